/* libmuxprobe.so: a measuring aid for bench.py and its test, not part of the
 * product boundary (include/ declares that).  Built by `python -m
 * muxserve_amd.build probe`. */
#ifndef MUX_PROBE_H
#define MUX_PROBE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Reads the K and V head-blocks named by block_ids (DEVICE int32 [n_blocks];
 * entries outside the pool are clamped) with the load pattern of the decode
 * kernel - four blocks per wave, all loads in flight - and does nothing else:
 * the rate it reaches is what the memory system gives to whole 4 KiB blocks
 * scattered over the pool, the yardstick next to the attention kernel's own
 * rate.  block_size must be 16.  sink: DEVICE uint32 [1] (only ever written
 * when the folded data equals an arbitrary constant).  Returns 0, -1 (invalid
 * argument), -2 (unsupported block size) or -4 (HIP error). */
int32_t mux_probe_gather_read(const void *k_pool, const void *v_pool, int64_t num_pool_blocks,
                              const int32_t *block_ids, int64_t n_blocks, int32_t block_size,
                              uint32_t *sink, void *stream);

/* Records where the workgroups of a launch run: out (DEVICE uint32
 * [num_workgroups, 2]) receives per workgroup the XCC_ID register (accelerator
 * die in its low 4 bits) and the HW_ID register (compute unit id in bits 8-11,
 * shader array in bit 12, shader engine in bits 13-15) of its compute unit; each
 * workgroup (one wave) then idles for spin_microseconds so that the launch
 * spreads over every compute unit its stream may use. */
int32_t mux_probe_where(uint32_t *out, int32_t num_workgroups, int32_t spin_microseconds, void *stream);

/* Copies nbytes (a multiple of 16; both pointers 16-byte aligned) from src to
 * dst with non-temporal 16-byte loads and stores, one chunk per thread: the
 * yardstick for kernels that read and write equal amounts (the cache write). */
int32_t mux_probe_copy(void *dst, const void *src, int64_t nbytes, void *stream);

/* The same copy with the cache write's destinations: block b (4 KiB) of k_src
 * and of v_src goes to pool block block_ids[b] (DEVICE int32 [n_blocks]; ids
 * outside the pool are clamped) of k_pool and v_pool, read contiguously, written
 * scattered - the byte movement of a prompt's cache write at block size 16
 * without its windows, slot arithmetic and transposition. */
int32_t mux_probe_scatter_copy(void *k_pool, void *v_pool, int64_t num_pool_blocks, const void *k_src,
                               const void *v_src, const int32_t *block_ids, int64_t n_blocks, void *stream);

/* What the matrix cores sustain: num_workgroups workgroups of
 * waves_per_workgroup (1..8) waves; waves below mfma_waves run `iterations`
 * iterations of `chains` (1, 2 or 4) independent v_mfma_f32_32x32x16_f16
 * accumulations from register operands (32768 flop each per wave) plus
 * valu_per_iteration (0; with 4 chains also 8 or 32) dependent v_fma_f32; the
 * remaining waves run 32 independent v_fma_f32 per iteration and no MFMA.  ticks
 * (DEVICE uint32 [num_workgroups, 2]) receives per workgroup the shader-clock
 * ticks and the 100 MHz ticks wave 0's loop took.  sink: DEVICE float [1].
 * Returns 0, -1 (invalid argument), -2 (combination not built) or -4. */
int32_t mux_probe_mfma(int32_t chains, int32_t valu_per_iteration, int32_t iterations, int32_t num_workgroups,
                       int32_t waves_per_workgroup, int32_t mfma_waves, uint32_t *ticks, float *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif
