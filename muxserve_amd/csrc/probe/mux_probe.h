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

#ifdef __cplusplus
}
#endif
#endif
