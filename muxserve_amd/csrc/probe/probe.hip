// Bare gather read of pool blocks, gfx950: the memory side of a decode step
// without its arithmetic, table walk or softmax.  A measuring aid: it shows
// what rate the access pattern of paged decode attention - whole 4 KiB K and
// V head-blocks scattered over the pool - gets from the memory system, next to
// which the attention kernel's own rate can be read.
//
// A wave takes four consecutive ids of the list (64 tokens at block size 16)
// and issues the loads the attention kernel issues for such a tile: lane t
// reads the 16 chunks of "its" token from the K block, then the wave reads the
// four V blocks as consecutive 1 KiB runs; all 32 loads are non-temporal and in
// flight together.  The data is folded into one word that is never stored
// unless it equals an arbitrary constant, so the loads cannot be optimised away.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mux_probe.h"

namespace mux {

typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void probe_gather_read_kernel(const uint4 *__restrict__ k_pool,
                                                                const uint4 *__restrict__ v_pool,
                                                                const int32_t *__restrict__ ids, int64_t n_blocks,
                                                                int64_t num_pool_blocks, uint32_t *sink) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t first = (static_cast<int64_t>(blockIdx.x) * 4 + wave) * 4;
  if (first >= n_blocks) return;
  // Ids past the list repeat its last entry; ids outside the pool are clamped.
  const int last_block = static_cast<int>(min(num_pool_blocks - 1, int64_t{0x7fffffff}));
  const int id = min(max(ids[min(first + (lane >> 4), n_blocks - 1)], 0), last_block);
  probe_u32x4 r[32];
  const uint4 *kp = k_pool + static_cast<int64_t>(id) * 256 + (lane & 15);
#pragma unroll
  for (int j = 0; j < 16; ++j) r[j] = __builtin_nontemporal_load(reinterpret_cast<const probe_u32x4 *>(&kp[j * 16]));
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const uint4 *vp = v_pool + static_cast<int64_t>(__builtin_amdgcn_readlane(id, 16 * b)) * 256 + lane;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      r[16 + 4 * b + j] = __builtin_nontemporal_load(reinterpret_cast<const probe_u32x4 *>(&vp[j * 64]));
  }
  uint32_t acc = 0;
#pragma unroll
  for (int j = 0; j < 32; ++j) acc += r[j].x ^ r[j].y ^ r[j].z ^ r[j].w;
  if (acc == 0x9e3779b9u) sink[0] = acc;
}

}  // namespace mux

extern "C" int32_t mux_probe_gather_read(const void *k_pool, const void *v_pool, int64_t num_pool_blocks,
                                         const int32_t *block_ids, int64_t n_blocks, int32_t block_size,
                                         uint32_t *sink, void *stream) {
  using namespace mux;
  if (!k_pool || !v_pool || !sink || num_pool_blocks <= 0 || n_blocks < 0) return -1;
  if (n_blocks > 0 && !block_ids) return -1;
  if ((reinterpret_cast<uintptr_t>(k_pool) | reinterpret_cast<uintptr_t>(v_pool)) & 15u) return -1;
  if (block_size != 16) return -2;       // 4 KiB head-blocks: 256 chunks of 16 bytes
  if (n_blocks == 0) return 0;
  const int64_t n_wg = (n_blocks + 15) / 16;
  if (n_wg > 0x7fffffff) return -2;
  hipLaunchKernelGGL(probe_gather_read_kernel, dim3(static_cast<uint32_t>(n_wg)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4 *>(k_pool),
                     static_cast<const uint4 *>(v_pool), block_ids, n_blocks, num_pool_blocks, sink);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}

// ---------------------------------------------------------------------------
// Where workgroups run: every workgroup of the launch records the accelerator
// die (XCC_ID register) and the hardware id word (HW_ID register: compute unit,
// shader array, shader engine, ...) of the compute unit it was started on, then
// spins for `spin_ticks` of the 100 MHz clock so that the launch spreads over
// every compute unit the stream may use.  The evidence behind CU-masked streams:
// which mask bit enables which compute unit.
// ---------------------------------------------------------------------------
namespace mux {

__global__ __launch_bounds__(64) void probe_where_kernel(uint32_t *out, int spin_ticks) {
  // s_getreg_b32: id | offset << 6 | (size - 1) << 11; HW_ID is register 4, XCC_ID register 20.
  const uint32_t hw_id = __builtin_amdgcn_s_getreg(4 | (0 << 6) | (31 << 11));
  const uint32_t xcc_id = __builtin_amdgcn_s_getreg(20 | (0 << 6) | (31 << 11));
  if (threadIdx.x == 0) {
    out[2 * blockIdx.x] = xcc_id;
    out[2 * blockIdx.x + 1] = hw_id;
  }
  const long long until = static_cast<long long>(__builtin_amdgcn_s_memrealtime()) + spin_ticks;
  while (static_cast<long long>(__builtin_amdgcn_s_memrealtime()) < until) __builtin_amdgcn_s_sleep(8);
}

}  // namespace mux

extern "C" int32_t mux_probe_where(uint32_t *out, int32_t num_workgroups, int32_t spin_microseconds, void *stream) {
  if (!out || num_workgroups <= 0 || spin_microseconds < 0 || spin_microseconds > 100000) return -1;
  hipLaunchKernelGGL(mux::probe_where_kernel, dim3(static_cast<uint32_t>(num_workgroups)), dim3(64), 0,
                     static_cast<hipStream_t>(stream), out, spin_microseconds * 100);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}

// ---------------------------------------------------------------------------
// Contiguous copy: what a read + write mix of a given size gets from the memory
// system, next to which the cache write's rate can be read.  One 16-byte chunk
// per thread, loads and stores non-temporal (the form that measured fastest:
// 6.2 TB/s for 109 MB in + 109 MB out against 5.15 TB/s for the framework's copy
// kernel; more chunks per thread, resident workgroups walking the buffer, or
// either hint dropped were all slower).
// ---------------------------------------------------------------------------
namespace mux {

__global__ __launch_bounds__(256) void probe_copy_kernel(probe_u32x4 *__restrict__ dst,
                                                         const probe_u32x4 *__restrict__ src, int64_t n_chunks) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n_chunks) __builtin_nontemporal_store(__builtin_nontemporal_load(&src[i]), &dst[i]);
}

}  // namespace mux

extern "C" int32_t mux_probe_copy(void *dst, const void *src, int64_t nbytes, void *stream) {
  if (!dst || !src || nbytes < 0 || (nbytes & 15)) return -1;
  if ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u) return -1;
  const int64_t n = nbytes / 16;
  if (n == 0) return 0;
  const int64_t n_wg = (n + 255) / 256;
  if (n_wg > 0x7fffffff) return -2;
  hipLaunchKernelGGL(mux::probe_copy_kernel, dim3(static_cast<uint32_t>(n_wg)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<mux::probe_u32x4 *>(dst),
                     static_cast<const mux::probe_u32x4 *>(src), n);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}
