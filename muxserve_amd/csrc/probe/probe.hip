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

// ---------------------------------------------------------------------------
// The same copy with the cache write's destinations: the sources are read
// contiguously, 4 KiB at a time, and every 4 KiB lands in the pool block the id
// list names - one K block and one V block per workgroup, as the cache write of a
// prompt leaves them, without its token windows, slot arithmetic and
// transposition.  What separates this from the contiguous copy is the cost of
// scattering the writes over the pool; what separates the cache write from this
// is the cost of its own structure.
// ---------------------------------------------------------------------------
namespace mux {

__global__ __launch_bounds__(256) void probe_scatter_copy_kernel(probe_u32x4 *__restrict__ k_dst,
                                                                 probe_u32x4 *__restrict__ v_dst,
                                                                 const probe_u32x4 *__restrict__ k_src,
                                                                 const probe_u32x4 *__restrict__ v_src,
                                                                 const int32_t *__restrict__ ids, int64_t num_pool_blocks) {
  const int64_t b = blockIdx.x;
  const int64_t last = num_pool_blocks - 1;
  int64_t id = ids[b];
  id = id < 0 ? 0 : (id > last ? last : id);               // ids outside the pool are clamped
  const probe_u32x4 kx = __builtin_nontemporal_load(&k_src[b * 256 + threadIdx.x]);
  const probe_u32x4 vx = __builtin_nontemporal_load(&v_src[b * 256 + threadIdx.x]);
  __builtin_nontemporal_store(kx, &k_dst[id * 256 + threadIdx.x]);
  __builtin_nontemporal_store(vx, &v_dst[id * 256 + threadIdx.x]);
}

}  // namespace mux

extern "C" int32_t mux_probe_scatter_copy(void *k_pool, void *v_pool, int64_t num_pool_blocks, const void *k_src,
                                          const void *v_src, const int32_t *block_ids, int64_t n_blocks, void *stream) {
  if (!k_pool || !v_pool || !k_src || !v_src || num_pool_blocks <= 0 || n_blocks < 0) return -1;
  if (n_blocks > 0 && !block_ids) return -1;
  if ((reinterpret_cast<uintptr_t>(k_pool) | reinterpret_cast<uintptr_t>(v_pool) | reinterpret_cast<uintptr_t>(k_src) |
       reinterpret_cast<uintptr_t>(v_src)) & 15u)
    return -1;
  if (n_blocks == 0) return 0;
  if (n_blocks > 0x7fffffff) return -2;
  hipLaunchKernelGGL(mux::probe_scatter_copy_kernel, dim3(static_cast<uint32_t>(n_blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<mux::probe_u32x4 *>(k_pool),
                     static_cast<mux::probe_u32x4 *>(v_pool), static_cast<const mux::probe_u32x4 *>(k_src),
                     static_cast<const mux::probe_u32x4 *>(v_src), block_ids, num_pool_blocks);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}

// ---------------------------------------------------------------------------
// What the matrix cores sustain, and what they sustain beside vector-ALU work:
// waves 0 .. mfma_waves-1 of a workgroup run `iters` iterations of CHAINS
// independent v_mfma_f32_32x32x16_f16 accumulations (operands in registers,
// nothing else in the loop) plus VALU dependent v_fma_f32 of their own; the
// other waves run 32 independent v_fma_f32 per iteration and no MFMA.  The
// figures the causal prefill kernel is priced against: the dense peak is quoted
// at 2.4 GHz, and under sustained matrix work the shader clock settles lower.
// Wave 0 of every workgroup reports the shader-clock and 100 MHz-clock ticks its
// loop took, which gives the clock the chip really ran at.
// ---------------------------------------------------------------------------
namespace mux {

typedef _Float16 probe_v8f16 __attribute__((ext_vector_type(8)));
typedef float probe_v16f32 __attribute__((ext_vector_type(16)));

template <int CHAINS, int VALU>
__global__ __launch_bounds__(512) void probe_mfma_kernel(int iters, int mfma_waves, uint32_t *__restrict__ ticks,
                                                         float *sink) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const long long c0 = __builtin_readcyclecounter();
  const long long r0 = static_cast<long long>(__builtin_amdgcn_s_memrealtime());
  float folded = 0.f;
  if (wave < mfma_waves) {
    probe_v8f16 a, b;
    // Operands with all mantissa bits in play (a multiplier fed with zeros or small
    // integers draws less power and would flatter the clock): hashed values in (-1, 1).
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t h = (threadIdx.x * 8u + i + blockIdx.x * 4099u) * 2654435761u;
      h ^= h >> 15;
      h *= 2246822519u;
      h ^= h >> 13;
      a[i] = static_cast<_Float16>(static_cast<float>(static_cast<int>(h & 0xffffu) - 32768) * (1.f / 32768.f));
      b[i] = static_cast<_Float16>(static_cast<float>(static_cast<int>(h >> 16) - 32768) * (1.f / 32768.f));
    }
    probe_v16f32 acc[CHAINS];
#pragma unroll
    for (int c = 0; c < CHAINS; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[c][i] = 0.f;
    float f = static_cast<float>(threadIdx.x), g = 1.0001f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int c = 0; c < CHAINS; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[c], 0, 0, 0);
#pragma unroll
      for (int v = 0; v < VALU; ++v) f = __builtin_fmaf(f, g, 0.5f);
      asm volatile("" : "+v"(f));
    }
#pragma unroll
    for (int c = 0; c < CHAINS; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) folded += acc[c][i];
    folded += f;
  } else {
    float f[32];
#pragma unroll
    for (int v = 0; v < 32; ++v) f[v] = static_cast<float>(threadIdx.x + v);
    const float g = 1.0001f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int v = 0; v < 32; ++v) {
        f[v] = __builtin_fmaf(f[v], g, 0.5f);
        asm volatile("" : "+v"(f[v]));
      }
    }
#pragma unroll
    for (int v = 0; v < 32; ++v) folded += f[v];
  }
  const long long c1 = __builtin_readcyclecounter();
  const long long r1 = static_cast<long long>(__builtin_amdgcn_s_memrealtime());
  if (threadIdx.x == 0) {
    ticks[2 * blockIdx.x] = static_cast<uint32_t>(c1 - c0);
    ticks[2 * blockIdx.x + 1] = static_cast<uint32_t>(r1 - r0);
  }
  if (folded == 123.456f) sink[0] = folded;     // keeps the loops alive; practically never taken
}

}  // namespace mux

extern "C" int32_t mux_probe_mfma(int32_t chains, int32_t valu_per_iteration, int32_t iterations,
                                  int32_t num_workgroups, int32_t waves_per_workgroup, int32_t mfma_waves,
                                  uint32_t *ticks, float *sink, void *stream) {
  using namespace mux;
  if (!ticks || !sink || iterations <= 0 || iterations > (1 << 24) || num_workgroups <= 0) return -1;
  if (waves_per_workgroup < 1 || waves_per_workgroup > 8 || mfma_waves < 0 || mfma_waves > waves_per_workgroup) return -1;
  const dim3 grid(static_cast<uint32_t>(num_workgroups)), block(static_cast<uint32_t>(64 * waves_per_workgroup));
  hipStream_t st = static_cast<hipStream_t>(stream);
#define MUX_PROBE_MFMA(C, V)                                                                                  \
  if (chains == C && valu_per_iteration == V) {                                                                \
    hipLaunchKernelGGL((probe_mfma_kernel<C, V>), grid, block, 0, st, iterations, mfma_waves, ticks, sink);    \
    return hipGetLastError() == hipSuccess ? 0 : -4;                                                           \
  }
  MUX_PROBE_MFMA(1, 0)
  MUX_PROBE_MFMA(2, 0)
  MUX_PROBE_MFMA(4, 0)
  MUX_PROBE_MFMA(4, 8)
  MUX_PROBE_MFMA(4, 32)
#undef MUX_PROBE_MFMA
  return -2;
}
