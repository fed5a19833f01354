// KV-cache write (reshape_and_cache) into the head-granular pool, gfx950.
//
// Pure byte movement.  A 256-thread workgroup takes 16 consecutive tokens of
// one kv head; thread (c, i) loads the 16-byte chunk c (dims 8c..8c+7) of
// token i of both K and V:
//   K pool [D/8][BS][8]: the chunk goes out as one 16-byte store; the 16
//     token-lanes of a chunk row are adjacent, so tokens in consecutive slots
//     of one block fill a contiguous 256-byte run.
//   V pool [D][BS]: 8 consecutive tokens of one dim are a 16-byte chunk of the
//     pool.  When 8 consecutive tokens of the workgroup go to 8 consecutive
//     slots starting at a multiple of 8 (every prompt written through a block
//     table does), the tile is transposed through LDS and thread (c, i) stores
//     the whole chunk of dim 8c + i%8 for token half i/8.  Any other mapping
//     (decode steps, arbitrary slots) takes the element path: the chunk's 8
//     dims as 8 two-byte stores BS*2 bytes apart.
#include "mux_common.h"

namespace mux {

constexpr int kVtRow = kHeadSize + 8;    // LDS row of one token: 256 B + 16 B so that rows shift banks

__global__ __launch_bounds__(256) void reshape_and_cache_kernel(
    const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, int64_t row_stride,
    uint4 *__restrict__ k_pool, uint16_t *__restrict__ v_pool, int64_t num_blocks,
    const int64_t *__restrict__ slots, int64_t slot_stride, int num_tokens, int block_size) {
  constexpr int D = kHeadSize;
  __shared__ __attribute__((aligned(16))) uint16_t vt[16][kVtRow];
  const int lane = threadIdx.x & 63;
  const int i = threadIdx.x & 15;
  const int c = threadIdx.x >> 4;
  const int t = blockIdx.x * 16 + i;
  const int h = blockIdx.y;
  int64_t slot = -1;
  if (t < num_tokens) slot = slots[static_cast<int64_t>(t) * slot_stride + h];
  const int64_t b = slot >= 0 ? slot / block_size : 0;
  const int o = static_cast<int>(slot - b * block_size);
  const bool live = slot >= 0 && b < num_blocks;   // never write outside the pool

  uint4 vx = make_uint4(0, 0, 0, 0);
  if (live) {
    const int64_t src = static_cast<int64_t>(t) * row_stride + h * D + c * 8;
    const uint4 kx = *reinterpret_cast<const uint4 *>(k + src);
    vx = *reinterpret_cast<const uint4 *>(v + src);
    k_pool[(b * (D / 8) + c) * block_size + o] = kx;
  }

  // Do the 8 tokens of this lane's half (lanes 8 j .. 8 j + 7 of the wave) go
  // to 8 consecutive slots that start a 16-byte chunk of the V pool?
  const int first = lane & ~7;
  const int64_t slot0 = (static_cast<int64_t>(__shfl(static_cast<int>(slot >> 32), first)) << 32) |
                        static_cast<uint32_t>(__shfl(static_cast<int>(slot), first));
  const bool in_run = live && slot == slot0 + (lane & 7) && (slot0 & 7) == 0;
  const unsigned long long runs = __builtin_amdgcn_ballot_w64(in_run);
  const bool chunked = ((runs >> first) & 0xffull) == 0xffull;

  *reinterpret_cast<uint4 *>(&vt[i][c * 8]) = vx;
  __syncthreads();
  if (chunked) {
    const int d = c * 8 + (i & 7);
    const int r0 = i & 8;                // first token row of this half
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      w[e] = static_cast<uint32_t>(vt[r0 + 2 * e][d]) | (static_cast<uint32_t>(vt[r0 + 2 * e + 1][d]) << 16);
    const int64_t b0 = slot0 / block_size;
    const int o0 = static_cast<int>(slot0 - b0 * block_size);
    *reinterpret_cast<uint4 *>(v_pool + (b0 * D + d) * block_size + o0) = make_uint4(w[0], w[1], w[2], w[3]);
  } else if (live) {
    uint16_t *vp = v_pool + (b * D + c * 8) * block_size + o;
    const uint32_t w[4] = {vx.x, vx.y, vx.z, vx.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      vp[(2 * e) * block_size] = static_cast<uint16_t>(w[e] & 0xffffu);
      vp[(2 * e + 1) * block_size] = static_cast<uint16_t>(w[e] >> 16);
    }
  }
}

}  // namespace mux

extern "C" int32_t mux_reshape_and_cache(const void *k, const void *v, int64_t kv_row_stride,
                                         void *k_pool, void *v_pool, int64_t num_pool_blocks,
                                         const int64_t *slot_mapping, int32_t layer, int32_t num_layers,
                                         int32_t num_tokens, int32_t num_kv_heads, int32_t head_size,
                                         int32_t block_size, int32_t dtype, void *stream) {
  using namespace mux;
  if (!k || !v || !k_pool || !v_pool || !slot_mapping) return MUXA_EINVAL;
  if (num_tokens < 0 || num_kv_heads <= 0 || num_pool_blocks <= 0) return MUXA_EINVAL;
  if (layer < 0 || layer >= num_layers) return MUXA_EINVAL;
  if (head_size != kHeadSize) return MUXA_EUNSUPPORTED;
  if (block_size != 8 && block_size != 16 && block_size != 32) return MUXA_EUNSUPPORTED;
  if (dtype != MUXA_DTYPE_F16 && dtype != MUXA_DTYPE_BF16) return MUXA_EUNSUPPORTED;
  if (kv_row_stride < static_cast<int64_t>(num_kv_heads) * kHeadSize || kv_row_stride % 8 != 0)
    return MUXA_EINVAL;
  const uintptr_t align = reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                          reinterpret_cast<uintptr_t>(k_pool) | reinterpret_cast<uintptr_t>(v_pool);
  if (align & 15u) return MUXA_EINVAL;
  if (num_kv_heads > 65535) return MUXA_EUNSUPPORTED;
  if (num_tokens == 0) return MUXA_OK;
  const int64_t slot_stride = static_cast<int64_t>(num_layers) * num_kv_heads;
  const int64_t *slots = slot_mapping + static_cast<int64_t>(layer) * num_kv_heads;
  dim3 grid((num_tokens + 15) / 16, num_kv_heads);
  hipLaunchKernelGGL(reshape_and_cache_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t *>(k), static_cast<const uint16_t *>(v), kv_row_stride,
                     static_cast<uint4 *>(k_pool), static_cast<uint16_t *>(v_pool), num_pool_blocks,
                     slots, slot_stride, num_tokens, block_size);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e);
  return MUXA_OK;
}
