// KV-cache write (reshape_and_cache) into the head-granular pool, gfx950.
//
// Pure byte movement.  A 256-thread workgroup takes about 16 consecutive
// tokens of one kv head; thread (c, i) loads the 16-byte chunk c (dims
// 8c..8c+7) of token i of both K and V:
//   K pool [D/8][BS][8]: the chunk goes out as one 16-byte store; the token
//     lanes of a chunk row are adjacent, so tokens in consecutive slots of one
//     block fill a contiguous run.
//   V pool [D][BS]: 8 consecutive tokens of one dim are a 16-byte chunk of the
//     pool.  Where 8 consecutive tokens go to 8 consecutive slots that start at
//     a multiple of 8 (every prompt written through a block table does, up to
//     its last few tokens) the tile is transposed through LDS and one thread
//     stores the whole chunk of a dim.  Tokens outside such runs (decode steps,
//     arbitrary slots, prompt tails) take the element path: a chunk's 8 dims
//     as 8 two-byte stores BS*2 bytes apart.
// Packed prompts start anywhere in the token stream, so runs are not aligned
// to multiples of 16 tokens.  The boundary between workgroups w-1 and w is
// therefore moved back from token 16w to the start of the run that contains
// token 16w, if there is one: both neighbours derive it from the same slots,
// the windows still tile the token stream exactly, each holds 9..23 tokens,
// and no run straddles two workgroups.
#include "mux_common.h"

namespace mux {

constexpr int kVtRow = kHeadSize + 8;    // LDS row of one token: 256 B + 16 B so that rows shift banks
constexpr int kSlotWin = 40;             // slots of tokens 16w-8 .. 16w+31 are examined

__global__ __launch_bounds__(256) void reshape_and_cache_kernel(
    const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, int64_t row_stride,
    uint4 *__restrict__ k_pool, uint16_t *__restrict__ v_pool, int64_t num_blocks,
    const int64_t *__restrict__ slots, int64_t slot_stride, int num_tokens, int block_size) {
  constexpr int D = kHeadSize;
  __shared__ __attribute__((aligned(16))) uint16_t vt[24][kVtRow];
  __shared__ int64_t s_slot[kSlotWin + 8];
  const int lane = threadIdx.x & 63;
  const int i = threadIdx.x & 15;
  const int c = threadIdx.x >> 4;
  const int h = blockIdx.y;
  const int T0 = blockIdx.x * 16;
  const int64_t pool_slots = num_blocks * block_size;

  // The nominal 16 tokens T0+i do not depend on the window: their loads go out
  // first and overlap the slot examination.
  const int t_nom = T0 + i;
  const int64_t src_nom = static_cast<int64_t>(t_nom) * row_stride + h * D + c * 8;
  uint4 kx = make_uint4(0, 0, 0, 0), vx = make_uint4(0, 0, 0, 0);
  if (t_nom < num_tokens) {
    kx = *reinterpret_cast<const uint4 *>(k + src_nom);
    vx = *reinterpret_cast<const uint4 *>(v + src_nom);
  }

  // Slots of tokens T0-8 .. T0+31; -1 for tokens outside the batch, skipped
  // tokens and slots outside the pool (never written).
  if (threadIdx.x < kSlotWin + 8) {
    const int t = T0 - 8 + static_cast<int>(threadIdx.x);
    int64_t sl = -1;
    if (threadIdx.x < kSlotWin && t >= 0 && t < num_tokens) sl = slots[static_cast<int64_t>(t) * slot_stride + h];
    s_slot[threadIdx.x] = (sl >= 0 && sl < pool_slots) ? sl : -1;
  }
  __syncthreads();
  // Bit j of `starts`: token T0-8+j begins a run (8 consecutive slots from a multiple of 8).
  bool is_start = false;
  if (lane < 32) {
    const int64_t s0 = s_slot[lane];
    is_start = s0 >= 0 && (s0 & 7) == 0;
#pragma unroll
    for (int e = 1; e < 8; ++e) is_start = is_start && s_slot[lane + e] == s0 + e;
  }
  const uint32_t starts = static_cast<uint32_t>(__builtin_amdgcn_ballot_w64(is_start));
  // Window [a, b) as bit positions [ja, jb): a run that contains a nominal
  // boundary token belongs to the later workgroup.
  const uint32_t before_lo = starts & 0x000000feu;        // runs starting at T0-7 .. T0-1
  const uint32_t before_hi = starts & 0x00fe0000u;        // runs starting at T0+9 .. T0+15
  const int ja = before_lo ? __ffs(before_lo) - 1 : 8;
  const int jb = before_hi ? __ffs(before_hi) - 1 : min(24, num_tokens - T0 + 8);
  const uint32_t in_win = starts & (~0u << ja) & ~(~0u << jb);   // runs that start inside the window

  // Rows of the LDS tile are bit positions: 8 + i for the nominal tokens, i for
  // the up to 7 tokens taken over from the previous workgroup's nominal range.
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int j = pass == 0 ? 8 + i : i;
    if (pass == 1) {
      if (i >= 8) break;
      kx = make_uint4(0, 0, 0, 0);
      vx = make_uint4(0, 0, 0, 0);
    }
    const int64_t slot = (j >= ja && j < jb) ? s_slot[j] : -1;
    if (slot >= 0) {
      const int64_t blk = slot / block_size;
      const int o = static_cast<int>(slot - blk * block_size);
      if (pass == 1) {
        const int64_t src = static_cast<int64_t>(T0 - 8 + j) * row_stride + h * D + c * 8;
        kx = *reinterpret_cast<const uint4 *>(k + src);
        vx = *reinterpret_cast<const uint4 *>(v + src);
      }
      k_pool[(blk * (D / 8) + c) * block_size + o] = kx;
      // Element path for tokens that no run covers (a run starts at most 7 tokens back).
      const uint32_t cover = in_win & (0xffu << (j > 7 ? j - 7 : 0)) & ~(~0u << (j + 1));
      if (cover == 0) {
        uint16_t *vp = v_pool + (blk * D + c * 8) * block_size + o;
        const uint32_t w[4] = {vx.x, vx.y, vx.z, vx.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          vp[(2 * e) * block_size] = static_cast<uint16_t>(w[e] & 0xffffu);
          vp[(2 * e + 1) * block_size] = static_cast<uint16_t>(w[e] >> 16);
        }
      }
    }
    if (in_win != 0) *reinterpret_cast<uint4 *>(&vt[j][c * 8]) = vx;
  }
  if (in_win == 0) return;                                 // uniform: no run in this window
  __syncthreads();
  // Up to two runs per window; thread (c, i) stores dim 8c + i%8 of run i/8.
  uint32_t m = in_win;
  if (i >= 8) m &= m - 1;                                  // drop the first run
  if (m != 0) {
    const int jp = __ffs(m) - 1;                           // bit, and LDS row, of the run's first token
    const int d = c * 8 + (i & 7);
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      w[e] = static_cast<uint32_t>(vt[jp + 2 * e][d]) | (static_cast<uint32_t>(vt[jp + 2 * e + 1][d]) << 16);
    const int64_t slot0 = s_slot[jp];
    const int64_t b0 = slot0 / block_size;
    const int o0 = static_cast<int>(slot0 - b0 * block_size);
    *reinterpret_cast<uint4 *>(v_pool + (b0 * D + d) * block_size + o0) = make_uint4(w[0], w[1], w[2], w[3]);
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
  if (num_pool_blocks > (int64_t{1} << 56)) return MUXA_EINVAL;   // slot arithmetic stays in 64 bits
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
