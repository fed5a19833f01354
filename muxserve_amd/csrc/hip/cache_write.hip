// KV-cache write (reshape_and_cache) into the head-granular pool, gfx950.
//
// Pure byte movement.  A 256-thread workgroup takes about 16 consecutive
// tokens of one kv head.  Loading, thread (i, c) takes the 16-byte chunk c (dims
// 8c..8c+7) of token i of both K and V, so that a token's 256-byte head slice is
// read by 16 neighbouring threads; the tile goes to LDS, one row per token, and
// is stored from there by thread (c, i):
//   K pool [D/8][BS][8]: the chunk goes out as one 16-byte store; the token
//     lanes of a chunk row are adjacent, so tokens in consecutive slots of one
//     block fill a contiguous run.
//   V pool [D][BS]: 8 consecutive tokens of one dim are a 16-byte chunk of the
//     pool.  Where 8 consecutive tokens go to 8 consecutive slots that start at
//     a multiple of 8 (every prompt written through a block table does, up to
//     its last few tokens) one thread gathers a dim's 8 values from the LDS rows
//     and stores the whole chunk.  Tokens outside such runs (decode steps,
//     arbitrary slots, prompt tails) take the element path: a chunk's 8 dims
//     as 8 two-byte stores BS*2 bytes apart.
// Packed prompts start anywhere in the token stream, so runs are not aligned
// to multiples of 16 tokens.  The boundary between workgroups w-1 and w is
// therefore moved back from token 16w to the start of the run that contains
// token 16w - and, when that run is the second half of a pool block whose first
// half precedes it, on to the start of the block: inside a prompt every window
// is then exactly one pool block (whole K and V rows, streamed past the L2),
// whatever the prompt's position in the stream.  Both neighbours derive the
// boundary from the same slots, the windows still tile the token stream
// exactly, each holds 1..31 tokens, and no run straddles two workgroups.  The
// slots are read first and only the window's own tokens are loaded.
//
// Fused variant (ROPE): the same kernel first applies the NeoX rotary embedding
// to k (and to the query heads that share this kv head) for the tokens of its
// window, in place, and scatters the rotated k - one launch and one pass over k
// instead of a rotary kernel followed by the cache write.  A thread's chunk c
// pairs with chunk c^8 (dims +-64) of the same token: both are read, the
// workgroup meets, then the rotated chunk goes back in place and into the pool.
#include "mux_common.h"

namespace mux {

struct RopeArgs {
  uint16_t *q;                 // rotated in place; may be null
  int64_t q_stride;
  int32_t ratio;               // query heads per kv head
  const int64_t *positions;    // [num_tokens]
  const float *cos_sin;        // [max_position, 128] = [cos | sin]
  int32_t max_position;
};

// out = own * cos + (is_y ? +1 : -1) * partner * sin, elementwise on 8 packed values.
template <typename T>
__device__ __forceinline__ uint4 rotate_chunk(const uint4 own, const uint4 partner, const float (&cs)[8],
                                              const float (&sn)[8], bool is_y) {
  const uint32_t a[4] = {own.x, own.y, own.z, own.w};
  const uint32_t b[4] = {partner.x, partner.y, partner.z, partner.w};
  uint32_t o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float a0, a1, b0, b1;
    if constexpr (__is_same(T, F16)) {
      const half2_t ah = as_half2(a[e]), bh = as_half2(b[e]);
      a0 = static_cast<float>(ah.x); a1 = static_cast<float>(ah.y);
      b0 = static_cast<float>(bh.x); b1 = static_cast<float>(bh.y);
    } else {
      a0 = bf16_lo(a[e]); a1 = bf16_hi(a[e]);
      b0 = bf16_lo(b[e]); b1 = bf16_hi(b[e]);
    }
    // x' = x c - y s for the low half of a head, y' = y c + x s for the high half.
    const float r0 = is_y ? a0 * cs[2 * e] + b0 * sn[2 * e] : a0 * cs[2 * e] - b0 * sn[2 * e];
    const float r1 = is_y ? a1 * cs[2 * e + 1] + b1 * sn[2 * e + 1] : a1 * cs[2 * e + 1] - b1 * sn[2 * e + 1];
    o[e] = static_cast<uint32_t>(to_storage<T>(r0)) | (static_cast<uint32_t>(to_storage<T>(r1)) << 16);
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

// Stores that fill whole 128-byte lines by themselves go out non-temporal
// (nothing to merge with, and the pool is not read back soon): K rows of a run
// of 8 consecutive slots, V rows when the workgroup holds every run of the row.
typedef uint32_t cw_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store16(void *p, const uint4 x, bool streaming) {
  const cw_u32x4 v = {x.x, x.y, x.z, x.w};
  if (streaming) {
    // Written as an instruction: as two C++ stores that differ only in the hint,
    // the optimiser folds the branches into one store and drops it.  The
    // compiler does not know that the instruction is still reading its data
    // registers when the next one issues, so the wait states between a 16-byte
    // store and a write of its data registers are spelled out (one was not
    // enough once the next store's operands were already in registers).
    asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 4" ::"v"(p), "v"(v) : "memory");
  } else {
    *static_cast<cw_u32x4 *>(p) = v;
  }
}

constexpr int kVtRow = kHeadSize + 8;    // LDS row of one token: 256 B + 16 B so that rows shift banks
constexpr int kBack = 16;                // tokens before the nominal 16 that a window may take over
constexpr int kSlotWin = 48;             // slots of tokens 16w-16 .. 16w+31 are examined
constexpr int kTileRows = 32;            // a window lies inside tokens 16w-16 .. 16w+15

// One workgroup's window: kv head h, tokens around T0 (a multiple of 16).
template <typename T, bool ROPE>
__device__ __forceinline__ void cache_write_window(
    uint16_t *k, const uint16_t *__restrict__ v, int64_t row_stride,
    uint4 *__restrict__ k_pool, uint16_t *__restrict__ v_pool, int64_t num_blocks,
    const int64_t *__restrict__ slots, int64_t slot_stride, int num_tokens, int block_size, const RopeArgs &R,
    const int h, const int T0) {
  constexpr int D = kHeadSize;
  __shared__ __attribute__((aligned(16))) uint16_t kt[kTileRows][kVtRow];
  __shared__ __attribute__((aligned(16))) uint16_t vt[kTileRows][kVtRow];
  __shared__ int64_t s_slot[kSlotWin + 8];
  const int lane = threadIdx.x & 63;
  const int i = threadIdx.x & 15;
  const int c = threadIdx.x >> 4;
  const int64_t pool_slots = num_blocks * block_size;
  // Block sizes are powers of two (8, 16, 32): slot -> (block, offset) by shift and mask.
  const int bs_shift = __builtin_ctz(static_cast<unsigned>(block_size));

  // Slots of tokens T0-16 .. T0+31 (bit j of the masks below is token T0-16+j);
  // -1 for tokens outside the batch, skipped tokens and slots outside the pool
  // (never written).
  if (threadIdx.x < kSlotWin + 8) {
    const int t = T0 - kBack + static_cast<int>(threadIdx.x);
    int64_t sl = -1;
    if (threadIdx.x < kSlotWin && t >= 0 && t < num_tokens) sl = slots[static_cast<int64_t>(t) * slot_stride + h];
    s_slot[threadIdx.x] = (sl >= 0 && sl < pool_slots) ? sl : -1;
  }
  __syncthreads();
  // Bit j of `starts`: token j begins a run (8 consecutive slots from a multiple of 8).
  bool is_start = false;
  if (lane < 40) {
    const int64_t s0 = s_slot[lane];
    is_start = s0 >= 0 && (s0 & 7) == 0;
#pragma unroll
    for (int e = 1; e < 8; ++e) is_start = is_start && s_slot[lane + e] == s0 + e;
  }
  const unsigned long long starts = __builtin_amdgcn_ballot_w64(is_start);
  // The boundary next to nominal bit n: the start of the run that contains
  // token n, moved on to the start of that run's pool block when the run is the
  // block's second half and the first half sits right before it - so that
  // inside a prompt a window is exactly one pool block.  Both neighbours derive
  // the boundary from the same slots.
  auto boundary = [&](int n) {
    const unsigned long long cand = starts & (0xffull << (n - 7));      // runs starting at n-7 .. n
    if (cand == 0) return n;
    int sbit = __ffsll(cand) - 1;
    if (block_size == 16 && (s_slot[sbit] & 15) == 8 && ((starts >> (sbit - 8)) & 1ull) != 0 &&
        s_slot[sbit - 8] == s_slot[sbit] - 8)
      sbit -= 8;
    return sbit;
  };
  const int ja = boundary(kBack);
  const int jb = min(boundary(kBack + 16), num_tokens - T0 + kBack);
  const unsigned long long in_win = starts & (~0ull << ja) & ~(~0ull << jb);   // runs that start inside the window
  // Does this window write whole pool rows and nothing else?  K rows of a run are
  // 128 bytes; a V row is block_size * 2 bytes: one run fills it at block size 8,
  // the two runs of a block at 16, never at 32.  Such a window streams its stores
  // past the L2 (uniform over the workgroup).
  const int n_runs = __popcll(in_win);
  const int first_bit = n_runs > 0 ? __ffsll(in_win) - 1 : 0;
  const bool rows_complete =
      n_runs > 0 && jb - ja == 8 * n_runs &&
      (block_size == 8 || (block_size == 16 && n_runs == 2 && ((in_win >> (first_bit + 8)) & 1ull) != 0 &&
                           (s_slot[first_bit] & 15) == 0 && s_slot[first_bit + 8] == s_slot[first_bit] + 8));

  // Loads: thread (token il, chunk cl) - the 16 threads of a token read its whole
  // 256-byte head slice, a wave four such slices, every line exactly once.
  // (Non-temporal loads make no difference whether k/v come from HBM or were
  // just written by the projection, and lose when the same buffers are read
  // again.)  Stores: thread
  // (chunk row c, token i) - the 16 threads of a chunk row write one whole
  // 256-byte K row of the block with a single store instruction (split over
  // two, the non-temporal stores would each leave partial lines).  In between
  // the tile sits in LDS, one row per token (rows are bit positions); V is
  // transposed on its way out.  A window has at most 31 tokens: two passes of
  // 16, the second one rare.
  const bool two_passes = jb - ja > 16;                    // uniform
  const int il = threadIdx.x >> 4, cl = threadIdx.x & 15;
  const int pc = (cl ^ 8) - cl;            // the partner chunk of the rotation, in chunks from this one
  uint4 kx2[2], vx2[2], kp2[2];
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    kx2[pass] = vx2[pass] = kp2[pass] = make_uint4(0, 0, 0, 0);
    if (pass == 1 && !two_passes) break;
    const int j = ja + 16 * pass + il;
    if (j < jb && (ROPE || s_slot[j] >= 0)) {
      const int64_t src = static_cast<int64_t>(T0 - kBack + j) * row_stride + h * D + cl * 8;
      kx2[pass] = *reinterpret_cast<const uint4 *>(k + src);
      vx2[pass] = *reinterpret_cast<const uint4 *>(v + src);
      if constexpr (ROPE) kp2[pass] = *reinterpret_cast<const uint4 *>(k + src + pc * 8);
    }
  }
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    if (pass == 1 && !two_passes) break;
    const int j = ja + 16 * pass + il;
    const bool mine = j < jb;                              // token T0-16+j is in this window
    uint4 kx = kx2[pass];
    if constexpr (ROPE) {
      // Rotate k of every token of the window (also tokens without a slot), and
      // the query heads of this kv head, four at a time; all reads of a group
      // precede its writes (the workgroup meets in between), because a thread's
      // partner chunk is another thread's own.
      const int t = T0 - kBack + j;
      const int64_t src = static_cast<int64_t>(t) * row_stride + h * D + cl * 8;
      float cs[8], sn[8];
      if (mine) {
        int64_t pos = R.positions[t];
        pos = pos < 0 ? 0 : (pos >= R.max_position ? R.max_position - 1 : pos);
        const float *row = R.cos_sin + pos * D + (cl & 7) * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          cs[e] = row[e];
          sn[e] = row[D / 2 + e];
        }
        kx = rotate_chunk<T>(kx, kp2[pass], cs, sn, cl >= 8);
      }
      const int n_q = R.q != nullptr ? R.ratio : 0;
      uint16_t *q0 = R.q + static_cast<int64_t>(t) * R.q_stride + static_cast<int64_t>(h) * R.ratio * D + cl * 8;
      for (int g0 = 0; g0 < max(n_q, 1); g0 += 4) {
        uint4 qx[4];
#pragma unroll
        for (int g = 0; g < 4; ++g)
          if (mine && g0 + g < n_q) {
            const uint16_t *qp = q0 + (g0 + g) * D;
            qx[g] = rotate_chunk<T>(*reinterpret_cast<const uint4 *>(qp),
                                    *reinterpret_cast<const uint4 *>(qp + pc * 8), cs, sn, cl >= 8);
          }
        __syncthreads();
        if (mine && g0 == 0) *reinterpret_cast<uint4 *>(k + src) = kx;
#pragma unroll
        for (int g = 0; g < 4; ++g)
          if (mine && g0 + g < n_q) *reinterpret_cast<uint4 *>(q0 + (g0 + g) * D) = qx[g];
      }
    }
    if (mine) {
      *reinterpret_cast<uint4 *>(&kt[j][cl * 8]) = kx;
      *reinterpret_cast<uint4 *>(&vt[j][cl * 8]) = vx2[pass];
    }
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    if (pass == 1 && !two_passes) break;
    const int j = ja + 16 * pass + i;
    const int64_t slot = j < jb ? s_slot[j] : -1;
    if (slot >= 0) {
      const int64_t blk = slot >> bs_shift;
      const int o = static_cast<int>(slot) & (block_size - 1);
      // Element path for tokens that no run covers (a run starts at most 7 tokens back).
      const unsigned long long cover = in_win & (0xffull << (j > 7 ? j - 7 : 0)) & ~(~0ull << (j + 1));
      store16(&k_pool[(blk * (D / 8) + c) * block_size + o], *reinterpret_cast<const uint4 *>(&kt[j][c * 8]),
              rows_complete);
      if (cover == 0) {
        uint16_t *vp = v_pool + (blk * D + c * 8) * block_size + o;
        const uint4 vx = *reinterpret_cast<const uint4 *>(&vt[j][c * 8]);
        const uint32_t w[4] = {vx.x, vx.y, vx.z, vx.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          vp[(2 * e) * block_size] = static_cast<uint16_t>(w[e] & 0xffffu);
          vp[(2 * e + 1) * block_size] = static_cast<uint16_t>(w[e] >> 16);
        }
      }
    }
  }
  // Up to three runs per window; thread (c, i) stores dim 8c + i%8 of runs i/8, i/8 + 2.
  for (int r = i >> 3; r < n_runs; r += 2) {
    unsigned long long m = in_win;
    for (int q = 0; q < r; ++q) m &= m - 1;                // drop the runs before run r
    const int jp = __ffsll(m) - 1;                         // bit, and LDS row, of the run's first token
    const int d = c * 8 + (i & 7);
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      w[e] = static_cast<uint32_t>(vt[jp + 2 * e][d]) | (static_cast<uint32_t>(vt[jp + 2 * e + 1][d]) << 16);
    const int64_t slot0 = s_slot[jp];
    const int64_t b0 = slot0 >> bs_shift;
    const int o0 = static_cast<int>(slot0) & (block_size - 1);
    store16(v_pool + (b0 * D + d) * block_size + o0, make_uint4(w[0], w[1], w[2], w[3]), rows_complete);
  }
}

// Heads vary fastest over the workgroup ids: workgroups that run together read
// the neighbouring 256-byte head slices of the same k/v rows (one DRAM page)
// rather than one slice out of each of many rows.
template <typename T, bool ROPE>
__global__ __launch_bounds__(256) void reshape_and_cache_kernel(
    uint16_t *k, const uint16_t *__restrict__ v, int64_t row_stride,
    uint4 *__restrict__ k_pool, uint16_t *__restrict__ v_pool, int64_t num_blocks,
    const int64_t *__restrict__ slots, int64_t slot_stride, int num_tokens, int block_size, const RopeArgs R) {
  cache_write_window<T, ROPE>(k, v, row_stride, k_pool, v_pool, num_blocks, slots, slot_stride, num_tokens,
                              block_size, R, blockIdx.x, blockIdx.y * 16);
}

// Several colocated models' cache writes of one step in one grid: the kernel
// argument carries one descriptor per model, a workgroup finds its model from
// the models' first workgroup ids and then does what the single-model kernel
// does (heads fastest within a model).
struct CacheWriteItemDev {
  uint16_t *k;
  const uint16_t *v;
  int64_t row_stride;
  const int64_t *slots;          // layer slice of the model's slot mapping
  int64_t slot_stride;
  RopeArgs rope;
  int32_t num_tokens;
  int32_t num_kv_heads;
  int32_t work_begin;            // first workgroup of this model
};
struct MultiCacheWriteParams {
  CacheWriteItemDev it[MUXA_MAX_DECODE_ITEMS];
  uint4 *k_pool;
  uint16_t *v_pool;
  int64_t num_blocks;
  int32_t n_items;
  int32_t block_size;
};

template <typename T, bool ROPE>
__global__ __launch_bounds__(256) void multi_reshape_and_cache_kernel(const MultiCacheWriteParams P) {
  const int w = blockIdx.x;
  int ii = 0;
#pragma unroll
  for (int i = 1; i < MUXA_MAX_DECODE_ITEMS; ++i)
    if (i < P.n_items && w >= P.it[i].work_begin) ii = i;
  const CacheWriteItemDev I = P.it[ii];
  const int local = w - I.work_begin;
  const int ty = local / I.num_kv_heads;
  const int h = local - ty * I.num_kv_heads;
  cache_write_window<T, ROPE>(I.k, I.v, I.row_stride, P.k_pool, P.v_pool, P.num_blocks, I.slots, I.slot_stride,
                              I.num_tokens, P.block_size, I.rope, h, ty * 16);
}

}  // namespace mux

namespace mux {
namespace {

int32_t check_cache_write(const void *k, const void *v, int64_t kv_row_stride, const void *k_pool,
                          const void *v_pool, int64_t num_pool_blocks, const int64_t *slot_mapping, int32_t layer,
                          int32_t num_layers, int32_t num_tokens, int32_t num_kv_heads, int32_t head_size,
                          int32_t block_size, int32_t dtype) {
  // (pointers are only required when there is something to do)
  if (num_tokens > 0 && (!k || !v || !k_pool || !v_pool || !slot_mapping)) return MUXA_EINVAL;
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
  if (num_tokens > 16 * 65535) return MUXA_EUNSUPPORTED;      // one grid row per 16 tokens
  if (num_pool_blocks > (int64_t{1} << 56)) return MUXA_EINVAL;   // slot arithmetic stays in 64 bits
  return MUXA_OK;
}

}  // namespace
}  // namespace mux

extern "C" int32_t mux_reshape_and_cache(const void *k, const void *v, int64_t kv_row_stride,
                                         void *k_pool, void *v_pool, int64_t num_pool_blocks,
                                         const int64_t *slot_mapping, int32_t layer, int32_t num_layers,
                                         int32_t num_tokens, int32_t num_kv_heads, int32_t head_size,
                                         int32_t block_size, int32_t dtype, void *stream) {
  using namespace mux;
  const int32_t rc = check_cache_write(k, v, kv_row_stride, k_pool, v_pool, num_pool_blocks, slot_mapping, layer,
                                       num_layers, num_tokens, num_kv_heads, head_size, block_size, dtype);
  if (rc != MUXA_OK) return rc;
  if (num_tokens == 0) return MUXA_OK;
  const int64_t slot_stride = static_cast<int64_t>(num_layers) * num_kv_heads;
  const int64_t *slots = slot_mapping + static_cast<int64_t>(layer) * num_kv_heads;
  dim3 grid(num_kv_heads, (num_tokens + 15) / 16);
  // Without the rotary part the kernel only moves bytes and never writes k.
  hipLaunchKernelGGL((reshape_and_cache_kernel<F16, false>), grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                     const_cast<uint16_t *>(static_cast<const uint16_t *>(k)), static_cast<const uint16_t *>(v),
                     kv_row_stride, static_cast<uint4 *>(k_pool), static_cast<uint16_t *>(v_pool), num_pool_blocks,
                     slots, slot_stride, num_tokens, block_size, RopeArgs{});
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e);
  return MUXA_OK;
}

extern "C" int32_t mux_rope_reshape_and_cache(const int64_t *positions, void *q, int64_t q_row_stride, void *k,
                                              const void *v, int64_t kv_row_stride, const float *cos_sin,
                                              int32_t max_position, int32_t rotary_dim, void *k_pool, void *v_pool,
                                              int64_t num_pool_blocks, const int64_t *slot_mapping, int32_t layer,
                                              int32_t num_layers, int32_t num_tokens, int32_t num_q_heads,
                                              int32_t num_kv_heads, int32_t head_size, int32_t block_size,
                                              int32_t dtype, void *stream) {
  using namespace mux;
  const int32_t rc = check_cache_write(k, v, kv_row_stride, k_pool, v_pool, num_pool_blocks, slot_mapping, layer,
                                       num_layers, num_tokens, num_kv_heads, head_size, block_size, dtype);
  if (rc != MUXA_OK) return rc;
  if ((num_tokens > 0 && (!positions || !cos_sin)) || max_position <= 0) return MUXA_EINVAL;
  if (rotary_dim != kHeadSize) return MUXA_EUNSUPPORTED;   // partial rotation: use mux_rotary_neox + mux_reshape_and_cache
  if (q != nullptr) {
    if (num_q_heads <= 0 || num_q_heads % num_kv_heads != 0) return MUXA_EINVAL;
    if (q_row_stride < static_cast<int64_t>(num_q_heads) * kHeadSize || q_row_stride % 8 != 0) return MUXA_EINVAL;
    if (reinterpret_cast<uintptr_t>(q) & 15u) return MUXA_EINVAL;
  }
  if (num_tokens == 0) return MUXA_OK;
  const int64_t slot_stride = static_cast<int64_t>(num_layers) * num_kv_heads;
  const int64_t *slots = slot_mapping + static_cast<int64_t>(layer) * num_kv_heads;
  RopeArgs R;
  R.q = static_cast<uint16_t *>(q);
  R.q_stride = q_row_stride;
  R.ratio = q ? num_q_heads / num_kv_heads : 0;
  R.positions = positions;
  R.cos_sin = cos_sin;
  R.max_position = max_position;
  dim3 grid(num_kv_heads, (num_tokens + 15) / 16);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == MUXA_DTYPE_F16)
    hipLaunchKernelGGL((reshape_and_cache_kernel<F16, true>), grid, dim3(256), 0, st, static_cast<uint16_t *>(k),
                       static_cast<const uint16_t *>(v), kv_row_stride, static_cast<uint4 *>(k_pool),
                       static_cast<uint16_t *>(v_pool), num_pool_blocks, slots, slot_stride, num_tokens, block_size, R);
  else
    hipLaunchKernelGGL((reshape_and_cache_kernel<BF16, true>), grid, dim3(256), 0, st, static_cast<uint16_t *>(k),
                       static_cast<const uint16_t *>(v), kv_row_stride, static_cast<uint4 *>(k_pool),
                       static_cast<uint16_t *>(v_pool), num_pool_blocks, slots, slot_stride, num_tokens, block_size, R);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e);
  return MUXA_OK;
}

extern "C" int32_t mux_multi_rope_reshape_and_cache(const MuxCacheWriteItem *items, int32_t n_items, void *k_pool,
                                                    void *v_pool, int64_t num_pool_blocks, int32_t head_size,
                                                    int32_t block_size, int32_t dtype, void *stream) {
  using namespace mux;
  if (!items || n_items <= 0 || n_items > MUXA_MAX_DECODE_ITEMS) return MUXA_EINVAL;
  MultiCacheWriteParams P = {};
  P.k_pool = static_cast<uint4 *>(k_pool);
  P.v_pool = static_cast<uint16_t *>(v_pool);
  P.num_blocks = num_pool_blocks;
  P.block_size = block_size;
  // Either every model of the call that has tokens rotates (positions given) or none does.
  bool rope = false;
  for (int i = 0; i < n_items; ++i)
    if (items[i].num_tokens > 0) {
      rope = items[i].positions != nullptr;
      break;
    }
  int64_t work = 0;
  for (int i = 0; i < n_items; ++i) {
    const MuxCacheWriteItem &it = items[i];
    const int32_t rc = check_cache_write(it.k, it.v, it.kv_row_stride, k_pool, v_pool, num_pool_blocks,
                                         it.slot_mapping, it.layer, it.num_layers, it.num_tokens, it.num_kv_heads,
                                         head_size, block_size, dtype);
    if (rc != MUXA_OK) return rc;
    if (it.num_tokens > 0 && (it.positions != nullptr) != rope) return MUXA_EINVAL;
    RopeArgs R{};
    if (rope && it.num_tokens > 0) {
      if ((it.num_tokens > 0 && !it.cos_sin) || it.max_position <= 0) return MUXA_EINVAL;
      if (it.rotary_dim != kHeadSize) return MUXA_EUNSUPPORTED;
      if (it.q != nullptr) {
        if (it.num_q_heads <= 0 || it.num_q_heads % it.num_kv_heads != 0) return MUXA_EINVAL;
        if (it.q_row_stride < static_cast<int64_t>(it.num_q_heads) * kHeadSize || it.q_row_stride % 8 != 0)
          return MUXA_EINVAL;
        if (reinterpret_cast<uintptr_t>(it.q) & 15u) return MUXA_EINVAL;
      }
      R.q = static_cast<uint16_t *>(it.q);
      R.q_stride = it.q_row_stride;
      R.ratio = it.q ? it.num_q_heads / it.num_kv_heads : 0;
      R.positions = it.positions;
      R.cos_sin = it.cos_sin;
      R.max_position = it.max_position;
    }
    if (it.num_tokens == 0) continue;
    CacheWriteItemDev &d = P.it[P.n_items++];
    d.k = static_cast<uint16_t *>(it.k);
    d.v = static_cast<const uint16_t *>(it.v);
    d.row_stride = it.kv_row_stride;
    d.slots = it.slot_mapping + static_cast<int64_t>(it.layer) * it.num_kv_heads;
    d.slot_stride = static_cast<int64_t>(it.num_layers) * it.num_kv_heads;
    d.rope = R;
    d.num_tokens = it.num_tokens;
    d.num_kv_heads = it.num_kv_heads;
    d.work_begin = static_cast<int32_t>(work);
    work += static_cast<int64_t>((it.num_tokens + 15) / 16) * it.num_kv_heads;
    if (work > 0x7fffffff) return MUXA_EUNSUPPORTED;
  }
  if (P.n_items == 0) return MUXA_OK;
  const dim3 grid(static_cast<unsigned>(work));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!rope)
    hipLaunchKernelGGL((multi_reshape_and_cache_kernel<F16, false>), grid, dim3(256), 0, st, P);
  else if (dtype == MUXA_DTYPE_F16)
    hipLaunchKernelGGL((multi_reshape_and_cache_kernel<F16, true>), grid, dim3(256), 0, st, P);
  else
    hipLaunchKernelGGL((multi_reshape_and_cache_kernel<BF16, true>), grid, dim3(256), 0, st, P);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e);
  return MUXA_OK;
}
