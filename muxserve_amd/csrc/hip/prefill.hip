// Causal prefill attention on the fresh q, k, v of a batch of packed prompts,
// gfx950 MFMA (v_mfma_f32_32x32x16_{f16,bf16}).
//
// One workgroup = 128 query rows of one head of one prompt, 4 waves x 32 rows.
// Keys/values stream through LDS in tiles of 32 tokens shared by the 4 waves
// (32 rather than 64: 160 VGPRs and 34 KB of LDS let three workgroups share a
// CU instead of two, and the causal edge is cut at 32 keys; measured 8 %
// faster on ragged short prompts, 1 - 3 % on 2048-token prompts).
// Each wave keeps the TRANSPOSED problem so that probabilities never leave
// registers:
//     S^T[key][q] = K . Q^T      A = K tile   (LDS, row-major, 16-byte frags)
//                                B = Q^T      (registers, loaded once)
//     O^T[d][q]  += V^T . P^T    A = V^T      (the row-major V tile in LDS, read
//                                              with the transposing LDS read)
//                                B = P^T      = the S^T accumulators, converted
// In the 32x32 accumulator layout a lane owns ONE query column (q = lane%32)
// and 16 of the 32 keys of a block, so softmax statistics are per-lane scalars
// (one exchange with lane^32), the rescale of O^T is a per-lane multiply, and
// the accumulator registers of S^T are, in order, exactly the 8-element
// B-operand fragments of the P.V products - provided the V^T fragments use the
// same key order (two groups of four keys), which costs nothing because V^T is
// read from LDS anyway.
// The next tile's global loads are issued before the current tile's math.
#include "mux_common.h"

#include <algorithm>
#include <vector>

namespace mux {

typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf16 __attribute__((ext_vector_type(8)));
typedef float v16f32 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kBM = 128;                 // query rows per workgroup
constexpr int kBN = 32;                  // keys per tile
constexpr int kNKB = kBN / 32;           // 32-key blocks (one MFMA row block) per tile

// Query tiles listed in the kernel argument (its size limit is 4 KiB).
constexpr int kMaxPairs = 768;

// Tracing build (-DMUX_TRACE, libmuxattn_trace.so; never the shipped library):
// thread 0 of every workgroup that has work stamps the 100 MHz clock into a
// caller-provided table, 8 int64 per workgroup: [0] entry, [1] the prompt's
// place and length known, [2] first key tile landed and the workgroup met (end
// of the prologue), [3] last key tile done, [4] output stores issued (a wave
// does not wait for them before it ends, and neither does the stamp), [5] key
// tiles of the workgroup, [6] prompt length, [7] first query row.
#ifdef MUX_TRACE
__device__ long long *g_prefill_trace = nullptr;
__device__ long long g_prefill_trace_rows = 0;
#endif

union Frag {
  u32x4 u;
  v8f16 h;
  v8bf16 b;
};

template <typename T>
__device__ __forceinline__ v16f32 mfma(const Frag &a, const Frag &b, v16f32 c) {
  if constexpr (__is_same(T, F16)) return __builtin_amdgcn_mfma_f32_32x32x16_f16(a.h, b.h, c, 0, 0, 0);
  else return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.b, b.b, c, 0, 0, 0);
}

// Two fp32 -> one packed pair in storage type T, round to nearest even
// (one v_cvt_pk_f16_f32 / v_cvt_pk_bf16_f32).
typedef float float2_t __attribute__((ext_vector_type(2)));
template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  const float2_t x = {lo, hi};
  if constexpr (__is_same(T, F16)) {
    union { half2_t h; uint32_t u; } c;
    c.h = __builtin_convertvector(x, half2_t);
    return c.u;
  } else {
    union { bf162_t h; uint32_t u; } c;
    c.h = __builtin_convertvector(x, bf162_t);
    return c.u;
  }
}

// One model's prompts (several colocated models can share a launch).
struct PrefillItemDev {
  uint16_t *out;
  const uint16_t *q, *k, *v;
  int64_t out_stride, q_stride, kv_stride;
  const int32_t *cu_seqlens;
  int32_t ratio;          // query heads per kv head
  int32_t num_kv_heads;
  int32_t num_prompts;
  int32_t kv_per_xcd;     // ceil(num_kv_heads / 8)
  float scale_log2;
  int32_t out_rows_16b;   // out and its row stride allow 16-byte stores
};

struct PrefillParams {
  PrefillItemDev it[MUXA_MAX_DECODE_ITEMS];
  const int32_t *prompt_order;   // dense grid, optional: prompts in the order their workgroups should start
  int32_t q_tiles;        // dense grid: 128-row query tiles per prompt (of the longest prompt)
  int32_t num_groups;     // dense grid: (prompt, kv head) pairs
  // Compact grid (the caller gave the prompt lengths on the host): the query
  // tiles that exist, the heaviest of all models first, as
  // model << 28 | prompt << 12 | tile; every pair takes slots_per_pair workgroups
  // on each XCD (the largest model's kv heads per XCD x query heads per kv head;
  // the surplus of smaller models leaves at once).  0 pairs = dense grid, one model.
  int32_t n_pairs;
  int32_t slots_per_pair;
  uint32_t pairs[kMaxPairs];
};
static_assert(sizeof(PrefillParams) <= 4096, "kernel argument segment");
constexpr int kPairTileBits = 12;       // tile in bits 0-11, prompt in bits 12-27, model in bits 28-30

// K and V tiles go from global memory straight into LDS
// (global_load_lds_dwordx4: lane l's 16 bytes land at base + 16 l), row-major
// [key][128 dims] with the 16-byte chunks of a row XOR-swizzled by the row
// number so that fragment reads spread over the banks; V^T fragments come out of
// the row-major tile with the transposing read ds_read_b64_tr_b16.  No staging
// registers, no LDS stores, no byte permutes; two tile buffers per operand, one
// barrier per tile.
typedef short v4i16 __attribute__((ext_vector_type(4)));
// A wave raises its issue priority while it feeds the matrix cores and drops
// it for the softmax, so that of the two waves of a SIMD the one in its MFMA
// phase goes first (1 - 5 % on prompts of 1024 - 2048 tokens).
#define MUX_PF_PRIO(x) __builtin_amdgcn_s_setprio(x)
#define MUX_PF_PRIO_MFMA 1
#define MUX_PF_PRIO_VALU 0
constexpr int kTileElems = kBN * kHeadSize;          // one unpadded row-major tile
// The swizzle: the 16-byte chunk c of tile row r sits at chunk position
// c ^ swz(r), swz(r) = the low three bits of r rotated left by one, bit 3 kept.
// LDS has 32 banks of 4 bytes: a 256-byte row covers them twice, so only the low
// three bits of a chunk position choose the banks.  The K fragments are read 8
// rows at a time (one chunk each, ds_read_b128): the rotated low bits of 8
// consecutive rows are all different.  The V^T fragments are read 16 lanes at a
// time (ds_read_b64_tr_b16) over 4 consecutive rows x 2 neighbouring chunks x
// the two halves of a chunk: the rows' two low bits land in position bits 1-2
// and the chunk pair in bit 0 - again all different.  (With the plain c ^ r the
// four rows and the chunk pair shared two position bits: a two-way conflict on
// every V^T read.)
__device__ __forceinline__ int swz(int row) { return ((row & 3) << 1) | ((row >> 2) & 1) | (row & 8); }

template <typename T>
__global__ __launch_bounds__(256, 3) void prefill_causal_kernel(const PrefillParams P) {
  constexpr int D = kHeadSize;
  // K[2], V[2] tile buffers.  The epilogue reuses the memory for the output rows
  // (4 waves x 32 rows of 272 bytes), which is the larger of the two.
  constexpr int kSmemElems = 4 * kTileElems > 4 * 32 * (D + 8) ? 4 * kTileElems : 4 * 32 * (D + 8);
  __shared__ __attribute__((aligned(16))) uint16_t smem[kSmemElems];

#ifdef MUX_TRACE
  const long long tr_entry = __builtin_amdgcn_s_memrealtime();
  long long tr_first = 0;
  long long *const tr_table = g_prefill_trace;   // read here, so that the write at the end waits for nothing
  const long long tr_rows = g_prefill_trace_rows;
#endif
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Workgroups are dealt to the 8 XCDs round-robin by id, and each XCD has its
  // own L2.  All workgroups that read the same K/V - the query tiles and query
  // heads of one (prompt, kv head) pair - are therefore given ids that are equal
  // mod 8.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  int item = 0, prompt, hk, hq, q0, rem = 0;
  uint32_t pair = 0;
  if (P.n_pairs > 0) {
    // Compact grid: only query tiles that exist, the heaviest of the whole launch first.
    const int pi = slot / P.slots_per_pair;
    if (pi >= P.n_pairs) return;
    rem = slot - pi * P.slots_per_pair;
    pair = P.pairs[pi];
    item = min(static_cast<int>(pair >> 28), MUXA_MAX_DECODE_ITEMS - 1);
  }
  const PrefillItemDev I = P.it[item];
  if (P.n_pairs > 0) {
    // kv head hk of prompt p lives on XCD (hk + p) % 8 (rotated by the prompt so
    // that head counts that are no multiple of 8 load the XCDs evenly).
    if (rem >= I.kv_per_xcd * I.ratio) return;
    // (clamped: a malformed list costs results, never a stray read)
    prompt = min(static_cast<int>((pair >> kPairTileBits) & 0xffffu), I.num_prompts - 1);
    q0 = static_cast<int>(pair & ((1u << kPairTileBits) - 1)) * kBM;
    hk = ((xcd - prompt) & 7) + 8 * (rem / I.ratio);
    if (hk >= I.num_kv_heads) return;
    hq = hk * I.ratio + rem % I.ratio;
  } else {
    // Dense grid: every prompt gets the tiles of the longest one, heaviest first;
    // (prompt, kv head) groups go round-robin over the XCDs.
    const int per_group = I.ratio * P.q_tiles;
    const int group = (slot / per_group) * 8 + xcd;
    if (group >= P.num_groups) return;
    const int in_group = slot % per_group;
    const int prompt_rank = group / I.num_kv_heads;
    // (an entry outside the batch is clamped, as above)
    prompt = P.prompt_order ? min(max(P.prompt_order[prompt_rank], 0), I.num_prompts - 1) : prompt_rank;
    hk = group % I.num_kv_heads;
    hq = hk * I.ratio + in_group / P.q_tiles;
    q0 = (P.q_tiles - 1 - in_group % P.q_tiles) * kBM;
  }
  const int seq_begin = I.cu_seqlens[prompt];
  const int len = I.cu_seqlens[prompt + 1] - seq_begin;
  if (q0 >= len) return;
#ifdef MUX_TRACE
  asm volatile("s_nop 0" ::"s"(len));    // (the stamp waits for the loads of the two offsets)
  const long long tr_len = __builtin_amdgcn_s_memrealtime();
#endif

  const int qcol = lane & 31;            // this lane's query column / fragment row
  const int half = lane >> 5;            // which 8 of a fragment's 16 k-slots
  const int wq0 = q0 + wave * 32;        // first query row of this wave
  const int my_q = wq0 + qcol;           // this lane's query position inside the prompt

  // ---- Q^T fragments: Q[my_q][16 s + 8 half .. +7], s = 0..7 ------------------------
  Frag qf[8];
  {
    const bool ok = my_q < len;
    const uint16_t *qp = I.q + static_cast<int64_t>(seq_begin + (ok ? my_q : 0)) * I.q_stride + hq * D + 8 * half;
#pragma unroll
    for (int s = 0; s < 8; ++s) qf[s].u = ok ? *reinterpret_cast<const u32x4 *>(qp + 16 * s) : u32x4{0, 0, 0, 0};
  }

  v16f32 oacc[4];                        // O^T[d = 32 mb + ...][q]
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[mb][i] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // Keys needed by this workgroup: positions 0 .. min(len, q0 + 128) - 1.
  const int kv_end = min(len, q0 + kBM);
  const int n_tiles = (kv_end + kBN - 1) / kBN;

  // ---- tile staging -------------------------------------------------------------------
  const uint32_t row_bytes = static_cast<uint32_t>(I.kv_stride) * 2u;
  const char *kbase = reinterpret_cast<const char *>(I.k + static_cast<int64_t>(seq_begin) * I.kv_stride + hk * D);
  const char *vbase = reinterpret_cast<const char *>(I.v + static_cast<int64_t>(seq_begin) * I.kv_stride + hk * D);
  const uint32_t tile_bytes = kBN * row_bytes;
  const uint32_t last_row = static_cast<uint32_t>(len - 1) * row_bytes;
  // Rows past the prompt re-read its last row: finite data whose probability is
  // exactly 0 (such a key is in the future of every valid query).

  // Instruction i of wave w fills KiB 4 i + w of a tile = rows 16 i + 4 w .. +3;
  // lane l sits at row 16 i + 4 w + l/16, position l%16, and fetches chunk
  // position ^ swz(row) - the same chunk for every i (rows 16 apart swizzle alike).
  constexpr int kLoads = kBN / 16;         // such instructions per wave, tile and operand
  uint32_t koff[kLoads];
  const int row0 = 4 * wave + (lane >> 4);
  const int chunk0 = (lane & 15) ^ swz(row0);
#pragma unroll
  for (int i = 0; i < kLoads; ++i) koff[i] = static_cast<uint32_t>(row0 + 16 * i) * row_bytes + 16u * chunk0;
  const uint32_t kmax = last_row + 16u * chunk0;
  auto dma_tile = [&](int buf) {           // the next tile in sequence into buffer buf
    typedef __attribute__((address_space(3))) void lds_void;
    typedef const __attribute__((address_space(1))) void global_void;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const uint32_t o = min(koff[i], kmax);
      uint16_t *kd = smem + buf * kTileElems + (4 * i + wave) * 512;
      uint16_t *vd = smem + (2 + buf) * kTileElems + (4 * i + wave) * 512;
      // (address-space casts need the C form)
      __builtin_amdgcn_global_load_lds((global_void *)(kbase + o), (lds_void *)kd, 16, 0, 0);
      __builtin_amdgcn_global_load_lds((global_void *)(vbase + o), (lds_void *)vd, 16, 0, 0);
      koff[i] += tile_bytes;
    }
  };

  // Lane-dependent part of the V^T fragment addresses (see read_v), in elements.
  int v_lane_base[2];
  {
    const int jrow = (lane & 15) >> 2, m = lane & 3;
    const int rl = 4 * half + jrow, cl = 2 * ((lane >> 4) & 1) + (m >> 1);
    // rl < 8, cl < 4: the lane's part of the position is cl ^ swz(rl), below 8.
    v_lane_base[0] = rl * D + 8 * (cl ^ swz(rl)) + 4 * (m & 1);
    v_lane_base[1] = rl * D + 8 * (cl ^ swz(rl) ^ 4) + 4 * (m & 1);
  }
  dma_tile(0);
  for (int t = 0; t < n_tiles; ++t) {
    const int k0 = t * kBN;
    const int cur = t & 1;
    // This wave's part of tile t has landed; after the barrier all of it has,
    // and everybody is done with the other buffer.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#ifdef MUX_TRACE
    if (t == 0) tr_first = __builtin_amdgcn_s_memrealtime();
#endif
    if (t + 1 < n_tiles) dma_tile(cur ^ 1);
    // Nothing to compute: every key of the tile is in this wave's future, or all
    // of the wave's rows are past the prompt's end.
    if (k0 > wq0 + 31 || wq0 >= len) continue;
    const uint16_t *const Kt = smem + cur * kTileElems;           // this tile's K
    const uint16_t *const Vr = smem + (2 + cur) * kTileElems;     // this tile's V (row-major)

    // ---- S^T = K . Q^T : kNKB 32-key blocks -----------------------------------------
    // LDS fragment reads run kDepth steps ahead of the MFMAs that consume them.
    // In the P.V product consecutive MFMAs go to different accumulators (4 dim
    // blocks); a single dependent chain, as here with one key block, runs at 3/4
    // of the rate.
    constexpr int kDepth = 4;
    v16f32 sacc[kNKB];
#pragma unroll
    for (int kb = 0; kb < kNKB; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[kb][i] = 0.f;
    {
      // Fragment j: key block j % kNKB, dims 16 (j / kNKB) + 8 half .. +7 of key row qcol.
      auto read_k = [&](int j) {
        Frag f;
        const int row = 32 * (j % kNKB) + qcol, chunk = 2 * (j / kNKB) + half;
        f.u = *reinterpret_cast<const u32x4 *>(Kt + row * D + 8 * (chunk ^ swz(row)));
        return f;
      };
      Frag ring[kDepth];
#pragma unroll
      for (int j = 0; j < kDepth; ++j) ring[j] = read_k(j);
      __builtin_amdgcn_sched_barrier(0);   // keep the scheduler from sinking the reads to their uses
      MUX_PF_PRIO(MUX_PF_PRIO_MFMA);
#pragma unroll
      for (int j = 0; j < 8 * kNKB; ++j) {
        sacc[j % kNKB] = mfma<T>(ring[j % kDepth], qf[j / kNKB], sacc[j % kNKB]);
        if (j + kDepth < 8 * kNKB) ring[j % kDepth] = read_k(j + kDepth);
        __builtin_amdgcn_sched_barrier(0);
      }
      MUX_PF_PRIO(MUX_PF_PRIO_VALU);
    }

    // ---- softmax over keys, per query column --------------------------------------
    // register i of block kb is key k0 + 32 kb + 8 (i/4) + 4 half + i%4.
    // Raw scores stay unscaled; scale (> 0) is folded into the exponent:
    // p = exp2(s * scale_log2 - m * scale_log2).
    // Exactly one tile per wave straddles the diagonal; only it pays for the mask.
    if (k0 + kBN - 1 > wq0) {
      const int rel = my_q - k0 - 4 * half;   // key offset inside the tile, less this lane's share
#pragma unroll
      for (int kb = 0; kb < kNKB; ++kb)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (32 * kb + 8 * (i / 4) + (i % 4) > rel) sacc[kb][i] = -INFINITY;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < kNKB; ++kb)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, sacc[kb][i]);
    mx = max_with_lane_xor32(mx);
    // The reference of the exponents (m_run) only moves when some row's maximum has
    // risen more than kRescaleStep (in the exponent's units) above it - and on the
    // wave's first tile, to that tile's maximum: probabilities then reach
    // 2^kRescaleStep at most, and the 64 accumulators and the running sum are
    // rescaled rarely instead of whenever a maximum rises at all (with 32 rows per
    // wave, that is in most tiles of a prompt's first hundreds of keys).
    constexpr float kRescaleStep = 8.f;
    const bool move = m_run == -INFINITY ? mx != -INFINITY : (mx - m_run) * I.scale_log2 > kRescaleStep;
    if (__builtin_amdgcn_ballot_w64(move) != 0) {
      const float m_new = fmaxf(m_run, mx);
      // Rows past the prompt may have no valid key at all; keep them finite.
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = fast_exp2((m_run - m_use) * I.scale_log2);
      l_run *= alpha;
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[mb][i] *= alpha;
      m_run = m_use;
    }
    // (a row that has not seen a valid key yet keeps a finite reference)
    const float neg_m = m_run == -INFINITY ? 0.f : -m_run * I.scale_log2;
    float psum = 0.f;
    Frag pf[2 * kNKB];                          // B fragments: [kb][step] -> index 2 kb + st
    // bf16 keeps only 8 mantissa bits of a probability, which alone would cost
    // more than the 2e-3 budget, so bf16 P is carried as hi + lo parts.
    constexpr bool kSplitP = __is_same(T, BF16);
    Frag pf_lo[kSplitP ? 2 * kNKB : 1];
#pragma unroll
    for (int kb = 0; kb < kNKB; ++kb) {
      float p[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) p[i] = fast_exp2(__builtin_fmaf(sacc[kb][i], I.scale_log2, neg_m));
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = pack2<T>(p[8 * st + 2 * j], p[8 * st + 2 * j + 1]);
        pf[2 * kb + st].u = u32x4{w[0], w[1], w[2], w[3]};
        if constexpr (kSplitP) {
          // The part of p that its bf16 rounding lost, as a second bf16.
          uint32_t lo[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            lo[j] = pack2<T>(p[8 * st + 2 * j] - bf16_lo(w[j]), p[8 * st + 2 * j + 1] - bf16_hi(w[j]));
            psum += p[8 * st + 2 * j] + p[8 * st + 2 * j + 1];
          }
          pf_lo[2 * kb + st].u = u32x4{lo[0], lo[1], lo[2], lo[3]};
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) psum += p[8 * st + j];
        }
      }
    }
    l_run += psum;

    // ---- O^T += V^T . P^T ---------------------------------------------------------------
    // k-slot j of lane half h in step (kb, st) is key 32 kb + 16 st + 8 (j/4) + 4 h + j%4
    {
      auto read_v = [&](int n) {         // fragment n = 4 ks + mb
        const int mb = n % 4, ks = n / 4;
        Frag f;
        // The transposing read works on groups of 16 lanes: lane 4 j + m of a
        // group points at dims 4 m .. 4 m + 3 of key row j, and lane i of the
        // group receives dim i of rows 0..3.  Here a group covers dims
        // 32 mb + 16 (lane/16 % 2) .. +15 and keys 16 ks + 4 half (+ 8) .. +3.
        // Address: row = 16 ks + 8 hsel + rl with rl = 4 half + jrow, chunk =
        // 4 mb + cl, position = chunk ^ swz(row) = (cl ^ swz(rl)) ^ 4 (mb ^ 2 hsel).
        // The lane part cl ^ rl is below 8, so bit 3 of the constant part adds
        // and only its bit 2 (mb odd) has to be folded into the lane's base:
        // two bases per lane, everything else is an immediate offset.
        typedef __attribute__((address_space(3))) v4i16 lds_v4i16;
        u32x2 part[2];
#pragma unroll
        for (int hsel = 0; hsel < 2; ++hsel) {
          const uint16_t *src = Vr + v_lane_base[mb & 1] + (16 * ks + 8 * hsel) * D + 64 * (((mb >> 1) ^ hsel) & 1);
          const v4i16 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16 *)src);
          union { v4i16 v; u32x2 u; } c;
          c.v = r;
          part[hsel] = c.u;
        }
        f.u = u32x4{part[0].x, part[0].y, part[1].x, part[1].y};
        return f;
      };
      Frag ring[kDepth];
#pragma unroll
      for (int j = 0; j < kDepth; ++j) ring[j] = read_v(j);
      __builtin_amdgcn_sched_barrier(0);
      MUX_PF_PRIO(MUX_PF_PRIO_MFMA);
#pragma unroll
      for (int j = 0; j < 8 * kNKB; ++j) {
        oacc[j % 4] = mfma<T>(ring[j % kDepth], pf[j / 4], oacc[j % 4]);
        if constexpr (kSplitP) oacc[j % 4] = mfma<T>(ring[j % kDepth], pf_lo[j / 4], oacc[j % 4]);
        if (j + kDepth < 8 * kNKB) ring[j % kDepth] = read_v(j + kDepth);
        __builtin_amdgcn_sched_barrier(0);
      }
      MUX_PF_PRIO(MUX_PF_PRIO_VALU);
    }
  }

#ifdef MUX_TRACE
  const long long tr_loop = __builtin_amdgcn_s_memrealtime();
#endif
  // ---- normalise and store: register i of block mb is d = 32 mb + 8 (i/4) + 4 half + i%4 ------
  const float l_tot = sum_with_lane_xor32(l_run);
  const float inv = 1.f / l_tot;
  if (I.out_rows_16b) {
    // Through LDS, so that the rows go out as whole 256-byte runs (16 bytes per
    // lane, four rows per instruction) instead of 8-byte pieces of 32 rows: the
    // tile buffers are free once every wave has left the loop.
    constexpr int kORow = D + 8;         // 272-byte rows
    static_assert(4 * 32 * kORow <= kSmemElems, "output staging fits the tile buffers");
    __syncthreads();
    uint16_t *stage = smem + wave * 32 * kORow;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<u32x2 *>(&stage[qcol * kORow + 32 * mb + 8 * g + 4 * half]) =
            u32x2{pack2<T>(oacc[mb][4 * g] * inv, oacc[mb][4 * g + 1] * inv),
                  pack2<T>(oacc[mb][4 * g + 2] * inv, oacc[mb][4 * g + 3] * inv)};
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int chunk = lane & 15;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int r = 4 * it + (lane >> 4);
      if (wq0 + r < len) {
        const u32x4 x = *reinterpret_cast<const u32x4 *>(&stage[r * kORow + 8 * chunk]);
        *reinterpret_cast<u32x4 *>(I.out + static_cast<int64_t>(seq_begin + wq0 + r) * I.out_stride + hq * D +
                                   8 * chunk) = x;
      }
    }
  } else if (my_q < len) {
    uint16_t *op = I.out + static_cast<int64_t>(seq_begin + my_q) * I.out_stride + hq * D + 4 * half;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const uint2 w2 = make_uint2(pack2<T>(oacc[mb][4 * g] * inv, oacc[mb][4 * g + 1] * inv),
                                    pack2<T>(oacc[mb][4 * g + 2] * inv, oacc[mb][4 * g + 3] * inv));
        *reinterpret_cast<uint2 *>(op + 32 * mb + 8 * g) = w2;
      }
  }
#ifdef MUX_TRACE
  if (tid == 0 && tr_table && blockIdx.x < tr_rows) {
    long long *row = tr_table + 8 * static_cast<long long>(blockIdx.x);
    row[0] = tr_entry, row[1] = tr_len, row[2] = tr_first, row[3] = tr_loop, row[4] = __builtin_amdgcn_s_memrealtime();
    row[5] = n_tiles, row[6] = len, row[7] = q0;
  }
#endif
}

}  // namespace mux

namespace mux {
namespace {

int32_t check_prefill_item(const MuxPrefillItem &it, int32_t head_size) {
  // (pointers are only required when there is something to do)
  const bool work = it.num_prompts > 0 && it.max_prompt_len > 0;
  if (work && (!it.out || !it.q || !it.k || !it.v || !it.cu_seqlens)) return MUXA_EINVAL;
  if (it.num_prompts < 0 || it.max_prompt_len < 0 || it.num_q_heads <= 0 || it.num_kv_heads <= 0) return MUXA_EINVAL;
  if (it.num_q_heads % it.num_kv_heads != 0) return MUXA_EINVAL;
  if (head_size != kHeadSize) return MUXA_EUNSUPPORTED;
  if (it.q_row_stride < static_cast<int64_t>(it.num_q_heads) * kHeadSize ||
      it.out_row_stride < static_cast<int64_t>(it.num_q_heads) * kHeadSize ||
      it.kv_row_stride < static_cast<int64_t>(it.num_kv_heads) * kHeadSize)
    return MUXA_EINVAL;
  // 16-byte fragment loads and 8-byte output stores.
  if (it.q_row_stride % 8 || it.kv_row_stride % 8 || it.out_row_stride % 4) return MUXA_EINVAL;
  const uintptr_t a16 =
      reinterpret_cast<uintptr_t>(it.q) | reinterpret_cast<uintptr_t>(it.k) | reinterpret_cast<uintptr_t>(it.v);
  if ((a16 & 15u) || (reinterpret_cast<uintptr_t>(it.out) & 7u)) return MUXA_EINVAL;
  // K/V rows of one prompt are addressed with 32-bit byte offsets.
  if (static_cast<int64_t>(it.max_prompt_len + kBM + 2 * kBN) * it.kv_row_stride * 2 >= (int64_t{1} << 32))
    return MUXA_EUNSUPPORTED;
  if (it.prompt_lens_host != nullptr)
    for (int p = 0; p < it.num_prompts; ++p)
      if (it.prompt_lens_host[p] < 0 || it.prompt_lens_host[p] > it.max_prompt_len) return MUXA_EINVAL;
  return MUXA_OK;
}

PrefillItemDev device_item(const MuxPrefillItem &it) {
  PrefillItemDev d;
  d.out = static_cast<uint16_t *>(it.out);
  d.q = static_cast<const uint16_t *>(it.q);
  d.k = static_cast<const uint16_t *>(it.k);
  d.v = static_cast<const uint16_t *>(it.v);
  d.out_stride = it.out_row_stride;
  d.q_stride = it.q_row_stride;
  d.kv_stride = it.kv_row_stride;
  d.cu_seqlens = it.cu_seqlens;
  d.ratio = it.num_q_heads / it.num_kv_heads;
  d.num_kv_heads = it.num_kv_heads;
  d.num_prompts = it.num_prompts;
  d.kv_per_xcd = (it.num_kv_heads + 7) / 8;
  d.scale_log2 = it.scale * 1.4426950408889634f;
  d.out_rows_16b = (reinterpret_cast<uintptr_t>(it.out) & 15u) == 0 && it.out_row_stride % 8 == 0;
  return d;
}

hipError_t launch_prefill(const PrefillParams &P, int64_t n_wg, int32_t dtype, hipStream_t st) {
  const dim3 grid(static_cast<uint32_t>(n_wg));
  if (dtype == MUXA_DTYPE_F16) hipLaunchKernelGGL((prefill_causal_kernel<F16>), grid, dim3(256), 0, st, P);
  else hipLaunchKernelGGL((prefill_causal_kernel<BF16>), grid, dim3(256), 0, st, P);
  return hipGetLastError();
}

// One model on the grid sized by its longest prompt (no host-side lengths, or too
// many query tiles for the kernel argument).
int32_t launch_dense(const MuxPrefillItem &it, const int32_t *prompt_order, int32_t dtype, hipStream_t st) {
  PrefillParams P = {};
  P.it[0] = device_item(it);
  P.prompt_order = prompt_order;
  P.q_tiles = (it.max_prompt_len + kBM - 1) / kBM;
  P.num_groups = it.num_prompts * it.num_kv_heads;
  const int64_t n_wg = static_cast<int64_t>((P.num_groups + 7) / 8) * 8 * P.it[0].ratio * P.q_tiles;
  if (n_wg > 0x7fffffff || P.q_tiles > 0xffff) return MUXA_EUNSUPPORTED;
  hipError_t e = launch_prefill(P, n_wg, dtype, st);
  if (e != hipSuccess) return hip_fail(e);
  return MUXA_OK;
}

// items[first .. first + n): one launch over the query tiles that exist, the
// heaviest (most keys) of all models first; false when they do not fit the
// kernel argument.
bool launch_compact(const MuxPrefillItem *items, int n, int32_t dtype, hipStream_t st, int32_t *rc) {
  PrefillParams P = {};
  int64_t total = 0;
  int max_tiles = 0, slots = 0, n_dev = 0;
  int dev_of[MUXA_MAX_DECODE_ITEMS];
  for (int i = 0; i < n; ++i) {
    const MuxPrefillItem &it = items[i];
    dev_of[i] = -1;
    if (it.num_prompts == 0 || it.max_prompt_len == 0) continue;
    if (it.prompt_lens_host == nullptr || it.num_prompts > 0xffff) return false;
    int64_t tiles = 0;
    for (int p = 0; p < it.num_prompts; ++p) tiles += (it.prompt_lens_host[p] + kBM - 1) / kBM;
    if (tiles == 0) continue;
    total += tiles;
    max_tiles = std::max(max_tiles, (it.max_prompt_len + kBM - 1) / kBM);
    dev_of[i] = n_dev;
    P.it[n_dev] = device_item(it);
    slots = std::max(slots, P.it[n_dev].kv_per_xcd * P.it[n_dev].ratio);
    ++n_dev;
  }
  *rc = MUXA_OK;
  if (total == 0) return true;
  if (total > kMaxPairs || max_tiles > (1 << kPairTileBits)) return false;
  // Order: prompt by prompt, the longest prompt of all models first, and within a
  // prompt the heaviest query tile (most keys) first.  The query tiles and query
  // heads that read the same K/V then run at the same time on one XCD and walk
  // the keys from the start together, so a K/V tile is fetched from memory once
  // and found in that XCD's L2 by the others (tile by tile over the whole batch
  // instead - every stream of the batch live at once - the 16 x 2048-token shape
  // re-read K/V from memory at 4.6 TB/s and ran 1.2 x slower), and the launch
  // ends with the short prompts' small tiles.
  struct Group {
    int item, prompt, len;
  };
  std::vector<Group> groups;
  for (int i = 0; i < n; ++i) {
    if (dev_of[i] < 0) continue;
    for (int p = 0; p < items[i].num_prompts; ++p)
      if (items[i].prompt_lens_host[p] > 0) groups.push_back({i, p, items[i].prompt_lens_host[p]});
  }
  std::stable_sort(groups.begin(), groups.end(), [](const Group &a, const Group &b) { return a.len > b.len; });
  int np = 0;
  for (const Group &g : groups)
    for (int t = (g.len + kBM - 1) / kBM - 1; t >= 0; --t)
      P.pairs[np++] = (static_cast<uint32_t>(dev_of[g.item]) << 28) |
                      (static_cast<uint32_t>(g.prompt) << kPairTileBits) | static_cast<uint32_t>(t);
  P.n_pairs = np;
  P.slots_per_pair = slots;
  const int64_t n_wg = static_cast<int64_t>(np) * slots * 8;
  if (n_wg > 0x7fffffff) {
    *rc = MUXA_EUNSUPPORTED;
    return true;
  }
  hipError_t e = launch_prefill(P, n_wg, dtype, st);
  if (e != hipSuccess) *rc = hip_fail(e);
  return true;
}

}  // namespace
}  // namespace mux

extern "C" int32_t mux_multi_prefill_causal(const MuxPrefillItem *items, int32_t n_items, int32_t head_size,
                                            int32_t dtype, void *stream) {
  using namespace mux;
  if (!items || n_items <= 0 || n_items > MUXA_MAX_DECODE_ITEMS) return MUXA_EINVAL;
  if (dtype != MUXA_DTYPE_F16 && dtype != MUXA_DTYPE_BF16) return MUXA_EUNSUPPORTED;
  for (int i = 0; i < n_items; ++i) {
    const int32_t rc = check_prefill_item(items[i], head_size);
    if (rc != MUXA_OK) return rc;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  int32_t rc = MUXA_OK;
  if (launch_compact(items, n_items, dtype, st, &rc)) return rc;
  // Not all in one kernel argument: one launch per model, compact where possible.
  for (int i = 0; i < n_items; ++i) {
    if (items[i].num_prompts == 0 || items[i].max_prompt_len == 0) continue;
    if (!launch_compact(items + i, 1, dtype, st, &rc)) rc = launch_dense(items[i], nullptr, dtype, st);
    if (rc != MUXA_OK) return rc;
  }
  return MUXA_OK;
}

extern "C" int32_t mux_prefill_causal(void *out, int64_t out_row_stride, const void *q, int64_t q_row_stride,
                                      const void *k, const void *v, int64_t kv_row_stride,
                                      const int32_t *cu_seqlens, const int32_t *prompt_order,
                                      const int32_t *prompt_lens_host, int32_t num_prompts,
                                      int32_t max_prompt_len, int32_t num_q_heads, int32_t num_kv_heads,
                                      int32_t head_size, float scale, int32_t dtype, void *stream) {
  using namespace mux;
  if (dtype != MUXA_DTYPE_F16 && dtype != MUXA_DTYPE_BF16) return MUXA_EUNSUPPORTED;
  MuxPrefillItem it = {};
  it.out = out;
  it.out_row_stride = out_row_stride;
  it.q = q;
  it.q_row_stride = q_row_stride;
  it.k = k;
  it.v = v;
  it.kv_row_stride = kv_row_stride;
  it.cu_seqlens = cu_seqlens;
  it.prompt_lens_host = prompt_lens_host;
  it.num_prompts = num_prompts;
  it.max_prompt_len = max_prompt_len;
  it.num_q_heads = num_q_heads;
  it.num_kv_heads = num_kv_heads;
  it.scale = scale;
  const int32_t rc0 = check_prefill_item(it, head_size);
  if (rc0 != MUXA_OK) return rc0;
  if (num_prompts == 0 || max_prompt_len == 0) return MUXA_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  int32_t rc = MUXA_OK;
  if (launch_compact(&it, 1, dtype, st, &rc)) return rc;
  return launch_dense(it, prompt_order, dtype, st);
}

#ifdef MUX_TRACE
// Tracing build only: where the prefill kernel's workgroups write their stamps
// (DEVICE int64 [rows, 8], zero-filled by the caller; NULL switches it off).
extern "C" int32_t mux_prefill_trace_set(void *table, int64_t rows) {
  long long *p = static_cast<long long *>(table);
  long long n = table ? rows : 0;
  MUX_HIP_TRY(hipMemcpyToSymbol(HIP_SYMBOL(mux::g_prefill_trace), &p, sizeof(p)));
  MUX_HIP_TRY(hipMemcpyToSymbol(HIP_SYMBOL(mux::g_prefill_trace_rows), &n, sizeof(n)));
  return MUXA_OK;
}
#endif
