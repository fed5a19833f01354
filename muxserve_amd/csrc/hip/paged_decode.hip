// Paged decode attention over the head-granular KV pool, gfx950.
//
// Work unit = (model, sequence, group of G query heads that share a kv head,
// partition of the context).  A workgroup of NW waves handles one unit at a
// time; wave w takes tiles w, w+NW, ... of 64 tokens:
//   * K: lane t owns token t of the tile.  Pool layout [D/8][BS][8] makes the
//     8 dims of one token a 16-byte chunk; 16 loads (one per d/8) bring the
//     token's whole key into 64 VGPRs, each load instruction reading whole
//     256-byte (BS=16) runs of the block.  q.k is then a private dot product
//     (v_dot2_f32_f16), no cross-lane traffic.
//   * softmax: running max via DPP row reductions + 4 readlanes, running sum
//     kept per lane and reduced once at the end.
//   * V: pool layout [D][BS] makes 8 consecutive tokens of one dim a 16-byte
//     chunk; lanes read consecutive chunks (1 KiB per instruction), the 64
//     probabilities of the tile are exchanged through 256 bytes of LDS and
//     each lane accumulates BS/4 output dims, partial over its 8 tokens; the
//     BS/8 partials per dim are summed once at the end with DPP.
// All 32 loads of a tile (16 KiB K + 16 KiB V per wave) are issued before the
// first use; the waves' partial results meet in LDS and wave 0 merges them.
//
// Contexts longer than `partition` tokens are split; each partition's partial
// (max, sum, unnormalised acc) goes to the workspace and the workgroup that
// arrives LAST for a (sequence, head group) - found with one atomic counter per
// group - combines them and writes the output, so a step is a single kernel.
// Sequences that fit one partition write their output directly.
//
// Units are enumerated compactly from the device-side context lengths (a
// wave-wide prefix sum), so the grid holds (almost) no empty workgroups; per
// model the split sequences come first and the sequences that need no combine
// last, which keeps the kernel's tail short.
//
// Several models (different head counts, tables, q/out tensors) are covered by
// one grid: the kernel argument carries up to MUXA_MAX_DECODE_ITEMS item
// descriptors.
#include "mux_common.h"

#include <algorithm>
#include <mutex>

namespace mux {

thread_local int32_t g_last_hip_error = 0;

// Tracing build (-DMUX_TRACE, libmuxattn_trace.so; never the shipped library):
// wave 0 of every workgroup of the vector-ALU decode kernel stamps the 100 MHz
// clock at the ends of its phases into a caller-provided table, 8 int64 per
// workgroup: [0] entry, [1] unit known, [2] block ids and q there, [3] K/V loads
// of the (last) tile issued, [4] tile consumed, [5] past the workgroup's barrier,
// [6] merge / publish / combine done, [7] tokens of the unit | split << 16.
// The matrix-core kernel of the grouped-query shapes stamps [0], [6] and [7] only.
#ifdef MUX_TRACE
__device__ long long *g_decode_trace = nullptr;
__device__ long long g_decode_trace_rows = 0;
#define MUX_TR(slot)                                                                         \
  do {                                                                                       \
    if (threadIdx.x == 0 && g_decode_trace && blockIdx.x < g_decode_trace_rows)              \
      g_decode_trace[blockIdx.x * 8 + (slot)] = __builtin_amdgcn_s_memrealtime();            \
  } while (0)
#define MUX_TRV(slot, v)                                                                     \
  do {                                                                                       \
    if (threadIdx.x == 0 && g_decode_trace && blockIdx.x < g_decode_trace_rows)              \
      g_decode_trace[blockIdx.x * 8 + (slot)] = (v);                                         \
  } while (0)
#else
#define MUX_TR(slot)
#define MUX_TRV(slot, v)
#endif

constexpr int kWavesPerGroup = 4;         // waves cooperating on one unit

struct DecodeItemDev {
  void *out;
  const void *q;
  int64_t out_stride, q_stride;   // elements per row
  const int32_t *tables;          // layer slice [B, Hkv, max_blocks]
  const int32_t *ctx;             // [B]
  float *ws_acc;                  // [B, Hq, max_splits, 128]
  float *ws_ml;                   // [B, Hq, max_splits, 2]  (running max in log2 units, sum)
  int32_t *counters;              // [B, Hq/G] arrivals per (sequence, head group); zero between launches
  const int4 *unit_table;         // large batches: (sequence, partition index, ctx, -) per pair, else null
  int32_t B, Hq, Hkv, ratio;      // ratio = Hq / Hkv
  int32_t max_blocks, max_splits, max_ctx;
  int32_t work_begin;             // first block of this item in the grid
  int32_t pair_begin;             // host-enumerated launches: first entry of this item in DecodeParams::pairs;
                                  // device-enumerated: how many of the item's pairs have a workgroup per head group of
                                  // their own (the grid is sized from the caller's bound on the sum of the context lengths)
  float scale_log2;               // scale * log2(e)
};

// Launches whose context lengths the caller also has on the host carry their
// (sequence, partition) pairs in the kernel argument itself: a workgroup then
// knows its unit after scalar loads from the (cached) argument segment instead
// of a round of vector loads of the device-side context lengths - one
// dependent memory latency less before its K/V loads go out.
constexpr int kMaxHostPairs = 384;

struct DecodeParams {
  DecodeItemDev it[MUXA_MAX_DECODE_ITEMS];
  const void *k_pool;
  const void *v_pool;
  int32_t n_items;
  int32_t partition;
  int32_t last_block;             // num_pool_blocks - 1: table entries are clamped to it
  int32_t n_host_pairs;           // > 0: units come from `pairs`, the device-side context lengths are not read
  int32_t rounds;                 // seq_units' R
  int32_t absorb;                 // seq_units' A
  uint2 pairs[kMaxHostPairs];     // x = sequence | unit index << 16, y = clamped context length
};
static_assert(sizeof(DecodeParams) <= 4096, "kernel argument segment");

// One unit of work, uniform across the workgroup.
struct Unit {
  int item, seq, split, ctx, wh, t0, t1, n_splits;
};

// How a context of c tokens is cut into units.  P = partition: the tokens the
// waves of a workgroup load in one round (a multiple of 64); R = rounds: the
// most full groups of P tokens one unit walks; A = absorb.
//   fg = c / P full groups, rem = c - fg P tokens behind them.  A remainder of
//   at most A tokens behind at least one full group is left to the unit that
//   holds the last group (one more, short, round for one of its waves) instead
//   of becoming a unit of its own.
//   nb = ceil(fg / R) units share the fg groups as evenly as possible (unit j
//   holds fg / nb groups, the first fg % nb units one more); a remainder unit,
//   index nb, follows when rem > 0.
// A context with a single unit writes its output directly; others go through
// the partials and the arrival counter.  Host and device enumerate with this one
// function, so the units - and with them the rounding of the results - do not
// depend on who enumerated.
struct SeqUnits {
  int fg, nb, rem;
  __host__ __device__ int count() const { return nb + (rem > 0 ? 1 : 0); }
};
__host__ __device__ inline SeqUnits seq_units(int c, int P, int R, int A) {
  SeqUnits s;
  s.fg = c / P;
  s.rem = c - s.fg * P;
  if (s.fg > 0 && s.rem <= A) s.rem = 0;
  s.nb = (s.fg + R - 1) / R;
  return s;
}
__host__ __device__ inline void unit_range(int c, int P, const SeqUnits &s, int j, int &t0, int &t1) {
  if (j < s.nb) {
    const int base = s.fg / s.nb, extra = s.fg - base * s.nb;
    const int g0 = j * base + (j < extra ? j : extra);
    const int g1 = g0 + base + (j < extra ? 1 : 0);
    t0 = g0 * P;
    t1 = (j == s.nb - 1 && s.rem == 0) ? c : g1 * P;      // an absorbed remainder rides on the last unit
  } else {
    t0 = s.fg * P;
    t1 = c;
  }
}

// Device-coherent accesses for data handed between workgroups of one kernel
// that may run on different XCDs (each XCD has its own L2).
__device__ __forceinline__ void coherent_store(float *p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float coherent_load(const float *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Orders a wave's own LDS writes before its following LDS reads of data other
// lanes wrote.  One wave's LDS instructions execute in order, so this only has
// to stop the compiler from moving them.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// K/V blocks are read exactly once per launch: non-temporal loads keep them
// from displacing the block tables, q and context lengths in the XCD's L2.
typedef uint32_t nt_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 stream_load(const uint4 *p) {
  const nt_u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x4 *>(p));
  return make_uint4(t.x, t.y, t.z, t.w);
}

template <int BS>
struct Geometry {
  static_assert(BS == 8 || BS == 16 || BS == 32, "block size");
  static constexpr int D = kHeadSize;
  static constexpr int BPT = 64 / BS;               // blocks per 64-token tile
  static constexpr int PARTS = BS / 8;              // 16-byte chunks per V row of a block
  static constexpr int VI = D * PARTS / 64;         // V load instructions per block
  static constexpr int BLOCK_CHUNKS = D * BS / 8;   // 16-byte chunks per K block (same for V)
};

// This lane's block id for token tb+lane of a sequence's table row (0 for
// tokens at or past t1).  Clamped so that a corrupt table entry reads the
// wrong block instead of faulting the GPU.
template <int BS>
__device__ __forceinline__ int load_block_id(const int32_t *trow, int tb, int t1, int lane, int last_block) {
  const int tok = tb + lane;
  int id = 0;
  if (tok < t1) id = min(max(trow[tok / BS], 0), last_block);
  return id;
}

// Issues every load of a tile: 16 K chunks for this lane's token, BPT*VI V chunks.
template <int BS>
__device__ __forceinline__ void issue_tile_loads(uint4 (&kreg)[16], uint4 (&vreg)[Geometry<BS>::BPT][Geometry<BS>::VI],
                                                 const uint4 *kpool, const uint4 *vpool, int id, int tb, int t1,
                                                 int lane) {
  using Geo = Geometry<BS>;
  const int tok = tb + lane;
  const int part = lane % Geo::PARTS;
  if (tok < t1) {
    const uint4 *kp = kpool + static_cast<int64_t>(id) * Geo::BLOCK_CHUNKS + (tok % BS);
#pragma unroll
    for (int j = 0; j < 16; ++j) kreg[j] = stream_load(&kp[j * BS]);
  } else {
#pragma unroll
    for (int j = 0; j < 16; ++j) kreg[j] = make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int b = 0; b < Geo::BPT; ++b) {
    const int idb = __builtin_amdgcn_readlane(id, b * BS);   // the block's id, uniform
    const uint4 *vp = vpool + static_cast<int64_t>(idb) * Geo::BLOCK_CHUNKS + lane;
    const bool chunk_ok = tb + b * BS + part * 8 < t1;
#pragma unroll
    for (int j = 0; j < Geo::VI; ++j) {
      if (chunk_ok) vreg[b][j] = stream_load(&vp[j * 64]);
      else vreg[b][j] = make_uint4(0, 0, 0, 0);
    }
  }
}

// Scores, online softmax and P.V for one loaded tile.
template <typename T, int BS, int G>
__device__ __forceinline__ void consume_tile(uint4 (&kreg)[16], uint4 (&vreg)[Geometry<BS>::BPT][Geometry<BS>::VI],
                                             const uint32_t (&q_s)[64], const uint32_t (*q_w)[64],
                                             float (*p_w)[64], float (&m)[G], float (&l)[G],
                                             float (&acc)[G][Geometry<BS>::VI], float scale_log2, int tb, int t1,
                                             int lane) {
  using Geo = Geometry<BS>;
  const int part = lane % Geo::PARTS;
  const bool valid = tb + lane < t1;
  // Tail tile: zero V elements of tokens >= t1 (their probability is 0 but
  // the slots were never written and may hold NaN/Inf bit patterns).
  if (tb + 64 > t1) {
#pragma unroll
    for (int b = 0; b < Geo::BPT; ++b) {
      const int n_ok = t1 - (tb + b * BS + part * 8);   // valid tokens in this lane's chunk
#pragma unroll
      for (int j = 0; j < Geo::VI; ++j) {
        uint32_t *wv = reinterpret_cast<uint32_t *>(&vreg[b][j]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (2 * e >= n_ok) wv[e] = 0u;
          else if (2 * e + 1 >= n_ok) wv[e] &= 0x0000ffffu;
        }
      }
    }
  }

  float s[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      uint4 qq;
      if constexpr (G == 1) qq = make_uint4(q_s[4 * j], q_s[4 * j + 1], q_s[4 * j + 2], q_s[4 * j + 3]);
      else qq = reinterpret_cast<const uint4 *>(q_w[g])[j];
      a0 = dot2<T>(kreg[j].x, qq.x, a0);
      a1 = dot2<T>(kreg[j].y, qq.y, a1);
      a0 = dot2<T>(kreg[j].z, qq.z, a0);
      a1 = dot2<T>(kreg[j].w, qq.w, a1);
    }
    s[g] = valid ? (a0 + a1) * scale_log2 : -INFINITY;
  }

  // fp16: the probabilities go to the P.V product as packed halves, one
  // v_dot2_f32_f16 per pair of tokens instead of two conversions and two
  // multiply-adds (a quarter of the product's instructions; the accumulation stays
  // fp32).  They are taken 2^15 times too large, so that the smallest half-precision
  // normal stands for a probability of 2e-9 rather than 6e-5; the running sum
  // carries the same factor, which therefore cancels in every ratio this kernel and
  // the merges form.  bf16 would keep 8 bits of a probability: it stays on the
  // fp32 path.
  constexpr bool kHalfP = __is_same(T, F16);
  constexpr float kPShift = kHalfP ? 15.f : 0.f;
  uint16_t(*p_h)[64] = reinterpret_cast<uint16_t(*)[64]>(p_w);     // the same LDS, as halves, one row per head
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const float m_new = fmaxf(m[g], wave_max(s[g]));
    const float alpha = fast_exp2(m[g] - m_new);
    const float p = fast_exp2(s[g] - m_new + kPShift);
    l[g] = l[g] * alpha + p;
#pragma unroll
    for (int j = 0; j < Geo::VI; ++j) acc[g][j] *= alpha;
    m[g] = m_new;
    if constexpr (kHalfP) p_h[2 * g][lane] = f32_to_f16_bits(p);     // (row 2 g: rows are 128 bytes, a float row 256)
    else p_w[g][lane] = p;
  }
  wave_lds_sync();

#pragma unroll
  for (int b = 0; b < Geo::BPT; ++b) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if constexpr (kHalfP) {
        const uint4 pp = *reinterpret_cast<const uint4 *>(&p_h[2 * g][b * BS + part * 8]);
#pragma unroll
        for (int j = 0; j < Geo::VI; ++j) {
          float a = acc[g][j];
          a = dot2<T>(vreg[b][j].x, pp.x, a);
          a = dot2<T>(vreg[b][j].y, pp.y, a);
          a = dot2<T>(vreg[b][j].z, pp.z, a);
          a = dot2<T>(vreg[b][j].w, pp.w, a);
          acc[g][j] = a;
        }
      } else {
        const float4 pa = *reinterpret_cast<const float4 *>(&p_w[g][b * BS + part * 8]);
        const float4 pb = *reinterpret_cast<const float4 *>(&p_w[g][b * BS + part * 8 + 4]);
#pragma unroll
        for (int j = 0; j < Geo::VI; ++j) {
          float a = acc[g][j];
          a = fma2<T>(vreg[b][j].x, pa.x, pa.y, a);
          a = fma2<T>(vreg[b][j].y, pa.z, pa.w, a);
          a = fma2<T>(vreg[b][j].z, pb.x, pb.y, a);
          a = fma2<T>(vreg[b][j].w, pb.z, pb.w, a);
          acc[g][j] = a;
        }
      }
    }
  }
  wave_lds_sync();
}

// This wave's partial (a wave without tiles contributes max=-inf, sum=0) to LDS.
template <int BS, int G>
__device__ __forceinline__ void stash_wave_partial(float (&m)[G], float (&l)[G], float (&acc)[G][Geometry<BS>::VI],
                                                   float (*xa)[kHeadSize], float (*xm)[2], int lane) {
  using Geo = Geometry<BS>;
  const int part = lane % Geo::PARTS;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const float L = wave_sum(l[g]);
#pragma unroll
    for (int j = 0; j < Geo::VI; ++j) {
      float a = acc[g][j];
      if constexpr (Geo::PARTS >= 2) a += dpp_mov<0xB1>(a);
      if constexpr (Geo::PARTS >= 4) a += dpp_mov<0x4E>(a);
      const int d = j * (64 / Geo::PARTS) + lane / Geo::PARTS;
      if (part == 0) xa[g][d] = a;
    }
    if (lane == 0) {
      xm[g][0] = m[g];
      xm[g][1] = L;
    }
  }
}

// Combine of one head's partitions by one wave: out = sum_i w_i acc_i / sum_i w_i l_i,
// w_i = 2^(m_i - max m).  Lane i of a 64-partition chunk holds (m_i, l_i); the
// partial accumulators are fetched eight partitions at a time, all loads in
// flight together (partition indices past the end re-read the last partition
// with weight 0).
template <typename T>
__device__ __forceinline__ void combine_head(const DecodeItemDev &I, int seq, int hq, int n_splits, int lane) {
  constexpr int D = kHeadSize;
  const int64_t base = (static_cast<int64_t>(seq) * I.Hq + hq) * I.max_splits;
  const float *ml = I.ws_ml + base * 2;
  const float *pa = I.ws_acc + base * D;
  float M = -INFINITY;
  for (int c0 = 0; c0 < n_splits; c0 += 64) {
    const int i = c0 + lane;
    if (i < n_splits) M = fmaxf(M, coherent_load(&ml[i * 2]));
  }
  M = wave_max(M);
  float Lsum = 0.f, a0 = 0.f, a1 = 0.f;
  for (int c0 = 0; c0 < n_splits; c0 += 64) {
    const int i = c0 + lane;
    float wl = 0.f;
    if (i < n_splits) {
      wl = fast_exp2(coherent_load(&ml[i * 2]) - M);
      Lsum += coherent_load(&ml[i * 2 + 1]) * wl;
    }
    const int cnt = min(64, n_splits - c0);
    for (int k0 = 0; k0 < cnt; k0 += 8) {
      float v0[8], v1[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int idx = min(c0 + k0 + j, n_splits - 1);
        v0[j] = coherent_load(&pa[idx * D + lane]);
        v1[j] = coherent_load(&pa[idx * D + 64 + lane]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float wj = k0 + j < 64 ? lane_bcast(wl, (k0 + j) & 63) : 0.f;
        a0 = __builtin_fmaf(v0[j], wj, a0);
        a1 = __builtin_fmaf(v1[j], wj, a1);
      }
    }
  }
  Lsum = wave_sum(Lsum);
  uint16_t *o = static_cast<uint16_t *>(I.out) + static_cast<int64_t>(seq) * I.out_stride + hq * D;
  o[lane] = to_storage<T>(a0 / Lsum);
  o[64 + lane] = to_storage<T>(a1 / Lsum);
}

// Wave 0: merge the workgroup's NW partials (lane owns dims lane and lane+64),
// then either write the output (context fits one partition) or publish the
// partition's partial and, if this was the last partition to arrive, combine
// them all.
template <typename T, int G, int NW>
__device__ __forceinline__ void merge_and_write(const DecodeItemDev &I, const Unit &u, int partition,
                                                const float (*xa)[G][kHeadSize], const float (*xm)[G][2],
                                                int n_active, int lane) {
  constexpr int D = kHeadSize;
  const bool single = u.n_splits == 1;
  const int hq0 = u.wh * G;
#pragma unroll 1
  for (int g = 0; g < G; ++g) {
    // Waves without tokens have left early and wrote nothing.
    float M = xm[0][g][0];
#pragma unroll
    for (int k = 1; k < NW; ++k)
      if (k < n_active) M = fmaxf(M, xm[k][g][0]);
    float L = 0.f, a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int k = 0; k < NW; ++k)
      if (k < n_active) {
        const float wgt = fast_exp2(xm[k][g][0] - M);
        L += xm[k][g][1] * wgt;
        a0 += xa[k][g][lane] * wgt;
        a1 += xa[k][g][64 + lane] * wgt;
      }
    const int hq = hq0 + g;
    if (single) {
      uint16_t *o = static_cast<uint16_t *>(I.out) + static_cast<int64_t>(u.seq) * I.out_stride + hq * D;
      o[lane] = to_storage<T>(a0 / L);
      o[64 + lane] = to_storage<T>(a1 / L);
    } else {
      const int64_t prow = (static_cast<int64_t>(u.seq) * I.Hq + hq) * I.max_splits + u.split;
      coherent_store(&I.ws_acc[prow * D + lane], a0);
      coherent_store(&I.ws_acc[prow * D + 64 + lane], a1);
      if (lane == 0) {
        coherent_store(&I.ws_ml[prow * 2], M);
        coherent_store(&I.ws_ml[prow * 2 + 1], L);
      }
    }
  }
  if (single) return;

  // Partials are written and read with device-coherent accesses (they bypass
  // the per-XCD L2 and are acknowledged from the memory side), so ordering them
  // against the arrival counter needs no L2 write-back/invalidate, only: (1) this
  // wave's partial stores have been acknowledged before the counter is bumped -
  // the explicit vmcnt wait; (2) the combiner's loads issue after its atomic
  // returned - they depend on its value.  The fences only pin the compiler.
  const int n_splits = u.n_splits;
  int32_t *counter = I.counters + static_cast<int64_t>(u.seq) * (I.Hq / G) + u.wh;
  wait_own_vector_memory();
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  int arrived = 0;
  if (lane == 0) arrived = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  arrived = __builtin_amdgcn_readfirstlane(arrived);
  if (arrived != n_splits - 1) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll 1
  for (int g = 0; g < G; ++g) combine_head<T>(I, u.seq, hq0 + g, n_splits, lane);
  // Ready for the next launch.
  if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The same merge, publish and combine for a group of G heads, spread over the
// workgroup's waves that had tokens (the first n_active; wave w takes heads w,
// w + n_active, ...).  Every one of them must call it.
template <typename T, int G, int NW>
__device__ __forceinline__ void merge_and_write_group(const DecodeItemDev &I, const Unit &u, int partition,
                                                      const float (*xa)[G][kHeadSize], const float (*xm)[G][2],
                                                      int *arrival_lds, int n_active, int lane, int wave) {
  constexpr int D = kHeadSize;
  const bool single = u.n_splits == 1;
  const int hq0 = u.wh * G;
  // (a wave that had no tokens but stayed - see the kernels' sweep - only keeps the barriers company)
  const int g_first = wave < n_active ? wave : G;
#pragma unroll 1
  for (int g = g_first; g < G; g += n_active) {
    // Waves without tokens have left early and wrote nothing.
    float M = xm[0][g][0];
#pragma unroll
    for (int k = 1; k < NW; ++k)
      if (k < n_active) M = fmaxf(M, xm[k][g][0]);
    float L = 0.f, a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int k = 0; k < NW; ++k)
      if (k < n_active) {
        const float wgt = fast_exp2(xm[k][g][0] - M);
        L += xm[k][g][1] * wgt;
        a0 += xa[k][g][lane] * wgt;
        a1 += xa[k][g][64 + lane] * wgt;
      }
    const int hq = hq0 + g;
    if (single) {
      uint16_t *o = static_cast<uint16_t *>(I.out) + static_cast<int64_t>(u.seq) * I.out_stride + hq * D;
      o[lane] = to_storage<T>(a0 / L);
      o[64 + lane] = to_storage<T>(a1 / L);
    } else {
      const int64_t prow = (static_cast<int64_t>(u.seq) * I.Hq + hq) * I.max_splits + u.split;
      coherent_store(&I.ws_acc[prow * D + lane], a0);
      coherent_store(&I.ws_acc[prow * D + 64 + lane], a1);
      if (lane == 0) {
        coherent_store(&I.ws_ml[prow * 2], M);
        coherent_store(&I.ws_ml[prow * 2 + 1], L);
      }
    }
  }
  if (single) return;

  // Each wave waits until its own partial stores have been acknowledged (they
  // bypass the per-XCD L2, so the acknowledgement is all that is needed), the
  // workgroup meets, one lane announces the arrival and tells the others
  // whether this workgroup came last.
  const int n_splits = u.n_splits;
  int32_t *counter = I.counters + static_cast<int64_t>(u.seq) * (I.Hq / G) + u.wh;
  wait_own_vector_memory();
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (wave == 0 && lane == 0)
    *arrival_lds = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (*arrival_lds != n_splits - 1) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll 1
  for (int g = g_first; g < G; g += n_active) combine_head<T>(I, u.seq, hq0 + g, n_splits, lane);
  // Ready for the next launch.
  if (wave == 0 && lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------
// Direct kernel: one workgroup per unit, unit found by scanning the context
// lengths in global memory.
// ---------------------------------------------------------------------------

// Maps pair index e to (sequence, unit index).  Every lane returns the same
// answer; false: e is past the last pair (grid padding).  Pairs are numbered in
// three classes, chosen so that the kernel's last workgroups are the ones that
// finish fastest:
//   1. the remainder unit of every context that has more than one unit -
//      dispatched first, so the unit that arrives last and combines a split
//      context is normally a full one in mid-kernel;
//   2. all other units of those contexts;
//   3. contexts with a single unit: no partials, no atomics, the output is
//      written straight from the workgroup.

// Lane index of the n-th (0-based) set bit of a wave mask that has more than n bits set.
__device__ __forceinline__ int nth_set_lane(unsigned long long mask, int n, int lane) {
  const int upto = __popcll(mask & (~0ull >> (63 - lane)));          // set bits in lanes 0..lane
  const unsigned long long hit = __builtin_amdgcn_ballot_w64(((mask >> lane) & 1ull) != 0 && upto == n + 1);
  return __ffsll(static_cast<long long>(hit)) - 1;
}

// Batches of at most 64 * kLocateChunks sequences: all context lengths are
// fetched with one round of loads (lane l keeps sequences l, l+64, ...) and the
// three classes are enumerated from registers, so the unit is known after a
// single memory latency.
constexpr int kLocateChunks = 4;
__device__ __forceinline__ bool locate_pair_small(const int32_t *ctx_arr, int B, int max_ctx, int partition,
                                                  int rounds, int absorb, int e, int lane, int &seq, int &split,
                                                  int &ctx) {
  int c[kLocateChunks], big[kLocateChunks];
#pragma unroll
  for (int j = 0; j < kLocateChunks; ++j) {
    const int s = 64 * j + lane;
    c[j] = s < B ? ctx_arr[s] : 0;
  }
  unsigned long long rem_mask[kLocateChunks], single_mask[kLocateChunks];
#pragma unroll
  for (int j = 0; j < kLocateChunks; ++j) {
    c[j] = max(min(c[j], max_ctx), 0);
    const SeqUnits su = seq_units(c[j], partition, rounds, absorb);
    const bool split_ctx = su.count() > 1;
    big[j] = split_ctx ? su.nb : 0;
    rem_mask[j] = __builtin_amdgcn_ballot_w64(split_ctx && su.rem > 0);
    single_mask[j] = __builtin_amdgcn_ballot_w64(c[j] > 0 && !split_ctx);
  }
  int base = 0;
  // class 1: remainder units of split contexts
#pragma unroll
  for (int j = 0; j < kLocateChunks; ++j) {
    const int cnt = __popcll(rem_mask[j]);
    if (e < base + cnt) {
      const int k = nth_set_lane(rem_mask[j], e - base, lane);
      seq = 64 * j + k;
      ctx = __builtin_amdgcn_readlane(c[j], k);
      split = __builtin_amdgcn_readlane(big[j], k);
      return true;
    }
    base += cnt;
  }
  // class 2: the other units of split contexts
#pragma unroll
  for (int j = 0; j < kLocateChunks; ++j) {
    const int incl = wave_inclusive_scan(big[j]);
    const int total = __builtin_amdgcn_readlane(incl, 63);
    if (e < base + total) {
      const int k = __popcll(__builtin_amdgcn_ballot_w64(base + incl <= e));
      seq = 64 * j + k;
      split = e - base - __builtin_amdgcn_readlane(incl - big[j], k);
      ctx = __builtin_amdgcn_readlane(c[j], k);
      return true;
    }
    base += total;
  }
  // class 3: contexts with a single unit
#pragma unroll
  for (int j = 0; j < kLocateChunks; ++j) {
    const int cnt = __popcll(single_mask[j]);
    if (e < base + cnt) {
      const int k = nth_set_lane(single_mask[j], e - base, lane);
      seq = 64 * j + k;
      ctx = __builtin_amdgcn_readlane(c[j], k);
      split = 0;
      return true;
    }
    base += cnt;
  }
  return false;
}

// Batches too large for that take the pair from a table that a small kernel
// (decode_plan_kernel below) writes ahead of the launch: one 16-byte load.
__device__ __forceinline__ bool locate_pair(const DecodeParams &P, const DecodeItemDev &I, int partition, int e,
                                            int lane, int &seq, int &split, int &ctx) {
  if (P.n_host_pairs > 0) {
    // The grid of such a launch holds exactly the enumerated pairs.
    const uint2 pr = P.pairs[min(I.pair_begin + e, kMaxHostPairs - 1)];
    seq = static_cast<int>(pr.x & 0xffffu);
    split = static_cast<int>(pr.x >> 16);
    ctx = static_cast<int>(pr.y);
    return true;
  }
  if (I.unit_table == nullptr)
    return locate_pair_small(I.ctx, I.B, I.max_ctx, partition, P.rounds, P.absorb, e, lane, seq, split, ctx);
  if (e >= I.B * I.max_splits) return false;      // the table holds a row for every pair there can be
  const int4 ent = I.unit_table[e];
  if (ent.x < 0) return false;
  seq = ent.x;
  split = ent.y;
  ctx = ent.z;
  return true;
}

// Writes the (sequence, unit) table of one item per workgroup, in the same
// three classes as above.  Thread t owns a contiguous range of sequences;
// class counts are prefix-summed over the threads in LDS.  Entries past the
// last pair (the grid is sized from an upper bound) get sequence -1.
struct PlanItem {
  const int32_t *ctx;
  int4 *table;
  int32_t B, max_ctx, capacity;   // capacity = entries in table
};
struct PlanParams {
  PlanItem it[MUXA_MAX_DECODE_ITEMS];
  int32_t partition, rounds, absorb;
};

__global__ __launch_bounds__(256) void decode_plan_kernel(const PlanParams PP) {
  __shared__ int scan[3][256];
  const PlanItem &I = PP.it[blockIdx.x];
  const int partition = PP.partition;
  const int t = threadIdx.x;
  const int per = (I.B + 255) / 256;
  const int s0 = min(t * per, I.B), s1 = min(s0 + per, I.B);
  int n[3] = {0, 0, 0};
  for (int s = s0; s < s1; ++s) {
    const int c = max(min(I.ctx[s], I.max_ctx), 0);
    const SeqUnits su = seq_units(c, partition, PP.rounds, PP.absorb);
    if (su.count() > 1) {
      n[1] += su.nb;
      if (su.rem > 0) n[0] += 1;
    } else if (c > 0) {
      n[2] += 1;
    }
  }
#pragma unroll
  for (int k = 0; k < 3; ++k) scan[k][t] = n[k];
  __syncthreads();
  for (int d = 1; d < 256; d <<= 1) {      // inclusive Hillis-Steele scan of the three rows
    int v[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) v[k] = t >= d ? scan[k][t - d] : 0;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 3; ++k) scan[k][t] += v[k];
    __syncthreads();
  }
  const int tot0 = scan[0][255], tot1 = scan[1][255], tot2 = scan[2][255];
  int at0 = scan[0][t] - n[0];
  int at1 = tot0 + scan[1][t] - n[1];
  int at2 = tot0 + tot1 + scan[2][t] - n[2];
  for (int s = s0; s < s1; ++s) {
    const int c = max(min(I.ctx[s], I.max_ctx), 0);
    const SeqUnits su = seq_units(c, partition, PP.rounds, PP.absorb);
    if (su.count() > 1) {
      for (int j = 0; j < su.nb; ++j)
        if (at1 < I.capacity) I.table[at1++] = make_int4(s, j, c, 0);
      if (su.rem > 0 && at0 < I.capacity) I.table[at0++] = make_int4(s, su.nb, c, 0);
    } else if (c > 0) {
      if (at2 < I.capacity) I.table[at2++] = make_int4(s, 0, c, 0);
    }
  }
  for (int i = tot0 + tot1 + tot2 + t; i < I.capacity; i += 256) I.table[i] = make_int4(-1, 0, 0, 0);
}

// q of the unit's head group for the tile code.  G == 1: one coalesced 256-byte
// load, then 64 readlanes make it uniform (SGPRs) so q.k needs no q registers
// per lane.  G > 1: this wave's LDS copy.
template <int G>
__device__ __forceinline__ void fetch_q(const DecodeItemDev &I, int seq, int hq0, int lane, uint32_t (&q_s)[64],
                                        uint32_t (*q_w)[64]) {
  const uint32_t *qv = reinterpret_cast<const uint32_t *>(
      static_cast<const uint16_t *>(I.q) + static_cast<int64_t>(seq) * I.q_stride + hq0 * kHeadSize);
  if constexpr (G == 1) {
    const uint32_t mine = qv[lane];
#pragma unroll
    for (int i = 0; i < 64; ++i) q_s[i] = __builtin_amdgcn_readlane(mine, i);
  } else {
#pragma unroll
    for (int g = 0; g < G; ++g) q_w[g][lane] = qv[g * 64 + lane];
    wave_lds_sync();
  }
}

#ifdef MUX_TRACE
// (the stamps cost two registers; the tracing build is held to the shipped kernel's
// three waves per SIMD so that the timeline is that of the same residency)
#define MUX_DECODE_BOUNDS __launch_bounds__(64 * NW, G == 1 ? 3 : 1)
#else
#define MUX_DECODE_BOUNDS __launch_bounds__(64 * NW)
#endif

// LDS of one workgroup of the vector-ALU kernel.
template <int G, int NW>
struct DecodeSmem {
  __attribute__((aligned(16))) float p[NW][G][64];      // per-wave probabilities of a tile
  __attribute__((aligned(16))) uint32_t q[NW][G][64];   // G > 1: per-wave copy of the group's q
  float x_acc[NW][G][kHeadSize];                        // per-wave partial outputs
  float x_ml[NW][G][2];
};

// One unit, start to finish, by the workgroup's NW waves.  STAY = false: waves
// that have nothing (more) to do return from the kernel (the function's result
// tells the caller to return); STAY = true, for a workgroup that goes on to
// another unit: every wave comes back, after a barrier that makes the LDS
// partials reusable.
template <typename T, int BS, int G, int NW, bool STAY>
__device__ __forceinline__ bool decode_unit(const DecodeParams &P, const DecodeItemDev &I, Unit &u, int e,
                                            DecodeSmem<G, NW> &sm, int lane, int wave) {
  using Geo = Geometry<BS>;
  const int partition = P.partition;
  // Every wave of the workgroup derives the same unit (or all of them leave).
  if (!locate_pair(P, I, partition, e, lane, u.seq, u.split, u.ctx)) return false;
  {
    const SeqUnits su = seq_units(u.ctx, partition, P.rounds, P.absorb);
    unit_range(u.ctx, partition, su, u.split, u.t0, u.t1);
    u.n_splits = su.count();
  }
  MUX_TR(1);
  MUX_TRV(7, static_cast<long long>(u.t1 - u.t0) | (static_cast<long long>(u.n_splits > 1) << 16));
  const int hq0 = u.wh * G;
  const int hk = hq0 / I.ratio;

  // The first tile's block ids and q are independent: both loads are issued
  // before either is waited for.
  const int32_t *trow = I.tables + (static_cast<int64_t>(u.seq) * I.Hkv + hk) * I.max_blocks;
  const uint4 *kpool = static_cast<const uint4 *>(P.k_pool);
  const uint4 *vpool = static_cast<const uint4 *>(P.v_pool);
  const int tb0 = u.t0 + wave * 64;
  // A wave without tokens leaves at once and frees its registers for the next
  // workgroup; the barrier below counts only the waves that are still there.
  const bool idle = tb0 >= u.t1;
  if constexpr (!STAY) {
    if (idle) return false;
  }
  const int n_active = min(NW, (u.t1 - u.t0 + 63) / 64);
  if (!STAY || !idle) {
    int id_next = load_block_id<BS>(trow, tb0, u.t1, lane, P.last_block);
    uint32_t q_s[64];
    fetch_q<G>(I, u.seq, hq0, lane, q_s, sm.q[wave]);
    MUX_TR(2);

    float m[G], l[G], acc[G][Geo::VI];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      m[g] = -INFINITY;
      l[g] = 0.f;
#pragma unroll
      for (int j = 0; j < Geo::VI; ++j) acc[g][j] = 0.f;
    }
    for (int tb = tb0; tb < u.t1; tb += 64 * NW) {
      const int id = id_next;
      if (tb + 64 * NW < u.t1) id_next = load_block_id<BS>(trow, tb + 64 * NW, u.t1, lane, P.last_block);
      uint4 kreg[16];
      uint4 vreg[Geo::BPT][Geo::VI];
      issue_tile_loads<BS>(kreg, vreg, kpool, vpool, id, tb, u.t1, lane);
      MUX_TR(3);
      consume_tile<T, BS, G>(kreg, vreg, q_s, sm.q[wave], sm.p[wave], m, l, acc, I.scale_log2, tb, u.t1, lane);
      MUX_TR(4);
    }
    stash_wave_partial<BS, G>(m, l, acc, sm.x_acc[wave], sm.x_ml[wave], lane);
  }
  __syncthreads();
  MUX_TR(5);
  if constexpr (!STAY) {
    if (wave != 0) return false;
  }
  if (wave == 0) merge_and_write<T, G, NW>(I, u, partition, sm.x_acc, sm.x_ml, n_active, lane);
  MUX_TR(6);
  if constexpr (STAY) __syncthreads();
  return true;
}

template <typename T, int BS, int G, int NW>
__global__ MUX_DECODE_BOUNDS void paged_decode_kernel(const DecodeParams P) {
  __shared__ DecodeSmem<G, NW> sm;
  MUX_TR(0);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int w = blockIdx.x;
  int ii = 0;
#pragma unroll
  for (int k = 1; k < MUXA_MAX_DECODE_ITEMS; ++k)
    if (k < P.n_items && w >= P.it[k].work_begin) ii = k;
  const DecodeItemDev I = P.it[ii];       // by value: one round of scalar loads for every field

  const int WH = I.Hq / G;                   // head groups per sequence
  const int local = w - I.work_begin;
  const int e = local / WH;
  Unit u;
  u.item = ii;
  u.wh = local - e * WH;
  decode_unit<T, BS, G, NW, false>(P, I, u, e, sm, lane, wave);
}

// A device-enumerated launch is sized from the caller's bound on the sum of the
// context lengths.  Should that bound have been too small, some (sequence, unit)
// pairs have no workgroup in the grid above; this kernel, launched behind it
// with one workgroup per item and head group, runs them one after the other
// (slow, but every output is written and every arrival counter returns to zero).
// With a bound that holds its workgroups find nothing and leave.
template <typename T, int BS, int G, int NW>
__global__ __launch_bounds__(64 * NW) void paged_decode_sweep_kernel(const DecodeParams P) {
  __shared__ DecodeSmem<G, NW> sm;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int w = blockIdx.x;
  int ii = 0;
#pragma unroll
  for (int k = 1; k < MUXA_MAX_DECODE_ITEMS; ++k)
    if (k < P.n_items && w >= P.it[k].work_begin) ii = k;
  const DecodeItemDev I = P.it[ii];
  Unit u;
  u.item = ii;
  u.wh = w - I.work_begin;                   // one workgroup per head group; work_begin counts those
  for (int e = I.pair_begin;; ++e)           // pair_begin: the pairs that had a place in the grid above
    if (!decode_unit<T, BS, G, NW, true>(P, I, u, e, sm, lane, wave)) return;
}

// ---------------------------------------------------------------------------
// Grouped-query kernel (G >= 4 query heads per kv head): the G heads of a group
// read the same K/V, so scores and P.V are small matrix products and go to the
// matrix cores (v_mfma_f32_16x16x32_{f16,bf16}), with the group padded to the 16
// columns of the instruction.  Both products are kept transposed so that a lane
// owns ONE head (lane % 16) throughout and the softmax state is a per-lane scalar:
//     S^T[tok][head] = K . Q^T     A = K   : lane (tok = l%16, g = l/16) holds dims
//                                            32 s + 8 g .. +7 of its token - exactly
//                                            the pool's 16-byte chunk (d/8, tok)
//                                  B = Q^T : lane (head = l%16, g), same dims
//     O^T[d][head]  += V^T . P^T   A = V^T : lane (d = 16 nb + l%16, g) holds tokens
//                                            32 ts + 8 g .. +7 of its dim - exactly
//                                            the pool's 16-byte chunk (d, tok/8)
//                                  B = P^T : lane (head = l%16, g), same tokens
// so every K and V load lands in its operand register straight from the pool.
// The score accumulators give a lane tokens 16 tg + 4 g + i of its head; the
// regrouping into runs of 8 tokens goes through 1 KiB of LDS per wave.
// A wave advances 32 tokens per step (16 KiB of K/V in 64 registers); three
// waves per SIMD keep the memory system busy while one of them computes.
// Work units, partitions, the cross-wave merge and the split combine are those
// of the kernel above.
// ---------------------------------------------------------------------------
typedef _Float16 v8f16_t __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf16_t __attribute__((ext_vector_type(8)));
typedef float v4f32_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

union Frag8 {
  u32x4_t u;
  v8f16_t h;
  v8bf16_t b;
};

template <typename T>
__device__ __forceinline__ v4f32_t mfma16(const Frag8 &a, const Frag8 &b, v4f32_t c) {
  if constexpr (__is_same(T, F16)) return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h, b.h, c, 0, 0, 0);
  else return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b.b, c, 0, 0, 0);
}

typedef float float2v_t __attribute__((ext_vector_type(2)));
template <typename T>
__device__ __forceinline__ uint32_t pack_pair(float lo, float hi) {
  const float2v_t x = {lo, hi};
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

constexpr int kGqaTile = 32;             // tokens per wave step
constexpr int kPRow = kGqaTile + 8;      // P^T row in LDS: 32 tokens + 16 bytes of padding

// Registers of one 32-token step: K as 2 token groups x 4 dim steps, V as 8 dim blocks.
struct GqaTile {
  u32x4_t k[2][4];
  u32x4_t v[8];
};

// LDS of one workgroup of the grouped-query kernel.
template <typename T, int G, int NW>
struct GqaSmem {
  static constexpr int kParts = __is_same(T, BF16) ? 2 : 1;    // bf16 keeps 8 bits of a probability: P as hi + lo parts
  __attribute__((aligned(16))) uint16_t p[NW][kParts][16][kPRow];
  __attribute__((aligned(16))) float x_acc[NW][G][kHeadSize];
  float x_ml[NW][G][2];
  int arrival;
};

// One unit by the workgroup's NW waves; STAY as in decode_unit above.
template <typename T, int BS, int G, int NW, bool STAY>
__device__ __forceinline__ bool decode_unit_gqa(const DecodeParams &P, const DecodeItemDev &I, Unit &u, int e,
                                                GqaSmem<T, G, NW> &sm, int lane, int wave) {
  using Geo = Geometry<BS>;
  static_assert(G >= 2 && G <= 16, "group size");
  constexpr int kParts = GqaSmem<T, G, NW>::kParts;
  constexpr int kStep = kGqaTile * NW;   // wave w takes tokens t0 + 32 w + kStep n .. +31
  auto &p_lds = sm.p;
  auto &x_acc = sm.x_acc;
  auto &x_ml = sm.x_ml;
  const int partition = P.partition;
  if (!locate_pair(P, I, partition, e, lane, u.seq, u.split, u.ctx)) return false;
  {
    const SeqUnits su = seq_units(u.ctx, partition, P.rounds, P.absorb);
    unit_range(u.ctx, partition, su, u.split, u.t0, u.t1);
    u.n_splits = su.count();
  }
  const int hq0 = u.wh * G;
  const int hk = hq0 / I.ratio;
  const int t1 = u.t1;

  // A wave without tokens leaves at once (see the kernel above).
  const bool idle = u.t0 + kGqaTile * wave >= t1;
  if constexpr (!STAY) {
    if (idle) return false;
  }
  const int n_active = min(NW, (t1 - u.t0 + kGqaTile - 1) / kGqaTile);

  const int h = lane & 15;               // this lane's head (columns >= G are padding)
  const int g = lane >> 4;               // which 8 of an operand's 32 k-slots

  // Q^T operand: dims 32 s + 8 g .. +7 of head h.
  Frag8 qf[4];
  {
    const uint16_t *qrow = static_cast<const uint16_t *>(I.q) + static_cast<int64_t>(u.seq) * I.q_stride +
                           (hq0 + (h < G ? h : 0)) * kHeadSize + 8 * g;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      // q rows are only 4-byte aligned in general.
      const uint32_t *qp = reinterpret_cast<const uint32_t *>(qrow + 32 * s);
      qf[s].u = h < G ? u32x4_t{qp[0], qp[1], qp[2], qp[3]} : u32x4_t{0, 0, 0, 0};
    }
  }

  const int32_t *trow = I.tables + (static_cast<int64_t>(u.seq) * I.Hkv + hk) * I.max_blocks;
  const u32x4_t *kpool = static_cast<const u32x4_t *>(P.k_pool);
  const u32x4_t *vpool = static_cast<const u32x4_t *>(P.v_pool);
  const int last_block = P.last_block;
  const float scale_log2 = I.scale_log2;

  v4f32_t oacc[8];                       // O^T[d = 16 nb + 4 g + i][head h]
#pragma unroll
  for (int nb = 0; nb < 8; ++nb) oacc[nb] = v4f32_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;          // running max (log2 units) and this lane's share of the sum

  // Block ids of the step at tb: x, y for the K tokens tb + h and tb + 16 + h,
  // z for the V tokens tb + 8 g .. +7 (0 past t1).  Clamped so that a corrupt
  // table entry reads the wrong block instead of faulting the GPU.
  // Raw table entries; they are clamped where they are used, so that nothing
  // waits for them at the point of the load.
  auto load_ids = [&](int tb) {
    int3 id = make_int3(0, 0, 0);
    if (tb + h < t1) id.x = trow[(tb + h) / BS];
    if (tb + 16 + h < t1) id.y = trow[(tb + 16 + h) / BS];
    if (tb + 8 * g < t1) id.z = trow[(tb + 8 * g) / BS];
    return id;
  };
  auto issue = [&](GqaTile &r, int tb, int3 id) {
    id.x = min(max(id.x, 0), last_block);
    id.y = min(max(id.y, 0), last_block);
    id.z = min(max(id.z, 0), last_block);
#pragma unroll
    for (int tg = 0; tg < 2; ++tg) {
      const int tok = tb + 16 * tg + h;
      const u32x4_t *kp = kpool + static_cast<int64_t>(tg ? id.y : id.x) * Geo::BLOCK_CHUNKS + (tok % BS);
#pragma unroll
      for (int s = 0; s < 4; ++s)
        r.k[tg][s] = tok < t1 ? __builtin_nontemporal_load(&kp[(4 * s + g) * BS]) : u32x4_t{0, 0, 0, 0};
    }
    const int tok = tb + 8 * g;
    const u32x4_t *vp = vpool + static_cast<int64_t>(id.z) * Geo::BLOCK_CHUNKS + (tok % BS) / 8;
#pragma unroll
    for (int nb = 0; nb < 8; ++nb)
      r.v[nb] = tok < t1 ? __builtin_nontemporal_load(&vp[(16 * nb + h) * Geo::PARTS]) : u32x4_t{0, 0, 0, 0};
  };
  auto compute = [&](GqaTile &r, int tb) {
    const bool tail = tb + kGqaTile > t1;
    if (tail) {
      // Slots of tokens >= t1 were never written and may hold NaN/Inf patterns;
      // their probability is 0 but 0 * NaN would still poison the product.
      const int n_ok = t1 - (tb + 8 * g);
#pragma unroll
      for (int nb = 0; nb < 8; ++nb)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          if (2 * c >= n_ok) r.v[nb][c] = 0u;
          else if (2 * c + 1 >= n_ok) r.v[nb][c] &= 0x0000ffffu;
        }
    }
    // ---- S^T = K . Q^T ---------------------------------------------------------
    v4f32_t sacc[2];
#pragma unroll
    for (int tg = 0; tg < 2; ++tg) {
      sacc[tg] = v4f32_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        Frag8 kf;
        kf.u = r.k[tg][s];
        sacc[tg] = mfma16<T>(kf, qf[s], sacc[tg]);
      }
    }
    // ---- online softmax: lane = head h, tokens tb + 16 tg + 4 g + i ----------------
    float mx = -INFINITY;
#pragma unroll
    for (int tg = 0; tg < 2; ++tg)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float sc = sacc[tg][i] * scale_log2;
        if (tail && tb + 16 * tg + 4 * g + i >= t1) sc = -INFINITY;
        sacc[tg][i] = sc;
        mx = fmaxf(mx, sc);
      }
    mx = max_with_lane_xor32(max_with_lane_xor16(mx));   // the step has at least one valid token: finite
    const float m_new = fmaxf(m, mx);
    const float alpha = fast_exp2(m - m_new);
    float psum = 0.f;
#pragma unroll
    for (int tg = 0; tg < 2; ++tg) {
      float p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p[i] = fast_exp2(sacc[tg][i] - m_new);
        psum += p[i];
      }
      const uint32_t w0 = pack_pair<T>(p[0], p[1]), w1 = pack_pair<T>(p[2], p[3]);
      *reinterpret_cast<u32x2_t *>(&p_lds[wave][0][h][16 * tg + 4 * g]) = u32x2_t{w0, w1};
      if constexpr (kParts == 2) {
        const float r0 = p[0] - bf16_lo(w0), r1 = p[1] - bf16_hi(w0);
        const float r2 = p[2] - bf16_lo(w1), r3 = p[3] - bf16_hi(w1);
        *reinterpret_cast<u32x2_t *>(&p_lds[wave][1][h][16 * tg + 4 * g]) =
            u32x2_t{pack_pair<T>(r0, r1), pack_pair<T>(r2, r3)};
      }
    }
    l = l * alpha + psum;
    if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {
#pragma unroll
      for (int nb = 0; nb < 8; ++nb)
#pragma unroll
        for (int i = 0; i < 4; ++i) oacc[nb][i] *= alpha;
    }
    m = m_new;
    wave_lds_sync();
    Frag8 pf[kParts];
#pragma unroll
    for (int part = 0; part < kParts; ++part)
      pf[part].u = *reinterpret_cast<const u32x4_t *>(&p_lds[wave][part][h][8 * g]);
    wave_lds_sync();
    // ---- O^T += V^T . P^T --------------------------------------------------------
#pragma unroll
    for (int nb = 0; nb < 8; ++nb) {
      Frag8 vf;
      vf.u = r.v[nb];
#pragma unroll
      for (int part = 0; part < kParts; ++part) oacc[nb] = mfma16<T>(vf, pf[part], oacc[nb]);
    }
  };

  // One register set per wave and three waves per SIMD: while a wave consumes
  // its step the SIMD's other two have theirs in flight (two sets and two waves
  // per SIMD moved as much on long launches and less on short ones: 76 against
  // 67 us on 16 contexts of 2048-8192 tokens, 46 against 37 us on 64 contexts of
  // 256-1024).  Vector loads return in order, so waiting for a step's block ids
  // also waits for every load issued before them: the ids of step s + 1 are
  // therefore requested BEFORE the K/V loads of step s go out, and waiting for
  // them never waits for K/V that is still wanted in flight.
  int tb = u.t0 + kGqaTile * wave;
  if (tb < t1) {
    GqaTile r;
    int3 ids_next = load_ids(tb);
    while (true) {
      const int3 ids = ids_next;
      const bool more = tb + kStep < t1;
      if (more) ids_next = load_ids(tb + kStep);
      issue(r, tb, ids);
      compute(r, tb);
      if (!more) break;
      tb += kStep;
    }
  }

  // ---- this wave's partial to LDS, in the layout the merge expects ----------------------
  l = sum_with_lane_xor32(sum_with_lane_xor16(l));
  if (h < G && !idle) {
#pragma unroll
    for (int nb = 0; nb < 8; ++nb)
      *reinterpret_cast<float4 *>(&x_acc[wave][h][16 * nb + 4 * g]) =
          make_float4(oacc[nb][0], oacc[nb][1], oacc[nb][2], oacc[nb][3]);
    if (g == 0) {
      x_ml[wave][h][0] = m;
      x_ml[wave][h][1] = l;
    }
  }
  __syncthreads();
  merge_and_write_group<T, G, NW>(I, u, partition, x_acc, x_ml, &sm.arrival, n_active, lane, wave);
  if constexpr (STAY) __syncthreads();      // the partials in LDS are reused by the next unit
  return true;
}

template <typename T, int BS, int G, int NW>
__global__ __launch_bounds__(64 * NW, 3) void paged_decode_gqa_kernel(const DecodeParams P) {
  MUX_TR(0);
  __shared__ GqaSmem<T, G, NW> sm;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int w = blockIdx.x;
  int ii = 0;
#pragma unroll
  for (int k = 1; k < MUXA_MAX_DECODE_ITEMS; ++k)
    if (k < P.n_items && w >= P.it[k].work_begin) ii = k;
  const DecodeItemDev I = P.it[ii];       // by value: one round of scalar loads for every field
  const int WH = I.Hq / G;
  const int local = w - I.work_begin;
  const int e = local / WH;
  Unit u;
  u.item = ii;
  u.wh = local - e * WH;
#ifdef MUX_TRACE
  u.t0 = u.t1 = 0, u.n_splits = 0;       // (a workgroup that finds no unit reports no tokens)
#endif
  decode_unit_gqa<T, BS, G, NW, false>(P, I, u, e, sm, lane, wave);
  // (tracing build: the matrix-core kernel stamps its entry and its end only)
  MUX_TR(6);
  MUX_TRV(7, static_cast<long long>(u.t1 - u.t0) | (static_cast<long long>(u.n_splits > 1) << 16));
}

// (pairs that got no place in the grid: see paged_decode_sweep_kernel)
template <typename T, int BS, int G, int NW>
__global__ __launch_bounds__(64 * NW, 3) void paged_decode_gqa_sweep_kernel(const DecodeParams P) {
  __shared__ GqaSmem<T, G, NW> sm;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int w = blockIdx.x;
  int ii = 0;
#pragma unroll
  for (int k = 1; k < MUXA_MAX_DECODE_ITEMS; ++k)
    if (k < P.n_items && w >= P.it[k].work_begin) ii = k;
  const DecodeItemDev I = P.it[ii];
  Unit u;
  u.item = ii;
  u.wh = w - I.work_begin;
  for (int e = I.pair_begin;; ++e)
    if (!decode_unit_gqa<T, BS, G, NW, true>(P, I, u, e, sm, lane, wave)) return;
}



// Zero-fills the arrival counters (a kernel rather than a memset node so the
// call can be captured into a graph).
__global__ void fill_zero_kernel(int32_t *p, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
namespace {

int pick_group(int ratio);

// Tokens per partition when the caller leaves the choice to the library: short
// partitions spread the batch over more workgroups, long ones amortise a unit's
// fixed cost and split fewer contexts.
int choose_partition(const MuxDecodeItem *items, int n_items, int requested) {
  if (requested > 0) return requested;
  int max_ctx = 0;
  bool all_grouped = true;
  // Tokens x head groups of the launch: the caller's bound on the sum of the
  // context lengths where it gave one, half the longest context per sequence
  // where it did not.
  int64_t token_heads = 0;
  for (int i = 0; i < n_items; ++i) {
    const MuxDecodeItem &it = items[i];
    max_ctx = std::max(max_ctx, it.max_context_len);
    const int group = it.num_kv_heads > 0 ? pick_group(it.num_q_heads / it.num_kv_heads) : 1;
    if (it.num_kv_heads <= 0 || group < 4) all_grouped = false;
    const int64_t tokens = it.total_context_len > 0
                               ? it.total_context_len
                               : static_cast<int64_t>(it.num_seqs) * (it.max_context_len / 2);
    token_heads += tokens * (it.num_q_heads / std::max(group, 1));
  }
  // Grouped-query launches: as many tokens per unit as a workgroup slot's share
  // of the launch (three workgroups on each of the 256 compute units), so that
  // the units fill the chip about once and few contexts are split at all; never
  // under 256.  Against the 1024 / 256 tokens used before: 230 against 237 us on
  // 64 contexts of 2048-8192 tokens, 245 against 315 us on 512 of 256-1024, 19.5
  // against 26 us on two long ones (their units now fill a fifth of the chip
  // instead of a twentieth).
  if (all_grouped) {
    constexpr int64_t kSlots = 3 * 256;
    const int64_t per_slot = (token_heads / kSlots + 255) / 256 * 256;
    return static_cast<int>(std::min<int64_t>(std::max<int64_t>(per_slot, 256), 1 << 20));
  }
  if (max_ctx > 4096) return 512;
  // A large launch does better with long partitions (fewer units, hardly any
  // hand-off: 1 - 6 % over launches of 0.8 - 1.7 GB of K/V, one model or three);
  // a small one needs the many short units to fill the chip and to end evenly
  // (1024-token partitions: +1 to +15 % there).
  if (token_heads >= 1500000) return 1024;
  return 256;
}

// The other two knobs of seq_units.  Measured on the mixed three-model batch
// (interleaved runs in one process, medians of eight): units of two to four
// groups per workgroup 79 - 80 us against 74.5 with one (a wave's second round
// starts with nothing in flight); a remainder of at most 8 / 16 / 24 tokens left
// to the last unit 73.6 - 73.7 us against 74.1 - 74.5 without (32: 74.4, 64:
// 74.7): a remainder of one pool block is cheaper as one more short round of one
// wave than as a workgroup of its own with its own partial and hand-off.
struct DecodePolicy {
  int rounds, absorb;
};
DecodePolicy choose_policy(const MuxDecodeItem *, int, int) { return DecodePolicy{1, 16}; }

int pick_group(int ratio) {
  if (ratio == 8 || ratio == 4 || ratio == 2) return ratio;
  if (ratio % 16 == 0) return 16;
  if (ratio % 8 == 0) return 8;
  if (ratio % 4 == 0) return 4;
  if (ratio % 2 == 0) return 2;
  return 1;
}

struct ItemPlan {
  size_t counters_off, acc_off, ml_off;
  int max_splits;
  int64_t units;      // (sequence, unit) pairs that get a place in the grid of a device-enumerated launch
  size_t table_off;   // pair table of a large batch (0: none)
};

// Workspace layout: a FIXED leading region of MUXA_DECODE_COUNTER_BYTES holds
// the arrival counters (one int32 per sequence and head group, items back to
// back) so that its position never depends on the shapes of a call and no
// call's partials can land on another call's counters; then per item acc
// [B,Hq,max_splits,128] fp32 and ml [B,Hq,max_splits,2] fp32, and for batches
// of more than 64 * kLocateChunks sequences the pair table (16 bytes per pair).
// Calls whose contexts all fit one partition and whose batches are small need no
// workspace.  Returns total bytes, or SIZE_MAX when the counters do not fit the
// fixed region.
size_t plan_workspace(const MuxDecodeItem *items, int n_items, int partition, ItemPlan *out) {
  size_t counters = 0;
  size_t off = MUXA_DECODE_COUNTER_BYTES;
  bool any = false;
  for (int i = 0; i < n_items; ++i) {
    const MuxDecodeItem &it = items[i];
    ItemPlan w{0, 0, 0, std::max(1, (it.max_context_len + partition - 1) / partition), 0, 0};
    // Upper bound on the number of pairs: every sequence has at most
    // max_splits of them, and all sequences together at most
    // floor(sum ctx / partition) full ones plus one remainder each.
    w.units = static_cast<int64_t>(it.num_seqs) * w.max_splits;
    if (it.total_context_len > 0)
      w.units = std::min<int64_t>(w.units, it.total_context_len / partition + it.num_seqs);
    if (w.max_splits > 1 && it.num_seqs > 0) {
      any = true;
      const int G = pick_group(it.num_q_heads / it.num_kv_heads);
      w.counters_off = counters;
      counters += static_cast<size_t>(it.num_seqs) * (it.num_q_heads / G) * sizeof(int32_t);
      const size_t rows = static_cast<size_t>(it.num_seqs) * it.num_q_heads * w.max_splits;
      w.acc_off = off;
      off += rows * kHeadSize * sizeof(float);
      w.ml_off = off;
      off += rows * 2 * sizeof(float);
      off = (off + 255) & ~static_cast<size_t>(255);
    }
    if (it.num_seqs > 64 * kLocateChunks && it.max_context_len > 0) {
      // A row for every pair there can be, whatever the caller's bound on the sum
      // says: the bound only sizes the grid, and pairs it leaves without a place
      // are still found in the table (by the sweep of the kernels).
      any = true;
      w.table_off = off;
      off += static_cast<size_t>(it.num_seqs) * w.max_splits * sizeof(int4);
      off = (off + 255) & ~static_cast<size_t>(255);
    }
    if (out) out[i] = w;
  }
  if (!any) return 0;
  if (counters > MUXA_DECODE_COUNTER_BYTES) return SIZE_MAX;
  return off;
}

// Host-side enumeration of one item's (sequence, unit) pairs, in the classes the
// device-side enumeration (locate_pair_small) uses: remainder units of split
// contexts, their other units, then the contexts with a single unit.  Appends
// to out[*n]; false when they do not fit the kernel argument's table or its
// 16-bit fields.
bool enumerate_pairs_on_host(const int32_t *ctx_host, int B, int max_ctx, int partition, int rounds, int absorb,
                             uint2 *out, int *n, int *first_single_out = nullptr) {
  if (B > 0xffff) return false;
  auto clamped = [&](int s) { return std::max(std::min(ctx_host[s], max_ctx), 0); };
  int at = *n;
  auto push = [&](int s, int split, int c) {
    if (at >= kMaxHostPairs || split > 0xffff) return false;
    out[at++] = make_uint2(static_cast<uint32_t>(s) | (static_cast<uint32_t>(split) << 16), static_cast<uint32_t>(c));
    return true;
  };
  for (int s = 0; s < B; ++s) {
    const int c = clamped(s);
    const SeqUnits su = seq_units(c, partition, rounds, absorb);
    if (su.count() > 1 && su.rem > 0 && !push(s, su.nb, c)) return false;
  }
  // (the remainders longest first: the same units, in the order that leaves the
  // short ones for when the others are under way; long-context grouped-query
  // batches 0.8 % faster, the three-model mix -0.7 to +0.2 us)
  {
    const uint32_t P = static_cast<uint32_t>(partition);
    std::stable_sort(out + *n, out + at, [P](const uint2 &a, const uint2 &b) { return a.y % P > b.y % P; });
  }
  for (int s = 0; s < B; ++s) {
    const int c = clamped(s);
    const SeqUnits su = seq_units(c, partition, rounds, absorb);
    if (su.count() > 1)
      for (int j = 0; j < su.nb; ++j)
        if (!push(s, j, c)) return false;
  }
  // The single-unit contexts end the item (and the last item's end the launch):
  // longest first, so that what is still running at the very end is short.  The
  // units are the same in any order, and so are the results.
  const int first_single = at;
  for (int s = 0; s < B; ++s) {
    const int c = clamped(s);
    if (c > 0 && seq_units(c, partition, rounds, absorb).count() == 1 && !push(s, 0, c)) return false;
  }
  std::stable_sort(out + first_single, out + at, [](const uint2 &a, const uint2 &b) { return a.y > b.y; });
  if (first_single_out) *first_single_out = first_single;
  *n = at;
  return true;
}

template <typename T, int BS, int G>
hipError_t launch_g(const DecodeParams &P, int grid, bool sweep, hipStream_t st) {
  constexpr int NW = kWavesPerGroup;
  if (sweep) hipLaunchKernelGGL((paged_decode_sweep_kernel<T, BS, G, NW>), dim3(grid), dim3(64 * NW), 0, st, P);
  else hipLaunchKernelGGL((paged_decode_kernel<T, BS, G, NW>), dim3(grid), dim3(64 * NW), 0, st, P);
  return hipGetLastError();
}

template <typename T, int BS, int G>
hipError_t launch_gqa(const DecodeParams &P, int grid, bool sweep, hipStream_t st) {
  constexpr int NW = kWavesPerGroup;
  if (sweep) hipLaunchKernelGGL((paged_decode_gqa_sweep_kernel<T, BS, G, NW>), dim3(grid), dim3(64 * NW), 0, st, P);
  else hipLaunchKernelGGL((paged_decode_gqa_kernel<T, BS, G, NW>), dim3(grid), dim3(64 * NW), 0, st, P);
  return hipGetLastError();
}

template <typename T, int BS>
hipError_t launch_main(int G, const DecodeParams &P, int grid, bool sweep, hipStream_t st) {
  switch (G) {
    case 1: return launch_g<T, BS, 1>(P, grid, sweep, st);
    case 2: return launch_g<T, BS, 2>(P, grid, sweep, st);
    case 4: return launch_gqa<T, BS, 4>(P, grid, sweep, st);
    case 8: return launch_gqa<T, BS, 8>(P, grid, sweep, st);
    case 16: return launch_gqa<T, BS, 16>(P, grid, sweep, st);
    default: return hipErrorInvalidValue;
  }
}

template <typename T>
hipError_t launch_bs(int BS, int G, const DecodeParams &P, int grid, bool sweep, hipStream_t st) {
  switch (BS) {
    case 8: return launch_main<T, 8>(G, P, grid, sweep, st);
    case 16: return launch_main<T, 16>(G, P, grid, sweep, st);
    case 32: return launch_main<T, 32>(G, P, grid, sweep, st);
    default: return hipErrorInvalidValue;
  }
}

int32_t validate_item(const MuxDecodeItem &it, int block_size) {
  // (pointers are only required when the item has sequences)
  if (it.num_seqs > 0 && (!it.out || !it.q || !it.block_tables || !it.context_lens)) return MUXA_EINVAL;
  if (it.num_seqs < 0 || it.num_q_heads <= 0 || it.num_kv_heads <= 0) return MUXA_EINVAL;
  if (it.num_q_heads % it.num_kv_heads != 0) return MUXA_EINVAL;
  if (it.layer < 0 || it.layer >= it.num_layers) return MUXA_EINVAL;
  if (it.max_blocks < 0 || it.max_context_len < 0 || it.total_context_len < 0) return MUXA_EINVAL;
  // The grid is sized from max_context_len and every table row must be able
  // to hold that many tokens.
  if (static_cast<int64_t>(it.max_context_len) > static_cast<int64_t>(it.max_blocks) * block_size)
    return MUXA_EINVAL;
  const int64_t width = static_cast<int64_t>(it.num_q_heads) * kHeadSize;
  if (it.q_row_stride < width || it.out_row_stride < width) return MUXA_EINVAL;
  // Packed-pair q loads and 2-byte output stores.
  if (it.q_row_stride % 2 != 0 || (reinterpret_cast<uintptr_t>(it.q) & 3u) != 0) return MUXA_EINVAL;
  if ((reinterpret_cast<uintptr_t>(it.out) & 1u) != 0) return MUXA_EINVAL;
  return MUXA_OK;
}

}  // namespace
}  // namespace mux

extern "C" {

size_t mux_paged_decode_workspace_bytes(const MuxDecodeItem *items, int32_t n_items,
                                        int32_t partition_size) {
  if (!items || n_items <= 0 || n_items > MUXA_MAX_DECODE_ITEMS) return 0;
  const int partition = mux::choose_partition(items, n_items, partition_size);
  size_t need = mux::plan_workspace(items, n_items, partition, nullptr);
  // Where the library chooses, the choice may change from launch to launch with
  // the caller's bound on the context sum: size for the shortest partition it picks.
  if (partition_size == 0 && partition > 256 && need != SIZE_MAX) {
    const size_t need_short = mux::plan_workspace(items, n_items, 256, nullptr);
    if (need_short != SIZE_MAX && need_short > need) need = need_short;
  }
  return need;
}

int32_t mux_paged_decode_host_pairs(const MuxDecodeItem *items, int32_t n_items, int32_t partition_size) {
  using namespace mux;
  if (!items || n_items <= 0 || n_items > MUXA_MAX_DECODE_ITEMS) return 0;
  if (partition_size < 0 || partition_size % 64 != 0) return 0;
  for (int i = 0; i < n_items; ++i)
    if (items[i].num_kv_heads <= 0 || items[i].num_q_heads <= 0 || items[i].num_q_heads % items[i].num_kv_heads != 0)
      return 0;
  const int partition = choose_partition(items, n_items, partition_size);
  const DecodePolicy pol = choose_policy(items, n_items, partition);
  // The first launch group: the items that share the first item's head grouping.
  const int G = pick_group(items[0].num_q_heads / items[0].num_kv_heads);
  uint2 pairs[kMaxHostPairs];
  int n_pairs = 0;
  for (int i = 0; i < n_items; ++i) {
    const MuxDecodeItem &it = items[i];
    if (pick_group(it.num_q_heads / it.num_kv_heads) != G) continue;
    if (it.num_seqs <= 0 || it.max_context_len <= 0) continue;
    if (!it.context_lens_host ||
        !enumerate_pairs_on_host(it.context_lens_host, it.num_seqs, it.max_context_len, partition, pol.rounds,
                                 pol.absorb, pairs, &n_pairs))
      return 0;
  }
  return n_pairs;
}

int32_t mux_paged_decode_workspace_init(void *workspace, size_t workspace_bytes, void *stream) {
  if (!workspace || workspace_bytes == 0) return MUXA_OK;
  if (reinterpret_cast<uintptr_t>(workspace) & 15u) return MUXA_EINVAL;
  const int64_t n = static_cast<int64_t>(std::min<size_t>(workspace_bytes, MUXA_DECODE_COUNTER_BYTES) /
                                        sizeof(int32_t));
  if (n == 0) return MUXA_OK;
  hipLaunchKernelGGL(mux::fill_zero_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<int32_t *>(workspace), n);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return mux::hip_fail(e);
  return MUXA_OK;
}

}  // extern "C"

namespace mux {
namespace {

// Everything about a call that can be refused before anything is launched.
int32_t validate_call(const MuxDecodeItem *items, int32_t n_items, const void *k_pool, const void *v_pool,
                      int64_t num_pool_blocks, int32_t head_size, int32_t block_size, int32_t dtype,
                      int32_t partition_size) {
  if (!items || n_items <= 0 || n_items > MUXA_MAX_DECODE_ITEMS) return MUXA_EINVAL;
  if (!k_pool || !v_pool || num_pool_blocks <= 0) return MUXA_EINVAL;
  if ((reinterpret_cast<uintptr_t>(k_pool) & 15u) || (reinterpret_cast<uintptr_t>(v_pool) & 15u))
    return MUXA_EINVAL;
  if (head_size != kHeadSize) return MUXA_EUNSUPPORTED;
  if (block_size != 8 && block_size != 16 && block_size != 32) return MUXA_EUNSUPPORTED;
  if (dtype != MUXA_DTYPE_F16 && dtype != MUXA_DTYPE_BF16) return MUXA_EUNSUPPORTED;
  if (partition_size < 0 || partition_size % 64 != 0) return MUXA_EINVAL;
  for (int i = 0; i < n_items; ++i) {
    const int32_t rc = validate_item(items[i], block_size);
    if (rc != MUXA_OK) return rc;
  }
  return MUXA_OK;
}

int32_t multi_decode_impl(const MuxDecodeItem *items, int32_t n_items,
                          const void *k_pool, const void *v_pool, int64_t num_pool_blocks,
                          int32_t head_size, int32_t block_size, int32_t dtype,
                          int32_t partition_size, void *workspace, size_t workspace_bytes,
                          void *stream) {
  const int32_t vrc = validate_call(items, n_items, k_pool, v_pool, num_pool_blocks, head_size, block_size, dtype,
                                    partition_size);
  if (vrc != MUXA_OK) return vrc;
  const int partition = choose_partition(items, n_items, partition_size);
  const DecodePolicy pol = choose_policy(items, n_items, partition);
  const int rounds = pol.rounds, absorb = pol.absorb;
  ItemPlan plan[MUXA_MAX_DECODE_ITEMS];
  const size_t need = plan_workspace(items, n_items, partition, plan);
  if (need == SIZE_MAX) return MUXA_EUNSUPPORTED;   // more (sequence, head group) pairs than counters
  if (need > 0 && (!workspace || workspace_bytes < need)) return MUXA_EWORKSPACE;
  if (need > 0 && (reinterpret_cast<uintptr_t>(workspace) & 15u)) return MUXA_EINVAL;
  hipStream_t st = static_cast<hipStream_t>(stream);
  char *ws = static_cast<char *>(workspace);

  // Items are launched in groups that share G (query heads per workgroup).
  // Within a launch the items' workgroups follow each other, the item with the
  // most sequences last: its many single-unit contexts, the cheapest units of the
  // launch, are then what the launch ends with (the three-model mix over four
  // sets of batches: 0.2 - 1.2 % faster than in the caller's order, which had the
  // largest batch first; no result depends on the order).
  int order[MUXA_MAX_DECODE_ITEMS];
  for (int i = 0; i < n_items; ++i) order[i] = i;
  std::stable_sort(order, order + n_items,
                   [&](int a, int b) { return items[a].num_seqs < items[b].num_seqs; });
  bool done[MUXA_MAX_DECODE_ITEMS] = {false};
  for (int of = 0; of < n_items; ++of) {
    const int first = order[of];
    if (done[first]) continue;
    const int G = pick_group(items[first].num_q_heads / items[first].num_kv_heads);
    DecodeParams P = {};
    PlanParams PP;
    PP.partition = partition;
    PP.rounds = rounds;
    PP.absorb = absorb;
    int n_tables = 0;
    P.k_pool = k_pool;
    P.v_pool = v_pool;
    P.partition = partition;
    P.rounds = rounds;
    P.absorb = absorb;
    P.last_block = static_cast<int32_t>(std::min<int64_t>(num_pool_blocks - 1, 0x7fffffff));
    P.n_items = 0;
    P.n_host_pairs = 0;
    // Host-enumerated units: every item of the launch group must come with its
    // context lengths on the host, and the pairs must fit the kernel argument.
    int pair_begin[MUXA_MAX_DECODE_ITEMS] = {0}, pair_end[MUXA_MAX_DECODE_ITEMS] = {0};
    int pair_single[MUXA_MAX_DECODE_ITEMS] = {0};          // the item's first single-unit context
    bool host_pairs = true;
    {
      int n_pairs = 0;
      for (int oi = of; oi < n_items && host_pairs; ++oi) {
        const int i = order[oi];
        const MuxDecodeItem &it = items[i];
        if (done[i] || pick_group(it.num_q_heads / it.num_kv_heads) != G) continue;
        if (it.num_seqs == 0 || it.max_context_len == 0) continue;
        pair_begin[i] = n_pairs;
        host_pairs = it.context_lens_host != nullptr &&
                     enumerate_pairs_on_host(it.context_lens_host, it.num_seqs, it.max_context_len, partition,
                                             rounds, absorb, P.pairs, &n_pairs, &pair_single[i]);
        pair_end[i] = n_pairs;
      }
      host_pairs = host_pairs && n_pairs > 0;
      if (host_pairs) P.n_host_pairs = n_pairs;
    }
    int64_t work = 0;
    bool tightened = false;
    // What every descriptor of an item has in common.
    auto describe = [&](DecodeItemDev &d, int i) {
      const MuxDecodeItem &it = items[i];
      const bool split = plan[i].max_splits > 1;
      d.out = it.out;
      d.q = it.q;
      d.out_stride = it.out_row_stride;
      d.q_stride = it.q_row_stride;
      d.tables = it.block_tables +
                 static_cast<int64_t>(it.layer) * it.num_seqs * it.num_kv_heads * it.max_blocks;
      d.ctx = it.context_lens;
      d.ws_acc = split ? reinterpret_cast<float *>(ws + plan[i].acc_off) : nullptr;
      d.ws_ml = split ? reinterpret_cast<float *>(ws + plan[i].ml_off) : nullptr;
      d.counters = split ? reinterpret_cast<int32_t *>(ws + plan[i].counters_off) : nullptr;
      d.unit_table = nullptr;
      d.B = it.num_seqs;
      d.Hq = it.num_q_heads;
      d.Hkv = it.num_kv_heads;
      d.ratio = it.num_q_heads / it.num_kv_heads;
      d.max_blocks = it.max_blocks;
      d.max_splits = plan[i].max_splits;
      d.max_ctx = it.max_context_len;
      d.scale_log2 = it.scale * 1.4426950408889634f;
    };
    int members[MUXA_MAX_DECODE_ITEMS], n_members = 0;
    for (int oi = of; oi < n_items; ++oi) {
      const int i = order[oi];
      if (done[i]) continue;
      const MuxDecodeItem &it = items[i];
      if (pick_group(it.num_q_heads / it.num_kv_heads) != G) continue;
      done[i] = true;
      if (it.num_seqs == 0 || it.max_context_len == 0) continue;
      members[n_members++] = i;
    }
    if (host_pairs) {
      // The grid holds exactly the enumerated pairs; no table, no padding.  A
      // descriptor is a run of pairs of one model; with room for two per model the
      // units of split contexts of ALL models come first and the single-unit
      // contexts of all models after them, so that the launch as a whole - not each
      // model's stretch of it - ends with its cheapest units.
      const bool two_runs = 2 * n_members <= MUXA_MAX_DECODE_ITEMS;
      for (int pass = 0; pass < (two_runs ? 2 : 1); ++pass)
        for (int m = 0; m < n_members; ++m) {
          const int i = members[m];
          const int lo = two_runs && pass == 1 ? pair_single[i] : pair_begin[i];
          const int hi = two_runs && pass == 0 ? pair_single[i] : pair_end[i];
          if (hi <= lo) continue;
          DecodeItemDev &d = P.it[P.n_items++];
          describe(d, i);
          d.pair_begin = lo;
          d.work_begin = static_cast<int32_t>(work);
          work += static_cast<int64_t>(hi - lo) * (items[i].num_q_heads / G);
        }
    } else {
      for (int m = 0; m < n_members; ++m) {
        const int i = members[m];
        const MuxDecodeItem &it = items[i];
        DecodeItemDev &d = P.it[P.n_items++];
        describe(d, i);
        if (plan[i].table_off != 0) {
          const int64_t rows = static_cast<int64_t>(it.num_seqs) * plan[i].max_splits;
          if (rows > 0x7fffffff) return MUXA_EUNSUPPORTED;
          PlanItem &t = PP.it[n_tables++];
          t.ctx = it.context_lens;
          t.table = reinterpret_cast<int4 *>(ws + plan[i].table_off);
          t.B = it.num_seqs;
          t.max_ctx = it.max_context_len;
          t.capacity = static_cast<int32_t>(rows);
          d.unit_table = t.table;
        }
        d.work_begin = static_cast<int32_t>(work);
        if (plan[i].units > 0x7fffffff) return MUXA_EUNSUPPORTED;
        d.pair_begin = static_cast<int32_t>(plan[i].units);       // pairs with a place in the grid
        if (plan[i].units < static_cast<int64_t>(it.num_seqs) * plan[i].max_splits) tightened = true;
        work += plan[i].units * (it.num_q_heads / G);
        if (work > 0x7fffffff) return MUXA_EUNSUPPORTED;
      }
    }
    if (P.n_items == 0) continue;
    if (n_tables > 0) {
      hipLaunchKernelGGL(decode_plan_kernel, dim3(n_tables), dim3(256), 0, st, PP);
      hipError_t pe = hipGetLastError();
      if (pe != hipSuccess) return hip_fail(pe);
    }
    const int grid = static_cast<int>(work);
    hipError_t e = dtype == MUXA_DTYPE_F16 ? launch_bs<F16>(block_size, G, P, grid, false, st)
                                           : launch_bs<BF16>(block_size, G, P, grid, false, st);
    if (e != hipSuccess) return hip_fail(e);
    // Where the caller's bound on the sum of the context lengths made the grid
    // smaller than the shapes allow, the pairs it may have left out are swept
    // up behind the launch: one workgroup per item and head group.
    if (tightened) {
      int sweep_grid = 0;
      for (int k = 0; k < P.n_items; ++k) {
        P.it[k].work_begin = sweep_grid;
        sweep_grid += P.it[k].Hq / G;
      }
      e = dtype == MUXA_DTYPE_F16 ? launch_bs<F16>(block_size, G, P, sweep_grid, true, st)
                                  : launch_bs<BF16>(block_size, G, P, sweep_grid, true, st);
      if (e != hipSuccess) return hip_fail(e);
    }
  }
  return MUXA_OK;
}

}  // namespace
}  // namespace mux

// Scratch of the allocation-free entry point: one copy per GPU the library's
// code object is loaded on, held until the process ends.  Host code must not
// use this name as an address; it asks the runtime for the device address once
// per device (static_scratch_base) and passes that pointer on.
static __device__ __align__(256) unsigned char scratch[MUXA_STATIC_SCRATCH_BYTES];

namespace mux {
namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {nullptr};

// Device address of `scratch` on the current device, looked up on the first
// call per device.  Returns MUXA_OK and sets *out, or a negative code.
int32_t static_scratch_base(void **out) {
  int dev = -1;
  MUX_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return MUXA_EUNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void *ptr = nullptr;
    MUX_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) return MUXA_EHIP;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return MUXA_OK;
}

}  // namespace
}  // namespace mux

extern "C" {

int32_t mux_multi_decode(const MuxDecodeItem *items, int32_t n_items,
                         const void *k_pool, const void *v_pool, int64_t num_pool_blocks,
                         int32_t head_size, int32_t block_size, int32_t dtype,
                         int32_t partition_size, void *workspace, size_t workspace_bytes,
                         void *stream) {
  return mux::multi_decode_impl(items, n_items, k_pool, v_pool, num_pool_blocks, head_size, block_size, dtype,
                                partition_size, workspace, workspace_bytes, stream);
}

size_t mux_multi_decode_noalloc_max_bytes(void) { return MUXA_STATIC_SCRATCH_BYTES; }

int32_t mux_multi_decode_noalloc(const MuxDecodeItem *items, int32_t n_items,
                                 const void *k_pool, const void *v_pool, int64_t num_pool_blocks,
                                 int32_t head_size, int32_t block_size, int32_t dtype,
                                 int32_t partition_size, void *stream) {
  using namespace mux;
  // Every check the launch makes is made first: a refused call has launched nothing.
  const int32_t vrc = validate_call(items, n_items, k_pool, v_pool, num_pool_blocks, head_size, block_size, dtype,
                                    partition_size);
  if (vrc != MUXA_OK) return vrc;
  // The call's scratch need against the fixed size of the static array.
  const int partition = choose_partition(items, n_items, partition_size);
  const size_t need = plan_workspace(items, n_items, partition, nullptr);
  if (need == SIZE_MAX) return MUXA_EUNSUPPORTED;
  if (need > MUXA_STATIC_SCRATCH_BYTES) return MUXA_ESCRATCH_LIMIT;
  void *base = nullptr;
  const int32_t rc = static_scratch_base(&base);
  if (rc != MUXA_OK) return rc;
  if (need > 0) {
    // The array keeps the previous call's contents.  Partials and the pair
    // table are written before they are read; the arrival counters must start
    // at zero and every completed launch leaves them so, but a launch that was
    // cut short would not - so they are cleared here, with a fill kernel (a
    // memset node must not end up in a captured graph).
    const int32_t irc = mux_paged_decode_workspace_init(base, MUXA_DECODE_COUNTER_BYTES, stream);
    if (irc != MUXA_OK) return irc;
  }
  return multi_decode_impl(items, n_items, k_pool, v_pool, num_pool_blocks, head_size, block_size, dtype,
                           partition_size, need > 0 ? base : nullptr, need > 0 ? MUXA_STATIC_SCRATCH_BYTES : 0,
                           stream);
}

int32_t mux_paged_decode(void *out, int64_t out_row_stride, const void *q, int64_t q_row_stride,
                         const void *k_pool, const void *v_pool, int64_t num_pool_blocks,
                         const int32_t *block_tables, const int32_t *context_lens,
                         int32_t layer, int32_t num_layers, int32_t num_seqs,
                         int32_t num_q_heads, int32_t num_kv_heads, int32_t head_size,
                         int32_t block_size, int32_t max_blocks, int32_t max_context_len,
                         float scale, int32_t dtype, int32_t partition_size,
                         void *workspace, size_t workspace_bytes, void *stream) {
  MuxDecodeItem it = {};     // every field the wrapper does not name (context_lens_host, ...) is null / zero
  it.out = out;
  it.q = q;
  it.out_row_stride = out_row_stride;
  it.q_row_stride = q_row_stride;
  it.block_tables = block_tables;
  it.context_lens = context_lens;
  it.total_context_len = 0;
  it.layer = layer;
  it.num_layers = num_layers;
  it.num_seqs = num_seqs;
  it.num_q_heads = num_q_heads;
  it.num_kv_heads = num_kv_heads;
  it.max_blocks = max_blocks;
  it.max_context_len = max_context_len;
  it.scale = scale;
  return mux_multi_decode(&it, 1, k_pool, v_pool, num_pool_blocks, head_size, block_size, dtype,
                          partition_size, workspace, workspace_bytes, stream);
}

}  // extern "C"

#ifdef MUX_TRACE
// Tracing build only: where the decode kernel's workgroups write their stamps
// (DEVICE int64 [rows, 8], zero-filled by the caller; NULL switches it off).
extern "C" int32_t mux_decode_trace_set(void *table, int64_t rows) {
  long long *p = static_cast<long long *>(table);
  long long n = table ? rows : 0;
  MUX_HIP_TRY(hipMemcpyToSymbol(HIP_SYMBOL(mux::g_decode_trace), &p, sizeof(p)));
  MUX_HIP_TRY(hipMemcpyToSymbol(HIP_SYMBOL(mux::g_decode_trace_rows), &n, sizeof(n)));
  return MUXA_OK;
}
#endif
