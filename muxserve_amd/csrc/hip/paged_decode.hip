// Paged decode attention over the head-granular KV pool, gfx950.
//
// Work unit = one wave64 = (model, sequence, group of G query heads that share
// a kv head, partition of the context).  A wave walks its partition in tiles
// of 64 tokens:
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
// first use, which is what keeps HBM busy; arithmetic is <15% of VALU time.
//
// Contexts longer than `partition` tokens are split; partials (max, sum,
// unnormalised acc) go to the workspace and a second small kernel combines
// them.  Sequences that fit one partition write their output directly.
//
// Several models (different head counts, tables, q/out tensors) are covered by
// one grid: the kernel argument carries up to MUXA_MAX_DECODE_ITEMS item
// descriptors and each wave finds its item from its block index.
#include "mux_common.h"

#include <algorithm>

namespace mux {

thread_local int32_t g_last_hip_error = 0;

struct DecodeItemDev {
  void *out;
  const void *q;
  int64_t out_stride, q_stride;   // elements per row
  const int32_t *tables;          // layer slice [B, Hkv, max_blocks]
  const int32_t *ctx;             // [B]
  float *ws_acc;                  // [B, Hq, max_splits, 128]
  float *ws_ml;                   // [B, Hq, max_splits, 2]  (running max in log2 units, sum)
  int32_t B, Hq, Hkv, ratio;      // ratio = Hq / Hkv
  int32_t max_blocks, max_splits, max_ctx;
  int32_t work_begin;             // first block of this item in the main grid
  int32_t row_begin;              // first (seq, hq) row of this item in the reduce grid
  float scale_log2;               // scale * log2(e)
};

struct DecodeParams {
  DecodeItemDev it[MUXA_MAX_DECODE_ITEMS];
  const void *k_pool;
  const void *v_pool;
  int32_t n_items;
  int32_t partition;
  int32_t last_block;             // num_pool_blocks - 1: table entries are clamped to it
};

template <typename T, int BS, int G>
__global__ __launch_bounds__(64) void paged_decode_kernel(const DecodeParams P) {
  constexpr int D = kHeadSize;
  constexpr int BPT = 64 / BS;               // blocks per tile
  constexpr int PARTS = BS / 8;              // 16-byte chunks per V row of a block
  constexpr int VI = D * PARTS / 64;         // V load instructions per block
  constexpr int BLOCK_CHUNKS = D * BS / 8;   // 16-byte chunks per K block (same for V)
  static_assert(BS == 8 || BS == 16 || BS == 32, "block size");

  __shared__ __attribute__((aligned(16))) float p_lds[G][64];
  __shared__ __attribute__((aligned(16))) uint32_t q_lds[G][64];

  const int lane = threadIdx.x;
  const int w = blockIdx.x;
  int ii = 0;
#pragma unroll
  for (int k = 1; k < MUXA_MAX_DECODE_ITEMS; ++k)
    if (k < P.n_items && w >= P.it[k].work_begin) ii = k;
  const DecodeItemDev &I = P.it[ii];

  const int WH = I.Hq / G;                   // work heads per sequence
  const int local = w - I.work_begin;
  const int per_split = I.B * WH;
  const int split = local / per_split;
  const int r = local - split * per_split;
  const int seq = r / WH;
  const int wh = r - seq * WH;
  const int hq0 = wh * G;
  const int hk = hq0 / I.ratio;
  const int ctx = min(I.ctx[seq], I.max_ctx);
  const int partition = P.partition;
  const int t0 = split * partition;
  if (t0 >= ctx) return;
  const int t1 = min(ctx, t0 + partition);
  const bool single = ctx <= partition;

  // ---- q: 128 dims = 64 packed pairs per head --------------------------------
  const uint32_t *qrow = reinterpret_cast<const uint32_t *>(
      static_cast<const uint16_t *>(I.q) + static_cast<int64_t>(seq) * I.q_stride + hq0 * D);
  uint32_t q_s[64];   // G == 1: the head's q, uniform across lanes (lives in SGPRs)
  if constexpr (G == 1) {
    const uint32_t qv = qrow[lane];
#pragma unroll
    for (int i = 0; i < 64; ++i) q_s[i] = __builtin_amdgcn_readlane(qv, i);
  } else {
#pragma unroll
    for (int g = 0; g < G; ++g) q_lds[g][lane] = qrow[g * 64 + lane];
    __syncthreads();
  }

  const int32_t *trow = I.tables + (static_cast<int64_t>(seq) * I.Hkv + hk) * I.max_blocks;
  const uint4 *kpool = static_cast<const uint4 *>(P.k_pool);
  const uint4 *vpool = static_cast<const uint4 *>(P.v_pool);
  const float scale_log2 = I.scale_log2;
  const int part = lane % PARTS;

  float m[G], l[G], acc[G][VI];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int j = 0; j < VI; ++j) acc[g][j] = 0.f;
  }

  for (int tb = t0; tb < t1; tb += 64) {
    const int tok = tb + lane;
    const bool valid = tok < t1;
    int id = 0;
    // Clamp so that a corrupt table entry reads the wrong block instead of
    // faulting the GPU.
    if (valid) id = min(max(trow[tok / BS], 0), P.last_block);

    // ---- issue every load of the tile ---------------------------------------
    uint4 kreg[16];
    if (valid) {
      const uint4 *kp = kpool + static_cast<int64_t>(id) * BLOCK_CHUNKS + (tok % BS);
#pragma unroll
      for (int j = 0; j < 16; ++j) kreg[j] = kp[j * BS];
    } else {
#pragma unroll
      for (int j = 0; j < 16; ++j) kreg[j] = make_uint4(0, 0, 0, 0);
    }
    uint4 vreg[BPT][VI];
#pragma unroll
    for (int b = 0; b < BPT; ++b) {
      const int idb = __builtin_amdgcn_readlane(id, b * BS);
      const uint4 *vp = vpool + static_cast<int64_t>(idb) * BLOCK_CHUNKS + lane;
      const bool chunk_ok = tb + b * BS + part * 8 < t1;
#pragma unroll
      for (int j = 0; j < VI; ++j) {
        if (chunk_ok) vreg[b][j] = vp[j * 64];
        else vreg[b][j] = make_uint4(0, 0, 0, 0);
      }
    }
    // Tail tile: zero V elements of tokens >= t1 (their probability is 0 but
    // the slots were never written and may hold NaN/Inf bit patterns).
    if (tb + 64 > t1) {
#pragma unroll
      for (int b = 0; b < BPT; ++b) {
        const int n_ok = t1 - (tb + b * BS + part * 8);   // valid tokens in this lane's chunk
#pragma unroll
        for (int j = 0; j < VI; ++j) {
          uint32_t *wv = reinterpret_cast<uint32_t *>(&vreg[b][j]);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (2 * e >= n_ok) wv[e] = 0u;
            else if (2 * e + 1 >= n_ok) wv[e] &= 0x0000ffffu;
          }
        }
      }
    }

    // ---- scores ---------------------------------------------------------------
    float s[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float a0 = 0.f, a1 = 0.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        uint4 qq;
        if constexpr (G == 1) qq = make_uint4(q_s[4 * j], q_s[4 * j + 1], q_s[4 * j + 2], q_s[4 * j + 3]);
        else qq = reinterpret_cast<const uint4 *>(q_lds[g])[j];
        a0 = dot2<T>(kreg[j].x, qq.x, a0);
        a1 = dot2<T>(kreg[j].y, qq.y, a1);
        a0 = dot2<T>(kreg[j].z, qq.z, a0);
        a1 = dot2<T>(kreg[j].w, qq.w, a1);
      }
      s[g] = valid ? (a0 + a1) * scale_log2 : -INFINITY;
    }

    // ---- online softmax -------------------------------------------------------
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float m_new = fmaxf(m[g], wave_max(s[g]));
      const float alpha = fast_exp2(m[g] - m_new);
      const float p = fast_exp2(s[g] - m_new);
      l[g] = l[g] * alpha + p;
#pragma unroll
      for (int j = 0; j < VI; ++j) acc[g][j] *= alpha;
      m[g] = m_new;
      p_lds[g][lane] = p;
    }
    __syncthreads();

    // ---- P.V --------------------------------------------------------------------
#pragma unroll
    for (int b = 0; b < BPT; ++b) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float4 pa = *reinterpret_cast<const float4 *>(&p_lds[g][b * BS + part * 8]);
        const float4 pb = *reinterpret_cast<const float4 *>(&p_lds[g][b * BS + part * 8 + 4]);
#pragma unroll
        for (int j = 0; j < VI; ++j) {
          float a = acc[g][j];
          a = fma2<T>(vreg[b][j].x, pa.x, pa.y, a);
          a = fma2<T>(vreg[b][j].y, pa.z, pa.w, a);
          a = fma2<T>(vreg[b][j].z, pb.x, pb.y, a);
          a = fma2<T>(vreg[b][j].w, pb.z, pb.w, a);
          acc[g][j] = a;
        }
      }
    }
    __syncthreads();
  }

  // ---- finish: sum the per-part partials, then write output or a partial ---------
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const float L = wave_sum(l[g]);
    const int hq = hq0 + g;
    const int64_t prow = (static_cast<int64_t>(seq) * I.Hq + hq) * I.max_splits + split;
#pragma unroll
    for (int j = 0; j < VI; ++j) {
      float a = acc[g][j];
      if constexpr (PARTS >= 2) a += dpp_mov<0xB1>(a);
      if constexpr (PARTS >= 4) a += dpp_mov<0x4E>(a);
      const int d = j * (64 / PARTS) + lane / PARTS;
      if (part == 0) {
        if (single) {
          uint16_t *o = static_cast<uint16_t *>(I.out) + static_cast<int64_t>(seq) * I.out_stride + hq * D;
          o[d] = to_storage<T>(a / L);
        } else {
          I.ws_acc[prow * D + d] = a;
        }
      }
    }
    if (!single && lane == 0) {
      I.ws_ml[prow * 2] = m[g];
      I.ws_ml[prow * 2 + 1] = L;
    }
  }
}

// One block of 128 threads per (sequence, query head) with more than one partition.
template <typename T>
__global__ __launch_bounds__(128) void paged_decode_reduce_kernel(const DecodeParams P) {
  constexpr int D = kHeadSize;
  const int row = blockIdx.x;
  int ii = 0;
#pragma unroll
  for (int k = 1; k < MUXA_MAX_DECODE_ITEMS; ++k)
    if (k < P.n_items && row >= P.it[k].row_begin) ii = k;
  const DecodeItemDev &I = P.it[ii];
  const int local = row - I.row_begin;
  const int seq = local / I.Hq;
  const int hq = local - seq * I.Hq;
  const int ctx = min(I.ctx[seq], I.max_ctx);
  if (ctx <= P.partition) return;   // written directly by the main kernel
  const int n = (ctx + P.partition - 1) / P.partition;
  const int64_t base = (static_cast<int64_t>(seq) * I.Hq + hq) * I.max_splits;
  const int d = threadIdx.x;
  float M = -INFINITY;
  for (int i = 0; i < n; ++i) M = fmaxf(M, I.ws_ml[(base + i) * 2]);
  float L = 0.f, a = 0.f;
  for (int i = 0; i < n; ++i) {
    const float wgt = fast_exp2(I.ws_ml[(base + i) * 2] - M);
    L += I.ws_ml[(base + i) * 2 + 1] * wgt;
    a += I.ws_acc[(base + i) * D + d] * wgt;
  }
  uint16_t *o = static_cast<uint16_t *>(I.out) + static_cast<int64_t>(seq) * I.out_stride + hq * D;
  o[d] = to_storage<T>(a / L);
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
namespace {

int choose_partition(const MuxDecodeItem *items, int n_items, int requested) {
  if (requested > 0) return requested;
  int max_ctx = 0;
  for (int i = 0; i < n_items; ++i) max_ctx = std::max(max_ctx, items[i].max_context_len);
  return max_ctx > 4096 ? 512 : 256;
}

int pick_group(int ratio) {
  if (ratio == 8 || ratio == 4 || ratio == 2) return ratio;
  if (ratio % 8 == 0) return 8;
  if (ratio % 4 == 0) return 4;
  if (ratio % 2 == 0) return 2;
  return 1;
}

struct ItemWs { size_t acc_off, ml_off; int max_splits; };

// Workspace layout: for every item, acc [B,Hq,max_splits,128] fp32 then ml
// [B,Hq,max_splits,2] fp32; items whose contexts fit one partition take none.
size_t plan_workspace(const MuxDecodeItem *items, int n_items, int partition, ItemWs *out) {
  size_t off = 0;
  for (int i = 0; i < n_items; ++i) {
    const int ms = std::max(1, (items[i].max_context_len + partition - 1) / partition);
    ItemWs w{0, 0, ms};
    if (ms > 1) {
      const size_t rows = static_cast<size_t>(items[i].num_seqs) * items[i].num_q_heads * ms;
      w.acc_off = off;
      off += rows * kHeadSize * sizeof(float);
      w.ml_off = off;
      off += rows * 2 * sizeof(float);
      off = (off + 255) & ~static_cast<size_t>(255);
    }
    if (out) out[i] = w;
  }
  return off;
}

template <typename T, int BS>
hipError_t launch_main(int G, const DecodeParams &P, int grid, hipStream_t st) {
  switch (G) {
    case 1: hipLaunchKernelGGL((paged_decode_kernel<T, BS, 1>), dim3(grid), dim3(64), 0, st, P); break;
    case 2: hipLaunchKernelGGL((paged_decode_kernel<T, BS, 2>), dim3(grid), dim3(64), 0, st, P); break;
    case 4: hipLaunchKernelGGL((paged_decode_kernel<T, BS, 4>), dim3(grid), dim3(64), 0, st, P); break;
    case 8: hipLaunchKernelGGL((paged_decode_kernel<T, BS, 8>), dim3(grid), dim3(64), 0, st, P); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

template <typename T>
hipError_t launch_bs(int BS, int G, const DecodeParams &P, int grid, hipStream_t st) {
  switch (BS) {
    case 8: return launch_main<T, 8>(G, P, grid, st);
    case 16: return launch_main<T, 16>(G, P, grid, st);
    case 32: return launch_main<T, 32>(G, P, grid, st);
    default: return hipErrorInvalidValue;
  }
}

int32_t validate_item(const MuxDecodeItem &it, int block_size) {
  if (!it.out || !it.q || !it.block_tables || !it.context_lens) return MUXA_EINVAL;
  if (it.num_seqs < 0 || it.num_q_heads <= 0 || it.num_kv_heads <= 0) return MUXA_EINVAL;
  if (it.num_q_heads % it.num_kv_heads != 0) return MUXA_EINVAL;
  if (it.layer < 0 || it.layer >= it.num_layers) return MUXA_EINVAL;
  if (it.max_blocks < 0 || it.max_context_len < 0) return MUXA_EINVAL;
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
  return mux::plan_workspace(items, n_items, partition, nullptr);
}

int32_t mux_multi_decode(const MuxDecodeItem *items, int32_t n_items,
                         const void *k_pool, const void *v_pool, int64_t num_pool_blocks,
                         int32_t head_size, int32_t block_size, int32_t dtype,
                         int32_t partition_size, void *workspace, size_t workspace_bytes,
                         void *stream) {
  using namespace mux;
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
  const int partition = choose_partition(items, n_items, partition_size);
  ItemWs ws[MUXA_MAX_DECODE_ITEMS];
  const size_t need = plan_workspace(items, n_items, partition, ws);
  if (need > 0 && (!workspace || workspace_bytes < need)) return MUXA_EWORKSPACE;
  if (need > 0 && (reinterpret_cast<uintptr_t>(workspace) & 15u)) return MUXA_EINVAL;
  hipStream_t st = static_cast<hipStream_t>(stream);

  // Items are launched in groups that share G (query heads per wave).
  bool done[MUXA_MAX_DECODE_ITEMS] = {false};
  for (int first = 0; first < n_items; ++first) {
    if (done[first]) continue;
    const int G = pick_group(items[first].num_q_heads / items[first].num_kv_heads);
    DecodeParams P;
    P.k_pool = k_pool;
    P.v_pool = v_pool;
    P.partition = partition;
    P.last_block = static_cast<int32_t>(std::min<int64_t>(num_pool_blocks - 1, 0x7fffffff));
    P.n_items = 0;
    int64_t work = 0, rows = 0;
    bool any_split = false;
    for (int i = first; i < n_items; ++i) {
      if (done[i]) continue;
      const MuxDecodeItem &it = items[i];
      if (pick_group(it.num_q_heads / it.num_kv_heads) != G) continue;
      done[i] = true;
      if (it.num_seqs == 0 || it.max_context_len == 0) continue;
      DecodeItemDev &d = P.it[P.n_items++];
      d.out = it.out;
      d.q = it.q;
      d.out_stride = it.out_row_stride;
      d.q_stride = it.q_row_stride;
      d.tables = it.block_tables +
                 static_cast<int64_t>(it.layer) * it.num_seqs * it.num_kv_heads * it.max_blocks;
      d.ctx = it.context_lens;
      d.ws_acc = ws[i].max_splits > 1
                     ? reinterpret_cast<float *>(static_cast<char *>(workspace) + ws[i].acc_off) : nullptr;
      d.ws_ml = ws[i].max_splits > 1
                    ? reinterpret_cast<float *>(static_cast<char *>(workspace) + ws[i].ml_off) : nullptr;
      d.B = it.num_seqs;
      d.Hq = it.num_q_heads;
      d.Hkv = it.num_kv_heads;
      d.ratio = it.num_q_heads / it.num_kv_heads;
      d.max_blocks = it.max_blocks;
      d.max_splits = ws[i].max_splits;
      d.max_ctx = it.max_context_len;
      d.work_begin = static_cast<int32_t>(work);
      d.row_begin = static_cast<int32_t>(rows);
      d.scale_log2 = it.scale * 1.4426950408889634f;
      work += static_cast<int64_t>(it.num_seqs) * (it.num_q_heads / G) * ws[i].max_splits;
      rows += static_cast<int64_t>(it.num_seqs) * it.num_q_heads;
      any_split = any_split || ws[i].max_splits > 1;
      if (work > 0x7fffffff || rows > 0x7fffffff) return MUXA_EUNSUPPORTED;
    }
    if (P.n_items == 0) continue;
    hipError_t e = dtype == MUXA_DTYPE_F16 ? launch_bs<F16>(block_size, G, P, static_cast<int>(work), st)
                                           : launch_bs<BF16>(block_size, G, P, static_cast<int>(work), st);
    if (e != hipSuccess) return hip_fail(e);
    if (any_split) {
      if (dtype == MUXA_DTYPE_F16)
        hipLaunchKernelGGL((paged_decode_reduce_kernel<F16>), dim3(static_cast<int>(rows)), dim3(128), 0, st, P);
      else
        hipLaunchKernelGGL((paged_decode_reduce_kernel<BF16>), dim3(static_cast<int>(rows)), dim3(128), 0, st, P);
      e = hipGetLastError();
      if (e != hipSuccess) return hip_fail(e);
    }
  }
  return MUXA_OK;
}

int32_t mux_paged_decode(void *out, int64_t out_row_stride, const void *q, int64_t q_row_stride,
                         const void *k_pool, const void *v_pool, int64_t num_pool_blocks,
                         const int32_t *block_tables, const int32_t *context_lens,
                         int32_t layer, int32_t num_layers, int32_t num_seqs,
                         int32_t num_q_heads, int32_t num_kv_heads, int32_t head_size,
                         int32_t block_size, int32_t max_blocks, int32_t max_context_len,
                         float scale, int32_t dtype, int32_t partition_size,
                         void *workspace, size_t workspace_bytes, void *stream) {
  MuxDecodeItem it;
  it.out = out;
  it.q = q;
  it.out_row_stride = out_row_stride;
  it.q_row_stride = q_row_stride;
  it.block_tables = block_tables;
  it.context_lens = context_lens;
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
