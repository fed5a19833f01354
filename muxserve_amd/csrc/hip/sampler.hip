// Greedy sampling for gfx950: logits = hidden . embedding^T and the argmax over
// the vocabulary in one pass over the embedding matrix
// (muxserve/flexserver/sampler.py:15-35).  The logits are never written: a step
// reads the [vocab, hidden] matrix once (262 MB for a 7B model) and a few rows of
// hidden states, so the kernel is bound by HBM.
//
// lm_head_argmax_kernel<T, NB>: a workgroup owns 64 vocabulary rows (16 per
// wave) and up to 16 NB sampled rows of hidden states, and walks the hidden
// dimension in tiles of 128.
//   * Hidden states: the tile [16 NB][128] is staged in LDS, shared by the four
//     waves, double-buffered, one barrier per tile.
//   * Embedding rows: the MFMA A operand wants lane l to hold row l % 16
//     (v_mfma_f32_16x16x32: columns 8 (l / 16) .. +7 of a 32-column slice) -
//     loaded that way, every 16 lanes would touch 16 different rows with 16 bytes
//     each.  Instead a load instruction takes 4 rows x 256 contiguous bytes
//     (16 lanes per row), two tiles ahead of their use, and the wave regroups
//     its 4 KiB tile through a private LDS area: 16-byte chunk c of row r sits at
//     position c ^ r of the row, so both the row-wise writes and the
//     column-wise fragment reads are free of bank conflicts.
// Accumulators hold logits[vocab row 4 (l / 16) + i][sampled row l % 16]; each is
// rounded to the storage type (the reference compares logits of that type),
// reduced to the workgroup's (max, lowest index) per sampled row and written to
// a partial table.  argmax_finish_kernel reduces the table: one wave per
// sampled row.
#include "mux_common.h"

namespace mux {

typedef _Float16 sm_v8f16 __attribute__((ext_vector_type(8)));
typedef __bf16 sm_v8bf16 __attribute__((ext_vector_type(8)));
typedef float sm_v4f32 __attribute__((ext_vector_type(4)));
typedef uint32_t sm_u32x4 __attribute__((ext_vector_type(4)));

union SmFrag {
  sm_u32x4 u;
  sm_v8f16 h;
  sm_v8bf16 b;
};

constexpr int kSmTile = 256;              // the hidden size must be a multiple of this
constexpr int kSmVocabPerWg = 64;

struct LmHeadParams {
  const uint16_t *hidden;
  int64_t hidden_stride;
  const int32_t *row_index;               // sampled row r reads hidden row row_index[r]; null: row r
  const uint16_t *weight;
  int64_t weight_stride;
  int32_t hidden_size, vocab, num_rows;
  float *part_val;                        // [workgroups][16 NB]
  int32_t *part_idx;
};

template <typename T>
__device__ __forceinline__ float sm_round(float f) {
  if constexpr (__is_same(T, F16)) return static_cast<float>(static_cast<_Float16>(f));
  else return __uint_as_float(static_cast<uint32_t>(f32_to_bf16_bits(f)) << 16);
}

// (value, index) pairs ordered by value, ties to the lower index.
__device__ __forceinline__ void take_better(float &v, int &i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) {
    v = ov;
    i = oi;
  }
}

template <typename T, int NB>
__global__ __launch_bounds__(256) void lm_head_argmax_kernel(const LmHeadParams P) {
  constexpr int KT = 128;                             // hidden elements per tile
  constexpr int ROWS = 16 * NB;                       // sampled rows held in LDS
  constexpr int CPR = KT / 8;                         // 16-byte chunks per tile row (16)
  constexpr int SJ = ROWS * CPR / 256;                // hidden-state staging chunks per thread (= NB)
  constexpr int NF = KT / 32;                         // MFMA column slices per tile (4)
  constexpr int kHRow = KT + 8;     // LDS row pitch: 16 bytes of padding keep b128 reads off each other's banks
  __shared__ __attribute__((aligned(16))) uint16_t htile[2][ROWS * kHRow];
  __shared__ __attribute__((aligned(16))) uint16_t wtile[4][16 * KT];      // one 4 KiB area per wave
  __shared__ float red_v[4][ROWS];
  __shared__ int red_i[4][ROWS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const int n_tiles = P.hidden_size / KT;

  // Embedding rows of this wave (rows past the vocabulary re-read its last row
  // and are masked at the end).  Load instruction j: lane l takes row
  // 4 j + l / 16, and of that row the chunk (l % 16) ^ row.
  const int vrow0 = blockIdx.x * kSmVocabPerWg + 16 * wave;
  const uint16_t *wsrc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = 4 * j + g;
    const int lrow = min(vrow0 + row, P.vocab - 1);
    wsrc[j] = P.weight + static_cast<int64_t>(lrow) * P.weight_stride + 8 * (r16 ^ row);
  }
  uint16_t *const wmine = &wtile[wave][0];

  // Hidden-state staging: chunk id = tid + 256 j -> (row id / 16, 16-byte chunk id % 16).
  const uint16_t *hsrc[SJ];
  bool hvalid[SJ];
#pragma unroll
  for (int j = 0; j < SJ; ++j) {
    const int row = (tid >> 4) + 16 * j;
    hvalid[j] = row < P.num_rows;
    const int src = hvalid[j] ? (P.row_index ? P.row_index[row] : row) : 0;
    hsrc[j] = P.hidden + static_cast<int64_t>(src) * P.hidden_stride + 8 * (tid & 15);
  }
  const int hoff = (tid >> 4) * kHRow + 8 * (tid & 15);
  sm_u32x4 st[SJ];
  auto stage_load = [&](int t) {
#pragma unroll
    for (int j = 0; j < SJ; ++j)
      st[j] = hvalid[j] ? *reinterpret_cast<const sm_u32x4 *>(hsrc[j] + t * KT) : sm_u32x4{0, 0, 0, 0};
  };
  auto stage_store = [&](int buf) {
#pragma unroll
    for (int j = 0; j < SJ; ++j) *reinterpret_cast<sm_u32x4 *>(&htile[buf][hoff + 16 * j * kHRow]) = st[j];
  };
  auto load_w = [&](sm_u32x4 (&w)[4], int t) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      w[j] = __builtin_nontemporal_load(reinterpret_cast<const sm_u32x4 *>(wsrc[j] + t * KT));
  };

  sm_v4f32 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) acc[nb] = sm_v4f32{0.f, 0.f, 0.f, 0.f};
  // Regroup one embedding tile through the wave's LDS area, then multiply.
  auto consume = [&](const sm_u32x4 (&w)[4], int buf) {
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<sm_u32x4 *>(wmine + (4 * j) * KT + 8 * lane) = w[j];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    SmFrag a[NF];
#pragma unroll
    for (int i = 0; i < NF; ++i)
      a[i].u = *reinterpret_cast<const sm_u32x4 *>(wmine + r16 * KT + 8 * ((4 * i + g) ^ r16));
    const uint16_t *base = &htile[buf][r16 * kHRow + 8 * g];
#pragma unroll
    for (int i = 0; i < NF; ++i) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        SmFrag b;
        b.u = *reinterpret_cast<const sm_u32x4 *>(base + 16 * nb * kHRow + 32 * i);
        if constexpr (__is_same(T, F16))
          acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i].h, b.h, acc[nb], 0, 0, 0);
        else
          acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i].b, b.b, acc[nb], 0, 0, 0);
      }
    }
    __builtin_amdgcn_wave_barrier();                    // fragment reads stay ahead of the next tile's writes
  };

  sm_u32x4 w0[4], w1[4];
  load_w(w0, 0);
  if (n_tiles > 1) load_w(w1, 1);
  stage_load(0);
  stage_store(0);
  __syncthreads();
  for (int t = 0; t < n_tiles; t += 2) {
    if (t + 1 < n_tiles) stage_load(t + 1);
    consume(w0, 0);
    if (t + 2 < n_tiles) load_w(w0, t + 2);
    if (t + 1 < n_tiles) stage_store(1);
    __syncthreads();
    if (t + 1 >= n_tiles) break;
    if (t + 2 < n_tiles) stage_load(t + 2);
    consume(w1, 1);
    if (t + 3 < n_tiles) load_w(w1, t + 3);
    if (t + 2 < n_tiles) stage_store(0);
    __syncthreads();
  }

  // Lane holds logits[vocab row vrow0 + 4 g + i][sampled row 16 nb + r16].
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    float bv = -__builtin_inff();
    int bi = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int vr = vrow0 + 4 * g + i;
      const float val = sm_round<T>(acc[nb][i]);
      if (vr < P.vocab) take_better(bv, bi, val, vr);
    }
#pragma unroll
    for (int off = 16; off <= 32; off <<= 1) {
      const float ov = __shfl_xor(bv, off);
      const int oi = __shfl_xor(bi, off);
      take_better(bv, bi, ov, oi);
    }
    if (g == 0) {
      red_v[wave][16 * nb + r16] = bv;
      red_i[wave][16 * nb + r16] = bi;
    }
  }
  __syncthreads();
  if (tid < ROWS) {
    float bv = red_v[0][tid];
    int bi = red_i[0][tid];
#pragma unroll
    for (int w = 1; w < 4; ++w) take_better(bv, bi, red_v[w][tid], red_i[w][tid]);
    P.part_val[static_cast<int64_t>(blockIdx.x) * ROWS + tid] = bv;
    P.part_idx[static_cast<int64_t>(blockIdx.x) * ROWS + tid] = bi;
  }
}

// One wave per sampled row: lanes stride over the workgroups' partial results.
__global__ __launch_bounds__(64) void argmax_finish_kernel(int64_t *__restrict__ next_tokens,
                                                           const float *__restrict__ part_val,
                                                           const int32_t *__restrict__ part_idx, int n_parts,
                                                           int rows_pitch) {
  const int r = blockIdx.x, lane = threadIdx.x;
  float bv = -__builtin_inff();
  int bi = 0x7fffffff;
  for (int b = lane; b < n_parts; b += 64)
    take_better(bv, bi, part_val[static_cast<int64_t>(b) * rows_pitch + r],
                part_idx[static_cast<int64_t>(b) * rows_pitch + r]);
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const float ov = __shfl_xor(bv, off);
    const int oi = __shfl_xor(bi, off);
    take_better(bv, bi, ov, oi);
  }
  if (lane == 0) next_tokens[r] = bi == 0x7fffffff ? 0 : bi;   // every logit NaN: token 0
}

constexpr int kSmMaxRowsPerPass = 64;

}  // namespace mux

extern "C" size_t mux_greedy_sample_workspace_bytes(int32_t vocab_size) {
  if (vocab_size <= 0) return 0;
  const size_t n_wg = (static_cast<size_t>(vocab_size) + mux::kSmVocabPerWg - 1) / mux::kSmVocabPerWg;
  return n_wg * mux::kSmMaxRowsPerPass * (sizeof(float) + sizeof(int32_t));
}

extern "C" int32_t mux_greedy_sample(int64_t *next_tokens, const void *hidden_states, int64_t hidden_row_stride,
                                     const int32_t *row_index, int32_t num_rows, const void *embedding,
                                     int64_t embedding_row_stride, int32_t embedding_rows, int32_t vocab_size,
                                     int32_t hidden_size, int32_t dtype, void *workspace, size_t workspace_bytes,
                                     void *stream) {
  using namespace mux;
  if (!next_tokens || !hidden_states || !embedding) return MUXA_EINVAL;
  if (num_rows < 0 || vocab_size <= 0 || hidden_size <= 0 || embedding_rows < vocab_size) return MUXA_EINVAL;
  if (dtype != MUXA_DTYPE_F16 && dtype != MUXA_DTYPE_BF16) return MUXA_EUNSUPPORTED;
  if (hidden_size % kSmTile) return MUXA_EUNSUPPORTED;
  if (hidden_row_stride < hidden_size || embedding_row_stride < hidden_size || hidden_row_stride % 8 ||
      embedding_row_stride % 8)
    return MUXA_EINVAL;
  if ((reinterpret_cast<uintptr_t>(hidden_states) | reinterpret_cast<uintptr_t>(embedding)) & 15u)
    return MUXA_EINVAL;
  if (num_rows == 0) return MUXA_OK;
  if (!workspace || workspace_bytes < mux_greedy_sample_workspace_bytes(vocab_size) ||
      (reinterpret_cast<uintptr_t>(workspace) & 15u))
    return MUXA_EWORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int n_wg = (vocab_size + kSmVocabPerWg - 1) / kSmVocabPerWg;
  float *part_val = static_cast<float *>(workspace);
  int32_t *part_idx = reinterpret_cast<int32_t *>(part_val + static_cast<size_t>(n_wg) * kSmMaxRowsPerPass);
  // At most 64 sampled rows per pass over the matrix; larger batches take
  // several passes that reuse the partial table one after the other.
  for (int r0 = 0; r0 < num_rows; r0 += kSmMaxRowsPerPass) {
    const int rows = min(num_rows - r0, kSmMaxRowsPerPass);
    LmHeadParams P;
    P.hidden = static_cast<const uint16_t *>(hidden_states) + (row_index ? 0 : static_cast<int64_t>(r0) * hidden_row_stride);
    P.hidden_stride = hidden_row_stride;
    P.row_index = row_index ? row_index + r0 : nullptr;
    P.weight = static_cast<const uint16_t *>(embedding);
    P.weight_stride = embedding_row_stride;
    P.hidden_size = hidden_size;
    P.vocab = vocab_size;
    P.num_rows = rows;
    P.part_val = part_val;
    P.part_idx = part_idx;
    const int nb = rows <= 16 ? 1 : (rows <= 32 ? 2 : 4);
    const dim3 grid(n_wg), block(256);
#define MUX_LM_LAUNCH(TT)                                                                   \
  do {                                                                                      \
    if (nb == 1) hipLaunchKernelGGL((lm_head_argmax_kernel<TT, 1>), grid, block, 0, st, P); \
    else if (nb == 2) hipLaunchKernelGGL((lm_head_argmax_kernel<TT, 2>), grid, block, 0, st, P); \
    else hipLaunchKernelGGL((lm_head_argmax_kernel<TT, 4>), grid, block, 0, st, P);         \
  } while (0)
    if (dtype == MUXA_DTYPE_F16) MUX_LM_LAUNCH(F16);
    else MUX_LM_LAUNCH(BF16);
#undef MUX_LM_LAUNCH
    hipLaunchKernelGGL(argmax_finish_kernel, dim3(rows), dim3(64), 0, st, next_tokens + r0, part_val, part_idx, n_wg,
                       16 * nb);
  }
  MUX_HIP_TRY(hipGetLastError());
  return MUXA_OK;
}
