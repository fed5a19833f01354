// Greedy sampling for gfx950: logits = hidden . embedding^T and the argmax over
// the vocabulary in one pass over the embedding matrix
// (muxserve/flexserver/sampler.py:15-35).  The logits are never written: a step
// reads the [vocab, hidden] matrix once (262 MB for a 7B model) and a few rows of
// hidden states, so the kernel is bound by HBM.
//
// lm_head_argmax_kernel<T, NB, NW, RB>: a workgroup of NW waves owns 16 NW RB
// vocabulary rows (RB blocks of 16 per wave) and up to 16 NB sampled rows of hidden states,
// and walks the hidden dimension in tiles of 128.
//   * Hidden states: the tile [16 NB][128] is staged in LDS, shared by the
//     waves, double-buffered, one barrier per tile.  Every workgroup reads all
//     of the sampled hidden states (from L2), so large vocabularies use 8 waves
//     per workgroup: half as many workgroups, half that traffic.
//   * Embedding rows: the MFMA A operand wants lane l to hold row l % 16
//     (v_mfma_f32_16x16x32: columns 8 (l / 16) .. +7 of a 32-column slice) -
//     loaded that way, every 16 lanes would touch 16 different rows with 16 bytes
//     each.  Instead a load instruction takes 4 rows x 256 contiguous bytes
//     (16 lanes per row), a tile ahead of their use (deeper makes no difference), and the wave regroups
//     its 4 KiB tile through a private LDS area: 16-byte chunk c of row r sits at
//     position c ^ r of the row, so both the row-wise writes and the
//     column-wise fragment reads are free of bank conflicts.
// Accumulators hold logits[vocab row 4 (l / 16) + i][sampled row l % 16]; each is
// rounded to the storage type (the reference compares logits of that type) and
// reduced to the workgroup's (max, lowest index) per sampled row, which goes to
// the workgroup's line of a table as a 64-bit key (ordered logit bits << 32 |
// ~index).  The last workgroup to arrive (a counter tells it) takes the maximum
// of every column of the table, writes the token ids and leaves the counter at
// zero for the next launch.  (Atomic max on one key per sampled row instead of
// the table serialises 16000 atomics on two cache lines: +30 us per launch.)
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
constexpr int kSmMaxRowsPerPass = 64;
#ifndef MUX_SM_PREFETCH_TILES
#define MUX_SM_PREFETCH_TILES 2
#endif

struct LmHeadParams {
  const uint16_t *hidden;
  int64_t hidden_stride;
  const int32_t *row_index;               // sampled row r reads hidden row row_index[r]; null: row r
  const uint16_t *weight;
  int64_t weight_stride;
  int32_t hidden_size, vocab, num_rows;
  int32_t hidden_rows;                    // rows of `hidden`: row_index entries are clamped to it
  uint32_t *counter;                      // workgroups arrived, zero between launches
  unsigned long long *table;              // [workgroups][16 NB] keys, written before they are read
  int64_t *next_tokens;
};

// Float bits that compare like the floats as unsigned integers.
__device__ __forceinline__ uint32_t ordered_bits(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

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

template <typename T, int NB, int NW, int RB>
__global__ __launch_bounds__(64 * NW) void lm_head_argmax_kernel(const LmHeadParams P) {
  constexpr int KT = 128;                             // hidden elements per tile
  constexpr int ROWS = 16 * NB;                       // sampled rows held in LDS
  constexpr int CPR = KT / 8;                         // 16-byte chunks per tile row (16)
  constexpr int RPP = 4 * NW;                         // hidden-state rows staged per pass of the workgroup
  constexpr int SJ = (ROWS + RPP - 1) / RPP;          // staging chunks per thread
  constexpr int NF = KT / 32;                         // MFMA column slices per tile (4)
  constexpr int kHRow = KT + 8;     // LDS row pitch: 16 bytes of padding keep b128 reads off each other's banks
  __shared__ __attribute__((aligned(16))) uint16_t htile[2][ROWS * kHRow];
  __shared__ __attribute__((aligned(16))) uint16_t wtile[NW][RB][16 * KT];  // 4 KiB per wave and row block
  __shared__ float red_v[NW][ROWS];
  __shared__ int red_i[NW][ROWS];
  __shared__ int s_last;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  const int n_tiles = P.hidden_size / KT;
  // Workgroups start their walk over the hidden dimension at different tiles
  // (a dot product does not care about the order): with a row pitch that is a
  // power of two - 8 KiB at hidden size 4096 - workgroups walking in step would
  // all be reading the same few memory channels at any moment.
  const int t_start = blockIdx.x % n_tiles;
  auto tile_of = [&](int t) {
    const int x = t + t_start;
    return x >= n_tiles ? x - n_tiles : x;
  };

  // Embedding rows of this wave (rows past the vocabulary re-read its last row
  // and are masked at the end).  Load instruction j: lane l takes row
  // 4 j + l / 16, and of that row the chunk (l % 16) ^ row.
  const int vrow0 = blockIdx.x * (16 * NW * RB) + 16 * RB * wave;
  const uint16_t *wsrc[RB][4];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = 4 * j + g;
      const int lrow = min(vrow0 + 16 * rb + row, P.vocab - 1);
      wsrc[rb][j] = P.weight + static_cast<int64_t>(lrow) * P.weight_stride + 8 * (r16 ^ row);
    }
  uint16_t *const wmine = &wtile[wave][0][0];

  // Hidden-state staging: thread -> (row tid / 16 + RPP j, 16-byte chunk tid % 16).
  const uint16_t *hsrc[SJ];
  bool hvalid[SJ], hstore[SJ];
#pragma unroll
  for (int j = 0; j < SJ; ++j) {
    const int row = (tid >> 4) + RPP * j;
    hstore[j] = row < ROWS;
    hvalid[j] = row < P.num_rows && hstore[j];
    const int src = hvalid[j] ? (P.row_index ? min(max(P.row_index[row], 0), P.hidden_rows - 1) : row) : 0;
    hsrc[j] = P.hidden + static_cast<int64_t>(src) * P.hidden_stride + 8 * (tid & 15);
  }
  const int hoff = (tid >> 4) * kHRow + 8 * (tid & 15);
  auto stage_load = [&](sm_u32x4 (&st)[SJ], int t) {
#pragma unroll
    for (int j = 0; j < SJ; ++j)
      st[j] = hvalid[j] ? *reinterpret_cast<const sm_u32x4 *>(hsrc[j] + tile_of(t) * KT) : sm_u32x4{0, 0, 0, 0};
  };
  auto stage_store = [&](const sm_u32x4 (&st)[SJ], int buf) {
#pragma unroll
    for (int j = 0; j < SJ; ++j)
      if (hstore[j]) *reinterpret_cast<sm_u32x4 *>(&htile[buf][hoff + RPP * j * kHRow]) = st[j];
  };
  auto load_w = [&](sm_u32x4 (&w)[RB][4], int t) {
    const int off = tile_of(t) * KT;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        w[rb][j] = __builtin_nontemporal_load(reinterpret_cast<const sm_u32x4 *>(wsrc[rb][j] + off));
  };

  sm_v4f32 acc[RB][NB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[rb][nb] = sm_v4f32{0.f, 0.f, 0.f, 0.f};
  // Regroup one embedding tile through the wave's LDS area, then multiply.
  auto consume = [&](const sm_u32x4 (&w)[RB][4], int buf) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        *reinterpret_cast<sm_u32x4 *>(wmine + rb * 16 * KT + (4 * j) * KT + 8 * lane) = w[rb][j];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    SmFrag a[RB][NF];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int i = 0; i < NF; ++i)
        a[rb][i].u = *reinterpret_cast<const sm_u32x4 *>(wmine + rb * 16 * KT + r16 * KT + 8 * ((4 * i + g) ^ r16));
    const uint16_t *base = &htile[buf][r16 * kHRow + 8 * g];
#pragma unroll
    for (int i = 0; i < NF; ++i) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        SmFrag b;
        b.u = *reinterpret_cast<const sm_u32x4 *>(base + 16 * nb * kHRow + 32 * i);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {      // one hidden-state fragment serves every row block of the wave
          if constexpr (__is_same(T, F16))
            acc[rb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[rb][i].h, b.h, acc[rb][nb], 0, 0, 0);
          else
            acc[rb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rb][i].b, b.b, acc[rb][nb], 0, 0, 0);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();                    // fragment reads stay ahead of the next tile's writes
  };

  // PD tiles per wave are in flight: register sets used in rotation (unrolled,
  // so every set is addressed statically).  Loads return in order, so the
  // hidden-state part of a tile is requested together with - and just before -
  // its embedding part: waiting for one never waits for a younger tile.
  constexpr int PD = MUX_SM_PREFETCH_TILES;
  static_assert(PD % 2 == 0, "the hidden-state buffers alternate with the tile parity");
  sm_u32x4 w[PD][RB][4], st[PD][SJ];
#pragma unroll
  for (int s2 = 0; s2 < PD; ++s2)
    if (s2 < n_tiles) {
      stage_load(st[s2], s2);
      load_w(w[s2], s2);
    }
  stage_store(st[0], 0);
  __syncthreads();
  for (int t0 = 0; t0 < n_tiles; t0 += PD) {
#pragma unroll
    for (int s2 = 0; s2 < PD; ++s2) {
      const int t = t0 + s2;
      if (t < n_tiles) {
        consume(w[s2], s2 & 1);
        if (t + 1 < n_tiles) stage_store(st[(s2 + 1) % PD], (s2 + 1) & 1);
        if (t + PD < n_tiles) {
          stage_load(st[s2], t + PD);
          load_w(w[s2], t + PD);
        }
        __syncthreads();
      }
    }
  }

  // Lane holds logits[vocab row vrow0 + 16 rb + 4 g + i][sampled row 16 nb + r16].
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    float bv = -__builtin_inff();
    int bi = 0x7fffffff;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int vr = vrow0 + 16 * rb + 4 * g + i;
        const float val = sm_round<T>(acc[rb][nb][i]);
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
  // The workgroup's result per sampled row goes to its line of the table as a
  // 64-bit key (ordered logit bits << 32 | ~index: a larger key is a better
  // logit or, between equal logits, a lower index).
  if (tid < ROWS) {
    float bv = red_v[0][tid];
    int bi = red_i[0][tid];
#pragma unroll
    for (int w = 1; w < NW; ++w) take_better(bv, bi, red_v[w][tid], red_i[w][tid]);
    const unsigned long long key = (static_cast<unsigned long long>(ordered_bits(bv)) << 32) |
                                   (0xffffffffu - static_cast<uint32_t>(bi));
    __hip_atomic_store(&P.table[static_cast<int64_t>(blockIdx.x) * ROWS + tid], key, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  }
  // The table is written and read with device-coherent accesses (they bypass
  // the per-XCD L2), so ordering them against the counter takes only a wait
  // for this wave's table stores to be acknowledged before the workgroup meets
  // and bumps the counter.  A device-scope fence would also write back and
  // invalidate this XCD's L2, which holds the hidden states every other
  // workgroup is still reading (measured: +30 us per launch).
  wait_own_vector_memory();
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (tid == 0)
    s_last = __hip_atomic_fetch_add(P.counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gridDim.x - 1;
  __syncthreads();
  if (!s_last) return;
  // Last workgroup to arrive: thread -> (sampled row tid % ROWS, slice
  // tid / ROWS of the workgroups), sixteen loads in flight.
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  constexpr int SLICES = 64 * NW / ROWS;
  __shared__ unsigned long long fin[SLICES][ROWS];
  const int row = tid % ROWS, slice = tid / ROWS;
  unsigned long long best = 0;
  const int n_wg = gridDim.x;
  for (int b0 = slice; b0 < n_wg; b0 += 16 * SLICES) {
    unsigned long long v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int b = b0 + j * SLICES;
      v[j] = b < n_wg ? __hip_atomic_load(&P.table[static_cast<int64_t>(b) * ROWS + row], __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT)
                      : 0ull;
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) best = v[j] > best ? v[j] : best;
  }
  fin[slice][row] = best;
  __syncthreads();
  if (tid < P.num_rows) {
    unsigned long long k = fin[0][tid];
#pragma unroll
    for (int sl = 1; sl < SLICES; ++sl) k = fin[sl][tid] > k ? fin[sl][tid] : k;
    const uint32_t idx = 0xffffffffu - static_cast<uint32_t>(k);
    P.next_tokens[tid] = idx < static_cast<uint32_t>(P.vocab) ? idx : 0;   // every logit NaN: token 0
  }
  if (tid == 0) __hip_atomic_store(P.counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__global__ void sampler_zero_kernel(uint32_t *p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

constexpr size_t kSmCounterBytes = 256;        // the arrival counter, then the table
#ifndef MUX_SM_EIGHT_WAVE_MIN_WGS
#define MUX_SM_EIGHT_WAVE_MIN_WGS 192
#endif
constexpr int kSmEightWaveMinWgs = MUX_SM_EIGHT_WAVE_MIN_WGS;

}  // namespace mux

extern "C" size_t mux_greedy_sample_workspace_bytes(int32_t vocab_size) {
  if (vocab_size <= 0) return 0;
  const size_t n_wg = (static_cast<size_t>(vocab_size) + 63) / 64;            // the most workgroups a launch uses
  return mux::kSmCounterBytes + n_wg * mux::kSmMaxRowsPerPass * sizeof(unsigned long long);
}

extern "C" int32_t mux_greedy_sample_workspace_init(void *workspace, size_t workspace_bytes, void *stream) {
  using namespace mux;
  if (!workspace || workspace_bytes < kSmCounterBytes || (reinterpret_cast<uintptr_t>(workspace) & 15u))
    return MUXA_EWORKSPACE;
  hipLaunchKernelGGL(sampler_zero_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<uint32_t *>(workspace), static_cast<int>(kSmCounterBytes / 4));
  MUX_HIP_TRY(hipGetLastError());
  return MUXA_OK;
}

extern "C" int32_t mux_greedy_sample(int64_t *next_tokens, const void *hidden_states, int64_t hidden_row_stride,
                                     int32_t num_hidden_rows, const int32_t *row_index, int32_t num_rows,
                                     const void *embedding,
                                     int64_t embedding_row_stride, int32_t embedding_rows, int32_t vocab_size,
                                     int32_t hidden_size, int32_t dtype, void *workspace, size_t workspace_bytes,
                                     void *stream) {
  using namespace mux;
  // (pointers are only required when there is something to do)
  if (num_rows > 0 && (!next_tokens || !hidden_states || !embedding)) return MUXA_EINVAL;
  if (num_rows < 0 || vocab_size <= 0 || hidden_size <= 0 || embedding_rows < vocab_size) return MUXA_EINVAL;
  if (num_hidden_rows < 1 || (!row_index && num_rows > num_hidden_rows)) return MUXA_EINVAL;
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
  // 128 vocabulary rows per workgroup (8 waves) once that still gives the chip
  // enough workgroups, else 64.  (Two row blocks per wave, RB = 2, halve the
  // hidden-state fragment reads but measured slower with 4 waves per workgroup:
  // 61 against 56 us at 64 sampled rows, hidden size 4096.)
  const bool wide = (vocab_size + 127) / 128 >= kSmEightWaveMinWgs;
  const int rows_per_wg = wide ? 128 : 64;
  const int n_wg = (vocab_size + rows_per_wg - 1) / rows_per_wg;
  // At most 64 sampled rows per pass over the matrix; larger batches take
  // several passes, one after the other on the stream.
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
    P.hidden_rows = row_index ? num_hidden_rows : num_hidden_rows - r0;
    P.counter = static_cast<uint32_t *>(workspace);
    P.table = reinterpret_cast<unsigned long long *>(static_cast<char *>(workspace) + kSmCounterBytes);
    P.next_tokens = next_tokens + r0;
    const int nb = rows <= 16 ? 1 : (rows <= 32 ? 2 : 4);
    const dim3 grid(n_wg);
#define MUX_LM_GO(TT, NBV, NWV, RBV) \
  hipLaunchKernelGGL((lm_head_argmax_kernel<TT, NBV, NWV, RBV>), grid, dim3(64 * NWV), 0, st, P)
#define MUX_LM_LAUNCH(TT)                  \
  do {                                     \
    if (!wide) {                           \
      if (nb == 1) MUX_LM_GO(TT, 1, 4, 1); \
      else if (nb == 2) MUX_LM_GO(TT, 2, 4, 1); \
      else MUX_LM_GO(TT, 4, 4, 1);         \
    } else if (nb == 1) MUX_LM_GO(TT, 1, 8, 1); \
    else if (nb == 2) MUX_LM_GO(TT, 2, 8, 1);   \
    else MUX_LM_GO(TT, 4, 8, 1);           \
  } while (0)
    if (dtype == MUXA_DTYPE_F16) MUX_LM_LAUNCH(F16);
    else MUX_LM_LAUNCH(BF16);
#undef MUX_LM_LAUNCH
#undef MUX_LM_GO
  }
  MUX_HIP_TRY(hipGetLastError());
  return MUXA_OK;
}
