// RMSNorm and SiluAndMul for gfx950: the two element-wise operators of a LLaMA
// layer next to the attention (muxserve/flexserver/models/llama.py:75-81,
// 200-232).  Both are bound by HBM: every input element is read once and every
// output element written once, in 16-byte pieces.
//
//   rms_norm      one wave per token row at a time: the row stays in registers
//                 between the sum of squares and the scaling, so x is read once
//                 (with non-temporal loads: 19.5 instead of 26 us for 4096 rows
//                 of 6656); the wave sum is a DPP reduction, no LDS, no barrier.
//                 out = T(x * rsqrt(mean(x^2) + eps)) * w, the product in T.
//   silu_and_mul  one thread per 8 outputs: out = T(a / (1 + exp(-a))) * b for
//                 x = [a | b], the product in T.
#include <algorithm>

#include "mux_common.h"

namespace mux {

typedef uint32_t mo_u32x4 __attribute__((ext_vector_type(4)));

#ifndef MUX_RMS_WAVES_PER_CU
#define MUX_RMS_WAVES_PER_CU 8
#endif
constexpr int kRmsWavesPerCu = MUX_RMS_WAVES_PER_CU;


template <typename T>
__device__ __forceinline__ void unpack8(const mo_u32x4 v, float (&f)[8]) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (__is_same(T, F16)) {
      const half2_t h = as_half2(w[i]);
      f[2 * i] = static_cast<float>(h.x);
      f[2 * i + 1] = static_cast<float>(h.y);
    } else {
      f[2 * i] = bf16_lo(w[i]);
      f[2 * i + 1] = bf16_hi(w[i]);
    }
  }
}

template <typename T>
__device__ __forceinline__ float round_to(float f) {         // the value of f after one rounding to T
  if constexpr (__is_same(T, F16)) return static_cast<float>(static_cast<_Float16>(f));
  else return __uint_as_float(static_cast<uint32_t>(f32_to_bf16_bits(f)) << 16);
}

template <typename T>
__device__ __forceinline__ mo_u32x4 pack8(const float (&f)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = static_cast<uint32_t>(to_storage<T>(f[2 * i])) | (static_cast<uint32_t>(to_storage<T>(f[2 * i + 1])) << 16);
  return mo_u32x4{w[0], w[1], w[2], w[3]};
}

// CPL = 16-byte chunks a lane keeps (a row has hidden / 8 chunks, lane l takes
// chunks l, l + 64, ...).  A wave walks rows wave, wave + W, wave + 2 W, ... (W
// waves in the grid) with the next row's loads issued before the current row is
// reduced and stored, so that across the chip reads and writes overlap instead
// of coming as one burst of each.  CPL = 0: rows of any length, x read twice.
template <typename T, int CPL>
__global__ __launch_bounds__(256) void rms_norm_kernel(uint16_t *__restrict__ out, int64_t out_stride,
                                                       const uint16_t *__restrict__ x, int64_t x_stride,
                                                       const uint16_t *__restrict__ weight, float eps, int hidden,
                                                       int num_rows) {
  const int lane = threadIdx.x & 63;
  const int first = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int step = gridDim.x * 4;
  if (first >= num_rows) return;
  const int nchunks = hidden >> 3;
  const mo_u32x4 *wr = reinterpret_cast<const mo_u32x4 *>(weight);
  const float inv_n = 1.0f / static_cast<float>(hidden);
  if constexpr (CPL > 0) {
    auto load_row = [&](mo_u32x4 (&v)[CPL], int row) {
      const mo_u32x4 *xr = reinterpret_cast<const mo_u32x4 *>(x + row * x_stride);
#pragma unroll
      for (int i = 0; i < CPL; ++i) {
        const int c = lane + 64 * i;
        v[i] = c < nchunks ? __builtin_nontemporal_load(&xr[c]) : mo_u32x4{0, 0, 0, 0};
      }
    };
    auto finish_row = [&](const mo_u32x4 (&v)[CPL], int row) {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < CPL; ++i) {
        float f[8];
        unpack8<T>(v[i], f);
#pragma unroll
        for (int j = 0; j < 8; ++j) ss = __builtin_fmaf(f[j], f[j], ss);
      }
      ss = wave_sum(ss);
      const float s = rsqrtf(ss * inv_n + eps);
      mo_u32x4 *outr = reinterpret_cast<mo_u32x4 *>(out + row * out_stride);
#pragma unroll
      for (int i = 0; i < CPL; ++i) {
        const int c = lane + 64 * i;
        if (c < nchunks) {
          float f[8], w[8];
          unpack8<T>(v[i], f);
          unpack8<T>(wr[c], w);
#pragma unroll
          for (int j = 0; j < 8; ++j) f[j] = round_to<T>(f[j] * s) * w[j];
          outr[c] = pack8<T>(f);
        }
      }
    };
    mo_u32x4 a[CPL], b[CPL];
    load_row(a, first);
    for (int row = first; row < num_rows; row += 2 * step) {
      if (row + step < num_rows) load_row(b, row + step);
      finish_row(a, row);
      if (row + step >= num_rows) break;
      if (row + 2 * step < num_rows) load_row(a, row + 2 * step);
      finish_row(b, row + step);
    }
  } else {
    for (int row = first; row < num_rows; row += step) {
      const mo_u32x4 *xr = reinterpret_cast<const mo_u32x4 *>(x + row * x_stride);
      mo_u32x4 *outr = reinterpret_cast<mo_u32x4 *>(out + row * out_stride);
      float ss = 0.f;
      for (int c = lane; c < nchunks; c += 64) {
        float f[8];
        unpack8<T>(xr[c], f);
#pragma unroll
        for (int j = 0; j < 8; ++j) ss = __builtin_fmaf(f[j], f[j], ss);
      }
      ss = wave_sum(ss);
      const float s = rsqrtf(ss * inv_n + eps);
      for (int c = lane; c < nchunks; c += 64) {
        float f[8], w[8];
        unpack8<T>(xr[c], f);
        unpack8<T>(wr[c], w);
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] = round_to<T>(f[j] * s) * w[j];
        outr[c] = pack8<T>(f);
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void silu_and_mul_kernel(uint16_t *__restrict__ out, int64_t out_stride,
                                                           const uint16_t *__restrict__ x, int64_t x_stride,
                                                           int d8, int64_t total) {
  const int64_t id = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (id >= total) return;
  const int64_t t = id / d8;
  const int c = static_cast<int>(id - t * d8);
  const mo_u32x4 *xr = reinterpret_cast<const mo_u32x4 *>(x + t * x_stride);
  const mo_u32x4 av = __builtin_nontemporal_load(&xr[c]), bv = __builtin_nontemporal_load(&xr[d8 + c]);
  float a[8], b[8];
  unpack8<T>(av, a);
  unpack8<T>(bv, b);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float e = fast_exp2(-1.4426950408889634f * a[j]);
    a[j] = round_to<T>(a[j] * __builtin_amdgcn_rcpf(1.0f + e)) * b[j];
  }
  reinterpret_cast<mo_u32x4 *>(out + t * out_stride)[c] = pack8<T>(a);
}

}  // namespace mux

extern "C" int32_t mux_rms_norm(void *out, int64_t out_row_stride, const void *x, int64_t x_row_stride,
                                const void *weight, float eps, int32_t num_tokens, int32_t hidden_size,
                                int32_t dtype, void *stream) {
  using namespace mux;
  // (pointers are only required when there is something to do)
  if (num_tokens > 0 && (!out || !x || !weight)) return MUXA_EINVAL;
  if (num_tokens < 0 || hidden_size <= 0 || !(eps >= 0.f)) return MUXA_EINVAL;
  if (dtype != MUXA_DTYPE_F16 && dtype != MUXA_DTYPE_BF16) return MUXA_EUNSUPPORTED;
  if (hidden_size % 8) return MUXA_EUNSUPPORTED;
  if (out_row_stride < hidden_size || x_row_stride < hidden_size || out_row_stride % 8 || x_row_stride % 8)
    return MUXA_EINVAL;
  if ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight)) & 15u)
    return MUXA_EINVAL;
  if (num_tokens == 0) return MUXA_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // At most kRmsWavesPerCu waves per CU; rows beyond that are walked in sequence.
  static const int cus = [] {                      // compute units of the current device, asked once
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      return v;
    return 256;
  }();
  const int max_wgs = cus * kRmsWavesPerCu / 4;
  const dim3 grid(std::min((num_tokens + 3) / 4, max_wgs)), block(256);
  uint16_t *o = static_cast<uint16_t *>(out);
  const uint16_t *xi = static_cast<const uint16_t *>(x), *w = static_cast<const uint16_t *>(weight);
  const int nchunks = hidden_size / 8;
#define MUX_RMS_LAUNCH(TT, CPL)                                                                              \
  hipLaunchKernelGGL((rms_norm_kernel<TT, CPL>), grid, block, 0, st, o, out_row_stride, xi, x_row_stride, w, \
                     eps, hidden_size, num_tokens)
#define MUX_RMS_PICK(TT)                              \
  do {                                                \
    if (nchunks <= 64 * 4) MUX_RMS_LAUNCH(TT, 4);     \
    else if (nchunks <= 64 * 8) MUX_RMS_LAUNCH(TT, 8); \
    else if (nchunks <= 64 * 16) MUX_RMS_LAUNCH(TT, 16); \
    else MUX_RMS_LAUNCH(TT, 0);                       \
  } while (0)
  if (dtype == MUXA_DTYPE_F16) MUX_RMS_PICK(F16);
  else MUX_RMS_PICK(BF16);
#undef MUX_RMS_PICK
#undef MUX_RMS_LAUNCH
  MUX_HIP_TRY(hipGetLastError());
  return MUXA_OK;
}

extern "C" int32_t mux_silu_and_mul(void *out, int64_t out_row_stride, const void *x, int64_t x_row_stride,
                                    int32_t num_tokens, int32_t d, int32_t dtype, void *stream) {
  using namespace mux;
  if (num_tokens > 0 && (!out || !x)) return MUXA_EINVAL;
  if (num_tokens < 0 || d <= 0) return MUXA_EINVAL;
  if (dtype != MUXA_DTYPE_F16 && dtype != MUXA_DTYPE_BF16) return MUXA_EUNSUPPORTED;
  if (d % 8) return MUXA_EUNSUPPORTED;
  if (out_row_stride < d || x_row_stride < 2 * static_cast<int64_t>(d) || out_row_stride % 8 || x_row_stride % 8)
    return MUXA_EINVAL;
  if ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(x)) & 15u) return MUXA_EINVAL;
  if (num_tokens == 0) return MUXA_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int d8 = d / 8;
  const int64_t total = static_cast<int64_t>(num_tokens) * d8;
  const int64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return MUXA_EUNSUPPORTED;
  const dim3 grid(static_cast<uint32_t>(blocks)), block(256);
  if (dtype == MUXA_DTYPE_F16)
    hipLaunchKernelGGL(silu_and_mul_kernel<F16>, grid, block, 0, st, static_cast<uint16_t *>(out), out_row_stride,
                       static_cast<const uint16_t *>(x), x_row_stride, d8, total);
  else
    hipLaunchKernelGGL(silu_and_mul_kernel<BF16>, grid, block, 0, st, static_cast<uint16_t *>(out), out_row_stride,
                       static_cast<const uint16_t *>(x), x_row_stride, d8, total);
  MUX_HIP_TRY(hipGetLastError());
  return MUXA_OK;
}
