// NeoX-style rotary position embedding applied in place to q and k, gfx950.
//
// For token t at position p, every head, pair index i < rot/2:
//     x = h[i], y = h[i + rot/2]
//     h[i]         = x * cos(p * f_i) - y * sin(p * f_i)
//     h[i + rot/2] = y * cos(p * f_i) + x * sin(p * f_i)
// cos/sin come from an fp32 table [max_position, rot] = [cos | sin] built on
// the host; arithmetic is fp32 and each result is rounded once to the storage
// type.  One workgroup per token; a thread handles two adjacent pair indices
// (4-byte loads/stores), heads of q first, then heads of k.
#include "mux_common.h"

namespace mux {

template <typename T>
__global__ __launch_bounds__(256) void rotary_neox_kernel(const int64_t *__restrict__ positions,
                                                          uint16_t *__restrict__ q, int64_t q_stride,
                                                          uint16_t *__restrict__ k, int64_t k_stride,
                                                          const float *__restrict__ cos_sin, int max_position,
                                                          int rot, int num_q_heads, int num_kv_heads) {
  constexpr int D = kHeadSize;
  const int t = blockIdx.x;
  int64_t pos = positions[t];
  pos = pos < 0 ? 0 : (pos >= max_position ? max_position - 1 : pos);
  const float *cs = cos_sin + pos * rot;
  const int half = rot / 2;
  const int per_head = half / 2;                       // thread items per head
  const int total = (num_q_heads + num_kv_heads) * per_head;
  for (int it = threadIdx.x; it < total; it += blockDim.x) {
    const int head = it / per_head;
    const int i = (it - head * per_head) * 2;
    uint16_t *row = head < num_q_heads ? q + t * q_stride + head * D
                                       : k + t * k_stride + (head - num_q_heads) * D;
    const uint32_t xv = *reinterpret_cast<const uint32_t *>(row + i);
    const uint32_t yv = *reinterpret_cast<const uint32_t *>(row + half + i);
    float x0, x1, y0, y1;
    if constexpr (__is_same(T, F16)) {
      const half2_t xh = as_half2(xv), yh = as_half2(yv);
      x0 = static_cast<float>(xh.x); x1 = static_cast<float>(xh.y);
      y0 = static_cast<float>(yh.x); y1 = static_cast<float>(yh.y);
    } else {
      x0 = bf16_lo(xv); x1 = bf16_hi(xv);
      y0 = bf16_lo(yv); y1 = bf16_hi(yv);
    }
    const float c0 = cs[i], c1 = cs[i + 1], s0 = cs[half + i], s1 = cs[half + i + 1];
    const uint32_t xo = static_cast<uint32_t>(to_storage<T>(x0 * c0 - y0 * s0)) |
                        (static_cast<uint32_t>(to_storage<T>(x1 * c1 - y1 * s1)) << 16);
    const uint32_t yo = static_cast<uint32_t>(to_storage<T>(y0 * c0 + x0 * s0)) |
                        (static_cast<uint32_t>(to_storage<T>(y1 * c1 + x1 * s1)) << 16);
    *reinterpret_cast<uint32_t *>(row + i) = xo;
    *reinterpret_cast<uint32_t *>(row + half + i) = yo;
  }
}

}  // namespace mux

extern "C" int32_t mux_rotary_neox(const int64_t *positions, void *q, int64_t q_row_stride, void *k,
                                   int64_t k_row_stride, const float *cos_sin, int32_t max_position,
                                   int32_t rotary_dim, int32_t num_tokens, int32_t num_q_heads,
                                   int32_t num_kv_heads, int32_t head_size, int32_t dtype, void *stream) {
  using namespace mux;
  // (pointers are only required when there is something to do)
  if (num_tokens > 0 && (!positions || !q || !k || !cos_sin)) return MUXA_EINVAL;
  if (num_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || max_position <= 0) return MUXA_EINVAL;
  if (head_size != kHeadSize) return MUXA_EUNSUPPORTED;
  if (rotary_dim <= 0 || rotary_dim > kHeadSize || rotary_dim % 4 != 0) return MUXA_EUNSUPPORTED;
  if (dtype != MUXA_DTYPE_F16 && dtype != MUXA_DTYPE_BF16) return MUXA_EUNSUPPORTED;
  if (q_row_stride < static_cast<int64_t>(num_q_heads) * kHeadSize ||
      k_row_stride < static_cast<int64_t>(num_kv_heads) * kHeadSize)
    return MUXA_EINVAL;
  if (q_row_stride % 2 || k_row_stride % 2) return MUXA_EINVAL;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k)) & 3u) return MUXA_EINVAL;
  if (num_tokens == 0) return MUXA_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == MUXA_DTYPE_F16)
    hipLaunchKernelGGL(rotary_neox_kernel<F16>, dim3(num_tokens), dim3(256), 0, st, positions,
                       static_cast<uint16_t *>(q), q_row_stride, static_cast<uint16_t *>(k), k_row_stride, cos_sin,
                       max_position, rotary_dim, num_q_heads, num_kv_heads);
  else
    hipLaunchKernelGGL(rotary_neox_kernel<BF16>, dim3(num_tokens), dim3(256), 0, st, positions,
                       static_cast<uint16_t *>(q), q_row_stride, static_cast<uint16_t *>(k), k_row_stride, cos_sin,
                       max_position, rotary_dim, num_q_heads, num_kv_heads);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e);
  return MUXA_OK;
}
