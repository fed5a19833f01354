// Shared device/host helpers for the gfx950 kernels of libmuxattn.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "muxserve_attn.h"

namespace mux {

constexpr int kHeadSize = 128;          // muxserve/flexstore/manager.py:337
constexpr int kWave = 64;               // CDNA wavefront
constexpr int kChunkElems = 8;          // one 16-byte chunk = 8 fp16/bf16 = the pool's "x"

// Last HIP error seen by this library on this thread.
extern thread_local int32_t g_last_hip_error;

inline int32_t hip_fail(hipError_t e) {
  g_last_hip_error = static_cast<int32_t>(e);
  return MUXA_EHIP;
}

#define MUX_HIP_TRY(expr)                                 \
  do {                                                    \
    hipError_t _e = (expr);                               \
    if (_e != hipSuccess) return ::mux::hip_fail(_e);     \
  } while (0)

// ---- scalar conversions -------------------------------------------------
struct F16 {};   // IEEE half storage
struct BF16 {};  // bfloat16 storage

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ half2_t as_half2(uint32_t u) {
  union { uint32_t u; half2_t h; } c;
  c.u = u;
  return c.h;
}

typedef __bf16 bf162_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ bf162_t as_bf162(uint32_t u) {
  union { uint32_t u; bf162_t h; } c;
  c.u = u;
  return c.h;
}

// fp32 -> bf16 bits, round to nearest even (NaN kept quiet).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  union { _Float16 h; uint16_t u; } c;
  c.h = static_cast<_Float16>(f);
  return c.u;
}

template <typename T>
__device__ __forceinline__ uint16_t to_storage(float f) {
  if constexpr (__is_same(T, F16)) return f32_to_f16_bits(f);
  else return f32_to_bf16_bits(f);
}

// acc + a.x*b.x + a.y*b.y with a, b packed pairs in storage type T, fp32 accumulate.
template <typename T>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
  if constexpr (__is_same(T, F16)) {
    return __builtin_amdgcn_fdot2(as_half2(a), as_half2(b), acc, false);
  } else {
    return __builtin_amdgcn_fdot2_f32_bf16(as_bf162(a), as_bf162(b), acc, false);   // v_dot2c_f32_bf16
  }
}

// acc + lo(v)*p0 + hi(v)*p1, v a packed pair in storage type T, p fp32.
template <typename T>
__device__ __forceinline__ float fma2(uint32_t v, float p0, float p1, float acc) {
  if constexpr (__is_same(T, F16)) {
    half2_t h = as_half2(v);
    acc = __builtin_fmaf(static_cast<float>(h.x), p0, acc);
    return __builtin_fmaf(static_cast<float>(h.y), p1, acc);
  } else {
    acc = __builtin_fmaf(bf16_lo(v), p0, acc);
    return __builtin_fmaf(bf16_hi(v), p1, acc);
  }
}

// ---- wave64 reductions with DPP (no LDS traffic) --------------------------
template <int kCtrl>
__device__ __forceinline__ float dpp_mov(float v) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xf, 0xf, true));
}

// After this every lane of a 16-lane row holds the row's max.
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_mov<0xB1>(v));    // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp_mov<0x4E>(v));    // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp_mov<0x141>(v));   // row_half_mirror
  v = fmaxf(v, dpp_mov<0x140>(v));   // row_mirror
  return v;
}
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_mov<0xB1>(v);
  v += dpp_mov<0x4E>(v);
  v += dpp_mov<0x141>(v);
  v += dpp_mov<0x140>(v);
  return v;
}
__device__ __forceinline__ float lane_bcast(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ float wave_max(float v) {
  v = row16_max(v);
  return fmaxf(fmaxf(lane_bcast(v, 0), lane_bcast(v, 16)), fmaxf(lane_bcast(v, 32), lane_bcast(v, 48)));
}
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  return (lane_bcast(v, 0) + lane_bcast(v, 16)) + (lane_bcast(v, 32) + lane_bcast(v, 48));
}

// A lane's value combined with that of lane ^ 32 (lane ^ 16), on the vector ALU:
// v_permlane32_swap exchanges the upper half of one register with the lower
// half of another (v_permlane16_swap: the odd 16-lane rows of one with the even
// rows of the other), so with the same value in both, every lane ends up with
// its own half's value in one result and the other half's in the other.  The
// usual __shfl_xor is a ds_bpermute, which queues behind the LDS traffic of the
// whole compute unit.
__device__ __forceinline__ float max_with_lane_xor32(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_with_lane_xor32(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float max_with_lane_xor16(float v) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_with_lane_xor16(float v) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Blocks this wave until every vector-memory access it has issued - loads AND
// stores - has completed (on gfx9 stores count in vmcnt and are acknowledged
// once they have reached the level their scope bits name).  A workgroup-scope
// fence does not emit this wait for agent-scope relaxed stores, so code that
// publishes data to other workgroups and then bumps an arrival counter calls it
// between the two.
__device__ __forceinline__ void wait_own_vector_memory() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Inclusive prefix sum over the 64 lanes of a wave (row shifts, then the two
// cross-row broadcasts of the GCN/CDNA DPP unit).  Lanes whose DPP source is
// outside the row or masked off receive 0.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ int dpp_or_zero(int v) {
  return __builtin_amdgcn_update_dpp(0, v, kCtrl, kRowMask, 0xf, false);
}
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  v += dpp_or_zero<0x111, 0xf>(v);   // row_shr:1
  v += dpp_or_zero<0x112, 0xf>(v);   // row_shr:2
  v += dpp_or_zero<0x114, 0xf>(v);   // row_shr:4
  v += dpp_or_zero<0x118, 0xf>(v);   // row_shr:8
  v += dpp_or_zero<0x142, 0xa>(v);   // row_bcast:15 -> rows 1 and 3
  v += dpp_or_zero<0x143, 0xc>(v);   // row_bcast:31 -> rows 2 and 3
  return v;
}

}  // namespace mux
