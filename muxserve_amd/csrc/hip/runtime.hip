// Library-level entry points: version, error state, CU-masked streams.
#include "mux_common.h"

#include <vector>

extern "C" {

int32_t mux_attn_version(void) { return 100; }

int32_t mux_last_hip_error(void) { return mux::g_last_hip_error; }

int32_t mux_device_cu_info(int32_t out[2]) {
  if (!out) return MUXA_EINVAL;
  int dev = 0;
  MUX_HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  MUX_HIP_TRY(hipGetDeviceProperties(&prop, dev));
  out[0] = prop.multiProcessorCount;
  // gfx950 (MI355X): 8 accelerator dies of 32 CUs each.
  out[1] = prop.multiProcessorCount % 32 == 0 ? prop.multiProcessorCount / 32 : 1;
  return MUXA_OK;
}

int32_t mux_stream_create_cu_range(void **stream_out, int32_t lo_percent, int32_t hi_percent,
                                   int32_t *num_cus_out) {
  if (!stream_out) return MUXA_EINVAL;
  if (lo_percent < 0 || hi_percent > 100 || lo_percent >= hi_percent) return MUXA_EINVAL;
  int32_t info[2];
  const int32_t rc = mux_device_cu_info(info);
  if (rc != MUXA_OK) return rc;
  const int n = info[0];
  const int lo = static_cast<int>(static_cast<int64_t>(n) * lo_percent / 100);
  const int hi = static_cast<int>(static_cast<int64_t>(n) * hi_percent / 100);
  if (hi <= lo) return MUXA_EINVAL;
  std::vector<uint32_t> mask((n + 31) / 32, 0u);
  for (int i = lo; i < hi; ++i) mask[i / 32] |= 1u << (i % 32);
  hipStream_t st = nullptr;
  // Default priority: streams of different priorities are never mixed.
  MUX_HIP_TRY(hipExtStreamCreateWithCUMask(&st, static_cast<uint32_t>(mask.size()), mask.data()));
  *stream_out = st;
  if (num_cus_out) *num_cus_out = hi - lo;
  return MUXA_OK;
}

int32_t mux_stream_destroy(void *stream) {
  if (!stream) return MUXA_EINVAL;
  MUX_HIP_TRY(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return MUXA_OK;
}

}  // extern "C"
