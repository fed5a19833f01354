// Library-level entry points: version, error state, CU-masked streams.
#include "mux_common.h"

#include <vector>

extern "C" {

int32_t mux_attn_version(void) { return 300; }

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

int32_t mux_cu_parts_mask(uint32_t part_mask, int32_t num_cus, uint32_t *words, int32_t n_words) {
  if (!words || num_cus <= 0 || n_words < (num_cus + 31) / 32) return MUXA_EINVAL;
  if (part_mask == 0 || (part_mask >> MUXA_CU_PARTS) != 0) return MUXA_EINVAL;
  for (int w = 0; w < n_words; ++w) words[w] = 0u;
  int32_t enabled = 0;
  for (int p = 0; p < MUXA_CU_PARTS; ++p) {
    if (((part_mask >> p) & 1u) == 0) continue;
    const int lo = static_cast<int>(static_cast<int64_t>(num_cus) * p / MUXA_CU_PARTS);
    const int hi = static_cast<int>(static_cast<int64_t>(num_cus) * (p + 1) / MUXA_CU_PARTS);
    for (int i = lo; i < hi; ++i) words[i / 32] |= 1u << (i % 32);
    enabled += hi - lo;
  }
  return enabled;
}

int32_t mux_stream_create_cu_parts(void **stream_out, uint32_t part_mask, int32_t *num_cus_out) {
  if (!stream_out) return MUXA_EINVAL;
  int32_t info[2];
  const int32_t rc = mux_device_cu_info(info);
  if (rc != MUXA_OK) return rc;
  std::vector<uint32_t> mask((info[0] + 31) / 32, 0u);
  const int32_t enabled = mux_cu_parts_mask(part_mask, info[0], mask.data(), static_cast<int32_t>(mask.size()));
  if (enabled <= 0) return MUXA_EINVAL;
  hipStream_t st = nullptr;
  // Default priority: streams of different priorities are never mixed.
  MUX_HIP_TRY(hipExtStreamCreateWithCUMask(&st, static_cast<uint32_t>(mask.size()), mask.data()));
  *stream_out = st;
  if (num_cus_out) *num_cus_out = enabled;
  return MUXA_OK;
}

int32_t mux_stream_destroy(void *stream) {
  if (!stream) return MUXA_EINVAL;
  MUX_HIP_TRY(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return MUXA_OK;
}

}  // extern "C"
