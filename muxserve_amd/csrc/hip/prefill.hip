// Causal prefill attention (placeholder until the MFMA kernel lands).
#include "mux_common.h"

extern "C" int32_t mux_prefill_causal(void *, int64_t, const void *, int64_t, const void *, const void *,
                                      int64_t, const int32_t *, int32_t, int32_t, int32_t, int32_t,
                                      int32_t, float, int32_t, void *) {
  return MUXA_EUNSUPPORTED;
}
