// Chunked-prefill attention over the paged cache (placeholder until the MFMA kernel lands).
#include "fp_common.h"

extern "C" int fp_paged_prefill(const void*, int64_t, int64_t, const void*, const void*, const int64_t*, int64_t,
                                const int64_t*, const int64_t*, const int32_t*, void*, int64_t, int64_t, float*,
                                int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, int64_t, float, int,
                                void*) {
  return fp::fail(FP_ERR_UNSUPPORTED, "fp_paged_prefill: not built yet");
}
