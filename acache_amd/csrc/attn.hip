// placeholder until the MFMA kernel lands: reports an error, launches nothing
#include "common.h"
extern "C" int acache_varlen_attn(
    void *, const void *, const void *, const void *, const int32_t *, const int32_t *, const int32_t *,
    float, int32_t, const int32_t *, const int32_t *, const float *, const float *, int32_t,
    int32_t, int64_t, int64_t, int32_t, int32_t, int32_t, int32_t, int64_t,
    int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, void *) {
  return acache::fail(ACACHE_E_MODE, "varlen_attn: kernel not built yet");
}
