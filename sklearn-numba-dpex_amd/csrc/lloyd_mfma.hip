// fp32 Lloyd step on the matrix cores (v_mfma_f32_32x32x2_f32).  Not selected yet:
// lloyd_layout() never returns KMX_VARIANT_MFMA, and these entry points refuse to run.
#include "lloyd_layout.h"

#include <cstdlib>
#include <cstring>

int kmx_forced_variant() {
    const char* v = std::getenv("KMX_LLOYD_VARIANT");
    if (v == nullptr) return -1;
    if (std::strcmp(v, "stream") == 0) return KMX_VARIANT_STREAM;
    if (std::strcmp(v, "register") == 0) return KMX_VARIANT_REGISTER;
    if (std::strcmp(v, "mfma") == 0) return KMX_VARIANT_MFMA;
    return -1;
}

int32_t kmx_lloyd_iter_mfma_f32(const LloydLayout&, const void*, const void*, const void*, void*,
                                const uint32_t*, uint32_t*, void*, uint32_t*, char*, int64_t, int,
                                int, hipStream_t, hipEvent_t*) {
    return KMX_ERR_UNSUPPORTED;
}

int32_t kmx_assign_labels_mfma_f32(const LloydLayout&, const void*, const void*, uint32_t*, char*,
                                   int64_t, int, int, hipStream_t) {
    return KMX_ERR_UNSUPPORTED;
}
