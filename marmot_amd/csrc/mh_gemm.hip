// Prefill GEMM route (dequantize-to-LDS + MFMA). Placeholder until the MFMA kernel lands: reports that no
// shape is supported so that callers take the small-batch route.
#include "mh_common.h"

namespace mh {

bool gemm_f16_supported(int, size_t, size_t, size_t) {
    return false;
}

int launch_gemm_f16(marmot_hip_device *, int, const void *, const void *, size_t, size_t, size_t, const void *, int,
                    void *, int) {
    return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "prefill GEMM route is not built");
}

} // namespace mh
