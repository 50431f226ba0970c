// MoE entry points (top-k, router softmax, grouped experts).
#include "mh_common.h"

using namespace mh;

extern "C" {

int marmot_hip_topk(marmot_hip_device_t *, const float *, size_t, size_t, size_t, float *, int32_t *) {
    return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "topk is not built yet");
}

int marmot_hip_softmax_rows(marmot_hip_device_t *, const float *, size_t, size_t, float *) {
    return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "softmax_rows is not built yet");
}

int marmot_hip_moe_experts(marmot_hip_device_t *, const float *, size_t, size_t, size_t, size_t, size_t, int, int,
                           const void *, const void *, const void *, const int32_t *, const float *, float, int, int,
                           float *) {
    return set_error(MARMOT_HIP_ERROR_NOT_IMPLEMENTED, "moe_experts is not built yet");
}

} // extern "C"
