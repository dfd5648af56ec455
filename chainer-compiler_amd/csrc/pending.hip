// Entry points declared in chx_hip.h whose kernels are not written yet.  Each one
// fails loudly; none computes anything.
#include "chx_internal.h"

extern "C" {

int chx_hip_qconv_plan_create(
        const chx_hip_tensor*, const chx_hip_tensor*, const chx_hip_tensor*, const chx_hip_tensor*,
        const chx_hip_conv_params*, void*, chx_hip_qconv_plan**) {
    CHX_FAIL(CHX_HIP_EUNSUPPORTED, "chx_hip_qconv_plan_create: not implemented");
}
int chx_hip_qconv_plan_run(
        const chx_hip_qconv_plan*, const chx_hip_tensor*, float, int32_t, float, int32_t, uint32_t, chx_hip_tensor*,
        void*) {
    CHX_FAIL(CHX_HIP_EUNSUPPORTED, "chx_hip_qconv_plan_run: not implemented");
}
void chx_hip_qconv_plan_destroy(chx_hip_qconv_plan*) {
}
}
