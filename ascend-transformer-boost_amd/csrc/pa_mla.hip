// Instantiations and dispatch of the 128-head decode-attention kernel for the combined MLA cache.
#include "pa_mla_kernel.h"

namespace atbmi {

int LaunchPaMlaWide(const AtbmiPaShape &s, const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream)
{
    if (!PaMlaWide(s)) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: shape does not fit the 128-head MLA kernel");
    }
    if (s.kvLayout == ATBMI_PA_KV_FRACTAL_NZ) {
        return s.qDtype == ATBMI_BF16 ? mla::LaunchAsm<true, true, true>(args, plan, stream)
                                      : mla::LaunchAsm<false, true, true>(args, plan, stream);
    }
    if (s.ropeDim != 0) {
        return s.qDtype == ATBMI_BF16 ? mla::LaunchAsm<true, true>(args, plan, stream)
                                      : mla::LaunchAsm<false, true>(args, plan, stream);
    }
    return s.qDtype == ATBMI_BF16 ? mla::LaunchAsm<true, false>(args, plan, stream)
                                  : mla::LaunchAsm<false, false>(args, plan, stream);
}

} // namespace atbmi
