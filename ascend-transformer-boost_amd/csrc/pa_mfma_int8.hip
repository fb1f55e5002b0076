// MFMA decode-attention instantiations for int8 caches (fp16 or bf16 queries;
// the matrix cores run in fp16 either way, int8 values are exact in fp16).
#include "pa_mfma_kernel.h"

namespace atbmi {

int LaunchPaMfmaInt8(const AtbmiPaShape &s, const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream)
{
    using namespace mfma;
    if (s.mlaCombined || s.headDimK != s.headDimV) {
        return -1;
    }
    switch (s.headDimK) { // every multiple of 32 from 64 to 256
        case 64:
            return Launch<false, true, 64, 64, false, true, 8>(args, plan, stream);
        case 96:
            return Launch<false, true, 96, 96, false, true, 8>(args, plan, stream);
        case 128:
            return Launch<false, true, 128, 128, false, true, 8>(args, plan, stream);
        case 160:
            return Launch<false, true, 160, 160, false, true, 4>(args, plan, stream);
        case 192:
            return Launch<false, true, 192, 192, false, true, 4>(args, plan, stream);
        case 224:
            return Launch<false, true, 224, 224, false, true, 4>(args, plan, stream);
        case 256:
            return Launch<false, true, 256, 256, false, true, 4>(args, plan, stream);
        default:
            return -1;
    }
}

} // namespace atbmi
