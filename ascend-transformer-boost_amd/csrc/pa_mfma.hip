// placeholder until the MFMA kernel lands
#include "pa_internal.h"
namespace atbmi {
bool PaMfmaSupports(const AtbmiPaShape &) { return false; }
int LaunchPaMfma(const AtbmiPaShape &, const PaArgs &, int, hipStream_t)
{
    return Fail(ERR_INVALID_PARAM, "pa_decode: MFMA kernel not built");
}
} // namespace atbmi
