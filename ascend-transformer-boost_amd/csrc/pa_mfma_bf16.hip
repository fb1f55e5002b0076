// MFMA decode-attention instantiations for bf16 queries and caches.
#define BF16_OPERANDS true
#define PA_MFMA_LAUNCH_NAME LaunchPaMfmaBf16
#include "pa_mfma_dispatch.inc"
