// MFMA decode-attention instantiations for fp16 queries and caches.
#define BF16_OPERANDS false
#define PA_MFMA_LAUNCH_NAME LaunchPaMfmaF16
#include "pa_mfma_dispatch.inc"
