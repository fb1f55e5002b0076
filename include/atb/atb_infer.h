// Umbrella header for inference callers (reference include/atb/atb_infer.h).
#ifndef ATB_ATB_INFER_H
#define ATB_ATB_INFER_H
#include "atb/types.h"
#include "atb/svector.h"
#include "atb/context.h"
#include "atb/operation.h"
#include "atb/utils.h"
#include "atb/infer_op_params.h"
#endif
