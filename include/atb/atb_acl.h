// The aclnn-style two-call C wrappers of the reference (include/atb/atb_acl.h) for the operations
// this library has: the first call creates the operation if *op is null, binds the tensors and
// runs Setup (returning the workspace size), the second runs Execute on what the first bound.
//   AtbMLAGetWorkspaceSize / AtbMLA                      reference include/atb/atb_acl.h:99-116
//   AtbMLAPreFillGetWorkspaceSize / AtbMLAPreFill        reference include/atb/atb_acl.h:141-156
//   AtbPagedCacheLoadGetWorkspaceSize / AtbPagedCacheLoad  reference include/atb/atb_acl.h:251-267
// contextLens and qSeqLen are host tensors: their aclTensor carries a host address.
#ifndef ATB_MI_ATB_ACL_H
#define ATB_MI_ATB_ACL_H
#include <acl/acl.h>
#include "atb/context.h"
#include "atb/infer_op_params.h"
#include "atb/operation.h"
#include "atb/types.h"

#ifdef __cplusplus
extern "C" {
#endif

// MultiLatentAttention (cacheMode KROPE_CTKV, NZCACHE or INT8_NZCACHE). mask is read when maskType is not
// UNDEFINED, qSeqLen when calcType is CALC_TYPE_SPEC, lse when calcType is CALC_TYPE_RING, qkDescale /
// pvDescale with the int8 cache mode. Pointers that are not read may be null.
atb::Status AtbMLAGetWorkspaceSize(const aclTensor *qNope, const aclTensor *qRope, const aclTensor *ctKV,
                                   const aclTensor *kRope, const aclTensor *blockTables, const aclTensor *contextLens,
                                   const aclTensor *mask, const aclTensor *qSeqLen, const aclTensor *qkDescale,
                                   const aclTensor *pvDescale, int32_t headNum, float qkScale, int32_t kvHeadNum,
                                   int maskType, int calcType, uint8_t cacheMode, aclTensor *attenOut, aclTensor *lse,
                                   uint64_t *workspaceSize, atb::Operation **op, atb::Context *context);
atb::Status AtbMLA(void *workspace, uint64_t workspaceSize, atb::Operation *op, atb::Context *context);

// MultiLatentAttention, calcType PREFILL (cacheMode KROPE_CTKV): attention of whole prompts over key / keyRope /
// value tensors. qSeqLen and kvSeqLen are host tensors; mask is read when maskType is MASK_TYPE_MASK_FREE.
atb::Status AtbMLAPreFillGetWorkspaceSize(const aclTensor *q, const aclTensor *qRope, const aclTensor *k,
                                          const aclTensor *kRope, const aclTensor *v, const aclTensor *qSeqLen,
                                          const aclTensor *kvSeqLen, const aclTensor *mask, int32_t headNum,
                                          float qkScale, int32_t kvHeadNum, int maskType, uint8_t cacheMode,
                                          aclTensor *attenOut, uint64_t *workspaceSize, atb::Operation **op,
                                          atb::Context *context);
atb::Status AtbMLAPreFill(void *workspace, uint64_t workspaceSize, atb::Operation *op, atb::Context *context);

// PagedCacheLoad. key and value are inputs and outputs at once; seqStarts is read when hasSeqStarts.
atb::Status AtbPagedCacheLoadGetWorkspaceSize(const aclTensor *keyCache, const aclTensor *valueCache,
                                              const aclTensor *blockTables, const aclTensor *contextLens,
                                              const aclTensor *key, const aclTensor *value, const aclTensor *seqStarts,
                                              int8_t kvCacheCfg, bool isSeqLensCumsumType, bool hasSeqStarts,
                                              uint64_t *workspaceSize, atb::Operation **op, atb::Context *context);
atb::Status AtbPagedCacheLoad(void *workspace, uint64_t workspaceSize, atb::Operation *op, atb::Context *context);

#ifdef __cplusplus
}
#endif
#endif
