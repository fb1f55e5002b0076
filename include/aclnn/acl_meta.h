// atb/types.h includes this CANN header next to acl/acl.h; nothing from it is
// used on the PagedAttention / ReshapeAndCache path.
#ifndef ATB_MI_ACLNN_META_SHIM_H
#define ATB_MI_ACLNN_META_SHIM_H
#include <acl/acl.h>
#endif
