// atb::Context - carries the stream an Operation launches on, plus the
// execute/launch mode switches of the reference API
// (reference include/atb/context.h:34-142 for the class, :153-194 for the
// factory functions).
#ifndef ATB_CONTEXT_H
#define ATB_CONTEXT_H
#include <cstddef>
#include <cstdint>
#include <functional>
#include <vector>
#include <acl/acl.h>
#include "atb/types.h"

namespace atb {
enum ExecuteType : int {
    EXECUTE_NORMAL = 0, // Execute checks, uploads the plan and launches
    EXECUTE_PRELAUNCH,  // first half only: checks + plan upload
    EXECUTE_LAUNCH,     // second half only: kernel launches
};

enum LaunchMode : int {
    KERNEL_LAUNCH_MODE = 0,
    GRAPH_LAUNCH_MODE // accepted and stored; kernels are still launched one by one
};

class Context {
public:
    Context() = default;
    virtual ~Context() = default;

    // The stream is a hipStream_t carried in an aclrtStream.
    virtual Status SetExecuteStream(aclrtStream stream) = 0;
    virtual aclrtStream GetExecuteStream() const = 0;

    virtual Status SetAsyncTilingCopyStatus(bool enable) = 0;
    virtual bool GetAsyncTilingCopyStatus() const = 0;

    virtual Status SetExecuteStreams(const std::vector<aclrtStream> &streams) = 0;
    virtual std::vector<aclrtStream> GetExecuteStreams() = 0;

    virtual Status SetExecuteType(ExecuteType type) = 0;
    virtual ExecuteType GetExecuteType() = 0;

    virtual Status SetLaunchMode(LaunchMode mode) = 0;
    virtual LaunchMode GetLaunchMode() = 0;
};

Status CreateContext(Context **context);
// The allocator pair and the tiling-block counts configure Ascend tiling
// buffers; they are validated like the reference does and otherwise unused.
Status CreateContext(Context **context, const std::function<void *(size_t)> &alloc,
                     const std::function<void(void *)> &dealloc);
Status CreateContext(Context **context, uint32_t hostTilingBlockNum, uint32_t deviceTilingBlockNum);
Status DestroyContext(Context *context);
} // namespace atb
#endif
