// Context factory and implementation (reference src/atb/context/context_base.cpp,
// include/atb/context.h:153-194).
#include "context_impl.h"
#include <new>
#include "log.h"

namespace atb {
namespace {
// The execute type is per thread in the reference (context_base.h:67): the
// two-thread pre-launch / launch split sets it from both threads.
thread_local ExecuteType t_executeType = EXECUTE_NORMAL;
} // namespace

Status ContextImpl::SetExecuteStream(aclrtStream stream)
{
    streams_.at(0) = stream;
    return NO_ERROR;
}
aclrtStream ContextImpl::GetExecuteStream() const
{
    return streams_.at(0);
}
Status ContextImpl::SetAsyncTilingCopyStatus(bool enable)
{
    // The plan upload already runs asynchronously on the execute stream.
    asyncTilingCopy_ = enable;
    return NO_ERROR;
}
bool ContextImpl::GetAsyncTilingCopyStatus() const
{
    return asyncTilingCopy_;
}
Status ContextImpl::SetExecuteStreams(const std::vector<aclrtStream> &streams)
{
    if (streams.empty()) {
        ATB_LOG(ERROR) << "SetExecuteStreams: empty stream list";
        return ERROR_INVALID_PARAM;
    }
    streams_ = streams;
    return NO_ERROR;
}
std::vector<aclrtStream> ContextImpl::GetExecuteStreams()
{
    return streams_;
}
Status ContextImpl::SetExecuteType(ExecuteType type)
{
    if (type < EXECUTE_NORMAL || type > EXECUTE_LAUNCH) {
        return ERROR_INVALID_PARAM;
    }
    t_executeType = type;
    return NO_ERROR;
}
ExecuteType ContextImpl::GetExecuteType()
{
    return t_executeType;
}
Status ContextImpl::SetLaunchMode(LaunchMode mode)
{
    if (mode < KERNEL_LAUNCH_MODE || mode > GRAPH_LAUNCH_MODE) {
        return ERROR_INVALID_PARAM;
    }
    launchMode_ = mode;
    return NO_ERROR;
}
LaunchMode ContextImpl::GetLaunchMode()
{
    return launchMode_;
}

Status CreateContext(Context **context)
{
    if (!context) {
        ATB_LOG(ERROR) << "CreateContext: null out pointer";
        return ERROR_INVALID_PARAM;
    }
    ContextImpl *impl = new (std::nothrow) ContextImpl();
    if (!impl) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    *context = impl;
    return NO_ERROR;
}

Status CreateContext(Context **context, const std::function<void *(size_t)> &alloc,
                     const std::function<void(void *)> &dealloc)
{
    if (!alloc || !dealloc) {
        ATB_LOG(ERROR) << "CreateContext: allocator pair must be callable";
        return ERROR_INVALID_PARAM;
    }
    return CreateContext(context);
}

Status CreateContext(Context **context, uint32_t hostTilingBlockNum, uint32_t deviceTilingBlockNum)
{
    if (hostTilingBlockNum < 128 || hostTilingBlockNum > 1024 || deviceTilingBlockNum < 32 ||
        deviceTilingBlockNum > 1024) {
        ATB_LOG(ERROR) << "CreateContext: tiling block counts out of range";
        return ERROR_INVALID_PARAM;
    }
    return CreateContext(context);
}

Status DestroyContext(Context *context)
{
    delete context;
    return NO_ERROR;
}
} // namespace atb
