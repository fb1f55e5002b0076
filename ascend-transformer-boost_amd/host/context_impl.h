// The one concrete atb::Context of this library: holds the execute stream(s)
// and the mode switches (reference src/atb/context/context_base.h:19-73).
#ifndef ATB_MI_CONTEXT_IMPL_H
#define ATB_MI_CONTEXT_IMPL_H
#include "atb/context.h"

namespace atb {
class ContextImpl : public Context {
public:
    Status SetExecuteStream(aclrtStream stream) override;
    aclrtStream GetExecuteStream() const override;
    Status SetAsyncTilingCopyStatus(bool enable) override;
    bool GetAsyncTilingCopyStatus() const override;
    Status SetExecuteStreams(const std::vector<aclrtStream> &streams) override;
    std::vector<aclrtStream> GetExecuteStreams() override;
    Status SetExecuteType(ExecuteType type) override;
    ExecuteType GetExecuteType() override;
    Status SetLaunchMode(LaunchMode mode) override;
    LaunchMode GetLaunchMode() override;

private:
    std::vector<aclrtStream> streams_{nullptr};
    bool asyncTilingCopy_ = false;
    LaunchMode launchMode_ = KERNEL_LAUNCH_MODE;
};
} // namespace atb
#endif
