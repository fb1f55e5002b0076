// Minimal stderr logger behind the ATB_LOG(LEVEL) << ... idiom.
// Level comes from ASCEND_GLOBAL_LOG_LEVEL (0 debug, 1 info, 2 warn, 3 error,
// 4 off; default error) or Utils::SetLogLevel at run time
// (reference include/atb/types.h:76-82, include/atb/utils.h:91-98).
#ifndef ATB_MI_LOG_H
#define ATB_MI_LOG_H
#include <sstream>
#include "atb/types.h"

namespace atb {
namespace logging {
bool Enabled(LogLevel level);
void SetLevel(LogLevel level);
void ResetLevel();
void Emit(LogLevel level, const char *file, int line, const std::string &text);

class Line {
public:
    Line(LogLevel level, const char *file, int line) : level_(level), file_(file), line_(line) {}
    ~Line() { Emit(level_, file_, line_, os_.str()); }
    std::ostringstream &Stream() { return os_; }

private:
    LogLevel level_;
    const char *file_;
    int line_;
    std::ostringstream os_;
};
} // namespace logging
} // namespace atb

#define ATB_LOG(LEVEL)                                       \
    if (!::atb::logging::Enabled(::atb::LogLevel::LEVEL)) {  \
    } else                                                   \
        ::atb::logging::Line(::atb::LogLevel::LEVEL, __FILE__, __LINE__).Stream()
#endif
