#include "log.h"
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace atb {
namespace logging {
namespace {
int EnvLevel()
{
    const char *v = getenv("ASCEND_GLOBAL_LOG_LEVEL");
    if (v && *v >= '0' && *v <= '4' && v[1] == '\0') {
        return *v - '0';
    }
    return static_cast<int>(LogLevel::ERROR);
}
std::atomic<int> g_level{-1};
int Level()
{
    int l = g_level.load(std::memory_order_relaxed);
    if (l < 0) {
        l = EnvLevel();
        g_level.store(l, std::memory_order_relaxed);
    }
    return l;
}
const char *Name(LogLevel l)
{
    switch (l) {
        case LogLevel::DEBUG: return "DEBUG";
        case LogLevel::INFO: return "INFO";
        case LogLevel::WARN: return "WARN";
        case LogLevel::ERROR: return "ERROR";
        default: return "NONE";
    }
}
} // namespace

bool Enabled(LogLevel level)
{
    return level != LogLevel::NONE && static_cast<int>(level) >= Level();
}
void SetLevel(LogLevel level)
{
    g_level.store(static_cast<int>(level), std::memory_order_relaxed);
}
void ResetLevel()
{
    g_level.store(EnvLevel(), std::memory_order_relaxed);
}
void Emit(LogLevel level, const char *file, int line, const std::string &text)
{
    const char *base = strrchr(file, '/');
    fprintf(stderr, "[atb][%s] %s:%d %s\n", Name(level), base ? base + 1 : file, line, text.c_str());
}
} // namespace logging
} // namespace atb
