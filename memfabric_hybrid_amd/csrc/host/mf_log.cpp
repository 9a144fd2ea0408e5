#include "mf_log.h"

#include <atomic>
#include <cstdio>
#include <cstring>

namespace mf {
namespace {
std::atomic<LogSink> g_sink{nullptr};
std::atomic<int> g_level{2};
thread_local std::string t_lastError;
const char *kNames[] = {"DEBUG", "INFO", "WARN", "ERROR"};
}  // namespace

void SetLogSink(LogSink sink)
{
    g_sink.store(sink);
}

int SetLogLevel(int level)
{
    if (level < 0 || level > 3) {
        return -1;
    }
    g_level.store(level);
    return 0;
}

int GetLogLevel()
{
    return g_level.load(std::memory_order_relaxed);
}

void LogMessage(int level, const char *file, int line, const std::string &text)
{
    if (level < 0) {
        level = 0;
    }
    if (level > 3) {
        level = 3;
    }
    const char *slash = std::strrchr(file, '/');
    std::string full = std::string("[mf_hip ") + (slash ? slash + 1 : file) + ":" + std::to_string(line) + "] " + text;
    LogSink sink = g_sink.load();
    if (sink != nullptr) {
        sink(level, full.c_str());
        return;
    }
    std::fprintf(stderr, "%s %s\n", kNames[level], full.c_str());
}

void SetLastError(const std::string &text)
{
    t_lastError = text;
}

const char *LastError()
{
    return t_lastError.c_str();
}

}  // namespace mf
