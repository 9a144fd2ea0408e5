// Process-wide logger with a replaceable sink and a thread-local "last
// error" text, the two facilities the reference exposes through
// hybm_set_extern_logger / hybm_set_log_level (src/hybm/csrc/hybm_entry.cpp:143-161)
// and smem_get_last_err_msg (src/smem/csrc/common/smem_last_error.h).
// Levels: 0 DEBUG, 1 INFO, 2 WARN, 3 ERROR.
#ifndef MF_LOG_H
#define MF_LOG_H

#include <sstream>
#include <string>

namespace mf {

using LogSink = void (*)(int level, const char *msg);

void SetLogSink(LogSink sink);
int SetLogLevel(int level);  // 0 on success, -1 for an unknown level
int GetLogLevel();
void LogMessage(int level, const char *file, int line, const std::string &text);
void SetLastError(const std::string &text);
const char *LastError();

}  // namespace mf

#define MF_LOG(level, expr)                                          \
    do {                                                             \
        if ((level) >= ::mf::GetLogLevel()) {                        \
            std::ostringstream mfLogStream_;                         \
            mfLogStream_ << expr;                                    \
            ::mf::LogMessage((level), __FILE__, __LINE__, mfLogStream_.str()); \
        }                                                            \
    } while (0)

#define MF_DEBUG(expr) MF_LOG(0, expr)
#define MF_INFO(expr) MF_LOG(1, expr)
#define MF_WARN(expr) MF_LOG(2, expr)
#define MF_ERROR(expr) MF_LOG(3, expr)

// Log, remember as the thread's last error, and return `code`.
#define MF_FAIL(code, expr)                         \
    do {                                            \
        std::ostringstream mfFailStream_;           \
        mfFailStream_ << expr;                      \
        ::mf::SetLastError(mfFailStream_.str());    \
        MF_ERROR(mfFailStream_.str());              \
        return (code);                              \
    } while (0)

#endif  // MF_LOG_H
