// Minimal logging / assertion front-end with the stream syntax the kuiper sources use
// (LOG(INFO) << ..., CHECK(cond) << ..., CHECK_EQ(a, b) ...).  The reference gets these from
// glog (kuiper/include/base/base.h:4); this build carries its own so that the library has no
// third-party dependency.  Semantics kept: a failed CHECK or a LOG(FATAL) prints file:line and
// the message to stderr and then terminates the process.
//
// For tests, base::set_fatal_handler() can replace "terminate" by a callback (for instance one
// that throws), which makes CHECK failures observable without losing the process.
#ifndef KUIPER_INCLUDE_BASE_LOG_H
#define KUIPER_INCLUDE_BASE_LOG_H

#include <sstream>
#include <string>

namespace base {

enum class LogSeverity : int { kInfo = 0, kWarning = 1, kError = 2, kFatal = 3 };

// Called with the full message of a fatal event.  If it returns, the process aborts.
using FatalHandler = void (*)(const std::string& message);
void set_fatal_handler(FatalHandler handler);

// Messages below this severity are dropped (default: kWarning, so LOG(INFO) is silent).
void set_min_log_severity(LogSeverity severity);

namespace detail {

class LogMessage {
public:
    LogMessage(const char* file, int line, LogSeverity severity);
    ~LogMessage() noexcept(false);
    std::ostream& stream() { return stream_; }

private:
    std::ostringstream stream_;
    LogSeverity severity_;
};

// Lets "cond ? (void)0 : Voidify() & LogMessage(...).stream() << x" type-check.
struct Voidify {
    void operator&(std::ostream&) {}
};

}  // namespace detail
}  // namespace base

#define KX_LOG_SEVERITY_INFO ::base::LogSeverity::kInfo
#define KX_LOG_SEVERITY_WARNING ::base::LogSeverity::kWarning
#define KX_LOG_SEVERITY_ERROR ::base::LogSeverity::kError
#define KX_LOG_SEVERITY_FATAL ::base::LogSeverity::kFatal

#define LOG(severity) ::base::detail::LogMessage(__FILE__, __LINE__, KX_LOG_SEVERITY_##severity).stream()

#define CHECK(condition)                                                                      \
    (condition) ? (void)0                                                                     \
                : ::base::detail::Voidify() &                                                 \
                      ::base::detail::LogMessage(__FILE__, __LINE__, ::base::LogSeverity::kFatal) \
                              .stream()                                                       \
                          << "Check failed: " #condition " "

#define KX_CHECK_OP(a, b, op)                                                                 \
    ((a)op(b)) ? (void)0                                                                      \
               : ::base::detail::Voidify() &                                                  \
                     ::base::detail::LogMessage(__FILE__, __LINE__, ::base::LogSeverity::kFatal) \
                             .stream()                                                        \
                         << "Check failed: " #a " " #op " " #b " "

#define CHECK_EQ(a, b) KX_CHECK_OP(a, b, ==)
#define CHECK_NE(a, b) KX_CHECK_OP(a, b, !=)
#define CHECK_LT(a, b) KX_CHECK_OP(a, b, <)
#define CHECK_LE(a, b) KX_CHECK_OP(a, b, <=)
#define CHECK_GT(a, b) KX_CHECK_OP(a, b, >)
#define CHECK_GE(a, b) KX_CHECK_OP(a, b, >=)

#endif  // KUIPER_INCLUDE_BASE_LOG_H
