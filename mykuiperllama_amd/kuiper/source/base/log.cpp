#include "base/log.h"

#include <cstdio>
#include <cstdlib>

namespace base {
namespace {
FatalHandler g_fatal_handler = nullptr;
LogSeverity g_min_severity = LogSeverity::kWarning;

const char* severity_tag(LogSeverity s) {
    switch (s) {
        case LogSeverity::kInfo: return "I";
        case LogSeverity::kWarning: return "W";
        case LogSeverity::kError: return "E";
        default: return "F";
    }
}
}  // namespace

void set_fatal_handler(FatalHandler handler) {
    g_fatal_handler = handler;
}

void set_min_log_severity(LogSeverity severity) {
    g_min_severity = severity;
}

namespace detail {

LogMessage::LogMessage(const char* file, int line, LogSeverity severity) : severity_(severity) {
    stream_ << severity_tag(severity) << " " << file << ":" << line << "] ";
}

LogMessage::~LogMessage() noexcept(false) {
    const std::string text = stream_.str();
    if (severity_ >= g_min_severity) {
        std::fprintf(stderr, "%s\n", text.c_str());
        std::fflush(stderr);
    }
    if (severity_ == LogSeverity::kFatal) {
        if (g_fatal_handler) {
            g_fatal_handler(text);  // may throw
        }
        std::abort();
    }
}

}  // namespace detail
}  // namespace base
