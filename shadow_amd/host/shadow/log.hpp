// Error and logging convention of the host layer: a failed CHECK or a
// LOG(FATAL) prints the message to stderr and throws std::runtime_error, the
// way Shadow's LogMessage destructor does (shadow/util/log.hpp:92-118).
// INFO goes to stdout, WARNING/ERROR to stderr.  DLOG/DCHECK vanish under
// NDEBUG (shadow/util/log.hpp:47-82).
#ifndef SHADOW_AMD_HOST_LOG_HPP_
#define SHADOW_AMD_HOST_LOG_HPP_

#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>

namespace Shadow {

enum class LogSeverity { kInfo, kWarning, kError, kFatal };

class LogLine {
 public:
  LogLine(LogSeverity severity, const char* file, int line) : severity_(severity) {
    static const char* const names[] = {"INFO", "WARNING", "ERROR", "FATAL"};
    std::string path(file);
    const auto slash = path.find_last_of("/\\");
    text_ << names[static_cast<int>(severity)] << ": "
          << (slash == std::string::npos ? path : path.substr(slash + 1)) << ":" << line << "] ";
  }
  LogLine(const LogLine&) = delete;
  LogLine& operator=(const LogLine&) = delete;

  // Throwing from a destructor is deliberate: it is what lets
  // `CHECK(x) << "why"` collect the whole message first.
  ~LogLine() noexcept(false) {
    const std::string message = text_.str();
    (severity_ == LogSeverity::kInfo ? std::cout : std::cerr) << message << std::endl;
    if (severity_ == LogSeverity::kFatal) throw std::runtime_error(message);
  }

  std::ostream& stream() { return text_; }

 private:
  LogSeverity severity_;
  std::ostringstream text_;
};

// Lets the CHECK macros be expressions (no dangling-else hazard).
struct LogVoidify {
  void operator&(std::ostream&) const {}
};

}  // namespace Shadow

#define SHADOW_LOG_INFO ::Shadow::LogLine(::Shadow::LogSeverity::kInfo, __FILE__, __LINE__)
#define SHADOW_LOG_WARNING ::Shadow::LogLine(::Shadow::LogSeverity::kWarning, __FILE__, __LINE__)
#define SHADOW_LOG_ERROR ::Shadow::LogLine(::Shadow::LogSeverity::kError, __FILE__, __LINE__)
#define SHADOW_LOG_FATAL ::Shadow::LogLine(::Shadow::LogSeverity::kFatal, __FILE__, __LINE__)

#define LOG(severity) SHADOW_LOG_##severity.stream()
#define LOG_IF(severity, condition) \
  !(condition) ? (void)0 : ::Shadow::LogVoidify() & LOG(severity)

#define CHECK(condition) \
  (condition) ? (void)0 : ::Shadow::LogVoidify() & LOG(FATAL) << "Check Failed: " #condition " "
#define CHECK_NOTNULL(pointer)   \
  ((pointer) != nullptr) ? (void)0 \
                         : ::Shadow::LogVoidify() & LOG(FATAL) << "Check Failed: '" #pointer "' Must be non NULL "
#define SHADOW_CHECK_OP(op, a, b)                                                           \
  ((a)op(b)) ? (void)0                                                                      \
             : ::Shadow::LogVoidify() & LOG(FATAL) << "Check Failed: " #a " " #op " " #b " (" \
                                                   << (a) << " vs " << (b) << ") "
#define CHECK_EQ(a, b) SHADOW_CHECK_OP(==, a, b)
#define CHECK_NE(a, b) SHADOW_CHECK_OP(!=, a, b)
#define CHECK_LE(a, b) SHADOW_CHECK_OP(<=, a, b)
#define CHECK_LT(a, b) SHADOW_CHECK_OP(<, a, b)
#define CHECK_GE(a, b) SHADOW_CHECK_OP(>=, a, b)
#define CHECK_GT(a, b) SHADOW_CHECK_OP(>, a, b)

#if defined(NDEBUG)
#define DLOG(severity) true ? (void)0 : ::Shadow::LogVoidify() & LOG(severity)
#define DLOG_IF(severity, condition) true ? (void)0 : ::Shadow::LogVoidify() & LOG(severity)
#define DCHECK(condition) true ? (void)0 : ::Shadow::LogVoidify() & LOG(FATAL)
#else
#define DLOG(severity) LOG(severity)
#define DLOG_IF(severity, condition) LOG_IF(severity, condition)
#define DCHECK(condition) CHECK(condition)
#endif

#endif  // SHADOW_AMD_HOST_LOG_HPP_
