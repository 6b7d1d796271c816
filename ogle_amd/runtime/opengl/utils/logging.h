// Minimal glog-shaped logging for the runtime.
//
// The reference aborts on any violated CHECK or LOG(FATAL)
// (ogl_runtime/opengl/utils/logging.h, macros.h:16-32).  Here a fatal message
// throws opengl::FatalError carrying "file:line message", so that a host
// application or test can observe the failure; set the environment variable
// OGLE_FATAL_ABORT=1 to get the reference's abort() instead.  The C API turns
// the exception into a negative status.
#ifndef OPENGL_UTILS_LOGGING_H_
#define OPENGL_UTILS_LOGGING_H_

#include <cstdlib>
#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>

namespace opengl {

class FatalError : public std::runtime_error {
 public:
  explicit FatalError(const std::string& what) : std::runtime_error(what) {}
};

namespace logging {

enum Severity { INFO = 0, WARNING = 1, ERROR = 2, FATAL = 3 };

inline int MinLogLevel() {
  static const int level = [] {
    const char* v = std::getenv("OGLE_MIN_LOG_LEVEL");
    return v ? std::atoi(v) : 1;  // warnings and above by default
  }();
  return level;
}

class Message {
 public:
  Message(const char* file, int line, Severity severity) : severity_(severity) {
    stream_ << file << ":" << line << " ";
  }
  // A fatal message throws from the destructor of a temporary, which is the
  // only place a streaming-style CHECK can act; noexcept(false) makes it legal.
  ~Message() noexcept(false) {
    if (severity_ == FATAL) {
      const char* v = std::getenv("OGLE_FATAL_ABORT");
      if (v != nullptr && v[0] == '1') {
        std::cerr << "F " << stream_.str() << std::endl;
        std::abort();
      }
      throw FatalError(stream_.str());
    }
    if (severity_ >= MinLogLevel()) {
      static const char kTag[] = {'I', 'W', 'E', 'F'};
      std::cerr << kTag[severity_] << " " << stream_.str() << std::endl;
    }
  }
  std::ostream& stream() { return stream_; }

 private:
  std::ostringstream stream_;
  Severity severity_;
};

// Swallows the stream of a disabled statement.
struct Voidify {
  void operator&(std::ostream&) {}
};

}  // namespace logging
}  // namespace opengl

#define LOG(severity) \
  ::opengl::logging::Message(__FILE__, __LINE__, ::opengl::logging::severity).stream()
#define DLOG(severity) \
  true ? (void)0 : ::opengl::logging::Voidify() & LOG(severity)
#define VLOG(level) DLOG(INFO)

#define CHECK(cond) \
  (cond) ? (void)0 : ::opengl::logging::Voidify() & LOG(FATAL) << "Check failed: " #cond " "
#define OGLE_CHECK_OP(a, b, op)                                                     \
  ((a)op(b)) ? (void)0                                                             \
             : ::opengl::logging::Voidify() &                                      \
                   LOG(FATAL) << "Check failed: " #a " " #op " " #b " (" << (a) << " vs " << (b) \
                              << ") "
#define CHECK_EQ(a, b) OGLE_CHECK_OP(a, b, ==)
#define CHECK_NE(a, b) OGLE_CHECK_OP(a, b, !=)
#define CHECK_LT(a, b) OGLE_CHECK_OP(a, b, <)
#define CHECK_LE(a, b) OGLE_CHECK_OP(a, b, <=)
#define CHECK_GT(a, b) OGLE_CHECK_OP(a, b, >)
#define CHECK_GE(a, b) OGLE_CHECK_OP(a, b, >=)
#define CHECK_NOTNULL(p) CHECK((p) != nullptr)

#endif  // OPENGL_UTILS_LOGGING_H_
