// Minimal leveled logging with the reference's macro names (TAO_VLOG, TAO_LOG,
// TAO_CHECK; reference: tao_compiler/mlir/ral/ral_logging.h).  Verbosity comes
// from TAO_CPP_MIN_VLOG_LEVEL, read once.
#ifndef RAL_RAL_LOGGING_H_
#define RAL_RAL_LOGGING_H_

#include <sstream>
#include <string>

namespace tao {
namespace ral {
namespace logging {

enum Severity { INFO = 0, WARNING = 1, ERROR = 2, FATAL = 3 };

int MinVLogLevel();

// Collects one message and emits it to stderr on destruction.  FATAL aborts.
class Message {
 public:
  Message(const char* file, int line, int severity);
  ~Message();
  std::ostringstream& stream() { return os_; }

 private:
  std::ostringstream os_;
  const char* file_;
  int line_;
  int severity_;
};

struct Voidify {
  void operator&(std::ostream&) {}
};

}  // namespace logging
}  // namespace ral
}  // namespace tao

#define TAO_VLOG_IS_ON(lvl) ((lvl) <= ::tao::ral::logging::MinVLogLevel())

#define TAO_LOG(severity)                                            \
  ::tao::ral::logging::Message(__FILE__, __LINE__,                   \
                               ::tao::ral::logging::severity)        \
      .stream()

#define TAO_VLOG(lvl)                  \
  !TAO_VLOG_IS_ON(lvl)                 \
      ? (void)0                        \
      : ::tao::ral::logging::Voidify() & TAO_LOG(INFO)

#define TAO_CHECK(cond) \
  (cond) ? (void)0 : ::tao::ral::logging::Voidify() & TAO_LOG(FATAL) << "Check failed: " #cond " "

#endif  // RAL_RAL_LOGGING_H_
