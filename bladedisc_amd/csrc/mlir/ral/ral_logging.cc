#include "mlir/ral/ral_logging.h"

#include <cstdio>
#include <cstdlib>

namespace tao {
namespace ral {
namespace logging {

int MinVLogLevel() {
  static const int level = [] {
    const char* v = std::getenv("TAO_CPP_MIN_VLOG_LEVEL");
    return v ? std::atoi(v) : -1;
  }();
  return level;
}

Message::Message(const char* file, int line, int severity)
    : file_(file), line_(line), severity_(severity) {}

Message::~Message() {
  static const char tags[] = "IWEF";
  std::fprintf(stderr, "[ral %c %s:%d] %s\n", tags[severity_ & 3], file_, line_,
               os_.str().c_str());
  if (severity_ == FATAL) std::abort();
}

}  // namespace logging
}  // namespace ral
}  // namespace tao
