// Library-wide pieces of the C ABI: version and per-thread error message.
#include "cxg_common.hpp"

namespace cxg {
namespace {
thread_local char g_error[512] = "";
}

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}
}  // namespace cxg

extern "C" {
int cxg_version(void) { return 100; }
const char* cxg_last_error(void) { return cxg::g_error; }
}
