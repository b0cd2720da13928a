// Error plumbing shared by every entry point: the last error text is kept per host thread.
#include <stdarg.h>
#include <string.h>

#include "common.hpp"

namespace gptoss {

static thread_local char g_last_error[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

const char *last_error() { return g_last_error; }

}  // namespace gptoss

extern "C" const char *gptoss_last_error_string(void) { return gptoss::last_error(); }
extern "C" int gptoss_abi_version(void) { return 100; }
