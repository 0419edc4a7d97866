// Version and error reporting for the C ABI.
#include "fsa_common.h"

namespace fsa {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
}  // namespace fsa

extern "C" int fsa_version(void) { return 100; }
extern "C" const char* fsa_last_error(void) { return fsa::g_err; }
