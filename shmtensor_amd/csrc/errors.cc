// Thread-local error channel behind shmt_last_error().
#include <stdarg.h>
#include <stdio.h>

#include "shmt.h"

namespace shmt {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

}  // namespace shmt

extern "C" {
int shmt_abi_version(void) { return SHMT_ABI_VERSION; }
const char *shmt_last_error(void) { return shmt::g_error; }
}
