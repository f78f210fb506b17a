// Thread-local error string behind ck_last_error_string().
#include <stdarg.h>
#include <stdio.h>

#include "ck_mi355.h"

namespace ck {
static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace ck

extern "C" const char* ck_last_error_string(void) { return ck::g_error; }
extern "C" int32_t ck_abi_version(void) { return 1; }
