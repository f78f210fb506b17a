// Thread-local error string behind ck_last_error_string(), the ABI revision and the debug options.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "ck_mi355.h"
#include "debug_options.h"

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
extern "C" int32_t ck_abi_version(void) { return 2; }

namespace ck {
DebugOptions& debug_options() {
  static DebugOptions options;
  return options;
}
}  // namespace ck

extern "C" int ck_debug_set_option(const char* name, int64_t value) {
  ck::DebugOptions& o = ck::debug_options();
  if (name != nullptr && strcmp(name, "gemm_line_kernel") == 0) o.gemm_line_kernel = value != 0;
  else if (name != nullptr && strcmp(name, "gemm_register_pipeline") == 0) o.gemm_register_pipeline = value != 0;
  else if (name != nullptr && strcmp(name, "gemm_four_waves") == 0) o.gemm_four_waves = value != 0;
  else if (name != nullptr && strcmp(name, "trace_buffer") == 0) o.trace_buffer = reinterpret_cast<void*>(static_cast<uintptr_t>(value));
  else {
    ck::set_error("ck_debug_set_option: unknown option '%s'", name ? name : "(null)");
    return CK_ERR_ARG;
  }
  return CK_OK;
}
