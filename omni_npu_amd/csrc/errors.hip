// Error reporting and version for the C-ABI: entry points return 0 or a negative code and leave a
// thread-local message behind.
#include <cstdarg>
#include <cstdio>
#include "mla_common.hpp"

namespace mlahip {
static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return MLA_OK;
  return fail(MLA_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
}
}  // namespace mlahip

extern "C" int mlahip_version(void) { return 100; }
extern "C" const char* mlahip_last_error_string(void) { return mlahip::g_err; }
