// Error reporting and version for the C-ABI: entry points return 0 or a negative code and leave a
// thread-local message behind.
#include <cstdarg>
#include <cstdio>
#include <mutex>
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
// Kernels that use more dynamic LDS than the default limit must raise the limit once per device (the attribute belongs
// to the device's copy of the function).  Remembered per (kernel, device); callers may come from several threads.
int ensure_dynamic_lds(const void* kernel, int bytes, const char* what) {
  constexpr int kMaxDev = 64, kMaxFn = 64;   // (the library has about twenty kernels that need the raised limit)
  static std::mutex mu;
  static const void* fns[kMaxFn];
  static bool done[kMaxFn][kMaxDev];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev)
    return fail(MLA_ERR_LAUNCH, "%s: cannot identify the current device", what);
  std::lock_guard<std::mutex> lock(mu);
  int slot = 0;
  while (slot < kMaxFn && fns[slot] && fns[slot] != kernel) slot++;
  if (slot == kMaxFn) return fail(MLA_ERR_LAUNCH, "%s: kernel table full", what);
  fns[slot] = kernel;
  if (done[slot][dev]) return MLA_OK;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return fail(MLA_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, bytes, hipGetErrorString(e));
  done[slot][dev] = true;
  return MLA_OK;
}
}  // namespace mlahip

extern "C" int mlahip_version(void) { return 100; }
extern "C" const char* mlahip_last_error_string(void) { return mlahip::g_err; }
