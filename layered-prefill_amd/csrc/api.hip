// Error reporting shared by every entry point of libmoe_gfx950.so.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace {
thread_local char g_last_error[512] = "";
}

int moe_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int moe_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return MOE_OK;
  return moe_fail(MOE_ERR_LAUNCH, "%s: kernel launch failed: %s", what, hipGetErrorString(e));
}

int moe_opt_in_lds(MoeLdsOptIn& flags, const void* kernel, int lds_bytes, const char* what) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) dev = 0;
  const bool tracked = dev < kMoeMaxDevices;  // devices beyond the table set the attribute on every call
  if (tracked && flags.done[dev].load(std::memory_order_acquire)) return MOE_OK;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  if (e != hipSuccess)
    return moe_fail(MOE_ERR_LAUNCH, "%s: cannot reserve %d B of LDS: %s", what, lds_bytes, hipGetErrorString(e));
  if (tracked) flags.done[dev].store(true, std::memory_order_release);  // two threads setting it twice is harmless
  return MOE_OK;
}

MOE_EXPORT const char* moe_last_error(void) { return g_last_error; }

MOE_EXPORT int moe_abi_version(void) { return 2; }
