// Library attributes and error reporting of the C ABI.
#include <stdarg.h>
#include <stdio.h>

#include "ac4k_common.h"

namespace ac4k {

static thread_local char g_last_error[512] = "";

int set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return 1;
}

int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

}  // namespace ac4k

extern "C" __attribute__((visibility("default"))) const char *ac4k_arch(void) { return "gfx950"; }
extern "C" __attribute__((visibility("default"))) const char *ac4k_arch_description(void) { return "AMD Instinct MI355X (CDNA4)"; }
extern "C" __attribute__((visibility("default"))) const char *ac4k_backend(void) { return "rocm"; }
extern "C" __attribute__((visibility("default"))) const char *ac4k_version(void) { return "0.1.0"; }
extern "C" __attribute__((visibility("default"))) const char *ac4k_last_error(void) { return ac4k::g_last_error; }
