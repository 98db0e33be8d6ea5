// Library-level entry points: version, architecture, per-thread error text.
#include <stdarg.h>
#include <stdio.h>

#include "samfast_internal.hpp"

namespace samfast {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return SAMFAST_E_LAUNCH;
  }
  return SAMFAST_OK;
}

}  // namespace samfast

extern "C" int samfast_version(void) { return SAMFAST_VERSION; }
extern "C" const char* samfast_arch(void) { return "gfx950"; }
extern "C" const char* samfast_last_error(void) { return samfast::g_error; }
