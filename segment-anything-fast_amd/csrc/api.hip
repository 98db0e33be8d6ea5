// Library-level entry points: version, architecture, per-thread error text.
#include <pthread.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "samfast_internal.hpp"
#include "samfast_bench.h"

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

static const char* const kKnobNames[KNOB_COUNT] = {
    "SAMFAST_GEMM_TM",      "SAMFAST_GEMM_WG3",    "SAMFAST_GEMM_TILE", "SAMFAST_GEMM_SMALL_BELOW",
    "SAMFAST_GEMM_PERSIST", "SAMFAST_GEMM_PERSIST_SKEW", "SAMFAST_GEMM_PERSIST_PRIO", "SAMFAST_GEMM_SPLITK", "SAMFAST_ATTN_WAVES", "SAMFAST_ATTN_WINDOW_ROWS",
    "SAMFAST_SPARSE_PERSIST"};
static int g_knobs[KNOB_COUNT];
static pthread_once_t g_knobs_once = PTHREAD_ONCE_INIT;

static void knobs_from_environment() {
  for (int k = 0; k < KNOB_COUNT; ++k) {
    const char* e = getenv(kKnobNames[k]);
    g_knobs[k] = (e && *e) ? atoi(e) : kKnobUnset;
  }
}

int knob(Knob k) {
  pthread_once(&g_knobs_once, knobs_from_environment);
  return __atomic_load_n(&g_knobs[k], __ATOMIC_RELAXED);
}

}  // namespace samfast

extern "C" int samfast_bench_set_knob(const char* name, int value, int unset) {
  using namespace samfast;
  SF_REQUIRE(name, "bench_set_knob: null name");
  pthread_once(&g_knobs_once, knobs_from_environment);
  for (int k = 0; k < KNOB_COUNT; ++k)
    if (strcmp(name, kKnobNames[k]) == 0) {
      __atomic_store_n(&g_knobs[k], unset ? kKnobUnset : value, __ATOMIC_RELAXED);
      return SAMFAST_OK;
    }
  SF_FAIL(SAMFAST_E_INVALID, "bench_set_knob: unknown knob %s", name);
}

extern "C" int samfast_version(void) { return SAMFAST_VERSION; }
extern "C" const char* samfast_arch(void) { return "gfx950"; }
extern "C" const char* samfast_last_error(void) { return samfast::g_error; }
