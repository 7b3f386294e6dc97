// Library-wide entry points of libolmax_hip: error reporting and version.
#include "common.h"
#include <string.h>
#include <dlfcn.h>
#include <atomic>
#include <mutex>

static thread_local char g_err[512] = "";

int olmax_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

extern "C" const char* olmax_last_error_string(void) { return g_err; }

extern "C" int32_t olmax_abi_version(void) { return 2; }

// ---- profiler ranges.  The reference wraps its modules in jax.named_scope / starts a JAX trace
// from ProfilerCallback (src/olmax/train/callbacks/profiler.py:33-50); here the whole-model entry
// points emit roctx ranges ("olmax.forward", "olmax.layers.<l>.backward", ...) that
// rocprofv3 --marker-trace shows on the host timeline.  The roctx library is looked up at run
// time the first time ranges are switched on; without it the switch reports an error and stays off.
static int (*g_roctx_push)(const char*) = nullptr;
static int (*g_roctx_pop)(void) = nullptr;
static std::atomic<bool> g_ranges_on{false};  // diagnostic switch, process-wide
static std::mutex g_roctx_mu;

extern "C" int32_t olmax_set_profiler_ranges(int32_t on) {
  std::lock_guard<std::mutex> lock(g_roctx_mu);
  if (on && !g_roctx_push) {
    // rocprofv3 listens to the SDK's roctx library; the roctracer one serves the older tools
    const char* names[] = {"librocprofiler-sdk-roctx.so", "librocprofiler-sdk-roctx.so.1", "libroctx64.so", "libroctx64.so.4"};
    void* h = nullptr;
    for (const char* n : names)
      if ((h = dlopen(n, RTLD_NOW | RTLD_GLOBAL))) break;
    if (h) {
      g_roctx_push = (int (*)(const char*))dlsym(h, "roctxRangePushA");
      g_roctx_pop = (int (*)(void))dlsym(h, "roctxRangePop");
    }
    if (!g_roctx_push || !g_roctx_pop) {
      g_roctx_push = nullptr;
      g_roctx_pop = nullptr;
      return olmax_set_error(OLMAX_ERR_ARG, "olmax_set_profiler_ranges: no roctx library (roctxRangePushA/Pop) found");
    }
  }
  g_ranges_on = on != 0;
  return OLMAX_OK;
}
void olmax_range_push(const char* fmt, ...) {
  if (!g_ranges_on) return;
  char name[96];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(name, sizeof(name), fmt, ap);
  va_end(ap);
  g_roctx_push(name);
}
void olmax_range_pop(void) {
  if (g_ranges_on) g_roctx_pop();
}
