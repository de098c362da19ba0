// Named ranges on a profiler's timeline, the counterpart of the reference's NVTX
// annotations (csrc/layerwise.cpp:1073, 1380; flexkv/transfer/worker.py:556-587).
// The ROCm marker library is loaded on first use and only when FKV_ROCTX=1, so
// the transfer library has no link-time dependency on it.
#include "fkv_internal.h"

#include <dlfcn.h>

#include <cstdarg>
#include <cstdlib>
#include <mutex>

namespace {
struct Markers {
  int (*push)(const char *) = nullptr;
  int (*pop)() = nullptr;
};
const Markers &markers() {
  static Markers m;
  static std::once_flag once;
  std::call_once(once, [] {
    const char *on = std::getenv("FKV_ROCTX");
    if (!on || *on != '1')
      return;
    // the library rocprofv3 listens to first, the older stand-alone one second
    for (const char *name : {"librocprofiler-sdk-roctx.so", "librocprofiler-sdk-roctx.so.1",
                             "libroctx64.so", "libroctx64.so.4"}) {
      void *h = dlopen(name, RTLD_NOW | RTLD_GLOBAL);
      if (!h)
        continue;
      auto push = reinterpret_cast<int (*)(const char *)>(dlsym(h, "roctxRangePushA"));
      auto pop = reinterpret_cast<int (*)()>(dlsym(h, "roctxRangePop"));
      if (push && pop) {
        m.push = push;
        m.pop = pop;
        return;
      }
    }
    fprintf(stderr, "[fkv] FKV_ROCTX=1 but no ROCm marker library could be loaded\n");
  });
  return m;
}
} // namespace

namespace fkv {
Range::Range(const char *fmt, ...) {
  const Markers &m = markers();
  if (!m.push)
    return;
  char label[160];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(label, sizeof(label), fmt, ap);
  va_end(ap);
  m.push(label);
  pushed_ = true;
}
Range::~Range() {
  if (pushed_)
    markers().pop();
}
} // namespace fkv

extern "C" {
int fkv_range_push(const char *label) try {
  const Markers &m = markers();
  if (!m.push || !label)
    return 0;
  m.push(label);
  return 1;
} catch (...) {
  return fkv::caught(__func__);
}
int fkv_range_pop(void) try {
  const Markers &m = markers();
  if (!m.pop)
    return 0;
  m.pop();
  return 1;
} catch (...) {
  return fkv::caught(__func__);
}
}
