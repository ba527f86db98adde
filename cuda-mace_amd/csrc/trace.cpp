// Optional ROCTx ranges around the ops, the counterpart of the NVTX ranges the reference opens around every autograd
// forward and backward (include/utils.h:9-21, e.g. src/linear.cpp:15, :24).  Off unless the environment variable
// CUDA_MACE_TRACE is set to a non-zero value when the first range is requested; the marker library is then looked up
// at run time, so the kernel library has no link-time dependency on a profiler.
#include <dlfcn.h>

#include <cstdlib>
#include <mutex>

#include "cuda_mace_hip.h"

namespace {

using push_fn = int (*)(const char *);
using pop_fn = int (*)();

struct Markers {
  push_fn push = nullptr;
  pop_fn pop = nullptr;
};

const Markers &markers() {
  static Markers m;
  static std::once_flag once;
  std::call_once(once, [] {
    const char *env = std::getenv("CUDA_MACE_TRACE");
    if (env == nullptr || env[0] == '\0' || env[0] == '0') return;
    // the marker library of the current profiler first, the older tracer's second
    for (const char *name : {"librocprofiler-sdk-roctx.so", "librocprofiler-sdk-roctx.so.1", "libroctx64.so", "libroctx64.so.4"}) {
      void *lib = dlopen(name, RTLD_NOW | RTLD_GLOBAL);
      if (lib == nullptr) continue;
      auto push = reinterpret_cast<push_fn>(dlsym(lib, "roctxRangePushA"));
      auto pop = reinterpret_cast<pop_fn>(dlsym(lib, "roctxRangePop"));
      if (push != nullptr && pop != nullptr) {
        m.push = push;
        m.pop = pop;
        return;
      }
    }
  });
  return m;
}

}  // namespace

extern "C" int cm_trace_enabled(void) { return markers().push != nullptr; }

extern "C" void cm_trace_push(const char *name) {
  const Markers &m = markers();
  if (m.push != nullptr) m.push(name != nullptr ? name : "cuda_mace");
}

extern "C" void cm_trace_pop(void) {
  const Markers &m = markers();
  if (m.pop != nullptr) m.pop();
}
