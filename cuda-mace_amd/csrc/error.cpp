// Thread-local error message and ABI version of the C library.
#include <cstdarg>
#include <cstdio>

#include "cuda_mace_hip.h"

namespace cm {
namespace {
thread_local char g_error[512] = "";
}

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace cm

extern "C" int cm_abi_version(void) { return 8; }
extern "C" const char *cm_last_error(void) { return cm::g_error; }
