// Error bookkeeping shared by every entry point of libhqekv.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace hq {

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return HQEKV_OK;
  snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
  return (int)e;
}

}  // namespace hq

extern "C" int hqekv_version(void) { return 1; }
extern "C" const char *hqekv_last_error(void) { return hq::g_err; }
