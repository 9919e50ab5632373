// Error state of the library: the last failure's message, per host thread.
#include "common.h"

static thread_local char g_error[1024] = "";

extern "C" const char* lev_last_error() { return g_error; }

int lev_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return -1;
}

int lev_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return lev_fail("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

extern "C" int lev_abi_version() { return 1; }
