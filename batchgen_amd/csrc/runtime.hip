// Error reporting and small host utilities of libbgmoe.
#include <stdarg.h>
#include <stdio.h>

#include "bgmoe_common.h"

static thread_local char g_err[512] = "";

void bgmoe_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int bgmoe_check_launch(const char* what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    bgmoe_set_error("%s: %s", what, hipGetErrorString(err));
    return BGMOE_ERR_HIP;
  }
  return BGMOE_OK;
}

extern "C" const char* bgmoe_last_error(void) { return g_err; }
extern "C" int bgmoe_version(void) { return 1; }
