#include "moe_common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_err[512] = "";

void moe_set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
}

extern "C" const char *moe_last_error(void) { return g_err; }

int moe_check_hip(hipError_t e, const char *what) {
  if (e == hipSuccess) return MOE_OK;
  moe_set_error("%s: %s", what, hipGetErrorString(e));
  return MOE_EHIP;
}

int moe_check_launch(const char *what) { return moe_check_hip(hipGetLastError(), what); }
