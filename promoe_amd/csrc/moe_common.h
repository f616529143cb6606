// Shared host-side helpers of the library (error string, launch check).
#pragma once
#include <hip/hip_runtime.h>

#include "moe_kernels.h"

void moe_set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int moe_check_launch(const char *what);
int moe_check_hip(hipError_t e, const char *what);
