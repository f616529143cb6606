// Shared host-side helpers of the library (error string, launch check).
#pragma once
#include <hip/hip_runtime.h>

#include "moe_kernels.h"

void moe_set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int moe_check_launch(const char *what);
int moe_check_hip(hipError_t e, const char *what);

// Optional per-kernel timing with HIP events on the launch stream (moe_kernel_timing*).
enum MoeKernelId { MOE_K_GATE = 0, MOE_K_TOPK, MOE_K_DISPATCH, MOE_K_W13, MOE_K_W2, MOE_K_COMBINE,
                   MOE_K_PREFILL_W13, MOE_K_PREFILL_W2, MOE_K_COUNT };
void moe_ktimer_begin(int kid, hipStream_t s);
void moe_ktimer_end(int kid, hipStream_t s);

// A kernel met a selected expert whose slot-table entry is 0: it skips the unit and raises the caller's
// error word.  A system-scope store (every raiser writes the same value), so the word may live in device
// memory or in pinned host memory that the host polls without a copy.
static __device__ __forceinline__ void moe_raise_err(int *err) {
  __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
