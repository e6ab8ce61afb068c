// Host-side helpers shared by the C-ABI translation units: thread-local error text,
// argument checks, device facts.  Replaces checkCuda / check_compatability of the
// reference (cpp/souffle_utils/cuda_utils.h:10-19,86-98): nothing here prints or aborts.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include "../../include/souffle_hip.h"

namespace souffle {

char *error_buffer();                       // thread-local, 512 bytes
int fail(int code, const char *fmt, ...);   // formats into error_buffer(), returns code

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

struct DeviceFacts {
  int ok;            // 0 until queried successfully
  int num_cus, lds_per_cu, cooperative;
  char arch[64];
};
// Cached per process for the current device; returns a negative status on failure.
int device_facts(DeviceFacts *out);

// 1: the Swin block pair runs four workgroups per window (souffle_set_swin_split / SOUFFLE_SWIN_SPLIT).
int swin_split_mode();

// 1: every hand-over between workgroups also runs the release / acquire fences of the memory model
// (souffle_set_strict_fences / SOUFFLE_STRICT_FENCES).
int strict_fences_mode();

// Process-wide stage-trace buffer set by souffle_set_stage_trace (NULL = tracing off).
void stage_trace(unsigned long long **buf, int *max_barriers, int nblk);

// Launch of a persistent kernel whose workgroups synchronise through the grid barrier: all
// `grid` workgroups must be resident at once.  Checks that with the occupancy query (cached
// per function), then launches plainly or, when souffle_set_cooperative_launch(1) was called,
// cooperatively.
int launch_persistent(const void *fn, int grid, int block, void **args, size_t lds_bytes, hipStream_t st);

inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

#define SOUFFLE_HIP_TRY(expr)                                                            \
  do {                                                                                   \
    hipError_t e_ = (expr);                                                              \
    if (e_ != hipSuccess)                                                                \
      return ::souffle::fail(SOUFFLE_ERR_LAUNCH, "%s failed: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

}  // namespace souffle
