// Shared host-side plumbing of libdopplerhip: error reporting, the single stream every op
// enqueues on, and launch helpers.  gfx950 only.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/doppler_hip.h"

namespace dh {

constexpr int kQK = 256;           // weights per Q4_K super-block
constexpr int kBlockBytes = 144;   // bytes per super-block
constexpr int kWave = 64;

// Records a message for dh_last_error() and returns the code to hand back to the caller.
int fail(int code, const char* fmt, ...);
hipStream_t stream();
bool ready();
int num_cus();

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace dh

#define DH_REQUIRE_INIT(op)                                                     \
  do {                                                                          \
    if (!dh::ready()) return dh::fail(1, "[%s] dh_init has not been called", op); \
  } while (0)

#define DH_CHECK_HIP(op, expr)                                                       \
  do {                                                                               \
    hipError_t e_ = (expr);                                                          \
    if (e_ != hipSuccess)                                                            \
      return dh::fail(2, "[%s] %s failed: %s", op, #expr, hipGetErrorString(e_));    \
  } while (0)

// After a kernel launch: surfaces launch-configuration errors at the call site.
#define DH_CHECK_LAUNCH(op) DH_CHECK_HIP(op, hipGetLastError())
