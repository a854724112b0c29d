// Shared host/device helpers for the gfx950 W4A16 library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/w4a16_gfx950.h"

namespace w4a16 {

// Records a printf-style message for w4a16_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define W4A16_CHECK(cond, ...)                                   \
  do {                                                           \
    if (!(cond)) return ::w4a16::fail(W4A16_EINVAL, __VA_ARGS__); \
  } while (0)

#define W4A16_HIP(expr)                                                          \
  do {                                                                           \
    hipError_t e_ = (expr);                                                      \
    if (e_ != hipSuccess)                                                        \
      return ::w4a16::fail(W4A16_EHIP, "%s failed: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Number of compute units of the current device (cached per device).
int num_cus();

}  // namespace w4a16
