// Shared host-side helpers of libtsmi.so: error reporting and launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/tsmi.h"

namespace tsmi {

// Stores a formatted message for tsmi_last_error() and returns `code`.
int fail(int code, const char *fmt, ...);
void clear_error();

inline int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TSMI_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return TSMI_OK;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// 1-D grids are capped at 2^31-1 blocks; every kernel here sizes its grid from
// an int64 element count through this helper and refuses anything larger.
inline bool grid_fits(int64_t blocks) { return blocks >= 0 && blocks < (int64_t(1) << 31); }

// Weight-gradient pair lists: pairs per reduction step (each offset's list is padded to a
// multiple of it) and the largest kernel volume the kernels keep a segment table for.
constexpr int kWgradPairStep = 32;
constexpr int kWgradMaxKvol = 511;

}  // namespace tsmi

#define TSMI_REQUIRE(cond, ...)                                            \
  do {                                                                     \
    if (!(cond)) return tsmi::fail(TSMI_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)
