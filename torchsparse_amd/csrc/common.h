// Shared host-side helpers of libtsmi.so: error reporting and launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
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

// Raises a kernel's dynamic-LDS limit to `bytes`, once per device: the attribute belongs to
// the device's copy of the code object.  `done` is the kernel's bit mask of configured devices.
inline int raise_dynamic_lds(const void *kernel, int bytes, std::atomic<uint64_t> &done,
                             const char *what) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(TSMI_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  const uint64_t bit = uint64_t(1) << (dev & 63);
  if (done.load(std::memory_order_relaxed) & bit) return TSMI_OK;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return fail(TSMI_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  done.fetch_or(bit, std::memory_order_relaxed);
  return TSMI_OK;
}

__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

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
