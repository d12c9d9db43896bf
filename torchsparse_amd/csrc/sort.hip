// Device-wide radix sorts used by kernel-map construction (output-coordinate
// ordering and the row permutation of the sorted implicit-GEMM map).  The sort
// itself is rocPRIM's; scratch comes from the caller.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

#include "common.h"

using namespace tsmi;

namespace {
constexpr int64_t kAlign = 256;
}

extern "C" int64_t tsmi_sort_temp_bytes(int64_t n) {
  if (n < 0) return -1;
  if (n == 0) n = 1;
  size_t a = 0, b = 0;
  hipError_t e1 = rocprim::radix_sort_keys(nullptr, a, (const unsigned long long *)nullptr,
                                           (unsigned long long *)nullptr, (size_t)n, 0, 64,
                                           (hipStream_t)0);
  hipError_t e2 = rocprim::radix_sort_pairs_desc(
      nullptr, b, (const int32_t *)nullptr, (int32_t *)nullptr,
      rocprim::counting_iterator<int32_t>(0), (int32_t *)nullptr, (size_t)n, 0, 32, (hipStream_t)0);
  if (e1 != hipSuccess || e2 != hipSuccess) {
    fail(TSMI_ERR_HIP, "sort_temp_bytes: size query failed");
    return -1;
  }
  int64_t m = (int64_t)(a > b ? a : b);
  return (m + kAlign - 1) / kAlign * kAlign + kAlign;
}

extern "C" int tsmi_sort_keys(tsmi_stream_t s, const int64_t *keys_in, int64_t *keys_out, int64_t n,
                              int end_bit, void *temp, int64_t temp_bytes) {
  TSMI_REQUIRE(n >= 0 && end_bit >= 1 && end_bit <= 64, "sort_keys: bad arguments");
  if (n == 0) return TSMI_OK;
  TSMI_REQUIRE(keys_in && keys_out && temp, "sort_keys: null pointer");
  size_t need = 0;
  (void)rocprim::radix_sort_keys(nullptr, need, (const unsigned long long *)keys_in,
                                 (unsigned long long *)keys_out, (size_t)n, 0, end_bit,
                                 (hipStream_t)s);
  TSMI_REQUIRE((int64_t)need <= temp_bytes, "sort_keys: scratch too small (%lld < %lld)",
               (long long)temp_bytes, (long long)need);
  hipError_t e = rocprim::radix_sort_keys(temp, need, (const unsigned long long *)keys_in,
                                          (unsigned long long *)keys_out, (size_t)n, 0, end_bit,
                                          (hipStream_t)s);
  if (e != hipSuccess) return fail(TSMI_ERR_HIP, "sort_keys: %s", hipGetErrorString(e));
  return check_launch("tsmi_sort_keys");
}

extern "C" int tsmi_argsort_desc(tsmi_stream_t s, const int32_t *keys_in, int32_t *keys_out,
                                 int32_t *idx_out, int rows, int64_t n, void *temp,
                                 int64_t temp_bytes) {
  TSMI_REQUIRE(rows >= 1 && n >= 0 && n < (int64_t(1) << 31), "argsort_desc: bad sizes");
  if (n == 0) return TSMI_OK;
  TSMI_REQUIRE(keys_in && keys_out && idx_out && temp, "argsort_desc: null pointer");
  size_t need = 0;
  (void)rocprim::radix_sort_pairs_desc(nullptr, need, keys_in, keys_out,
                                       rocprim::counting_iterator<int32_t>(0), idx_out, (size_t)n,
                                       0, 32, (hipStream_t)s);
  TSMI_REQUIRE((int64_t)need <= temp_bytes, "argsort_desc: scratch too small (%lld < %lld)",
               (long long)temp_bytes, (long long)need);
  for (int r = 0; r < rows; ++r) {
    hipError_t e = rocprim::radix_sort_pairs_desc(
        temp, need, keys_in + (int64_t)r * n, keys_out + (int64_t)r * n,
        rocprim::counting_iterator<int32_t>(0), idx_out + (int64_t)r * n, (size_t)n, 0, 32,
        (hipStream_t)s);
    if (e != hipSuccess) return fail(TSMI_ERR_HIP, "argsort_desc: %s", hipGetErrorString(e));
  }
  return check_launch("tsmi_argsort_desc");
}
