// Device-wide radix sorts used by kernel-map construction (output-coordinate
// ordering and the row permutation of the sorted implicit-GEMM map).  The sort
// itself is rocPRIM's; scratch comes from the caller.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>
#include <rocprim/iterator/transform_iterator.hpp>

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

// ---------------------------------------------------------------- grouping by index
// order = the entries of idx with a value in [0, n_groups), sorted by (value, position);
// starts[v] = first position of value v in `order`.  Row sums over the entries of a group
// (voxelize, the gradient of devoxelize) then run without atomics and in a fixed order.

namespace {

struct GroupKey {
  uint32_t n_groups;
  __device__ uint32_t operator()(int32_t v) const {
    return (v < 0 || (uint32_t)v >= n_groups) ? n_groups : (uint32_t)v;  // sentinel sorts last
  }
};

using GroupKeyIter = rocprim::transform_iterator<const int32_t *, GroupKey, uint32_t>;

inline int group_bits(int64_t n_groups) {
  int bits = 1;
  while (bits < 32 && (int64_t(1) << bits) <= n_groups) ++bits;  // values 0..n_groups inclusive
  return bits;
}

__global__ void group_starts_kernel(const uint32_t *sorted, int64_t m, int64_t n_groups,
                                    int32_t *starts) {
  const int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (v > n_groups) return;
  int64_t lo = 0, hi = m;  // first position with sorted[pos] >= v
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if ((int64_t)sorted[mid] < v) lo = mid + 1; else hi = mid;
  }
  starts[v] = (int32_t)lo;
}

inline int64_t align_up(int64_t v) { return (v + kAlign - 1) / kAlign * kAlign; }

}  // namespace

extern "C" int64_t tsmi_group_temp_bytes(int64_t m) {
  if (m < 0) return -1;
  if (m == 0) m = 1;
  size_t need = 0;
  hipError_t e = rocprim::radix_sort_pairs(nullptr, need, GroupKeyIter((const int32_t *)nullptr, GroupKey{1}),
                                           (uint32_t *)nullptr, rocprim::counting_iterator<int32_t>(0),
                                           (int32_t *)nullptr, (size_t)m, 0, 32, (hipStream_t)0);
  if (e != hipSuccess) {
    fail(TSMI_ERR_HIP, "group_temp_bytes: size query failed");
    return -1;
  }
  return align_up(m * 4) + align_up((int64_t)need);
}

extern "C" int tsmi_group_by_index(tsmi_stream_t s, const int32_t *idx, int64_t m, int64_t n_groups,
                                   void *temp, int64_t temp_bytes, int32_t *order, int32_t *starts) {
  TSMI_REQUIRE(m >= 0 && m < (int64_t(1) << 31) && n_groups >= 0 && n_groups < (int64_t(1) << 31),
               "group_by_index: bad sizes");
  TSMI_REQUIRE(starts, "group_by_index: null starts");
  if (m == 0) {
    const int64_t blocks0 = ceil_div(n_groups + 1, 256);
    TSMI_REQUIRE(grid_fits(blocks0), "group_by_index: too many groups");
    hipLaunchKernelGGL(group_starts_kernel, dim3((unsigned)blocks0), dim3(256), 0, (hipStream_t)s,
                       (const uint32_t *)nullptr, (int64_t)0, n_groups, starts);
    return check_launch("tsmi_group_by_index");
  }
  TSMI_REQUIRE(idx && order && temp, "group_by_index: null pointer");
  uint32_t *sorted = (uint32_t *)temp;
  void *sort_temp = (char *)temp + align_up(m * 4);
  const int bits = group_bits(n_groups);
  GroupKeyIter keys(idx, GroupKey{(uint32_t)n_groups});
  size_t need = 0;
  (void)rocprim::radix_sort_pairs(nullptr, need, keys, sorted, rocprim::counting_iterator<int32_t>(0),
                                  order, (size_t)m, 0, bits, (hipStream_t)s);
  TSMI_REQUIRE(align_up(m * 4) + (int64_t)need <= temp_bytes,
               "group_by_index: scratch too small (%lld < %lld)", (long long)temp_bytes,
               (long long)(align_up(m * 4) + (int64_t)need));
  hipError_t e = rocprim::radix_sort_pairs(sort_temp, need, keys, sorted,
                                           rocprim::counting_iterator<int32_t>(0), order, (size_t)m, 0,
                                           bits, (hipStream_t)s);
  if (e != hipSuccess) return fail(TSMI_ERR_HIP, "group_by_index: %s", hipGetErrorString(e));
  const int64_t blocks = ceil_div(n_groups + 1, 256);
  TSMI_REQUIRE(grid_fits(blocks), "group_by_index: too many groups");
  hipLaunchKernelGGL(group_starts_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)s,
                     (const uint32_t *)sorted, m, n_groups, starts);
  return check_launch("tsmi_group_by_index");
}
