// Batch normalisation of a row-major feature matrix [N, C] in training mode for gfx950:
// per-channel statistics over the N rows, the normalised output, and the backward.
//
// Every pass is HBM-bound: a thread owns one 16-byte piece of a row (8 half / bf16 or 4 float
// channels), neighbouring lanes read neighbouring addresses, and column sums are kept in fp32
// registers while a block strides over its rows.  Blocks leave their partial sums in a
// [blocks, 2, C] fp32 array that one small launch adds up in a fixed order: no atomics, the
// same bits on every run.  The variance comes from sums of (x - x[0, c]) and its square: the
// shift by the column's first row keeps E[d^2] - E[d]^2 away from cancellation when a column's
// mean is large next to its spread.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace tsmi {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxBlocks = 256;  // partial sums per column

template <typename T>
struct Vec;
template <>
struct Vec<float> {
  static constexpr int V = 4;
};
template <>
struct Vec<_Float16> {
  static constexpr int V = 8;
};
template <>
struct Vec<__bf16> {
  static constexpr int V = 8;
};

template <typename T, int V>
struct alignas(sizeof(T) * V) Pack {
  T v[V];
};

template <typename T, int V>
__device__ __forceinline__ void load_piece(const T *p, float *out) {
  const Pack<T, V> q = *(const Pack<T, V> *)p;
#pragma unroll
  for (int e = 0; e < V; ++e) out[e] = (float)q.v[e];
}

template <typename T, int V>
__device__ __forceinline__ void store_piece(T *p, const float *in) {
  Pack<T, V> q;
#pragma unroll
  for (int e = 0; e < V; ++e) q.v[e] = (T)in[e];
  *(Pack<T, V> *)p = q;
}

// Parameters and running statistics come in the module's own type.
__device__ __forceinline__ float load_param(const void *p, int i, int code, float missing) {
  if (!p) return missing;
  if (code == TSMI_F32) return ((const float *)p)[i];
  if (code == TSMI_F16) return (float)((const _Float16 *)p)[i];
  return (float)((const __bf16 *)p)[i];
}

__device__ __forceinline__ void store_param(void *p, int i, int code, float v) {
  if (code == TSMI_F32)
    ((float *)p)[i] = v;
  else if (code == TSMI_F16)
    ((_Float16 *)p)[i] = (_Float16)v;
  else
    ((__bf16 *)p)[i] = (__bf16)v;
}

// Column sums of one block's rows.  Forward: sum (x - k) and sum (x - k)^2 with k = x[0, c].
// Backward: sum dy and sum dy * xhat, xhat = (x - mean) * invstd.
// Threads: piece g = tid % (C / V) of row tid / (C / V); 256 / (C / V) rows per sweep.
template <typename T, int V, bool kBackward>
__global__ __launch_bounds__(kBlock) void bn_reduce_kernel(const T *x, const T *dy, const float *mean,
                                                           const float *invstd, int64_t n, int c,
                                                           float *partial) {
  extern __shared__ float red[];  // [rows per sweep][2 * C]
  const int cg = c / V;
  const int rows = kBlock / cg;
  const int r = threadIdx.x / cg, g = threadIdx.x - r * cg;
  const bool active = r < rows;
  float a1[V], a2[V], k[V], inv[V];
#pragma unroll
  for (int e = 0; e < V; ++e) a1[e] = a2[e] = k[e] = inv[e] = 0.f;
  if (active) {
    if (kBackward) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        k[e] = mean[g * V + e];
        inv[e] = invstd[g * V + e];
      }
    } else {
      load_piece<T, V>(x + g * V, k);
    }
    for (int64_t row = (int64_t)blockIdx.x * rows + r; row < n; row += (int64_t)gridDim.x * rows) {
      float xv[V];
      load_piece<T, V>(x + row * c + g * V, xv);
      if (kBackward) {
        float dv[V];
        load_piece<T, V>(dy + row * c + g * V, dv);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          a1[e] += dv[e];
          a2[e] += dv[e] * ((xv[e] - k[e]) * inv[e]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const float d = xv[e] - k[e];
          a1[e] += d;
          a2[e] += d * d;
        }
      }
    }
#pragma unroll
    for (int e = 0; e < V; ++e) {
      red[r * 2 * c + g * V + e] = a1[e];
      red[r * 2 * c + c + g * V + e] = a2[e];
    }
  }
  __syncthreads();
  for (int t = threadIdx.x; t < 2 * c; t += kBlock) {
    float s = 0.f;
    for (int q = 0; q < rows; ++q) s += red[q * 2 * c + t];
    partial[(int64_t)blockIdx.x * 2 * c + t] = s;
  }
}

// Adds the blocks' partial sums per column in a fixed order and derives the per-column
// constants of the element-wise pass.  A block of 1024 threads serves 32 columns: 16 slices
// of the partial sums x 2 sums x 32 columns, added up through LDS.
//   forward  (stats != 0): out[0:c] = mean, out[c:2c] = 1/sqrt(var + eps), and the output is
//            y = (x - mean) * out[2c:3c] + out[3c:4c]; running statistics updated.
//   backward: out[0:c] = sum dy, out[c:2c] = sum dy * xhat, and the input gradient is
//            dx = dy * out[2c:3c] + (x - mean) * out[3c:4c] + out[4c:5c].
constexpr int kFinalizeCols = 32;
constexpr int kFinalizeSlices = 16;

template <typename T>
__global__ __launch_bounds__(1024) void bn_finalize_kernel(
    const float *partial, int blocks, const T *x, int64_t n, int c, int stats, float eps, float momentum,
    const void *weight, const void *bias, void *running_mean, void *running_var, int param_code,
    const float *mean_in, const float *invstd_in, float *out, void *out_param) {
  __shared__ float red[kFinalizeSlices][2][kFinalizeCols];
  const int lc = threadIdx.x % kFinalizeCols;
  const int which = (threadIdx.x / kFinalizeCols) % 2;
  const int slice = threadIdx.x / (2 * kFinalizeCols);
  const int col = blockIdx.x * kFinalizeCols + lc;
  float acc = 0.f;
  if (col < c)
    for (int b = slice; b < blocks; b += kFinalizeSlices) acc += partial[(int64_t)b * 2 * c + which * c + col];
  red[slice][which][lc] = acc;
  __syncthreads();
  if (threadIdx.x >= kFinalizeCols || col >= c) return;
  float t1 = 0.f, t2 = 0.f;
#pragma unroll
  for (int q = 0; q < kFinalizeSlices; ++q) {
    t1 += red[q][0][lc];
    t2 += red[q][1][lc];
  }
  const float inv_n = 1.f / (float)n;
  const float w = load_param(weight, col, param_code, 1.f);
  if (!stats) {
    const float mean = mean_in[col], invstd = invstd_in[col];
    const float s = w * invstd;
    const float bx = -s * t2 * invstd * inv_n;
    out[col] = t1;
    out[c + col] = t2;
    out[2 * c + col] = s;
    out[3 * c + col] = bx;
    out[4 * c + col] = -s * t1 * inv_n;
    if (out_param) {  // the two gradients once more, in the parameters' type
      store_param(out_param, col, param_code, t1);
      store_param(out_param, c + col, param_code, t2);
    }
    return;
  }
  const float shift = t1 * inv_n;
  const float mean = (float)x[col] + shift;
  const float var = fmaxf(t2 * inv_n - shift * shift, 0.f);  // biased, as used for normalising
  const float invstd = rsqrtf(var + eps);
  out[col] = mean;
  out[c + col] = invstd;
  out[2 * c + col] = invstd * w;
  out[3 * c + col] = load_param(bias, col, param_code, 0.f);
  if (running_mean) {
    const float rm = load_param(running_mean, col, param_code, 0.f);
    store_param(running_mean, col, param_code, (1.f - momentum) * rm + momentum * mean);
  }
  if (running_var) {
    const float unbiased = n > 1 ? var * ((float)n / (float)(n - 1)) : var;
    const float rv = load_param(running_var, col, param_code, 1.f);
    store_param(running_var, col, param_code, (1.f - momentum) * rv + momentum * unbiased);
  }
}

// Per column: out = (a - cm) * ca + cc, or with two inputs out = a * ca + (b - cm) * cb + cc
// (the mean is subtracted before scaling, as torch does: x * scale + (bias - mean * scale) would
// lose the small difference of two large terms when a column's mean is large).  Thread layout as
// in the reduction; the column constants are read once per thread and serve kSweeps rows.
constexpr int kSweeps = 8;

template <typename T, int V, bool kTwo>
__global__ __launch_bounds__(kBlock) void bn_apply_kernel(const T *a, const T *b, int64_t n, int c,
                                                          const float *cm, const float *ca, const float *cb,
                                                          const float *cc, T *out) {
  const int cg = c / V;
  const int rows = kBlock / cg;
  const int r = threadIdx.x / cg, g = threadIdx.x - r * cg;
  if (r >= rows) return;
  float km[V], ka[V], kb[V], kc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) {
    km[e] = cm[g * V + e];
    ka[e] = ca[g * V + e];
    kb[e] = kTwo ? cb[g * V + e] : 0.f;
    kc[e] = cc[g * V + e];
  }
  const int64_t row0 = (int64_t)blockIdx.x * rows * kSweeps + r;
#pragma unroll
  for (int sweep = 0; sweep < kSweeps; ++sweep) {
    const int64_t row = row0 + (int64_t)sweep * rows;
    if (row >= n) break;
    float av[V], bv[V];
    load_piece<T, V>(a + row * c + g * V, av);
    if (kTwo) load_piece<T, V>(b + row * c + g * V, bv);
#pragma unroll
    for (int e = 0; e < V; ++e)
      av[e] = kTwo ? av[e] * ka[e] + (bv[e] - km[e]) * kb[e] + kc[e] : (av[e] - km[e]) * ka[e] + kc[e];
    store_piece<T, V>(out + row * c + g * V, av);
  }
}

int check_shape(const char *what, int64_t n, int c, int dtype, int param_dtype, int *v) {
  TSMI_REQUIRE(dtype == TSMI_F32 || dtype == TSMI_F16 || dtype == TSMI_BF16, "%s: bad dtype %d", what, dtype);
  TSMI_REQUIRE(param_dtype == TSMI_F32 || param_dtype == TSMI_F16 || param_dtype == TSMI_BF16,
               "%s: bad parameter dtype %d", what, param_dtype);
  *v = dtype == TSMI_F32 ? 4 : 8;
  TSMI_REQUIRE(n >= 1, "%s: needs at least one row", what);
  TSMI_REQUIRE(c >= *v && c % *v == 0 && c / *v <= kBlock,
               "%s: the channel count must be a multiple of %d and at most %d (got %d)", what, *v,
               *v * kBlock, c);
  TSMI_REQUIRE(grid_fits(ceil_div(n * (c / *v), kBlock)), "%s: problem too large for one launch", what);
  return TSMI_OK;
}

int reduce_blocks(int64_t n, int c, int v) {
  const int rows = kBlock / (c / v);
  const int64_t b = ceil_div(n, rows);
  return (int)(b < kMaxBlocks ? b : kMaxBlocks);
}

template <typename T>
int forward_t(hipStream_t s, const T *x, int64_t n, int c, const void *weight, const void *bias,
              int param_dtype, void *running_mean, void *running_var, float momentum, float eps,
              float *partial, float *stats, T *y) {
  constexpr int V = Vec<T>::V;
  const int blocks = reduce_blocks(n, c, V);
  const int rows = kBlock / (c / V);
  const size_t lds = (size_t)rows * 2 * c * sizeof(float);
  hipLaunchKernelGGL((bn_reduce_kernel<T, V, false>), dim3(blocks), dim3(kBlock), lds, s, x, (const T *)nullptr,
                     (const float *)nullptr, (const float *)nullptr, n, c, partial);
  hipLaunchKernelGGL((bn_finalize_kernel<T>), dim3((unsigned)ceil_div(c, kFinalizeCols)), dim3(1024), 0, s,
                     (const float *)partial, blocks, x, n, c, 1, eps, momentum, weight, bias, running_mean,
                     running_var, param_dtype, (const float *)nullptr, (const float *)nullptr, stats,
                     (void *)nullptr);
  hipLaunchKernelGGL((bn_apply_kernel<T, V, false>), dim3((unsigned)ceil_div(n, (int64_t)rows * kSweeps)),
                     dim3(kBlock), 0, s, x, (const T *)nullptr, n, c, (const float *)stats,
                     (const float *)(stats + 2 * c), (const float *)nullptr, (const float *)(stats + 3 * c), y);
  return check_launch("tsmi_bn_forward_train");
}

template <typename T>
int backward_t(hipStream_t s, const T *dy, const T *x, int64_t n, int c, const void *weight, int param_dtype,
               const float *mean, const float *invstd, float *partial, float *sums, void *grads, T *dx) {
  constexpr int V = Vec<T>::V;
  const int blocks = reduce_blocks(n, c, V);
  const int rows = kBlock / (c / V);
  const size_t lds = (size_t)rows * 2 * c * sizeof(float);
  hipLaunchKernelGGL((bn_reduce_kernel<T, V, true>), dim3(blocks), dim3(kBlock), lds, s, x, dy, mean, invstd, n,
                     c, partial);
  hipLaunchKernelGGL((bn_finalize_kernel<T>), dim3((unsigned)ceil_div(c, kFinalizeCols)), dim3(1024), 0, s,
                     (const float *)partial, blocks, x, n, c, 0, 0.f, 0.f, weight, (const void *)nullptr,
                     (void *)nullptr, (void *)nullptr, param_dtype, mean, invstd, sums, grads);
  hipLaunchKernelGGL((bn_apply_kernel<T, V, true>), dim3((unsigned)ceil_div(n, (int64_t)rows * kSweeps)),
                     dim3(kBlock), 0, s, dy, x, n, c, mean, (const float *)(sums + 2 * c),
                     (const float *)(sums + 3 * c), (const float *)(sums + 4 * c), dx);
  return check_launch("tsmi_bn_backward");
}

}  // namespace
}  // namespace tsmi

using namespace tsmi;

extern "C" int64_t tsmi_bn_partial_elems(int c) { return (int64_t)kMaxBlocks * 2 * (c > 0 ? c : 0); }

extern "C" int tsmi_bn_forward_train(tsmi_stream_t s, const void *x, int64_t n, int c, int dtype,
                                     const void *weight, const void *bias, int param_dtype,
                                     void *running_mean, void *running_var, float momentum, float eps,
                                     float *partial, float *stats, void *y) {
  int v;
  if (int e = check_shape("bn_forward_train", n, c, dtype, param_dtype, &v)) return e;
  TSMI_REQUIRE(x && y && partial && stats, "bn_forward_train: null pointer");
  TSMI_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0, "bn_forward_train: x and y must be 16-byte aligned");
  hipStream_t st = (hipStream_t)s;
  if (dtype == TSMI_F32)
    return forward_t<float>(st, (const float *)x, n, c, weight, bias, param_dtype, running_mean, running_var,
                            momentum, eps, partial, stats, (float *)y);
  if (dtype == TSMI_F16)
    return forward_t<_Float16>(st, (const _Float16 *)x, n, c, weight, bias, param_dtype, running_mean,
                               running_var, momentum, eps, partial, stats, (_Float16 *)y);
  return forward_t<__bf16>(st, (const __bf16 *)x, n, c, weight, bias, param_dtype, running_mean, running_var,
                           momentum, eps, partial, stats, (__bf16 *)y);
}

extern "C" int tsmi_bn_backward(tsmi_stream_t s, const void *dy, const void *x, int64_t n, int c, int dtype,
                                const void *weight, int param_dtype, const float *mean,
                                const float *invstd, float *partial, float *sums, void *grads,
                                void *dx) {
  int v;
  if (int e = check_shape("bn_backward", n, c, dtype, param_dtype, &v)) return e;
  TSMI_REQUIRE(dy && x && dx && partial && mean && invstd && sums, "bn_backward: null pointer");
  TSMI_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)dy % 16 == 0 && (uintptr_t)dx % 16 == 0,
               "bn_backward: dy, x and dx must be 16-byte aligned");
  hipStream_t st = (hipStream_t)s;
  if (dtype == TSMI_F32)
    return backward_t<float>(st, (const float *)dy, (const float *)x, n, c, weight, param_dtype, mean, invstd,
                             partial, sums, grads, (float *)dx);
  if (dtype == TSMI_F16)
    return backward_t<_Float16>(st, (const _Float16 *)dy, (const _Float16 *)x, n, c, weight, param_dtype, mean,
                                invstd, partial, sums, grads, (_Float16 *)dx);
  return backward_t<__bf16>(st, (const __bf16 *)dy, (const __bf16 *)x, n, c, weight, param_dtype, mean, invstd,
                            partial, sums, grads, (__bf16 *)dx);
}
