// Per-element-type operation table of the convolution kernels.  Each element
// type is compiled in its own translation unit (conv_igemm_{f16,bf16,f32}.hip)
// and exposes one of these tables; conv_api.cpp dispatches on the dtype code.
#pragma once

#include <algorithm>
#include <cstdlib>

#include "common.h"

namespace tsmi {

// Where a convolution's result rows go when not into a dense [n_out, cout] tensor: row pitch of y
// in elements (0: cout), and an optional second destination that receives the same values (a
// column slice of a wider buffer, say).  Honoured by the launches that finish their rows
// themselves (igemm with its in-kernel epilogue, segment_sum).
struct OutPlace {
  int64_t ldy;
  void *y2;
  int64_t ldy2;
};

struct ConvOps {
  int step;  // reduction elements per MFMA step (Cin is padded to a multiple)
  int (*pack)(hipStream_t s, const void *w, void *wp, int kvol, int cin, int cout);
  // floats of scratch igemm wants for this problem (0 = none)
  int64_t (*workspace)(int64_t n_tile_rows, int64_t n_out, int kvol, int split, int cin, int cout,
                       int sorted);
  // row_out == nullptr: plain implicit GEMM over `map`; otherwise sorted mode.  order64 / order128
  // (sorted mode, one split, n_tile_rows a multiple of 128): the 64-row / 128-row tiles of the map
  // listed heaviest first (tsmi_map_group_rows); the tiles start in that order where the plan allows.
  int (*igemm)(hipStream_t s, const void *x, const void *wp, const int32_t *map,
               int64_t n_map_rows, int64_t n_tile_rows, int64_t n_out, int kvol, int cin, int cout,
               const void *bias, const void *residual, int relu, void *y, const int32_t *row_out,
               int64_t row_out_stride, int split, float *partial, int64_t partial_elems,
               int32_t *counters, int64_t n_counters, const int32_t *order64, const int32_t *order128,
               const OutPlace *place);
  // out[nbaddrs[k] + p, :] = X[rows[nbaddrs[k] + p], :] W[k] over 128-padded pair lists
  int (*pairs)(hipStream_t s, const void *x, const void *wp, const int32_t *rows,
               const int32_t *nbaddrs, const int32_t *qnbaddrs, int64_t qnnz, int kvol, int cin,
               int cout, void *out);
  int (*sum_partials)(hipStream_t s, const float *partial, int split, int64_t n_out, int cout,
                      const void *bias, const void *residual, int relu, void *y);
  int (*scatter)(hipStream_t s, const void *pbuf, const int32_t *nbaddrs, const int32_t *mask,
                 int64_t n_out, int kvol, int cout, int center_k, const void *bias,
                 const void *residual, int relu, void *y);
  int (*gather)(hipStream_t s, const void *x, const int32_t *pairs, int64_t nnz, int cin, int col,
                void *buffer);
  // dW[k] = sum over input rows i of X[i]^T dY[map_bwd[i,k]]
  int64_t (*wgrad_workspace)(int64_t n_in, int kvol, int cin, int cout);
  int (*wgrad)(hipStream_t s, const void *x, const void *dy, const int32_t *map_bwd, int64_t n_in,
               int kvol, int cin, int cout, float *partial, int64_t partial_elems, void *dw);
  // the same sums over padded pair lists (tsmi_wgrad_pairs_build); pairs[:, x_col] indexes x
  int64_t (*wgrad_pairs_workspace)(int64_t pair_cap, int kvol, int cin, int cout);
  int (*wgrad_pairs)(hipStream_t s, const void *x, const void *dy, const int32_t *pairs,
                     const int32_t *seg_steps, int64_t pair_cap, int x_col, int kvol, int cin,
                     int cout, float *partial, int64_t partial_elems, void *dw);
  // 1 when `segments` has a variant for the shape
  int (*segments_supported)(int kvol, int cin, int cout);
  // products[k * seg_rows + j, :] = X[in_rows[k * seg_rows + j], :] W[k] for j < counts[k]
  int (*segments)(hipStream_t s, const void *x, const void *wp, const int32_t *in_rows,
                  const int32_t *counts, int64_t seg_rows, int kvol, int cin, int cout,
                  void *products);
  // y[o, :] = sum over k of products[k * seg_rows + pos[k * n_out + o], :] where pos >= 0
  int (*segment_sum)(hipStream_t s, const void *products, const int32_t *pos, int64_t n_out, int kvol,
                     int64_t seg_rows, int cout, const void *bias, const void *residual, int relu,
                     void *y, const OutPlace *place);
};

const ConvOps &conv_ops_f16();
const ConvOps &conv_ops_bf16();
const ConvOps &conv_ops_f32();

inline int pad_to(int v, int m) { return (v + m - 1) / m * m; }

}  // namespace tsmi
