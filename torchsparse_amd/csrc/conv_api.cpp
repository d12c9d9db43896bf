// C entry points of the convolution dataflows: argument checks and dispatch on
// the element type.  The kernels live in conv_igemm.inc.
#include "conv_ops.h"

using namespace tsmi;

namespace {

const ConvOps *ops_for(int dtype) {
  switch (dtype) {
    case TSMI_F32: return &conv_ops_f32();
    case TSMI_F16: return &conv_ops_f16();
    case TSMI_BF16: return &conv_ops_bf16();
    default: return nullptr;
  }
}

int check_shapes(const char *who, const ConvOps *ops, int kvol, int cin, int cout) {
  if (!ops) return fail(TSMI_ERR_INVALID_ARGUMENT, "%s: unsupported dtype", who);
  TSMI_REQUIRE(kvol >= 1 && cin >= 1 && cout >= 1, "%s: bad kernel shape [%d,%d,%d]", who, kvol,
               cin, cout);
  return TSMI_OK;
}

bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

extern "C" int64_t tsmi_packed_weight_elems(int kvol, int cin, int cout) {
  if (kvol < 1 || cin < 1 || cout < 1) return -1;
  // sized for the coarsest reduction step (32 elements) so one size fits every dtype
  return (int64_t)kvol * pad_to(cout, 16) * pad_to(cin, 32);
}

extern "C" int tsmi_pack_weights(tsmi_stream_t s, const void *w, void *w_packed, int kvol, int cin,
                                 int cout, int dtype) {
  const ConvOps *ops = ops_for(dtype);
  if (int e = check_shapes("pack_weights", ops, kvol, cin, cout)) return e;
  TSMI_REQUIRE(w && w_packed, "pack_weights: null pointer");
  return ops->pack((hipStream_t)s, w, w_packed, kvol, cin, cout);
}

extern "C" int64_t tsmi_conv_workspace_elems(int64_t n_tile_rows, int64_t n_out, int kvol,
                                             int split, int cin, int cout, int dtype, int sorted) {
  const ConvOps *ops = ops_for(dtype);
  if (!ops || n_tile_rows < 0 || n_out < 0 || kvol < 1 || split < 1 || cin < 1 || cout < 1) return -1;
  return ops->workspace(n_tile_rows, n_out, kvol, split, cin, cout, sorted);
}

// A placed result (tsmi.h: the *_packed entry points): pitches in whole 16-byte pieces that hold
// a row, the second destination aligned like the first.
static int check_place(const char *who, const OutPlace *place, int cout) {
  if (!place) return TSMI_OK;
  TSMI_REQUIRE(place->ldy == 0 || (place->ldy >= cout && place->ldy % 8 == 0),
               "%s: the row pitch of y (%lld) must be a multiple of 8 elements that holds %d channels", who,
               (long long)place->ldy, cout);
  TSMI_REQUIRE(!place->y2 || (aligned16(place->y2) && place->ldy2 >= cout && place->ldy2 % 8 == 0),
               "%s: the second destination must be 16-byte aligned, its row pitch (%lld) a multiple of 8 "
               "elements that holds %d channels", who, (long long)place->ldy2, cout);
  return TSMI_OK;
}

static int implicit_gemm(tsmi_stream_t s, const void *x, const void *w_packed, const int32_t *map,
                         int64_t n_map_rows, int64_t n_out, int kvol, int cin, int cout, int dtype,
                         const void *bias, const void *residual, int relu, float *workspace,
                         int64_t workspace_elems, int32_t *tile_counters, int64_t n_tile_counters, void *y,
                         const OutPlace *place) {
  const ConvOps *ops = ops_for(dtype);
  if (int e = check_shapes("conv_implicit_gemm", ops, kvol, cin, cout)) return e;
  if (int e = check_place("conv_implicit_gemm", place, cout)) return e;
  TSMI_REQUIRE(n_out >= 0 && n_map_rows >= n_out, "conv_implicit_gemm: map has %lld rows, need %lld",
               (long long)n_map_rows, (long long)n_out);
  if (n_out == 0) return TSMI_OK;
  TSMI_REQUIRE(x && w_packed && map && y, "conv_implicit_gemm: null pointer");
  TSMI_REQUIRE(aligned16(x) && aligned16(w_packed) && aligned16(y),
               "conv_implicit_gemm: x, w_packed and y must be 16-byte aligned");
  return ops->igemm((hipStream_t)s, x, w_packed, map, n_map_rows, n_out, n_out, kvol, cin, cout,
                    bias, residual, relu, y, nullptr, 0, 1, workspace, workspace_elems,
                    tile_counters, tile_counters ? n_tile_counters : 0, nullptr, nullptr, place);
}

extern "C" int tsmi_conv_implicit_gemm(tsmi_stream_t s, const void *x, const void *w_packed,
                                       const int32_t *map, int64_t n_map_rows, int64_t n_out,
                                       int kvol, int cin, int cout, int dtype, const void *bias,
                                       const void *residual, int relu, float *workspace,
                                       int64_t workspace_elems, int32_t *tile_counters,
                                       int64_t n_tile_counters, void *y) {
  return implicit_gemm(s, x, w_packed, map, n_map_rows, n_out, kvol, cin, cout, dtype, bias, residual, relu,
                       workspace, workspace_elems, tile_counters, n_tile_counters, y, nullptr);
}

extern "C" int tsmi_conv_implicit_gemm_sorted(tsmi_stream_t s, const void *x, const void *w_packed,
                                              const int32_t *reorder_map,
                                              const int32_t *reduced_mask,
                                              const int32_t *reorder_loc, int64_t n_pad,
                                              int64_t n_out, int kvol, int split, int cin, int cout,
                                              int dtype, const void *bias, const void *residual,
                                              int relu, float *workspace, int64_t workspace_elems,
                                              int32_t *tile_counters, int64_t n_tile_counters,
                                              void *y) {
  (void)reduced_mask;  // tile skipping is derived from the staged map itself
  const ConvOps *ops = ops_for(dtype);
  if (int e = check_shapes("conv_implicit_gemm_sorted", ops, kvol, cin, cout)) return e;
  TSMI_REQUIRE(split >= 1 && split <= kvol, "conv_implicit_gemm_sorted: bad split %d", split);
  TSMI_REQUIRE((int64_t)(split - 1) * ((kvol + split - 1) / split) < kvol,
               "conv_implicit_gemm_sorted: split_mask_num %d leaves an empty split", split);
  TSMI_REQUIRE(n_out >= 0 && n_pad >= n_out, "conv_implicit_gemm_sorted: n_pad < n_out");
  if (n_out == 0) return TSMI_OK;
  TSMI_REQUIRE(x && w_packed && reorder_map && reorder_loc && y,
               "conv_implicit_gemm_sorted: null pointer");
  TSMI_REQUIRE(split == 1 || workspace, "conv_implicit_gemm_sorted: split > 1 needs a workspace");
  TSMI_REQUIRE(aligned16(x) && aligned16(w_packed) && aligned16(y),
               "conv_implicit_gemm_sorted: x, w_packed and y must be 16-byte aligned");
  return ops->igemm((hipStream_t)s, x, w_packed, reorder_map, n_pad, n_pad, n_out, kvol, cin, cout,
                    bias, residual, relu, y, reorder_loc, n_pad, split, workspace, workspace_elems,
                    tile_counters, tile_counters ? n_tile_counters : 0, nullptr, nullptr, nullptr);
}

static int implicit_gemm_grouped(tsmi_stream_t s, const void *x, const void *w_packed,
                                               const int32_t *grouped_map, const int32_t *row_of,
                                               const int32_t *order64, const int32_t *order128,
                                               int64_t n_grouped, int64_t n_out, int kvol, int cin,
                                               int cout, int dtype, const void *bias,
                                               const void *residual, int relu, void *y, const OutPlace *place) {
  const ConvOps *ops = ops_for(dtype);
  if (int e = check_shapes("conv_implicit_gemm_grouped", ops, kvol, cin, cout)) return e;
  if (int e = check_place("conv_implicit_gemm_grouped", place, cout)) return e;
  TSMI_REQUIRE(n_out >= 0 && n_grouped >= n_out && n_grouped % 128 == 0,
               "conv_implicit_gemm_grouped: bad sizes (%lld grouped rows for %lld outputs)",
               (long long)n_grouped, (long long)n_out);
  if (n_out == 0) return TSMI_OK;
  TSMI_REQUIRE(x && w_packed && grouped_map && row_of && order64 && order128 && y,
               "conv_implicit_gemm_grouped: null pointer");
  TSMI_REQUIRE(aligned16(x) && aligned16(w_packed) && aligned16(y),
               "conv_implicit_gemm_grouped: x, w_packed and y must be 16-byte aligned");
  return ops->igemm((hipStream_t)s, x, w_packed, grouped_map, n_grouped, n_grouped, n_out, kvol, cin,
                    cout, bias, residual, relu, y, row_of, n_grouped, 1, nullptr, 0, nullptr, 0, order64,
                    order128, place);
}

extern "C" int tsmi_conv_implicit_gemm_grouped(tsmi_stream_t s, const void *x, const void *w_packed,
                                               const int32_t *grouped_map, const int32_t *row_of,
                                               const int32_t *order64, const int32_t *order128,
                                               int64_t n_grouped, int64_t n_out, int kvol, int cin,
                                               int cout, int dtype, const void *bias,
                                               const void *residual, int relu, void *y) {
  return implicit_gemm_grouped(s, x, w_packed, grouped_map, row_of, order64, order128, n_grouped, n_out, kvol,
                               cin, cout, dtype, bias, residual, relu, y, nullptr);
}

extern "C" int64_t tsmi_conv_wgrad_workspace_elems(int64_t n_in, int kvol, int cin, int cout,
                                                   int dtype) {
  const ConvOps *ops = ops_for(dtype);
  if (!ops || n_in < 0 || kvol < 1 || cin < 1 || cout < 1) return 0;
  return ops->wgrad_workspace(n_in, kvol, cin, cout);
}

extern "C" int tsmi_conv_wgrad(tsmi_stream_t s, const void *x, const void *dy,
                               const int32_t *map_bwd, int64_t n_map_rows, int64_t n_in, int kvol,
                               int cin, int cout, int dtype, float *workspace,
                               int64_t workspace_elems, void *dw) {
  const ConvOps *ops = ops_for(dtype);
  if (int e = check_shapes("conv_wgrad", ops, kvol, cin, cout)) return e;
  TSMI_REQUIRE(n_in >= 0 && n_map_rows >= n_in, "conv_wgrad: map has %lld rows, need %lld",
               (long long)n_map_rows, (long long)n_in);
  TSMI_REQUIRE(dw && workspace, "conv_wgrad: null output or workspace");
  TSMI_REQUIRE(n_in == 0 || (x && dy && map_bwd), "conv_wgrad: null pointer");
  TSMI_REQUIRE(aligned16(x) && aligned16(dy), "conv_wgrad: x and dy must be 16-byte aligned");
  return ops->wgrad((hipStream_t)s, x, dy, map_bwd, n_in, kvol, cin, cout, workspace,
                    workspace_elems, dw);
}

extern "C" int64_t tsmi_conv_wgrad_pairs_workspace_elems(int64_t pair_cap, int kvol, int cin,
                                                         int cout, int dtype) {
  const ConvOps *ops = ops_for(dtype);
  if (!ops || pair_cap < 0 || kvol < 1 || cin < 1 || cout < 1) return 0;
  return ops->wgrad_pairs_workspace(pair_cap, kvol, cin, cout);
}

extern "C" int tsmi_conv_wgrad_pairs(tsmi_stream_t s, const void *x, const void *dy,
                                     const int32_t *pairs, const int32_t *seg_steps,
                                     int64_t pair_cap, int x_col, int kvol, int cin, int cout,
                                     int dtype, float *workspace, int64_t workspace_elems,
                                     void *dw) {
  const ConvOps *ops = ops_for(dtype);
  if (int e = check_shapes("conv_wgrad_pairs", ops, kvol, cin, cout)) return e;
  TSMI_REQUIRE(pair_cap >= 0 && (x_col == 0 || x_col == 1), "conv_wgrad_pairs: bad arguments");
  TSMI_REQUIRE(dw && workspace && seg_steps, "conv_wgrad_pairs: null output, workspace or seg_steps");
  TSMI_REQUIRE(pair_cap == 0 || (x && dy && pairs), "conv_wgrad_pairs: null pointer");
  TSMI_REQUIRE(aligned16(x) && aligned16(dy) && ((uintptr_t)pairs & 7) == 0,
               "conv_wgrad_pairs: x and dy must be 16-byte aligned, pairs 8-byte aligned");
  return ops->wgrad_pairs((hipStream_t)s, x, dy, pairs, seg_steps, pair_cap, x_col, kvol, cin, cout,
                          workspace, workspace_elems, dw);
}

extern "C" int tsmi_conv_fetch_on_demand(tsmi_stream_t s, const void *x, const void *w_packed,
                                         const int32_t *nbmaps_planar, int64_t nnz,
                                         const int32_t *nbaddrs, const int32_t *qnbaddrs,
                                         int64_t qnnz, const int32_t *row_mask, int64_t n_out,
                                         int kvol, int cin, int cout, int dtype, int transpose,
                                         int center_k, const void *bias, const void *residual,
                                         int relu, void *partial, void *y) {
  const ConvOps *ops = ops_for(dtype);
  if (int e = check_shapes("conv_fetch_on_demand", ops, kvol, cin, cout)) return e;
  TSMI_REQUIRE(nnz >= 0 && qnnz >= nnz && qnnz % 128 == 0 && n_out >= 0,
               "conv_fetch_on_demand: bad sizes (nnz %lld, qnnz %lld)", (long long)nnz,
               (long long)qnnz);
  TSMI_REQUIRE(center_k >= -1 && center_k < kvol, "conv_fetch_on_demand: bad center_k");
  if (n_out == 0) return TSMI_OK;
  TSMI_REQUIRE(x && w_packed && nbaddrs && qnbaddrs && row_mask && y,
               "conv_fetch_on_demand: null pointer");
  TSMI_REQUIRE(nnz == 0 || (nbmaps_planar && partial), "conv_fetch_on_demand: null pair list");
  TSMI_REQUIRE(aligned16(x) && aligned16(w_packed) && aligned16(partial),
               "conv_fetch_on_demand: x, w_packed and partial must be 16-byte aligned");
  const int32_t *rows = transpose ? nbmaps_planar + nnz : nbmaps_planar;
  if (nnz > 0)
    if (int e = ops->pairs((hipStream_t)s, x, w_packed, rows, nbaddrs, qnbaddrs, qnnz, kvol, cin,
                           cout, partial))
      return e;
  return ops->scatter((hipStream_t)s, partial, nbaddrs, row_mask, n_out, kvol, cout, center_k, bias,
                      residual, relu, y);
}

extern "C" int tsmi_conv_segments_supported(int kvol, int cin, int cout, int dtype) {
  const ConvOps *ops = ops_for(dtype);
  if (!ops || kvol < 1 || cin < 1 || cout < 1) return 0;
  return ops->segments_supported(kvol, cin, cout);
}

static int implicit_gemm_segments(tsmi_stream_t s, const void *x, const void *w_packed,
                                  const int32_t *in_rows, const int32_t *counts, const int32_t *pos,
                                  int64_t seg_rows, int64_t n_out, int kvol, int cin, int cout, int dtype,
                                  const void *bias, const void *residual, int relu, void *products, void *y,
                                  const OutPlace *place) {
  const ConvOps *ops = ops_for(dtype);
  if (int e = check_shapes("conv_implicit_gemm_segments", ops, kvol, cin, cout)) return e;
  if (int e = check_place("conv_implicit_gemm_segments", place, cout)) return e;
  TSMI_REQUIRE(n_out >= 0 && seg_rows >= n_out && seg_rows % 64 == 0,
               "conv_implicit_gemm_segments: bad sizes (n_out %lld, seg_rows %lld)", (long long)n_out,
               (long long)seg_rows);
  if (n_out == 0) return TSMI_OK;
  TSMI_REQUIRE(x && w_packed && in_rows && counts && pos && products && y,
               "conv_implicit_gemm_segments: null pointer");
  TSMI_REQUIRE(aligned16(x) && aligned16(w_packed) && aligned16(products) && aligned16(y),
               "conv_implicit_gemm_segments: x, w_packed, products and y must be 16-byte aligned");
  if (int e = ops->segments((hipStream_t)s, x, w_packed, in_rows, counts, seg_rows, kvol, cin, cout,
                            products))
    return e;
  return ops->segment_sum((hipStream_t)s, products, pos, n_out, kvol, seg_rows, cout, bias, residual,
                          relu, y, place);
}

extern "C" int tsmi_conv_implicit_gemm_segments(tsmi_stream_t s, const void *x, const void *w_packed,
                                               const int32_t *in_rows, const int32_t *counts,
                                               const int32_t *pos, int64_t seg_rows, int64_t n_out,
                                               int kvol, int cin, int cout, int dtype,
                                               const void *bias, const void *residual, int relu,
                                               void *products, void *y) {
  return implicit_gemm_segments(s, x, w_packed, in_rows, counts, pos, seg_rows, n_out, kvol, cin, cout, dtype,
                                bias, residual, relu, products, y, nullptr);
}

extern "C" int tsmi_gs_gather(tsmi_stream_t s, const void *x, const int32_t *nbmaps_inter,
                              int64_t nnz, int cin, int dtype, int transpose, void *buffer) {
  const ConvOps *ops = ops_for(dtype);
  if (!ops) return fail(TSMI_ERR_INVALID_ARGUMENT, "gs_gather: unsupported dtype");
  TSMI_REQUIRE(nnz >= 0 && cin >= 1, "gs_gather: bad sizes");
  if (nnz == 0) return TSMI_OK;
  TSMI_REQUIRE(x && nbmaps_inter && buffer, "gs_gather: null pointer");
  return ops->gather((hipStream_t)s, x, nbmaps_inter, nnz, cin, transpose ? 1 : 0, buffer);
}

extern "C" int tsmi_gs_gemm(tsmi_stream_t s, const void *buffer, const void *w_packed,
                            const int32_t *nbaddrs, const int32_t *qnbaddrs, int64_t nnz,
                            int64_t qnnz, int kvol, int cin, int cout, int dtype,
                            void *out_buffer) {
  const ConvOps *ops = ops_for(dtype);
  if (int e = check_shapes("gs_gemm", ops, kvol, cin, cout)) return e;
  TSMI_REQUIRE(nnz >= 0 && qnnz >= nnz && qnnz % 128 == 0, "gs_gemm: bad sizes");
  if (nnz == 0) return TSMI_OK;
  TSMI_REQUIRE(buffer && w_packed && nbaddrs && qnbaddrs && out_buffer, "gs_gemm: null pointer");
  TSMI_REQUIRE(aligned16(buffer) && aligned16(w_packed) && aligned16(out_buffer),
               "gs_gemm: buffers must be 16-byte aligned");
  return ops->pairs((hipStream_t)s, buffer, w_packed, nullptr, nbaddrs, qnbaddrs, qnnz, kvol, cin,
                    cout, out_buffer);
}

extern "C" int tsmi_gs_scatter(tsmi_stream_t s, const void *out_buffer, const int32_t *nbaddrs,
                               const int32_t *row_mask, int64_t n_out, int kvol, int cout,
                               int dtype, int center_k, const void *bias, const void *residual,
                               int relu, void *y) {
  const ConvOps *ops = ops_for(dtype);
  if (!ops) return fail(TSMI_ERR_INVALID_ARGUMENT, "gs_scatter: unsupported dtype");
  TSMI_REQUIRE(n_out >= 0 && kvol >= 1 && cout >= 1 && center_k >= -1 && center_k < kvol,
               "gs_scatter: bad sizes");
  if (n_out == 0) return TSMI_OK;
  TSMI_REQUIRE(out_buffer && nbaddrs && row_mask && y, "gs_scatter: null pointer");
  return ops->scatter((hipStream_t)s, out_buffer, nbaddrs, row_mask, n_out, kvol, cout, center_k,
                      bias, residual, relu, y);
}

// The two calls a forward makes most often, with their arguments in one block: a binding that
// converts arguments one by one (ctypes: 0.1 us each) passes one pointer instead of 17 or 18.
static inline const void *as_ptr(int64_t v) { return (const void *)(uintptr_t)v; }

// The placement of a packed call's result: three more entries (row pitch of y, second destination,
// its row pitch); all zero: a dense y and nothing else.
static const OutPlace *place_of(const int64_t *w, OutPlace *place) {
  if (w[0] == 0 && w[1] == 0) return nullptr;
  place->ldy = w[0];
  place->y2 = (void *)as_ptr(w[1]);
  place->ldy2 = w[2];
  return place;
}

extern "C" int tsmi_conv_implicit_gemm_packed(const int64_t *a) {
  TSMI_REQUIRE(a, "conv_implicit_gemm_packed: null argument block");
  OutPlace place;
  return implicit_gemm((tsmi_stream_t)as_ptr(a[0]), as_ptr(a[1]), as_ptr(a[2]), (const int32_t *)as_ptr(a[3]),
                       a[4], a[5], (int)a[6], (int)a[7], (int)a[8], (int)a[9], as_ptr(a[10]),
                       as_ptr(a[11]), (int)a[12], (float *)as_ptr(a[13]), a[14],
                       (int32_t *)as_ptr(a[15]), a[16], (void *)as_ptr(a[17]), place_of(a + 18, &place));
}

extern "C" int tsmi_conv_implicit_gemm_grouped_packed(const int64_t *a) {
  TSMI_REQUIRE(a, "conv_implicit_gemm_grouped_packed: null argument block");
  OutPlace place;
  return implicit_gemm_grouped((tsmi_stream_t)as_ptr(a[0]), as_ptr(a[1]), as_ptr(a[2]),
                               (const int32_t *)as_ptr(a[3]), (const int32_t *)as_ptr(a[4]),
                               (const int32_t *)as_ptr(a[5]), (const int32_t *)as_ptr(a[6]), a[7], a[8],
                               (int)a[9], (int)a[10], (int)a[11], (int)a[12], as_ptr(a[13]),
                               as_ptr(a[14]), (int)a[15], (void *)as_ptr(a[16]), place_of(a + 17, &place));
}

extern "C" int tsmi_conv_implicit_gemm_segments_packed(const int64_t *a) {
  TSMI_REQUIRE(a, "conv_implicit_gemm_segments_packed: null argument block");
  OutPlace place;
  return implicit_gemm_segments((tsmi_stream_t)as_ptr(a[0]), as_ptr(a[1]), as_ptr(a[2]),
                                (const int32_t *)as_ptr(a[3]), (const int32_t *)as_ptr(a[4]),
                                (const int32_t *)as_ptr(a[5]), a[6], a[7], (int)a[8], (int)a[9],
                                (int)a[10], (int)a[11], as_ptr(a[12]), as_ptr(a[13]), (int)a[14],
                                (void *)as_ptr(a[15]), (void *)as_ptr(a[16]), place_of(a + 17, &place));
}
