/*
 * CPU oracle for the sparse-convolution forward path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT THE PRODUCT.  It restates, in plain C, the
 * algorithms of the reference (mit-han-lab/torchsparse v2.1.0) so that the HIP
 * path can be checked bit-exactly (integer work) or to tolerance (float work).
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may call it.
 *
 * Every function cites the reference file:line whose behaviour it follows.
 * Pinning status (what independent evidence fixes each function) is listed in
 * oracle/__init__.py next to the ctypes wrappers.
 *
 * Conventions shared with the reference:
 *   coords      int32 [N,4] rows (b, x, y, z)
 *   out_in_map  int32 [N_pad, K_vol], -1 = no neighbour, N_pad = ceil128(N_out)
 *   weights     [K_vol, Cin, Cout] row-major
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif


#define TSO_EXPORT __attribute__((visibility("default")))

/* Thread count of the parallel loops below (timing only; results do not depend on it).
 * Returns the count now in force. */
TSO_EXPORT int tso_set_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
  return omp_get_max_threads();
#else
  (void)n;
  return 1;
#endif
}

/* ------------------------------------------------------------------ helpers */

typedef struct {
  int64_t key;
  int32_t idx;
} tso_pair;

static int pair_cmp(const void *a, const void *b) {
  const tso_pair *pa = (const tso_pair *)a, *pb = (const tso_pair *)b;
  if (pa->key < pb->key) return -1;
  if (pa->key > pb->key) return 1;
  return (pa->idx > pb->idx) - (pa->idx < pb->idx);
}

static int i64_cmp(const void *a, const void *b) {
  int64_t x = *(const int64_t *)a, y = *(const int64_t *)b;
  return (x > y) - (x < y);
}

/* Row-major ravel of (b,x,y,z) over the extents max-min+1.
 * Follows backend/others/sparsemapping_cuda.cu:12-26 (transform_coords). */
static int64_t ravel4(const int *c, const int *cmin, const int *cmax) {
  int64_t cur = 0;
  for (int i = 0; i < 4; i++) {
    int64_t size = (int64_t)cmax[i] - cmin[i] + 1;
    cur = cur * size + ((int64_t)c[i] - cmin[i]);
  }
  return cur;
}

/* Inverse of ravel4.  Follows sparsemapping_cuda.cu:28-42. */
static void unravel4(int64_t key, const int *cmin, const int *cmax, int *out) {
  for (int i = 3; i >= 0; i--) {
    int64_t size = (int64_t)cmax[i] - cmin[i] + 1;
    out[i] = cmin[i] + (int)(key % size);
    key /= size;
  }
}

static int kernel_volume(const int *ks) { return ks[0] * ks[1] * ks[2]; }

/* Decode a flat kernel index into per-axis digits (x,y,z).
 * Odd kernel volume: x is the fastest digit; even volume: z is the fastest.
 * Follows sparsemapping_cuda.cu:165-170 (odd) and :209-214 (even). */
static void decode_digits(int k, const int *ks, int odd, int *d) {
  if (odd) {
    for (int a = 0; a < 3; a++) {
      d[a] = k % ks[a];
      k /= ks[a];
    }
  } else {
    for (int a = 2; a >= 0; a--) {
      d[a] = k % ks[a];
      k /= ks[a];
    }
  }
}

/* Binary search of a sorted (key, idx) table; returns idx or -1. */
static int32_t table_find(const tso_pair *t, int n, int64_t key) {
  int lo = 0, hi = n - 1;
  while (lo <= hi) {
    int mid = lo + (hi - lo) / 2;
    if (t[mid].key == key) return t[mid].idx;
    if (t[mid].key < key)
      lo = mid + 1;
    else
      hi = mid - 1;
  }
  return -1;
}

static tso_pair *build_table(const int *coords, int n, const int *cmin,
                             const int *cmax) {
  tso_pair *t = (tso_pair *)malloc(sizeof(tso_pair) * (size_t)(n > 0 ? n : 1));
  for (int i = 0; i < n; i++) {
    t[i].key = ravel4(coords + 4 * i, cmin, cmax);
    t[i].idx = i;
  }
  qsort(t, (size_t)n, sizeof(tso_pair), pair_cmp);
  return t;
}

static int in_bounds3(const int *c, const int *cmin, const int *cmax) {
  for (int a = 1; a < 4; a++)
    if (c[a] < cmin[a] || c[a] > cmax[a]) return 0;
  return 1;
}

/* ---------------------------------------------------------- kernel offsets */

/* Canonical offset table, shape [K_vol,3].
 * Follows nn/utils/kernel.py:21-35: per axis arange(-size//2+1, size//2+1)
 * (Python floor division) times stride*dilation; odd volume enumerates x
 * fastest, even volume enumerates z fastest. */
TSO_EXPORT int tso_kernel_offsets(const int *ks, const int *stride,
                                  const int *dilation, int *out) {
  int kvol = kernel_volume(ks);
  int odd = kvol % 2 == 1;
  for (int k = 0; k < kvol; k++) {
    int d[3];
    decode_digits(k, ks, odd, d);
    for (int a = 0; a < 3; a++) {
      /* python: -size // 2 + 1 with floor division */
      int lo = -((ks[a] + 1) / 2) + 1;
      out[3 * k + a] = (lo + d[a]) * stride[a] * dilation[a];
    }
  }
  return kvol;
}

/* ----------------------------------------------------- submanifold kernel map */

/* out_in_map[i,k] = j  iff  coords[j] == coords[i] + off(k), same batch.
 * Follows sparsemapping_cuda.cu:129-231 and host code :303-345:
 *  - odd volume: off = digit - (ks-1)/2, x fastest, mirrored write of
 *    map[j, K_vol-1-k] = i while scanning the first half, centre column = i;
 *  - even volume: off = digit (0..ks-1), z fastest, no mirroring;
 *  - neighbours outside [cmin,cmax] on a spatial axis are rejected before the
 *    lookup; rows N..N_pad-1 stay -1.
 * map must hold n_pad*K_vol ints. */
TSO_EXPORT void tso_kmap_subm(const int *coords, int n, const int *cmin,
                              const int *cmax, const int *ks, int n_pad,
                              int *map) {
  int kvol = kernel_volume(ks);
  int odd = kvol % 2 == 1;
  for (int64_t t = 0; t < (int64_t)n_pad * kvol; t++) map[t] = -1;
  tso_pair *table = build_table(coords, n, cmin, cmax);
  for (int i = 0; i < n; i++) {
    const int *c = coords + 4 * i;
    int nk = odd ? kvol / 2 : kvol;
    if (odd) map[(int64_t)i * kvol + kvol / 2] = i;
    for (int k = 0; k < nk; k++) {
      int d[3], q[4];
      decode_digits(k, ks, odd, d);
      q[0] = c[0];
      for (int a = 0; a < 3; a++)
        q[a + 1] = c[a + 1] + (odd ? d[a] - (ks[a] - 1) / 2 : d[a]);
      if (!in_bounds3(q, cmin, cmax)) continue;
      int32_t j = table_find(table, n, ravel4(q, cmin, cmax));
      if (j < 0) continue;
      map[(int64_t)i * kvol + k] = j;
      if (odd) map[(int64_t)j * kvol + kvol - 1 - k] = i;
    }
  }
  free(table);
}

/* ------------------------------------------------------ downsample kernel map */

/* Enumerate the candidate output of (input i, kernel index k); returns 1 and
 * fills o[4] when valid.  Follows sparsemapping_cuda.cu:60-107 (stage 1):
 * o = (in + pad + digit - (ks-1)) / stride, required divisible (C remainder,
 * so a negative numerator only passes when it is an exact multiple) and inside
 * [cmin,cmax] on the three spatial axes. */
static int downsample_candidate(const int *c, int k, const int *ks,
                                const int *stride, const int *pad,
                                const int *cmin, const int *cmax, int odd,
                                int *o) {
  int d[3];
  decode_digits(k, ks, odd, d);
  o[0] = c[0];
  for (int a = 0; a < 3; a++) {
    int v = c[a + 1] + pad[a] + d[a] - (ks[a] - 1);
    if (v % stride[a] != 0) return 0;
    o[a + 1] = v / stride[a];
  }
  return in_bounds3(o, cmin, cmax);
}

/* Output coordinates of a strided convolution, ascending in ravel order
 * (= lexicographic (b,x,y,z)).  Follows sparsemapping_cuda.cu:464-493: all
 * valid candidates, torch::_unique (sorted), unravel.  out_coords must hold
 * n*K_vol rows; returns N_out. */
TSO_EXPORT int tso_downsample_coords(const int *coords, int n, const int *cmin,
                                     const int *cmax, const int *ks,
                                     const int *stride, const int *pad,
                                     int *out_coords) {
  int kvol = kernel_volume(ks);
  int odd = kvol % 2 == 1;
  int64_t *keys = (int64_t *)malloc(sizeof(int64_t) * ((size_t)n * kvol + 1));
  int64_t cnt = 0;
  for (int i = 0; i < n; i++)
    for (int k = 0; k < kvol; k++) {
      int o[4];
      if (downsample_candidate(coords + 4 * i, k, ks, stride, pad, cmin, cmax,
                               odd, o))
        keys[cnt++] = ravel4(o, cmin, cmax);
    }
  qsort(keys, (size_t)cnt, sizeof(int64_t), i64_cmp);
  int n_out = 0;
  for (int64_t t = 0; t < cnt; t++) {
    if (t > 0 && keys[t] == keys[t - 1]) continue;
    unravel4(keys[t], cmin, cmax, out_coords + 4 * n_out);
    n_out++;
  }
  free(keys);
  return n_out;
}

/* out_in_map for a strided convolution given its output coordinates.
 * Follows sparsemapping_cuda.cu:110-126 (stage 3): for every valid candidate
 * (i, k) with output row o: map[o, K_vol-1-k] = i.  (The reference narrows the
 * 64-bit ravel key to int at :120; this restatement keeps 64 bits.) */
TSO_EXPORT void tso_kmap_downsample(const int *coords, int n,
                                    const int *out_coords, int n_out,
                                    const int *cmin, const int *cmax,
                                    const int *ks, const int *stride,
                                    const int *pad, int n_pad, int *map) {
  int kvol = kernel_volume(ks);
  int odd = kvol % 2 == 1;
  for (int64_t t = 0; t < (int64_t)n_pad * kvol; t++) map[t] = -1;
  tso_pair *table = build_table(out_coords, n_out, cmin, cmax);
  for (int i = 0; i < n; i++)
    for (int k = 0; k < kvol; k++) {
      int o[4];
      if (!downsample_candidate(coords + 4 * i, k, ks, stride, pad, cmin, cmax,
                                odd, o))
        continue;
      int32_t r = table_find(table, n_out, ravel4(o, cmin, cmax));
      if (r >= 0) map[(int64_t)r * kvol + kvol - 1 - k] = i;
    }
  free(table);
}

/* ------------------------------------------- kmap_mode="hashmap" primitives */

/* unique(floor(coords / stride)) sorted lexicographically.
 * Follows nn/functional/conv/kmap/downsample.py:30-37 (torch.unique(dim=0)
 * returns rows in ascending lexicographic order).  Returns N_out. */
TSO_EXPORT int tso_spdownsample_floor(const int *coords, int n,
                                      const int *stride, int *out_coords) {
  int *tmp = (int *)malloc(sizeof(int) * 4 * (size_t)(n > 0 ? n : 1));
  int cmin[4] = {0, 0, 0, 0}, cmax[4] = {0, 0, 0, 0};
  for (int i = 0; i < n; i++) {
    tmp[4 * i] = coords[4 * i];
    for (int a = 0; a < 3; a++) {
      int v = coords[4 * i + 1 + a];
      int s = stride[a];
      int q = v / s;
      if ((v % s != 0) && ((v < 0) != (s < 0))) q--; /* floor */
      tmp[4 * i + 1 + a] = q;
    }
    for (int a = 0; a < 4; a++) {
      int v = tmp[4 * i + a];
      if (i == 0 || v < cmin[a]) cmin[a] = v;
      if (i == 0 || v > cmax[a]) cmax[a] = v;
    }
  }
  int64_t *keys = (int64_t *)malloc(sizeof(int64_t) * (size_t)(n > 0 ? n : 1));
  for (int i = 0; i < n; i++) keys[i] = ravel4(tmp + 4 * i, cmin, cmax);
  qsort(keys, (size_t)n, sizeof(int64_t), i64_cmp);
  int n_out = 0;
  for (int i = 0; i < n; i++) {
    if (i > 0 && keys[i] == keys[i - 1]) continue;
    unravel4(keys[i], cmin, cmax, out_coords + 4 * n_out);
    n_out++;
  }
  free(keys);
  free(tmp);
  return n_out;
}

/* map[o,k] = i  iff  in_coords[i] == out_coords[o]*stride + digit-(ks-1)/2.
 * Follows backend/hashmap/hashmap_cuda.cuh:199-253 (lookup_coords_kernel):
 * padding never enters, odd volume x fastest / even volume z fastest, integer
 * (ks-1)/2 so even sizes use offsets 0..ks-1.  The reference keys its table by
 * a 64-bit FNV hash of the coordinate; this restatement matches coordinates
 * exactly (what the reference does whenever the hash does not collide). */
TSO_EXPORT void tso_lookup_coords(const int *in_coords, int n_in,
                                  const int *out_coords, int n_out,
                                  const int *ks, const int *stride, int n_pad,
                                  int *map) {
  int kvol = kernel_volume(ks);
  int odd = kvol % 2 == 1;
  int cmin[4], cmax[4];
  for (int a = 0; a < 4; a++) cmin[a] = cmax[a] = n_in > 0 ? in_coords[a] : 0;
  for (int i = 0; i < n_in; i++)
    for (int a = 0; a < 4; a++) {
      int v = in_coords[4 * i + a];
      if (v < cmin[a]) cmin[a] = v;
      if (v > cmax[a]) cmax[a] = v;
    }
  for (int64_t t = 0; t < (int64_t)n_pad * kvol; t++) map[t] = -1;
  tso_pair *table = build_table(in_coords, n_in, cmin, cmax);
  for (int o = 0; o < n_out; o++)
    for (int k = 0; k < kvol; k++) {
      int d[3], q[4];
      decode_digits(k, ks, odd, d);
      q[0] = out_coords[4 * o];
      for (int a = 0; a < 3; a++)
        q[a + 1] = out_coords[4 * o + 1 + a] * stride[a] + d[a] - (ks[a] - 1) / 2;
      if (q[0] < cmin[0] || q[0] > cmax[0] || !in_bounds3(q, cmin, cmax)) continue;
      map[(int64_t)o * kvol + k] = table_find(table, n_in, ravel4(q, cmin, cmax));
    }
  free(table);
}

/* ------------------------------------------------------- derived map products */

/* map_t[in,k] = out for every map[out,k] = in >= 0; map_t pre-filled with -1.
 * Follows backend/others/query_cuda.cu:9-15 and conv/hash/query.py:47-55. */
TSO_EXPORT void tso_transpose_map(const int *map, int n_rows, int kvol,
                                  int n_rows_t, int *map_t) {
  for (int64_t t = 0; t < (int64_t)n_rows_t * kvol; t++) map_t[t] = -1;
  for (int64_t t = 0; t < (int64_t)n_rows * kvol; t++) {
    int in = map[t];
    if (in < 0) continue;
    map_t[(int64_t)in * kvol + t % kvol] = (int)(t / kvol);
  }
}

/* bitmask[s, r] = sum_i (map[r, s*L+i] >= 0) << i for r < valid_n, -1 for the
 * padding rows.  L = ceil(K_vol/split); the last split takes the remainder.
 * Follows query_cuda.cu:17-31 and :59-65. */
TSO_EXPORT void tso_derive_bitmask(const int *map, int n_pad, int kvol,
                                   int split, int valid_n, int *bitmask) {
  int len = (kvol + split - 1) / split;
  for (int64_t t = 0; t < (int64_t)split * n_pad; t++) bitmask[t] = -1;
  for (int r = 0; r < valid_n; r++)
    for (int s = 0; s < split; s++) {
      int l = (s == split - 1) ? kvol - s * len : len;
      uint32_t m = 0;
      for (int i = 0; i < l; i++)
        if (map[(int64_t)r * kvol + s * len + i] >= 0) m += 1u << i;
      bitmask[(int64_t)s * n_pad + r] = (int)m;
    }
}

/* reordered[r,c] = map[loc[split(c), r], c].  Follows reorder_map_cuda.cu:8-23. */
TSO_EXPORT void tso_reorder_map(const int *map, const int *loc, int n_pad,
                                int kvol, int split, int *out) {
  int len = (kvol + split - 1) / split;
  for (int r = 0; r < n_pad; r++)
    for (int c = 0; c < kvol; c++) {
      int src = loc[(int64_t)(c / len) * n_pad + r];
      out[(int64_t)r * kvol + c] = map[(int64_t)src * kvol + c];
    }
}

/* reduced[s,t] = OR of sorted_mask[s, t*tile .. (t+1)*tile-1] (clipped).
 * Follows reduce_bitmask_cuda.cu:13-57 and host :60-84. */
TSO_EXPORT void tso_reduce_bitmask(const int *mask, int split, int n_pad,
                                   int tile, int *reduced) {
  int rows = (n_pad - 1) / tile + 1;
  for (int s = 0; s < split; s++)
    for (int t = 0; t < rows; t++) {
      int acc = 0;
      for (int r = t * tile; r < (t + 1) * tile && r < n_pad; r++)
        acc |= mask[(int64_t)s * n_pad + r];
      reduced[(int64_t)s * rows + t] = acc;
    }
}

/* Pair lists from an out_in_map: for k ascending, out ascending, every
 * map[out,k] = in != -1 yields the pair (in, out).  nbmaps is interleaved
 * [nnz,2]; nbsizes [K_vol].  Follows kmap/func/hashmap_on_the_fly.py:138-141
 * (transpose, count != -1, nonzero in row-major order).  Returns nnz. */
TSO_EXPORT int64_t tso_pair_lists(const int *map, int n_pad, int kvol,
                                  int *nbmaps, int *nbsizes) {
  int64_t nnz = 0;
  for (int k = 0; k < kvol; k++) {
    int cnt = 0;
    for (int o = 0; o < n_pad; o++) {
      int in = map[(int64_t)o * kvol + k];
      if (in == -1) continue;
      if (nbmaps) {
        nbmaps[2 * nnz] = in;
        nbmaps[2 * nnz + 1] = o;
      }
      nnz++;
      cnt++;
    }
    nbsizes[k] = cnt;
  }
  return nnz;
}

/* input_mask[k*n_in + in] = output_mask[k*n_out + out] = position of the pair
 * inside offset k's list, -1 elsewhere; the centre offset of an odd-volume
 * submanifold map (n_in == n_out) is skipped.
 * Follows sparsemapping_cuda.cu:235-256 and :510-548. */
TSO_EXPORT void tso_build_masks(int n_in, int n_out, const int *nbmaps,
                                const int *nbsizes, int kvol, int *input_mask,
                                int *output_mask) {
  for (int64_t t = 0; t < (int64_t)kvol * n_in; t++) input_mask[t] = -1;
  for (int64_t t = 0; t < (int64_t)kvol * n_out; t++) output_mask[t] = -1;
  int64_t base = 0;
  for (int k = 0; k < kvol; k++) {
    int skip = (n_in == n_out && kvol % 2 == 1 && k == kvol / 2);
    if (!skip)
      for (int p = 0; p < nbsizes[k]; p++) {
        input_mask[(int64_t)k * n_in + nbmaps[2 * (base + p)]] = p;
        output_mask[(int64_t)k * n_out + nbmaps[2 * (base + p) + 1]] = p;
      }
    base += nbsizes[k];
  }
}

/* nbaddrs = exclusive scan of nbsizes, qnbaddrs = exclusive scan of nbsizes
 * rounded up to q; both [K_vol+1].  Follows exclusive_scan_cuda.cu:7-45. */
TSO_EXPORT void tso_exclusive_scan_quantified(int kvol, const int *nbsizes,
                                              int q, int *nbaddrs,
                                              int *qnbaddrs) {
  int acc = 0, qacc = 0;
  nbaddrs[0] = 0;
  qnbaddrs[0] = 0;
  for (int k = 0; k < kvol; k++) {
    acc += nbsizes[k];
    qacc += (nbsizes[k] + q - 1) / q * q;
    nbaddrs[k + 1] = acc;
    qnbaddrs[k + 1] = qacc;
  }
}

/* ------------------------------------------------------------- convolutions */

/* Closed form of every dataflow: Y[i,:] = sum_k [m=map[i,k]>=0] X[m,:] W[k],
 * accumulated in double and rounded once to float.
 * Follows the contract of convolution_forward_implicit_gemm_cuda.cu:1527-1986
 * (every output row written, all-miss rows are zero). */
TSO_EXPORT void tso_conv_implicit_gemm(const float *x, const float *w,
                                       const int *map, int n_out, int kvol,
                                       int cin, int cout, float *y) {
#pragma omp parallel
  {
    double *acc = (double *)malloc(sizeof(double) * (size_t)cout);
#pragma omp for schedule(static)
    for (int i = 0; i < n_out; i++) {
      for (int c = 0; c < cout; c++) acc[c] = 0.0;
      for (int k = 0; k < kvol; k++) {
        int m = map[(int64_t)i * kvol + k];
        if (m < 0) continue;
        const float *xr = x + (int64_t)m * cin;
        const float *wk = w + (int64_t)k * cin * cout;
        for (int ci = 0; ci < cin; ci++) {
          double xv = xr[ci];
          const float *wr = wk + (int64_t)ci * cout;
          for (int c = 0; c < cout; c++) acc[c] += xv * wr[c];
        }
      }
      for (int c = 0; c < cout; c++) y[(int64_t)i * cout + c] = (float)acc[c];
    }
    free(acc);
  }
}

/* C[m,n] += A[m,k] B[k,n], fp32. */
static void sgemm_acc(const float *a, const float *b, float *c, int m, int k,
                      int n, int parallel_rows) {
#pragma omp parallel for schedule(static) if (parallel_rows)
  for (int i = 0; i < m; i++) {
    float *cr = c + (int64_t)i * n;
    for (int p = 0; p < k; p++) {
      float av = a[(int64_t)i * k + p];
      const float *br = b + (int64_t)p * n;
      for (int j = 0; j < n; j++) cr[j] += av * br[j];
    }
  }
}

/* fp32 gather -> GEMM -> scatter-add, one kernel offset at a time.
 * Follows convolution_gather_scatter_cpu.cpp:8-109: output zeroed; for an
 * odd-volume map with n_out == n_in the centre offset is a plain X*W[centre]
 * and its pair list is skipped; pairs are interleaved (in,out) and `transpose`
 * swaps their roles; negative indices are skipped.
 * variant 0 = the reference's threading (a parallel region per row over the
 * channel loop of gather and scatter, :16 and :31); variant 1 = threads over
 * rows (gather and GEMM) and a serial scatter. */
TSO_EXPORT int tso_conv_gather_scatter(const float *x, int n_in, int cin,
                                       const float *w, int kvol, int cout,
                                       const int *nbmaps, const int *nbsizes,
                                       float *y, int n_out, int transpose,
                                       int variant) {
  memset(y, 0, sizeof(float) * (size_t)n_out * cout);
  int flag = (kvol % 2 == 1) && (n_out == n_in);
  int buf_rows = 1;
  for (int k = 0; k < kvol; k++) {
    if (flag && k == kvol / 2) continue;
    if (nbsizes[k] > buf_rows) buf_rows = nbsizes[k];
  }
  if (flag)
    sgemm_acc(x, w + (int64_t)(kvol / 2) * cin * cout, y, n_in, cin, cout,
              variant == 1);
  float *ib = (float *)malloc(sizeof(float) * (size_t)buf_rows * cin);
  float *ob = (float *)malloc(sizeof(float) * (size_t)buf_rows * cout);
  int64_t cur = 0;
  for (int k = 0; k < kvol; k++) {
    int nk = nbsizes[k];
    if ((flag && k == kvol / 2) || nk == 0) {
      cur += 2 * (int64_t)nk;
      continue;
    }
    const int *pairs = nbmaps + cur;
    /* gather */
    if (variant == 0) {
      for (int p = 0; p < nk; p++) {
        int src = pairs[2 * p + transpose];
        if (src < 0) continue;
#pragma omp parallel for
        for (int c = 0; c < cin; c++)
          ib[(int64_t)p * cin + c] = x[(int64_t)src * cin + c];
      }
    } else {
#pragma omp parallel for schedule(static)
      for (int p = 0; p < nk; p++) {
        int src = pairs[2 * p + transpose];
        if (src < 0) continue;
        memcpy(ib + (int64_t)p * cin, x + (int64_t)src * cin,
               sizeof(float) * (size_t)cin);
      }
    }
    /* matmul */
    memset(ob, 0, sizeof(float) * (size_t)nk * cout);
    sgemm_acc(ib, w + (int64_t)k * cin * cout, ob, nk, cin, cout, variant == 1);
    /* scatter */
    for (int p = 0; p < nk; p++) {
      int dst = pairs[2 * p + 1 - transpose];
      if (dst < 0) continue;
      if (variant == 0) {
#pragma omp parallel for
        for (int c = 0; c < cout; c++)
          y[(int64_t)dst * cout + c] += ob[(int64_t)p * cout + c];
      } else {
        for (int c = 0; c < cout; c++)
          y[(int64_t)dst * cout + c] += ob[(int64_t)p * cout + c];
      }
    }
    cur += 2 * (int64_t)nk;
  }
  free(ib);
  free(ob);
  return 0;
}

/* Backward of the gather-scatter convolution, pair lists in (in, out) columns:
 *   dX[in] += dY[out] W[k]^T,   dW[k] = sum_pairs X[in]^T dY[out]
 * for every pair of every offset (no centre shortcut: `flag` is false in the
 * reference).  transpose swaps the roles of the two columns.  Accumulates in
 * double.  Follows conv_backward_gather_scatter_cpu
 * (convolution/convolution_gather_scatter_cpu.cpp:111-188). */
TSO_EXPORT void tso_conv_backward_gather_scatter(
    const float *x, int n_in, int cin, const float *w, int kvol, int cout,
    const int *nbmaps, const int *nbsizes, const float *dy, float *dx, float *dw,
    int transpose) {
  double *dxa = (double *)calloc((size_t)n_in * cin, sizeof(double));
  double *dwa = (double *)calloc((size_t)kvol * cin * cout, sizeof(double));
  int64_t cur = 0;
  for (int k = 0; k < kvol; k++) {
    int nk = nbsizes[k];
    const int *pairs = nbmaps + cur;
    const float *wk = w + (int64_t)k * cin * cout;
    double *dwk = dwa + (int64_t)k * cin * cout;
    for (int p = 0; p < nk; p++) {
      int in = pairs[2 * p + transpose];
      int out = pairs[2 * p + 1 - transpose];
      if (in < 0 || out < 0) continue;
      const float *g = dy + (int64_t)out * cout;
      const float *xr = x + (int64_t)in * cin;
      double *dxr = dxa + (int64_t)in * cin;
      for (int ci = 0; ci < cin; ci++) {
        double a = 0.0, xv = xr[ci];
        for (int c = 0; c < cout; c++) {
          a += (double)g[c] * wk[(int64_t)ci * cout + c];
          dwk[(int64_t)ci * cout + c] += xv * g[c];
        }
        dxr[ci] += a;
      }
    }
    cur += 2 * (int64_t)nk;
  }
  for (int64_t i = 0; i < (int64_t)n_in * cin; i++) dx[i] = (float)dxa[i];
  for (int64_t i = 0; i < (int64_t)kvol * cin * cout; i++) dw[i] = (float)dwa[i];
  free(dxa);
  free(dwa);
}

/* The same gradients from the forward map: for map[i,k] = m >= 0,
 *   dX[m] += dY[i] W[k]^T,   dW[k] += X[m]^T dY[i].
 * This is what the reference's dgrad (the forward kernel over out_in_map_bwd with
 * W[k]^T) and wgrad kernels compute (nn/functional/conv/func/implicit_gemm.py:129-190). */
TSO_EXPORT void tso_conv_backward_implicit_gemm(const float *x, int n_in, int cin,
                                                const float *w, int kvol, int cout,
                                                const int *map, int n_out,
                                                const float *dy, float *dx, float *dw) {
  double *dxa = (double *)calloc((size_t)n_in * cin, sizeof(double));
  double *dwa = (double *)calloc((size_t)kvol * cin * cout, sizeof(double));
  for (int i = 0; i < n_out; i++) {
    const float *g = dy + (int64_t)i * cout;
    for (int k = 0; k < kvol; k++) {
      int m = map[(int64_t)i * kvol + k];
      if (m < 0) continue;
      const float *wk = w + (int64_t)k * cin * cout;
      double *dwk = dwa + (int64_t)k * cin * cout;
      const float *xr = x + (int64_t)m * cin;
      double *dxr = dxa + (int64_t)m * cin;
      for (int ci = 0; ci < cin; ci++) {
        double a = 0.0, xv = xr[ci];
        for (int c = 0; c < cout; c++) {
          a += (double)g[c] * wk[(int64_t)ci * cout + c];
          dwk[(int64_t)ci * cout + c] += xv * g[c];
        }
        dxr[ci] += a;
      }
    }
  }
  for (int64_t i = 0; i < (int64_t)n_in * cin; i++) dx[i] = (float)dxa[i];
  for (int64_t i = 0; i < (int64_t)kvol * cin * cout; i++) dw[i] = (float)dwa[i];
  free(dxa);
  free(dwa);
}

/* ---------------------------------------- CPU map recipe of the CPU backend */

/* 64-bit FNV-1a over the four int32 fields of a row, then the 60-bit fold.
 * Follows backend/hash/hash_cpu.cpp:7-19.  `data` rows are hashed in the
 * order given (the reference's callers pass (x,y,z,b)). */
static uint64_t fnv_row(const int *row) {
  uint64_t h = 14695981039346656037ULL;
  for (int j = 0; j < 4; j++) {
    h ^= (unsigned int)row[j];
    h *= 1099511628211ULL;
  }
  return (h >> 60) ^ (h & 0xFFFFFFFFFFFFFFFULL);
}

TSO_EXPORT void tso_hash_cpu(const int *data, int n, int64_t *out) {
  for (int i = 0; i < n; i++) out[i] = (int64_t)fnv_row(data + 4 * i);
}

/* out[k*n+i] = hash(data[i,:3] + offsets[k], data[i,3]).
 * Follows backend/hash/hash_cpu.cpp:21-41. */
TSO_EXPORT void tso_kernel_hash_cpu(const int *data, int n, const int *offsets,
                                    int kvol, int64_t *out) {
#pragma omp parallel for schedule(static)
  for (int k = 0; k < kvol; k++)
    for (int i = 0; i < n; i++) {
      int row[4];
      for (int j = 0; j < 3; j++) row[j] = data[4 * i + j] + offsets[3 * k + j];
      row[3] = data[4 * i + 3];
      out[(int64_t)k * n + i] = (int64_t)fnv_row(row);
    }
}

/* out[q] = idx_target[t]+1 where hash_target[t] == hash_query[q], else 0.
 * Follows backend/others/query_cpu.cpp:12-37 (exact-match dictionary; the
 * reference uses google::dense_hash_map with empty key 0, first insert wins).
 * Implemented as an open-addressing table owned by this function. */
TSO_EXPORT void tso_hash_query_cpu(const int64_t *hash_query, int64_t n_query,
                                   const int64_t *hash_target,
                                   const int64_t *idx_target, int n_target,
                                   int64_t *out) {
  uint64_t cap = 16;
  while (cap < 2 * (uint64_t)n_target) cap <<= 1;
  int64_t *tk = (int64_t *)calloc(cap, sizeof(int64_t));
  int64_t *tv = (int64_t *)calloc(cap, sizeof(int64_t));
  for (int i = 0; i < n_target; i++) {
    int64_t key = hash_target[i];
    uint64_t s = ((uint64_t)key * 0x9E3779B97F4A7C15ULL) >> 20 & (cap - 1);
    while (tk[s] != 0 && tk[s] != key) s = (s + 1) & (cap - 1);
    if (tk[s] == 0) {
      tk[s] = key;
      tv[s] = idx_target[i] + 1;
    }
  }
#pragma omp parallel for schedule(static)
  for (int64_t q = 0; q < n_query; q++) {
    int64_t key = hash_query[q];
    uint64_t s = ((uint64_t)key * 0x9E3779B97F4A7C15ULL) >> 20 & (cap - 1);
    int64_t r = 0;
    while (tk[s] != 0) {
      if (tk[s] == key) {
        r = tv[s];
        break;
      }
      s = (s + 1) & (cap - 1);
    }
    out[q] = r;
  }
  free(tk);
  free(tv);
}

/* ------------------------------------------------ point-voxel operators */

/* The GPU hash of a coordinate row: 64-bit FNV-1a over its four int32 fields, WITHOUT the
 * 60-bit fold of the CPU version.  Follows backend/hash/hash_cuda.cu:9-22 (the fold is
 * commented out there). */
static uint64_t fnv_row_nofold(const int *row) {
  uint64_t h = 14695981039346656037ULL;
  for (int j = 0; j < 4; j++) {
    h ^= (unsigned int)row[j];
    h *= 1099511628211ULL;
  }
  return h;
}

TSO_EXPORT void tso_hash_gpu(const int *data, int64_t n, int64_t *out) {
  for (int64_t i = 0; i < n; i++) out[i] = (int64_t)fnv_row_nofold(data + 4 * i);
}

/* out[k*n+i] = hash(data[i,0], data[i,1:4] + offsets[k]): the offsets move the three
 * spatial fields, the batch field in column 0 stays.  Follows hash_cuda.cu:26-52. */
TSO_EXPORT void tso_kernel_hash_gpu(const int *data, int64_t n, const int *offsets, int kvol,
                                    int64_t *out) {
  for (int k = 0; k < kvol; k++)
    for (int64_t i = 0; i < n; i++) {
      int row[4];
      row[0] = data[4 * i];
      for (int j = 1; j < 4; j++) row[j] = data[4 * i + j] + offsets[3 * k + j - 1];
      out[(int64_t)k * n + i] = (int64_t)fnv_row_nofold(row);
    }
}

/* out[v] = number of i with idx[i] == v; negative indices are skipped.
 * Follows backend/others/count_cpu.cpp:7-23 (count_cuda.cu:10-17 is the same sum). */
TSO_EXPORT void tso_count(const int *idx, int64_t n, int s, int *out) {
  memset(out, 0, sizeof(int) * (size_t)s);
  for (int64_t i = 0; i < n; i++)
    if (idx[i] >= 0 && idx[i] < s) out[idx[i]]++;
}

/* out[v,:] = sum over points i with idx[i] == v of feats[i,:] / counts[v].  Points whose
 * index is outside [0, n1) or whose voxel has count 0 contribute nothing.
 * Follows backend/voxelize/voxelize_cpu.cpp:7-25 with the index guard of
 * voxelize_cuda.cu:55-57; accumulation in double. */
TSO_EXPORT void tso_voxelize_forward(const float *feats, int64_t n, int c, const int *idx,
                                     const int *counts, int64_t n1, float *out) {
  double *acc = (double *)calloc((size_t)(n1 * c > 0 ? n1 * c : 1), sizeof(double));
  for (int64_t i = 0; i < n; i++) {
    const int pos = idx[i];
    if (pos < 0 || pos >= n1 || counts[pos] == 0) continue;
    for (int j = 0; j < c; j++) acc[(int64_t)pos * c + j] += (double)feats[i * c + j] / (double)counts[pos];
  }
  for (int64_t i = 0; i < n1 * c; i++) out[i] = (float)acc[i];
  free(acc);
}

/* bottom[i,:] = top[idx[i],:] / counts[idx[i]] (0 for skipped points).
 * Follows voxelize_cpu.cpp:27-43. */
TSO_EXPORT void tso_voxelize_backward(const float *top, const int *idx, const int *counts,
                                      int64_t n, int c, int64_t n1, float *bottom) {
  for (int64_t i = 0; i < n; i++) {
    const int pos = idx[i];
    const int ok = !(pos < 0 || pos >= n1 || counts[pos] == 0);
    for (int j = 0; j < c; j++)
      bottom[i * c + j] = ok ? (float)((double)top[(int64_t)pos * c + j] / (double)counts[pos]) : 0.f;
  }
}

/* out[i,:] = sum_k weight[i,k] * feat[indices[i,k],:] over the 8 corner voxels, negative
 * index = absent corner.  Follows backend/devoxelize/devoxelize_cpu.cpp:10-32. */
TSO_EXPORT void tso_devoxelize_forward(const float *feat, int c, const int *indices,
                                       const float *weight, int64_t n, float *out) {
  for (int64_t i = 0; i < n; i++)
    for (int j = 0; j < c; j++) {
      double acc = 0.0;
      for (int k = 0; k < 8; k++) {
        const int v = indices[8 * i + k];
        if (v >= 0) acc += (double)weight[8 * i + k] * (double)feat[(int64_t)v * c + j];
      }
      out[i * c + j] = (float)acc;
    }
}

/* bottom[v,:] = sum over (i,k) with indices[i,k] == v of weight[i,k] * top[i,:]: the adjoint
 * of the forward.  Follows backend/devoxelize/devoxelize_cuda.cu:37-58.  (The CPU file's
 * backward, devoxelize_cpu.cpp:36-59, reads top_grad at the VOXEL index and writes through
 * negative indices; it is not the adjoint and is not followed.) */
TSO_EXPORT void tso_devoxelize_backward(const float *top, const int *indices, const float *weight,
                                        int64_t n, int64_t n_vox, int c, float *bottom) {
  double *acc = (double *)calloc((size_t)(n_vox * c > 0 ? n_vox * c : 1), sizeof(double));
  for (int64_t i = 0; i < n; i++)
    for (int k = 0; k < 8; k++) {
      const int v = indices[8 * i + k];
      if (v < 0 || v >= n_vox) continue;
      for (int j = 0; j < c; j++)
        acc[(int64_t)v * c + j] += (double)weight[8 * i + k] * (double)top[i * c + j];
    }
  for (int64_t i = 0; i < n_vox * c; i++) bottom[i] = (float)acc[i];
  free(acc);
}

/* dense[b,x,y,z,:] = feats[i,:] for coords[i] = (b,x,y,z); `dense` is zero elsewhere.
 * Follows backend/voxelize/voxelize_cuda.cu:10-24 (to_dense_forward_kernel). */
TSO_EXPORT void tso_to_dense_forward(const float *feats, const int *coords, int64_t n, int c,
                                     const int *range, float *dense) {
  const int64_t cells = (int64_t)range[0] * range[1] * range[2] * range[3];
  memset(dense, 0, sizeof(float) * (size_t)(cells * c));
  for (int64_t i = 0; i < n; i++) {
    const int *q = coords + 4 * i;
    const int64_t pos = (((int64_t)q[0] * range[1] + q[1]) * range[2] + q[2]) * range[3] + q[3];
    memcpy(dense + pos * c, feats + i * c, sizeof(float) * (size_t)c);
  }
}

/* bottom[i,:] = top[b,x,y,z,:].  Follows voxelize_cuda.cu:26-40. */
TSO_EXPORT void tso_to_dense_backward(const float *top, const int *coords, int64_t n, int c,
                                      const int *range, float *bottom) {
  for (int64_t i = 0; i < n; i++) {
    const int *q = coords + 4 * i;
    const int64_t pos = (((int64_t)q[0] * range[1] + q[1]) * range[2] + q[2]) * range[3] + q[3];
    memcpy(bottom + i * c, top + pos * c, sizeof(float) * (size_t)c);
  }
}
