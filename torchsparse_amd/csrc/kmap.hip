// Integer kernels of kernel-map construction for gfx950 and their C entry points.
//
// All kernels are HBM/L2-bound index work: one thread per produced element,
// 256-thread blocks, coalesced stores; the only random accesses are hash-table
// probes (see hashtable.h for how neighbouring coordinates share cache lines).
#include "common.h"
#include "hashtable.h"

namespace tsmi {
namespace {

constexpr int kBlock = 256;

struct Geom {
  int ks[3];
  int stride[3];
  int pad[3];
  int kvol;
  int odd;
};

__device__ __forceinline__ void decode_digits(int k, const Geom &g, int *d) {
  if (g.odd) {  // x is the fastest digit
    d[0] = k % g.ks[0];
    k /= g.ks[0];
    d[1] = k % g.ks[1];
    d[2] = k / g.ks[1];
  } else {  // z is the fastest digit
    d[2] = k % g.ks[2];
    k /= g.ks[2];
    d[1] = k % g.ks[1];
    d[0] = k / g.ks[1];
  }
}

template <typename T>
__global__ void fill_kernel(T *p, int64_t n, T v) {
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) p[i] = v;
}

// n4 int4 stores of one value (16-byte aligned p).
__global__ void fill_i32x4_kernel(int4 *p, int64_t n4, int32_t v) {
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n4) p[i] = make_int4(v, v, v, v);
}

__global__ void table_clear_kernel(unsigned long long *keys, int32_t *vals, int64_t cap) {
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < cap) {
    keys[i] = 0ULL;
    vals[i] = 0;
  }
}

__global__ void insert_coords_kernel(TableView t, const int4 *coords, int64_t n, int32_t *status) {
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  int4 c = coords[i];  // (b, x, y, z)
  if (!coords_packable(c.x, c.y, c.z, c.w)) {
    if (status) atomicOr(status, 2);  // a row the packed key cannot hold: the caller must not go on
    return;
  }
  bool fresh;
  uint32_t slot = table_insert<false>(t, pack_coords(c.x, c.y, c.z, c.w), &fresh);  // rows are distinct
  if (slot == 0xFFFFFFFFu) {
    if (status) atomicOr(status, 1);
    return;
  }
  t.vals[slot] = (int32_t)(i + 1);
}

// What a submanifold build needs before its insert pass, in one launch: an empty table and a
// map of -1.  Both are 16-byte stores; thread i takes the i-th int4 of each region it covers.
__global__ void subm_prepare_kernel(int4 *keys, int64_t keys4, int4 *vals, int64_t vals4, int4 *map,
                                    int64_t map4, int32_t *status) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i == 0 && status) *status = 0;
  if (i < keys4) keys[i] = make_int4(0, 0, 0, 0);
  if (i < vals4) vals[i] = make_int4(0, 0, 0, 0);
  if (i < map4) map[i] = make_int4(-1, -1, -1, -1);
}

__global__ void insert_keys_kernel(TableView t, const long long *user_keys, int64_t n,
                                   int32_t *status) {
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  bool fresh;
  uint32_t slot = table_insert(t, (unsigned long long)user_keys[i], &fresh);
  if (slot == 0xFFFFFFFFu) {
    if (status) *status = 1;
    return;
  }
  t.vals[slot] = (int32_t)(i + 1);
}

__global__ void lookup_keys_kernel(TableView t, const long long *user_keys, int64_t n,
                                   int32_t *out) {
  int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  uint32_t slot = table_find(t, (unsigned long long)user_keys[i]);
  out[i] = slot == 0xFFFFFFFFu ? 0 : t.vals[slot];
}

// One thread per (output row, kernel offset); a wave's 64 stores are contiguous.
__global__ void kmap_query_kernel(TableView t, const int4 *out_coords, int64_t n_out,
                                  int64_t total, Geom g, int32_t *map) {
  int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (tid >= total) return;
  int64_t row = tid / g.kvol;
  int k = (int)(tid - row * g.kvol);
  int32_t result = -1;
  if (row < n_out) {
    int4 c = out_coords[row];
    int d[3];
    decode_digits(k, g, d);
    int x = c.y * g.stride[0] - g.pad[0] + d[0];
    int y = c.z * g.stride[1] - g.pad[1] + d[1];
    int z = c.w * g.stride[2] - g.pad[2] + d[2];
    if (coords_packable(c.x, x, y, z)) {
      uint32_t slot = table_find(t, pack_coords(c.x, x, y, z));
      if (slot != 0xFFFFFFFFu) result = t.vals[slot] - 1;
    }
  }
  map[tid] = result;
}

// Submanifold map of a centred odd kernel at stride 1 over the table's own coordinates (row i
// was inserted with value i + 1).  map[i, k] = j  <=>  map[j, K_vol-1-k] = i, so only the first
// half of the offsets and the centre are probed; a hit also writes the mirrored entry.  The map
// must hold -1 everywhere before the launch.  One thread per (row, offset <= K_vol/2).
__global__ void kmap_query_subm_kernel(TableView t, const int4 *coords, int64_t n, int64_t total,
                                       Geom g, int32_t *map) {
  int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (tid >= total) return;
  const int half = g.kvol >> 1;
  int64_t row = tid / (half + 1);
  int k = (int)(tid - row * (half + 1));
  int4 c = coords[row];
  int d[3];
  decode_digits(k, g, d);
  int x = c.y - g.pad[0] + d[0];
  int y = c.z - g.pad[1] + d[1];
  int z = c.w - g.pad[2] + d[2];
  if (!coords_packable(c.x, x, y, z)) return;
  uint32_t slot = table_find(t, pack_coords(c.x, x, y, z));
  if (slot == 0xFFFFFFFFu) return;
  const int32_t j = t.vals[slot] - 1;
  map[row * g.kvol + k] = j;
  // a table that indexes other rows than `coords` must not send the mirrored store astray
  if (k != half && (uint64_t)j < (uint64_t)n) map[(int64_t)j * g.kvol + (g.kvol - 1 - k)] = (int32_t)row;
}

__global__ void coords_max_kernel(const int4 *coords, int64_t n, int32_t *out_max) {
  __shared__ int smax[kBlock / 64][4];
  // a bounded number of blocks strides over the rows: every block ends in atomics on the same
  // four words, which the memory side works off one after the other
  int v[4] = {0, 0, 0, 0};
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
    const int4 c = coords[i];
    v[0] = max(v[0], c.x);
    v[1] = max(v[1], c.y);
    v[2] = max(v[2], c.z);
    v[3] = max(v[3], c.w);
  }
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    int m = v[a];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = max(m, __shfl_xor(m, off));
    if ((threadIdx.x & 63) == 0) smax[threadIdx.x >> 6][a] = m;
  }
  __syncthreads();
  if (threadIdx.x < 4) {  // one atomic per block and column
    int m = max(max(smax[0][threadIdx.x], smax[1][threadIdx.x]),
                max(smax[2][threadIdx.x], smax[3][threadIdx.x]));
    // the maxima only grow: a stale read that is already large enough spares the atomic
    if (m > 0 && m > out_max[threadIdx.x]) atomicMax(&out_max[threadIdx.x], m);
  }
}

__host__ __device__ __forceinline__ int floor_div(int a, int b) {
  int q = a / b;
  return (a % b != 0 && ((a < 0) != (b < 0))) ? q - 1 : q;
}

// Output range of axis a: upper bound from the host or floor((max + 2 pad - (ks-1)) / stride)
// of the largest input coordinate; lower bound 0, or, when negative coordinates are allowed
// (in_min_dev given), (min - 2 pad + (ks-1)) / stride rounded toward zero.
__host__ __device__ __forceinline__ void output_range(const Geom &g, int a, int3 out_max_host,
                                             const int32_t *in_max_dev, const int32_t *in_min_dev,
                                             int *lo, int *hi) {
  *hi = in_max_dev ? floor_div(in_max_dev[1 + a] + 2 * g.pad[a] - (g.ks[a] - 1), g.stride[a])
                   : (a == 0 ? out_max_host.x : (a == 1 ? out_max_host.y : out_max_host.z));
  *lo = in_min_dev ? (in_min_dev[1 + a] - 2 * g.pad[a] + (g.ks[a] - 1)) / g.stride[a] : 0;
}

// Candidate j of the input coordinate c = (b, x, y, z) for modes 0, 1 and 2 (one candidate,
// j = 0, in modes 1 and 2) inside the output range [lo, hi] per axis (unused in mode 1); false
// when there is none.
// *unpackable (when given) is set if the candidate exists but the packed key cannot hold it.
__device__ __forceinline__ bool strided_candidate_in(int4 c, int j, const Geom &g, const int *lo,
                                                     const int *hi, int mode, int *b, int *o,
                                                     bool *unpackable = nullptr) {
  *b = c.x;
  const int v[3] = {c.y, c.z, c.w};
  if (mode != 0) {
    // one candidate per input: o = floor(in / stride).  mode 1 keeps it unbounded; mode 2
    // is the strided-convolution rule specialised to kernel size == stride, zero padding
    // (o*s <= in < o*s + k has exactly one solution), bounded like mode 0.
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      int q = v[a] / g.stride[a];
      if (v[a] % g.stride[a] != 0 && v[a] < 0) --q;
      o[a] = q;
      if (mode == 2 && (o[a] < lo[a] || o[a] > hi[a])) return false;
    }
  } else {
    // o = (in + pad + d - (ks-1)) / stride for the digits d in [0, ks) that make the division
    // exact: per axis d = r, r + stride, ... with r = (ks-1 - in - pad) mod stride, at most
    // ceil(ks / stride) of them; j numbers the combinations of such digits.
    const int f0 = (g.ks[0] + g.stride[0] - 1) / g.stride[0];
    const int f1 = (g.ks[1] + g.stride[1] - 1) / g.stride[1];
    const int jj[3] = {j % f0, (j / f0) % f1, j / (f0 * f1)};
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      int r = (g.ks[a] - 1 - v[a] - g.pad[a]) % g.stride[a];
      if (r < 0) r += g.stride[a];
      const int d = r + jj[a] * g.stride[a];
      if (d >= g.ks[a]) return false;
      o[a] = (v[a] + g.pad[a] + d - (g.ks[a] - 1)) / g.stride[a];  // exact
      if (o[a] < lo[a] || o[a] > hi[a]) return false;
    }
  }
  const bool ok = coords_packable(*b, o[0], o[1], o[2]);
  if (!ok && unpackable) *unpackable = true;
  return ok;
}

__device__ __forceinline__ void output_ranges(const Geom &g, int3 out_max_host, const int32_t *in_max_dev,
                                              const int32_t *in_min_dev, int mode, int *lo, int *hi) {
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    lo[a] = hi[a] = 0;
    if (mode != 1) output_range(g, a, out_max_host, in_max_dev, in_min_dev, &lo[a], &hi[a]);
  }
}

__device__ __forceinline__ bool strided_candidate(int4 c, int j, const Geom &g, int3 out_max_host,
                                                  const int32_t *in_max_dev, const int32_t *in_min_dev,
                                                  int mode, int *b, int *o, bool *unpackable = nullptr) {
  int lo[3], hi[3];
  output_ranges(g, out_max_host, in_max_dev, in_min_dev, mode, lo, hi);
  return strided_candidate_in(c, j, g, lo, hi, mode, b, o, unpackable);
}

__device__ __forceinline__ int strided_fan(const Geom &g) {
  return ((g.ks[0] + g.stride[0] - 1) / g.stride[0]) * ((g.ks[1] + g.stride[1] - 1) / g.stride[1]) *
         ((g.ks[2] + g.stride[2] - 1) / g.stride[2]);
}

// The candidate output coordinate of thread `tid`; false when the thread has none.
// mode 0: thread per (input, exactly dividing offset); modes 1 and 2: thread per input; mode 3 (generative
// upsampling): thread per (input, offset), o = clamp(in * stride + digit - (ks-1)/2, 0, max).
__device__ __forceinline__ bool downsample_candidate(int64_t tid, const int4 *in_coords, const Geom &g,
                                                     int3 out_max_host, const int32_t *in_max_dev,
                                                     const int32_t *in_min_dev, int mode, int *b,
                                                     int *o, bool *unpackable = nullptr) {
  if (mode == 3) {
    int64_t i = tid / g.kvol;
    int k = (int)(tid - i * g.kvol);
    int4 c = in_coords[i];
    *b = c.x;
    int d[3];
    decode_digits(k, g, d);
    int v[3] = {c.y, c.z, c.w};
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int hi = a == 0 ? out_max_host.x : (a == 1 ? out_max_host.y : out_max_host.z);
      o[a] = min(max(v[a] * g.stride[a] + d[a] - (g.ks[a] - 1) / 2, 0), hi);
    }
    const bool ok = coords_packable(*b, o[0], o[1], o[2]);
    if (unpackable && (!ok || !coords_packable(c.x, c.y, c.z, c.w))) *unpackable = true;
    return ok;
  }
  const int fan = mode == 0 ? strided_fan(g) : 1;
  const int64_t i = tid / fan;
  const int4 c = in_coords[i];
  // an input the packed key cannot hold is missing from every table built from these rows
  if (unpackable && !coords_packable(c.x, c.y, c.z, c.w)) *unpackable = true;
  return strided_candidate(c, (int)(tid - i * fan), g, out_max_host, in_max_dev, in_min_dev, mode, b, o,
                           unpackable);
}

__global__ void downsample_candidates_kernel(const int4 *in_coords, int64_t n_in, int64_t total,
                                             Geom g, int3 out_max_host, const int32_t *in_max_dev,
                                             const int32_t *in_min_dev, int mode, TableView t,
                                             int32_t *counters) {
  int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (tid >= total) return;
  int b, o[3];
  bool unpackable = false;
  const bool have = downsample_candidate(tid, in_coords, g, out_max_host, in_max_dev, in_min_dev, mode, &b,
                                         o, &unpackable);
  if (unpackable) counters[3] = 1;  // the caller must not go on: rows or outputs would be missing
  if (!have) return;
  bool fresh;
  if (table_insert(t, pack_coords(b, o[0], o[1], o[2]), &fresh) == 0xFFFFFFFFu) counters[1] = 1;
}

// ---- strided output coordinates through an occupancy bitmap -------------------------------
//
// When the output grid (batches x extents, known on the device from the largest input
// coordinate) has at most `cap_bits` cells, the distinct outputs in ascending (b, x, y, z) order
// are the set bits of a bitmap indexed by the mixed-radix cell number in ascending bit order: no
// hash insertion of the candidates, no compaction, no sort.  Four passes over the used part
// of the bitmap (mark, count per 512-word chunk, emit and clear) and a one-block scan of the
// chunk counts.
constexpr int kGridChunkWords = 512;  // 2 words per thread of a 256-thread block

struct GridDims {
  int e[3];            // extents of the three axes (largest output coordinate + 1)
  int64_t used_words;  // bitmap words that cover every cell, rounded up to whole chunks
  bool fits;
};

// Cell numbers stay below 2^30 (the largest bitmap), so everything after the fit test is
// 32-bit arithmetic.
__host__ __device__ __forceinline__ GridDims grid_dims(const Geom &g, int3 out_max_host, int has_host_max,
                                                       const int32_t *in_max_dev, int64_t cap_words) {
  GridDims d;
  int64_t cells = (int64_t)in_max_dev[0] + 1;
  bool ok = true;
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    int lo, hi;
    output_range(g, a, out_max_host, has_host_max ? nullptr : in_max_dev, nullptr, &lo, &hi);
    d.e[a] = hi + 1;
    if (hi < 0) ok = false;  // no output at all: nothing to mark
    // the product stays below 2^63: every factor is below 2^31 and the running product is
    // compared with the capacity (at most 2^30) before the next factor
    if (ok) cells *= d.e[a];
    if (cells > cap_words * 32) ok = false;
  }
  const bool empty = d.e[0] <= 0 || d.e[1] <= 0 || d.e[2] <= 0;
  d.fits = ok || empty;
  const uint32_t c = (ok && !empty) ? (uint32_t)cells : 0u;
  constexpr uint32_t kChunkCells = kGridChunkWords * 32;
  d.used_words = (int64_t)((c + kChunkCells - 1) / kChunkCells) * kGridChunkWords;  // power of two: shifts
  return d;
}

__global__ void grid_clear_kernel(uint4 *bitmap, int64_t cap_words, Geom g, int3 out_max_host,
                                  int has_host_max, const int32_t *in_max_dev) {
  const GridDims d = grid_dims(g, out_max_host, has_host_max, in_max_dev, cap_words);
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i * 4 < d.used_words) bitmap[i] = make_uint4(0u, 0u, 0u, 0u);
}

// Inputs usually arrive sorted, so the candidates of neighbouring lanes fall into the same
// bitmap word: lanes OR their bits into the last lane of each run of equal words and only
// that lane issues the atomic (any split of the runs is still right, only less thrifty).
// Per-column maximum of the block's (b, x, y, z), raised into out_max[4] (zero before the
// launch; threads without a coordinate pass zeros).  Every thread of the block must call it.
__device__ __forceinline__ void block_raise_max(int b, int x, int y, int z, int32_t *out_max) {
  __shared__ int wave_max[kBlock / 64][4];
  int v[4] = {b, x, y, z};
#pragma unroll
  for (int a = 0; a < 4; ++a) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v[a] = max(v[a], __shfl_xor(v[a], off));
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6][a] = v[a];
  }
  __syncthreads();
  if (threadIdx.x < 4) {
    const int m = max(max(wave_max[0][threadIdx.x], wave_max[1][threadIdx.x]),
                      max(wave_max[2][threadIdx.x], wave_max[3][threadIdx.x]));
    // the maxima only grow: a stale read that is already large enough spares the atomic
    if (m > 0 && m > out_max[threadIdx.x]) atomicMax(&out_max[threadIdx.x], m);
  }
}

__global__ void grid_mark_kernel(const int4 *in_coords, int64_t total, Geom g, int3 out_max_host,
                                 int has_host_max, const int32_t *in_max_dev, int mode,
                                 uint32_t *bitmap, int64_t cap_words, int32_t *next_in_max,
                                 int32_t *counters, const int32_t *n_in_dev) {
  const int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  // the rows may be the emit pass's output of the previous level of a chain, whose count has
  // not been read back: `total` is then the capacity and the count comes from the device
  if (n_in_dev) total = min(total, (int64_t)*n_in_dev * (mode == 0 ? strided_fan(g) : 1));
  const GridDims d = grid_dims(g, out_max_host, has_host_max, in_max_dev, cap_words);
  if (!d.fits || d.used_words == 0) return;  // the same for every thread
  int word = -1;
  uint32_t bits = 0;
  int b, o[3];
  bool unpackable = false;
  const bool have = tid < total &&
                    downsample_candidate(tid, in_coords, g, out_max_host,
                                         has_host_max ? nullptr : in_max_dev, nullptr, mode, &b, o,
                                         &unpackable) &&
                    b <= in_max_dev[0];
  if (unpackable) counters[3] = 1;
  if (have) {
    const uint32_t cell = (((uint32_t)b * d.e[0] + o[0]) * d.e[1] + o[1]) * d.e[2] + o[2];
    word = (int)(cell >> 5);
    bits = 1u << (cell & 31);
  }
  if (next_in_max) block_raise_max(have ? b : 0, have ? o[0] : 0, have ? o[1] : 0, have ? o[2] : 0, next_in_max);
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int w = __shfl_up(word, off);
    const uint32_t v = __shfl_up(bits, off);
    if (lane >= off && w == word) bits |= v;
  }
  const int next = __shfl_down(word, 1);
  if (word >= 0 && (lane == 63 || next != word)) {
    // bits are only ever set: a stale read of set bits is still right, a stale read of clear
    // bits only costs the atomic
    if ((bitmap[word] & bits) != bits) atomicOr(&bitmap[word], bits);
  }
}

// grid_mark_kernel for the strided-convolution rule (mode 0) with several candidates per
// input, one thread per INPUT: the outputs along each axis (at most kMaxFanAxis) are worked out
// once and the thread walks their combinations; candidates that share a bitmap word (neighbours
// along z, of the thread itself and of the other lanes of its wavefront) are merged before the
// pre-checked atomic, and the block raises the maxima once per input instead of once per
// candidate.  Marks exactly the bits grid_mark_kernel marks.
constexpr int kMaxFanAxis = 4;

__global__ __launch_bounds__(kBlock) void grid_mark_fan_kernel(
    const int4 *in_coords, int64_t n_in, Geom g, int3 out_max_host, int has_host_max,
    const int32_t *in_max_dev, uint32_t *bitmap, int64_t cap_words, int32_t *next_in_max,
    int32_t *counters) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const GridDims d = grid_dims(g, out_max_host, has_host_max, in_max_dev, cap_words);
  if (!d.fits || d.used_words == 0) return;  // the same for every thread
  int lo[3], hi[3];
  output_ranges(g, out_max_host, has_host_max ? nullptr : in_max_dev, nullptr, 0, lo, hi);
  int mb = 0, m0 = 0, m1 = 0, m2 = 0;
  bool unpackable = false;
  int4 c = make_int4(0, 0, 0, 0);
  int cnt[3] = {0, 0, 0};
  int ov[3][kMaxFanAxis];
  bool live = false;
  if (i < n_in) {
    c = in_coords[i];
    // an input the packed key cannot hold is missing from every table built from these rows
    if (!coords_packable(c.x, c.y, c.z, c.w)) unpackable = true;
    const int v[3] = {c.y, c.z, c.w};
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      // o = (in + pad + digit - (ks-1)) / stride for the digits that make the division exact
      int r = (g.ks[a] - 1 - v[a] - g.pad[a]) % g.stride[a];
      if (r < 0) r += g.stride[a];
#pragma unroll
      for (int j = 0; j < kMaxFanAxis; ++j) {
        const int digit = r + j * g.stride[a];
        if (digit >= g.ks[a]) break;
        const int o = (v[a] + g.pad[a] + digit - (g.ks[a] - 1)) / g.stride[a];  // exact
        if (o >= lo[a] && o <= hi[a]) ov[a][cnt[a]++] = o;
      }
    }
    live = c.x <= in_max_dev[0];
  }
  // Every lane walks the same (x, y) slots, so that the lanes of a wavefront - neighbours along
  // z where the inputs are sorted - can merge the words they mark: lanes OR their bits into the
  // last lane of each run of equal words and only that lane issues the pre-checked atomic.
  const int lane = threadIdx.x & 63;
  const int f0 = min(kMaxFanAxis, (g.ks[0] + g.stride[0] - 1) / g.stride[0]);
  const int f1 = min(kMaxFanAxis, (g.ks[1] + g.stride[1] - 1) / g.stride[1]);
  for (int i0 = 0; i0 < f0; ++i0) {
    for (int i1 = 0; i1 < f1; ++i1) {
      int word = -1;
      uint32_t bits = 0;
      if (live && i0 < cnt[0] && i1 < cnt[1]) {
        for (int i2 = 0; i2 < cnt[2]; ++i2) {
          const int o0 = ov[0][i0], o1 = ov[1][i1], o2 = ov[2][i2];
          if (!coords_packable(c.x, o0, o1, o2)) {
            unpackable = true;
            continue;
          }
          const uint32_t cell = (((uint32_t)c.x * d.e[0] + o0) * d.e[1] + o1) * d.e[2] + o2;
          const int w = (int)(cell >> 5);
          if (w != word) {
            // (the z run crosses into the next word: the earlier word goes out by itself)
            // bits are only ever set: a stale read of set bits is still right, a stale read
            // of clear bits only costs the atomic
            if (word >= 0 && (bitmap[word] & bits) != bits) atomicOr(&bitmap[word], bits);
            word = w;
            bits = 0;
          }
          bits |= 1u << (cell & 31);
          mb = max(mb, c.x);
          m0 = max(m0, o0);
          m1 = max(m1, o1);
          m2 = max(m2, o2);
        }
      }
      if (__ballot(word >= 0) == 0) continue;  // (the same for the whole wavefront)
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int w = __shfl_up(word, off);
        const uint32_t v = __shfl_up(bits, off);
        if (lane >= off && w == word) bits |= v;
      }
      const int next = __shfl_down(word, 1);
      if (word >= 0 && (lane == 63 || next != word) && (bitmap[word] & bits) != bits)
        atomicOr(&bitmap[word], bits);
    }
  }
  if (unpackable) counters[3] = 1;
  if (next_in_max) block_raise_max(mb, m0, m1, m2, next_in_max);
}

__device__ __forceinline__ int grid_thread_words(const uint32_t *bitmap, int64_t chunk, uint32_t *w);

// The same marking for the NEXT level of a chain of equal strided convolutions: its inputs are
// the set bits of the previous level's bitmap (prev_in_max: the maxima that bitmap's extents
// derive from; in_max: the maxima of its set bits, raised by the launch that marked it).
// A bounded number of blocks strides over the previous bitmap's chunks; like the emit kernel,
// a block keeps the chunk's words and the prefix of their bit counts in LDS and thread i takes
// the chunk's set bits i, i + 256, ... - a walk of each thread's own words would leave the
// threads over dense words with tens of divisions-heavy candidates and the rest with none.
__global__ __launch_bounds__(kBlock) void grid_mark_next_kernel(
    const uint32_t *prev_bitmap, int64_t prev_cap_words, const int32_t *prev_in_max, Geom g, int mode,
    const int32_t *in_max, uint32_t *bitmap, int64_t cap_words, int32_t *next_in_max) {
  __shared__ int wave_sum[kBlock / 64];
  __shared__ uint32_t words[kGridChunkWords];
  __shared__ int before[kGridChunkWords];
  const int3 none = make_int3(0, 0, 0);
  const GridDims pd = grid_dims(g, none, 0, prev_in_max, prev_cap_words);
  const GridDims d = grid_dims(g, none, 0, in_max, cap_words);
  if (!pd.fits || !d.fits || d.used_words == 0) return;  // the same for every thread
  const int fan = mode == 2 ? 1 : strided_fan(g);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t e0 = pd.e[0], e1 = pd.e[1], e2 = pd.e[2];
  int range_lo[3], range_hi[3];
  output_ranges(g, none, in_max, nullptr, mode, range_lo, range_hi);
  const int max_batch = in_max[0];
  int mb = 0, mx = 0, my = 0, mz = 0;
  const int64_t chunks = pd.used_words / kGridChunkWords;
  for (int64_t chunk = blockIdx.x; chunk < chunks; chunk += gridDim.x) {
    uint32_t w[2];
    const int mine = grid_thread_words(prev_bitmap, chunk, w);
    int incl = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int v = __shfl_up(incl, off);
      if (lane >= off) incl += v;
    }
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    int first = incl - mine;
    for (int v = 0; v < wave; ++v) first += wave_sum[v];
    words[threadIdx.x * 2] = w[0];
    words[threadIdx.x * 2 + 1] = w[1];
    before[threadIdx.x * 2] = first;
    before[threadIdx.x * 2 + 1] = first + __popc(w[0]);
    const int chunk_total = wave_sum[0] + wave_sum[1] + wave_sum[2] + wave_sum[3];
    __syncthreads();
    for (int i = threadIdx.x; i < chunk_total; i += kBlock) {
      int lo = 0;
#pragma unroll
      for (int step = kGridChunkWords / 2; step > 0; step >>= 1)
        if (before[lo + step] <= i) lo += step;
      uint32_t x = words[lo];
      int k = i - before[lo], pos = 0;
#pragma unroll
      for (int half = 16; half > 0; half >>= 1) {
        const int c = __popc(x & ((1u << half) - 1u));
        if (k >= c) {
          k -= c;
          x >>= half;
          pos += half;
        }
      }
      uint32_t cell = ((uint32_t)chunk * kGridChunkWords + lo) * 32 + pos;
      int4 c;
      c.w = (int)(cell % e2);
      cell /= e2;
      c.z = (int)(cell % e1);
      cell /= e1;
      c.y = (int)(cell % e0);
      c.x = (int)(cell / e0);
      for (int j = 0; j < fan; ++j) {
        int b, o[3];
        if (!strided_candidate_in(c, j, g, range_lo, range_hi, mode, &b, o) || b > max_batch) continue;
        const uint32_t out = (((uint32_t)b * d.e[0] + o[0]) * d.e[1] + o[1]) * d.e[2] + o[2];
        atomicOr(&bitmap[out >> 5], 1u << (out & 31));  // result unused: nothing waits for it
        mb = max(mb, b);
        mx = max(mx, o[0]);
        my = max(my, o[1]);
        mz = max(mz, o[2]);
      }
    }
    __syncthreads();  // the LDS arrays are rewritten by the next chunk
  }
  if (next_in_max) block_raise_max(mb, mx, my, mz, next_in_max);
}

__device__ __forceinline__ int grid_thread_words(const uint32_t *bitmap, int64_t chunk, uint32_t *w) {
  const uint2 v = *(const uint2 *)(bitmap + chunk * kGridChunkWords + threadIdx.x * 2);
  w[0] = v.x;
  w[1] = v.y;
  return __popc(v.x) + __popc(v.y);
}

// Set bits of every chunk -> chunk_counts; the blocks `first`, `first + step`, ... share the chunks.
__device__ __forceinline__ void grid_count_chunks(const uint32_t *bitmap, int64_t cap_words, const Geom &g,
                                                  int3 out_max_host, int has_host_max,
                                                  const int32_t *in_max_dev, int32_t *chunk_counts,
                                                  unsigned first, unsigned step) {
  // The extents live on the device, so the launch cannot be sized to the grid; a block that
  // only learns it has nothing to do still waits ~2 us for them, and thousands of such blocks
  // queue up behind each other.  A bounded number of blocks stride over the chunks instead.
  __shared__ int wave_sum[kBlock / 64];
  const GridDims d = grid_dims(g, out_max_host, has_host_max, in_max_dev, cap_words);
  const int64_t chunks = d.used_words / kGridChunkWords;
  for (int64_t chunk = first; chunk < chunks; chunk += step) {
    uint32_t w[2];
    int c = grid_thread_words(bitmap, chunk, w);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off);
    if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) chunk_counts[chunk] = wave_sum[0] + wave_sum[1] + wave_sum[2] + wave_sum[3];
    __syncthreads();
  }
}

__global__ __launch_bounds__(kBlock) void grid_count_kernel(const uint32_t *bitmap, int64_t cap_words,
                                                            Geom g, int3 out_max_host, int has_host_max,
                                                            const int32_t *in_max_dev,
                                                            int32_t *chunk_counts) {
  grid_count_chunks(bitmap, cap_words, g, out_max_host, has_host_max, in_max_dev, chunk_counts, blockIdx.x,
                    gridDim.x);
}

// One block: chunk_counts[0 .. used chunks) -> exclusive prefix in place, total -> counters[0].
__device__ __forceinline__ void grid_scan_chunks(int32_t *chunk_counts, int64_t cap_words, const Geom &g,
                                                 int3 out_max_host, int has_host_max,
                                                 const int32_t *in_max_dev, int32_t *counters) {
  __shared__ int wave_sum[16];
  const GridDims d = grid_dims(g, out_max_host, has_host_max, in_max_dev, cap_words);
  const int n = (int)(d.used_words / kGridChunkWords);
  const int per = (n + 1023) / 1024;
  const int first = threadIdx.x * per;
  int mine = 0;
  for (int i = first; i < min(first + per, n); ++i) mine += chunk_counts[i];
  int incl = mine;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int v = __shfl_up(incl, off);
    if (lane >= off) incl += v;
  }
  if (lane == 63) wave_sum[wave] = incl;
  __syncthreads();
  int base = 0;
  for (int w = 0; w < wave; ++w) base += wave_sum[w];
  int run = base + incl - mine;
  for (int i = first; i < min(first + per, n); ++i) {
    const int c = chunk_counts[i];
    chunk_counts[i] = run;
    run += c;
  }
  if (threadIdx.x == 1023) {
    counters[0] = base + incl;
    counters[2] = d.fits ? 0 : 1;
  }
}

__global__ __launch_bounds__(1024) void grid_scan_kernel(int32_t *chunk_counts, int64_t cap_words, Geom g,
                                                         int3 out_max_host, int has_host_max,
                                                         const int32_t *in_max_dev, int32_t *counters) {
  grid_scan_chunks(chunk_counts, cap_words, g, out_max_host, has_host_max, in_max_dev, counters);
}

// Set bits in ascending order -> out_coords rows; every word read is cleared again.
// Occupied cells cluster (surfaces): a few words of a chunk can hold most of its outputs, so
// the block does not walk bits word by word.  It keeps the chunk's words and the exclusive
// prefix of their bit counts in LDS, and thread i takes output rank i, i + 256, ...: a binary
// search of the prefix finds the word, five halvings find the bit.  The table entries
// (coordinate -> row + 1) are a separate launch of one thread per row.
__device__ __forceinline__ void grid_emit_chunks(uint32_t *bitmap, int64_t cap_words,
                                                 const int32_t *chunk_prefix, const Geom &g,
                                                 int3 out_max_host, int has_host_max,
                                                 const int32_t *in_max_dev, const GridDims &host_dims,
                                                 int have_host_dims, int4 *out_coords, int64_t n_out,
                                                 unsigned first_chunk, unsigned step) {
  __shared__ int wave_sum[kBlock / 64];
  __shared__ uint32_t words[kGridChunkWords];
  __shared__ int before[kGridChunkWords];  // set bits of the chunk before each word
  const GridDims d = have_host_dims ? host_dims
                                    : grid_dims(g, out_max_host, has_host_max, in_max_dev, cap_words);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // one block per chunk when the host knows the extents; otherwise a bounded number of blocks
  // strides over the chunks the device-side extents cover
  for (int64_t chunk = first_chunk; chunk * kGridChunkWords < d.used_words; chunk += step) {
  uint32_t w[2];
  const int mine = grid_thread_words(bitmap, chunk, w);
  if (mine)  // leave the bitmap all clear for the next call
    *(uint2 *)(bitmap + chunk * kGridChunkWords + threadIdx.x * 2) = make_uint2(0u, 0u);
  int incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int v = __shfl_up(incl, off);
    if (lane >= off) incl += v;
  }
  if (lane == 63) wave_sum[wave] = incl;
  __syncthreads();
  int first = incl - mine;
  for (int v = 0; v < wave; ++v) first += wave_sum[v];
  words[threadIdx.x * 2] = w[0];
  words[threadIdx.x * 2 + 1] = w[1];
  before[threadIdx.x * 2] = first;
  before[threadIdx.x * 2 + 1] = first + __popc(w[0]);
  const int chunk_total = wave_sum[0] + wave_sum[1] + wave_sum[2] + wave_sum[3];
  __syncthreads();
  const uint32_t chunk_cell0 = (uint32_t)chunk * (kGridChunkWords * 32);
  const int64_t chunk_rank0 = chunk_prefix[chunk];
  for (int i = threadIdx.x; i < chunk_total; i += kBlock) {
    // the last word with before[word] <= i holds rank i (an empty word shares its successor's count)
    int lo = 0;
#pragma unroll
    for (int step = kGridChunkWords / 2; step > 0; step >>= 1)
      if (before[lo + step] <= i) lo += step;
    uint32_t x = words[lo];
    int k = i - before[lo], pos = 0;
#pragma unroll
    for (int half = 16; half > 0; half >>= 1) {
      const int c = __popc(x & ((1u << half) - 1u));
      if (k >= c) {
        k -= c;
        x >>= half;
        pos += half;
      }
    }
    uint32_t cell = chunk_cell0 + lo * 32 + pos;
    const int z = (int)(cell % d.e[2]);
    cell /= d.e[2];
    const int y = (int)(cell % d.e[1]);
    cell /= d.e[1];
    const int x_ = (int)(cell % d.e[0]);
    const int b = (int)(cell / d.e[0]);
    // always true: n_out is the total of the counts the ranks come from (or the capacity of
    // out_coords when the total is still on the device)
    if (chunk_rank0 + i < n_out) out_coords[chunk_rank0 + i] = make_int4(b, x_, y, z);
  }
  __syncthreads();  // the LDS arrays are rewritten by the next chunk
  }
}

__global__ __launch_bounds__(kBlock) void grid_emit_kernel(uint32_t *bitmap, int64_t cap_words,
                                                           const int32_t *chunk_prefix, Geom g,
                                                           int3 out_max_host, int has_host_max,
                                                           const int32_t *in_max_dev, GridDims host_dims,
                                                           int have_host_dims, int4 *out_coords,
                                                           int64_t n_out) {
  grid_emit_chunks(bitmap, cap_words, chunk_prefix, g, out_max_host, has_host_max, in_max_dev, host_dims,
                   have_host_dims, out_coords, n_out, blockIdx.x, gridDim.x);
}

// ---- a chain of equal strided layers with one output per input, every level marked from the
// chain's ROOT rows.  Level l's cells are those of the root's rows carried down l + 1 layers, so
// the marks of level l need the maxima of its inputs (the extents of its grid, and which outputs
// the rule keeps) but not the rows of level l - 1: one launch per level marks it and raises the
// maxima of the next, and then ONE launch counts the chunks of every level, one scans them, one
// emits every level's rows.  levels + 3 launches (and tsmi_coords_max before them) where level
// after level takes 4 each.
constexpr int kChainMaxLevels = 8;
struct ChainLayout {
  int64_t bitmap_at[kChainMaxLevels];   // word of `scratch` where the level's bitmap starts
  int64_t words[kChainMaxLevels];       // ... and its capacity
  int64_t chunks_at[kChainMaxLevels];   // ... and where its chunk counts start
  unsigned first_block[kChainMaxLevels + 1];  // blocks of the counting / emitting launch per level
  int levels;
};

// One thread per root row: follow it down to `level` (dropped where the rule leaves a layer's
// output out: beyond floor((max - (ks - 1)) / stride) of that layer's inputs, or unpackable) and
// mark its cell there.  counters: 8 per level, [4..8) the maxima of the level's inputs - complete
// for the levels up to `level`, raised here for `level + 1`.
__global__ __launch_bounds__(kBlock) void chain_mark_kernel(const int4 *coords, int64_t n, Geom g, int level,
                                                            ChainLayout lay, int32_t *scratch,
                                                            int32_t *counters) {
  const int3 none = make_int3(0, 0, 0);
  GridDims d;
  for (int j = 0; j <= level; ++j) {  // (the same for every thread)
    d = grid_dims(g, none, 0, counters + 8 * j + 4, lay.words[j]);
    if (!d.fits || d.used_words == 0) return;  // a level without outputs leaves none to the later ones
  }
  const int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  bool have = tid < n;
  int4 c = have ? coords[tid] : make_int4(0, 0, 0, 0);
  // an input the packed key cannot hold is missing from every table built from these rows
  if (have && level == 0 && !coords_packable(c.x, c.y, c.z, c.w)) counters[3] = 1;
  for (int j = 0; j <= level && have; ++j) {
    const int32_t *in_max = counters + 8 * j + 4;
    int lo[3], hi[3], b, o[3];
    output_ranges(g, none, in_max, nullptr, 2, lo, hi);
    bool unpackable = false;
    have = strided_candidate_in(c, 0, g, lo, hi, 2, &b, o, &unpackable) && b <= in_max[0];
    if (unpackable && j == level) counters[8 * level + 3] = 1;
    c = make_int4(b, o[0], o[1], o[2]);
  }
  int word = -1;
  uint32_t bits = 0;
  if (have) {
    const uint32_t cell = (((uint32_t)c.x * d.e[0] + c.y) * d.e[1] + c.z) * d.e[2] + c.w;
    word = (int)(cell >> 5);
    bits = 1u << (cell & 31);
  }
  if (level + 1 < lay.levels)
    block_raise_max(have ? c.x : 0, have ? c.y : 0, have ? c.z : 0, have ? c.w : 0, counters + 8 * (level + 1) + 4);
  uint32_t *bitmap = (uint32_t *)scratch + lay.bitmap_at[level];
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int w = __shfl_up(word, off);
    const uint32_t v = __shfl_up(bits, off);
    if (lane >= off && w == word) bits |= v;
  }
  const int next = __shfl_down(word, 1);
  if (word >= 0 && (lane == 63 || next != word)) {
    if ((bitmap[word] & bits) != bits) atomicOr(&bitmap[word], bits);
  }
}

__device__ __forceinline__ int chain_level_of_block(const ChainLayout &lay, unsigned *first, unsigned *step) {
  int level = 0;
  while (level + 1 < lay.levels && blockIdx.x >= lay.first_block[level + 1]) ++level;
  *first = blockIdx.x - lay.first_block[level];
  *step = lay.first_block[level + 1] - lay.first_block[level];
  return level;
}

__global__ __launch_bounds__(kBlock) void chain_count_kernel(Geom g, ChainLayout lay, const int32_t *scratch,
                                                             int32_t *chunk_scratch, const int32_t *counters) {
  unsigned first, step;
  const int level = chain_level_of_block(lay, &first, &step);
  grid_count_chunks((const uint32_t *)scratch + lay.bitmap_at[level], lay.words[level], g, make_int3(0, 0, 0), 0,
                    counters + 8 * level + 4, chunk_scratch + lay.chunks_at[level], first, step);
}

__global__ __launch_bounds__(1024) void chain_scan_kernel(Geom g, ChainLayout lay, int32_t *scratch,
                                                          int32_t *counters) {
  const int level = blockIdx.x;
  grid_scan_chunks(scratch + lay.chunks_at[level], lay.words[level], g, make_int3(0, 0, 0), 0,
                   counters + 8 * level + 4, counters + 8 * level);
}

__global__ __launch_bounds__(kBlock) void chain_emit_kernel(Geom g, ChainLayout lay, int32_t *scratch,
                                                            const int32_t *counters, int4 *rows, int64_t n) {
  unsigned first, step;
  const int level = chain_level_of_block(lay, &first, &step);
  grid_emit_chunks((uint32_t *)scratch + lay.bitmap_at[level], lay.words[level], scratch + lay.chunks_at[level], g,
                   make_int3(0, 0, 0), 0, counters + 8 * level + 4, GridDims{}, 0, rows + (int64_t)level * n, n,
                   first, step);
}

// Occupied slots of a table, gathered in arbitrary order: one atomic per workgroup
// reserves the output range (a counter bumped once per wavefront or per key would
// serialise on its one address).
__global__ __launch_bounds__(kBlock) void compact_keys_kernel(const unsigned long long *keys,
                                                              int64_t cap, unsigned long long *out,
                                                              int32_t *count) {
  __shared__ int wave_base[kBlock / 64];
  __shared__ int block_base;
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const unsigned long long k = i < cap ? keys[i] : 0ULL;
  const unsigned long long b = __ballot(k != 0ULL);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) wave_base[wave] = __popcll(b);
  __syncthreads();
  if (threadIdx.x == 0) {
    int total = 0;
    for (int w = 0; w < kBlock / 64; ++w) {
      const int c = wave_base[w];
      wave_base[w] = total;
      total += c;
    }
    block_base = total ? atomicAdd(count, total) : 0;
  }
  __syncthreads();
  if (k != 0ULL)
    out[block_base + wave_base[wave] + __popcll(b & ((1ULL << lane) - 1ULL))] = k;
}

__global__ void downsample_finalize_kernel(const unsigned long long *sorted, int64_t n_out,
                                           TableView t, int4 *out_coords) {
  int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r >= n_out) return;
  unsigned long long key = sorted[r] - 1ULL;  // the table stores key + 1
  int c[4];
  unpack_coords(key, c);
  out_coords[r] = make_int4(c[0], c[1], c[2], c[3]);
  uint32_t slot = table_find(t, key);
  if (slot != 0xFFFFFFFFu) t.vals[slot] = (int32_t)(r + 1);
}

__global__ void transpose_map_kernel(const int32_t *map, int64_t total, int kvol, int32_t *map_t,
                                     int64_t n_rows_t) {
  int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (tid >= total) return;
  int32_t in = map[tid];
  if (in < 0 || in >= n_rows_t) return;
  int64_t out = tid / kvol;
  int k = (int)(tid - out * kvol);
  map_t[(int64_t)in * kvol + k] = (int32_t)out;
}


__global__ void reorder_map_kernel(const int32_t *map, const int32_t *loc, int64_t n_pad, int kvol,
                                   int len, int32_t *out) {
  int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (tid >= n_pad * kvol) return;
  int64_t r = tid / kvol;
  int c = (int)(tid - r * kvol);
  int32_t src = loc[(int64_t)(c / len) * n_pad + r];
  out[tid] = map[(int64_t)src * kvol + c];
}

__global__ void reduce_bitmask_kernel(const int32_t *mask, int split, int64_t n_pad, int tile,
                                      int64_t rows, int32_t *reduced) {
  int64_t tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (tid >= rows * split) return;
  int s = (int)(tid / rows);
  int64_t t = tid - (int64_t)s * rows;
  const int32_t *p = mask + (int64_t)s * n_pad;
  int64_t end = min((t + 1) * (int64_t)tile, n_pad);
  int32_t acc = 0;
  for (int64_t r = t * tile; r < end; ++r) acc |= p[r];
  reduced[tid] = acc;
}

// ---- pair lists: per-block counts, in-place scan, ordered fill ---------------

// Pair lists, shared structure of the kernels below: a block owns 256 consecutive map rows
// (one per thread) and walks the offsets in chunks of kPairChunk.  The chunk's part of the
// block's rows is staged in LDS with coalesced loads (for K_vol <= 32 the block's whole span
// of the map, contiguous) — a thread walking its own row straight from memory makes every
// wavefront load touch 54 cache lines, and with a few dozen wavefronts per CU those lines
// do not survive in the L1 until the next offset (measured: 340 GB/s of map).  Per offset a
// wavefront then ballots "row has an entry" out of LDS (row stride odd: no bank conflicts).
constexpr int kPairMaxKvol = 512;  // offsets the per-block start table holds
constexpr int kPairChunk = 32;     // offsets staged at a time
constexpr int kPairStride = kPairChunk + 1;

// tile[r * kPairStride + j] = map[row0 + r][k0 + j] for r < 256, j < kc (-1 past the end)
__device__ __forceinline__ void pair_stage_rows(const int32_t *map, int64_t row0, int64_t n_rows,
                                                int kvol, int k0, int kc, int32_t *tile) {
  const float inv = 1.0f / (float)kc;
  for (int idx = threadIdx.x; idx < kBlock * kc; idx += kBlock) {
    const int r = (int)(((float)idx + 0.5f) * inv);  // idx / kc, exact for idx < 2^20
    const int j = idx - r * kc;
    const int64_t row = row0 + r;
    tile[r * kPairStride + j] = row < n_rows ? map[row * kvol + k0 + j] : -1;
  }
}

// bitmask[s][r] bit i = row r has an entry at offset s*len + i (-1 for rows >= valid_n).  A
// block stages the split's offsets of its 256 rows through LDS like the pair-list kernels.
__global__ __launch_bounds__(kBlock) void derive_bitmask_kernel(const int32_t *map, int64_t n_pad,
                                                                int kvol, int split, int len,
                                                                int64_t valid_n, int32_t *bitmask) {
  __shared__ int32_t tile[kBlock * kPairStride];
  const int s = blockIdx.y;
  const int64_t row0 = (int64_t)blockIdx.x * kBlock, r = row0 + threadIdx.x;
  const int begin = s * len;
  const int l = min(len, kvol - begin);
  pair_stage_rows(map, row0, valid_n, kvol, begin, l, tile);
  __syncthreads();
  if (r >= n_pad) return;
  int32_t result = -1;
  if (r < valid_n) {
    uint32_t m = 0;
    for (int i = 0; i < l; ++i) m |= (uint32_t)(tile[threadIdx.x * kPairStride + i] >= 0) << i;
    result = (int32_t)m;
  }
  bitmask[(int64_t)s * n_pad + r] = result;
}

__global__ __launch_bounds__(kBlock) void pair_count_kernel(const int32_t *map, int64_t n_rows,
                                                            int kvol, int64_t nblk,
                                                            int32_t *block_counts) {
  __shared__ int32_t tile[kBlock * kPairStride];
  __shared__ int wave_cnt[kBlock / 64][kPairChunk];
  const int64_t row0 = (int64_t)blockIdx.x * kBlock;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int k0 = 0; k0 < kvol; k0 += kPairChunk) {
    const int kc = min(kPairChunk, kvol - k0);
    pair_stage_rows(map, row0, n_rows, kvol, k0, kc, tile);
    __syncthreads();
    int my = 0;  // lane j keeps the count of offset k0 + j
    for (int j = 0; j < kc; ++j) {
      const int c = __popcll(__ballot(tile[threadIdx.x * kPairStride + j] != -1));
      if (lane == j) my = c;
    }
    if (lane < kc) wave_cnt[wave][lane] = my;
    __syncthreads();
    if (threadIdx.x < kc)
      block_counts[(int64_t)(k0 + threadIdx.x) * nblk + blockIdx.x] =
          wave_cnt[0][threadIdx.x] + wave_cnt[1][threadIdx.x] + wave_cnt[2][threadIdx.x] +
          wave_cnt[3][threadIdx.x];
  }
}

// The pairs of every kernel offset, compacted into that offset's fixed segment, in one launch:
// in_rows[k * seg_rows + j] = map[row][k] of the j-th pair of offset k, pos[k * n_rows + row] = j
// (-1 where the row has no pair at k), counts[k] (zero on entry) = pairs of offset k.  A block
// reserves its share of each segment with one atomic add per offset, so the order of the blocks'
// shares inside a segment varies from launch to launch; pos names the place either way.
// KV > 0: the kernel volume, known at compile time: a thread keeps its row's entries in
// registers (one round trip to memory, no staging).  KV == 0: any volume, staged through LDS
// in chunks of kPairChunk offsets.
// `pool` (NULL, or kvol + 1 int32 that are zero on entry): the blocks then add up in the pool,
// and the block that finishes last moves the sums into `counts` and leaves the pool zero for
// the next launch, so that `counts` needs no clearing beforehand.
template <int KV>
__global__ __launch_bounds__(kBlock) void pair_segments_kernel(const int32_t *map, int64_t n_rows,
                                                               int kvol, int64_t seg_rows,
                                                               int32_t *pool, int32_t *counts,
                                                               int32_t *in_rows, int32_t *pos) {
  constexpr int kChunk = KV > 0 ? KV : kPairChunk;
  __shared__ int32_t tile[KV > 0 ? 1 : kBlock * kPairStride];
  __shared__ int wave_cnt[kBlock / 64][kChunk];
  __shared__ int wave_base[kBlock / 64][kChunk];
  const int64_t row0 = (int64_t)blockIdx.x * kBlock, row = row0 + threadIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const unsigned long long below = (1ULL << lane) - 1ULL;
  for (int k0 = 0; k0 < kvol; k0 += kChunk) {
    const int kc = KV > 0 ? KV : min(kChunk, kvol - k0);
    int32_t m[KV > 0 ? KV : 1];
    if (KV > 0) {
#pragma unroll
      for (int j = 0; j < KV; ++j) m[j] = row < n_rows ? map[row * KV + j] : -1;
    } else {
      __syncthreads();  // the previous chunk's tile and bases are no longer read
      pair_stage_rows(map, row0, n_rows, kvol, k0, kc, tile);
      __syncthreads();
    }
    auto entry = [&](int j) __attribute__((always_inline)) -> int32_t {
      return KV > 0 ? m[KV > 0 ? j : 0] : tile[threadIdx.x * kPairStride + j];
    };
#pragma unroll
    for (int j = 0; j < kChunk; ++j) {
      if (j >= kc) break;
      const int c = __popcll(__ballot(entry(j) >= 0));
      if (lane == 0) wave_cnt[wave][j] = c;
    }
    __syncthreads();
    if (threadIdx.x < kc) {
      const int t = threadIdx.x;
      const int a = wave_cnt[0][t], b = wave_cnt[1][t], c = wave_cnt[2][t], d = wave_cnt[3][t];
      const int total = a + b + c + d;
      const int base = total > 0 ? atomicAdd(&(pool ? pool : counts)[k0 + t], total) : 0;
      wave_base[0][t] = base;
      wave_base[1][t] = base + a;
      wave_base[2][t] = base + a + b;
      wave_base[3][t] = base + a + b + c;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kChunk; ++j) {
      if (j >= kc) break;
      const int32_t v = entry(j);
      const unsigned long long b = __ballot(v >= 0);
      const int rank = wave_base[wave][j] + __popcll(b & below);
      if (v >= 0) in_rows[(int64_t)(k0 + j) * seg_rows + rank] = v;
      if (row < n_rows) pos[(int64_t)(k0 + j) * n_rows + row] = v >= 0 ? rank : -1;
    }
  }
  if (pool) {
    __shared__ int last;
    __syncthreads();  // this block's adds are issued
    if (threadIdx.x == 0) {
      __threadfence();
      last = atomicAdd(&pool[kvol], 1) == (int)gridDim.x - 1;
    }
    __syncthreads();
    if (last) {  // every other block's adds precede its ticket: the sums are complete
      for (int k = threadIdx.x; k < kvol; k += kBlock) counts[k] = atomicExch(&pool[k], 0);
      if (threadIdx.x == 0) atomicExch(&pool[kvol], 0);
    }
  }
}

// Block k: exclusive scan of offset k's per-block counts in place (positions relative to the
// start of the offset's list); nbsizes[k] = their sum.
__global__ __launch_bounds__(1024) void pair_scan_kernel(int32_t *counts, int kvol, int64_t nblk,
                                                         int32_t *nbsizes) {
  __shared__ int part[1024];
  const int t = threadIdx.x;
  int32_t *mine = counts + (int64_t)blockIdx.x * nblk;
  const int64_t chunk = (nblk + 1023) / 1024;
  const int64_t begin = min((int64_t)t * chunk, nblk), end = min(begin + chunk, nblk);
  int sum = 0;
  for (int64_t i = begin; i < end; ++i) sum += mine[i];
  part[t] = sum;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {  // Hillis-Steele inclusive scan of the partial sums
    const int v = t >= off ? part[t - off] : 0;
    __syncthreads();
    part[t] += v;
    __syncthreads();
  }
  int run = part[t] - sum;
  for (int64_t i = begin; i < end; ++i) {
    const int c = mine[i];
    mine[i] = run;
    run += c;
  }
  if (t == 1023) nbsizes[blockIdx.x] = part[t];
}

// start[k] = first position of offset k's list: the sum of the earlier offsets' sizes, each
// rounded up to a multiple of `quantum` entries first.
__device__ __forceinline__ void pair_list_starts(const int32_t *nbsizes, int kvol, int quantum,
                                                 int *start) {
  for (int k = threadIdx.x; k < kvol; k += kBlock) start[k + 1] = nbsizes[k];
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int k = 0; k < kvol; ++k) {
      const int c = start[k + 1];
      start[k] = run;
      run += (c + quantum - 1) / quantum * quantum;
    }
    start[kvol] = run;
  }
  __syncthreads();
}

// Rank of every entry of the staged chunk inside its (block, offset) run, by two ballot
// passes around one barrier; `emit(k, value, row, position inside the offset's list)` is
// called for every entry.
template <typename Emit>
__device__ __forceinline__ void pair_for_each(const int32_t *map, int64_t n_rows, int kvol,
                                              int64_t nblk, const int32_t *offsets, int32_t *tile,
                                              int (*wave_cnt)[kPairChunk], Emit emit) {
  const int64_t row0 = (int64_t)blockIdx.x * kBlock;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int k0 = 0; k0 < kvol; k0 += kPairChunk) {
    const int kc = min(kPairChunk, kvol - k0);
    __syncthreads();  // the previous chunk's tile and counts are no longer read
    pair_stage_rows(map, row0, n_rows, kvol, k0, kc, tile);
    __syncthreads();
    int my = 0;
    for (int j = 0; j < kc; ++j) {
      const int c = __popcll(__ballot(tile[threadIdx.x * kPairStride + j] != -1));
      if (lane == j) my = c;
    }
    if (lane < kc) wave_cnt[wave][lane] = my;
    __syncthreads();
    for (int j = 0; j < kc; ++j) {
      const int32_t v = tile[threadIdx.x * kPairStride + j];
      const unsigned long long b = __ballot(v != -1);
      if (v == -1) continue;
      int before = 0;
      for (int w = 0; w < wave; ++w) before += wave_cnt[w][j];
      const int in_list = offsets[(int64_t)(k0 + j) * nblk + blockIdx.x] + before +
                          __popcll(b & ((1ULL << lane) - 1ULL));
      emit(k0 + j, v, (int32_t)(row0 + threadIdx.x), in_list);
    }
  }
}

__global__ __launch_bounds__(kBlock) void pair_fill_kernel(
    const int32_t *map, int64_t n_rows, int kvol, int64_t nblk, const int32_t *offsets,
    const int32_t *nbsizes, int64_t nnz, int32_t *inter, int32_t *planar, int64_t n_in, int64_t n_out,
    int32_t *input_mask, int32_t *output_mask, int skip_k) {
  __shared__ int32_t tile[kBlock * kPairStride];
  __shared__ int wave_cnt[kBlock / 64][kPairChunk];
  __shared__ int start[kPairMaxKvol + 1];
  pair_list_starts(nbsizes, kvol, 1, start);
  pair_for_each(map, n_rows, kvol, nblk, offsets, tile, wave_cnt,
                [&](int k, int32_t in, int32_t row, int in_list) {
                  const int64_t pos = (int64_t)start[k] + in_list;
                  if (pos >= nnz) return;
                  if (inter) {
                    inter[2 * pos] = in;
                    inter[2 * pos + 1] = row;
                  }
                  if (planar) {
                    planar[pos] = in;
                    planar[nnz + pos] = row;
                  }
                  if (k != skip_k) {
                    if (input_mask && in >= 0 && in < n_in) input_mask[(int64_t)k * n_in + in] = in_list;
                    if (output_mask && row < n_out) output_mask[(int64_t)k * n_out + row] = in_list;
                  }
                });
}

// Pair lists for the weight gradient: offset k's pairs (map value, row), ordered by row,
// start at entry seg_steps[k] * kWgradPairStep and are padded with (-1, -1) up to the next
// multiple of kWgradPairStep, so that a block of kWgradPairStep consecutive entries never
// mixes two offsets.  `offsets` holds each block's first position inside its offset's list.
__global__ __launch_bounds__(kBlock) void wgrad_pair_fill_kernel(
    const int32_t *map, int64_t n_rows, int kvol, int64_t nblk, const int32_t *offsets,
    const int32_t *nbsizes, int32_t *pairs, int32_t *seg_steps) {
  __shared__ int32_t tile[kBlock * kPairStride];
  __shared__ int wave_cnt[kBlock / 64][kPairChunk];
  __shared__ int start[kPairMaxKvol + 1];
  pair_list_starts(nbsizes, kvol, kWgradPairStep, start);
  if (blockIdx.x == 0) {
    for (int k = threadIdx.x; k <= kvol; k += kBlock) seg_steps[k] = start[k] / kWgradPairStep;
    // the padding entries behind each list
    for (int k = 0; k < kvol; ++k) {
      const int64_t pos = (int64_t)start[k] + nbsizes[k] + threadIdx.x;
      if (pos < start[k + 1]) {
        pairs[2 * pos] = -1;
        pairs[2 * pos + 1] = -1;
      }
    }
  }
  pair_for_each(map, n_rows, kvol, nblk, offsets, tile, wave_cnt,
                [&](int k, int32_t v, int32_t row, int in_list) {
                  const int64_t pos = (int64_t)start[k] + in_list;
                  pairs[2 * pos] = v;
                  pairs[2 * pos + 1] = row;
                });
}

// Padded copy of existing interleaved pair lists (offset k's nbsizes[k] pairs follow each
// other without gaps): the layout wgrad_pair_fill_kernel writes.  One thread per entry of
// the padded array; `limit` bounds the entries a launch may touch.
__global__ void wgrad_pair_pad_kernel(const int32_t *nbmaps, int64_t nnz, const int32_t *nbsizes,
                                      int kvol, int64_t limit, int32_t *pairs,
                                      int32_t *seg_steps) {
  __shared__ int seg[kWgradMaxKvol + 1];   // padded start of each list, in steps
  __shared__ int src[kWgradMaxKvol + 1];   // start of each list in nbmaps
  for (int k = threadIdx.x; k < kvol; k += kBlock) seg[k + 1] = nbsizes[k];
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0, raw = 0;
    for (int k = 0; k < kvol; ++k) {
      const int c = seg[k + 1];
      seg[k] = run;
      src[k] = raw;
      run += (c + kWgradPairStep - 1) / kWgradPairStep;
      raw += c;
    }
    seg[kvol] = run;
    src[kvol] = raw;
  }
  __syncthreads();
  if (blockIdx.x == 0)
    for (int k = threadIdx.x; k <= kvol; k += kBlock) seg_steps[k] = seg[k];
  const int64_t pos = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (pos >= limit || pos >= (int64_t)seg[kvol] * kWgradPairStep) return;
  const int step = (int)(pos / kWgradPairStep);
  int lo = 0, hi = kvol;  // largest k with seg[k] <= step
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (seg[mid] <= step) lo = mid; else hi = mid;
  }
  const int64_t j = pos - (int64_t)seg[lo] * kWgradPairStep;
  int32_t a = -1, b = -1;
  if (j < src[lo + 1] - src[lo] && src[lo] + j < nnz) {
    a = nbmaps[2 * (src[lo] + j)];
    b = nbmaps[2 * (src[lo] + j) + 1];
  }
  pairs[2 * pos] = a;
  pairs[2 * pos + 1] = b;
}

// One thread per pair: offset by binary search over the exclusive scan, position
// inside the offset's list by subtraction.
__global__ void masks_from_pairs_kernel(const int32_t *pairs, int64_t nnz, const int32_t *nbaddrs,
                                        int kvol, int64_t n_in, int64_t n_out, int skip_k,
                                        int32_t *input_mask, int32_t *output_mask) {
  int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= nnz) return;
  int lo = 0, hi = kvol;  // largest k with nbaddrs[k] <= p
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if ((int64_t)nbaddrs[mid] <= p) lo = mid; else hi = mid;
  }
  if (lo == skip_k) return;
  int32_t pos = (int32_t)(p - nbaddrs[lo]);
  int32_t in = pairs[2 * p], out = pairs[2 * p + 1];
  if (in >= 0 && in < n_in) input_mask[(int64_t)lo * n_in + in] = pos;
  if (out >= 0 && out < n_out) output_mask[(int64_t)lo * n_out + out] = pos;
}

__global__ void scan_quantified_kernel(int kvol, const int32_t *nbsizes, int q, int32_t *nbaddrs,
                                       int32_t *qnbaddrs) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int acc = 0, qacc = 0;
  nbaddrs[0] = 0;
  qnbaddrs[0] = 0;
  for (int k = 0; k < kvol; ++k) {
    acc += nbsizes[k];
    qacc += (nbsizes[k] + q - 1) / q * q;
    nbaddrs[k + 1] = acc;
    qnbaddrs[k + 1] = qacc;
  }
}

#include "kmap_sorted.inc"

int make_table(TableView *t, const int64_t *keys, const int32_t *vals, int64_t cap) {
  TSMI_REQUIRE(keys != nullptr && vals != nullptr, "hash table: null keys/vals");
  TSMI_REQUIRE(cap >= 8 && cap % 8 == 0 && cap < (int64_t(1) << 31),
               "hash table: capacity %lld must be a multiple of 8 in [8, 2^31)", (long long)cap);
  t->keys = (unsigned long long *)keys;
  t->vals = (int32_t *)vals;
  t->cap = (uint32_t)cap;
  t->groups = (uint32_t)(cap / 4);
  return TSMI_OK;
}

int make_geom(Geom *g, const int32_t ks[3], const int32_t stride[3], const int32_t pad[3]) {
  TSMI_REQUIRE(ks && stride && pad, "kernel geometry: null pointer");
  int64_t kvol = 1;
  for (int a = 0; a < 3; ++a) {
    TSMI_REQUIRE(ks[a] >= 1 && stride[a] >= 1, "kernel geometry: kernel size and stride must be >= 1");
    g->ks[a] = ks[a];
    g->stride[a] = stride[a];
    g->pad[a] = pad[a];
    kvol *= ks[a];
  }
  TSMI_REQUIRE(kvol <= 4096, "kernel volume %lld too large", (long long)kvol);
  g->kvol = (int)kvol;
  g->odd = kvol % 2 == 1;
  return TSMI_OK;
}

inline dim3 grid_for(int64_t n) { return dim3((unsigned)ceil_div(n > 0 ? n : 1, kBlock)); }

}  // namespace
}  // namespace tsmi

using namespace tsmi;

#define TSMI_GRID_CHECK(n) \
  TSMI_REQUIRE(grid_fits(ceil_div((n), kBlock)), "problem too large for one launch (%lld elements)", (long long)(n))

extern "C" int tsmi_hashtable_clear(tsmi_stream_t s, int64_t *keys, int32_t *vals, int64_t cap) {
  TableView t;
  if (int e = make_table(&t, keys, vals, cap)) return e;
  hipLaunchKernelGGL(table_clear_kernel, grid_for(cap), dim3(kBlock), 0, (hipStream_t)s, t.keys,
                     t.vals, cap);
  return check_launch("tsmi_hashtable_clear");
}

extern "C" int tsmi_hashtable_insert_coords(tsmi_stream_t s, int64_t *keys, int32_t *vals,
                                            int64_t cap, const int32_t *coords, int64_t n,
                                            int32_t *status) {
  TableView t;
  if (int e = make_table(&t, keys, vals, cap)) return e;
  TSMI_REQUIRE(n >= 0 && (n == 0 || coords), "insert_coords: bad coords");
  TSMI_REQUIRE(n <= cap, "The capacity of hashtable is not sufficient (%lld keys, capacity %lld)",
               (long long)n, (long long)cap);
  if (n == 0) return TSMI_OK;
  TSMI_GRID_CHECK(n);
  hipLaunchKernelGGL(insert_coords_kernel, grid_for(n), dim3(kBlock), 0, (hipStream_t)s, t,
                     (const int4 *)coords, n, status);
  return check_launch("tsmi_hashtable_insert_coords");
}

extern "C" int tsmi_hashtable_insert_keys(tsmi_stream_t s, int64_t *keys, int32_t *vals,
                                          int64_t cap, const int64_t *user_keys, int64_t n,
                                          int32_t *status) {
  TableView t;
  if (int e = make_table(&t, keys, vals, cap)) return e;
  TSMI_REQUIRE(n >= 0 && (n == 0 || user_keys), "insert_keys: bad keys");
  TSMI_REQUIRE(n <= cap, "The capacity of hashtable is not sufficient (%lld keys, capacity %lld)",
               (long long)n, (long long)cap);
  if (n == 0) return TSMI_OK;
  TSMI_GRID_CHECK(n);
  hipLaunchKernelGGL(insert_keys_kernel, grid_for(n), dim3(kBlock), 0, (hipStream_t)s, t,
                     (const long long *)user_keys, n, status);
  return check_launch("tsmi_hashtable_insert_keys");
}

extern "C" int tsmi_hashtable_lookup_keys(tsmi_stream_t s, const int64_t *keys,
                                          const int32_t *vals, int64_t cap,
                                          const int64_t *user_keys, int64_t n, int32_t *out) {
  TableView t;
  if (int e = make_table(&t, keys, vals, cap)) return e;
  TSMI_REQUIRE(n >= 0 && (n == 0 || (user_keys && out)), "lookup_keys: bad arguments");
  if (n == 0) return TSMI_OK;
  TSMI_GRID_CHECK(n);
  hipLaunchKernelGGL(lookup_keys_kernel, grid_for(n), dim3(kBlock), 0, (hipStream_t)s, t,
                     (const long long *)user_keys, n, out);
  return check_launch("tsmi_hashtable_lookup_keys");
}

extern "C" int tsmi_kmap_query(tsmi_stream_t s, const int64_t *keys, const int32_t *vals,
                               int64_t cap, const int32_t *out_coords, int64_t n_out,
                               int64_t n_out_pad, const int32_t ks[3], const int32_t stride[3],
                               const int32_t pad[3], int32_t *out_in_map) {
  TableView t;
  Geom g;
  if (int e = make_table(&t, keys, vals, cap)) return e;
  if (int e = make_geom(&g, ks, stride, pad)) return e;
  TSMI_REQUIRE(n_out >= 0 && n_out_pad >= n_out, "kmap_query: n_out_pad < n_out");
  TSMI_REQUIRE(n_out == 0 || out_coords, "kmap_query: null out_coords");
  int64_t total = n_out_pad * g.kvol;
  if (total == 0) return TSMI_OK;
  TSMI_REQUIRE(out_in_map, "kmap_query: null out_in_map");
  TSMI_GRID_CHECK(total);
  hipLaunchKernelGGL(kmap_query_kernel, grid_for(total), dim3(kBlock), 0, (hipStream_t)s, t,
                     (const int4 *)out_coords, n_out, total, g, out_in_map);
  return check_launch("tsmi_kmap_query");
}

extern "C" int tsmi_kmap_query_subm(tsmi_stream_t s, const int64_t *keys, const int32_t *vals,
                                    int64_t cap, const int32_t *coords, int64_t n, int64_t n_pad,
                                    const int32_t ks[3], int32_t *out_in_map) {
  TableView t;
  Geom g;
  if (int e = make_table(&t, keys, vals, cap)) return e;
  TSMI_REQUIRE(ks && ks[0] % 2 == 1 && ks[1] % 2 == 1 && ks[2] % 2 == 1,
               "kmap_query_subm: every kernel size must be odd");
  const int32_t one[3] = {1, 1, 1};
  const int32_t pad[3] = {(ks[0] - 1) / 2, (ks[1] - 1) / 2, (ks[2] - 1) / 2};
  if (int e = make_geom(&g, ks, one, pad)) return e;
  TSMI_REQUIRE(n >= 0 && n_pad >= n, "kmap_query_subm: n_pad < n");
  TSMI_REQUIRE(n == 0 || coords, "kmap_query_subm: null coords");
  TSMI_REQUIRE(n <= cap, "kmap_query_subm: more rows than table slots");
  const int64_t cells = n_pad * g.kvol;
  if (cells == 0) return TSMI_OK;
  TSMI_REQUIRE(out_in_map, "kmap_query_subm: null out_in_map");
  TSMI_GRID_CHECK(cells);
  if (cells % 4 == 0 && (uintptr_t)out_in_map % 16 == 0)
    hipLaunchKernelGGL(fill_i32x4_kernel, grid_for(cells / 4), dim3(kBlock), 0, (hipStream_t)s,
                       (int4 *)out_in_map, cells / 4, -1);
  else
    hipLaunchKernelGGL(fill_kernel<int32_t>, grid_for(cells), dim3(kBlock), 0, (hipStream_t)s,
                       out_in_map, cells, -1);
  const int64_t total = n * (g.kvol / 2 + 1);
  if (total > 0)
    hipLaunchKernelGGL(kmap_query_subm_kernel, grid_for(total), dim3(kBlock), 0, (hipStream_t)s, t,
                       (const int4 *)coords, n, total, g, out_in_map);
  return check_launch("tsmi_kmap_query_subm");
}

extern "C" int tsmi_kmap_build_subm(tsmi_stream_t s, int64_t *keys, int32_t *vals, int64_t cap,
                                    const int32_t *coords, int64_t n, int64_t n_pad,
                                    const int32_t ks[3], int32_t *out_in_map, int32_t *status) {
  TableView t;
  Geom g;
  if (int e = make_table(&t, keys, vals, cap)) return e;
  TSMI_REQUIRE(ks && ks[0] >= 1 && ks[1] >= 1 && ks[2] >= 1, "kmap_build_subm: bad kernel size");
  const bool odd = ks[0] % 2 == 1 && ks[1] % 2 == 1 && ks[2] % 2 == 1;
  const bool odd_volume = ((int64_t)ks[0] * ks[1] * ks[2]) % 2 == 1;
  const int32_t one[3] = {1, 1, 1};
  const int32_t pad[3] = {odd_volume ? (ks[0] - 1) / 2 : 0, odd_volume ? (ks[1] - 1) / 2 : 0,
                          odd_volume ? (ks[2] - 1) / 2 : 0};
  if (int e = make_geom(&g, ks, one, pad)) return e;
  TSMI_REQUIRE(n >= 0 && n_pad >= n, "kmap_build_subm: n_pad < n");
  TSMI_REQUIRE(n == 0 || coords, "kmap_build_subm: null coords");
  TSMI_REQUIRE(n <= cap, "The capacity of hashtable is not sufficient (%lld keys, capacity %lld)",
               (long long)n, (long long)cap);
  const int64_t cells = n_pad * g.kvol;
  TSMI_REQUIRE(cells == 0 || out_in_map, "kmap_build_subm: null out_in_map");
  TSMI_REQUIRE((uintptr_t)keys % 16 == 0 && (uintptr_t)vals % 16 == 0 && (uintptr_t)out_in_map % 16 == 0,
               "kmap_build_subm: table and map must be 16-byte aligned");
  // capacity is a multiple of 8 and n_pad * kvol a multiple of 4 (n_pad is a multiple of 128
  // in every caller; any other n_pad takes the scalar fill below)
  const bool vec_map = cells % 4 == 0;
  const int64_t keys4 = cap / 2, vals4 = cap / 4, map4 = (odd && vec_map) ? cells / 4 : 0;
  const int64_t prep = std::max(keys4, std::max(vals4, map4));
  TSMI_GRID_CHECK(std::max(prep, cells));
  hipLaunchKernelGGL(subm_prepare_kernel, grid_for(prep), dim3(kBlock), 0, (hipStream_t)s, (int4 *)keys,
                     keys4, (int4 *)vals, vals4, (int4 *)out_in_map, map4, status);
  if (odd && !vec_map && cells > 0)
    hipLaunchKernelGGL(fill_kernel<int32_t>, grid_for(cells), dim3(kBlock), 0, (hipStream_t)s,
                       out_in_map, cells, -1);
  if (n > 0)
    hipLaunchKernelGGL(insert_coords_kernel, grid_for(n), dim3(kBlock), 0, (hipStream_t)s, t,
                       (const int4 *)coords, n, status);
  if (odd) {
    const int64_t total = n * (g.kvol / 2 + 1);
    if (total > 0)
      hipLaunchKernelGGL(kmap_query_subm_kernel, grid_for(total), dim3(kBlock), 0, (hipStream_t)s, t,
                         (const int4 *)coords, n, total, g, out_in_map);
  } else if (cells > 0) {
    hipLaunchKernelGGL(kmap_query_kernel, grid_for(cells), dim3(kBlock), 0, (hipStream_t)s, t,
                       (const int4 *)coords, n, cells, g, out_in_map);
  }
  return check_launch("tsmi_kmap_build_subm");
}

extern "C" int tsmi_coords_check(tsmi_stream_t s, const int32_t *coords, int64_t n, int32_t *flags) {
  TSMI_REQUIRE(flags && n >= 0 && (n == 0 || coords), "coords_check: bad arguments");
  if (n == 0) return TSMI_OK;
  TSMI_GRID_CHECK(n);
  hipLaunchKernelGGL(coords_check_kernel, grid_for(n), dim3(kBlock), 0, (hipStream_t)s,
                     (const int4 *)coords, n, flags);
  return check_launch("tsmi_coords_check");
}

extern "C" int tsmi_kmap_sorted_supported(const int32_t ks[3]) {
  if (!ks || ks[0] < 1 || ks[1] < 1 || ks[2] < 1) return 0;
  const int64_t kvol = (int64_t)ks[0] * ks[1] * ks[2];
  return ks[0] <= kSortedMaxKs0 && ks[1] <= kSortedMaxKs1 && kvol <= kSortedTileInts;
}

extern "C" int64_t tsmi_kmap_sorted_samples_elems(int64_t n_in) {
  if (n_in <= (int64_t)kSortedSamples * kSortedDirect || n_in >= (int64_t(1) << 31)) return 0;
  return (int64_t)kSortedSamples * (1 + kSortedCell);
}

extern "C" int tsmi_kmap_sorted_samples(tsmi_stream_t s, const int32_t *in_coords, int64_t n_in,
                                        int64_t *samples) {
  TSMI_REQUIRE(tsmi_kmap_sorted_samples_elems(n_in) > 0, "kmap_sorted_samples: inputs of this size need none");
  TSMI_REQUIRE(in_coords && samples, "kmap_sorted_samples: null pointer");
  const int n = (int)n_in;
  const int sa = (n + kSortedSamples - 1) / kSortedSamples, n_a = (n + sa - 1) / sa;
  const int sb = (sa + kSortedCell - 1) / kSortedCell;
  hipLaunchKernelGGL(kmap_sorted_samples_kernel, grid_for((int64_t)n_a * kSortedCell), dim3(kBlock), 0,
                     (hipStream_t)s, (const int4 *)in_coords, n, sa, sb, n_a,
                     (unsigned long long *)samples, (unsigned long long *)samples + kSortedSamples);
  return check_launch("tsmi_kmap_sorted_samples");
}

// Checks the operands of one sorted-map build and fills its kernel arguments.  *cube: the
// compile-time kernel size that serves it (2, 3) or 0; *blocks: its workgroups (0: nothing to do).
static int sorted_args(SortedArgs *a, int *cube, int64_t *blocks, const int32_t *in_coords, int64_t n_in,
                       const int32_t *out_coords, int64_t n_out, int64_t n_out_pad, const int32_t ks[3],
                       const int32_t stride[3], const int32_t pad[3], const int64_t *samples,
                       int32_t *out_in_map, int32_t *map_t, int64_t n_t_pad, int64_t *pair_words,
                       int64_t *pair_out, const int32_t *n_in_dev = nullptr, const int32_t *n_out_dev = nullptr) {
  if (int e = make_geom(&a->g, ks, stride, pad)) return e;
  TSMI_REQUIRE(tsmi_kmap_sorted_supported(ks), "kmap_sorted: kernel size (%d, %d, %d) not supported",
               ks[0], ks[1], ks[2]);
  TSMI_REQUIRE(n_in >= 0 && n_in < (int64_t(1) << 31) && (n_in == 0 || in_coords), "kmap_sorted: bad in_coords");
  TSMI_REQUIRE(n_out >= 0 && n_out_pad >= n_out && n_out_pad < (int64_t(1) << 31),
               "kmap_sorted: n_out_pad < n_out");
  TSMI_REQUIRE(n_out == 0 || out_coords, "kmap_sorted: null out_coords");
  *blocks = 0;
  *cube = 0;
  TSMI_REQUIRE(!map_t || (n_t_pad >= n_in && n_t_pad < (int64_t(1) << 31)),
               "kmap_sorted: the transposed map needs n_t_pad >= n_in rows");
  TSMI_REQUIRE((pair_words == nullptr) == (pair_out == nullptr), "kmap_sorted: pair_words and pair_out go together");
  TSMI_REQUIRE(!pair_out || n_out_pad > 0, "kmap_sorted: a map without rows has no pairs to count");
  if (n_out_pad == 0) return TSMI_OK;
  TSMI_REQUIRE(out_in_map, "kmap_sorted: null out_in_map");
  a->in_coords = (const int4 *)in_coords;
  a->out_coords = (const int4 *)out_coords;
  a->map = out_in_map;
  a->n_in = n_in;
  a->n_out = n_out;
  a->n_out_pad = n_out_pad;
  a->rows = std::min(kBlock, kSortedTileInts / a->g.kvol);
  TSMI_REQUIRE(!n_in_dev || tsmi_kmap_sorted_samples_elems(n_in) == 0,
               "kmap_sorted: inputs whose count is on the device must be small enough to need no samples");
  const bool sampled = samples != nullptr && tsmi_kmap_sorted_samples_elems(n_in) > 0;
  a->first = sampled ? (const unsigned long long *)samples : nullptr;
  a->cell = sampled ? (const unsigned long long *)samples + kSortedSamples : nullptr;
  a->map_t = map_t;
  a->n_t_pad = n_t_pad;
  a->pair_acc = (unsigned long long *)pair_words;
  a->pair_ticket = pair_words ? (unsigned int *)(pair_words + 1) : nullptr;
  a->pair_out = (long long *)pair_out;
  a->n_in_dev = n_in_dev;
  a->n_out_dev = n_out_dev;
  *blocks = ceil_div(n_out_pad, a->rows);
  TSMI_REQUIRE(grid_fits(*blocks), "kmap_sorted: too many rows for one launch");
  a->n_blocks = (unsigned)*blocks;
  *cube = (ks[0] == ks[1] && ks[1] == ks[2] && a->rows == kBlock) ? ks[0] : 0;
  if (*cube != 2 && *cube != 3) *cube = 0;
  return TSMI_OK;
}

static int sorted_launch(hipStream_t s, const SortedArgs &a, int cube, int64_t blocks) {
  if (blocks == 0) return TSMI_OK;
  const dim3 grid((unsigned)blocks), block(kBlock);
  switch (cube) {
    case 2: hipLaunchKernelGGL(kmap_sorted_kernel<2>, grid, block, 0, s, a); break;
    case 3: hipLaunchKernelGGL(kmap_sorted_kernel<3>, grid, block, 0, s, a); break;
    default: hipLaunchKernelGGL(kmap_sorted_kernel<0>, grid, block, 0, s, a); break;
  }
  return check_launch("tsmi_kmap_sorted");
}

extern "C" int tsmi_kmap_sorted(tsmi_stream_t s, const int32_t *in_coords, int64_t n_in,
                                const int32_t *out_coords, int64_t n_out, int64_t n_out_pad,
                                const int32_t ks[3], const int32_t stride[3], const int32_t pad[3],
                                const int64_t *samples, int32_t *out_in_map) {
  SortedArgs a;
  int cube;
  int64_t blocks;
  if (int e = sorted_args(&a, &cube, &blocks, in_coords, n_in, out_coords, n_out, n_out_pad, ks, stride, pad,
                          samples, out_in_map, nullptr, 0, nullptr, nullptr))
    return e;
  return sorted_launch((hipStream_t)s, a, cube, blocks);
}

extern "C" int tsmi_kmap_sorted_batch(tsmi_stream_t s, int count, const int64_t *args) {
  TSMI_REQUIRE(count >= 0 && (count == 0 || args), "kmap_sorted_batch: bad arguments");
  constexpr int kWords = 22;  // int64 words per map
  int done = 0;
  while (done < count) {
    // as many of the next maps as one launch takes: 2^3 and 3^3 kernels, up to kSortedBatchMax
    SortedBatch b;
    b.count = 0;
    b.first_block[0] = 0;
    SortedArgs single;
    int single_cube = 0;
    int64_t single_blocks = 0;
    bool have_single = false;
    while (done < count && b.count < kSortedBatchMax) {
      const int64_t *a = args + (int64_t)kWords * done;
      int32_t geom[9];
      for (int j = 0; j < 9; ++j) geom[j] = (int32_t)a[7 + j];
      SortedArgs one;
      int cube;
      int64_t blocks;
      if (int e = sorted_args(&one, &cube, &blocks, (const int32_t *)(uintptr_t)a[0], a[1],
                              (const int32_t *)(uintptr_t)a[2], a[3], a[4], geom, geom + 3, geom + 6,
                              (const int64_t *)(uintptr_t)a[5], (int32_t *)(uintptr_t)a[6],
                              (int32_t *)(uintptr_t)a[16], a[17], (int64_t *)(uintptr_t)a[18],
                              (int64_t *)(uintptr_t)a[19], (const int32_t *)(uintptr_t)a[20],
                              (const int32_t *)(uintptr_t)a[21]))
        return e;
      if (blocks == 0) {
        ++done;
        continue;
      }
      if (cube == 0 || !grid_fits((int64_t)b.first_block[b.count] + blocks)) {
        if (b.count > 0) break;  // launch what has been gathered first
        single = one;
        single_cube = cube;
        single_blocks = blocks;
        have_single = true;
        ++done;
        break;
      }
      b.a[b.count] = one;
      b.kc[b.count] = cube;
      b.first_block[b.count + 1] = b.first_block[b.count] + (unsigned)blocks;
      ++b.count;
      ++done;
    }
    if (have_single) {
      if (int e = sorted_launch((hipStream_t)s, single, single_cube, single_blocks)) return e;
    } else if (b.count == 1) {
      if (int e = sorted_launch((hipStream_t)s, b.a[0], b.kc[0], b.first_block[1])) return e;
    } else if (b.count > 1) {
      for (int i = b.count; i < kSortedBatchMax; ++i) {
        b.a[i] = b.a[0];
        b.kc[i] = b.kc[0];
        b.first_block[i + 1] = b.first_block[b.count];
      }
      hipLaunchKernelGGL(kmap_sorted_batch_kernel, dim3(b.first_block[b.count]), dim3(kBlock), 0, (hipStream_t)s, b);
      if (int e = check_launch("tsmi_kmap_sorted_batch")) return e;
    }
  }
  return TSMI_OK;
}

extern "C" int tsmi_coords_max(tsmi_stream_t s, const int32_t *coords, int64_t n,
                               int32_t *out_max, int clear_first) {
  TSMI_REQUIRE(out_max && n >= 0 && (n == 0 || coords), "coords_max: bad arguments");
  if (clear_first)
    hipLaunchKernelGGL(fill_kernel<int32_t>, dim3(1), dim3(kBlock), 0, (hipStream_t)s, out_max,
                       (int64_t)4, 0);
  if (n > 0) {
    TSMI_GRID_CHECK(n);
    hipLaunchKernelGGL(coords_max_kernel, dim3(std::min(grid_for(n).x, 512u)), dim3(kBlock), 0,
                       (hipStream_t)s, (const int4 *)coords, n, out_max);
  }
  return check_launch("tsmi_coords_max");
}

extern "C" int tsmi_downsample_candidates(tsmi_stream_t s, const int32_t *in_coords, int64_t n_in,
                                          const int32_t ks[3], const int32_t stride[3],
                                          const int32_t pad[3], const int32_t out_max_host[3],
                                          const int32_t *in_max_dev, const int32_t *in_min_dev,
                                          int mode, int64_t *keys, int64_t cap,
                                          int32_t *counters) {
  TableView t;
  Geom g;
  static int32_t dummy_vals;  // the de-duplication pass never touches vals
  if (int e = make_table(&t, keys, &dummy_vals, cap)) return e;
  if (int e = make_geom(&g, ks, stride, pad)) return e;
  TSMI_REQUIRE(mode == 0 || mode == 1 || mode == 3, "downsample_candidates: mode must be 0, 1 or 3");
  TSMI_REQUIRE(mode != 3 || out_max_host, "downsample_candidates: mode 3 needs out_max_host");
  // kernel size == stride and zero padding: every input has exactly one candidate
  if (mode == 0 && ks[0] == stride[0] && ks[1] == stride[1] && ks[2] == stride[2] &&
      pad[0] == 0 && pad[1] == 0 && pad[2] == 0)
    mode = 2;
  TSMI_REQUIRE(n_in >= 0 && (n_in == 0 || in_coords), "downsample_candidates: bad coords");
  TSMI_REQUIRE(counters, "downsample_candidates: null counters");
  TSMI_REQUIRE(mode == 1 || in_max_dev || out_max_host, "downsample_candidates: no output bound");
  if (n_in == 0) return TSMI_OK;
  int64_t per_input = g.kvol;  // mode 3: every offset
  if (mode == 1 || mode == 2) per_input = 1;
  if (mode == 0)  // the digits that divide exactly: at most ceil(ks / stride) per axis
    per_input = (int64_t)((ks[0] + stride[0] - 1) / stride[0]) * ((ks[1] + stride[1] - 1) / stride[1]) *
                ((ks[2] + stride[2] - 1) / stride[2]);
  int64_t total = n_in * per_input;
  TSMI_GRID_CHECK(total);
  int3 hm = make_int3(0, 0, 0);
  if (out_max_host) hm = make_int3(out_max_host[0], out_max_host[1], out_max_host[2]);
  hipLaunchKernelGGL(downsample_candidates_kernel, grid_for(total), dim3(kBlock), 0,
                     (hipStream_t)s, (const int4 *)in_coords, n_in, total, g, hm, in_max_dev,
                     in_min_dev, mode, t, counters);
  return check_launch("tsmi_downsample_candidates");
}

extern "C" int tsmi_hashtable_compact_keys(tsmi_stream_t s, const int64_t *keys, int64_t cap,
                                           int64_t *stored_keys_out, int32_t *count_out) {
  TSMI_REQUIRE(keys && stored_keys_out && count_out && cap >= 1 && cap < (int64_t(1) << 31),
               "hashtable_compact_keys: bad arguments");
  TSMI_GRID_CHECK(cap);
  hipLaunchKernelGGL(compact_keys_kernel, grid_for(cap), dim3(kBlock), 0, (hipStream_t)s,
                     (const unsigned long long *)keys, cap, (unsigned long long *)stored_keys_out,
                     count_out);
  return check_launch("tsmi_hashtable_compact_keys");
}

extern "C" int tsmi_downsample_finalize(tsmi_stream_t s, const int64_t *sorted_keys, int64_t n_out,
                                        const int64_t *keys, int32_t *vals, int64_t cap,
                                        int32_t *out_coords) {
  TableView t;
  if (int e = make_table(&t, keys, vals, cap)) return e;
  TSMI_REQUIRE(n_out >= 0 && (n_out == 0 || (sorted_keys && out_coords)),
               "downsample_finalize: bad arguments");
  TSMI_REQUIRE(n_out <= cap,
               "The capacity of hashtable is not sufficient. Please enlarge reserved space for "
               "hashtable (backends.hash_rsv_ratio): %lld outputs, capacity %lld",
               (long long)n_out, (long long)cap);
  if (n_out == 0) return TSMI_OK;
  TSMI_GRID_CHECK(n_out);
  hipLaunchKernelGGL(downsample_finalize_kernel, grid_for(n_out), dim3(kBlock), 0, (hipStream_t)s,
                     (const unsigned long long *)sorted_keys, n_out, t, (int4 *)out_coords);
  return check_launch("tsmi_downsample_finalize");
}

namespace {
// Shared argument checks of the two occupancy-bitmap entry points.
int grid_args(Geom *g, int *mode, int3 *hm, const int32_t ks[3], const int32_t stride[3],
              const int32_t pad[3], const int32_t out_max_host[3], const int32_t *in_max_dev,
              const void *bitmap, int64_t bitmap_words, const void *chunk_counts, const void *counters) {
  if (int e = make_geom(g, ks, stride, pad)) return e;
  TSMI_REQUIRE(in_max_dev && bitmap && chunk_counts && counters, "downsample_grid: null pointer");
  TSMI_REQUIRE((uintptr_t)bitmap % 16 == 0, "downsample_grid: bitmap must be 16-byte aligned");
  TSMI_REQUIRE(bitmap_words >= kGridChunkWords && bitmap_words % kGridChunkWords == 0 &&
                   bitmap_words <= (int64_t(1) << 25),
               "downsample_grid: bitmap_words must be a multiple of %d and at most 2^25", kGridChunkWords);
  *mode = (ks[0] == stride[0] && ks[1] == stride[1] && ks[2] == stride[2] && pad[0] == 0 &&
           pad[1] == 0 && pad[2] == 0) ? 2 : 0;
  *hm = out_max_host ? make_int3(out_max_host[0], out_max_host[1], out_max_host[2]) : make_int3(0, 0, 0);
  return TSMI_OK;
}
}  // namespace

static int64_t per_input_fan(const int32_t ks[3], const int32_t stride[3]) {
  return (int64_t)((ks[0] + stride[0] - 1) / stride[0]) * ((ks[1] + stride[1] - 1) / stride[1]) *
         ((ks[2] + stride[2] - 1) / stride[2]);
}

extern "C" int tsmi_downsample_grid_count(tsmi_stream_t s, const int32_t *in_coords, int64_t n_in,
                                          const int32_t ks[3], const int32_t stride[3],
                                          const int32_t pad[3], const int32_t out_max_host[3],
                                          const int32_t *in_max_dev, int32_t *bitmap,
                                          int64_t bitmap_words, int clear_first,
                                          int32_t *chunk_counts, int32_t *counters,
                                          int32_t *next_in_max_dev, const int32_t *n_in_dev) {
  Geom g;
  int mode;
  int3 hm;
  if (int e = grid_args(&g, &mode, &hm, ks, stride, pad, out_max_host, in_max_dev, bitmap, bitmap_words,
                        chunk_counts, counters))
    return e;
  TSMI_REQUIRE(n_in >= 0 && (n_in == 0 || in_coords), "downsample_grid_count: bad coords");
  const int has_hm = out_max_host != nullptr;
  const int64_t total = n_in * (mode == 2 ? 1 : per_input_fan(ks, stride));
  TSMI_GRID_CHECK(total);
  hipStream_t st = (hipStream_t)s;
  const unsigned chunks = (unsigned)(bitmap_words / kGridChunkWords);
  if (clear_first)
    hipLaunchKernelGGL(grid_clear_kernel, grid_for(bitmap_words / 4), dim3(kBlock), 0, st, (uint4 *)bitmap,
                       bitmap_words, g, hm, has_hm, in_max_dev);
  bool per_input = mode == 0 && per_input_fan(ks, stride) > 1 && !n_in_dev;
  for (int a = 0; a < 3; ++a) per_input = per_input && (ks[a] + stride[a] - 1) / stride[a] <= kMaxFanAxis;
  if (total > 0 && per_input)
    hipLaunchKernelGGL(grid_mark_fan_kernel, grid_for(n_in), dim3(kBlock), 0, st, (const int4 *)in_coords,
                       n_in, g, hm, has_hm, in_max_dev, (uint32_t *)bitmap, bitmap_words, next_in_max_dev,
                       counters);
  else if (total > 0)
    hipLaunchKernelGGL(grid_mark_kernel, grid_for(total), dim3(kBlock), 0, st, (const int4 *)in_coords,
                       total, g, hm, has_hm, in_max_dev, mode, (uint32_t *)bitmap, bitmap_words,
                       next_in_max_dev, counters, n_in_dev);
  hipLaunchKernelGGL(grid_count_kernel, dim3(chunks < 2048u ? chunks : 2048u), dim3(kBlock), 0, st,
                     (const uint32_t *)bitmap,
                     bitmap_words, g, hm, has_hm, in_max_dev, chunk_counts);
  hipLaunchKernelGGL(grid_scan_kernel, dim3(1), dim3(1024), 0, st, chunk_counts, bitmap_words, g, hm,
                     has_hm, in_max_dev, counters);
  return check_launch("tsmi_downsample_grid_count");
}

extern "C" int tsmi_downsample_grid_count_next(tsmi_stream_t s, const int32_t ks[3],
                                               const int32_t stride[3], const int32_t pad[3],
                                               const int32_t *prev_in_max_dev, const int32_t *prev_bitmap,
                                               int64_t prev_bitmap_words, const int32_t *in_max_dev,
                                               int32_t *bitmap, int64_t bitmap_words,
                                               int32_t *chunk_counts, int32_t *counters,
                                               int32_t *next_in_max_dev) {
  Geom g;
  int mode;
  int3 hm;
  if (int e = grid_args(&g, &mode, &hm, ks, stride, pad, nullptr, in_max_dev, bitmap, bitmap_words,
                        chunk_counts, counters))
    return e;
  TSMI_REQUIRE(prev_in_max_dev && prev_bitmap && prev_bitmap_words >= kGridChunkWords &&
                   prev_bitmap_words % kGridChunkWords == 0 && prev_bitmap_words <= (int64_t(1) << 25),
               "downsample_grid_count_next: bad previous bitmap");
  hipStream_t st = (hipStream_t)s;
  const int64_t prev_chunks = prev_bitmap_words / kGridChunkWords;
  hipLaunchKernelGGL(grid_mark_next_kernel, dim3((unsigned)(prev_chunks < 2048 ? prev_chunks : 2048)),
                     dim3(kBlock), 0, st, (const uint32_t *)prev_bitmap, prev_bitmap_words,
                     prev_in_max_dev, g, mode, in_max_dev, (uint32_t *)bitmap, bitmap_words,
                     next_in_max_dev);
  const unsigned chunks = (unsigned)(bitmap_words / kGridChunkWords);
  hipLaunchKernelGGL(grid_count_kernel, dim3(chunks < 2048u ? chunks : 2048u), dim3(kBlock), 0, st,
                     (const uint32_t *)bitmap, bitmap_words, g, hm, 0, in_max_dev, chunk_counts);
  hipLaunchKernelGGL(grid_scan_kernel, dim3(1), dim3(1024), 0, st, chunk_counts, bitmap_words, g, hm, 0,
                     in_max_dev, counters);
  return check_launch("tsmi_downsample_grid_count_next");
}

extern "C" int tsmi_downsample_grid_emit(tsmi_stream_t s, const int32_t ks[3], const int32_t stride[3],
                                         const int32_t pad[3], const int32_t out_max_host[3],
                                         const int32_t *in_max_dev, const int32_t *in_max_host,
                                         int32_t *bitmap, int64_t bitmap_words,
                                         const int32_t *chunk_prefix, int64_t n_out, int64_t *keys,
                                         int32_t *vals, int64_t cap, int32_t *out_coords,
                                         int32_t *counters) {
  Geom g;
  int mode;
  int3 hm;
  TableView t;
  if (int e = grid_args(&g, &mode, &hm, ks, stride, pad, out_max_host, in_max_dev, bitmap, bitmap_words,
                        chunk_prefix, counters))
    return e;
  const bool want_table = keys != nullptr;
  if (want_table)
    if (int e = make_table(&t, keys, vals, cap)) return e;
  // n_out < 0: the count is still on the device and out_coords holds -n_out rows; every chunk
  // the device-side extents cover is emitted by a bounded grid, no table is filled
  const bool on_device = n_out < 0;
  if (on_device) {
    TSMI_REQUIRE(!want_table && !in_max_host && out_coords, "downsample_grid_emit: a device-side count takes no table");
    const int64_t chunks_cap = bitmap_words / kGridChunkWords;
    hipLaunchKernelGGL(grid_emit_kernel, dim3((unsigned)std::min<int64_t>(chunks_cap, 2048)), dim3(kBlock), 0,
                       (hipStream_t)s, (uint32_t *)bitmap, bitmap_words, chunk_prefix, g, hm,
                       out_max_host != nullptr, in_max_dev, GridDims{}, 0, (int4 *)out_coords, -n_out);
    return check_launch("tsmi_downsample_grid_emit");
  }
  TSMI_REQUIRE(n_out >= 0 && (n_out == 0 || out_coords), "downsample_grid_emit: bad arguments");
  TSMI_REQUIRE(!want_table || n_out <= cap,
               "The capacity of hashtable is not sufficient. Please enlarge reserved space for "
               "hashtable (backends.hash_rsv_ratio): %lld outputs, capacity %lld",
               (long long)n_out, (long long)cap);
  if (n_out == 0) return TSMI_OK;
  TSMI_GRID_CHECK(n_out);
  // with the maxima on the host the extents are computed here: the kernel neither waits for
  // them nor launches the chunks beyond the grid
  GridDims hd = {};
  int64_t chunks = bitmap_words / kGridChunkWords;
  if (in_max_host) {
    hd = grid_dims(g, hm, out_max_host != nullptr, in_max_host, bitmap_words);
    TSMI_REQUIRE(hd.fits, "downsample_grid_emit: the grid does not fit the bitmap");
    chunks = hd.used_words / kGridChunkWords;
    if (chunks == 0) return TSMI_OK;
  }
  hipLaunchKernelGGL(grid_emit_kernel, dim3((unsigned)chunks), dim3(kBlock), 0, (hipStream_t)s,
                     (uint32_t *)bitmap, bitmap_words, chunk_prefix, g, hm, out_max_host != nullptr,
                     in_max_dev, hd, in_max_host != nullptr, (int4 *)out_coords, n_out);
  if (want_table)
    hipLaunchKernelGGL(insert_coords_kernel, grid_for(n_out), dim3(kBlock), 0, (hipStream_t)s, t,
                       (const int4 *)out_coords, n_out, counters + 1);
  return check_launch("tsmi_downsample_grid_emit");
}

extern "C" int tsmi_downsample_chain_rows(tsmi_stream_t s, const int32_t *coords, int64_t n,
                                          const int32_t ks[3], const int32_t stride[3],
                                          const int32_t pad[3], int levels, int32_t *scratch,
                                          const int64_t *bitmap_at, const int64_t *bitmap_words,
                                          const int64_t *chunks_at, int32_t *counters, int32_t *rows,
                                          int phase) {
  TSMI_REQUIRE(levels >= 1 && levels <= kChainMaxLevels && n > 0 && coords && scratch && bitmap_at &&
                   bitmap_words && chunks_at && counters && rows && phase >= 0 && phase <= 2,
               "downsample_chain_rows: bad arguments");
  for (int a = 0; a < 3; ++a)
    TSMI_REQUIRE(ks[a] == stride[a] && pad[a] == 0 && ks[a] >= 1,
                 "downsample_chain_rows: one output per input needs kernel size == stride and no padding");
  Geom g;
  if (int e = make_geom(&g, ks, stride, pad)) return e;
  TSMI_REQUIRE((uintptr_t)scratch % 16 == 0, "downsample_chain_rows: scratch must be 16-byte aligned");
  TSMI_GRID_CHECK(n);
  // blocks of the launches that walk chunks: the extents are on the device, so a bounded number
  // per level strides over the chunks there are
  constexpr int64_t kBlocksPerLevel = 512;
  ChainLayout lay;
  lay.levels = levels;
  lay.first_block[0] = 0;
  for (int l = 0; l < kChainMaxLevels; ++l) {
    const int u = l < levels ? l : 0;  // (unused entries repeat level 0)
    TSMI_REQUIRE(bitmap_words[u] >= kGridChunkWords && bitmap_words[u] % kGridChunkWords == 0 &&
                     bitmap_words[u] <= (int64_t(1) << 25) && bitmap_at[u] >= 0 && bitmap_at[u] % 4 == 0 &&
                     chunks_at[u] >= 0,
                 "downsample_chain_rows: bitmap_words must be a multiple of %d and at most 2^25, bitmaps 16-byte aligned",
                 kGridChunkWords);
    lay.bitmap_at[l] = bitmap_at[u];
    lay.words[l] = bitmap_words[u];
    lay.chunks_at[l] = chunks_at[u];
    const int64_t blocks = l < levels ? std::min(bitmap_words[u] / kGridChunkWords, kBlocksPerLevel) : 0;
    lay.first_block[l + 1] = lay.first_block[l] + (unsigned)blocks;
  }
  hipStream_t st = (hipStream_t)s;
  if (phase != 2) {
    // counters: 8 per level, [4..8) of a level = the maxima of its INPUT rows
    if (int e = tsmi_coords_max(s, coords, n, counters + 4, 0)) return e;
    for (int level = 0; level < levels; ++level)
      hipLaunchKernelGGL(chain_mark_kernel, grid_for(n), dim3(kBlock), 0, st, (const int4 *)coords, n, g, level,
                         lay, scratch, counters);
    hipLaunchKernelGGL(chain_count_kernel, dim3(lay.first_block[levels]), dim3(kBlock), 0, st, g, lay,
                       (const int32_t *)scratch, scratch, (const int32_t *)counters);
    hipLaunchKernelGGL(chain_scan_kernel, dim3((unsigned)levels), dim3(1024), 0, st, g, lay, scratch, counters);
  }
  if (phase != 1)
    hipLaunchKernelGGL(chain_emit_kernel, dim3(lay.first_block[levels]), dim3(kBlock), 0, st, g, lay, scratch,
                       (const int32_t *)counters, (int4 *)rows, n);
  return check_launch("tsmi_downsample_chain_rows");
}

extern "C" int tsmi_transpose_map(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                                  int32_t *map_t, int64_t n_rows_t) {
  TSMI_REQUIRE(kvol >= 1 && n_rows >= 0 && n_rows_t >= 0, "transpose_map: bad sizes");
  int64_t total_t = n_rows_t * kvol, total = n_rows * kvol;
  if (total_t > 0) {
    TSMI_REQUIRE(map_t, "transpose_map: null map_t");
    TSMI_GRID_CHECK(total_t);
    hipLaunchKernelGGL(fill_kernel<int32_t>, grid_for(total_t), dim3(kBlock), 0, (hipStream_t)s,
                       map_t, total_t, -1);
  }
  if (total > 0 && total_t > 0) {
    TSMI_REQUIRE(map, "transpose_map: null map");
    TSMI_GRID_CHECK(total);
    hipLaunchKernelGGL(transpose_map_kernel, grid_for(total), dim3(kBlock), 0, (hipStream_t)s, map,
                       total, kvol, map_t, n_rows_t);
  }
  return check_launch("tsmi_transpose_map");
}

extern "C" int tsmi_derive_bitmask(tsmi_stream_t s, const int32_t *map, int64_t n_pad, int kvol,
                                   int split, int64_t valid_n, int32_t *bitmask) {
  TSMI_REQUIRE(kvol >= 1 && split >= 1 && n_pad >= 0 && valid_n >= 0 && valid_n <= n_pad,
               "derive_bitmask: bad sizes");
  int len = (kvol + split - 1) / split;
  TSMI_REQUIRE(len <= 32, "derive_bitmask: %d offsets per split exceed the 32 mask bits", len);
  TSMI_REQUIRE((int64_t)(split - 1) * len < kvol, "derive_bitmask: split_mask_num %d leaves an empty split", split);
  int64_t total = n_pad * split;
  if (total == 0) return TSMI_OK;
  TSMI_REQUIRE(map && bitmask, "derive_bitmask: null pointer");
  TSMI_GRID_CHECK(n_pad);
  hipLaunchKernelGGL(derive_bitmask_kernel, dim3(grid_for(n_pad).x, split), dim3(kBlock), 0,
                     (hipStream_t)s, map, n_pad, kvol, split, len, valid_n, bitmask);
  return check_launch("tsmi_derive_bitmask");
}

extern "C" int tsmi_reorder_map(tsmi_stream_t s, const int32_t *map, const int32_t *reorder_loc,
                                int64_t n_pad, int kvol, int split, int32_t *out) {
  TSMI_REQUIRE(kvol >= 1 && split >= 1 && n_pad >= 0, "reorder_map: bad sizes");
  int64_t total = n_pad * kvol;
  if (total == 0) return TSMI_OK;
  TSMI_REQUIRE(map && reorder_loc && out, "reorder_map: null pointer");
  TSMI_GRID_CHECK(total);
  int len = (kvol + split - 1) / split;
  hipLaunchKernelGGL(reorder_map_kernel, grid_for(total), dim3(kBlock), 0, (hipStream_t)s, map,
                     reorder_loc, n_pad, kvol, len, out);
  return check_launch("tsmi_reorder_map");
}

extern "C" int tsmi_reduce_bitmask(tsmi_stream_t s, const int32_t *sorted_mask, int split,
                                   int64_t n_pad, int tile, int32_t *reduced) {
  if (tile < 4 || tile % 4 != 0)
    return fail(TSMI_ERR_RUNTIME, "[Bitmask reduce] reduce tile size must be multiple of 4.");
  TSMI_REQUIRE(split >= 1 && n_pad >= 0, "reduce_bitmask: bad sizes");
  if (n_pad == 0) return TSMI_OK;  // a map without rows has no tiles
  TSMI_REQUIRE(sorted_mask && reduced, "reduce_bitmask: null pointer");
  int64_t rows = (n_pad - 1) / tile + 1;
  int64_t total = rows * split;
  TSMI_GRID_CHECK(total);
  hipLaunchKernelGGL(reduce_bitmask_kernel, grid_for(total), dim3(kBlock), 0, (hipStream_t)s,
                     sorted_mask, split, n_pad, tile, rows, reduced);
  return check_launch("tsmi_reduce_bitmask");
}

extern "C" int tsmi_pair_lists_count(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                                     int32_t *block_counts, int32_t *nbsizes) {
  TSMI_REQUIRE(kvol >= 1 && kvol <= kPairMaxKvol && n_rows >= 0 && nbsizes,
               "pair_lists_count: bad arguments (kernel volume %d, at most %d)", kvol, kPairMaxKvol);
  int64_t nblk = ceil_div(n_rows, kBlock);
  if (n_rows == 0) {
    hipLaunchKernelGGL(fill_kernel<int32_t>, grid_for(kvol), dim3(kBlock), 0, (hipStream_t)s,
                       nbsizes, (int64_t)kvol, 0);
    return check_launch("tsmi_pair_lists_count");
  }
  TSMI_REQUIRE(map && block_counts, "pair_lists_count: null pointer");
  TSMI_REQUIRE(grid_fits(nblk), "pair_lists_count: too many rows");
  hipLaunchKernelGGL(pair_count_kernel, dim3((unsigned)nblk), dim3(kBlock), 0, (hipStream_t)s, map,
                     n_rows, kvol, nblk, block_counts);
  hipLaunchKernelGGL(pair_scan_kernel, dim3(kvol), dim3(1024), 0, (hipStream_t)s, block_counts, kvol,
                     nblk, nbsizes);
  return check_launch("tsmi_pair_lists_count");
}

extern "C" int tsmi_pair_lists_fill(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                                    int32_t *block_counts, const int32_t *nbsizes, int64_t nnz,
                                    int32_t *nbmaps_inter, int32_t *nbmaps_planar, int64_t n_in,
                                    int64_t n_out, int mask_skip_k, int32_t *input_mask,
                                    int32_t *output_mask) {
  TSMI_REQUIRE(mask_skip_k >= -2 && mask_skip_k < kvol, "pair_lists_fill: bad mask_skip_k %d", mask_skip_k);
  TSMI_REQUIRE(kvol >= 1 && kvol <= kPairMaxKvol && n_rows >= 0 && nnz >= 0 && n_in >= 0 && n_out >= 0,
               "pair_lists_fill: bad sizes");
  if (input_mask && n_in > 0) {
    TSMI_GRID_CHECK(n_in * kvol);
    hipLaunchKernelGGL(fill_kernel<int32_t>, grid_for(n_in * kvol), dim3(kBlock), 0,
                       (hipStream_t)s, input_mask, n_in * kvol, -1);
  }
  if (output_mask && n_out > 0) {
    TSMI_GRID_CHECK(n_out * kvol);
    hipLaunchKernelGGL(fill_kernel<int32_t>, grid_for(n_out * kvol), dim3(kBlock), 0,
                       (hipStream_t)s, output_mask, n_out * kvol, -1);
  }
  if (n_rows > 0 && nnz > 0) {
    TSMI_REQUIRE(map && block_counts && nbsizes, "pair_lists_fill: null pointer");
    int64_t nblk = ceil_div(n_rows, kBlock);
    TSMI_REQUIRE(grid_fits(nblk), "pair_lists_fill: too many rows");
    int skip_k = mask_skip_k;
    if (skip_k == -2) skip_k = (n_in == n_out && kvol % 2 == 1) ? kvol / 2 : -1;  // the reference's rule
    hipLaunchKernelGGL(pair_fill_kernel, dim3((unsigned)nblk), dim3(kBlock), 0, (hipStream_t)s,
                       map, n_rows, kvol, nblk, block_counts, nbsizes, nnz, nbmaps_inter,
                       nbmaps_planar, n_in, n_out, input_mask, output_mask, skip_k);
  }
  return check_launch("tsmi_pair_lists_fill");
}

extern "C" int tsmi_pair_segments(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                                  int64_t seg_rows, int32_t *pool, int32_t *counts, int32_t *in_rows,
                                  int32_t *pos) {
  TSMI_REQUIRE(kvol >= 1 && kvol <= kPairMaxKvol && n_rows >= 0 && seg_rows >= n_rows,
               "pair_segments: bad sizes (kernel volume %d, at most %d; %lld rows, segments of %lld)",
               kvol, kPairMaxKvol, (long long)n_rows, (long long)seg_rows);
  TSMI_REQUIRE((int64_t)kvol * seg_rows < (int64_t(1) << 31), "pair_segments: kvol * seg_rows exceeds int32");
  TSMI_REQUIRE(counts, "pair_segments: null counts");
  if (!pool || n_rows == 0)
    hipLaunchKernelGGL(fill_kernel<int32_t>, grid_for(kvol), dim3(kBlock), 0, (hipStream_t)s, counts,
                       (int64_t)kvol, 0);
  if (n_rows == 0) return check_launch("tsmi_pair_segments");
  TSMI_REQUIRE(map && in_rows && pos, "pair_segments: null pointer");
  const int64_t nblk = ceil_div(n_rows, kBlock);
  TSMI_REQUIRE(grid_fits(nblk), "pair_segments: too many rows");
  const dim3 grid((unsigned)nblk), block(kBlock);
  switch (kvol) {
    case 27:
      hipLaunchKernelGGL(pair_segments_kernel<27>, grid, block, 0, (hipStream_t)s, map, n_rows, kvol,
                         seg_rows, pool, counts, in_rows, pos);
      break;
    case 8:
      hipLaunchKernelGGL(pair_segments_kernel<8>, grid, block, 0, (hipStream_t)s, map, n_rows, kvol,
                         seg_rows, pool, counts, in_rows, pos);
      break;
    default:
      hipLaunchKernelGGL(pair_segments_kernel<0>, grid, block, 0, (hipStream_t)s, map, n_rows, kvol,
                         seg_rows, pool, counts, in_rows, pos);
  }
  return check_launch("tsmi_pair_segments");
}

extern "C" int tsmi_pair_segments_batch(tsmi_stream_t s, int count, const int64_t *args) {
  TSMI_REQUIRE(count >= 0 && (count == 0 || args), "pair_segments_batch: bad arguments");
  for (int i = 0; i < count; ++i) {
    const int64_t *a = args + 8 * (int64_t)i;
    TSMI_REQUIRE(a[2] >= 1 && a[2] <= kPairMaxKvol, "pair_segments_batch: bad kernel volume");
    if (int e = tsmi_pair_segments(s, (const int32_t *)(uintptr_t)a[0], a[1], (int)a[2], a[3],
                                   (int32_t *)(uintptr_t)a[4], (int32_t *)(uintptr_t)a[5],
                                   (int32_t *)(uintptr_t)a[6], (int32_t *)(uintptr_t)a[7]))
      return e;
  }
  return TSMI_OK;
}

// ---- rows of a 3x3x3 map grouped by the planes of the kernel they use ------------------------
// An implicit-GEMM workgroup multiplies every kernel offset that ANY row of its tile uses; on a
// surface scan in coordinate order four of five such products are for absent neighbours.  Rows
// whose neighbours lie in the same outer planes of the kernel (digit 0 or 2 along each axis: six
// planes) use nearly the same offsets, so inside windows of `window` consecutive rows (near
// enough in space for the rows they gather to share an L2) the rows are counting-sorted by
//   key = rank of (offsets the occupied planes span) << 6 | plane bits    (1024 bins, padding rows last)
// where a row with neighbours in e_a of the three layers along axis a (the centre layer always
// counts) spans e_0 * e_1 * e_2 offsets - one of 1, 2, 3, 4, 6, 8, 9, 12, 18, 27 -, and the map
// is written out in that order together with the row each position came from and, per 64
// positions, the union of the offsets their rows use.  A second launch (one workgroup) lists
// the 64-row and the 128-row tiles by the size of that union, largest first: the order in which
// the convolution starts them.  The order inside a bin (and among tiles of one size) depends on
// the order in which threads draw their slots; what is computed through these arrays does not.
constexpr int kGroupThreads = 1024;
constexpr int kGroupMaxPerThread = 8;  // windows of at most 8192 rows

// used[row] = bit k per kernel offset the row has a neighbour at (thread per row, all CUs: a
// workgroup per window reading whole rows would have a handful of CUs pull the map through
// their load units row by row - 60 us for a 90k-row map, against 4 for this pass)
__global__ __launch_bounds__(kBlock) void map_row_masks_kernel(const int32_t *__restrict__ map,
                                                              int64_t n_rows, int32_t *__restrict__ used) {
  const int64_t row = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (row >= n_rows) return;
  const int32_t *m = map + row * 27;
  int mask = 0;
#pragma unroll
  for (int o = 0; o < 27; ++o)
    if (m[o] >= 0) mask |= 1 << o;
  used[row] = mask;
}

// One workgroup per window: the counting sort of its rows by key (from their masks), row_of, and
// the union of the masks of every 64 positions.
__global__ __launch_bounds__(kGroupThreads) void map_group_rows_kernel(
    const int32_t *__restrict__ used, int64_t n_rows, int window, int32_t *__restrict__ row_of,
    int32_t *__restrict__ masks64) {
  __shared__ int hist[1024];
  __shared__ int offs[1024];
  __shared__ int lmask[kGroupThreads * kGroupMaxPerThread];
  const int tid = threadIdx.x;
  const int64_t base = (int64_t)blockIdx.x * window;
  hist[tid] = 0;
  __syncthreads();
  int key[kGroupMaxPerThread], mine[kGroupMaxPerThread];
#pragma unroll
  for (int j = 0; j < kGroupMaxPerThread; ++j) {
    const int r = tid + j * kGroupThreads;
    key[j] = -1;
    mine[j] = 0;
    if (r >= window) continue;
    const int64_t row = base + r;
    int k = 1023;
    if (row < n_rows) {
      const int mask = used[row];
      // plane bits 0..5: a neighbour with digit 0 / digit 2 along axis 0, 1, 2 (the first digit of
      // an offset runs fastest: offset o has digits o % 3, o / 3 % 3, o / 9)
      constexpr int kD0_0 = 0x1249249, kD0_2 = 0x4924924;  // offsets with first digit 0 / 2
      constexpr int kD1_0 = 0x01C0E07, kD1_2 = 0x70381C0;  // second digit 0 / 2
      constexpr int kD2_0 = 0x00001FF, kD2_2 = 0x7FC0000;  // third digit 0 / 2
      const int planes = ((mask & kD0_0) ? 1 : 0) | ((mask & kD0_2) ? 2 : 0) | ((mask & kD1_0) ? 4 : 0) |
                         ((mask & kD1_2) ? 8 : 0) | ((mask & kD2_0) ? 16 : 0) | ((mask & kD2_2) ? 32 : 0);
      const int span = (1 + __popc(planes & 3)) * (1 + __popc(planes & 12)) * (1 + __popc(planes & 48));
      // rank of the span among 1, 2, 3, 4, 6, 8, 9, 12, 18, 27
      const int rank = span <= 4 ? span - 1 : (span == 6 ? 4 : span == 8 ? 5 : span == 9 ? 6 : span == 12 ? 7 : span == 18 ? 8 : 9);
      k = (rank << 6) | planes;
      mine[j] = mask;
    }
    key[j] = k;
    atomicAdd(&hist[k], 1);
  }
  __syncthreads();
  if (tid < 64) {  // exclusive scan of the 1024 bins: 16 per lane, then across the wavefront
    int local[16], sum = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      local[i] = sum;
      sum += hist[tid * 16 + i];
    }
    int incl = sum;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d);
      if (tid >= d) incl += up;
    }
    const int excl = incl - sum;
#pragma unroll
    for (int i = 0; i < 16; ++i) offs[tid * 16 + i] = excl + local[i];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kGroupMaxPerThread; ++j) {
    if (key[j] < 0) continue;
    const int64_t row = base + tid + j * kGroupThreads;
    const int slot = atomicAdd(&offs[key[j]], 1);  // < window: the bins hold `window` rows in all
    lmask[slot] = mine[j];
    row_of[base + slot] = row < n_rows ? (int32_t)row : -1;
  }
  __syncthreads();
  // union of the offsets used by every 64 consecutive positions (window is a multiple of 128)
  const int wave = tid >> 6, lane = tid & 63;
  for (int g = wave; g < window / 64; g += kGroupThreads / 64) {
    int v = lmask[g * 64 + lane];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v |= __shfl_xor(v, d);
    if (lane == 0) masks64[base / 64 + g] = v;
  }
}

// grouped[p, :] = map[row_of[p], :] (all -1 for a padding position): a thread per entry, so the
// writes are contiguous and the reads walk whole rows of the window's part of the map
__global__ __launch_bounds__(kBlock) void map_group_copy_kernel(const int32_t *__restrict__ map,
                                                               const int32_t *__restrict__ row_of,
                                                               int64_t n_entries,
                                                               int32_t *__restrict__ grouped) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n_entries) return;
  const unsigned p = (unsigned)i / 27u;  // (fewer than 2^31 entries: checked by the host)
  const int o = (int)((unsigned)i - p * 27u);
  const int32_t row = row_of[p];
  grouped[i] = row >= 0 ? map[(int64_t)row * 27 + o] : -1;
}

// The order in which a convolution starts the T tiles of 64 (order64) or 128 (order128) rows:
// workgroup b runs on XCD b % 8, so the tiles are cut into 8 runs of S = ceil(T / 8) consecutive
// tiles (consecutive windows are neighbours in space: the rows a run gathers stay in one L2) and
// order[8 j + c] = the tile of run c with the j-th most offsets, -1 when the run has fewer than
// j + 1 tiles: every XCD starts its long tiles first, and the workgroups that share a CU are
// a long, a middling and a short one.
__global__ __launch_bounds__(kGroupThreads) void group_tile_order_kernel(
    const int32_t *__restrict__ masks64, int n64, int32_t *__restrict__ order64,
    int32_t *__restrict__ order128) {
  __shared__ int hist[2][8][32];
  __shared__ int offs[2][8][32];
  const int tid = threadIdx.x;
  const int n128 = n64 / 2;  // (n64 is even: the grouped map holds a multiple of 128 positions)
  const int s64 = (n64 + 7) / 8, s128 = (n128 + 7) / 8;
  if (tid < 512) (&hist[0][0][0])[tid] = 0;
  for (int i = tid; i < 8 * s64; i += kGroupThreads) order64[i] = -1;
  for (int i = tid; i < 8 * s128; i += kGroupThreads) order128[i] = -1;
  __syncthreads();
  for (int i = tid; i < n64; i += kGroupThreads) {
    const int a = masks64[i];
    atomicAdd(&hist[0][i / s64][27 - __popc(a)], 1);
    if ((i & 1) == 0) atomicAdd(&hist[1][(i >> 1) / s128][27 - __popc(a | masks64[i + 1])], 1);
  }
  __syncthreads();
  if (tid < 16) {
    int sum = 0;
    for (int c = 0; c < 28; ++c) {
      offs[tid >> 3][tid & 7][c] = sum;
      sum += hist[tid >> 3][tid & 7][c];
    }
  }
  __syncthreads();
  for (int i = tid; i < n64; i += kGroupThreads) {
    const int a = masks64[i];
    const int c64 = i / s64;
    order64[8 * atomicAdd(&offs[0][c64][27 - __popc(a)], 1) + c64] = i;
    if ((i & 1) == 0) {
      const int c128 = (i >> 1) / s128;
      order128[8 * atomicAdd(&offs[1][c128][27 - __popc(a | masks64[i + 1])], 1) + c128] = i >> 1;
    }
  }
}

extern "C" int64_t tsmi_map_group_rows_padded(int64_t n_rows, int window) {
  if (n_rows < 0 || window < 128 || window > kGroupThreads * kGroupMaxPerThread || window % 128 != 0) return -1;
  return ceil_div(n_rows, window) * window;
}

extern "C" int tsmi_map_group_rows(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                                   int window, int32_t *grouped, int32_t *row_of, int32_t *masks64,
                                   int32_t *order64, int32_t *order128) {
  TSMI_REQUIRE(kvol == 27, "map_group_rows: 3x3x3 maps only (kernel volume %d)", kvol);
  const int64_t padded = tsmi_map_group_rows_padded(n_rows, window);
  TSMI_REQUIRE(padded >= 0, "map_group_rows: bad sizes (%lld rows, windows of %d: a multiple of 128, at most %d)",
               (long long)n_rows, window, kGroupThreads * kGroupMaxPerThread);
  TSMI_REQUIRE(padded < (int64_t(1) << 31) / 27, "map_group_rows: too many map entries");
  if (n_rows == 0) return TSMI_OK;
  TSMI_REQUIRE(map && grouped && row_of && masks64 && order64 && order128, "map_group_rows: null pointer");
  // the row masks go into the first n_rows ints of `grouped` (rewritten by the copy at the end,
  // which reads row_of and map only)
  int32_t *used = grouped;
  hipLaunchKernelGGL(map_row_masks_kernel, grid_for(n_rows), dim3(kBlock), 0, (hipStream_t)s, map, n_rows, used);
  hipLaunchKernelGGL(map_group_rows_kernel, dim3((unsigned)(padded / window)), dim3(kGroupThreads), 0,
                     (hipStream_t)s, used, n_rows, window, row_of, masks64);
  hipLaunchKernelGGL(group_tile_order_kernel, dim3(1), dim3(kGroupThreads), 0, (hipStream_t)s, masks64,
                     (int)(padded / 64), order64, order128);
  hipLaunchKernelGGL(map_group_copy_kernel, grid_for(padded * 27), dim3(kBlock), 0, (hipStream_t)s, map, row_of,
                     padded * 27, grouped);
  return check_launch("tsmi_map_group_rows");
}

extern "C" int64_t tsmi_wgrad_pairs_capacity(int64_t n_rows, int kvol) {
  if (n_rows < 0 || kvol < 1) return 0;
  return n_rows * kvol + (int64_t)kvol * (kWgradPairStep - 1);
}

extern "C" int tsmi_wgrad_pairs_build(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                                      int32_t *block_counts, int32_t *nbsizes, int32_t *pairs,
                                      int32_t *seg_steps) {
  TSMI_REQUIRE(kvol >= 1 && kvol <= kWgradMaxKvol && n_rows >= 0,
               "wgrad_pairs_build: bad sizes (kernel volume %d, at most %d)", kvol, kWgradMaxKvol);
  TSMI_REQUIRE(nbsizes && seg_steps, "wgrad_pairs_build: null pointer");
  TSMI_REQUIRE(n_rows * kvol < (int64_t(1) << 31), "wgrad_pairs_build: too many map entries");
  if (n_rows == 0) {
    hipLaunchKernelGGL(fill_kernel<int32_t>, grid_for(kvol + 1), dim3(kBlock), 0, (hipStream_t)s,
                       seg_steps, (int64_t)kvol + 1, 0);
    hipLaunchKernelGGL(fill_kernel<int32_t>, grid_for(kvol), dim3(kBlock), 0, (hipStream_t)s,
                       nbsizes, (int64_t)kvol, 0);
    return check_launch("tsmi_wgrad_pairs_build");
  }
  if (int e = tsmi_pair_lists_count(s, map, n_rows, kvol, block_counts, nbsizes)) return e;
  TSMI_REQUIRE(pairs, "wgrad_pairs_build: null pairs");
  int64_t nblk = ceil_div(n_rows, kBlock);
  hipLaunchKernelGGL(wgrad_pair_fill_kernel, dim3((unsigned)nblk), dim3(kBlock), 0, (hipStream_t)s,
                     map, n_rows, kvol, nblk, block_counts, nbsizes, pairs, seg_steps);
  return check_launch("tsmi_wgrad_pairs_build");
}

// ---- the entry point that allocates nothing -------------------------------------------------
// Scratch of the pair-list build (per-block counts of every offset) for callers that cannot
// bring a buffer of their own.  Each GPU holds its own copy of the array at its own address;
// host code only ever uses the per-device address obtained below, never the array's name.
constexpr int64_t kStaticScratchInts = int64_t(1) << 20;  // 4 MiB per GPU
static __device__ __align__(256) int32_t scratch[kStaticScratchInts];
constexpr int kStaticScratchMaxDevices = 64;
static std::atomic<int32_t *> g_scratch_ptr[kStaticScratchMaxDevices];

// Device address of `scratch` on the current device, looked up once per device.
static int static_scratch(int32_t **out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return tsmi::fail(TSMI_ERR_HIP, "static scratch: %s", hipGetErrorString(e));
  TSMI_REQUIRE(dev >= 0 && dev < kStaticScratchMaxDevices, "static scratch: device %d out of range", dev);
  int32_t *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    void *addr = nullptr;
    e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !addr)
      return tsmi::fail(TSMI_ERR_HIP, "static scratch: hipGetSymbolAddress: %s", hipGetErrorString(e));
    p = static_cast<int32_t *>(addr);
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return TSMI_OK;
}

extern "C" int tsmi_wgrad_pairs_build_static(tsmi_stream_t s, const int32_t *map, int64_t n_rows,
                                             int kvol, int32_t *nbsizes, int32_t *pairs,
                                             int32_t *seg_steps) {
  TSMI_REQUIRE(kvol >= 1 && kvol <= kWgradMaxKvol && n_rows >= 0,
               "wgrad_pairs_build_static: bad sizes (kernel volume %d, at most %d)", kvol, kWgradMaxKvol);
  const int64_t need = (int64_t)kvol * ceil_div(n_rows, kBlock);
  TSMI_REQUIRE(need <= kStaticScratchInts,
               "wgrad_pairs_build_static: K_vol * ceil(n_rows / 256) = %lld exceeds the %lld "
               "entries of the built-in scratch; use tsmi_wgrad_pairs_build with a buffer",
               (long long)need, (long long)kStaticScratchInts);
  int32_t *block_counts = nullptr;
  if (int e = static_scratch(&block_counts)) return e;
  // every entry the kernels read is written by the counting pass first: nothing to clear
  return tsmi_wgrad_pairs_build(s, map, n_rows, kvol, block_counts, nbsizes, pairs, seg_steps);
}

extern "C" int tsmi_wgrad_pairs_pad(tsmi_stream_t s, const int32_t *nbmaps_inter, int64_t nnz,
                                    const int32_t *nbsizes, int kvol, int32_t *pairs,
                                    int32_t *seg_steps) {
  TSMI_REQUIRE(kvol >= 1 && kvol <= kWgradMaxKvol && nnz >= 0,
               "wgrad_pairs_pad: bad sizes (kernel volume %d, at most %d)", kvol, kWgradMaxKvol);
  TSMI_REQUIRE(nbsizes && seg_steps && pairs, "wgrad_pairs_pad: null pointer");
  TSMI_REQUIRE(nnz == 0 || nbmaps_inter, "wgrad_pairs_pad: null pair list");
  const int64_t limit = nnz + (int64_t)kvol * (kWgradPairStep - 1);
  TSMI_GRID_CHECK(limit);
  hipLaunchKernelGGL(wgrad_pair_pad_kernel, grid_for(std::max<int64_t>(limit, 1)), dim3(kBlock), 0,
                     (hipStream_t)s, nbmaps_inter, nnz, nbsizes, kvol, limit, pairs, seg_steps);
  return check_launch("tsmi_wgrad_pairs_pad");
}

extern "C" int tsmi_exclusive_scan_quantified(tsmi_stream_t s, int kvol, const int32_t *nbsizes,
                                              int q, int32_t *nbaddrs, int32_t *qnbaddrs) {
  TSMI_REQUIRE(kvol >= 1 && q >= 1 && nbsizes && nbaddrs && qnbaddrs,
               "exclusive_scan_quantified: bad arguments");
  hipLaunchKernelGGL(scan_quantified_kernel, dim3(1), dim3(64), 0, (hipStream_t)s, kvol, nbsizes,
                     q, nbaddrs, qnbaddrs);
  return check_launch("tsmi_exclusive_scan_quantified");
}

extern "C" int tsmi_build_masks(tsmi_stream_t s, const int32_t *nbmaps_inter, int64_t nnz,
                                const int32_t *nbaddrs, int kvol, int64_t n_in, int64_t n_out,
                                int32_t *input_mask, int32_t *output_mask) {
  TSMI_REQUIRE(kvol >= 1 && nnz >= 0 && n_in >= 0 && n_out >= 0, "build_masks: bad sizes");
  TSMI_REQUIRE(input_mask || n_in == 0, "build_masks: null input_mask");
  TSMI_REQUIRE(output_mask || n_out == 0, "build_masks: null output_mask");
  if (n_in > 0) {
    TSMI_GRID_CHECK(n_in * kvol);
    hipLaunchKernelGGL(fill_kernel<int32_t>, grid_for(n_in * kvol), dim3(kBlock), 0,
                       (hipStream_t)s, input_mask, n_in * kvol, -1);
  }
  if (n_out > 0) {
    TSMI_GRID_CHECK(n_out * kvol);
    hipLaunchKernelGGL(fill_kernel<int32_t>, grid_for(n_out * kvol), dim3(kBlock), 0,
                       (hipStream_t)s, output_mask, n_out * kvol, -1);
  }
  if (nnz > 0) {
    TSMI_REQUIRE(nbmaps_inter && nbaddrs, "build_masks: null pair list");
    TSMI_GRID_CHECK(nnz);
    int skip_k = (n_in == n_out && kvol % 2 == 1) ? kvol / 2 : -1;
    hipLaunchKernelGGL(masks_from_pairs_kernel, grid_for(nnz), dim3(kBlock), 0, (hipStream_t)s,
                       nbmaps_inter, nnz, nbaddrs, kvol, n_in, n_out, skip_k, input_mask,
                       output_mask);
  }
  return check_launch("tsmi_build_masks");
}
