/*
 * tsmi.h — C ABI of libtsmi.so: the MI355X (gfx950) forward sparse-convolution
 * hot path (kernel-map construction, implicit-GEMM / gather-scatter /
 * fetch-on-demand convolution).
 *
 * Every entry point is `extern "C"`, takes plain device pointers and sizes,
 * launches on the HIP stream it is given and returns a status code.  The
 * caller owns (and allocates) every buffer, including scratch; nothing here
 * allocates device memory or synchronises the stream unless stated.  After a
 * non-zero return, tsmi_last_error() describes the failure (thread local).
 *
 * Each declaration cites the interface of the reference (torchsparse v2.1.0,
 * pybind module `torchsparse.backend`, backend/pybind_cuda.cu:29-83) it
 * replaces.  Paths are relative to the reference's torchsparse/backend/.
 *
 * Shared conventions
 *   coords       int32 [N,4] rows (b, x, y, z); -2^17 <= x,y,z < 2^17, 0 <= b < 512
 *   out_in_map   int32 [N_pad, K_vol], -1 = no neighbour, N_pad = ceil128(N_out)
 *   kernel index odd K_vol: x is the fastest digit; even K_vol: z is the fastest
 *   hash table   two caller-owned arrays keys int64[cap], vals int32[cap];
 *                cap must be a multiple of 8; an empty slot has key 0; a stored
 *                key is (packed coordinate or user key) + 1, a stored value is
 *                row index + 1 (the reference's biasing, hashmap_cuda.cuh:13,132)
 *   dtype        TSMI_F32 / TSMI_F16 / TSMI_BF16; 16-bit types accumulate in fp32
 */
#ifndef TSMI_H_
#define TSMI_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

typedef void *tsmi_stream_t; /* a hipStream_t */

enum { TSMI_OK = 0, TSMI_ERR_INVALID_ARGUMENT = 1, TSMI_ERR_RUNTIME = 2, TSMI_ERR_HIP = 3 };
enum { TSMI_F32 = 0, TSMI_F16 = 1, TSMI_BF16 = 2 };

/* ----------------------------------------------------------------- general */

/* Message of the last failure on the calling thread ("" when none).
 * Replaces the C++ exceptions pybind turns into Python errors
 * (std::invalid_argument -> ValueError, std::runtime_error -> RuntimeError). */
const char *tsmi_last_error(void);

/* ABI version of the library (bumped on any signature change). */
int tsmi_version(void);

/* ------------------------------------------------------------- hash table */

/* Empty the table (keys and vals := 0).
 * Replaces torch.zeros for hashmap_keys / hashmap_vals
 * (nn/functional/conv/kmap/func/hashmap_on_the_fly.py:59-67). */
int tsmi_hashtable_clear(tsmi_stream_t s, int64_t *keys, int32_t *vals, int64_t cap);

/* Insert coords[i] -> i+1 for i < n.
 * Replaces subm_hashmap_kmap_stage1 (others/sparsemapping_cuda.cu:129-140) and
 * GPUHashTable::insert_coords (hashmap/hashmap_cuda.cuh:149-169).
 * `status` (device int32[1], pre-zeroed by the caller or NULL) collects two bits: 1 when a
 * key could not be placed because the table is full, 2 when a row cannot be packed into a
 * table key (x, y or z outside [-2^17, 2^17) or batch outside [0, 512)) and was left out.
 * The reference ravels over the measured extents and takes any int32 coordinate
 * (others/sparsemapping_cuda.cu:12-26); a caller that does not check bit 2 gets maps
 * that miss those rows. */
int tsmi_hashtable_insert_coords(tsmi_stream_t s, int64_t *keys, int32_t *vals, int64_t cap,
                                 const int32_t *coords, int64_t n, int32_t *status);

/* Insert user_keys[i] -> i+1.  Replaces GPUHashTable::insert_vals
 * (hashmap/hashmap_cuda.cuh:124-146; wrapper :95-96). */
int tsmi_hashtable_insert_keys(tsmi_stream_t s, int64_t *keys, int32_t *vals, int64_t cap,
                               const int64_t *user_keys, int64_t n, int32_t *status);

/* out[i] = stored value of user_keys[i] (row index + 1) or 0 when absent.
 * Replaces GPUHashTable::lookup_vals (hashmap/hashmap_cuda.cuh:173-196). */
int tsmi_hashtable_lookup_keys(tsmi_stream_t s, const int64_t *keys, const int32_t *vals,
                               int64_t cap, const int64_t *user_keys, int64_t n, int32_t *out);

/* ------------------------------------------------------------- kernel maps */

/* out_in_map[o,k] = i  iff  in_coords[i] == out_coords[o]*stride - pad + digit(k)
 * (same batch), for o < n_out; rows n_out..n_out_pad-1 are written as -1, so the
 * map needs no prior fill.  (keys, vals, cap) index the INPUT coordinates.
 * One entry point covers
 *   build_kernel_map_subm_hashmap stage 2 (others/sparsemapping_cuda.cu:144-231,
 *     host :303-345): out_coords = in_coords, stride 1, pad = (ks-1)/2 for an odd
 *     kernel volume and 0 for an even one;
 *   build_kernel_map_downsample_hashmap stage 3 (:110-126, host :429-507):
 *     pad = the convolution's padding;
 *   GPUHashTable::lookup_coords (hashmap/hashmap_cuda.cuh:199-253): pad = (ks-1)/2. */
int tsmi_kmap_query(tsmi_stream_t s, const int64_t *keys, const int32_t *vals, int64_t cap,
                    const int32_t *out_coords, int64_t n_out, int64_t n_out_pad,
                    const int32_t ks[3], const int32_t stride[3], const int32_t pad[3],
                    int32_t *out_in_map);

/* The same map for the submanifold case of an odd kernel (every ks[a] odd, stride 1,
 * pad = (ks-1)/2) when `coords` are the table's own rows (row i inserted with value i, as
 * tsmi_hashtable_insert_coords does): map[i,k] = j <=> map[j,K_vol-1-k] = i, so half of the
 * offsets are probed and each hit is stored twice.  Fills the map with -1 first (n_pad
 * rows).  Identical output to tsmi_kmap_query for coordinates without duplicates
 * (others/sparsemapping_cuda.cu:144-231 probes all K_vol offsets). */
int tsmi_kmap_query_subm(tsmi_stream_t s, const int64_t *keys, const int32_t *vals, int64_t cap,
                         const int32_t *coords, int64_t n, int64_t n_pad, const int32_t ks[3],
                         int32_t *out_in_map);

/* A whole submanifold map in one call: empty the table and fill the map with -1 (one
 * launch), insert coords[i] -> i+1, query (mirrored for an all-odd kernel, all offsets
 * otherwise; pad = (ks-1)/2 for an odd kernel volume, 0 for an even one).  keys / vals need
 * not be initialised.  `status` as in tsmi_hashtable_insert_coords, except that this call
 * clears it first.  Same table and map, bit
 * for bit, as tsmi_hashtable_clear + tsmi_hashtable_insert_coords + tsmi_kmap_query_subm (or
 * tsmi_kmap_query).  Replaces build_kernel_map_subm_hashmap with to_insert = true
 * (others/sparsemapping_cuda.cu:303-345) together with the torch.zeros of its table
 * (kmap/func/hashmap_on_the_fly.py:59-67). */
int tsmi_kmap_build_subm(tsmi_stream_t s, int64_t *keys, int32_t *vals, int64_t cap,
                         const int32_t *coords, int64_t n, int64_t n_pad, const int32_t ks[3],
                         int32_t *out_in_map, int32_t *status);

/* flags[0] (device int32[1], zeroed by the caller) |= 1 when the rows of coords do not ascend
 * strictly in (b, x, y, z), |= 2 when a row cannot be packed into a table key (see
 * tsmi_hashtable_insert_coords).  What a caller reads once per coordinate tensor to choose
 * between tsmi_kmap_sorted and the hash-table builders; no counterpart in the reference. */
int tsmi_coords_check(tsmi_stream_t s, const int32_t *coords, int64_t n, int32_t *flags);

/* out_in_map[o, k] = i with in_coords[i] == out_coords[o] * stride - pad + digits(k), -1 when
 * there is none — the map of tsmi_kmap_query (same digit order, same padding rows), computed
 * WITHOUT a hash table for inputs whose rows ascend strictly in (b, x, y, z) and are all
 * packable, and outputs that ascend too (out_coords == in_coords for a submanifold map;
 * tsmi_downsample_grid_emit and tsmi_downsample_finalize emit ascending rows): the input row
 * of a target is found by binary search inside a short segment of the input that a block of
 * output rows stages in LDS.  One launch, every entry of the n_out_pad rows written.
 * Replaces build_kernel_map_subm_hashmap and stages 1 and 3 of
 * build_kernel_map_downsample_hashmap (others/sparsemapping_cuda.cu:303-345, 429-507) for
 * such inputs.  tsmi_kmap_sorted_supported: 1 when the kernel size fits the kernel's LDS
 * layout (ks[0] <= 6, ks[1] <= 8, volume <= 7168). */
int tsmi_kmap_sorted_supported(const int32_t ks[3]);
int tsmi_kmap_sorted(tsmi_stream_t s, const int32_t *in_coords, int64_t n_in,
                     const int32_t *out_coords, int64_t n_out, int64_t n_out_pad,
                     const int32_t ks[3], const int32_t stride[3], const int32_t pad[3],
                     const int64_t *samples, int32_t *out_in_map);
/* `count` builds of tsmi_kmap_sorted queued by one call (a network's maps over the levels of a
 * strided chain, built ahead of their use): maps with 2^3 and 3^3 kernels share one launch, up to
 * eight at a time; others get a launch each.  args: host int64[22 * count], per map
 * [in_coords, n_in, out_coords, n_out, n_out_pad, samples (0: none), out_in_map, ks[3],
 * stride[3], pad[3], map_t, n_t_pad, pair_words, pair_out, n_in_dev, n_out_dev] with the pointers as
 * integers.  n_in_dev / n_out_dev (0: none): device int32 that hold the row counts when these are
 * not on the host yet (the rows come out of launches queued just before, tsmi_downsample_chain_rows):
 * n_in, n_out and n_out_pad are then upper bounds that size the launch and the buffers, the kernel
 * works on min(count, bound) rows and pads the map to the next multiple of 128 of the count; only for
 * inputs of at most 131,072 rows (no samples).  map_t .. pair_out are optional products of the same
 * launch (0: not wanted):
 *   map_t int32[n_t_pad * K_vol] (n_t_pad >= n_in), filled with -1 by the caller beforehand:
 *     receives map_t[in, k] = out for every pair found, which makes it the transposed map
 *     (tsmi_transpose_map's result; the reference's others/query_cuda.cu:9-15 after the fill of
 *     conv/hash/query.py:47-55).
 *   pair_words int64[2], zero before the first use and left zero by every launch, and pair_out
 *     int64[1]: receives the number of entries >= 0 of the whole map.
 * No counterpart in the reference. */
int tsmi_kmap_sorted_batch(tsmi_stream_t s, int count, const int64_t *args);
/* Optional for tsmi_kmap_sorted, and only for inputs of more than 131072 rows (smaller ones
 * need none: tsmi_kmap_sorted_samples_elems returns 0): the keys every block of that kernel
 * searches before it stages its segment, gathered once per INPUT into
 * samples int64[tsmi_kmap_sorted_samples_elems(n_in)] — every map over the same input rows
 * (the submanifold and the strided map of a level) can share them.  With samples == NULL the
 * kernel reads the same keys row by row (one cache line per key and block). */
int64_t tsmi_kmap_sorted_samples_elems(int64_t n_in);
int tsmi_kmap_sorted_samples(tsmi_stream_t s, const int32_t *in_coords, int64_t n_in, int64_t *samples);

/* Per-column maximum of non-negative coords -> out_max int32[4] (device).  n may be 0 (result 0).
 * clear_first = 0 when out_max already holds zeros (saves the fill launch).
 * Replaces coords.max(0).values (hashmap_on_the_fly.py:33). */
int tsmi_coords_max(tsmi_stream_t s, const int32_t *coords, int64_t n, int32_t *out_max,
                    int clear_first);

/* Candidate output coordinates of a strided convolution, de-duplicated by inserting
 * them, packed as (b<<54 | x'<<36 | y'<<18 | z') with x' = x + 2^17, into the (empty) OUTPUT table
 * (keys, cap); vals are not touched.  counters (device int32[4], zero on entry):
 * counters[1] is set to 1 if the table overflowed, counters[3] to 1 if an input row or one
 * of its in-range candidates cannot be packed (x, y or z outside [-2^17, 2^17), batch
 * outside [0, 512)) — the reference has no such limit (others/sparsemapping_cuda.cu:12-26)
 * and the caller must treat it as an error.
 *   mode 0: o = (in + pad + digit - (ks-1)) / stride where divisible and
 *           out_min <= o <= out_max per axis — downsample_grid_kmap_stage1_specialized_fast
 *           (others/sparsemapping_cuda.cu:60-107) and get_output_coords_kernel
 *           (others/downsample_cuda.cu:62-141).  When ks == stride and pad == 0 every
 *           input has exactly one candidate, floor(in / stride), and one thread per
 *           input is launched instead of one per (input, offset).
 *   mode 1: o = floor(in / stride), unbounded — spdownsample for stride in {1, ks}
 *           or "minkowski" mode (nn/functional/conv/kmap/downsample.py:30-37).
 *   mode 3: o = clamp(in * stride + digit - (ks-1)/2, 0, out_max_host) for every offset —
 *           the output coordinates of a generative transposed convolution
 *           (nn/functional/conv/kmap/upsample.py:12-41).
 * The upper bound is out_max_host[3] when in_max_dev is NULL, otherwise it is derived on
 * the device as floor((in_max_dev[1+a] + 2*pad - (ks-1)) / stride)
 * (hashmap_on_the_fly.py:33-37).  The lower bound is 0 when in_min_dev is NULL; with
 * in_min_dev (device int32[4], the per-column minima of the input coordinates: negative
 * coordinates allowed) it is (in_min_dev[1+a] - 2*pad + (ks-1)) / stride rounded toward zero
 * (hashmap_on_the_fly.py:39-43), and in_max_dev must then hold the true maxima. */
int tsmi_downsample_candidates(tsmi_stream_t s, const int32_t *in_coords, int64_t n_in,
                               const int32_t ks[3], const int32_t stride[3],
                               const int32_t pad[3], const int32_t out_max_host[3],
                               const int32_t *in_max_dev, const int32_t *in_min_dev, int mode,
                               int64_t *keys, int64_t cap, int32_t *counters);

/* Gather the non-empty slots of a table: stored_keys_out[0..count) = the stored keys
 * (key + 1) in arbitrary order, *count_out (device int32, zero on entry) += their
 * number.  Together with tsmi_sort_keys this is the de-duplicated, sorted candidate
 * list torch::_unique returns (others/sparsemapping_cuda.cu:478); a compaction with
 * one atomic per workgroup replaces the reference's one-atomic-per-candidate append
 * (others/sparsemapping_cuda.cu:103-105). */
int tsmi_hashtable_compact_keys(tsmi_stream_t s, const int64_t *keys, int64_t cap,
                                int64_t *stored_keys_out, int32_t *count_out);

/* Bytes of scratch tsmi_sort_keys / tsmi_argsort_desc need for n items. */
int64_t tsmi_sort_temp_bytes(int64_t n);

/* Ascending sort of n int64 keys (bits [0,end_bit) significant).
 * Replaces torch::_unique's sort (others/sparsemapping_cuda.cu:478). */
int tsmi_sort_keys(tsmi_stream_t s, const int64_t *keys_in, int64_t *keys_out, int64_t n,
                   int end_bit, void *temp, int64_t temp_bytes);

/* Unpack sorted unique STORED keys (key + 1, as tsmi_hashtable_compact_keys emits
 * them) into out_coords int32[n_out,4] and store row+1 as the value of each key in
 * the OUTPUT table.  Replaces
 * inverse_transform_coords_and_insert_kernel (others/sparsemapping_cuda.cu:44-57). */
int tsmi_downsample_finalize(tsmi_stream_t s, const int64_t *sorted_keys, int64_t n_out,
                             const int64_t *keys, int32_t *vals, int64_t cap,
                             int32_t *out_coords);

/* Output coordinates of a strided convolution through an occupancy bitmap of the output
 * grid: the same result as tsmi_downsample_candidates (mode 0) + compact + sort + finalize
 * when every coordinate is non-negative and the grid (batches x extents) has at most
 * 32 * bitmap_words cells; no hash insertion of candidates and no sort.  Replaces
 * downsample_cuda's candidate / unique passes (others/downsample_cuda.cu:147-190,
 * others/sparsemapping_cuda.cu:429-507).
 *
 * tsmi_downsample_grid_count marks the bitmap (after clearing the part THIS call uses when
 * clear_first is set, for callers that pass uninitialised scratch every time; otherwise the
 * caller guarantees it is all zero) and counts its set bits:
 * counters[0] = number of outputs, counters[2] = 1 when the grid does not fit (nothing is
 * then marked and the caller takes the sorting path), counters[3] = 1 when an input row or
 * an in-range candidate cannot be packed into a table key (as in tsmi_downsample_candidates;
 * the caller zeroes counters[3] before the call).  next_in_max_dev, when given, is a
 * zero-filled device int32[4] that receives the per-column maximum of the outputs (what
 * tsmi_coords_max would find over out_coords).  in_max_dev is the device int32[4]
 * per-column maximum of in_coords (tsmi_coords_max); out_max_host, when given, bounds the
 * three spatial axes instead.  bitmap int32[bitmap_words] (16-byte aligned, a multiple of
 * 512 words, at most 2^25) and chunk_counts int32[bitmap_words / 512] are scratch that
 * tsmi_downsample_grid_emit reads back: it writes out_coords int32[n_out,4] in ascending
 * (b,x,y,z) order, inserts coordinate -> row + 1 into the EMPTY output table
 * (keys, vals, cap; counters[1] = 1 if the table was too small; keys == NULL: no table) and leaves the bitmap
 * all zero again, so that one bitmap can serve call after call without clear_first.
 * in_max_host, when given, is a host copy of in_max_dev (read back with the counters): the
 * extents are then computed on the host and only the chunks inside the grid are launched.
 * Chains without a read-back in between: tsmi_downsample_grid_emit with n_out = -capacity
 * emits every set bit into out_coords int32[capacity, 4] while the count is still on the
 * device (no table; capacity >= the count, e.g. the number of inputs when every input has one
 * output), and tsmi_downsample_grid_count with n_in_dev (device int32[1], e.g. counters[0] of
 * the previous level; n_in is then the capacity of in_coords) marks from such rows.  NULL:
 * n_in rows. */
int tsmi_downsample_grid_count(tsmi_stream_t s, const int32_t *in_coords, int64_t n_in,
                               const int32_t ks[3], const int32_t stride[3], const int32_t pad[3],
                               const int32_t out_max_host[3], const int32_t *in_max_dev,
                               int32_t *bitmap, int64_t bitmap_words, int clear_first,
                               int32_t *chunk_counts, int32_t *counters, int32_t *next_in_max_dev,
                               const int32_t *n_in_dev);
/* The next level of a chain of strided convolutions with the same geometry, before the
 * previous level's outputs exist as rows: the inputs are the set bits of the previous
 * level's bitmap (marked by tsmi_downsample_grid_count / _count_next with next_in_max_dev =
 * this call's in_max_dev, a zero-filled device int32[4] that receives the per-column maximum
 * of the outputs; prev_in_max_dev is the in_max_dev of that call).  Same outputs in counters,
 * bitmap and chunk_counts as tsmi_downsample_grid_count; a level whose predecessor did not fit
 * marks nothing.  No counterpart in the reference, which reads the number of outputs back
 * after every level (others/sparsemapping_cuda.cu:477-479); with this entry one read-back
 * serves the whole chain. */
int tsmi_downsample_grid_count_next(tsmi_stream_t s, const int32_t ks[3], const int32_t stride[3],
                                    const int32_t pad[3], const int32_t *prev_in_max_dev,
                                    const int32_t *prev_bitmap, int64_t prev_bitmap_words,
                                    const int32_t *in_max_dev, int32_t *bitmap, int64_t bitmap_words,
                                    int32_t *chunk_counts, int32_t *counters,
                                    int32_t *next_in_max_dev);
int tsmi_downsample_grid_emit(tsmi_stream_t s, const int32_t ks[3], const int32_t stride[3],
                              const int32_t pad[3], const int32_t out_max_host[3],
                              const int32_t *in_max_dev, const int32_t *in_max_host,
                              int32_t *bitmap, int64_t bitmap_words, const int32_t *chunk_prefix, int64_t n_out, int64_t *keys,
                              int32_t *vals, int64_t cap, int32_t *out_coords, int32_t *counters);

/* A whole chain of `levels` equal strided layers with one output per input (kernel size ==
 * stride, no padding) queued by one call.  The outputs of level l are the cells of the ROOT's
 * rows carried down l + 1 layers (a row drops out where a layer's rule leaves its output out:
 * beyond floor((max - (ks - 1)) / stride) of that layer's inputs), so no level needs the rows
 * of the one before, only the maxima of its inputs: tsmi_coords_max over coords, one launch per
 * level that marks its bitmap from the root's rows and raises the maxima of the next level, then
 * one launch that counts the chunks of every level, one that scans them (the counters are
 * complete), one that emits every level's rows and clears the bitmaps: levels + 4 launches.
 * phase 0: all of them; 1: up to the counters (what a caller copies to the host); 2: the rows
 * (after phase 1 with the same arguments, on the same stream).  scratch is the int32 buffer that
 * holds every level's bitmap (at word bitmap_at[level], a multiple of 4, bitmap_words[level]
 * words, all zero on entry and after phase 2) and chunk counts (at word chunks_at[level]); the
 * three arrays are host int64[levels].  counters: zero-filled device int32[8 * levels], per level
 * [n_out, -, grid too large, unpackable, maxima (b, x, y, z) of the level's INPUT rows]; rows:
 * device int32[levels, n, 4], level i's first counters[8 i] rows are its output coordinates in
 * ascending order.  A level whose grid does not fit its bitmap is flagged and leaves no rows, nor
 * do the levels after it.  Nothing is read back.  No counterpart in the reference, which builds
 * level after level with a read-back each (others/sparsemapping_cuda.cu:429-507, called once per
 * strided layer). */
int tsmi_downsample_chain_rows(tsmi_stream_t s, const int32_t *coords, int64_t n,
                               const int32_t ks[3], const int32_t stride[3], const int32_t pad[3],
                               int levels, int32_t *scratch, const int64_t *bitmap_at,
                               const int64_t *bitmap_words, const int64_t *chunks_at,
                               int32_t *counters, int32_t *rows, int phase);

/* map_t[in,k] = out for every map[out,k] = in >= 0, out < n_rows; map_t
 * [n_rows_t, K_vol] is filled with -1 first.  Replaces
 * convert_transposed_out_in_map (others/query_cuda.cu:9-15,50-54) plus the
 * torch.full of nn/functional/conv/hash/query.py:47-55. */
int tsmi_transpose_map(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                       int32_t *map_t, int64_t n_rows_t);

/* bitmask[s,r] = sum_i (map[r, s*L+i] >= 0) << i for r < valid_n, -1 for padding
 * rows; L = ceil(K_vol/split) (must be <= 32).  Replaces
 * derive_bitmask_from_out_in_map (others/query_cuda.cu:17-31,59-65). */
int tsmi_derive_bitmask(tsmi_stream_t s, const int32_t *map, int64_t n_pad, int kvol,
                        int split, int64_t valid_n, int32_t *bitmask);

/* Descending (signed) sort of each of `rows` rows of keys_in int32[rows,n]:
 * keys_out = sorted values, idx_out = source positions.  Ties keep no particular
 * order.  Replaces torch.sort(bitmask, descending=True) (hashmap_on_the_fly.py:96). */
int tsmi_argsort_desc(tsmi_stream_t s, const int32_t *keys_in, int32_t *keys_out,
                      int32_t *idx_out, int rows, int64_t n, void *temp, int64_t temp_bytes);

/* out[r,c] = map[reorder_loc[c / L, r], c].  Replaces reorder_out_in_map_cuda
 * (others/reorder_map_cuda.cu:8-48). */
int tsmi_reorder_map(tsmi_stream_t s, const int32_t *map, const int32_t *reorder_loc,
                     int64_t n_pad, int kvol, int split, int32_t *out);

/* reduced[s,t] = OR of sorted_mask[s, t*tile .. (t+1)*tile-1]; tile % 4 == 0.
 * Replaces reduce_bitmask_cuda (others/reduce_bitmask_cuda.cu:13-84). */
int tsmi_reduce_bitmask(tsmi_stream_t s, const int32_t *sorted_mask, int split,
                        int64_t n_pad, int tile, int32_t *reduced);

/* Pair lists, phase 1: per-offset counts.  nbsizes int32[K_vol] := number of
 * rows < n_rows with map[row,k] != -1; block_counts int32[K_vol * nblk] is
 * scratch for phase 2, nblk = ceil(n_rows / 256).  K_vol <= 512.  Replaces
 * torch.sum(results != -1, dim=1) (hashmap_on_the_fly.py:139,186). */
int tsmi_pair_lists_count(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                          int32_t *block_counts, int32_t *nbsizes);

/* Pair lists, phase 2 (after phase 1 on the same stream).  Pairs are ordered by
 * (k, out).  Any of the outputs may be NULL:
 *   nbmaps_inter int32[nnz,2] rows (in,out)     — GatherScatter layout (:141-143)
 *   nbmaps_planar int32[2,nnz] all in, then out — FetchOnDemand layout (:187-200)
 *   input_mask int32[K_vol*n_in], output_mask int32[K_vol*n_out]: position of the
 *     pair inside offset k's list (pre-filled with -1 here).  Offset mask_skip_k is left
 *     out of the masks: the identity offset of an odd-volume submanifold map, whose pair
 *     list needs no look-up (-1: none).  -2 applies the reference's rule, the centre
 *     offset whenever the volume is odd and n_in == n_out — build_mask_from_kmap
 *     (others/sparsemapping_cuda.cu:235-256,510-548) — which also fires for a strided
 *     map that happens to have as many outputs as inputs.
 * nbsizes is phase 1's (device); nnz is its sum (the caller read it back to size the
 * arrays). */
int tsmi_pair_lists_fill(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                         int32_t *block_counts, const int32_t *nbsizes, int64_t nnz,
                         int32_t *nbmaps_inter, int32_t *nbmaps_planar, int64_t n_in,
                         int64_t n_out, int mask_skip_k, int32_t *input_mask, int32_t *output_mask);

/* input_mask / output_mask (see tsmi_pair_lists_fill) from an existing interleaved
 * pair list and nbaddrs = exclusive scan of its per-offset sizes.  Replaces
 * build_mask_from_kmap (others/sparsemapping_cuda.cu:235-256,510-548). */
int tsmi_build_masks(tsmi_stream_t s, const int32_t *nbmaps_inter, int64_t nnz,
                     const int32_t *nbaddrs, int kvol, int64_t n_in, int64_t n_out,
                     int32_t *input_mask, int32_t *output_mask);

/* nbaddrs / qnbaddrs int32[K_vol+1]: exclusive scans of nbsizes and of nbsizes
 * rounded up to q.  Replaces exclusive_scan_quantified_wrapper
 * (others/exclusive_scan_cuda.cu:7-45). */
int tsmi_exclusive_scan_quantified(tsmi_stream_t s, int kvol, const int32_t *nbsizes, int q,
                                   int32_t *nbaddrs, int32_t *qnbaddrs);

/* ------------------------------------------------------------ convolutions */

/* Elements of the packed-weight buffer for a [K_vol, Cin, Cout] kernel. */
int64_t tsmi_packed_weight_elems(int kvol, int cin, int cout);

/* Re-lay a [K_vol, Cin, Cout] kernel as [K_vol, Cout_pad, Cin_pad] (reduction
 * axis contiguous, zero padded to multiples of 16 / 32) for the MFMA kernels.
 * No counterpart in the reference (its kernels read [K_vol,Cin,Cout] directly). */
int tsmi_pack_weights(tsmi_stream_t s, const void *w, void *w_packed, int kvol, int cin,
                      int cout, int dtype);

/* Floats of scratch the implicit-GEMM entry points want for a problem of
 * n_tile_rows map rows (n_out for the unsorted call, n_pad and sorted = 1 for the
 * sorted one) and `split` mask splits; 0 when none is needed.  Small problems cut the kernel offsets
 * into ranges that run as separate workgroups and add their fp32 partial sums, the
 * role split-K plays in the reference's wgrad kernels
 * (convolution/convolution_backward_wgrad_implicit_gemm_cuda.cu:1614-2042). */
int64_t tsmi_conv_workspace_elems(int64_t n_tile_rows, int64_t n_out, int kvol, int split,
                                  int cin, int cout, int dtype, int sorted);

/* Y[i,:] = sum_k [m = map[i,k] >= 0] X[m,:] W[k] (+ bias) for i < n_out; every
 * output row is written.  `map` has at least n_out rows.  `workspace` (float
 * [workspace_elems], may be NULL) enables the offset split described above.
 * `tile_counters` (int32 [n_tile_counters], may be NULL) lets the workgroup that
 * finishes a tile's last partial sum add them up itself instead of a second
 * launch: the array must be all zero on entry and is all zero again when the
 * launch completes, so one zero-filled array can serve every call on a stream
 * (calls that overlap on the GPU must not share it); 4096 entries cover every
 * problem that is split.
 * Epilogue, shared by every convolution entry point: y = act(sum + bias +
 * residual), with bias [cout] and residual [n_out, cout] of the I/O type (either
 * may be NULL) and act = max(., 0) when relu != 0 — the bias add of
 * nn/functional/conv/conv.py:123-124 and the BatchNorm-folded / ReLU / shortcut
 * adds of the residual blocks, fused into the producing kernel.
 * Replaces conv_forward_implicit_gemm_cuda
 * (convolution/convolution_forward_implicit_gemm_cuda.cu:1527-1986). */
int tsmi_conv_implicit_gemm(tsmi_stream_t s, const void *x, const void *w_packed,
                            const int32_t *map, int64_t n_map_rows, int64_t n_out, int kvol,
                            int cin, int cout, int dtype, const void *bias, const void *residual,
                            int relu, float *workspace, int64_t workspace_elems,
                            int32_t *tile_counters, int64_t n_tile_counters, void *y);

/* Same sum over a row-sorted map: tile row r of split s reads
 * reorder_map[r, s*L..] and adds into output row reorder_loc[s, r].
 * `workspace` (tsmi_conv_workspace_elems floats; required for split > 1) receives
 * the per-split fp32 sums, which are then added into y; tile_counters as above
 * (used when split == 1).  reduced_mask may be NULL
 * (the kernel derives its skipping from the map itself).  Replaces
 * conv_forward_implicit_gemm_sorted_cuda
 * (convolution/convolution_forward_implicit_gemm_sorted_cuda.cu:1755-2230). */
int tsmi_conv_implicit_gemm_sorted(tsmi_stream_t s, const void *x, const void *w_packed,
                                   const int32_t *reorder_map, const int32_t *reduced_mask,
                                   const int32_t *reorder_loc, int64_t n_pad, int64_t n_out,
                                   int kvol, int split, int cin, int cout, int dtype,
                                   const void *bias, const void *residual, int relu,
                                   float *workspace, int64_t workspace_elems,
                                   int32_t *tile_counters, int64_t n_tile_counters, void *y);

/* Weight gradient: dw[k][c][n] = sum_i [m = map_bwd[i,k] >= 0] x[i][c] * dy[m][n], with
 * map_bwd int32 [n_map_rows >= n_in, K_vol] the transposed kernel map (tsmi_transpose_map
 * of the forward map: input row, offset -> output row), dy [n_out, cout] and dw
 * [K_vol, cin, cout] of the I/O type, fp32 accumulation.  `workspace` holds
 * tsmi_conv_wgrad_workspace_elems floats (per-split partial sums, added by a second
 * launch).  The input gradient needs no entry point of its own: it is
 * tsmi_conv_implicit_gemm over map_bwd with the weights transposed per offset
 * (nn/functional/conv/func/implicit_gemm.py:171-180).  Replaces
 * conv_backward_wgrad_implicit_gemm_cuda
 * (convolution/convolution_backward_wgrad_implicit_gemm_cuda.cu:1614-2042), which
 * returns the same sums as [K_vol*cout, cin]. */
int64_t tsmi_conv_wgrad_workspace_elems(int64_t n_in, int kvol, int cin, int cout, int dtype);
int tsmi_conv_wgrad(tsmi_stream_t s, const void *x, const void *dy, const int32_t *map_bwd,
                    int64_t n_map_rows, int64_t n_in, int kvol, int cin, int cout, int dtype,
                    float *workspace, int64_t workspace_elems, void *dw);

/* Weight gradient over pair lists.  tsmi_wgrad_pairs_build turns a kernel map (int32
 * [n_rows, K_vol], -1 = none) into per-offset lists of (map value, row) pairs ordered by
 * row: offset k's list starts at entry 32 * seg_steps[k] of `pairs` and is padded with
 * (-1, -1) to a multiple of 32 entries; seg_steps int32[K_vol + 1] counts those blocks of
 * 32, nbsizes int32[K_vol] the pairs themselves.  `pairs` holds
 * tsmi_wgrad_pairs_capacity(n_rows, K_vol) entries of two int32 (only the part the lists
 * need is written), block_counts is scratch of K_vol * ceil(n_rows / 256) int32.  Nothing
 * is read back to the host.  K_vol <= 511.
 *
 * tsmi_conv_wgrad_pairs: dw[k][c][n] = sum over offset k's pairs of x[a][c] * dy[b][n],
 * a = pair[x_col], b = pair[1 - x_col] (x_col 0: the map values index x, as in a forward
 * map out_in_map[out, k] = in; x_col 1: the rows index x, as for a transposed
 * convolution over the same map).  Only rows that take part in an offset are read.  cin
 * and cout must be multiples of 16 bytes of elements (other widths: tsmi_conv_wgrad).
 * `workspace` holds tsmi_conv_wgrad_pairs_workspace_elems floats; pair_cap is the
 * capacity `pairs` was built with.  Same sums as conv_backward_gather_scatter_cuda's
 * grad_kernel (convolution/convolution_gather_scatter_cuda.cu:815-915) and as
 * conv_backward_wgrad_implicit_gemm_cuda, accumulated in fp32.
 *
 * tsmi_wgrad_pairs_pad makes the same padded lists from pair lists that already exist
 * (nbmaps_inter int32[nnz,2], offset k's nbsizes[k] pairs one after the other, as the
 * gather-scatter dataflow holds them); `pairs` then needs nnz + 31 * K_vol entries. */
int64_t tsmi_wgrad_pairs_capacity(int64_t n_rows, int kvol);
int tsmi_wgrad_pairs_pad(tsmi_stream_t s, const int32_t *nbmaps_inter, int64_t nnz,
                         const int32_t *nbsizes, int kvol, int32_t *pairs, int32_t *seg_steps);
int tsmi_wgrad_pairs_build(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                           int32_t *block_counts, int32_t *nbsizes, int32_t *pairs,
                           int32_t *seg_steps);
/* tsmi_wgrad_pairs_build without the caller's scratch buffer, for callers that cannot
 * allocate device memory (code under HIP graph capture, serving loops and harnesses that
 * forbid hipMalloc).  It has no counterpart in the reference.  The per-block counts live in
 * an array built into the library (4 MiB of device memory on every GPU the library runs
 * on, held until the process ends); inputs and outputs are still the caller's.  Limit:
 * K_vol * ceil(n_rows / 256) <= 1,048,576 (e.g. 9.9M map rows at K_vol = 27), otherwise
 * TSMI_ERR_INVALID_ARGUMENT.  The call allocates nothing; its first call on a device looks
 * the array's address up (hipGetSymbolAddress) and should therefore happen outside stream
 * capture.  All calls on one GPU share the array: calls that overlap on one GPU (two
 * streams, two threads) race, calls queued on one stream do not.  Same outputs, bit for
 * bit, as tsmi_wgrad_pairs_build. */
int tsmi_wgrad_pairs_build_static(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                                  int32_t *nbsizes, int32_t *pairs, int32_t *seg_steps);
int64_t tsmi_conv_wgrad_pairs_workspace_elems(int64_t pair_cap, int kvol, int cin, int cout,
                                              int dtype);
int tsmi_conv_wgrad_pairs(tsmi_stream_t s, const void *x, const void *dy, const int32_t *pairs,
                          const int32_t *seg_steps, int64_t pair_cap, int x_col, int kvol, int cin,
                          int cout, int dtype, float *workspace, int64_t workspace_elems, void *dw);

/* Fetch-on-demand: one launch over 128-padded pair lists gathers X rows, multiplies
 * by W[k] and writes partial[qnbaddrs[k] + p, :] (fp32 for TSMI_F32, else the I/O
 * type); a second launch sums the partials of each output row through output_mask
 * (atomic free).  `transpose` swaps the roles of the two pair columns; row_mask is
 * the output_mask (input_mask when transposed).  center_k >= 0 names an offset
 * whose pair list is the identity (p-th pair = (p, p)) and which the masks skip:
 * the centre of an odd-volume submanifold map; -1 otherwise.  `partial` holds
 * nnz x cout elements of the I/O type.
 * Replaces conv_forward_fetch_on_demand_cuda
 * (convolution/convolution_forward_fetch_on_demand_cuda.cu:1981-2119). */
int tsmi_conv_fetch_on_demand(tsmi_stream_t s, const void *x, const void *w_packed,
                              const int32_t *nbmaps_planar, int64_t nnz,
                              const int32_t *nbaddrs, const int32_t *qnbaddrs, int64_t qnnz,
                              const int32_t *row_mask, int64_t n_out, int kvol, int cin,
                              int cout, int dtype, int transpose, int center_k,
                              const void *bias, const void *residual, int relu, void *partial,
                              void *y);

/* Convolution over pair segments: the form the implicit-GEMM dataflow takes on small, wide
 * layers (a few thousand to a few ten thousand rows, 128 or more channels), where a dense
 * pass over all K_vol offsets of every row tile would stream the whole weight tensor once
 * per tile.  tsmi_pair_segments compacts the pairs of a kernel map (int32 [n_rows, K_vol],
 * negative = none) per kernel offset, in one launch and without a host read-back:
 * in_rows[k * seg_rows + j] = map value of the j-th pair of offset k, pos[k * n_rows + row] =
 * j (-1: the row has no pair at k), counts[k] = pairs of offset k.  seg_rows >= n_rows is the
 * fixed capacity of a segment (a multiple of 64 for the convolution below); in_rows holds
 * K_vol * seg_rows int32 (only the first counts[k] of a segment are written), pos
 * K_vol * n_rows, counts K_vol.  The order of the pairs inside a segment is not fixed
 * (blocks reserve their share with an atomic add); pos names each pair's place, and every
 * result computed through the two arrays is the same whatever the order.  `pool`: NULL, or
 * K_vol + 1 int32 that are zero on entry and zero again when the call has run (the blocks
 * add up there and the last one moves the sums into `counts`); with NULL `counts` is cleared
 * by a launch of its own first.  Calls that share a pool must not overlap.
 * tsmi_conv_implicit_gemm_segments: products[k * seg_rows + j, :] = X[in_rows[k * seg_rows + j], :]
 * W[k] for j < counts[k] (one launch: a workgroup takes a run of 64-pair tiles and keeps the
 * weights of their offset in registers), then Y[o, :] = sum over k of products[k * seg_rows +
 * pos[k * n_out + o], :] + bias + residual, optional ReLU (second launch; fp32 sums in the
 * order of k, atomic free).  `products` holds K_vol * seg_rows * cout elements of the I/O
 * type, of which only the rows of existing pairs are touched.  tsmi_conv_segments_supported:
 * 1 for the shapes that have a variant (fp16 / bf16, K_vol <= 64, cin one of 128, 192, 256,
 * 384, cout a multiple of 8).  Same sums as conv_forward_implicit_gemm_cuda
 * (convolution/convolution_forward_implicit_gemm_cuda.cu:1527-1986) with the per-offset
 * products rounded to the I/O type as conv_forward_fetch_on_demand_cuda's are
 * (convolution/convolution_forward_fetch_on_demand_cuda.cu:1981-2119). */
int tsmi_conv_segments_supported(int kvol, int cin, int cout, int dtype);
int tsmi_pair_segments(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol,
                       int64_t seg_rows, int32_t *pool, int32_t *counts, int32_t *in_rows,
                       int32_t *pos);
/* `count` calls of tsmi_pair_segments queued by one (the segments of several maps of a network,
 * built ahead of their layers): args is host int64[8 * count], per build [map, n_rows, kvol,
 * seg_rows, pool, counts, in_rows, pos] with the pointers as integers.  The builds run one after
 * the other on the stream and may share a pool. */
int tsmi_pair_segments_batch(tsmi_stream_t s, int count, const int64_t *args);
int tsmi_conv_implicit_gemm_segments(tsmi_stream_t s, const void *x, const void *w_packed,
                                     const int32_t *in_rows, const int32_t *counts,
                                     const int32_t *pos, int64_t seg_rows, int64_t n_out, int kvol,
                                     int cin, int cout, int dtype, const void *bias,
                                     const void *residual, int relu, void *products, void *y);

/* Implicit GEMM over a 3x3x3 map whose rows are grouped by the kernel planes they use - the
 * counterpart of the reference's mask-sorted dataflow (bitmask -> sort -> reordered map,
 * nn/functional/conv/kmap/func/hashmap_on_the_fly.py:92-107, and
 * convolution/convolution_forward_implicit_gemm_sorted_cuda.cu:94-95,341-342, which skips
 * the offsets a 128-row tile does not use) without its device sort.
 * tsmi_map_group_rows: inside windows of `window` consecutive rows (a multiple of 128, at
 * most 8192) the rows of `map` (int32 [>= n_rows, 27], negative = none) are counting-sorted
 * by the outer planes of the kernel that hold a neighbour (digit 0 or 2 along each axis: six
 * bits; key = rank of the number of offsets those planes span << 6 | bits, ascending, so the
 * rows with the most offsets end a window).  With P = tsmi_map_group_rows_padded(n_rows,
 * window) = ceil(n_rows / window) * window positions (-1: bad sizes): grouped[p, :] =
 * map[row_of[p], :] and row_of[p] = the row at position p (int32 [P, 27] and [P]; -1 and an
 * all -1 map row for the padding positions behind n_rows); masks64[t] (int32 [P / 64]) = the
 * union, bit k per kernel offset, of the offsets the rows at positions 64 t .. 64 t + 63 use;
 * order64 (int32 [8 ceil(P / 512)]) / order128 (int32 [8 ceil(P / 1024)]) = the order in which a
 * convolution starts the T = P / 64 (P / 128) tiles of 64 (128) rows: the tiles are cut into 8 runs
 * of S = ceil(T / 8) consecutive ones, one per XCD (workgroup b runs on XCD b % 8), and
 * order[8 j + c] = the tile of run c with the j-th most offsets (-1: the run has no such
 * tile).  Two launches, no host read-back; the order of
 * equal keys (and of tiles with equally many offsets) is not fixed, and what the convolution
 * below computes is the same bit for bit whatever it is.
 * tsmi_conv_implicit_gemm_grouped: Y[row_of[p], :] = sum over k of X[grouped[p, k], :] W[k]
 * + bias + residual, optional ReLU - tsmi_conv_implicit_gemm's sums, row by row - with one
 * workgroup per row tile, started in the listed order: on every XCD the long tiles first, the
 * short ones fill the machine behind them.  n_grouped = P. */
int64_t tsmi_map_group_rows_padded(int64_t n_rows, int window);
int tsmi_map_group_rows(tsmi_stream_t s, const int32_t *map, int64_t n_rows, int kvol, int window,
                        int32_t *grouped, int32_t *row_of, int32_t *masks64, int32_t *order64,
                        int32_t *order128);
int tsmi_conv_implicit_gemm_grouped(tsmi_stream_t s, const void *x, const void *w_packed,
                                    const int32_t *grouped_map, const int32_t *row_of,
                                    const int32_t *order64, const int32_t *order128,
                                    int64_t n_grouped, int64_t n_out, int kvol, int cin, int cout,
                                    int dtype, const void *bias, const void *residual, int relu,
                                    void *y);

/* tsmi_conv_implicit_gemm, tsmi_conv_implicit_gemm_segments and tsmi_conv_implicit_gemm_grouped
 * with their arguments in one block of host int64, in the order of the declarations above
 * (pointers and the stream as integers: 18, 17 and 17 entries) followed by three entries that
 * place the result: [ldy, y2, ldy2] - the calls a forward makes most often, about 60 per forward
 * of a U-Net, for bindings that pay per argument (ctypes converts one in 0.1 us).
 *   ldy   row pitch of y in elements (0: cout, a dense result); a multiple of 8 that holds a row
 *   y2    optional second destination of the same rows (0: none), 16-byte aligned, row pitch ldy2
 * With them a layer writes into a column slice of a wider buffer, and a layer whose result a
 * later concatenation would copy writes it there as well: torch.cat([a, b], 1) of two layers'
 * results (the decoder of a U-Net, the reference's backbones/unet.py:99-103) costs no launch.
 * All three zero: same checks, same launches, same status as the unpacked call.  Calls that would
 * finish their rows in a second launch (the offset split without tile counters) refuse a placed
 * result.  No counterpart in the reference (pybind11 converts its arguments in compiled code). */
int tsmi_conv_implicit_gemm_packed(const int64_t *args);          /* 21 entries */
int tsmi_conv_implicit_gemm_segments_packed(const int64_t *args); /* 20 entries */
int tsmi_conv_implicit_gemm_grouped_packed(const int64_t *args);  /* 20 entries */

/* A launch thread for the convolution calls of a forward (no counterpart in the reference, whose
 * calls are made one by one from the interpreter's thread).  Between _open and _close the three
 * packed convolution calls can be handed to one worker thread, which carries them out in the order
 * they were handed over while the caller prepares the next call: a call costs its caller ~0.5 us
 * instead of ~5.
 *   tsmi_launch_thread_submit(kind, args, n_words): kind 0 / 1 / 2 = tsmi_conv_implicit_gemm_packed
 *     / _segments_packed / _grouped_packed with the same argument block (copied).  Returns the
 *     call's ticket (> 0), or -1 when no region is open (make the call yourself then).
 *   tsmi_launch_thread_completed(): address of an int64 that holds the ticket of the last call
 *     carried out.  The buffers of a submitted call must stay allocated until it has reached the
 *     call's ticket.
 *   tsmi_launch_thread_flush(): returns once every submitted call has been carried out, with the
 *     status of the first that failed since the last flush (its message in tsmi_last_error()).
 *     The ONLY ordering between submitted calls and anything else the caller queues on the same
 *     streams (other entry points of this library, the framework's kernels, event records):
 *     flush before queuing whatever reads a submitted call's result or overwrites its operands.
 *   tsmi_launch_thread_close(): flush, then the region ends.
 * Regions nest and may be opened by several host threads; calls handed over by one thread keep
 * their order.  Not for streams that are being captured into a graph. */
int tsmi_launch_thread_open(void);
int64_t tsmi_launch_thread_submit(int kind, const int64_t *args, int n_words);
const int64_t *tsmi_launch_thread_completed(void);
int tsmi_launch_thread_flush(void);
int tsmi_launch_thread_close(void);

/* Gather-GEMM-scatter, step 1: buffer[nbaddrs[k] + p, :] = X[in(k,p), :].
 * Replaces gather_all_kernel_pad_sep_with_mask / gather_kernel
 * (convolution/convolution_gather_scatter_cuda.cu:17-40,70-112). */
int tsmi_gs_gather(tsmi_stream_t s, const void *x, const int32_t *nbmaps_inter, int64_t nnz,
                   int cin, int dtype, int transpose, void *buffer);

/* Gather-GEMM-scatter, step 2: out_buffer[p,:] = buffer[p,:] W[k(p)] for every pair,
 * one launch for all offsets (qnbaddrs / qnnz: the 128-padded scan that maps a
 * workgroup to its offset).  Replaces the torch::mm_out / bmm_out groups
 * (convolution/convolution_gather_scatter_cuda.cu:597-673). */
int tsmi_gs_gemm(tsmi_stream_t s, const void *buffer, const void *w_packed,
                 const int32_t *nbaddrs, const int32_t *qnbaddrs, int64_t nnz, int64_t qnnz,
                 int kvol, int cin, int cout, int dtype, void *out_buffer);

/* Gather-GEMM-scatter, step 3: Y[o,:] = sum_k out_buffer[nbaddrs[k] + mask[k,o], :]
 * (+ bias), atomic free.  Replaces scatter_all_kernel_pad_sep_with_mask_{half,float}
 * (convolution/convolution_gather_scatter_cuda.cu:150-250). */
int tsmi_gs_scatter(tsmi_stream_t s, const void *out_buffer, const int32_t *nbaddrs,
                    const int32_t *row_mask, int64_t n_out, int kvol, int cout, int dtype,
                    int center_k, const void *bias, const void *residual, int relu, void *y);

/* ------------------------------------------------------ point-voxel operators
 * Row tensors are [rows, c] of dtype TSMI_F32 / TSMI_F16 / TSMI_BF16, sums run in fp32.
 * Rows are moved 16 bytes per thread when c is a multiple of 16 bytes of elements and the
 * tensors are 16-byte aligned, element by element otherwise. */

/* out[i] = 64-bit FNV-1a hash of the four int32 fields of coords[i] (no 60-bit fold).
 * Replaces hash_cuda (hash/hash_cuda.cu:9-22,64-70). */
int tsmi_hash_coords(tsmi_stream_t s, const int32_t *coords, int64_t n, int64_t *out);

/* out[k*n + i] = hash of (coords[i,0], coords[i,1:4] + offsets[k]); offsets int32[kvol,3] on
 * the device, out int64[kvol,n].  Replaces kernel_hash_cuda (hash/hash_cuda.cu:26-57,72-83). */
int tsmi_kernel_hash(tsmi_stream_t s, const int32_t *coords, int64_t n, const int32_t *offsets,
                     int kvol, int64_t *out);

/* out[v] = number of i with idx[i] == v for v in [0, num); other indices are skipped.  `out`
 * is cleared here.  Replaces count_cuda (others/count_cuda.cu:10-31). */
int tsmi_count(tsmi_stream_t s, const int32_t *idx, int64_t n, int32_t *out, int num);

/* Grouping of an index array, the preparation of the two row sums below: `order` int32[m]
 * receives the positions e of idx with 0 <= idx[e] < n_groups sorted by (idx[e], e) — only the
 * first starts[n_groups] entries are meaningful — and starts int32[n_groups + 1] the beginning of
 * every group's run.  `temp` holds tsmi_group_temp_bytes(m) bytes.  A radix sort over the bits
 * n_groups needs plus one binary search per group; no host read-back.  No counterpart in the
 * reference, which adds with atomicAdd instead. */
int64_t tsmi_group_temp_bytes(int64_t m);
int tsmi_group_by_index(tsmi_stream_t s, const int32_t *idx, int64_t m, int64_t n_groups, void *temp,
                        int64_t temp_bytes, int32_t *order, int32_t *starts);

/* out[v,:] = (sum of feats[i,:] over the points i of voxel v) / counts[v], zero when counts[v]
 * is 0; (order, starts) = tsmi_group_by_index of the points' voxel indices idx int32[n] with
 * n_groups = n1, so points with an index outside [0, n1) add nothing.  The points of a voxel
 * are added in ascending order: results do not vary from run to run.
 * Replaces voxelize_forward_cuda (voxelize/voxelize_cuda.cu:42-60,82-100). */
int tsmi_voxelize_forward(tsmi_stream_t s, const void *feats, const int32_t *counts,
                          const int32_t *order, const int32_t *starts, int64_t n, int c, int64_t n1,
                          int dtype, void *out);

/* bottom_grad[i,:] = top_grad[idx[i],:] / counts[idx[i]] (zero for skipped points).
 * Replaces voxelize_backward_cuda (voxelize/voxelize_cuda.cu:62-80,102-120), without its
 * atomics: every output row has one writer. */
int tsmi_voxelize_backward(tsmi_stream_t s, const void *top_grad, const int32_t *idx,
                           const int32_t *counts, int64_t n, int c, int64_t n1, int dtype,
                           void *bottom_grad);

/* out[i,:] = sum_k weight[i,k] * feat[indices[i,k],:] over the 8 corners, indices int32[n,8]
 * (negative = absent), weight fp32 [n,8], feat [n_vox, c].
 * Replaces devoxelize_forward_cuda (devoxelize/devoxelize_cuda.cu:11-33,62-79); the weights are
 * always fp32 here. */
int tsmi_devoxelize_forward(tsmi_stream_t s, const void *feat, const int32_t *indices,
                            const float *weight, int64_t n, int64_t n_vox, int c, int dtype,
                            void *out);

/* bottom_grad[v,:] = sum over (i,k) with indices[i,k] == v of weight[i,k] * top_grad[i,:];
 * (order, starts) = tsmi_group_by_index of the flattened indices int32[8n] with n_groups = n_vox.
 * Replaces devoxelize_backward_cuda (devoxelize/devoxelize_cuda.cu:37-58,83-98). */
int tsmi_devoxelize_backward(tsmi_stream_t s, const void *top_grad, const float *weight,
                             const int32_t *order, const int32_t *starts, int64_t n, int64_t n_vox,
                             int c, int dtype, void *bottom_grad);

/* dense[b,x,y,z,:] = feats[i,:] for coords[i] = (b,x,y,z) inside spatial_range (HOST int32[4],
 * extents B,X,Y,Z); the caller clears `dense` first.  The backward copies the other way
 * (rows outside the range receive zeros).
 * Replace to_dense_forward_cuda / to_dense_backward_cuda (voxelize/voxelize_cuda.cu:10-40,122-141). */
int tsmi_to_dense_forward(tsmi_stream_t s, const void *feats, const int32_t *coords, int64_t n, int c,
                          const int32_t *spatial_range, int dtype, void *dense);
int tsmi_to_dense_backward(tsmi_stream_t s, const void *top_grad, const int32_t *coords, int64_t n,
                           int c, const int32_t *spatial_range, int dtype, void *bottom_grad);

/* ---- batch normalisation of feats [n, c] in training mode ------------------------------
 * Replaces what nn/modules/norm.py:13-17 reaches through torch.nn.BatchNorm1d on
 * SparseTensor.feats (forward with batch statistics, running-statistics update, backward).
 * x, y, dy, dx: [n, c] row-major of `dtype`, 16-byte aligned, c a multiple of 16 bytes' worth
 * of elements (8 for 16-bit types, 4 for fp32) and at most 256 such pieces.  weight, bias,
 * running_mean, running_var: [c] of `param_dtype`, each may be null (no affine term, no
 * running statistics).  partial: fp32 scratch of tsmi_bn_partial_elems(c) elements.  Sums run
 * in fp32 in a fixed order: results are identical from run to run.
 *
 * forward:  stats[4c] (fp32) receives mean[c] and invstd[c] (biased variance,
 *           1/sqrt(var + eps)), which the backward takes, and 2c values of scratch;
 *           y = (x - mean) * invstd * weight + bias;
 *           running_mean = (1 - momentum) * running_mean + momentum * mean,
 *           running_var likewise with the unbiased variance.
 * backward: sums[5c] (fp32) receives sum_rows dy (the bias gradient) in [0:c], sum_rows
 *           dy * xhat (the weight gradient) in [c:2c], xhat = (x - mean) * invstd, and 3c values
 *           of scratch; grads, when given, receives the same two gradients as [2c] of
 *           param_dtype;
 *           dx = weight * invstd * (dy - sums[0:c] / n - xhat * sums[c:2c] / n). */
int64_t tsmi_bn_partial_elems(int c);
int tsmi_bn_forward_train(tsmi_stream_t s, const void *x, int64_t n, int c, int dtype,
                          const void *weight, const void *bias, int param_dtype, void *running_mean,
                          void *running_var, float momentum, float eps, float *partial, float *stats,
                          void *y);
int tsmi_bn_backward(tsmi_stream_t s, const void *dy, const void *x, int64_t n, int c, int dtype,
                     const void *weight, int param_dtype, const float *mean, const float *invstd,
                     float *partial, float *sums, void *grads, void *dx);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* TSMI_H_ */
