"""CPU oracle of the sparse-convolution forward path (numpy/ctypes front end).

TEST INFRASTRUCTURE, NOT THE PRODUCT: only ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py`` may import this package.  The
product (``torchsparse_amd``) never does.

Each wrapper calls the plain-C restatement in ``oracle/oracle.c``; the C
functions cite the reference file:line they follow.

Pinning status (what fixes each function independently of its own formula;
the checks live in ``tests/test_oracle_*.py``):

  kernel_offsets           literal tables for k=2,3 and (3,1,1) written out by hand
                           from nn/utils/kernel.py:21-35
  kmap_subm                brute-force O(N^2) coordinate comparison; symmetry and
                           centre-column invariants; dense torch.nn.Conv3d
                           equivalence (the reference's own test method,
                           tests/python/test_single_layer_conv.py:186-220)
  downsample_coords /      brute-force set construction; k == s case equals
  kmap_downsample          unique(coords // s); dense nn.Conv3d equivalence for
                           k in {2,3,5} x s in {1,2,3}
  spdownsample_floor /     numpy unique(axis=0); dense nn.Conv3d equivalence
  lookup_coords
  upsample_generative_     numpy restatement of the torch recipe; with lookup_coords (pinned
  coords / kmap_generative above) the convolution over the map equals a dense
                           torch conv_transpose3d with the flipped kernel (odd kernels,
                           inputs away from the clamped border)
  transpose_map            exact inverse relation, checked by brute force;
                           torch.nn.ConvTranspose3d equivalence (k == s)
  derive_bitmask /         closed-form definitions re-derived with numpy bit ops on
  reorder_map /            random maps
  reduce_bitmask
  pair_lists / build_masks numpy nonzero on the transposed map (the reference's
  / exclusive_scan         own recipe, hashmap_on_the_fly.py:138-141), inverse-
                           permutation property of the masks, numpy cumsum
  conv_implicit_gemm       float64 numpy einsum; dense nn.Conv3d; identity map
                           reduces to X @ W
  conv_gather_scatter      the compiled reference CPU conv (oracle/_ref) on golden
                           vectors in tests/golden/; float64 closed form
  conv_backward_*          the compiled reference CPU backward (oracle/_ref) on golden
                           vectors in tests/golden/; torch autograd through the
                           dense nn.Conv3d equivalent; finite differences of the
                           oracle's own forward
  hash_cpu /               golden value hash_cpu([[0,1,2,3]]) = 321218472033932309
  kernel_hash_cpu          and vectors from the compiled reference (tests/golden/)
  hash_gpu /               hash_cpu's golden vectors: folding hash_gpu's value to 60 bits
  kernel_hash_gpu          must give them (hash_cuda.cu only drops the fold); kernel_hash
                           = hash of the shifted rows
  count                    compiled reference count_cpu (golden), numpy bincount
  voxelize_forward /       compiled reference voxelize_{forward,backward}_cpu (golden);
  voxelize_backward        numpy add.at closed form; backward = adjoint of forward
  devoxelize_forward       compiled reference devoxelize_forward_cpu (golden); einsum
  devoxelize_backward      adjoint identity <devox(f), g> = <f, devox_bwd(g)> with the
                           pinned forward, and a scatter-add closed form.  The reference's
                           CPU backward is defective (indexes the gradient by voxel) and
                           is deliberately not used as evidence
  to_dense_forward /       numpy fancy indexing; backward(forward(x)) == x
  to_dense_backward
  hash_query_cpu           python dict; third-party google::dense_hash_map is not
                           vendored by the reference and no reference test covers
                           it: parity unpinned beyond "exact-match dictionary"
"""
import ctypes
import importlib.util
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)
_f32p = ctypes.POINTER(ctypes.c_float)


def lib():
    """Load (building on first use when absent) oracle/liboracle.so."""
    global _LIB
    if _LIB is None:
        from . import build as _build

        # (ASAN=1: the build with the host sanitizers, see build.py)
        path = os.path.join(_HERE, "liboracle_asan.so" if _build.SANITIZE else "liboracle.so")
        if not os.path.exists(path):
            _build.build_oracle()
        _LIB = ctypes.CDLL(path)
        _LIB.tso_pair_lists.restype = ctypes.c_int64
    return _LIB


def ref_module():
    """The reference's own CPU sources compiled by oracle/build.py --ref, or None."""
    path = os.path.join(_HERE, "_ref", "tsref_cpu.so")
    if not os.path.exists(path):
        return None
    import torch  # noqa: F401  (the module links against libtorch)

    spec = importlib.util.spec_from_file_location("tsref_cpu", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a, t):
    return a.ctypes.data_as(t)


def _triple(x):
    if isinstance(x, (int, np.integer)):
        return _i32([x, x, x])
    x = _i32(list(x))
    assert x.shape == (3,)
    return x


def ceil128(n):
    return (n + 127) // 128 * 128


def kernel_offsets(kernel_size, stride=1, dilation=1):
    ks, st, dl = _triple(kernel_size), _triple(stride), _triple(dilation)
    out = np.empty((int(np.prod(ks)), 3), np.int32)
    lib().tso_kernel_offsets(_p(ks, _i32p), _p(st, _i32p), _p(dl, _i32p), _p(out, _i32p))
    return out


def kmap_subm(coords, kernel_size, coords_min=None, coords_max=None):
    coords = _i32(coords)
    n = coords.shape[0]
    ks = _triple(kernel_size)
    cmin = _i32([0, 0, 0, 0] if coords_min is None else coords_min)
    cmax = _i32(coords.max(0) if coords_max is None else coords_max)
    n_pad = ceil128(n)
    out = np.empty((n_pad, int(np.prod(ks))), np.int32)
    lib().tso_kmap_subm(_p(coords, _i32p), n, _p(cmin, _i32p), _p(cmax, _i32p),
                        _p(ks, _i32p), n_pad, _p(out, _i32p))
    return out


def downsample_bounds(coords, kernel_size, stride, padding, spatial_range=None, allow_negative=False):
    """coords_min / coords_max of the OUTPUT grid, as kmap/func/hashmap_on_the_fly.py:27-45
    computes them (spatial_range here is the already-strided one of build_kmap.py:65-72).
    With allow_negative the minimum is (min - 2 pad + (ks-1)) / stride, a true division
    stored into an int tensor, i.e. rounded toward zero (:39-43)."""
    ks, st, pd = _triple(kernel_size), _triple(stride), _triple(padding)
    if spatial_range is not None:
        cmax = _i32([x - 1 for x in spatial_range])
    else:
        cmax = _i32(coords).max(0).astype(np.int64)
        cmax[1:] = (cmax[1:] + 2 * pd - (ks - 1)) // st
        cmax = _i32(cmax)
    if allow_negative:
        cmin = _i32(coords).min(0).astype(np.int64)
        cmin[1:] = np.trunc((cmin[1:] - 2 * pd + (ks - 1)) / st).astype(np.int64)
        return _i32(cmin), cmax
    return _i32([0, 0, 0, 0]), cmax


def kmap_downsample(coords, kernel_size, stride, padding, spatial_range=None, allow_negative=False):
    """Returns (out_in_map [ceil128(N_out),K_vol], out_coords [N_out,4])."""
    coords = _i32(coords)
    n = coords.shape[0]
    ks, st, pd = _triple(kernel_size), _triple(stride), _triple(padding)
    cmin, cmax = downsample_bounds(coords, ks, st, pd, spatial_range, allow_negative)
    kvol = int(np.prod(ks))
    buf = np.empty((max(n * kvol, 1), 4), np.int32)
    n_out = lib().tso_downsample_coords(_p(coords, _i32p), n, _p(cmin, _i32p), _p(cmax, _i32p),
                                        _p(ks, _i32p), _p(st, _i32p), _p(pd, _i32p),
                                        _p(buf, _i32p))
    out_coords = np.ascontiguousarray(buf[:n_out])
    n_pad = ceil128(n_out)
    omap = np.empty((n_pad, kvol), np.int32)
    lib().tso_kmap_downsample(_p(coords, _i32p), n, _p(out_coords, _i32p), n_out,
                              _p(cmin, _i32p), _p(cmax, _i32p), _p(ks, _i32p),
                              _p(st, _i32p), _p(pd, _i32p), n_pad, _p(omap, _i32p))
    return omap, out_coords


def spdownsample_floor(coords, stride):
    coords = _i32(coords)
    st = _triple(stride)
    buf = np.empty((max(coords.shape[0], 1), 4), np.int32)
    n_out = lib().tso_spdownsample_floor(_p(coords, _i32p), coords.shape[0], _p(st, _i32p),
                                         _p(buf, _i32p))
    return np.ascontiguousarray(buf[:n_out])


def lookup_coords(in_coords, out_coords, kernel_size, stride):
    in_coords, out_coords = _i32(in_coords), _i32(out_coords)
    ks, st = _triple(kernel_size), _triple(stride)
    n_pad = ceil128(out_coords.shape[0])
    omap = np.empty((n_pad, int(np.prod(ks))), np.int32)
    lib().tso_lookup_coords(_p(in_coords, _i32p), in_coords.shape[0], _p(out_coords, _i32p),
                            out_coords.shape[0], _p(ks, _i32p), _p(st, _i32p), n_pad,
                            _p(omap, _i32p))
    return omap


def upsample_generative_coords(coords, kernel_size, stride, spatial_range):
    """unique(clamp(coords * stride + offset, 0, range - 1)) over all kernel offsets, ascending
    (b,x,y,z) — nn/functional/conv/kmap/upsample.py:12-41 (torch.unique(dim=0) sorts rows)."""
    coords = _i32(coords)
    ks, st = _triple(kernel_size), _triple(stride)
    offs = kernel_offsets(ks)
    c = coords.astype(np.int64)
    c[:, 1:] *= st
    cand = np.repeat(c[:, None, :], offs.shape[0], axis=1)
    cand[:, :, 1:] += offs[None]
    for a in range(1, 4):
        np.clip(cand[:, :, a], 0, int(spatial_range[a]) - 1, out=cand[:, :, a])
    return np.unique(cand.reshape(-1, 4), axis=0).astype(np.int32)


def kmap_generative(coords, kernel_size, stride, spatial_range):
    """(out_in_map, out_coords) of a generative transposed convolution —
    kmap/func/hashmap.py:24-83: the table holds coords * stride, the outputs are looked up
    with stride 1 (lookup_coords)."""
    coords = _i32(coords)
    st = _triple(stride)
    out_coords = upsample_generative_coords(coords, kernel_size, stride, spatial_range)
    scaled = coords.copy()
    scaled[:, 1:] *= st
    return lookup_coords(scaled, out_coords, kernel_size, 1), out_coords


def transpose_map(out_in_map, n_in):
    m = _i32(out_in_map)
    n_rows_t = ceil128(n_in)
    out = np.empty((n_rows_t, m.shape[1]), np.int32)
    lib().tso_transpose_map(_p(m, _i32p), m.shape[0], m.shape[1], n_rows_t, _p(out, _i32p))
    return out


def derive_bitmask(out_in_map, split, valid_n):
    m = _i32(out_in_map)
    out = np.empty((split, m.shape[0]), np.int32)
    lib().tso_derive_bitmask(_p(m, _i32p), m.shape[0], m.shape[1], split, valid_n, _p(out, _i32p))
    return out


def reorder_map(out_in_map, reorder_loc):
    m, loc = _i32(out_in_map), _i32(reorder_loc)
    out = np.empty_like(m)
    lib().tso_reorder_map(_p(m, _i32p), _p(loc, _i32p), m.shape[0], m.shape[1], loc.shape[0],
                          _p(out, _i32p))
    return out


def reduce_bitmask(sorted_mask, tile):
    m = _i32(sorted_mask)
    rows = (m.shape[1] - 1) // tile + 1
    out = np.empty((m.shape[0], rows), np.int32)
    lib().tso_reduce_bitmask(_p(m, _i32p), m.shape[0], m.shape[1], tile, _p(out, _i32p))
    return out


def pair_lists(out_in_map):
    """Returns (nbmaps int32 [nnz,2] interleaved (in,out), nbsizes int32 [K_vol])."""
    m = _i32(out_in_map)
    nbsizes = np.empty(m.shape[1], np.int32)
    nnz = lib().tso_pair_lists(_p(m, _i32p), m.shape[0], m.shape[1], None, _p(nbsizes, _i32p))
    nbmaps = np.empty((nnz, 2), np.int32)
    lib().tso_pair_lists(_p(m, _i32p), m.shape[0], m.shape[1], _p(nbmaps, _i32p),
                         _p(nbsizes, _i32p))
    return nbmaps, nbsizes


def build_masks(n_in, n_out, nbmaps, nbsizes):
    nbmaps, nbsizes = _i32(nbmaps), _i32(nbsizes)
    kvol = nbsizes.shape[0]
    im = np.empty(kvol * n_in, np.int32)
    om = np.empty(kvol * n_out, np.int32)
    lib().tso_build_masks(n_in, n_out, _p(nbmaps, _i32p), _p(nbsizes, _i32p), kvol,
                          _p(im, _i32p), _p(om, _i32p))
    return im, om


def exclusive_scan_quantified(nbsizes, q=128):
    nbsizes = _i32(nbsizes)
    kvol = nbsizes.shape[0]
    a = np.empty(kvol + 1, np.int32)
    b = np.empty(kvol + 1, np.int32)
    lib().tso_exclusive_scan_quantified(kvol, _p(nbsizes, _i32p), q, _p(a, _i32p), _p(b, _i32p))
    return a, b


def conv_implicit_gemm(x, w, out_in_map, n_out):
    x, w, m = _f32(x), _f32(w), _i32(out_in_map)
    kvol, cin, cout = w.shape
    assert x.shape[1] == cin and m.shape[1] == kvol
    y = np.empty((n_out, cout), np.float32)
    lib().tso_conv_implicit_gemm(_p(x, _f32p), _p(w, _f32p), _p(m, _i32p), n_out, kvol, cin, cout,
                                 _p(y, _f32p))
    return y


def set_threads(n: int = 0) -> int:
    """Set (n > 0) and return the OpenMP thread count of the C restatement; timing only."""
    return int(lib().tso_set_threads(int(n)))


def conv_gather_scatter(x, w, nbmaps, nbsizes, n_out, transpose=False, variant=1):
    x, w, nbmaps, nbsizes = _f32(x), _f32(w), _i32(nbmaps), _i32(nbsizes)
    kvol, cin, cout = w.shape
    if x.shape[1] != cin:
        raise ValueError("Input feature size and kernel size mismatch")
    y = np.empty((n_out, cout), np.float32)
    lib().tso_conv_gather_scatter(_p(x, _f32p), x.shape[0], cin, _p(w, _f32p), kvol, cout,
                                  _p(nbmaps, _i32p), _p(nbsizes, _i32p), _p(y, _f32p), n_out,
                                  int(bool(transpose)), int(variant))
    return y


def conv_backward_gather_scatter(x, w, nbmaps, nbsizes, dy, transpose=False):
    """(dx, dw) of conv_gather_scatter with respect to x and w."""
    x, w, nbmaps, nbsizes, dy = _f32(x), _f32(w), _i32(nbmaps), _i32(nbsizes), _f32(dy)
    kvol, cin, cout = w.shape
    dx, dw = np.empty_like(x), np.empty_like(w)
    lib().tso_conv_backward_gather_scatter(_p(x, _f32p), x.shape[0], cin, _p(w, _f32p), kvol, cout,
                                           _p(nbmaps, _i32p), _p(nbsizes, _i32p), _p(dy, _f32p),
                                           _p(dx, _f32p), _p(dw, _f32p), int(bool(transpose)))
    return dx, dw


def conv_backward_implicit_gemm(x, w, out_in_map, dy):
    """(dx, dw) of conv_implicit_gemm over the first len(dy) rows of the forward map."""
    x, w, m, dy = _f32(x), _f32(w), _i32(out_in_map), _f32(dy)
    kvol, cin, cout = w.shape
    dx, dw = np.empty_like(x), np.empty_like(w)
    lib().tso_conv_backward_implicit_gemm(_p(x, _f32p), x.shape[0], cin, _p(w, _f32p), kvol, cout,
                                          _p(m, _i32p), dy.shape[0], _p(dy, _f32p), _p(dx, _f32p),
                                          _p(dw, _f32p))
    return dx, dw


def hash_cpu(rows):
    rows = _i32(rows)
    out = np.empty(rows.shape[0], np.int64)
    lib().tso_hash_cpu(_p(rows, _i32p), rows.shape[0], _p(out, _i64p))
    return out


def kernel_hash_cpu(rows, offsets):
    rows, offsets = _i32(rows), _i32(offsets)
    out = np.empty((offsets.shape[0], rows.shape[0]), np.int64)
    lib().tso_kernel_hash_cpu(_p(rows, _i32p), rows.shape[0], _p(offsets, _i32p), offsets.shape[0],
                              _p(out, _i64p))
    return out


def hash_query_cpu(hash_query, hash_target, idx_target):
    hq = np.ascontiguousarray(hash_query, dtype=np.int64)
    ht = np.ascontiguousarray(hash_target, dtype=np.int64)
    it = np.ascontiguousarray(idx_target, dtype=np.int64)
    out = np.empty(hq.shape, np.int64)
    lib().tso_hash_query_cpu(_p(hq, _i64p), hq.size, _p(ht, _i64p), _p(it, _i64p), ht.shape[0],
                             _p(out, _i64p))
    return out


def kmap_cpu_backend(coords, kernel_size):
    """Submanifold pair lists the way the reference's CPU-capable primitives build
    them (v2.0 recipe): FNV hash of (x,y,z,b) rows, hash of every shifted row,
    dictionary query.  Returns (nbmaps [nnz,2] (in,out), nbsizes [K_vol]).
    Follows nn/functional/hash.py + query.py call pattern over
    nn/utils/kernel.py offsets; used by the cpu_baseline timing."""
    coords = _i32(coords)
    xyzb = np.ascontiguousarray(coords[:, [1, 2, 3, 0]])
    offsets = kernel_offsets(kernel_size)
    references = hash_cpu(xyzb)
    queries = kernel_hash_cpu(xyzb, offsets)
    idx = np.arange(coords.shape[0], dtype=np.int64)
    res = hash_query_cpu(queries, references, idx) - 1  # [K, N], -1 = miss
    nbsizes = (res != -1).sum(1).astype(np.int32)
    k_idx, out_idx = np.nonzero(res != -1)
    nbmaps = np.stack([res[k_idx, out_idx], out_idx], 1).astype(np.int32)
    return nbmaps, nbsizes


# ---------------------------------------------------------------- point-voxel operators


def hash_gpu(rows):
    rows = _i32(rows)
    out = np.empty(rows.shape[0], np.int64)
    lib().tso_hash_gpu(_p(rows, _i32p), ctypes.c_int64(rows.shape[0]), _p(out, _i64p))
    return out


def kernel_hash_gpu(rows, offsets):
    rows, offsets = _i32(rows), _i32(offsets)
    out = np.empty((offsets.shape[0], rows.shape[0]), np.int64)
    lib().tso_kernel_hash_gpu(_p(rows, _i32p), ctypes.c_int64(rows.shape[0]), _p(offsets, _i32p),
                              offsets.shape[0], _p(out, _i64p))
    return out


def count(idx, s):
    idx = _i32(idx)
    out = np.empty(int(s), np.int32)
    lib().tso_count(_p(idx, _i32p), ctypes.c_int64(idx.shape[0]), int(s), _p(out, _i32p))
    return out


def voxelize_forward(feats, idx, counts):
    feats, idx, counts = _f32(feats), _i32(idx), _i32(counts)
    out = np.empty((counts.shape[0], feats.shape[1]), np.float32)
    lib().tso_voxelize_forward(_p(feats, _f32p), ctypes.c_int64(feats.shape[0]), feats.shape[1],
                               _p(idx, _i32p), _p(counts, _i32p), ctypes.c_int64(counts.shape[0]),
                               _p(out, _f32p))
    return out


def voxelize_backward(top, idx, counts, n):
    top, idx, counts = _f32(top), _i32(idx), _i32(counts)
    out = np.empty((int(n), top.shape[1]), np.float32)
    lib().tso_voxelize_backward(_p(top, _f32p), _p(idx, _i32p), _p(counts, _i32p), ctypes.c_int64(int(n)),
                                top.shape[1], ctypes.c_int64(counts.shape[0]), _p(out, _f32p))
    return out


def devoxelize_forward(feat, indices, weight):
    feat, indices, weight = _f32(feat), _i32(indices), _f32(weight)
    out = np.empty((indices.shape[0], feat.shape[1]), np.float32)
    lib().tso_devoxelize_forward(_p(feat, _f32p), feat.shape[1], _p(indices, _i32p), _p(weight, _f32p),
                                 ctypes.c_int64(indices.shape[0]), _p(out, _f32p))
    return out


def devoxelize_backward(top, indices, weight, n_vox):
    top, indices, weight = _f32(top), _i32(indices), _f32(weight)
    out = np.empty((int(n_vox), top.shape[1]), np.float32)
    lib().tso_devoxelize_backward(_p(top, _f32p), _p(indices, _i32p), _p(weight, _f32p),
                                  ctypes.c_int64(indices.shape[0]), ctypes.c_int64(int(n_vox)),
                                  top.shape[1], _p(out, _f32p))
    return out


def to_dense_forward(feats, coords, spatial_range):
    feats, coords, rng = _f32(feats), _i32(coords), _i32(spatial_range)
    out = np.empty(tuple(int(v) for v in rng) + (feats.shape[1],), np.float32)
    lib().tso_to_dense_forward(_p(feats, _f32p), _p(coords, _i32p), ctypes.c_int64(feats.shape[0]),
                               feats.shape[1], _p(rng, _i32p), _p(out, _f32p))
    return out


def to_dense_backward(top, coords, spatial_range):
    top, coords, rng = _f32(top), _i32(coords), _i32(spatial_range)
    out = np.empty((coords.shape[0], top.shape[-1]), np.float32)
    lib().tso_to_dense_backward(_p(top, _f32p), _p(coords, _i32p), ctypes.c_int64(coords.shape[0]),
                                top.shape[-1], _p(rng, _i32p), _p(out, _f32p))
    return out
