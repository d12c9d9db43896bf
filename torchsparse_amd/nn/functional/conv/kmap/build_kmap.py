"""Kernel-map construction glue (the reference's nn/functional/conv/kmap/build_kmap.py
and kmap/func/{hashmap_on_the_fly,hashmap}.py): spatial-range arithmetic, hash-table
reuse, and the per-dataflow products, all computed by the HIP kernels behind
``torchsparse_amd.backend``.

The returned dict carries the reference's keys (build_kmap.py:39-60):
  out_in_map, coords, sizes, spatial_range, hashmap_keys, hashmap_vals,
  reorder_out_in_map, reduced_sorted_mask, reorder_loc, sorted_mask      (ifsort)
  nbmaps, nbsizes, input_mask, output_mask                               (GatherScatter)
  nbmaps, nbsizes, nbaddrs, qnbaddrs, qmapsize                           (FetchOnDemand)
plus two of its own: ``in_hashmap`` / ``out_hashmap`` = (keys, vals) of the tables
that index the input / output coordinates, so the caller can cache each under
the stride level it belongs to.
"""
from typing import Dict, Optional, Tuple, Union

import torch

from torchsparse_amd import backend, backends
from torchsparse_amd.utils import make_divisible, make_ntuple
from ..conv_config import Dataflow

__all__ = ["build_kernel_map", "transpose_kernel_map"]

cta_M = 128  # row padding of every map and tile size of the reduced masks
cta_M_wgrad = 64  # reduce tile of the sorted weight-gradient mask (build_kmap.py:16)


def _empty_kmap(hashmap_keys, hashmap_vals, spatial_range) -> Dict:
    keys = ("out_in_map", "coords", "sizes", "reorder_out_in_map", "reduced_sorted_mask",
            "reorder_loc", "sorted_mask", "nbmaps", "nbsizes", "input_mask", "output_mask",
            "nbaddrs", "qnbaddrs", "qmapsize", "in_hashmap", "out_hashmap",
            "out_in_map_bwd", "reorder_out_in_map_bwd", "reduced_sorted_mask_bwd_wgrad",
            "reduced_sorted_mask_bwd_dgrad", "reorder_loc_bwd")
    kmap = dict.fromkeys(keys)
    kmap["hashmap_keys"], kmap["hashmap_vals"] = hashmap_keys, hashmap_vals
    kmap["spatial_range"] = spatial_range
    return kmap


def _strided_range(spatial_range, kernel_size, stride, padding):
    """(B, X', Y', Z') with X' = (X + 2p - (k-1) - 1)//s + 1 — build_kmap.py:65-72."""
    if spatial_range is None:
        return None
    return tuple(spatial_range[:1]) + tuple(
        (spatial_range[a + 1] + 2 * padding[a] - (kernel_size[a] - 1) - 1) // stride[a] + 1
        for a in range(3))


def _sort_products(kmap: Dict, out_in_map: torch.Tensor, valid_n: int, split_mask_num: int, suffix=""):
    """bitmask -> descending sort -> row-permuted map -> per-tile OR
    (kmap/func/hashmap_on_the_fly.py:92-107)."""
    bitmask = backend.derive_bitmask_from_out_in_map(out_in_map, split_mask_num, valid_n)
    sorted_mask, reorder_loc = backend.sort_bitmask_descending(bitmask)
    kmap["reorder_out_in_map" + suffix] = backend.reorder_out_in_map_cuda(out_in_map, reorder_loc)
    kmap["reduced_sorted_mask" + suffix] = backend.reduce_bitmask_cuda(sorted_mask, cta_M)
    kmap["reorder_loc" + suffix] = reorder_loc
    kmap["sorted_mask" + suffix] = sorted_mask


def _backward_products(kmap: Dict, ifsort: bool, split_mask_num_bwd: int) -> None:
    """Training-time products (build_kmap.py:191-220): the transposed map the input gradient
    runs over and, for sorted mode, its sort products with the reference's two reduce tiles
    (64 rows for the weight gradient, 128 for the input gradient).  The input gradient of a
    sorted configuration runs over them; the weight gradient works from pair lists and
    needs none."""
    n_in, n_out = kmap["sizes"]
    bwd = backend.convert_transposed_out_in_map(kmap["out_in_map"], make_divisible(n_in, cta_M), n_out)
    kmap["out_in_map_bwd"] = bwd
    if not ifsort:
        return
    bitmask = backend.derive_bitmask_from_out_in_map(bwd, split_mask_num_bwd, n_in)
    sorted_mask, reorder_loc = backend.sort_bitmask_descending(bitmask)
    kmap["reorder_out_in_map_bwd"] = backend.reorder_out_in_map_cuda(bwd, reorder_loc)
    kmap["reduced_sorted_mask_bwd_wgrad"] = backend.reduce_bitmask_cuda(sorted_mask, cta_M_wgrad)
    kmap["reduced_sorted_mask_bwd_dgrad"] = backend.reduce_bitmask_cuda(sorted_mask, cta_M)
    kmap["reorder_loc_bwd"] = reorder_loc


def _generative_kmap(kmap: Dict, coords: torch.Tensor, input_node_num: int, kernel_size, stride,
                     padding, new_range, dataflow, ifsort: bool, split_mask_num: int) -> Dict:
    """Map of a generative transposed convolution (kmap/func/hashmap.py:24-83): the outputs are
    generated around the inputs scaled by the stride (kmap/upsample.py), the table indexes the
    scaled inputs, and out_in_map[o, k] = the input whose scaled coordinate is o + offset k
    (a stride-1 centred look-up).  The output range is the reference's: the STRIDED range of
    build_kmap.py:65-74, also for this upsampling map."""
    from .upsample import spupsample_generative
    out_coords, out_table = spupsample_generative(coords, stride, kernel_size, padding, new_range,
                                                  return_table=True)
    scaled = coords.clone()
    scaled[:, 1:] *= torch.tensor(stride, dtype=coords.dtype, device=coords.device)
    in_table = backend.GPUHashTable(backend.hash_capacity(coords.shape[0], backends.hash_rsv_ratio),
                                    device=coords.device)
    in_table.insert_bxyz(scaled)
    pad = tuple((k - 1) // 2 for k in kernel_size)
    kmap["out_in_map"] = in_table.query_bxyz(out_coords, kernel_size, (1, 1, 1), pad)
    kmap["coords"] = out_coords
    kmap["sizes"] = (input_node_num, out_coords.shape[0])
    kmap["in_hashmap"] = (in_table.keys, in_table.vals)
    kmap["out_hashmap"] = (out_table.keys, out_table.vals)
    kmap["hashmap_keys"], kmap["hashmap_vals"] = in_table.keys, in_table.vals
    if dataflow == Dataflow.ImplicitGEMM:
        if ifsort:
            _sort_products(kmap, kmap["out_in_map"], kmap["sizes"][1], split_mask_num)
    else:
        _pair_products(kmap, dataflow)
    return kmap


def _pair_products(kmap: Dict, dataflow: Dataflow) -> None:
    """Pair lists, masks and scans for the GatherScatter / FetchOnDemand dataflows
    (kmap/func/hashmap_on_the_fly.py:112-207).  Both dataflows get the masks and the
    scans here: they make the reduction over offsets atomic free."""
    n_in, n_out = kmap["sizes"]
    fod = dataflow == Dataflow.FetchOnDemand
    kvol = kmap["out_in_map"].shape[1]
    # the masks leave out the identity offset of an odd submanifold map, and only that
    skip = kvol // 2 if (kmap.get("subm", False) and kvol % 2 == 1) else -1
    prod = backend.pair_lists(kmap["out_in_map"], n_in, n_out, want_inter=not fod, want_planar=fod,
                              mask_skip_k=skip)
    dev = kmap["out_in_map"].device
    nbaddrs = torch.empty(kvol + 1, dtype=torch.int32, device=dev)
    qnbaddrs = torch.empty(kvol + 1, dtype=torch.int32, device=dev)
    backend.exclusive_scan_quantified_wrapper(kvol, prod["nbsizes"], nbaddrs, qnbaddrs)
    kmap["nbmaps"] = prod["nbmaps_planar"] if fod else prod["nbmaps_inter"]
    kmap["nbsizes"] = prod["nbsizes"]
    kmap["input_mask"], kmap["output_mask"] = prod["input_mask"], prod["output_mask"]
    kmap["nbaddrs"], kmap["qnbaddrs"] = nbaddrs, qnbaddrs
    kmap["qmapsize"] = qnbaddrs[-1].cpu().int()
    kmap["nnz"] = prod["nnz"]


def build_kernel_map(_coords: torch.Tensor, input_node_num: int,
                     kernel_size: Union[int, Tuple[int, ...]] = 2,
                     stride: Union[int, Tuple[int, ...]] = 2,
                     padding: Union[int, Tuple[int, ...]] = 0,
                     hashmap_keys: torch.Tensor = None, hashmap_vals: torch.Tensor = None,
                     spatial_range: Optional[Tuple[int, ...]] = None, mode: str = "hashmap",
                     dataflow=Dataflow.ImplicitGEMM, downsample_mode: str = "spconv",
                     training: bool = False, ifsort: bool = False, generative: bool = False,
                     split_mask_num: int = 1, split_mask_num_bwd: int = 1) -> Dict:
    """Build the kernel map of one convolution geometry.

    ``hashmap_keys`` / ``hashmap_vals`` — when given — are a table that already
    indexes the INPUT coordinates ``_coords`` (it is reused instead of rebuilt)."""
    if mode not in ("hashmap_on_the_fly", "hashmap"):
        if mode == "grid":
            raise AssertionError("grid mode is temporarily deprecated.")
        raise ValueError("[Build kernel map] unknown mode: {}".format(mode))
    if dataflow not in (Dataflow.ImplicitGEMM, Dataflow.GatherScatter, Dataflow.FetchOnDemand):
        raise ValueError("[Build kernel map] unsupported dataflow: {}".format(dataflow))
    assert backends.hash_rsv_ratio >= 2, (
        f"hash_rsv_ratio should be no less than 2, now {backends.hash_rsv_ratio}.")

    if generative and mode == "hashmap_on_the_fly":
        raise ValueError(f"Unsupported kmap_mode: {mode} for generative convolution "
                         "(please switch to kmap_mode=hashmap).")

    kernel_size, stride, padding = (make_ntuple(v, ndim=3) for v in (kernel_size, stride, padding))
    new_range = _strided_range(spatial_range, kernel_size, stride, padding)
    kmap = _empty_kmap(hashmap_keys, hashmap_vals, new_range)
    if generative:
        return _generative_kmap(kmap, _coords.contiguous(), input_node_num, kernel_size, stride,
                                padding, new_range, dataflow, ifsort, split_mask_num)
    subm = all(s == 1 for s in stride)
    coords = _coords.contiguous()
    n_in = coords.shape[0]

    fresh = hashmap_keys is None or hashmap_vals is None
    out_in_map = None
    in_table = out_table = None
    # Ascending input rows (voxelisation by a ravelled key, every strided builder here): the
    # map is searched over the rows themselves and no table is built at all.
    by_search = (mode == "hashmap_on_the_fly" and n_in > 0 and backend.kmap_sorted_supported(kernel_size)
                 and backend.coords_ascending(_coords))
    if by_search:
        if subm:
            backend.strided_lookahead(_coords)  # the strided chain that follows such rows, queued early
            out_coords = coords
            out_in_map = backend.kmap_sorted(coords, coords, kernel_size, stride, backend._subm_pad(kernel_size))
            # rows that thinned out like a surface on their way here (at most 1 / 0.3 occupied
            # cells per occupied block of the strided layer before) have few neighbours each
            thinning = backend.level_thinning(_coords)
            if thinning is not None and thinning >= 0.3:
                backend.hint_sparse_map(out_in_map)
        else:
            host_max = None if new_range is None else tuple(x - 1 for x in new_range[1:])
            from torchsparse_amd.tensor import get_allow_negative_coordinates
            out_coords, out_table = backend.downsample_coords(
                coords, kernel_size, stride, padding, host_max, 0, backends.hash_rsv_ratio,
                allow_negative=get_allow_negative_coordinates(), want_table=False)
            out_in_map = backend.kmap_sorted(coords, out_coords, kernel_size, stride, padding)
        if not fresh:
            in_table = backend.GPUHashTable(hashmap_keys, hashmap_vals)
    else:
        # table over the input coordinates: reuse or build
        if subm and mode == "hashmap_on_the_fly":
            backend.strided_lookahead(_coords)  # (a caller's rows whose order is not known yet take this path)
        if fresh and subm and (mode == "hashmap_on_the_fly" or all(k % 2 == 1 for k in kernel_size)):
            # table and map in one call (an even kernel in "hashmap" mode is centred differently)
            in_table, out_in_map = backend.GPUHashTable.build_subm(coords, kernel_size, backends.hash_rsv_ratio)
        elif fresh:
            in_table = backend.GPUHashTable(backend.hash_capacity(n_in, backends.hash_rsv_ratio),
                                            device=coords.device)
            in_table.insert_bxyz(coords)
        else:
            in_table = backend.GPUHashTable(hashmap_keys, hashmap_vals)

        if subm:
            out_coords = coords
            pad_eff = backend._subm_pad(kernel_size)
            out_table = in_table
        elif mode == "hashmap_on_the_fly":
            host_max = None if new_range is None else tuple(x - 1 for x in new_range[1:])
            from torchsparse_amd.tensor import get_allow_negative_coordinates
            out_coords, out_table = backend.downsample_coords(
                coords, kernel_size, stride, padding, host_max, 0, backends.hash_rsv_ratio,
                allow_negative=get_allow_negative_coordinates())
            pad_eff = padding
        else:  # "hashmap": coordinates first, then a padding-free centred lookup
            from .downsample import spdownsample
            out_coords, out_table = spdownsample(coords, stride, kernel_size, padding, new_range,
                                                 downsample_mode, return_table=True)
            pad_eff = tuple((k - 1) // 2 for k in kernel_size)
        if subm and mode == "hashmap":
            pad_eff = tuple((k - 1) // 2 for k in kernel_size)

        if out_in_map is not None:
            pass
        elif subm and all(k % 2 == 1 for k in kernel_size):
            out_in_map = in_table.query_subm_bxyz(out_coords, kernel_size)  # centred in both modes
        else:
            out_in_map = in_table.query_bxyz(out_coords, kernel_size, stride, pad_eff)

    def pair(table):
        return None if table is None else (table.keys, table.vals)

    kmap["out_in_map"] = out_in_map
    kmap["subm"] = subm  # stride 1: outputs are the inputs, the centre offset is the identity
    kmap["coords"] = out_coords if not subm else _coords
    kmap["sizes"] = (input_node_num, out_coords.shape[0])
    # tables of the input / output coordinates: None when the map was searched over sorted rows
    kmap["in_hashmap"] = pair(in_table)
    kmap["out_hashmap"] = pair(in_table if (subm and out_table is None) else out_table)
    owner = in_table if (subm or mode == "hashmap") else out_table
    kmap["hashmap_keys"], kmap["hashmap_vals"] = pair(owner) if owner is not None else (None, None)

    if dataflow == Dataflow.ImplicitGEMM:
        if ifsort:
            _sort_products(kmap, out_in_map, kmap["sizes"][1], split_mask_num)
        if training:
            _backward_products(kmap, ifsort, split_mask_num_bwd)
    else:
        _pair_products(kmap, dataflow)
    return kmap


def transpose_kernel_map(kmap: Dict, ifsort: bool = False, training: bool = False,
                         split_mask_num: int = 1, split_mask_num_bwd: int = 1) -> Dict:
    """Add the products a transposed convolution needs to an existing strided map:
    out_in_map_t[in, k] = out (and its sort products when ifsort).  Computed once
    and kept under the ``*_t`` keys (the reference recomputes them on every call,
    build_kmap.py:224-309)."""
    if kmap is None:
        raise ValueError("transposed convolution needs the kernel map of the matching strided "
                         "convolution; run that layer on this tensor's ancestors first")
    n_in, n_out = kmap["sizes"]
    if kmap.get("out_in_map_t") is None:
        kmap["out_in_map_t"] = backend.convert_transposed_out_in_map(
            kmap["out_in_map"], make_divisible(n_in, cta_M), n_out)
    if ifsort:
        if kmap.get("reorder_out_in_map_t") is None or kmap.get("_split_t") != split_mask_num:
            _sort_products(kmap, kmap["out_in_map_t"], n_in, split_mask_num, suffix="_t")
            kmap["_split_t"] = split_mask_num
    else:
        kmap.setdefault("reorder_out_in_map_t", None)
        kmap.setdefault("reduced_sorted_mask_t", None)
        kmap.setdefault("reorder_loc_t", None)
    for key in ("out_in_map_bwd_t", "reorder_out_in_map_bwd_t", "reduced_sorted_mask_bwd_wgrad_t",
                "reduced_sorted_mask_bwd_dgrad_t", "reorder_loc_bwd_t"):
        kmap.setdefault(key, None)
    return kmap
