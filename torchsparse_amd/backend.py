"""Host side of the C ABI: loads ``libtsmi.so`` with ctypes and exposes it under
the names and argument meanings of the reference's pybind module
``torchsparse.backend`` (backend/pybind_cuda.cu:29-83), forward path only.

PyTorch is used for device memory and the current HIP stream; every computation
below happens in the hand-written HIP kernels of ``csrc/``.  There is no CPU or
eager fallback: if the shared object is missing, importing this module raises.
"""
import collections
import ctypes
import functools
import os
import struct
import threading
import weakref
from typing import List, Optional, Sequence, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# (ASAN=1 / SANITIZE=address: the build whose host code carries AddressSanitizer, for CPU runs of
# the host logic under a preloaded sanitizer runtime; csrc/build.py makes it under the same switch)
_SANITIZE = os.environ.get("ASAN", "0") not in ("", "0") or os.environ.get("SANITIZE") == "address"
_LIB_PATH = os.path.join(_HERE, "libtsmi_asan.so" if _SANITIZE else "libtsmi.so")

F32, F16, BF16 = 0, 1, 2
_DTYPE_CODE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

_vp, _i64, _i32, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
_I3 = ctypes.c_int32 * 3
_I4 = ctypes.c_int32 * 4


def _load():
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            f"{_LIB_PATH} is missing: build the HIP extension first "
            "(python torchsparse_amd/csrc/build.py, or __graft_entry__.build())")
    lib = ctypes.CDLL(_LIB_PATH)
    lib.tsmi_last_error.restype = ctypes.c_char_p
    lib.tsmi_launch_thread_submit.restype = _i64
    lib.tsmi_launch_thread_submit.argtypes = [_i32, ctypes.c_char_p, _i32]
    lib.tsmi_launch_thread_completed.restype = ctypes.POINTER(ctypes.c_int64)
    lib.tsmi_launch_thread_completed.argtypes = []
    lib.tsmi_sort_temp_bytes.restype = _i64
    lib.tsmi_sort_temp_bytes.argtypes = [_i64]
    lib.tsmi_packed_weight_elems.restype = _i64
    lib.tsmi_packed_weight_elems.argtypes = [_i32, _i32, _i32]
    lib.tsmi_conv_workspace_elems.restype = _i64
    lib.tsmi_conv_wgrad_workspace_elems.restype = _i64
    lib.tsmi_conv_wgrad_workspace_elems.argtypes = [_i64, _i32, _i32, _i32, _i32]
    lib.tsmi_conv_workspace_elems.argtypes = [_i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32]
    lib.tsmi_group_temp_bytes.restype = _i64
    lib.tsmi_group_temp_bytes.argtypes = [_i64]
    lib.tsmi_wgrad_pairs_capacity.restype = _i64
    lib.tsmi_wgrad_pairs_capacity.argtypes = [_i64, _i32]
    lib.tsmi_conv_wgrad_pairs_workspace_elems.restype = _i64
    lib.tsmi_conv_wgrad_pairs_workspace_elems.argtypes = [_i64, _i32, _i32, _i32, _i32]
    lib.tsmi_map_group_rows_padded.restype = _i64
    lib.tsmi_map_group_rows_padded.argtypes = [_i64, _i32]
    lib.tsmi_kmap_sorted_samples_elems.restype = _i64
    lib.tsmi_kmap_sorted_samples_elems.argtypes = [_i64]
    sig = {
        "tsmi_hashtable_clear": [_vp, _vp, _vp, _i64],
        "tsmi_hashtable_insert_coords": [_vp, _vp, _vp, _i64, _vp, _i64, _vp],
        "tsmi_hashtable_insert_keys": [_vp, _vp, _vp, _i64, _vp, _i64, _vp],
        "tsmi_hashtable_lookup_keys": [_vp, _vp, _vp, _i64, _vp, _i64, _vp],
        "tsmi_kmap_query": [_vp, _vp, _vp, _i64, _vp, _i64, _i64, _I3, _I3, _I3, _vp],
        "tsmi_kmap_query_subm": [_vp, _vp, _vp, _i64, _vp, _i64, _i64, _I3, _vp],
        "tsmi_coords_max": [_vp, _vp, _i64, _vp, _i32],
        "tsmi_kmap_sorted_batch": [_vp, _i32, _vp],
        "tsmi_downsample_candidates": [_vp, _vp, _i64, _I3, _I3, _I3, _vp, _vp, _vp, _i32, _vp, _i64, _vp],
        "tsmi_hashtable_compact_keys": [_vp, _vp, _i64, _vp, _vp],
        "tsmi_sort_keys": [_vp, _vp, _vp, _i64, _i32, _vp, _i64],
        "tsmi_downsample_finalize": [_vp, _vp, _i64, _vp, _vp, _i64, _vp],
        "tsmi_downsample_grid_count": [_vp, _vp, _i64, _I3, _I3, _I3, _vp, _vp, _vp, _i64, _i32, _vp, _vp,
                                       _vp, _vp],
        "tsmi_downsample_grid_count_next": [_vp, _I3, _I3, _I3, _vp, _vp, _i64, _vp, _vp, _i64, _vp, _vp, _vp],
        "tsmi_downsample_grid_emit": [_vp, _I3, _I3, _I3, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _vp,
                                      _i64, _vp, _vp],
        "tsmi_downsample_chain_rows": [_vp, _vp, _i64, _I3, _I3, _I3, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _i32],
        "tsmi_transpose_map": [_vp, _vp, _i64, _i32, _vp, _i64],
        "tsmi_derive_bitmask": [_vp, _vp, _i64, _i32, _i32, _i64, _vp],
        "tsmi_argsort_desc": [_vp, _vp, _vp, _vp, _i32, _i64, _vp, _i64],
        "tsmi_reorder_map": [_vp, _vp, _vp, _i64, _i32, _i32, _vp],
        "tsmi_reduce_bitmask": [_vp, _vp, _i32, _i64, _i32, _vp],
        "tsmi_pair_lists_count": [_vp, _vp, _i64, _i32, _vp, _vp],
        "tsmi_pair_lists_fill": [_vp, _vp, _i64, _i32, _vp, _vp, _i64, _vp, _vp, _i64, _i64, _i32, _vp, _vp],
        "tsmi_exclusive_scan_quantified": [_vp, _i32, _vp, _i32, _vp, _vp],
        "tsmi_build_masks": [_vp, _vp, _i64, _vp, _i32, _i64, _i64, _vp, _vp],
        "tsmi_pack_weights": [_vp, _vp, _vp, _i32, _i32, _i32, _i32],
        "tsmi_conv_implicit_gemm": [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _i32, _i32, _vp, _vp,
                                    _i32, _vp, _i64, _vp, _i64, _vp],
        "tsmi_conv_implicit_gemm_sorted": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32,
                                           _i32, _i32, _i32, _vp, _vp, _i32, _vp, _i64, _vp, _i64,
                                           _vp],
        "tsmi_conv_wgrad": [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _i32, _i32, _vp, _i64, _vp],
        "tsmi_wgrad_pairs_build": [_vp, _vp, _i64, _i32, _vp, _vp, _vp, _vp],
        "tsmi_wgrad_pairs_build_static": [_vp, _vp, _i64, _i32, _vp, _vp, _vp],
        "tsmi_kmap_build_subm": [_vp, _vp, _vp, _i64, _vp, _i64, _i64, _I3, _vp, _vp],
        "tsmi_coords_check": [_vp, _vp, _i64, _vp],
        "tsmi_kmap_sorted_supported": [_I3],
        "tsmi_kmap_sorted": [_vp, _vp, _i64, _vp, _i64, _i64, _I3, _I3, _I3, _vp, _vp],
        "tsmi_kmap_sorted_samples": [_vp, _vp, _i64, _vp],
        "tsmi_wgrad_pairs_pad": [_vp, _vp, _i64, _vp, _i32, _vp, _vp],
        "tsmi_conv_wgrad_pairs": [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32, _vp,
                                  _i64, _vp],
        "tsmi_conv_fetch_on_demand": [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _i64, _vp, _i64, _i32,
                                      _i32, _i32, _i32, _i32, _i32, _vp, _vp, _i32, _vp, _vp],
        "tsmi_conv_segments_supported": [_i32, _i32, _i32, _i32],
        "tsmi_pair_segments": [_vp, _vp, _i64, _i32, _i64, _vp, _vp, _vp, _vp],
        "tsmi_pair_segments_batch": [_vp, _i32, _vp],
        "tsmi_conv_implicit_gemm_segments": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _i32,
                                             _i32, _vp, _vp, _i32, _vp, _vp],
        "tsmi_launch_thread_open": [],
        "tsmi_launch_thread_flush": [],
        "tsmi_launch_thread_close": [],
        "tsmi_conv_implicit_gemm_packed": [ctypes.c_char_p],
        "tsmi_conv_implicit_gemm_segments_packed": [ctypes.c_char_p],
        "tsmi_conv_implicit_gemm_grouped_packed": [ctypes.c_char_p],
        "tsmi_conv_implicit_gemm_grouped": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _i32, _i32,
                                            _vp, _vp, _i32, _vp],
        "tsmi_map_group_rows": [_vp, _vp, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _vp],
        "tsmi_hash_coords": [_vp, _vp, _i64, _vp],
        "tsmi_kernel_hash": [_vp, _vp, _i64, _vp, _i32, _vp],
        "tsmi_count": [_vp, _vp, _i64, _vp, _i32],
        "tsmi_group_by_index": [_vp, _vp, _i64, _i64, _vp, _i64, _vp, _vp],
        "tsmi_voxelize_forward": [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i64, _i32, _vp],
        "tsmi_voxelize_backward": [_vp, _vp, _vp, _vp, _i64, _i32, _i64, _i32, _vp],
        "tsmi_devoxelize_forward": [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _vp],
        "tsmi_devoxelize_backward": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _vp],
        "tsmi_to_dense_forward": [_vp, _vp, _vp, _i64, _i32, _I4, _i32, _vp],
        "tsmi_to_dense_backward": [_vp, _vp, _vp, _i64, _i32, _I4, _i32, _vp],
        "tsmi_bn_forward_train": [_vp, _vp, _i64, _i32, _i32, _vp, _vp, _i32, _vp, _vp, _f32, _f32, _vp, _vp,
                                  _vp],
        "tsmi_bn_partial_elems": [_i32],
        "tsmi_bn_backward": [_vp, _vp, _vp, _i64, _i32, _i32, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _vp],
        "tsmi_gs_gather": [_vp, _vp, _vp, _i64, _i32, _i32, _i32, _vp],
        "tsmi_gs_gemm": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _i32, _i32, _vp],
        "tsmi_gs_scatter": [_vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _vp, _vp, _i32, _vp],
    }
    for name, argtypes in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _i32
    return lib


class _Library:
    """The entry points of the loaded library.  Every call that can queue work first waits for
    the convolution calls that were handed to the library's launch thread (launch_region below):
    whatever is queued from this thread then comes after them on the stream.  The packed
    convolution calls, which go to that thread inside a region, the thread's own entry points and
    the entry points that only answer a question are passed through as they are."""

    _ASIS = ("tsmi_conv_implicit_gemm_packed", "tsmi_conv_implicit_gemm_segments_packed",
             "tsmi_conv_implicit_gemm_grouped_packed", "tsmi_last_error", "tsmi_version")
    _ASIS_ENDINGS = ("_elems", "_supported", "_bytes", "_capacity", "_padded")

    def __init__(self, lib):
        self._lib = lib

    def __getattr__(self, name):  # (once per name: the result becomes an attribute)
        fn = getattr(self._lib, name)
        if not (name in self._ASIS or name.startswith("tsmi_launch_thread_") or name.endswith(self._ASIS_ENDINGS)):
            raw = fn

            def fn(*args, _raw=raw):
                if _region_calls:
                    flush_launches()
                return _raw(*args)
        setattr(self, name, fn)
        return fn


_C = _Library(_load())


def _check(status: int) -> None:
    """Status code -> the exception class pybind raises for the reference
    (std::invalid_argument -> ValueError, std::runtime_error -> RuntimeError)."""
    if status == 0:
        return
    msg = _C.tsmi_last_error().decode()
    if status == 1:
        raise ValueError(msg)
    raise RuntimeError(msg)


_raw_stream = torch._C._cuda_getCurrentRawStream
_cur_device = torch._C._cuda_getDevice


def _stream() -> int:
    """hipStream_t of torch's current stream on the current device (as an int)."""
    return _raw_stream(_cur_device())


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _need(t: torch.Tensor, dtype, name: str) -> torch.Tensor:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got {t.device}); there is no CPU path")
    if t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    return t if t.is_contiguous() else t.contiguous()


@functools.lru_cache(maxsize=512)
def _i3(t: Tuple[int, int, int]):
    """int32[3] argument of a triple (one shared, read-only instance per value)."""
    return _I3(*t)


@functools.lru_cache(maxsize=512)
def _triple_of_tuple(x: tuple) -> Tuple[int, int, int]:
    x = tuple(int(v) for v in x)
    assert len(x) == 3, x
    return x


def _triple(x) -> Tuple[int, int, int]:
    if type(x) is tuple:
        return _triple_of_tuple(x)
    if isinstance(x, torch.Tensor):
        x = x.view(-1).tolist()
    if isinstance(x, int):
        return (x, x, x)
    x = tuple(int(v) for v in x)
    assert len(x) == 3, x
    return x


def make_divisible(x: int, divisor: int) -> int:
    return (x + divisor - 1) // divisor * divisor


def hash_capacity(n: int, ratio: float = 2.0) -> int:
    """Table capacity for n keys: max(512, ratio*n) as in
    kmap/func/hashmap_on_the_fly.py:56-58, rounded up to the slot-group size."""
    return make_divisible(max(512, int(ratio * n)), 8)


# --------------------------------------------------------------------- hash table


# The table key packs 18 bits per spatial axis and 9 for the batch index.  The reference
# ravels over the measured extents and takes any int32 coordinate
# (others/sparsemapping_cuda.cu:12-26); here a row outside the packed range must stop the
# call: the kernels flag it and the shim raises.  A flag costs a read-back, so a coordinate
# tensor is looked at once: what is known of it — it is in range; its rows ascend strictly in
# (b, x, y, z) or do not — is remembered by identity, version and address.  The strided
# builders produce ascending rows in range and say so for their outputs.
COORD_LIMIT = 1 << 17
BATCH_LIMIT = 512
_range_ok = {}  # id(tensor) -> (weak reference, version, address, ascending: True / False / None = not known, origin)
# A tensor the library has not seen is checked by one small kernel, and its verdict is read
# back: that stops the host until everything queued on the stream has run (a quarter of a U-Net
# forward when forwards follow each other).  The wait also stands for a fact the library
# cannot see: rows produced by work queued on the caller's stream are complete only once that
# work has run, and the strided chain that follows (whose row counts must reach the host
# before anything can be sized) cannot start before.  A caller who knows that the rows are
# complete - a data loader's own stream, a scan uploaded earlier - says so with
# rows_ready(coords): the check then runs without a read-back (its verdict is copied to pinned
# memory and picked up by a later call), the chain starts at once on the second stream, and
# until the verdict is in the rows count as unordered (their own maps go through the hash
# table, which takes any order).  A row outside the packed range of such a tensor raises its
# ValueError from the call that picks the verdict up (settle_checks() picks up all of them).
coords_check_deferred = True
# ... unless the check runs on the device's second stream, where nothing of the caller's stream is
# in its way: the host then waits for the verdict at once (a kernel and a copy) and rows that
# ascend take the table-free builders from their first map on.
coords_check_aside = True
# The first check of any other tensor is read back at once; the strided chain that followed such
# rows last time is queued before the host waits for the verdict (False: after it).
coords_check_overlap = True
_rows_ready = {}  # id(tensor) -> (weak reference, version, address)
_pending_verdicts = []  # (weak reference, version, address, pinned slot, event)
_verdict_slots = None   # pinned int32 ring the verdicts are copied into
_verdict_host = None    # ... as a numpy array over the same memory (an element read costs 0.2 us against 3)
_verdict_next = 0
_VERDICT_SLOTS = 64
# Kernel maps of ascending inputs are built by binary search over the coordinates themselves
# (no hash table); False sends every map through the tables.
kmap_through_sorted = True


_tables_lock = threading.Lock()  # guards the insertions and prunings of the module's tables


def _remember(table: dict, key, value, limit: int) -> None:
    """``table[key] = value``; a table that holds ``limit`` entries first drops those whose
    tensor (``entry[0]``, a weak reference) is gone, and everything if none is.  One host thread
    at a time: a second one would otherwise iterate a table the first is resizing."""
    with _tables_lock:
        if len(table) >= limit:
            for k in [k for k, v in table.items() if v[0]() is None]:
                del table[k]
            if len(table) >= limit:
                table.clear()
        table[key] = value


def _range_error() -> ValueError:
    return ValueError(
        f"coordinates outside the range of the packed hash key: x, y, z must lie in "
        f"[{-COORD_LIMIT}, {COORD_LIMIT}) and the batch index in [0, {BATCH_LIMIT})")


def _range_entry(coords: torch.Tensor):
    hit = _range_ok.get(id(coords))
    if (hit is not None and hit[0]() is coords and hit[1] == coords._version
            and hit[2] == coords.data_ptr()):
        return hit
    return None


def _range_known(coords: torch.Tensor) -> bool:
    return _range_entry(coords) is not None


def _range_origin(coords: torch.Tensor) -> Optional[str]:
    """"user": a caller's tensor that coords_ascending looked at (complete: its verdict was
    read back, or the caller declared it so); "library": rows a strided builder produced; None:
    not known."""
    hit = _range_entry(coords)
    return None if hit is None else hit[4]


def _mark_range_ok(coords: torch.Tensor, ascending: Optional[bool] = None, origin: str = "library") -> None:
    """``coords`` is in range; ``ascending`` says whether its rows ascend strictly (None keeps
    what is already known)."""
    if ascending is None:
        hit = _range_entry(coords)
        if hit is not None:
            return
        origin = "user"  # vouched for by a flag read-back over a caller's rows
    _remember(_range_ok, id(coords), (weakref.ref(coords), coords._version, coords.data_ptr(), ascending, origin),
              512)


def settle_checks(block: bool = True) -> None:
    """Pick up the verdicts of coordinate checks that were left on their way to the host
    (coords_check_deferred): all of them, waiting for their copies, or with ``block=False``
    those that have arrived.  Raises the ValueError of a tensor with a row outside the packed
    range."""
    global _pending_verdicts
    if not _pending_verdicts:
        return
    bad = False
    left = []
    for item in _pending_verdicts:
        ref, version, address, slot, event = item
        if not block and not event.query():
            left.append(item)
            continue
        if block:
            event.synchronize()
        bits = int(_verdict_host[slot])
        t = ref()
        if bits & 2:
            bad = True
            if t is not None:
                _range_ok.pop(id(t), None)
            continue
        hit = _range_ok.get(id(t)) if t is not None else None
        if hit is not None and hit[0]() is t and hit[1] == version and hit[2] == address:
            _range_ok[id(t)] = (hit[0], version, address, not (bits & 1), "user")
    _pending_verdicts = left
    if bad:
        raise _range_error()


def rows_ready(coords: torch.Tensor) -> torch.Tensor:
    """Declare that the rows of ``coords`` are complete: no work still queued on any stream
    writes them.  The library then neither waits for the caller's stream before it reads them
    on its second stream nor reads the verdict of their first check back at once.  Returns
    ``coords``.  Holds until the tensor is written in place."""
    _remember(_rows_ready, id(coords), (weakref.ref(coords), coords._version, coords.data_ptr()), 256)
    return coords


def _declared_ready(coords: torch.Tensor) -> bool:
    hit = _rows_ready.get(id(coords))
    return (hit is not None and hit[0]() is coords and hit[1] == coords._version
            and hit[2] == coords.data_ptr())


def coords_ascending(coords: torch.Tensor) -> bool:
    """Whether the rows of ``coords`` ascend strictly in (b, x, y, z); raises ValueError for a
    row outside the packed key's range.  One kernel and one read-back the first time a tensor
    is seen, nothing afterwards.  Rows declared complete (rows_ready) are checked on the second
    stream, so that the read-back waits for nothing else (or, with coords_check_aside off, have
    their verdict picked up later: False is the answer until then)."""
    if _pending_verdicts:
        settle_checks(block=False)
    hit = _range_entry(coords)
    if hit is not None and hit[3] is not None:
        return hit[3]
    rows = _need(coords, torch.int32, "coords")
    if coords_check_aside and rows is coords and _declared_ready(coords):
        return _verdict(coords, _check_aside(rows))
    overlap = coords_check_overlap and rows is coords and not _declared_ready(coords)
    if overlap:
        # The read-back below waits for everything the stream has queued - the whole forward
        # before, in a loop over new tensors - and until it returns the device gets nothing new.
        # What does not depend on the verdict is therefore queued first: the strided chain that
        # followed rows like these last time (any order of rows will do for it, and rows it cannot
        # take are flagged, not followed), on the second stream, behind this point of the caller's
        # stream - in front of the check, which the chain does not need.
        ready = torch.cuda.Event()
        ready.record()
        strided_lookahead(coords, behind=ready)
    flags = torch.zeros(1, dtype=torch.int32, device=rows.device)
    _check(_C.tsmi_coords_check(_stream(), _ptr(rows), rows.shape[0], _ptr(flags)))
    if coords_check_deferred and rows is coords and _declared_ready(coords):
        slot = _verdict_slot()
        _verdict_slots[slot:slot + 1].copy_(flags, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        _pending_verdicts.append((weakref.ref(coords), coords._version, coords.data_ptr(), slot, event))
        _mark_range_ok(coords, ascending=False, origin="user")  # (complete: the caller said so)
        return False
    elif overlap:
        slot = _verdict_slot()
        _verdict_slots[slot:slot + 1].copy_(flags, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        _queue_root_map(coords)  # (taken or dropped with the verdict)
        event.synchronize()
        _drained[(rows.device.index, _stream())] = weakref.ref(coords)  # (nothing is queued on this stream now)
        bits = int(_verdict_host[slot])
        if bits and _root_maps:
            with _tables_lock:
                for key in [k for k in _root_maps if k[0] == id(coords)]:
                    _root_maps.pop(key, None)  # (searched over rows that do not ascend)
            if bits & 1:
                _root_geoms.pop((coords.device.index, _stream()), None)
    else:
        bits = int(flags.item())
    return _verdict(coords, bits)


def _verdict(coords: torch.Tensor, bits: int) -> bool:
    if bits & 2:
        raise _range_error()
    _mark_range_ok(coords, ascending=not (bits & 1), origin="user")
    return not (bits & 1)


def _verdict_slot() -> int:
    """A free element of the pinned ring the verdicts are copied into."""
    global _verdict_slots, _verdict_next, _verdict_host
    if _verdict_slots is None:
        _verdict_slots = torch.zeros(_VERDICT_SLOTS, dtype=torch.int32, pin_memory=True)
        _verdict_host = _verdict_slots.numpy()
    if len(_pending_verdicts) >= _VERDICT_SLOTS - 1:
        settle_checks(block=True)  # (every slot is on its way: wait for them)
    slot = _verdict_next
    while any(item[3] == slot for item in _pending_verdicts):  # (a verdict still on its way keeps its slot)
        slot = (slot + 1) % _VERDICT_SLOTS
    _verdict_next = (slot + 1) % _VERDICT_SLOTS
    return slot


def _check_aside(rows: torch.Tensor) -> int:
    """The check of rows that are complete (rows_ready), on the device's second stream: the host
    waits for that stream only - a kernel and a copy - whatever the caller's stream still has
    queued.  Returns the flags."""
    dev = rows.device
    with _state_lock:
        state = _strided_state(dev)
        if state.side is None:
            state.side = torch.cuda.Stream(device=dev)
        side = state.side
    slot = _verdict_slot()
    main = torch.cuda.current_stream(dev)
    torch.cuda.set_stream(side)
    try:
        flags = torch.zeros(1, dtype=torch.int32, device=dev)
        _check(_C.tsmi_coords_check(_stream(), _ptr(rows), rows.shape[0], _ptr(flags)))
        _verdict_slots[slot:slot + 1].copy_(flags, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
    finally:
        torch.cuda.set_stream(main)
    event.synchronize()
    return int(_verdict_host[slot])


@functools.lru_cache(maxsize=256)
def _sorted_supported(ks: Tuple[int, int, int]) -> bool:
    return bool(_C.tsmi_kmap_sorted_supported(_I3(*ks)))


def kmap_sorted_supported(kernel_size) -> bool:
    return bool(kmap_through_sorted and _sorted_supported(_triple(kernel_size)))


def kmap_sorted(in_coords: torch.Tensor, out_coords: torch.Tensor, kernel_size, stride, pad) -> torch.Tensor:
    """out_in_map int32 [ceil128(N_out), K_vol] of ascending in-range inputs and ascending
    outputs, by binary search over the input rows: no hash table, one launch."""
    in_coords = _need(in_coords, torch.int32, "coords")
    out_coords = _need(out_coords, torch.int32, "coords")
    ks, st, pd = _triple(kernel_size), _triple(stride), _triple(pad)
    if in_coords is out_coords and _root_maps:
        hit = _root_maps.pop((id(in_coords), ks, st, pd), None)
        if (hit is not None and hit[0]() is in_coords and hit[1] == in_coords._version
                and hit[2] == in_coords.data_ptr() and hit[3] == _stream()):
            if hit[5] is not None and not hit[5].query():  # (built on the second stream a moment ago)
                torch.cuda.current_stream(in_coords.device).wait_event(hit[5])
            return hit[4]
    if kmap_queue_ahead:
        ahead = _map_queued_ahead(in_coords, out_coords, ks, st, pd)
        if ahead is not None:
            return ahead
    if in_coords is out_coords and _range_origin(in_coords) == "user":
        _root_geoms[(in_coords.device.index, _stream())] = (ks, st, pd)  # (see _queue_root_map)
    return _kmap_sorted_launch(in_coords, out_coords, ks, st, pd)


# The submanifold map over a caller's own rows, queued while their first check is still on its
# way.  A loop over new coordinate tensors waits for each tensor's check with the device drained,
# and the first thing the forward then needs is this map; when the stream's last such tensor
# had ascending rows and asked for the map, it is queued right behind the check of the next one,
# before the host waits for the verdict: the device builds it while the host wakes up.  Rows
# that turn out not to ascend make it a wasted launch (the search stays inside the rows whatever
# their order; its result is dropped).
_drained = {}     # (device index, stream) -> weak reference to the tensor whose check the host last waited for there
_root_geoms = {}  # (device index, stream) -> geometry of the last map built over a caller's ascending rows
_root_maps = {}   # (id(coords), ks, st, pd) -> (weak reference, version, address, stream, map)


def _queue_root_map(coords: torch.Tensor, main=None) -> None:
    """``main`` None: on the current stream, for its own layers.  Else the current stream is the
    second stream of ``main`` (rows that are complete: the map is built beside what ``main`` still has
    queued, and the layer that takes it puts ``main`` behind an event)."""
    stream = _stream() if main is None else main.cuda_stream
    geom = _root_geoms.get((coords.device.index, stream))
    if geom is None or not kmap_through_sorted or coords.shape[0] == 0:
        return
    with _tables_lock:  # (another host thread may be adding its own)
        left = [k for k, v in _root_maps.items() if v[3] == stream]
        for k in left:
            _root_maps.pop(k, None)
    if left:
        # the map queued for the tensor before was never asked for: another network runs now;
        # nothing is queued until a forward asks for such a map again
        _root_geoms.pop((coords.device.index, stream), None)
        return
    ks, st, pd = geom
    omap = _kmap_sorted_launch(coords, coords, ks, st, pd)
    event = None
    if main is not None:
        omap.record_stream(main)
        event = torch.cuda.Event()
        event.record()
    _remember(_root_maps, (id(coords), ks, st, pd),
              (weakref.ref(coords), coords._version, coords.data_ptr(), stream, omap, event), 8)


# The maps a network builds over the levels of its strided chain (the submanifold map of every
# level, the strided map to the next) depend on nothing but those levels' rows, which exist
# - on the chain's second stream - long before the layers that ask for the maps are reached.
# Once a forward has asked for such maps, the next forward queues the same builds on that
# stream as soon as the row counts are on the host, beside the convolutions of the levels
# above; the caller's stream waits once, for the end of that queue, when it takes the first
# of them.  Maps queued and never asked for cost their kernels.
kmap_queue_ahead = True
# The launch that builds the maps queued ahead also counts their pairs (entries >= 0); the counts
# travel to pinned memory behind it and tell the convolutions how dense each map is.
map_pairs_counted = True
_PAIR_SLOTS = 16
_map_requests = {}  # id(map) -> (weak reference, stream state, request, transposed map or None)


def map_density(out_in_map: torch.Tensor) -> Optional[float]:
    """Pairs per entry of a kernel map that was queued ahead of its use, once its count has
    reached the host (None: not such a map, or not yet).  Never waits."""
    index = out_in_map.device.index
    state = _stream_states.get((index if index is not None else _cur_device(), _stream()))
    if state is None:
        return None
    hit = state.pairs_of.get(id(out_in_map))
    if hit is None or hit[0]() is not out_in_map:
        return None
    if state.pair_vals is None:
        event = state.pair_event
        if event is None or not event.query():
            return None
        state.pair_vals, state.pair_event = state.pair_host.tolist(), None
    return state.pair_vals[hit[1]] / max(hit[2], 1)


def _map_queued_ahead(in_coords, out_coords, ks, st, pd) -> Optional[torch.Tensor]:
    """The map of kmap_sorted(in_coords, out_coords, ...) if it was queued ahead on the second
    stream; notes the request when both operands are levels of the chain in flight."""
    index = in_coords.device.index
    state = _stream_states.get((index if index is not None else _cur_device(), _stream()))
    if state is None:
        return None
    a = state.level_index.get(id(in_coords))
    if a is None:  # (the common miss, answered without the lock: neither table is changed here)
        return None
    with _state_lock:
        b = state.level_index.get(id(out_coords))
        if b is None or a[0]() is not in_coords or b[0]() is not out_coords:
            return None
        request = (a[1], b[1], ks, st, pd)
        if request not in state.map_plan_seen:
            state.map_plan_seen.append(request)
        hit = state.maps_ahead.pop((id(in_coords), id(out_coords), ks, st, pd), None)
        if (hit is None or hit[0]() is not in_coords or hit[1]() is not out_coords
                or hit[3] != (in_coords._version, out_coords._version)):
            return None
        main = state.maps_main  # the caller's stream (this state belongs to it)
        if state.maps_event is not None:
            # usually the second stream is long done: then nothing has to wait on the device (a
            # wait on a pending event costs the host 25 us, the query 2); later takers on this
            # stream are ordered behind the wait
            if not state.maps_event.query():
                main.wait_event(state.maps_event)
            state.maps_event = None
        state.maps_ahead_hits += 1
        _remember(_map_requests, id(hit[2]), (weakref.ref(hit[2]), state, request, hit[4]), 64)
        if state.segments_todo is not None and any(j[0] is hit[2] for j in state.segments_todo):
            jobs, state.segments_todo = state.segments_todo, None
            main_handle = _stream()
            for (omap, n_rows, kvol), seg in zip(jobs, _build_pair_segments_batch(jobs, hit[2].device)):
                _remember(_segments_of, id(omap), (weakref.ref(omap), omap._version, omap.data_ptr(),
                                                   main_handle, n_rows, seg), 64)
            state.segments_hits += len(jobs)
            state.segments_ids = tuple(id(j[0]) for j in jobs)
        return hit[2]


# Maps queued before the row counts are known.  A chain that emits its rows before the read-back
# leaves every level's count on the device; the launch that searches the planned maps can take the
# counts from there (tsmi_kmap_sorted_batch: n_in_dev / n_out_dev), sized by the one bound the host
# has - no level has more rows than the chain's root.  The maps are then queued right behind the
# chain, before the host has seen a count, instead of after the read-back and the host work that
# follows it: with a new coordinate tensor every forward, when nothing of the previous forward
# hides that start-up, the first strided layer finds its map ~0.15 ms earlier.  Only for roots of
# at most 131,072 rows (larger inputs search through samples gathered per input).
kmap_queue_before_counts = True
# A forward that starts with the device drained hands its maps out without the second stream's
# event traffic (see _queue_maps_ahead).
kmap_register_on_drained_stream = True
# The map over a caller's own rows - the first a network asks for - is built on the second stream
# when its chain is queued there ahead of the forward (rows known to be complete): 23 us of the
# caller's stream, where a forward over known rows is bound by its kernels.
kmap_root_on_second_stream = True
_EARLY_MAX_ROWS = 131072


def _launch_maps_early(state, job, coords) -> None:
    """Queues the maps of the plan over the levels ``job`` is emitting, on the current (second)
    stream, with the row counts read from ``job.ctr`` on the device.  Leaves what
    _queue_maps_ahead needs to hand the maps out in ``job.early``.  _state_lock held."""
    plan = tuple(state.map_plan_seen)
    n = coords.shape[0]
    if not plan or n > _EARLY_MAX_ROWS or _sample_elems(n) != 0:
        return
    transposed, dev = frozenset(state.transposed_seen), coords.device
    # rows to provide for per level: the root's count is the only bound there is, but the chain of
    # the forward before is the better guess - an eighth and 1024 rows above its counts, and a
    # level that turns out larger has its maps queued again once the counts are known (the launch
    # never looks past the rows it was given room for)
    seen = state.level_counts
    bound = [n] + [min(n, seen[l] + seen[l] // 8 + 1024) if l < len(seen) else n for l in range(job.levels)]
    todo, rows_of, t_ints = [], {}, 0
    for request in plan:
        i, o, ks, st, pd = request
        if max(i, o) > job.levels or max(i, o) == 0:
            continue
        kvol = ks[0] * ks[1] * ks[2]
        first = rows_of.get(kvol, 0)
        rows_of[kvol] = first + make_divisible(bound[o], 128)
        t_first = -1
        if request in transposed:
            t_first = t_ints
            t_ints += make_divisible(bound[i], 128) * kvol
        todo.append((request, kvol, first, t_first))
    if not todo:
        return
    buffers = {kvol: torch.empty((rows, kvol), dtype=torch.int32, device=dev) for kvol, rows in rows_of.items()}
    t_buffer = torch.full((t_ints,), -1, dtype=torch.int32, device=dev) if t_ints else None
    counted = map_pairs_counted and len(todo) <= _PAIR_SLOTS
    if counted and state.pair_dev is None:
        state.pair_dev = torch.zeros(3 * _PAIR_SLOTS, dtype=torch.int64, device=dev)
        state.pair_host = torch.zeros(_PAIR_SLOTS, dtype=torch.int64, pin_memory=True)
    pair_ptr = state.pair_dev.data_ptr() if counted else 0
    root, rows_ptr, ctr_ptr = coords.data_ptr(), job.rows.data_ptr(), job.ctr.data_ptr()
    flat = []
    for slot, ((i, o, ks, st, pd), kvol, first, t_first) in enumerate(todo):
        # level 0: the root (its count is on the host); level l >= 1: rows[l - 1], count in ctr[8 (l - 1)]
        flat += (root if i == 0 else rows_ptr + (i - 1) * n * 16, bound[i],
                 root if o == 0 else rows_ptr + (o - 1) * n * 16, bound[o], make_divisible(bound[o], 128), 0,
                 buffers[kvol].data_ptr() + first * kvol * 4, *ks, *st, *pd,
                 0 if t_first < 0 else t_buffer.data_ptr() + 4 * t_first, make_divisible(bound[i], 128),
                 pair_ptr + 16 * slot if counted else 0, pair_ptr + 8 * (2 * _PAIR_SLOTS + slot) if counted else 0,
                 0 if i == 0 else ctr_ptr + 32 * (i - 1), 0 if o == 0 else ctr_ptr + 32 * (o - 1))
    _check(_C.tsmi_kmap_sorted_batch(_stream(), len(todo), (ctypes.c_int64 * len(flat))(*flat)))
    # (what follows the launch needs no count either: off the host's hands before the counts arrive)
    if counted:
        if state.pair_out is None:
            state.pair_out = state.pair_dev[2 * _PAIR_SLOTS:]
        state.pair_host.copy_(state.pair_out, non_blocking=True)
    event = torch.cuda.Event()
    event.record()
    main = state.main_stream
    if main is not None:
        for buf in buffers.values():
            buf.record_stream(main)  # allocated on the second stream, read and freed on the caller's
        if t_buffer is not None:
            t_buffer.record_stream(main)
    job.early = (tuple(t[0] for t in todo), todo, buffers, t_buffer, counted, transposed, bound, main, event)


def _queue_maps_ahead(state, chain_rows, on_side: bool, job=None) -> None:
    """Called when the rows of a chain's levels (``chain_rows[0]``: its root) have become known
    on the host: the requests of the forward before become this forward's plan, and - when the
    rows were emitted on the second stream - the planned maps are queued there, or, where
    _launch_maps_early has queued them already, cut to their sizes and handed out.  Runs with
    _state_lock held, the caller's stream current."""
    state.level_index = {id(t): (weakref.ref(t), i) for i, t in enumerate(chain_rows)}
    plan, state.map_plan_seen = tuple(state.map_plan_seen), []
    state.map_plan = plan
    state.transposed_plan, state.transposed_seen = frozenset(state.transposed_seen), set()
    state.segments_plan, state.segments_seen = frozenset(state.segments_seen), set()
    state.maps_ahead = {}
    state.maps_event = None
    state.segments_todo = None
    if state.segments_ids:
        # (the segments built ahead for the forward before, over maps that are gone: up to 20 MB a forward)
        for key in state.segments_ids:
            hit = _segments_of.get(key)
            if hit is not None and hit[0]() is None:
                _segments_of.pop(key, None)
        state.segments_ids = ()
    state.pairs_of, state.pair_event, state.pair_vals = {}, None, None

    def behind_rows():
        # (_grid_finish left the caller's stream in front of the launch that emitted the rows)
        if job is not None and job.rows_wait_deferred:
            job.rows_wait_deferred = False
            if job.rows_event is not None and not job.rows_event.query():
                torch.cuda.current_stream(chain_rows[0].device).wait_event(job.rows_event)

    if not (kmap_queue_ahead and on_side and plan and state.side is not None and kmap_through_sorted):
        return behind_rows()
    early = getattr(job, "early", None)
    if early is not None and (early[0] != tuple(r for r in plan if 0 < max(r[0], r[1]) <= job.levels)
                              or any((r in early[5]) != (r in state.transposed_plan) for r in early[0])):
        early = None  # (the plan changed between the two halves of the chain: queue the maps now)
    if early is not None and any(t.shape[0] > early[6][l] for l, t in enumerate(chain_rows)):
        early = None  # (a level outgrew the room its maps were given)
    # maps of one kernel volume share an allocation, the transposed maps another: one hand-over
    # between the streams each
    todo, rows_of, t_ints = [], {}, 0
    if early is not None:
        _, early_todo, buffers, t_buffer, counted, _, _, recorded_for, early_event = early
        state.maps_early_hits += 1
        for slot, (request, kvol, first, t_first) in enumerate(early_todo):
            i, o, ks, st, pd = request
            with_segments = request in state.segments_plan
            if max(i, o) >= len(chain_rows) or chain_rows[i].shape[0] == 0 or chain_rows[o].shape[0] == 0:
                continue  # (a chain that ended early: the launch found no rows and wrote nothing)
            todo.append((chain_rows[i], chain_rows[o], ks, st, pd, kvol, first, t_first, with_segments, slot))
    else:
        for request in plan:
            i, o, ks, st, pd = request
            if max(i, o) >= len(chain_rows) or max(i, o) == 0:  # (the root's own map is asked for before this point)
                continue
            a, b = chain_rows[i], chain_rows[o]
            if a.shape[0] == 0 or b.shape[0] == 0:
                continue
            kvol = ks[0] * ks[1] * ks[2]
            first = rows_of.get(kvol, 0)
            rows_of[kvol] = first + make_divisible(b.shape[0], 128)
            # the transposed map comes out of the same launch where the forward before asked for it
            t_first = -1
            if request in state.transposed_plan:
                t_first = t_ints
                t_ints += make_divisible(a.shape[0], 128) * kvol
            with_segments = request in state.segments_plan
            todo.append((a, b, ks, st, pd, kvol, first, t_first, with_segments, len(todo)))
    if not todo:
        return behind_rows()
    dev = chain_rows[0].device
    main = state.main_stream  # (asking torch for the current stream costs 5 us)
    if main is None or main.cuda_stream != _stream():
        main = state.main_stream = torch.cuda.current_stream(dev)
    state.maps_main = main
    if early is None:
        recorded_for = None
    # A forward that began with the device drained (the read-back of a new tensor's check) has the
    # device waiting for the host here: nothing is to be gained from the second stream, and an event
    # record plus the wait for it at the first map cost the host 30 us.  The pair segments then go
    # to the caller's stream, behind the maps, which were queued before the row counts arrived.
    drained = False
    if early is not None and _drained:
        hit = _drained.pop((dev.index, main.cuda_stream), None)
        drained = kmap_register_on_drained_stream and hit is not None and hit() is chain_rows[0]
    behind_rows()  # (by now a query of the event that finds it complete)
    if not drained:
        torch.cuda.set_stream(state.side)  # (the context manager costs 6 us, two switches 0.8)
    try:
        if early is None:
            buffers = {kvol: torch.empty((rows, kvol), dtype=torch.int32, device=dev) for kvol, rows in rows_of.items()}
            # (one fill for the transposed maps of all levels; the map launch stores their entries)
            t_buffer = torch.full((t_ints,), -1, dtype=torch.int32, device=dev) if t_ints else None
            counted = map_pairs_counted and len(todo) <= _PAIR_SLOTS
            if counted and state.pair_dev is None:
                state.pair_dev = torch.zeros(3 * _PAIR_SLOTS, dtype=torch.int64, device=dev)
                state.pair_host = torch.zeros(_PAIR_SLOTS, dtype=torch.int64, pin_memory=True)
        pair_ptr = state.pair_dev.data_ptr() if counted else 0
        flat, queued, pairs_of = [], {}, {}
        segment_jobs = []
        for a, b, ks, st, pd, kvol, first, t_first, with_segments, slot in todo:
            n_pad = make_divisible(b.shape[0], 128)
            omap = buffers[kvol].narrow(0, first, n_pad)
            omap_t, t_pad = None, make_divisible(a.shape[0], 128)
            if t_first >= 0:  # (where the transposed map lies: the view is cut when a layer asks for it)
                omap_t = (t_buffer, t_first, t_pad, kvol)
            if early is None:
                samples = _sorted_samples(a)
                flat += (a.data_ptr(), a.shape[0], b.data_ptr(), b.shape[0], n_pad,
                         0 if samples is None else samples.data_ptr(), omap.data_ptr(), *ks, *st, *pd,
                         0 if omap_t is None else t_buffer.data_ptr() + 4 * t_first, t_pad,
                         pair_ptr + 16 * slot if counted else 0,
                         pair_ptr + 8 * (2 * _PAIR_SLOTS + slot) if counted else 0, 0, 0)
            queued[(id(a), id(b), ks, st, pd)] = (weakref.ref(a), weakref.ref(b), omap, (a._version, b._version),
                                                  omap_t)
            if counted:
                pairs_of[id(omap)] = (weakref.ref(omap), slot, b.shape[0] * kvol)
            if with_segments:
                segment_jobs.append((omap, b.shape[0], kvol))
        if early is None:
            _check(_C.tsmi_kmap_sorted_batch(_stream(), len(todo), (ctypes.c_int64 * len(flat))(*flat)))
        # the pair segments the forward before built over these maps, behind the maps on this
        # stream instead of in front of their first layer on the caller's
        if segment_jobs and drained:
            # (on the caller's stream, which is not behind the maps yet: queued when the first of
            # these maps is taken - the first map taken at all has waited for them by then)
            state.segments_todo, segment_jobs = segment_jobs, None
        if segment_jobs:
            segs = _build_pair_segments_batch(segment_jobs, dev)
            segs[0].buffer.record_stream(main)
            main_handle = main.cuda_stream
            for (omap, n_rows, kvol), seg in zip(segment_jobs, segs):
                _remember(_segments_of, id(omap), (weakref.ref(omap), omap._version, omap.data_ptr(),
                                                   main_handle, n_rows, seg), 64)
            state.segments_hits += len(segs)
            state.segments_ids = tuple(id(j[0]) for j in segment_jobs)
        if counted and early is None:  # (counts of maps queued before the row counts are on their way already)
            if state.pair_out is None:
                state.pair_out = state.pair_dev[2 * _PAIR_SLOTS:]
            state.pair_host.copy_(state.pair_out, non_blocking=True)
        if drained:
            event = early_event
        else:
            event = torch.cuda.Event()
            event.record()
    finally:
        if not drained:
            torch.cuda.set_stream(main)
    if recorded_for is None or recorded_for.cuda_stream != main.cuda_stream:
        for buf in buffers.values():
            buf.record_stream(main)  # allocated on the second stream, read and freed on the caller's
        if t_buffer is not None:
            t_buffer.record_stream(main)
    # (only now: a call that failed above leaves no map behind that was never written)
    state.maps_ahead, state.maps_event = queued, event
    if counted:
        state.pairs_of, state.pair_event = pairs_of, event


def _kmap_sorted_launch(in_coords, out_coords, ks, st, pd, omap=None) -> torch.Tensor:
    """The launch of kmap_sorted on the current stream (operands checked by the caller), into
    ``omap`` (int32 [ceil128(N_out), K_vol]) when given."""
    n_out = out_coords.shape[0]
    n_pad = make_divisible(n_out, 128)
    if omap is None:
        omap = out_coords.new_empty(n_pad, ks[0] * ks[1] * ks[2])
    samples = _sorted_samples(in_coords)
    _check(_C.tsmi_kmap_sorted(_stream(), in_coords.data_ptr(), in_coords.shape[0], out_coords.data_ptr(),
                               n_out, n_pad, _i3(ks), _i3(st), _i3(pd), _ptr(samples), omap.data_ptr()))
    return omap


@functools.lru_cache(maxsize=1024)
def _sample_elems(n: int) -> int:
    return _C.tsmi_kmap_sorted_samples_elems(n)


_samples_of = {}  # id(coords) -> (weak reference, version, address, stream, samples)


def _sorted_samples(coords: torch.Tensor) -> Optional[torch.Tensor]:
    """The search samples of a large input (None below 131073 rows), gathered once per
    coordinate tensor and stream: the submanifold and the strided map of a level share them."""
    n = coords.shape[0]
    elems = _sample_elems(n)
    if elems == 0:
        return None
    stream = _stream()
    hit = _samples_of.get(id(coords))
    if (hit is not None and hit[0]() is coords and hit[1] == coords._version
            and hit[2] == coords.data_ptr() and hit[3] == stream):
        return hit[4]
    samples = torch.empty(elems, dtype=torch.int64, device=coords.device)
    _check(_C.tsmi_kmap_sorted_samples(stream, _ptr(coords), n, _ptr(samples)))
    _remember(_samples_of, id(coords), (weakref.ref(coords), coords._version, coords.data_ptr(), stream, samples),
              64)
    return samples


def _settle_insert(coords: torch.Tensor, status: torch.Tensor) -> None:
    """After an insert pass over ``coords`` that collected its flags in ``status``: read them
    (one synchronisation) unless these rows are known to be in range."""
    if _range_known(coords):
        return
    flags = int(status.item())
    if flags & 2:
        raise _range_error()
    if flags & 1:
        raise ValueError("The capacity of hashtable is not sufficient.")
    _mark_range_ok(coords)


class GPUHashTable:
    """Non-owning view of (keys int64[cap], vals int32[cap]) or, given an int, an
    owning table of that capacity — hashmap/hashmap_cuda.cuh:65-121."""

    def __init__(self, keys, vals: Optional[torch.Tensor] = None, device="cuda", zero: bool = True):
        self.counters = None
        if isinstance(keys, int):
            # one allocation: keys (int64 view), vals, 8 spare counters; zero-filled unless the
            # caller's first pass over the table clears it (build_subm)
            cap = make_divisible(max(int(keys), 8), 8)
            buf = (torch.zeros if zero else torch.empty)(3 * cap + 8, dtype=torch.int32, device=device)
            self.keys = buf[:2 * cap].view(torch.int64)
            self.vals = buf[2 * cap:3 * cap]
            if zero:
                self.counters = buf[3 * cap:]
            self._status = buf[3 * cap + 3:3 * cap + 4]
        else:
            self.keys = _need(keys, torch.int64, "hashmap_keys")
            self.vals = _need(vals, torch.int32, "hashmap_vals")
            if self.keys.numel() != self.vals.numel():
                raise ValueError("hashmap_keys and hashmap_vals differ in length")
        self.capacity = self.keys.numel()

    def get_capacity(self) -> int:
        return self.capacity

    def clear(self) -> None:
        _check(_C.tsmi_hashtable_clear(_stream(), _ptr(self.keys), _ptr(self.vals), self.capacity))

    def insert_bxyz(self, coords: torch.Tensor) -> None:
        given = coords
        coords = _need(coords, torch.int32, "coords")
        known = _range_known(given)
        status = None
        if not known:
            status = torch.zeros(1, dtype=torch.int32, device=coords.device)
        _check(_C.tsmi_hashtable_insert_coords(_stream(), _ptr(self.keys), _ptr(self.vals),
                                               self.capacity, _ptr(coords), coords.shape[0], _ptr(status)))
        if not known:
            _settle_insert(given, status)

    @classmethod
    def build_subm(cls, coords: torch.Tensor, kernel_size, rsv_ratio: float = 2.0):
        """(table over ``coords``, stride-1 map of ``kernel_size``) in one call: the table is
        emptied and the map filled by one launch, then insert, then query."""
        given = coords
        coords = _need(coords, torch.int32, "coords")
        ks = _triple(kernel_size)
        n = coords.shape[0]
        table = cls(hash_capacity(n, rsv_ratio), device=coords.device, zero=False)
        n_pad = make_divisible(n, 128)
        omap = torch.empty((n_pad, ks[0] * ks[1] * ks[2]), dtype=torch.int32, device=coords.device)
        _check(_C.tsmi_kmap_build_subm(_stream(), _ptr(table.keys), _ptr(table.vals), table.capacity,
                                       _ptr(coords), n, n_pad, _I3(*ks), _ptr(omap), _ptr(table._status)))
        _settle_insert(given, table._status)
        return table, omap

    def query_subm_bxyz(self, coords, kernel_size) -> torch.Tensor:
        """Stride-1 map over the table's own coordinates (row i inserted with value i).  Odd
        kernels probe half of the offsets and mirror the hits; even ones take the general
        query with offsets 0..ks-1."""
        ks = _triple(kernel_size)
        if any(k % 2 == 0 for k in ks):
            return self.query_bxyz(coords, ks, (1, 1, 1), _subm_pad(ks))
        coords = _need(coords, torch.int32, "coords")
        n = coords.shape[0]
        n_pad = make_divisible(n, 128)
        omap = torch.empty((n_pad, ks[0] * ks[1] * ks[2]), dtype=torch.int32, device=coords.device)
        _check(_C.tsmi_kmap_query_subm(_stream(), _ptr(self.keys), _ptr(self.vals), self.capacity,
                                       _ptr(coords), n, n_pad, _I3(*ks), _ptr(omap)))
        return omap

    def query_bxyz(self, out_coords, kernel_size, stride, pad, n_pad=None) -> torch.Tensor:
        out_coords = _need(out_coords, torch.int32, "coords")
        ks, st, pd = _triple(kernel_size), _triple(stride), _triple(pad)
        n = out_coords.shape[0]
        n_pad = make_divisible(n, 128) if n_pad is None else n_pad
        omap = out_coords.new_empty(n_pad, ks[0] * ks[1] * ks[2])
        _check(_C.tsmi_kmap_query(_stream(), _ptr(self.keys), _ptr(self.vals), self.capacity,
                                  _ptr(out_coords), n, n_pad, _I3(*ks), _I3(*st), _I3(*pd),
                                  _ptr(omap)))
        return omap

    # --- the reference's method names; its coordinate rows are (x, y, z, b) ---

    def insert_coords(self, coords_xyzb: torch.Tensor) -> None:
        self.insert_bxyz(coords_xyzb[:, [3, 0, 1, 2]].contiguous())

    def lookup_coords(self, coords_xyzb, kernel_sizes, strides, kernel_volume=None) -> torch.Tensor:
        """int32 [ceil128(N), K_vol] of row index + 1, 0 = miss
        (hashmap/hashmap_cuda.cuh:199-253: in = out*stride + digit - (ks-1)/2)."""
        ks = _triple(kernel_sizes)
        pad = tuple((k - 1) // 2 for k in ks)
        omap = self.query_bxyz(coords_xyzb[:, [3, 0, 1, 2]].contiguous(), ks, strides, pad)
        return omap.add_(1)

    def insert_vals(self, keys: torch.Tensor) -> None:
        keys = _need(keys, torch.int64, "keys")
        _check(_C.tsmi_hashtable_insert_keys(_stream(), _ptr(self.keys), _ptr(self.vals),
                                             self.capacity, _ptr(keys), keys.numel(), None))

    def lookup_vals(self, keys: torch.Tensor) -> torch.Tensor:
        keys = _need(keys, torch.int64, "keys")
        out = torch.empty(keys.numel(), dtype=torch.int32, device=keys.device)
        _check(_C.tsmi_hashtable_lookup_keys(_stream(), _ptr(self.keys), _ptr(self.vals),
                                             self.capacity, _ptr(keys), keys.numel(), _ptr(out)))
        return out


# --------------------------------------------------------------------- kernel maps


def _subm_pad(ks: Sequence[int]) -> Tuple[int, ...]:
    """Effective padding of a stride-1 map: centred offsets for an odd kernel volume,
    offsets 0..ks-1 for an even one (others/sparsemapping_cuda.cu:165-170,209-214)."""
    odd = (ks[0] * ks[1] * ks[2]) % 2 == 1
    return tuple((k - 1) // 2 if odd else 0 for k in ks)


def build_kernel_map_subm_hashmap(table: GPUHashTable, coords, coords_min, coords_max,
                                  kernel_sizes, stride, padding, to_insert: bool) -> List[torch.Tensor]:
    """[out_in_map int32 [ceil128(N), K_vol]] — others/sparsemapping_cuda.cu:303-345.
    coords_min / coords_max are accepted for signature compatibility; the table key
    is the packed coordinate itself, so no extent is needed."""
    ks = _triple(kernel_sizes)
    if to_insert:
        table.insert_bxyz(coords)
    return [table.query_subm_bxyz(coords, ks)]


def coords_max(coords: torch.Tensor) -> torch.Tensor:
    """Device int32[4] per-column maximum (no host synchronisation)."""
    coords = _need(coords, torch.int32, "coords")
    out = torch.empty(4, dtype=torch.int32, device=coords.device)
    _check(_C.tsmi_coords_max(_stream(), _ptr(coords), coords.shape[0], _ptr(out), 1))
    return out


def downsample_coords(coords: torch.Tensor, kernel_sizes, stride, padding, coords_max_host=None,
                      mode: int = 0, rsv_ratio: float = 2.0, allow_negative: bool = False,
                      _reserve_all: bool = False, want_table: bool = True):
    """Output coordinates of a strided convolution in ascending (b,x,y,z) order and
    the hash table that indexes them.  Returns (out_coords, GPUHashTable); with
    ``want_table=False`` the table may be None (callers that search the sorted rows).
    One host read-back (the number of outputs) — the reference has two
    (others/sparsemapping_cuda.cu:477-479).  With ``allow_negative`` the outputs are bounded
    below by the reference's coords_min (hashmap_on_the_fly.py:39-43) instead of 0."""
    coords = _need(coords, torch.int32, "coords")
    ks, st, pd = _triple(kernel_sizes), _triple(stride), _triple(padding)
    n = coords.shape[0]
    dev = coords.device
    # a voxel has up to prod(ceil(ks/stride)) outputs; reserve for the ones a surface
    # typically produces, and for all of them on a second attempt when that was too few (the
    # reference sizes its table for two outputs per input and raises, hashmap_on_the_fly.py:56-58)
    fan = 1
    if mode == 0:
        for k, s in zip(ks, st):
            fan *= -(-k // s)
    if mode == 3:  # generative upsampling: up to one output per (input, offset)
        cap = hash_capacity(n * ks[0] * ks[1] * ks[2], rsv_ratio)
    else:
        cap = hash_capacity(n * (fan if _reserve_all else min(fan, 2)), rsv_ratio)
    through_grid = (mode == 0 and not allow_negative and n > 0 and downsample_through_grid
                    and not _reserve_all)
    table = None
    if through_grid:
        with _state_lock:
            state = _strided_state(dev)
            chain = (ks, st, pd, rsv_ratio) if coords_max_host is None else None
            job, state.pending = state.pending, None
            ahead = state.chain_step(coords, chain)
            if not isinstance(ahead, int):  # computed ahead when the previous level of the chain was
                if want_table and ahead[1] is None:
                    tbl = GPUHashTable(hash_capacity(ahead[0].shape[0], rsv_ratio), device=dev)
                    tbl.insert_bxyz(ahead[0])
                    return ahead[0], tbl
                return ahead
            if _range_origin(coords) == "user":
                # what strided_lookahead starts next time (None: a call it cannot serve, e.g. one
                # bounded by a spatial range - nothing is queued ahead for such rows any more)
                state.root_chain = chain
            if (job is not None and job.coords is coords and job.geom == (ks, st, pd)
                    and job.coords_max_host is None and coords_max_host is None
                    and job.levels == 1 + ahead and state.pending_rsv == rsv_ratio):
                state.lookahead_hits += 1
                done = _grid_finish(state, job, rsv_ratio, cap, want_table)
            else:
                # (a look-ahead that does not fit this call left marks behind: bitmap() clears them)
                done = _downsample_coords_grid(state, coords, ks, st, pd, coords_max_host, fan, rsv_ratio,
                                               cap, ahead, want_table)
            if done is not None:
                state.chain_last = weakref.ref(done[0])
                return done
    if table is None:
        table = GPUHashTable(cap, device=dev)
    counters = table.counters  # zero on a fresh table
    in_max = in_min = None
    host_max = None
    if mode == 3:
        host_max = _I3(*[int(v) for v in coords_max_host])
    elif mode == 0:
        if coords_max_host is not None:
            host_max = _I3(*[int(v) for v in coords_max_host])
        elif allow_negative and n > 0:
            in_max = coords.max(0).values.contiguous()  # the true maxima, possibly negative
        else:
            in_max = counters[4:8]  # still zero: the maximum lands here without a fill launch
            _check(_C.tsmi_coords_max(_stream(), _ptr(coords), n, _ptr(in_max), 0))
        if allow_negative and n > 0:
            in_min = coords.min(0).values.contiguous()
    s = _stream()
    _check(_C.tsmi_downsample_candidates(s, _ptr(coords), n, _I3(*ks), _I3(*st), _I3(*pd), host_max,
                                         _ptr(in_max), _ptr(in_min), mode, _ptr(table.keys), cap,
                                         _ptr(counters)))
    # unique keys = the occupied slots of the table: compact, read the count back, sort
    temp_bytes = _C.tsmi_sort_temp_bytes(cap)
    scratch = torch.empty(2 * cap + temp_bytes // 8 + 1, dtype=torch.int64, device=dev)
    uniq, sorted_keys, temp = scratch[:cap], scratch[cap:2 * cap], scratch[2 * cap:]
    _check(_C.tsmi_hashtable_compact_keys(s, _ptr(table.keys), cap, _ptr(uniq), _ptr(counters)))
    n_out, overflow, _, unpackable = counters[:4].tolist()
    if unpackable:
        raise _range_error()
    _mark_range_ok(coords)
    if overflow and mode == 0 and fan > 2 and not _reserve_all:
        return downsample_coords(coords, kernel_sizes, stride, padding, coords_max_host, mode, rsv_ratio,
                                 allow_negative, _reserve_all=True)
    if overflow:
        raise ValueError(
            "The capacity of hashtable is not sufficient. Please enlarge reserved space for "
            "hashtable:\n # Python \nimport torchsparse_amd.backends\n"
            "torchsparse_amd.backends.hash_rsv_ratio=#Value")
    out_coords = torch.empty((n_out, 4), dtype=torch.int32, device=dev)
    if n_out > 0:
        _check(_C.tsmi_sort_keys(s, _ptr(uniq), _ptr(sorted_keys), n_out, 63, _ptr(temp), temp_bytes))
        _check(_C.tsmi_downsample_finalize(s, _ptr(sorted_keys), n_out, _ptr(table.keys),
                                           _ptr(table.vals), cap, _ptr(out_coords)))
    _mark_range_ok(out_coords, ascending=True)  # unpacked from sorted keys
    return out_coords, table


# Strided output coordinates go through an occupancy bitmap of the output grid when it is small
# enough (no sort); False keeps every call on the hash-and-sort path.
downsample_through_grid = True
# Networks apply the same strided convolution level after level (k2 s2 four times in a U-Net).
# Once such a chain has been seen, the call for its first level also computes the following
# levels (each from the previous level's bitmap) before the one read-back of the output counts,
# so the later calls return at once and the forward synchronises once instead of once per
# level.  Levels computed ahead and never asked for cost their kernels, not a read-back.
downsample_chain_ahead = True
_GRID_CHUNK_WORDS = 512
_GRID_LEVELS = 4  # the level asked for and up to three ahead
_MAX_STREAM_STATES = 8  # (device, stream) pairs whose scratch is kept; the least recently used goes


class _StridedState:
    """What the strided-coordinate path keeps between calls, for ONE (device, stream): the
    occupancy-bitmap scratch, the chain of equal strided calls in progress, the lengths of the
    chains seen, and the levels computed ahead.  Everything in it was produced by work queued
    on that stream, so a later call on the same stream is ordered after it; calls on another
    stream (or device) get a state of their own and never see these tensors."""
    __slots__ = ("grid_buf", "grid_words", "grid_dirty", "chain_geom", "chain_last", "chain_count",
                 "chain_len", "ahead", "ahead_hits", "host_counters", "pending", "pending_rsv", "root_chain",
                 "lookahead_hits", "side", "grid_event", "grid_event_stream", "grid_old", "level_index", "map_plan",
                 "map_plan_seen", "maps_ahead", "maps_event", "maps_ahead_hits", "maps_main", "transposed_plan",
                 "maps_early_hits", "level_counts", "main_stream", "pair_out", "segments_todo", "segments_ids",
                 "transposed_seen", "transposed_hits", "pair_dev", "pair_host", "pair_event", "pair_vals", "pairs_of",
                 "segments_plan", "segments_seen", "segments_hits")

    def __init__(self):
        self.grid_buf = None      # int32 scratch: bitmaps and chunk counts of every level
        self.grid_words = 0       # bitmap words of level 0 the scratch was laid out for
        self.grid_dirty = False   # a call marked bits and did not reach its emit passes
        self.chain_geom = None    # geometry of the chain in progress
        self.chain_last = None    # weak reference to the last output of that chain
        self.chain_count = 0
        self.chain_len = {}       # geometry -> length of the last chain that ended
        self.ahead = {}           # id(coords) -> (weakref(coords), geometry, out_coords, table)
        self.ahead_hits = 0       # calls answered from `ahead` (diagnostic)
        self.host_counters = None  # pinned int32 buffer the counters are copied into
        self.pending = None       # _GridJob started at a submanifold build, not yet asked for
        self.pending_rsv = None
        self.root_chain = None    # geometry of the last chain that started from a caller's own rows
        self.lookahead_hits = 0   # chains whose first half was already queued (diagnostic)
        self.side = None          # second stream of the device, for chains queued ahead of their use
        self.grid_event = None    # end of the last work queued on the bitmap scratch, on either stream
        self.grid_event_stream = 0  # ... and the stream it was queued on
        self.grid_old = None      # the scratch before it last grew (kept until the next growth)
        self.level_index = {}     # id(rows) -> (weak reference, position in the chain in flight; 0: its root)
        self.map_plan = ()        # sorted-map builds the last forward asked for over its chain's levels
        self.map_plan_seen = []   # ... the forward in flight has asked for so far
        self.maps_ahead = {}      # (id(in), id(out), ks, st, pd) -> (refs, map) queued on the side stream
        self.maps_event = None    # end of that queue; None once the caller's stream has waited for it
        self.maps_ahead_hits = 0  # maps answered from `maps_ahead` (diagnostic)
        self.maps_early_hits = 0  # forwards whose maps were queued before the counts were read (diagnostic)
        self.main_stream = None   # torch's object for the stream this state belongs to
        self.pair_out = None      # the last third of pair_dev (the counts)
        self.segments_todo = None  # pair-segment builds left for the first take of one of their maps
        self.segments_ids = ()     # ids of the maps whose segments were built ahead last
        self.level_counts = []    # rows of the levels of the last chain (the root's not among them)
        self.maps_main = None     # the caller's stream object at the time of that queue
        self.transposed_plan = frozenset()  # requests of map_plan whose transposed map was asked for too
        self.transposed_seen = set()
        self.transposed_hits = 0  # transposed maps answered by the launch of their strided map (diagnostic)
        # pair counts of the maps queued ahead: int64 [3 * 16] on the device (two words the blocks add
        # up in and take tickets from, then the count, per map), pinned copy of the counts, the event
        # behind that copy (None once it was seen done), the counts as a list, id(map) -> (ref, slot, entries)
        self.segments_plan = frozenset()  # requests of map_plan whose pair segments were asked for too
        self.segments_seen = set()
        self.segments_hits = 0     # pair segments that were built on the second stream (diagnostic)
        self.pair_dev = None
        self.pair_host = None
        self.pair_event = None
        self.pair_vals = None
        self.pairs_of = {}

    def chain_step(self, coords, geom):
        """Book-keeping of chains of equal strided calls (each on the previous one's outputs).
        Returns the (out_coords, table) computed ahead for ``coords``, or the number of levels
        to compute ahead now."""
        hit = self.ahead.pop(id(coords), None)
        last = self.chain_last() if self.chain_last is not None else None
        if geom is not None and self.chain_geom == geom and last is coords:
            self.chain_count += 1
            if hit is not None and hit[0]() is coords and hit[1] == geom and downsample_chain_ahead:
                self.chain_last = weakref.ref(hit[2])
                self.ahead_hits += 1
                return hit[2], hit[3]
            return 0
        if self.chain_geom is not None:
            self.chain_len[self.chain_geom] = self.chain_count
        self.chain_geom, self.chain_count, self.chain_last = geom, 1, None
        self.ahead.clear()
        if geom is None or not downsample_chain_ahead:
            return 0
        return min(self.chain_len.get(geom, 1) - 1, _GRID_LEVELS - 1)

    def bitmap(self, dev: torch.device, words: int):
        """The all-zero scratch whose first bitmap has at least ``words`` words.  Every call
        leaves the bitmaps zero again; one that did not finish has them cleared here."""
        if self.grid_buf is None or self.grid_words < words:
            self.grid_old = self.grid_buf  # work queued on the other stream may still hold its address
            self.grid_buf = torch.zeros(_grid_layout(words)[1], dtype=torch.int32, device=dev)
            self.grid_words, self.grid_dirty = words, False
        elif self.grid_dirty:
            self.grid_buf.zero_()
            self.grid_dirty = False
        return self.grid_buf


_stream_states = collections.OrderedDict()  # (device index, stream) -> _StridedState
_state_lock = threading.RLock()  # guards _stream_states and every _StridedState


def _strided_state(dev: torch.device) -> _StridedState:
    """State of the current stream of ``dev`` (call with _state_lock held)."""
    key = (dev.index if dev.index is not None else _cur_device(), _stream())
    st = _stream_states.get(key)
    if st is None:
        st = _stream_states[key] = _StridedState()
        while len(_stream_states) > _MAX_STREAM_STATES:
            _stream_states.popitem(last=False)
    else:
        _stream_states.move_to_end(key)
    return st


def release_scratch() -> None:
    """Drop the scratch bitmaps, the levels computed ahead and the chain history of every
    stream (up to ~170 MB of device memory per stream that ran a large strided map), and the
    buffers the convolutions of a stream share for partial sums and per-pair products (they
    grow to the largest layer seen: K_vol * ceil128(N_out) * Cout elements for a layer over
    pair segments)."""
    with _state_lock:
        _stream_states.clear()
    with _scratch_lock:
        _SCRATCH.clear()


def _grid_layout(words0: int):
    """(bitmap offset, bitmap words, chunk-count offset) of each level inside the scratch buffer:
    a level's grid has at most a quarter of the cells of the one before in any strided geometry
    worth chaining (half the extent on two axes or more), and a level that does not fit only
    ends the look-ahead."""
    out, off = [], 0
    for level in range(_GRID_LEVELS):
        w = max(words0 >> (2 * level), 1 << 15)
        out.append((off, w, off + w))
        off += w + w // _GRID_CHUNK_WORDS
    return out, off


class _GridJob:
    """The first half of a strided-coordinate build through the occupancy bitmaps — extents,
    marks and counts of every level queued, the counters on their way to pinned host memory —
    whose second half (emit) needs the counts on the host."""
    __slots__ = ("coords", "geom", "coords_max_host", "fan", "levels", "ctr", "host", "event", "stream", "rows",
                 "early", "rows_event", "rows_wait_deferred")


def _strided_fan(ks, st) -> int:
    fan = 1
    for k, s in zip(ks, st):
        fan *= -(-k // s)
    return fan


def _grid_start(state, coords, ks, st, pd, coords_max_host, fan, ahead, early=False) -> _GridJob:
    """Queue the marking and counting passes of ``1 + ahead`` levels and the copy of their
    counters to the host; nothing waits.  Runs with _state_lock held."""
    n = coords.shape[0]
    dev = coords.device
    if state.grid_event is not None and state.grid_event_stream != _stream():
        # the scratch was last used on the other stream (work of the same stream is ordered anyway)
        torch.cuda.current_stream(dev).wait_event(state.grid_event)
    bits = min(max(1 << (n * fan * 2048 - 1).bit_length(), 1 << 20), 1 << 30)
    buf = state.bitmap(dev, bits // 32)
    layout, _ = _grid_layout(state.grid_words)
    levels = 1 + ahead
    # per level 8 counters: [n_out, table overflow, grid too large, unpackable, max b, x, y, z of the INPUTS]
    ctr = torch.zeros(8 * levels, dtype=torch.int32, device=dev)
    s = _stream()
    g = (_i3(ks), _i3(st), _i3(pd))
    host_max = _I3(*[int(v) for v in coords_max_host]) if coords_max_host is not None else None
    buf_ptr, ctr_ptr = buf.data_ptr(), ctr.data_ptr()
    part = lambda level, what: _grid_part(buf_ptr, ctr_ptr, layout, levels, level, what)  # noqa: E731
    # One output per input (kernel size == stride, no padding: a level never has more rows than
    # the one before): every level's rows are emitted at once into a buffer of n rows while
    # their count is still on the device, and the next level marks from those rows.  Nothing is
    # left to launch once the counts are on the host.  Other geometries mark the next level
    # from the previous level's bitmap and emit after the read-back; so does a single level,
    # whose emit pass is cheaper once the host knows the extents.
    rows = None
    if (levels > 1 and fan == 1 and ks == st and pd == (0, 0, 0) and coords_max_host is None
            and downsample_emit_before_readback):
        rows = torch.empty((levels, n, 4), dtype=torch.int32, device=dev)  # level i: rows[i, :n_out_i]
        state.grid_dirty = True
        # (first what the counters need; the rows follow behind the copy of the counters)
        chain_args = (s, _ptr(coords), n, *g, levels, buf_ptr, *_layout_arrays(layout), ctr_ptr, rows.data_ptr())
        _check(_C.tsmi_downsample_chain_rows(*chain_args, 1))
    else:
        _check(_C.tsmi_coords_max(s, _ptr(coords), n, part(0, "in_max"), 0))
        state.grid_dirty = True  # marked bits stay behind unless the emit passes run
        _check(_C.tsmi_downsample_grid_count(s, _ptr(coords), n, *g, host_max, part(0, "in_max"),
                                             part(0, "bitmap"), layout[0][1], 0,
                                             part(0, "chunks"), part(0, "counters"),
                                             part(1, "in_max"), None))
        for level in range(1, levels):
            _check(_C.tsmi_downsample_grid_count_next(
                s, *g, part(level - 1, "in_max"), part(level - 1, "bitmap"), layout[level - 1][1],
                part(level, "in_max"), part(level, "bitmap"), layout[level][1],
                part(level, "chunks"), part(level, "counters"), part(level + 1, "in_max")))
    job = _GridJob()
    job.early = job.rows_event = None
    job.rows_wait_deferred = False
    job.rows = rows
    job.coords, job.geom, job.coords_max_host, job.fan = coords, (ks, st, pd), coords_max_host, fan
    job.levels, job.ctr, job.stream = levels, ctr, s
    job.host = job.event = None
    if early:
        # a job started ahead of its use copies its counters to pinned memory (allocated once
        # per stream state: allocating it is slow) and marks the end of the copy with an event,
        # so the counts are usually on the host by the time they are asked for; a job whose
        # counts are needed at once reads them back directly, which is the quicker way then
        if state.host_counters is None:
            state.host_counters = torch.empty(8 * _GRID_LEVELS, dtype=torch.int32, pin_memory=True)
        job.host = state.host_counters[:8 * levels]
        job.host.copy_(ctr, non_blocking=True)
        job.event = torch.cuda.Event()
        job.event.record()
        if rows is not None:
            _check(_C.tsmi_downsample_chain_rows(*chain_args, 2))
            # (the scratch is free again behind the rows, not behind the counters)
            job.rows_event = state.grid_event = torch.cuda.Event()
            state.grid_event.record()
            state.grid_event_stream = s
        else:
            state.grid_event, state.grid_event_stream = job.event, s
        if (rows is not None and kmap_queue_before_counts and kmap_queue_ahead and kmap_through_sorted
                and state.side is not None and s == state.side.cuda_stream):
            _launch_maps_early(state, job, coords)  # (behind the counters' copy: the host gets those first)
    else:
        if rows is not None:
            _check(_C.tsmi_downsample_chain_rows(*chain_args, 2))
        if state.side is not None:  # (a state that never used its side stream needs no events)
            state.grid_event, state.grid_event_stream = torch.cuda.Event(), s
            state.grid_event.record()
    return job


_LAYOUT_ARRAYS = {}


def _layout_arrays(layout):
    """(bitmap offsets, bitmap words, chunk-count offsets) of a scratch layout as int64 arrays."""
    key = tuple(layout)
    hit = _LAYOUT_ARRAYS.get(key)
    if hit is None:
        if len(_LAYOUT_ARRAYS) >= 64:
            _LAYOUT_ARRAYS.clear()
        arr = ctypes.c_int64 * len(layout)
        hit = _LAYOUT_ARRAYS[key] = (arr(*[v[0] for v in layout]), arr(*[v[1] for v in layout]),
                                     arr(*[v[2] for v in layout]))
    return hit


def _grid_part(buf_ptr, ctr_ptr, layout, levels, level, what):
    """Address of one part of the bitmap scratch (int32 words at ``buf_ptr``) or of the counters
    (8 int32 per level at ``ctr_ptr``): plain integers, no tensor views (a view costs more
    host time than the launch it feeds)."""
    if what == "in_max":
        return ctr_ptr + 4 * (8 * level + 4) if level < levels else None
    off, w, cc = layout[level]
    if what == "bitmap":
        return buf_ptr + 4 * off
    if what == "chunks":
        return buf_ptr + 4 * cc
    return ctr_ptr + 4 * 8 * level  # "counters"


def _grid_finish(state, job: _GridJob, rsv_ratio, cap, want_table):
    """The second half: wait for the counters, emit the rows of every level.  Returns what
    downsample_coords returns for the first level (None: the grid did not fit) and leaves
    the later levels in ``state.ahead``.  Runs with _state_lock held."""
    coords = job.coords
    ks, st, pd = job.geom
    fan, levels, ctr = job.fan, job.levels, job.ctr
    n = coords.shape[0]
    dev = coords.device
    s = job.stream
    if job.rows is None:  # (what the emit launches below take; rows emitted already need none of it)
        buf = state.grid_buf
        layout, _ = _grid_layout(state.grid_words)
        g = (_i3(ks), _i3(st), _i3(pd))
        host_max = _I3(*[int(v) for v in job.coords_max_host]) if job.coords_max_host is not None else None
        buf_ptr, ctr_ptr = buf.data_ptr(), ctr.data_ptr()
        part = lambda level, what: _grid_part(buf_ptr, ctr_ptr, layout, levels, level, what)  # noqa: E731
    if job.event is not None:
        job.event.synchronize()
        host = job.host.tolist()
        # the rows were emitted behind the counters' copy: a launch or two that the caller's stream,
        # if it is another one, has to be behind as well (usually they are over by now)
        # (not where the maps queued behind the rows are about to be waited for: _queue_maps_ahead, drained)
        hit = _drained.get((dev.index, _stream())) if job.early is not None and _drained else None
        if hit is not None and hit() is coords and kmap_register_on_drained_stream and levels > 1:
            job.rows_wait_deferred = True
        elif job.rows_event is not None and s != _stream() and not job.rows_event.query():
            torch.cuda.current_stream(dev).wait_event(job.rows_event)
    else:
        host = ctr.tolist()
    if _pending_verdicts:
        settle_checks(block=False)  # (checks queued before this chain have arrived with it)
    if host[2]:
        state.grid_dirty = False  # nothing was marked, at any level
        return None
    if host[3]:  # a row or an in-range output the packed key cannot hold
        raise _range_error()  # the marks stay: grid_dirty has the next call clear them
    if host[0] > 0:  # the marking pass looked at every input row
        _mark_range_ok(coords)

    def emit(level, n_in, capacity):
        n_out = host[8 * level]
        if job.rows is not None:  # emitted before the read-back: the level is a view of its buffer
            out = job.rows.as_strided((n_out, 4), (4, 1), job.rows.storage_offset() + level * n * 4)  # (= rows[level, :n_out])
            tbl = None
            if want_table:
                _mark_range_ok(out, ascending=True)  # (known: the insert below does not read a flag back)
                tbl = GPUHashTable(capacity, device=dev)
                tbl.insert_bxyz(out)
            return out, tbl
        if n_out > capacity and fan > 2:  # more than the two outputs per input reserved
            capacity = hash_capacity(n_in * fan, rsv_ratio)
        if n_out > capacity:  # the reference's limit, with or without a table to overflow
            raise ValueError(
                "The capacity of hashtable is not sufficient. Please enlarge reserved space for "
                "hashtable:\n # Python \nimport torchsparse_amd.backends\n"
                "torchsparse_amd.backends.hash_rsv_ratio=#Value")
        tbl = GPUHashTable(capacity, device=dev) if want_table else None
        out = torch.empty((n_out, 4), dtype=torch.int32, device=dev)
        if n_out > 0:
            _check(_C.tsmi_downsample_grid_emit(
                s, *g, host_max, part(level, "in_max"),
                (ctypes.c_int32 * 4)(*host[8 * level + 4:8 * level + 8]), part(level, "bitmap"),
                layout[level][1], part(level, "chunks"), n_out,
                _ptr(tbl.keys) if tbl is not None else None, _ptr(tbl.vals) if tbl is not None else None,
                capacity, _ptr(out), _ptr(tbl.counters) if tbl is not None else part(level, "counters")))
        return out, tbl

    first = emit(0, n, cap)
    # cells of a grid whose every in-range candidate was packable, in ascending order
    _mark_range_ok(first[0], ascending=True)
    thin = fan == 1 and ks == st and pd == (0, 0, 0)  # every output stands for one block of cells
    if thin:
        _note_level(first[0], n)
    prev = first[0]
    chain_rows = [coords, prev]
    clean = True
    for level in range(1, levels):
        if prev.shape[0] == 0:
            break  # no inputs: nothing was marked from here on
        if host[8 * level + 2]:
            break  # this level's grid did not fit its bitmap: it and the later ones marked nothing
        n_in = prev.shape[0]
        try:
            nxt = emit(level, n_in, hash_capacity(n_in * min(fan, 2), rsv_ratio))
        except ValueError:  # not asked for yet: let the call that asks raise it
            clean = False  # this level's marks (and the later ones') are still in the bitmaps
            break
        state.ahead[id(prev)] = (weakref.ref(prev), (ks, st, pd, rsv_ratio), nxt[0], nxt[1])
        chain_rows.append(nxt[0])
        if thin:
            _note_level(nxt[0], n_in)
        # the later levels are not flagged on the device; their inputs' maxima are on the host
        h = 8 * level
        if (host[h + 4] < BATCH_LIMIT and host[h + 5] + 2 * pd[0] < COORD_LIMIT
                and host[h + 6] + 2 * pd[1] < COORD_LIMIT and host[h + 7] + 2 * pd[2] < COORD_LIMIT):
            _mark_range_ok(nxt[0], ascending=True)
        prev = nxt[0]
    # rows emitted before the read-back cleared every bitmap they read, asked for or not
    state.grid_dirty = (not clean) and job.rows is None
    state.level_counts = [t.shape[0] for t in chain_rows[1:]]
    if levels > 1:
        _queue_maps_ahead(state, chain_rows, job.rows is not None and state.side is not None
                          and job.stream == state.side.cuda_stream, job)
    if state.side is not None and job.rows is None:  # emit passes ran on this stream just now
        state.grid_event, state.grid_event_stream = torch.cuda.Event(), _stream()
        state.grid_event.record()
    return first


def _downsample_coords_grid(state, coords, ks, st, pd, coords_max_host, fan, rsv_ratio, cap, ahead=0,
                            want_table=True):
    """downsample_coords for non-negative coordinates when the output grid has at most
    2048 cells per candidate (and at most 2^30): mark an occupancy bitmap, count, read the
    number of outputs back, emit rows and table entries in ascending order.  None when the grid
    is larger than that (decided on the device; costs the same one read-back).  ``ahead`` more
    levels of the same geometry are computed before the read-back and left in ``state.ahead``.
    Runs with _state_lock held: one call at a time between marking a bitmap and emitting."""
    job = _grid_start(state, coords, ks, st, pd, coords_max_host, fan, ahead)
    return _grid_finish(state, job, rsv_ratio, cap, want_table)


# A network that starts with submanifold layers and then enters a chain of strided ones (a
# U-Net's stem and encoder) asks for the chain's coordinates a few convolutions after the
# first map of the same rows.  Once such a chain has been seen, the first half of its build
# (marks, counts, the copy of the counters) is queued when the submanifold map of those rows is
# built, so the counts are on the host by the time the strided layer asks and the forward no
# longer stops to wait for the queue to drain.  A look-ahead nobody asks for costs its kernels
# and a clear of the bitmaps.
downsample_lookahead_at_subm = True
# Chains in which every input has exactly one output emit each level's rows before the counts
# are read back (False: mark the next level from the bitmap, emit afterwards).
downsample_emit_before_readback = True
# Such a chain, queued at the submanifold build, runs on a second stream of the device (False:
# on the caller's stream, behind everything already queued there).
downsample_side_stream = True


def strided_lookahead(coords: torch.Tensor, behind=None) -> None:
    """Called when a submanifold map is built over ``coords``: start the strided chain that
    followed such rows last time on this stream, if any.  ``behind``: an event on the caller's
    stream that the rows are complete behind - for a caller's rows whose check is still on its
    way (no verdict yet: the chain takes rows in any order and flags those it cannot take)."""
    if not (downsample_lookahead_at_subm and downsample_through_grid and downsample_chain_ahead):
        return
    if coords.shape[0] == 0:
        return
    if behind is None and _range_origin(coords) != "user":  # (most calls: a deeper level's rows)
        return
    with _state_lock:
        state = _strided_state(coords.device)
        root = state.root_chain  # geometry of the last chain that started from rows like these
        if root is None:
            return
        if state.pending is not None:
            if state.pending.coords is coords:
                return
            # never asked for (its marks are cleared by the next bitmap() call): the network that
            # runs now is not the one the chain was learnt from; queue nothing ahead until a
            # strided call over a caller's own rows names a chain again
            state.pending = None
            state.root_chain = None
            return
        ks, st, pd, rsv_ratio = root
        ahead = min(state.chain_len.get(root, 1) - 1, _GRID_LEVELS - 1)
        fan = _strided_fan(ks, st)
        # A chain that emits its rows before the read-back needs nothing but these rows, and rows
        # of origin "user" were read back (with a synchronisation) when the library first saw
        # them: they are complete whatever the stream still has queued.  Such a chain runs on a
        # second stream, beside the tail of the previous forward, instead of behind it; the
        # caller's stream never waits for it on the device: the host waits for the counters
        # (the last thing the side stream does) before it queues anything that reads the rows.
        aside = (downsample_side_stream and ahead > 0 and fan == 1 and ks == st and pd == (0, 0, 0)
                 and downsample_emit_before_readback)
        if aside:
            main = torch.cuda.current_stream(coords.device)
            if state.side is None:
                state.side = torch.cuda.Stream(device=coords.device)
            torch.cuda.set_stream(state.side)  # (the context manager costs 6 us, two switches 0.8)
            try:
                if behind is not None:
                    state.side.wait_event(behind)
                elif kmap_root_on_second_stream:
                    _queue_root_map(coords, main)  # (first: the forward's first layer takes it)
                job = _grid_start(state, coords, ks, st, pd, None, fan, ahead, early=True)
            finally:
                torch.cuda.set_stream(main)
            if job.rows is not None:
                job.rows.record_stream(main)  # allocated on the side stream, read and freed on the caller's
        else:
            job = _grid_start(state, coords, ks, st, pd, None, fan, ahead, early=True)
        state.pending = job
        state.pending_rsv = rsv_ratio


def build_kernel_map_downsample_hashmap(in_table: Optional[GPUHashTable], coords, coords_min,
                                        coords_max_host, kernel_sizes, stride, padding,
                                        to_insert: bool = True, rsv_ratio: float = 2.0):
    """[out_in_map int32 [ceil128(N_out), K_vol], out_coords int32 [N_out,4], out_table]
    — others/sparsemapping_cuda.cu:429-507.  ``in_table`` indexes the INPUT
    coordinates (built here when None or when to_insert); the returned table
    indexes the OUTPUT coordinates and serves the next stride level."""
    ks, st, pd = _triple(kernel_sizes), _triple(stride), _triple(padding)
    out_coords, out_table = downsample_coords(coords, ks, st, pd, coords_max_host, 0, rsv_ratio)
    if in_table is None:
        in_table = GPUHashTable(hash_capacity(coords.shape[0], rsv_ratio), device=coords.device)
        to_insert = True
    if to_insert:
        in_table.insert_bxyz(coords)
    omap = in_table.query_bxyz(out_coords, ks, st, pd)
    return [omap, out_coords, out_table]


def downsample_cuda(coords, coords_max_host, coords_min, kernel_sizes, stride, padding) -> torch.Tensor:
    """Output coordinates only — others/downsample_cuda.cu:147-190."""
    return downsample_coords(coords, kernel_sizes, stride, padding, coords_max_host, 0)[0]


def convert_transposed_out_in_map(out_in_map: torch.Tensor, n_rows_t: int, n_rows: Optional[int] = None) -> torch.Tensor:
    """int32 [n_rows_t, K_vol] with map_t[in,k] = out — others/query_cuda.cu:9-15,50-54
    together with the -1 fill of nn/functional/conv/hash/query.py:47-55."""
    out_in_map = _need(out_in_map, torch.int32, "out_in_map")
    kvol = out_in_map.shape[1]
    n_rows = out_in_map.shape[0] if n_rows is None else n_rows
    hit = _map_requests.get(id(out_in_map))
    if hit is not None and hit[0]() is out_in_map:
        # a map of the chain in flight: the next forward's launch of this map writes the transposed
        # one too; this forward's did if the forward before asked
        hit[1].transposed_seen.add(hit[2])
        ready = hit[3]
        if ready is not None and ready[2] == n_rows_t:
            _map_requests[id(out_in_map)] = hit[:3] + (None,)
            hit[1].transposed_hits += 1
            t_buffer, t_first, t_pad, kvol = ready
            # (= t_buffer[t_first:t_first + t_pad * kvol].view(t_pad, kvol), in one call)
            return t_buffer.as_strided((t_pad, kvol), (kvol, 1), t_buffer.storage_offset() + t_first)
    map_t = out_in_map.new_empty(n_rows_t, kvol)
    _check(_C.tsmi_transpose_map(_stream(), _ptr(out_in_map), n_rows, kvol, _ptr(map_t), n_rows_t))
    return map_t


def derive_bitmask_from_out_in_map(out_in_map: torch.Tensor, split_mask_num: int, valid_n: int) -> torch.Tensor:
    """int32 [split, N_pad] — others/query_cuda.cu:17-31,59-65."""
    out_in_map = _need(out_in_map, torch.int32, "out_in_map")
    n_pad, kvol = out_in_map.shape
    bitmask = torch.empty((split_mask_num, n_pad), dtype=torch.int32, device=out_in_map.device)
    _check(_C.tsmi_derive_bitmask(_stream(), _ptr(out_in_map), n_pad, kvol, split_mask_num, valid_n,
                                  _ptr(bitmask)))
    return bitmask


def sort_bitmask_descending(bitmask: torch.Tensor):
    """(sorted_mask, reorder_loc int32), the role of torch.sort(bitmask, descending=True)
    at kmap/func/hashmap_on_the_fly.py:96."""
    bitmask = _need(bitmask, torch.int32, "bitmask")
    rows, n = bitmask.shape
    sorted_mask = torch.empty_like(bitmask)
    loc = torch.empty_like(bitmask)
    temp_bytes = _C.tsmi_sort_temp_bytes(n)
    temp = torch.empty(temp_bytes, dtype=torch.uint8, device=bitmask.device)
    _check(_C.tsmi_argsort_desc(_stream(), _ptr(bitmask), _ptr(sorted_mask), _ptr(loc), rows, n,
                                _ptr(temp), temp_bytes))
    return sorted_mask, loc


def reorder_out_in_map_cuda(out_in_map: torch.Tensor, reorder_loc: torch.Tensor) -> torch.Tensor:
    """others/reorder_map_cuda.cu:25-48."""
    out_in_map = _need(out_in_map, torch.int32, "out_in_map")
    reorder_loc = _need(reorder_loc, torch.int32, "reorder_loc")
    n_pad, kvol = out_in_map.shape
    out = torch.empty_like(out_in_map)
    _check(_C.tsmi_reorder_map(_stream(), _ptr(out_in_map), _ptr(reorder_loc), n_pad, kvol,
                               reorder_loc.shape[0], _ptr(out)))
    return out


def reduce_bitmask_cuda(sorted_mask: torch.Tensor, tile: int) -> torch.Tensor:
    """others/reduce_bitmask_cuda.cu:60-84."""
    sorted_mask = _need(sorted_mask, torch.int32, "bitmask")
    split, n_pad = sorted_mask.shape
    rows = (n_pad - 1) // tile + 1 if n_pad > 0 else 0
    out = torch.empty((split, rows), dtype=torch.int32, device=sorted_mask.device)
    _check(_C.tsmi_reduce_bitmask(_stream(), _ptr(sorted_mask), split, n_pad, tile, _ptr(out)))
    return out


def pair_lists(out_in_map: torch.Tensor, n_in: int, n_out: int, want_inter=True, want_planar=False,
               want_masks=True, mask_skip_k: int = -2):
    """Pair lists of a map, ordered by (offset, output row): the products of
    kmap/func/hashmap_on_the_fly.py:138-151 and :185-205 in one pass.
    Returns dict(nbmaps_inter, nbmaps_planar, nbsizes, input_mask, output_mask, nnz).
    One host read-back (nnz).  ``mask_skip_k``: the offset the masks leave out (the identity
    offset of an odd submanifold map), -1 for none, -2 for the reference's rule (the centre
    offset whenever the volume is odd and n_in == n_out)."""
    out_in_map = _need(out_in_map, torch.int32, "out_in_map")
    dev = out_in_map.device
    kvol = out_in_map.shape[1]
    nblk = max((n_out + 255) // 256, 1)
    block_counts = torch.empty(kvol * nblk, dtype=torch.int32, device=dev)
    nbsizes = torch.empty(kvol, dtype=torch.int32, device=dev)
    _check(_C.tsmi_pair_lists_count(_stream(), _ptr(out_in_map), n_out, kvol, _ptr(block_counts),
                                    _ptr(nbsizes)))
    nnz = int(nbsizes.sum().item())
    inter = torch.empty((nnz, 2), dtype=torch.int32, device=dev) if want_inter else None
    planar = torch.empty((2, nnz), dtype=torch.int32, device=dev) if want_planar else None
    imask = torch.empty(kvol * n_in, dtype=torch.int32, device=dev) if want_masks else None
    omask = torch.empty(kvol * n_out, dtype=torch.int32, device=dev) if want_masks else None
    _check(_C.tsmi_pair_lists_fill(_stream(), _ptr(out_in_map), n_out, kvol, _ptr(block_counts),
                                   _ptr(nbsizes), nnz, _ptr(inter), _ptr(planar), n_in, n_out,
                                   int(mask_skip_k), _ptr(imask), _ptr(omask)))
    return dict(nbmaps_inter=inter, nbmaps_planar=planar, nbsizes=nbsizes, input_mask=imask,
                output_mask=omask, nnz=nnz)


def build_mask_from_kmap(n_in: int, n_out: int, nbmaps: torch.Tensor, nbsizes: torch.Tensor):
    """[input_mask, output_mask] from interleaved pair lists —
    others/sparsemapping_cuda.cu:510-548.  (pair_lists() produces the masks in the
    same pass as the pairs; this entry serves callers that already hold pairs.)"""
    nbmaps = _need(nbmaps, torch.int32, "nbmaps")
    nbsizes = _need(nbsizes, torch.int32, "nbsizes")
    kvol = nbsizes.numel()
    dev = nbmaps.device
    nbaddrs = torch.empty(kvol + 1, dtype=torch.int32, device=dev)
    qnbaddrs = torch.empty(kvol + 1, dtype=torch.int32, device=dev)
    exclusive_scan_quantified_wrapper(kvol, nbsizes, nbaddrs, qnbaddrs)
    imask = torch.empty(kvol * n_in, dtype=torch.int32, device=dev)
    omask = torch.empty(kvol * n_out, dtype=torch.int32, device=dev)
    _check(_C.tsmi_build_masks(_stream(), _ptr(nbmaps), nbmaps.shape[0], _ptr(nbaddrs), kvol, n_in,
                               n_out, _ptr(imask), _ptr(omask)))
    return [imask, omask]


def exclusive_scan_quantified_wrapper(kvol: int, nbsizes: torch.Tensor, nbaddrs: torch.Tensor,
                                      qnbaddrs: torch.Tensor, q: int = 128) -> None:
    """others/exclusive_scan_cuda.cu:31-45 (writes nbaddrs / qnbaddrs in place)."""
    nbsizes = _need(nbsizes, torch.int32, "nbsizes")
    _check(_C.tsmi_exclusive_scan_quantified(_stream(), kvol, _ptr(nbsizes), q, _ptr(nbaddrs),
                                             _ptr(qnbaddrs)))


# -------------------------------------------------------------------- convolutions


def _dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported feature dtype {t.dtype}") from None


def pack_weights(kernel: torch.Tensor) -> torch.Tensor:
    """[K_vol, Cin, Cout] -> the MFMA-friendly [K_vol, Cout_pad, Cin_pad] layout.
    Cached on the tensor object and refreshed when its version counter moves."""
    cached = getattr(kernel, "_tsmi_packed", None)
    if cached is not None and cached[0] == kernel._version and cached[1] == kernel.data_ptr():
        if _pin_sinks:
            _pin(cached[2])
        return cached[2]
    w = kernel.detach()
    if w.dim() == 2:
        w = w.unsqueeze(0)
    w = w.contiguous()
    kvol, cin, cout = w.shape
    packed = torch.empty(_C.tsmi_packed_weight_elems(kvol, cin, cout), dtype=w.dtype, device=w.device)
    _check(_C.tsmi_pack_weights(_stream(), _ptr(w), _ptr(packed), kvol, cin, cout, _dtype_code(w)))
    try:
        kernel._tsmi_packed = (kernel._version, kernel.data_ptr(), packed)
    except AttributeError:
        pass
    if _pin_sinks:
        _pin(packed)
    return packed


def _conv_common(in_feats: torch.Tensor, kernel: torch.Tensor):
    if not in_feats.is_cuda:
        raise RuntimeError("sparse convolution needs GPU tensors; there is no CPU path")
    if in_feats.dtype != kernel.dtype:
        raise ValueError(f"feature dtype {in_feats.dtype} and kernel dtype {kernel.dtype} differ")
    kshape = kernel.shape if kernel.dim() == 3 else (1,) + tuple(kernel.shape)
    if in_feats.shape[1] != kshape[1]:
        raise ValueError("Input feature size and kernel size mismatch")
    x = in_feats if in_feats.is_contiguous() else in_feats.contiguous()
    return x, pack_weights(kernel), kshape


def _epilogue_args(bias, residual, x, n_out, cout):
    pb = pr = None
    if bias is not None:
        if bias.dtype != x.dtype or bias.dim() != 1 or bias.shape[0] != cout or not bias.is_contiguous():
            raise ValueError(f"bias must be a contiguous {x.dtype} tensor of shape {(cout,)}")
        pb = bias.data_ptr()
    if residual is not None:
        if (residual.dtype != x.dtype or residual.dim() != 2 or residual.shape[0] != n_out
                or residual.shape[1] != cout or not residual.is_contiguous()):
            raise ValueError(f"residual must be a contiguous {x.dtype} tensor of shape {(n_out, cout)}")
        pr = residual.data_ptr()
    return pb, pr


# ---- a launch thread for the convolution calls of a forward --------------------------------
#
# Inside ``with launch_region():`` the convolution calls of this module hand their packed
# argument block to the library's launch thread (tsmi_launch_thread_submit) instead of launching
# themselves: the ~5 us a call spends inside the library (checks, plan, hipLaunchKernel) run beside
# the ~5 us Python spends on the next call.  The launch thread keeps the order of the calls; what
# this thread queues itself - other library calls, torch's kernels, event records - is ordered
# against them only by flush_launches(), which every function here that consumes a convolution's
# result or reuses its operands calls first (and which the region calls when it ends).  The
# tensors of a handed-over call are kept referenced until the launch thread has carried it out.
# The networks in ``backbones`` open a region around their inference forward when
# ``launch_thread = True``.
launch_thread = True
_region_depth = 0
_region_calls = collections.deque()  # (ticket, tensors the call reads and writes)
_completed = None                    # the launch thread's counter of calls carried out (a ctypes int64)


class launch_region:
    """Context: convolution calls inside are carried out by the library's launch thread (see
    above).  A no-op where ``launch_thread`` is False, while a graph is being recorded, and on
    CPU-only builds."""
    __slots__ = ("opened",)

    def __enter__(self):
        global _region_depth, _completed
        self.opened = False
        if launch_thread and torch.cuda.is_available() and not torch.cuda.is_current_stream_capturing():
            if _completed is None:
                _completed = _C.tsmi_launch_thread_completed().contents
            _check(_C.tsmi_launch_thread_open())
            _region_depth += 1
            self.opened = True
        return self

    def __exit__(self, *exc):
        global _region_depth
        if self.opened:
            _region_depth -= 1
            status = _C.tsmi_launch_thread_close()  # (waits for every call handed over)
            _region_calls.clear()
            if exc[0] is None:
                _check(status)
        return False


class direct_launches:
    """Context inside a launch_region in which convolution calls launch themselves again (after
    waiting for those handed over): for code that looks at results as soon as a layer returns -
    forward hooks, debugging."""
    __slots__ = ("depth",)

    def __enter__(self):
        global _region_depth
        flush_launches()
        self.depth, _region_depth = _region_depth, 0
        return self

    def __exit__(self, *exc):
        global _region_depth
        _region_depth = self.depth
        return False


def flush_launches() -> None:
    """Returns once every convolution call handed to the launch thread has been launched; raises
    the error of the first that failed.  Cheap when no region is open or nothing is pending."""
    if _region_depth and _region_calls:
        status = _C.tsmi_launch_thread_flush()
        _region_calls.clear()
        _check(status)


def _hand_over(kind: int, block: bytes, words: int, keep) -> bool:
    """Hands a packed convolution call to the launch thread; False: no region, make the call."""
    ticket = _C.tsmi_launch_thread_submit(kind, block, words)
    if ticket < 0:
        return False
    calls = _region_calls
    done = _completed.value
    while calls and calls[0][0] <= done:
        calls.popleft()
    calls.append((ticket, keep))
    return True


_PACK20 = struct.Struct("20q").pack
_PACK21 = struct.Struct("21q").pack


class ColumnSlice:
    """Columns [first, first + cols) of a contiguous 2-D ``buffer``, for ``out=`` / ``also=`` of a
    convolution: the same as the view ``buffer[:, first:first + cols]`` without making one (a
    view costs 2 us, a forward of a U-Net places eight results).  A call placed through
    ``out=ColumnSlice(...)`` returns the whole buffer as its result tensor."""
    __slots__ = ("buffer", "ptr", "pitch", "rows", "cols")

    def __init__(self, buffer: torch.Tensor, first: int, cols: int):
        if buffer.dim() != 2 or not buffer.is_contiguous() or first < 0 or cols < 1 or first + cols > buffer.shape[1]:
            raise ValueError("a column slice needs a contiguous 2-D buffer that holds its columns")
        self.buffer, self.rows, self.cols, self.pitch = buffer, buffer.shape[0], cols, buffer.shape[1]
        self.ptr = buffer.data_ptr() + first * buffer.element_size()
        if self.pitch % 8 or self.ptr % 16:
            raise ValueError("a placed result needs rows a multiple of 8 elements apart and 16-byte aligned")


def _placed(x, num_out_feats: int, cout: int, out, also):
    """(result tensor, address of y, row pitch of y or 0, address of the second destination or 0,
    its row pitch) of a
    convolution whose result goes into ``out`` (None: a new dense tensor) and, a second time, into
    ``also``: [num_out_feats, cout] views of the features' dtype with unit column stride, rows a
    multiple of 8 elements apart and 16-byte aligned (column slices of wider buffers)."""
    ldy = a2 = ld2 = 0
    for t in (out, also):
        if t is None:
            continue
        if t.__class__ is ColumnSlice:
            if t.rows != num_out_feats or t.cols != cout or t.buffer.dtype != x.dtype or t.buffer.device != x.device:
                raise ValueError(f"a placed result needs {x.dtype} columns for [{num_out_feats}, {cout}] values")
            continue
        if (t.dtype != x.dtype or t.dim() != 2 or t.shape[0] != num_out_feats or t.shape[1] != cout
                or t.stride(1) != 1 or t.stride(0) % 8 or t.stride(0) < cout or t.data_ptr() % 16
                or t.device != x.device):
            raise ValueError(f"a placed result needs a {x.dtype} [{num_out_feats}, {cout}] view with unit column "
                             "stride, rows a multiple of 8 elements apart and 16-byte aligned")
    if out is None:
        y = x.new_empty(num_out_feats, cout)
        at = y.data_ptr()
    elif out.__class__ is ColumnSlice:
        y, at, ldy = out.buffer, out.ptr, out.pitch
    else:
        y, at, ldy = out, out.data_ptr(), out.stride(0)
    if also is not None:
        a2, ld2 = (also.ptr, also.pitch) if also.__class__ is ColumnSlice else (also.data_ptr(), also.stride(0))
    return y, at, ldy, a2, ld2

# Buffers the library owns (the scratch of a stream, its tile counters, identity maps, pair
# segments, grouped maps, packed weights) live in tables that drop or replace their entries.  A
# caller that keeps their ADDRESSES beyond the call - a recorded HIP graph - collects the tensors
# themselves while it records: every accessor below hands each buffer it returns to the open
# collectors, and a tensor that is referenced is not freed whatever the tables do.
_pin_sinks = []


class pinned:
    """``with pinned() as held:`` - ``held`` (a list) receives every library-owned tensor whose
    address is handed to a launch inside the block, once per tensor."""

    def __enter__(self):
        self.held, self._seen = [], set()
        _pin_sinks.append(self)
        return self.held

    def __exit__(self, *exc):
        _pin_sinks.remove(self)
        return False

    def add(self, t):
        if id(t) not in self._seen:
            self._seen.add(id(t))
            self.held.append(t)


def _pin(t):
    for sink in _pin_sinks:
        sink.add(t)
    return t


_SCRATCH = {}  # (device index, stream) -> uint8 tensor, grown on demand
# held while a call that goes through the scratch buffer queues its launches: two host threads
# that feed one stream must not interleave the launches of two such calls
_scratch_lock = threading.Lock()


def _scratch(device, stream: int, nbytes: int) -> int:
    """Address of at least ``nbytes`` of device memory that the convolutions queued on one stream
    share for their intermediate results (partial sums, per-pair products): every such launch
    pair writes before it reads, and the stream runs them one after the other, so the buffer
    needs no allocation per call.  It only grows; a replaced buffer goes back to torch's
    stream-ordered allocator like any temporary."""
    key = (device.index, stream)
    t = _SCRATCH.get(key)
    if t is None or t.numel() < nbytes:
        with _tables_lock:  # (two host threads that miss together must end with one buffer)
            t = _SCRATCH.get(key)
            if t is None or t.numel() < nbytes:
                t = _SCRATCH[key] = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
    if _pin_sinks:
        _pin(t)
    return t.data_ptr()


@functools.lru_cache(maxsize=4096)
def _workspace_elems(n_out: int, kvol: int, cin: int, cout: int, code: int) -> int:
    return _C.tsmi_conv_workspace_elems(n_out, n_out, kvol, 1, cin, cout, code, 0)


@functools.lru_cache(maxsize=4096)
def _segments_supported(kvol: int, cin: int, cout: int, code: int) -> bool:
    return bool(_C.tsmi_conv_segments_supported(kvol, cin, cout, code))


_TILE_COUNTERS = {}
_N_TILE_COUNTERS = 4096


def _tile_counters(device, stream: int):
    """Zero-filled int32 array shared by the split convolutions of one stream (each
    launch leaves it zero again)."""
    key = (device.index, stream)
    t = _TILE_COUNTERS.get(key)
    if t is None:
        with _tables_lock:
            t = _TILE_COUNTERS.get(key)
            if t is None:
                t = _TILE_COUNTERS[key] = torch.zeros(_N_TILE_COUNTERS, dtype=torch.int32, device=device)
    if _pin_sinks:
        _pin(t)
    return t


def conv_forward_implicit_gemm_cuda(in_feats, kernel, out_in_map, num_out_feats, num_out_channels,
                                    allow_tf32=False, allow_fp16=True, bias=None, residual=None,
                                    relu=False, segments=None) -> torch.Tensor:
    """convolution/convolution_forward_implicit_gemm_cuda.cu:1527-1986.  allow_tf32 /
    allow_fp16 are accepted and ignored: fp32 runs in true fp32, 16-bit types
    accumulate in fp32."""
    x, wp, (kvol, cin, cout) = _conv_common(in_feats, kernel)
    if cout != num_out_channels:
        raise ValueError("num_out_channels does not match the kernel")
    return _implicit_gemm(x, wp, kvol, cin, cout, out_in_map, num_out_feats, bias, residual, relu, segments)


# Small, wide layers of the implicit-GEMM dataflow run over pair segments (a per-offset
# compaction of the map, built once per map and kept with it) instead of the dense pass over
# all offsets of every row tile, where the map is known to have few pairs per row (True), wherever
# the kernels have a variant ("always"), or never (False).
igemm_through_segments = True
# The pair form costs about 0.2 + 2.3 d of the dense pass on the layers it is made for (d: pairs
# per map entry; fitted to 0.74 at d = 0.24 and 1.58 at d = 0.61, the two workloads measured in
# _segments_pay's note): it is the cheaper one below d = 0.35.  Used where the density of the map
# is known (map_density); other maps go by the hint of the level's thinning.
segments_max_density = 0.35

_segments_of = {}  # id(map) -> (weak reference, version, address, stream, rows, segments)
_SEGMENT_POOLS = {}  # (device index, stream) -> zero int32 tensor the builder's blocks add up in


class PairSegments:
    """Per-offset pair lists of a kernel map (tsmi_pair_segments), in one int32 allocation:
    ``counts`` [K_vol], ``in_rows`` [K_vol, seg_rows], ``pos`` [K_vol, n_rows] (views, made when
    asked for; the convolution works from the addresses)."""
    __slots__ = ("buffer", "first", "kvol", "n_rows", "seg_rows", "counts_ptr", "in_rows_ptr", "pos_ptr")

    @staticmethod
    def elems(kvol: int, n_rows: int, seg_rows: int) -> int:
        """int32 elements of one set of lists, rounded so that the next set in the same allocation
        starts 256-byte aligned as well."""
        return make_divisible(make_divisible(kvol, 64) + kvol * seg_rows + kvol * n_rows, 64)

    def __init__(self, kvol: int, n_rows: int, seg_rows: int, device, buffer=None, first: int = 0):
        """``buffer`` / ``first``: an int32 allocation shared with other sets and the element
        this one starts at (a multiple of 64); None: an allocation of its own."""
        self.kvol, self.n_rows, self.seg_rows, self.first = kvol, n_rows, seg_rows, first
        head = make_divisible(kvol, 64)  # keeps the two lists 256-byte aligned
        if buffer is None:
            buffer = torch.empty(head + kvol * seg_rows + kvol * n_rows, dtype=torch.int32, device=device)
        self.buffer = buffer
        self.counts_ptr = buffer.data_ptr() + 4 * first
        self.in_rows_ptr = self.counts_ptr + 4 * head
        self.pos_ptr = self.in_rows_ptr + 4 * kvol * seg_rows

    @property
    def counts(self) -> torch.Tensor:
        return self.buffer[self.first:self.first + self.kvol]

    @property
    def in_rows(self) -> torch.Tensor:
        head = self.first + make_divisible(self.kvol, 64)
        return self.buffer[head:head + self.kvol * self.seg_rows].view(self.kvol, self.seg_rows)

    @property
    def pos(self) -> torch.Tensor:
        start = self.first + make_divisible(self.kvol, 64) + self.kvol * self.seg_rows
        return self.buffer[start:start + self.kvol * self.n_rows].view(self.kvol, self.n_rows)

    def __iter__(self):  # (counts, in_rows, pos, seg_rows)
        return iter((self.counts, self.in_rows, self.pos, self.seg_rows))


def _build_pair_segments(out_in_map: torch.Tensor, n_rows: int, kvol: int, dev) -> PairSegments:
    """One launch on the current stream (operands checked by the caller)."""
    stream = _stream()
    seg = PairSegments(kvol, n_rows, make_divisible(max(n_rows, 1), 128), dev)
    key = (dev.index, stream)
    pool = _SEGMENT_POOLS.get(key)
    if pool is None:
        with _tables_lock:
            pool = _SEGMENT_POOLS.get(key)
            if pool is None:
                pool = _SEGMENT_POOLS[key] = torch.zeros(520, dtype=torch.int32, device=dev)
    if _pin_sinks:
        _pin(pool)
        _pin(seg.buffer)
    with _scratch_lock:  # (the pool is shared by the builds of one stream)
        _check(_C.tsmi_pair_segments(stream, out_in_map.data_ptr(), n_rows, kvol, seg.seg_rows,
                                     pool.data_ptr() if kvol < 520 else None, seg.counts_ptr,
                                     seg.in_rows_ptr, seg.pos_ptr))
    return seg


def _build_pair_segments_batch(jobs, dev):
    """The segments of several maps (``jobs``: (map, rows, kernel volume)) in one allocation,
    queued by one call on the current stream."""
    stream = _stream()
    sizes = [PairSegments.elems(kvol, n_rows, make_divisible(max(n_rows, 1), 128)) for _, n_rows, kvol in jobs]
    buffer = torch.empty(sum(sizes), dtype=torch.int32, device=dev)
    key = (dev.index, stream)
    pool = _SEGMENT_POOLS.get(key)
    if pool is None:
        with _tables_lock:
            pool = _SEGMENT_POOLS.get(key)
            if pool is None:
                pool = _SEGMENT_POOLS[key] = torch.zeros(520, dtype=torch.int32, device=dev)
    if _pin_sinks:
        _pin(pool)
        _pin(buffer)
    pool_ptr = pool.data_ptr()
    segs, flat, first = [], [], 0
    for (omap, n_rows, kvol), size in zip(jobs, sizes):
        seg = PairSegments(kvol, n_rows, make_divisible(max(n_rows, 1), 128), dev, buffer, first)
        first += size
        flat += (omap.data_ptr(), n_rows, kvol, seg.seg_rows, pool_ptr if kvol < 520 else 0, seg.counts_ptr,
                 seg.in_rows_ptr, seg.pos_ptr)
        segs.append(seg)
    with _scratch_lock:  # (the pool is shared by the builds of one stream)
        _check(_C.tsmi_pair_segments_batch(stream, len(jobs), (ctypes.c_int64 * len(flat))(*flat)))
    return segs


def pair_segments(out_in_map: torch.Tensor, n_rows: int) -> PairSegments:
    """The pair segments of a kernel map's first ``n_rows`` rows: per kernel offset the input
    rows of its pairs, compacted (``in_rows``), their number (``counts``) and for every (offset,
    row) the place of the pair in that list (``pos``, -1: none).  Built in one launch, once per
    map tensor and stream."""
    stream = _stream()
    request = _map_requests.get(id(out_in_map))
    if request is not None and request[0]() is out_in_map:
        # a map of the chain in flight: its segments are built ahead in the next forward (asked for
        # here whether they were built ahead this time or not: segments no layer takes drop out)
        request[1].segments_seen.add(request[2])
    hit = _segments_of.get(id(out_in_map))
    if (hit is not None and hit[0]() is out_in_map and hit[1] == out_in_map._version
            and hit[2] == out_in_map.data_ptr() and hit[3] == stream and hit[4] == n_rows):
        if _pin_sinks:
            _pin(hit[5].buffer)
        return hit[5]
    out_in_map = _need(out_in_map, torch.int32, "out_in_map")
    kvol = out_in_map.shape[1]
    if n_rows > out_in_map.shape[0]:
        raise ValueError(f"the map has {out_in_map.shape[0]} rows, fewer than the {n_rows} asked for")
    seg = _build_pair_segments(out_in_map, n_rows, kvol, out_in_map.device)
    if torch.cuda.is_current_stream_capturing():
        return seg  # filled by the recording's replays only: not for the table
    _remember(_segments_of, id(out_in_map), (weakref.ref(out_in_map), out_in_map._version, out_in_map.data_ptr(),
                                             stream, n_rows, seg), 64)
    return seg


_level_thinning = {}  # id(coords) -> (weak reference, rows kept per input row by the layer that made them)
_sparse_maps = {}     # id(map) -> weak reference: maps over rows known to have few neighbours
_hint_lock = threading.Lock()  # guards the two tables above


# Large 3x3x3 layers of the implicit-GEMM dataflow can run over a copy of the map whose rows are
# grouped, inside windows of consecutive rows, by the planes of the kernel they use
# (tsmi_map_group_rows): a row tile then multiplies about half as many kernel offsets as a tile
# of rows in coordinate order (a surface scan: 25 of 27 offsets per 128-row tile in coordinate
# order, 14 grouped), and the tiles run heaviest first.  Building the copy takes four launches
# (about 20 us of kernels and 12 us of host time for a 90k-row map) and a layer gains 2 - 7 us
# from it (96 -> 96 channels at 90k rows: 49 -> 42 us), so it pays from about the tenth layer
# that runs over the same map tensor on: maps kept over several forwards (cached kernel maps, a
# model applied again to the same SparseTensor), not the five to eight layers that share a map
# inside one forward.  True: a map's copy is built at its group_after_uses-th eligible use and
# used from then on; "always": at the first; False: never.
igemm_group_rows = True
group_window = 8192      # rows per window (a multiple of 128, at most 8192)
group_min_rows = 32768   # smaller maps have too few tiles for the order to matter
group_after_uses = 10
_group_uses = {}  # id(map) -> [weak reference, version, address, eligible uses so far]

_grouped_of = {}  # id(map) -> (weak reference, version, address, stream, rows, window, GroupedMap)


class GroupedMap:
    """What tsmi_map_group_rows leaves, in one int32 allocation: ``grouped`` [P, 27], ``row_of`` [P],
    ``masks64`` [P / 64], ``order64`` [8 ceil(P / 512)], ``order128`` [8 ceil(P / 1024)] (views, made when asked for;
    the convolution works from the addresses)."""
    __slots__ = ("buffer", "padded", "window", "ptrs")

    def __init__(self, padded: int, window: int, device):
        self.padded, self.window = padded, window
        sizes = self._sizes()
        self.buffer = torch.empty(sum(sizes), dtype=torch.int32, device=device)
        base, self.ptrs, off = self.buffer.data_ptr(), [], 0
        for n in sizes:
            self.ptrs.append(base + 4 * off)
            off += n

    def _sizes(self):
        p = self.padded
        return (p * 27, p, p // 64, 8 * -(-(p // 64) // 8), 8 * -(-(p // 128) // 8))

    def _part(self, i):
        sizes = self._sizes()
        start = sum(sizes[:i])
        return self.buffer[start:start + sizes[i]]

    grouped = property(lambda self: self._part(0).view(self.padded, 27))
    row_of = property(lambda self: self._part(1))
    masks64 = property(lambda self: self._part(2))
    order64 = property(lambda self: self._part(3))
    order128 = property(lambda self: self._part(4))


def grouped_map(out_in_map: torch.Tensor, n_rows: int, window: Optional[int] = None) -> GroupedMap:
    """The grouped copy of a 3x3x3 kernel map's first ``n_rows`` rows: grouped[p] =
    out_in_map[row_of[p]], positions sorted inside windows of ``window`` rows by the kernel
    planes a row uses, padding positions (-1) last; and its row tiles listed heaviest first.
    Four launches, once per map tensor and stream."""
    window = group_window if window is None else int(window)
    stream = _stream()
    hit = _grouped_of.get(id(out_in_map))
    if (hit is not None and hit[0]() is out_in_map and hit[1] == out_in_map._version
            and hit[2] == out_in_map.data_ptr() and hit[3] == stream and hit[4] == n_rows and hit[5] == window):
        if _pin_sinks:
            _pin(hit[6].buffer)
        return hit[6]
    out_in_map = _need(out_in_map, torch.int32, "out_in_map")
    if out_in_map.dim() != 2 or out_in_map.shape[1] != 27:
        raise ValueError("rows are grouped for 3x3x3 maps only (27 kernel offsets)")
    if n_rows > out_in_map.shape[0]:
        raise ValueError(f"the map has {out_in_map.shape[0]} rows, fewer than the {n_rows} asked for")
    padded = _C.tsmi_map_group_rows_padded(n_rows, window)
    if padded < 0:
        raise ValueError(f"bad window of {window} rows: a multiple of 128 between 128 and 8192")
    if n_rows == 0:
        raise ValueError("no rows to group")
    g = GroupedMap(padded, window, out_in_map.device)
    if _pin_sinks:
        _pin(g.buffer)
    _check(_C.tsmi_map_group_rows(stream, out_in_map.data_ptr(), n_rows, 27, window, *g.ptrs))
    if torch.cuda.is_current_stream_capturing():
        return g  # filled by the recording's replays only: not for the table
    _remember(_grouped_of, id(out_in_map), (weakref.ref(out_in_map), out_in_map._version, out_in_map.data_ptr(),
                                            stream, n_rows, window, g), 64)
    return g


def _grouping_fits(x, kvol: int, cin: int, cout: int, num_out_feats: int) -> bool:
    """Layers that can run over the grouped map: 3x3x3, enough rows for several hundred tiles,
    features in whole 16-byte pieces, and a channel count the one-column-tile kernels cover
    (wider layers of fewer than 65536 rows run the tiled kernel, which keeps its order)."""
    return bool(igemm_group_rows and kvol == 27 and num_out_feats >= group_min_rows
                and cin > 8 and (cin * x.element_size()) % 16 == 0
                and (cout < 128 or num_out_feats >= 65536))


def _grouping_pays(x, kvol: int, cin: int, cout: int, num_out_feats: int, out_in_map=None) -> bool:
    """Whether this call runs over the grouped copy of ``out_in_map``: an eligible layer, and a
    map that has been used often enough for the copy to pay (or has its copy already)."""
    if not _grouping_fits(x, kvol, cin, cout, num_out_feats):
        return False
    if igemm_group_rows == "always" or out_in_map is None:
        return True
    key = id(out_in_map)
    if key in _grouped_of and _grouped_of[key][0]() is out_in_map:
        return True
    hit = _group_uses.get(key)
    if (hit is None or hit[0]() is not out_in_map or hit[1] != out_in_map._version
            or hit[2] != out_in_map.data_ptr()):
        hit = [weakref.ref(out_in_map), out_in_map._version, out_in_map.data_ptr(), 0]
        _remember(_group_uses, key, hit, 256)
    hit[3] += 1
    # (a copy built while a graph is being recorded would hold nothing until the first replay)
    return hit[3] >= group_after_uses and not torch.cuda.is_current_stream_capturing()


def conv_implicit_gemm_grouped(x, wp, kvol, cin, cout, out_in_map, num_out_feats, bias=None,
                               residual=None, relu=False, out=None, also=None) -> torch.Tensor:
    """The implicit-GEMM sums over the grouped copy of the map (same results bit for bit)."""
    g = grouped_map(out_in_map, num_out_feats)
    if out is None and also is None:
        y = x.new_empty(num_out_feats, cout)
        at, ldy, a2, ld2 = y.data_ptr(), 0, 0, 0
    else:
        y, at, ldy, a2, ld2 = _placed(x, num_out_feats, cout, out, also)
    pb, pr = _epilogue_args(bias, residual, x, num_out_feats, cout)
    ptrs = g.ptrs
    block = _PACK20(_stream(), x.data_ptr(), wp.data_ptr(), ptrs[0], ptrs[1], ptrs[3], ptrs[4], g.padded,
                    num_out_feats, kvol, cin, cout, _dtype_code(x), pb or 0, pr or 0, int(relu), at, ldy, a2, ld2)
    if not (_region_depth and _hand_over(2, block, 20, (x, wp, g, bias, residual, y, also))):
        _check(_C.tsmi_conv_implicit_gemm_grouped_packed(block))
    return y


def _note_level(out_coords: torch.Tensor, n_in: int) -> None:
    """``out_coords`` came out of a kernel size = stride, pad 0 layer over ``n_in`` rows."""
    with _hint_lock:
        if len(_level_thinning) >= 256:
            for key in [k for k, v in _level_thinning.items() if v[0]() is None]:
                del _level_thinning[key]
            if len(_level_thinning) >= 256:
                _level_thinning.clear()
        _level_thinning[id(out_coords)] = (weakref.ref(out_coords), out_coords.shape[0] / max(n_in, 1))


def level_thinning(coords: torch.Tensor) -> Optional[float]:
    """N_out / N_in of the kernel size = stride, pad 0 strided layer that produced ``coords``
    (None: not such rows).  Each output of such a layer stands for a block of prod(stride) cells,
    so N_out / N_in = 1 / (occupied cells per occupied block): 1/8 for solid volumes under 2^3
    blocks, 0.4 - 0.5 for surfaces (a LiDAR scan's levels: 0.50, 0.44, 0.41, 0.39)."""
    hit = _level_thinning.get(id(coords))
    return hit[1] if hit is not None and hit[0]() is coords else None


def hint_sparse_map(out_in_map: torch.Tensor) -> None:
    """Mark a kernel map as one over thin rows (few neighbours per row): the implicit-GEMM
    dataflow then runs its small, wide layers over pair segments."""
    with _hint_lock:
        if len(_sparse_maps) >= 256:
            for key in [k for k, v in _sparse_maps.items() if v() is None]:
                del _sparse_maps[key]
            if len(_sparse_maps) >= 256:
                _sparse_maps.clear()
        _sparse_maps[id(out_in_map)] = weakref.ref(out_in_map)


def _segments_pay(x, kvol, cin, cout, num_out_feats, out_in_map=None, force=None) -> bool:
    """Whether a layer runs over pair segments: 16-bit features, a 3^3 or larger kernel, few rows
    and many channels (the regime in which the dense pass is bound by the weight slabs it streams
    per row tile) and a map with few pairs per row.  The cost of the pair form grows with the
    number of pairs (every product row crosses memory twice), the dense pass keeps its sums in
    registers: measured on the levels of an 89,834-voxel scan (24 % of the map entries are pairs):
    8,045 rows 256 -> 256 32 vs 43 us, 384 -> 256 39 vs 57, 19,815 rows 128 -> 128 30 vs 36,
    192 -> 128 33 vs 47, 3,105 rows 256 -> 256 22 vs 28 (8,045 rows 128 -> 128, 21 vs 20, stays
    dense); on a detection backbone's 55,578-row level (61 %): 128 -> 128 134 vs 85.  With
    ``igemm_through_segments = True`` the pair form is taken where the map's measured density
    (map_density: maps built ahead of their use count their pairs) is at most
    ``segments_max_density``; a map without a count goes by hint_sparse_map (build_kernel_map marks
    the maps over rows that thin out like surfaces, see level_thinning); "always" takes the pair
    form wherever a variant exists.  ``force`` (a
    layer's conv_config "pair_segments": True / False) overrides the module-wide setting; the
    row and channel limits hold either way."""
    mode = igemm_through_segments
    if force is not None:  # a layer's own configuration (conv_config "pair_segments") decides
        mode = "always" if force else False
    if not mode or not (kvol >= 27 and 0 < num_out_feats < 65536 and cout >= 128
                        and (cin * cout > 128 * 128 or num_out_feats >= 12000)
                        and _segments_supported(kvol, cin, cout, _dtype_code(x))):
        return False
    if mode == "always":
        return True
    if out_in_map is None:
        return False
    density = map_density(out_in_map)  # measured, where the map's build counted its pairs
    if density is not None:
        return density <= segments_max_density
    hit = _sparse_maps.get(id(out_in_map))
    return hit is not None and hit() is out_in_map


def conv_implicit_gemm_segments(x, wp, kvol, cin, cout, out_in_map, num_out_feats, bias=None,
                                residual=None, relu=False, out=None, also=None) -> torch.Tensor:
    """The implicit-GEMM sums over pair segments: one launch multiplies every pair's input row
    by its offset's weights (a workgroup reads one offset's weights only), a second adds each
    output row's products."""
    seg = pair_segments(out_in_map, num_out_feats)
    seg_rows = seg.seg_rows
    if out is None and also is None:
        y = x.new_empty(num_out_feats, cout)  # (the cheapest form of the call: 1.2 us against 1.6)
        at, ldy, a2, ld2 = y.data_ptr(), 0, 0, 0
    else:
        y, at, ldy, a2, ld2 = _placed(x, num_out_feats, cout, out, also)
    stream = _stream()
    pb, pr = _epilogue_args(bias, residual, x, num_out_feats, cout)
    with _scratch_lock:
        products = _scratch(x.device, stream, kvol * seg_rows * cout * x.element_size())
        block = _PACK20(stream, x.data_ptr(), wp.data_ptr(), seg.in_rows_ptr, seg.counts_ptr, seg.pos_ptr, seg_rows,
                        num_out_feats, kvol, cin, cout, _dtype_code(x), pb or 0, pr or 0, int(relu), products,
                        at, ldy, a2, ld2)
        if not (_region_depth and _hand_over(1, block, 20, (x, wp, seg, bias, residual, y, also,
                                                            _SCRATCH.get((x.device.index, stream))))):
            _check(_C.tsmi_conv_implicit_gemm_segments_packed(block))
    return y


def _implicit_gemm(x, wp, kvol, cin, cout, out_in_map, num_out_feats, bias=None, residual=None,
                   relu=False, segments=None, out=None, also=None) -> torch.Tensor:
    """``out`` / ``also``: the result goes into ``out`` instead of a new tensor, and a second time
    into ``also`` (see _placed: column slices of wider buffers, which spares the copy of a later
    concatenation)."""
    if _segments_pay(x, kvol, cin, cout, num_out_feats, out_in_map, segments):
        return conv_implicit_gemm_segments(x, wp, kvol, cin, cout, out_in_map, num_out_feats, bias,
                                           residual, relu, out, also)
    if _grouping_pays(x, kvol, cin, cout, num_out_feats, out_in_map):
        return conv_implicit_gemm_grouped(x, wp, kvol, cin, cout, out_in_map, num_out_feats, bias,
                                          residual, relu, out, also)
    if out is None and also is None:
        y = x.new_empty(num_out_feats, cout)  # (the cheapest form of the call: 1.2 us against 1.6)
        at, ldy, a2, ld2 = y.data_ptr(), 0, 0, 0
    else:
        y, at, ldy, a2, ld2 = _placed(x, num_out_feats, cout, out, also)
    code = _dtype_code(x)
    stream = _stream()
    pb, pr = _epilogue_args(bias, residual, x, num_out_feats, cout)
    # (the arguments of tsmi_conv_implicit_gemm in one block: one conversion instead of 18)
    ws_elems = _workspace_elems(num_out_feats, kvol, cin, cout, code) if num_out_feats < 65536 else 0
    if ws_elems > 0:  # (only maps with few row tiles use the offset split)
        with _scratch_lock:
            block = _PACK21(stream, x.data_ptr(), wp.data_ptr(), out_in_map.data_ptr(), out_in_map.shape[0],
                            num_out_feats, kvol, cin, cout, code, pb or 0, pr or 0, int(relu),
                            _scratch(x.device, stream, 4 * ws_elems), ws_elems,
                            _tile_counters(x.device, stream).data_ptr(), _N_TILE_COUNTERS, at, ldy, a2, ld2)
            if not (_region_depth and _hand_over(0, block, 21, (x, wp, out_in_map, bias, residual, y, also,
                                                                _SCRATCH.get((x.device.index, stream))))):
                _check(_C.tsmi_conv_implicit_gemm_packed(block))
    else:
        block = _PACK21(stream, x.data_ptr(), wp.data_ptr(), out_in_map.data_ptr(), out_in_map.shape[0], num_out_feats,
                        kvol, cin, cout, code, pb or 0, pr or 0, int(relu), 0, 0, 0, _N_TILE_COUNTERS, at, ldy, a2, ld2)
        if not (_region_depth and _hand_over(0, block, 21, (x, wp, out_in_map, bias, residual, y, also))):
            _check(_C.tsmi_conv_implicit_gemm_packed(block))
    return y


_IDENTITY_MAPS = {}


def _identity_map(n: int, device) -> torch.Tensor:
    """int32 [ceil128(n), 1]: row i -> i, pad rows -1 (the map of a 1x1x1 convolution).  The
    few most recent sizes are kept."""
    key = (device.index if device.index is not None else _cur_device(), n)
    m = _IDENTITY_MAPS.get(key)
    if m is None:
        m = torch.full((make_divisible(n, 128), 1), -1, dtype=torch.int32, device=device)
        m[:n, 0] = torch.arange(n, dtype=torch.int32, device=device)
        with _tables_lock:
            if len(_IDENTITY_MAPS) >= 16:
                _IDENTITY_MAPS.pop(next(iter(_IDENTITY_MAPS)), None)
            _IDENTITY_MAPS[key] = m
    if _pin_sinks:
        _pin(m)
    return m


def conv_pointwise_cuda(in_feats, kernel, bias=None, residual=None, relu=False) -> torch.Tensor:
    """1x1x1 convolution act(X W + bias + residual) through the implicit-GEMM kernels over the
    identity map: bias, residual add and ReLU stay in the kernel epilogue (the reference's
    conv.py:65-75 calls torch.mm and adds the bias afterwards)."""
    n = in_feats.shape[0]
    w = kernel if kernel.dim() == 3 else kernel.unsqueeze(0)
    if n == 0:
        return torch.empty((0, w.shape[2]), dtype=in_feats.dtype, device=in_feats.device)
    return conv_forward_implicit_gemm_cuda(in_feats, kernel, _identity_map(n, in_feats.device), n,
                                           w.shape[2], bias=bias, residual=residual, relu=relu)


def conv_dgrad_implicit_gemm_cuda(grad_out, kernel, in_out_map, num_in_feats) -> torch.Tensor:
    """Input gradient dX[m] = sum_k dY[map[m, k]] W[k]^T: the forward kernel over the
    (input row, offset) -> output row map with the weights transposed per offset
    (the reference's func/implicit_gemm.py:124-141).  The packed layout of W[k]^T is
    [Cin padded, Cout padded] row-major, which is W[k] itself when neither channel count
    needs padding: then the kernel tensor is passed as it is."""
    w = kernel if kernel.dim() == 3 else kernel.unsqueeze(0)
    kvol, cin, cout = w.shape
    if grad_out.shape[0] == 0:  # a convolution without outputs: nothing flows back
        return torch.zeros((num_in_feats, cin), dtype=grad_out.dtype, device=grad_out.device)
    if w.is_contiguous() and _C.tsmi_packed_weight_elems(kvol, cout, cin) == w.numel():
        if grad_out.dtype != w.dtype:
            raise ValueError(f"feature dtype {grad_out.dtype} and kernel dtype {w.dtype} differ")
        if grad_out.shape[1] != cout:
            raise ValueError("Input feature size and kernel size mismatch")
        dy = grad_out if grad_out.is_contiguous() else grad_out.contiguous()
        return _implicit_gemm(dy, w.detach(), kvol, cout, cin, in_out_map, num_in_feats)
    return conv_forward_implicit_gemm_cuda(grad_out, w.transpose(1, 2).contiguous(), in_out_map,
                                           num_in_feats, cin)


def conv_forward_implicit_gemm_sorted_cuda(in_feats, kernel, reorder_out_in_map, reduced_mask,
                                           reorder_loc, num_out_feats, num_out_channels,
                                           allow_tf32=False, allow_fp16=True, bias=None,
                                           residual=None, relu=False) -> torch.Tensor:
    """convolution/convolution_forward_implicit_gemm_sorted_cuda.cu:1755-2230."""
    x, wp, (kvol, cin, cout) = _conv_common(in_feats, kernel)
    return _implicit_gemm_sorted(x, wp, kvol, cin, cout, reorder_out_in_map, reduced_mask, reorder_loc,
                                 num_out_feats, bias, residual, relu)


def _implicit_gemm_sorted(x, wp, kvol, cin, cout, reorder_out_in_map, reduced_mask, reorder_loc,
                          num_out_feats, bias=None, residual=None, relu=False) -> torch.Tensor:
    split = reorder_loc.shape[0]
    n_pad = reorder_out_in_map.shape[0]
    y = x.new_empty(num_out_feats, cout)  # (the cheapest form of the call: 1.2 us against 1.6)
    code = _dtype_code(x)
    ws, ws_elems = None, 0
    if split > 1 or n_pad < 65536:
        ws_elems = _C.tsmi_conv_workspace_elems(n_pad, num_out_feats, kvol, split, cin, cout, code, 1)
        if ws_elems > 0:
            ws = torch.empty(ws_elems, dtype=torch.float32, device=x.device)
    pb, pr = _epilogue_args(bias, residual, x, num_out_feats, cout)
    _check(_C.tsmi_conv_implicit_gemm_sorted(_stream(), _ptr(x), _ptr(wp), _ptr(reorder_out_in_map),
                                             _ptr(reduced_mask), _ptr(reorder_loc), n_pad,
                                             num_out_feats, kvol, split, cin, cout, code,
                                             pb, pr, int(relu), _ptr(ws), ws_elems,
                                             _ptr(_tile_counters(x.device, _stream())) if ws is not None else None,
                                             _N_TILE_COUNTERS, _ptr(y)))
    return y


def conv_dgrad_implicit_gemm_sorted_cuda(grad_out, kernel, reorder_in_out_map, reduced_mask,
                                         reorder_loc, num_in_feats) -> torch.Tensor:
    """conv_dgrad_implicit_gemm_cuda over the mask-sorted (input row, offset) -> output row map:
    the input gradient of the reference's sorted branch (func/implicit_gemm.py:130-141)."""
    w = kernel if kernel.dim() == 3 else kernel.unsqueeze(0)
    kvol, cin, cout = w.shape
    if grad_out.shape[0] == 0:
        return torch.zeros((num_in_feats, cin), dtype=grad_out.dtype, device=grad_out.device)
    if w.is_contiguous() and _C.tsmi_packed_weight_elems(kvol, cout, cin) == w.numel():
        if grad_out.dtype != w.dtype:
            raise ValueError(f"feature dtype {grad_out.dtype} and kernel dtype {w.dtype} differ")
        if grad_out.shape[1] != cout:
            raise ValueError("Input feature size and kernel size mismatch")
        dy = grad_out if grad_out.is_contiguous() else grad_out.contiguous()
        return _implicit_gemm_sorted(dy, w.detach(), kvol, cout, cin, reorder_in_out_map, reduced_mask,
                                     reorder_loc, num_in_feats)
    return conv_forward_implicit_gemm_sorted_cuda(grad_out, w.transpose(1, 2).contiguous(),
                                                  reorder_in_out_map, reduced_mask, reorder_loc,
                                                  num_in_feats, cin)


def conv_backward_wgrad_implicit_gemm_cuda(grad_out: torch.Tensor, in_feats: torch.Tensor,
                                           out_in_map_bwd: torch.Tensor, num_in_feats: int,
                                           split_k_iters: int = 32, allow_tf32=False,
                                           allow_fp16=True) -> torch.Tensor:
    """Weight gradient [K_vol, Cin, Cout] of the I/O type —
    convolution/convolution_backward_wgrad_implicit_gemm_cuda.cu:1614-2042, which returns
    the same sums laid out [K_vol*Cout, Cin].  out_in_map_bwd maps (input row, offset) to
    the output row; split_k_iters is accepted and ignored (the row split is chosen by the
    library)."""
    if in_feats.dtype != grad_out.dtype:
        raise ValueError("in_feats and grad_out must have the same dtype")
    x = _need(in_feats, in_feats.dtype, "in_feats")
    dy = _need(grad_out, grad_out.dtype, "grad_out")
    m = _need(out_in_map_bwd, torch.int32, "out_in_map_bwd")
    kvol, cin, cout = m.shape[1], x.shape[1], dy.shape[1]
    code = _dtype_code(x)
    dw = torch.empty((kvol, cin, cout), dtype=x.dtype, device=x.device)
    ws_elems = _C.tsmi_conv_wgrad_workspace_elems(num_in_feats, kvol, cin, cout, code)
    ws = torch.empty(max(ws_elems, 1), dtype=torch.float32, device=x.device)
    _check(_C.tsmi_conv_wgrad(_stream(), _ptr(x), _ptr(dy), _ptr(m), m.shape[0], num_in_feats, kvol,
                              cin, cout, code, _ptr(ws), ws_elems, _ptr(dw)))
    return dw


def wgrad_pair_lists(out_in_map: torch.Tensor, n_rows: int) -> dict:
    """Per-offset (map value, row) pair lists of a kernel map, padded to blocks of 32, for
    conv_backward_wgrad_pairs_cuda.  No host read-back: `pairs` is sized for a full map and
    only the part the lists need is written.  Returns dict(pairs int32 [cap, 2], seg_steps
    int32 [K_vol+1] (first 32-pair block of each offset), nbsizes int32 [K_vol])."""
    m = _need(out_in_map, torch.int32, "out_in_map")
    if n_rows > m.shape[0]:
        raise ValueError(f"map has {m.shape[0]} rows, need {n_rows}")
    kvol, dev = m.shape[1], m.device
    cap = _C.tsmi_wgrad_pairs_capacity(n_rows, kvol)
    pairs = torch.empty((max(cap, 1), 2), dtype=torch.int32, device=dev)
    block_counts = torch.empty(kvol * max((n_rows + 255) // 256, 1), dtype=torch.int32, device=dev)
    nbsizes = torch.empty(kvol, dtype=torch.int32, device=dev)
    seg_steps = torch.empty(kvol + 1, dtype=torch.int32, device=dev)
    _check(_C.tsmi_wgrad_pairs_build(_stream(), _ptr(m), n_rows, kvol, _ptr(block_counts),
                                     _ptr(nbsizes), _ptr(pairs), _ptr(seg_steps)))
    return dict(pairs=pairs, seg_steps=seg_steps, nbsizes=nbsizes, cap=cap)


def wgrad_pair_lists_from_nbmaps(nbmaps: torch.Tensor, nbsizes: torch.Tensor) -> dict:
    """The padded lists of wgrad_pair_lists from the gather-scatter dataflow's own pair
    lists: nbmaps int32 [nnz, 2] rows (in, out) ordered by offset, nbsizes [K_vol]."""
    nbmaps = _need(nbmaps, torch.int32, "nbmaps")
    dev = nbmaps.device
    sizes = nbsizes.to(device=dev, dtype=torch.int32).contiguous()
    kvol, nnz = sizes.numel(), nbmaps.shape[0]
    cap = nnz + 31 * kvol
    pairs = torch.empty((max(cap, 1), 2), dtype=torch.int32, device=dev)
    seg_steps = torch.empty(kvol + 1, dtype=torch.int32, device=dev)
    _check(_C.tsmi_wgrad_pairs_pad(_stream(), _ptr(nbmaps), nnz, _ptr(sizes), kvol, _ptr(pairs),
                                   _ptr(seg_steps)))
    return dict(pairs=pairs, seg_steps=seg_steps, nbsizes=sizes, cap=cap)


def wgrad_pairs_supported(in_feats: torch.Tensor, grad_out: torch.Tensor, kernel_volume: int = 1) -> bool:
    """The pair-list weight gradient moves 16-byte pieces of rows: both channel counts
    must be multiples of 16 bytes of elements; its segment table holds 511 offsets."""
    per = 16 // in_feats.element_size()
    return (in_feats.shape[1] % per == 0 and grad_out.shape[1] % per == 0
            and kernel_volume <= 511)


def conv_backward_wgrad_pairs_cuda(grad_out: torch.Tensor, in_feats: torch.Tensor, pair_lists: dict,
                                   x_col: int = 0) -> torch.Tensor:
    """Weight gradient [K_vol, Cin, Cout] of the I/O type from the pair lists of
    wgrad_pair_lists: dW[k] = sum over offset k's pairs of in_feats[pair[x_col]]^T
    grad_out[pair[1 - x_col]].  The sums of conv_backward_gather_scatter_cuda's grad_kernel
    (convolution/convolution_gather_scatter_cuda.cu:815-915), reading only rows that take
    part in an offset."""
    if in_feats.dtype != grad_out.dtype:
        raise ValueError("in_feats and grad_out must have the same dtype")
    x = _need(in_feats, in_feats.dtype, "in_feats")
    dy = _need(grad_out, grad_out.dtype, "grad_out")
    pairs = _need(pair_lists["pairs"], torch.int32, "pairs")
    seg_steps = _need(pair_lists["seg_steps"], torch.int32, "seg_steps")
    kvol, cin, cout = seg_steps.numel() - 1, x.shape[1], dy.shape[1]
    if x.shape[0] == 0 or dy.shape[0] == 0:
        return torch.zeros((kvol, cin, cout), dtype=x.dtype, device=x.device)
    code = _dtype_code(x)
    cap = int(pair_lists["cap"])
    dw = torch.empty((kvol, cin, cout), dtype=x.dtype, device=x.device)
    ws_elems = _C.tsmi_conv_wgrad_pairs_workspace_elems(cap, kvol, cin, cout, code)
    ws = torch.empty(max(ws_elems, 1), dtype=torch.float32, device=x.device)
    _check(_C.tsmi_conv_wgrad_pairs(_stream(), _ptr(x), _ptr(dy), _ptr(pairs), _ptr(seg_steps), cap,
                                    int(x_col), kvol, cin, cout, code, _ptr(ws), ws_elems, _ptr(dw)))
    return dw


def conv_backward_gather_scatter_cuda(in_feat: torch.Tensor, grad_in_feat: torch.Tensor,
                                      grad_out_feat: torch.Tensor, kernel: torch.Tensor,
                                      grad_kernel: torch.Tensor, neighbor_map: torch.Tensor,
                                      neighbor_offset: torch.Tensor, transpose: bool) -> None:
    """convolution/convolution_gather_scatter_cuda.cu:815-915: fills grad_in_feat (shape of
    in_feat) and grad_kernel (shape of kernel) in place from the pair lists neighbor_map
    int32 [nnz, 2] rows (in, out) and their per-offset sizes neighbor_offset.

    grad_in  = the forward dataflow over the same lists with the two columns exchanged and
               the weights transposed per offset (sums through the masks, no atomics);
    grad_w   = the pair-list weight-gradient kernel (the map form's sums for channel counts
               that are not a multiple of 16 bytes are not reachable from pair lists:
               those raise)."""
    x = _need(in_feat, in_feat.dtype, "in_feat")
    dy = _need(grad_out_feat, x.dtype, "grad_out_feat")
    nbmaps = _need(neighbor_map, torch.int32, "neighbor_map")
    w = kernel if kernel.dim() == 3 else kernel.unsqueeze(0)
    kvol = w.shape[0]
    if not transpose:
        n_in, n_out = x.shape[0], dy.shape[0]   # sizes of the pair columns (in, out)
    else:
        n_in, n_out = dy.shape[0], x.shape[0]
    sizes = neighbor_offset.to(device=x.device, dtype=torch.int32)
    imask, omask = build_mask_from_kmap(n_in, n_out, nbmaps, sizes)
    # pair lists alone do not say whether the centre offset is the identity: masks and scatter
    # both follow the reference's rule here (odd volume and as many outputs as inputs)
    center = kvol // 2 if (n_in == n_out and kvol % 2 == 1) else -1
    dx = conv_forward_gather_scatter_cuda(dy, w.transpose(1, 2).contiguous(), nbmaps, sizes, imask, omask,
                                          x.shape[0], transpose=not transpose, center_k=center)
    lists = wgrad_pair_lists_from_nbmaps(nbmaps, sizes)
    dw = conv_backward_wgrad_pairs_cuda(dy, x, lists, 1 if transpose else 0)
    grad_in_feat.resize_(x.shape).copy_(dx)
    grad_kernel.resize_(kernel.shape).copy_(dw.reshape(kernel.shape))


def conv_forward_fetch_on_demand_cuda(in_feats, kernel, nbmaps, sum_nnz, nbaddrs, qnbaddrs,
                                      output_size, qsum_nnz, transpose, allow_tf32=False,
                                      allow_fp16=True, row_mask=None, center_k=-1, bias=None,
                                      residual=None, relu=False) -> torch.Tensor:
    """convolution/convolution_forward_fetch_on_demand_cuda.cu:1981-2119.  nbmaps is the
    planar [2, nnz] list; row_mask is the kmap's output_mask (input_mask when
    transposed) that makes the reduction atomic free."""
    x, wp, (kvol, cin, cout) = _conv_common(in_feats, kernel)
    if row_mask is None:
        raise ValueError("fetch-on-demand needs the kmap's row mask (output_mask / input_mask)")
    y = torch.empty((output_size, cout), dtype=x.dtype, device=x.device)
    partial = torch.empty((max(int(sum_nnz), 1), cout), dtype=x.dtype, device=x.device)
    pb, pr = _epilogue_args(bias, residual, x, output_size, cout)
    _check(_C.tsmi_conv_fetch_on_demand(_stream(), _ptr(x), _ptr(wp), _ptr(nbmaps), int(sum_nnz),
                                        _ptr(nbaddrs), _ptr(qnbaddrs), int(qsum_nnz), _ptr(row_mask),
                                        output_size, kvol, cin, cout, _dtype_code(x),
                                        int(bool(transpose)), center_k, pb, pr, int(relu),
                                        _ptr(partial), _ptr(y)))
    return y


def conv_forward_gather_scatter_cuda(in_feats, kernel, nbmaps, nbsizes, input_mask, output_mask,
                                     output_size, epsilon=0.0, mm_thresh=0, conv_mode=0,
                                     transpose=False, buffer=None, nbaddrs=None, qnbaddrs=None,
                                     qsum_nnz=None, center_k=-1, bias=None, residual=None,
                                     relu=False) -> torch.Tensor:
    """convolution/convolution_gather_scatter_cuda.cu:279-814: gather -> GEMM per
    offset -> scatter, here always as three launches over all offsets.  epsilon,
    mm_thresh and conv_mode only steer grouping in the reference; results do not
    depend on them and they are accepted and ignored.  nbmaps is the interleaved
    int32 [nnz, 2] list."""
    x, wp, (kvol, cin, cout) = _conv_common(in_feats, kernel)
    nbmaps = _need(nbmaps, torch.int32, "nbmaps")
    nnz = nbmaps.shape[0]
    dev = x.device
    if nbaddrs is None or qnbaddrs is None:
        sizes = nbsizes.to(device=dev, dtype=torch.int32)
        nbaddrs = torch.zeros(kvol + 1, dtype=torch.int32, device=dev)
        qnbaddrs = torch.zeros(kvol + 1, dtype=torch.int32, device=dev)
        exclusive_scan_quantified_wrapper(kvol, sizes, nbaddrs, qnbaddrs)
        qsum_nnz = None
    if qsum_nnz is None:
        qsum_nnz = int(qnbaddrs[-1].item())
    row_mask = input_mask if transpose else output_mask
    code = _dtype_code(x)
    gathered = torch.empty((max(nnz, 1), cin), dtype=x.dtype, device=dev)
    products = torch.empty((max(nnz, 1), cout), dtype=x.dtype, device=dev)
    y = torch.empty((output_size, cout), dtype=x.dtype, device=dev)
    s = _stream()
    _check(_C.tsmi_gs_gather(s, _ptr(x), _ptr(nbmaps), nnz, cin, code, int(bool(transpose)),
                             _ptr(gathered)))
    _check(_C.tsmi_gs_gemm(s, _ptr(gathered), _ptr(wp), _ptr(nbaddrs), _ptr(qnbaddrs), nnz,
                           int(qsum_nnz), kvol, cin, cout, code, _ptr(products)))
    pb, pr = _epilogue_args(bias, residual, x, output_size, cout)
    _check(_C.tsmi_gs_scatter(s, _ptr(products), _ptr(nbaddrs), _ptr(row_mask), output_size, kvol,
                              cout, code, center_k, pb, pr, int(relu), _ptr(y)))
    return y


# ------------------------------------------------------------ point-voxel operators


def hash_cuda(coords: torch.Tensor) -> torch.Tensor:
    """hash/hash_cuda.cu:64-70: int64 [N] FNV-1a hashes of int32 [N,4] rows."""
    coords = _need(coords, torch.int32, "coords")
    out = torch.empty(coords.shape[0], dtype=torch.int64, device=coords.device)
    _check(_C.tsmi_hash_coords(_stream(), _ptr(coords), coords.shape[0], _ptr(out)))
    return out


def kernel_hash_cuda(coords: torch.Tensor, kernel_offset: torch.Tensor) -> torch.Tensor:
    """hash/hash_cuda.cu:72-83: int64 [K,N] hashes of the rows shifted by each offset."""
    coords = _need(coords, torch.int32, "coords")
    offsets = _need(kernel_offset, torch.int32, "kernel_offset")
    out = torch.empty((offsets.shape[0], coords.shape[0]), dtype=torch.int64, device=coords.device)
    _check(_C.tsmi_kernel_hash(_stream(), _ptr(coords), coords.shape[0], _ptr(offsets),
                               offsets.shape[0], _ptr(out)))
    return out


def count_cuda(idx: torch.Tensor, num: int) -> torch.Tensor:
    """others/count_cuda.cu:24-31: int32 [num] occurrences of each index (negatives skipped)."""
    idx = _need(idx, torch.int32, "idx")
    out = torch.empty(int(num), dtype=torch.int32, device=idx.device)
    _check(_C.tsmi_count(_stream(), _ptr(idx), idx.numel(), _ptr(out), int(num)))
    return out


def group_by_index(idx: torch.Tensor, n_groups: int):
    """(order, starts) of an int32 index tensor: the positions of the entries with a value in
    [0, n_groups) sorted by (value, position), and the start of every value's run.  Kept on
    the tensor (and rebuilt when it is modified in place): a network voxelizes and
    devoxelizes through the same indices many times."""
    idx = _need(idx, torch.int32, "idx")
    cached = getattr(idx, "_tsmi_groups", None)
    if cached is not None and cached[0] == (idx._version, int(n_groups)):
        return cached[1], cached[2]
    m, dev = idx.numel(), idx.device
    temp_bytes = _C.tsmi_group_temp_bytes(m)
    temp = torch.empty(max(temp_bytes, 1), dtype=torch.uint8, device=dev)
    order = torch.empty(max(m, 1), dtype=torch.int32, device=dev)
    starts = torch.empty(int(n_groups) + 1, dtype=torch.int32, device=dev)
    _check(_C.tsmi_group_by_index(_stream(), _ptr(idx), m, int(n_groups), _ptr(temp), temp_bytes,
                                  _ptr(order), _ptr(starts)))
    idx._tsmi_groups = ((idx._version, int(n_groups)), order, starts)
    return order, starts


def voxelize_forward_cuda(inputs: torch.Tensor, idx: torch.Tensor, counts: torch.Tensor) -> torch.Tensor:
    """voxelize/voxelize_cuda.cu:82-100: [N1, C] means of the points of each voxel."""
    x = _need(inputs, inputs.dtype, "inputs")
    idx, counts = _need(idx, torch.int32, "idx"), _need(counts, torch.int32, "counts")
    n, c, n1 = x.shape[0], x.shape[1], counts.shape[0]
    if idx.numel() != n:
        raise ValueError(f"idx has {idx.numel()} entries for {n} points")
    order, starts = group_by_index(idx, n1)
    out = torch.empty((n1, c), dtype=x.dtype, device=x.device)
    _check(_C.tsmi_voxelize_forward(_stream(), _ptr(x), _ptr(counts), _ptr(order), _ptr(starts), n, c,
                                    n1, _dtype_code(x), _ptr(out)))
    return out


def voxelize_backward_cuda(top_grad: torch.Tensor, idx: torch.Tensor, counts: torch.Tensor,
                           n: int) -> torch.Tensor:
    """voxelize/voxelize_cuda.cu:102-120."""
    g = _need(top_grad, top_grad.dtype, "top_grad")
    idx, counts = _need(idx, torch.int32, "idx"), _need(counts, torch.int32, "counts")
    out = torch.empty((int(n), g.shape[1]), dtype=g.dtype, device=g.device)
    _check(_C.tsmi_voxelize_backward(_stream(), _ptr(g), _ptr(idx), _ptr(counts), int(n), g.shape[1],
                                     counts.shape[0], _dtype_code(g), _ptr(out)))
    return out


def devoxelize_forward_cuda(feat: torch.Tensor, indices: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """devoxelize/devoxelize_cuda.cu:62-79: [N, C] interpolations from 8 corner voxels
    (indices int32 [N,8], weight [N,8]; the weights are used in fp32)."""
    f = _need(feat, feat.dtype, "feat")
    indices = _need(indices, torch.int32, "indices")
    w = _need(weight.float(), torch.float32, "weight")
    n = indices.shape[0]
    out = torch.empty((n, f.shape[1]), dtype=f.dtype, device=f.device)
    _check(_C.tsmi_devoxelize_forward(_stream(), _ptr(f), _ptr(indices), _ptr(w), n, f.shape[0],
                                      f.shape[1], _dtype_code(f), _ptr(out)))
    return out


def devoxelize_backward_cuda(top_grad: torch.Tensor, indices: torch.Tensor, weight: torch.Tensor,
                             n: int) -> torch.Tensor:
    """devoxelize/devoxelize_cuda.cu:83-98: [n, C] gradient with respect to the voxel features."""
    g = _need(top_grad, top_grad.dtype, "top_grad")
    indices = _need(indices, torch.int32, "indices")
    w = _need(weight.float(), torch.float32, "weight")
    if indices.shape[0] != g.shape[0] or w.numel() != indices.numel():
        raise ValueError("top_grad, indices and weight disagree on the number of points")
    order, starts = group_by_index(indices, int(n))
    out = torch.empty((int(n), g.shape[1]), dtype=g.dtype, device=g.device)
    _check(_C.tsmi_devoxelize_backward(_stream(), _ptr(g), _ptr(w), _ptr(order), _ptr(starts),
                                       indices.shape[0], int(n), g.shape[1], _dtype_code(g), _ptr(out)))
    return out


def to_dense_forward_cuda(inputs: torch.Tensor, idx: torch.Tensor, spatial_range, outputs: torch.Tensor) -> None:
    """voxelize/voxelize_cuda.cu:122-131: outputs [B,X,Y,Z,C] (already zero) receives the rows."""
    x = _need(inputs, inputs.dtype, "inputs")
    idx = _need(idx, torch.int32, "idx")
    out = _need(outputs, x.dtype, "outputs")
    rng = [int(v) for v in (spatial_range.tolist() if torch.is_tensor(spatial_range) else spatial_range)]
    _check(_C.tsmi_to_dense_forward(_stream(), _ptr(x), _ptr(idx), x.shape[0], x.shape[1], _I4(*rng),
                                    _dtype_code(x), _ptr(out)))


def to_dense_backward_cuda(top_grad: torch.Tensor, idx: torch.Tensor, spatial_range,
                           bottom_grad: torch.Tensor) -> None:
    """voxelize/voxelize_cuda.cu:133-141."""
    g = _need(top_grad, top_grad.dtype, "top_grad")
    idx = _need(idx, torch.int32, "idx")
    out = _need(bottom_grad, g.dtype, "bottom_grad")
    rng = [int(v) for v in (spatial_range.tolist() if torch.is_tensor(spatial_range) else spatial_range)]
    _check(_C.tsmi_to_dense_backward(_stream(), _ptr(g), _ptr(idx), out.shape[0], out.shape[1], _I4(*rng),
                                     _dtype_code(g), _ptr(out)))


# ------------------------------------------------------------------ batch normalisation


def bn_supported(x: torch.Tensor, *params) -> bool:
    """Whether the batch-norm kernels take this [N, C] matrix: GPU, contiguous, a supported
    type, N >= 2, C a multiple of 16 bytes' worth of elements (at most 256 such pieces), and
    every parameter / running statistic given of one supported type."""
    if not (x.is_cuda and x.dim() == 2 and x.dtype in _DTYPE_CODE and x.is_contiguous() and x.shape[0] >= 2):
        return False
    v = 4 if x.dtype == torch.float32 else 8
    if x.shape[1] < v or x.shape[1] % v or x.shape[1] // v > 256 or x.data_ptr() % 16:
        return False
    given = [p for p in params if p is not None]
    return all(p.is_cuda and p.dtype in _DTYPE_CODE and p.dtype == given[0].dtype and p.is_contiguous()
               and p.numel() == x.shape[1] for p in given)


def bn_forward_train(x, weight, bias, running_mean, running_var, momentum: float, eps: float):
    """(y, mean, invstd): batch statistics over the rows of x [N, C], running statistics updated in
    place — what torch.nn.functional.batch_norm(training=True) does for nn/modules/norm.py:13-17."""
    n, c = x.shape
    given = [p for p in (weight, bias, running_mean, running_var) if p is not None]
    pcode = _dtype_code(given[0]) if given else F32
    work = torch.empty(_C.tsmi_bn_partial_elems(c), dtype=torch.float32, device=x.device)
    stats = torch.empty(4 * c, dtype=torch.float32, device=x.device)
    y = torch.empty_like(x)
    _check(_C.tsmi_bn_forward_train(_stream(), _ptr(x), n, c, _dtype_code(x), _ptr(weight), _ptr(bias), pcode,
                                    _ptr(running_mean), _ptr(running_var), float(momentum), float(eps),
                                    _ptr(work), _ptr(stats), _ptr(y)))
    return y, stats[:c], stats[c:2 * c]


def bn_backward(dy, x, weight, mean, invstd):
    """(dx, sum_rows dy * xhat, sum_rows dy): the input, weight and bias gradients (the last two in
    the weight's type; fp32 without a weight)."""
    n, c = x.shape
    work = torch.empty(_C.tsmi_bn_partial_elems(c), dtype=torch.float32, device=x.device)
    sums = torch.empty(5 * c, dtype=torch.float32, device=x.device)
    dx = torch.empty_like(x)
    pcode = _dtype_code(weight) if weight is not None else F32
    grads = torch.empty(2 * c, dtype=weight.dtype, device=x.device) if weight is not None else None
    _check(_C.tsmi_bn_backward(_stream(), _ptr(dy), _ptr(x), n, c, _dtype_code(x), _ptr(weight), pcode,
                               _ptr(mean), _ptr(invstd), _ptr(work), _ptr(sums), _ptr(grads), _ptr(dx)))
    if grads is not None:
        return dx, grads[c:], grads[:c]
    return dx, sums[c:2 * c], sums[:c]
