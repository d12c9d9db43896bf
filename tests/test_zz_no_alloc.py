"""The entry point that allocates nothing: tsmi_wgrad_pairs_build_static keeps the per-block
counts of the pair-list build in an array built into the library instead of a caller's buffer.
Called through the C ABI with preallocated inputs and outputs, twice in a row (the second map
smaller, so the array still holds the first call's counts), it must give the bits of
tsmi_wgrad_pairs_build; sizes beyond the built-in array are refused."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import random_coords

pytestmark = pytest.mark.gpu


def _build(backend, C, omap, n_rows, static, check_free=False):
    kvol = omap.shape[1]
    dev = omap.device
    cap = C.tsmi_wgrad_pairs_capacity(n_rows, kvol)
    pairs = torch.full((max(cap, 1), 2), -7, dtype=torch.int32, device=dev)
    nbsizes = torch.full((kvol,), -7, dtype=torch.int32, device=dev)
    seg_steps = torch.full((kvol + 1,), -7, dtype=torch.int32, device=dev)
    stream = backend._stream()
    if static:
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"], torch.cuda.mem_get_info()[0]
        status = C.tsmi_wgrad_pairs_build_static(stream, omap.data_ptr(), n_rows, kvol, nbsizes.data_ptr(),
                                                 pairs.data_ptr(), seg_steps.data_ptr())
        torch.cuda.synchronize()
        after = torch.cuda.memory_stats()["allocation.all.allocated"], torch.cuda.mem_get_info()[0]
        assert before[0] == after[0]  # nothing came from torch's allocator
        if check_free:  # ... and nothing from the device behind its back (hipMalloc inside the library)
            assert before[1] == after[1], (before[1], after[1])
    else:
        nblk = max((n_rows + 255) // 256, 1)
        counts = torch.empty(kvol * nblk, dtype=torch.int32, device=dev)
        status = C.tsmi_wgrad_pairs_build(stream, omap.data_ptr(), n_rows, kvol, counts.data_ptr(),
                                          nbsizes.data_ptr(), pairs.data_ptr(), seg_steps.data_ptr())
    assert status == 0, C.tsmi_last_error()
    return pairs, nbsizes, seg_steps


def test_static_scratch_entry_point_matches_the_buffer_one():
    from torchsparse_amd import backend
    from torchsparse_amd.nn import functional as F
    C = backend._C
    rng = np.random.default_rng(3)
    first = True
    for n, shape, ks in ((60000, (120, 110, 30), 3), (7001, (40, 40, 20), 3), (900, (12, 12, 12), (5, 3, 1)),
                         (0, (4, 4, 4), 3)):
        coords = torch.from_numpy(random_coords(rng, n, shape)).cuda() if n else \
            torch.zeros((0, 4), dtype=torch.int32, device="cuda")
        if n:
            omap = F.build_kernel_map(coords, n, ks, 1, 1, mode="hashmap_on_the_fly")["out_in_map"]
        else:
            omap = torch.zeros((0, 27), dtype=torch.int32, device="cuda")
        want = _build(backend, C, omap, n, static=False)
        if first:  # the first call on a device looks the array's address up; repeat it for the check
            _build(backend, C, omap, n, static=True)
            first = False
        got = _build(backend, C, omap, n, static=True, check_free=True)
        for g, w in zip(got, want):
            assert torch.equal(g, w), (n, ks)
        assert int(got[1].sum()) == int((omap[:n] >= 0).sum())
    # a map whose counts do not fit the built-in array is refused, with a message, before any launch
    fake = torch.zeros(1, dtype=torch.int32, device="cuda")
    too_many = (1 << 20) // 27 * 256 + 257
    status = C.tsmi_wgrad_pairs_build_static(backend._stream(), fake.data_ptr(), too_many, 27, fake.data_ptr(),
                                             fake.data_ptr(), fake.data_ptr())
    assert status == 1 and b"built-in scratch" in C.tsmi_last_error()
    torch.cuda.synchronize()


def test_static_calls_queued_back_to_back_on_one_stream():
    """Two calls on one stream with no synchronisation between them, the second over a smaller
    map: the stream orders their use of the built-in array, each gives the bits of the buffer
    entry point, and the free device memory is the same before and after."""
    from torchsparse_amd import backend
    from torchsparse_amd.nn import functional as F
    C = backend._C
    rng = np.random.default_rng(11)
    cases = []
    for n, shape in ((50000, (100, 100, 30)), (3000, (30, 30, 20))):
        coords = torch.from_numpy(random_coords(rng, n, shape)).cuda()
        omap = F.build_kernel_map(coords, n, 3, 1, 1, mode="hashmap_on_the_fly")["out_in_map"]
        cap = C.tsmi_wgrad_pairs_capacity(n, 27)
        outs = (torch.full((max(cap, 1), 2), -7, dtype=torch.int32, device="cuda"),
                torch.full((27,), -7, dtype=torch.int32, device="cuda"),
                torch.full((28,), -7, dtype=torch.int32, device="cuda"))
        cases.append((omap, n, outs, _build(backend, C, omap, n, static=False)))
    stream = backend._stream()
    _build(backend, C, cases[1][0], cases[1][1], static=True)  # (the address look-up of a fresh process)
    torch.cuda.synchronize()
    free = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        for omap, n, (pairs, nbsizes, seg_steps), _ in cases:
            assert C.tsmi_wgrad_pairs_build_static(stream, omap.data_ptr(), n, 27, nbsizes.data_ptr(),
                                                   pairs.data_ptr(), seg_steps.data_ptr()) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free
    for omap, n, (pairs, nbsizes, seg_steps), want in cases:
        for g, w in zip((nbsizes, pairs, seg_steps), (want[1], want[0], want[2])):
            assert torch.equal(g, w), n
