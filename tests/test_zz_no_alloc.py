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


def _build(backend, C, omap, n_rows, static):
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
        got = _build(backend, C, omap, n, static=True)
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
