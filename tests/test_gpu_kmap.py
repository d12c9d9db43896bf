"""GPU parity of kernel-map construction: the HIP path (through libtsmi.so's C ABI,
via torchsparse_amd.backend) against the CPU oracle.  Bit-exact."""
import numpy as np
import pytest
import torch

import oracle
from helpers import lidar_like_coords, random_coords

pytestmark = pytest.mark.gpu

backend = None
F = None


@pytest.fixture(scope="module", autouse=True)
def _load():
    global backend, F
    from torchsparse_amd import backend as b
    from torchsparse_amd.nn import functional as f
    backend, F = b, f
    assert b._C.tsmi_version() >= 1


def dev(a, dtype=torch.int32):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", dtype)


def t3(v):
    return (v,) * 3 if isinstance(v, int) else tuple(v)


SUBM_CASES = [3, 2, 5, (3, 1, 1), (1, 3, 1), (2, 3, 3), (3, 5, 3)]


@pytest.mark.parametrize("ks", SUBM_CASES)
@pytest.mark.parametrize("batch", [1, 3])
def test_subm_map_matches_oracle(ks, batch):
    rng = np.random.default_rng(100)
    coords = random_coords(rng, 900, (14, 12, 10), batch)
    coords = coords[rng.permutation(len(coords))]
    kmap = F.build_kernel_map(dev(coords), len(coords), t3(ks), 1, 0, mode="hashmap_on_the_fly")
    want = oracle.kmap_subm(coords, t3(ks))
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want)
    assert kmap["sizes"] == (len(coords), len(coords))
    assert kmap["out_in_map"].shape[0] % 128 == 0


DOWN_CASES = [(2, 2, 0), (3, 2, 1), (3, 3, 1), (5, 2, 2), (5, 3, 2), (2, 3, 0), (3, 2, 0),
              ((3, 1, 1), (2, 1, 1), (0, 0, 0)), ((3, 3, 3), (2, 2, 2), (0, 1, 1)),
              ((1, 3, 1), (1, 2, 1), 0)]


@pytest.mark.parametrize("ks,stride,pad", DOWN_CASES)
@pytest.mark.parametrize("with_range", [False, True])
@pytest.mark.parametrize("through_grid", [True, False])
def test_downsample_map_matches_oracle(ks, stride, pad, with_range, through_grid, monkeypatch):
    monkeypatch.setattr(backend, "downsample_through_grid", through_grid)
    rng = np.random.default_rng(101)
    shape = (19, 17, 13)
    coords = random_coords(rng, 700, shape, batch=2)
    coords = coords[rng.permutation(len(coords))]
    ks, stride, pad = t3(ks), t3(stride), t3(pad)
    sr = (2,) + shape if with_range else None
    kmap = F.build_kernel_map(dev(coords), len(coords), ks, stride, pad, spatial_range=sr,
                              mode="hashmap_on_the_fly")
    new_sr = None
    if with_range:
        new_sr = (2,) + tuple((shape[a] + 2 * pad[a] - (ks[a] - 1) - 1) // stride[a] + 1 for a in range(3))
        assert kmap["spatial_range"] == new_sr
    want_map, want_coords = oracle.kmap_downsample(coords, ks, stride, pad, spatial_range=new_sr)
    np.testing.assert_array_equal(kmap["coords"].cpu().numpy(), want_coords)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want_map)
    assert kmap["sizes"] == (len(coords), len(want_coords))


@pytest.mark.parametrize("ks,stride", [(2, 2), (3, 2), (3, 1), (2, 1), (5, 3), (3, 3)])
def test_hashmap_mode_matches_oracle(ks, stride):
    rng = np.random.default_rng(102)
    coords = random_coords(rng, 800, (16, 16, 16), batch=2)
    pad = (ks - 1) // 2 if ks % 2 == 1 else 0
    kmap = F.build_kernel_map(dev(coords), len(coords), ks, stride, pad, mode="hashmap")
    if stride == 1:
        want_coords = coords
    elif stride == ks:
        want_coords = oracle.spdownsample_floor(coords, stride)
    else:
        want_coords = oracle.kmap_downsample(coords, ks, stride, pad)[1]
    np.testing.assert_array_equal(kmap["coords"].cpu().numpy(), want_coords)
    want = oracle.lookup_coords(coords, want_coords, ks, stride)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want)
    # GPUHashTable.lookup_coords keeps the reference's (x,y,z,b) rows and +1 bias
    table = backend.GPUHashTable(*kmap["in_hashmap"])
    got = table.lookup_coords(dev(want_coords)[:, [1, 2, 3, 0]], t3(ks), t3(stride), ks ** 3)
    np.testing.assert_array_equal(got.cpu().numpy() - 1, want)


def test_spdownsample_minkowski_and_spconv():
    rng = np.random.default_rng(103)
    coords = random_coords(rng, 500, (20, 20, 20), batch=2)
    got = F.spdownsample(dev(coords), 2, 3, 1, downsample_mode="minkowski").cpu().numpy()
    np.testing.assert_array_equal(got, oracle.spdownsample_floor(coords, 2))
    got = F.spdownsample(dev(coords), 2, 3, 1).cpu().numpy()
    np.testing.assert_array_equal(got, oracle.kmap_downsample(coords, 3, 2, 1)[1])


@pytest.mark.parametrize("n,shape,batch", [(1, (3, 3, 3), 1), (40000, (300, 280, 24), 1),
                                           (30000, (90, 70, 40), 5), (3000, (4000, 3000, 900), 2),
                                           (2000, (100000, 90000, 70000), 1)])
@pytest.mark.parametrize("geom", [(2, 2, 0), (3, 2, 1), (5, 3, 2)])
def test_downsample_through_grid_equals_hash_and_sort(n, shape, batch, geom, monkeypatch):
    """The occupancy-bitmap path and the hash-and-sort path give the same output coordinates,
    in the same order, and tables that index them alike: small grids, grids of many 2048-word
    chunks, several batches, and grids too large for the bitmap (the call falls back)."""
    rng = np.random.default_rng(n + batch)
    cols = [rng.integers(0, batch, n)] + [rng.integers(0, e, n) for e in shape]
    coords = np.unique(np.stack(cols, 1).astype(np.int32), axis=0)
    coords = coords[rng.permutation(len(coords))]
    ks, st, pd = t3(geom[0]), t3(geom[1]), t3(geom[2])
    results = []
    for through_grid in (True, False):
        monkeypatch.setattr(backend, "downsample_through_grid", through_grid)
        out, table = backend.downsample_coords(dev(coords), ks, st, pd)
        omap = table.query_bxyz(out, (1, 1, 1), (1, 1, 1), (0, 0, 0))[:out.shape[0], 0]
        results.append((out.cpu().numpy(), omap.cpu().numpy()))
    np.testing.assert_array_equal(results[0][0], results[1][0])
    np.testing.assert_array_equal(results[0][1], np.arange(len(results[0][0])))
    np.testing.assert_array_equal(results[1][1], np.arange(len(results[1][0])))
    np.testing.assert_array_equal(results[0][0], oracle.kmap_downsample(coords, ks, st, pd)[1])


def test_downsample_grid_recovers_from_an_unfinished_call(monkeypatch):
    """The occupancy bitmap is shared by the calls on a stream and must be all zero between them:
    a call that stopped after marking (here: forged, then a real one that raises because the
    output table is too small) is noticed and the bitmap cleared before the next use."""
    monkeypatch.setattr(backend, "downsample_chain_ahead", False)
    rng = np.random.default_rng(7)
    coords = random_coords(rng, 5000, (60, 50, 40), batch=2)
    want = oracle.kmap_downsample(coords, t3(3), t3(2), t3(1))[1]
    args = (dev(coords), t3(3), t3(2), t3(1))
    np.testing.assert_array_equal(backend.downsample_coords(*args)[0].cpu().numpy(), want)
    assert backend._stream_states
    for state in backend._stream_states.values():
        state.grid_buf[:state.grid_words].fill_(-1)
        state.grid_dirty = True
    np.testing.assert_array_equal(backend.downsample_coords(*args)[0].cpu().numpy(), want)
    with pytest.raises(ValueError, match="capacity of hashtable"):
        backend.downsample_coords(*args, rsv_ratio=0.001)
    np.testing.assert_array_equal(backend.downsample_coords(*args)[0].cpu().numpy(), want)
    assert not any(state.grid_dirty for state in backend._stream_states.values())


@pytest.mark.parametrize("geom", [(2, 2, 0), (3, 2, 1), ((2, 2, 1), (2, 2, 1), (0, 0, 0))])
def test_strided_chain_computed_ahead_equals_level_by_level(geom, monkeypatch):
    """A chain of equal strided calls, each on the previous one's outputs: once the chain has
    been seen, its first call computes the later levels before its one read-back.  Same
    coordinates, same order, tables that index them, as level by level and as the oracle."""
    rng = np.random.default_rng(11)
    coords = lidar_like_coords(rng, 30000) if geom[0] == 2 else random_coords(rng, 20000, (150, 140, 30), 2)
    ks, st, pd = t3(geom[0]), t3(geom[1]), t3(geom[2])
    calls = []
    real = backend._downsample_coords_grid
    monkeypatch.setattr(backend, "_downsample_coords_grid",
                        lambda *a, **k: (calls.append(a[9] if len(a) > 9 else k.get("ahead")), real(*a, **k))[1])
    backend.release_scratch()  # no chain history from earlier tests

    def chain(ahead):
        monkeypatch.setattr(backend, "downsample_chain_ahead", ahead)
        outs, c = [], dev(coords)
        for _ in range(4):
            out, table = backend.downsample_coords(c, ks, st, pd)
            rows = table.query_bxyz(out, (1, 1, 1), (1, 1, 1), (0, 0, 0))[:out.shape[0], 0]
            outs.append((out.cpu().numpy(), rows.cpu().numpy()))
            c = out
        return outs

    base = chain(False)
    chain(True)  # the chain is learnt here
    del calls[:]
    ahead = chain(True)
    assert calls == [3], calls  # one call marks four levels, three calls return what it left
    want = coords
    for (a, ra), (b, rb) in zip(base, ahead):
        want = oracle.kmap_downsample(want, ks, st, pd)[1]
        np.testing.assert_array_equal(a, want)
        np.testing.assert_array_equal(b, want)
        np.testing.assert_array_equal(ra, np.arange(len(want)))
        np.testing.assert_array_equal(rb, np.arange(len(want)))
    # a different geometry on a level computed ahead ignores what was left for it
    out, _ = backend.downsample_coords(dev(coords), ks, st, pd)
    got = backend.downsample_coords(out, t3(3), t3(2), t3(0))[0].cpu().numpy()
    np.testing.assert_array_equal(got, oracle.kmap_downsample(base[0][0], t3(3), t3(2), t3(0))[1])
    assert not any(state.grid_dirty for state in backend._stream_states.values())
    # levels computed ahead and never asked for are dropped by the next chain
    chain(True)
    out, _ = backend.downsample_coords(dev(coords), ks, st, pd)
    state, = backend._stream_states.values()
    assert state.ahead and state.ahead_hits > 0
    np.testing.assert_array_equal(backend.downsample_coords(dev(coords), ks, st, pd)[0].cpu().numpy(), base[0][0])
    chain(True)
    assert not state.grid_dirty and not state.ahead


def test_table_reuse_across_levels():
    """The table a strided map leaves behind indexes its outputs and serves the next
    submanifold map at that level without re-insertion."""
    rng = np.random.default_rng(104)
    coords = random_coords(rng, 2000, (30, 30, 20))
    k1 = F.build_kernel_map(dev(coords), len(coords), 2, 2, 0, mode="hashmap_on_the_fly")
    keys, vals = k1["out_hashmap"]
    oc = k1["coords"]
    k2 = F.build_kernel_map(oc, oc.shape[0], 3, 1, 1, keys, vals, mode="hashmap_on_the_fly")
    np.testing.assert_array_equal(k2["out_in_map"].cpu().numpy(), oracle.kmap_subm(oc.cpu().numpy(), 3))


def test_transpose_and_sort_products():
    rng = np.random.default_rng(105)
    coords = random_coords(rng, 3000, (40, 40, 10))
    for ks, stride, pad, split in [(3, 1, 1, 1), (3, 1, 1, 3), (2, 2, 0, 1), (2, 2, 0, 2), (5, 1, 2, 5)]:
        kmap = F.build_kernel_map(dev(coords), len(coords), ks, stride, pad, mode="hashmap_on_the_fly",
                                  ifsort=True, split_mask_num=split)
        omap = kmap["out_in_map"].cpu().numpy()
        n_out = kmap["sizes"][1]
        want_bm = oracle.derive_bitmask(omap, split, n_out)
        np.testing.assert_array_equal(
            backend.derive_bitmask_from_out_in_map(kmap["out_in_map"], split, n_out).cpu().numpy(), want_bm)
        srt, loc = kmap["sorted_mask"].cpu().numpy(), kmap["reorder_loc"].cpu().numpy()
        np.testing.assert_array_equal(srt, -np.sort(-want_bm.astype(np.int64), axis=1))
        for s in range(split):  # loc is a permutation that realises the sort (ties in any order)
            assert sorted(loc[s].tolist()) == list(range(omap.shape[0]))
            np.testing.assert_array_equal(want_bm[s][loc[s]], srt[s])
        np.testing.assert_array_equal(kmap["reorder_out_in_map"].cpu().numpy(), oracle.reorder_map(omap, loc))
        np.testing.assert_array_equal(kmap["reduced_sorted_mask"].cpu().numpy(), oracle.reduce_bitmask(srt, 128))
        np.testing.assert_array_equal(backend.reduce_bitmask_cuda(kmap["sorted_mask"], 64).cpu().numpy(),
                                      oracle.reduce_bitmask(srt, 64))
        if stride > 1:
            F.transpose_kernel_map(kmap, ifsort=False)
            np.testing.assert_array_equal(kmap["out_in_map_t"].cpu().numpy(),
                                          oracle.transpose_map(omap, len(coords)))
            np.testing.assert_array_equal(
                F.convert_transposed_out_in_map(kmap["out_in_map"], oracle.ceil128(len(coords))).cpu().numpy(),
                oracle.transpose_map(omap, len(coords)))


@pytest.mark.parametrize("geom", [(3, 1, 1), (2, 2, 0), (3, 2, 1), (2, 1, 0)])
def test_pair_lists_masks_scans(geom):
    ks, stride, pad = geom
    rng = np.random.default_rng(106)
    coords = random_coords(rng, 2500, (30, 30, 12), batch=2)
    for dataflow in (F.Dataflow.GatherScatter, F.Dataflow.FetchOnDemand):
        kmap = F.build_kernel_map(dev(coords), len(coords), ks, stride, pad, mode="hashmap_on_the_fly",
                                  dataflow=dataflow)
        omap = kmap["out_in_map"].cpu().numpy()
        n_in, n_out = kmap["sizes"]
        nb, sz = oracle.pair_lists(omap)
        np.testing.assert_array_equal(kmap["nbsizes"].cpu().numpy(), sz)
        got = kmap["nbmaps"].cpu().numpy()
        if dataflow == F.Dataflow.FetchOnDemand:
            assert got.shape == (2, len(nb)) and kmap["nbmaps"].is_contiguous()
            got = got.T
        np.testing.assert_array_equal(got, nb)
        im, om = oracle.build_masks(n_in, n_out, nb, sz)
        np.testing.assert_array_equal(kmap["input_mask"].cpu().numpy(), im)
        np.testing.assert_array_equal(kmap["output_mask"].cpu().numpy(), om)
        a, q = oracle.exclusive_scan_quantified(sz)
        np.testing.assert_array_equal(kmap["nbaddrs"].cpu().numpy(), a)
        np.testing.assert_array_equal(kmap["qnbaddrs"].cpu().numpy(), q)
        assert int(kmap["qmapsize"]) == q[-1]
        im2, om2 = backend.build_mask_from_kmap(n_in, n_out, dev(nb), dev(sz))
        np.testing.assert_array_equal(im2.cpu().numpy(), im)
        np.testing.assert_array_equal(om2.cpu().numpy(), om)


def test_hashtable_vals_api_and_errors():
    rng = np.random.default_rng(107)
    keys = np.unique(rng.integers(0, 1 << 50, 5000))
    table = backend.GPUHashTable(2 * len(keys))
    table.insert_vals(dev(keys, torch.int64))
    qry = np.concatenate([keys[::7], rng.integers(1 << 51, 1 << 52, 50)])
    got = table.lookup_vals(dev(qry, torch.int64)).cpu().numpy()
    want = np.concatenate([np.arange(len(keys))[::7] + 1, np.zeros(50, np.int64)])
    np.testing.assert_array_equal(got, want)
    small = backend.GPUHashTable(8)
    with pytest.raises(ValueError, match="capacity"):
        small.insert_vals(dev(keys, torch.int64))
    with pytest.raises(ValueError):
        backend.GPUHashTable(torch.zeros(7, dtype=torch.int64, device="cuda"),
                             torch.zeros(7, dtype=torch.int32, device="cuda")).clear()
    with pytest.raises(RuntimeError, match="multiple of 4"):
        backend.reduce_bitmask_cuda(torch.zeros((1, 128), dtype=torch.int32, device="cuda"), 6)
    with pytest.raises(RuntimeError, match="GPU"):
        backend.GPUHashTable(64).insert_bxyz(torch.zeros((4, 4), dtype=torch.int32))


def test_empty_and_single_voxel():
    one = dev(np.array([[0, 3, 3, 3]]))
    kmap = F.build_kernel_map(one, 1, 3, 1, 1, mode="hashmap_on_the_fly")
    m = kmap["out_in_map"].cpu().numpy()
    assert m.shape == (128, 27) and m[0, 13] == 0 and (m >= 0).sum() == 1
    kmap = F.build_kernel_map(one, 1, 2, 2, 0, mode="hashmap_on_the_fly")
    assert kmap["coords"].cpu().tolist() == [[0, 1, 1, 1]] and (kmap["out_in_map"] >= 0).sum().item() == 1
    empty = torch.zeros((0, 4), dtype=torch.int32, device="cuda")
    kmap = F.build_kernel_map(empty, 0, 3, 1, 1, mode="hashmap_on_the_fly")
    assert kmap["out_in_map"].shape == (0, 27)
    kmap = F.build_kernel_map(empty, 0, 2, 2, 0, mode="hashmap_on_the_fly", dataflow=F.Dataflow.GatherScatter)
    assert kmap["coords"].shape == (0, 4) and kmap["nbmaps"].shape == (0, 2)


def test_medium_scan_maps_and_invariants():
    """~60k surface-like voxels: exact against the oracle, plus the size-independent
    invariants used at full benchmark sizes."""
    rng = np.random.default_rng(108)
    coords = lidar_like_coords(rng, 60000)
    c = dev(coords)
    kmap = F.build_kernel_map(c, len(coords), 3, 1, 1, mode="hashmap_on_the_fly")
    m = kmap["out_in_map"]
    np.testing.assert_array_equal(m.cpu().numpy(), oracle.kmap_subm(coords, 3))
    n = len(coords)
    assert (m[:n, 13] == torch.arange(n, device="cuda")).all()
    rows, ks = torch.nonzero(m[:n] >= 0, as_tuple=True)
    assert (m[m[rows, ks].long(), 26 - ks] == rows).all()
    k2 = F.build_kernel_map(c, n, 2, 2, 0, mode="hashmap_on_the_fly")
    want_map, want_coords = oracle.kmap_downsample(coords, 2, 2, 0)
    np.testing.assert_array_equal(k2["coords"].cpu().numpy(), want_coords)
    np.testing.assert_array_equal(k2["out_in_map"].cpu().numpy(), want_map)
    k3 = F.build_kernel_map(c, n, 3, 2, 1, mode="hashmap_on_the_fly")
    want_map, want_coords = oracle.kmap_downsample(coords, 3, 2, 1)
    np.testing.assert_array_equal(k3["coords"].cpu().numpy(), want_coords)
    np.testing.assert_array_equal(k3["out_in_map"].cpu().numpy(), want_map)


@pytest.mark.parametrize("ks", [(3, 3, 3), (5, 5, 5), (3, 1, 1), (1, 3, 5), (1, 1, 1)])
@pytest.mark.parametrize("n,shape", [(0, (4, 4, 4)), (1, (4, 4, 4)), (129, (6, 6, 5)), (5000, (30, 28, 12))])
def test_mirrored_subm_query_equals_the_full_query(ks, n, shape):
    """tsmi_kmap_query_subm (half of the offsets probed, hits stored twice) against
    tsmi_kmap_query (every offset probed): identical maps, pad rows included; coordinates at the
    edge of the packable range (negative ones too) and several batches."""
    rng = np.random.default_rng(sum(ks) + n)
    coords = random_coords(rng, n, shape, batch=2) if n else np.zeros((0, 4), np.int32)
    if n > 100:
        coords = coords.copy()
        coords[: n // 2, 1:] -= np.array(shape, np.int32) // 2          # negative coordinates
        coords[:8, 1] = (1 << 17) - 1 - np.arange(8)                    # largest packable x
        coords[8:16, 3] = -(1 << 17) + np.arange(8)                     # smallest packable z
        coords = np.unique(coords, axis=0)
    table = backend.GPUHashTable(backend.hash_capacity(max(len(coords), 1), 2), device="cuda")
    c = dev(coords)
    table.insert_bxyz(c)
    pad = tuple((k - 1) // 2 for k in ks)
    full = table.query_bxyz(c, ks, (1, 1, 1), pad)
    mirrored = table.query_subm_bxyz(c, ks)
    assert mirrored.shape == full.shape and mirrored.dtype == torch.int32
    assert torch.equal(mirrored, full)
    if len(coords):
        shifted = coords.copy()  # the map does not change under translation; the oracle ravels from 0
        shifted[:, 1:] -= coords[:, 1:].min(0)
        want = oracle.kmap_subm(shifted, ks)
        np.testing.assert_array_equal(mirrored.cpu().numpy()[:len(coords)], want[:len(coords)])
    with pytest.raises(ValueError):
        backend._check(backend._C.tsmi_kmap_query_subm(
            None, backend._ptr(table.keys), backend._ptr(table.vals), table.capacity, backend._ptr(c),
            len(coords), len(coords), backend._I3(2, 3, 3), backend._ptr(full)))


@pytest.mark.parametrize("n", [1, 2, 3, 1000, 4096, 4097, 16384, 16385, 60000])
def test_sort_keys_small_and_large(n):
    """tsmi_sort_keys (device-wide radix sort of packed coordinate keys): ascending, exact,
    repeated keys kept, input untouched."""
    rng = np.random.default_rng(n)
    keys = rng.integers(0, 1 << 62, n, dtype=np.int64)
    if n > 10:
        keys[: n // 4] = keys[n // 2: n // 2 + n // 4]  # duplicates
    C = backend._C
    d_in = torch.from_numpy(keys).cuda()
    d_out = torch.empty_like(d_in)
    temp_bytes = C.tsmi_sort_temp_bytes(n)
    temp = torch.empty(temp_bytes, dtype=torch.uint8, device="cuda")
    backend._check(C.tsmi_sort_keys(None, backend._ptr(d_in), backend._ptr(d_out), n, 63,
                                    backend._ptr(temp), temp_bytes))
    np.testing.assert_array_equal(d_out.cpu().numpy(), np.sort(keys))
    assert torch.equal(d_in.cpu(), torch.from_numpy(keys))  # the input is left alone


# Coordinates the packed table key cannot hold (18 bits per axis, 9 for the batch) must stop the
# call with a ValueError, in every builder; the reference takes any int32 coordinate
# (others/sparsemapping_cuda.cu:12-26), so a silent drop would be a wrong map with status 0.
BAD_ROWS = [(0, 131072, 3, 3), (0, 3, -131073, 3), (0, 3, 3, 1 << 20), (512, 3, 3, 3), (-1, 3, 3, 3)]


def _coords_with(bad_row):
    rng = np.random.default_rng(5)
    coords = random_coords(rng, 300, (12, 12, 12))
    coords[137] = bad_row
    return coords


@pytest.mark.parametrize("bad_row", BAD_ROWS)
def test_unpackable_coordinates_raise_in_the_submanifold_build(bad_row):
    coords = dev(_coords_with(bad_row))
    with pytest.raises(ValueError, match="packed hash key"):
        F.build_kernel_map(coords, coords.shape[0], 3, 1, 0, mode="hashmap_on_the_fly")
    table = backend.GPUHashTable(backend.hash_capacity(coords.shape[0]), device="cuda")
    with pytest.raises(ValueError, match="packed hash key"):
        table.insert_bxyz(coords)
    with pytest.raises(ValueError, match="packed hash key"):
        table.insert_coords(coords[:, [1, 2, 3, 0]].contiguous())


@pytest.mark.parametrize("bad_row", BAD_ROWS)
@pytest.mark.parametrize("through_grid", [True, False])
@pytest.mark.parametrize("mode", ["hashmap_on_the_fly", "hashmap"])
def test_unpackable_coordinates_raise_in_the_strided_builds(bad_row, through_grid, mode, monkeypatch):
    monkeypatch.setattr(backend, "downsample_through_grid", through_grid)
    coords = dev(_coords_with(bad_row))
    with pytest.raises(ValueError, match="packed hash key"):
        F.build_kernel_map(coords, coords.shape[0], 2, 2, 0, mode=mode)
    with pytest.raises(ValueError, match="packed hash key"):
        F.build_kernel_map(coords, coords.shape[0], 3, 2, 1, mode=mode)
    backend.release_scratch()  # a refused call leaves marks in the stream's bitmap: start clean


def test_coordinates_at_the_edge_of_the_packed_range_are_exact():
    """The largest and smallest packable coordinates, in every builder, against the oracle."""
    rng = np.random.default_rng(6)
    base = random_coords(rng, 400, (9, 9, 9))
    hi = base.copy()
    hi[:, 1:] += 131072 - 9
    kmap = F.build_kernel_map(dev(hi), len(hi), 3, 1, 0, mode="hashmap_on_the_fly")
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), oracle.kmap_subm(hi, 3))
    for through_grid in (True, False):
        backend.downsample_through_grid = through_grid
        try:
            kmap = F.build_kernel_map(dev(hi), len(hi), 2, 2, 0, mode="hashmap_on_the_fly")
        finally:
            backend.downsample_through_grid = True
        want_map, want_coords = oracle.kmap_downsample(hi, 2, 2, 0)
        np.testing.assert_array_equal(kmap["coords"].cpu().numpy(), want_coords)
        np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want_map)
    lo = base.copy()
    lo[:, 1:] -= 131072
    lo[:, 0] = 511
    kmap = F.build_kernel_map(dev(lo), len(lo), 3, 1, 0, mode="hashmap_on_the_fly")
    want = oracle.kmap_subm(lo, 3, coords_min=lo.min(0), coords_max=lo.max(0))
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want)


def test_a_checked_tensor_is_not_read_back_again_and_a_changed_one_is():
    rng = np.random.default_rng(7)
    coords = dev(random_coords(rng, 500, (10, 10, 10)))
    assert not backend._range_known(coords)
    F.build_kernel_map(coords, coords.shape[0], 3, 1, 0, mode="hashmap_on_the_fly")
    assert backend._range_known(coords)
    coords[3, 1] = 1 << 18  # an in-place write bumps the version: the tensor is checked again
    assert not backend._range_known(coords)
    with pytest.raises(ValueError, match="packed hash key"):
        F.build_kernel_map(coords, coords.shape[0], 3, 1, 0, mode="hashmap_on_the_fly")
    # outputs of a strided build are known to be in range: their own builds do not synchronise
    good = dev(random_coords(rng, 500, (10, 10, 10)))
    kmap = F.build_kernel_map(good, good.shape[0], 2, 2, 0, mode="hashmap_on_the_fly")
    assert backend._range_known(good) and backend._range_known(kmap["coords"])


def test_fused_submanifold_build_equals_the_separate_calls():
    """tsmi_kmap_build_subm against clear + insert + query on the same rows: table and map."""
    rng = np.random.default_rng(8)
    for n, ks in ((0, 3), (1, 3), (777, 3), (5000, (3, 1, 5)), (3001, 2), (2000, (2, 3, 3))):
        coords = dev(random_coords(rng, n, (30, 20, 10))) if n else torch.zeros((0, 4), dtype=torch.int32,
                                                                                 device="cuda")
        table, omap = backend.GPUHashTable.build_subm(coords, ks)
        ref = backend.GPUHashTable(backend.hash_capacity(n), device="cuda")
        ref.insert_bxyz(coords)
        want = ref.query_subm_bxyz(coords, t3(ks))
        assert torch.equal(omap, want), (n, ks)
        # slots may differ only where two keys raced for one; the key -> value relation may not
        assert torch.equal(torch.sort(table.keys)[0], torch.sort(ref.keys)[0])
        looked = table.query_bxyz(coords, (1, 1, 1), (1, 1, 1), (0, 0, 0))
        assert torch.equal(looked[:n, 0], torch.arange(n, dtype=torch.int32, device="cuda"))
        if n:
            np.testing.assert_array_equal(omap.cpu().numpy(), oracle.kmap_subm(coords.cpu().numpy(), t3(ks)))


@pytest.mark.parametrize("side", [True, False])
def test_chain_started_at_the_submanifold_build(side):
    """The strided chain's first half queued when the submanifold map of the same rows is built
    (what a U-Net's stem does), on a second stream of the device or on the caller's: same
    coordinates and maps as without, a look-ahead nobody asks for leaves no marks behind, and other
    rows or another geometry in between do not take it."""
    keep_side = backend.downsample_side_stream
    backend.downsample_side_stream = side
    try:
        _chain_started_at_the_submanifold_build(side)
    finally:
        backend.downsample_side_stream = keep_side


def _chain_started_at_the_submanifold_build(side):
    rng = np.random.default_rng(21)
    rows = lidar_like_coords(rng, 30000)
    rows = rows[np.lexsort((rows[:, 3], rows[:, 2], rows[:, 1], rows[:, 0]))]
    want = []
    level = rows
    for _ in range(3):
        m, level = oracle.kmap_downsample(level, 2, 2, 0)
        want.append((m, level))
    backend.release_scratch()

    def forward(coords, strided=3, geom=(2, 2, 0)):
        F.build_kernel_map(coords, coords.shape[0], 3, 1, 1, mode="hashmap_on_the_fly")
        got, level = [], coords
        for _ in range(strided):
            km = F.build_kernel_map(level, level.shape[0], geom[0], geom[1], geom[2], mode="hashmap_on_the_fly")
            got.append(km)
            level = km["coords"]
        return got

    coords = dev(rows)
    for _ in range(4):
        got = forward(coords)
        for km, (m, c) in zip(got, want):
            np.testing.assert_array_equal(km["coords"].cpu().numpy(), c)
            np.testing.assert_array_equal(km["out_in_map"].cpu().numpy(), m)
    state, = backend._stream_states.values()
    assert state.lookahead_hits == 2 and state.pending is None  # forwards three and four
    assert (state.side is not None) == side
    # the maps over the chain's levels (here the strided ones) that a forward asked for are queued
    # on the second stream by the next forward that emits its rows there: forwards three and four
    assert state.maps_ahead_hits == (6 if side else 0)
    assert [r[:2] for r in state.map_plan if r[:2] != (0, 0)] == [(0, 1), (1, 2), (2, 3)]
    # a forward that stops after the stem leaves a look-ahead behind; the next strided call of
    # other rows must not take it, and must find clean bitmaps
    F.build_kernel_map(coords, coords.shape[0], 3, 1, 1, mode="hashmap_on_the_fly")
    assert state.pending is not None
    other = rows[: len(rows) // 2].copy()
    other[:, 1] += 3
    km = F.build_kernel_map(dev(other), len(other), 2, 2, 0, mode="hashmap_on_the_fly")
    m, c = oracle.kmap_downsample(other, 2, 2, 0)
    np.testing.assert_array_equal(km["coords"].cpu().numpy(), c)
    np.testing.assert_array_equal(km["out_in_map"].cpu().numpy(), m)
    assert state.pending is None
    # the same rows with another geometry: the look-ahead is for k2 s2 and is dropped
    F.build_kernel_map(coords, coords.shape[0], 3, 1, 1, mode="hashmap_on_the_fly")
    km = F.build_kernel_map(coords, coords.shape[0], 3, 2, 1, mode="hashmap_on_the_fly")
    m, c = oracle.kmap_downsample(rows, 3, 2, 1)
    np.testing.assert_array_equal(km["coords"].cpu().numpy(), c)
    np.testing.assert_array_equal(km["out_in_map"].cpu().numpy(), m)
    # a network without that chain (submanifold maps of fresh rows, no strided call, or a strided
    # call bounded by a spatial range) stops the queueing ahead after one miss
    forward(coords)
    assert state.root_chain is not None
    F.build_kernel_map(coords, coords.shape[0], 3, 1, 1, mode="hashmap_on_the_fly")
    assert state.pending is not None
    fresh = dev(rows)
    F.build_kernel_map(fresh, fresh.shape[0], 3, 1, 1, mode="hashmap_on_the_fly")
    assert state.pending is None and state.root_chain is None
    F.build_kernel_map(dev(rows), len(rows), 3, 1, 1, mode="hashmap_on_the_fly")
    assert state.pending is None
    forward(coords)
    assert state.root_chain is not None  # learnt again from the strided call over the caller's rows
    bounded = dev(rows)
    F.build_kernel_map(bounded, len(rows), 3, 1, 1, mode="hashmap_on_the_fly")
    extent = tuple(int(v) + 1 for v in rows[:, 1:].max(0))
    km = F.build_kernel_map(bounded, len(rows), 2, 2, 0, mode="hashmap_on_the_fly",
                            spatial_range=(int(rows[:, 0].max()) + 1,) + extent)
    strided = (int(rows[:, 0].max()) + 1,) + tuple((e - 2) // 2 + 1 for e in extent)
    m, c = oracle.kmap_downsample(rows, 2, 2, 0, spatial_range=strided)
    np.testing.assert_array_equal(km["coords"].cpu().numpy(), c)
    np.testing.assert_array_equal(km["out_in_map"].cpu().numpy(), m)
    assert state.pending is None and state.root_chain is None
    forward(coords)
    # and switched off, nothing is queued early
    backend.downsample_lookahead_at_subm = False
    try:
        forward(coords)
        assert state.pending is None
        hits = state.lookahead_hits
        forward(coords)
        assert state.lookahead_hits == hits
    finally:
        backend.downsample_lookahead_at_subm = True
    assert not any(st.grid_dirty for st in backend._stream_states.values())


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_maps_queued_ahead_match_the_oracle(seed):
    """Chains of kernel size = stride layers with a submanifold map per level, passed five times
    (a new coordinate tensor on every other pass): from the third pass on the maps over the
    chain's levels are built ahead on the second stream; every map of every pass equals the
    oracle's, whatever the stride, the submanifold kernel of a level or the depth of the chain."""
    rng = np.random.default_rng(400 + seed)
    st = t3([(2, 2, 2), (2, 1, 2), (3, 3, 2), (2, 3, 2)][seed])
    n = [3000, 30000, 60000, 500][seed]
    ext = [(40, 100, 40), (100, 100, 40), (400, 40, 100), (40, 40, 40)][seed]
    batch = 1 + seed % 2
    cols = [rng.integers(0, batch, n)] + [rng.integers(0, e, n) for e in ext]
    coords = np.unique(np.stack(cols, 1).astype(np.int32), axis=0)  # ascending rows
    depth = [2, 3, 2, 3][seed]
    sub_k = [t3(k) for k in [(3, 3, 3), (3, 1, 3), (1, 3, 3), (3, 3, 3)]][:depth + 1]
    want, want_sub, c = [], [oracle.kmap_subm(coords, sub_k[0])], coords
    for d in range(depth):
        m, c2 = oracle.kmap_downsample(c, st, st, 0)
        assert len(c2) > 0
        want.append((m, c2))
        want_sub.append(oracle.kmap_subm(c2, sub_k[d + 1]))
        c = c2
    backend.release_scratch()
    x = None
    for rep in range(5):
        x = dev(coords) if rep % 2 == 0 else x
        km = F.build_kernel_map(x, x.shape[0], sub_k[0], 1, 1, mode="hashmap_on_the_fly")
        np.testing.assert_array_equal(km["out_in_map"].cpu().numpy(), want_sub[0])
        lvl = x
        for d, (m, c2) in enumerate(want):
            km = F.build_kernel_map(lvl, lvl.shape[0], st, st, 0, mode="hashmap_on_the_fly")
            np.testing.assert_array_equal(km["coords"].cpu().numpy(), c2)
            np.testing.assert_array_equal(km["out_in_map"].cpu().numpy(), m)
            lvl = km["coords"]
            ks = sub_k[d + 1]
            km = F.build_kernel_map(lvl, lvl.shape[0], ks, 1, tuple((k - 1) // 2 for k in ks),
                                    mode="hashmap_on_the_fly")
            np.testing.assert_array_equal(km["out_in_map"].cpu().numpy(), want_sub[d + 1])
    state, = backend._stream_states.values()
    assert state.maps_ahead_hits >= 2 * depth  # at least one pass took its maps from the queue


def _chain_cases():
    rng = np.random.default_rng(321)
    scan = lidar_like_coords(rng, 30000)
    # a cloud whose largest coordinates are lone rows: the row with the largest x has an even y
    # at the largest y (the layer's rule leaves its output out), so the maxima of the next level
    # come from other rows than the maxima of this one; the same again one level further down
    cloud = random_coords(rng, 3000, (200, 180, 40), 1)
    lone = np.array([[0, 260, 250, 17], [0, 259, 3, 77], [0, 4, 249, 76], [0, 258, 7, 2], [0, 131, 125, 39]], np.int32)
    spiky = np.concatenate([cloud, lone])
    # ... and one whose largest row is alone far out: the next level's largest x is not half of it
    gap = np.concatenate([random_coords(rng, 3000, (198, 180, 40), 1), np.array([[0, 260, 250, 17]], np.int32)])
    batches = random_coords(rng, 5000, (60, 50, 30), 3)
    few = np.array([[0, 1, 1, 0], [0, 0, 1, 1], [0, 1, 0, 0]], np.int32)  # gone after two layers
    below = np.concatenate([random_coords(rng, 500, (40, 40, 20), 1), np.array([[0, -3, 5, 5], [0, 7, -1, 2]], np.int32)])
    return [("scan", scan, 2, 4), ("spiky", spiky, 2, 4), ("gap", gap, 2, 4), ("batches", batches, 2, 3),
            ("threes", scan, 3, 3),
            ("flat", spiky, (2, 2, 1), 4), ("few", few, 2, 4), ("one", few[:1], 2, 2), ("below", below, 2, 3),
            ("shuffled", scan[rng.permutation(len(scan))], 2, 4)]


@pytest.mark.parametrize("name,coords,ks,levels", _chain_cases(), ids=[c[0] for c in _chain_cases()])
def test_chain_of_strided_levels_from_the_root_rows(name, coords, ks, levels):
    """tsmi_downsample_chain_rows marks every level from the chain's root: the rows of each level
    equal the oracle's strided layer applied to the level before (whose outputs and extents
    follow from the largest coordinates of ITS inputs), the counters hold the counts and those
    maxima, the bitmaps are clear again; in one call and in the two phases a caller puts its copy
    of the counters between."""
    import ctypes
    ks = t3(ks)
    want, c = [], coords
    while len(want) < levels and len(c):
        c = oracle.kmap_downsample(c, ks, ks, 0)[1]
        want.append(c)
    n = len(coords)
    words = max(1 << 15, (1 << (n * 2048 - 1).bit_length()) // 32)
    layout, total = backend._grid_layout(words)
    arrays = backend._layout_arrays(layout)
    g = (backend._i3(ks), backend._i3(ks), backend._i3((0, 0, 0)))
    root = dev(coords)
    for phases in ((0,), (1, 2)):
        scratch = torch.zeros(total, dtype=torch.int32, device="cuda")
        ctr = torch.zeros(8 * levels, dtype=torch.int32, device="cuda")
        rows = torch.full((levels, n, 4), -7, dtype=torch.int32, device="cuda")
        for phase in phases:
            status = backend._C.tsmi_downsample_chain_rows(backend._stream(), root.data_ptr(), n, *g, levels,
                                                           scratch.data_ptr(), *arrays, ctr.data_ptr(),
                                                           rows.data_ptr(), phase)
            assert status == 0, backend._C.tsmi_last_error()
            if phase == 1:
                counts_first = ctr.cpu().numpy().copy()
        host, got = ctr.cpu().numpy().reshape(levels, 8), rows.cpu().numpy()
        if phases == (1, 2):
            np.testing.assert_array_equal(counts_first, host.reshape(-1))  # complete before the rows
        assert not any(scratch[at:at + w].any() for at, w, _ in layout[:levels])  # (the chunk counts stay)
        inputs = coords
        for level in range(levels):
            out = want[level] if level < len(want) else np.zeros((0, 4), np.int32)
            assert host[level, 0] == len(out), (name, level)
            assert host[level, 2] == 0 and host[level, 3] == 0
            np.testing.assert_array_equal(got[level, :len(out)], out)
            assert (got[level, len(out):] == -7).all()
            if len(inputs):
                np.testing.assert_array_equal(host[level, 4:], np.maximum(inputs.max(0), 0))
            inputs = out
