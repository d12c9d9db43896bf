"""Kernel maps searched over sorted coordinates (tsmi_kmap_sorted: no hash table) against the
CPU oracle, bit-exact, and against the hash-table builders on the same rows.  Inputs ascend
strictly in (b, x, y, z), which is what voxelisation by a ravelled key produces and what selects
this path in build_kernel_map."""
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


def dev(a, dtype=torch.int32):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", dtype)


def t3(v):
    return (v,) * 3 if isinstance(v, int) else tuple(v)


def ascending(coords):
    """Rows in ascending (b, x, y, z) order."""
    return coords[np.lexsort((coords[:, 3], coords[:, 2], coords[:, 1], coords[:, 0]))]


def build(coords, ks, stride, pad, **kw):
    kmap = F.build_kernel_map(dev(coords), len(coords), t3(ks), t3(stride), t3(pad), mode="hashmap_on_the_fly", **kw)
    assert kmap["in_hashmap"] is None  # searched: no table over the inputs
    return kmap


@pytest.mark.parametrize("ks", [3, 2, 5, (3, 1, 1), (1, 3, 1), (2, 3, 3), (3, 5, 3), (1, 1, 1), (5, 7, 2)])
@pytest.mark.parametrize("batch", [1, 3])
def test_subm_map_over_sorted_rows_matches_oracle(ks, batch):
    rng = np.random.default_rng(200)
    coords = ascending(random_coords(rng, 900, (14, 12, 10), batch))
    kmap = build(coords, ks, 1, 0)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), oracle.kmap_subm(coords, t3(ks)))
    assert kmap["sizes"] == (len(coords), len(coords)) and kmap["out_in_map"].shape[0] % 128 == 0


DOWN_CASES = [(2, 2, 0), (3, 2, 1), (3, 3, 1), (5, 2, 2), (5, 3, 2), (2, 3, 0), (3, 2, 0),
              ((3, 1, 1), (2, 1, 1), (0, 0, 0)), ((3, 3, 3), (2, 2, 2), (0, 1, 1)),
              ((1, 3, 1), (1, 2, 1), 0), ((4, 2, 6), (2, 2, 3), (1, 0, 2))]


@pytest.mark.parametrize("ks,stride,pad", DOWN_CASES)
@pytest.mark.parametrize("with_range", [False, True])
@pytest.mark.parametrize("through_grid", [True, False])
def test_strided_map_over_sorted_rows_matches_oracle(ks, stride, pad, with_range, through_grid, monkeypatch):
    monkeypatch.setattr(backend, "downsample_through_grid", through_grid)
    rng = np.random.default_rng(201)
    shape = (19, 17, 13)
    coords = ascending(random_coords(rng, 700, shape, batch=2))
    ks, stride, pad = t3(ks), t3(stride), t3(pad)
    sr = (2,) + shape if with_range else None
    kmap = build(coords, ks, stride, pad, spatial_range=sr)
    new_sr = None
    if with_range:
        new_sr = (2,) + tuple((shape[a] + 2 * pad[a] - (ks[a] - 1) - 1) // stride[a] + 1 for a in range(3))
    want_map, want_coords = oracle.kmap_downsample(coords, ks, stride, pad, spatial_range=new_sr)
    np.testing.assert_array_equal(kmap["coords"].cpu().numpy(), want_coords)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want_map)


def test_unsorted_or_repeated_rows_take_the_tables():
    rng = np.random.default_rng(202)
    coords = ascending(random_coords(rng, 500, (10, 10, 10)))
    swapped = coords.copy()
    swapped[[100, 101]] = swapped[[101, 100]]
    repeated = np.concatenate([coords[:200], coords[199:]])
    for rows in (swapped, repeated):
        t = dev(rows)
        assert not backend.coords_ascending(t)
        kmap = F.build_kernel_map(t, len(rows), 3, 1, 0, mode="hashmap_on_the_fly")
        assert kmap["in_hashmap"] is not None
    assert backend.coords_ascending(dev(coords))
    assert backend.coords_ascending(dev(coords[:1])) and backend.coords_ascending(dev(coords[:0]))


def test_rows_declared_ready_are_checked_on_the_second_stream(monkeypatch):
    """rows_ready(): the check of such rows is queued on the device's second stream and the host
    waits for that stream alone (on a device whose hardware queues are not shared between the two
    streams the verdict does not wait for what the caller's stream has queued): ascending rows
    take the table-free builder from their first map on, unsorted rows the tables, a row outside
    the packed range raises from the call that looks at the tensor first."""
    rng = np.random.default_rng(303)
    coords = ascending(random_coords(rng, 3000, (30, 30, 12)))
    seen = []
    real = backend._C.tsmi_coords_check
    main = backend._stream()

    class Spy:  # (the library object, with the one entry point watched)
        def __getattr__(self, name):
            return getattr(real_lib, name)

        def tsmi_coords_check(self, stream, *args):
            seen.append(stream)
            return real(stream, *args)
    real_lib = backend._C
    monkeypatch.setattr(backend, "_C", Spy())
    t = backend.rows_ready(dev(coords))
    assert backend.coords_ascending(t)
    state = backend._stream_states[(torch.cuda.current_device(), main)]
    assert seen == [state.side.cuda_stream] and seen[0] != main
    assert backend._stream() == main
    kmap = F.build_kernel_map(t, len(coords), 3, 1, 0, mode="hashmap_on_the_fly")
    assert kmap["in_hashmap"] is None  # (the table-free builder)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), oracle.kmap_subm(coords, 3))
    swapped = coords.copy()
    swapped[[100, 101]] = swapped[[101, 100]]
    u = backend.rows_ready(dev(swapped))
    assert not backend.coords_ascending(u)
    kmap = F.build_kernel_map(u, len(swapped), 3, 1, 0, mode="hashmap_on_the_fly")
    assert kmap["in_hashmap"] is not None
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), oracle.kmap_subm(swapped, 3))
    far = coords.copy()
    far[-1, 2] = 1 << 20  # beyond the 18 bits a packed key holds per axis
    v = backend.rows_ready(dev(far))
    with pytest.raises(ValueError, match="range"):
        backend.coords_ascending(v)
    assert not backend._pending_verdicts


def test_rows_declared_ready_are_checked_without_waiting_for_the_verdict(monkeypatch):
    """coords_check_aside off: the check of rows_ready() rows is queued on the caller's stream and
    nobody waits for it.  The first map over such a tensor is built through the tables (the verdict of
    the ordering check is still on its way), equals the oracle's, and later maps take the
    table-free builder once the verdict has been picked up; unsorted rows keep the tables; a row
    outside the packed range raises at the latest when settle_checks() is called."""
    monkeypatch.setattr(backend, "coords_check_aside", False)
    rng = np.random.default_rng(303)
    coords = ascending(random_coords(rng, 3000, (30, 30, 12)))
    t = backend.rows_ready(dev(coords))
    assert backend._declared_ready(t)
    assert not backend.coords_ascending(t)  # the verdict has not been read
    kmap = F.build_kernel_map(t, len(coords), 3, 1, 0, mode="hashmap_on_the_fly")
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), oracle.kmap_subm(coords, 3))
    backend.settle_checks()
    assert not backend._pending_verdicts and backend.coords_ascending(t)
    kmap = F.build_kernel_map(t, len(coords), 3, 2, 1, mode="hashmap_on_the_fly")
    assert kmap["in_hashmap"] is None  # (the table-free builder)
    want_map, want_coords = oracle.kmap_downsample(coords, 3, 2, 1)
    np.testing.assert_array_equal(kmap["coords"].cpu().numpy(), want_coords)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want_map)

    swapped = coords.copy()
    swapped[[100, 101]] = swapped[[101, 100]]
    u = backend.rows_ready(dev(swapped))
    assert not backend.coords_ascending(u)
    backend.settle_checks()
    assert not backend.coords_ascending(u)
    kmap = F.build_kernel_map(u, len(swapped), 3, 1, 0, mode="hashmap_on_the_fly")
    assert kmap["in_hashmap"] is not None
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), oracle.kmap_subm(swapped, 3))

    # written in place afterwards: the declaration no longer holds
    t.add_(0)
    assert not backend._declared_ready(t)

    far = coords.copy()
    far[-1, 2] = 1 << 20  # beyond the 18 bits a packed key holds per axis
    v = backend.rows_ready(dev(far))
    backend.coords_ascending(v)
    with pytest.raises(ValueError, match="range"):
        backend.settle_checks()
    assert not backend._pending_verdicts
    backend.settle_checks()  # raised once


def test_segments_longer_than_the_staging_area_are_searched_in_memory():
    """A thin slab next to a dense one: the block that holds the thin slab's rows needs the
    whole dense slab as its segment for the x-digit that points there."""
    ys, zs = np.meshgrid(np.arange(120), np.arange(60), indexing="ij")
    dense = np.stack([np.zeros(ys.size), np.full(ys.size, 5), ys.ravel(), zs.ravel()], 1)
    thin_y = np.arange(0, 120, 3)
    thin = np.stack([np.zeros(thin_y.size), np.full(thin_y.size, 4), thin_y, np.full(thin_y.size, 7)], 1)
    far = np.stack([np.zeros(50), np.full(50, 9), np.arange(50), np.arange(50)], 1)
    coords = ascending(np.concatenate([thin, dense, far]).astype(np.int32))
    kmap = build(coords, 3, 1, 0)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), oracle.kmap_subm(coords, 3))
    kmap = build(coords, (3, 3, 3), (1, 2, 2), (1, 1, 1))
    want_map, want_coords = oracle.kmap_downsample(coords, (3, 3, 3), (1, 2, 2), (1, 1, 1))
    np.testing.assert_array_equal(kmap["coords"].cpu().numpy(), want_coords)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want_map)


@pytest.mark.parametrize("n,extent", [(1, (3, 3, 3)), (2, (2, 2, 2)), (255, (9, 9, 9)), (256, (9, 9, 9)),
                                      (257, (9, 9, 9)), (70000, (300, 300, 12)), (300000, (900, 900, 30))])
def test_sizes_around_the_sampling_levels(n, extent):
    """One and two sampling levels (more than 65536 rows: second-level samples every other row
    and beyond), tiny inputs, sizes around one block."""
    rng = np.random.default_rng(n)
    coords = ascending(random_coords(rng, n, extent))
    kmap = build(coords, 3, 1, 0)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), oracle.kmap_subm(coords, 3))
    kmap = build(coords, 2, 2, 0)
    want_map, want_coords = oracle.kmap_downsample(coords, 2, 2, 0)
    np.testing.assert_array_equal(kmap["coords"].cpu().numpy(), want_coords)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want_map)


def test_sorted_search_equals_the_table_builders_on_random_geometries():
    """Per-axis kernel, stride and padding drawn at random; the searched map against the
    hash-table map of the same rows (itself pinned by the oracle elsewhere)."""
    rng = np.random.default_rng(203)
    for case in range(40):
        ks = tuple(int(v) for v in rng.integers(1, 5, 3))
        st = tuple(int(v) for v in rng.integers(1, 4, 3))
        pd = tuple(int(v) for v in rng.integers(0, 3, 3))
        n = int(rng.integers(1, 6000))
        extent = tuple(int(v) for v in rng.integers(3, 60, 3))
        n = min(n, int(np.prod(extent)))
        coords = ascending(random_coords(rng, n, extent, batch=int(rng.integers(1, 3))))
        if case % 2:
            coords[:, 1:] -= np.array(extent) // 2  # negative coordinates: the biased key keeps the order
        ins = dev(coords)
        outs = dev(ascending(random_coords(rng, max(n // 2, 1), extent)))
        table = backend.GPUHashTable(backend.hash_capacity(len(coords)), device="cuda")
        table.insert_bxyz(ins)
        want = table.query_bxyz(outs, ks, st, pd)
        got = backend.kmap_sorted(ins, outs, ks, st, pd)
        assert torch.equal(got, want), (case, ks, st, pd, n, extent)


def test_negative_coordinates_and_the_edge_of_the_packed_range():
    import torchsparse_amd as ts
    rng = np.random.default_rng(204)
    base = random_coords(rng, 600, (11, 11, 11))
    lo = base.copy()
    lo[:, 1:] -= 131072
    lo = ascending(lo)
    kmap = build(lo, 3, 1, 0)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(),
                                  oracle.kmap_subm(lo, 3, coords_min=lo.min(0), coords_max=lo.max(0)))
    hi = base.copy()
    hi[:, 1:] += 131072 - 11
    hi[:, 0] = 511
    hi = ascending(hi)
    kmap = build(hi, 3, 1, 0)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), oracle.kmap_subm(hi, 3))
    kmap = build(hi, 2, 2, 0)
    want_map, want_coords = oracle.kmap_downsample(hi, 2, 2, 0)
    np.testing.assert_array_equal(kmap["coords"].cpu().numpy(), want_coords)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want_map)
    mid = base.copy()
    mid[:, 1:] -= 5
    mid = ascending(mid)
    ts.set_allow_negative_coordinates(True)
    try:
        kmap = build(mid, 3, 2, 1)
        want_map, want_coords = oracle.kmap_downsample(mid, 3, 2, 1, allow_negative=True)
    finally:
        ts.set_allow_negative_coordinates(False)
    np.testing.assert_array_equal(kmap["coords"].cpu().numpy(), want_coords)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want_map)


@pytest.mark.parametrize("edge", ["low", "high"])
def test_blocks_that_start_inside_a_plane_at_the_edge_of_the_packed_range(edge):
    """Runs of 300 rows per (x, y) line, lines at the first (last) packable x and y: the blocks of
    256 rows start and end inside the edge lines, where the targets one step outside clamp.  The
    bounds of a block's segment must still hold the neighbours of its rows in the next line."""
    xs = np.arange(2) + (-131072 if edge == "low" else 131070)
    ys = np.arange(3) + (-131072 if edge == "low" else 131069)
    zs = np.arange(300) + (-131072 if edge == "low" else 131072 - 300)
    x, y, z = np.meshgrid(xs, ys, zs, indexing="ij")
    coords = np.stack([np.zeros(x.size), x.ravel(), y.ravel(), z.ravel()], 1).astype(np.int32)
    rng = np.random.default_rng(7)
    coords = ascending(coords[rng.random(len(coords)) < 0.9])  # (a few holes: not every target exists)
    lo, hi = coords.min(0), coords.max(0)
    for ks in (3, (3, 5, 3), (5, 3, 3)):
        kmap = build(coords, ks, 1, 0)
        want = oracle.kmap_subm(coords, ks, coords_min=lo, coords_max=hi)
        np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want)
        assert (want[:len(coords)] >= 0).mean() > 0.2
    if edge == "high":
        for ks, st, pd in ((3, 2, 1), (2, 2, 0), ((3, 3, 3), (1, 2, 2), (1, 1, 1))):
            kmap = build(coords, ks, st, pd)
            want_map, want_coords = oracle.kmap_downsample(coords, ks, st, pd)
            np.testing.assert_array_equal(kmap["coords"].cpu().numpy(), want_coords)
            np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want_map)


def test_scan_like_surface_and_switch():
    rng = np.random.default_rng(205)
    coords = ascending(lidar_like_coords(rng, 60000))
    kmap = build(coords, 3, 1, 0)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), oracle.kmap_subm(coords, 3))
    backend.kmap_through_sorted = False
    try:
        hashed = F.build_kernel_map(dev(coords), len(coords), 3, 1, 0, mode="hashmap_on_the_fly")
    finally:
        backend.kmap_through_sorted = True
    assert hashed["in_hashmap"] is not None
    assert torch.equal(hashed["out_in_map"], kmap["out_in_map"])


def test_batch_of_maps_in_one_call_with_transposed_maps_and_pair_counts():
    """tsmi_kmap_sorted_batch over the levels of a strided chain: submanifold 3^3 maps and 2^3
    stride-2 maps in one launch, a (3, 1, 1) map beside them in its own; every map bit for bit
    the oracle's, the transposed maps whose entries the same launch stores (into buffers filled
    with -1) equal to the oracle's transposition, the pair counts equal to the number of entries >= 0, and
    the two words the blocks add up in zero again (the call is repeated over them)."""
    import ctypes
    rng = np.random.default_rng(404)
    c1 = ascending(lidar_like_coords(rng, 30000))
    d1, c2 = oracle.kmap_downsample(c1, 2, 2, 0)
    d2, c3 = oracle.kmap_downsample(c2, 2, 2, 0)
    t1, t2, t3 = dev(c1), dev(c2), dev(c3)
    jobs = [  # (inputs, outputs, ks, st, pd, transposed?, oracle map)
        (t1, t1, (3, 3, 3), (1, 1, 1), (1, 1, 1), True, oracle.kmap_subm(c1, 3)),
        (t1, t2, (2, 2, 2), (2, 2, 2), (0, 0, 0), True, d1),
        (t2, t2, (3, 3, 3), (1, 1, 1), (1, 1, 1), False, oracle.kmap_subm(c2, 3)),
        (t2, t2, (3, 1, 1), (1, 1, 1), (1, 0, 0), False, oracle.kmap_subm(c2, (3, 1, 1))),
        (t2, t3, (2, 2, 2), (2, 2, 2), (0, 0, 0), True, d2),
        (t3, t3, (3, 3, 3), (1, 1, 1), (1, 1, 1), False, oracle.kmap_subm(c3, 3)),
    ]
    words = torch.zeros(3 * len(jobs), dtype=torch.int64, device="cuda")
    for attempt in range(2):
        flat, outs = [], []
        for slot, (a, b, ks, st, pd, tr, want) in enumerate(jobs):
            kvol = ks[0] * ks[1] * ks[2]
            n_pad = -(-b.shape[0] // 128) * 128
            t_pad = -(-a.shape[0] // 128) * 128
            omap = torch.full((n_pad, kvol), -9, dtype=torch.int32, device="cuda")
            omap_t = torch.full((t_pad, kvol), -1, dtype=torch.int32, device="cuda") if tr else None
            flat += [a.data_ptr(), a.shape[0], b.data_ptr(), b.shape[0], n_pad, 0, omap.data_ptr(), *ks, *st, *pd,
                     omap_t.data_ptr() if tr else 0, t_pad, words.data_ptr() + 16 * slot,
                     words.data_ptr() + 8 * (2 * len(jobs) + slot), 0, 0]
            outs.append((omap, omap_t))
        status = backend._C.tsmi_kmap_sorted_batch(backend._stream(), len(jobs), (ctypes.c_int64 * len(flat))(*flat))
        assert status == 0, backend._C.tsmi_last_error()
        torch.cuda.synchronize()
        host = words.cpu().numpy()
        assert (host[:2 * len(jobs)] == 0).all()
        for slot, ((a, b, ks, st, pd, tr, want), (omap, omap_t)) in enumerate(zip(jobs, outs)):
            np.testing.assert_array_equal(omap.cpu().numpy(), want)
            assert host[2 * len(jobs) + slot] == (want >= 0).sum()
            if tr:
                n_in = a.shape[0]
                want_t = oracle.transpose_map(want, n_in)
                got_t = omap_t.cpu().numpy()
                np.testing.assert_array_equal(got_t[:n_in], want_t[:n_in])
                assert (got_t[n_in:] == -1).all()
    # a transposed map with fewer rows than there are inputs is refused
    bad = list(flat[22:44])
    bad[17] = jobs[1][0].shape[0] - 1
    status = backend._C.tsmi_kmap_sorted_batch(backend._stream(), 1, (ctypes.c_int64 * 22)(*bad))
    assert status != 0 and b"transposed" in backend._C.tsmi_last_error()


@pytest.mark.parametrize("rows", [30000, 700, 0])
def test_batch_of_maps_whose_row_counts_are_on_the_device(rows):
    """tsmi_kmap_sorted_batch with the counts of the levels left on the device: the call gets only
    a bound (the root's rows) for every level, buffers sized by it, and pointers to the counts.
    The rows of each map up to ceil128 of its real count equal the oracle's map, rows beyond stay
    untouched, transposed maps and pair counts are those of the real counts; a level without rows
    (count 0 on the device) writes nothing and counts no pairs."""
    import ctypes
    rng = np.random.default_rng(405)
    c1 = ascending(lidar_like_coords(rng, 30000))
    d1, c2 = oracle.kmap_downsample(c1, 2, 2, 0)
    d2, c3 = oracle.kmap_downsample(c2, 2, 2, 0)
    sub2, sub3 = oracle.kmap_subm(c2, 3), oracle.kmap_subm(c3, 3)
    if rows < 30000:
        # the later levels hold fewer rows than the chain found (down to none): a prefix of the
        # ascending rows keeps its indices, so the maps are the full ones cut to the prefix, with
        # the entries that pointed beyond the inputs' prefix gone
        def cut(full, n_out, n_in):
            m = full[:n_out].copy()
            m[m >= n_in] = -1
            return m
        n2, n3 = rows, min(rows, len(c3)) // 2
        d1, d2 = cut(d1, n2, len(c1)), cut(d2, n3, n2)
        sub2, sub3 = cut(sub2, n2, n2), cut(sub3, n3, n3)
        c2, c3 = c2[:n2], c3[:n3]
    n = c1.shape[0]
    n_pad = -(-n // 128) * 128
    # the levels in one buffer of n rows each (what a chain that emits before the read-back leaves)
    levels = torch.full((2, n, 4), 0x7fffffff, dtype=torch.int32, device="cuda")
    if len(c2):
        levels[0, :len(c2)] = dev(c2)
    if len(c3):
        levels[1, :len(c3)] = dev(c3)
    counts = torch.zeros(16, dtype=torch.int32, device="cuda")
    counts[0], counts[8] = len(c2), len(c3)
    t1 = dev(c1)
    jobs = [  # (input level, output level, ks, st, pd, transposed?, oracle map)
        (0, 1, (2, 2, 2), (2, 2, 2), (0, 0, 0), True, d1),
        (1, 1, (3, 3, 3), (1, 1, 1), (1, 1, 1), False, sub2),
        (1, 2, (2, 2, 2), (2, 2, 2), (0, 0, 0), True, d2),
        (2, 2, (3, 3, 3), (1, 1, 1), (1, 1, 1), True, sub3),
    ]
    real = [n, len(c2), len(c3)]
    rows_ptr = lambda l: t1.data_ptr() if l == 0 else levels.data_ptr() + (l - 1) * n * 16  # noqa: E731
    count_ptr = lambda l: 0 if l == 0 else counts.data_ptr() + 32 * (l - 1)  # noqa: E731
    words = torch.zeros(3 * len(jobs), dtype=torch.int64, device="cuda")
    for attempt in range(2):
        flat, outs = [], []
        for slot, (i, o, ks, st, pd, tr, want) in enumerate(jobs):
            kvol = ks[0] * ks[1] * ks[2]
            omap = torch.full((n_pad, kvol), -9, dtype=torch.int32, device="cuda")
            omap_t = torch.full((n_pad, kvol), -1, dtype=torch.int32, device="cuda") if tr else None
            flat += [rows_ptr(i), n, rows_ptr(o), n, n_pad, 0, omap.data_ptr(), *ks, *st, *pd,
                     omap_t.data_ptr() if tr else 0, n_pad, words.data_ptr() + 16 * slot,
                     words.data_ptr() + 8 * (2 * len(jobs) + slot), count_ptr(i), count_ptr(o)]
            outs.append((omap, omap_t))
        status = backend._C.tsmi_kmap_sorted_batch(backend._stream(), len(jobs), (ctypes.c_int64 * len(flat))(*flat))
        assert status == 0, backend._C.tsmi_last_error()
        torch.cuda.synchronize()
        host = words.cpu().numpy()
        assert (host[:2 * len(jobs)] == 0).all()
        for slot, ((i, o, ks, st, pd, tr, want), (omap, omap_t)) in enumerate(zip(jobs, outs)):
            n_out, n_in = real[o], real[i]
            pad = -(-n_out // 128) * 128
            got = omap.cpu().numpy()
            np.testing.assert_array_equal(got[:n_out], want[:n_out])
            assert (got[n_out:pad] == -1).all() and (got[pad:] == -9).all()
            assert host[2 * len(jobs) + slot] == (want[:n_out] >= 0).sum()
            if tr:
                want_t = (oracle.transpose_map(want[:n_out], n_in) if n_out and n_in
                          else np.full((n_in, got.shape[1]), -1))
                got_t = omap_t.cpu().numpy()
                np.testing.assert_array_equal(got_t[:n_in], want_t[:n_in])
                assert (got_t[n_in:] == -1).all()
    # counts on the device go with inputs small enough to be searched without samples
    big = list(flat[22:44])
    big[1] = 200000
    status = backend._C.tsmi_kmap_sorted_batch(backend._stream(), 1, (ctypes.c_int64 * 22)(*big))
    assert status != 0 and b"samples" in backend._C.tsmi_last_error()


def test_root_map_queued_before_the_verdict_of_a_new_tensor(monkeypatch):
    """The submanifold map over a caller's rows is queued behind the first check of a new tensor,
    before the host has the verdict, once the tensor before on this stream asked for such a map:
    one launch per tensor either way, the oracle's map for ascending rows; rows that do not ascend
    get theirs through the table (the queued search is dropped, and nothing is queued ahead for the
    next tensor); a map nobody asks for ends the queueing as well."""
    rng = np.random.default_rng(77)
    base = ascending(lidar_like_coords(rng, 20000))
    want = oracle.kmap_subm(base, 3)
    launches = []
    real = backend._kmap_sorted_launch
    monkeypatch.setattr(backend, "_kmap_sorted_launch", lambda *a, **k: (launches.append(a[2]), real(*a, **k))[1])
    backend._root_geoms.clear()
    backend._root_maps.clear()

    def build(rows):
        t = dev(rows)
        launches.clear()
        m = F.build_kernel_map(t, len(rows), (3, 3, 3), 1, 0, mode="hashmap_on_the_fly")["out_in_map"]
        return m.cpu().numpy(), len(launches)

    got, n = build(base)  # learns the geometry
    np.testing.assert_array_equal(got, want)
    assert n == 1 and backend._root_geoms and not backend._root_maps
    for _ in range(2):  # queued before the verdict, taken after it
        got, n = build(base)
        np.testing.assert_array_equal(got, want)
        assert n == 1 and not backend._root_maps
    shuffled = base[rng.permutation(len(base))]
    got, n = build(shuffled)
    np.testing.assert_array_equal(got, oracle.kmap_subm(shuffled, 3))
    assert n == 1 and not backend._root_maps and not backend._root_geoms  # (the one launch was the dropped one)
    got, n = build(base)
    np.testing.assert_array_equal(got, want)
    assert n == 1 and backend._root_geoms
    # a new tensor whose map nobody asks for, then another one: nothing queued for it
    t = dev(base)
    launches.clear()
    assert backend.coords_ascending(t) and len(launches) == 1 and len(backend._root_maps) == 1
    t2 = dev(base)
    assert backend.coords_ascending(t2) and len(launches) == 1
    assert not backend._root_maps and not backend._root_geoms
    torch.cuda.synchronize()


def test_root_map_of_rows_known_to_be_complete_is_built_on_the_second_stream(monkeypatch):
    """Once a network's strided chain is queued ahead on the second stream (the rows are known to be
    complete: declared so, or checked before), the submanifold map over the rows themselves is
    launched there too, in front of the chain, and the layer that asks for it takes it from there:
    the oracle's map, one launch per tensor, on the second stream."""
    rng = np.random.default_rng(99)
    base = ascending(lidar_like_coords(rng, 20000))
    want = oracle.kmap_subm(base, 3)
    want_down, level2 = oracle.kmap_downsample(base, 2, 2, 0)
    launches = []
    real = backend._kmap_sorted_launch
    monkeypatch.setattr(backend, "_kmap_sorted_launch",
                        lambda *a, **k: (launches.append((a[0] is a[1], backend._stream())), real(*a, **k))[1])
    backend.release_scratch()
    backend._root_geoms.clear()
    backend._root_maps.clear()
    main = backend._stream()
    for turn in range(5):
        t = backend.rows_ready(dev(base))
        launches.clear()
        subm = F.build_kernel_map(t, len(base), (3, 3, 3), 1, 0, mode="hashmap_on_the_fly")
        down = F.build_kernel_map(t, len(base), (2, 2, 2), 2, 0, mode="hashmap_on_the_fly")
        down2 = F.build_kernel_map(down["coords"], len(level2), (2, 2, 2), 2, 0, mode="hashmap_on_the_fly")
        np.testing.assert_array_equal(subm["out_in_map"].cpu().numpy(), want)
        np.testing.assert_array_equal(down["out_in_map"].cpu().numpy(), want_down)
        np.testing.assert_array_equal(down["coords"].cpu().numpy(), level2)
        assert down2["out_in_map"].shape[1] == 8
        roots = [s for is_root, s in launches if is_root]
        assert len(roots) == 1
        state = backend._stream_states[(torch.cuda.current_device(), main)]
        if state.lookahead_hits:  # the chain of this tensor was queued at its submanifold build
            assert state.side is not None and roots[0] == state.side.cuda_stream
    assert state.lookahead_hits >= 2 and not backend._root_maps
    torch.cuda.synchronize()
