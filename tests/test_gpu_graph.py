"""A forward over cached kernel maps recorded as a HIP graph (utils.graph.GraphedForward):
every replay equals the eager forward of the same features, with eager work and
synchronisations of the program's own between the replays, for the U-Net (pair-segment layers,
offset splits with their shared scratch and counters, transposed layers, concatenations) and for
the detection backbone (a spatial range, batches)."""
import copy

import numpy as np
import pytest
import torch

from helpers import random_coords

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _stat_norms(model):
    for m in model.modules():  # non-trivial norm statistics
        if isinstance(m, torch.nn.BatchNorm1d):
            m.running_mean.normal_(0, 0.3)
            m.running_var.uniform_(0.5, 1.5)
            m.weight.data.uniform_(0.5, 1.5)
            m.bias.data.normal_(0, 0.2)


def _check_replays(ts, model, coords, cin, spatial_range=None, pick=lambda out: out):
    from torchsparse_amd.utils.graph import GraphedForward
    n = coords.shape[0]
    torch.manual_seed(5)
    feats = [torch.randn(n, cin, device="cuda", dtype=torch.float16) for _ in range(4)]
    x = ts.SparseTensor(feats[0], coords, spatial_range=spatial_range)
    runner = GraphedForward(model, x)
    for i in (1, 2, 3, 0, 2):
        got = [t.clone() for t in pick(runner(feats[i]))]
        # the program's own eager work between replays: a fresh tensor, maps rebuilt
        with torch.no_grad():
            want = pick(model(ts.SparseTensor(feats[i], coords.clone(), spatial_range=spatial_range)))
        torch.cuda.synchronize()
        assert len(got) == len(want) > 0
        for g, w in zip(got, want):
            assert g.shape == w.shape and torch.isfinite(w.float()).all()
            assert torch.equal(g, w), (i, float((g.float() - w.float()).abs().max()))
    with pytest.raises(ValueError):
        runner(feats[0][:-1])


def test_unet_replays_equal_eager_forwards():
    import torchsparse_amd as ts
    from torchsparse_amd.backbones import SparseResUNet42
    from torchsparse_amd.nn.utils import fuse_inference
    from torchsparse_amd.utils.synthetic import lidar_scan_voxels
    torch.manual_seed(1)
    coords = dev(lidar_scan_voxels(seed=1)[::3].copy())  # a thinned scan: deep levels over pair segments
    model = SparseResUNet42(in_channels=4).cuda().eval()
    _stat_norms(model)
    model = fuse_inference(copy.deepcopy(model)).half()
    _check_replays(ts, model, coords, 4, pick=lambda out: [o.feats for o in out])


def test_detection_backbone_replays_equal_eager_forwards():
    import torchsparse_amd as ts
    from torchsparse_amd.backbones import VoxelResBackBone8x
    from torchsparse_amd.nn.utils import fuse_inference
    torch.manual_seed(2)
    rng = np.random.default_rng(12)
    coords = random_coords(rng, 9000, (41, 96, 96), batch=2)
    coords = dev(coords[np.lexsort((coords[:, 3], coords[:, 2], coords[:, 1], coords[:, 0]))])
    model = VoxelResBackBone8x(in_channels=5).cuda().eval()
    _stat_norms(model)
    model = fuse_inference(model).half()
    _check_replays(ts, model, coords, 5, spatial_range=(2, 41, 96, 96),
                   pick=lambda out: [v.feats for v in out.values()])


def test_replays_survive_the_eviction_of_every_library_table():
    """After the recording: release_scratch(), 1x1x1 layers over seventeen other row counts (the
    identity-map table keeps sixteen), pair segments of seventy other maps (that table is cleared
    at sixty-four), and eager forwards of a larger input on
    the recording's own stream (its scratch regrown).  The recording keeps the buffers it was
    made over: they are still where they were, and the replay still equals the eager forward."""
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd.backbones import SparseResUNet42
    from torchsparse_amd.nn.utils import fuse_inference
    from torchsparse_amd.utils.graph import GraphedForward
    from torchsparse_amd.utils.synthetic import lidar_scan_voxels
    import oracle
    torch.manual_seed(1)
    scan = lidar_scan_voxels(seed=1)
    coords = dev(scan[::3].copy())
    n = coords.shape[0]
    model = SparseResUNet42(in_channels=4).cuda().eval()
    _stat_norms(model)
    model = fuse_inference(copy.deepcopy(model)).half()
    pick = lambda out: [o.feats for o in out]  # noqa: E731
    feats = [torch.randn(n, 4, device="cuda", dtype=torch.float16) for _ in range(2)]
    runner = GraphedForward(model, ts.SparseTensor(feats[0], coords))
    assert len(runner.pinned) >= 40  # the packed weights of 49 layers, scratch, counters, segments ...
    recorded = [t.data_ptr() for t in runner.pinned]
    sizes = {t.numel() * t.element_size() for t in runner.pinned}
    assert max(sizes) >= 1 << 20  # the stream's scratch is among them
    with torch.no_grad():
        want = [[t.clone() for t in pick(model(ts.SparseTensor(f, coords.clone())))] for f in feats]

    backend.release_scratch()
    w1 = torch.randn(16, 16, device="cuda", dtype=torch.float16)
    for m in range(2000, 2017):
        backend.conv_pointwise_cuda(torch.randn(m, 16, device="cuda", dtype=torch.float16), w1)
    rng = np.random.default_rng(3)
    small = oracle.kmap_subm(random_coords(rng, 200, (8, 8, 8)), 3)
    keep = [dev(small.copy()) for _ in range(70)]
    for m in keep:
        backend.pair_segments(m, 200)
    assert len(backend._segments_of) < 64  # (cleared on the way)
    big = dev(scan)
    fb = torch.randn(big.shape[0], 4, device="cuda", dtype=torch.float16)
    torch.cuda.synchronize()
    with torch.no_grad(), torch.cuda.stream(runner.stream):
        model(ts.SparseTensor(fb, big))
    runner.stream.synchronize()
    junk = [torch.full((1 << 22,), 7, dtype=torch.int32, device="cuda") for _ in range(8)]  # reuse freed blocks
    torch.cuda.synchronize()
    assert [t.data_ptr() for t in runner.pinned] == recorded
    for i in (1, 0, 1):
        got = pick(runner(feats[i]))
        torch.cuda.synchronize()
        for g, w in zip(got, want[i]):
            assert torch.equal(g, w), i
    del junk
    # a moved buffer is refused
    runner.pinned[0].resize_(runner.pinned[0].numel() * 4 + (1 << 24))
    with pytest.raises(RuntimeError, match="moved"):
        runner(feats[0])


def test_convolution_calls_through_the_launch_thread():
    """Inside backend.launch_region() the convolution calls are carried out by the library's launch
    thread: same results bit for bit, in order with the calls this thread makes itself once
    flush_launches() has returned, nothing handed over while hooks are registered or outside a
    region, and a call the library refuses raises at the flush."""
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.backbones import SparseResUNet42
    from torchsparse_amd.nn.utils import fuse_inference
    from torchsparse_amd.utils.synthetic import lidar_scan_voxels
    assert backend.launch_thread
    torch.manual_seed(2)
    coords = dev(lidar_scan_voxels(seed=1)[::2].copy())
    n = coords.shape[0]
    model = SparseResUNet42(in_channels=4).cuda().eval()
    _stat_norms(model)
    model = fuse_inference(copy.deepcopy(model)).half()
    feats = torch.randn(n, 4, device="cuda", dtype=torch.float16)
    done = backend._C.tsmi_launch_thread_completed().contents
    with torch.no_grad():
        before = done.value
        threaded = [o.feats.clone() for o in model(ts.SparseTensor(feats, coords.clone()))]
        handed = done.value - before
        assert handed >= 49 and not backend._region_calls and backend._region_depth == 0
        backend.launch_thread = False
        try:
            before = done.value
            direct = [o.feats.clone() for o in model(ts.SparseTensor(feats, coords.clone()))]
            assert done.value == before
        finally:
            backend.launch_thread = True
        for a, b in zip(threaded, direct):
            assert torch.equal(a, b)
        # layers called one by one inside a region: torch reads a result only after the flush
        layer = spnn.Conv3d(4, 32, 3).cuda().half().eval()
        x = ts.SparseTensor(feats, coords)
        want = layer(x).feats.clone()
        with backend.launch_region():
            for _ in range(20):
                y = layer(x)
            assert backend._region_calls  # (handed over, possibly not launched yet)
            backend.flush_launches()
            assert not backend._region_calls
            assert torch.equal(y.feats, want)
            # a forward hook looks at the result as soon as the layer returns
            seen = []
            handle = layer.register_forward_hook(lambda m, a, out: seen.append(out.feats.clone()))
            from torchsparse_amd.nn.utils.fuse import call_module
            before = done.value
            call_module(layer, x)
            handle.remove()
            assert done.value == before and torch.equal(seen[0], want)
        # a call the library refuses (a null map pointer) surfaces when the region flushes
        with pytest.raises(ValueError, match="null pointer"):
            with backend.launch_region():
                bad = backend._PACK21(backend._stream(), feats.data_ptr(), feats.data_ptr(), 0, n, n, 27, 4, 32, 1,
                                      0, 0, 0, 0, 0, 0, 0, feats.data_ptr(), 0, 0, 0)
                assert backend._hand_over(0, bad, 21, (feats,))
        assert backend._region_depth == 0
        assert backend._C.tsmi_launch_thread_submit(0, bad, 21) == -1  # no region open: nothing is taken
        y = layer(x)
        assert torch.equal(y.feats, want)
