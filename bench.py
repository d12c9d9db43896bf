"""Benchmark of the sparse-convolution forward hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-layers] [--no-backward] [--no-tune] [--no-pointops] [--no-configs]
  python bench.py --summarize DIR     (no GPU: rocprofv3 output -> profiles/)

One step = one MinkUNet (SparseResUNet42 + 19-class linear head) forward in fp16 on a
synthetic 64-beam LiDAR scan (~90k voxels, 4 input channels), starting from a coordinate
tensor the library has not seen (a device copy of the resident scan, queued in the step) and a
fresh SparseTensor: every step pays the first-sight check of the rows and rebuilds its 9 kernel
maps.  Scan, features and weights are resident in HBM before the timed region.  The same loop
over one and the same coordinate tensor, and over new tensors that were complete beforehand and
are declared so (backend.rows_ready), is reported in `config`.  The network runs in inference
form: eval-mode BatchNorm folded into the convolutions, ReLU and shortcut adds in the
convolution epilogues (nn.utils.fuse_inference; same function, checked in the tests);
the unfused module-by-module time is reported beside it.  Prints ONE JSON line.

Also measured (same JSON line):
  layers        the five single layers of the layer sweep on the same scan: kernel-map
                build ms (cold), conv ms (warm map), effective TFLOP/s, kmap GB/s
  roofline      the layer whose kernel takes the largest share of the forward, timed
                alone with HIP events on the launch stream
  cpu_baseline  the CPU oracle (a C restatement of the reference's CPU backend) running
                the network's sparse convolutions and kernel maps on the host cores
  tuned         utils.tune.tune over the three dataflows and the sorted variants, and the
                step time of the tuned network beside the default configuration's
  pointops      the point-voxel operators (hash, query, count, voxelize, devoxelize) on a
                synthetic 1M-point cloud: ms and GB/s of the bytes each has to touch
  backward      input- and weight-gradient kernels of the sweep's submanifold layers, the
                pair-list build the weight gradient needs, one training step of the network
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-layers", action="store_true", help="skip the single-layer sweep")
    ap.add_argument("--no-roofline", action="store_true", help="skip the per-kernel roofline timing")
    ap.add_argument("--no-backward", action="store_true", help="skip the backward (training) figures")
    ap.add_argument("--no-tune", action="store_true", help="skip the per-group tuner run")
    ap.add_argument("--no-pointops", action="store_true", help="skip the point-voxel operator sweep")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the detection-backbone and 1M-voxel figures")
    ap.add_argument("--pmc-target", default=None, metavar="KERNEL",
                    help="run only a 256 MiB device copy (5 launches) and one conv kernel (5 launches) "
                         "for a hardware-counter pass; KERNEL is the description a normal run prints "
                         "in roofline.kernel, or 'auto' for the kernel that run would pick")
    ap.add_argument("--pmc-kernels", action="store_true",
                    help="for a hardware-counter pass over the kernels outside the dominant convolution: "
                         "a 256 MiB device copy (5 launches), then 5 launches each of the kernel-map "
                         "builders (searched and hashed, scan and 1M voxels), the gather and scatter "
                         "kernels (64 channels) and the 1M-voxel 256 -> 256 convolution")
    ap.add_argument("--dense-deep", action="store_true",
                    help="run the small wide layers as a dense pass over the map instead of over pair "
                         "segments (for the counter passes that compare the two forms)")
    ap.add_argument("--summarize", default=None, metavar="DIR",
                    help="no GPU work: turn the rocprofv3 output of the passes listed in "
                         "profiles/*.md (DIR/kt, DIR/pmc_fetch, DIR/pmc_write, DIR/pmc_sq, DIR/bench.json) "
                         "into profiles/*.md and profiles/roofline_traffic.json")
    ap.add_argument("--sorted", type=int, default=-1,
                    help="1: run the implicit GEMM over row-sorted maps (conv_mode 1); 0: unsorted; "
                         "-1: the default of this benchmark")
    return ap.parse_args()


def event_ms(fn, iters=20, warm=3):
    """Average milliseconds of fn() measured with HIP events on the current stream."""
    for _ in range(warm):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def conv_work(n_in, n_out, n_pad, nnz, kvol, cin, cout, elem_bytes):
    """Algorithmic work of one sparse convolution: effective flops and minimum bytes
    (features in, features out, weights, the kernel map)."""
    flops = 2.0 * nnz * cin * cout
    nbytes = elem_bytes * (n_in * cin + n_out * cout + kvol * cin * cout) + 4.0 * n_pad * kvol
    return flops, nbytes


def kmap_bytes_subm(n, n_pad, cap, kvol):
    """Algorithmic bytes of a submanifold map build: coords, table init, inserts, one
    probe per queried neighbour of the half kernel, the map itself."""
    return 16.0 * n + 12.0 * cap + 12.0 * n + 12.0 * (kvol // 2) * n + 4.0 * kvol * n_pad


def kmap_bytes_down(n, n_out, n_out_pad, cap, cand, kvol):
    return (16.0 * n + 16.0 * cand + 12.0 * cap + 12.0 * n_out + 16.0 * n_out + 12.0 * cand
            + 4.0 * kvol * n_out_pad)


# HBM bytes per launch of the roofline kernel from hardware counters (FETCH_SIZE and
# WRITE_SIZE passes of `rocprofv3 --pmc ... -- python bench.py --pmc-target KERNEL`, each scaled
# by what the same counter reads for the 256 MiB copy of that run): `bench.py --summarize DIR`
# writes them, keyed by the kernel description this script prints, into this file next to the
# summaries the figures come from.  No entry for the kernel that dominates: `traffic` is null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "roofline_traffic.json")
MARKER_ELEMS = 31337  # an int16 fill of this many elements brackets the timed loop in a kernel trace


def pmc_traffic_bytes(desc):
    try:
        with open(TRAFFIC_FILE) as f:
            entry = json.load(f).get(desc)
    except (OSError, ValueError):
        return None
    return None if entry is None else int(entry["fetch_bytes"] + entry["write_bytes"])


def roofline_of(flops, nbytes, ms):
    t_f = flops / (MFMA_F16_PEAK_TFLOPS * 1e12)
    t_b = nbytes / (HBM_PEAK_GBS * 1e9)
    if t_f > t_b:
        ach = flops / (ms * 1e-3) / 1e12
        return {"bound": "mfma", "achieved": ach, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": ach / MFMA_F16_PEAK_TFLOPS, "traffic": None}
    ach = nbytes / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": ach / HBM_PEAK_GBS, "traffic": None}


def achievable_peaks():
    """What this GPU sustains on the two textbook kernels, beside the published peaks the
    roofline is priced against: a 1 GiB device-to-device copy (bytes read + written per second)
    and a large fp16 GEMM through torch (hipBLASLt), fp32 accumulation."""
    a = torch.empty(256 * 1024 * 1024, dtype=torch.float32, device="cuda")
    b = torch.empty_like(a)
    t_copy = event_ms(lambda: b.copy_(a), iters=10)
    del a, b
    m = 8192
    x = torch.randn(m, m, device="cuda", dtype=torch.float16)
    y = torch.randn(m, m, device="cuda", dtype=torch.float16)
    t_gemm = event_ms(lambda: torch.matmul(x, y), iters=10)
    return {"device_copy_GBps": round(2 * 1024 ** 3 / (t_copy * 1e-3) / 1e9, 1),
            "gemm_f16_8192_TFLOPs": round(2 * m ** 3 / (t_gemm * 1e-3) / 1e12, 1)}


def layer_sweep(ts, spnn, F, backend, coords_dev, n):
    """The five single layers of the sweep, fp16."""
    out = []
    specs = [("subm_k3_32_32", 32, 32, 3, 1, False), ("subm_k3_64_64", 64, 64, 3, 1, False),
             ("subm_k3_128_128", 128, 128, 3, 1, False), ("down_k2s2_64_128", 64, 128, 2, 2, False),
             ("up_k2s2_128_64", 128, 64, 2, 2, True)]
    for name, cin, cout, k, s, transposed in specs:
        kvol = k ** 3
        if transposed:
            base = ts.SparseTensor(torch.zeros(n, 1, device="cuda", dtype=torch.float16), coords_dev)
            down = spnn.Conv3d(1, cin, k, stride=s).cuda().half()
            mid = down(base)
            x = torch.randn(mid.feats.shape[0], cin, device="cuda", dtype=torch.float16)
            inp = ts.SparseTensor(x, mid.coords, stride=mid.stride)
            inp._caches = mid._caches
        else:
            x = torch.randn(n, cin, device="cuda", dtype=torch.float16)
            inp = ts.SparseTensor(x, coords_dev)
        layer = spnn.Conv3d(cin, cout, k, stride=s, transposed=transposed).cuda().half()

        def build():
            if transposed:
                km = mid._caches.kmaps[((1, 1, 1), (k,) * 3, (s,) * 3, (1, 1, 1))]
                km["out_in_map_t"] = None
                F.transpose_kernel_map(km)
            else:
                F.build_kernel_map(coords_dev, n, k, s, 0 if s > 1 else (k - 1) // 2,
                                   mode="hashmap_on_the_fly")
        kmap_ms = event_ms(build, iters=10)
        y = layer(inp)  # builds and caches the map
        conv_ms = event_ms(lambda: layer(inp), iters=20)
        if transposed:
            km = mid._caches.kmaps[((1, 1, 1), (k,) * 3, (s,) * 3, (1, 1, 1))]
            omap = km["out_in_map_t"]
            n_in, n_out = km["sizes"][1], km["sizes"][0]
        else:
            km = inp._caches.kmaps[((1, 1, 1), (k,) * 3, (s,) * 3, (1, 1, 1))]
            omap = km["out_in_map"]
            n_in, n_out = km["sizes"]
        nnz = int((omap >= 0).sum().item())
        n_pad = omap.shape[0]
        flops, nbytes = conv_work(n_in, n_out, n_pad, nnz, kvol, cin, cout, 2)
        cap = backend.hash_capacity(n)
        if s == 1:
            kbytes = kmap_bytes_subm(n, n_pad, cap, kvol)
        elif transposed:
            kbytes = 4.0 * kvol * (km["out_in_map"].shape[0] + n_pad)  # read one map, write the other
        else:
            kbytes = kmap_bytes_down(n, n_out, n_pad, cap, nnz, kvol)
        row = {"layer": name, "n_in": n_in, "n_out": n_out, "nnz": nnz,
               "kmap_ms": round(kmap_ms, 4), "kmap_GBps": round(kbytes / kmap_ms / 1e6, 1),
               "conv_ms": round(conv_ms, 4),
               "eff_TFLOPs": round(flops / conv_ms / 1e9, 2),
               "min_bytes_GBps": round(nbytes / conv_ms / 1e6, 1)}
        row.update(pair_dataflows(ts, spnn, F, backend, layer, inp, mid if transposed else None,
                                  k, s, transposed, cin, cout, flops))
        out.append(row)
        del y
    return out


def pair_dataflows(ts, spnn, F, backend, layer, inp, mid, k, s, transposed, cin, cout, flops):
    """The same layer through the two pair-list dataflows (warm map products): the whole layer,
    and for gather-scatter its gather and scatter kernels on their own with the bytes they have
    to move — gather: every pair's input row read and written plus its index
    (nnz * (2 * Cin * 2 + 4)); scatter: every product row and its mask entry read, every output
    row written (nnz * (Cout * 2 + 4) + N_out * Cout * 2)."""
    out = {}
    key = ((1, 1, 1), (k,) * 3, (s,) * 3, (1, 1, 1))
    for flow, tag in ((F.Dataflow.GatherScatter, "gather_scatter"), (F.Dataflow.FetchOnDemand, "fetch_on_demand")):
        cfg = F.conv_config.get_default_conv_config()
        cfg.dataflow = flow
        twin = spnn.Conv3d(cin, cout, k, stride=s, transposed=transposed, config=cfg).cuda().half()
        twin.kernel.data.copy_(layer.kernel.data)
        if transposed:
            lower = spnn.Conv3d(1, cin, k, stride=s, config=cfg).cuda().half()
            fine = ts.SparseTensor(torch.zeros(mid._caches.cmaps[(1, 1, 1)][0].shape[0], 1, device="cuda",
                                               dtype=torch.float16), mid._caches.cmaps[(1, 1, 1)][0])
            coarse = lower(fine)  # this dataflow's products of the strided map
            x = ts.SparseTensor(inp.feats, coarse.coords, stride=coarse.stride)
            x._caches = coarse._caches
        else:
            x = ts.SparseTensor(inp.feats, inp.coords)
        with torch.no_grad():
            twin(x)  # builds the pair lists once
            ms = event_ms(lambda: twin(x), iters=20)
        out[tag + "_ms"] = round(ms, 4)
        out[tag + "_eff_TFLOPs"] = round(flops / ms / 1e9, 2)
        if flow == F.Dataflow.GatherScatter:
            km = x._caches.kmaps[key]
            nb = km["nbmaps"]
            nnz = nb.shape[0]
            n_rows_out = km["sizes"][0] if transposed else km["sizes"][1]
            code = 1
            C = backend._C
            st = backend._stream()
            gathered = torch.empty((max(nnz, 1), cin), dtype=torch.float16, device="cuda")
            products = torch.randn((max(nnz, 1), cout), dtype=torch.float16, device="cuda")
            y = torch.empty((n_rows_out, cout), dtype=torch.float16, device="cuda")
            feats = inp.feats
            g_ms = event_ms(lambda: C.tsmi_gs_gather(st, feats.data_ptr(), nb.data_ptr(), nnz, cin, code,
                                                     int(transposed), gathered.data_ptr()), iters=20)
            mask = km["input_mask"] if transposed else km["output_mask"]
            center = k ** 3 // 2 if (s == 1 and k % 2 == 1) else -1
            s_ms = event_ms(lambda: C.tsmi_gs_scatter(st, products.data_ptr(), km["nbaddrs"].data_ptr(),
                                                      mask.data_ptr(), n_rows_out, k ** 3, cout, code, center,
                                                      None, None, 0, y.data_ptr()), iters=20)
            out["gather_ms"] = round(g_ms, 4)
            out["gather_GBps"] = round(nnz * (2 * cin * 2 + 4) / g_ms / 1e6, 1)
            out["scatter_ms"] = round(s_ms, 4)
            out["scatter_GBps"] = round((nnz * (cout * 2 + 4) + n_rows_out * cout * 2) / s_ms / 1e6, 1)
    return out


def backward_sweep(ts, spnn, F, backend, coords_dev, n, feats):
    """Backward of the sweep's submanifold layers on the same scan (fp16, HIP events): input
    gradient (the forward kernel over the transposed map), weight gradient over pair lists,
    the build of those lists; and one training step (forward + backward, batch-norm in
    training mode) of the whole network."""
    from torchsparse_amd.backbones import SparseResUNet42
    km = F.build_kernel_map(coords_dev, n, 3, 1, 1, mode="hashmap_on_the_fly")
    omap = km["out_in_map"]
    nnz = int((omap[:n] >= 0).sum().item())
    map_bwd = backend.convert_transposed_out_in_map(omap, omap.shape[0], n)
    lists = backend.wgrad_pair_lists(omap, n)
    out = {"pair_lists_ms": round(event_ms(lambda: backend.wgrad_pair_lists(omap, n), iters=10), 4),
           "transposed_map_ms": round(event_ms(
               lambda: backend.convert_transposed_out_in_map(omap, omap.shape[0], n), iters=10), 4),
           "layers": []}
    for c in (32, 64, 96, 128):
        x = torch.randn(n, c, device="cuda", dtype=torch.float16)
        dy = torch.randn(n, c, device="cuda", dtype=torch.float16)
        wt = torch.randn(27, c, c, device="cuda", dtype=torch.float16) * 0.05
        dgrad = event_ms(lambda: backend.conv_forward_implicit_gemm_cuda(dy, wt, map_bwd, n, c), iters=20)
        wgrad = event_ms(lambda: backend.conv_backward_wgrad_pairs_cuda(dy, x, lists, 0), iters=20)
        flops = 2.0 * nnz * c * c
        # bytes the weight gradient has to move: every pair's two rows once, the pair list, dW
        wbytes = nnz * (2 * c * 2 + 8) + 27 * c * c * 2
        out["layers"].append({"layer": f"subm_k3_{c}_{c}", "nnz": nnz,
                              "dgrad_ms": round(dgrad, 4), "dgrad_eff_TFLOPs": round(flops / dgrad / 1e9, 2),
                              "wgrad_ms": round(wgrad, 4), "wgrad_eff_TFLOPs": round(flops / wgrad / 1e9, 2),
                              "wgrad_gathered_GBps": round(wbytes / wgrad / 1e6, 1)})
    net = SparseResUNet42(in_channels=4).cuda().half().train()

    def step():
        net.zero_grad(set_to_none=True)
        y = net(ts.SparseTensor(feats, coords_dev))[-1].feats
        y.float().square().mean().backward()
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(10):
        step()
    torch.cuda.synchronize()
    out["train_step_ms"] = round((time.perf_counter() - t0) * 100, 4)
    return out


def other_configs(ts, spnn, F, backend):
    """The two larger configurations of the benchmark set, as single figures: the detection
    backbone (batch 2, merged sweeps, (41, 1440, 1440) grid, 5 input channels, fp16, inference form)
    and one 256 -> 256 submanifold layer on ~1M voxels (sphere shells in 512^3), unsorted and sorted."""
    from torchsparse_amd.backbones import VoxelResBackBone8x
    from torchsparse_amd.nn.utils import fuse_inference
    from torchsparse_amd.utils import synthetic
    out = {}
    coords_np, spatial_range = synthetic.multisweep_voxels(seed=2)
    coords = torch.from_numpy(coords_np).cuda()
    n = coords.shape[0]
    feats = torch.randn(n, 5, device="cuda", dtype=torch.float16)
    torch.manual_seed(1)
    net = fuse_inference(VoxelResBackBone8x(in_channels=5).cuda().half().eval())
    warm = ts.SparseTensor(feats, coords, spatial_range=spatial_range)

    def run(x):
        with torch.no_grad():
            return net(x)
    out["detection_backbone"] = {
        "voxels": n, "batch": 2, "spatial_range": list(spatial_range),
        "ms_maps_rebuilt": round(event_ms(lambda: run(ts.SparseTensor(feats, coords, spatial_range=spatial_range)),
                                          iters=10), 4),
        "ms_maps_cached": round(event_ms(lambda: run(warm), iters=10), 4)}
    from torchsparse_amd.utils.graph import GraphedForward
    runner = GraphedForward(net, warm)
    out["detection_backbone"]["ms_maps_cached_graph_replay"] = round(event_ms(runner, iters=10), 4)
    del runner
    del net, warm, feats, coords
    coords = torch.from_numpy(synthetic.sphere_shell_voxels(seed=3)).cuda()
    n = coords.shape[0]
    t_map = event_ms(lambda: F.build_kernel_map(coords, n, 3, 1, 1, mode="hashmap_on_the_fly"), iters=5)
    t_map_sorted = event_ms(lambda: F.build_kernel_map(coords, n, 3, 1, 1, mode="hashmap_on_the_fly", ifsort=True),
                            iters=5)
    km = F.build_kernel_map(coords, n, 3, 1, 1, mode="hashmap_on_the_fly", ifsort=True)
    nnz = int((km["out_in_map"][:n] >= 0).sum().item())
    x = torch.randn(n, 256, device="cuda", dtype=torch.float16)
    w = torch.randn(27, 256, 256, device="cuda", dtype=torch.float16) * 0.02
    setting, backend.igemm_group_rows = backend.igemm_group_rows, False
    t = event_ms(lambda: backend.conv_forward_implicit_gemm_cuda(x, w, km["out_in_map"], n, 256), iters=5)
    # the same layer over the grouped copy of the map (rows counting-sorted by kernel planes inside
    # windows, tiles heaviest first), and what building that copy takes
    backend.igemm_group_rows = "always"
    omap = km["out_in_map"]

    def regroup():
        backend._grouped_of.pop(id(omap), None)
        backend.grouped_map(omap, n)
    t_group = event_ms(regroup, iters=5)
    t_grouped = event_ms(lambda: backend.conv_forward_implicit_gemm_cuda(x, w, omap, n, 256), iters=5)
    backend.igemm_group_rows = setting
    t_sorted = event_ms(lambda: backend.conv_forward_implicit_gemm_sorted_cuda(
        x, w, km["reorder_out_in_map"], km["reduced_sorted_mask"], km["reorder_loc"], n, 256), iters=5)
    flops = 2.0 * nnz * 256 * 256
    out["subm_k3_256_256_1M"] = {
        "voxels": n, "nnz": nnz, "kmap_ms": round(t_map, 4), "kmap_with_sort_products_ms": round(t_map_sorted, 4),
        "conv_ms": round(t, 4), "eff_TFLOPs": round(flops / (t * 1e-3) / 1e12, 1),
        "conv_sorted_ms": round(t_sorted, 4), "sorted_eff_TFLOPs": round(flops / (t_sorted * 1e-3) / 1e12, 1),
        "group_rows_ms": round(t_group, 4), "conv_grouped_ms": round(t_grouped, 4),
        "grouped_eff_TFLOPs": round(flops / (t_grouped * 1e-3) / 1e12, 1)}
    return out


def pointops_sweep(F):
    """The point-voxel operators on a synthetic cloud (1M points in ~200k voxels, 64 channels,
    fp16): HIP-event time and the rate at which the bytes each op has to touch move."""
    n, c, b = 1_000_000, 64, 2
    g = torch.Generator(device="cuda").manual_seed(0)
    pts = torch.rand(n, 3, device="cuda", generator=g) * torch.tensor([160.0, 160.0, 8.0], device="cuda")
    pc = torch.cat([torch.zeros(n, 1, device="cuda", dtype=torch.int32), pts.floor().int()], 1).contiguous()
    offsets = torch.tensor([[dx, dy, dz] for dx in (0, 1) for dy in (0, 1) for dz in (0, 1)],
                           device="cuda", dtype=torch.int32)
    pc_hash = F.sphash(pc)
    vox_hash = torch.unique(pc_hash)
    n_vox = vox_hash.numel()
    idx = F.sphashquery(pc_hash, vox_hash)
    counts = F.spcount(idx, n_vox)
    corner = F.sphashquery(F.sphash(pc, offsets).t().contiguous(), vox_hash)
    w = F.calc_ti_weights(pts, corner, scale=1)
    feats = torch.randn(n, c, device="cuda", dtype=torch.float16)
    vfeat = torch.randn(n_vox, c, device="cuda", dtype=torch.float16)
    from torchsparse_amd import backend
    rows = []

    def add(name, fn, nbytes):
        ms = event_ms(fn, iters=20)
        rows.append({"op": name, "ms": round(ms, 4), "GBps": round(nbytes / ms / 1e6, 1)})

    add("sphash", lambda: F.sphash(pc), 24 * n)
    add("sphash_8_offsets", lambda: F.sphash(pc, offsets), 16 * n + 64 * n)
    add("sphashquery", lambda: F.sphashquery(pc_hash, vox_hash), 12 * backend.hash_capacity(n_vox) * 2 + 8 * n_vox + 12 * n)
    add("spcount", lambda: F.spcount(idx, n_vox), 4 * n + 8 * n_vox)
    def regroup(t, groups):
        t._tsmi_groups = None
        backend.group_by_index(t, groups)

    add("group_points_by_voxel", lambda: regroup(idx, n_vox), 2 * 8 * n * 2 + 4 * n_vox)
    add("group_corners_by_voxel", lambda: regroup(corner, n_vox), 2 * 8 * 8 * n * 2 + 4 * n_vox)
    add("spvoxelize", lambda: backend.voxelize_forward_cuda(feats, idx, counts), n * (c * b + 4) + n_vox * c * b)
    add("spvoxelize_backward", lambda: backend.voxelize_backward_cuda(vfeat, idx, counts, n),
        n * (c * b + 4) + n_vox * c * b)
    add("spdevoxelize", lambda: backend.devoxelize_forward_cuda(vfeat, corner, w), n * (c * b + 64) + n_vox * c * b)
    add("spdevoxelize_backward", lambda: backend.devoxelize_backward_cuda(feats, corner, w, n_vox),
        n * (c * b + 64) + n_vox * c * b)
    return {"points": n, "voxels": n_vox, "channels": c, "dtype": "f16", "ops": rows}


def network_layers(model, inp):
    """One forward with hooks: per sparse conv the geometry and sizes it ran at."""
    from torchsparse_amd import nn as spnn
    records = []

    def hook(mod, args, output):
        x = args[0]
        records.append({"mod": mod, "cin": mod.in_channels, "cout": mod.out_channels,
                        "ks": mod.kernel_size, "stride": mod.stride, "transposed": mod.transposed,
                        "level": x.stride, "n_in": x.feats.shape[0], "n_out": output.feats.shape[0]})

    handles = [m.register_forward_hook(hook) for m in model.modules() if isinstance(m, spnn.Conv3d)]
    out = model(inp)
    for h in handles:
        h.remove()
    return records, out


def dominant_layer_roofline(ts, F, records, caches, pmc_target=None):
    """Group the network's conv launches by (level, geometry, channels), time each
    group's kernel alone with HIP events on the launch stream, and report the roofline
    of the group with the largest total time."""
    from torchsparse_amd import backend
    groups = {}
    for r in records:
        if r["ks"] == (1, 1, 1):
            continue
        key = (r["level"], r["ks"], r["stride"], r["transposed"], r["cin"], r["cout"])
        groups.setdefault(key, []).append(r)
    best = None
    every = []
    for key, rs in groups.items():
        level, ks, stride, transposed, cin, cout = key
        r = rs[0]
        fine = tuple(level[a] // stride[a] for a in range(3)) if transposed else level
        km = caches.kmaps[(fine, ks, stride, (1, 1, 1))]
        omap = km["out_in_map_t"] if transposed else km["out_in_map"]
        x = torch.randn(r["n_in"], cin, device="cuda", dtype=torch.float16)
        w = r["mod"].kernel.detach()
        run = (lambda x=x, w=w, omap=omap, n_out=r["n_out"], cout=cout:
               backend.conv_forward_implicit_gemm_cuda(x, w, omap, n_out, cout))
        # as a step with rebuilt maps runs it: rows in coordinate order (a map's grouped copy is
        # built only once the map has been used about ten times, see backend.igemm_group_rows)
        setting, backend.igemm_group_rows = backend.igemm_group_rows, False
        ms = event_ms(run, iters=30, warm=5)
        backend.igemm_group_rows = setting
        total = ms * len(rs)
        kvol = ks[0] * ks[1] * ks[2]
        nnz = int((omap[:r["n_out"]] >= 0).sum().item())
        desc = (f"igemm k{ks} s{stride} {'T ' if transposed else ''}{cin}->{cout} "
                f"level{level} n_out={r['n_out']} nnz={nnz}")
        if pmc_target not in (None, "auto"):
            total = 1.0 if desc == pmc_target else 0.0
        flops, nbytes = conv_work(r["n_in"], r["n_out"], omap.shape[0], nnz, kvol, cin, cout, 2)
        one = roofline_of(flops, nbytes, ms)
        form = ("pair segments (segment_products_kernel + segment_sum_kernel)"
                if backend._segments_pay(x, kvol, cin, cout, r["n_out"], omap) else "dense pass over the map")
        share = None
        if form.startswith("dense") and backend._grouping_fits(x, kvol, cin, cout, r["n_out"]):
            # the same layer over the grouped copy of its map (maps kept over several forwards)
            backend.igemm_group_rows = "always"
            share = tile_offset_share(backend, omap, r["n_out"], w)
            share["launch_ms_over_grouped_map"] = round(event_ms(run, iters=30, warm=5), 5)
            backend.igemm_group_rows = setting
        every.append({"kernel": desc, "form": form, "launches_per_step": len(rs), "launch_ms": round(ms, 5),
                      "step_ms": round(ms * len(rs), 4), "bound": one["bound"],
                      "achieved": round(one["achieved"], 2), "peak": one["peak"], "unit": one["unit"],
                      "frac": round(one["frac"], 4),
                      "dense_map_TFLOPs": round(2.0 * omap.shape[0] * kvol * cin * cout / (ms * 1e-3) / 1e12, 1),
                      **({"rows_grouped_by_kernel_planes": share} if share else {})})
        if best is None or total > best["total_ms"]:
            best = {"total_ms": total, "ms": ms, "launches": len(rs), "flops": flops, "bytes": nbytes,
                    "run": run, "issued": 2.0 * omap.shape[0] * kvol * cin * cout,
                    "desc": desc}
    if pmc_target:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        for _ in range(5):
            best["run"]()
        torch.cuda.synchronize()
        return {"kernel": best["desc"]}
    roof = roofline_of(best["flops"], best["bytes"], best["ms"])
    roof["traffic"] = pmc_traffic_bytes(best["desc"])
    if roof["traffic"] is None:
        roof["traffic_note"] = "no FETCH_SIZE / WRITE_SIZE pass recorded for this kernel and shape"
    roof["kernel"] = best["desc"]
    # every convolution group of the step, largest share first: the deep, wide layers run
    # furthest below their roofline and carry the largest share of the step
    roof["all_groups"] = sorted(every, key=lambda e: -e["step_ms"])
    roof["launch_ms"] = round(best["ms"], 5)
    roof["launches_per_step"] = best["launches"]
    roof["algorithmic_bytes"] = best["bytes"]
    roof["algorithmic_flops"] = best["flops"]
    # the dense work over the whole map (every (row, offset) pair multiplied): what the MFMA
    # pipe would execute without any skipping
    roof["dense_map_flops"] = best["issued"]
    roof["dense_map_TFLOPs"] = round(best["issued"] / (best["ms"] * 1e-3) / 1e12, 1)
    roof["achieved"] = round(roof["achieved"], 2)
    roof["frac"] = round(roof["frac"], 4)
    roof["measured_on_this_gpu"] = achievable_peaks()
    return roof


def tile_offset_share(backend, omap, n_out, w):
    """(wavefront of 32 rows, kernel offset) blocks a dense pass multiplies, as a share of all of
    them: over the rows in coordinate order, and over the grouped copy of the map the layer
    runs on."""
    valid = (omap[:n_out] >= 0)
    pad = (-n_out) % 32
    if pad:
        valid = torch.cat([valid, torch.zeros((pad, valid.shape[1]), dtype=torch.bool, device=valid.device)])
    natural = float(valid.view(-1, 32, valid.shape[1]).any(1).float().mean())
    g = backend.grouped_map(omap, n_out)
    gv = g.grouped >= 0
    grouped = float(gv.view(-1, 32, gv.shape[1]).any(1).float().sum() / (valid.shape[0] // 32 * valid.shape[1]))
    return {"wavefront_offset_blocks_multiplied_coordinate_order": round(natural, 3),
            "wavefront_offset_blocks_multiplied_grouped": round(grouped, 3)}


def pmc_kernels(ts, spnn, F, backend, coords, n):
    """The launches a counter pass (rocprofv3 --pmc) looks at, five of each after five 256 MiB
    copies whose known size scales the counters: kernel maps of the scan and of the 1M-voxel
    input (searched over sorted rows, then through the hash table), the strided k2 s2 chain
    of the scan, gather and scatter of a 64 -> 64 layer, the 1M-voxel 256 -> 256 convolution."""
    from torchsparse_amd.utils import synthetic
    src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    for _ in range(5):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst
    big = torch.from_numpy(synthetic.sphere_shell_voxels(seed=3)).cuda()
    for rows in (coords, big):
        for searched in (True, False):
            backend.kmap_through_sorted = searched
            for _ in range(5):
                F.build_kernel_map(rows, rows.shape[0], 3, 1, 1, mode="hashmap_on_the_fly")
            torch.cuda.synchronize()
    backend.kmap_through_sorted = True
    for _ in range(5):
        level = coords
        for _ in range(4):
            level = F.build_kernel_map(level, level.shape[0], 2, 2, 0, mode="hashmap_on_the_fly")["coords"]
    torch.cuda.synchronize()
    cfg = F.conv_config.get_default_conv_config()
    cfg.dataflow = F.Dataflow.GatherScatter
    layer = spnn.Conv3d(64, 64, 3, config=cfg).cuda().half()
    x = ts.SparseTensor(torch.randn(n, 64, device="cuda", dtype=torch.float16), coords)
    with torch.no_grad():
        for _ in range(6):
            layer(x)
    torch.cuda.synchronize()
    km = F.build_kernel_map(big, big.shape[0], 3, 1, 1, mode="hashmap_on_the_fly")
    xb = torch.randn(big.shape[0], 256, device="cuda", dtype=torch.float16)
    w = torch.randn(27, 256, 256, device="cuda", dtype=torch.float16) * 0.02
    for _ in range(5):
        backend.conv_forward_implicit_gemm_cuda(xb, w, km["out_in_map"], big.shape[0], 256)
    torch.cuda.synchronize()
    print(json.dumps({"pmc_kernels": "done", "scan_voxels": n, "big_voxels": int(big.shape[0])}))


def kmap_roofline(F, backend, coords, n):
    """The submanifold k3 map of the scan (one launch over ascending rows): HIP-event time of
    the build, priced with the bytes a hash-table build has to touch (coordinates, table
    init, inserts, one probe per queried neighbour of the half kernel, the map) and with the
    least any builder moves (coordinates in, map out)."""
    ms = event_ms(lambda: F.build_kernel_map(coords, n, 3, 1, 1, mode="hashmap_on_the_fly"), iters=30, warm=5)
    n_pad = (n + 127) // 128 * 128
    hashed = kmap_bytes_subm(n, n_pad, backend.hash_capacity(n), 27)
    least = 16.0 * n + 4.0 * 27 * n_pad
    searched = backend.kmap_sorted_supported(3) and backend.coords_ascending(coords)
    return {"bound": "hbm", "achieved": round(hashed / ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(hashed / ms / 1e6 / HBM_PEAK_GBS, 4), "traffic": None,
            "kernel": ("kmap_sorted_kernel<3>" if searched else "subm_prepare + insert_coords + kmap_query_subm")
                      + f" k3 s1 n={n}",
            "launch_ms": round(ms, 5), "algorithmic_bytes": hashed,
            "coords_plus_map_bytes": least, "coords_plus_map_GBps": round(least / ms / 1e6, 1)}


def cpu_baseline(records, level_coords):
    """The oracle's CPU convolution (gather -> GEMM -> scatter, fp32, threads over rows)
    and kernel-map builders over the network's sparse conv layers and maps, once."""
    import oracle
    cores = oracle.set_threads(int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    rng = np.random.default_rng(0)
    t_map = t_conv = t_ref = t_conv_same = 0.0
    pair_cache = {}
    n_layers = n_ref_layers = 0
    timed_layers = []
    ref_budget_s = 15.0  # the compiled reference convolution is slow: stop timing it after this
    ref = oracle.ref_module()  # the reference's own CPU convolution, compiled in place
    for r in records:
        if r["ks"] == (1, 1, 1):
            continue
        level, ks, stride, transposed = r["level"], r["ks"], r["stride"], r["transposed"]
        fine = tuple(level[a] // stride[a] for a in range(3)) if transposed else level
        key = (fine, ks, stride)
        if key not in pair_cache:
            coords = level_coords[fine]
            t0 = time.perf_counter()
            if all(s == 1 for s in stride):
                nb, sz = oracle.kmap_cpu_backend(coords, ks)
            else:
                omap, _ = oracle.kmap_downsample(coords, ks, stride, (0, 0, 0))
                nb, sz = oracle.pair_lists(omap)
            t_map += time.perf_counter() - t0
            pair_cache[key] = (nb, sz)
        nb, sz = pair_cache[key]
        x = rng.standard_normal((r["n_in"], r["cin"])).astype(np.float32)
        w = rng.standard_normal((len(sz), r["cin"], r["cout"])).astype(np.float32)
        t0 = time.perf_counter()
        oracle.conv_gather_scatter(x, w, nb, sz, r["n_out"], transpose=transposed, variant=1)
        dt = time.perf_counter() - t0
        t_conv += dt
        timed_layers.append((dict(r, key=key), dt))
        if ref is not None and t_ref < ref_budget_s:
            n_y = r["n_out"]
            y = torch.zeros(n_y, r["cout"])
            tx, tw, tnb, tsz = torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(nb), torch.from_numpy(sz)
            t0 = time.perf_counter()
            ref.conv_forward_gather_scatter_cpu(tx, y, tw, tnb, tsz, transposed)
            t_ref += time.perf_counter() - t0
            t_conv_same += dt
            n_ref_layers += 1
        n_layers += 1
    extra = {}
    if ref is not None:
        extra = {"reference_conv_ms": round(t_ref * 1e3, 1),
                 "reference_conv": "conv_forward_gather_scatter_cpu of the reference (its own sources, "
                                   f"compiled) over the first {n_ref_layers} of the layers (stopped "
                                   f"after {ref_budget_s:.0f} s), torch threads = "
                                   f"{torch.get_num_threads()}; the port takes "
                                   f"{t_conv_same * 1e3:.0f} ms on those layers"}
    # the same convolutions with the reference's own threading (a parallel region per row over
    # the channel loop) and on one thread, each on a bounded prefix of the layers
    for name, variant, threads in (("faithful_threading", 0, cores), ("one_thread", 1, 1)):
        oracle.set_threads(threads)
        t_v = t_same = 0.0
        n_v = 0
        for r, dt in timed_layers:
            if t_v > 5.0:
                break
            nb, sz = pair_cache[r["key"]]
            x = rng.standard_normal((r["n_in"], r["cin"])).astype(np.float32)
            w = rng.standard_normal((len(sz), r["cin"], r["cout"])).astype(np.float32)
            t0 = time.perf_counter()
            oracle.conv_gather_scatter(x, w, nb, sz, r["n_out"], transpose=r["transposed"], variant=variant)
            t_v += time.perf_counter() - t0
            t_same += dt
            n_v += 1
        extra[name] = {"conv_ms": round(t_v * 1e3, 1), "layers": n_v, "threads": threads,
                       "row_parallel_ms_same_layers": round(t_same * 1e3, 1)}
    oracle.set_threads(cores)
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {**extra, "value": round((t_map + t_conv) * 1e3, 1), "unit": "ms", "cores": cores, "kind": "port",
            "cpu_model": model, "host_cpus": os.cpu_count(),
            "sample": f"{n_layers} sparse conv layers (fp32) + {len(pair_cache)} kernel maps of one "
                      f"MinkUNet forward on the same scan; BN/ReLU/concat/1x1x1 layers excluded; "
                      f"maps {t_map * 1e3:.0f} ms, convs {t_conv * 1e3:.0f} ms",
            "kmap_ms": round(t_map * 1e3, 1), "conv_ms": round(t_conv * 1e3, 1)}


def _short_kernel(name):
    import re
    n = name.replace("(anonymous namespace)::", "")
    n = re.sub(r"\(.*", "", n)
    n = n.replace("void ", "").replace("tsmi::f16::", "").replace("tsmi::", "")
    n = n.replace("rocprim::ROCPRIM_400200_NS::detail::", "rocprim::")
    m = re.match(r"_ZN4tsmi3f16\d+([a-z_0-9]+?)E", n)
    if m:
        n = m.group(1)
    return n[:70]


def summarize(meas):
    """No GPU work: the rocprofv3 output under ``meas`` (written by the commands quoted in the
    summaries) -> profiles/bench_minkunet_kernel_trace.md, profiles/igemm_roofline_kernel_pmc.md,
    profiles/roofline_traffic.json."""
    import collections
    import csv
    import re
    prof = os.path.join(ROOT, "profiles")
    bench = json.loads(open(os.path.join(meas, "bench.json")).read())
    roof = bench["roofline"]
    desc = roof["kernel"]
    steps, warmup = bench["steps"], bench["warmup"]

    # ---- kernel trace: stats, and the timed loop between the two marker fills ----
    rows = list(csv.DictReader(open(os.path.join(meas, "kt", "kt_kernel_stats.csv"))))
    out = ["# rocprofv3 kernel trace of bench.py (MinkUNet fp16 forward, %d-voxel synthetic scan)\n" % bench["config"]["voxels"],
           "Command (from the repository root on one MI355X; `cd /tmp && export TMPDIR=/tmp` first; OUT: a scratch "
           "directory that also holds the output of a plain `python bench.py > OUT/bench.json`), then "
           "`python bench.py --summarize OUT` for this file:\n",
           "```\nrocprofv3 --kernel-trace --stats --output-format csv -d OUT/kt -o kt -- python bench.py "
           f"--steps {steps} --warmup {warmup} --no-cpu --no-layers --no-backward --no-tune --no-pointops --no-configs\n```\n",
           "The process also runs the unfused network, the same-tensor and resident-tensor loops, warm-map forwards and the "
           "per-group roofline timing, so `calls` mixes those phases; the second table isolates the timed loop "
           "(the kernels between the two int16 marker fills that bracket it).\n",
           "## Kernel stats of the whole process (top 24 by total time)\n",
           "| kernel | calls | total µs | avg µs | % |\n|---|---:|---:|---:|---:|"]
    for r in rows[:24]:
        out.append(f"| `{_short_kernel(r['Name'])}` | {r['Calls']} | {float(r['TotalDurationNs']) / 1e3:.0f} | "
                   f"{float(r['AverageNs']) / 1e3:.1f} | {float(r['Percentage']):.2f} |")
    tr = list(csv.DictReader(open(os.path.join(meas, "kt", "kt_kernel_trace.csv"))))
    tr.sort(key=lambda r: int(r["Start_Timestamp"]))
    marks = [i for i, r in enumerate(tr) if "FillFunctor<short>" in r["Kernel_Name"]]
    assert len(marks) == 2, f"expected the two marker fills around the timed loop, found {len(marks)}"
    seg = tr[marks[0] + 1:marks[1]]
    streams = collections.Counter(r["Stream_Id"] for r in seg)
    main = streams.most_common(1)[0][0]
    per = collections.defaultdict(lambda: [0, 0.0, 0.0])
    busy = {True: 0.0, False: 0.0}
    count = {True: 0, False: 0}
    for r in seg:
        n = _short_kernel(r["Kernel_Name"])
        if n.startswith("Cijk"):
            n = "hipBLASLt GEMM (linear head)"
        elif n.startswith("rocprim"):
            n = "rocprim (sort / select / scan)"
        elif n.startswith("at::native") or n.startswith("__amd"):
            n = "torch elementwise / copy / fill / cat"
        dur = (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3
        on_main = r["Stream_Id"] == main
        per[n][0] += 1
        per[n][1 if on_main else 2] += dur
        busy[on_main] += dur
        count[on_main] += 1
    wall = (int(seg[-1]["End_Timestamp"]) - int(seg[0]["Start_Timestamp"])) / 1e3
    out.append(f"\n## The timed loop: {steps} steps (fused network, a new coordinate tensor and 9 kernel maps every step), per step\n")
    out.append(f"{len(seg) / steps:.1f} kernels per step; kernel time {(busy[True] + busy[False]) / steps:.0f} µs per step, of it "
               f"{busy[True] / steps:.0f} µs ({count[True] / steps:.1f} kernels) on the caller's stream and "
               f"{busy[False] / steps:.0f} µs ({count[False] / steps:.1f} kernels) on the library's second stream; "
               f"first kernel to last {wall / steps:.0f} µs per step; `ms_per_step` of this run "
               f"{bench['ms_per_step'] * 1e3:.0f} µs.\n")
    out.append("| kernel | launches / step | µs / step, caller's stream | µs / step, second stream |\n|---|---:|---:|---:|")
    for k, v in sorted(per.items(), key=lambda kv: -(kv[1][1] + kv[1][2])):
        out.append(f"| `{k}` | {v[0] / steps:.1f} | {v[1] / steps:.1f} | {v[2] / steps:.1f} |")
    out.append("\n`igemm2_kernel<MF,NT,KS,OS>`: MF·64 output rows × NT·16 output channels per workgroup, KS·64 bytes of input "
               "channels and OS kernel offsets per reduction step; `tile_kernel<..,WM,WN,KS,ST>`: 32·WM rows × 32·WN channels, "
               "ST-stage LDS ring; `map_group_rows_kernel` / `group_tile_order_kernel`: the grouped copy of a level's 3×3×3 map.")
    open(os.path.join(prof, "bench_minkunet_kernel_trace.md"), "w").write("\n".join(out) + "\n")

    # ---- counters of the roofline kernel ----
    def counter_rows(sub, stem):
        path = os.path.join(meas, sub, stem + "_counter_collection.csv")
        rs = list(csv.DictReader(open(path)))
        rs.sort(key=lambda r: int(r["Dispatch_Id"]))
        return rs

    def last5(rs, ctr):
        vals = [(r["Kernel_Name"], float(r["Counter_Value"]), int(r["Grid_Size"]),
                 int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) for r in rs if r["Counter_Name"] == ctr]
        tgt = [v for v in vals if re.search(r"igemm2?_kernel|tile_kernel|segment_products", v[0])][-5:]
        cp = [v for v in vals if "copyBuffer" in v[0] and v[2] == 131072][-5:]
        return tgt, cp

    avg = lambda v, i=1: sum(x[i] for x in v) / len(v)  # noqa: E731
    ft, fc = last5(counter_rows("pmc_fetch", "f"), "FETCH_SIZE")
    wt, wc = last5(counter_rows("pmc_write", "w"), "WRITE_SIZE")
    kib = 256 * 1024
    f_fac, w_fac = kib / avg(fc), kib / avg(wc)
    fetch, write = avg(ft) * f_fac, avg(wt) * w_fac
    kname = _short_kernel(ft[0][0])
    o = ["# Hardware counters of the roofline kernel\n", f"Kernel: `{kname}` — {desc}\n",
         "Commands (one pass per run; `bench.py --pmc-target KERNEL` launches a 256 MiB device-to-device copy five times "
         "and then the kernel five times), then `python bench.py --summarize OUT`:\n",
         f"```\nrocprofv3 --pmc FETCH_SIZE --output-format csv -d OUT/pmc_fetch -o f -- python bench.py --pmc-target \"{desc}\"\n"
         f"rocprofv3 --pmc WRITE_SIZE --output-format csv -d OUT/pmc_write -o w -- python bench.py --pmc-target \"{desc}\"\n"
         "rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_VALU_MFMA_MOPS_F16 SQ_WAIT_INST_ANY SQ_ACTIVE_INST_LDS SQ_WAVE_CYCLES "
         f"SQ_BUSY_CYCLES GRBM_GUI_ACTIVE --output-format csv -d OUT/pmc_sq -o q -- python bench.py --pmc-target \"{desc}\"\n```\n",
         "## HBM traffic\n",
         "| counter (KiB per dispatch) | 256 MiB copy reads | scale to true KiB | kernel reads | kernel, scaled |\n|---|---:|---:|---:|---:|",
         f"| FETCH_SIZE | {avg(fc):.0f} | {f_fac:.3f} | {avg(ft):.0f} | {fetch:.0f} |",
         f"| WRITE_SIZE | {avg(wc):.0f} | {w_fac:.3f} | {avg(wt):.0f} | {write:.0f} |"]
    tot = (fetch + write) * 1024
    o.append(f"\nHBM traffic per launch: {tot / 1e6:.1f} MB ({fetch * 1024 / 1e6:.1f} read + {write * 1024 / 1e6:.1f} written); "
             f"algorithmic bytes {roof['algorithmic_bytes'] / 1e6:.1f} MB, algorithmic flops {roof['algorithmic_flops'] / 1e9:.2f} G; "
             f"launch duration by HIP events in bench.py {roof['launch_ms'] * 1e3:.1f} µs "
             f"({avg(ft, 3) / 1e3:.1f} µs under the counter pass).")
    sq_path = os.path.join(meas, "pmc_sq", "q_counter_collection.csv")
    if os.path.exists(sq_path):
        rs = counter_rows("pmc_sq", "q")
        names = ["SQ_VALU_MFMA_BUSY_CYCLES", "SQ_INSTS_VALU_MFMA_MOPS_F16", "SQ_WAIT_INST_ANY", "SQ_ACTIVE_INST_LDS",
                 "SQ_WAVE_CYCLES", "SQ_BUSY_CYCLES", "GRBM_GUI_ACTIVE"]
        got = {}
        dur_ns = None
        for nm in names:
            tgt, _ = last5(rs, nm)
            if tgt:
                got[nm] = avg(tgt)
                dur_ns = avg(tgt, 3)
        o.append("\n## Matrix pipe, LDS and waiting (per launch, summed over the device)\n")
        o.append("| counter | value |\n|---|---:|")
        for nm in names:
            if nm in got:
                o.append(f"| {nm} | {got[nm]:.4g} |")
        if "SQ_VALU_MFMA_BUSY_CYCLES" in got and "GRBM_GUI_ACTIVE" in got:
            # SIMD cycles of the launch: its duration at the 2.4 GHz peak engine clock x 256 CUs x 4 SIMDs
            # (GRBM_GUI_ACTIVE is summed over the XCDs' instances and is listed as read)
            simd_cycles = dur_ns * 1e-9 * 2.4e9 * 1024
            o.append(f"\nMatrix pipe busy {100 * got['SQ_VALU_MFMA_BUSY_CYCLES'] / simd_cycles:.1f} % of the SIMD cycles "
                     f"(SQ_VALU_MFMA_BUSY_CYCLES ÷ (duration × 2.4 GHz × 1024 SIMDs)); kernel duration under this "
                     f"pass {dur_ns / 1e3:.1f} µs.")
        if "SQ_INSTS_VALU_MFMA_MOPS_F16" in got:
            # one count = 512 multiply-adds... report raw and the flops it stands for (MOPS counts units of 512 flops)
            o.append(f"fp16 matrix operations counted: {got['SQ_INSTS_VALU_MFMA_MOPS_F16']:.4g} × 512 flop = "
                     f"{got['SQ_INSTS_VALU_MFMA_MOPS_F16'] * 512 / 1e9:.2f} GFLOP executed, against {roof['algorithmic_flops'] / 1e9:.2f} "
                     f"GFLOP of pairs and {roof['dense_map_flops'] / 1e9:.2f} GFLOP of the whole map"
                     + (f" ({got['SQ_INSTS_VALU_MFMA_MOPS_F16'] * 512 / (dur_ns * 1e-9) / 1e12:.0f} TFLOP/s executed, "
                        f"{100 * got['SQ_INSTS_VALU_MFMA_MOPS_F16'] * 512 / (dur_ns * 1e-9) / 2.5e15:.1f} % of the dense "
                        "fp16 peak)." if dur_ns else "."))
        if "SQ_WAIT_INST_ANY" in got and "SQ_WAVE_CYCLES" in got:
            o.append(f"Wavefronts wait for an instruction {100 * got['SQ_WAIT_INST_ANY'] / got['SQ_WAVE_CYCLES']:.0f} % of "
                     f"their cycles; LDS instructions are active {100 * got.get('SQ_ACTIVE_INST_LDS', 0) / got['SQ_WAVE_CYCLES']:.0f} %.")
    open(os.path.join(prof, "igemm_roofline_kernel_pmc.md"), "w").write("\n".join(o) + "\n")
    try:
        table = json.load(open(TRAFFIC_FILE))
    except (OSError, ValueError):
        table = {}
    table[desc] = {"fetch_bytes": int(fetch * 1024), "write_bytes": int(write * 1024), "kernel": kname,
                   "copy_scale_fetch": round(f_fac, 4), "copy_scale_write": round(w_fac, 4)}
    json.dump(table, open(TRAFFIC_FILE, "w"), indent=1, sort_keys=True)
    print(desc, int(tot))


def main():
    args = parse()
    if args.summarize:
        summarize(args.summarize)
        return
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}); nothing in this path "
              "communicates between GPUs", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.backbones import SparseResUNet42
    from torchsparse_amd.nn import functional as F
    from torchsparse_amd.utils.synthetic import lidar_scan_voxels

    torch.manual_seed(0)
    coords_np = lidar_scan_voxels(seed=1)
    n = coords_np.shape[0]
    coords = torch.from_numpy(coords_np).cuda()
    feats = torch.randn(n, 4, device="cuda", dtype=torch.float16)
    import copy
    from torchsparse_amd.nn.utils import fuse_inference
    unfused = SparseResUNet42(in_channels=4).cuda().half().eval()
    model = fuse_inference(copy.deepcopy(unfused))
    head = torch.nn.Linear(96, 19).cuda().half().eval()
    if args.sorted == 1:
        F.set_conv_mode(1)
    if args.dense_deep:
        backend.igemm_through_segments = False

    def timed(net, steps, warmup, rows="new", mark=False):
        """ms per forward.  rows = "new": a coordinate tensor the library has not seen, every step
        (a device copy queued in the step: what a loader that hands over one scan after the
        other amounts to; the library checks its range and row order - one small kernel and
        one read-back - and every kernel map is rebuilt); "resident": a new tensor every step
        that was complete before the loop and is declared so (backend.rows_ready), so its
        check runs on the second stream and waits for nothing the forward before has queued; "same": the same tensor every step (the check is
        remembered, the strided chain runs ahead on the second stream; the maps are rebuilt)."""
        pool = [coords.clone() for _ in range(steps + warmup)] if rows == "resident" else None
        k = [0]

        def step():
            with torch.no_grad():
                if rows == "new":
                    c = coords.clone()
                elif rows == "resident":
                    c = backend.rows_ready(pool[k[0]])
                    k[0] += 1
                else:
                    c = coords
                return head(net(ts.SparseTensor(feats, c))[-1].feats)
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        marker = torch.empty(MARKER_ELEMS, dtype=torch.int16, device="cuda") if mark else None
        if mark:
            marker.fill_(1)  # (brackets the timed loop in a kernel trace)
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        if mark:
            marker.fill_(2)
            torch.cuda.synchronize()
        backend.settle_checks()
        return ms

    if args.pmc_kernels:
        pmc_kernels(ts, spnn, F, backend, coords, n)
        return
    if args.pmc_target:
        with torch.no_grad():
            inp = ts.SparseTensor(feats, coords)
            records, _ = network_layers(model, inp)
            print(json.dumps(dominant_layer_roofline(ts, F, records, inp._caches,
                                                     pmc_target=args.pmc_target)))
        return

    # the secondary figures first: the clocks, the allocator and the library's own look-ahead
    # state settle over the first few dozen forwards of a process (the headline loop measured
    # first reads ~5 % higher than the same loop a moment later)
    ms_unfused = timed(unfused, max(args.steps // 2, 1), 2, rows="same")
    ms_same = timed(model, args.steps, args.warmup, rows="same")
    ms_resident = timed(model, args.steps, args.warmup, rows="resident")
    # the same new-tensor loop with the convolution calls launched by this thread instead of the
    # library's launch thread, and what queuing one forward costs the host (device idle at its start)
    backend.launch_thread = False
    ms_direct = timed(model, args.steps, args.warmup, rows="new")
    backend.launch_thread = True

    def host_ms(iters=20):
        total = 0.0
        with torch.no_grad():
            for _ in range(iters):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                head(model(ts.SparseTensor(feats, coords))[-1].feats)
                total += time.perf_counter() - t0
        torch.cuda.synchronize()
        return total * 1e3 / iters
    ms_host = host_ms()
    ms_per_step = timed(model, args.steps, args.warmup, rows="new", mark=True)

    with torch.no_grad():
        inp = ts.SparseTensor(feats, coords)
        records, outs = network_layers(model, inp)
        warm_ms = event_ms(lambda: model(inp), iters=10, warm=2)  # kernel maps cached
        # the same forward (with the linear head) over cached maps, recorded as a HIP graph and replayed
        from torchsparse_amd.utils.graph import GraphedForward
        runner = GraphedForward(lambda t: head(model(t)[-1].feats), ts.SparseTensor(feats, coords))
        graph_ms = event_ms(runner, iters=20, warm=3)
        del runner
        roof = None if args.no_roofline else dominant_layer_roofline(ts, F, records, inp._caches)
        level_coords = {lvl: c[0].cpu().numpy() for lvl, c in inp._caches.cmaps.items()}
        layers = None if args.no_layers else layer_sweep(ts, spnn, F, backend, coords, n)
        roof_kmap = None if args.no_roofline else kmap_roofline(F, backend, coords, n)
    backward = None if args.no_backward else backward_sweep(ts, spnn, F, backend, coords, n, feats)
    pointops = None if args.no_pointops else pointops_sweep(F)
    configs = None if args.no_configs else other_configs(ts, spnn, F, backend)
    tuned = None
    if not args.no_tune:
        # the per-group tuner over all three dataflows and the sorted variants, then the same
        # timed loop on the tuned copy of the network
        import tempfile
        from torchsparse_amd.utils.tune import tune
        tuned_model = copy.deepcopy(model)
        with tempfile.TemporaryDirectory() as tmp:
            chosen = tune(tuned_model, [ts.SparseTensor(feats, coords) for _ in range(12)], n_samples=12,
                          save_dir=tmp, tune_tag="bench", verbose=False, skip_warning=True,
                          dataflow_range=[F.Dataflow.ImplicitGEMM, F.Dataflow.FetchOnDemand,
                                          F.Dataflow.GatherScatter])
        tuned = {"ms_per_step": round(timed(tuned_model, args.steps, args.warmup, rows="same"), 4),
                 "default_ms_per_step": round(timed(model, args.steps, args.warmup, rows="same"), 4),
                 "groups": [{"level": g[0], "kernel": g[1], "stride": g[2],
                             "dataflow": c["dataflow"].name, "ifsort": c["ifsort"],
                             "split_mask_num": c["split_mask_num"]} for g, c in chosen.items()]}
    cpu = None if args.no_cpu else cpu_baseline(records, level_coords)

    result = {
        "metric": "MinkUNet fwd ms @~100k voxels fp16; per-layer eff. TFLOP/s + kmap GB/s",
        "value": round(ms_per_step, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "MinkUNet (SparseResUNet42, cr=1.0) + Linear(96,19) forward, batch 1, "
                               f"synthetic 64-beam scan seed 1, {n} voxels, 4 input channels, "
                               "a new coordinate tensor (checked on first sight) and 9 kernel maps every step",
                   "voxels": n, "warm_map_ms_per_step": round(warm_ms, 4),
                   "warm_map_graph_replay_ms_per_step": round(graph_ms, 4),
                   "unfused_ms_per_step": round(ms_unfused, 4),
                   "same_coordinate_tensor_ms_per_step": round(ms_same, 4),
                   "resident_new_coordinate_tensor_declared_ready_ms_per_step": round(ms_resident, 4),
                   "host_ms_to_queue_one_forward": round(ms_host, 4),
                   "new_tensor_ms_per_step_without_launch_thread": round(ms_direct, 4),
                   "conv_mode": F.get_conv_mode().value},
        "roofline": roof, "roofline_kmap": roof_kmap, "cpu_baseline": cpu, "layers": layers,
        "backward": backward,
        "tuned": tuned, "pointops": pointops, "other_configs": configs,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
