"""Writes tests/golden/*.npz from the reference's own CPU sources.

Run in the build container only (needs /root/reference and
`python oracle/build.py --ref`).  The fixtures hold inputs and the outputs the
compiled reference produced for them; no reference source text is stored.

  conv_gs_cpu.npz   conv_forward_gather_scatter_cpu
                    (backend/convolution/convolution_gather_scatter_cpu.cpp:38-109)
                    on submanifold k=3, strided k=2/s=2, its transposed use, and
                    strided k=3/s=2 pair lists
  hash_cpu.npz      hash_cpu / kernel_hash_cpu (backend/hash/hash_cpu.cpp:43-59)
  pointops_cpu.npz  count_cpu (others/count_cpu.cpp:7-23), voxelize_forward_cpu /
                    voxelize_backward_cpu (voxelize/voxelize_cpu.cpp:7-43),
                    devoxelize_forward_cpu (devoxelize/devoxelize_cpu.cpp:10-32)
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import oracle  # noqa: E402
from helpers import random_coords  # noqa: E402


def main():
    ref = oracle.ref_module()
    assert ref is not None, "build oracle/_ref first: python oracle/build.py --ref"
    torch.set_num_threads(1)
    rng = np.random.default_rng(2024)
    out = {}
    coords = random_coords(rng, 400, (12, 11, 10), batch=2)
    cases = {
        "subm3": (oracle.kmap_subm(coords, 3), len(coords), False, 12, 20),
        "down2": (oracle.kmap_downsample(coords, 2, 2, 0)[0], None, False, 8, 16),
        "up2": (oracle.kmap_downsample(coords, 2, 2, 0)[0], None, True, 16, 8),
        "down3": (oracle.kmap_downsample(coords, 3, 2, 1)[0], None, False, 5, 7),
    }
    out["coords"] = coords
    bwd = {}
    for name, (omap, n_out, transpose, cin, cout) in cases.items():
        if n_out is None:
            n_out = int((omap >= 0).any(1).sum())
        nbmaps, nbsizes = oracle.pair_lists(omap)
        kvol = omap.shape[1]
        n_x = n_out if transpose else len(coords)
        n_y = len(coords) if transpose else n_out
        x = rng.standard_normal((n_x, cin)).astype(np.float32)
        w = rng.uniform(-0.2, 0.2, (kvol, cin, cout)).astype(np.float32)
        y = torch.zeros(n_y, cout)
        ref.conv_forward_gather_scatter_cpu(torch.from_numpy(x), y, torch.from_numpy(w),
                                            torch.from_numpy(nbmaps), torch.from_numpy(nbsizes),
                                            transpose)
        out[name + "_map"] = omap
        out[name + "_nbmaps"] = nbmaps
        out[name + "_nbsizes"] = nbsizes
        out[name + "_x"] = x
        out[name + "_w"] = w
        out[name + "_y"] = y.numpy()
        out[name + "_transpose"] = np.array(transpose)
        # backward of the same case
        dy = rng.standard_normal((n_y, cout)).astype(np.float32)
        dx, dw = torch.zeros(n_x, cin), torch.zeros(kvol, cin, cout)
        ref.conv_backward_gather_scatter_cpu(torch.from_numpy(x), dx, torch.from_numpy(dy),
                                             torch.from_numpy(w), dw, torch.from_numpy(nbmaps),
                                             torch.from_numpy(nbsizes), transpose)
        bwd[name + "_dy"] = dy
        bwd[name + "_dx"] = dx.numpy()
        bwd[name + "_dw"] = dw.numpy()
    np.savez_compressed(os.path.join(HERE, "conv_gs_cpu.npz"), **out)
    np.savez_compressed(os.path.join(HERE, "conv_gs_bwd_cpu.npz"), **bwd)

    rows = rng.integers(-50, 3000, (64, 4)).astype(np.int32)
    rows[0] = [0, 1, 2, 3]
    offs = oracle.kernel_offsets(3)
    h = ref.hash_cpu(torch.from_numpy(rows)).numpy()
    kh = ref.kernel_hash_cpu(torch.from_numpy(rows), torch.from_numpy(offs)).numpy()
    np.savez_compressed(os.path.join(HERE, "hash_cpu.npz"), rows=rows, offsets=offs, hash=h,
                        kernel_hash=kh)
    # point-voxel operators: 300 points falling into 90 voxels (some empty), 5 channels
    n_pts, n_vox, ch = 300, 90, 5
    idx = rng.integers(0, 80, n_pts).astype(np.int32)        # voxels 80..89 stay empty
    idx[rng.integers(0, n_pts, 20)] = -1                     # points outside every voxel
    counts = ref.count_cpu(torch.from_numpy(idx), n_vox).numpy()
    valid = idx >= 0                                          # the CPU kernels do not guard the index
    pts = rng.standard_normal((n_pts, ch)).astype(np.float32)
    vox = ref.voxelize_forward_cpu(torch.from_numpy(pts[valid]), torch.from_numpy(idx[valid]),
                                   torch.from_numpy(counts)).numpy()
    top = rng.standard_normal((n_vox, ch)).astype(np.float32)
    vox_bwd = ref.voxelize_backward_cpu(torch.from_numpy(top), torch.from_numpy(idx[valid]),
                                        torch.from_numpy(counts), int(valid.sum())).numpy()
    corner = rng.integers(-1, n_vox, (n_pts, 8)).astype(np.int32)
    wts = rng.uniform(0, 1, (n_pts, 8)).astype(np.float32)
    vfeat = rng.standard_normal((n_vox, ch)).astype(np.float32)
    devox = ref.devoxelize_forward_cpu(torch.from_numpy(vfeat), torch.from_numpy(corner),
                                       torch.from_numpy(wts)).numpy()
    np.savez_compressed(os.path.join(HERE, "pointops_cpu.npz"), idx=idx, n_vox=np.array(n_vox),
                        counts=counts, pts=pts, vox=vox, top=top, vox_bwd=vox_bwd, corner=corner,
                        wts=wts, vfeat=vfeat, devox=devox)
    print("written", os.listdir(HERE))


if __name__ == "__main__":
    main()
