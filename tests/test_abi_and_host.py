"""CPU-side checks: the C-ABI library loads and exports every symbol include/tsmi.h
declares (no compute calls), and the host logic mirrors the reference's formulas."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "tsmi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tsmi_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    path = os.path.join(ROOT, "torchsparse_amd", "libtsmi.so")
    assert os.path.exists(path), "build first: python torchsparse_amd/csrc/build.py"
    lib = ctypes.CDLL(path)
    names = _declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/tsmi.h but not exported"
    lib.tsmi_version.restype = ctypes.c_int
    assert lib.tsmi_version() >= 1
    lib.tsmi_last_error.restype = ctypes.c_char_p
    assert lib.tsmi_last_error() == b""


def test_host_side_argument_errors_without_gpu():
    """Entry points validate sizes before touching the device."""
    lib = ctypes.CDLL(os.path.join(ROOT, "torchsparse_amd", "libtsmi.so"))
    lib.tsmi_last_error.restype = ctypes.c_char_p
    lib.tsmi_packed_weight_elems.restype = ctypes.c_int64
    assert lib.tsmi_packed_weight_elems(27, 96, 96) == 27 * 96 * 96
    assert lib.tsmi_packed_weight_elems(27, 4, 19) == 27 * 32 * 32
    assert lib.tsmi_packed_weight_elems(0, 4, 4) == -1
    lib.tsmi_reduce_bitmask.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64,
                                        ctypes.c_int, ctypes.c_void_p]
    assert lib.tsmi_reduce_bitmask(None, None, 1, 128, 6, None) == 2  # runtime_error in the reference
    assert b"multiple of 4" in lib.tsmi_last_error()
    lib.tsmi_hashtable_clear.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
    assert lib.tsmi_hashtable_clear(None, None, None, 64) == 1
    lib.tsmi_derive_bitmask.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
                                        ctypes.c_int, ctypes.c_int64, ctypes.c_void_p]
    assert lib.tsmi_derive_bitmask(None, None, 128, 125, 1, 100, None) == 1
    assert b"32 mask bits" in lib.tsmi_last_error()


def test_python_front_end_mirrors_reference_rules():
    import torchsparse_amd as ts
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.nn import functional as F
    from torchsparse_amd.nn.functional.conv.kmap.build_kmap import _strided_range
    from torchsparse_amd.nn.utils import get_kernel_offsets

    # padding override (nn/modules/conv.py:42-48)
    assert spnn.Conv3d(4, 4, 3, padding=0).padding == (1, 1, 1)
    assert spnn.Conv3d(4, 4, (3, 1, 3), stride=(1, 1, 2), padding=(0, 5, 7)).padding == (1, 0, 7)
    # kernel shapes and init bound (conv.py:56-66, 87-94)
    assert spnn.Conv3d(8, 16, 3).kernel.shape == (27, 8, 16)
    assert spnn.Conv3d(8, 16, 1).kernel.shape == (8, 16)
    assert spnn.Conv3d(8, 16, 1, stride=2).kernel.shape == (1, 8, 16)
    torch.manual_seed(0)
    up = spnn.Conv3d(8, 16, 2, stride=2, transposed=True, bias=True)
    assert float(up.kernel.detach().abs().max()) <= 1 / np.sqrt(16 * 8)
    assert set(up.state_dict().keys()) == {"kernel", "bias"}
    # strided spatial range (build_kmap.py:65-72)
    assert _strided_range((2, 41, 1440, 1440), (3, 3, 3), (2, 2, 2), (1, 1, 1)) == (2, 21, 720, 720)
    assert _strided_range((1, 5, 5, 5), (2, 2, 2), (2, 2, 2), (0, 0, 0)) == (1, 2, 2, 2)
    assert _strided_range(None, (3, 3, 3), (1, 1, 1), (1, 1, 1)) is None
    # offset tables equal the oracle's (nn/utils/kernel.py:21-35)
    for size in (3, 2, 5, (3, 1, 1), (2, 3, 3), 4):
        np.testing.assert_array_equal(get_kernel_offsets(size).numpy(), oracle.kernel_offsets(size))
    np.testing.assert_array_equal(get_kernel_offsets(3, 2, 3).numpy(), oracle.kernel_offsets(3, 2, 3))
    # config knobs
    cfg = F.conv_config.get_default_conv_config()
    assert cfg.dataflow == F.Dataflow.ImplicitGEMM and cfg["kmap_mode"] == "hashmap_on_the_fly"
    assert (cfg.ifsort, cfg.split_mask_num, cfg.epsilon, cfg.mm_thresh, cfg.FOD_fusion) == (False, 1, 0.0, 0, True)
    cfg.ifsort = True
    assert F.conv_config.get_default_conv_config().ifsort is False  # copies, not one shared object
    assert F.conv_config.get_default_conv_config(F.ConvMode.mode2).split_mask_num == 3
    partial = F.conv_config.AttributeDict(dataflow=F.Dataflow.GatherScatter)
    F.conv_config.set_global_conv_config(partial)
    assert F.conv_config.get_global_conv_config()["epsilon"] == 0.0
    F.conv_config.clear_global_conv_config()
    with pytest.raises(AssertionError):
        F.set_kmap_mode("grid")
    F.set_conv_mode(1)
    assert F.get_conv_mode() == F.ConvMode.mode1
    F.set_conv_mode(0)
    # tensor container and caches
    x = ts.SparseTensor(torch.zeros(3, 2), torch.zeros(3, 4, dtype=torch.int32), stride=2)
    assert x.stride == (2, 2, 2) and x.s == (2, 2, 2) and x.F is x.feats and x.C is x.coords
    y = x + x
    assert y._caches is x._caches
    z = ts.cat([x, y])
    assert z.feats.shape == (3, 4) and z._caches is x._caches
    from torchsparse_amd.utils import TensorCacheMode, clear_global_tensor_cache, set_tensor_cache_mode
    set_tensor_cache_mode(TensorCacheMode.GLOBAL_TENSOR_CACHE)
    a = ts.SparseTensor(torch.zeros(1, 1), torch.zeros(1, 4, dtype=torch.int32))
    b = ts.SparseTensor(torch.zeros(1, 1), torch.zeros(1, 4, dtype=torch.int32))
    assert a._caches is b._caches
    set_tensor_cache_mode(TensorCacheMode.SEPARATE_TENSOR_CACHE)
    clear_global_tensor_cache()
    # no CPU path: convolutions refuse host tensors loudly
    with pytest.raises(RuntimeError, match="GPU"):
        spnn.Conv3d(2, 2, 3)(ts.SparseTensor(torch.zeros(3, 2), torch.zeros(3, 4, dtype=torch.int32)))


def test_fuse_inference_on_cpu_modules():
    """Folding is pure parameter arithmetic; check it against the unfused affine map."""
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.nn.utils.fuse import _fold
    torch.manual_seed(0)
    conv, bn = spnn.Conv3d(5, 7, 3, bias=True), spnn.BatchNorm(7).eval()
    bn.running_mean.normal_(); bn.running_var.uniform_(0.5, 2); bn.weight.data.uniform_(0.5, 2); bn.bias.data.normal_()
    w0, b0 = conv.kernel.detach().clone(), conv.bias.detach().clone()
    _fold(conv, bn)
    g = bn.weight / torch.sqrt(bn.running_var + bn.eps)
    torch.testing.assert_close(conv.kernel.detach(), w0 * g)
    torch.testing.assert_close(conv.bias.detach(), (b0 - bn.running_mean) * g + bn.bias)


def test_synthetic_workloads_are_seeded_and_sized():
    from torchsparse_amd.utils.synthetic import lidar_scan_voxels, uniform_voxels
    a, b = lidar_scan_voxels(seed=1), lidar_scan_voxels(seed=1)
    np.testing.assert_array_equal(a, b)
    assert 80_000 < len(a) < 100_000 and a.min() >= 0 and a.dtype == np.int32
    assert len(np.unique(a, axis=0)) == len(a)
    c = uniform_voxels(20000, 128, seed=0)
    assert c.shape == (20000, 4) and len(np.unique(c, axis=0)) == 20000 and c[:, 1:].max() < 128


def test_strided_chain_bookkeeping_with_interleaved_chains():
    """The look-ahead of chains of equal strided convolutions is book-keeping per (device,
    stream).  Two states fed interleaved chains never see each other's levels; inside one
    state a chain interrupted by another geometry hands out nothing computed for the old one."""
    import weakref
    from torchsparse_amd import backend
    geom_a, geom_b = ((2, 2, 2), (2, 2, 2), (0, 0, 0), 2.0), ((3, 3, 3), (2, 2, 2), (1, 1, 1), 2.0)
    mk = lambda: torch.zeros(1, 4, dtype=torch.int32)

    def run_chain(state, geom, length, levels):
        """Calls chain_step like downsample_coords does; returns what each call got."""
        got, c = [], levels[0]
        for i in range(length):
            r = state.chain_step(c, geom)
            got.append(r)
            if isinstance(r, int):
                for j in range(r):  # what the grid path leaves behind for the levels ahead
                    state.ahead[id(levels[i + j + 1])] = (weakref.ref(levels[i + j + 1]), geom,
                                                          levels[i + j + 2], "table%d" % (i + j + 2))
                state.chain_last = weakref.ref(levels[i + 1])
            c = levels[i + 1]
        return got

    s1, s2 = backend._StridedState(), backend._StridedState()
    lv1, lv2 = [mk() for _ in range(6)], [mk() for _ in range(6)]
    assert run_chain(s1, geom_a, 4, lv1) == [0, 0, 0, 0]       # nothing known yet
    assert run_chain(s2, geom_b, 2, lv2) == [0, 0]
    second = run_chain(s1, geom_a, 4, lv1)                      # learnt: 3 levels ahead, then hits
    assert second[0] == 3 and [r[0] is lv1[i + 1] for i, r in enumerate(second[1:], 1)] == [True] * 3
    assert s1.ahead_hits == 3 and s2.ahead_hits == 0 and not s2.ahead
    third = run_chain(s2, geom_b, 2, lv2)                       # the other state learnt its own length
    assert third[0] == 1 and third[1][0] is lv2[2] and s1.chain_len == {geom_a: 4}
    # one state, chains interleaved: A starts (computes ahead), B interrupts, A's next level asks
    assert s1.chain_step(lv1[0], geom_a) == 3
    for j in range(1, 4):
        s1.ahead[id(lv1[j])] = (weakref.ref(lv1[j]), geom_a, lv1[j + 1], "t")
    s1.chain_last = weakref.ref(lv1[1])
    assert s1.chain_step(lv2[0], geom_b) == 0 and not s1.ahead  # B starts: A's levels are dropped
    r = s1.chain_step(lv1[1], geom_a)                           # A resumes as a new chain
    assert isinstance(r, int)
    # a level computed ahead for a tensor that died is not handed to a new tensor at its address
    s3 = backend._StridedState()
    dead = mk()
    s3.ahead[id(dead)] = (weakref.ref(dead), geom_a, lv1[1], "t")
    s3.chain_geom, s3.chain_last = geom_a, weakref.ref(dead)
    key = id(dead)
    del dead
    fresh = mk()
    s3.ahead[id(fresh)] = s3.ahead.pop(key)  # worst case: the allocator reused the address
    assert isinstance(s3.chain_step(fresh, geom_a), int)


def test_coordinate_range_bookkeeping_on_the_host():
    """Which coordinate tensors count as checked: the same object, unchanged; nothing else."""
    from torchsparse_amd import backend
    a = torch.zeros((5, 4), dtype=torch.int32)
    assert not backend._range_known(a)
    backend._mark_range_ok(a)
    assert backend._range_known(a)
    assert not backend._range_known(a.clone())
    a[0, 0] = 1
    assert not backend._range_known(a)
    for _ in range(600):  # the table of checked tensors stays bounded
        backend._mark_range_ok(torch.zeros((1, 4), dtype=torch.int32))
    assert len(backend._range_ok) <= 512
    msg = str(backend._range_error())
    assert "-131072" in msg and "131072)" in msg and "512" in msg
    assert backend.COORD_LIMIT == 1 << 17 and backend.BATCH_LIMIT == 512


def test_buffers_collected_while_recording_outlive_the_tables():
    """backend.pinned(): every library-owned buffer an accessor returns inside the block is
    collected once; dropping the scratch of every stream and pushing seventeen other sizes
    through the identity-map table (it keeps sixteen) leaves the collected tensors where they
    were, with their contents (host tensors stand in for device memory here)."""
    from torchsparse_amd import backend
    cpu = torch.device("cpu", 0)
    with backend.pinned() as held:
        at = backend._scratch(cpu, 1234, 4096)
        assert backend._scratch(cpu, 1234, 100) == at  # same buffer: collected once
        counters = backend._tile_counters(cpu, 1234)
        ident = backend._identity_map(300, cpu)
        w = torch.randn(27, 8, 8)
        w._tsmi_packed = (w._version, w.data_ptr(), torch.zeros(5))
        packed = backend.pack_weights(w)
        with backend.pinned() as inner:  # recordings may nest: both collect
            assert backend._identity_map(300, cpu) is ident
        assert len(inner) == 1 and inner[0] is ident
    assert not backend._pin_sinks
    assert [t.data_ptr() for t in held] == [at, counters.data_ptr(), ident.data_ptr(), packed.data_ptr()]
    backend._identity_map(301, cpu)  # outside the block: not collected
    assert len(held) == 4
    recorded = [t.data_ptr() for t in held]
    backend.release_scratch()
    assert (cpu.index, 1234) not in backend._SCRATCH
    for n in range(1000, 1017):
        backend._identity_map(n, cpu)
    assert (0, 300) not in backend._IDENTITY_MAPS and len(backend._IDENTITY_MAPS) == 16
    w.add_(1)  # a new version of the weights: the cached packing is replaced on the next use
    assert [t.data_ptr() for t in held] == recorded
    assert held[0].numel() >= 4096
    np.testing.assert_array_equal(ident[:300, 0].numpy(), np.arange(300))
    assert (ident[300:] == -1).all() and ident.shape == (384, 1)
    assert backend._scratch(cpu, 1234, 4096) != at  # the table allocates anew; the old block is still held
    backend.release_scratch()
    backend._IDENTITY_MAPS.clear()
    backend._TILE_COUNTERS.pop((0, 1234), None)


def test_launch_thread_without_a_device():
    """The launch thread starts, takes nothing while no device can be asked for its index (or no
    region is open), and flushing and closing return at once."""
    import struct
    from torchsparse_amd import backend
    C = backend._C
    block = struct.pack("21q", *([0] * 21))
    assert C.tsmi_launch_thread_submit(0, block, 21) == -1  # no region open
    assert C.tsmi_launch_thread_open() == 0
    done = C.tsmi_launch_thread_completed().contents.value
    assert C.tsmi_launch_thread_submit(3, block, 21) == -1 and C.tsmi_launch_thread_submit(0, block, 22) == -1
    if not torch.cuda.is_available():
        assert C.tsmi_launch_thread_submit(0, block, 21) == -1  # (no device: the caller makes the call itself)
    assert C.tsmi_launch_thread_flush() == 0
    assert C.tsmi_launch_thread_close() == 0
    assert C.tsmi_launch_thread_completed().contents.value == done
    assert C.tsmi_launch_thread_submit(0, block, 21) == -1
    # the Python region is a no-op without a GPU
    with backend.launch_region() as region:
        assert region.opened == torch.cuda.is_available()
    assert backend._region_depth == 0
