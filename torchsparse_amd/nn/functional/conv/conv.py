from typing import Dict, List, Optional, Tuple, Union

import torch

from ....tensor import SparseTensor
from ....utils import make_ntuple
from . import conv_config as _cfg
from .conv_mode import get_conv_mode
from .func import (FetchOnDemandConvolutionFuntion, GatherScatterConvolutionFuntion,
                   ImplicitGEMMConvolutionFuntion)
from .kmap import build_kernel_map, transpose_kernel_map

__all__ = ["conv3d", "conv3d_cached"]

_DATAFLOWS = {
    _cfg.Dataflow.ImplicitGEMM: ImplicitGEMMConvolutionFuntion,
    _cfg.Dataflow.GatherScatter: GatherScatterConvolutionFuntion,
    _cfg.Dataflow.FetchOnDemand: FetchOnDemandConvolutionFuntion,
}


def conv3d(input: SparseTensor, weight: torch.Tensor,
           kernel_size: Union[int, List[int], Tuple[int, ...]],
           bias: Optional[torch.Tensor] = None,
           stride: Union[int, List[int], Tuple[int, ...]] = 1,
           padding: Union[int, Tuple[int, ...]] = 0,
           dilation: Union[int, Tuple[int, ...]] = 1, config: Dict = None,
           transposed: bool = False, generative: bool = False,
           training: bool = False, residual: Optional[torch.Tensor] = None,
           activation: Optional[str] = None, out: Optional[torch.Tensor] = None,
           also: Optional[torch.Tensor] = None) -> SparseTensor:
    """Sparse convolution on a SparseTensor (the reference's
    nn/functional/conv/conv.py:15-210): config resolution (per call -> global ->
    default), 1x1x1 fast path, kernel-map cache lookup / build, dataflow dispatch,
    transposed branch, cache propagation to the output tensor.

    Differences kept on purpose: hash tables are cached under the stride of the
    coordinates they index; the config is never mutated; transposed-map products
    are computed once per map; the bias is added inside the kernel epilogue.

    Two optional extras fuse what usually follows a convolution into its epilogue:
    ``residual`` (a [N_out, Cout] tensor added to the result) and ``activation``
    (None or "relu"): output = act(conv(input) + bias + residual).

    ``out`` / ``also`` place the result: it is written into ``out`` (a [N_out, Cout] view with
    unit column stride, e.g. a column slice of a wider buffer) instead of a new tensor, and a
    second time into ``also``.  A layer whose result a later ``cat`` would copy writes it where
    the concatenation wants it; the implicit-GEMM inference launch stores there directly, any
    other path copies."""
    if activation not in (None, "relu"):
        raise ValueError(f"unsupported fused activation: {activation}")
    relu = activation == "relu"
    feats, coords = input.feats, input.coords
    kernel_size = make_ntuple(kernel_size, ndim=3)
    stride = make_ntuple(stride, ndim=3)
    dilation = make_ntuple(dilation, ndim=3)

    if config is None:
        config = _cfg.get_global_conv_config()
        if config is None:
            config = _cfg._shared_default_config(get_conv_mode())
    dataflow = config["dataflow"]
    if dataflow == _cfg.Dataflow.CodedCSR:
        raise AssertionError("CodedCSR has not been integrated.")
    try:
        conv_fn = _DATAFLOWS[dataflow]
    except KeyError:
        raise ValueError("unsupported dataflow: {}".format(dataflow)) from None
    if dataflow != _cfg.Dataflow.ImplicitGEMM and config["ifsort"]:
        config = dict(config, ifsort=False)  # pair-list dataflows never sort
    caches = input._caches
    # the input's own level is registered too, so a transposed layer can return to a
    # level no earlier layer produced (the reference only registers outputs)
    if input.stride not in caches.cmaps:
        caches.cmaps[input.stride] = (coords, input.spatial_range)

    if kernel_size == (1, 1, 1) and stride == (1, 1, 1) and dilation == (1, 1, 1):
        needs_grad = torch.is_grad_enabled() and any(
            t is not None and t.requires_grad for t in (feats, weight, bias, residual))
        if feats.is_cuda and not needs_grad and feats.dtype == weight.dtype and weight.dim() == 2:
            # the implicit-GEMM kernels over the identity map: bias, residual and ReLU fused
            from torchsparse_amd import backend
            out_feats = backend.conv_pointwise_cuda(
                feats, weight, None if bias is None else bias.to(feats.dtype),
                None if residual is None else residual.contiguous(), relu)
        else:
            if feats.is_cuda:
                from torchsparse_amd import backend
                backend.flush_launches()
            out_feats = feats.matmul(weight) if bias is None else torch.addmm(bias, feats, weight)
            if residual is not None:
                out_feats += residual
            if relu:
                out_feats = torch.relu_(out_feats)
        output = SparseTensor._make(out_feats, coords, input.stride, input.spatial_range, caches)
    elif not transposed:
        key = (input.stride, kernel_size, stride, dilation)
        ist = input.stride
        out_stride = (ist[0] * stride[0], ist[1] * stride[1], ist[2] * stride[2])
        kmap = caches.kmaps.get(key)
        if kmap is None:
            in_hashmap = caches.hashmaps.get(input.stride)
            keys, vals = in_hashmap if in_hashmap is not None else (None, None)
            kmap = build_kernel_map(
                coords, feats.shape[0], kernel_size, stride, padding, keys, vals,
                input.spatial_range, config["kmap_mode"], dataflow,
                downsample_mode=config["downsample_mode"], training=training,
                ifsort=config["ifsort"], split_mask_num=config["split_mask_num"],
                split_mask_num_bwd=config["split_mask_num_bwd"])
            caches.kmaps[key] = kmap
            # tables exist only where a map was built through one (unsorted coordinates, "hashmap" mode)
            for level, table in ((input.stride, kmap["in_hashmap"]), (out_stride, kmap["out_hashmap"])):
                if table is not None and caches.hashmaps.get(level) is None:
                    caches.hashmaps[level] = table
        if (weight.dim() == 3 and feats.shape[1] == weight.shape[1]
                and _direct_ok(feats, weight, bias, residual, config)):
            # (what conv_fn.apply comes down to for an inference call in the unsorted implicit GEMM)
            from torchsparse_amd import backend
            out_feats = backend._implicit_gemm(feats, backend.pack_weights(weight), *weight.shape,
                                               kmap["out_in_map"], kmap["sizes"][1], bias, residual, relu,
                                               config.get("pair_segments"), out, also)
            out = also = None  # (placed by the launch)
        else:
            out_feats = conv_fn.apply(feats, weight, kmap, config, False, bias, residual, relu)
        output = SparseTensor._make(out_feats, kmap["coords"], out_stride, kmap["spatial_range"], caches)
    elif generative:
        # generative transposed convolution (conv.py:162-204): outputs are created around
        # every input; the map is never cached and the caches of coarser levels are dropped
        fine_stride = tuple(input.stride[a] // stride[a] for a in range(3))
        kmap = build_kernel_map(
            coords, feats.shape[0], kernel_size, stride, padding, None, None,
            input.spatial_range, config["kmap_mode"], dataflow,
            downsample_mode=config["downsample_mode"], training=training,
            ifsort=config["ifsort"], generative=True, split_mask_num=config["split_mask_num"])
        out_feats = conv_fn.apply(feats, weight, kmap, config, False, bias, residual, relu)
        caches.cmaps[fine_stride] = (kmap["coords"], kmap.get("spatial_range"))
        caches.kmaps = dict()
        caches.hashmaps = dict()
        output = SparseTensor._make(out_feats, kmap["coords"], fine_stride, kmap.get("spatial_range"),
                                    caches)
    else:
        fine_stride = tuple(input.stride[a] // stride[a] for a in range(3))
        kmap = caches.kmaps.get((fine_stride, kernel_size, stride, dilation))
        kmap = transpose_kernel_map(kmap, config["ifsort"], training=training,
                                    split_mask_num=config["split_mask_num"],
                                    split_mask_num_bwd=config["split_mask_num_bwd"])
        if (weight.dim() == 3 and feats.shape[1] == weight.shape[1]
                and _direct_ok(feats, weight, bias, residual, config)):
            from torchsparse_amd import backend
            out_feats = backend._implicit_gemm(feats, backend.pack_weights(weight), *weight.shape,
                                               kmap["out_in_map_t"], kmap["sizes"][0], bias, residual, relu,
                                               config.get("pair_segments"), out, also)
            out = also = None  # (placed by the launch)
        else:
            out_feats = conv_fn.apply(feats, weight, kmap, config, True, bias, residual, relu)
        fine_coords, fine_range = caches.cmaps[fine_stride]
        output = SparseTensor._make(out_feats, fine_coords, fine_stride, fine_range, caches)

    if also is not None or out is not None:  # (a path that does not place its result itself)
        from torchsparse_amd.backend import ColumnSlice, flush_launches
        flush_launches()

        def view(t):
            if t.__class__ is not ColumnSlice:
                return t
            first = (t.ptr - t.buffer.data_ptr()) // t.buffer.element_size()
            return t.buffer[:, first:first + t.cols]
        if also is not None:
            view(also).copy_(output.feats)
        if out is not None:
            view(out).copy_(output.feats)
            output = SparseTensor._make(out.buffer if out.__class__ is ColumnSlice else out, output.coords,
                                        output.stride, output.spatial_range, caches)
    if output.stride not in caches.cmaps:
        caches.cmaps[output.stride] = (output.coords, output.spatial_range)
    return output


def _direct_ok(feats, kernel, bias, residual, config) -> bool:
    """Whether a call may go straight to the unsorted implicit-GEMM launch: that dataflow, no
    gradient to record, operands that need no conversion."""
    if config["dataflow"] != _cfg.Dataflow.ImplicitGEMM or config["ifsort"]:
        return False
    dtype = feats.dtype
    if (not feats.is_cuda or dtype != kernel.dtype or not feats.is_contiguous()
            or (bias is not None and bias.dtype != dtype)
            or (residual is not None and (residual.dtype != dtype or not residual.is_contiguous()))):
        return False
    if torch.is_grad_enabled() and (feats.requires_grad or kernel.requires_grad
                                    or (bias is not None and bias.requires_grad)
                                    or (residual is not None and residual.requires_grad)):
        return False
    return True


def conv3d_cached(input: SparseTensor, kernel: torch.Tensor, bias: Optional[torch.Tensor],
                  kernel_size: Tuple[int, int, int], stride: Tuple[int, int, int],
                  dilation: Tuple[int, int, int], transposed: bool, config: Optional[Dict],
                  residual: Optional[torch.Tensor], activation: Optional[str],
                  out: Optional[torch.Tensor] = None, also: Optional[torch.Tensor] = None) -> Optional[SparseTensor]:
    """The hot case of ``conv3d`` with most of its bookkeeping left out: an inference call
    (no gradient flows) of a real-kernel, non-generative layer in the unsorted implicit-GEMM
    dataflow whose kernel map is already in the tensor's cache and whose operands need no
    conversion.  Returns None for everything else (the caller then takes ``conv3d``); what it
    returns is what ``conv3d`` returns.  Kernel size, stride and dilation come as 3-tuples."""
    if config is None:
        config = _cfg.get_global_conv_config()
        if config is None:
            config = _cfg._shared_default_config(get_conv_mode())
    feats = input.feats
    if not _direct_ok(feats, kernel, bias, residual, config):
        return None
    caches = input._caches
    ist = input.stride
    if kernel.dim() != 3:  # a 1x1x1 stride-1 layer: no map, the outputs are the inputs
        if kernel_size != (1, 1, 1) or stride != (1, 1, 1) or dilation != (1, 1, 1) or feats.shape[0] == 0 \
                or feats.shape[1] != kernel.shape[0] or out is not None or also is not None:
            return None
        from torchsparse_amd import backend
        if ist not in caches.cmaps:
            caches.cmaps[ist] = (input.coords, input.spatial_range)
        out_feats = backend.conv_pointwise_cuda(feats, kernel, bias, residual, activation == "relu")
        return SparseTensor._make(out_feats, input.coords, ist, input.spatial_range, caches)
    if not transposed:
        kmap = caches.kmaps.get((ist, kernel_size, stride, dilation))
        if kmap is None:
            return None
        omap = kmap["out_in_map"]
        n_out = kmap["sizes"][1]
        out_stride = (ist[0] * stride[0], ist[1] * stride[1], ist[2] * stride[2])
        out_coords, out_range = kmap["coords"], kmap["spatial_range"]
    else:
        out_stride = (ist[0] // stride[0], ist[1] // stride[1], ist[2] // stride[2])
        kmap = caches.kmaps.get((out_stride, kernel_size, stride, dilation))
        level = caches.cmaps.get(out_stride)
        if kmap is None or level is None:
            return None
        omap = kmap.get("out_in_map_t")
        if omap is None:
            return None
        n_out = kmap["sizes"][0]
        out_coords, out_range = level
    if ist not in caches.cmaps:
        caches.cmaps[ist] = (input.coords, input.spatial_range)
    from torchsparse_amd import backend
    kvol, cin, cout = kernel.shape
    if feats.shape[1] != cin:
        return None  # (conv3d raises the reference's error)
    out_feats = backend._implicit_gemm(feats, backend.pack_weights(kernel), kvol, cin, cout, omap, n_out,
                                       bias, residual, activation == "relu", config.get("pair_segments"),
                                       out, also)
    output = SparseTensor._make(out_feats, out_coords, out_stride, out_range, caches)
    if out_stride not in caches.cmaps:
        caches.cmaps[out_stride] = (out_coords, out_range)
    return output
