from typing import Dict, Optional

import torch

from torchsparse_amd import backend
from .implicit_gemm import _coerce

from .autograd import differentiable  # noqa: E402

__all__ = ["GatherScatterConvolutionFuntion"]


def _center_offset(kmap: Dict, kvol: int) -> int:
    """Index of the identity offset of an odd-volume submanifold map (its pairs are (i, i) in
    row order, so the scatter needs no mask look-up for it), or -1.  Decided by the map's
    geometry: a strided map can have as many outputs as inputs without being one (the
    reference tells by the sizes, convolution_gather_scatter_cuda.cu:497-499)."""
    return kvol // 2 if (kmap.get("subm", False) and kvol % 2 == 1) else -1


class GatherScatterConvolutionFuntion:
    """Forward of the gather-GEMM-scatter dataflow (the reference's
    func/gather_scatter.py:16-102).  ``epsilon`` / ``mm_thresh`` are read from the
    config for compatibility; they never change the result."""

    @staticmethod
    def _forward(input: torch.Tensor, weight: torch.Tensor, kmap: Dict, config: Dict,
                 transposed: bool = False, bias: Optional[torch.Tensor] = None,
                 residual: Optional[torch.Tensor] = None, relu: bool = False) -> torch.Tensor:
        sizes = kmap["sizes"]
        out_dtype = weight.dtype
        input, weight = _coerce(input, weight)
        if bias is not None and bias.dtype != input.dtype:
            bias = bias.to(input.dtype)
        if residual is not None and residual.dtype != input.dtype:
            residual = residual.to(input.dtype)
        nbmaps = kmap["nbmaps"]
        if nbmaps.dtype != torch.int32:
            nbmaps = nbmaps.int()
        kvol = weight.shape[0] if weight.dim() == 3 else 1
        out = backend.conv_forward_gather_scatter_cuda(
            input, weight, nbmaps, kmap["nbsizes"], kmap["input_mask"], kmap["output_mask"],
            sizes[0] if transposed else sizes[1], config["epsilon"], int(config["mm_thresh"]), 0,
            transposed, None, nbaddrs=kmap.get("nbaddrs"), qnbaddrs=kmap.get("qnbaddrs"),
            qsum_nnz=None if kmap.get("qmapsize") is None else int(kmap["qmapsize"]),
            center_k=_center_offset(kmap, kvol), bias=bias, residual=residual, relu=relu)
        return out if out.dtype == out_dtype else out.to(out_dtype)


GatherScatterConvolutionFuntion.apply = staticmethod(differentiable(GatherScatterConvolutionFuntion._forward))
