from typing import Dict, Optional

import torch

from torchsparse_amd import backend, backends
from .gather_scatter import _center_offset
from .implicit_gemm import _coerce

from .autograd import differentiable  # noqa: E402

__all__ = ["FetchOnDemandConvolutionFuntion"]


class FetchOnDemandConvolutionFuntion:
    """Forward of the fetch-on-demand dataflow (the reference's
    func/fetch_on_demand.py:17-111): input rows are fetched through the pair lists
    inside the GEMM kernel, no gathered copy is materialised.  ``FOD_fusion`` is
    read for compatibility; all offsets always run in one launch."""

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
        nbmaps = kmap["nbmaps"]  # int32 [2, nnz]
        kvol = weight.shape[0] if weight.dim() == 3 else 1
        out = backend.conv_forward_fetch_on_demand_cuda(
            input, weight, nbmaps, nbmaps.size(1), kmap["nbaddrs"], kmap["qnbaddrs"],
            sizes[0] if transposed else sizes[1], int(kmap["qmapsize"]), transposed,
            backends.allow_tf32, backends.allow_fp16,
            row_mask=kmap["input_mask"] if transposed else kmap["output_mask"],
            center_k=_center_offset(kmap, kvol), bias=bias, residual=residual, relu=relu)
        return out if out.dtype == out_dtype else out.to(out_dtype)


FetchOnDemandConvolutionFuntion.apply = staticmethod(differentiable(FetchOnDemandConvolutionFuntion._forward))
