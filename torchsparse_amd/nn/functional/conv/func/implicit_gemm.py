from typing import Dict, Optional

import torch

from torchsparse_amd import backend, backends

from .autograd import differentiable  # noqa: E402

__all__ = ["ImplicitGEMMConvolutionFuntion"]


def _coerce(input: torch.Tensor, weight: torch.Tensor):
    """If either operand is half precision both are used in half
    (the reference's func/implicit_gemm.py:64-66)."""
    if input.dtype != weight.dtype:
        for dt in (torch.float16, torch.bfloat16):
            if dt in (input.dtype, weight.dtype):
                return input.to(dt), weight.to(dt)
        weight = weight.to(input.dtype)
    return input, weight


class ImplicitGEMMConvolutionFuntion:
    """The implicit-GEMM dataflow (the reference's func/implicit_gemm.py:15-190);
    ``apply`` is differentiable (func/autograd.py)."""

    @staticmethod
    def _forward(input: torch.Tensor, weight: torch.Tensor, kmap: Dict, config: Dict,
                 transposed: bool = False, bias: Optional[torch.Tensor] = None,
                 residual: Optional[torch.Tensor] = None, relu: bool = False) -> torch.Tensor:
        sizes = kmap["sizes"]
        sfx = "_t" if transposed else ""
        num_out_feats = sizes[0] if transposed else sizes[1]
        out_dtype = weight.dtype
        input, weight = _coerce(input, weight)
        if bias is not None and bias.dtype != input.dtype:
            bias = bias.to(input.dtype)
        if residual is not None and residual.dtype != input.dtype:
            residual = residual.to(input.dtype)
        if not config["ifsort"]:
            out = backend.conv_forward_implicit_gemm_cuda(
                input, weight, kmap["out_in_map" + sfx], num_out_feats, weight.shape[-1],
                backends.allow_tf32, backends.allow_fp16, bias=bias, residual=residual, relu=relu,
                segments=config.get("pair_segments"))
        else:
            out = backend.conv_forward_implicit_gemm_sorted_cuda(
                input, weight, kmap["reorder_out_in_map" + sfx], kmap["reduced_sorted_mask" + sfx],
                kmap["reorder_loc" + sfx], num_out_feats, weight.shape[-1],
                backends.allow_tf32, backends.allow_fp16, bias=bias, residual=residual, relu=relu)
        return out if out.dtype == out_dtype else out.to(out_dtype)


ImplicitGEMMConvolutionFuntion.apply = staticmethod(differentiable(ImplicitGEMMConvolutionFuntion._forward))
