"""Backward of the sparse convolution, shared by the three dataflows.

    dX[m]  += dY[i] W[k]^T          (input gradient)
    dW[k]  += X[m]^T dY[i]          for every map entry  map[i, k] = m >= 0

The input gradient is the forward implicit-GEMM kernel over the transposed map with
the weights transposed per offset; a sorted configuration (``ifsort``) whose map carries
the backward sort products runs it over the mask-sorted transposed map, as the
reference's sorted branch does.  The weight gradient runs over per-offset pair lists
derived from the map (tsmi_conv_wgrad_pairs: only rows that take part in an offset are
read); channel counts that are not a multiple of 16 bytes use the map form
(tsmi_conv_wgrad).  Both follow the reference's func/implicit_gemm.py:108-190 (unsorted
branch); the gather-scatter and fetch-on-demand dataflows get the same gradients from
the same maps (the reference computes theirs with conv_backward_gather_scatter_cuda,
func/gather_scatter.py:104-160 — same sums)."""
from typing import Callable, Dict

import torch

from torchsparse_amd import backend
from torchsparse_amd.utils import make_divisible

__all__ = ["SparseConvFunction", "backward_map", "backward_sort_products", "wgrad_pairs"]


def backward_map(kmap: Dict, transposed: bool) -> torch.Tensor:
    """(input row, offset) -> output row of the convolution, int32 [ceil128(N_in), K_vol].
    For a transposed convolution that is the strided map itself; otherwise the transposed
    map, built once and kept under ``out_in_map_bwd`` (build_kmap.py:191-194)."""
    if transposed:
        return kmap["out_in_map"]
    if kmap.get("out_in_map_bwd") is None:
        if kmap.get("out_in_map_t") is not None:  # a transposed convolution already built it
            kmap["out_in_map_bwd"] = kmap["out_in_map_t"]
        else:
            n_in, n_out = kmap["sizes"]
            kmap["out_in_map_bwd"] = backend.convert_transposed_out_in_map(
                kmap["out_in_map"], make_divisible(n_in, 128), n_out)
    return kmap["out_in_map_bwd"]


def backward_sort_products(kmap: Dict, transposed: bool):
    """(mask-sorted backward map, its reduced masks for 128-row tiles, row order) when the map
    was built with them, else None.  A plain convolution's are the ``*_bwd`` products of a
    training-time sorted map (build_kmap.py:195-220); a transposed convolution runs its
    input gradient over the strided map itself, whose products are the forward ones."""
    names = (("reorder_out_in_map", "reduced_sorted_mask", "reorder_loc") if transposed else
             ("reorder_out_in_map_bwd", "reduced_sorted_mask_bwd_dgrad", "reorder_loc_bwd"))
    products = tuple(kmap.get(n) for n in names)
    return None if any(p is None for p in products) else products


def wgrad_pairs(kmap: Dict) -> Dict:
    """Per-offset (input row, output row) pair lists of the strided / submanifold map, built
    once per map and shared by every convolution (transposed ones included) that uses it."""
    if kmap.get("wgrad_pairs") is None:
        kmap["wgrad_pairs"] = backend.wgrad_pair_lists(kmap["out_in_map"], kmap["sizes"][1])
    return kmap["wgrad_pairs"]


class SparseConvFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input: torch.Tensor, weight: torch.Tensor, kmap: Dict, config: Dict,
                transposed: bool, forward_impl: Callable) -> torch.Tensor:
        out = forward_impl(input, weight, kmap, config, transposed, None, None, False)
        ctx.save_for_backward(input, weight)
        ctx.kmap, ctx.transposed = kmap, transposed
        ctx.ifsort = bool(config.get("ifsort", False)) if config is not None else False
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        input, weight = ctx.saved_tensors
        kmap, transposed = ctx.kmap, ctx.transposed
        from .implicit_gemm import _coerce
        x, w = _coerce(input.detach(), weight.detach())
        if w.dim() == 2:
            w = w.unsqueeze(0)
        dy = grad_output.contiguous()
        if dy.dtype != x.dtype:
            dy = dy.to(x.dtype)
        sizes = kmap["sizes"]
        n_in = sizes[1] if transposed else sizes[0]
        grad_input = grad_weight = None
        if dy.shape[0] == 0 or x.shape[0] == 0:  # no outputs (or no inputs): nothing flows back
            return (torch.zeros_like(input) if ctx.needs_input_grad[0] else None,
                    torch.zeros_like(weight) if ctx.needs_input_grad[1] else None, None, None, None, None)
        if ctx.needs_input_grad[0]:
            products = backward_sort_products(kmap, transposed) if ctx.ifsort else None
            if products is not None:
                grad_input = backend.conv_dgrad_implicit_gemm_sorted_cuda(dy, w, *products, n_in)
            else:
                grad_input = backend.conv_dgrad_implicit_gemm_cuda(
                    dy, w, backward_map(kmap, transposed), n_in)
            if grad_input.dtype != input.dtype:
                grad_input = grad_input.to(input.dtype)
        if ctx.needs_input_grad[1]:
            if backend.wgrad_pairs_supported(x, dy, w.shape[0]):
                # the map's values index the strided convolution's input: x for a plain
                # convolution (column 0), dy for a transposed one
                grad_weight = backend.conv_backward_wgrad_pairs_cuda(
                    dy, x, wgrad_pairs(kmap), 1 if transposed else 0)
            else:
                grad_weight = backend.conv_backward_wgrad_implicit_gemm_cuda(
                    dy, x, backward_map(kmap, transposed), n_in)
            grad_weight = grad_weight.reshape(weight.shape)
            if grad_weight.dtype != weight.dtype:
                grad_weight = grad_weight.to(weight.dtype)
        return grad_input, grad_weight, None, None, None, None


def differentiable(forward_impl: Callable):
    """Wrap a dataflow's forward: with autograd active the convolution goes through
    SparseConvFunction and bias / residual / ReLU are applied by autograd-aware ops."""
    def apply(input, weight, kmap, config, transposed=False, bias=None, residual=None, relu=False):
        if torch.is_grad_enabled() and any(
                t is not None and t.requires_grad for t in (input, weight, bias, residual)):
            if input.requires_grad or weight.requires_grad:
                out = SparseConvFunction.apply(input, weight, kmap, config, transposed, forward_impl)
            else:  # only the bias or the residual is trainable: they enter through torch ops below
                out = forward_impl(input, weight, kmap, config, transposed, None, None, False)
            if bias is not None:
                out = out + bias.to(out.dtype)
            if residual is not None:
                out = out + residual.to(out.dtype)
            return torch.relu(out) if relu else out
        return forward_impl(input, weight, kmap, config, transposed, bias, residual, relu)
    return apply
