"""SparseTensor: features [N, C] + integer coordinates [N, 4] = (batch, x, y, z)
(the reference's torchsparse/tensor.py:29-110)."""
from typing import Optional, Tuple, Union

import torch

from .utils import make_ntuple
from .utils.tensor_cache import (TensorCache, TensorCacheMode, get_global_tensor_cache,
                                 get_tensor_cache_mode, set_global_tensor_cache)

__all__ = ["SparseTensor", "PointTensor", "get_allow_negative_coordinates",
           "set_allow_negative_coordinates"]

_allow_negative_coordinates = False


def get_allow_negative_coordinates() -> bool:
    return _allow_negative_coordinates


def set_allow_negative_coordinates(flag: bool) -> None:
    """Let strided convolutions produce outputs at negative coordinates (tensor.py:24-26):
    the lower bound of the output range becomes the reference's coords_min instead of 0.
    Submanifold maps and the hash tables accept coordinates in [-2^17, 2^17) either way."""
    global _allow_negative_coordinates
    _allow_negative_coordinates = bool(flag)


class SparseTensor:
    def __init__(self, feats: torch.Tensor, coords: torch.Tensor,
                 stride: Union[int, Tuple[int, ...]] = 1,
                 spatial_range: Optional[Tuple[int, ...]] = None) -> None:
        self.feats = feats
        self.coords = coords
        self.stride = make_ntuple(stride, ndim=3)
        self.spatial_range = None if spatial_range is None else make_ntuple(
            spatial_range, ndim=len(spatial_range))
        if get_tensor_cache_mode() == TensorCacheMode.GLOBAL_TENSOR_CACHE:
            cache = get_global_tensor_cache()
            if cache is None:
                cache = TensorCache()
                set_global_tensor_cache(cache)
            self._caches = cache
        else:
            self._caches = TensorCache()

    # short aliases used throughout user code
    F = property(lambda self: self.feats, lambda self, v: setattr(self, "feats", v))
    C = property(lambda self: self.coords, lambda self, v: setattr(self, "coords", v))
    s = property(lambda self: self.stride,
                 lambda self, v: setattr(self, "stride", make_ntuple(v, ndim=3)))

    @classmethod
    def _make(cls, feats, coords, stride, spatial_range, caches) -> "SparseTensor":
        """Constructor for already-normalised fields (used on the convolution path)."""
        out = cls.__new__(cls)
        out.feats, out.coords = feats, coords
        out.stride, out.spatial_range = stride, spatial_range
        out._caches = caches
        return out

    def _like(self, feats: torch.Tensor) -> "SparseTensor":
        out = SparseTensor.__new__(SparseTensor)
        out.feats, out.coords = feats, self.coords
        out.stride, out.spatial_range = self.stride, self.spatial_range
        out._caches = self._caches
        return out

    def cpu(self):
        self.coords, self.feats = self.coords.cpu(), self.feats.cpu()
        return self

    def cuda(self):
        self.coords, self.feats = self.coords.cuda(), self.feats.cuda()
        return self

    def half(self):
        self.feats = self.feats.half()
        return self

    def detach(self):
        self.coords, self.feats = self.coords.detach(), self.feats.detach()
        return self

    def to(self, device, non_blocking: bool = True):
        self.coords = self.coords.to(device, non_blocking=non_blocking)
        self.feats = self.feats.to(device, non_blocking=non_blocking)
        return self

    def dense(self) -> torch.Tensor:
        """[B, X, Y, Z, C] dense tensor (needs spatial_range)."""
        assert self.spatial_range is not None
        from .utils.to_dense import to_dense
        return to_dense(self.feats, self.coords, self.spatial_range)

    def __add__(self, other: "SparseTensor") -> "SparseTensor":
        if self.feats.is_cuda:
            from . import backend
            backend.flush_launches()  # (either operand may still be with the launch thread)
        return self._like(self.feats + other.feats)


class PointTensor:
    """Features [N, C] at floating-point positions [N, 4], with the per-stride voxel indices
    and interpolation weights point-voxel networks cache on it
    (the reference's torchsparse/tensor.py:116-140)."""

    def __init__(self, feats, coords, idx_query=None, weights=None):
        self.F = feats
        self.C = coords
        self.idx_query = idx_query if idx_query is not None else {}
        self.weights = weights if weights is not None else {}
        self.additional_features = {"idx_query": {}, "counts": {}}

    def cuda(self):
        self.F, self.C = self.F.cuda(), self.C.cuda()
        return self

    def detach(self):
        self.F, self.C = self.F.detach(), self.C.detach()
        return self

    def to(self, device, non_blocking: bool = True):
        self.F = self.F.to(device, non_blocking=non_blocking)
        self.C = self.C.to(device, non_blocking=non_blocking)
        return self
