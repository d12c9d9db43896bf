"""Per-input caches shared by every tensor derived from one SparseTensor
(the reference's torchsparse/utils/tensor_cache.py:33-39):

  cmaps[stride]                   -> (coords, spatial_range) of that stride level
  kmaps[(stride, ks, s, dil)]     -> kernel-map dict
  hashmaps[stride]                -> (hashmap_keys, hashmap_vals) indexing the
                                     coordinates of that stride level
"""
from enum import Enum


class TensorCacheMode(Enum):
    SEPARATE_TENSOR_CACHE = 0
    GLOBAL_TENSOR_CACHE = 1


class TensorCache:
    __slots__ = ("cmaps", "kmaps", "hashmaps")

    def __init__(self) -> None:
        self.cmaps = {}
        self.kmaps = {}
        self.hashmaps = {}


_mode = TensorCacheMode.SEPARATE_TENSOR_CACHE
_global_cache = None


def set_tensor_cache_mode(mode: TensorCacheMode) -> None:
    """With GLOBAL_TENSOR_CACHE every new SparseTensor shares one cache, which the
    caller must clear after each forward pass."""
    global _mode
    assert isinstance(mode, TensorCacheMode), "Input must be an instance of TensorCacheMode"
    _mode = mode


def get_tensor_cache_mode() -> TensorCacheMode:
    return _mode


def get_global_tensor_cache():
    return _global_cache


def set_global_tensor_cache(cache) -> None:
    global _global_cache
    _global_cache = cache


def clear_global_tensor_cache() -> None:
    set_global_tensor_cache(None)
