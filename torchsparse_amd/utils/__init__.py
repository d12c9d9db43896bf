from .utils import make_divisible, make_ntuple, make_tensor
from .tensor_cache import (TensorCache, TensorCacheMode, clear_global_tensor_cache,
                           get_global_tensor_cache, get_tensor_cache_mode,
                           set_global_tensor_cache, set_tensor_cache_mode)

from .to_dense import to_dense

__all__ = ["to_dense", "make_ntuple", "make_tensor", "make_divisible", "TensorCache", "TensorCacheMode",
           "set_tensor_cache_mode", "get_tensor_cache_mode", "get_global_tensor_cache",
           "set_global_tensor_cache", "clear_global_tensor_cache"]
