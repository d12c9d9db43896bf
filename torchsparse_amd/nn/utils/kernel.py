import itertools
from typing import Tuple, Union

import numpy as np
import torch

from ...utils import make_ntuple

__all__ = ["get_kernel_offsets"]


def get_kernel_offsets(size: Union[int, Tuple[int, ...]], stride: Union[int, Tuple[int, ...]] = 1,
                       dilation: Union[int, Tuple[int, ...]] = 1, device="cpu") -> torch.Tensor:
    """Canonical [K_vol, 3] offset table; row k is the offset weight k applies to.

    Per axis the offsets run from -size//2 + 1 to size//2 (so 3 -> -1..1, 2 -> 0..1),
    scaled by stride*dilation.  An odd kernel volume enumerates x fastest, an even
    one z fastest — the same convention the kernel-map kernels use
    (the reference's nn/utils/kernel.py:21-35)."""
    size, stride, dilation = (make_ntuple(v, ndim=3) for v in (size, stride, dilation))
    axes = [np.arange(-size[a] // 2 + 1, size[a] // 2 + 1) * stride[a] * dilation[a] for a in range(3)]
    if int(np.prod(size)) % 2 == 1:
        rows = [(x, y, z) for z, y, x in itertools.product(axes[2], axes[1], axes[0])]
    else:
        rows = list(itertools.product(axes[0], axes[1], axes[2]))
    return torch.tensor(np.array(rows, dtype=np.int32).reshape(-1, 3), dtype=torch.int, device=device)
