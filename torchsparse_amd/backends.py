"""Process-wide switches read by the convolution path (the reference's
torchsparse/backends.py:4-11).  Unlike the reference nothing here queries the
device at import time.

  benchmark       GatherScatter: the reference switches to its fused kernels; here
                  the fused three-launch pipeline is always used.
  allow_tf32      accepted for compatibility; fp32 convolutions run in true fp32.
  allow_fp16      accepted for compatibility; gfx950 always has fp16/bf16 MFMA.
  hash_rsv_ratio  hash-table slots reserved per input voxel (>= 2).
"""
benchmark = False
allow_tf32 = True
allow_fp16 = True
hash_rsv_ratio = 2


def init():
    """Kept so that code calling torchsparse.backends.init() keeps working."""
    global benchmark, allow_tf32, allow_fp16, hash_rsv_ratio
    benchmark = False
    allow_tf32 = True
    allow_fp16 = True
    hash_rsv_ratio = 2
