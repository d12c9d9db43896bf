"""torchsparse_amd: the forward sparse-convolution hot path of TorchSparse++ for
AMD MI355X (gfx950), behind the reference's own Python API.

    import torchsparse_amd as torchsparse
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.nn import functional as F
"""
from . import backends
from .operators import *  # noqa: F401,F403
from .tensor import *  # noqa: F401,F403
from .version import __version__  # noqa: F401

backends.init()
