from .apply import fapply  # noqa: F401
from .kernel import get_kernel_offsets  # noqa: F401
from .fuse import fuse_inference  # noqa: F401
