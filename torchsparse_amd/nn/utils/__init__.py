from .apply import fapply  # noqa: F401
from .kernel import get_kernel_offsets  # noqa: F401
