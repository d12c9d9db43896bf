from .fetch_on_demand import *  # noqa: F401,F403
from .gather_scatter import *  # noqa: F401,F403
from .implicit_gemm import *  # noqa: F401,F403
