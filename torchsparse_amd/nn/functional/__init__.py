from .activation import *  # noqa: F401,F403
from .conv import *  # noqa: F401,F403
from .conv import conv_config  # noqa: F401
from .count import *  # noqa: F401,F403
from .devoxelize import *  # noqa: F401,F403
from .hash import *  # noqa: F401,F403
from .query import *  # noqa: F401,F403
from .voxelize import *  # noqa: F401,F403
