from . import conv_config  # noqa: F401
from .conv import *  # noqa: F401,F403
from .conv_config import *  # noqa: F401,F403
from .conv_mode import *  # noqa: F401,F403
from .func import *  # noqa: F401,F403
from .hash import *  # noqa: F401,F403
from .kmap import *  # noqa: F401,F403
