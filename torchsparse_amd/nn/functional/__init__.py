from .activation import *  # noqa: F401,F403
from .conv import *  # noqa: F401,F403
from .conv import conv_config  # noqa: F401
