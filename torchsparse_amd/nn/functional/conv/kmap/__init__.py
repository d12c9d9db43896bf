from .build_kmap import *  # noqa: F401,F403
from .downsample import *  # noqa: F401,F403
from .upsample import *  # noqa: F401,F403
