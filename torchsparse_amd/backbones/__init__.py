from .detection import *  # noqa: F401,F403
from .resnet import *  # noqa: F401,F403
from .unet import *  # noqa: F401,F403
