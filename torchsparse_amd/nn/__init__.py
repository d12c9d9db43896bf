from . import functional  # noqa: F401
from .modules import *  # noqa: F401,F403
