from .blocks import *  # noqa: F401,F403
