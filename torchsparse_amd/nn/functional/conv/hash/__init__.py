from .query import *  # noqa: F401,F403
