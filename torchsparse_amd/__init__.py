"""torchsparse_amd: the forward sparse-convolution hot path of TorchSparse++ for
AMD MI355X (gfx950), behind the reference's own Python API.

    import torchsparse_amd as torchsparse
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.nn import functional as F

or, for code that must keep its ``import torchsparse`` lines (model files, plugins):

    import torchsparse_amd
    torchsparse_amd.install_as("torchsparse")
    import torchsparse, torchsparse.nn as spnn          # the same module objects
"""
import importlib
import importlib.abc
import importlib.util
import sys

from . import backends
from .operators import *  # noqa: F401,F403
from .tensor import *  # noqa: F401,F403
from .version import __version__  # noqa: F401

backends.init()


def __getattr__(name):
    # torchsparse/__init__.py:5 exports tune at the top level; imported on first use because
    # utils.tune itself imports this package
    if name == "tune":
        from .utils.tune import tune
        return tune
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")


class _AliasFinder(importlib.abc.MetaPathFinder, importlib.abc.Loader):
    """Resolves ``alias`` and ``alias.x.y`` to the module objects of this package, so that
    ``alias.nn is torchsparse_amd.nn``: one set of classes, one set of process-wide switches."""

    def __init__(self, alias: str):
        self.alias = alias

    def _real(self, fullname: str):
        if fullname == self.alias or fullname.startswith(self.alias + "."):
            return __name__ + fullname[len(self.alias):]
        return None

    def find_spec(self, fullname, path=None, target=None):
        real = self._real(fullname)
        if real is None:
            return None
        try:
            importlib.import_module(real)
        except ModuleNotFoundError as e:
            if e.name == real:  # no such sub-module here: let the import fail under the alias
                return None
            raise
        return importlib.util.spec_from_loader(fullname, self)

    def create_module(self, spec):
        return sys.modules[self._real(spec.name)]

    def exec_module(self, module):
        pass


def install_as(alias: str = "torchsparse") -> None:
    """Make ``import <alias>`` (and every ``<alias>.sub.module``) give this package, so that
    code written against the reference's import block (backbones/unet.py:5-9) runs unchanged.
    Refuses to shadow a different package already imported under that name."""
    this = sys.modules[__name__]
    have = sys.modules.get(alias)
    if have is not None and have is not this:
        raise ImportError(f"a different module is already imported as {alias!r}: {have!r}")
    if not any(isinstance(f, _AliasFinder) and f.alias == alias for f in sys.meta_path):
        sys.meta_path.insert(0, _AliasFinder(alias))
    for name in [n for n in sys.modules if n == __name__ or n.startswith(__name__ + ".")]:
        sys.modules[alias + name[len(__name__):]] = sys.modules[name]
