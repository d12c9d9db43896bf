"""Convolution configuration knobs (the reference's
nn/functional/conv/conv_config.py:8-94).

A config is a dict whose keys are also attributes (``config.dataflow``,
``config["epsilon"]``, ``config.copy()``).  Unlike the reference,
get_default_conv_config() hands out a fresh copy each time, so a caller editing it
cannot change what other layers see."""
from enum import Enum

from .conv_mode import ConvMode

__all__ = ["Dataflow", "AttributeDict", "get_default_conv_config", "get_global_conv_config",
           "set_global_conv_config", "clear_global_conv_config", "keys_check"]


class Dataflow(Enum):
    ImplicitGEMM = 0
    GatherScatter = 1
    FetchOnDemand = 2
    CodedCSR = 3


class AttributeDict(dict):
    """dict with attribute access to its keys."""

    def __getattr__(self, key):
        try:
            return self[key]
        except KeyError:
            raise AttributeError(key) from None

    def __setattr__(self, key, value):
        self[key] = value

    def __delattr__(self, key):
        try:
            del self[key]
        except KeyError:
            raise AttributeError(key) from None

    def copy(self):
        return AttributeDict(self)


_DEFAULTS = (
    ("dataflow", Dataflow.ImplicitGEMM),
    ("ifsort", False),
    ("kmap_mode", "hashmap_on_the_fly"),
    ("downsample_mode", "spconv"),
    ("split_mask_num", 1),
    ("split_mask_num_bwd", 3),
    ("epsilon", 0.0),
    ("mm_thresh", 0),
    ("FOD_fusion", True),
    # implicit GEMM over pair segments on small, wide layers: None = where the library knows the
    # map to be thin, True = wherever the kernels have a variant, False = never (the tuner times both)
    ("pair_segments", None),
)

_global_conv_config = None


def keys_check(conv_config) -> None:
    """Fill missing fields with their defaults (and say so once)."""
    missing = [k for k, _ in _DEFAULTS if k not in conv_config]
    for k, v in _DEFAULTS:
        if k not in conv_config:
            conv_config[k] = v
    if missing:
        print("Warning: Missing fields for ConvConfig. Use default configs for these fields.")


def get_global_conv_config():
    return _global_conv_config


def set_global_conv_config(conv_config) -> None:
    global _global_conv_config
    keys_check(conv_config)
    _global_conv_config = conv_config


def clear_global_conv_config() -> None:
    global _global_conv_config
    _global_conv_config = None


_SHARED_DEFAULTS = {}


def _shared_default_config(conv_mode: ConvMode):
    """One read-only default config per conv mode for conv3d's own use (never handed
    to callers, never mutated)."""
    cfg = _SHARED_DEFAULTS.get(conv_mode)
    if cfg is None:
        cfg = _SHARED_DEFAULTS[conv_mode] = get_default_conv_config(conv_mode)
    return cfg


def get_default_conv_config(conv_mode: ConvMode = ConvMode.mode0, training: bool = False):
    config = AttributeDict(_DEFAULTS)
    if conv_mode == ConvMode.mode1:
        config.ifsort = True
    elif conv_mode == ConvMode.mode2:
        config.ifsort = True
        config.split_mask_num = 3
    return config
