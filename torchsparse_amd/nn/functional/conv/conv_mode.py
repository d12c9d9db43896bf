"""Global kernel-map / downsample / conv modes (the reference's
nn/functional/conv/conv_mode.py:3-65)."""
from enum import Enum

__all__ = ["ConvMode", "get_kmap_mode", "set_kmap_mode", "get_downsample_mode",
           "set_downsample_mode", "get_conv_mode", "set_conv_mode"]

_KMAP_MODES = ("hashmap_on_the_fly", "hashmap")
_DOWNSAMPLE_MODES = ("spconv", "minkowski")


class ConvMode(Enum):
    mode0 = 0  # unsorted forward
    mode1 = 1  # sorted forward, one mask split
    mode2 = 2  # sorted forward, three mask splits


_state = {"kmap": "hashmap_on_the_fly", "downsample": "spconv", "conv": ConvMode.mode0}


def get_kmap_mode() -> str:
    return _state["kmap"]


def set_kmap_mode(kmap_mode: str) -> None:
    assert kmap_mode in _KMAP_MODES, (
        f'Unsupport kmap_mode: {kmap_mode}. Please set kmap_mode to "hashmap_on_the_fly" or "hashmap".')
    _state["kmap"] = kmap_mode


def get_downsample_mode() -> str:
    return _state["downsample"]


def set_downsample_mode(downsample_mode: str) -> None:
    assert downsample_mode in _DOWNSAMPLE_MODES, (
        f'Unsupport downsample_mode {downsample_mode}. Please set downsample_mode to "spconv" or "minkowski".')
    _state["downsample"] = downsample_mode


def get_conv_mode() -> ConvMode:
    return _state["conv"]


def set_conv_mode(conv_mode) -> None:
    if isinstance(conv_mode, int):
        assert conv_mode in (0, 1, 2), f"Undefined conv_mode:{conv_mode}"
        conv_mode = ConvMode(conv_mode)
    assert isinstance(conv_mode, ConvMode), "Unsupport conv_mode input type"
    _state["conv"] = conv_mode
