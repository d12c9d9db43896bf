"""SpConv checkpoints -> this library's kernel layout (the reference's examples/converter.py).

A sparse convolution weight here is ``kernel [K_vol, Cin, Cout]`` (``[Cin, Cout]`` when
K_vol = 1) whose row k applies to offset ``get_kernel_offsets(size)[k]``: an odd kernel
volume enumerates x fastest, an even one z fastest.  SpConv keeps the three kernel axes
separate and flattens them x-major:

    SpConv v1  weight [kx, ky, kz, Cin, Cout]      (examples/converter.py:54-90)
    SpConv v2  weight [Cout, kx, ky, kz, Cin]      (examples/converter.py:14-51)

so a conversion is a transpose of the channel axes plus, for odd volumes, the x<->z
reordering of the offsets.  Keys are renamed ``*.weight`` -> ``*.kernel``.

Differences from the reference, on purpose:
  * every odd kernel volume is reordered, not only 27 (the reference leaves e.g. 5x5x5
    and 3x3x1 kernels in SpConv order, which is not the order its own offset table uses);
  * sparse convolution weights are recognised by the class NAME of the module that owns
    them (SubMConv3d, SparseConv3d, SparseInverseConv3d, ...), or by an explicit key
    list, so SpConv itself need not be importable;
  * checkpoints are read with ``torch.load(weights_only=True)``.
"""
from typing import Dict, Iterable, Optional, Tuple

import torch

__all__ = ["convert_weights_v1", "convert_weights_v2", "convert_state_dict", "convert_model_weights",
           "sparse_conv_weight_keys"]

_SPCONV_CLASSES = {
    "SparseConv1d", "SparseConv2d", "SparseConv3d", "SparseConv4d",
    "SubMConv1d", "SubMConv2d", "SubMConv3d", "SubMConv4d",
    "SparseConvTranspose1d", "SparseConvTranspose2d", "SparseConvTranspose3d",
    "SparseInverseConv1d", "SparseInverseConv2d", "SparseInverseConv3d",
}


def _reorder(w: torch.Tensor, sizes: Tuple[int, int, int]) -> torch.Tensor:
    """[kx*ky*kz (x-major), Cin, Cout] -> rows in this library's offset order."""
    kx, ky, kz = sizes
    kvol = kx * ky * kz
    if kvol == 1:
        return w[0]
    if kvol % 2 == 0:
        return w  # even volumes enumerate z fastest: the x-major flattening already
    index = [(x * ky + y) * kz + z for z in range(kz) for y in range(ky) for x in range(kx)]
    return w[torch.tensor(index, dtype=torch.int64, device=w.device)]


def convert_weights_v1(key: str, model: Dict[str, torch.Tensor]) -> Tuple[str, torch.Tensor]:
    """One SpConv v1 weight ``model[key]`` of shape [kx, ky, kz, Cin, Cout]."""
    w = model[key]
    if w.dim() != 5:
        raise ValueError(f"{key}: expected a 5-d SpConv v1 weight, got shape {tuple(w.shape)}")
    kx, ky, kz, cin, cout = w.shape
    return key.replace(".weight", ".kernel"), _reorder(w.reshape(-1, cin, cout), (kx, ky, kz)).contiguous()


def convert_weights_v2(key: str, model: Dict[str, torch.Tensor]) -> Tuple[str, torch.Tensor]:
    """One SpConv v2 weight ``model[key]`` of shape [Cout, kx, ky, kz, Cin]."""
    w = model[key]
    if w.dim() != 5:
        raise ValueError(f"{key}: expected a 5-d SpConv v2 weight, got shape {tuple(w.shape)}")
    cout, kx, ky, kz, cin = w.shape
    flat = w.reshape(cout, -1, cin).permute(1, 2, 0)
    return key.replace(".weight", ".kernel"), _reorder(flat, (kx, ky, kz)).contiguous()


def sparse_conv_weight_keys(model: torch.nn.Module) -> Iterable[str]:
    """State-dict keys of the sparse convolution weights of ``model``: ``<module>.weight`` of
    every module whose class is one of SpConv's convolution classes (matched by name)."""
    return [f"{name}.weight" for name, m in model.named_modules()
            if any(c.__name__ in _SPCONV_CLASSES for c in type(m).__mro__)]


def convert_state_dict(state_dict: Dict[str, torch.Tensor], sparse_keys: Optional[Iterable[str]] = None,
                       legacy: bool = False) -> Dict[str, torch.Tensor]:
    """Convert the weights named in ``sparse_keys`` (default: every 5-d ``*.weight``) from the
    SpConv v1 (``legacy=True``) or v2 layout; every other entry is passed through."""
    if sparse_keys is None:
        keys = {k for k, v in state_dict.items() if k.endswith(".weight") and v.dim() == 5}
    else:
        keys = set(sparse_keys)
    convert = convert_weights_v1 if legacy else convert_weights_v2
    out = {}
    for k, v in state_dict.items():
        if k in keys and v.dim() == 5:
            nk, nv = convert(k, state_dict)
            out[nk] = nv
        else:
            out[k] = v
    return out


def convert_model_weights(ckpt_before: str, ckpt_after: str, model: Optional[torch.nn.Module] = None,
                          legacy: bool = False) -> None:
    """Read the checkpoint ``ckpt_before`` (its weights under ``state_dict``, mmdet3d, or
    ``model_state``, OpenPCDet), convert the sparse convolution weights of ``model`` (every 5-d
    weight when no model is given) and write the checkpoint to ``ckpt_after``."""
    ckpt = torch.load(ckpt_before, map_location="cpu", weights_only=True)
    field = "state_dict" if "state_dict" in ckpt else "model_state"
    if field not in ckpt:
        raise ValueError("checkpoint has neither 'state_dict' nor 'model_state'")
    keys = sparse_conv_weight_keys(model) if model is not None else None
    ckpt[field] = convert_state_dict(ckpt[field], keys, legacy)
    torch.save(ckpt, ckpt_after)
