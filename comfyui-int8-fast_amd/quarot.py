"""QuaRot block rotation, host side.

Same surface as the reference's quarot.py (build_hadamard, rotate_weight,
rotate_activation), but the rotation itself runs in the HIP library as a
fixed-order 128-point butterfly (i8f_rotate128); in the forward pass it is not a
separate step at all: Linear.forward asks the quantiser to rotate while it reads
the activations (i8f_quant_rowwise with rotate_block=128).
"""
from __future__ import annotations

import torch

from . import _lib

GROUP_SIZE = 128  # the only group size the reference ever passes (int8_quant.py:602,743)

_cache: dict[tuple[int, str, torch.dtype], torch.Tensor] = {}


def build_hadamard(size: int, device="cpu", dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Normalised Sylvester-Hadamard matrix H (H @ H.T = I), cached per (size, device, dtype).

    Follows the reference's construction (quarot.py:18-39): a +-1 matrix of `dtype`
    divided by the Python float size**0.5, so the entries are 1/sqrt(size) rounded
    to `dtype`.  The +-1 pattern is H[k, j] = (-1)^popcount(k & j).
    """
    if size <= 0 or size & (size - 1):
        raise ValueError(f"Hadamard size must be power of 2, got {size}")
    key = (size, str(device), dtype)
    H = _cache.get(key)
    if H is None:
        idx = torch.arange(size)
        both = idx[:, None] & idx[None, :]
        parity = torch.zeros_like(both)
        while bool(both.any()):
            parity ^= both & 1
            both = both >> 1
        signs = 1 - 2 * parity
        H = signs.to(dtype=dtype, device=device) / (size**0.5)
        _cache[key] = H
    return H


def _check(last: int, group_size: int, what: str) -> None:
    if last % group_size:
        raise ValueError(f"{what} {last} not divisible by group_size {group_size}")
    if group_size != GROUP_SIZE:
        raise ValueError(f"the HIP rotation is built for group_size {GROUP_SIZE} only, got {group_size}")


def rotate_weight(weight: torch.Tensor, H: torch.Tensor | None = None, group_size: int = GROUP_SIZE) -> torch.Tensor:
    """W_rot = W @ blockdiag(H).T for a [out, in] weight (quarot.py:42-70).  H is accepted for
    signature compatibility; the kernel applies the normalised Hadamard of weight.dtype."""
    if weight.dim() != 2:
        raise ValueError("weight must be 2-D")
    _check(weight.shape[1], group_size, "in_features")
    return _lib.rotate128(weight)


def rotate_activation(x: torch.Tensor, H: torch.Tensor | None = None, group_size: int = GROUP_SIZE) -> torch.Tensor:
    """x_rot = x @ blockdiag(H) over the last dimension (quarot.py:73-102)."""
    _check(x.shape[-1], group_size, "features")
    shape = x.shape
    return _lib.rotate128(x.reshape(-1, shape[-1])).view(shape)
