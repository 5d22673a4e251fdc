"""Second restatement of the reference's CPU path, in torch CPU tensor ops.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  The reference's slow path IS a
chain of torch tensor ops (int8_quant.py:20-62, 75-88, 106-119); this module writes
that chain down again so that
  * the C oracle can be pinned against the library routines the reference calls
    (torch.round, torch._int_mm, tensor/scalar division, dtype casts), and
  * bench.py can time "the reference's torch CPU fallback" on the host cores.
Everything here runs on CPU tensors.
"""
from __future__ import annotations

import torch


def quant_rowwise(x: torch.Tensor):
    """int8_quant.py:28-31 with :20-21: per-row absmax scale, multiply by the reciprocal, round half to even."""
    amax = x.abs().amax(dim=-1, keepdim=True)
    scale = (amax.float() / 127.0).clamp(min=1e-30)
    q = x.float().mul(1.0 / scale).round_().clamp_(-128.0, 127.0).to(torch.int8)
    return q, scale


def quant_tensorwise(x: torch.Tensor):
    """int8_quant.py:23-26."""
    scale = (x.abs().max().float() / 127.0).clamp(min=1e-30)
    q = x.float().mul(1.0 / scale).round_().clamp_(-128.0, 127.0).to(torch.int8)
    return q, scale


def hadamard(n: int, dtype: torch.dtype) -> torch.Tensor:
    """quarot.py:35-36: scipy's Sylvester matrix in `dtype`, divided by the Python float sqrt(n)."""
    from scipy.linalg import hadamard as scipy_hadamard

    return torch.tensor(scipy_hadamard(n), dtype=dtype) / (n**0.5)


def rotate(x: torch.Tensor, block: int = 128) -> torch.Tensor:
    """quarot.py:99-102 / 66-70: dense product of each block with H, in x's dtype (BLAS summation order)."""
    H = hadamard(block, x.dtype)
    return torch.matmul(x.view(*x.shape[:-1], x.shape[-1] // block, block), H).view(x.shape)


def linear_w8a8(x, w_q, w_scale, bias, compute_dtype, rotate_block: int = 0):
    """int8_quant.py:75-88 (one scale: float or 0-dim tensor) and :106-119 (w_scale [N,1])."""
    if rotate_block:
        x = rotate(x, rotate_block)
    x8, xs = quant_rowwise(x)
    acc = torch._int_mm(x8, w_q.T)
    if isinstance(w_scale, torch.Tensor) and w_scale.numel() > 1:
        y = acc.float().mul_(xs).mul_(w_scale.T).to(compute_dtype)
    else:
        y = acc.float().mul_(w_scale * xs).to(compute_dtype)
    if bias is not None:
        y = y + bias.to(compute_dtype)
    return y


def linear_w8a16(x, w_q, w_scale, bias):
    """int8_quant.py:756-760."""
    w_float = (w_q.float() * w_scale).to(x.dtype)
    return torch.nn.functional.linear(x, w_float, None if bias is None else bias.to(x.dtype))


def sr_delta(x, scale, noise):
    """int8_quant.py:47-62 with the random values supplied."""
    xs = x / scale
    fl = torch.floor(xs)
    frac = xs - fl
    return torch.clamp(torch.where(noise < frac, fl + 1, fl), -128, 127).to(torch.int8)


def merge_i8(w, dq):
    """int8_quant.py:313-316."""
    return torch.clamp(w.to(torch.int32) + dq.to(torch.int32), -128, 127).to(torch.int8)
