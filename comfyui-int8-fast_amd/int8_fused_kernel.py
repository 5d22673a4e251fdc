"""Fused W8A8 linear pipeline on the HIP library.

Same entry points as the reference's int8_fused_kernel.py, which launches Triton
kernels; here each call goes through the C ABI of libi8f_gfx950.so:

    hip_quantize_rowwise      <- triton_quantize_rowwise      (int8_fused_kernel.py:55-73)
    hip_int8_linear           <- triton_int8_linear           (int8_fused_kernel.py:179-235)
    hip_int8_linear_per_row   <- triton_int8_linear_per_row   (int8_fused_kernel.py:330-372)

The triton_* names are kept as aliases so that callers written against the
reference keep working.
"""
from __future__ import annotations

import torch

from . import _lib
from ._lib import EPI_FUSED, EPI_TORCH  # noqa: F401  (re-exported)

# Order of the epilogue's float operations used by the wrappers below.  EPI_TORCH
# reproduces the reference's torch path bit for bit; EPI_FUSED is the single-rounding
# order of the reference's Triton kernels.
DEFAULT_EPILOGUE = EPI_TORCH


def hip_quantize_rowwise(x: torch.Tensor, rotate: bool = False):
    """[rows, cols] float -> (int8 [rows, cols], float32 [rows, 1]) per-row absmax quantisation;
    rotate=True applies the online QuaRot rotation in the same pass."""
    if x.dim() != 2:
        raise ValueError(f"expected a 2-D tensor, got shape {tuple(x.shape)}")
    return _lib.quant_rowwise(x, rotate=rotate)


def _linear(x, weight, weight_scale, bias, compute_dtype, rotate, order, addend=None, prologue=None, side=None, gate=None):
    lead = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1])
    kind, mod_scale, mod_shift, eps, norm_weight, fused_add = \
        (tuple(prologue) + (1e-6, None, False)[len(prologue) - 3:])[:6] if prologue else (_lib.PRO_NONE, None, None, 1e-6, None, False)
    q, s = _lib.quant_rowwise(x2, rotate=rotate, prologue=kind, mod_scale=mod_scale, mod_shift=mod_shift, eps=eps, norm_weight=norm_weight,
                              fused_add=fused_add)
    order = DEFAULT_EPILOGUE if order is None else order
    if side is not None:   # (side_t [M,r], side_b [N,r], alpha or None): the low-rank branch formed inside the epilogue
        if gate is not None or addend is not None:
            raise ValueError("the low-rank side branch takes neither a gate nor an addend")
        y = _lib.linear_w8a8_lora(q, s, weight, weight_scale, bias, side[0], side[1], side[2], compute_dtype, order)
    else:
        y = _lib.linear_w8a8(q, s, weight, weight_scale, bias, compute_dtype, order, addend=addend, gate=gate)
    return y.reshape(*lead, weight.shape[0])


def hip_int8_linear(x, weight, weight_scale, bias=None, compute_dtype=torch.float16, rotate=False, order=None,
                    addend=None, prologue=None, side=None, gate=None):
    """W8A8 linear with ONE weight scale (Python float or 1-element tensor).  `addend`, a tensor of the
    output's shape and dtype, is added to the result inside the epilogue (and the sum rounded again).
    `prologue` = (kind, mod_scale, mod_shift[, eps[, norm_weight[, fused_add]]]) applies _lib.PRO_GELU_TANH, _lib.PRO_GELU_ERF, _lib.PRO_MODULATE,
    _lib.PRO_SILU_GATE, _lib.PRO_NORM_MODULATE, _lib.PRO_RMS_NORM or _lib.PRO_CONCAT_GELU to x inside the quantiser.  `side` = (side_t [M,r], side_b [N,r], alpha or None) adds the low-rank product side_t @ side_b.T,
    formed inside the epilogue (see _lib.linear_w8a8_lora), instead of a ready-made addend.  `gate` ([.., 1, N] or [N],
    one vector per group of consecutive rows) multiplies the rounded result before the addend is added:
    addend + gate * y, the gated residual of an adaLN-Zero block."""
    if isinstance(weight_scale, torch.Tensor) and weight_scale.numel() != 1:
        # the reference's kernel reads element 0 only (int8_fused_kernel.py:153)
        weight_scale = weight_scale.reshape(-1)[:1]
    return _linear(x, weight, weight_scale, bias, compute_dtype, rotate, order, addend, prologue, side, gate)


def hip_int8_linear_per_row(x, weight, weight_scale, bias=None, compute_dtype=torch.float16, rotate=False, order=None,
                            addend=None, prologue=None, side=None, gate=None):
    """W8A8 linear with one weight scale per output row ([N,1] or [N] float32 tensor)."""
    if not isinstance(weight_scale, torch.Tensor) or weight_scale.numel() != weight.shape[0]:
        raise ValueError("per-row weight scale must be a tensor with one element per weight row")
    return _linear(x, weight, weight_scale, bias, compute_dtype, rotate, order, addend, prologue, side, gate)


def hip_int8_linear_pair(xs, weights, weight_scales, biases=(None, None), compute_dtype=torch.float16, rotate=False, order=None,
                         gates=None, residuals=None):
    """The same layer type applied to several token streams, each with its own weight (the image and the text stream
    of a double-stream transformer block; the reference calls its operator once per stream, int8_quant.py:703-778):
    the activations of all streams are quantised in ONE launch (they share their width and dtype), and their GEMMs
    go out as one launch where the small stream's tiles fit into the compute units the large one leaves idle (else one
    launch per stream).  gates / residuals: per stream, a gate ([.., 1, N] or [N]) and a residual of the output's shape
    and dtype, or None: residual + gate * y in the epilogue.
    -> list of outputs, bit-identical to separate hip_int8_linear[_per_row] calls."""
    leads = [x.shape[:-1] for x in xs]
    quantised = _lib.quant_rowwise_grouped([x.reshape(-1, x.shape[-1]) for x in xs], rotate=rotate)
    order = DEFAULT_EPILOGUE if order is None else order
    problems = []
    gates = gates or [None] * len(xs)
    residuals = residuals or [None] * len(xs)
    for (q, s), w, ws, b, gt, rs in zip(quantised, weights, weight_scales, biases, gates, residuals):
        if isinstance(ws, torch.Tensor) and ws.numel() not in (1, w.shape[0]):
            ws = ws.reshape(-1)[:1]
        problems.append((q, s, w, ws, b, None if rs is None else rs.reshape(-1, rs.shape[-1]), gt))
    outs = _lib.linear_w8a8_grouped(problems, compute_dtype, order)
    return [o.reshape(*lead, o.shape[-1]) for o, lead in zip(outs, leads)]


triton_quantize_rowwise = hip_quantize_rowwise
triton_int8_linear = hip_int8_linear
triton_int8_linear_per_row = hip_int8_linear_per_row
