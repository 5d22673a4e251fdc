"""torch.library registration of the INT8 linear path, so that torch.compile traces through it.

The reference reaches its full speed-up only under torch.compile (README.md:4,56 of the reference);
there the Triton kernels are traceable by construction.  Here the kernels sit behind ctypes calls,
which Dynamo cannot trace, so every call of the forward path is registered as a custom operator in
the namespace `i8f` with a shape-only ("fake") implementation:

    torch.ops.i8f.quantize_rowwise      <- triton_quantize_rowwise             (int8_fused_kernel.py:55-73)
    torch.ops.i8f.linear_w8a8           <- the GEMM + dequant launch            (int8_fused_kernel.py:216-232, 357-369)
    torch.ops.i8f.int8_linear           <- triton_int8_linear[_per_row]         (int8_fused_kernel.py:179-235, 330-372)
    torch.ops.i8f.linear_w8a16_small_m  <- the M <= 16 branch of Linear.forward (int8_quant.py:756-760)
    torch.ops.i8f.rotate128             <- rotate_activation                    (quarot.py:73-102)

`Int8TensorwiseOps.Linear.forward` switches to these operators while a graph is being traced
(`torch.compiler.is_compiling()`); in eager mode it calls the library directly, which saves the
dispatcher overhead per layer.  A weight scale is passed either as a tensor or, for the
single-scale layout, as a float beside a `None` tensor.
"""
from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _lib

NAMESPACE = "i8f"


def _scale_arg(weight_scale: Optional[Tensor], weight_scale_value: float):
    return weight_scale if weight_scale is not None else float(weight_scale_value)


@torch.library.custom_op(f"{NAMESPACE}::quantize_rowwise", mutates_args=())
def quantize_rowwise(x: Tensor, rotate: bool) -> Tuple[Tensor, Tensor]:
    return _lib.quant_rowwise(x, rotate=rotate)


@quantize_rowwise.register_fake
def _(x, rotate):
    if x.dim() != 2:
        raise ValueError(f"expected a 2-D tensor, got shape {tuple(x.shape)}")
    return (x.new_empty(x.shape, dtype=torch.int8), x.new_empty((x.shape[0], 1), dtype=torch.float32))


@torch.library.custom_op(f"{NAMESPACE}::rotate128", mutates_args=())
def rotate128(x: Tensor) -> Tensor:
    return _lib.rotate128(x)


@rotate128.register_fake
def _(x):
    return x.new_empty(x.shape)


@torch.library.custom_op(f"{NAMESPACE}::linear_w8a8", mutates_args=())
def linear_w8a8(a: Tensor, a_scale: Tensor, weight: Tensor, weight_scale: Optional[Tensor],
                weight_scale_value: float, bias: Optional[Tensor], out_dtype: torch.dtype, order: int) -> Tensor:
    return _lib.linear_w8a8(a, a_scale, weight, _scale_arg(weight_scale, weight_scale_value), bias, out_dtype, order)


@linear_w8a8.register_fake
def _(a, a_scale, weight, weight_scale, weight_scale_value, bias, out_dtype, order):
    return a.new_empty((a.shape[0], weight.shape[0]), dtype=out_dtype)


@torch.library.custom_op(f"{NAMESPACE}::int8_linear", mutates_args=())
def int8_linear(x: Tensor, weight: Tensor, weight_scale: Optional[Tensor], weight_scale_value: float,
                bias: Optional[Tensor], compute_dtype: torch.dtype, rotate: bool, order: int,
                addend: Optional[Tensor] = None) -> Tensor:
    """Quantise the activations per token (rotated first when `rotate`) and run the W8A8 linear;
    `addend` (shape and dtype of the result) is added inside the epilogue."""
    lead = x.shape[:-1]
    q, s = _lib.quant_rowwise(x.reshape(-1, x.shape[-1]), rotate=rotate)
    y = _lib.linear_w8a8(q, s, weight, _scale_arg(weight_scale, weight_scale_value), bias, compute_dtype, order,
                         addend=addend)
    return y.reshape(*lead, weight.shape[0])


@int8_linear.register_fake
def _(x, weight, weight_scale, weight_scale_value, bias, compute_dtype, rotate, order, addend=None):
    return x.new_empty((*x.shape[:-1], weight.shape[0]), dtype=compute_dtype)


@torch.library.custom_op(f"{NAMESPACE}::linear_w8a16_small_m", mutates_args=())
def linear_w8a16_small_m(x: Tensor, weight: Tensor, weight_scale: Optional[Tensor], weight_scale_value: float,
                         bias: Optional[Tensor], rotate: bool) -> Tensor:
    x2 = x.reshape(-1, x.shape[-1])
    if rotate:
        x2 = _lib.rotate128(x2)
    y = _lib.linear_w8a16_small_m(x2, weight, _scale_arg(weight_scale, weight_scale_value), bias)
    return y.reshape(*x.shape[:-1], weight.shape[0])


@linear_w8a16_small_m.register_fake
def _(x, weight, weight_scale, weight_scale_value, bias, rotate):
    return x.new_empty((*x.shape[:-1], weight.shape[0]))


OPS = ("quantize_rowwise", "rotate128", "linear_w8a8", "int8_linear", "linear_w8a16_small_m")


def split_scale(weight_scale):
    """(tensor or None, float): the two-argument form in which the operators take a weight scale."""
    if isinstance(weight_scale, Tensor):
        return weight_scale, 0.0
    return None, float(weight_scale)
