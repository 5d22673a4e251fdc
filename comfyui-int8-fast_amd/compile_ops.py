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
    torch.ops.i8f.int8_linear_lora      <- the same with the dynamic-LoRA side branch formed in the epilogue (int8_quant.py:762-774)
    torch.ops.i8f.int8_linear_prologue  <- int8_linear with the elementwise operation in front of the layer
                                           (adaLN modulation, tanh-GELU) applied inside the quantiser: what
                                           torch.compile's fusion into the Triton quantiser gives the reference

`Int8TensorwiseOps.Linear.forward` switches to these operators while a graph is being traced
(`torch.compiler.is_compiling()`); in eager mode it calls the library directly, which saves the
dispatcher overhead per layer.  A weight scale is passed either as a tensor or, for the
single-scale layout, as a float beside a `None` tensor.

`fuse_prologues(graph_module)` rewrites a traced graph so that the elementwise producer of a layer's activations
(GELU, adaLN modulation with its LayerNorm or RMSNorm, `silu(a) * b`, `cat((a, gelu(b)), -1)`) becomes the prologue of
its quantiser, `fuse_epilogues` moves `res + gate * layer(h)` into the GEMM epilogue, `share_quantisation` gives layers
that read one tensor a single quantiser, and `backend(inner)` is a torch.compile backend that applies the three and
hands the graph to `inner` ("inductor" by default):

    model = torch.compile(model, backend=compile_ops.backend())
"""
import copy
import logging
import operator
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


@torch.library.custom_op(f"{NAMESPACE}::quantize_rowwise_prologue", mutates_args=())
def quantize_rowwise_prologue(x: Tensor, rotate: bool, prologue: int, mod_scale: Optional[Tensor], mod_shift: Optional[Tensor],
                              eps: float = 1e-6, norm_weight: Optional[Tensor] = None, fused_add: bool = False) -> Tuple[Tensor, Tensor]:
    """quantize_rowwise on prologue(x) (the kinds of int8_linear_prologue), x with any leading dimensions:
    -> int8 [rows, K'] and float32 [rows, 1], K' the width behind the prologue.  What the layers that read one
    activation tensor share when the graph rewrite gives them a single quantiser."""
    return _lib.quant_rowwise(x.reshape(-1, x.shape[-1]), rotate=rotate, prologue=prologue, mod_scale=mod_scale,
                              mod_shift=mod_shift, eps=eps, norm_weight=norm_weight, fused_add=fused_add)


@quantize_rowwise_prologue.register_fake
def _(x, rotate, prologue, mod_scale, mod_shift, eps=1e-6, norm_weight=None, fused_add=False):
    rows = x.numel() // max(1, x.shape[-1])
    width = x.shape[-1] + (mod_scale.shape[-1] if prologue == _lib.PRO_CONCAT_GELU else 0)
    return (x.new_empty((rows, width), dtype=torch.int8), x.new_empty((rows, 1), dtype=torch.float32))


@torch.library.custom_op(f"{NAMESPACE}::rotate128", mutates_args=())
def rotate128(x: Tensor) -> Tensor:
    return _lib.rotate128(x)


@rotate128.register_fake
def _(x):
    return x.new_empty(x.shape)


@torch.library.custom_op(f"{NAMESPACE}::linear_w8a8", mutates_args=())
def linear_w8a8(a: Tensor, a_scale: Tensor, weight: Tensor, weight_scale: Optional[Tensor],
                weight_scale_value: float, bias: Optional[Tensor], out_dtype: torch.dtype, order: int,
                addend: Optional[Tensor] = None, gate: Optional[Tensor] = None) -> Tensor:
    """The GEMM on quantised activations [M,K]; addend / gate as for int8_linear.  -> [M,N]"""
    return _lib.linear_w8a8(a, a_scale, weight, _scale_arg(weight_scale, weight_scale_value), bias, out_dtype, order,
                            addend=addend, gate=gate)


@linear_w8a8.register_fake
def _(a, a_scale, weight, weight_scale, weight_scale_value, bias, out_dtype, order, addend=None, gate=None):
    return a.new_empty((a.shape[0], weight.shape[0]), dtype=out_dtype)


@torch.library.custom_op(f"{NAMESPACE}::int8_linear", mutates_args=())
def int8_linear(x: Tensor, weight: Tensor, weight_scale: Optional[Tensor], weight_scale_value: float,
                bias: Optional[Tensor], compute_dtype: torch.dtype, rotate: bool, order: int,
                addend: Optional[Tensor] = None, gate: Optional[Tensor] = None) -> Tensor:
    """Quantise the activations per token (rotated first when `rotate`) and run the W8A8 linear;
    `addend` (as many elements as the result, its dtype) is added inside the epilogue, after `gate` (vectors of the
    result's width, one per group of consecutive rows) has multiplied the result: addend + gate * y."""
    lead = x.shape[:-1]
    q, s = _lib.quant_rowwise(x.reshape(-1, x.shape[-1]), rotate=rotate)
    y = _lib.linear_w8a8(q, s, weight, _scale_arg(weight_scale, weight_scale_value), bias, compute_dtype, order,
                         addend=addend, gate=gate)
    return y.reshape(*lead, weight.shape[0])


@int8_linear.register_fake
def _(x, weight, weight_scale, weight_scale_value, bias, compute_dtype, rotate, order, addend=None, gate=None):
    return x.new_empty((*x.shape[:-1], weight.shape[0]), dtype=compute_dtype)


@torch.library.custom_op(f"{NAMESPACE}::int8_linear_lora", mutates_args=())
def int8_linear_lora(x: Tensor, weight: Tensor, weight_scale: Optional[Tensor], weight_scale_value: float,
                     bias: Optional[Tensor], compute_dtype: torch.dtype, rotate: bool, order: int,
                     side_t: Tensor, side_b: Tensor, alpha: Optional[float] = None) -> Tensor:
    """int8_linear plus the dynamic-LoRA side branch (int8_quant.py:762-774 of the reference): side_t [rows, r] is the
    first low-rank product x @ A.T, side_b [N, r] the second factor; their product, the scaling by alpha and the sum
    with the main result happen inside the GEMM epilogue, so the [rows, N] side tensor never exists."""
    lead = x.shape[:-1]
    q, s = _lib.quant_rowwise(x.reshape(-1, x.shape[-1]), rotate=rotate)
    y = _lib.linear_w8a8_lora(q, s, weight, _scale_arg(weight_scale, weight_scale_value), bias, side_t, side_b, alpha,
                              compute_dtype, order)
    return y.reshape(*lead, weight.shape[0])


@int8_linear_lora.register_fake
def _(x, weight, weight_scale, weight_scale_value, bias, compute_dtype, rotate, order, side_t, side_b, alpha=None):
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


@torch.library.custom_op(f"{NAMESPACE}::int8_linear_prologue", mutates_args=())
def int8_linear_prologue(x: Tensor, prologue: int, mod_scale: Optional[Tensor], mod_shift: Optional[Tensor],
                         weight: Tensor, weight_scale: Optional[Tensor], weight_scale_value: float,
                         bias: Optional[Tensor], compute_dtype: torch.dtype, rotate: bool, order: int, eps: float = 1e-6,
                         addend: Optional[Tensor] = None, gate: Optional[Tensor] = None,
                         norm_weight: Optional[Tensor] = None, fused_add: bool = False) -> Tensor:
    """int8_linear on prologue(x): GELU (tanh or exact form), (1 + mod_scale) * x + mod_shift with one pair of vectors per
    group of consecutive rows (PRO_NORM_MODULATE: of layer_norm(x, eps) without affine parameters; PRO_RMS_NORM: of
    rms_norm(x, norm_weight, eps), scale and shift each optional; fused_add: product and sum rounded once, as
    torch.addcmul(mod_shift, x, 1 + mod_scale)), silu(x) * mod_scale with a gate operand of x's shape,
    or cat((x, gelu(mod_scale)), -1); the transformed activations exist only inside the quantiser."""
    lead = x.shape[:-1]
    q, s = _lib.quant_rowwise(x.reshape(-1, x.shape[-1]), rotate=rotate, prologue=prologue, mod_scale=mod_scale,
                              mod_shift=mod_shift, eps=eps, norm_weight=norm_weight, fused_add=fused_add)
    y = _lib.linear_w8a8(q, s, weight, _scale_arg(weight_scale, weight_scale_value), bias, compute_dtype, order, addend=addend, gate=gate)
    return y.reshape(*lead, weight.shape[0])


@int8_linear_prologue.register_fake
def _(x, prologue, mod_scale, mod_shift, weight, weight_scale, weight_scale_value, bias, compute_dtype, rotate, order, eps=1e-6,
      addend=None, gate=None, norm_weight=None, fused_add=False):
    width = weight.shape[0]
    return x.new_empty((*x.shape[:-1], width), dtype=compute_dtype)


OPS = ("quantize_rowwise", "quantize_rowwise_prologue", "rotate128", "linear_w8a8", "int8_linear", "int8_linear_lora",
       "linear_w8a16_small_m", "int8_linear_prologue")


# --------------------------------------------------------------------------- graph rewrite
_VIEW_METHODS = ("reshape", "view", "contiguous", "flatten")


def _is_call(node, *targets):
    return node.op == "call_function" and node.target in targets


_OWN_META = "i8f_shape_and_dtype"   # what the rewrites record for the nodes they create (a meta-device tensor)


def _meta_val(node):
    if not isinstance(node, torch.fx.Node):
        return None
    return node.meta.get("example_value", node.meta.get("val", node.meta.get(_OWN_META)))


def _meta_shape(node):
    v = _meta_val(node)
    return None if v is None else tuple(v.shape)


def _record(node, shape, dtype):
    node.meta[_OWN_META] = torch.empty(tuple(int(d) for d in shape), dtype=dtype, device="meta")
    return node


def _through_views(node):
    """The producer of `node` behind shape-only steps that have no other user and only regroup the LEADING
    dimensions: a step whose traced shapes do not show the same last dimension on both sides (a view that splits or
    merges the feature dimension, or a graph without shape metadata) ends the walk."""
    while isinstance(node, torch.fx.Node) and len(node.users) == 1 and (
            (node.op == "call_method" and node.target in _VIEW_METHODS)
            or _is_call(node, torch.reshape, torch.flatten)):
        src = node.args[0]
        out_shape, in_shape = _meta_shape(node), _meta_shape(src)
        if not out_shape or not in_shape or out_shape[-1] != in_shape[-1]:
            break
        node = src
    return node


def _match_gelu(node):
    if not (_is_call(node, torch.nn.functional.gelu, torch._C._nn.gelu) and len(node.users) == 1):
        return None
    approx = node.kwargs.get("approximate", node.args[1] if len(node.args) > 1 else "none")
    return node.args[0] if approx == "tanh" else None


def _match_gelu_erf(node):
    """gelu(h) in its exact form (approximate="none", the default), used nowhere else -> h."""
    if not (_is_call(node, torch.nn.functional.gelu, torch._C._nn.gelu) and len(node.users) == 1):
        return None
    approx = node.kwargs.get("approximate", node.args[1] if len(node.args) > 1 else "none")
    return node.args[0] if approx == "none" else None


def _match_concat_gelu(node):
    """cat((a, gelu(b, approximate="tanh")), dim=-1) with a, b of one 16-bit dtype and equal leading dimensions, widths
    in multiples of 16 that add up to at most 16384, the activated tensor used nowhere else -> (a, b) nodes."""
    if not (_is_call(node, torch.cat, torch.concat, torch.concatenate) and len(node.users) == 1):
        return None
    parts = node.args[0] if node.args else node.kwargs.get("tensors")
    dim = node.args[1] if len(node.args) > 1 else node.kwargs.get("dim", 0)
    if not isinstance(parts, (list, tuple)) or len(parts) != 2 or not all(isinstance(p, torch.fx.Node) for p in parts):
        return None
    a, act = parts
    b = _match_gelu(act)
    va, vb = _meta_val(a), _meta_val(b) if b is not None else None
    if va is None or vb is None or dim not in (-1, len(va.shape) - 1):
        return None
    if va.dtype != vb.dtype or va.dtype not in (torch.bfloat16, torch.float16) or tuple(va.shape[:-1]) != tuple(vb.shape[:-1]) or len(va.shape) < 2:
        return None
    ka, kb = int(va.shape[-1]), int(vb.shape[-1])
    return (a, b) if ka % 16 == 0 and kb % 16 == 0 and ka > 0 and kb > 0 and ka + kb <= 16384 else None


def _match_silu_gate(node):
    """silu(a) * b in either operand order (a, b of one shape and dtype by the traced metadata) -> (a, b) nodes."""
    if not (_is_call(node, operator.mul, torch.mul) and len(node.users) == 1 and len(node.args) == 2):
        return None
    for act, gate in (node.args, node.args[::-1]):
        if not (isinstance(act, torch.fx.Node) and isinstance(gate, torch.fx.Node) and len(act.users) == 1
                and _is_call(act, torch.nn.functional.silu)):
            continue
        a = act.args[0]
        va, vb = _meta_val(a), _meta_val(gate)
        if va is not None and vb is not None and tuple(va.shape) == tuple(vb.shape) and va.dtype == vb.dtype:
            return a, gate
    return None


def _match_modulate(node):
    """(1 + scale) * x + shift in any operand order -> (x, scale, shift) nodes."""
    if not (_is_call(node, operator.add, torch.add) and len(node.users) == 1 and len(node.args) == 2):
        return None
    for prod, shift in (node.args, node.args[::-1]):
        if not (isinstance(prod, torch.fx.Node) and _is_call(prod, operator.mul, torch.mul) and len(prod.users) == 1):
            continue
        for gain, x in (prod.args, prod.args[::-1]):
            if isinstance(gain, torch.fx.Node) and _is_call(gain, operator.add, torch.add) and len(gain.users) == 1 and len(gain.args) == 2:
                for one, scale in (gain.args, gain.args[::-1]):
                    if isinstance(one, (int, float)) and one == 1 and isinstance(scale, torch.fx.Node) \
                            and isinstance(x, torch.fx.Node) and isinstance(shift, torch.fx.Node):
                        return x, scale, shift
    return None


def _match_scale_only(node):
    """(1 + scale) * x in either operand order -> (x, scale) nodes."""
    if not (_is_call(node, operator.mul, torch.mul) and len(node.users) == 1 and len(node.args) == 2):
        return None
    for gain, x in (node.args, node.args[::-1]):
        if isinstance(gain, torch.fx.Node) and _is_call(gain, operator.add, torch.add) and len(gain.users) == 1 and len(gain.args) == 2:
            for one, scale in (gain.args, gain.args[::-1]):
                if isinstance(one, (int, float)) and one == 1 and isinstance(scale, torch.fx.Node) and isinstance(x, torch.fx.Node):
                    return x, scale
    return None


def _match_rms_norm(node):
    """rms_norm(h, (K,), weight, eps) over the last dimension, used nowhere else, on 16-bit rows of a width the
    normalising quantiser takes, the weight absent or [K] of h's dtype -> (h, weight or None, eps)."""
    if not (_is_call(node, torch.nn.functional.rms_norm, torch.rms_norm) and len(node.users) == 1):
        return None
    a = dict(zip(("input", "normalized_shape", "weight", "eps"), node.args))
    a.update(node.kwargs)
    h, shape, w = a.get("input"), a.get("normalized_shape"), a.get("weight")
    v = _meta_val(h)
    if v is None or v.dtype not in (torch.bfloat16, torch.float16) or len(v.shape) < 2:
        return None
    K = int(v.shape[-1])
    if tuple(int(d) for d in (shape if isinstance(shape, (tuple, list, torch.Size)) else (shape,))) != (K,) or K % 16 or K > 16384:
        return None
    if w is not None:
        vw = _meta_val(w)
        if vw is None or vw.dtype != v.dtype or tuple(vw.shape) != (K,):
            return None
    eps = a.get("eps")
    if eps is None:
        eps = torch.finfo(v.dtype).eps      # what torch takes when none is given
    return (h, w, float(eps)) if isinstance(eps, (int, float)) else None


def _match_modulate_addcmul(node):
    """torch.addcmul(shift, x, 1 + scale) (the two factors in either order, value 1) on 16-bit tensors -> (x, scale, shift)."""
    if not (_is_call(node, torch.addcmul) and len(node.users) == 1):
        return None
    a = dict(zip(("input", "tensor1", "tensor2"), node.args))
    a.update(node.kwargs)
    if a.get("value", 1) != 1 or a.get("out") is not None:
        return None
    shift, f1, f2 = a.get("input"), a.get("tensor1"), a.get("tensor2")
    for gain, x in ((f1, f2), (f2, f1)):
        if isinstance(gain, torch.fx.Node) and _is_call(gain, operator.add, torch.add) and len(gain.users) == 1 and len(gain.args) == 2:
            for one, scale in (gain.args, gain.args[::-1]):
                if isinstance(one, (int, float)) and one == 1 and all(isinstance(n, torch.fx.Node) for n in (scale, x, shift)):
                    v = _meta_val(x)
                    if v is not None and v.dtype in (torch.bfloat16, torch.float16):
                        return x, scale, shift
    return None


def _match_plain_layer_norm(node):
    """layer_norm(h, (K,), eps=...) over the last dimension without weight and bias, used nowhere else, on 16-bit rows
    of a width the normalising quantiser takes -> (h, eps)."""
    if not (_is_call(node, torch.nn.functional.layer_norm) and len(node.users) == 1):
        return None
    names = ("input", "normalized_shape", "weight", "bias", "eps")
    a = dict(zip(names, node.args))
    a.update(node.kwargs)
    h, shape = a.get("input"), a.get("normalized_shape")
    if a.get("weight") is not None or a.get("bias") is not None or not isinstance(h, torch.fx.Node):
        return None
    v = _meta_val(h)
    if v is None or v.dtype not in (torch.bfloat16, torch.float16):
        return None
    K = int(v.shape[-1])
    if tuple(int(d) for d in (shape if isinstance(shape, (tuple, list, torch.Size)) else (shape,))) != (K,) or K % 16 or K > 16384:
        return None
    eps = a.get("eps", 1e-5)
    return (h, float(eps)) if isinstance(eps, (int, float)) else None


def _vectors_broadcast_over_tokens(x, scale, shift) -> bool:
    """True if the traced shapes say scale/shift are [.., 1, K] (or [K]) against x [.., T, K]: one vector per
    leading index, shared by the T rows that become consecutive rows of the flattened activations."""
    if any(_meta_val(n) is None for n in (x, scale, shift)):
        return False
    return modulation_broadcasts_over_tokens(_meta_val(x), _meta_val(scale), _meta_val(shift))


def modulation_broadcasts_over_tokens(x, scale, shift) -> bool:
    """Whether (1 + scale) * x + shift can run inside the quantiser: scale and shift of x's dtype and of one shape,
    [K] or [.., 1, K] against x [.., T, K] with the same leading dimensions, i.e. one vector per leading index,
    shared by the T rows that are consecutive rows of the flattened activations.  (Mixed dtypes promote in torch,
    other shapes broadcast differently: those stay torch expressions.)"""
    xs, ss, ts = tuple(x.shape), tuple(scale.shape), tuple(shift.shape)
    if ss != ts or len(xs) < 2 or not (x.dtype == scale.dtype == shift.dtype):
        return False
    if len(ss) == 1:
        return ss[0] == xs[-1]
    return len(ss) == len(xs) and ss[-1] == xs[-1] and ss[-2] == 1 and ss[:-2] == xs[:-2]


_INPLACE_FUNCTIONS = tuple(getattr(operator, n) for n in ("iadd", "isub", "imul", "itruediv", "ifloordiv", "imod", "ipow", "iand", "ior",
                                                          "ixor", "ilshift", "irshift", "imatmul", "setitem"))


def _writes_in_place(node) -> bool:
    """Whether a traced node may overwrite one of its tensor operands: an in-place method (name ending in an underscore),
    an augmented assignment or an item assignment, or an `out=` argument."""
    if node.op == "call_method":
        return node.target.endswith("_") and not node.target.endswith("__")
    if node.op == "call_function":
        name = getattr(node.target, "__name__", "")
        return node.target in _INPLACE_FUNCTIONS or (name.endswith("_") and not name.endswith("__")) or "out" in node.kwargs
    return False


def _in_place_write_between(first, last) -> bool:
    """True if a node that may write in place sits between `first` and `last` in graph order.  The rewrites move a read of
    a tensor from where the model reads it to where the fused operator runs; with a write in between they would read
    another value, so they leave such stretches alone (inference graphs rarely have any)."""
    node = first.next
    while node is not last and node.op != "root":
        if _writes_in_place(node):
            return True
        node = node.next
    return False


def _match_producer(src, rotate):
    """The producer of a layer's activations as a prologue kind -> (h, kind, mod_scale, mod_shift, eps, norm_weight,
    fused_add) nodes / values, or None.  Every node matched is used nowhere else."""
    h = _match_gelu(src)
    if h is not None:
        return h, _lib.PRO_GELU_TANH, None, None, 1e-6, None, False
    h = _match_gelu_erf(src)
    if h is not None:
        return h, _lib.PRO_GELU_ERF, None, None, 1e-6, None, False
    r = _match_rms_norm(src)
    if r is not None:                                               # the norm alone
        return r[0], _lib.PRO_RMS_NORM, None, None, r[2], r[1], False
    so = _match_scale_only(src)
    if so is not None:                                              # modulate(norm(x), scale) = norm(x) * (1 + scale)
        r = _match_rms_norm(so[0])
        if r is not None and _vectors_broadcast_over_tokens(r[0], so[1], so[1]):
            return r[0], _lib.PRO_RMS_NORM, so[1], None, r[2], r[1], False
    m, fused = _match_modulate(src), False
    if m is None:
        m, fused = _match_modulate_addcmul(src), True               # the one-kernel spelling: product and sum rounded once
    if m is not None:
        if not _vectors_broadcast_over_tokens(*m):
            return None
        ln = _match_plain_layer_norm(m[0])   # the modulated tensor is a LayerNorm without affine: that goes in too
        if ln is not None:
            return ln[0], _lib.PRO_NORM_MODULATE, m[1], m[2], ln[1], None, fused
        rn = _match_rms_norm(m[0])           # or an RMSNorm
        if rn is not None and _vectors_broadcast_over_tokens(rn[0], m[1], m[2]):
            return rn[0], _lib.PRO_RMS_NORM, m[1], m[2], rn[2], rn[1], fused
        return m[0], _lib.PRO_MODULATE, m[1], m[2], 1e-6, None, fused
    g = _match_silu_gate(src)
    if g is not None:
        return g[0], _lib.PRO_SILU_GATE, g[1], None, 1e-6, None, False
    c = _match_concat_gelu(src)
    if c is not None and not (rotate and (_meta_shape(c[0])[-1] % 128 or _meta_shape(c[1])[-1] % 128)):
        return c[0], _lib.PRO_CONCAT_GELU, c[1], None, 1e-6, None, False
    return None


def fuse_prologues(gm: torch.fx.GraphModule) -> int:
    """Rewrite int8_linear(gelu(h)) (either form), int8_linear((1 + s) * h + t), int8_linear((1 + s) * layer_norm(h) + t),
    int8_linear(rms_norm(h, w) [* (1 + s)] [+ t]), int8_linear(silu(h) * g) and int8_linear(cat((a, gelu_tanh(b)), -1))
    (no dynamic-LoRA addend, producers used nowhere else) into int8_linear_prologue(h, ...); the same producers in front
    of a quantize_rowwise that several layers share (share_quantisation) into quantize_rowwise_prologue(h, ...).
    Returns the number of consumers rewritten."""
    n_fused = 0
    lin_targets = (torch.ops.i8f.int8_linear, torch.ops.i8f.int8_linear.default)
    quant_targets = (torch.ops.i8f.quantize_rowwise, torch.ops.i8f.quantize_rowwise.default)
    order_of = {n: i for i, n in enumerate(gm.graph.nodes)}
    for node in list(gm.graph.nodes):
        is_lin = _is_call(node, *lin_targets)
        if not is_lin and not _is_call(node, *quant_targets):
            continue
        if is_lin:
            args = list(node.args) + [node.kwargs.get("addend")] * (9 - len(node.args))
            x_in, weight, ws_t, ws_v, bias, cdt, rotate, order, addend = args[:9]
            if addend is not None:
                continue
        else:
            x_in, rotate = node.args[0], node.args[1]
        if not isinstance(x_in, torch.fx.Node):
            continue
        src = _through_views(x_in)
        x_shape = _meta_shape(x_in)
        if not isinstance(src, torch.fx.Node) or x_shape is None:
            continue
        found = _match_producer(src, rotate)
        if found is None:
            continue
        h, kind, mod_scale, mod_shift, eps, norm_w, fused_add = found
        earliest = min((n for n in (h, mod_scale, mod_shift, norm_w) if isinstance(n, torch.fx.Node)), key=lambda n: order_of.get(n, 1 << 30))   # (nodes this pass created sit where a later node was)
        if _in_place_write_between(earliest, node):
            continue
        # The fused operator returns the leading shape of h, the original one that of x_in: the same when nothing
        # sat between them; a layer that flattened h to 2-D gets its 2-D result back by a reshape; anything else
        # (a direct caller with another regrouping of the rows) is left alone.
        h_shape = _meta_shape(h)
        if h_shape is None:
            continue
        if kind == _lib.PRO_CONCAT_GELU:   # the layer's input is wider than h by the second tensor: compare the rows
            if h_shape[-1] + _meta_shape(mod_scale)[-1] != x_shape[-1]:
                continue
            h_shape = (*h_shape[:-1], x_shape[-1])
        if h_shape[-1] != x_shape[-1]:
            continue
        if h_shape != x_shape and len(x_shape) != 2:
            continue
        if not is_lin:   # the shared quantiser: its outputs are 2-D whatever h's leading dimensions are
            with gm.graph.inserting_before(node):
                fused = gm.graph.call_function(torch.ops.i8f.quantize_rowwise_prologue,
                                               (h, rotate, kind, mod_scale, mod_shift, eps, norm_w, fused_add))
            node.replace_all_uses_with(fused)
            gm.graph.erase_node(node)
            n_fused += 1
            continue
        with gm.graph.inserting_before(node):
            fused = gm.graph.call_function(torch.ops.i8f.int8_linear_prologue,
                                           (h, kind, mod_scale, mod_shift, weight, ws_t, ws_v, bias, cdt, rotate, order, eps),
                                           {k: v for k, v in (("norm_weight", norm_w), ("fused_add", fused_add)) if v})
            n_out, old = _out_features(weight), _meta_val(node)
            if old is not None:   # shapes for the passes that follow (the epilogue rewrite reads them)
                _record(fused, (*h_shape[:-1], n_out), old.dtype)
            restored = fused
            if h_shape != x_shape:
                restored = gm.graph.call_method("reshape", (fused, -1, n_out))
                if old is not None:
                    _record(restored, old.shape, old.dtype)
        node.replace_all_uses_with(restored)
        gm.graph.erase_node(node)
        n_fused += 1
    if n_fused:
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()
    return n_fused


def share_quantisation(gm: torch.fx.GraphModule) -> int:
    """Layers that read the same activations (separate q, k and v projections, the two up-projections of a SwiGLU
    feed-forward) each quantise them, int8_linear being one operator: give every such group ONE quantize_rowwise and
    its layers the GEMM operator on the shared int8 rows (bit-identical: the quantiser is a function of its input).
    Shape-only steps between the shared tensor and the layers (each layer flattens its input) are looked through.
    Returns the number of layers rewritten."""
    lin_targets = (torch.ops.i8f.int8_linear, torch.ops.i8f.int8_linear.default)
    groups = {}
    for node in gm.graph.nodes:
        if not _is_call(node, *lin_targets) or not isinstance(node.args[0], torch.fx.Node):
            continue
        x_val, y_val = _meta_val(node.args[0]), _meta_val(node)
        if x_val is None or y_val is None or len(x_val.shape) < 1:
            continue
        src = _through_views(node.args[0])
        groups.setdefault((src, bool(node.args[6])), []).append(node)
    n_shared = 0
    for (src, rotate), nodes in groups.items():
        if len(nodes) < 2:
            continue
        first = nodes[0]                                   # (graph order: everything the group reads exists before it)
        if _in_place_write_between(first, nodes[-1]):      # the later layers might read another value than the first
            continue
        x_in = first.args[0]
        x_val = _meta_val(x_in)
        K = int(x_val.shape[-1])
        rows = int(x_val.numel()) // max(1, K)
        with gm.graph.inserting_before(first):
            x2d = x_in
            if len(x_val.shape) != 2:
                x2d = _record(gm.graph.call_method("reshape", (x_in, -1, K)), (rows, K), x_val.dtype)
            qs = gm.graph.call_function(torch.ops.i8f.quantize_rowwise, (x2d, rotate))
            q = gm.graph.call_function(operator.getitem, (qs, 0))
            s = gm.graph.call_function(operator.getitem, (qs, 1))
        for node in nodes:
            args = list(node.args) + [None] * (10 - len(node.args))
            _, weight, ws_t, ws_v, bias, cdt, _, order, addend, gate = args[:10]
            addend = node.kwargs.get("addend", addend)
            gate = node.kwargs.get("gate", gate)
            y_val = _meta_val(node)
            n_out = int(y_val.shape[-1])
            with gm.graph.inserting_before(node):
                y = _record(gm.graph.call_function(torch.ops.i8f.linear_w8a8, (q, s, weight, ws_t, ws_v, bias, cdt, order),
                                                   {"addend": addend, "gate": gate}), (rows, n_out), y_val.dtype)
                restored = y
                if tuple(y_val.shape) != (rows, n_out):
                    restored = _record(gm.graph.call_method("reshape", (y, *(int(d) for d in y_val.shape))), y_val.shape, y_val.dtype)
            node.replace_all_uses_with(restored)
            gm.graph.erase_node(node)
            n_shared += 1
    if n_shared:
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()
    return n_shared


def _sole_user(node):
    return next(iter(node.users)) if len(node.users) == 1 else None


_FRESH_TENSOR_FUNCTIONS = (operator.add, operator.sub, operator.mul, operator.truediv, operator.iadd, operator.isub, operator.imul,
                           torch.add, torch.sub, torch.mul, torch.cat, torch.nn.functional.linear, torch.nn.functional.layer_norm,
                           torch.nn.functional.rms_norm, torch.nn.functional.gelu, torch.nn.functional.silu)


def _update_in_place_is_private(res, update, order_of) -> bool:
    """`update` is `res += v` (operator.iadd).  Replacing it by an operator that RETURNS res + v leaves res itself as it
    was, which nobody can tell if (a) everything else that reads res does so before the update, and (b) res is not a
    window onto storage that something else reads: it is the result of an operation that makes a new tensor (arithmetic,
    a layer, one of this package's operators), possibly behind shape-only steps that have no other user.  Graph inputs,
    parameters, slices and anything unknown fail (b)."""
    pos = order_of.get(update, 1 << 30)
    for user in res.users:
        if user is not update and order_of.get(user, 1 << 30) > pos:
            return False
    base = res
    while (base.op == "call_method" and base.target in _VIEW_METHODS) or _is_call(base, torch.reshape, torch.flatten):
        src = base.args[0]
        if not isinstance(src, torch.fx.Node) or len(src.users) != 1:
            return False
        base = src
    if base.op == "call_module":
        return True
    return base.op == "call_function" and (base.target in _FRESH_TENSOR_FUNCTIONS or "i8f" in str(base.target))


def fuse_epilogues(gm: torch.fx.GraphModule) -> int:
    """Rewrite res + gate * int8_linear(...) -- the gated residual behind the projections of an adaLN-Zero block, gate
    one vector per leading index broadcast over the tokens, res of the result's shape, all of the compute dtype, in any
    operand order, with shape-only steps between the layer and the multiplication -- into the layer's own epilogue
    (addend=res, gate=gate); also gate * linear(...) and res + linear(...) alone, and the in-place spelling
    `res += gate * linear(...)` where nobody can tell the difference (_update_in_place_is_private).  Layers that already
    carry an addend (a dynamic-LoRA side tensor) are left alone.  Returns the number of layers rewritten."""
    n_fused = 0
    order_of = {n: i for i, n in enumerate(gm.graph.nodes)}
    lin_targets = (torch.ops.i8f.int8_linear, torch.ops.i8f.int8_linear.default,
                   torch.ops.i8f.int8_linear_prologue, torch.ops.i8f.int8_linear_prologue.default,
                   torch.ops.i8f.linear_w8a8, torch.ops.i8f.linear_w8a8.default)
    for node in list(gm.graph.nodes):
        if not _is_call(node, *lin_targets):
            continue
        n_pos = 12 if "prologue" in str(node.target) else 8      # arguments in front of addend, gate
        given = list(node.args[n_pos:]) + [None, None]
        if given[0] is not None or given[1] is not None or node.kwargs.get("addend") is not None or node.kwargs.get("gate") is not None:
            continue
        y_val = _meta_val(node)
        if y_val is None:
            continue
        cur = node                                 # forward through shape-only steps that keep the feature dimension
        while True:
            u = _sole_user(cur)
            if u is None or not ((u.op == "call_method" and u.target in _VIEW_METHODS) or _is_call(u, torch.reshape, torch.flatten)):
                break
            if u.args[0] is not cur or not _meta_shape(u) or _meta_shape(u)[-1] != y_val.shape[-1]:
                break
            cur = u
        u = _sole_user(cur)
        if u is None:
            continue
        cur_val = _meta_val(cur)
        gate = res = None
        last = None

        def other(n, operand):
            return n.args[1] if n.args[0] is operand else n.args[0]

        if _is_call(u, operator.mul, torch.mul) and len(u.args) == 2:
            g_node = other(u, cur)
            g_val = _meta_val(g_node)
            if g_val is None or cur_val is None or not modulation_broadcasts_over_tokens(cur_val, g_val, g_val):
                continue
            gate, last = g_node, u
            a = _sole_user(u)
            if a is not None and _is_call(a, operator.add, torch.add) and len(a.args) == 2 and not a.kwargs:
                r_node = other(a, u)
                r_val = _meta_val(r_node)
                if r_val is not None and tuple(r_val.shape) == tuple(_meta_shape(u)) and r_val.dtype == cur_val.dtype and r_node is not u:
                    res, last = r_node, a
            elif a is not None and _is_call(a, operator.iadd) and len(a.args) == 2 and a.args[1] is u and isinstance(a.args[0], torch.fx.Node):
                r_node = a.args[0]                                   # res += gate * y
                r_val = _meta_val(r_node)
                if (r_val is not None and tuple(r_val.shape) == tuple(_meta_shape(u)) and r_val.dtype == cur_val.dtype
                        and _update_in_place_is_private(r_node, a, order_of)):
                    res, last = r_node, a
        elif _is_call(u, operator.iadd) and len(u.args) == 2 and u.args[1] is cur and isinstance(u.args[0], torch.fx.Node):
            r_node = u.args[0]                                       # res += y
            r_val = _meta_val(r_node)
            if (r_val is None or cur_val is None or tuple(r_val.shape) != tuple(cur_val.shape) or r_val.dtype != cur_val.dtype
                    or not _update_in_place_is_private(r_node, u, order_of)):
                continue
            res, last = r_node, u
        elif _is_call(u, operator.add, torch.add) and len(u.args) == 2 and not u.kwargs:
            r_node = other(u, cur)
            r_val = _meta_val(r_node)
            if r_val is None or cur_val is None or tuple(r_val.shape) != tuple(cur_val.shape) or r_val.dtype != cur_val.dtype or r_node is cur:
                continue
            res, last = r_node, u
        else:
            continue
        final_shape = _meta_shape(last)
        if final_shape is None or final_shape[-1] != y_val.shape[-1]:
            continue
        if _in_place_write_between(node, last):   # the layer would run later than the model ran it
            continue
        with gm.graph.inserting_before(last):
            kwargs = dict(node.kwargs)
            kwargs.update(addend=res, gate=gate)
            fused = _record(gm.graph.call_function(node.target, tuple(node.args[:n_pos]), kwargs), y_val.shape, y_val.dtype)
            restored = fused
            if tuple(final_shape) != tuple(y_val.shape):
                restored = _record(gm.graph.call_method("reshape", (fused, *final_shape)), final_shape, y_val.dtype)
        last.replace_all_uses_with(restored)
        n_fused += 1
    if n_fused:
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()
    return n_fused


def _out_features(weight_node):
    v = _meta_val(weight_node)
    if v is None:
        raise RuntimeError("the traced graph carries no shape for the weight")
    return int(v.shape[0])


def backend(inner="inductor"):
    """A torch.compile backend: share_quantisation, fuse_prologues and fuse_epilogues, then `inner` (a registered backend
    name or a callable)."""
    def compile_fn(gm, example_inputs):
        rewrite(gm)
        fn = inner
        if isinstance(inner, str):
            from torch._dynamo.backends.registry import lookup_backend

            fn = lookup_backend(inner)
        return fn(gm, example_inputs)
    return compile_fn


LAST_PASS_COUNTS = None   # (layers sharing a quantiser, prologues, epilogues) of the most recent graph the installed pass saw


def rewrite(gm: torch.fx.GraphModule):
    """The three rewrites in the order in which they build on each other -> their counts."""
    return share_quantisation(gm), fuse_prologues(gm), fuse_epilogues(gm)


def install_inductor_pass() -> bool:
    """Make plain `torch.compile(model)` -- the inductor backend, what ComfyUI's compile nodes call, as the reference's
    README has its users do (README.md:4,56) -- apply the rewrites without `backend=compile_ops.backend()`: they are
    registered as inductor's pre-grad custom pass, behind a pass that is already registered there.  Idempotent;
    returns False where this torch has no such hook."""
    global _installed
    try:
        import torch._inductor.config as inductor_config
    except ImportError:
        return False
    if not hasattr(inductor_config, "pre_grad_custom_pass"):
        return False
    if _installed:
        return True
    before = inductor_config.pre_grad_custom_pass

    def i8f_pre_grad_pass(graph: torch.fx.Graph):
        global LAST_PASS_COUNTS
        if before is not None:
            before(graph)
        gm = graph.owning_module
        if gm is None or not any("i8f" in str(n.target) for n in graph.nodes if n.op == "call_function"):
            return
        # Somebody else's compile must not fail over a graph these rewrites were not written for: they are tried on a
        # copy first, and a graph on which they raise is compiled as it is.
        try:
            rewrite(copy.deepcopy(gm))
        except Exception as e:  # noqa: BLE001
            logging.getLogger(__name__).warning("INT8 Fast: graph rewrites skipped for this graph (%s: %s)", type(e).__name__, e)
            return
        LAST_PASS_COUNTS = rewrite(gm)

    inductor_config.pre_grad_custom_pass = i8f_pre_grad_pass
    _installed = True
    return True


_installed = False


def split_scale(weight_scale):
    """(tensor or None, float): the two-argument form in which the operators take a weight scale."""
    if isinstance(weight_scale, Tensor):
        return weight_scale, 0.0
    return None, float(weight_scale)
