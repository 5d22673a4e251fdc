"""INT8 W8A8 linear layer for ComfyUI on the gfx950 HIP library.

Host-side mirror of the reference's int8_quant.py: same free functions, same
`Int8TensorwiseOps` custom-operations class (attribute names, state-dict
behaviour, dispatch rules) and the same LoRA patch adapters, so that ComfyUI
code written against the reference runs unchanged.  All device work goes through
libi8f_gfx950.so; there is no torch._int_mm or CPU path.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from . import _lib, compile_ops, int8_fused_kernel
from ._comfy_compat import (
    LoRAAdapter,
    cast_bias_weight,
    compute_device,
    manual_cast,
    uncast_bias_weight,
)
from .int8_fused_kernel import hip_int8_linear, hip_int8_linear_per_row
from .dynamic_lora import DynamicLoRAHook  # noqa: F401  (int8_dynamic_lora.py:40 of the reference imports it from here)

# Rows at or below this use the W8A16 small-batch kernel (int8_quant.py:751 of the reference).
SMALL_BATCH_ROWS = 16


# --------------------------------------------------------------------------- quantisation helpers
def quantize_int8(x: Tensor, scale) -> Tensor:
    """round(x / scale) saturated to int8 for a GIVEN scale (int8_quant.py:20-21).
    A load-time utility (elementwise torch on x's device); the hot path never calls it."""
    return x.float().mul(1.0 / scale).round_().clamp_(-128.0, 127.0).to(torch.int8)


def quantize_int8_tensorwise(x: Tensor):
    """One absmax scale for the whole tensor (int8_quant.py:23-26), in two launches over all CUs.
    Returns (int8 like x, 0-dim float32 scale)."""
    return _lib.quant_tensorwise(x)


def quantize_int8_axiswise(x: Tensor, dim: int):
    """Absmax scale per slice along `dim`, which must be the last dimension
    (int8_quant.py:28-31; the reference only ever passes the last one)."""
    if dim not in (-1, x.dim() - 1):
        raise ValueError("the HIP quantiser reduces over the last dimension only")
    lead = x.shape[:-1]
    q, s = _lib.quant_rowwise(x.reshape(-1, x.shape[-1]))
    return q.view(x.shape), s.view(*lead, 1)


def dequantize(q: Tensor, scale) -> Tensor:
    return q.float() * scale


def stochastic_round_int8_delta(x: Tensor, scale, seed: int = 0, noise: Tensor | None = None) -> Tensor:
    """Stochastic rounding of x / scale to int8 (int8_quant.py:36-62).

    The uniform noise is drawn like the reference does (a generator seeded with `seed` on the
    compute device) unless `noise` is supplied; with supplied noise the result is reproducible
    on any device and bit-identical to the reference's arithmetic.
    """
    orig_device, shape = x.device, x.shape
    xd = x if x.is_cuda else x.to(compute_device())
    xd = xd.float().reshape(-1, shape[-1]) if x.dim() != 2 else xd.float()
    if noise is None:
        gen = torch.Generator(device=xd.device)
        gen.manual_seed(seed)
        noise = torch.rand(xd.shape, generator=gen, device=xd.device, dtype=torch.float32)
    else:
        noise = noise.to(xd.device).reshape(xd.shape)
    if isinstance(scale, Tensor) and scale.numel() > 1:
        scale = scale.reshape(-1)
    out = _lib.sr_quant_delta(xd, scale, noise).view(shape)
    return out if out.device == orig_device else out.to(orig_device)


# --------------------------------------------------------------------------- forward functions
@torch.no_grad()
def int8_forward_dynamic(x: Tensor, weight: Tensor, weight_scale, bias, compute_dtype: torch.dtype,
                         rotate: bool = False, addend: Tensor | None = None, prologue=None, side=None, gate=None) -> Tensor:
    """Dynamic per-token activation quantisation, ONE weight scale (int8_quant.py:68-88)."""
    return hip_int8_linear(x, weight, weight_scale, bias, compute_dtype, rotate=rotate, addend=addend, prologue=prologue,
                           side=side, gate=gate)


@torch.no_grad()
def int8_forward_dynamic_per_row(x: Tensor, weight: Tensor, weight_scale: Tensor, bias,
                                 compute_dtype: torch.dtype, rotate: bool = False, addend: Tensor | None = None,
                                 prologue=None, side=None, gate=None) -> Tensor:
    """Dynamic per-token activation quantisation, per-row weight scales [N,1] (int8_quant.py:92-119)."""
    return hip_int8_linear_per_row(x, weight, weight_scale, bias, compute_dtype, rotate=rotate, addend=addend,
                                   prologue=prologue, side=side, gate=gate)


class _ShapeAndDtype:
    """What modulation_broadcasts_over_tokens looks at, for a tensor that does not exist yet (a layer's output)."""

    def __init__(self, shape, dtype):
        self.shape, self.dtype = tuple(shape), dtype


def forward_pair(layers, xs, gates=None, residuals=None):
    """Linear.forward for several quantised layers of one shape at once, e.g. the same projection of the image and of
    the text stream of a double-stream block: [layer(x) for layer, x in zip(layers, xs)], with the activations of all
    streams quantised by ONE kernel launch where the layers allow it (W8A8 path on every stream: more than 16 rows,
    quantised weights on the inputs' device, no dynamic LoRA, no managed casting, the same rotation flag, inputs of one
    width and one 16-bit dtype, eager mode).  gates / residuals: per layer, what forward(x, gate=, residual=) takes
    (the gated residual of the block in the epilogue), or None.  Anything else falls back to the layers' own forward;
    results are bit-identical either way."""
    layers, xs = list(layers), list(xs)
    gates = list(gates) if gates is not None else [None] * len(xs)
    residuals = list(residuals) if residuals is not None else [None] * len(xs)
    ok = len(layers) >= 2 and len(layers) == len(xs) == len(gates) == len(residuals) and not torch.compiler.is_compiling()
    if ok:
        x0 = xs[0]
        rot = bool(getattr(layers[0], "_use_quarot", False))
        for lin, x in zip(layers, xs):
            managed = lin.comfy_cast_weights or len(lin.weight_function) > 0 or len(lin.bias_function) > 0
            ok = ok and (getattr(lin, "_is_quantized", False) and not managed and lin.lora_A is None and x.is_cuda
                         and lin.weight.device == x.device and (lin.bias is None or lin.bias.device == x.device)
                         and x.dtype == x0.dtype and x.dtype in (torch.float16, torch.bfloat16) and x.shape[-1] == x0.shape[-1]
                         and x.device == x0.device and x.numel() // max(1, x.shape[-1]) > SMALL_BATCH_ROWS
                         and bool(getattr(lin, "_use_quarot", False)) == rot)
    if ok:   # gates and residuals in the form the epilogue takes, else every layer goes alone
        for lin, x, gt, rs in zip(layers, xs, gates, residuals):
            shape = (*x.shape[:-1], lin.weight.shape[0])
            ok = ok and (rs is None or (tuple(rs.shape) == shape and rs.dtype == x.dtype and rs.device == x.device))
            ok = ok and (gt is None or (gt.device == x.device and x.dim() >= 2
                                        and compile_ops.modulation_broadcasts_over_tokens(_ShapeAndDtype(shape, x.dtype), gt, gt)))
    if not ok:
        return [lin(x, gate=gt, residual=rs) for lin, x, gt, rs in zip(layers, xs, gates, residuals)]
    scales = []
    for lin in layers:
        ws = lin._get_weight_scale()
        if isinstance(ws, Tensor) and ws.device != xs[0].device:
            ws = ws.to(xs[0].device, non_blocking=True)
        scales.append(ws)
    return int8_fused_kernel.hip_int8_linear_pair(xs, [lin.weight for lin in layers], scales, [lin.bias for lin in layers],
                                                  xs[0].dtype, rotate=rot, gates=gates, residuals=residuals)


def forward_fanout(layers, x, prologue: int = _lib.PRO_NONE, mod_scale=None, mod_shift=None, eps: float = 1e-6, norm_weight=None,
                   fused_add: bool = False):
    """[layer(x) for layer in layers] for quantised layers that read the same activations (separate q, k and v projections,
    the two up-projections of a SwiGLU feed-forward): x is quantised ONCE -- with `prologue` and its operands applied
    inside that quantiser, as forward(x, prologue=...) does for one layer -- and every layer runs its GEMM on the shared
    int8 rows.  The reference quantises in every Linear.forward (int8_quant.py:703-778); the quantiser being a function
    of its input, results are bit-identical to the layers' own forward calls, which is also the fall-back where a layer
    is not on the W8A8 path (dynamic LoRA, managed casting, different rotation flags, tracing).  With 16 rows or fewer
    (no prologue) the layers' small-batch W8A16 kernels go out as one launch instead."""
    layers = list(layers)
    if prologue == _lib.PRO_MODULATE_FUSED:
        prologue, fused_add = _lib.PRO_MODULATE, True
    rot = bool(getattr(layers[0], "_use_quarot", False)) if layers else False
    # 16 rows or fewer (the modulation projections of a block, which read the conditioning vector): the small-batch
    # W8A16 kernel of all the layers in one launch
    if (len(layers) >= 2 and prologue == _lib.PRO_NONE and not torch.compiler.is_compiling() and x.is_cuda and x.dim() >= 1
            and 0 < x.numel() // max(1, x.shape[-1]) <= SMALL_BATCH_ROWS and x.dtype in (torch.float16, torch.bfloat16)
            and all(getattr(lin, "_is_quantized", False) and lin.lora_A is None and lin.weight.device == x.device
                    and not (lin.comfy_cast_weights or len(lin.weight_function) > 0 or len(lin.bias_function) > 0)
                    and (lin.bias is None or lin.bias.device == x.device) and bool(getattr(lin, "_use_quarot", False)) == rot
                    and lin.weight.shape[1] == x.shape[-1] for lin in layers)):
        x_2d = x.reshape(-1, x.shape[-1])
        x_in = _lib.rotate128(x_2d) if rot else x_2d
        problems = []
        for lin in layers:
            ws = lin._get_weight_scale()
            if isinstance(ws, Tensor):
                if ws.device != x.device:
                    ws = ws.to(x.device, non_blocking=True)
                if not lin._is_per_row and ws.numel() != 1:
                    ws = ws.reshape(-1)[:1]
            problems.append((x_in, lin.weight, ws, lin.bias))
        return [y.reshape(*x.shape[:-1], y.shape[-1]) for y in _lib.linear_w8a16_small_m_grouped(problems)]
    ok = len(layers) >= 2 and not torch.compiler.is_compiling() and x.is_cuda and x.dim() >= 2 \
        and x.numel() // max(1, x.shape[-1]) > SMALL_BATCH_ROWS and x.dtype in (torch.float16, torch.bfloat16)
    for lin in layers:
        managed = lin.comfy_cast_weights or len(lin.weight_function) > 0 or len(lin.bias_function) > 0
        ok = ok and (getattr(lin, "_is_quantized", False) and not managed and lin.lora_A is None and lin.weight.device == x.device
                     and (lin.bias is None or lin.bias.device == x.device) and bool(getattr(lin, "_use_quarot", False)) == rot)
    if ok and prologue != _lib.PRO_NONE:
        # the checks of forward(): operands the quantiser does not take make every layer go alone (torch applies the operation)
        if prologue == _lib.PRO_CONCAT_GELU:
            ok = (isinstance(mod_scale, Tensor) and mod_scale.shape[:-1] == x.shape[:-1]
                  and _lib.concat_gelu_fusable(x.reshape(-1, x.shape[-1]), mod_scale.reshape(-1, mod_scale.shape[-1]))
                  and not (rot and (x.shape[-1] % 128 or mod_scale.shape[-1] % 128)))
        elif prologue == _lib.PRO_SILU_GATE:
            ok = isinstance(mod_scale, Tensor) and mod_scale.shape == x.shape and mod_scale.dtype == x.dtype
        elif prologue in (_lib.PRO_MODULATE, _lib.PRO_NORM_MODULATE):
            ok = (isinstance(mod_scale, Tensor) and isinstance(mod_shift, Tensor)
                  and compile_ops.modulation_broadcasts_over_tokens(x, mod_scale, mod_shift)
                  and (prologue == _lib.PRO_MODULATE or _lib.norm_modulate_fusable(x.reshape(-1, x.shape[-1]))))
        elif prologue == _lib.PRO_RMS_NORM:
            vecs = [v for v in (mod_scale, mod_shift) if v is not None]
            ok = (_lib.norm_modulate_fusable(x.reshape(-1, x.shape[-1]))
                  and (norm_weight is None or (norm_weight.dtype == x.dtype and tuple(norm_weight.shape) == (x.shape[-1],)
                                               and norm_weight.device == x.device))
                  and all(isinstance(v, Tensor) and v.device == x.device
                          and compile_ops.modulation_broadcasts_over_tokens(x, v, v) for v in vecs))
    width = x.shape[-1] + (mod_scale.shape[-1] if ok and prologue == _lib.PRO_CONCAT_GELU else 0)
    ok = ok and all(lin.weight.shape[1] == width for lin in layers)
    if not ok:
        return [lin(x, prologue=prologue, mod_scale=mod_scale, mod_shift=mod_shift, eps=eps, norm_weight=norm_weight, fused_add=fused_add)
                for lin in layers]
    lead = x.shape[:-1]
    q, s = _lib.quant_rowwise(x.reshape(-1, x.shape[-1]), rotate=rot, prologue=prologue, mod_scale=mod_scale, mod_shift=mod_shift,
                              eps=eps, norm_weight=norm_weight, fused_add=fused_add)
    outs = []
    for lin in layers:
        ws = lin._get_weight_scale()
        if isinstance(ws, Tensor):
            if ws.device != x.device:
                ws = ws.to(x.device, non_blocking=True)
            if not lin._is_per_row and ws.numel() != 1:
                ws = ws.reshape(-1)[:1]
        y = _lib.linear_w8a8(q, s, lin.weight, ws, lin.bias, x.dtype, int8_fused_kernel.DEFAULT_EPILOGUE)
        outs.append(y.reshape(*lead, lin.weight.shape[0]))
    return outs


# --------------------------------------------------------------------------- LoRA delta reconstruction
def reconstruct_lora_diff(weights, target_shape, device, dtype, strength):
    """Float delta of a LoRA / LoHA / LoKr patch and its scalar multiplier (int8_quant.py:128-208).
    Host-side torch; only the plain-LoRA product has a fused kernel (see the adapters)."""

    def dev(t):
        return t.to(device=device, dtype=dtype)

    def rank_scale(alpha, rank):
        return (alpha / rank) * strength if alpha is not None and rank is not None else strength

    n = len(weights)
    if n == 6:  # LoRA: (up, down, alpha, mid, dora_scale, reshape)
        up, down, alpha, mid = weights[0], weights[1], weights[2], weights[3]
        right = dev(down).flatten(1)
        if mid is not None:
            right = torch.mm(dev(mid).flatten(1), right)
        diff = torch.mm(dev(up).flatten(1), right)
        return diff.reshape(target_shape), rank_scale(alpha, down.shape[0])
    if n == 8:  # LoHA: (w1a, w1b, alpha, w2a, w2b, t1, t2, dora_scale)
        w1a, w1b, alpha, w2a, w2b, t1, t2 = weights[:7]
        if t1 is None:
            m1, m2 = torch.mm(dev(w1a), dev(w1b)), torch.mm(dev(w2a), dev(w2b))
        else:
            eq = "i j k l, j r, i p -> p r k l"
            m1 = torch.einsum(eq, dev(t1), dev(w1b), dev(w1a))
            m2 = torch.einsum(eq, dev(t2), dev(w2b), dev(w2a))
        return (m1 * m2).reshape(target_shape), rank_scale(alpha, w1b.shape[0])
    if n == 9:  # LoKr: (w1, w2, alpha, w1a, w1b, w2a, w2b, t2, dora_scale)
        w1, w2, alpha, w1a, w1b, w2a, w2b, t2 = weights[:8]
        rank = None
        if w1 is None:
            rank = w1b.shape[0]
            left = torch.mm(dev(w1a), dev(w1b))
        else:
            left = dev(w1)
        if w2 is None:
            rank = w2b.shape[0]
            if t2 is None:
                right = torch.mm(dev(w2a), dev(w2b))
            else:
                right = torch.einsum("i j k l, j r, i p -> p r k l", dev(t2), dev(w2b), dev(w2a))
        else:
            right = dev(w2)
        if right.dim() == 4:
            left = left.unsqueeze(2).unsqueeze(2)
        return torch.kron(left, right).reshape(target_shape), rank_scale(alpha, rank)
    return None, 1.0


def _slice_scale_offset_first(ws, delta_rows: int, offset):
    """Weight scale matching a (possibly narrowed) weight: INT8LoRAPatchAdapter's rule
    (the second definition at int8_quant.py:249-272 is the one in effect)."""
    if not isinstance(ws, Tensor) or ws.numel() == 1:
        return ws
    if offset is not None:
        dim, start, size = offset
        if dim < ws.dim() and ws.shape[dim] > start:
            return ws.narrow(dim, start, min(size, ws.shape[dim] - start))
    if ws.shape[0] != delta_rows and ws.shape[0] % delta_rows == 0:
        return ws[:delta_rows]
    return ws


def _slice_scale_mismatch_only(ws, delta_rows: int, offset):
    """INT8MergedLoRAPatchAdapter's older rule (int8_quant.py:341-352)."""
    if not isinstance(ws, Tensor) or ws.numel() == 1:
        return ws
    if offset is not None and ws.shape[0] != delta_rows:
        dim, start, size = offset
        if dim == 0:
            return ws.narrow(0, start, size)
    if ws.shape[0] != delta_rows and ws.shape[0] % delta_rows == 0:
        return ws[:delta_rows]
    return ws


def _draw_noise(shape, seed: int, device) -> Tensor:
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    return torch.rand(shape, generator=gen, device=device, dtype=torch.float32)


def _quarot_applies(weight: Tensor) -> bool:
    # the reference gates on the GLOBAL flag and K % 128, not on the module (int8_quant.py:300,387)
    return bool(getattr(Int8TensorwiseOps, "enable_quarot", False)) and weight.shape[1] % 128 == 0


def _plain_lora(weights):
    """(up, down) as 2-D matrices when the patch is a plain low-rank LoRA without a Tucker core."""
    if len(weights) == 6 and weights[3] is None and weights[0].dim() >= 2 and weights[1].dim() >= 2:
        return weights[0].flatten(1), weights[1].flatten(1)
    return None


class INT8LoRAPatchAdapter(LoRAAdapter):
    """Patches an int8 weight in int8 space: w' = sat8(w + SR(delta / w_scale))
    (int8_quant.py:218-323).  A plain LoRA is merged by the fused kernel straight from its
    factors; other adapter types are reconstructed in float first."""

    fuse_low_rank = True  # False: build delta with torch.mm like the reference, then merge

    def __init__(self, loaded_keys, weights, weight_scale, seed=0):
        super().__init__(loaded_keys, weights)
        self.weight_scale = weight_scale
        self.seed = seed

    def _get_effective_scale(self, delta_f, offset):
        rows = delta_f if isinstance(delta_f, int) else delta_f.shape[0]
        return _slice_scale_offset_first(self.weight_scale, rows, offset)

    def calculate_weight(self, weight, key, strength, strength_model, offset, function,
                         intermediate_dtype=torch.float32, original_weight=None):
        if intermediate_dtype == torch.int8:
            intermediate_dtype = torch.float32
        if weight.dtype != torch.int8:
            diff, mult = reconstruct_lora_diff(self.weights, weight.shape, weight.device, intermediate_dtype, strength)
            return weight if diff is None else weight + (diff * mult).to(weight.device, weight.dtype)

        home = weight.device
        dev = compute_device()
        w_dev = weight.to(dev)
        rotate = _quarot_applies(weight)
        eff = self._get_effective_scale(weight.shape[0], offset)
        noise = _draw_noise(tuple(weight.shape), self.seed, dev)
        plain = _plain_lora(self.weights) if self.fuse_low_rank else None
        if plain is not None and intermediate_dtype == torch.float32 and plain[1].shape[0] <= 256:
            up, down = (t.to(dev, torch.float32) for t in plain)
            alpha = self.weights[2]
            mult = (alpha / down.shape[0]) * strength if alpha is not None else strength
            if rotate:  # rotating the rows of up @ down is rotating the rows of down
                down = _lib.rotate128(down)
            merged = _lib.lora_merge_sr(w_dev, eff, noise, up=up, down=down, lora_scale=mult)
        else:
            diff, mult = reconstruct_lora_diff(self.weights, weight.shape, dev, intermediate_dtype, strength)
            if diff is None:
                return weight
            delta = (diff * mult).float()
            if rotate:
                delta = _lib.rotate128(delta, out=delta)
            merged = _lib.lora_merge_sr(w_dev, eff, noise, delta=delta)
        return merged.to(home)


class INT8MergedLoRAPatchAdapter(LoRAAdapter):
    """Sums several LoRA deltas in float and applies ONE stochastic rounding step
    (int8_quant.py:325-408).  `patches` is a list of (adapter, strength)."""

    def __init__(self, patches, weight_scale, seed=0):
        first = patches[0][0]
        super().__init__(first.loaded_keys, first.weights)
        self.patches = patches
        self.weight_scale = weight_scale
        self.seed = seed

    def _get_effective_scale(self, delta_f, offset):
        rows = delta_f if isinstance(delta_f, int) else delta_f.shape[0]
        return _slice_scale_mismatch_only(self.weight_scale, rows, offset)

    def calculate_weight(self, weight, key, strength, strength_model, offset, function,
                         intermediate_dtype=torch.float32, original_weight=None):
        if intermediate_dtype == torch.int8:
            intermediate_dtype = torch.float32
        home = weight.device
        dev = compute_device() if weight.dtype == torch.int8 else home
        total = None
        for adapter, lora_strength in self.patches:  # ComfyUI's own `strength` is ignored here, as in the reference
            diff, mult = reconstruct_lora_diff(adapter.weights, weight.shape, dev, intermediate_dtype, lora_strength)
            if diff is None:
                continue
            total = diff * mult if total is None else total.add_(diff * mult)
        if total is None:
            return weight
        if weight.dtype != torch.int8:
            return weight + total.to(home, weight.dtype)
        total = total.float()
        if _quarot_applies(weight):
            total = _lib.rotate128(total, out=total)
        eff = self._get_effective_scale(weight.shape[0], offset)
        noise = _draw_noise(tuple(weight.shape), self.seed, dev)
        return _lib.lora_merge_sr(weight.to(dev), eff, noise, delta=total).to(home)


# --------------------------------------------------------------------------- ComfyUI custom operations
class Int8TensorwiseOps(manual_cast):
    """`custom_operations` class for comfy.sd.load_diffusion_model (int8_quant.py:522-792)."""

    excluded_names: list = []
    dynamic_quantize = False   # quantise float checkpoints while loading
    enable_quarot = False      # rotate weights at load, activations in the quantiser
    use_triton = True          # kept for callers that set it; there is one (HIP) path
    _is_prequantized = False

    class Linear(manual_cast.Linear):
        def __init__(self, *args, **kwargs):
            super().__init__(*args, **kwargs)
            self.register_buffer("weight_scale", None)
            self._is_quantized = False
            self._is_per_row = False
            self._use_quarot = False
            self._weight_scale_scalar = None
            self.compute_dtype = torch.bfloat16
            self.lora_A = None
            self.lora_B = None
            self.lora_alpha = None

        def reset_parameters(self):
            return None

        # -- loading ---------------------------------------------------------------------
        def _adopt_scale(self, scale) -> None:
            """Scalar -> Python float (tensorwise); [N,1] -> per-row buffer; other tensors are kept
            as a buffer and treated as one scale (int8_quant.py:568-585)."""
            if isinstance(scale, Tensor) and scale.numel() != 1:
                self.register_buffer("weight_scale", scale.float())
                self._weight_scale_scalar = None
                self._is_per_row = scale.dim() == 2 and scale.shape[1] == 1
            else:
                self._weight_scale_scalar = float(scale.float().item()) if isinstance(scale, Tensor) else float(scale)
                self.weight_scale = None
                self._is_per_row = False

        def _quantize_on_load(self, w: Tensor) -> None:
            """Float checkpoint weight -> rowwise int8 (+ QuaRot) on the GPU, stored on the CPU for
            ComfyUI to place (int8_quant.py:595-620).  Rotation and quantisation are one kernel."""
            w_dev = w.to(compute_device(), non_blocking=True).float()
            self._use_quarot = bool(Int8TensorwiseOps.enable_quarot) and self.in_features % 128 == 0
            q, s = _lib.quant_rowwise(w_dev, rotate=self._use_quarot)
            self.weight = nn.Parameter(q.cpu(), requires_grad=False)
            self.register_buffer("weight_scale", s.cpu())
            self._weight_scale_scalar = None
            self._is_quantized = True
            self._is_per_row = True

        def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys,
                                  unexpected_keys, error_msgs):
            scale = state_dict.pop(prefix + "weight_scale", None)
            state_dict.pop(prefix + "comfy_quant", None)
            state_dict.pop(prefix + "input_scale", None)  # static activation scales are not used
            w = state_dict.pop(prefix + "weight", None)
            bias = state_dict.pop(prefix + "bias", None)

            if w is None:
                missing_keys.append(prefix + "weight")
            elif w.dtype == torch.int8 and scale is not None:
                self._is_quantized = True
                self.weight = nn.Parameter(w, requires_grad=False)
                Int8TensorwiseOps._is_prequantized = True
                self._adopt_scale(scale)
            elif w.dtype in (torch.float16, torch.bfloat16, torch.float32):
                skip = (
                    any(name in prefix for name in Int8TensorwiseOps.excluded_names)
                    or self.in_features == 1 or self.out_features == 1 or w.ndim == 1
                    or not Int8TensorwiseOps.dynamic_quantize
                )
                if skip:
                    self._is_quantized = False
                    self.weight = nn.Parameter(w, requires_grad=False)
                else:
                    self._quantize_on_load(w)
            else:
                self._is_quantized = False
                self.weight = nn.Parameter(w, requires_grad=False)

            self.bias = None if bias is None else nn.Parameter(bias, requires_grad=False)

            # ComfyUI sizes its staging buffers from these; they were recorded before loading
            if self.weight is not None:
                self.weight_comfy_model_dtype = self.weight.dtype
            if self.weight_scale is not None:
                self.weight_scale_comfy_model_dtype = self.weight_scale.dtype
            if self.bias is not None:
                self.bias_comfy_model_dtype = self.bias.dtype

        def _get_weight_scale(self):
            return self._weight_scale_scalar if self._weight_scale_scalar is not None else self.weight_scale

        # -- ModelPatcher hooks -------------------------------------------------------------
        def convert_weight(self, _weight, inplace=False):
            return self.weight if self._is_quantized else _weight

        def _install_weight(self, new_weight, inplace_update):
            if inplace_update:
                self.weight.data.copy_(new_weight)
            else:
                self.weight = nn.Parameter(new_weight, requires_grad=False)

        def set_weight(self, out_weight, inplace_update=False, seed=0, return_weight=False, **kwargs):
            if not self._is_quantized:
                new_weight = out_weight.to(self.weight.dtype)
            elif out_weight.dtype == torch.int8:
                new_weight = out_weight
            else:  # a float patch fell through: requantise with this layer's own scale
                new_weight = stochastic_round_int8_delta(out_weight, self._get_weight_scale(), seed)
            if return_weight:
                return new_weight
            self._install_weight(new_weight, inplace_update)

        def set_bias(self, out_bias, inplace_update=False, seed=0, return_weight=False, **kwargs):
            if out_bias is None:
                return None
            if return_weight:
                return out_bias
            if inplace_update:
                if self.bias is not None:
                    self.bias.data.copy_(out_bias)
            else:
                self.bias = nn.Parameter(out_bias, requires_grad=False)

        # -- forward ------------------------------------------------------------------------
        def forward(self, x: Tensor, prologue: int = _lib.PRO_NONE, mod_scale: Tensor | None = None,
                    mod_shift: Tensor | None = None, eps: float = 1e-6, gate: Tensor | None = None,
                    residual: Tensor | None = None, norm_weight: Tensor | None = None, fused_add: bool = False) -> Tensor:
            """The reference's forward(x) (int8_quant.py:703-778).  The optional arguments name the elementwise
            operation the caller would otherwise apply to x first -- _lib.PRO_GELU_TANH, _lib.PRO_MODULATE with
            (1 + mod_scale) * x + mod_shift, vectors broadcast over the token dimension, _lib.PRO_NORM_MODULATE with
            the same modulation of layer_norm(x, eps) (no affine parameters: the whole adaLN producer of a DiT
            block), _lib.PRO_CONCAT_GELU with cat((x, gelu(mod_scale)), -1), the input of the second projection of a
            single-stream block, _lib.PRO_GELU_ERF (GELU in its exact form), _lib.PRO_RMS_NORM with
            rms_norm(x, norm_weight, eps) followed by * (1 + mod_scale) and + mod_shift where those are given (the
            producer in blocks that normalise with an RMSNorm; fused_add=True in the three modulating kinds: product and
            sum rounded once, as torch.addcmul(mod_shift, x, 1 + mod_scale) computes them), or _lib.PRO_SILU_GATE with silu(x) * mod_scale, the gate operand of x's shape -- which the W8A8
            path then applies inside its quantiser instead of in passes of their own (under torch.compile the graph
            rewrite of compile_ops does this without the caller's help).  `gate` / `residual` name what the caller would
            apply to the result: forward(h, gate=g, residual=x) returns x + g * linear(h), the gated residual of an
            adaLN-Zero block (g broadcast over the token dimension like the modulation vectors), formed inside the GEMM
            epilogue with the roundings of torch's two operations; gate or residual alone work the same way."""
            managed = self.comfy_cast_weights or len(self.weight_function) > 0 or len(self.bias_function) > 0
            fuse_epilogue = False
            if gate is not None or residual is not None:
                cdt = x.dtype if x.dtype in (torch.float16, torch.bfloat16) else torch.bfloat16
                out_shape = (*x.shape[:-1], self.weight.shape[0])
                fuse_epilogue = (self._is_quantized and x.numel() // max(1, x.shape[-1]) > SMALL_BATCH_ROWS and self.lora_A is None
                                 and not torch.compiler.is_compiling() and x.dim() >= 2
                                 and (residual is None or (tuple(residual.shape) == out_shape and residual.dtype == cdt
                                                           and residual.device == x.device))
                                 and (gate is None or (gate.device == x.device and compile_ops.modulation_broadcasts_over_tokens(
                                     _ShapeAndDtype(out_shape, cdt), gate, gate))))
                if not fuse_epilogue:   # torch applies the two operations, as the caller would have
                    y = self.forward(x, prologue, mod_scale, mod_shift, eps, norm_weight=norm_weight, fused_add=fused_add)
                    if gate is not None:
                        y = gate * y
                    return y if residual is None else residual + y
            if prologue != _lib.PRO_NONE:
                rows = x.numel() // max(1, x.shape[-1])
                fusable = (self._is_quantized and rows > SMALL_BATCH_ROWS and self.lora_A is None
                           and not torch.compiler.is_compiling())
                if prologue == _lib.PRO_MODULATE_FUSED:
                    prologue, fused_add = _lib.PRO_MODULATE, True
                if fused_add and x.dtype not in (torch.float16, torch.bfloat16):
                    fusable = False                      # (the one-rounding form exists for 16-bit tensors)
                if fusable and prologue == _lib.PRO_CONCAT_GELU:   # x followed by gelu(mod_scale) along the feature dimension
                    fusable = (isinstance(mod_scale, Tensor) and mod_scale.shape[:-1] == x.shape[:-1]
                               and x.shape[-1] + mod_scale.shape[-1] == self.weight.shape[1]
                               and _lib.concat_gelu_fusable(x.reshape(-1, x.shape[-1]), mod_scale.reshape(-1, mod_scale.shape[-1]))
                               and not (getattr(self, "_use_quarot", False) and (x.shape[-1] % 128 or mod_scale.shape[-1] % 128)))
                    if fusable:
                        mod_scale = mod_scale.reshape(-1, mod_scale.shape[-1])
                if fusable and prologue == _lib.PRO_SILU_GATE:   # the gate operand has x's shape and dtype, or torch does it
                    fusable = isinstance(mod_scale, Tensor) and mod_scale.shape == x.shape and mod_scale.dtype == x.dtype
                if fusable and prologue in (_lib.PRO_MODULATE, _lib.PRO_NORM_MODULATE):
                    # vectors of another dtype or another broadcast pattern are torch's business (as under compile)
                    fusable = (isinstance(mod_scale, Tensor) and isinstance(mod_shift, Tensor) and x.dim() >= 2
                               and compile_ops.modulation_broadcasts_over_tokens(x, mod_scale, mod_shift))
                if fusable and prologue == _lib.PRO_RMS_NORM:
                    vecs = [v for v in (mod_scale, mod_shift) if v is not None]
                    fusable = (x.dim() >= 2 and _lib.norm_modulate_fusable(x.reshape(-1, x.shape[-1]))
                               and (norm_weight is None or (norm_weight.dtype == x.dtype and tuple(norm_weight.shape) == (x.shape[-1],)
                                                            and norm_weight.device == x.device))
                               and all(isinstance(v, Tensor) and v.device == x.device
                                       and compile_ops.modulation_broadcasts_over_tokens(x, v, v) for v in vecs))
                if prologue == _lib.PRO_NORM_MODULATE and not (fusable and _lib.norm_modulate_fusable(x.reshape(-1, x.shape[-1]))):
                    # rows the normalising quantiser does not take: torch normalises, the modulation may still be fused
                    x = F.layer_norm(x, (x.shape[-1],), eps=eps)
                    prologue = _lib.PRO_MODULATE
                if not fusable:   # every other path takes the operation as torch would have applied it
                    if prologue == _lib.PRO_GELU_TANH:
                        x = F.gelu(x, approximate="tanh")
                    elif prologue == _lib.PRO_GELU_ERF:
                        x = F.gelu(x)
                    elif prologue == _lib.PRO_RMS_NORM:
                        x = F.rms_norm(x, (x.shape[-1],), norm_weight, eps)
                        if fused_add and mod_scale is not None and mod_shift is not None:
                            x = torch.addcmul(mod_shift, x, 1 + mod_scale)
                        else:
                            if mod_scale is not None:
                                x = x * (1 + mod_scale)
                            if mod_shift is not None:
                                x = x + mod_shift
                    elif prologue == _lib.PRO_CONCAT_GELU:
                        x = torch.cat((x, F.gelu(mod_scale, approximate="tanh")), -1)
                    elif prologue == _lib.PRO_SILU_GATE:
                        x = F.silu(x) * mod_scale
                    elif fused_add:
                        x = torch.addcmul(mod_shift, x, 1 + mod_scale)
                    else:
                        x = (1 + mod_scale) * x + mod_shift
                    prologue = _lib.PRO_NONE

            if not self._is_quantized:
                if not managed:
                    return F.linear(x, self.weight, self.bias)
                weight, bias, offload_stream = cast_bias_weight(self, x, offloadable=True)
                out = F.linear(x, weight, bias)
                uncast_bias_weight(self, weight, bias, offload_stream)
                return out

            if managed:
                weight, bias, offload_stream = cast_bias_weight(
                    self, input=None, dtype=torch.int8, device=x.device, bias_dtype=x.dtype, offloadable=True)
            else:
                weight, bias, offload_stream = self.weight, self.bias, None
                if weight.device != x.device:  # outside ComfyUI nobody placed the module
                    weight = weight.to(x.device)
                    bias = None if bias is None else bias.to(x.device)

            w_scale = self._get_weight_scale()
            if isinstance(w_scale, Tensor) and w_scale.device != x.device:
                w_scale = w_scale.to(x.device, non_blocking=True)
            if isinstance(w_scale, Tensor) and not self._is_per_row and w_scale.numel() != 1:
                # a one-scale layer whose scale tensor has several elements: element 0 counts, in eager mode and
                # under torch.compile alike (the reference's kernel reads b_scale_ptr[0], int8_fused_kernel.py:153)
                w_scale = w_scale.reshape(-1)[:1]

            compute_dtype = x.dtype if x.dtype in (torch.float16, torch.bfloat16) else torch.bfloat16
            x_2d = x.reshape(-1, x.shape[-1])
            rotate = bool(getattr(self, "_use_quarot", False))

            # Dynamic (unmerged) LoRA side branch, float; it is fed the rotated activations when QuaRot
            # is on, as in the reference (int8_quant.py:741-744,768).  On the W8A8 path its second product
            # and its sum with the main result happen inside the GEMM epilogue when the factors have the
            # compute dtype and a rank up to 64 (no [M,N] side tensor at all); otherwise the side tensor is
            # formed by torch and only added inside the epilogue (same rounding as the reference's
            # `y + lora_out.to(y.dtype)`, one pass over [M,N] less).
            side = None
            side_factors = None   # (lora_x, lB, alpha): the second product happens inside the GEMM epilogue
            compiling = torch.compiler.is_compiling()
            if self.lora_A is not None and self.lora_B is not None:
                lA = self.lora_A.to(x.device, non_blocking=True)
                lB = self.lora_B.to(x.device, non_blocking=True)
                if not rotate:
                    x_side = x_2d
                elif compiling:
                    x_side = torch.ops.i8f.rotate128(x_2d)
                else:
                    x_side = _lib.rotate128(x_2d)
                x_side = x_side.to(lA.dtype)
                rows = x_2d.shape[0]
                if (rows > SMALL_BATCH_ROWS and lB.dtype == lA.dtype
                        and (self.lora_alpha is None or isinstance(self.lora_alpha, (int, float)))
                        and _lib.lora_side_fusable(rows, weight.shape[0], weight.shape[1], lA.shape[0], compute_dtype, lA.dtype)):
                    # (the first product stays with torch: it is bound by the same per-CU load path whoever issues the
                    # loads, and an own kernel for it measured no faster than the BLAS library's 9.5 us at 4608 x 3072)
                    side_factors = (F.linear(x_side, lA), lB, self.lora_alpha)
                else:
                    side = F.linear(F.linear(x_side, lA), lB)
                    if self.lora_alpha is not None:
                        side = side * self.lora_alpha

            if x_2d.shape[0] > SMALL_BATCH_ROWS:
                addend = None if side is None else side.to(compute_dtype)
                if compiling:  # under torch.compile the call goes through the registered operators
                    ws_t, ws_v = compile_ops.split_scale(w_scale)
                    if side_factors is not None:
                        alpha = None if self.lora_alpha is None else float(self.lora_alpha)
                        y = torch.ops.i8f.int8_linear_lora(x_2d, weight, ws_t, ws_v, bias, compute_dtype, rotate,
                                                           int8_fused_kernel.DEFAULT_EPILOGUE, side_factors[0], lB, alpha)
                    else:
                        y = torch.ops.i8f.int8_linear(x_2d, weight, ws_t, ws_v, bias, compute_dtype, rotate,
                                                      int8_fused_kernel.DEFAULT_EPILOGUE, addend)
                else:
                    fwd = int8_forward_dynamic_per_row if self._is_per_row else int8_forward_dynamic
                    pro = None if prologue == _lib.PRO_NONE else (prologue, mod_scale, mod_shift, eps, norm_weight, fused_add)
                    if fuse_epilogue:   # (no dynamic LoRA here: the addend slot is free for the residual stream)
                        addend = None if residual is None else residual.reshape(-1, residual.shape[-1])
                    y = fwd(x_2d, weight, w_scale, bias, compute_dtype, rotate=rotate, addend=addend, prologue=pro,
                            side=side_factors, gate=gate if fuse_epilogue else None)
            else:
                # W8A16: activations keep their dtype (rotated first when the weight is rotated)
                if compiling:
                    ws_t, ws_v = compile_ops.split_scale(w_scale)
                    y = torch.ops.i8f.linear_w8a16_small_m(x_2d, weight, ws_t, ws_v, bias, rotate)
                else:
                    x_in = _lib.rotate128(x_2d) if rotate else x_2d
                    y = _lib.linear_w8a16_small_m(x_in, weight, w_scale, bias)
                if side is not None:
                    y = y + side.to(y.dtype)

            if managed:
                uncast_bias_weight(self, weight, bias, offload_stream)
            return y.reshape(*x.shape[:-1], y.shape[-1])

    class GroupNorm(manual_cast.GroupNorm):
        pass

    class LayerNorm(manual_cast.LayerNorm):
        pass

    class Conv2d(manual_cast.Conv2d):
        pass

    class Conv3d(manual_cast.Conv3d):
        pass

    class ConvTranspose2d(manual_cast.ConvTranspose2d):
        pass

    class Embedding(manual_cast.Embedding):
        pass

    @classmethod
    def conv_nd(cls, dims, *args, **kwargs):
        if dims == 2:
            return cls.Conv2d(*args, **kwargs)
        if dims == 3:
            return cls.Conv3d(*args, **kwargs)
        raise ValueError(f"unsupported dimensions: {dims}")
