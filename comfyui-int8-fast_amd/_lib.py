"""ctypes binding of libi8f_gfx950.so (the C ABI declared in include/i8f.h).

This is the only place the package touches the native library.  There is no
fallback: if the library is missing or the tensors are not on a gfx950 device,
the functions raise.  Tensors are torch tensors used as device memory; the
library launches on torch's current HIP stream.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libi8f_gfx950.so")

BF16, F16, F32 = 0, 1, 2
SCALE_TENSOR, SCALE_ROW = 0, 1
EPI_TORCH, EPI_FUSED = 0, 1
PRO_NONE, PRO_MODULATE, PRO_GELU_TANH, PRO_SILU_GATE, PRO_NORM_MODULATE, PRO_CONCAT_GELU, PRO_GELU_ERF, PRO_RMS_NORM = 0, 1, 2, 3, 4, 5, 6, 7
PRO_MODULATE_FUSED = 8   # the modulation as torch.addcmul(shift, x, 1 + scale): product and sum rounded once

_DT = {torch.bfloat16: BF16, torch.float16: F16, torch.float32: F32}

_lib = None


class I8FError(RuntimeError):
    """A call into libi8f_gfx950.so returned a negative status."""

    def __init__(self, what: str, status: int, text: str, hip_error: int = 0):
        self.status = status
        self.hip_error = hip_error
        extra = f", hipError {hip_error}" if hip_error else ""
        super().__init__(f"{what}: status {status} ({text}{extra})")


def lib() -> ctypes.CDLL:
    """Load the library once.  Raises RuntimeError with the build command if it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python {os.path.join(_HERE, 'build.py')}` "
            "(needs hipcc; the INT8 path has no other implementation)."
        )
    L = ctypes.CDLL(LIB_PATH)
    vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
    L.i8f_version.restype = i32
    L.i8f_status_string.restype = ctypes.c_char_p
    L.i8f_status_string.argtypes = [i32]
    L.i8f_last_hip_error.restype = i32
    L.i8f_quant_rowwise.argtypes = [vp, i32, i64, i64, i64, i32, vp, vp, vp]
    L.i8f_rotate128.argtypes = [vp, i32, i64, i64, i64, vp, vp]
    L.i8f_quant_rowwise_grouped.argtypes = [vp, i32, i32, i64, i32, vp]
    L.i8f_quant_rowwise_prologue.argtypes = [vp, i32, i64, i64, i64, i32, vp, vp, i64, i32, vp, vp, vp]
    L.i8f_quant_rowwise_norm_modulate.argtypes = [vp, i32, i64, i64, i64, f32, vp, vp, i64, i32, i32, vp, vp, vp]
    L.i8f_quant_rowwise_rms_norm.argtypes = [vp, i32, i64, i64, i64, f32, vp, vp, vp, i64, i32, i32, vp, vp, vp]
    L.i8f_quant_rowwise_concat_gelu.argtypes = [vp, i32, i64, i64, i64, vp, i64, i64, i32, vp, vp, vp]
    L.i8f_quant_tensorwise_workspace_bytes.argtypes = [i64]
    L.i8f_quant_tensorwise_workspace_bytes.restype = i64
    L.i8f_quant_tensorwise.argtypes = [vp, i32, i64, vp, vp, vp, i64, vp]
    L.i8f_quant_tensorwise_static.argtypes = [vp, i32, i64, vp, vp, vp]
    L.i8f_gemm_i32.argtypes = [vp, vp, i64, i64, i64, vp, vp]
    L.i8f_gemm_tile.argtypes = [i64, i64, i64, ctypes.POINTER(i32), ctypes.POINTER(i32), ctypes.POINTER(i32)]
    L.i8f_gemm_tile.restype = i32
    L.i8f_linear_w8a8.argtypes = [vp, vp, vp, vp, f32, i32, vp, i32, vp, i32, i64, i64, i64, i32, vp]
    L.i8f_linear_w8a8_add.argtypes = [vp, vp, vp, vp, f32, i32, vp, i32, vp, vp, i32, i64, i64, i64, i32, vp]
    L.i8f_linear_w8a8_splitk.argtypes = [vp, vp, vp, vp, f32, i32, vp, i32, vp, vp, i32, i64, i64, i64, i32, vp, i64, vp]
    L.i8f_linear_w8a8_grouped.argtypes = [vp, i32, i32, i32, i32, i64, i64, i32, vp, i64, vp]
    L.i8f_linear_w8a8_gated.argtypes = [vp, vp, vp, vp, f32, i32, vp, i32, vp, i64, vp, vp, i32, i64, i64, i64, i32, vp, i64, vp]
    L.i8f_linear_w8a8_workspace_bytes.argtypes = []
    L.i8f_linear_w8a8_workspace_bytes.restype = i64
    L.i8f_linear_w8a8_lora.argtypes = [vp, vp, vp, vp, f32, i32, vp, i32, vp, vp, i64, i32, f32, vp, i32, i64, i64, i64, i32, vp]
    L.i8f_linear_w8a16_small_m.argtypes = [vp, i32, i64, i64, i64, vp, vp, f32, i32, vp, i32, vp, i64, vp]
    L.i8f_linear_w8a16_small_m_grouped.argtypes = [vp, i32, i32, i32, i32, vp]
    L.i8f_sr_quant_delta.argtypes = [vp, vp, f32, i32, vp, i64, i64, vp, vp]
    L.i8f_lora_merge_sr.argtypes = [vp, vp, f32, i32, vp, vp, vp, i64, f32, vp, i64, i64, vp, vp]
    for name in ("i8f_quant_rowwise_concat_gelu", "i8f_quant_rowwise_rms_norm", "i8f_linear_w8a8_gated", "i8f_quant_rowwise", "i8f_quant_rowwise_grouped", "i8f_quant_rowwise_prologue", "i8f_quant_rowwise_norm_modulate", "i8f_quant_tensorwise", "i8f_quant_tensorwise_static", "i8f_rotate128", "i8f_gemm_i32", "i8f_linear_w8a8", "i8f_linear_w8a8_add", "i8f_linear_w8a8_splitk", "i8f_linear_w8a8_grouped", "i8f_linear_w8a8_lora",
                 "i8f_linear_w8a16_small_m", "i8f_linear_w8a16_small_m_grouped", "i8f_sr_quant_delta", "i8f_lora_merge_sr"):
        getattr(L, name).restype = i32
    _lib = L
    return L


EXPORTS = (
    "i8f_version", "i8f_status_string", "i8f_last_hip_error", "i8f_quant_rowwise", "i8f_quant_rowwise_grouped", "i8f_rotate128",
    "i8f_quant_tensorwise_workspace_bytes", "i8f_quant_tensorwise", "i8f_quant_tensorwise_static", "i8f_quant_rowwise_prologue", "i8f_quant_rowwise_norm_modulate", "i8f_quant_rowwise_concat_gelu",
    "i8f_quant_rowwise_rms_norm",
    "i8f_gemm_i32", "i8f_gemm_tile", "i8f_linear_w8a8", "i8f_linear_w8a8_add", "i8f_linear_w8a8_workspace_bytes", "i8f_linear_w8a8_splitk", "i8f_linear_w8a8_gated", "i8f_linear_w8a8_grouped", "i8f_linear_w8a8_lora", "i8f_linear_w8a16_small_m", "i8f_linear_w8a16_small_m_grouped", "i8f_sr_quant_delta", "i8f_lora_merge_sr",
)


def _check(status: int, what: str) -> None:
    if status != 0:
        L = lib()
        text = L.i8f_status_string(status).decode()
        raise I8FError(what, status, text, L.i8f_last_hip_error() if status == -3 else 0)


def _dev(t: torch.Tensor, name: str) -> None:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} is on {t.device}: the INT8 engine runs on a gfx950 GPU only (no CPU path)")


class _Nop:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NOP = _Nop()


def _on(device):
    """Context that makes `device` current for the call: nothing to do (and nothing to pay) when it already is."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NOP
    return torch.cuda.device(device)


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor):
    """torch's current stream on t's device as the void * the library takes (the raw handle: building a
    torch.cuda.Stream object for it costs several microseconds per call)."""
    if _raw_stream is not None and t.device.index is not None:
        return ctypes.c_void_p(_raw_stream(t.device.index))
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DT[dt]
    except KeyError:
        raise TypeError(f"unsupported dtype {dt}; expected bfloat16, float16 or float32") from None


def _rows(x: torch.Tensor, name: str) -> torch.Tensor:
    """A 2-D view whose rows are contiguous (row stride may exceed K)."""
    if x.dim() != 2:
        raise ValueError(f"{name} must be 2-D, got shape {tuple(x.shape)}")
    if x.shape[1] > 1 and x.stride(1) != 1:
        x = x.contiguous()
    if x.shape[0] > 1 and x.stride(0) < x.shape[1]:
        x = x.contiguous()
    return x


def _scale(ws, N: int, device):
    """-> (device tensor or None, host float, mode).  Python floats travel by value."""
    if isinstance(ws, torch.Tensor):
        if ws.numel() == 1 and not ws.is_cuda:
            return None, float(ws.item()), SCALE_TENSOR
        if ws.device != device:
            ws = ws.to(device, non_blocking=True)
        ws = ws.reshape(-1)
        if ws.dtype != torch.float32:
            ws = ws.float()
        ws = ws.contiguous()
        if ws.numel() == 1:
            return ws, 0.0, SCALE_TENSOR
        if ws.numel() != N:
            raise ValueError(f"weight scale has {ws.numel()} elements, expected 1 or {N}")
        return ws, 0.0, SCALE_ROW
    return None, float(ws), SCALE_TENSOR


# --------------------------------------------------------------------------- entry points
def concat_gelu_fusable(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Whether the quantiser takes cat(a, gelu(b)) itself (PRO_CONCAT_GELU): 2-D tensors of one 16-bit dtype and one row
    count on one GPU, widths in multiples of 16 that add up to at most 16384, contiguous 16-byte aligned rows."""
    def rows_ok(t):
        return t.stride(1) == 1 and (t.shape[0] <= 1 or (t.stride(0) % 8 == 0 and t.stride(0) >= t.shape[1])) and t.data_ptr() % 16 == 0

    return (a.is_cuda and a.dim() == 2 and b.dim() == 2 and a.dtype == b.dtype and a.dtype in (torch.bfloat16, torch.float16)
            and a.device == b.device and a.shape[0] == b.shape[0] and a.shape[0] > 0 and a.shape[1] % 16 == 0 and b.shape[1] % 16 == 0
            and a.shape[1] > 0 and b.shape[1] > 0 and a.shape[1] + b.shape[1] <= 16384 and rows_ok(a) and rows_ok(b))


def quant_rowwise_concat_gelu(a: torch.Tensor, b: torch.Tensor, rotate: bool = False):
    """quant_rowwise(cat((a, gelu(b, approximate="tanh")), -1)) without the activated tensor or the concatenation ever
    existing: the input of the second projection of a single-stream transformer block.  a [M,Ka], b [M,Kb]
    -> (int8 [M, Ka+Kb], float32 [M,1])."""
    _dev(a, "a")
    _dev(b, "b")
    if a.dim() > 2:   # leading dimensions are rows
        a = a.reshape(-1, a.shape[-1])
    if b.dim() > 2:
        b = b.reshape(-1, b.shape[-1])
    if a.dim() == 2 and b.dim() == 2 and not concat_gelu_fusable(a, b):   # rows that are not contiguous or aligned: copies
        a, b = a.contiguous(), b.contiguous()
    if a.dim() != 2 or b.dim() != 2 or not concat_gelu_fusable(a, b):
        raise ValueError("these tensors have no fused concatenation (see concat_gelu_fusable)")
    M, Ka = a.shape
    Kb = b.shape[1]
    if rotate and (Ka % 128 or Kb % 128):
        raise ValueError(f"rotation needs both widths in multiples of 128, got {Ka} and {Kb}")
    q = torch.empty((M, Ka + Kb), dtype=torch.int8, device=a.device)
    s = torch.empty((M, 1), dtype=torch.float32, device=a.device)
    with _on(a.device):
        _check(lib().i8f_quant_rowwise_concat_gelu(_ptr(a), dtype_code(a.dtype), M, Ka, a.stride(0) if M > 1 else Ka, _ptr(b), Kb,
                                                   b.stride(0) if M > 1 else Kb, 128 if rotate else 0, _ptr(q), _ptr(s), _stream(a)),
               "i8f_quant_rowwise_concat_gelu")
    return q, s


def norm_modulate_fusable(x: torch.Tensor) -> bool:
    """Whether the quantiser takes PRO_NORM_MODULATE for these rows (the row stays in the registers of one to four wavefronts): 16-bit elements,
    a width of at most 16384 in multiples of 16, 16-byte aligned rows."""
    return (x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and x.dim() == 2 and 0 < x.shape[1] <= 16384 and x.shape[1] % 16 == 0
            and x.stride(1) == 1 and (x.shape[0] <= 1 or x.stride(0) % 8 == 0) and x.data_ptr() % 16 == 0)


def quant_rowwise_rms_norm(x: torch.Tensor, eps: float = 1e-6, weight=None, mod_scale=None, mod_shift=None, rotate: bool = False,
                           fused_add: bool = False):
    """quant_rowwise of rms_norm(x, weight, eps) [* (1 + mod_scale)] [+ mod_shift] with no intermediate tensor in memory:
    the producer of the projections of blocks that normalise with an RMSNorm.  x [M,K] as norm_modulate_fusable
    describes; weight [K]; mod_scale / mod_shift [V,K] (or [K]), M // V consecutive rows to a vector; each optional."""
    _dev(x, "x")
    if not norm_modulate_fusable(x):
        raise ValueError("the normalising quantiser takes contiguous 16-bit rows of at most 16384 elements in multiples of 16 "
                         "(see norm_modulate_fusable); normalise with torch")
    M, K = x.shape
    if rotate and K % 128:
        raise ValueError(f"rotation needs K % 128 == 0, got K={K}")
    if weight is not None:
        _dev(weight, "weight")
        if weight.dtype != x.dtype or weight.device != x.device or weight.numel() != K:
            raise ValueError(f"weight must be [{K}] of {x.dtype} on {x.device}")
        weight = weight.reshape(K).contiguous()
    rows_per_vec, vecs = 1, []
    for name, v in (("mod_scale", mod_scale), ("mod_shift", mod_shift)):
        if v is not None:
            _dev(v, name)
            if v.dtype != x.dtype or v.device != x.device or v.numel() % K or v.shape[-1] != K:
                raise ValueError(f"{name} must be [V,{K}] of {x.dtype} on {x.device}")
            v = v.reshape(-1, K).contiguous()
            if v.shape[0] == 0 or M % v.shape[0] or (vecs and vecs[0] is not None and vecs[0].shape[0] != v.shape[0]):
                raise ValueError(f"{M} rows do not split evenly over the modulation vectors")
            rows_per_vec = max(1, M // v.shape[0])
        vecs.append(v)
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    s = torch.empty((M, 1), dtype=torch.float32, device=x.device)
    with _on(x.device):
        _check(lib().i8f_quant_rowwise_rms_norm(_ptr(x), dtype_code(x.dtype), M, K, x.stride(0) if M > 1 else K, float(eps),
                                                _ptr(weight) if weight is not None else None, *(None if v is None else _ptr(v) for v in vecs),
                                                rows_per_vec, int(bool(fused_add)), 128 if rotate else 0, _ptr(q), _ptr(s), _stream(x)),
               "i8f_quant_rowwise_rms_norm")
    return q, s


def quant_rowwise(x: torch.Tensor, rotate: bool = False, prologue: int = PRO_NONE, mod_scale=None, mod_shift=None, eps: float = 1e-6,
                  norm_weight=None, fused_add: bool = False):
    """x [M,K] (bf16/fp16/fp32, cuda) -> (int8 [M,K], float32 [M,1]); rotate=True applies the 128-block Hadamard first.
    prologue applies an elementwise operation while the rows are read: PRO_GELU_TANH, or PRO_MODULATE with
    mod_scale / mod_shift of x's dtype, [V,K] (or [K]): (1 + mod_scale) * x + mod_shift, M // V consecutive rows
    to a vector, or PRO_SILU_GATE with the gate operand as mod_scale (x's dtype, [M,K], or [V,K] like the vectors
    above): silu(x) * mod_scale, or PRO_NORM_MODULATE: the modulation applied to layer_norm(x, eps) without affine
    parameters (see norm_modulate_fusable for the rows it takes), or PRO_CONCAT_GELU with a second tensor [M,Kb] as
    mod_scale: cat((x, gelu(mod_scale)), -1) (see quant_rowwise_concat_gelu), or PRO_GELU_ERF, GELU in its exact form, or
    PRO_RMS_NORM: rms_norm(x, norm_weight, eps), then the modulation's operations where mod_scale / mod_shift are given
    (see quant_rowwise_rms_norm).  fused_add (or PRO_MODULATE_FUSED): the modulation as torch.addcmul(mod_shift, x, 1 + mod_scale)
    computes it, product and sum rounded once (16-bit tensors), in the three kinds that modulate."""
    _dev(x, "x")
    if prologue == PRO_RMS_NORM:
        return quant_rowwise_rms_norm(x, eps, norm_weight, mod_scale, mod_shift, rotate=rotate, fused_add=fused_add)
    if prologue == PRO_CONCAT_GELU:   # x followed by gelu(mod_scale) along the row
        return quant_rowwise_concat_gelu(x, mod_scale, rotate=rotate)
    x = _rows(x, "x")
    M, K = x.shape
    if rotate and K % 128:
        raise ValueError(f"rotation needs K % 128 == 0, got K={K}")
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    s = torch.empty((M, 1), dtype=torch.float32, device=x.device)
    ldx = x.stride(0) if M > 1 else K
    rows_per_vec = 1
    if prologue == PRO_MODULATE and fused_add:
        prologue = PRO_MODULATE_FUSED
    if prologue == PRO_MODULATE_FUSED and x.dtype == torch.float32:
        raise ValueError("the fused form of the modulation exists for 16-bit tensors")
    if prologue in (PRO_MODULATE, PRO_MODULATE_FUSED, PRO_SILU_GATE, PRO_NORM_MODULATE):
        if prologue == PRO_NORM_MODULATE and not norm_modulate_fusable(x):
            raise ValueError("PRO_NORM_MODULATE takes contiguous 16-bit rows of at most 16384 elements in multiples of 16 "
                             "(see norm_modulate_fusable); normalise with torch and use PRO_MODULATE")
        vecs = []
        if prologue == PRO_SILU_GATE:
            mod_shift = mod_scale      # one operand: the gate
        for name, v in (("mod_scale", mod_scale), ("mod_shift", mod_shift)):
            _dev(v, name)
            if v.dtype != x.dtype or v.device != x.device or v.numel() % max(K, 1) or v.shape[-1] != K:
                raise ValueError(f"{name} must be [V,{K}] of {x.dtype} on {x.device}")
            vecs.append(v.reshape(-1, K).contiguous())
        mod_scale, mod_shift = vecs
        V = mod_scale.shape[0]
        if mod_shift.shape[0] != V or V == 0 or M % V:
            raise ValueError(f"{M} rows do not split evenly over {V} modulation vectors")
        rows_per_vec = max(1, M // V)
    elif prologue not in (PRO_NONE, PRO_GELU_TANH, PRO_GELU_ERF):
        raise ValueError(f"unknown prologue {prologue}")
    else:
        mod_scale = mod_shift = None
    with _on(x.device):
        if prologue == PRO_NONE:
            _check(lib().i8f_quant_rowwise(_ptr(x), dtype_code(x.dtype), M, K, ldx, 128 if rotate else 0, _ptr(q), _ptr(s),
                                           _stream(x)), "i8f_quant_rowwise")
        elif prologue == PRO_NORM_MODULATE:
            _check(lib().i8f_quant_rowwise_norm_modulate(_ptr(x), dtype_code(x.dtype), M, K, ldx, float(eps), _ptr(mod_scale),
                                                         _ptr(mod_shift), rows_per_vec, int(bool(fused_add)), 128 if rotate else 0, _ptr(q),
                                                         _ptr(s), _stream(x)), "i8f_quant_rowwise_norm_modulate")
        else:
            _check(lib().i8f_quant_rowwise_prologue(_ptr(x), dtype_code(x.dtype), M, K, ldx, prologue, _ptr(mod_scale),
                                                    _ptr(mod_shift), rows_per_vec, 128 if rotate else 0, _ptr(q), _ptr(s),
                                                    _stream(x)), "i8f_quant_rowwise_prologue")
    return q, s


class _QuantGroup(ctypes.Structure):
    _fields_ = [("x", ctypes.c_void_p), ("M", ctypes.c_int64), ("ldx", ctypes.c_int64), ("q", ctypes.c_void_p),
                ("scale", ctypes.c_void_p)]


def quant_rowwise_grouped(xs, rotate: bool = False):
    """quant_rowwise for several [M_i, K] tensors of one dtype, one width and one device in a single launch
    -> [(int8 [M_i,K], float32 [M_i,1]), ...], bit-identical to the separate calls."""
    xs = list(xs)
    if not xs:
        return []
    for i, x in enumerate(xs):
        _dev(x, f"xs[{i}]")
        xs[i] = _rows(x, f"xs[{i}]")
    K, dt, device = xs[0].shape[1], xs[0].dtype, xs[0].device
    if any(x.shape[1] != K or x.dtype != dt or x.device != device for x in xs):
        raise ValueError("the tensors of a group launch share their width, dtype and device")
    if rotate and K % 128:
        raise ValueError(f"rotation needs K % 128 == 0, got K={K}")
    outs = [(torch.empty((x.shape[0], K), dtype=torch.int8, device=device), torch.empty((x.shape[0], 1), dtype=torch.float32, device=device))
            for x in xs]
    groups = (_QuantGroup * len(xs))()
    for g, x, (q, s) in zip(groups, xs, outs):
        g.x, g.M, g.ldx, g.q, g.scale = x.data_ptr(), x.shape[0], (x.stride(0) if x.shape[0] > 1 else K), q.data_ptr(), s.data_ptr()
    with _on(device):
        _check(lib().i8f_quant_rowwise_grouped(ctypes.byref(groups), len(xs), dtype_code(dt), K, 128 if rotate else 0, _stream(xs[0])),
               "i8f_quant_rowwise_grouped")
    return outs


def quant_tensorwise(x: torch.Tensor, static_scratch: bool = False):
    """x (any shape; bf16/fp16/fp32, cuda) -> (int8 like x, 0-dim float32 scale): one absmax scale for the tensor.
    static_scratch=True uses the library's own device array for the partial maxima instead of a torch workspace
    (the call then allocates nothing beyond q and scale, which the caller may also preallocate via the C ABI)."""
    _dev(x, "x")
    if x.dtype not in _DT:
        raise TypeError(f"unsupported dtype {x.dtype}; expected bfloat16, float16 or float32")
    xc = x if x.is_contiguous() else x.contiguous()
    n = xc.numel()
    q = torch.empty(xc.shape, dtype=torch.int8, device=x.device)
    s = torch.empty((), dtype=torch.float32, device=x.device)
    with _on(x.device):
        if static_scratch:
            _check(lib().i8f_quant_tensorwise_static(_ptr(xc), dtype_code(x.dtype), n, _ptr(q), _ptr(s), _stream(x)),
                   "i8f_quant_tensorwise_static")
        else:
            nbytes = lib().i8f_quant_tensorwise_workspace_bytes(n)
            ws = torch.empty(max(1, nbytes // 4), dtype=torch.float32, device=x.device)
            _check(lib().i8f_quant_tensorwise(_ptr(xc), dtype_code(x.dtype), n, _ptr(q), _ptr(s), _ptr(ws), ws.numel() * 4,
                                              _stream(x)), "i8f_quant_tensorwise")
    return q, s


def rotate128(x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    _dev(x, "x")
    x = _rows(x, "x")
    M, K = x.shape
    if K % 128:
        raise ValueError(f"rotation needs K % 128 == 0, got K={K}")
    if out is None:
        out = torch.empty((M, K), dtype=x.dtype, device=x.device)
    elif out.shape != x.shape or out.dtype != x.dtype or not out.is_contiguous() or out.device != x.device:
        raise ValueError("out must be a contiguous tensor like x")
    ldx = x.stride(0) if M > 1 else K
    with _on(x.device):
        _check(lib().i8f_rotate128(_ptr(x), dtype_code(x.dtype), M, K, ldx, _ptr(out), _stream(x)), "i8f_rotate128")
    return out


def _i8_matrix(t: torch.Tensor, name: str) -> torch.Tensor:
    _dev(t, name)
    if t.dtype != torch.int8 or t.dim() != 2:
        raise TypeError(f"{name} must be a 2-D int8 tensor, got {t.dtype} {tuple(t.shape)}")
    return t if t.is_contiguous() else t.contiguous()


def gemm_tile(M: int, N: int, K: int):
    """(tile rows, tile columns, LDS stages) of the GEMM kernel variant an aligned M x N x K problem takes."""
    bm, bn, st = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    _check(lib().i8f_gemm_tile(M, N, K, ctypes.byref(bm), ctypes.byref(bn), ctypes.byref(st)), "i8f_gemm_tile")
    return bm.value, bn.value, st.value


def gemm_i32(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """a [M,K] int8, w [N,K] int8 -> int32 [M,N] = a @ w.T"""
    a, w = _i8_matrix(a, "a"), _i8_matrix(w, "w")
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise ValueError(f"K mismatch: a has {K}, w has {K2}")
    acc = torch.empty((M, N), dtype=torch.int32, device=a.device)
    with _on(a.device):
        _check(lib().i8f_gemm_i32(_ptr(a), _ptr(w), M, N, K, _ptr(acc), _stream(a)), "i8f_gemm_i32")
    return acc


def _bias_arg(bias, N, device):
    if bias is None:
        return None, BF16
    if bias.device != device:
        bias = bias.to(device, non_blocking=True)
    bias = bias.reshape(-1).contiguous()
    if bias.numel() != N:
        raise ValueError(f"bias has {bias.numel()} elements, expected {N}")
    return bias, dtype_code(bias.dtype)


_SPLITK_WORKSPACES = {}
_SPLITK_COUNTER_BYTES = 4096


def _splitk_workspace(t: torch.Tensor, M: int, N: int, K: int):
    """The K-split workspace for shapes that can use one (a long K and few output tiles), else None.

    The library's contract is one launch at a time per workspace (launches that overlap in time race on the partial
    sums).  Eager calls: one workspace per (device, stream), allocated and zeroed once and kept until
    clear_splitk_workspaces(); launches on one stream run one after the other, so they can share it.  While the
    stream is capturing a graph the eager workspace is never used (a replay of the graph on another stream could
    overlap eager calls on this one): the call gets a workspace of its own from the graph's memory pool, with a
    fill kernel in front of it that clears the arrival words on every replay, and the memory goes back to the pool
    of the graph when the call returns (later nodes of the same graph run after this one)."""
    if K < 10240 or M * N > 128 * 128 * 128:
        return None
    nbytes = lib().i8f_linear_w8a8_workspace_bytes()
    if torch.cuda.is_current_stream_capturing():
        ws = torch.empty(nbytes, dtype=torch.uint8, device=t.device)
        ws[:_SPLITK_COUNTER_BYTES].zero_()
        return ws
    key = (t.device.index, torch.cuda.current_stream(t.device).cuda_stream)
    ws = _SPLITK_WORKSPACES.get(key)
    if ws is None:
        ws = torch.zeros(nbytes, dtype=torch.uint8, device=t.device)
        _SPLITK_WORKSPACES[key] = ws
    return ws


def clear_splitk_workspaces() -> None:
    """Drop the cached K-split workspaces (16 MB per device and stream that used one); the next call allocates anew."""
    _SPLITK_WORKSPACES.clear()


def linear_w8a8(a, a_scale, w, w_scale, bias=None, out_dtype=torch.bfloat16, order=EPI_TORCH, out=None, addend=None, gate=None):
    """Quantised activations (a int8 [M,K], a_scale [M,1]) times int8 weight [N,K] with the fused dequant epilogue.
    addend ([M,N] of the output dtype) is added to the rounded result in the epilogue and the sum rounded again.
    gate ([V,N] or [N] of the output dtype, M // V consecutive rows to a vector) multiplies the rounded result first
    (rounded again): out = addend + gate * y, the gated residual of an adaLN-Zero block."""
    a, w = _i8_matrix(a, "a"), _i8_matrix(w, "w")
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise ValueError(f"K mismatch: a has {K}, w has {K2}")
    _dev(a_scale, "a_scale")
    a_scale = a_scale.reshape(-1)
    if a_scale.numel() != M or a_scale.dtype != torch.float32:
        raise ValueError("a_scale must be float32 with M elements")
    a_scale = a_scale.contiguous()
    ws, ws_host, mode = _scale(w_scale, N, a.device)
    bias, bcode = _bias_arg(bias, N, a.device)
    for name, t in (("w", w), ("a_scale", a_scale), ("addend", addend), ("out", out)):
        if isinstance(t, torch.Tensor) and t.device != a.device:
            raise ValueError(f"{name} is on {t.device}, a is on {a.device}")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    elif tuple(out.shape) != (M, N) or not out.is_contiguous() or out.dtype not in _DT:
        raise ValueError(f"out must be a contiguous [{M},{N}] tensor of bfloat16, float16 or float32")
    if addend is not None:
        _dev(addend, "addend")
        if addend.numel() != M * N or addend.dtype != out.dtype:
            raise ValueError(f"addend must have {M * N} elements of {out.dtype}")
        addend = addend.reshape(M, N).contiguous()
    rows_per_gate = 1
    if gate is not None:
        _dev(gate, "gate")
        if gate.dtype != out.dtype or gate.device != a.device or gate.numel() % max(N, 1) or gate.shape[-1] != N:
            raise ValueError(f"gate must be [V,{N}] of {out.dtype} on {a.device}")
        gate = gate.reshape(-1, N).contiguous()
        V = gate.shape[0]
        if V == 0 or M % V:
            raise ValueError(f"{M} rows do not split evenly over {V} gate vectors")
        rows_per_gate = max(1, M // V)
    with _on(a.device):
        work = _splitk_workspace(a, M, N, K)
        _check(lib().i8f_linear_w8a8_gated(_ptr(a), _ptr(a_scale), _ptr(w), _ptr(ws), ws_host, mode, _ptr(bias), bcode, _ptr(gate),
                                           rows_per_gate, _ptr(addend), _ptr(out), dtype_code(out.dtype), M, N, K, order, _ptr(work),
                                           0 if work is None else work.numel(), _stream(a)),
               "i8f_linear_w8a8_gated")
    return out


class _LinearGroup(ctypes.Structure):
    _fields_ = [("a", ctypes.c_void_p), ("a_scale", ctypes.c_void_p), ("w", ctypes.c_void_p), ("w_scale", ctypes.c_void_p),
                ("w_scale_host", ctypes.c_float), ("bias", ctypes.c_void_p), ("addend", ctypes.c_void_p), ("out", ctypes.c_void_p),
                ("M", ctypes.c_int64), ("gate", ctypes.c_void_p), ("rows_per_gate", ctypes.c_int64)]


MAX_LINEAR_GROUPS = 4


def _addr(t):
    return None if t is None else t.data_ptr()


def linear_w8a8_grouped(problems, out_dtype=torch.bfloat16, order=EPI_TORCH, outs=None):
    """linear_w8a8 for several problems of one layer shape, each (a, a_scale, w, w_scale, bias[, addend[, gate]])
    with its own tensors (addend and gate as for linear_w8a8): the image and the text tokens of a double-stream
    transformer block through the same projection.  One launch where the library finds that the small problems' tiles
    fit into the compute units the largest one's last round leaves idle, else one launch per problem; problems that do
    not share N, K, the scale mode and the bias dtype (or more than MAX_LINEAR_GROUPS of them) are launched one by one
    from here.  outs: optional list of contiguous [M_i, N] tensors of out_dtype to write into.
    -> list of outputs, bit-identical to separate linear_w8a8 calls."""
    problems = [tuple(p) + (None,) * (7 - len(p)) for p in problems]
    if not problems:
        return []
    if outs is not None and len(outs) != len(problems):
        raise ValueError("outs must hold one tensor per problem")
    prepared = []
    for a, a_scale, w, w_scale, bias, addend, gate in problems:
        a, w = _i8_matrix(a, "a"), _i8_matrix(w, "w")
        M, K = a.shape
        N, K2 = w.shape
        if K != K2:
            raise ValueError(f"K mismatch: a has {K}, w has {K2}")
        _dev(a_scale, "a_scale")
        a_scale = a_scale.reshape(-1).contiguous()
        if a_scale.numel() != M or a_scale.dtype != torch.float32:
            raise ValueError("a_scale must be float32 with M elements")
        ws, ws_host, mode = _scale(w_scale, N, a.device)
        bias, bcode = _bias_arg(bias, N, a.device)
        if addend is not None:
            _dev(addend, "addend")
            if addend.numel() != M * N or addend.dtype != out_dtype:
                raise ValueError(f"addend must have {M * N} elements of {out_dtype}")
            addend = addend.reshape(M, N).contiguous()
        rows_per_gate = 1
        if gate is not None:
            _dev(gate, "gate")
            if gate.dtype != out_dtype or gate.numel() % max(N, 1) or gate.shape[-1] != N:
                raise ValueError(f"gate must be [V,{N}] of {out_dtype}")
            gate = gate.reshape(-1, N).contiguous()
            if gate.shape[0] == 0 or M % gate.shape[0]:
                raise ValueError(f"{M} rows do not split evenly over {gate.shape[0]} gate vectors")
            rows_per_gate = max(1, M // gate.shape[0])
        for name, t in (("w", w), ("a_scale", a_scale), ("addend", addend), ("gate", gate)):
            if isinstance(t, torch.Tensor) and t.device != a.device:
                raise ValueError(f"{name} is on {t.device}, a is on {a.device}")
        prepared.append((a, a_scale, w, ws, ws_host, mode, bias, bcode, addend, M, N, K, gate, rows_per_gate))
    first = prepared[0]
    bcodes = {p[7] for p in prepared if p[6] is not None}
    same = (len(prepared) <= MAX_LINEAR_GROUPS and len(bcodes) <= 1
            and all(p[10] == first[10] and p[11] == first[11] and p[5] == first[5] and p[0].device == first[0].device for p in prepared))
    if not same:
        return [linear_w8a8(p[0], p[1], p[2], src[3], p[6], out_dtype, order, None if outs is None else outs[i], addend=p[8], gate=p[12])
                for i, (p, src) in enumerate(zip(prepared, problems))]
    N, K, mode, device = first[10], first[11], first[5], first[0].device
    if outs is None:
        outs = [torch.empty((p[9], N), dtype=out_dtype, device=device) for p in prepared]
    else:
        for p, o in zip(prepared, outs):
            if tuple(o.shape) != (p[9], N) or not o.is_contiguous() or o.dtype != out_dtype or o.device != device:
                raise ValueError(f"outs: expected a contiguous [{p[9]},{N}] tensor of {out_dtype} on {device}")
    groups = (_LinearGroup * len(prepared))()
    for g, p, o in zip(groups, prepared, outs):
        g.a, g.a_scale, g.w, g.w_scale, g.w_scale_host = _addr(p[0]), _addr(p[1]), _addr(p[2]), _addr(p[3]), p[4]
        g.bias, g.addend, g.out, g.M = _addr(p[6]), _addr(p[8]), _addr(o), p[9]
        g.gate, g.rows_per_gate = _addr(p[12]), p[13]
    with _on(device):
        work = None
        for p in prepared:   # (used only if the library launches the problems one by one and one of them has a long K)
            work = work if work is not None else _splitk_workspace(p[0], p[9], N, K)
        _check(lib().i8f_linear_w8a8_grouped(ctypes.byref(groups), len(prepared), mode, bcodes.pop() if bcodes else 0,
                                             dtype_code(out_dtype), N, K, order, _ptr(work), 0 if work is None else work.numel(),
                                             _stream(first[0])), "i8f_linear_w8a8_grouped")
    return outs


def lora_side_fusable(M: int, N: int, K: int, rank: int, out_dtype, side_dtype) -> bool:
    """Whether linear_w8a8_lora takes this problem (else: a side tensor and linear_w8a8(addend=...))."""
    return (out_dtype in (torch.bfloat16, torch.float16) and side_dtype == out_dtype and 0 < rank <= 64
            and K % 128 == 0 and N % 8 == 0 and M > 0)


def linear_w8a8_lora(a, a_scale, w, w_scale, bias, side_t, side_b, alpha=None, out_dtype=torch.bfloat16, order=EPI_TORCH, out=None):
    """linear_w8a8 plus the low-rank side branch side_t [M,r] @ side_b [N,r].T (both of out_dtype), formed inside the
    GEMM epilogue: round(y + round(round(side) * alpha)).  A rank that is not a multiple of 16 is padded with zero
    columns (they add exact zeros)."""
    a, w = _i8_matrix(a, "a"), _i8_matrix(w, "w")
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise ValueError(f"K mismatch: a has {K}, w has {K2}")
    for name, t, rows in (("side_t", side_t, M), ("side_b", side_b, N)):
        _dev(t, name)
        if t.dim() != 2 or t.shape[0] != rows or t.dtype != out_dtype or t.device != a.device:
            raise ValueError(f"{name} must be [{rows}, rank] of {out_dtype} on {a.device}")
    r = side_t.shape[1]
    if side_b.shape[1] != r:
        raise ValueError("side_t and side_b disagree on the rank")
    if not lora_side_fusable(M, N, K, r, out_dtype, side_t.dtype):
        raise ValueError("this problem has no fused side branch (see lora_side_fusable)")
    if r % 16:
        pad = 16 - r % 16
        side_t = torch.nn.functional.pad(side_t, (0, pad))
        side_b = torch.nn.functional.pad(side_b, (0, pad))
        r += pad
    side_t, side_b = side_t.contiguous(), side_b.contiguous()
    a_scale = a_scale.reshape(-1).contiguous()
    if a_scale.numel() != M or a_scale.dtype != torch.float32:
        raise ValueError("a_scale must be float32 with M elements")
    ws, ws_host, mode = _scale(w_scale, N, a.device)
    bias, bcode = _bias_arg(bias, N, a.device)
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    elif tuple(out.shape) != (M, N) or not out.is_contiguous() or out.dtype != out_dtype or out.device != a.device:
        raise ValueError(f"out must be a contiguous [{M},{N}] tensor of {out_dtype} on {a.device}")
    with _on(a.device):
        _check(lib().i8f_linear_w8a8_lora(_ptr(a), _ptr(a_scale), _ptr(w), _ptr(ws), ws_host, mode, _ptr(bias), bcode,
                                          _ptr(side_t), _ptr(side_b), r, 0 if alpha is None else 1,
                                          0.0 if alpha is None else float(alpha), _ptr(out), dtype_code(out_dtype), M, N, K, order,
                                          _stream(a)), "i8f_linear_w8a8_lora")
    return out


def linear_w8a16_small_m(x, w, w_scale, bias=None):
    """x [M<=16,K] float, w int8 [N,K] -> [M,N] in x's dtype (weight dequantised on the fly)."""
    _dev(x, "x")
    x = _rows(x, "x")
    w = _i8_matrix(w, "w")
    M, K = x.shape
    N, K2 = w.shape
    if K != K2:
        raise ValueError(f"K mismatch: x has {K}, w has {K2}")
    ws, ws_host, mode = _scale(w_scale, N, x.device)
    bias, bcode = _bias_arg(bias, N, x.device)
    out = torch.empty((M, N), dtype=x.dtype, device=x.device)
    ldx = x.stride(0) if M > 1 else K
    with _on(x.device):
        _check(lib().i8f_linear_w8a16_small_m(_ptr(x), dtype_code(x.dtype), M, K, ldx, _ptr(w), _ptr(ws), ws_host, mode,
                                              _ptr(bias), bcode, _ptr(out), N, _stream(x)), "i8f_linear_w8a16_small_m")
    return out


class _SmallMGroup(ctypes.Structure):
    _fields_ = [("a", ctypes.c_void_p), ("M", ctypes.c_int64), ("K", ctypes.c_int64), ("ldx", ctypes.c_int64), ("w", ctypes.c_void_p),
                ("w_scale", ctypes.c_void_p), ("w_scale_host", ctypes.c_float), ("bias", ctypes.c_void_p), ("out", ctypes.c_void_p),
                ("N", ctypes.c_int64)]


def linear_w8a16_small_m_grouped(problems):
    """[linear_w8a16_small_m(x, w, w_scale, bias) for (x, w, w_scale, bias) in problems] with all layers in one launch
    where the library has a grouped kernel for them (up to 4 layers, 16-bit activations of one dtype, one scale mode and
    one bias dtype); anything else goes layer by layer.  Results are those of the separate calls bit for bit."""
    problems = [tuple(p) + (None,) * (4 - len(p)) for p in problems]
    if not problems:
        return []
    x0 = problems[0][0]
    _dev(x0, "x")
    prepared, keep = [], []
    for x, w, w_scale, bias in problems:
        _dev(x, "x")
        x = _rows(x, "x")
        w = _i8_matrix(w, "w")
        if x.shape[1] != w.shape[1]:
            raise ValueError(f"K mismatch: x has {x.shape[1]}, w has {w.shape[1]}")
        ws, ws_host, mode = _scale(w_scale, w.shape[0], x.device)
        b, bcode = _bias_arg(bias, w.shape[0], x.device)
        prepared.append((x, w, ws, ws_host, mode, b, bcode))
    modes = {p[4] for p in prepared}
    bcodes = {p[6] for p in prepared if p[5] is not None}
    same = (len(problems) <= MAX_LINEAR_GROUPS and len(modes) == 1 and len(bcodes) <= 1
            and all(p[0].dtype == x0.dtype and p[0].device == x0.device for p in prepared))
    if not same:
        return [linear_w8a16_small_m(x, w, w_scale, bias) for x, w, w_scale, bias in problems]
    groups = (_SmallMGroup * len(prepared))()
    outs = []
    for g, (x, w, ws, ws_host, mode, b, bcode) in zip(groups, prepared):
        M, K = x.shape
        out = torch.empty((M, w.shape[0]), dtype=x.dtype, device=x.device)
        g.a, g.M, g.K, g.ldx, g.w = _addr(x), M, K, (x.stride(0) if M > 1 else K), _addr(w)
        g.w_scale, g.w_scale_host, g.bias, g.out, g.N = _addr(ws), ws_host, _addr(b), _addr(out), w.shape[0]
        outs.append(out)
        keep.append((x, w, ws, b))
    with _on(x0.device):
        _check(lib().i8f_linear_w8a16_small_m_grouped(groups, len(prepared), dtype_code(x0.dtype), modes.pop(),
                                                      bcodes.pop() if bcodes else BF16, _stream(x0)), "i8f_linear_w8a16_small_m_grouped")
    return outs


def _f32_matrix(t, name, device):
    if t.device != device:
        t = t.to(device)
    if t.dtype != torch.float32:
        t = t.float()
    if t.dim() != 2:
        raise ValueError(f"{name} must be 2-D")
    return t.contiguous()


def sr_quant_delta(x, scale, noise):
    """Stochastic rounding of x / scale to int8 with the supplied uniform noise (both [N,K] float32)."""
    _dev(x, "x")
    x = _f32_matrix(x, "x", x.device)
    noise = _f32_matrix(noise, "noise", x.device)
    if noise.shape != x.shape:
        raise ValueError("noise must have the shape of x")
    N, K = x.shape
    ws, ws_host, mode = _scale(scale, N, x.device)
    dq = torch.empty((N, K), dtype=torch.int8, device=x.device)
    with _on(x.device):
        _check(lib().i8f_sr_quant_delta(_ptr(x), _ptr(ws), ws_host, mode, _ptr(noise), N, K, _ptr(dq), _stream(x)),
               "i8f_sr_quant_delta")
    return dq


def lora_merge_sr(w, w_scale, noise, delta=None, up=None, down=None, lora_scale=1.0, out=None):
    """w' = sat8(w + SR(delta / w_scale)); delta given, or rebuilt from up [N,r] / down [r,K] (times lora_scale)."""
    w = _i8_matrix(w, "w")
    N, K = w.shape
    noise = _f32_matrix(noise, "noise", w.device)
    if noise.shape != w.shape:
        raise ValueError("noise must have the shape of w")
    rank = 0
    if delta is not None:
        delta = _f32_matrix(delta, "delta", w.device)
        if delta.shape != w.shape:
            raise ValueError("delta must have the shape of w")
    else:
        if up is None or down is None:
            raise ValueError("give either delta or both up and down")
        up = _f32_matrix(up, "up", w.device)
        down = _f32_matrix(down, "down", w.device)
        rank = up.shape[1]
        if up.shape[0] != N or down.shape != (rank, K):
            raise ValueError(f"up must be [{N},r] and down [r,{K}]")
    ws, ws_host, mode = _scale(w_scale, N, w.device)
    if out is None:
        out = torch.empty_like(w)
    elif out.shape != w.shape or out.dtype != torch.int8 or not out.is_contiguous():
        raise ValueError("out must be a contiguous int8 tensor like w")
    with _on(w.device):
        _check(lib().i8f_lora_merge_sr(_ptr(w), _ptr(ws), ws_host, mode, _ptr(delta), _ptr(up), _ptr(down), rank,
                                       float(lora_scale), _ptr(noise), N, K, _ptr(out), _stream(w)), "i8f_lora_merge_sr")
    return out


def version() -> int:
    return int(lib().i8f_version())
