"""ctypes front end of the CPU oracle (``i8f_oracle.c``).

TEST INFRASTRUCTURE ONLY.  The oracle restates the reference's arithmetic on the
CPU so that the HIP library can be checked against it.  It may be imported by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py`` and by nothing else; the shipped package never imports it and has
no CPU fallback.

Arrays are numpy.  bfloat16 and float16 data travel as ``uint16`` bit patterns
together with a dtype code (``BF16``, ``F16``, ``F32``); ``from_torch`` /
``to_torch`` convert CPU torch tensors without touching the values.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

BF16, F16, F32 = 0, 1, 2
SCALE_TENSOR, SCALE_ROW = 0, 1
EPI_TORCH, EPI_FUSED = 0, 1

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libi8f_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile beside this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
        L.orc_quant_rowwise.argtypes = [vp, i32, i64, i64, i64, i32, vp, vp]
        L.orc_quant_tensorwise.argtypes = [vp, i32, i64, vp, vp]
        L.orc_prologue.argtypes = [vp, i32, i64, i64, i64, i32, vp, vp, i64, vp]
        L.orc_norm_modulate.argtypes = [vp, i32, i64, i64, i64, f32, vp, vp, i64, i32, vp]
        L.orc_rms_norm.argtypes = [vp, i32, i64, i64, i64, f32, vp, vp, vp, i64, i32, vp]
        L.orc_gemm_i32.argtypes = [vp, vp, i64, i64, i64, vp]
        L.orc_epilogue.argtypes = [vp, vp, vp, i32, vp, i32, vp, i32, i64, i64, i32]
        L.orc_linear_w8a8.argtypes = [vp, i32, i64, i64, i64, i32, vp, vp, i32, vp, i32, vp, i32, i64, i32]
        L.orc_gate_residual.argtypes = [vp, i32, i64, i64, vp, i64, vp, vp]
        L.orc_linear_w8a16.argtypes = [vp, i32, i64, i64, i64, vp, vp, i32, vp, i32, vp, i64]
        L.orc_sr_delta.argtypes = [vp, vp, i32, vp, i64, i64, vp]
        L.orc_merge_i8.argtypes = [vp, vp, i64, vp]
        L.orc_scale_by_127_mismatches.argtypes = [vp, i64, vp]
        L.orc_scale_by_127_mismatches.restype = i64
        L.orc_quotient_by_reciprocal_mismatches.argtypes = [vp, vp, i64, vp]
        L.orc_quotient_by_reciprocal_mismatches.restype = i64
        L.orc_lora_delta.argtypes = [vp, vp, i64, i64, i64, f32, vp]
        L.orc_lora_merge_sr.argtypes = [vp, vp, i32, vp, vp, vp, i64, f32, vp, i64, i64, vp]
        L.orc_fwht_f32.argtypes = [vp, i32]
        L.orc_rotate_row.argtypes = [vp, i64, i32, i32]
        L.orc_hadamard_entry.argtypes = [i32]
        L.orc_hadamard_entry.restype = f32
        L.orc_f32_to_bf16.argtypes = [f32]
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_f32_to_f16.argtypes = [f32]
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_bf16_to_f32.restype = f32
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f16_to_f32.restype = f32
        L.orc_set_num_threads.argtypes = [i32]
        L.orc_num_threads.restype = i32
        _lib = L
    return _lib


# --------------------------------------------------------------------------- helpers
_NP_OF = {BF16: np.uint16, F16: np.uint16, F32: np.float32}


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _chk(rc, what):
    if rc != 0:
        raise RuntimeError(f"oracle {what} failed with status {rc}")


def _arr(a, dtype_code):
    a = np.ascontiguousarray(a)
    want = _NP_OF[dtype_code]
    if a.dtype != want:
        if dtype_code == F16 and a.dtype == np.float16:
            a = a.view(np.uint16)
        else:
            raise TypeError(f"expected {want} for dtype code {dtype_code}, got {a.dtype}")
    return a


def from_torch(t):
    """CPU torch tensor -> (numpy array, dtype code); bf16/fp16 become uint16 bits."""
    import torch

    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16), BF16
    if t.dtype == torch.float16:
        return t.view(torch.int16).numpy().view(np.uint16), F16
    if t.dtype == torch.float32:
        return t.numpy(), F32
    raise TypeError(f"unsupported dtype {t.dtype}")


def to_torch(a, dtype_code):
    import torch

    a = np.ascontiguousarray(a)
    if dtype_code == BF16:
        return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    if dtype_code == F16:
        return torch.from_numpy(a.view(np.int16).copy()).view(torch.float16)
    return torch.from_numpy(a.copy())


def to_f32(a, dtype_code):
    """Widen a stored array to float32 values (exact)."""
    if dtype_code == BF16:
        return (a.astype(np.uint32) << 16).view(np.float32)
    if dtype_code == F16:
        return a.view(np.float16).astype(np.float32)
    return np.asarray(a, dtype=np.float32)


def round_to(v, dtype_code):
    """float32 values -> storage array of dtype_code, round-to-nearest-even (numpy bit arithmetic, not the C routine)."""
    v = np.ascontiguousarray(v, dtype=np.float32)
    if dtype_code == F32:
        return v.copy()
    if dtype_code == F16:
        return v.astype(np.float16).view(np.uint16)
    u = v.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[np.isnan(v)] = 0x7FC0
    return r


# --------------------------------------------------------------------------- the restated functions
def quant_rowwise(x, dtype_code, rotate_block=0):
    """int8_quant.py:28-31 (+ quarot.py:73-102 when rotate_block): x [M,K] -> (q int8 [M,K], scale f32 [M,1])."""
    x = _arr(x, dtype_code)
    M, K = x.shape
    q = np.empty((M, K), dtype=np.int8)
    s = np.empty((M, 1), dtype=np.float32)
    _chk(lib().orc_quant_rowwise(_p(x), dtype_code, M, K, K, rotate_block, _p(q), _p(s)), "quant_rowwise")
    return q, s


def quant_tensorwise(x, dtype_code):
    """int8_quant.py:23-26: one scale for the whole tensor."""
    x = _arr(x, dtype_code)
    q = np.empty(x.shape, dtype=np.int8)
    s = np.empty((1,), dtype=np.float32)
    _chk(lib().orc_quant_tensorwise(_p(x), dtype_code, x.size, _p(q), _p(s)), "quant_tensorwise")
    return q, s


PRO_MODULATE, PRO_GELU_TANH, PRO_SILU_GATE, PRO_NORM_MODULATE, PRO_GELU_ERF, PRO_MODULATE_FUSED = 1, 2, 3, 4, 6, 8


def prologue(x, dtype_code, kind, s=None, t=None, rows_per_vec=1):
    """The elementwise operation in front of a quantised linear (adaLN modulation or tanh-GELU), evaluated as
    torch's eager kernels do; returns the storage array of dtype_code, shape of x."""
    x = _arr(x, dtype_code)
    M, K = x.shape
    if kind in (PRO_MODULATE, PRO_MODULATE_FUSED):
        s, t = _arr(s, dtype_code).reshape(-1, K), _arr(t, dtype_code).reshape(-1, K)
        assert s.shape == t.shape and s.shape[0] * rows_per_vec >= M
    elif kind == PRO_SILU_GATE:
        s, t = _arr(s, dtype_code).reshape(-1, K), None
        assert s.shape[0] * rows_per_vec >= M
    out = np.empty((M, K), dtype=x.dtype)
    _chk(lib().orc_prologue(_p(x), dtype_code, M, K, K, kind, _p(s) if s is not None else None,
                            _p(t) if t is not None else None, rows_per_vec, _p(out)), "prologue")
    return out


def norm_modulate(x, dtype_code, eps, s, t, rows_per_vec=1, fused=False):
    """(1 + s) * layer_norm(x, eps) + t without affine parameters, every tensor operation rounded to the dtype as
    torch's eager kernels do (fused: the product and the sum as torch.addcmul, one rounding); returns the storage array
    of dtype_code, shape of x."""
    x = _arr(x, dtype_code)
    M, K = x.shape
    s, t = _arr(s, dtype_code).reshape(-1, K), _arr(t, dtype_code).reshape(-1, K)
    assert s.shape == t.shape and s.shape[0] * rows_per_vec >= M
    out = np.empty((M, K), dtype=x.dtype)
    _chk(lib().orc_norm_modulate(_p(x), dtype_code, M, K, K, float(eps), _p(s), _p(t), rows_per_vec, int(bool(fused)), _p(out)), "norm_modulate")
    return out


def rms_norm(x, dtype_code, eps, w=None, s=None, t=None, rows_per_vec=1, fused=False):
    """rms_norm(x, w, eps) rounded once to the dtype as torch's kernel does, then (1 + s) * y and + t where given, each
    rounded; returns the storage array of dtype_code, shape of x."""
    x = _arr(x, dtype_code)
    M, K = x.shape
    w = None if w is None else _arr(w, dtype_code).reshape(K)
    s = None if s is None else _arr(s, dtype_code).reshape(-1, K)
    t = None if t is None else _arr(t, dtype_code).reshape(-1, K)
    for v in (s, t):
        assert v is None or v.shape[0] * rows_per_vec >= M
    out = np.empty((M, K), dtype=x.dtype)
    _chk(lib().orc_rms_norm(_p(x), dtype_code, M, K, K, float(eps), *(None if v is None else _p(v) for v in (w, s, t)),
                            rows_per_vec, int(bool(fused)), _p(out)), "rms_norm")
    return out


def rotate(x, dtype_code, block=128):
    """quarot.py:73-102 / 42-70 restated with the fixed butterfly order; returns the storage array of dtype_code."""
    x = _arr(x, dtype_code)
    M, K = x.shape
    if K % block:
        raise ValueError("K must be a multiple of the block")
    v = np.array(to_f32(x, dtype_code), dtype=np.float32, order="C", copy=True)
    for m in range(M):
        row = v[m]
        lib().orc_rotate_row(_p(row), K, dtype_code, block)
    if dtype_code == BF16:
        return (v.view(np.uint32) >> 16).astype(np.uint16)
    if dtype_code == F16:
        return v.astype(np.float16).view(np.uint16)  # values are already on the f16 grid: exact
    return v


def fwht(v):
    """Unnormalised fixed-order transform of one float32 block (copy)."""
    v = np.ascontiguousarray(v, dtype=np.float32).copy()
    lib().orc_fwht_f32(_p(v), v.size)
    return v


def gemm_i32(a, w):
    """int8_quant.py:80,110: a [M,K] int8, w [N,K] int8 -> int32 [M,N]."""
    a = np.ascontiguousarray(a, dtype=np.int8)
    w = np.ascontiguousarray(w, dtype=np.int8)
    M, K = a.shape
    N, K2 = w.shape
    if K != K2:
        raise ValueError("K mismatch")
    acc = np.empty((M, N), dtype=np.int32)
    _chk(lib().orc_gemm_i32(_p(a), _p(w), M, N, K, _p(acc)), "gemm_i32")
    return acc


def _scale_arg(ws, N):
    ws = np.ascontiguousarray(np.asarray(ws, dtype=np.float32).reshape(-1))
    if ws.size == 1:
        return ws, SCALE_TENSOR
    if ws.size != N:
        raise ValueError("weight scale must have 1 or N elements")
    return ws, SCALE_ROW


def epilogue(acc, xs, ws, bias=None, bias_dtype=BF16, out_dtype=BF16, order=EPI_TORCH):
    """int8_quant.py:84-87 / 115-118 (EPI_TORCH) or int8_fused_kernel.py:156-173 / 310-324 (EPI_FUSED)."""
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    M, N = acc.shape
    xs = np.ascontiguousarray(np.asarray(xs, dtype=np.float32).reshape(-1))
    ws, mode = _scale_arg(ws, N)
    if bias is not None:
        bias = _arr(bias, bias_dtype).reshape(-1)
    out = np.empty((M, N), dtype=_NP_OF[out_dtype])
    _chk(lib().orc_epilogue(_p(acc), _p(xs), _p(ws), mode, _p(bias), bias_dtype, _p(out), out_dtype, M, N, order), "epilogue")
    return out


def linear_w8a8(x, x_dtype, w, ws, bias=None, bias_dtype=BF16, out_dtype=BF16, rotate_block=0, order=EPI_TORCH):
    """int8_quant.py:75-88 / 106-119 (after the rotation of :741-744): returns the storage array of out_dtype."""
    x = _arr(x, x_dtype)
    w = np.ascontiguousarray(w, dtype=np.int8)
    M, K = x.shape
    N = w.shape[0]
    ws, mode = _scale_arg(ws, N)
    if bias is not None:
        bias = _arr(bias, bias_dtype).reshape(-1)
    out = np.empty((M, N), dtype=_NP_OF[out_dtype])
    _chk(lib().orc_linear_w8a8(_p(x), x_dtype, M, K, K, rotate_block, _p(w), _p(ws), mode, _p(bias), bias_dtype,
                               _p(out), out_dtype, N, order), "linear_w8a8")
    return out


def gate_residual(y, dtype_code, gate=None, residual=None, rows_per_gate=1):
    """residual + gate * y as two tensor operations of one dtype (arrays as from_torch gives them; gate [V,N] with
    rows_per_gate consecutive rows of y to a vector); returns the storage array of dtype_code."""
    y = _arr(y, dtype_code)
    M, N = y.shape
    if gate is not None:
        gate = _arr(gate, dtype_code).reshape(-1, N)
        assert gate.shape[0] * rows_per_gate >= M
    if residual is not None:
        residual = _arr(residual, dtype_code).reshape(M, N)
    out = np.empty((M, N), dtype=y.dtype)
    _chk(lib().orc_gate_residual(_p(y), dtype_code, M, N, _p(gate) if gate is not None else None, rows_per_gate,
                                 _p(residual) if residual is not None else None, _p(out)), "gate_residual")
    return out


def linear_w8a16(x, x_dtype, w, ws, bias=None, bias_dtype=BF16):
    """int8_quant.py:756-760 (rows <= 16): tolerance reference, float64 accumulation."""
    x = _arr(x, x_dtype)
    w = np.ascontiguousarray(w, dtype=np.int8)
    M, K = x.shape
    N = w.shape[0]
    ws, mode = _scale_arg(ws, N)
    if bias is not None:
        bias = _arr(bias, bias_dtype).reshape(-1)
    out = np.empty((M, N), dtype=_NP_OF[x_dtype])
    _chk(lib().orc_linear_w8a16(_p(x), x_dtype, M, K, K, _p(w), _p(ws), mode, _p(bias), bias_dtype, _p(out), N), "linear_w8a16")
    return out


def sr_delta(x, scale, noise):
    """int8_quant.py:36-62 with supplied noise: x, noise [N,K] f32 -> int8 [N,K]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    noise = np.ascontiguousarray(noise, dtype=np.float32)
    N, K = x.shape
    scale, mode = _scale_arg(scale, N)
    dq = np.empty((N, K), dtype=np.int8)
    _chk(lib().orc_sr_delta(_p(x), _p(scale), mode, _p(noise), N, K, _p(dq)), "sr_delta")
    return dq


def scale_by_127_mismatches(a):
    """(count, first index or -1) of values whose fma-corrected product with 1/127 differs from max(a / 127, 1e-30)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    first = ctypes.c_int64(-1)
    n = lib().orc_scale_by_127_mismatches(_p(a), a.size, ctypes.byref(first))
    return int(n), int(first.value)


def quotient_by_reciprocal_mismatches(a, b):
    """How many pairs the reciprocal-and-two-corrections quotient gets differently from a / b, and the first index."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    first = ctypes.c_int64(-1)
    n = lib().orc_quotient_by_reciprocal_mismatches(_p(a), _p(b), a.size, ctypes.byref(first))
    return int(n), int(first.value)


def merge_i8(w, dq):
    """int8_quant.py:313-316: saturating int8 add."""
    w = np.ascontiguousarray(w, dtype=np.int8)
    dq = np.ascontiguousarray(dq, dtype=np.int8)
    out = np.empty(w.shape, dtype=np.int8)
    _chk(lib().orc_merge_i8(_p(w), _p(dq), w.size, _p(out)), "merge_i8")
    return out


def lora_delta(up, down, scale):
    """int8_quant.py:143-157,:295 with the fixed fma order: (up @ down) * scale."""
    up = np.ascontiguousarray(up, dtype=np.float32)
    down = np.ascontiguousarray(down, dtype=np.float32)
    N, r = up.shape
    r2, K = down.shape
    if r != r2:
        raise ValueError("rank mismatch")
    d = np.empty((N, K), dtype=np.float32)
    _chk(lib().orc_lora_delta(_p(up), _p(down), N, K, r, float(scale), _p(d)), "lora_delta")
    return d


def lora_merge_sr(w, w_scale, noise, delta=None, up=None, down=None, lora_scale=1.0):
    """int8_quant.py:293-318 from delta_f onward (delta given) or with the fixed-order product (up/down given)."""
    w = np.ascontiguousarray(w, dtype=np.int8)
    N, K = w.shape
    noise = np.ascontiguousarray(noise, dtype=np.float32)
    w_scale, mode = _scale_arg(w_scale, N)
    r = 0
    if delta is not None:
        delta = np.ascontiguousarray(delta, dtype=np.float32)
    else:
        up = np.ascontiguousarray(up, dtype=np.float32)
        down = np.ascontiguousarray(down, dtype=np.float32)
        r = up.shape[1]
    out = np.empty((N, K), dtype=np.int8)
    _chk(lib().orc_lora_merge_sr(_p(w), _p(w_scale), mode, _p(delta), _p(up), _p(down), r, float(lora_scale),
                                 _p(noise), N, K, _p(out)), "lora_merge_sr")
    return out


def set_num_threads(n: int) -> None:
    lib().orc_set_num_threads(int(n))


def num_threads() -> int:
    return int(lib().orc_num_threads())
