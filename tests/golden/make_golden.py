"""Writes tests/golden/vectors.npz: small input/output vectors for every hot-path function.

The reference ships no test vectors, and it is not imported here.  Expected outputs are
produced by the torch CPU routines the reference's slow path is made of
(oracle/torch_path.py) and, for the rotation, by a numpy float32 butterfly written out
below; none of them goes through the C oracle or the HIP library, which are the
things the vectors are used to check.  bfloat16 data is stored as uint16 bit patterns.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import torch_path as T  # noqa: E402


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def butterfly_rotate_bf16(x):
    """128-block rotation of a bf16 tensor: float32 butterfly, strides 1..64, (lo+hi, lo-hi), times 181/2048, round to bf16."""
    v = x.float().numpy().reshape(-1, 128).copy()
    stride = 1
    while stride < 128:
        w = v.reshape(v.shape[0], -1, 2, stride)
        lo, hi = w[:, :, 0, :].copy(), w[:, :, 1, :].copy()
        w[:, :, 0, :], w[:, :, 1, :] = lo + hi, lo - hi
        v = w.reshape(v.shape[0], 128)
        stride *= 2
    v = (v * np.float32(0.08837890625)).astype(np.float32)
    return torch.from_numpy(v.reshape(x.shape)).bfloat16()


def main():
    g = torch.Generator().manual_seed(20251125)
    out = {}

    x = torch.randn(8, 256, generator=g)
    x[:, [3, 77, 130]] *= 20
    x[5] = 0
    x = x.bfloat16()
    q, s = T.quant_rowwise(x)
    out.update(quant_x=bits(x), quant_q=q.numpy(), quant_s=s.numpy())

    xr = butterfly_rotate_bf16(x)
    qr, sr = T.quant_rowwise(xr)
    out.update(rot_x=bits(x), rot_xr=bits(xr), rot_q=qr.numpy(), rot_s=sr.numpy())

    a = torch.randint(-128, 128, (24, 256), dtype=torch.int8, generator=g)
    w = torch.randint(-128, 128, (16, 256), dtype=torch.int8, generator=g)
    out.update(gemm_a=a.numpy(), gemm_w=w.numpy(), gemm_acc=torch._int_mm(a, w.T).numpy())

    xl = torch.randn(24, 256, generator=g)
    xl[:, 9] *= 20
    xl = xl.bfloat16()
    wf = torch.randn(16, 256, generator=g) * 0.02
    bias = (torch.randn(16, generator=g) * 0.01).bfloat16()
    wq_r, ws_r = T.quant_rowwise(wf)
    wq_t, ws_t = T.quant_tensorwise(wf)
    out.update(lin_x=bits(xl), lin_bias=bits(bias),
               lin_wq_row=wq_r.numpy(), lin_ws_row=ws_r.numpy(),
               lin_wq_tensor=wq_t.numpy(), lin_ws_tensor=ws_t.numpy().reshape(1),
               lin_y_row_bias=bits(T.linear_w8a8(xl, wq_r, ws_r, bias, torch.bfloat16)),
               lin_y_row_nobias=bits(T.linear_w8a8(xl, wq_r, ws_r, None, torch.bfloat16)),
               lin_y_tensor_bias=bits(T.linear_w8a8(xl, wq_t, ws_t.item(), bias, torch.bfloat16)),
               lin_y_tensor_nobias_f16=bits(T.linear_w8a8(xl.half(), wq_t, ws_t.item(), None, torch.float16)),
               lin_x_f16=bits(xl.half()))

    wm = torch.randint(-128, 128, (4, 128), dtype=torch.int8, generator=g)
    wsm = torch.rand(4, 1, generator=g) * 1e-3 + 2e-4
    delta = torch.randn(4, 128, generator=g) * 2e-3
    delta[0, :2] = torch.tensor([1.0, -1.0])
    noise = torch.rand(4, 128, generator=g)
    dq = T.sr_delta(delta, wsm, noise)
    out.update(sr_w=wm.numpy(), sr_ws=wsm.numpy(), sr_delta=delta.numpy(), sr_noise=noise.numpy(),
               sr_dq=dq.numpy(), sr_merged=T.merge_i8(wm, dq).numpy(),
               sr_dq_scalar=T.sr_delta(delta, 0.0005, noise).numpy())

    np.savez_compressed(os.path.join(HERE, "vectors.npz"), **out)
    print("wrote", os.path.join(HERE, "vectors.npz"), {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
