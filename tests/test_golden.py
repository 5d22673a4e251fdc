"""Committed vectors (tests/golden/vectors.npz, written by tests/golden/make_golden.py from torch CPU
routines): the oracle must reproduce them on the CPU, the HIP library on the GPU."""
import os

import numpy as np
import pytest
import torch

import oracle as O

V = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz"))


def bf(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def f16(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.float16)


# ------------------------------------------------------------------ CPU: the oracle
def test_oracle_quant():
    q, s = O.quant_rowwise(V["quant_x"], O.BF16)
    assert np.array_equal(q, V["quant_q"]) and np.array_equal(s, V["quant_s"])


def test_oracle_rotate_and_quant():
    assert np.array_equal(O.rotate(V["rot_x"], O.BF16), V["rot_xr"])
    q, s = O.quant_rowwise(V["rot_x"], O.BF16, 128)
    assert np.array_equal(q, V["rot_q"]) and np.array_equal(s, V["rot_s"])


def test_oracle_gemm():
    assert np.array_equal(O.gemm_i32(V["gemm_a"], V["gemm_w"]), V["gemm_acc"])


def test_oracle_linear():
    x, b = V["lin_x"], V["lin_bias"]
    assert np.array_equal(O.linear_w8a8(x, O.BF16, V["lin_wq_row"], V["lin_ws_row"], b), V["lin_y_row_bias"])
    assert np.array_equal(O.linear_w8a8(x, O.BF16, V["lin_wq_row"], V["lin_ws_row"]), V["lin_y_row_nobias"])
    assert np.array_equal(O.linear_w8a8(x, O.BF16, V["lin_wq_tensor"], V["lin_ws_tensor"], b), V["lin_y_tensor_bias"])
    assert np.array_equal(O.linear_w8a8(V["lin_x_f16"], O.F16, V["lin_wq_tensor"], V["lin_ws_tensor"], out_dtype=O.F16),
                          V["lin_y_tensor_nobias_f16"])


def test_oracle_sr_merge():
    assert np.array_equal(O.sr_delta(V["sr_delta"], V["sr_ws"], V["sr_noise"]), V["sr_dq"])
    assert np.array_equal(O.sr_delta(V["sr_delta"], np.float32(0.0005), V["sr_noise"]), V["sr_dq_scalar"])
    assert np.array_equal(O.lora_merge_sr(V["sr_w"], V["sr_ws"], V["sr_noise"], delta=V["sr_delta"]), V["sr_merged"])


# ------------------------------------------------------------------ GPU: the HIP library
@pytest.mark.gpu
def test_hip_quant(L, dev):
    q, s = L.quant_rowwise(bf(V["quant_x"]).to(dev))
    assert np.array_equal(q.cpu().numpy(), V["quant_q"]) and np.array_equal(s.cpu().numpy(), V["quant_s"])


@pytest.mark.gpu
def test_hip_rotate_and_quant(L, dev):
    x = bf(V["rot_x"]).to(dev)
    assert np.array_equal(O.from_torch(L.rotate128(x).cpu())[0], V["rot_xr"])
    q, s = L.quant_rowwise(x, rotate=True)
    assert np.array_equal(q.cpu().numpy(), V["rot_q"]) and np.array_equal(s.cpu().numpy(), V["rot_s"])


@pytest.mark.gpu
def test_hip_gemm(L, dev):
    acc = L.gemm_i32(torch.from_numpy(V["gemm_a"]).to(dev), torch.from_numpy(V["gemm_w"]).to(dev))
    assert np.array_equal(acc.cpu().numpy(), V["gemm_acc"])


@pytest.mark.gpu
def test_hip_linear(pkg, dev):
    x, b = bf(V["lin_x"]).to(dev), bf(V["lin_bias"]).to(dev)
    wr, sr = torch.from_numpy(V["lin_wq_row"]).to(dev), torch.from_numpy(V["lin_ws_row"]).to(dev)
    wt, st = torch.from_numpy(V["lin_wq_tensor"]).to(dev), float(V["lin_ws_tensor"][0])

    def bits(t):
        return O.from_torch(t.cpu())[0]

    assert np.array_equal(bits(pkg.int8_forward_dynamic_per_row(x, wr, sr, b, torch.bfloat16)), V["lin_y_row_bias"])
    assert np.array_equal(bits(pkg.int8_forward_dynamic_per_row(x, wr, sr, None, torch.bfloat16)), V["lin_y_row_nobias"])
    assert np.array_equal(bits(pkg.int8_forward_dynamic(x, wt, st, b, torch.bfloat16)), V["lin_y_tensor_bias"])
    xh = f16(V["lin_x_f16"]).to(dev)
    assert np.array_equal(bits(pkg.int8_forward_dynamic(xh, wt, st, None, torch.float16)), V["lin_y_tensor_nobias_f16"])


@pytest.mark.gpu
def test_hip_sr_merge(pkg, L, dev):
    d, n = torch.from_numpy(V["sr_delta"]).to(dev), torch.from_numpy(V["sr_noise"]).to(dev)
    ws, w = torch.from_numpy(V["sr_ws"]).to(dev), torch.from_numpy(V["sr_w"]).to(dev)
    assert np.array_equal(L.sr_quant_delta(d, ws, n).cpu().numpy(), V["sr_dq"])
    assert np.array_equal(pkg.stochastic_round_int8_delta(d, 0.0005, noise=n).cpu().numpy(), V["sr_dq_scalar"])
    assert np.array_equal(L.lora_merge_sr(w, ws, n, delta=d).cpu().numpy(), V["sr_merged"])
