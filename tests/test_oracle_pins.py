"""Pins the CPU oracle (oracle/i8f_oracle.c) before anything is compared with it.

Each oracle function is checked against something that does not share its code:
the torch CPU routines the reference itself calls (oracle/torch_path.py), exact
rational arithmetic on tiny inputs, closed forms and invariants of the maths.
A wrong sign, index, rounding mode or operand order fails at least one of them.
"""
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle as O
from oracle import torch_path as T

G = torch.Generator().manual_seed(1234)


def randn(*shape, scale=1.0):
    return torch.randn(*shape, generator=G) * scale


def rn_f32(fr: Fraction) -> Fraction:
    """Correctly rounded (nearest, ties to even) binary32 value of a rational, as a Fraction; normal range only."""
    if fr == 0:
        return Fraction(0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = 0
    while a >= 2:
        a /= 2
        e += 1
    while a < 1:
        a *= 2
        e -= 1
    scaled = a * (1 << 23)
    fl = scaled.numerator // scaled.denominator
    rem = scaled - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return sign * Fraction(fl, 1 << 23) * (Fraction(2) ** e)


def rne_int(fr: Fraction) -> int:
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return fl


# ------------------------------------------------------------------ storage conversions
def test_bf16_widening_all_patterns():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).float().numpy()
    got = np.array([O.lib().orc_bf16_to_f32(int(b)) for b in bits[::7]], dtype=np.float32)
    ok = ~np.isnan(want[::7])   # a signalling NaN is quieted on its way back through the C float return
    assert np.array_equal(got.view(np.uint32)[ok], want[::7].view(np.uint32)[ok]) and np.isnan(got[~ok]).all()
    assert np.array_equal(O.to_f32(bits, O.BF16).view(np.uint32), want.view(np.uint32))


def test_f16_widening_all_patterns():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([O.lib().orc_f16_to_f32(int(b)) for b in bits[::5]], dtype=np.float32)
    ok = ~np.isnan(want[::5])
    assert np.array_equal(got.view(np.uint32)[ok], want[::5].view(np.uint32)[ok]) and np.isnan(got[~ok]).all()


@pytest.mark.parametrize("code,tdt", [(O.BF16, torch.bfloat16), (O.F16, torch.float16)])
def test_narrowing_matches_torch_cast(code, tdt):
    v = torch.cat([
        randn(4000), randn(2000, scale=1e-6), randn(2000, scale=3e4), randn(500, scale=1e-8),
        torch.tensor([0.0, -0.0, 1.0, 65504.0, 65519.9, 65520.0, 1e38, -1e38, 2.0**-24, 2.0**-25, 3 * 2.0**-25,
                      float("inf"), -float("inf"), 1.00390625, 1.01171875, 1.005859375]),
    ])
    # exact ties of both formats
    base = randn(500).bfloat16().float() if code == O.BF16 else randn(500).half().float()
    ulp = (base.abs() * 2.0**-8) if code == O.BF16 else (base.abs() * 2.0**-11)
    v = torch.cat([v, base + ulp])
    want = v.to(tdt).view(torch.int16).numpy().view(np.uint16)
    fn = O.lib().orc_f32_to_bf16 if code == O.BF16 else O.lib().orc_f32_to_f16
    got = np.array([fn(float(t)) for t in v.numpy()], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(O.round_to(v.numpy(), code), want)


# ------------------------------------------------------------------ a1: row quantiser
@pytest.mark.parametrize("tdt", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(37, 512), (5, 3072), (3, 77), (1, 1)])
def test_quant_rowwise_equals_torch_ops(tdt, shape):
    x = randn(*shape)
    x[:, :: max(1, shape[1] // 7)] *= 20
    x = x.to(tdt)
    xa, code = O.from_torch(x)
    q, s = O.quant_rowwise(xa, code)
    qt, st = T.quant_rowwise(x)
    assert np.array_equal(q, qt.numpy())
    assert np.array_equal(s.view(np.uint32), st.numpy().view(np.uint32))


def test_quant_rowwise_exact_rational_bruteforce():
    x = randn(6, 9).bfloat16()
    xa, code = O.from_torch(x)
    q, s = O.quant_rowwise(xa, code)
    for m in range(6):
        vals = [Fraction(float(v)) for v in x[m].float()]
        amax = max(abs(v) for v in vals)
        sc = rn_f32(amax / 127)
        inv = rn_f32(1 / sc)
        assert Fraction(float(s[m, 0])) == sc
        for k, v in enumerate(vals):
            assert int(q[m, k]) == max(-128, min(127, rne_int(rn_f32(v * inv))))


def test_quant_rowwise_properties():
    x = randn(64, 256).bfloat16()
    x[3] = 0
    x[5, :] = 0
    x[5, 17] = -3.0
    xa, code = O.from_torch(x)
    q, s = O.quant_rowwise(xa, code)
    assert s[3, 0] == np.float32(1e-30) and not q[3].any()           # zero row: clamp on the scale
    nz = [m for m in range(64) if m != 3]
    assert (np.abs(q[nz].astype(np.int32)).max(axis=1) == 127).all()  # the absmax element lands on +-127
    assert q[5, 17] == -127 and np.count_nonzero(q[5]) == 1
    err = np.abs(x.float().numpy() - q.astype(np.float32) * s)
    assert (err <= s * 0.5 + np.abs(x.float().numpy()) * 1e-6).all()  # half a quantisation step
    # ties go to even: x = (n + 0.5) * scale exactly
    row = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5]])
    q2, s2 = O.quant_rowwise(row.numpy(), O.F32)
    assert s2[0, 0] == 1.0 and q2.tolist() == [[127, 0, 2, 2, 0, -2, -2, 4]]
    # idempotence: quantising the dequantised grid returns the same integers
    deq = (q.astype(np.float32) * s).astype(np.float32)
    q3, s3 = O.quant_rowwise(deq, O.F32)
    assert np.array_equal(q3[nz], q[nz])


def test_quant_tensorwise_equals_torch_ops():
    w = (randn(96, 160) * 0.02).bfloat16()
    wa, code = O.from_torch(w)
    q, s = O.quant_tensorwise(wa, code)
    qt, st = T.quant_tensorwise(w)
    assert np.array_equal(q, qt.numpy()) and s[0] == st.item()


# ------------------------------------------------------------------ a3/a4: rotation
def test_hadamard_entry_constants():
    for code, tdt in [(O.BF16, torch.bfloat16), (O.F16, torch.float16), (O.F32, torch.float32)]:
        H = T.hadamard(128, tdt)
        assert float(H[0, 0].float()) == O.lib().orc_hadamard_entry(code)
        assert torch.equal(H.abs(), torch.full_like(H, H[0, 0].item()))


@pytest.mark.parametrize("n", [2, 8, 128])
def test_fwht_is_sylvester_hadamard_exactly_on_integers(n):
    from scipy.linalg import hadamard

    # small integers: every butterfly sum is exact in binary32, so any order gives the dense product exactly
    v = torch.randint(-512, 513, (n,), generator=G).float().numpy()
    want = v.astype(np.float64) @ hadamard(n).astype(np.float64)
    assert np.array_equal(O.fwht(v).astype(np.float64), want)
    assert np.array_equal(O.fwht(O.fwht(v)), v * n)                  # H H = n I
    e = np.zeros(n, dtype=np.float32)
    e[5 % n] = 1
    assert np.array_equal(O.fwht(e), hadamard(n)[5 % n].astype(np.float32))  # one row of H: fixes the sign pattern


def test_fwht_stage_order_is_the_documented_one():
    # the rounding of binary32 sums depends on the order: restate the butterfly in numpy float32
    v = (randn(128) * torch.logspace(-3, 3, 128)).numpy().astype(np.float32)
    w = v.copy()
    stride = 1
    while stride < 128:
        w = w.reshape(-1, 2, stride)
        lo, hi = w[:, 0, :].copy(), w[:, 1, :].copy()
        w[:, 0, :], w[:, 1, :] = lo + hi, lo - hi
        w = w.reshape(-1)
        stride *= 2
    assert np.array_equal(O.fwht(v).view(np.uint32), w.view(np.uint32))


@pytest.mark.parametrize("code,tdt,tol_ulp", [(O.BF16, torch.bfloat16, 2.0**-8), (O.F16, torch.float16, 2.0**-11),
                                              (O.F32, torch.float32, 2.0**-22)])
def test_rotate_close_to_dense_matmul(code, tdt, tol_ulp):
    x = randn(24, 512)
    x[:, ::37] *= 50
    x = x.to(tdt)
    xa, _ = O.from_torch(x)
    got = O.to_f32(O.rotate(xa, code), code).astype(np.float64)
    H = T.hadamard(128, tdt).double().numpy()
    dense = (x.double().numpy().reshape(24, 4, 128) @ H).reshape(24, 512)   # exact product, float64
    # error budget: one rounding of the result to the dtype, plus binary32 accumulation error, which is
    # relative to the sum of the magnitudes (8 adds deep), not to the possibly cancelled result
    mags = (np.abs(x.double().numpy()).reshape(24, 4, 128) @ np.abs(H)).reshape(24, 512)
    budget = tol_ulp * np.abs(dense) * 1.01 + 8 * 2.0**-24 * mags
    assert (np.abs(got - dense) <= budget).all()
    # and against the library product the reference actually runs (its summation order is BLAS's)
    lib = T.rotate(x).double().numpy()
    assert (np.abs(got - lib) <= 2 * tol_ulp * np.abs(dense) * 1.01 + 64 * 2.0**-24 * mags).all()


def test_rotated_quantisation_agrees_with_torch_path_statistically():
    x = randn(64, 3840)
    x[:, torch.randperm(3840, generator=G)[:77]] *= 50
    x = x.bfloat16()
    xa, code = O.from_torch(x)
    q, s = O.quant_rowwise(xa, code, 128)
    qt, st = T.quant_rowwise(T.rotate(x))
    diff = np.abs(q.astype(np.int32) - qt.numpy().astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 1e-3              # only summation-order ties differ
    assert np.allclose(s, st.numpy(), rtol=2.0**-7)                   # scales within one bf16 ulp


def test_rotation_is_orthogonal_and_cancels_in_the_product():
    x, w = randn(16, 256).numpy(), randn(24, 256, scale=0.02).numpy()
    xr, wr = O.rotate(x, O.F32), O.rotate(w, O.F32)
    assert np.allclose((xr**2).sum(1), (x**2).sum(1), rtol=1e-5)
    assert np.allclose(xr @ wr.T, x @ w.T, rtol=1e-4, atol=1e-5)
    assert np.allclose(O.rotate(xr, O.F32), x, rtol=1e-5, atol=1e-6)  # H is an involution


def test_rotation_spreads_outliers():
    x = randn(32, 1024)
    x[:, 100] = 50.0
    xa, code = O.from_torch(x.bfloat16())
    _, s_plain = O.quant_rowwise(xa, code)
    _, s_rot = O.quant_rowwise(xa, code, 128)
    assert (s_rot < s_plain * 0.5).all()


# ------------------------------------------------------------------ a5: integer product
@pytest.mark.parametrize("M,N,K", [(32, 24, 64), (17, 40, 3072), (33, 8, 8), (64, 16, 1000)])
def test_gemm_i32_equals_int_mm_and_int64(M, N, K):
    a = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=G)
    w = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=G)
    acc = O.gemm_i32(a.numpy(), w.numpy())
    assert np.array_equal(acc, a.numpy().astype(np.int64) @ w.numpy().astype(np.int64).T)
    if M > 16 and K % 8 == 0 and N % 8 == 0:
        assert np.array_equal(acc, torch._int_mm(a, w.T).numpy())


def test_gemm_i32_extremes_do_not_overflow():
    K = 12288
    a = np.full((2, K), -128, dtype=np.int8)
    w = np.stack([np.full(K, -128, dtype=np.int8), np.full(K, 127, dtype=np.int8)])
    acc = O.gemm_i32(a, w)
    assert acc.tolist() == [[K * 16384, -K * 16256]] * 2
    ident = np.eye(64, dtype=np.int8)
    b = np.random.default_rng(0).integers(-128, 128, (9, 64), dtype=np.int8)
    assert np.array_equal(O.gemm_i32(b, ident), b.astype(np.int32))   # a @ I.T = a: operands are not swapped
    assert O.gemm_i32(np.zeros((3, 0), np.int8), np.zeros((5, 0), np.int8)).tolist() == [[0] * 5] * 3


# ------------------------------------------------------------------ a6/a7: epilogue
def _epi_inputs(M=40, N=56):
    acc = torch.randint(-2_000_000, 2_000_000, (M, N), dtype=torch.int32, generator=G)
    acc[0, 0], acc[0, 1] = 2**27 + 5, -(2**27) - 3                    # beyond 2^24: int -> float rounds
    xs = (torch.rand(M, 1, generator=G) * 0.05 + 1e-3)
    ws_row = (torch.rand(N, 1, generator=G) * 2e-3 + 1e-4)
    bias = randn(N, scale=0.3)
    return acc, xs, ws_row, bias


@pytest.mark.parametrize("tdt,code", [(torch.bfloat16, O.BF16), (torch.float16, O.F16)])
@pytest.mark.parametrize("row", [False, True])
@pytest.mark.parametrize("with_bias", [False, True])
def test_epilogue_torch_order_equals_torch_ops(tdt, code, row, with_bias):
    acc, xs, ws_row, bias = _epi_inputs()
    b = bias.to(tdt) if with_bias else None
    if row:
        want = acc.float().mul_(xs).mul_(ws_row.T).to(tdt)
        ws = ws_row
    else:
        ws = 0.00123
        want = acc.float().mul_(ws * xs).to(tdt)
    if with_bias:
        want = want + b.to(tdt)
    got = O.epilogue(acc.numpy(), xs.numpy(), ws_row.numpy() if row else np.float32(ws),
                     None if b is None else O.from_torch(b)[0], code, code, O.EPI_TORCH)
    assert np.array_equal(got, O.from_torch(want)[0])


def test_epilogue_float32_bias_is_rounded_to_output_dtype_first():
    acc, xs, ws_row, bias = _epi_inputs()
    want = acc.float().mul_(xs).mul_(ws_row.T).to(torch.bfloat16) + bias.to(torch.bfloat16)
    got = O.epilogue(acc.numpy(), xs.numpy(), ws_row.numpy(), bias.numpy(), O.F32, O.BF16, O.EPI_TORCH)
    assert np.array_equal(got, O.from_torch(want)[0])


@pytest.mark.parametrize("row", [False, True])
def test_epilogue_fused_order_closed_form(row):
    acc, xs, ws_row, bias = _epi_inputs()
    ws = ws_row if row else torch.tensor([[0.00123]])
    got32 = O.epilogue(acc.numpy(), xs.numpy(), ws.numpy(), bias.numpy(), O.F32, O.F32, O.EPI_FUSED)
    sc = (xs * ws.T).float()                                          # one rounded product of the scales
    want32 = (acc.float() * sc + bias).numpy()                        # torch: separate multiply and add
    assert np.array_equal(got32.view(np.uint32), want32.view(np.uint32))
    exact = acc.double() * xs.double() * ws.T.double() + bias.double()
    mag = (acc.double() * xs.double() * ws.T.double()).abs() + bias.double().abs()
    assert ((torch.from_numpy(got32).double() - exact).abs() <= 4 * 2.0**-24 * mag).all()
    got16 = O.epilogue(acc.numpy(), xs.numpy(), ws.numpy(), O.from_torch(bias.bfloat16())[0], O.BF16, O.BF16, O.EPI_FUSED)
    want16 = (acc.float() * sc + bias.bfloat16().float()).bfloat16()
    assert np.array_equal(got16, O.from_torch(want16)[0])


@pytest.mark.parametrize("row", [False, True])
@pytest.mark.parametrize("rot", [0, 128])
def test_linear_w8a8_equals_torch_path(row, rot):
    x = randn(48, 256)
    x[:, 7] *= 20
    x = x.bfloat16()
    wf = randn(40, 256, scale=0.02)
    wq, ws = (T.quant_rowwise(wf) if row else T.quant_tensorwise(wf))
    bias = randn(40, scale=0.01).bfloat16()
    xa, code = O.from_torch(x)
    got = O.linear_w8a8(xa, code, wq.numpy(), ws.numpy(), O.from_torch(bias)[0], O.BF16, O.BF16, rot)
    if rot:   # the torch path rotates with a BLAS product: compare from the oracle's own rotated activations on
        xr = O.to_torch(O.rotate(xa, code), code)
        want = T.linear_w8a8(xr, wq, ws if row else ws.item(), bias, torch.bfloat16)
    else:
        want = T.linear_w8a8(x, wq, ws if row else ws.item(), bias, torch.bfloat16)
    assert np.array_equal(got, O.from_torch(want)[0])


# ------------------------------------------------------------------ a8: small batch W8A16
@pytest.mark.parametrize("tdt,tol", [(torch.bfloat16, 2.0**-7), (torch.float16, 2.0**-10), (torch.float32, 1e-5)])
def test_linear_w8a16_within_tolerance_of_f_linear(tdt, tol):
    x = randn(5, 384).to(tdt)
    wq = torch.randint(-128, 128, (72, 384), dtype=torch.int8, generator=G)
    ws = torch.rand(72, 1, generator=G) * 1e-2 + 1e-3
    bias = randn(72, scale=0.1).to(tdt)
    want = T.linear_w8a16(x, wq, ws, bias).float().numpy()
    xa, code = O.from_torch(x)
    got = O.to_f32(O.linear_w8a16(xa, code, wq.numpy(), ws.numpy(), O.from_torch(bias)[0], code), code)
    assert (np.abs(got - want) <= tol * np.abs(want) + tol * 0.05).all()


# ------------------------------------------------------------------ a9/a10/a11: stochastic merge
@pytest.mark.parametrize("row", [False, True])
def test_sr_delta_equals_torch_ops(row):
    x = randn(64, 96, scale=0.01)
    x[0, :4] = torch.tensor([1.0, -1.0, 0.5, 3.0])                    # saturation on both sides
    scale = (torch.rand(64, 1, generator=G) * 1e-3 + 1e-4) if row else 0.00037
    noise = torch.rand(64, 96, generator=G)
    want = T.sr_delta(x, scale, noise)
    got = O.sr_delta(x.numpy(), scale.numpy() if row else np.float32(scale), noise.numpy())
    assert np.array_equal(got, want.numpy())
    assert got.min() == -128 and got.max() == 127


def test_sr_delta_special_cases():
    scale = np.float32(0.25)
    x = np.array([[0.5, 0.3, -0.3, 0.26, -0.26, 0.0, 40.0, -40.0]], dtype=np.float32)   # x/scale = 2, 1.2, -1.2, 1.04, ...
    zeros, almost1 = np.zeros_like(x), np.full_like(x, 1 - 2.0**-24)
    assert O.sr_delta(x, scale, zeros).tolist() == [[2, 2, -1, 2, -1, 0, 127, -128]]     # noise 0: up whenever frac > 0, never when frac == 0
    assert O.sr_delta(x, scale, almost1).tolist() == [[2, 1, -2, 1, -2, 0, 127, -128]]   # noise -> 1: floor
    # strict compare: noise == frac rounds down
    assert O.sr_delta(np.array([[0.375]], np.float32), scale, np.array([[0.5]], np.float32)).tolist() == [[1]]
    # unbiased: the mean over many draws approaches x / scale
    xs = np.full((1, 200000), 0.3, dtype=np.float32)
    noise = torch.rand(1, 200000, generator=G).numpy()
    assert abs(O.sr_delta(xs, scale, noise).astype(np.float64).mean() - 1.2) < 5e-3


def test_row_scale_without_a_division_is_the_division_for_every_16_bit_maximum():
    """The HIP quantiser for bfloat16 / binary16 rows takes amax / 127 as fma(fma(-127, q, amax), y, q), q = amax y,
    y = RN(1/127).  amax is a value of the row's dtype, so every case there is can be checked: all finite
    non-negative patterns of both dtypes (and, for good measure, 4 M random binary32 values)."""
    bf = (np.arange(0, 0x7F80, dtype=np.uint32) << 16).view(np.float32)
    h = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    assert O.scale_by_127_mismatches(bf) == (0, -1)
    assert O.scale_by_127_mismatches(h) == (0, -1)
    rng = np.random.default_rng(5)
    r32 = rng.integers(0, 0x7F000000, 4_000_000, dtype=np.int64).astype(np.uint32).view(np.float32)
    assert O.scale_by_127_mismatches(r32) == (0, -1)


def test_quotient_by_reciprocal_is_the_correctly_rounded_division():
    """The HIP merge kernels compute delta / scale as q = delta * y, twice q += fma(-scale, q, delta) * y with
    y = 1 / scale, where 2^-20 <= scale <= 2^20 and 2^-102 <= |delta| <= 2^80 (everything else takes the division).
    That this equals the IEEE quotient is a theorem (Markstein) for a quotient estimate within one ulp, which the
    first correction provides; here it is checked on random operands over the whole permitted range, on mantissas at
    the ends of a binade and, the hard cases for a correctly rounded result, on quotients that lie as close to the
    midpoint of two neighbouring floats as two 24-bit significands allow."""
    rng = np.random.default_rng(11)
    n = 2_000_000

    def floats(mant, expo, sign=None):
        bits = (mant.astype(np.uint32) & 0x7FFFFF) | ((expo + 127).astype(np.uint32) << 23)
        if sign is not None:
            bits |= sign.astype(np.uint32) << 31
        return bits.view(np.float32)

    # random mantissas, every permitted exponent, both signs of the numerator
    a = floats(rng.integers(0, 1 << 23, n), rng.integers(-102, 81, n), rng.integers(0, 2, n))
    b = floats(rng.integers(0, 1 << 23, n), rng.integers(-20, 21, n))
    assert O.quotient_by_reciprocal_mismatches(a, b) == (0, -1)
    # mantissas next to 1 and next to 2 on either side, and numerators next to the denominator
    edge = np.concatenate([np.arange(0, 16), np.arange((1 << 23) - 16, 1 << 23)])
    mb = rng.choice(edge, n)
    ma = np.where(rng.integers(0, 2, n) == 0, rng.choice(edge, n), (mb + rng.integers(-2, 3, n)) & 0x7FFFFF)
    a = floats(ma, rng.integers(-102, 81, n), rng.integers(0, 2, n))
    b = floats(mb, rng.integers(-20, 21, n))
    assert O.quotient_by_reciprocal_mismatches(a, b) == (0, -1)
    a = floats(rng.integers(0, 1 << 23, n), rng.integers(-102, 81, n))
    assert O.quotient_by_reciprocal_mismatches(a, floats(mb, rng.integers(-20, 21, n))) == (0, -1)
    # Quotients next to a rounding boundary.  With integer significands A, B (24 bits) and an odd 25-bit M (the
    # midpoint of two neighbouring floats), A / B lies closest to the midpoint when A 2^s - B M = k for a small odd k,
    # s = 24 for quotients in [1, 2) and 25 for those in [1/2, 1): M = -k / B modulo 2^s, then A follows.
    for s_bits in (24, 25):
        B = (rng.integers(1 << 22, 1 << 23, n).astype(np.uint64) << np.uint64(1)) | np.uint64(1)   # odd, 24 bits
        k = rng.choice(np.array([-3, -1, 1, 3]), n)
        mask = np.uint64((1 << s_bits) - 1)
        inv = B.copy()
        for _ in range(5):                                                       # Newton: inverse of B modulo 2^s
            inv = (inv * (np.uint64(2) - B * inv)) & mask
        assert np.all((B * inv) & mask == 1)
        M = ((-k).astype(np.int64).astype(np.uint64) * inv) & mask
        if s_bits == 24:
            M = M | np.uint64(1 << 24)
        num = (B * M).astype(np.int64) + k
        assert np.all(num % (1 << s_bits) == 0)
        A = num >> s_bits
        ok = (M >= (1 << 24)) & (A >= (1 << 23)) & (A < (1 << 24))
        assert ok.mean() > 0.2
        A, Bk, M, k = A[ok], B[ok].astype(np.int64), M[ok].astype(np.int64), k[ok]
        a, b = A.astype(np.float32), Bk.astype(np.float32)                       # exact: 24-bit integers
        # distance from the midpoint in units of the quotient's ulp (2^-23 below 2, 2^-24 below 1): |k| / B
        assert np.all(A * (1 << s_bits) - Bk * M == k) and np.abs(k / Bk).max() < 2.0**-21
        for ea, eb in ((0, 0), (-90, 13), (70, -19)):                            # scaling by powers of two changes nothing
            assert O.quotient_by_reciprocal_mismatches(np.ldexp(a, ea), np.ldexp(b, eb)) == (0, -1)
            assert O.quotient_by_reciprocal_mismatches(-np.ldexp(a, ea), np.ldexp(b, eb)) == (0, -1)
    # and the check itself can fail: one correction fewer than needed for a poor reciprocal shows up
    bad, first = O.quotient_by_reciprocal_mismatches(np.float32([1.0, np.inf, 1e-44]), np.float32([3.0, 2.0, 3.0]))
    assert bad >= 1 and first >= 1                         # inf and denormal numerators are outside the permitted range


def test_merge_i8_all_pairs():
    a = np.arange(-128, 128, dtype=np.int8)
    w, dq = np.meshgrid(a, a, indexing="ij")
    got = O.merge_i8(np.ascontiguousarray(w), np.ascontiguousarray(dq))
    assert np.array_equal(got, np.clip(w.astype(np.int32) + dq.astype(np.int32), -128, 127).astype(np.int8))
    assert np.array_equal(got, T.merge_i8(torch.from_numpy(np.ascontiguousarray(w)), torch.from_numpy(np.ascontiguousarray(dq))).numpy())


def test_lora_delta_fma_chain_exact_and_close_to_mm():
    up, down = randn(6, 4, scale=0.1), randn(4, 5, scale=0.1)
    got = O.lora_delta(up.numpy(), down.numpy(), 0.7)
    s32 = Fraction(float(np.float32(0.7)))
    for n in range(6):
        for k in range(5):
            acc = Fraction(0)
            for j in range(4):   # fma: one rounding of the exact a*b + c
                acc = rn_f32(Fraction(float(up[n, j])) * Fraction(float(down[j, k])) + acc)
            assert Fraction(float(got[n, k])) == rn_f32(acc * s32)
    up, down = randn(128, 32, scale=0.01), randn(32, 96, scale=0.01)
    got = O.lora_delta(up.numpy(), down.numpy(), 1.0)
    assert np.allclose(got, torch.mm(up, down).numpy(), rtol=1e-4, atol=1e-9)


def test_lora_merge_composes_the_three_steps():
    N, K, r = 48, 64, 8
    w = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=G)
    ws = torch.rand(N, 1, generator=G) * 1e-3 + 2e-4
    up, down = randn(N, r, scale=0.05), randn(r, K, scale=0.05)
    noise = torch.rand(N, K, generator=G)
    delta = O.lora_delta(up.numpy(), down.numpy(), 0.5)
    want = T.merge_i8(w, T.sr_delta(torch.from_numpy(delta), ws, noise)).numpy()
    assert np.array_equal(O.lora_merge_sr(w.numpy(), ws.numpy(), noise.numpy(), delta=delta), want)
    assert np.array_equal(O.lora_merge_sr(w.numpy(), ws.numpy(), noise.numpy(), up=up.numpy(), down=down.numpy(), lora_scale=0.5), want)
    assert (want != w.numpy()).mean() > 0.5


# ------------------------------------------------------------------ prologue in front of the quantiser
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32])
def test_prologue_modulate_equals_torch_eager_ops(dt):
    """(1 + s) * x + t as three torch tensor operations in the tensor's dtype, bit for bit; two images of a
    batch with their own vectors."""
    g = torch.Generator().manual_seed(31)
    x = torch.randn(2 * 6, 200, generator=g).to(dt)
    sc, sh = (torch.randn(2, 200, generator=g) * 0.3).to(dt), torch.randn(2, 200, generator=g).to(dt)
    want = ((1 + sc[:, None, :]) * x.view(2, 6, 200) + sh[:, None, :]).reshape(12, 200)
    xa, code = O.from_torch(x)
    got = O.prologue(xa, code, O.PRO_MODULATE, O.from_torch(sc)[0], O.from_torch(sh)[0], rows_per_vec=6)
    assert np.array_equal(got, O.from_torch(want)[0])


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32])
def test_prologue_gelu_tanh_agrees_with_torch(dt):
    """torch's gelu(approximate="tanh") uses its own vectorised tanh: equal up to the last bits of binary32,
    i.e. at most one unit in the last place of the storage dtype, and that only rarely."""
    g = torch.Generator().manual_seed(32)
    x = (torch.randn(64, 512, generator=g) * 3).to(dt)
    x[0, :8] = torch.tensor([0.0, -0.0, 1e-6, -1e-6, 20.0, -20.0, 100.0, -100.0]).to(dt)
    want = torch.nn.functional.gelu(x, approximate="tanh")
    xa, code = O.from_torch(x)
    got = O.to_f32(O.prologue(xa, code, O.PRO_GELU_TANH), code)
    w = want.float().numpy()
    ulp = {torch.bfloat16: 2.0**-7, torch.float16: 2.0**-10, torch.float32: 2.0**-22}[dt]   # the largest spacing relative to the value
    # far in the negative tail 1 + tanh cancels to the last bit of binary32: an absolute 2^-23 |x| on top
    assert (np.abs(got - w) <= ulp * np.abs(w) + 2.0**-23 * np.abs(x.float().numpy())).all()
    assert (got != w).mean() < (1e-2 if dt != torch.float32 else 0.5)
    assert got[0, 4] == 20.0 and got[0, 5] == 0.0 and got[0, 0] == 0.0


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32])
def test_prologue_silu_gate_agrees_with_torch(dt):
    """silu(a) * b as torch's two eager kernels compute it: the oracle divides by 1 + expf(-a) with the C library's
    expf, torch with its own vectorised exp, so the activated value may differ in the last bit of binary32, i.e. now
    and then by one unit in the last place of the dtype before the product; the product of equal activations is equal."""
    g = torch.Generator().manual_seed(33)
    a = (torch.randn(64, 512, generator=g) * 3).to(dt)
    b = torch.randn(64, 512, generator=g).to(dt)
    a[0, :8] = torch.tensor([0.0, -0.0, 1e-6, -1e-6, 20.0, -20.0, 100.0, -100.0]).to(dt)
    want = torch.nn.functional.silu(a) * b
    got = O.to_f32(O.prologue(O.from_torch(a)[0], O.from_torch(a)[1], O.PRO_SILU_GATE, O.from_torch(b)[0], rows_per_vec=1), O.from_torch(a)[1])
    w = want.float().numpy()
    ulp = {torch.bfloat16: 2.0**-7, torch.float16: 2.0**-10, torch.float32: 2.0**-22}[dt]
    # one unit of the activated value, carried through the product and its rounding
    assert (np.abs(got - w) <= 2 * ulp * np.abs(w) + 1e-30).all()
    assert (got != w).mean() < (1e-2 if dt != torch.float32 else 0.5)
    assert got[0, 0] == 0.0 and got[0, 4] == np.float32((torch.tensor(20.0).to(dt) * b[0, 4]).float())   # silu(0) = 0, silu(20) rounds to 20
    # one gate row for every three rows of a (the layout the kernel's vector form shares with the modulation)
    b3 = torch.randn(4, 512, generator=g).to(dt)
    a3 = a[:12]
    got3 = O.prologue(O.from_torch(a3)[0], O.from_torch(a3)[1], O.PRO_SILU_GATE, O.from_torch(b3)[0], rows_per_vec=3)
    want3 = O.prologue(O.from_torch(a3)[0], O.from_torch(a3)[1], O.PRO_SILU_GATE, O.from_torch(b3.repeat_interleave(3, 0))[0], rows_per_vec=1)
    assert np.array_equal(got3, want3)


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_norm_modulate_agrees_with_torch(dt):
    """(1 + s) * layer_norm(x) + t as torch's eager kernels compute it on 16-bit tensors (LayerNorm without affine in
    binary32 with its own order of the sums, then three rounded tensor operations).  The oracle takes the row's sums
    in double, so the normalised value may differ from torch's by one unit in the last place of the dtype at rounding
    boundaries; that unit is carried through the modulation.  Also pinned: the closed form on a row whose statistics
    are exact (values +-1: mean 0, variance 1) and the row-group layout of the vectors."""
    g = torch.Generator().manual_seed(41)
    M, K, eps = 48, 768, 1e-6
    x = (torch.randn(M, K, generator=g) * 2 + 0.3).to(dt)
    x[:, 5] *= 30                                             # an outlier channel, as adaLN inputs have
    s = (torch.randn(1, K, generator=g) * 0.3).to(dt)
    t = (torch.randn(1, K, generator=g) * 0.2).to(dt)
    want = (1 + s) * torch.nn.functional.layer_norm(x, (K,), eps=eps) + t
    code = O.from_torch(x)[1]
    got = O.to_f32(O.norm_modulate(O.from_torch(x)[0], code, eps, O.from_torch(s)[0], O.from_torch(t)[0], rows_per_vec=M), code)
    w = want.float().numpy()
    ulp = {torch.bfloat16: 2.0**-7, torch.float16: 2.0**-10}[dt]
    y = torch.nn.functional.layer_norm(x.float(), (K,), eps=eps).numpy()
    # one unit of the normalised value times the gain, plus the roundings of the product and of the sum
    bound = ulp * (np.abs(y) * np.abs(1 + s.float().numpy()) + np.abs(w)) + 1e-30
    assert (np.abs(got - w) <= bound).all()
    assert (got != w).mean() < 2e-2
    # exact statistics: +-1 in equal numbers has mean 0 and variance 1, so y = x / sqrt(1 + eps), which rounds to x
    pm = torch.ones(4, 256)
    pm[:, ::2] = -1
    sv, tv = (torch.randn(2, 256, generator=g) * 0.5).to(dt), torch.randn(2, 256, generator=g).to(dt)
    got2 = O.to_torch(O.norm_modulate(O.from_torch(pm.to(dt))[0], code, 1e-6, O.from_torch(sv)[0], O.from_torch(tv)[0], rows_per_vec=2), code)
    want2 = ((1 + sv).repeat_interleave(2, 0) * pm.to(dt)) + tv.repeat_interleave(2, 0)
    assert torch.equal(got2.view(torch.int16), want2.view(torch.int16))
    # a constant row: variance 0, y = 0 exactly, the result is the shift
    const = torch.full((1, 64), 3.25).to(dt)
    got3 = O.to_torch(O.norm_modulate(O.from_torch(const)[0], code, 1e-5, O.from_torch(sv[:1, :64].contiguous())[0], O.from_torch(tv[:1, :64].contiguous())[0]), code)
    assert torch.equal(got3.view(torch.int16), tv[:1, :64].contiguous().view(torch.int16))


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_prologue_fused_modulation_equals_torch_addcmul(dt):
    """torch.addcmul(shift, x, 1 + scale), the one-kernel spelling of the modulation (the gain a rounded tensor of its
    own, product and sum rounded once): bit-equal on 16-bit CPU tensors, vectors dealt over groups of rows; it differs
    from the three-operation form exactly where the extra rounding of the product matters; and the two normalising
    oracles' fused forms equal this kind applied to their own normalised tensor."""
    g = torch.Generator().manual_seed(35)
    x = (torch.randn(2 * 6, 200, generator=g) * 3).to(dt)
    sc, sh = (torch.randn(2, 200, generator=g) * 0.3).to(dt), torch.randn(2, 200, generator=g).to(dt)
    want = torch.addcmul(sh[:, None, :], x.view(2, 6, 200), 1 + sc[:, None, :]).reshape(12, 200)
    xa, code = O.from_torch(x)
    got = O.prologue(xa, code, O.PRO_MODULATE_FUSED, O.from_torch(sc)[0], O.from_torch(sh)[0], rows_per_vec=6)
    assert np.array_equal(got, O.from_torch(want)[0])
    three = O.prologue(xa, code, O.PRO_MODULATE, O.from_torch(sc)[0], O.from_torch(sh)[0], rows_per_vec=6)
    assert 0.01 < (got != three).mean() < 0.6
    w = (torch.randn(200, generator=g) * 0.2 + 1).to(dt)
    y = O.rms_norm(xa, code, 1e-5, O.from_torch(w)[0])
    fused = O.rms_norm(xa, code, 1e-5, O.from_torch(w)[0], O.from_torch(sc)[0], O.from_torch(sh)[0], rows_per_vec=6, fused=True)
    assert np.array_equal(fused, O.prologue(y, code, O.PRO_MODULATE_FUSED, O.from_torch(sc)[0], O.from_torch(sh)[0], rows_per_vec=6))
    only_s = O.rms_norm(xa, code, 1e-5, O.from_torch(w)[0], O.from_torch(sc)[0], None, rows_per_vec=6, fused=True)   # no shift: nothing to fuse
    assert np.array_equal(only_s, O.rms_norm(xa, code, 1e-5, O.from_torch(w)[0], O.from_torch(sc)[0], None, rows_per_vec=6))
    # LayerNorm form: against torch end to end within the tolerance of the normalised value, and tighter than the
    # three-operation form is to the same target
    want_ln = torch.addcmul(sh[:, None, :], torch.nn.functional.layer_norm(x, (200,), eps=1e-6).view(2, 6, 200), 1 + sc[:, None, :]).reshape(12, 200)
    got_ln = O.to_f32(O.norm_modulate(xa, code, 1e-6, O.from_torch(sc)[0], O.from_torch(sh)[0], rows_per_vec=6, fused=True), code)
    wl = want_ln.float().numpy()
    ulp = {torch.bfloat16: 2.0**-7, torch.float16: 2.0**-10}[dt]
    yl = torch.nn.functional.layer_norm(x.float(), (200,), eps=1e-6).numpy()
    gain = np.abs(1 + sc.float().numpy()).repeat(6, 0)
    assert (np.abs(got_ln - wl) <= ulp * (np.abs(yl) * gain + np.abs(wl)) + 1e-30).all() and (got_ln != wl).mean() < 2e-2


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32])
def test_prologue_gelu_erf_agrees_with_torch_and_with_the_normal_distribution(dt):
    """GELU in its exact form, x Phi(x): against torch's gelu (same binary32 expression, its own vectorised erf: at most
    one unit in the last place of the storage dtype apart, and rarely) and against scipy's normal distribution function
    in double (what the mathematics fixes; the binary32 expression 1 + erf cancels in the negative tail, so the bound
    carries a few units of 2^-24 |x| on top of the dtype's rounding)."""
    from scipy.special import ndtr
    g = torch.Generator().manual_seed(34)
    x = (torch.randn(64, 512, generator=g) * 3).to(dt)
    x[0, :8] = torch.tensor([0.0, -0.0, 1e-6, -1e-6, 20.0, -20.0, 100.0, -100.0]).to(dt)
    want = torch.nn.functional.gelu(x)
    xa, code = O.from_torch(x)
    got = O.to_f32(O.prologue(xa, code, O.PRO_GELU_ERF), code)
    w = want.float().numpy()
    ulp = {torch.bfloat16: 2.0**-7, torch.float16: 2.0**-10, torch.float32: 2.0**-22}[dt]
    xf = x.float().numpy()
    tiny = 2.0**-24 if dt == torch.float16 else 0.0      # the spacing of fp16's subnormals, where the far tail ends up
    # (torch's vectorised binary32 erf is itself a rational-exponential form good to about 1e-6: in binary32 the comparison
    # with torch is that loose, the one with the normal distribution below is the tight one)
    slack = 2.0**-19 if dt == torch.float32 else 2.0**-22
    assert (np.abs(got - w) <= ulp * np.abs(w) + slack * np.abs(xf) + tiny).all()
    # left of -2 the sum 1 + erf keeps few bits of the erf (torch's and the C library's differ in the last one), and
    # the result is below 0.05 in magnitude: there a fifth of the 16-bit values may sit one unit apart; elsewhere none
    if dt != torch.float32:
        assert (got != w)[xf > -2].mean() < 1e-3 and (got != w).mean() < 0.1
    exact = xf.astype(np.float64) * ndtr(xf.astype(np.float64))
    assert (np.abs(got - exact) <= ulp * np.abs(exact) + 2.0**-21 * np.abs(xf) + tiny + 1e-30).all()
    assert got[0, 4] == 20.0 and got[0, 5] == 0.0 and got[0, 0] == 0.0
    # and it is not the tanh form: the two differ by up to 5e-4 around |x| = 2, which binary32 resolves
    if dt == torch.float32:
        tanh_form = O.to_f32(O.prologue(xa, code, O.PRO_GELU_TANH), code)
        assert np.abs(got - tanh_form).max() > 1e-4


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_rms_norm_agrees_with_torch(dt):
    """rms_norm(x, w, eps) as torch computes it on 16-bit tensors (binary32, one rounding), then the modulation's
    operations.  The oracle takes the row's sum of squares in double, torch in binary32 in its own order: the
    normalised value may land on the other side of a rounding boundary, rarely.  Also pinned: the closed form on rows
    of +-c (rms = c, so y = +-w to the rounding of 1 / sqrt(1 + eps / c^2) = 1), the modulation half against the
    modulation prologue applied to the oracle's own normalised tensor, and each optional operand left out."""
    g = torch.Generator().manual_seed(42)
    M, K, eps = 48, 768, 1e-6
    x = (torch.randn(M, K, generator=g) * 2 + 0.3).to(dt)
    x[:, 5] *= 30
    w = (torch.randn(K, generator=g) * 0.2 + 1).to(dt)
    s = (torch.randn(2, K, generator=g) * 0.3).to(dt)
    t = (torch.randn(2, K, generator=g) * 0.2).to(dt)
    xa, code = O.from_torch(x)
    ulp = {torch.bfloat16: 2.0**-7, torch.float16: 2.0**-10}[dt]
    for weight in (w, None):
        want = torch.nn.functional.rms_norm(x, (K,), weight, eps)
        got = O.to_f32(O.rms_norm(xa, code, eps, None if weight is None else O.from_torch(weight)[0]), code)
        wn = want.float().numpy()
        assert (np.abs(got - wn) <= ulp * np.abs(wn) + 1e-30).all()
        assert (got != wn).mean() < 5e-3
    # the modulation half: the same three roundings as the modulation prologue on the normalised tensor
    y = O.rms_norm(xa, code, eps, O.from_torch(w)[0])
    both = O.rms_norm(xa, code, eps, O.from_torch(w)[0], O.from_torch(s)[0], O.from_torch(t)[0], rows_per_vec=M // 2)
    assert np.array_equal(both, O.prologue(y, code, O.PRO_MODULATE, O.from_torch(s)[0], O.from_torch(t)[0], rows_per_vec=M // 2))
    zero = torch.zeros(2, K).to(dt)
    only_s = O.rms_norm(xa, code, eps, O.from_torch(w)[0], O.from_torch(s)[0], None, rows_per_vec=M // 2)
    assert np.array_equal(only_s, O.prologue(y, code, O.PRO_MODULATE, O.from_torch(s)[0], O.from_torch(zero)[0], rows_per_vec=M // 2))
    only_t = O.rms_norm(xa, code, eps, O.from_torch(w)[0], None, O.from_torch(t)[0], rows_per_vec=M // 2)
    assert np.array_equal(only_t, O.prologue(y, code, O.PRO_MODULATE, O.from_torch(zero)[0], O.from_torch(t)[0], rows_per_vec=M // 2))
    # against torch end to end (z-image's modulate(norm(x), scale) and ltx's rms_norm(x) * (1 + scale) + shift)
    want = torch.nn.functional.rms_norm(x, (K,), w, eps).view(2, M // 2, K) * (1 + s[:, None])
    wn = want.reshape(M, K).float().numpy()
    got = O.to_f32(only_s, code)
    assert (np.abs(got - wn) <= 2 * ulp * np.abs(wn) + 1e-30).all() and (got != wn).mean() < 1e-2
    # closed form: rows of +-4 have rms 4 exactly, y = +-1 * w
    pm = torch.full((4, 256), 4.0)
    pm[:, ::2] = -4.0
    wv = (torch.randn(256, generator=g) * 0.5 + 1).to(dt)
    got2 = O.to_torch(O.rms_norm(O.from_torch(pm.to(dt))[0], code, 1e-6, O.from_torch(wv)[0]), code)
    assert torch.equal(got2.view(torch.int16), (torch.sign(pm).to(dt) * wv).view(torch.int16))
    # a row of zeros stays zero (rstd = 1 / sqrt(eps) is finite)
    got3 = O.to_f32(O.rms_norm(O.from_torch(torch.zeros(1, 64).to(dt))[0], code, 1e-6, O.from_torch(wv[:64].contiguous())[0]), code)
    assert (got3 == 0).all()


@pytest.mark.parametrize("tdt", [torch.bfloat16, torch.float16, torch.float32])
def test_gate_residual_equals_torch_ops(tdt):
    """x + gate * y on tensors of one dtype: two elementwise torch operations, each rounded to the dtype; with the gate
    one vector per group of rows (one per image of a batch), with the gate alone and with the residual alone."""
    g = torch.Generator().manual_seed(51)
    y = (torch.randn(3, 8, 96, generator=g) * 3).to(tdt)
    gate = torch.randn(3, 1, 96, generator=g).to(tdt)
    res = (torch.randn(3, 8, 96, generator=g) * 2).to(tdt)
    code = O.from_torch(y)[1]
    ya, ga, ra = O.from_torch(y.reshape(24, 96))[0], O.from_torch(gate.reshape(3, 96))[0], O.from_torch(res.reshape(24, 96))[0]
    for want, kw in ((res + gate * y, dict(gate=ga, residual=ra, rows_per_gate=8)), (gate * y, dict(gate=ga, rows_per_gate=8)),
                     (res + y, dict(residual=ra))):
        got = O.gate_residual(ya, code, **kw)
        assert np.array_equal(got, O.from_torch(want.reshape(24, 96))[0])
