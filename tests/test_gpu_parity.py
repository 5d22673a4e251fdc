"""Parity of the HIP library with the CPU oracle on identical seeded inputs, through the C ABI.

Bars: int8 activations, their scales, int32 accumulators and merged int8 weights are
bit-exact; bf16/fp16 outputs of the W8A8 linear are bit-exact as well, in BOTH epilogue
orders (the oracle restates each order operation for operation); the small-batch W8A16
path, whose reference is a BLAS product of unspecified order, is held per element to
|y - y_ref| <= ulp(dtype) |y_ref| + K 2^-24 sum_k |x||w|   (ulp = 2^-8 bf16, 2^-11 fp16, 2^-23 fp32).
"""
import numpy as np
import pytest
import torch

import oracle as O
from bench import make_config

pytestmark = pytest.mark.gpu

G = torch.Generator().manual_seed(4321)


def acts(M, K, dt=torch.bfloat16, frac=0.01, mul=20.0):
    x = torch.randn(M, K, generator=G)
    if K > 8:
        x[:, torch.randperm(K, generator=G)[: max(1, int(K * frac))]] *= mul
    return x.to(dt)


def i8(*shape):
    return torch.randint(-128, 128, shape, dtype=torch.int8, generator=G)


def bits(t):
    return O.from_torch(t.cpu())[0]


def _raw16(t):
    return t.contiguous().view(torch.int16)


# ------------------------------------------------------------------ quantiser (a1, a3, a4)
QUANT_CASES = [
    # M, K, dtype, rotate
    (64, 3072, torch.bfloat16, False), (64, 3072, torch.bfloat16, True), (33, 3840, torch.bfloat16, True),
    (17, 12288, torch.bfloat16, False), (9, 12288, torch.bfloat16, True), (5, 18432, torch.bfloat16, False),
    (16, 1000, torch.bfloat16, False), (7, 1001, torch.bfloat16, False), (3, 77, torch.float16, False), (4, 1, torch.float32, False),
    (8, 3072, torch.float32, True), (8, 3072, torch.float16, True), (5, 24576, torch.float32, True),
    (6, 40960, torch.float32, True), (2, 70000, torch.bfloat16, False), (3, 66048, torch.bfloat16, True),
    (4, 384, torch.bfloat16, True), (1, 128, torch.float32, True), (257, 512, torch.float16, False), (1, 8, torch.bfloat16, False),
    # row counts just beyond a multiple of 1024: the rows beyond it are quantised as half rows by two waves each
    (4608, 3072, torch.bfloat16, True), (1536, 1024, torch.float16, True), (1028, 2048, torch.bfloat16, True), (2052, 4096, torch.bfloat16, True),
]


@pytest.mark.parametrize("M,K,dt,rot", QUANT_CASES)
def test_quant_rowwise_bit_exact(L, dev, M, K, dt, rot):
    x = acts(M, K, dt)
    if M > 2:
        x[1] = 0                                   # an all-zero row: scale clamps to 1e-30
    xa, code = O.from_torch(x)
    qo, so = O.quant_rowwise(xa, code, 128 if rot else 0)
    q, s = L.quant_rowwise(x.to(dev), rotate=rot)
    assert np.array_equal(q.cpu().numpy(), qo)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_quant_rowwise_every_possible_row_maximum(L, dev, dt):
    """The 16-bit quantiser takes its scale and the reciprocal of the scale without the division sequence; the row
    maximum is a value of the dtype, so every case there is gets a row of its own: each finite positive pattern as
    the maximum of a row of 128 values (fractions of it, both signs, the maximum at a varying position), and scales
    and int8 are the oracle's bit for bit."""
    if dt == torch.bfloat16:
        amax = (torch.arange(1, 0x7F80, dtype=torch.int32) << 16).view(torch.float32)
    else:
        amax = torch.arange(1, 0x7C00, dtype=torch.int16).view(torch.float16).float()
    M, K = amax.numel(), 128
    frac = torch.rand(M, K, generator=G) * 2 - 1
    x = (frac * amax[:, None]).to(dt)
    x[torch.arange(M), torch.arange(M) % K] = amax.to(dt) * torch.where(torch.arange(M) % 2 == 0, 1.0, -1.0).to(dt)
    xa, code = O.from_torch(x)
    qo, so = O.quant_rowwise(xa, code, 0)
    q, s = L.quant_rowwise(x.to(dev))
    bad = (s.cpu().numpy().view(np.uint32) != so.view(np.uint32)).reshape(-1)
    assert not bad.any(), f"{bad.sum()} scales differ, first for a row maximum of {amax[int(bad.argmax())].item()!r}"
    assert np.array_equal(q.cpu().numpy(), qo)


@pytest.mark.parametrize("rot,dt,K", [(False, torch.bfloat16, 3072), (True, torch.bfloat16, 3072), (True, torch.float16, 1024),
                                       (False, torch.bfloat16, 12288), (False, torch.float16, 200), (False, torch.float32, 256)])
def test_quant_rowwise_grouped_equals_separate_calls_and_the_oracle(L, dev, rot, dt, K):
    """Several row blocks in one launch (i8f_quant_rowwise_grouped): every group's int8 and scales are the oracle's and
    those of a launch of its own, for row counts that do and do not fill a workgroup, an empty group, a strided group,
    and the shapes (binary32, odd widths) that the entry point launches group by group."""
    Ms = [130, 0, 33, 4, 257]
    xs = [acts(M, K, dt) for M in Ms]
    wide = acts(19, K + 16, dt)
    dev_xs = [x.to(dev) for x in xs] + [wide.to(dev)[:, :K]]
    xs.append(wide[:, :K].contiguous())
    got = L.quant_rowwise_grouped(dev_xs, rotate=rot)
    assert len(got) == len(xs)
    for x, xd, (q, s) in zip(xs, dev_xs, got):
        if x.shape[0] == 0:
            assert q.shape == (0, K) and s.shape == (0, 1)
            continue
        xa, code = O.from_torch(x)
        qo, so = O.quant_rowwise(xa, code, 128 if rot else 0)
        assert np.array_equal(q.cpu().numpy(), qo)
        assert np.array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))
        q1, s1 = L.quant_rowwise(xd, rotate=rot)
        assert torch.equal(q1, q) and torch.equal(s1, s)
    with pytest.raises(ValueError):
        L.quant_rowwise_grouped([dev_xs[0], dev_xs[0][:, : K // 2]])
    # groups whose rows fill their workgroups (and, for the model widths, whose K fills every lane): the instantiation
    # without bounds tests
    full = [acts(M, K, dt) for M in (128, 64, 4)]
    for x, (q, s) in zip(full, L.quant_rowwise_grouped([x.to(dev) for x in full], rotate=rot)):
        xa, code = O.from_torch(x)
        qo, so = O.quant_rowwise(xa, code, 128 if rot else 0)
        assert np.array_equal(q.cpu().numpy(), qo) and np.array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))


PROLOGUE_CASES = [
    # M, K, dtype, rotate, vectors
    (64, 3072, torch.bfloat16, False, 1), (48, 3072, torch.bfloat16, True, 2), (12, 12288, torch.bfloat16, False, 3),
    (10, 1000, torch.bfloat16, False, 2), (6, 384, torch.float16, True, 1), (5, 77, torch.float32, False, 1), (8, 256, torch.float32, True, 4),
]


@pytest.mark.parametrize("M,K,dt,rot,V", PROLOGUE_CASES)
def test_quant_rowwise_modulate_prologue_bit_exact(L, dev, M, K, dt, rot, V):
    """adaLN modulation applied inside the quantiser == torch's three eager operations, then the quantiser."""
    x = acts(M, K, dt)
    sc, sh = (torch.randn(V, K, generator=G) * 0.3).to(dt), torch.randn(V, K, generator=G).to(dt)
    xa, code = O.from_torch(x)
    mod = O.prologue(xa, code, O.PRO_MODULATE, O.from_torch(sc)[0], O.from_torch(sh)[0], rows_per_vec=M // V)
    qo, so = O.quant_rowwise(mod, code, 128 if rot else 0)
    q, s = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_MODULATE, mod_scale=sc.to(dev), mod_shift=sh.to(dev))
    assert np.array_equal(q.cpu().numpy(), qo)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))
    # and against torch on the device followed by the plain quantiser
    xd = x.to(dev)
    t = ((1 + sc.to(dev)[:, None, :]) * xd.view(V, M // V, K) + sh.to(dev)[:, None, :]).reshape(M, K)
    q2, s2 = L.quant_rowwise(t, rotate=rot)
    assert torch.equal(q, q2) and torch.equal(s, s2)
    if dt != torch.float32:   # the one-kernel spelling, torch.addcmul(shift, x, 1 + scale): product and sum rounded once
        modf = O.prologue(xa, code, O.PRO_MODULATE_FUSED, O.from_torch(sc)[0], O.from_torch(sh)[0], rows_per_vec=M // V)
        qo, so = O.quant_rowwise(modf, code, 128 if rot else 0)
        q, s = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_MODULATE_FUSED, mod_scale=sc.to(dev), mod_shift=sh.to(dev))
        assert np.array_equal(q.cpu().numpy(), qo) and np.array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))
        t = torch.addcmul(sh.to(dev)[:, None, :], xd.view(V, M // V, K), 1 + sc.to(dev)[:, None, :]).reshape(M, K)
        q2, s2 = L.quant_rowwise(t, rotate=rot)
        assert torch.equal(q, q2) and torch.equal(s, s2)
    else:
        with pytest.raises(ValueError):
            L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_MODULATE_FUSED, mod_scale=sc.to(dev), mod_shift=sh.to(dev))


@pytest.mark.parametrize("M,K,dt,rot,V", PROLOGUE_CASES)
def test_quant_rowwise_gelu_prologue_within_tolerance(L, dev, M, K, dt, rot, V):
    """tanh-GELU inside the quantiser against the oracle (C tanhf) and against torch's gelu on the device followed
    by the plain quantiser.  The activations agree to the last bits of binary32 before they are rounded to the
    dtype, so: scales equal or one ulp of the dtype apart, int8 values at most 1 apart, at least 99.9 % equal
    (un-rotated; a rotation spreads a one-ulp difference over its 128-block: 99 %)."""
    x = (acts(M, K, dt).float() * 0.5).to(dt)
    xa, code = O.from_torch(x)
    qo, so = O.quant_rowwise(O.prologue(xa, code, O.PRO_GELU_TANH), code, 128 if rot else 0)
    q, s = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_GELU_TANH)
    q2, s2 = L.quant_rowwise(torch.nn.functional.gelu(x.to(dev), approximate="tanh"), rotate=rot)
    ulp = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11, torch.float32: 2.0**-22}[dt]
    for qr, sr in ((qo, so), (q2.cpu().numpy(), s2.cpu().numpy())):
        d = np.abs(q.cpu().numpy().astype(np.int32) - qr.astype(np.int32))
        assert d.max() <= 1 and (d != 0).mean() <= (1e-2 if rot else 1e-3)
        assert (np.abs(s.cpu().numpy() - sr) <= 2 * ulp * np.abs(sr)).all()


@pytest.mark.parametrize("M,K,dt,rot,V", PROLOGUE_CASES)
def test_quant_rowwise_silu_gate_prologue_within_tolerance(L, dev, M, K, dt, rot, V):
    """silu(a) * b inside the quantiser (the gated activation in front of a SwiGLU down projection) against the oracle
    (C expf) and against torch's silu and mul on the device followed by the plain quantiser; same bar as the GELU
    prologue: scales within 2 ulp of the dtype, int8 at most 1 apart, at least 99.9 % equal (99 % with rotation)."""
    a = (acts(M, K, dt).float() * 0.5).to(dt)
    b = torch.randn(M, K, generator=G).to(dt)
    aa, code = O.from_torch(a)
    qo, so = O.quant_rowwise(O.prologue(aa, code, O.PRO_SILU_GATE, O.from_torch(b)[0], rows_per_vec=1), code, 128 if rot else 0)
    q, s = L.quant_rowwise(a.to(dev), rotate=rot, prologue=L.PRO_SILU_GATE, mod_scale=b.to(dev))
    q2, s2 = L.quant_rowwise(torch.nn.functional.silu(a.to(dev)) * b.to(dev), rotate=rot)
    ulp = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11, torch.float32: 2.0**-22}[dt]
    for qr, sr in ((qo, so), (q2.cpu().numpy(), s2.cpu().numpy())):
        d = np.abs(q.cpu().numpy().astype(np.int32) - qr.astype(np.int32))
        assert d.max() <= 1 and (d != 0).mean() <= (1e-2 if rot else 1e-3)
        assert (np.abs(s.cpu().numpy() - sr) <= 2 * ulp * np.abs(sr)).all()
    if M % V == 0 and V > 1:   # one gate row per group of rows (the vector form)
        bv = torch.randn(V, K, generator=G).to(dt)
        qa, sa = L.quant_rowwise(a.to(dev), rotate=rot, prologue=L.PRO_SILU_GATE, mod_scale=bv.to(dev))
        qb, sb = L.quant_rowwise(a.to(dev), rotate=rot, prologue=L.PRO_SILU_GATE, mod_scale=bv.repeat_interleave(M // V, 0).to(dev))
        assert torch.equal(qa, qb) and torch.equal(sa, sb)


@pytest.mark.parametrize("M,K,dt,rot,V,eps", [
    (64, 3072, torch.bfloat16, False, 1, 1e-6), (48, 3072, torch.bfloat16, True, 2, 1e-6), (33, 4096, torch.float16, False, 3, 1e-5),
    (10, 1008, torch.bfloat16, False, 2, 1e-6), (6, 384, torch.float16, True, 1, 1e-5), (5, 16, torch.bfloat16, False, 1, 1e-6),
    (4608, 3072, torch.bfloat16, False, 1, 1e-6), (40, 5120, torch.bfloat16, False, 2, 1e-6), (9, 16384, torch.float16, True, 1, 1e-5),
    (6, 4112, torch.bfloat16, False, 1, 1e-6),
])
def test_quant_rowwise_norm_modulate_prologue_within_tolerance(L, dev, M, K, dt, rot, V, eps):
    """LayerNorm (no affine) and the adaLN modulation inside the quantiser (i8f_quant_rowwise_norm_modulate) against the
    oracle (row sums in double) and against torch's layer_norm and three eager operations on the device followed by
    the plain quantiser.  The kernel takes the row's sums in binary32 in its own order, so a normalised value may land
    on the other side of a rounding boundary of the dtype: scales within 2 ulp of the dtype, int8 at most 1 apart, at
    least 99.5 % equal (98 % with rotation, which spreads every such step over 128 values)."""
    rows = M - M % V
    x = (acts(rows, K, dt).float() * 3 + 0.25).to(dt)
    s = (torch.randn(V, K, generator=G) * 0.3).to(dt)
    t = (torch.randn(V, K, generator=G) * 0.2).to(dt)
    xa, code = O.from_torch(x)
    z = O.norm_modulate(xa, code, eps, O.from_torch(s)[0], O.from_torch(t)[0], rows_per_vec=rows // V)
    qo, so = O.quant_rowwise(z, code, 128 if rot else 0)
    q, sc = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_NORM_MODULATE, mod_scale=s.to(dev), mod_shift=t.to(dev), eps=eps)
    xd = x.to(dev).reshape(V, rows // V, K)
    zt = ((1 + s.to(dev)[:, None]) * torch.nn.functional.layer_norm(xd, (K,), eps=eps) + t.to(dev)[:, None]).reshape(rows, K)
    q2, s2 = L.quant_rowwise(zt, rotate=rot)
    ulp = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}[dt]
    for qr, sr in ((qo, so), (q2.cpu().numpy(), s2.cpu().numpy())):
        d = np.abs(q.cpu().numpy().astype(np.int32) - qr.astype(np.int32))
        assert d.max() <= 1 and (d != 0).mean() <= (2e-2 if rot else 5e-3)
        assert (np.abs(sc.cpu().numpy() - sr) <= 2 * ulp * np.abs(sr)).all()
    again = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_NORM_MODULATE, mod_scale=s.to(dev), mod_shift=t.to(dev), eps=eps)
    assert torch.equal(again[0], q) and torch.equal(again[1], sc)     # fixed order of the sums: launches agree bit for bit
    # the modulation as torch.addcmul (one rounding for product and sum): same bar against the oracle's fused form and torch's
    zf = O.norm_modulate(xa, code, eps, O.from_torch(s)[0], O.from_torch(t)[0], rows_per_vec=rows // V, fused=True)
    qo, so = O.quant_rowwise(zf, code, 128 if rot else 0)
    q, sc = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_NORM_MODULATE, mod_scale=s.to(dev), mod_shift=t.to(dev), eps=eps, fused_add=True)
    zt = torch.addcmul(t.to(dev)[:, None], torch.nn.functional.layer_norm(xd, (K,), eps=eps), 1 + s.to(dev)[:, None]).reshape(rows, K)
    q2, s2 = L.quant_rowwise(zt, rotate=rot)
    for qr, sr in ((qo, so), (q2.cpu().numpy(), s2.cpu().numpy())):
        d = np.abs(q.cpu().numpy().astype(np.int32) - qr.astype(np.int32))
        assert d.max() <= 1 and (d != 0).mean() <= (2e-2 if rot else 5e-3)
        assert (np.abs(sc.cpu().numpy() - sr) <= 2 * ulp * np.abs(sr)).all()


@pytest.mark.parametrize("M,K,dt,rot,V", PROLOGUE_CASES)
def test_quant_rowwise_gelu_erf_prologue_within_tolerance(L, dev, M, K, dt, rot, V):
    """GELU in its exact form inside the quantiser (x Phi(x), the complementary error function by a rational-exponential
    form good to 1.5e-7 of Phi) against the oracle (C erff) and against torch's gelu on the device followed by the plain
    quantiser: the bar of the tanh form -- scales within 2 ulp of the dtype, int8 at most 1 apart, at least 99.9 % equal
    (99 % with rotation); in binary32, where nothing hides the approximation, int8 still at most 1 apart."""
    x = (acts(M, K, dt).float() * 0.5).to(dt)
    xa, code = O.from_torch(x)
    qo, so = O.quant_rowwise(O.prologue(xa, code, O.PRO_GELU_ERF), code, 128 if rot else 0)
    q, s = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_GELU_ERF)
    q2, s2 = L.quant_rowwise(torch.nn.functional.gelu(x.to(dev)), rotate=rot)
    ulp = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11, torch.float32: 2.0**-20}[dt]
    for qr, sr in ((qo, so), (q2.cpu().numpy(), s2.cpu().numpy())):
        d = np.abs(q.cpu().numpy().astype(np.int32) - qr.astype(np.int32))
        assert d.max() <= 1 and (d != 0).mean() <= (1e-2 if rot else 1e-3)
        assert (np.abs(s.cpu().numpy() - sr) <= 2 * ulp * np.abs(sr)).all()
    qt, _ = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_GELU_TANH)
    if M * K > 10000 and not rot:
        assert not torch.equal(q, qt)     # the two forms differ by up to 5e-4: visible in int8 on enough elements


@pytest.mark.parametrize("M,K,dt,rot,V,eps,parts", [
    (64, 3072, torch.bfloat16, False, 1, 1e-6, "wst"), (48, 3072, torch.bfloat16, True, 2, 1e-6, "ws"), (33, 4096, torch.float16, False, 3, 1e-5, "w"),
    (10, 1008, torch.bfloat16, False, 2, 1e-6, "st"), (6, 384, torch.float16, True, 1, 1e-5, ""), (5, 16, torch.bfloat16, False, 1, 1e-6, "wt"),
    (4608, 3840, torch.bfloat16, False, 1, 1e-5, "ws"), (40, 5120, torch.bfloat16, False, 2, 1e-6, "wst"), (9, 16384, torch.float16, True, 1, 1e-5, "ws"),
    (6, 4112, torch.bfloat16, False, 1, 1e-6, "w"),
])
def test_quant_rowwise_rms_norm_prologue_within_tolerance(L, dev, M, K, dt, rot, V, eps, parts):
    """RMSNorm with its weight and the modulation behind it inside the quantiser (i8f_quant_rowwise_rms_norm; each of
    weight, scale and shift present or not) against the oracle (row sum in double) and against torch's rms_norm and
    eager operations on the device followed by the plain quantiser.  The bar of the LayerNorm form: scales within 2 ulp
    of the dtype, int8 at most 1 apart, at least 99.5 % equal (98 % with rotation)."""
    rows = M - M % V
    x = (acts(rows, K, dt).float() * 3 + 0.25).to(dt)
    w = (torch.randn(K, generator=G) * 0.2 + 1).to(dt) if "w" in parts else None
    s = (torch.randn(V, K, generator=G) * 0.3).to(dt) if "s" in parts else None
    t = (torch.randn(V, K, generator=G) * 0.2).to(dt) if "t" in parts else None
    xa, code = O.from_torch(x)
    z = O.rms_norm(xa, code, eps, *(None if v is None else O.from_torch(v)[0] for v in (w, s, t)), rows_per_vec=rows // V)
    qo, so = O.quant_rowwise(z, code, 128 if rot else 0)
    d = lambda v: None if v is None else v.to(dev)
    q, sc = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_RMS_NORM, norm_weight=d(w), mod_scale=d(s), mod_shift=d(t), eps=eps)
    zt = torch.nn.functional.rms_norm(x.to(dev), (K,), d(w), eps).reshape(V, rows // V, K)
    if s is not None:
        zt = zt * (1 + d(s)[:, None])
    if t is not None:
        zt = zt + d(t)[:, None]
    q2, s2 = L.quant_rowwise(zt.reshape(rows, K), rotate=rot)
    ulp = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}[dt]
    for qr, sr in ((qo, so), (q2.cpu().numpy(), s2.cpu().numpy())):
        df = np.abs(q.cpu().numpy().astype(np.int32) - qr.astype(np.int32))
        assert df.max() <= 1 and (df != 0).mean() <= (2e-2 if rot else 5e-3)
        assert (np.abs(sc.cpu().numpy() - sr) <= 2 * ulp * np.abs(sr)).all()
    again = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_RMS_NORM, norm_weight=d(w), mod_scale=d(s), mod_shift=d(t), eps=eps)
    assert torch.equal(again[0], q) and torch.equal(again[1], sc)
    if s is not None and t is not None:   # with both: the fused spelling, torch.addcmul(shift, norm(x), 1 + scale)
        zf = O.rms_norm(xa, code, eps, *(None if v is None else O.from_torch(v)[0] for v in (w, s, t)), rows_per_vec=rows // V, fused=True)
        qo, so = O.quant_rowwise(zf, code, 128 if rot else 0)
        q, sc = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_RMS_NORM, norm_weight=d(w), mod_scale=d(s), mod_shift=d(t), eps=eps, fused_add=True)
        zt = torch.addcmul(d(t)[:, None], torch.nn.functional.rms_norm(x.to(dev), (K,), d(w), eps).reshape(V, rows // V, K), 1 + d(s)[:, None])
        q2, s2 = L.quant_rowwise(zt.reshape(rows, K), rotate=rot)
        for qr, sr in ((qo, so), (q2.cpu().numpy(), s2.cpu().numpy())):
            df = np.abs(q.cpu().numpy().astype(np.int32) - qr.astype(np.int32))
            assert df.max() <= 1 and (df != 0).mean() <= (2e-2 if rot else 5e-3)
            assert (np.abs(sc.cpu().numpy() - sr) <= 2 * ulp * np.abs(sr)).all()
    if parts == "":      # nothing but the normalisation: invariant under a positive power-of-two factor (eps scaled with it)
        q4, s4 = L.quant_rowwise((x.float() * 4).to(dt).to(dev), rotate=rot, prologue=L.PRO_RMS_NORM, eps=eps * 16)
        assert torch.equal(q4, q) and torch.equal(s4, sc)


def test_quant_rowwise_norm_modulate_refuses_rows_it_does_not_take(L, dev):
    s = torch.zeros(1, 16400, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        L.quant_rowwise(torch.zeros(4, 16400, dtype=torch.bfloat16, device=dev), prologue=L.PRO_NORM_MODULATE, mod_scale=s, mod_shift=s)
    with pytest.raises(ValueError):
        L.quant_rowwise(torch.zeros(4, 256, device=dev), prologue=L.PRO_NORM_MODULATE, mod_scale=s[:, :256].float(), mod_shift=s[:, :256].float())
    with pytest.raises(ValueError):
        L.quant_rowwise(torch.zeros(4, 16400, dtype=torch.bfloat16, device=dev), prologue=L.PRO_RMS_NORM)
    with pytest.raises(ValueError):
        L.quant_rowwise(torch.zeros(4, 256, dtype=torch.bfloat16, device=dev), prologue=L.PRO_RMS_NORM, norm_weight=s[0, :128])


@pytest.mark.parametrize("M,Ka,Kb,dt,rot", [
    (64, 3072, 12288, torch.bfloat16, False), (33, 3072, 12288, torch.bfloat16, True), (10, 1024, 2048, torch.float16, False),
    (7, 16, 48, torch.bfloat16, False), (12, 384, 128, torch.float16, True), (4608, 3072, 12288, torch.bfloat16, False),
    (9, 3200, 800, torch.bfloat16, False),
])
def test_quant_rowwise_concat_gelu_prologue(L, dev, M, Ka, Kb, dt, rot):
    """cat(a, gelu(b)) along the row inside the quantiser (i8f_quant_rowwise_concat_gelu; the input of linear2 of a
    single-stream block) against the oracle's GELU on b, numpy's concatenation and the oracle's quantiser, and against
    torch's gelu and cat on the device followed by the plain quantiser: the bar of the GELU prologue (scales within 2 ulp
    of the dtype, int8 at most 1 apart, at least 99.9 % equal, 99 % with rotation).  The columns that come from a are
    exact whenever the row's scale is; with an empty-handed GELU (b = 0) the whole result is the plain quantiser's."""
    a = acts(M, Ka, dt)
    b = (acts(M, Kb, dt).float() * 0.5).to(dt)
    aa, code = O.from_torch(a)
    z = np.concatenate([aa, O.prologue(O.from_torch(b)[0], code, O.PRO_GELU_TANH)], axis=1)
    qo, so = O.quant_rowwise(z, code, 128 if rot else 0)
    wide_a, wide_b = acts(M, Ka + 32, dt), None
    q, s = L.quant_rowwise(a.to(dev), rotate=rot, prologue=L.PRO_CONCAT_GELU, mod_scale=b.to(dev))
    assert q.shape == (M, Ka + Kb)
    zt = torch.cat((a.to(dev), torch.nn.functional.gelu(b.to(dev), approximate="tanh")), -1)
    q2, s2 = L.quant_rowwise(zt, rotate=rot)
    ulp = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}[dt]
    for qr, sr in ((qo, so), (q2.cpu().numpy(), s2.cpu().numpy())):
        d = np.abs(q.cpu().numpy().astype(np.int32) - qr.astype(np.int32))
        assert d.max() <= 1 and (d != 0).mean() <= (1e-2 if rot else 1e-3)
        assert (np.abs(s.cpu().numpy() - sr) <= 2 * ulp * np.abs(sr)).all()
    zero_b = torch.zeros(M, Kb, dtype=dt, device=dev)                       # gelu(0) = 0: nothing toleranced is left
    q0, s0 = L.quant_rowwise(a.to(dev), rotate=rot, prologue=L.PRO_CONCAT_GELU, mod_scale=zero_b)
    q1, s1 = L.quant_rowwise(torch.cat((a.to(dev), zero_b), -1), rotate=rot)
    assert torch.equal(q0, q1) and torch.equal(s0, s1)
    a_str = wide_a.to(dev)[:, :Ka]                                          # a row stride larger than the width
    q3, s3 = L.quant_rowwise(a_str, rotate=rot, prologue=L.PRO_CONCAT_GELU, mod_scale=b.to(dev))
    q4, s4 = L.quant_rowwise(a_str.contiguous(), rotate=rot, prologue=L.PRO_CONCAT_GELU, mod_scale=b.to(dev))
    assert torch.equal(q3, q4) and torch.equal(s3, s4)


TENSORWISE_CASES = [
    # shape, dtype
    ((3072, 3072), torch.bfloat16), ((3072, 3072), torch.float32), ((1, 1), torch.float32), ((7,), torch.float16),
    ((5, 1001), torch.bfloat16), ((16 * 1024 + 3,), torch.float32), ((1024 * 16 * 1024 + 40,), torch.bfloat16),
    ((257, 4099), torch.float16), ((12288, 3072), torch.float32),
]


@pytest.mark.parametrize("shape,dt", TENSORWISE_CASES)
def test_quant_tensorwise_bit_exact(L, dev, shape, dt):
    """quantize_int8_tensorwise through i8f_quant_tensorwise: one slice, ragged slices, more slices than
    partial slots; int8 and the scale bit-exact against the oracle."""
    x = (torch.randn(*shape, generator=G) * 0.02).to(dt)
    xa, code = O.from_torch(x)
    qo, so = O.quant_tensorwise(xa, code)
    q, s = L.quant_tensorwise(x.to(dev))
    assert q.shape == x.shape and s.shape == ()
    assert np.array_equal(q.cpu().numpy(), qo.reshape(x.shape))
    assert np.array_equal(s.cpu().numpy().reshape(1).view(np.uint32), np.asarray(so).reshape(1).view(np.uint32))


def test_quant_tensorwise_edge_cases(L, dev):
    z = torch.zeros(4, 300, dtype=torch.bfloat16, device=dev)          # all zero: scale clamps to 1e-30
    q, s = L.quant_tensorwise(z)
    assert not q.any() and s.item() == np.float32(1e-30)
    e = torch.empty(0, dtype=torch.float32, device=dev)                # empty: scale only
    q, s = L.quant_tensorwise(e)
    assert q.numel() == 0 and s.item() == np.float32(1e-30)
    base = torch.randn(70001, generator=G).to(dev)                     # misaligned views take the scalar kernels
    for view in (base[1:], base[3:40000]):
        qo, so = O.quant_tensorwise(view.cpu().numpy().copy(), O.F32)
        q, s = L.quant_tensorwise(view)
        assert np.array_equal(q.cpu().numpy(), qo) and s.item() == so[0].item()


def test_quant_rowwise_strided_and_misaligned_views(L, dev):
    big = acts(40, 1100).to(dev)
    for view in (big[:, :1024], big[:, 3:1027], big[::2, 8:520], big[5:6, 1:130]):
        xa, code = O.from_torch(view.cpu())
        for rot in (False, True) if view.shape[1] % 128 == 0 else (False,):
            qo, so = O.quant_rowwise(xa, code, 128 if rot else 0)
            q, s = L.quant_rowwise(view, rotate=rot)
            assert np.array_equal(q.cpu().numpy(), qo) and np.array_equal(s.cpu().numpy(), so)


def test_quant_rowwise_more_than_2_pow_31_elements(L, dev):
    M, K = 131200, 16384                         # 2.15e9 elements: offsets need 64 bits
    x = torch.randn(M, K, device=dev, dtype=torch.bfloat16)
    rows = torch.cat([torch.arange(0, 8), torch.arange(131072 - 8, 131072 + 8), torch.arange(M - 8, M)])
    for rot in (False, True):
        q, s = L.quant_rowwise(x, rotate=rot)
        xa, code = O.from_torch(x[rows].cpu())
        qo, so = O.quant_rowwise(xa, code, 128 if rot else 0)
        assert np.array_equal(q[rows].cpu().numpy(), qo) and np.array_equal(s[rows].cpu().numpy(), so)
        del q, s


def test_quant_rowwise_empty(L, dev):
    q, s = L.quant_rowwise(torch.empty(0, 256, dtype=torch.bfloat16, device=dev))
    assert q.shape == (0, 256) and s.shape == (0, 1)
    q, s = L.quant_rowwise(torch.empty(5, 0, dtype=torch.bfloat16, device=dev))
    assert q.shape == (5, 0) and (s.cpu() == 1e-30).all()


def test_quant_extreme_magnitudes(L, dev):
    x = torch.tensor([[1e-38, -2e-38, 0.0, 5e-39], [3e38, -1e38, 1.0, 0.0], [1e-45, 0, 0, 0], [6e4, -6.5e4, 1e-3, 7.0]],
                     dtype=torch.float32).repeat(1, 32)
    for dt in (torch.float32, torch.bfloat16):
        xa, code = O.from_torch(x.to(dt))
        qo, so = O.quant_rowwise(xa, code)
        q, s = L.quant_rowwise(x.to(dt).to(dev))
        assert np.array_equal(q.cpu().numpy(), qo) and np.array_equal(s.cpu().numpy(), so)


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32])
def test_rotate128_bit_exact_and_in_place(L, dev, dt):
    x = acts(19, 640, dt, 0.02, 50.0)
    xa, code = O.from_torch(x)
    want = O.rotate(xa, code)
    xd = x.to(dev)
    assert np.array_equal(bits(L.rotate128(xd)), want)
    assert np.array_equal(bits(L.rotate128(xd[:, 128:512])), O.rotate(np.ascontiguousarray(xa[:, 128:512]), code))
    L.rotate128(xd, out=xd)
    assert np.array_equal(bits(xd), want)


def test_weight_prep_matches_oracle_for_rotated_rowwise_weights(L, dev):
    w = torch.randn(96, 3840, generator=G) * 0.02
    qo, so = O.quant_rowwise(w.numpy(), O.F32, 128)
    q, s = L.quant_rowwise(w.to(dev), rotate=True)
    assert np.array_equal(q.cpu().numpy(), qo) and np.array_equal(s.cpu().numpy(), so)


# ------------------------------------------------------------------ integer product (a5)
GEMM_CASES = [(256, 256, 64), (256, 256, 3072), (300, 520, 1040), (128, 128, 128), (100, 72, 48), (64, 64, 50),
              (1, 8, 16), (17, 3072, 3072), (1024, 768, 12288), (513, 1032, 80), (40, 24, 16), (31, 33, 35), (512, 512, 0),
              # one ragged case per tile configuration of the fast kernel: 128x128, 256x192, 256x256 (K tails included)
              (2048, 2048, 256), (2000, 2056, 200), (4100, 2056, 144), (3000, 4104, 80), (3000, 4104, 256),
              # 288x256 tiles of twelve waves (chosen where they save a round over 256 CUs), ragged in M, N and K
              (4500, 4088, 144), (4330, 4096, 256),
              # 256x288 tiles of twelve waves
              (4090, 4600, 144), (4096, 4608, 128),
              # long K, few tiles: the four-stage configurations (128x128, 128x64, 64x64, 128x96)
              (1000, 3080, 8200), (500, 3072, 8192), (200, 520, 8320), (250, 9200, 144), (256, 12288, 256),
              # 256x96 tiles, three stages (one round of them instead of two 128x128 tiles per CU)
              (500, 9200, 144), (512, 12288, 384)]


@pytest.mark.parametrize("M,N,K", GEMM_CASES)
def test_gemm_i32_bit_exact(L, dev, M, N, K):
    a, w = i8(M, K), i8(N, K)
    acc = L.gemm_i32(a.to(dev), w.to(dev))
    assert np.array_equal(acc.cpu().numpy(), O.gemm_i32(a.numpy(), w.numpy()))


def test_gemm_i32_random_shapes(L, dev):
    """40 seeded random shapes, ragged in every dimension, spread over all tile configurations."""
    rng = np.random.default_rng(20240)
    for _ in range(40):
        M = int(rng.integers(1, 2600))
        N = int(rng.integers(1, 330)) * 8 if rng.random() < 0.8 else int(rng.integers(1, 2600))
        K = int(rng.integers(1, 80)) * 16 if rng.random() < 0.8 else int(rng.integers(1, 1300))
        if rng.random() < 0.15:
            K = int(rng.integers(512, 640)) * 16            # long K: the four-stage configurations
        a, w = i8(M, K), i8(N, K)
        acc = L.gemm_i32(a.to(dev), w.to(dev))
        assert np.array_equal(acc.cpu().numpy(), O.gemm_i32(a.numpy(), w.numpy())), (M, N, K)


def test_linear_with_more_than_2_gib_of_activations(L, dev):
    """M * K >= 2^31 bytes: the launcher walks the rows in blocks; rows on both sides of the seam are checked."""
    M, N, K = 131200, 16, 16384
    a = torch.randint(-128, 128, (M, K), dtype=torch.int8, device=dev)
    w = torch.randint(-128, 128, (N, K), dtype=torch.int8, device=dev)
    xs = torch.rand(M, device=dev) * 0.01
    ws = torch.rand(N, device=dev) * 0.01
    y = L.linear_w8a8(a, xs, w, ws, None, torch.bfloat16, 0)
    acc = L.gemm_i32(a, w)
    rows = torch.cat([torch.arange(0, 40), torch.arange(131072 - 300, 131072 + 128), torch.arange(M - 40, M)])
    acc_o = O.gemm_i32(a[rows].cpu().numpy(), w.cpu().numpy())
    assert np.array_equal(acc[rows].cpu().numpy(), acc_o)
    want = O.epilogue(acc_o, xs[rows].cpu().numpy(), ws.cpu().numpy(), None, O.BF16, O.BF16)
    assert np.array_equal(bits(y[rows]), want)


def test_gemm_i32_saturating_inputs_at_largest_k(L, dev):
    K = 12288
    a = torch.full((64, K), -128, dtype=torch.int8)
    w = torch.cat([torch.full((32, K), -128, dtype=torch.int8), torch.full((32, K), 127, dtype=torch.int8)])
    acc = L.gemm_i32(a.to(dev), w.to(dev)).cpu()
    assert (acc[:, :32] == K * 16384).all() and (acc[:, 32:] == -K * 16256).all()


def test_gemm_i32_misaligned_operands_use_the_generic_kernel(L, dev):
    a, w = i8(70, 161), i8(90, 161)
    a_d, w_d = a.to(dev), w.to(dev)
    flat = torch.empty(70 * 160 + 1, dtype=torch.int8, device=dev)
    a_off = flat[1:].view(70, 160)
    a_off.copy_(a_d[:, :160])
    acc = L.gemm_i32(a_off, w_d[:, :160].contiguous())
    assert np.array_equal(acc.cpu().numpy(), O.gemm_i32(np.ascontiguousarray(a.numpy()[:, :160]), np.ascontiguousarray(w.numpy()[:, :160])))


# ------------------------------------------------------------------ fused linear (a6, a7)
LIN_CASES = [
    # M, N, K, row, bias dtype or None, out dtype, order
    (256, 256, 512, True, torch.bfloat16, torch.bfloat16, 0), (300, 520, 1040, False, None, torch.bfloat16, 0),
    (512, 768, 3072, True, torch.float16, torch.float16, 0), (512, 768, 3072, True, torch.bfloat16, torch.bfloat16, 1),
    (256, 256, 512, False, torch.bfloat16, torch.float32, 0), (100, 72, 48, True, torch.float32, torch.bfloat16, 0),
    (17, 3072, 3072, True, torch.bfloat16, torch.bfloat16, 0), (64, 50, 50, True, torch.bfloat16, torch.bfloat16, 0),
    (1030, 264, 272, False, torch.float32, torch.float16, 1), (40, 24, 16, False, None, torch.float16, 1),
    (2000, 2056, 200, True, torch.bfloat16, torch.bfloat16, 0), (4100, 2056, 144, True, torch.float16, torch.float16, 1),
    (3000, 4104, 80, False, torch.bfloat16, torch.bfloat16, 0), (3000, 4104, 256, True, None, torch.float32, 1),
    # 288x256 tiles
    (4500, 4088, 80, True, torch.bfloat16, torch.bfloat16, 0), (4400, 4088, 128, False, torch.float16, torch.float32, 1),
    (4608, 4096, 144, True, torch.float32, torch.float16, 1),
    # 256x288 tiles
    (4090, 4600, 80, True, torch.bfloat16, torch.bfloat16, 0), (4096, 4608, 128, False, torch.float32, torch.float32, 1),
    # 128x96 tiles (four waves of 32x96)
    (250, 9200, 144, True, torch.bfloat16, torch.bfloat16, 0), (256, 9216, 128, False, torch.float16, torch.float32, 1),
    # 256x96 tiles
    (500, 9200, 144, True, torch.bfloat16, torch.bfloat16, 0), (512, 9216, 128, False, torch.float32, torch.float32, 1),
    (384, 12288, 272, True, torch.float16, torch.float16, 1),
]


@pytest.mark.parametrize("M,N,K,row,bdt,odt,order", LIN_CASES)
def test_linear_w8a8_bit_exact(L, dev, M, N, K, row, bdt, odt, order):
    x = acts(M, K)
    wf = torch.randn(N, K, generator=G) * 0.02
    wq, ws = O.quant_rowwise(wf.numpy(), O.F32) if row else O.quant_tensorwise(wf.numpy(), O.F32)
    bias = None if bdt is None else (torch.randn(N, generator=G) * 0.01).to(bdt)
    xa, code = O.from_torch(x)
    ocode = {torch.bfloat16: O.BF16, torch.float16: O.F16, torch.float32: O.F32}[odt]
    ba, bcode = (None, O.BF16) if bias is None else O.from_torch(bias)
    want = O.linear_w8a8(xa, code, wq, ws, ba, bcode, ocode, 0, order)
    q, s = L.quant_rowwise(x.to(dev))
    ws_arg = torch.from_numpy(ws).to(dev) if row else float(ws[0])
    got = L.linear_w8a8(q, s, torch.from_numpy(wq).to(dev), ws_arg, None if bias is None else bias.to(dev), odt, order)
    assert np.array_equal(bits(got), want)
    if not row:   # the scale may also arrive as a one-element device tensor
        got2 = L.linear_w8a8(q, s, torch.from_numpy(wq).to(dev), torch.from_numpy(ws).to(dev), None if bias is None else bias.to(dev), odt, order)
        assert np.array_equal(bits(got2), want)


GATED_CASES = [
    # M, N, K, per-row scales, output dtype, gate vectors, residual: the gated residual x + gate * linear(h) in the epilogue
    (4608, 3072, 256, True, torch.bfloat16, 1, True), (4096, 3072, 384, True, torch.bfloat16, 2, True),      # 256-wide tiles
    (4600, 12288, 128, True, torch.float16, 1, True), (1000, 264, 384, False, torch.bfloat16, 4, True),      # 288 x 256; ragged
    (512, 3072, 12288, True, torch.bfloat16, 2, True),                                                       # few tiles, K split
    (300, 512, 256, True, torch.float32, 3, True), (130, 96, 128, True, torch.bfloat16, 1, False),           # binary32; gate alone
    (257, 3076, 640, True, torch.float16, 1, True),                                                          # N % 8 != 0: the one-thread-per-output kernel
]


@pytest.mark.parametrize("M,N,K,row,odt,V,with_res", GATED_CASES)
def test_linear_w8a8_gated_residual_bit_exact(L, dev, M, N, K, row, odt, V, with_res):
    """out = residual + gate * linear(h) with both elementwise operations inside the GEMM epilogue (i8f_linear_w8a8_gated):
    bit-equal to the oracle's linear followed by its restatement of torch's two tensor operations, and to the same two
    torch operations on the device applied to this library's own linear output; also in place (out = residual)."""
    M -= M % V
    x = acts(M, K)
    wf = torch.randn(N, K, generator=G) * 0.02
    wq, ws = O.quant_rowwise(wf.numpy(), O.F32) if row else O.quant_tensorwise(wf.numpy(), O.F32)
    bias = (torch.randn(N, generator=G) * 0.01).to(torch.bfloat16)
    gate = torch.randn(V, N, generator=G).to(odt)
    res = (torch.randn(M, N, generator=G) * 0.5).to(odt) if with_res else None
    ocode = {torch.bfloat16: O.BF16, torch.float16: O.F16, torch.float32: O.F32}[odt]
    xa, code = O.from_torch(x)
    y = O.linear_w8a8(xa, code, wq, ws, O.from_torch(bias)[0], O.BF16, ocode, 0, 0)
    want = O.gate_residual(y, ocode, gate=O.from_torch(gate)[0], residual=None if res is None else O.from_torch(res)[0], rows_per_gate=M // V)
    q, s = L.quant_rowwise(x.to(dev))
    ws_arg = torch.from_numpy(ws).to(dev) if row else float(ws[0])
    wd, bd, gd = torch.from_numpy(wq).to(dev), bias.to(dev), gate.to(dev)
    rd = None if res is None else res.to(dev)
    got = L.linear_w8a8(q, s, wd, ws_arg, bd, odt, L.EPI_TORCH, addend=rd, gate=gd)
    assert np.array_equal(bits(got), want)
    plain = L.linear_w8a8(q, s, wd, ws_arg, bd, odt, L.EPI_TORCH)
    torch_way = gd.repeat_interleave(M // V, 0) * plain
    if rd is not None:
        torch_way = rd + torch_way
    assert torch.equal(torch_way, got)
    if rd is not None:                                  # the residual stream updated in place
        buf = rd.clone()
        L.linear_w8a8(q, s, wd, ws_arg, bd, odt, L.EPI_TORCH, out=buf, addend=buf, gate=gd)
        assert torch.equal(buf, got)


GROUPED_CASES = [
    # row counts of the groups, N, K, per-row scales, bias dtype, output dtype, order, residual addend
    ((4096, 512), 3072, 384, True, torch.bfloat16, torch.bfloat16, 0, False),    # 192 + 24 tiles of 256 x 256: one launch
    ((4090, 500, 130), 3064, 256, True, torch.float16, torch.float16, 1, True),  # ragged everywhere, three groups, addends
    ((4096, 512), 9216, 3072, True, torch.bfloat16, torch.bfloat16, 0, False),   # the small group would cost a round: separate launches
    ((4096, 512), 2304, 256, False, None, torch.float32, 0, False),              # 192 + 24 tiles of 256 x 192, one scale per group
    ((4032, 288), 4096, 128, True, torch.bfloat16, torch.bfloat16, 0, True),     # 224 + 16 tiles of 288 x 256
    ((3584, 250), 4608, 128, True, torch.float16, torch.float16, 0, False),      # 224 + 16 tiles of 256 x 288
    ((512, 4096, 0, 17), 3072, 128, True, torch.bfloat16, torch.bfloat16, 0, False),  # the large group second, an empty one, a tiny one
    ((300, 200), 512, 200, True, torch.bfloat16, torch.bfloat16, 0, False),      # K not a multiple of 128: separate launches
]


@pytest.mark.parametrize("Ms,N,K,row,bdt,odt,order,add", GROUPED_CASES)
def test_linear_w8a8_grouped_equals_separate_calls_and_the_oracle(L, dev, Ms, N, K, row, bdt, odt, order, add):
    """i8f_linear_w8a8_grouped: several problems of one layer shape, each with its own activations, weights, scales, bias
    and addend, in one launch where the library groups them and group by group where it does not: every output is
    the oracle's bit for bit and that of a linear_w8a8 call of its own."""
    ocode = {torch.bfloat16: O.BF16, torch.float16: O.F16, torch.float32: O.F32}[odt]
    problems, wants = [], []
    for M in Ms:
        x = acts(M, K)
        wf = torch.randn(N, K, generator=G) * 0.02
        wq, ws = O.quant_rowwise(wf.numpy(), O.F32) if row else O.quant_tensorwise(wf.numpy(), O.F32)
        bias = None if bdt is None else (torch.randn(N, generator=G) * 0.01).to(bdt)
        addend = (torch.randn(M, N, generator=G) * 0.3).to(odt) if add else None
        gate = torch.randn(2 if M % 2 == 0 and M else 1, N, generator=G).to(odt) if add and M else None   # (with the addends: gated residuals)
        q, s = L.quant_rowwise(x.to(dev)) if M else (torch.empty(0, K, dtype=torch.int8, device=dev), torch.empty(0, 1, device=dev))
        ws_arg = torch.from_numpy(ws).to(dev) if row else float(ws[0])
        problems.append((q, s, torch.from_numpy(wq).to(dev), ws_arg, None if bias is None else bias.to(dev), None if addend is None else addend.to(dev),
                         None if gate is None else gate.to(dev)))
        if M:
            xa, code = O.from_torch(x)
            ba, bcode = (None, O.BF16) if bias is None else O.from_torch(bias)
            y = O.linear_w8a8(xa, code, wq, ws, ba, bcode, ocode, 0, order)
            if add:
                y = O.gate_residual(y, ocode, gate=O.from_torch(gate)[0], residual=O.from_torch(addend)[0], rows_per_gate=M // gate.shape[0])
            wants.append(y)
        else:
            wants.append(None)
    got = L.linear_w8a8_grouped(problems, odt, order)
    assert len(got) == len(Ms)
    for M, p, g, want in zip(Ms, problems, got, wants):
        assert tuple(g.shape) == (M, N) and g.dtype == odt
        if M == 0:
            continue
        assert np.array_equal(bits(g), want)
        alone = L.linear_w8a8(p[0], p[1], p[2], p[3], p[4], odt, order, addend=p[5], gate=p[6])
        assert torch.equal(alone, g)


def test_linear_w8a8_grouped_mixed_problems_fall_back_to_separate_launches(L, dev):
    """Problems that do not share N, the scale mode or the bias dtype are launched one by one by the Python layer."""
    xa, xb = acts(300, 256), acts(40, 256)
    qa, sa = L.quant_rowwise(xa.to(dev))
    qb, sb = L.quant_rowwise(xb.to(dev))
    wa, wb = i8(512, 256).to(dev), i8(264, 256).to(dev)
    wsa = (torch.rand(512, generator=G) * 0.002 + 0.0005).to(dev)
    got = L.linear_w8a8_grouped([(qa, sa, wa, wsa, None), (qb, sb, wb, 0.001, (torch.randn(264, generator=G) * 0.1).to(dev))], torch.bfloat16)
    assert torch.equal(got[0], L.linear_w8a8(qa, sa, wa, wsa, None, torch.bfloat16))
    assert tuple(got[1].shape) == (40, 264)
    with pytest.raises(ValueError):
        L.linear_w8a8_grouped([(qa, sa, wa, wsa, None), (qb, sb, i8(64, 128).to(dev), 0.001, None)], torch.bfloat16)   # K mismatch


SPLITK_CASES = [
    # M, N, K, output dtype: few tiles and a long K, where the tile's K range is dealt over several workgroups
    (512, 3072, 12288, torch.bfloat16),   # 128 x 96 tiles, two slices
    (250, 3064, 12304, torch.float16),    # ragged everywhere, K not a multiple of the 128-byte K-tile
    (64, 3072, 12288, torch.bfloat16),    # 64 x 64 tiles, five slices of unequal length
    (100, 1000, 16400, torch.float32),
    (16, 12288, 10240, torch.bfloat16),   # the shortest K that is split
]


@pytest.mark.parametrize("M,N,K,odt", SPLITK_CASES)
def test_linear_w8a8_k_split_bit_exact(L, dev, M, N, K, odt):
    """Outputs of few tiles with K >= 10240 take the K split when a workspace is given (the Python layer keeps one
    per stream): bit-equal to the oracle and to the same call without a workspace, the arrival counters are zero
    again afterwards, and a second call on the same workspace gives the same result."""
    x = acts(M, K)
    wq = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=G)
    ws = (torch.rand(N, generator=G) * 0.002 + 0.0005)
    bias = (torch.randn(N, generator=G) * 0.01).to(torch.bfloat16)
    xa, code = O.from_torch(x)
    ocode = {torch.bfloat16: O.BF16, torch.float16: O.F16, torch.float32: O.F32}[odt]
    ba, bcode = O.from_torch(bias)
    want = O.linear_w8a8(xa, code, wq.numpy(), ws.numpy(), ba, bcode, ocode, 0, L.EPI_TORCH)
    q, s = L.quant_rowwise(x.to(dev))
    wd, wsd, bd = wq.to(dev), ws.to(dev), bias.to(dev)
    got = L.linear_w8a8(q, s, wd, wsd, bd, odt, L.EPI_TORCH)
    assert np.array_equal(bits(got), want)
    work = L._splitk_workspace(q, M, N, K)
    assert work is not None and int(work[:4096].view(torch.int32).abs().sum()) == 0
    again = L.linear_w8a8(q, s, wd, wsd, bd, odt, L.EPI_TORCH)
    assert torch.equal(again.view(torch.uint8), got.view(torch.uint8))
    plain = torch.empty_like(got)
    rc = L.lib().i8f_linear_w8a8(q.data_ptr(), s.data_ptr(), wd.data_ptr(), wsd.data_ptr(), 0.0, L.SCALE_ROW, bd.data_ptr(), L.BF16,
                                 plain.data_ptr(), L.dtype_code(odt), M, N, K, L.EPI_TORCH, None)
    torch.cuda.synchronize()
    assert rc == 0 and torch.equal(plain.view(torch.uint8), got.view(torch.uint8))


def test_linear_w8a8_k_split_on_leftover_arrival_words(L, dev):
    """The arrival words of the K split as launches that never finished would have left them: another launch's tag
    with every count a slice can leave, counts no slice can leave, all ones.  Every kernel still exits, the result
    is the oracle's bit for bit, and the words are zero afterwards (a launch stamps the words with its own tag and
    takes a word with another tag as `nobody has arrived`)."""
    M, N, K = 64, 3072, 12288    # 64 x 64 tiles, five slices per tile
    x = acts(M, K)
    wq = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=G)
    ws = (torch.rand(N, generator=G) * 0.002 + 0.0005)
    xa, code = O.from_torch(x)
    want = O.linear_w8a8(xa, code, wq.numpy(), ws.numpy(), None, O.BF16, O.BF16, 0, L.EPI_TORCH)
    q, s = L.quant_rowwise(x.to(dev))
    wd, wsd = wq.to(dev), ws.to(dev)
    nbytes = L.lib().i8f_linear_w8a8_workspace_bytes()
    work = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    words = work[:4096].view(torch.int32)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    stale_tag = 0x123456
    leftovers = [[(stale_tag << 8) | c for c in (1, 2, 3, 4, 5)], [1, 2, 3, 4], [0xff, 0x7fffffff, -1, 0xabcdef07]]
    for fill in leftovers:
        words.copy_(torch.tensor([fill[i % len(fill)] for i in range(1024)], dtype=torch.int64).to(torch.int32))
        out.zero_()
        rc = L.lib().i8f_linear_w8a8_splitk(q.data_ptr(), s.data_ptr(), wd.data_ptr(), wsd.data_ptr(), 0.0, L.SCALE_ROW, None, L.BF16,
                                            None, out.data_ptr(), L.BF16, M, N, K, L.EPI_TORCH, work.data_ptr(), nbytes, None)
        torch.cuda.synchronize()
        assert rc == 0
        assert np.array_equal(bits(out), want), f"leftover words {fill[:3]}..."
        tiles = (N + 63) // 64
        assert int(words[:tiles].abs().sum()) == 0, "the words of the tiles in use are zero after a completed launch"


def test_linear_w8a8_long_k_under_hip_graph_equals_eager(L, dev):
    """A shape that takes the K split, captured in a HIP graph: while a stream captures, the Python layer gives the
    call a workspace from the graph's own memory pool with a fill kernel in front that clears the arrival words on
    every replay (never the eager workspace of the stream), so the split is taken inside the graph too; every replay
    gives the eager result bit for bit, with eager split launches between the replays."""
    M, N, K = 64, 1024, 12288
    q = torch.randint(-127, 128, (M, K), dtype=torch.int8, generator=G).to(dev)
    w = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=G).to(dev)
    s = (torch.rand(M, 1, generator=G) * 0.01 + 0.001).to(dev)
    ws = (torch.rand(N, generator=G) * 0.01 + 0.001).to(dev)
    eager = L.linear_w8a8(q, s, w, ws)
    static_q = q.clone()
    graph = torch.cuda.CUDAGraph()
    seen = []
    real = L._splitk_workspace
    try:
        L._splitk_workspace = lambda *a: seen.append(real(*a)) or seen[-1]
        with torch.cuda.graph(graph):
            static_y = L.linear_w8a8(static_q, s, w, ws)
    finally:
        L._splitk_workspace = real
    eager_ws = real(q, M, N, K)
    assert len(seen) == 1 and seen[0] is not None and seen[0].data_ptr() != eager_ws.data_ptr(), \
        "the captured call has a workspace of its own"
    del seen
    for i in range(3):
        q2 = torch.randint(-127, 128, (M, K), dtype=torch.int8, generator=G).to(dev)
        want = L.linear_w8a8(q2, s, w, ws)      # eager work (with the split) between the replays
        torch.cuda.synchronize()
        static_q.copy_(q2)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y.view(torch.int16), want.view(torch.int16)), f"replay {i}"
    assert torch.equal(L.linear_w8a8(q, s, w, ws).view(torch.int16), eager.view(torch.int16))


def test_linear_w8a8_random_shapes_and_flags(L, dev):
    """24 seeded cases over the whole range of output sizes (every tile configuration the host can pick),
    with the scale mode, bias dtype, output dtype and operation order drawn at random; K stays short so
    that the CPU side finishes in seconds."""
    rng = np.random.default_rng(777)
    dts = [torch.bfloat16, torch.float16, torch.float32]
    sizes = [(4608, 12288), (4096, 9216), (4608, 3072), (2048, 4096), (640, 12288), (512, 12288), (512, 9216), (256, 9216),
             (512, 3072), (256, 3072), (1024, 3072), (100, 18432)]
    for case in range(24):
        M0, N0 = sizes[case % len(sizes)]
        M = int(M0 - rng.integers(0, 40))
        N = int(N0 - 8 * rng.integers(0, 12))
        K = int(rng.integers(1, 20)) * 16
        row, order = bool(rng.integers(0, 2)), int(rng.integers(0, 2))
        bdt = [None, *dts][int(rng.integers(0, 4))]
        odt = dts[int(rng.integers(0, 3))] if case % 4 == 0 else dts[int(rng.integers(0, 2))]
        x = acts(M, K)
        wf = torch.randn(N, K, generator=G) * 0.02
        wq, ws = O.quant_rowwise(wf.numpy(), O.F32) if row else O.quant_tensorwise(wf.numpy(), O.F32)
        bias = None if bdt is None else (torch.randn(N, generator=G) * 0.01).to(bdt)
        xa, code = O.from_torch(x)
        ocode = {torch.bfloat16: O.BF16, torch.float16: O.F16, torch.float32: O.F32}[odt]
        ba, bcode = (None, O.BF16) if bias is None else O.from_torch(bias)
        want = O.linear_w8a8(xa, code, wq, ws, ba, bcode, ocode, 0, order)
        q, s = L.quant_rowwise(x.to(dev))
        ws_arg = torch.from_numpy(ws).to(dev) if row else float(ws[0])
        got = L.linear_w8a8(q, s, torch.from_numpy(wq).to(dev), ws_arg, None if bias is None else bias.to(dev), odt, order)
        assert np.array_equal(bits(got), want), (M, N, K, row, bdt, odt, order)


@pytest.mark.parametrize("M,N,K,odt,order", [(300, 520, 1040, torch.bfloat16, 0), (2000, 2056, 200, torch.float16, 1),
                                             (4100, 2056, 144, torch.bfloat16, 0), (64, 50, 50, torch.bfloat16, 0),
                                             (256, 256, 512, torch.float32, 0),
                                             (4500, 4088, 144, torch.bfloat16, 0),    # 288x256 tiles
                                             (4090, 4600, 80, torch.float16, 1)])     # 256x288 tiles
def test_linear_w8a8_with_addend_rounds_like_a_tensor_addition(L, dev, M, N, K, odt, order):
    """out = round(linear + addend): the sum of two ROUNDED tensors, rounded once more (int8_quant.py:774)."""
    x = acts(M, K)
    wq, ws = L.quant_rowwise((torch.randn(N, K, generator=G) * 0.02).to(dev))
    bias = (torch.randn(N, generator=G) * 0.01).to(odt).to(dev)
    addend = (torch.randn(M, N, generator=G) * 0.3).to(odt).to(dev)
    q, s = L.quant_rowwise(x.to(dev))
    plain = L.linear_w8a8(q, s, wq, ws, bias, odt, order)          # bit-exact against the oracle by the tests above
    got = L.linear_w8a8(q, s, wq, ws, bias, odt, order, addend=addend)
    code = {torch.bfloat16: O.BF16, torch.float16: O.F16, torch.float32: O.F32}[odt]
    want = O.round_to(O.to_f32(bits(plain), code) + O.to_f32(bits(addend), code), code)
    assert np.array_equal(bits(got), want)
    assert torch.equal(got, plain + addend)                          # and what torch's own addition gives


@pytest.mark.parametrize("M,N,K", [(4608, 3072, 3072), (512, 3072, 12288), (4096, 9216, 3072)])
def test_linear_w8a8_gives_the_same_bits_on_every_launch(L, dev, M, N, K):
    """300 back-to-back launches (no synchronisation between them) against the first result: a missing
    wait or barrier in the pipelined loop would show up as a rare differing tile."""
    q, s = L.quant_rowwise(acts(M, K).to(dev))
    wq, ws = L.quant_rowwise((torch.randn(N, K, generator=G) * 0.02).to(dev))
    first = L.linear_w8a8(q, s, wq, ws, None, torch.bfloat16, 0)
    out = torch.empty_like(first)
    bad = torch.zeros((), dtype=torch.int64, device=dev)
    for _ in range(300):
        L.linear_w8a8(q, s, wq, ws, None, torch.bfloat16, 0, out)
        bad += (out.view(torch.int16) != first.view(torch.int16)).sum()
    assert int(bad.item()) == 0


def test_linear_accumulator_beyond_2_pow_24_rounds_like_the_oracle(L, dev):
    K = 4096
    a = torch.full((32, K), 127, dtype=torch.int8)
    a[:, ::3] = 126
    w = torch.full((16, K), 127, dtype=torch.int8)
    w[:, ::5] = -128
    xs = np.full(32, 1e-3, dtype=np.float32)
    ws = np.linspace(1e-4, 2e-4, 16, dtype=np.float32)
    acc = O.gemm_i32(a.numpy(), w.numpy())
    assert np.abs(acc).max() > 2**24
    want = O.epilogue(acc, xs, ws, None, O.BF16, O.F32, O.EPI_TORCH)
    got = L.linear_w8a8(a.to(dev), torch.from_numpy(xs).to(dev), w.to(dev), torch.from_numpy(ws).to(dev), None, torch.float32, 0)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


# ------------------------------------------------------------------ BASELINE configs at full size
def _check_rows(L, dev, x, wq_d, ws_d, bias, rows, rotate=False, scalar=None):
    """Full-size launch, oracle on a row sample (bit-exact), integer checksum over everything."""
    xd = x.to(dev)
    q, s = L.quant_rowwise(xd, rotate=rotate)
    xa, code = O.from_torch(x[rows])
    qo, so = O.quant_rowwise(xa, code, 128 if rotate else 0)
    assert np.array_equal(q[rows].cpu().numpy(), qo) and np.array_equal(s[rows].cpu().numpy(), so)
    acc = L.gemm_i32(q, wq_d)
    wq = wq_d.cpu().numpy()
    assert np.array_equal(acc[rows].cpu().numpy(), O.gemm_i32(qo, wq))
    # checksum of checksums: sum_n acc[m,n] == q[m,:] . sum_n w[n,:]   for EVERY row, in int64
    col = wq.astype(np.int64).sum(axis=0)
    assert np.array_equal(acc.sum(dim=1, dtype=torch.int64).cpu().numpy(), q.cpu().numpy().astype(np.int64) @ col)
    ws_arg = ws_d if scalar is None else scalar
    y = L.linear_w8a8(q, s, wq_d, ws_arg, None if bias is None else bias.to(dev), torch.bfloat16, 0)
    ws_np = ws_d.cpu().numpy() if scalar is None else np.float32(scalar)
    want = O.epilogue(O.gemm_i32(qo, wq), so, ws_np, None if bias is None else O.from_torch(bias)[0], O.BF16, O.BF16)
    assert np.array_equal(bits(y[rows]), want)
    return y


def test_config0_tensorwise_full_size(L, dev):
    c = make_config(0)
    wq, ws = O.quant_tensorwise(O.from_torch(c["w"])[0], O.BF16)
    rows = torch.randperm(4096, generator=G)[:48].sort().values
    _check_rows(L, dev, c["x"], torch.from_numpy(wq).to(dev), None, None, rows, scalar=float(ws[0]))


def test_config1_flux_mlp_full_size(L, dev):
    c = make_config(1)
    rows = torch.randperm(4608, generator=G)[:32].sort().values
    wq, ws = L.quant_rowwise(c["w_up"].to(dev))
    qo, so = O.quant_rowwise(c["w_up"][:64].numpy(), O.F32)
    assert np.array_equal(wq[:64].cpu().numpy(), qo) and np.array_equal(ws[:64].cpu().numpy(), so)
    _check_rows(L, dev, c["x"], wq, ws, c["b_up"], rows)
    wq, ws = L.quant_rowwise(c["w_dn"].to(dev))
    _check_rows(L, dev, c["h"], wq, ws, c["b_dn"], rows[:16])


def test_config2_quarot_full_size_and_error_vs_bf16(L, dev):
    c = make_config(2)
    x, w = c["x"], c["w"]
    rows = torch.randperm(4096, generator=G)[:32].sort().values
    wq_r, ws_r = L.quant_rowwise(w.to(dev), rotate=True)
    y_rot = _check_rows(L, dev, x, wq_r, ws_r, None, rows, rotate=True).float()
    wq_p, ws_p = L.quant_rowwise(w.to(dev))
    q, s = L.quant_rowwise(x.to(dev))
    y_plain = L.linear_w8a8(q, s, wq_p, ws_p, None, torch.bfloat16, 0).float()
    ref = (x.to(dev).float() @ w.to(dev).bfloat16().float().T)
    err_rot = ((y_rot - ref).norm() / ref.norm()).item()
    err_plain = ((y_plain - ref).norm() / ref.norm()).item()
    assert err_rot < 0.5 * err_plain and err_rot < 0.03       # the rotation is what makes the outliers quantisable


def test_config3_dit_block_linears_full_size(L, dev):
    """Every W8A8 linear of the double-stream block (image stream M = 4096, text stream M = 512) and the
    adaLN projection at M = 1: the first two run through each tile configuration the host picks for them."""
    c = make_config(3)
    g = torch.Generator().manual_seed(1003)
    for name in ("qkv", "proj", "up", "down"):
        n_out, k_in = c["linears"][name]
        w = torch.randn(n_out, k_in, generator=g) * 0.02
        b = (torch.randn(n_out, generator=g) * 0.01).bfloat16()
        wq, ws = L.quant_rowwise(w.to(dev))
        for m in (c["img"], c["txt"]):
            x = acts(m, k_in)
            rows = torch.randperm(m, generator=G)[:12].sort().values
            _check_rows(L, dev, x, wq, ws, b, rows)
    n_out, k_in = c["linears"]["adaln"]
    w = torch.randn(n_out, k_in, generator=g) * 0.02
    wq, ws = L.quant_rowwise(w.to(dev))
    vec = torch.randn(1, k_in, generator=g).bfloat16()
    y = L.linear_w8a16_small_m(vec.to(dev), wq, ws, None).float().cpu().numpy()
    xa, code = O.from_torch(vec)
    ref = O.to_f32(O.linear_w8a16(xa, code, wq.cpu().numpy(), ws.cpu().numpy()), code)
    assert np.all(np.abs(y - ref) <= w8a16_bound(vec, wq.cpu(), ws.cpu().reshape(-1), ref, torch.bfloat16))


def test_config4_merge_full_size_then_skinny_gemm(L, dev):
    c = make_config(4)
    wq, ws = L.quant_rowwise(c["w"].to(dev))
    noise, up, down = c["noise"], c["up"], c["down"]
    merged = L.lora_merge_sr(wq, ws, noise.to(dev), up=up.to(dev), down=down.to(dev), lora_scale=c["alpha"] / 32)
    rows = torch.randperm(12288, generator=G)[:96].sort().values
    want = O.lora_merge_sr(wq[rows].cpu().numpy(), ws[rows].cpu().numpy(), noise[rows].numpy(),
                           up=up[rows].numpy(), down=down.numpy(), lora_scale=1.0)
    assert np.array_equal(merged[rows].cpu().numpy(), want)
    changed = (merged != wq).float().mean().item()
    assert 0.05 < changed < 0.95
    # in place gives the same bytes
    w2 = wq.clone()
    L.lora_merge_sr(w2, ws, noise.to(dev), up=up.to(dev), down=down.to(dev), lora_scale=1.0, out=w2)
    assert torch.equal(w2, merged)
    # skinny GEMM on the merged weight, M = 256
    x = c["x"]
    q, s = L.quant_rowwise(x.to(dev))
    y = L.linear_w8a8(q, s, merged, ws, None, torch.bfloat16, 0)
    xa, code = O.from_torch(x)
    want_y = O.linear_w8a8(xa, code, merged.cpu().numpy(), ws.cpu().numpy())
    assert np.array_equal(bits(y), want_y)


def test_config4_fused_merge_against_library_product_delta(L, dev):
    """The fused merge rebuilds the rank-32 delta as an fma chain; the reference forms it with torch.mm
    (int8_quant.py:143-157, :295), whose summation order is the BLAS library's.  The two deltas differ in
    the last bits, which flips a stochastic rounding only where the noise falls within that difference of
    the fraction: at most one merged byte in a million may differ, and none by more than one step."""
    c = make_config(4)
    wq, ws = L.quant_rowwise(c["w"].to(dev))
    noise, up, down = c["noise"].to(dev), c["up"].to(dev), c["down"].to(dev)
    scale = c["alpha"] / 32
    fused = L.lora_merge_sr(wq, ws, noise, up=up, down=down, lora_scale=scale)
    delta = torch.mm(up, down) * scale
    given = L.lora_merge_sr(wq, ws, noise, delta=delta)
    diff = (fused.int() - given.int()).abs()
    frac = (diff != 0).float().mean().item()
    assert diff.max().item() <= 1 and frac <= 1e-6, f"{frac:.2e} of the merged bytes differ"


# ------------------------------------------------------------------ dynamic LoRA side branch in the epilogue (f4)
@pytest.mark.parametrize("M,N,K,r,dt,alpha,row", [
    (300, 512, 256, 32, torch.bfloat16, None, True), (1000, 264, 384, 16, torch.float16, 0.5, True),
    (4608, 3072, 3072, 32, torch.bfloat16, None, True), (512, 12288, 3072, 64, torch.bfloat16, 1.25, True),
    (4608, 12288, 3072, 32, torch.bfloat16, None, True), (130, 96, 128, 24, torch.bfloat16, None, False),
    (257, 3080, 640, 8, torch.float16, 2.0, True),
    # the twelve-wave tiles: 256 x 288 (rank 48), 288 x 256 with a ragged last row and column of tiles
    (4096, 9216, 256, 48, torch.bfloat16, None, True), (4600, 12280, 128, 16, torch.float16, 0.75, True),
])
def test_linear_w8a8_lora_side_branch(L, dev, M, N, K, r, dt, alpha, row):
    """out = round(y + round(round(t @ B.T) * alpha)) with the rank-r product formed inside the GEMM epilogue, against
    (1) the same arithmetic with the product taken in float64 on the oracle's bit-exact y and (2) the unfused path
    (torch F.linear on the device, added by i8f_linear_w8a8_add).  The matrix core accumulates the r products in binary32
    in its own order, so a side value may round the other way now and then: results at most one ulp of the dtype
    apart, at least 99 % identical."""
    x = acts(M, K, dt)
    w = i8(N, K)
    ws = torch.rand(N if row else 1, generator=G) * 0.002 + 0.0005
    bias = (torch.randn(N, generator=G) * 0.1).to(dt)
    t = (torch.randn(M, r, generator=G) * 0.5).to(dt)
    B = (torch.randn(N, r, generator=G) * 0.2).to(dt)
    q, s = L.quant_rowwise(x.to(dev))
    ws_arg = ws.to(dev) if row else float(ws[0])
    got = L.linear_w8a8_lora(q, s, w.to(dev), ws_arg, bias.to(dev), t.to(dev), B.to(dev), alpha, dt)
    side = torch.nn.functional.linear(t.to(dev), B.to(dev))
    if alpha is not None:
        side = side * alpha
    unfused = L.linear_w8a8(q, s, w.to(dev), ws_arg, bias.to(dev), dt, L.EPI_TORCH, addend=side)
    xa, code = O.from_torch(x)
    y = O.to_f32(O.linear_w8a8(xa, code, w.numpy(), ws.numpy(), O.from_torch(bias)[0], code, code), code)
    sd = torch.from_numpy(t.double().numpy() @ B.double().numpy().T).to(dt)
    if alpha is not None:
        sd = (sd.float() * alpha).to(dt)
    want = (torch.from_numpy(y) + sd.float()).to(dt)
    # Element by element: the result is round(y + s') where s' is the reference's side value or a NEIGHBOUR of it in the
    # dtype (one step when the rank-r sum rounds the other way, two with alpha, whose product is rounded again): nothing
    # else is allowed, and all but 1 % of the elements take the reference's side value itself.
    steps = 1 if alpha is None else 2
    yt = torch.from_numpy(y)
    for side_ref, ref in ((sd, want), (side.cpu().to(dt), unfused.cpu())):
        ok = torch.zeros(got.shape, dtype=torch.bool)
        for k in range(-steps, steps + 1):
            ok |= _raw16((yt + step_16(side_ref, k).float()).to(dt)) == _raw16(got.cpu())
        assert ok.all(), f"{(~ok).sum().item()} elements are not y + (side value or a neighbour), first at {(~ok).flatten().nonzero()[0].item()}"
        assert (_raw16(got.cpu()) != _raw16(ref)).float().mean().item() <= 0.01


def step_16(t, k):
    """t (bfloat16 / float16) moved k representable values up (k < 0: down), through zero if need be."""
    b = t.contiguous().view(torch.int16).to(torch.int32)
    o = torch.where(b < 0, -(b & 0x7fff), b) + k          # sign-magnitude patterns as ordered integers
    b2 = torch.where(o < 0, (-o) | 0x8000, o)
    return torch.where(b2 >= 0x8000, b2 - 0x10000, b2).to(torch.int16).view(t.dtype)


# ------------------------------------------------------------------ small batch W8A16 (a8)
ULP = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11, torch.float32: 2.0**-23}
MANT_BITS = {torch.bfloat16: 7, torch.float16: 10, torch.float32: 23}


def spacing(v, dt):
    """Distance between neighbouring values of dtype dt at |v| (one unit in the last place: between 2^-(p+1) and
    2^-p of |v| for p mantissa bits, the larger just above a power of two)."""
    a = np.maximum(np.abs(np.asarray(v, dtype=np.float64)), 2.0**-126)
    return np.ldexp(1.0, np.floor(np.log2(a)).astype(np.int64) - MANT_BITS[dt])


def w8a16_bound(x, wq, ws, ref, dt):
    """Per-element bound for a product of dtype-rounded operands accumulated in binary32 in any order and
    rounded once: one unit in the last place of the result's dtype at the result (two sums on either side of a
    rounding boundary land on neighbouring values) plus K * 2^-24 * sum_k |x||w| for the accumulation (no term
    that scales with the largest output of the tensor)."""
    K = x.shape[1]
    wdq = (wq.float() * ws.reshape(-1, 1)).to(dt).double().abs()
    S = (x.double().abs() @ wdq.T).numpy()
    return spacing(ref, dt) + K * 2.0**-24 * S + 1e-30


@pytest.mark.parametrize("M,N,K,dt", [
    (1, 18432, 3072, torch.bfloat16), (16, 260, 1024, torch.bfloat16), (3, 100, 77, torch.float16), (2, 64, 256, torch.float32),
    (7, 33, 4096, torch.float16), (5, 48, 272, torch.bfloat16), (16, 31, 144, torch.float16), (1, 1, 16, torch.bfloat16),
    (13, 513, 2064, torch.bfloat16), (2, 96, 12288, torch.float16),
])
def test_small_m_w8a16_within_tolerance(L, dev, M, N, K, dt):
    x = torch.randn(M, K, generator=G).to(dt)
    wq = i8(N, K)
    ws = torch.rand(N, generator=G) * 0.01 + 0.001
    bias = (torch.randn(N, generator=G) * 0.1).to(dt)
    xa, code = O.from_torch(x)
    ref = O.to_f32(O.linear_w8a16(xa, code, wq.numpy(), ws.numpy(), O.from_torch(bias)[0], code), code)
    got = L.linear_w8a16_small_m(x.to(dev), wq.to(dev), ws.to(dev), bias.to(dev)).float().cpu().numpy()
    err = np.abs(got - ref)
    assert (err <= w8a16_bound(x, wq, ws, ref, dt)).all()
    # The worst case above grows with K; rounding errors of a binary32 accumulation add up like a random walk, so
    # all but a few elements also meet the bound with sqrt(K) in place of K (a kernel that is off by a unit in the
    # last place everywhere passes the first bound at K = 3072 and fails this one) ...
    tight = spacing(ref, dt) + (w8a16_bound(x, wq, ws, ref, dt) - spacing(ref, dt)) / np.sqrt(K)
    assert (err <= tight).mean() >= 0.995
    if dt != torch.float32:   # ... and a 16-bit result differs from the reference's only where a sum sat next to a rounding boundary
        assert (err != 0).mean() <= 0.10 + 2.0 / err.size
    got_t = L.linear_w8a16_small_m(x.to(dev), wq.to(dev), 0.004, None).float().cpu().numpy()
    ref_t = O.to_f32(O.linear_w8a16(xa, code, wq.numpy(), np.float32(0.004)), code)
    assert (np.abs(got_t - ref_t) <= w8a16_bound(x, wq, torch.full((N,), 0.004), ref_t, dt)).all()


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_small_m_rows_are_independent_and_strided_rows_work(L, dev, dt):
    """A token's result must not depend on how many other tokens share the call (the matrix-core
    kernel computes 16 token columns at once), nor on the row stride of x."""
    N, K = 200, 1040
    wide = torch.randn(16, K + 24, generator=G).to(dt).to(dev)
    x = wide[:, :K]                               # row stride K + 24 elements
    wq = i8(N, K).to(dev)
    ws = (torch.rand(N, generator=G) * 0.01 + 0.001).to(dev)
    bias = (torch.randn(N, generator=G) * 0.1).to(dt).to(dev)
    y16 = L.linear_w8a16_small_m(x, wq, ws, bias)
    assert torch.equal(_raw16(y16), _raw16(L.linear_w8a16_small_m(x.contiguous(), wq, ws, bias)))
    for m in (0, 3, 15):
        y1 = L.linear_w8a16_small_m(x[m:m + 1].contiguous(), wq, ws, bias)
        assert torch.equal(_raw16(y1[0]), _raw16(y16[m]))
    y5 = L.linear_w8a16_small_m(x[4:9], wq, ws, bias)
    assert torch.equal(_raw16(y5), _raw16(y16[4:9]))


# ------------------------------------------------------------------ stochastic merge (a9, a10, a11)
@pytest.mark.parametrize("N,K,r,row", [(256, 1024, 32, True), (100, 77, 8, False), (512, 3072, 32, True), (3, 5, 1, True), (64, 130, 256, False),
                                          (100, 96, 8, True), (70, 128, 4, False), (33, 64, 16, True), (1, 32, 32, True),
                                          (64, 100, 8, True), (300, 544, 32, True), (96, 288, 16, False)])
def test_lora_merge_bit_exact(L, dev, N, K, r, row):
    w = i8(N, K)
    ws = torch.rand(N if row else 1, generator=G) * 0.002 + 0.0005
    up, down = torch.randn(N, r, generator=G) * 0.05, torch.randn(r, K, generator=G) * 0.05
    noise = torch.rand(N, K, generator=G)
    delta = O.lora_delta(up.numpy(), down.numpy(), 0.7)
    ws_arg = ws.to(dev) if row else float(ws[0])
    fused = L.lora_merge_sr(w.to(dev), ws_arg, noise.to(dev), up=up.to(dev), down=down.to(dev), lora_scale=0.7)
    given = L.lora_merge_sr(w.to(dev), ws_arg, noise.to(dev), delta=torch.from_numpy(delta).to(dev))
    dq = L.sr_quant_delta(torch.from_numpy(delta).to(dev), ws_arg, noise.to(dev))
    assert np.array_equal(fused.cpu().numpy(), O.lora_merge_sr(w.numpy(), ws.numpy(), noise.numpy(), up=up.numpy(), down=down.numpy(), lora_scale=0.7))
    assert np.array_equal(given.cpu().numpy(), O.lora_merge_sr(w.numpy(), ws.numpy(), noise.numpy(), delta=delta))
    assert np.array_equal(dq.cpu().numpy(), O.sr_delta(delta, ws.numpy(), noise.numpy()))


@pytest.mark.parametrize("N,K,r", [(64, 256, 32), (96, 288, 16), (40, 100, 8)])
def test_lora_merge_denormal_products_bit_exact(L, dev, N, K, r):
    """Rank-r products and partial sums in the binary32 denormal range (|up*down| ~ 1e-40), with a weight
    scale small enough that they still decide the rounded delta: the matrix-core form of the fused merge
    (K % 32 == 0, ranks 4..32) and the vector form must both keep them as the oracle's fmaf chain does."""
    w = i8(N, K)
    up = torch.randn(N, r, generator=G) * 1e-20
    down = torch.randn(r, K, generator=G) * 1e-20
    noise = torch.rand(N, K, generator=G)
    ws = float(np.float32(2e-40))                       # denormal scale: delta / scale is of order one
    delta = O.lora_delta(up.numpy(), down.numpy(), 1.0)
    assert (delta != 0).mean() > 0.9 and np.abs(delta).max() < 1.2e-38
    want = O.lora_merge_sr(w.numpy(), np.asarray([ws], dtype=np.float32), noise.numpy(), up=up.numpy(), down=down.numpy(), lora_scale=1.0)
    assert (want != w.numpy()).mean() > 0.2             # the denormal deltas do move the weights
    fused = L.lora_merge_sr(w.to(dev), ws, noise.to(dev), up=up.to(dev), down=down.to(dev), lora_scale=1.0)
    assert np.array_equal(fused.cpu().numpy(), want)


@pytest.mark.parametrize("K", [256, 100, 37])
def test_sr_quotient_shortcut_and_division_agree_on_awkward_inputs(L, dev, K):
    """The merge kernels take delta / scale from a reciprocal and two fma corrections where that is provably the
    correctly rounded quotient, and from the division elsewhere.  Rows of tiny, zero, huge and infinite deltas,
    noise that is zero, denormal, negative, >= 1 or NaN, and scales outside the shortcut's range must all come out
    as the oracle's division gives them, in the matrix-core form (K = 256), the vector form (K = 100), the
    per-element form (K = 37) and the form that reads a given delta; weights at both ends of the int8 range
    exercise the saturating conversion that packs the result."""
    small = [0.0, -0.0, 1e-45, -3e-42, 1e-36, -2e-33, 7e-31, 3e-7, -0.01, 0.37, -1.5, 90.0, -200.0]
    large = [3e20, -5e25, 1e38, float("inf"), float("-inf")]  # no NaN: the reference's conversion of a NaN to int8 is undefined
    near, far = [1e-3, 2.5e-3, 0.25, 1.0], [3e-7, 1e-12, 2e-40, 4e6, 1e30]
    # 64 rows that qualify for the shortcut (a wave of the matrix-core form decides for 32 rows at once), then the rest
    rows = [(m, sc) for m in small for sc in near] + [(m, near[0]) for m in small[:12]]
    rows += [(m, sc) for m in small for sc in far] + [(m, sc) for m in large for sc in near + far]
    N = len(rows)
    u = torch.tensor([r[0] for r in rows], dtype=torch.float32)
    ws = torch.tensor([r[1] for r in rows], dtype=torch.float32)
    v = torch.tensor([1.0, -1.0, 0.5, 3.0, 1e-3, -7.0, 0.125, 1.0 + 2.0**-23] * ((K + 7) // 8), dtype=torch.float32)[:K]
    special = [0.0, 1e-45, 1e-30, 2.0**-82, 2.0**-83, 1 - 2.0**-24, 1.0, 1.5, -0.25, -0.0, float("nan"), 0.5]
    noise = torch.rand(N, K, generator=G)
    pick = torch.randint(0, 3 * len(special), (N, K), generator=G)
    pick[:, : K // 4] = 3 * len(special)  # the first columns keep ordinary noise, so that whole waves qualify
    for i, val in enumerate(special):
        noise[pick == i] = val
    w = i8(N, K)
    w[:, ::5] = 127
    w[:, 1::5] = -128
    up = torch.zeros(N, 4)
    up[:, 0] = u
    down = torch.zeros(4, K)
    down[0] = v
    with np.errstate(all="ignore"):
        want = O.lora_merge_sr(w.numpy(), ws.numpy(), noise.numpy(), up=up.numpy(), down=down.numpy(), lora_scale=1.0)
        delta = O.lora_delta(up.numpy(), down.numpy(), 1.0)
        want_given = O.lora_merge_sr(w.numpy(), ws.numpy(), noise.numpy(), delta=delta)
        want_dq = O.sr_delta(delta, ws.numpy(), noise.numpy())
    fused = L.lora_merge_sr(w.to(dev), ws.to(dev), noise.to(dev), up=up.to(dev), down=down.to(dev), lora_scale=1.0)
    given = L.lora_merge_sr(w.to(dev), ws.to(dev), noise.to(dev), delta=torch.from_numpy(delta).to(dev))
    dq = L.sr_quant_delta(torch.from_numpy(delta).to(dev), ws.to(dev), noise.to(dev))
    assert np.array_equal(fused.cpu().numpy(), want)
    assert np.array_equal(given.cpu().numpy(), want_given)
    assert np.array_equal(dq.cpu().numpy(), want_dq)
    assert len(np.unique(want_dq)) > 40  # the deltas are not all saturated or all zero


def test_sr_special_noise_values(L, dev):
    x = torch.tensor([[0.5, 0.3, -0.3, 0.26, -0.26, 0.0, 40.0, -40.0]])
    for noise in (torch.zeros(1, 8), torch.full((1, 8), 1 - 2.0**-24), torch.tensor([[0.0, 0.2, 0.8, 0.04, 0.96, 0.5, 0.5, 0.5]])):
        got = L.sr_quant_delta(x.to(dev), 0.25, noise.to(dev)).cpu().numpy()
        assert np.array_equal(got, O.sr_delta(x.numpy(), np.float32(0.25), noise.numpy()))


# ------------------------------------------------------------------ seeded sweeps with generators of their own
def test_lora_merge_matrix_core_form_shape_sweep(L, dev):
    """The matrix-core merge over shapes drawn at random: row counts that leave ragged last blocks and uneven bands,
    one to many column blocks of 256 (K a multiple of 32), every rank it takes, both scale modes."""
    g = torch.Generator().manual_seed(4242)
    rng = np.random.default_rng(4242)
    for case in range(12):
        N = int(rng.integers(1, 2600))
        K = 32 * int(rng.integers(1, 40))
        r = int(rng.choice([4, 8, 16, 32]))
        row = bool(rng.integers(0, 2))
        w = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=g)
        ws = torch.rand(N if row else 1, generator=g) * 0.002 + 0.0005
        up, down = torch.randn(N, r, generator=g) * 0.05, torch.randn(r, K, generator=g) * 0.05
        noise = torch.rand(N, K, generator=g)
        scale = float(rng.choice([1.0, 0.7, -1.3]))
        want = O.lora_merge_sr(w.numpy(), ws.numpy(), noise.numpy(), up=up.numpy(), down=down.numpy(), lora_scale=scale)
        got = L.lora_merge_sr(w.to(dev), ws.to(dev) if row else float(ws[0]), noise.to(dev), up=up.to(dev), down=down.to(dev), lora_scale=scale)
        assert np.array_equal(got.cpu().numpy(), want), f"case {case}: N={N} K={K} r={r} row={row}"


def test_linear_w8a8_k_split_flags_sweep(L, dev):
    """The K split with every epilogue flavour: tensor and row scales, with and without bias, both operation orders,
    an addend, every output dtype; against the oracle."""
    g = torch.Generator().manual_seed(777)
    rng = np.random.default_rng(777)
    dts = [torch.bfloat16, torch.float16, torch.float32]
    for case in range(8):
        M = int(rng.integers(17, 300))
        N = 8 * int(rng.integers(8, 200))
        K = 16 * int(rng.integers(640, 900))
        row, with_bias, order = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), int(rng.integers(0, 2))
        odt = dts[case % 3]
        x = (torch.randn(M, K, generator=g) * 0.5).to(torch.bfloat16)
        wq = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=g)
        ws = torch.rand(N if row else 1, generator=g) * 0.002 + 0.0005
        bias = (torch.randn(N, generator=g) * 0.01).to(dts[(case + 1) % 3]) if with_bias else None
        xa, code = O.from_torch(x)
        ocode = {torch.bfloat16: O.BF16, torch.float16: O.F16, torch.float32: O.F32}[odt]
        ba, bcode = (None, O.BF16) if bias is None else O.from_torch(bias)
        want = O.linear_w8a8(xa, code, wq.numpy(), ws.numpy(), ba, bcode, ocode, 0, order)
        q, s = L.quant_rowwise(x.to(dev))
        assert L._splitk_workspace(q, M, N, K) is not None
        got = L.linear_w8a8(q, s, wq.to(dev), ws.to(dev) if row else float(ws[0]), None if bias is None else bias.to(dev), odt, order)
        assert np.array_equal(bits(got), want), f"case {case}: {M}x{N}x{K} row={row} bias={with_bias} order={order} {odt}"
        if case % 2 == 0:   # and with an addend in the epilogue: bit-equal to adding it afterwards
            add = (torch.randn(M, N, generator=g) * 0.1).to(odt).to(dev)
            fused = L.linear_w8a8(q, s, wq.to(dev), ws.to(dev) if row else float(ws[0]), None if bias is None else bias.to(dev), odt, order, addend=add)
            assert torch.equal(fused, (got + add).to(odt))



@pytest.mark.parametrize("dt,M,shapes,bias,per_row", [
    (torch.bfloat16, 1, [(18432, 3072), (18432, 3072)], True, True), (torch.float16, 16, [(512, 1024), (96, 1024), (2048, 1024)], False, True),
    (torch.bfloat16, 5, [(33, 272), (17, 272)], True, False), (torch.bfloat16, 3, [(64, 256)] * 4, True, True),
    (torch.float32, 4, [(64, 256), (32, 256)], True, True), (torch.bfloat16, 2, [(64, 256)] * 5, False, True),
    (torch.bfloat16, 2, [(64, 200), (64, 264)], True, True),
])
def test_linear_w8a16_small_m_grouped_equals_separate_calls(L, dev, dt, M, shapes, bias, per_row):
    """Several small-batch layers in one launch (the modulation projections of both streams of a block) == the
    separate calls bit for bit: layers of different widths and depths, with and without bias, one weight scale or one
    per row, and the shapes without a grouped kernel (binary32 activations, more than four layers, K % 16 != 0), which
    go layer by layer."""
    g = torch.Generator().manual_seed(71)
    problems = []
    for (N, K) in shapes:
        x = torch.randn(M, K, generator=g).to(dt).to(dev)
        w = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=g).to(dev)
        ws = (torch.rand(N, 1, generator=g) * 0.002 + 1e-3).to(dev) if per_row else 0.0017
        b = torch.randn(N, generator=g).to(dt).to(dev) if bias else None
        problems.append((x, w, ws, b))
    outs = L.linear_w8a16_small_m_grouped(problems)
    assert len(outs) == len(problems)
    for (x, w, ws, b), y in zip(problems, outs):
        want = L.linear_w8a16_small_m(x, w, ws, b)
        assert y.shape == want.shape and y.dtype == want.dtype
        assert torch.equal(y.view(torch.int32) if dt == torch.float32 else y.view(torch.int16), want.view(torch.int32) if dt == torch.float32 else want.view(torch.int16))
