"""Seeded random shapes, dtypes and flags for every entry point, each case checked against the CPU oracle.

The hand-picked cases of test_gpu_parity.py sit on the boundaries that the kernels' tilings are known to have;
these draws look for boundaries nobody thought of.  Every family owns its generators, so adding or removing a
test elsewhere never changes what is drawn here.  Bars are those of test_gpu_parity.py: bit-exact for all integer
outputs, scales and the W8A8 linear's floating-point outputs; the spacing bound for the small-batch W8A16 path.
"""
import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu

DTS = [torch.bfloat16, torch.float16, torch.float32]
CODE = {torch.bfloat16: O.BF16, torch.float16: O.F16, torch.float32: O.F32}
CASES = 120


def gens(seed):
    return np.random.default_rng(seed), torch.Generator().manual_seed(seed)


def pick(rng, seq):
    return seq[int(rng.integers(0, len(seq)))]


def raw(t):
    return O.from_torch(t.cpu())[0]


def same(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    if a.dtype == np.float32:
        a, b = a.view(np.uint32), np.asarray(b, dtype=np.float32).view(np.uint32)
    return a.shape == b.shape and np.array_equal(a, b)


def check(bad):
    assert not bad, f"{len(bad)} of {CASES} draws differ from the oracle: {bad[:6]}"


def test_random_quant_rowwise(L, dev):
    """Plain and rotated row quantisation (int8_quant.py:59-70, 115-131) at arbitrary M and K, rows of zeros among them."""
    rng, g = gens(101)
    bad = []
    for _ in range(CASES):
        dt, rot = pick(rng, DTS), bool(rng.integers(0, 2))
        M = int(rng.integers(1, 700))
        K = 128 * int(rng.integers(1, 40)) if rot else int(rng.integers(1, 5000))
        x = (torch.randn(M, K, generator=g) * pick(rng, [1e-3, 1.0, 50.0])).to(dt)
        if rng.integers(0, 4) == 0:
            x[int(rng.integers(0, M))] = 0
        xa, code = O.from_torch(x)
        qo, so = O.quant_rowwise(xa, code, 128 if rot else 0)
        q, s = L.quant_rowwise(x.to(dev), rotate=rot)
        if not (same(q.cpu().numpy(), qo) and same(s.cpu().numpy().reshape(-1), so.reshape(-1))):
            bad.append((M, K, dt, rot))
    check(bad)


def test_random_quant_rowwise_modulate(L, dev):
    """(1 + scale) x + shift in front of the quantiser, one vector pair per group of consecutive rows."""
    rng, g = gens(102)
    bad = []
    for _ in range(CASES):
        dt, rot = pick(rng, DTS), bool(rng.integers(0, 2))
        V, per = int(rng.integers(1, 4)), int(rng.integers(1, 200))
        M = V * per
        K = 128 * int(rng.integers(1, 40)) if rot else int(rng.integers(1, 4000))
        x = torch.randn(M, K, generator=g).to(dt)
        sc, sh = ((torch.randn(V, K, generator=g) * 0.3).to(dt) for _ in range(2))
        xa, code = O.from_torch(x)
        mod = O.prologue(xa, code, O.PRO_MODULATE, O.from_torch(sc)[0], O.from_torch(sh)[0], rows_per_vec=per)
        qo, so = O.quant_rowwise(mod, code, 128 if rot else 0)
        q, s = L.quant_rowwise(x.to(dev), rotate=rot, prologue=L.PRO_MODULATE, mod_scale=sc.to(dev), mod_shift=sh.to(dev))
        if not (same(q.cpu().numpy(), qo) and same(s.cpu().numpy().reshape(-1), so.reshape(-1))):
            bad.append((M, K, V, dt, rot))
    check(bad)


def test_random_rotate_and_tensorwise(L, dev):
    """The stand-alone block rotation (int8_quant.py:115-131) and the whole-tensor quantiser (int8_quant.py:46-57),
    the latter through both of its scratch variants."""
    rng, g = gens(103)
    bad = []
    for _ in range(CASES):
        dt = pick(rng, DTS)
        M, K = int(rng.integers(1, 300)), 128 * int(rng.integers(1, 30))
        x = torch.randn(M, K, generator=g).to(dt)
        xa, code = O.from_torch(x)
        if not same(raw(L.rotate128(x.to(dev))), O.rotate(xa, code)):
            bad.append(("rotate", M, K, dt))
        n = int(rng.integers(1, 300000))
        v = (torch.randn(n, generator=g) * 0.02).to(dt)
        va, code = O.from_torch(v)
        qo, so = O.quant_tensorwise(va, code)
        q, s = L.quant_tensorwise(v.to(dev), static_scratch=bool(rng.integers(0, 2)))
        if not (same(q.cpu().numpy().reshape(-1), qo.reshape(-1)) and same(s.cpu().numpy().reshape(1), np.asarray(so, dtype=np.float32).reshape(1))):
            bad.append(("tensorwise", n, dt))
    check(bad)


def linear_case(L, dev, rng, g, M, N, K, with_addend):
    row, order, odt = bool(rng.integers(0, 2)), int(rng.integers(0, 2)), pick(rng, DTS)
    x = (torch.randn(M, K, generator=g) * 0.5).to(torch.bfloat16)
    wq = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=g)
    ws = torch.rand(N if row else 1, generator=g) * 0.002 + 0.0005
    bias = (torch.randn(N, generator=g) * 0.01).to(pick(rng, DTS)) if rng.integers(0, 2) else None
    xa, code = O.from_torch(x)
    ba, bcode = (None, O.BF16) if bias is None else O.from_torch(bias)
    want = O.linear_w8a8(xa, code, wq.numpy(), ws.numpy(), ba, bcode, CODE[odt], 0, order)
    q, s = L.quant_rowwise(x.to(dev))
    wsa = ws.to(dev) if row else float(ws[0])
    bd = None if bias is None else bias.to(dev)
    got = L.linear_w8a8(q, s, wq.to(dev), wsa, bd, odt, order)
    ok = same(raw(got), want)
    if ok and with_addend:     # the fused residual equals torch's own addition of the two rounded tensors
        add = (torch.randn(M, N, generator=g) * 0.3).to(odt).to(dev)
        ok = torch.equal(L.linear_w8a8(q, s, wq.to(dev), wsa, bd, odt, order, addend=add), got + add)
    return ok, (M, N, K, row, order, odt, None if bias is None else bias.dtype)


def test_random_linear_w8a8(L, dev):
    """W8A8 linear (int8_quant.py:73-104, int8_fused_kernel.py:285-318), ragged M, N and K, both epilogue orders,
    every bias and output dtype, with and without a residual addend."""
    rng, g = gens(104)
    bad = []
    for case in range(CASES):
        M = int(rng.integers(1, 1200))
        N = 8 * int(rng.integers(1, 400)) if rng.integers(0, 5) else int(rng.integers(1, 900))
        K = 16 * int(rng.integers(1, 40)) if rng.integers(0, 5) else int(rng.integers(1, 500))
        ok, what = linear_case(L, dev, rng, g, M, N, K, case % 3 == 0)
        if not ok:
            bad.append(what)
    check(bad)


def test_random_linear_w8a8_long_k(L, dev):
    """Few output tiles under a long K: the shapes whose K range the library may divide among workgroups."""
    rng, g = gens(105)
    bad = []
    for case in range(CASES):
        M, N, K = int(rng.integers(1, 200)), 8 * int(rng.integers(1, 160)), 16 * int(rng.integers(640, 1100))
        ok, what = linear_case(L, dev, rng, g, M, N, K, case % 3 == 0)
        if not ok:
            bad.append(what)
    check(bad)


def test_random_linear_w8a8_large(L, dev):
    """Outputs of hundreds of 256-row tiles, ragged on every side: the one-workgroup-per-CU configurations
    (256x256, 256x192, 288x256, 256x288 and the rounds they are chosen by), which the draws above seldom reach."""
    rng, g = gens(108)
    bad, tiles = [], set()
    for case in range(32):
        M, N, K = int(rng.integers(900, 6000)), 8 * int(rng.integers(100, 1700)), 16 * int(rng.integers(1, 130))
        tiles.add(L.gemm_tile(M, N, K)[:2])
        ok, what = linear_case(L, dev, rng, g, M, N, K, case % 4 == 0)
        if not ok:
            bad.append(what)
    assert not bad, f"{len(bad)} of 32 draws differ from the oracle: {bad[:6]}"
    assert len(tiles) >= 4, tiles


def test_random_small_m_w8a16(L, dev):
    """Small-batch W8A16 (int8_quant.py:666-674): |y - y_ref| <= spacing(y_ref) + K 2^-24 sum |x||w|."""
    rng, g = gens(106)
    bad = []
    for _ in range(CASES):
        dt = pick(rng, DTS[:2])
        M, N = int(rng.integers(1, 17)), int(rng.integers(1, 3000))
        K = 16 * int(rng.integers(1, 300)) if rng.integers(0, 4) else int(rng.integers(1, 2000))
        x = torch.randn(M, K, generator=g).to(dt)
        wq = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=g)
        ws = torch.rand(N, generator=g) * 0.01 + 0.001
        xa, code = O.from_torch(x)
        ref = O.to_f32(O.linear_w8a16(xa, code, wq.numpy(), ws.numpy()), code)
        got = L.linear_w8a16_small_m(x.to(dev), wq.to(dev), ws.to(dev), None).float().cpu().numpy()
        mant = 7 if dt == torch.bfloat16 else 10
        sp = np.ldexp(1.0, np.floor(np.log2(np.maximum(np.abs(ref), 2.0 ** -126))).astype(np.int64) - mant)
        mag = (x.double().abs() @ (wq.float() * ws.reshape(-1, 1)).to(dt).double().abs().T).numpy()
        if not (np.abs(got - ref) <= sp + K * 2.0 ** -24 * mag + 1e-30).all():
            bad.append((M, N, K, dt))
    check(bad)


def test_random_stochastic_rounding_and_merge(L, dev):
    """Stochastic rounding of a given delta (int8_quant.py:161-170), the merge of a given delta and the merge of a
    low-rank product (int8_dynamic_lora.py:321-338), all ranks and ragged shapes, both scale layouts."""
    rng, g = gens(107)
    bad = []
    for _ in range(CASES):
        row = bool(rng.integers(0, 2))
        N, K = int(rng.integers(1, 800)), int(rng.integers(1, 1200))
        d = torch.randn(N, K, generator=g) * pick(rng, [0.01, 1.0, 300.0])
        ws = torch.rand(N if row else 1, generator=g) * 0.02 + 0.0005
        noise = torch.rand(N, K, generator=g)
        w = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=g)
        wsa = ws.to(dev) if row else float(ws[0])
        if not same(L.sr_quant_delta(d.to(dev), wsa, noise.to(dev)).cpu().numpy(), O.sr_delta(d.numpy(), ws.numpy(), noise.numpy())):
            bad.append(("sr", N, K, row))
        if not same(L.lora_merge_sr(w.to(dev), wsa, noise.to(dev), delta=d.to(dev)).cpu().numpy(),
                    O.lora_merge_sr(w.numpy(), ws.numpy(), noise.numpy(), delta=d.numpy())):
            bad.append(("merge delta", N, K, row))
        r = pick(rng, [1, 3, 4, 8, 16, 32, 64])
        N = int(rng.integers(1, 1500))
        K = 32 * int(rng.integers(1, 30)) if rng.integers(0, 3) else int(rng.integers(1, 900))
        sc = pick(rng, [1.0, 0.7, -1.3])
        w = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=g)
        ws = torch.rand(N if row else 1, generator=g) * 0.002 + 0.0005
        up, down = torch.randn(N, r, generator=g) * 0.05, torch.randn(r, K, generator=g) * 0.05
        noise = torch.rand(N, K, generator=g)
        got = L.lora_merge_sr(w.to(dev), ws.to(dev) if row else float(ws[0]), noise.to(dev), up=up.to(dev), down=down.to(dev), lora_scale=sc)
        if not same(got.cpu().numpy(), O.lora_merge_sr(w.numpy(), ws.numpy(), noise.numpy(), up=up.numpy(), down=down.numpy(), lora_scale=sc)):
            bad.append(("merge lora", N, K, r, row, sc))
    check(bad)
