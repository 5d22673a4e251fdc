"""The ComfyUI-facing layer on the GPU: Int8TensorwiseOps.Linear and the INT8 LoRA adapters
produce what the oracle computes from the same inputs."""
import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu
G = torch.Generator().manual_seed(777)


@pytest.fixture(autouse=True)
def reset_flags(pkg):
    ops = pkg.Int8TensorwiseOps
    saved = (list(ops.excluded_names), ops.dynamic_quantize, ops.enable_quarot)
    yield
    ops.excluded_names, ops.dynamic_quantize, ops.enable_quarot = saved


def load(layer, sd, prefix="l."):
    layer._load_from_state_dict(dict(sd), prefix, {}, True, [], [], [])
    return layer


def bits(t):
    return O.from_torch(t.cpu())[0]


@pytest.mark.parametrize("quarot", [False, True])
def test_on_the_fly_quantised_linear_forward(pkg, dev, quarot):
    ops = pkg.Int8TensorwiseOps
    ops.dynamic_quantize, ops.enable_quarot = True, quarot
    w = (torch.randn(384, 512, generator=G) * 0.02).bfloat16()
    b = (torch.randn(384, generator=G) * 0.01).bfloat16()
    lin = load(ops.Linear(512, 384, bias=True), {"l.weight": w, "l.bias": b})
    rb = 128 if quarot else 0
    wq, ws = O.quant_rowwise(w.float().numpy(), O.F32, rb)          # the loader widens to float32 first
    assert lin._is_quantized and lin._is_per_row and lin._use_quarot == quarot
    assert lin.weight.device.type == "cpu" and np.array_equal(lin.weight.numpy(), wq) and np.array_equal(lin.weight_scale.numpy(), ws)

    x = torch.randn(2, 40, 512, generator=G)
    x[..., 5] *= 30
    x = x.bfloat16()
    y = lin(x.to(dev))
    assert y.shape == (2, 40, 384) and y.dtype == torch.bfloat16
    xa, code = O.from_torch(x.reshape(80, 512))
    want = O.linear_w8a8(xa, code, wq, ws, O.from_torch(b)[0], O.BF16, O.BF16, rb)
    assert np.array_equal(bits(y.reshape(80, 384)), want)

    # fp32 activations are computed and returned in bf16; fp16 activations in fp16
    y32 = lin(x.float().to(dev))
    assert y32.dtype == torch.bfloat16
    xa32, _ = O.from_torch(x.float().reshape(80, 512))
    assert np.array_equal(bits(y32.reshape(80, 384)), O.linear_w8a8(xa32, O.F32, wq, ws, O.from_torch(b)[0], O.BF16, O.BF16, rb))
    y16 = lin(x.half().to(dev))
    assert y16.dtype == torch.float16

    # 16 rows or fewer: W8A16 path, output in x's dtype, within the small-batch tolerance
    xs = x[0, :9]
    ys = lin(xs.to(dev))
    xin = O.rotate(O.from_torch(xs)[0], O.BF16) if quarot else O.from_torch(xs)[0]
    ref = O.to_f32(O.linear_w8a16(xin, O.BF16, wq, ws, O.from_torch(b)[0], O.BF16), O.BF16)
    got = ys.float().cpu().numpy()
    assert ys.shape == (9, 384) and (np.abs(got - ref) <= 2.0**-7 * np.abs(ref) + 2.0**-8 * np.abs(ref).max()).all()


def test_prequantised_tensorwise_linear_forward(pkg, dev):
    wf = torch.randn(256, 384, generator=G) * 0.02
    wq, ws = O.quant_tensorwise(wf.numpy(), O.F32)
    lin = load(pkg.Int8TensorwiseOps.Linear(384, 256, bias=False),
               {"l.weight": torch.from_numpy(wq), "l.weight_scale": torch.tensor(float(ws[0]))})
    x = torch.randn(33, 384, generator=G).bfloat16()
    y = lin.to(dev)(x.to(dev))
    xa, code = O.from_torch(x)
    assert np.array_equal(bits(y), O.linear_w8a8(xa, code, wq, ws))


def test_dynamic_lora_side_branch(pkg, dev):
    wq = torch.randint(-128, 128, (64, 128), dtype=torch.int8, generator=G)
    lin = load(pkg.Int8TensorwiseOps.Linear(128, 64, bias=False), {"l.weight": wq, "l.weight_scale": torch.rand(64, 1) * 0.01}).to(dev)
    x = torch.randn(20, 128, generator=G).bfloat16().to(dev)
    base = lin(x)
    lin.lora_A, lin.lora_B = torch.randn(4, 128, generator=G).bfloat16(), torch.randn(64, 4, generator=G).bfloat16()
    withl = lin(x)
    side = torch.nn.functional.linear(torch.nn.functional.linear(x, lin.lora_A.to(dev)), lin.lora_B.to(dev))
    assert torch.equal(withl, base + side.to(base.dtype))


def test_set_weight_requantises_a_float_patch_with_the_layers_scale(pkg, dev):
    wq = torch.randint(-100, 100, (32, 64), dtype=torch.int8, generator=G)
    ws = torch.rand(32, 1, generator=G) * 0.01 + 0.001
    lin = load(pkg.Int8TensorwiseOps.Linear(64, 32, bias=False), {"l.weight": wq, "l.weight_scale": ws})
    patched = wq.float() * ws + 0.0004                                 # what a float fallback would hand over
    noise = torch.rand(32, 64, generator=G)
    want = O.sr_delta(patched.numpy(), ws.numpy(), noise.numpy())
    got = pkg.stochastic_round_int8_delta(patched.to(dev), ws, noise=noise)
    assert np.array_equal(got.cpu().numpy(), want)
    out = lin.set_weight(patched, seed=3, return_weight=True)           # device-drawn noise: check the bracket only
    assert out.dtype == torch.int8 and out.device.type == "cpu"
    xs = patched / ws
    assert ((out.float() - torch.floor(xs)).abs() <= 1).all()


@pytest.mark.parametrize("quarot", [False, True])
@pytest.mark.parametrize("fused", [True, False])
def test_lora_patch_adapter_merges_like_the_oracle(pkg, dev, quarot, fused):
    ops = pkg.Int8TensorwiseOps
    ops.enable_quarot = quarot
    N, K, r = 192, 256, 8
    wq = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=G)
    ws = torch.rand(N, 1, generator=G) * 0.002 + 0.0005
    up, down = torch.randn(N, r, generator=G) * 0.05, torch.randn(r, K, generator=G) * 0.05
    ad = pkg.INT8LoRAPatchAdapter({"k"}, (up, down, 4.0, None, None, None), ws, seed=318008)
    ad.fuse_low_rank = fused
    out = ad.calculate_weight(wq, "k", 0.8, 1.0, None, None)
    assert out.dtype == torch.int8 and out.device == wq.device and out.shape == wq.shape
    noise = pkg.int8_quant._draw_noise((N, K), 318008, dev).cpu()      # the adapter's own draw
    mult = (4.0 / r) * 0.8
    if fused:
        dn = O.rotate(down.numpy(), O.F32) if quarot else down.numpy()
        want = O.lora_merge_sr(wq.numpy(), ws.numpy(), noise.numpy(), up=up.numpy(), down=dn, lora_scale=mult)
        assert np.array_equal(out.numpy(), want)
    else:   # delta comes from a device BLAS product: compare against the oracle fed with that very delta
        delta = (torch.mm(up.to(dev), down.to(dev)) * mult).cpu()
        if quarot:
            delta = torch.from_numpy(O.rotate(delta.numpy(), O.F32))
        want = O.lora_merge_sr(wq.numpy(), ws.numpy(), noise.numpy(), delta=delta.numpy())
        assert np.array_equal(out.numpy(), want)
    # narrowed weight (fused QKV): ComfyUI hands over the slice and its LoRA, the scale is still the full tensor
    sl = slice(64, 128)
    ad_q = pkg.INT8LoRAPatchAdapter({"k"}, (up[sl], down, 4.0, None, None, None), ws, seed=318008)
    ad_ref = pkg.INT8LoRAPatchAdapter({"k"}, (up[sl], down, 4.0, None, None, None), ws[sl], seed=318008)
    ad_q.fuse_low_rank = ad_ref.fuse_low_rank = fused
    part = ad_q.calculate_weight(wq[sl].contiguous(), "k", 0.8, 1.0, (0, 64, 64), None)
    assert torch.equal(part, ad_ref.calculate_weight(wq[sl].contiguous(), "k", 0.8, 1.0, None, None))
    assert not torch.equal(part, wq[sl])


def test_merged_adapter_sums_deltas_then_rounds_once(pkg, dev):
    N, K = 96, 128
    wq = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=G)
    ws = torch.rand(N, 1, generator=G) * 0.002 + 0.0005
    mk = lambda r: (torch.randn(N, r, generator=G) * 0.05, torch.randn(r, K, generator=G) * 0.05, float(r), None, None, None)
    a1, a2 = pkg.INT8LoRAPatchAdapter({"a"}, mk(4), ws), pkg.INT8LoRAPatchAdapter({"b"}, mk(8), ws)
    merged = pkg.INT8MergedLoRAPatchAdapter([(a1, 0.5), (a2, -0.25)], ws, seed=11)
    out = merged.calculate_weight(wq, "k", 1.0, 1.0, None, None)
    total = (torch.mm(a1.weights[0].to(dev), a1.weights[1].to(dev)) * 0.5)
    total += torch.mm(a2.weights[0].to(dev), a2.weights[1].to(dev)) * -0.25
    noise = pkg.int8_quant._draw_noise((N, K), 11, dev).cpu()
    want = O.lora_merge_sr(wq.numpy(), ws.numpy(), noise.numpy(), delta=total.cpu().numpy())
    assert np.array_equal(out.numpy(), want)
    # float weights take the float branch
    wf = torch.randn(N, K, generator=G)
    outf = merged.calculate_weight(wf, "k", 1.0, 1.0, None, None)
    assert outf.dtype == torch.float32 and not torch.equal(outf, wf)


def test_quantize_helpers_on_device(pkg, dev):
    x = (torch.randn(40, 96, generator=G) * 0.02).bfloat16()
    q, s = pkg.quantize_int8_tensorwise(x.to(dev))
    qo, so = O.quant_tensorwise(O.from_torch(x)[0], O.BF16)
    assert s.dim() == 0 and np.array_equal(q.cpu().numpy(), qo) and float(s) == float(so[0])
    x3 = torch.randn(3, 5, 64, generator=G).to(dev)
    q3, s3 = pkg.quantize_int8_axiswise(x3, dim=-1)
    qo3, so3 = O.quant_rowwise(x3.cpu().reshape(15, 64).numpy(), O.F32)
    assert s3.shape == (3, 5, 1) and np.array_equal(q3.cpu().numpy().reshape(15, 64), qo3)
    r = pkg.quarot.rotate_activation(x3[..., :128].contiguous() if x3.shape[-1] >= 128 else torch.randn(2, 3, 128, device=dev))
    assert r.shape[-1] == 128


@pytest.mark.parametrize("rows", [64, 8])
def test_forward_under_hip_graph_replays_like_eager(pkg, dev, rows):
    """The library allocates nothing, synchronises nothing and launches on the caller's stream, so a
    forward can be captured in a HIP graph.  Every replay, with new input contents and eager work in
    between, must give the eager result bit for bit."""
    ops = pkg.Int8TensorwiseOps
    ops.dynamic_quantize, ops.enable_quarot = True, True
    w = (torch.randn(256, 384, generator=G) * 0.02).bfloat16()
    b = (torch.randn(256, generator=G) * 0.01).bfloat16()
    lin = load(ops.Linear(384, 256, bias=True), {"l.weight": w, "l.bias": b}).to(dev)
    static_x = torch.zeros(rows, 384, dtype=torch.bfloat16, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            lin(static_x)                       # warm-up outside the capture (library load, device check)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = lin(static_x)
    for i in range(4):
        x = torch.randn(rows, 384, generator=G).bfloat16().to(dev) * (i + 1)
        want = lin(x)                           # eager work between the replays
        torch.cuda.synchronize()
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y.view(torch.int16), want.view(torch.int16)), f"replay {i}"


@pytest.mark.parametrize("rows,quarot", [(40, False), (40, True), (6, True)])
def test_dynamic_lora_side_branch_is_added_like_the_reference(pkg, dev, rows, quarot):
    """lora_A / lora_B set: y = y + ((x @ A.T) @ B.T * alpha).to(y.dtype), the sum formed inside the GEMM
    epilogue on the W8A8 path (int8_quant.py:762-774)."""
    ops = pkg.Int8TensorwiseOps
    ops.dynamic_quantize, ops.enable_quarot = True, quarot
    w = (torch.randn(256, 384, generator=G) * 0.02).bfloat16()
    b = (torch.randn(256, generator=G) * 0.01).bfloat16()
    lin = load(ops.Linear(384, 256, bias=True), {"l.weight": w, "l.bias": b}).to(dev)
    x = torch.randn(rows, 384, generator=G).bfloat16().to(dev)
    plain = lin(x)
    A = (torch.randn(16, 384, generator=G) * 0.05).bfloat16().to(dev)
    B = (torch.randn(256, 16, generator=G) * 0.05).bfloat16().to(dev)
    lin.lora_A, lin.lora_B, lin.lora_alpha = A, B, 0.5
    got = lin(x)
    x_side = pkg._lib.rotate128(x) if quarot else x
    side = torch.nn.functional.linear(torch.nn.functional.linear(x_side, A), B) * 0.5
    want = plain + side.to(plain.dtype)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_dynamic_lora_hook_drives_the_side_branch(pkg, dev):
    """transformer_options["dynamic_loras"] -> hook -> lora_A / lora_B of the layer -> forward with the side branch
    (int8_quant.py:415-507 feeding :762-774)."""
    dl = pkg.dynamic_lora

    class Tiny(torch.nn.Module):
        def __init__(self, lin):
            super().__init__()
            self.proj = lin

        def forward(self, x, transformer_options=None):
            return self.proj(x)

    wq = torch.randint(-128, 128, (64, 128), dtype=torch.int8, generator=G)
    lin = load(pkg.Int8TensorwiseOps.Linear(128, 64, bias=False), {"l.weight": wq, "l.weight_scale": torch.rand(64, 1) * 0.01})
    model = Tiny(lin).to(dev)
    x = torch.randn(40, 128, generator=G).bfloat16().to(dev)
    base = model(x)

    class Adapter:
        def __init__(self, up, down, alpha):
            self.weights = (up, down, alpha, None, None, None)

    up, down = (torch.randn(64, 4, generator=G) * 0.1).bfloat16(), (torch.randn(4, 128, generator=G) * 0.1).bfloat16()
    options = {}
    dl.append_entry(options, "a", 0.5, {"diffusion_model.proj.weight": Adapter(up, down, 8.0)})
    dl.DynamicLoRAHook.register(model)
    got = model(x, transformer_options=options["transformer_options"])
    a_dev = (down * (8.0 / 4 * 0.5)).to(dev)
    side = torch.nn.functional.linear(torch.nn.functional.linear(x, a_dev), up.to(dev))
    assert model.proj.lora_A.device.type == "cuda"
    assert torch.equal(got, base + side.to(base.dtype))
    assert torch.equal(model(x), base)                     # no entries in this call: the branch is gone again


def test_forward_with_a_prologue_equals_the_unfused_sequence(pkg, dev):
    """forward(x, prologue=...) against the same layer fed the tensor torch computes first: bit-identical for the
    modulation, within one step of the output dtype for the GELU (whose last binary32 bits differ from torch's)."""
    import torch.nn.functional as F
    L = pkg._lib
    g = torch.Generator().manual_seed(21)
    lin = pkg.Int8TensorwiseOps.Linear(384, 96, bias=True)
    lin._load_from_state_dict({"l.weight": torch.randint(-127, 128, (96, 384), dtype=torch.int8, generator=g),
                               "l.weight_scale": torch.rand(96, 1, generator=g) * 0.002 + 1e-3,
                               "l.bias": torch.randn(96, generator=g).bfloat16()}, "l.", {}, True, [], [], [])
    lin = lin.to(dev)
    x = torch.randn(2, 20, 384, generator=g).bfloat16().to(dev)
    sc, sh = (torch.randn(2, 1, 384, generator=g) * 0.3).bfloat16().to(dev), torch.randn(2, 1, 384, generator=g).bfloat16().to(dev)
    for quarot in (False, True):
        lin._use_quarot = quarot
        a = lin(x, prologue=L.PRO_MODULATE, mod_scale=sc, mod_shift=sh)
        b = lin((1 + sc) * x + sh)
        assert a.shape == (2, 20, 96) and torch.equal(a, b)
        a = lin(x, prologue=L.PRO_GELU_TANH)
        b = lin(F.gelu(x, approximate="tanh"))
        assert (a.float() - b.float()).abs().max() <= 2.0**-7 * b.float().abs().max()
        gate = torch.randn(2, 20, 384, generator=g).bfloat16().to(dev)
        a = lin(x, prologue=L.PRO_SILU_GATE, mod_scale=gate)
        b = lin(F.silu(x) * gate)
        assert (a.float() - b.float()).abs().max() <= 2.0**-7 * b.float().abs().max()
        wide = x[..., :256].contiguous()                                       # cat((a, gelu(b)), -1): 256 + 128 features
        tail = torch.randn(2, 20, 128, generator=g).bfloat16().to(dev)
        a = lin(wide, prologue=L.PRO_CONCAT_GELU, mod_scale=tail)
        b = lin(torch.cat((wide, F.gelu(tail, approximate="tanh")), -1))
        assert a.shape == (2, 20, 96) and (a.float() - b.float()).abs().max() <= 2.0**-7 * b.float().abs().max()
        a = lin(x, prologue=L.PRO_NORM_MODULATE, mod_scale=sc, mod_shift=sh, eps=1e-6)   # the whole adaLN producer
        b = lin((1 + sc) * F.layer_norm(x, (384,), eps=1e-6) + sh)
        assert a.shape == (2, 20, 96) and (a.float() - b.float()).abs().max() <= 2.0**-6 * b.float().abs().max()
        assert (a != b).float().mean().item() <= 0.2
        a = lin(x, prologue=L.PRO_MODULATE, mod_scale=sc, mod_shift=sh, fused_add=True)     # the one-kernel spelling of the modulation
        assert torch.equal(a, lin(torch.addcmul(sh, x, 1 + sc))) and torch.equal(a, lin(x, prologue=L.PRO_MODULATE_FUSED, mod_scale=sc, mod_shift=sh))
        a = lin(x, prologue=L.PRO_NORM_MODULATE, mod_scale=sc, mod_shift=sh, eps=1e-6, fused_add=True)
        b = lin(torch.addcmul(sh, F.layer_norm(x, (384,), eps=1e-6), 1 + sc))
        assert (a.float() - b.float()).abs().max() <= 2.0**-6 * b.float().abs().max() and (a != b).float().mean().item() <= 0.2
        a = lin(x, prologue=L.PRO_GELU_ERF)
        b = lin(F.gelu(x))
        assert (a.float() - b.float()).abs().max() <= 2.0**-7 * b.float().abs().max()
        nw = (torch.randn(384, generator=g) * 0.2 + 1).bfloat16().to(dev)
        for w_, s_, t_ in ((nw, sc, None), (None, sc, sh), (nw, None, None)):   # z-image's and ltx's producers, a bare RMSNorm
            a = lin(x, prologue=L.PRO_RMS_NORM, norm_weight=w_, mod_scale=s_, mod_shift=t_, eps=1e-5)
            h = F.rms_norm(x, (384,), w_, 1e-5)
            h = h if s_ is None else h * (1 + s_)
            b = lin(h if t_ is None else h + t_)
            assert a.shape == (2, 20, 96) and (a.float() - b.float()).abs().max() <= 2.0**-6 * b.float().abs().max()
            assert (a != b).float().mean().item() <= 0.2
    # vectors that torch would broadcast differently, or of another dtype, are left to torch: same result as the
    # unfused expression (a [1, T, K] vector against a batch of 2 must not be dealt over the rows as if it were [2, 1, K])
    lin._use_quarot = False
    per_token = (torch.randn(1, 20, 384, generator=g) * 0.3).bfloat16().to(dev)
    assert torch.equal(lin(x, prologue=L.PRO_MODULATE, mod_scale=per_token, mod_shift=per_token), lin((1 + per_token) * x + per_token))
    sc32, sh32 = sc.float(), sh.float()
    assert torch.equal(lin(x, prologue=L.PRO_MODULATE, mod_scale=sc32, mod_shift=sh32), lin((1 + sc32) * x + sh32))
    small = x[:1, :4]                     # four rows: the W8A16 path applies the operation in torch
    assert torch.equal(lin(small, prologue=L.PRO_GELU_TANH), lin(F.gelu(small, approximate="tanh")))
    assert torch.equal(lin(small, prologue=L.PRO_NORM_MODULATE, mod_scale=sc[:1], mod_shift=sh[:1], eps=1e-5),
                       lin((1 + sc[:1]) * F.layer_norm(small, (384,), eps=1e-5) + sh[:1]))
    assert torch.equal(lin(small, prologue=L.PRO_RMS_NORM, norm_weight=nw, mod_scale=sc[:1], eps=1e-5),
                       lin(F.rms_norm(small, (384,), nw, 1e-5) * (1 + sc[:1])))
    assert torch.equal(lin(x, prologue=L.PRO_RMS_NORM, norm_weight=nw.float(), eps=1e-5), lin(F.rms_norm(x, (384,), nw.float(), 1e-5)))
    assert torch.equal(lin(small, prologue=L.PRO_GELU_ERF), lin(F.gelu(small)))
    assert torch.equal(lin(small, prologue=L.PRO_MODULATE, mod_scale=sc[:1], mod_shift=sh[:1], fused_add=True), lin(torch.addcmul(sh[:1], small, 1 + sc[:1])))
    assert torch.equal(lin(x.float(), prologue=L.PRO_MODULATE_FUSED, mod_scale=sc.float(), mod_shift=sh.float()),
                       lin(torch.addcmul(sh.float(), x.float(), 1 + sc.float())))
    # rows that the normalising quantiser does not take (binary32 here): torch normalises, and the result is that of
    # the unfused expression
    x32, sc_, sh_ = x.float(), sc.float(), sh.float()
    assert torch.equal(lin(x32, prologue=L.PRO_NORM_MODULATE, mod_scale=sc_, mod_shift=sh_), lin((1 + sc_) * F.layer_norm(x32, (384,), eps=1e-6) + sh_))


def test_forward_with_gate_and_residual_equals_the_unfused_sequence(pkg, dev):
    """forward(h, gate=g, residual=x) == x + g * forward(h) bit for bit (two torch operations of the compute dtype, formed
    inside the GEMM epilogue), with either one alone, combined with a prologue, on the QuaRot path, and on every path
    that leaves the operations to torch (small batch, a gate torch would broadcast differently, binary32 residual)."""
    L = pkg._lib
    g = torch.Generator().manual_seed(23)
    lin = pkg.Int8TensorwiseOps.Linear(384, 256, bias=True)
    lin._load_from_state_dict({"l.weight": torch.randint(-127, 128, (256, 384), dtype=torch.int8, generator=g),
                               "l.weight_scale": torch.rand(256, 1, generator=g) * 0.002 + 1e-3,
                               "l.bias": torch.randn(256, generator=g).bfloat16()}, "l.", {}, True, [], [], [])
    lin = lin.to(dev)
    h = torch.randn(2, 40, 384, generator=g).bfloat16().to(dev)
    x = torch.randn(2, 40, 256, generator=g).bfloat16().to(dev)
    gate = torch.randn(2, 1, 256, generator=g).bfloat16().to(dev)
    sc, sh = (torch.randn(2, 1, 384, generator=g) * 0.3).bfloat16().to(dev), torch.randn(2, 1, 384, generator=g).bfloat16().to(dev)
    for quarot in (False, True):
        lin._use_quarot = quarot
        y = lin(h)
        assert torch.equal(lin(h, gate=gate, residual=x), x + gate * y)
        assert torch.equal(lin(h, gate=gate), gate * y)
        assert torch.equal(lin(h, residual=x), x + y)
        assert torch.equal(lin(h, gate=gate.reshape(2, 256)[0], residual=x), x + gate.reshape(2, 256)[0] * y)   # one vector for all rows
        ym = lin(h, prologue=L.PRO_MODULATE, mod_scale=sc, mod_shift=sh)
        assert torch.equal(lin(h, prologue=L.PRO_MODULATE, mod_scale=sc, mod_shift=sh, gate=gate, residual=x), x + gate * ym)
    lin._use_quarot = False
    y = lin(h)
    per_token = torch.randn(1, 40, 256, generator=g).bfloat16().to(dev)      # torch broadcasts this over the batch, not over the tokens
    assert torch.equal(lin(h, gate=per_token, residual=x), x + per_token * y)
    assert torch.equal(lin(h, gate=gate, residual=x.float()), x.float() + gate * y)
    small = h[:1, :4]
    assert torch.equal(lin(small, gate=gate[:1], residual=x[:1, :4]), x[:1, :4] + gate[:1] * lin(small))


@pytest.mark.parametrize("quarot", [False, True])
def test_forward_pair_equals_the_layers_own_forward(pkg, dev, quarot):
    """forward_pair: the same projection of two token streams with their own weights, activations quantised in one
    launch, bit-identical to calling each layer; layers that cannot share the launch (a small batch) fall back."""
    g = torch.Generator().manual_seed(31)

    def layer(n, k):
        lin = pkg.Int8TensorwiseOps.Linear(k, n, bias=True)
        lin._load_from_state_dict({"l.weight": torch.randint(-127, 128, (n, k), dtype=torch.int8, generator=g),
                                   "l.weight_scale": torch.rand(n, 1, generator=g) * 0.002 + 1e-3,
                                   "l.bias": torch.randn(n, generator=g).bfloat16()}, "l.", {}, True, [], [], [])
        lin._use_quarot = quarot
        return lin.to(dev)
    img, txt = layer(192, 384), layer(192, 384)
    x_img = torch.randn(2, 100, 384, generator=g).bfloat16().to(dev)
    x_txt = torch.randn(2, 20, 384, generator=g).bfloat16().to(dev)
    y_img, y_txt = pkg.forward_pair([img, txt], [x_img, x_txt])
    assert y_img.shape == (2, 100, 192) and y_txt.shape == (2, 20, 192)
    assert torch.equal(y_img, img(x_img)) and torch.equal(y_txt, txt(x_txt))
    small = x_txt[:1, :3]                                  # three rows: that stream takes the W8A16 path, so no shared launch
    y_img2, y_small = pkg.forward_pair([img, txt], [x_img, small])
    assert torch.equal(y_img2, y_img) and torch.equal(y_small, txt(small))
    # the residual update of both streams in the same launch: x + gate * layer(h) per stream, gate for one stream only,
    # and a pair that falls back (the small batch) with its gates applied by torch
    r_img, r_txt = torch.randn(2, 100, 192, generator=g).bfloat16().to(dev), torch.randn(2, 20, 192, generator=g).bfloat16().to(dev)
    g_img, g_txt = torch.randn(2, 1, 192, generator=g).bfloat16().to(dev), torch.randn(2, 1, 192, generator=g).bfloat16().to(dev)
    o_img, o_txt = pkg.forward_pair([img, txt], [x_img, x_txt], gates=[g_img, g_txt], residuals=[r_img, r_txt])
    assert torch.equal(o_img, r_img + g_img * y_img) and torch.equal(o_txt, r_txt + g_txt * y_txt)
    o_img, o_txt = pkg.forward_pair([img, txt], [x_img, x_txt], gates=[g_img, None], residuals=[None, r_txt])
    assert torch.equal(o_img, g_img * y_img) and torch.equal(o_txt, r_txt + y_txt)
    o_img, o_small = pkg.forward_pair([img, txt], [x_img, small], gates=[g_img, g_txt[:1]], residuals=[r_img, r_txt[:1, :3]])
    assert torch.equal(o_img, r_img + g_img * y_img) and torch.equal(o_small, r_txt[:1, :3] + g_txt[:1] * txt(small))


@pytest.mark.parametrize("quarot", [False, True])
def test_forward_fanout_equals_the_layers_own_forward(pkg, dev, quarot):
    """forward_fanout: layers that read the same activations (q, k, v of different widths) on ONE quantisation, bit-identical
    to calling each layer; with a prologue applied inside that one quantiser (an RMSNorm with scale-only modulation in
    front of a SwiGLU's two up-projections) bit-identical to each layer's own forward with that prologue; fall-backs
    (a small batch, a layer with another rotation flag) give the layers' own results."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(37)
    L = pkg._lib

    def layer(n, k, per_row=True):
        lin = pkg.Int8TensorwiseOps.Linear(k, n, bias=True)
        lin._load_from_state_dict({"l.weight": torch.randint(-127, 128, (n, k), dtype=torch.int8, generator=g),
                                   "l.weight_scale": (torch.rand(n, 1, generator=g) * 0.002 + 1e-3) if per_row else torch.tensor(0.0021),
                                   "l.bias": torch.randn(n, generator=g).bfloat16()}, "l.", {}, True, [], [], [])
        lin._use_quarot = quarot
        return lin.to(dev)
    q, k, v = layer(192, 384), layer(96, 384, per_row=False), layer(64, 384)
    x = torch.randn(2, 50, 384, generator=g).bfloat16().to(dev)
    outs = pkg.forward_fanout([q, k, v], x)
    assert [tuple(o.shape) for o in outs] == [(2, 50, 192), (2, 50, 96), (2, 50, 64)]
    assert all(torch.equal(o, lin(x)) for o, lin in zip(outs, (q, k, v)))
    nw = (torch.randn(384, generator=g) * 0.2 + 1).bfloat16().to(dev)
    sc = (torch.randn(2, 1, 384, generator=g) * 0.3).bfloat16().to(dev)
    outs = pkg.forward_fanout([q, v], x, prologue=L.PRO_RMS_NORM, norm_weight=nw, mod_scale=sc, eps=1e-5)
    assert all(torch.equal(o, lin(x, prologue=L.PRO_RMS_NORM, norm_weight=nw, mod_scale=sc, eps=1e-5)) for o, lin in zip(outs, (q, v)))
    h = F.rms_norm(x, (384,), nw, 1e-5) * (1 + sc)
    assert all((o.float() - lin(h).float()).abs().max() <= 2.0**-6 * lin(h).float().abs().max() for o, lin in zip(outs, (q, v)))
    small = x[:1, :5]
    assert all(torch.equal(o, lin(small)) for o, lin in zip(pkg.forward_fanout([q, k], small), (q, k)))
    vec = x[:, 0]                                      # [2, 384]: the small-batch kernels of all three layers in one launch
    outs = pkg.forward_fanout([q, k, v], vec)
    assert [tuple(o.shape) for o in outs] == [(2, 192), (2, 96), (2, 64)] and all(torch.equal(o, lin(vec)) for o, lin in zip(outs, (q, k, v)))
    k._use_quarot = not quarot
    assert all(torch.equal(o, lin(x)) for o, lin in zip(pkg.forward_fanout([q, k], x), (q, k)))
    per_token = (torch.randn(1, 50, 384, generator=g) * 0.3).bfloat16().to(dev)      # a scale torch would broadcast differently
    outs = pkg.forward_fanout([q, v], x, prologue=L.PRO_RMS_NORM, norm_weight=nw, mod_scale=per_token, eps=1e-5)
    assert all(torch.equal(o, lin(F.rms_norm(x, (384,), nw, 1e-5) * (1 + per_token))) for o, lin in zip(outs, (q, v)))
