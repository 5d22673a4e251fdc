"""torch.library registration of the forward path: schemas and shape-only implementations on the CPU,
Dynamo tracing of Linear.forward without graph breaks, the graph rewrite that moves the elementwise
operation in front of a layer into its quantiser, and (GPU) the compiled forward (aot_eager and
inductor) against eager and against the CPU oracle."""
import numpy as np
import operator

import pytest
import torch
import torch.nn.functional as F


def _load(lin, sd, prefix="l."):
    lin._load_from_state_dict({prefix + k: v for k, v in sd.items()}, prefix, {}, True, [], [], [])
    return lin


def _per_row_layer(pkg, n=64, k=256, bias=True, quarot=False):
    lin = pkg.Int8TensorwiseOps.Linear(k, n, bias=bias)
    sd = {"weight": torch.randint(-127, 128, (n, k), dtype=torch.int8), "weight_scale": torch.rand(n, 1) * 0.01 + 1e-3}
    if bias:
        sd["bias"] = torch.randn(n).bfloat16()
    _load(lin, sd)
    lin._use_quarot = quarot
    return lin


def test_operators_are_registered_with_the_expected_schemas(pkg):
    for name in pkg.compile_ops.OPS:
        assert hasattr(torch.ops.i8f, name)
    s = str(torch.ops.i8f.int8_linear.default._schema)
    assert "Tensor? weight_scale" in s and "float weight_scale_value" in s and "ScalarType compute_dtype" in s
    assert str(torch.ops.i8f.quantize_rowwise.default._schema).endswith("-> (Tensor, Tensor)")


def test_shape_only_implementations(pkg):
    ops = torch.ops.i8f
    x = torch.empty(3, 7, 256, dtype=torch.float16, device="meta")
    w = torch.empty(96, 256, dtype=torch.int8, device="meta")
    ws = torch.empty(96, 1, device="meta")
    b = torch.empty(96, dtype=torch.float16, device="meta")
    y = ops.int8_linear(x, w, ws, 0.0, b, torch.float16, False, 0)
    assert y.shape == (3, 7, 96) and y.dtype == torch.float16
    y = ops.int8_linear(x, w, None, 0.02, None, torch.bfloat16, True, 1)
    assert y.shape == (3, 7, 96) and y.dtype == torch.bfloat16
    y = ops.int8_linear(x, w, None, 0.02, None, torch.bfloat16, True, 1, torch.empty(3, 7, 96, dtype=torch.bfloat16, device="meta"))
    assert y.shape == (3, 7, 96)
    q, s = ops.quantize_rowwise(x.reshape(21, 256), True)
    assert q.shape == (21, 256) and q.dtype == torch.int8 and s.shape == (21, 1) and s.dtype == torch.float32
    y = ops.linear_w8a8(q, s, w, ws, 0.0, None, torch.float32, 0)
    assert y.shape == (21, 96) and y.dtype == torch.float32
    y = ops.linear_w8a16_small_m(x[:1, :4], w, ws, 0.0, b, False)
    assert y.shape == (1, 4, 96) and y.dtype == torch.float16
    assert ops.rotate128(x.reshape(21, 256)).shape == (21, 256)
    y = ops.int8_linear_lora(x, w, ws, 0.0, b, torch.float16, False, 0, torch.empty(21, 8, dtype=torch.float16, device="meta"),
                             torch.empty(96, 8, dtype=torch.float16, device="meta"), 0.5)
    assert y.shape == (3, 7, 96) and y.dtype == torch.float16
    q, s = ops.quantize_rowwise_prologue(x, False, pkg._lib.PRO_GELU_ERF, None, None)
    assert q.shape == (21, 256) and q.dtype == torch.int8 and s.shape == (21, 1)
    q, s = ops.quantize_rowwise_prologue(x, False, pkg._lib.PRO_CONCAT_GELU, torch.empty(3, 7, 128, dtype=torch.float16, device="meta"), None)
    assert q.shape == (21, 384)
    y = ops.linear_w8a8(q[:, :256], s, w, ws, 0.0, None, torch.float16, 0, torch.empty(21, 96, dtype=torch.float16, device="meta"), b)
    assert y.shape == (21, 96)
    with pytest.raises(Exception):
        ops.quantize_rowwise(x, False)     # 3-D input is rejected by the shape function as by the library


def test_split_scale(pkg):
    t = torch.ones(4, 1)
    assert pkg.compile_ops.split_scale(t) == (t, 0.0)
    assert pkg.compile_ops.split_scale(0.25) == (None, 0.25)


@pytest.mark.parametrize("rows,op", [(32, "int8_linear"), (4, "linear_w8a16_small_m")])
def test_forward_traces_into_one_operator_without_graph_breaks(pkg, rows, op):
    """Dynamo export traces with fake tensors only, so it runs without a GPU; a graph break would raise."""
    lin = _per_row_layer(pkg, quarot=True)
    x = torch.randn(2, rows // 2, 256).bfloat16()
    gm = torch._dynamo.export(lin)(x).graph_module
    targets = [str(n.target) for n in gm.graph.nodes if n.op == "call_function"]
    assert any(op in t for t in targets), targets
    assert not any("rotate128" in t for t in targets)          # rotation is folded into the operator
    other = "linear_w8a16_small_m" if op == "int8_linear" else "int8_linear"
    assert not any(other in t for t in targets)


class _ModulatedMlp(torch.nn.Module):
    """The MLP branch of a DiT block: adaLN modulation -> up projection -> tanh-GELU -> down projection."""

    def __init__(self, up, down):
        super().__init__()
        self.up, self.down = up, down

    def forward(self, x, scale, shift):
        h = (1 + scale) * x + shift
        return self.down(F.gelu(self.up(h), approximate="tanh"))


def _mlp(pkg, k=256, hidden=512):
    g = torch.Generator().manual_seed(11)
    layers = []
    for n_out, k_in in ((hidden, k), (k, hidden)):
        lin = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=True)
        _load(lin, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                    "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3, "bias": (torch.randn(n_out, generator=g) * 0.1).bfloat16()})
        layers.append(lin)
    return _ModulatedMlp(*layers)


def test_graph_rewrite_moves_modulation_and_gelu_into_the_quantiser(pkg):
    m = _mlp(pkg)
    x, sc, sh = torch.randn(2, 24, 256).bfloat16(), torch.randn(2, 1, 256).bfloat16(), torch.randn(2, 1, 256).bfloat16()
    gm = torch._dynamo.export(m)(x, sc, sh).graph_module
    assert pkg.compile_ops.fuse_prologues(gm) == 2
    calls = [n for n in gm.graph.nodes if n.op == "call_function"]
    fused = [n for n in calls if "int8_linear_prologue" in str(n.target)]
    assert [n.args[1] for n in fused] == [pkg._lib.PRO_MODULATE, pkg._lib.PRO_GELU_TANH]
    assert not any("gelu" in str(n.target) or n.target.__name__ in ("add", "mul") for n in calls if hasattr(n.target, "__name__"))
    assert not any(str(n.target).endswith("int8_linear") for n in calls)


def test_graph_rewrite_leaves_other_producers_alone(pkg):
    m = _mlp(pkg)

    class Other(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.m = m

        def forward(self, x, scale, shift):
            h = (1 + scale) * x + shift            # scale has one vector per TOKEN here: not the adaLN broadcast
            g = F.gelu(self.m.up(h))               # exact (erf) GELU: not the tanh form
            return self.m.down(g) + g.sum()        # and its result is used twice
    x, sc, sh = torch.randn(2, 24, 256).bfloat16(), torch.randn(2, 24, 256).bfloat16(), torch.randn(2, 24, 256).bfloat16()
    gm = torch._dynamo.export(Other())(x, sc, sh).graph_module
    assert pkg.compile_ops.fuse_prologues(gm) == 0


def test_graph_rewrite_respects_views_and_the_callers_shape(pkg):
    """A view between the producer and the layer that regroups the FEATURE dimension is not walked through (the
    quantiser would see rows of another length), and a direct 3-D caller of the operator keeps its 3-D result."""
    m = _mlp(pkg, k=256, hidden=512)
    ops = torch.ops.i8f

    class Regrouped(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.up = m.up

        def forward(self, x):                      # x [4, 24, 128]: gelu on rows of 128, the layer on rows of 256
            return self.up(F.gelu(x, approximate="tanh").reshape(4, 12, 256))

    gm = torch._dynamo.export(Regrouped())(torch.randn(4, 24, 128).bfloat16()).graph_module
    assert pkg.compile_ops.fuse_prologues(gm) == 0

    class Direct(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.w = torch.nn.Parameter(m.up.weight.data, requires_grad=False)
            self.ws = torch.nn.Parameter(m.up.weight_scale.data, requires_grad=False)

        def forward(self, x):                      # the operator called on a 3-D tensor, as its schema allows
            return ops.int8_linear(F.gelu(x, approximate="tanh"), self.w, self.ws, 0.0, None, torch.bfloat16, False, 0)

    x = torch.randn(2, 24, 256).bfloat16()
    gm = torch._dynamo.export(Direct())(x).graph_module
    assert pkg.compile_ops.fuse_prologues(gm) == 1
    outs = [n for n in gm.graph.nodes if n.op == "output"][0].args[0]
    out = outs[0] if isinstance(outs, (tuple, list)) else outs
    assert "int8_linear_prologue" in str(out.target), "no reshape to 2-D is put behind a 3-D caller's operator"
    fake = torch._subclasses.FakeTensorMode()
    with fake:
        y = ops.int8_linear_prologue(torch.empty(2, 24, 256, dtype=torch.bfloat16), 2, None, None, torch.empty(512, 256, dtype=torch.int8),
                                     torch.empty(512, 1), 0.0, None, torch.bfloat16, False, 0)
    assert tuple(y.shape) == (2, 24, 512)


def test_graph_rewrite_moves_the_swiglu_gate_into_the_quantiser(pkg):
    """w2(silu(w1 x) * w3 x): the product feeding the down projection becomes its prologue, in either operand order;
    a gate of another shape (broadcast by torch) is left alone."""
    g = torch.Generator().manual_seed(12)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=False)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3})

    class SwiGlu(torch.nn.Module):
        def __init__(self, flip):
            super().__init__()
            self.w1, self.w3, self.w2, self.flip = lin(512, 256), lin(512, 256), lin(256, 512), flip

        def forward(self, x):
            a, b = self.w1(x), self.w3(x)
            return self.w2(b * F.silu(a) if self.flip else F.silu(a) * b)

    x = torch.randn(2, 24, 256).bfloat16()
    for flip in (False, True):
        gm = torch._dynamo.export(SwiGlu(flip))(x).graph_module
        assert pkg.compile_ops.fuse_prologues(gm) == 1
        fused = [n for n in gm.graph.nodes if n.op == "call_function" and "int8_linear_prologue" in str(n.target)]
        assert len(fused) == 1 and fused[0].args[1] == pkg._lib.PRO_SILU_GATE and fused[0].args[3] is None
        assert not any("silu" in str(n.target) for n in gm.graph.nodes if n.op == "call_function")

    class Broadcast(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.w1, self.w2 = lin(512, 256), lin(256, 512)

        def forward(self, x, gate):                      # gate [512]: not a tensor of the activation's shape
            return self.w2(F.silu(self.w1(x)) * gate)
    gm = torch._dynamo.export(Broadcast())(x, torch.randn(512).bfloat16()).graph_module
    assert pkg.compile_ops.fuse_prologues(gm) == 0


def test_graph_rewrite_moves_layer_norm_and_modulation_into_the_quantiser(pkg):
    """(1 + scale) * LayerNorm(h) + shift -> linear, the adaLN producer of a DiT block: LayerNorm without affine goes into
    the quantiser together with the modulation (with its eps); a LayerNorm with affine parameters, one that is used
    elsewhere too, or rows wider than the registers hold (16384) stay torch's and only the modulation is fused."""
    g = torch.Generator().manual_seed(13)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=False)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3})

    class Block(torch.nn.Module):
        def __init__(self, k, affine=False, reuse=False):
            super().__init__()
            self.norm = torch.nn.LayerNorm(k, elementwise_affine=affine, eps=1e-6).bfloat16()
            self.qkv, self.reuse = lin(64, k), reuse

        def forward(self, x, scale, shift):
            h = self.norm(x)
            y = self.qkv((1 + scale) * h + shift)
            return y + h.sum() if self.reuse else y

    def fused_nodes(mod, k):
        x, v = torch.randn(2, 24, k).bfloat16(), torch.randn(2, 1, k).bfloat16()
        gm = torch._dynamo.export(mod)(x, v, v).graph_module
        assert pkg.compile_ops.fuse_prologues(gm) == 1
        nodes = [n for n in gm.graph.nodes if n.op == "call_function" and "int8_linear_prologue" in str(n.target)]
        assert len(nodes) == 1
        return nodes[0], any("layer_norm" in str(n.target) for n in gm.graph.nodes if n.op == "call_function")

    node, ln_left = fused_nodes(Block(256), 256)
    assert node.args[1] == pkg._lib.PRO_NORM_MODULATE and not ln_left and abs(node.args[-1] - 1e-6) < 1e-12
    for mod, k in ((Block(256, affine=True), 256), (Block(256, reuse=True), 256), (Block(16400), 16400)):
        node, ln_left = fused_nodes(mod, k)
        assert node.args[1] == pkg._lib.PRO_MODULATE and ln_left


def test_graph_rewrite_moves_rms_norm_and_exact_gelu_into_the_quantiser(pkg):
    """rms_norm(h, w) * (1 + scale) -> linear (z-image's modulate(norm(x), scale)), (1 + scale) * rms_norm(h) + shift ->
    linear (ltx), a bare rms_norm -> linear, and gelu(h) in its exact form -> linear: all become the layer's prologue,
    the weight of the norm travelling as the operator's norm_weight; an RMSNorm whose weight has another dtype, one used
    elsewhere too, or rows wider than the registers hold (16384) stay torch's."""
    g = torch.Generator().manual_seed(14)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=False)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3})

    class Block(torch.nn.Module):
        def __init__(self, k, form, wdt=torch.bfloat16):
            super().__init__()
            self.norm = torch.nn.RMSNorm(k, eps=1e-5, elementwise_affine=form != "ltx").to(wdt)
            self.qkv, self.form = lin(64, k), form

        def forward(self, x, scale, shift):
            h = self.norm(x)
            if self.form == "zimage":
                return self.qkv(h * (1 + scale))
            if self.form == "ltx":
                return self.qkv(h * (1 + scale) + shift)
            if self.form == "reuse":
                return self.qkv(h * (1 + scale)) + h.sum()
            return self.qkv(h)

    def rewrite(mod, k):
        x, v = torch.randn(2, 24, k).bfloat16(), torch.randn(2, 1, k).bfloat16()
        gm = torch._dynamo.export(mod)(x, v, v).graph_module
        n = pkg.compile_ops.fuse_prologues(gm)
        nodes = [n_ for n_ in gm.graph.nodes if n_.op == "call_function" and "int8_linear_prologue" in str(n_.target)]
        return n, nodes, any("rms_norm" in str(n_.target) for n_ in gm.graph.nodes if n_.op == "call_function")

    for form, has_w, has_s, has_t in (("zimage", True, True, False), ("ltx", False, True, True), ("bare", True, False, False)):
        n, nodes, norm_left = rewrite(Block(256, form), 256)
        assert n == 1 and len(nodes) == 1 and not norm_left
        node = nodes[0]
        assert node.args[1] == pkg._lib.PRO_RMS_NORM and abs(node.args[11] - 1e-5) < 1e-12
        assert (node.kwargs.get("norm_weight") is not None) == has_w
        assert (node.args[2] is not None) == has_s and (node.args[3] is not None) == has_t
    for mod, k in ((Block(256, "zimage", torch.float32), 256), (Block(256, "reuse"), 256), (Block(16400, "zimage"), 16400)):
        n, nodes, norm_left = rewrite(mod, k)
        assert n == 0 and norm_left

    class Mlp(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.up, self.down = lin(128, 64), lin(64, 128)

        def forward(self, x):
            return self.down(F.gelu(self.up(x)))

    gm = torch._dynamo.export(Mlp())(torch.randn(2, 24, 64).bfloat16()).graph_module
    assert pkg.compile_ops.fuse_prologues(gm) == 1
    node = [n_ for n_ in gm.graph.nodes if n_.op == "call_function" and "int8_linear_prologue" in str(n_.target)][0]
    assert node.args[1] == pkg._lib.PRO_GELU_ERF
    assert not any(n_.target is F.gelu for n_ in gm.graph.nodes if n_.op == "call_function")


def test_graph_rewrite_takes_the_addcmul_spelling_of_the_modulation(pkg):
    """torch.addcmul(shift, norm(x), 1 + scale) -> linear, the modulation as one torch kernel (product and sum rounded once):
    fused with the flag that keeps that rounding, behind a LayerNorm without affine, an RMSNorm or no norm at all, the
    factors in either order; another `value`, binary32 tensors or a gain that is not 1 + scale stay torch's."""
    g = torch.Generator().manual_seed(26)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=False)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3})

    class Block(torch.nn.Module):
        def __init__(self, norm, form="plain"):
            super().__init__()
            self.norm = {"ln": torch.nn.LayerNorm(128, elementwise_affine=False, eps=1e-6), "rms": torch.nn.RMSNorm(128, eps=1e-5).bfloat16(),
                         "none": torch.nn.Identity()}[norm]
            self.qkv, self.form = lin(64, 128), form

        def forward(self, x, scale, shift):
            h = self.norm(x)
            if self.form == "swapped":
                z = torch.addcmul(shift, 1 + scale, h)
            elif self.form == "value":
                z = torch.addcmul(shift, h, 1 + scale, value=2)
            elif self.form == "gain":
                z = torch.addcmul(shift, h, scale)
            else:
                z = torch.addcmul(shift, h, 1 + scale)
            return self.qkv(z)

    x, v = torch.randn(2, 24, 128).bfloat16(), torch.randn(2, 1, 128).bfloat16()
    for norm, form, kind in (("ln", "plain", "PRO_NORM_MODULATE"), ("rms", "plain", "PRO_RMS_NORM"), ("none", "plain", "PRO_MODULATE"),
                             ("ln", "swapped", "PRO_NORM_MODULATE")):
        gm = torch._dynamo.export(Block(norm, form))(x, v, v).graph_module
        assert pkg.compile_ops.fuse_prologues(gm) == 1
        node = [n for n in gm.graph.nodes if n.op == "call_function" and "int8_linear_prologue" in str(n.target)][0]
        assert node.args[1] == getattr(pkg._lib, kind) and node.kwargs.get("fused_add") is True
        assert not any(n.target is torch.addcmul for n in gm.graph.nodes if n.op == "call_function")
    for norm, form in (("ln", "value"), ("ln", "gain")):
        gm = torch._dynamo.export(Block(norm, form))(x, v, v).graph_module
        assert pkg.compile_ops.fuse_prologues(gm) == 0
    gm = torch._dynamo.export(Block("none"))(x.float(), v.float(), v.float()).graph_module
    assert pkg.compile_ops.fuse_prologues(gm) == 0


def test_graph_rewrite_moves_concatenation_and_gelu_into_the_quantiser(pkg):
    """linear2(cat((attn, gelu(mlp)), -1)), the second projection of a single-stream block: both producers become the
    layer's prologue; a concatenation along another dimension, of three tensors, or with an exact GELU stays torch's."""
    g = torch.Generator().manual_seed(15)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=False)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3})

    class Single(torch.nn.Module):
        def __init__(self, form):
            super().__init__()
            self.linear2, self.form = lin(128, 128 + 512 if form != 2 else 128 + 512 + 128), form

        def forward(self, attn, mlp):
            if self.form == 0:
                z = torch.cat((attn, F.gelu(mlp, approximate="tanh")), 2)
            elif self.form == 1:
                z = torch.cat((attn, F.gelu(mlp)), -1)                       # exact GELU
            else:
                z = torch.cat((attn, F.gelu(mlp, approximate="tanh"), attn), -1)
            return self.linear2(z)

    attn, mlp = torch.randn(2, 24, 128).bfloat16(), torch.randn(2, 24, 512).bfloat16()
    for form, fused in ((0, 1), (1, 0), (2, 0)):
        gm = torch._dynamo.export(Single(form))(attn, mlp).graph_module
        assert pkg.compile_ops.fuse_prologues(gm) == fused
        nodes = [n for n in gm.graph.nodes if n.op == "call_function" and "int8_linear_prologue" in str(n.target)]
        assert len(nodes) == fused
        if fused:
            assert nodes[0].args[1] == pkg._lib.PRO_CONCAT_GELU
            assert not any(n.target in (torch.cat, F.gelu) for n in gm.graph.nodes if n.op == "call_function")


def test_graph_rewrite_gives_layers_that_read_one_tensor_a_single_quantiser(pkg):
    """Separate q, k, v projections of one tensor: one quantize_rowwise and three GEMM operators instead of three
    int8_linear.  A SwiGLU feed-forward behind an RMSNorm with modulation, w2(silu(w1(h)) * w3(h)) with
    h = norm(x) * (1 + scale): w1 and w3 share one quantiser, which takes the norm and the modulation as its prologue
    (the normalised tensor never exists), and w2 takes the gate as its own; layers with different rotation flags, or a
    single layer, are left alone."""
    g = torch.Generator().manual_seed(18)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=False)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3})

    def calls(gm, name):
        return [n for n in gm.graph.nodes if n.op == "call_function" and str(n.target).split(".")[-2 if str(n.target).endswith("default") else -1] == name]

    class Qkv(torch.nn.Module):
        def __init__(self, rot_k=False):
            super().__init__()
            self.q, self.k, self.v = lin(64, 128), lin(64, 128), lin(32, 128)
            self.k._use_quarot = rot_k

        def forward(self, x):
            return self.q(x) + self.k(x), self.v(x)

    x = torch.randn(2, 24, 128).bfloat16()
    gm = torch._dynamo.export(Qkv())(x).graph_module
    assert pkg.compile_ops.share_quantisation(gm) == 3
    assert len(calls(gm, "quantize_rowwise")) == 1 and len(calls(gm, "linear_w8a8")) == 3 and not calls(gm, "int8_linear")
    out = gm.graph.find_nodes(op="output")[0]
    shapes = [tuple(pkg.compile_ops._meta_val(n).shape) for n in out.args[0]]
    assert shapes == [(2, 24, 64), (2, 24, 32)]
    gm = torch._dynamo.export(Qkv(rot_k=True))(x).graph_module     # k reads rotated activations: q and v share, k stays
    assert pkg.compile_ops.share_quantisation(gm) == 2
    assert len(calls(gm, "quantize_rowwise")) == 1 and len(calls(gm, "linear_w8a8")) == 2 and len(calls(gm, "int8_linear")) == 1

    class SwiGlu(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.norm = torch.nn.RMSNorm(128, eps=1e-5).bfloat16()
            self.w1, self.w3, self.w2 = lin(256, 128), lin(256, 128), lin(128, 256)

        def forward(self, x, scale):
            h = self.norm(x) * (1 + scale)
            return self.w2(F.silu(self.w1(h)) * self.w3(h))

    gm = torch._dynamo.export(SwiGlu())(x, torch.randn(2, 1, 128).bfloat16()).graph_module
    assert pkg.compile_ops.share_quantisation(gm) == 2
    assert pkg.compile_ops.fuse_prologues(gm) == 2
    quant = calls(gm, "quantize_rowwise_prologue")
    assert len(quant) == 1 and quant[0].args[2] == pkg._lib.PRO_RMS_NORM and quant[0].args[3] is not None and quant[0].args[6] is not None
    assert len(calls(gm, "linear_w8a8")) == 2 and not calls(gm, "quantize_rowwise")
    down = calls(gm, "int8_linear_prologue")
    assert len(down) == 1 and down[0].args[1] == pkg._lib.PRO_SILU_GATE
    assert not any("rms_norm" in str(n.target) or n.target in (operator.mul, F.silu) for n in gm.graph.nodes if n.op == "call_function")


def test_graph_rewrite_takes_the_in_place_residual_update_where_nobody_can_tell(pkg):
    """`txt += gate * proj(h)`, the in-place spelling of the residual update: folded into the layer's epilogue when txt is
    an intermediate of the graph that nothing reads afterwards except through the update's result; left to torch (with
    only the gate folded in) when txt is a graph input, a slice of something else, or read again after the update."""
    g = torch.Generator().manual_seed(24)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=False)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3})

    class Block(torch.nn.Module):
        def __init__(self, form):
            super().__init__()
            self.proj, self.form = lin(64, 64), form

        def forward(self, x, h, gate):
            if self.form == "input":
                txt = x
            elif self.form == "slice":
                txt = torch.cat((x, x), 1)[:, :24]
            else:
                txt = x + 1.0
            before = txt.sum() if self.form == "read_before" else None
            keep = txt                                   # the same tensor: sees the update in eager mode
            txt += gate * self.proj(h)
            out = txt * 2.0
            if self.form == "read_after":
                return out, keep.mean()
            return (out, before) if before is not None else out

    x, h, gate = torch.randn(2, 24, 64).bfloat16(), torch.randn(2, 24, 64).bfloat16(), torch.randn(2, 1, 64).bfloat16()
    for form, with_residual in (("fresh", True), ("read_before", True), ("input", False), ("slice", False), ("read_after", False)):
        gm = torch._dynamo.export(Block(form))(x, h, gate).graph_module
        assert pkg.compile_ops.fuse_epilogues(gm) == 1
        node = [n for n in gm.graph.nodes if n.op == "call_function" and "int8_linear" in str(n.target)][0]
        assert node.kwargs.get("gate") is not None and (node.kwargs.get("addend") is not None) == with_residual, form
        assert any(n.target is operator.iadd for n in gm.graph.nodes if n.op == "call_function") == (not with_residual), form


def test_installed_pass_rewrites_a_graph_and_steps_aside_when_a_rewrite_raises(pkg, monkeypatch):
    """compile_ops.install_inductor_pass(): the function it registers with inductor rewrites a graph that holds this
    package's operators, leaves other graphs alone, chains to a pass that was registered before it, and compiles a graph
    as it is when a rewrite raises on it (tried on a copy first)."""
    import torch._inductor.config as inductor_config
    g = torch.Generator().manual_seed(28)
    lin = pkg.Int8TensorwiseOps.Linear(64, 128, bias=False)
    _load(lin, {"weight": torch.randint(-127, 128, (128, 64), dtype=torch.int8, generator=g), "weight_scale": torch.rand(128, 1, generator=g) * 0.002 + 1e-3})

    class Mlp(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.up = lin

        def forward(self, x):
            return self.up(F.gelu(x, approximate="tanh"))

    seen = []
    monkeypatch.setattr(inductor_config, "pre_grad_custom_pass", lambda graph: seen.append("earlier pass"))
    monkeypatch.setattr(pkg.compile_ops, "_installed", False)
    assert pkg.compile_ops.install_inductor_pass()
    hook = inductor_config.pre_grad_custom_pass
    x = torch.randn(2, 24, 64).bfloat16()
    gm = torch._dynamo.export(Mlp())(x).graph_module
    hook(gm.graph)
    assert seen == ["earlier pass"] and pkg.compile_ops.LAST_PASS_COUNTS == (0, 1, 0)
    assert any("int8_linear_prologue" in str(n.target) for n in gm.graph.nodes)
    other = torch._dynamo.export(torch.nn.GELU())(x).graph_module           # no operator of this package: untouched
    before = [str(n.target) for n in other.graph.nodes]
    hook(other.graph)
    assert [str(n.target) for n in other.graph.nodes] == before
    gm = torch._dynamo.export(Mlp())(x).graph_module
    before = [str(n.target) for n in gm.graph.nodes]

    def broken(_gm):
        raise RuntimeError("a graph this rewrite was not written for")

    monkeypatch.setattr(pkg.compile_ops, "fuse_prologues", broken)
    hook(gm.graph)
    assert [str(n.target) for n in gm.graph.nodes] == before


def test_graph_rewrites_keep_away_from_in_place_writes(pkg):
    """A tensor overwritten in place between the point where the model reads it and the layer that would read it inside
    a fused operator: the rewrites leave that stretch of the graph alone (the fused read would see the new value)."""
    g = torch.Generator().manual_seed(20)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=False)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3})

    class Mlp(torch.nn.Module):
        def __init__(self, clobber):
            super().__init__()
            self.up, self.down, self.clobber = lin(128, 64), lin(64, 128), clobber

        def forward(self, x):
            h = self.up(x)
            a = F.gelu(h, approximate="tanh")
            if self.clobber:
                h.mul_(2.0)
            return self.down(a), h

    class Qk(torch.nn.Module):
        def __init__(self, clobber):
            super().__init__()
            self.q, self.k, self.clobber = lin(64, 64), lin(64, 64), clobber

        def forward(self, x):
            x = x * 1.0
            a = self.q(x)
            if self.clobber:
                x += 1.0
            return a, self.k(x)

    x = torch.randn(2, 24, 64).bfloat16()
    for clobber, fused in ((False, 1), (True, 0)):
        gm = torch._dynamo.export(Mlp(clobber))(x).graph_module
        assert pkg.compile_ops.fuse_prologues(gm) == fused
        gm = torch._dynamo.export(Qk(clobber))(x).graph_module
        assert pkg.compile_ops.share_quantisation(gm) == 2 * fused


def test_graph_rewrite_moves_the_gated_residual_into_the_epilogue(pkg):
    """x + gate * proj(h), the residual update of an adaLN-Zero block: multiplication and addition become the layer's
    epilogue (in any operand order); the gate alone and the residual alone are taken too; a gate of another dtype, a
    result that is used elsewhere as well, or a residual that torch would broadcast are left to torch."""
    g = torch.Generator().manual_seed(14)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=False)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3})

    class Block(torch.nn.Module):
        def __init__(self, form):
            super().__init__()
            self.proj, self.form = lin(256, 128), form

        def forward(self, x, h, gate):
            y = self.proj(h)
            if self.form == 0:
                return x + gate * y
            if self.form == 1:
                return y * gate + x
            if self.form == 2:
                return gate * y
            if self.form == 3:
                return x + y
            if self.form == 4:
                return x + gate.float() * y          # promotes: torch's business
            if self.form == 5:
                return x + gate * y + y.mean()         # the layer's result has another user
            return x[:, :1] + gate * y               # a residual that broadcasts

    x, h, gate = torch.randn(2, 24, 256).bfloat16(), torch.randn(2, 24, 128).bfloat16(), torch.randn(2, 1, 256).bfloat16()
    for form, want in ((0, (True, True)), (1, (True, True)), (2, (True, False)), (3, (False, True)), (4, None), (5, None), (6, (True, False))):
        gm = torch._dynamo.export(Block(form))(x, h, gate).graph_module
        n = pkg.compile_ops.fuse_epilogues(gm)
        lins = [nd for nd in gm.graph.nodes if nd.op == "call_function" and "int8_linear" in str(nd.target)]
        assert len(lins) == 1
        if want is None:
            assert n == 0 and lins[0].kwargs.get("gate") is None and lins[0].kwargs.get("addend") is None
            continue
        assert n == 1
        assert (lins[0].kwargs.get("gate") is not None, lins[0].kwargs.get("addend") is not None) == want
        left = [str(nd.target) for nd in gm.graph.nodes if nd.op == "call_function" and nd.target in (operator.mul, operator.add, torch.mul, torch.add)]
        assert len(left) == (1 if form == 6 else 0), left     # (form 6 keeps its broadcasting addition)


def test_modulation_broadcast_rule(pkg):
    ok = pkg.compile_ops.modulation_broadcasts_over_tokens
    x = torch.empty(2, 24, 256, dtype=torch.bfloat16)
    v = lambda *shape, dt=torch.bfloat16: torch.empty(*shape, dtype=dt)
    assert ok(x, v(2, 1, 256), v(2, 1, 256)) and ok(x, v(256), v(256))
    assert not ok(x, v(1, 24, 256), v(1, 24, 256))          # one vector per token of ONE image, broadcast over the batch
    assert not ok(x, v(1, 1, 256), v(1, 1, 256))            # batch 2 against one pair of vectors: torch broadcasts, rows do not split
    assert not ok(x, v(2, 1, 256, dt=torch.float32), v(2, 1, 256, dt=torch.float32))
    assert not ok(x, v(2, 1, 256), v(256))
    assert ok(torch.empty(1, 24, 256, dtype=torch.bfloat16), v(1, 1, 256), v(1, 1, 256))


def _oracle_linear(O, x2d, lin):
    xa, code = O.from_torch(x2d)
    return O.linear_w8a8(xa, code, lin.weight.cpu().numpy(), lin.weight_scale.cpu().numpy().reshape(-1),
                         O.from_torch(lin.bias.cpu())[0], O.BF16, O.BF16, 0)


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [48, 8])
def test_inductor_compiled_forward_equals_the_oracle(pkg, dev, O, rows):
    """Linear.forward under torch.compile(backend="inductor", fullgraph=True), plus an elementwise consumer that
    inductor generates code for, against the CPU oracle (W8A8 rows bit for bit; the W8A16 rows within the bound
    of that path)."""
    m = _mlp(pkg).to(dev)
    lin = m.up
    x = torch.randn(rows, 256, generator=torch.Generator().manual_seed(5)).bfloat16()

    def fn(t):
        return lin(t) * 2

    got = torch.compile(fn, backend="inductor", fullgraph=True)(x.to(dev))
    if rows > 16:
        want = O.to_f32(_oracle_linear(O, x, lin), O.BF16) * 2        # doubling a bf16 value is exact
        assert np.array_equal(got.float().cpu().numpy(), want)
    else:
        xa, code = O.from_torch(x)
        ref = O.to_f32(O.linear_w8a16(xa, code, lin.weight.cpu().numpy(), lin.weight_scale.cpu().numpy().reshape(-1),
                                      O.from_torch(lin.bias.cpu())[0], code), code) * 2
        assert (np.abs(got.float().cpu().numpy() - ref) <= 2.0**-7 * np.abs(ref) + 1e-3).all()


@pytest.mark.gpu
def test_compiled_mlp_with_fused_prologues_equals_the_oracle(pkg, dev, O):
    """Modulation -> up -> GELU -> down compiled with the rewriting backend over inductor: the first layer is
    bit-identical to the oracle (modulation restated operation for operation), the second, whose GELU differs from
    the C library's in the last bits of binary32, within two bf16 ulps of the output scale."""
    m = _mlp(pkg).to(dev)
    g = torch.Generator().manual_seed(6)
    x = torch.randn(2, 24, 256, generator=g).bfloat16()
    sc, sh = (torch.randn(2, 1, 256, generator=g) * 0.3).bfloat16(), torch.randn(2, 1, 256, generator=g).bfloat16()
    seen = []

    def counting(gm, inputs):
        seen.append(sum("int8_linear_prologue" in str(n.target) for n in gm.graph.nodes))
        from torch._dynamo.backends.registry import lookup_backend
        return lookup_backend("inductor")(gm, inputs)

    got = torch.compile(m, backend=pkg.compile_ops.backend(counting), fullgraph=True)(x.to(dev), sc.to(dev), sh.to(dev))
    assert seen == [2]
    xa, code = O.from_torch(x.reshape(48, 256))
    h = O.prologue(xa, code, O.PRO_MODULATE, O.from_torch(sc.reshape(2, 256))[0], O.from_torch(sh.reshape(2, 256))[0], rows_per_vec=24)
    y1 = O.linear_w8a8(h, code, m.up.weight.cpu().numpy(), m.up.weight_scale.cpu().numpy().reshape(-1),
                       O.from_torch(m.up.bias.cpu())[0], O.BF16, O.BF16, 0)
    assert np.array_equal(O.from_torch(m.up((1 + sc.to(dev)) * x.to(dev) + sh.to(dev)).reshape(48, -1).cpu())[0], y1)   # eager == oracle
    y2 = O.linear_w8a8(O.prologue(y1, code, O.PRO_GELU_TANH), code, m.down.weight.cpu().numpy(),
                       m.down.weight_scale.cpu().numpy().reshape(-1), O.from_torch(m.down.bias.cpu())[0], O.BF16, O.BF16, 0)
    want = O.to_f32(y2, O.BF16).reshape(2, 24, 256)
    diff = np.abs(got.float().cpu().numpy() - want)
    assert diff.max() <= 2.0**-7 * np.abs(want).max()
    assert (diff != 0).mean() < 0.02


@pytest.mark.gpu
def test_compiled_adaln_block_with_the_layer_norm_in_the_quantiser(pkg, dev, O):
    """LayerNorm (no affine) -> modulation -> quantised projection compiled with the rewriting backend over inductor:
    one fused operator, no LayerNorm kernel left, and the output agrees with the oracle's chain (row sums in double)
    to the rounding of the normalised values: within two bf16 ulps of the output scale, at least 90 % identical."""
    g = torch.Generator().manual_seed(8)
    lin = pkg.Int8TensorwiseOps.Linear(512, 192, bias=True)
    _load(lin, {"weight": torch.randint(-127, 128, (192, 512), dtype=torch.int8, generator=g),
                "weight_scale": torch.rand(192, 1, generator=g) * 0.002 + 1e-3, "bias": torch.randn(192, generator=g).bfloat16()})

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.norm, self.qkv = torch.nn.LayerNorm(512, elementwise_affine=False, eps=1e-6), lin

        def forward(self, x, scale, shift):
            return self.qkv((1 + scale) * self.norm(x) + shift)

    m = Block().to(dev)
    x = (torch.randn(2, 40, 512, generator=g) * 2 + 0.5).bfloat16()
    sc, sh = (torch.randn(2, 1, 512, generator=g) * 0.3).bfloat16(), torch.randn(2, 1, 512, generator=g).bfloat16()
    seen = []

    def counting(gm, inputs):
        seen.append((sum("int8_linear_prologue" in str(n.target) for n in gm.graph.nodes),
                     sum("layer_norm" in str(n.target) for n in gm.graph.nodes)))
        from torch._dynamo.backends.registry import lookup_backend
        return lookup_backend("inductor")(gm, inputs)

    got = torch.compile(m, backend=pkg.compile_ops.backend(counting), fullgraph=True)(x.to(dev), sc.to(dev), sh.to(dev))
    assert seen == [(1, 0)]
    xa, code = O.from_torch(x.reshape(80, 512))
    z = O.norm_modulate(xa, code, 1e-6, O.from_torch(sc.reshape(2, 512))[0], O.from_torch(sh.reshape(2, 512))[0], rows_per_vec=40)
    want = O.to_f32(O.linear_w8a8(z, code, lin.weight.cpu().numpy(), lin.weight_scale.cpu().numpy().reshape(-1),
                                  O.from_torch(lin.bias.cpu())[0], O.BF16, O.BF16, 0), O.BF16).reshape(2, 40, 192)
    diff = np.abs(got.float().cpu().numpy() - want)
    assert diff.max() <= 2.0**-7 * np.abs(want).max()
    assert (diff != 0).mean() < 0.1
    eager = m(x.to(dev), sc.to(dev), sh.to(dev))       # torch's LayerNorm and modulation, then the layer
    assert (got.float() - eager.float()).abs().max().item() <= 2.0**-7 * eager.float().abs().max().item()


@pytest.mark.gpu
def test_compiled_adaln_zero_block_equals_eager_bit_for_bit(pkg, dev):
    """x + gate * proj(gelu(up((1 + scale) * norm(x) + shift))) compiled with the rewriting backend over inductor: both
    layers carry a prologue, the second also the gated residual in its epilogue, and no elementwise kernel of the block
    is left for inductor; the result equals the same module run with this library's eager fused forward calls."""
    g = torch.Generator().manual_seed(9)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=True)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3, "bias": (torch.randn(n_out, generator=g) * 0.1).bfloat16()})

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.norm = torch.nn.LayerNorm(256, elementwise_affine=False, eps=1e-6)
            self.up, self.down = lin(512, 256), lin(256, 512)

        def forward(self, x, scale, shift, gate):
            h = self.up((1 + scale) * self.norm(x) + shift)
            return x + gate * self.down(F.gelu(h, approximate="tanh"))

    m = Block().to(dev)
    x = (torch.randn(2, 40, 256, generator=g) * 2).bfloat16().to(dev)
    sc, sh, gate = ((torch.randn(2, 1, 256, generator=g) * 0.3).bfloat16().to(dev) for _ in range(3))
    seen = []

    def counting(gm, inputs):
        calls = [n for n in gm.graph.nodes if n.op == "call_function"]
        seen.append((sum("int8_linear_prologue" in str(n.target) for n in calls),
                     sum(n.kwargs.get("gate") is not None and n.kwargs.get("addend") is not None for n in calls),
                     sum(n.target in (operator.mul, operator.add, torch.mul, torch.add) or "gelu" in str(n.target) or "layer_norm" in str(n.target)
                         for n in calls)))
        from torch._dynamo.backends.registry import lookup_backend
        return lookup_backend("inductor")(gm, inputs)

    got = torch.compile(m, backend=pkg.compile_ops.backend(counting), fullgraph=True)(x, sc, sh, gate)
    assert seen == [(2, 1, 0)]
    L = pkg._lib
    h = m.up(x, prologue=L.PRO_NORM_MODULATE, mod_scale=sc, mod_shift=sh, eps=1e-6)
    want = m.down(h, prologue=L.PRO_GELU_TANH, gate=gate, residual=x)
    assert torch.equal(got, want)
    loose = m(x, sc, sh, gate)                           # torch's LayerNorm, modulation, gelu, gate and residual around the layers
    assert (got.float() - loose.float()).abs().max().item() <= 2.0**-6 * loose.float().abs().max().item()


@pytest.mark.gpu
def test_compiled_rms_norm_producer_and_exact_gelu_equal_eager_bit_for_bit(pkg, dev):
    """down(gelu(up(norm(x) * (1 + scale)))) with an RMSNorm that has a weight and GELU in its exact form, compiled with the
    rewriting backend over inductor: two fused operators, neither an rms_norm nor a gelu kernel left; equal to the
    eager fused forward calls bit for bit and within rounding of torch's operations around the layers."""
    g = torch.Generator().manual_seed(17)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=True)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3, "bias": (torch.randn(n_out, generator=g) * 0.1).bfloat16()})

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.norm = torch.nn.RMSNorm(256, eps=1e-5).bfloat16()
            self.up, self.down = lin(512, 256), lin(256, 512)

        def forward(self, x, scale):
            return self.down(F.gelu(self.up(self.norm(x) * (1 + scale))))

    m = Block().to(dev)
    with torch.no_grad():
        m.norm.weight.copy_((torch.randn(256, generator=g) * 0.2 + 1).bfloat16())
    x = (torch.randn(2, 40, 256, generator=g) * 2).bfloat16().to(dev)
    scale = (torch.randn(2, 1, 256, generator=g) * 0.3).bfloat16().to(dev)
    seen = []

    def counting(gm, inputs):
        calls = [n for n in gm.graph.nodes if n.op == "call_function"]
        seen.append((sum("int8_linear_prologue" in str(n.target) for n in calls),
                     sum("rms_norm" in str(n.target) or "gelu" in str(n.target) or n.target in (operator.mul, operator.add) for n in calls)))
        from torch._dynamo.backends.registry import lookup_backend
        return lookup_backend("inductor")(gm, inputs)

    with torch.no_grad():
        got = torch.compile(m, backend=pkg.compile_ops.backend(counting), fullgraph=True)(x, scale)
        assert seen == [(2, 0)]
        L = pkg._lib
        h = m.up(x, prologue=L.PRO_RMS_NORM, norm_weight=m.norm.weight, mod_scale=scale, eps=1e-5)
        want = m.down(h, prologue=L.PRO_GELU_ERF)
        assert torch.equal(got, want)
        loose = m(x, scale)
    assert (got.float() - loose.float()).abs().max().item() <= 2.0**-6 * loose.float().abs().max().item()


@pytest.mark.gpu
def test_compiled_swiglu_block_shares_one_quantiser_and_equals_eager(pkg, dev):
    """x + tanh(gate) * w2(silu(w1(h)) * w3(h)), h = norm(x) * (1 + scale) with an RMSNorm (the feed-forward half of a
    z-image block) and separate q / k / v projections of the same h, compiled with the rewriting backend over inductor:
    the five layers that read h share ONE quantiser, which also normalises and modulates (h never exists), w2 takes the
    gate as its prologue and the residual in its epilogue.  Equal to the eager fused calls bit for bit."""
    g = torch.Generator().manual_seed(19)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=False)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3})

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.norm = torch.nn.RMSNorm(256, eps=1e-5).bfloat16()
            self.q, self.k, self.v = lin(128, 256), lin(64, 256), lin(64, 256)
            self.w1, self.w3, self.w2 = lin(512, 256), lin(512, 256), lin(256, 512)

        def forward(self, x, scale, gate):
            h = self.norm(x) * (1 + scale)
            y = x + gate.tanh() * self.w2(F.silu(self.w1(h)) * self.w3(h))
            return y, self.q(h), self.k(h), self.v(h)

    m = Block().to(dev)
    with torch.no_grad():
        m.norm.weight.copy_((torch.randn(256, generator=g) * 0.2 + 1).bfloat16())
    x = (torch.randn(2, 40, 256, generator=g) * 2).bfloat16().to(dev)
    scale, gate = ((torch.randn(2, 1, 256, generator=g) * 0.3).bfloat16().to(dev) for _ in range(2))
    seen = []

    def counting(gm, inputs):
        names = [str(n.target) for n in gm.graph.nodes if n.op == "call_function"]
        seen.append((sum("quantize_rowwise" in t for t in names), sum("linear_w8a8" in t for t in names),
                     sum("int8_linear_prologue" in t for t in names), sum("rms_norm" in t or "silu" in t for t in names)))
        from torch._dynamo.backends.registry import lookup_backend
        return lookup_backend("inductor")(gm, inputs)

    with torch.no_grad():
        got = torch.compile(m, backend=pkg.compile_ops.backend(counting), fullgraph=True)(x, scale, gate)
        assert seen == [(1, 5, 1, 0)]
        L = pkg._lib
        kw = dict(prologue=L.PRO_RMS_NORM, norm_weight=m.norm.weight, mod_scale=scale, eps=1e-5)
        a, b, q, k, v = pkg.forward_fanout([m.w1, m.w3, m.q, m.k, m.v], x, **kw)
        y = m.w2(a, prologue=L.PRO_SILU_GATE, mod_scale=b, gate=gate.tanh(), residual=x)
        for have, want in zip(got, (y, q, k, v)):
            assert torch.equal(have, want)
        loose = m(x, scale, gate)
    for have, want in zip(got, loose):
        assert (have.float() - want.float()).abs().max().item() <= 2.0**-6 * want.float().abs().max().item()


@pytest.mark.gpu
@pytest.mark.parametrize("quarot", [False, True])
def test_compiled_dynamic_lora_takes_the_side_branch_in_the_epilogue(pkg, dev, quarot):
    """A layer with dynamic LoRA factors under torch.compile: the traced graph holds the first low-rank product and ONE
    operator that forms the second product, the scaling and the sum inside the GEMM epilogue (no [rows, N] side tensor),
    as the eager path does; result equal to eager's, which the module tests hold to the reference's expression."""
    g = torch.Generator().manual_seed(23)
    lin = pkg.Int8TensorwiseOps.Linear(384, 256, bias=True)
    _load(lin, {"weight": torch.randint(-127, 128, (256, 384), dtype=torch.int8, generator=g),
                "weight_scale": torch.rand(256, 1, generator=g) * 0.002 + 1e-3, "bias": (torch.randn(256, generator=g) * 0.1).bfloat16()})
    lin = lin.to(dev)
    lin._use_quarot = quarot
    lin.lora_A = (torch.randn(16, 384, generator=g) * 0.05).bfloat16().to(dev)
    lin.lora_B = (torch.randn(256, 16, generator=g) * 0.05).bfloat16().to(dev)
    lin.lora_alpha = 0.5
    x = torch.randn(2, 30, 384, generator=g).bfloat16().to(dev)
    seen = []

    def counting(gm, inputs):
        names = [str(n.target) for n in gm.graph.nodes if n.op == "call_function"]
        seen.append((sum("int8_linear_lora" in t for t in names), sum(t.endswith("int8_linear.default") or t.endswith("int8_linear") for t in names)))
        from torch._dynamo.backends.registry import lookup_backend
        return lookup_backend("inductor")(gm, inputs)

    with torch.no_grad():
        got = torch.compile(lin, backend=pkg.compile_ops.backend(counting), fullgraph=True)(x)
        want = lin(x)
    assert seen == [(1, 0)]
    assert got.shape == (2, 30, 256)
    assert (got.float() - want.float()).abs().max().item() <= 2.0**-8 * want.float().abs().max().item()
    assert (got != want).float().mean().item() < 0.01      # (the first product is the BLAS library's in both runs)


@pytest.mark.gpu
def test_compiled_shared_quantiser_with_a_gated_residual_on_one_layer(pkg, dev):
    """Two layers read one tensor and the first one's result goes into res + gate * y: the rewriting backend shares the
    quantiser (two GEMM operators) and still folds the gated residual into the first GEMM's epilogue; equal to the
    eager calls bit for bit."""
    g = torch.Generator().manual_seed(21)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=True)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3, "bias": (torch.randn(n_out, generator=g) * 0.1).bfloat16()})

    class Two(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a, self.b = lin(256, 256), lin(128, 256)

        def forward(self, x, res, gate):
            return res + gate * self.a(x), self.b(x)

    m = Two().to(dev)
    x = torch.randn(2, 40, 256, generator=g).bfloat16().to(dev)
    res = torch.randn(2, 40, 256, generator=g).bfloat16().to(dev)
    gate = (torch.randn(2, 1, 256, generator=g) * 0.3).bfloat16().to(dev)
    seen = []

    def counting(gm, inputs):
        calls = [n for n in gm.graph.nodes if n.op == "call_function"]
        seen.append((sum("quantize_rowwise" in str(n.target) for n in calls),
                     sum("linear_w8a8" in str(n.target) and n.kwargs.get("gate") is not None and n.kwargs.get("addend") is not None for n in calls),
                     sum("linear_w8a8" in str(n.target) for n in calls),
                     sum(n.target in (operator.mul, operator.add) for n in calls)))
        from torch._dynamo.backends.registry import lookup_backend
        return lookup_backend("inductor")(gm, inputs)

    with torch.no_grad():
        got = torch.compile(m, backend=pkg.compile_ops.backend(counting), fullgraph=True)(x, res, gate)
        assert seen == [(1, 1, 2, 0)]
        assert torch.equal(got[0], m.a(x, gate=gate, residual=res)) and torch.equal(got[1], m.b(x))
        assert torch.equal(got[0], res + gate * m.a(x))


@pytest.mark.gpu
def test_plain_torch_compile_applies_the_rewrites_once_the_pass_is_installed(pkg, dev):
    """torch.compile(model) with the default backend, after compile_ops.install_inductor_pass(): the adaLN-Zero MLP is
    rewritten by inductor's pre-grad hook exactly as by compile_ops.backend() -- two prologues, one gated residual --
    and the result is that of the eager fused calls bit for bit."""
    import torch._inductor.config as inductor_config
    g = torch.Generator().manual_seed(22)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=True)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3, "bias": (torch.randn(n_out, generator=g) * 0.1).bfloat16()})

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.norm = torch.nn.LayerNorm(256, elementwise_affine=False, eps=1e-6)
            self.up, self.down = lin(512, 256), lin(256, 512)

        def forward(self, x, scale, shift, gate):
            h = self.up((1 + scale) * self.norm(x) + shift)
            return x + gate * self.down(F.gelu(h, approximate="tanh"))

    m = Block().to(dev)
    x = (torch.randn(2, 40, 256, generator=g) * 2).bfloat16().to(dev)
    sc, sh, gate = ((torch.randn(2, 1, 256, generator=g) * 0.3).bfloat16().to(dev) for _ in range(3))
    before = inductor_config.pre_grad_custom_pass
    try:
        assert pkg.compile_ops.install_inductor_pass() and pkg.compile_ops.install_inductor_pass()
        pkg.compile_ops.LAST_PASS_COUNTS = None
        with torch.no_grad():
            got = torch.compile(m, fullgraph=True)(x, sc, sh, gate)
        assert pkg.compile_ops.LAST_PASS_COUNTS == (0, 2, 1)
        L = pkg._lib
        h = m.up(x, prologue=L.PRO_NORM_MODULATE, mod_scale=sc, mod_shift=sh, eps=1e-6)
        assert torch.equal(got, m.down(h, prologue=L.PRO_GELU_TANH, gate=gate, residual=x))
    finally:
        inductor_config.pre_grad_custom_pass = before
        pkg.compile_ops._installed = False


@pytest.mark.gpu
def test_compiled_in_place_residual_update_equals_eager(pkg, dev):
    """The residual updates of a double-stream block as the model code spells them, `img = img + g * proj(a)` and
    `txt += g * proj(a)`: both end up in their layer's epilogue under the rewriting backend, and the results are those
    of eager mode bit for bit (torch's two rounded operations either way)."""
    g = torch.Generator().manual_seed(25)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=True)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3, "bias": (torch.randn(n_out, generator=g) * 0.1).bfloat16()})

    class Pair(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.img_proj, self.txt_proj, self.embed = lin(256, 256), lin(256, 256), lin(256, 128)

        def forward(self, img, txt_tokens, a_img, a_txt, g_img, g_txt):
            txt = self.embed(txt_tokens)
            img = img + g_img * self.img_proj(a_img)
            txt += g_txt * self.txt_proj(a_txt)
            return img, txt

    m = Pair().to(dev)
    img, a_img = (torch.randn(2, 64, 256, generator=g).bfloat16().to(dev) for _ in range(2))
    tok, a_txt = torch.randn(2, 24, 128, generator=g).bfloat16().to(dev), torch.randn(2, 24, 256, generator=g).bfloat16().to(dev)
    g_img, g_txt = ((torch.randn(2, 1, 256, generator=g) * 0.3).bfloat16().to(dev) for _ in range(2))
    seen = []

    def counting(gm, inputs):
        calls = [n for n in gm.graph.nodes if n.op == "call_function"]
        seen.append((sum(n.kwargs.get("gate") is not None and n.kwargs.get("addend") is not None for n in calls),
                     sum(n.target in (operator.mul, operator.add, operator.iadd) for n in calls)))
        from torch._dynamo.backends.registry import lookup_backend
        return lookup_backend("inductor")(gm, inputs)

    with torch.no_grad():
        got = torch.compile(m, backend=pkg.compile_ops.backend(counting), fullgraph=True)(img, tok, a_img, a_txt, g_img, g_txt)
        assert seen == [(2, 0)]
        want = m(img, tok, a_img, a_txt, g_img, g_txt)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


@pytest.mark.gpu
def test_compiled_block_in_the_spelling_of_the_model_code_equals_eager(pkg, dev):
    """One stream of a double-stream block as the model's Python writes it -- apply_mod(t, m, a) = torch.addcmul(a, t, m),
    apply_mod(t, m) = t * m: qkv(apply_mod(norm1(x), 1 + scale1, shift1)), x = x + apply_mod(proj(a), gate1),
    x += apply_mod(mlp(apply_mod(norm2(x), 1 + scale2, shift2)), gate2) -- under the rewriting backend: every layer
    carries its producer or its residual update, nothing elementwise is left for inductor but the attention stand-in,
    and the result is that of the eager fused calls bit for bit (and that of the module in eager mode up to the
    roundings of the in-quantiser LayerNorm, carried through four layers)."""
    g = torch.Generator().manual_seed(27)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=True)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3, "bias": (torch.randn(n_out, generator=g) * 0.1).bfloat16()})

    def apply_mod(tensor, m_mult, m_add=None):
        return torch.addcmul(m_add, tensor, m_mult) if m_add is not None else tensor * m_mult

    class Stream(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.norm1 = torch.nn.LayerNorm(256, elementwise_affine=False, eps=1e-6)
            self.norm2 = torch.nn.LayerNorm(256, elementwise_affine=False, eps=1e-6)
            self.qkv, self.proj, self.up, self.down = lin(768, 256), lin(256, 256), lin(1024, 256), lin(256, 1024)

        def forward(self, x, shift1, scale1, gate1, shift2, scale2, gate2):
            x = x * 1.0                                                   # (an intermediate, as inside a model)
            q, k, v = self.qkv(apply_mod(self.norm1(x), 1 + scale1, shift1)).chunk(3, dim=-1)
            attn = q + v                                                  # (stands in for the attention: ONE rounded operation, as inductor keeps chains in binary32)
            x = x + apply_mod(self.proj(attn), gate1)
            x += apply_mod(self.down(F.gelu(self.up(apply_mod(self.norm2(x), 1 + scale2, shift2)), approximate="tanh")), gate2)
            return x

    m = Stream().to(dev)
    x = (torch.randn(2, 48, 256, generator=g) * 2).bfloat16().to(dev)
    mods = [(torch.randn(2, 1, 256, generator=g) * 0.3).bfloat16().to(dev) for _ in range(6)]
    seen = []

    def counting(gm, inputs):
        calls = [n for n in gm.graph.nodes if n.op == "call_function"]
        seen.append((sum("int8_linear_prologue" in str(n.target) for n in calls),
                     sum(n.kwargs.get("gate") is not None and n.kwargs.get("addend") is not None for n in calls),
                     sum(n.target in (torch.addcmul, operator.iadd) or "layer_norm" in str(n.target) or "gelu" in str(n.target) for n in calls)))
        from torch._dynamo.backends.registry import lookup_backend
        return lookup_backend("inductor")(gm, inputs)

    with torch.no_grad():
        got = torch.compile(m, backend=pkg.compile_ops.backend(counting), fullgraph=True)(x, *mods)
        assert seen == [(3, 2, 0)]            # qkv, up, down carry a prologue; proj and down the gated residual
        L = pkg._lib
        shift1, scale1, gate1, shift2, scale2, gate2 = mods
        x0 = x * 1.0
        q, k, v = m.qkv(x0, prologue=L.PRO_NORM_MODULATE, mod_scale=scale1, mod_shift=shift1, eps=1e-6, fused_add=True).chunk(3, dim=-1)
        x1 = m.proj(q + v, gate=gate1, residual=x0)
        h = m.up(x1, prologue=L.PRO_NORM_MODULATE, mod_scale=scale2, mod_shift=shift2, eps=1e-6, fused_add=True)
        want = m.down(h, prologue=L.PRO_GELU_TANH, gate=gate2, residual=x1)
        assert torch.equal(got, want)
        loose = m(x, *mods)
    diff = (got.float() - loose.float()).abs()
    assert diff.max().item() <= 2.0**-4 * loose.float().abs().max().item() and diff.mean().item() <= 2.0**-9 * loose.float().abs().max().item()


@pytest.mark.gpu
def test_compiled_single_stream_block_equals_eager_bit_for_bit(pkg, dev):
    """x + gate * linear2(cat((a, gelu(mlp)), -1)) with a and mlp split from linear1's output, the shape of a
    single-stream block: the split halves reach the quantiser as strided views, neither the activated tensor nor the
    concatenation exists, the gated residual sits in linear2's epilogue; equal to the eager fused forward calls and
    within rounding of torch's operations around the layers."""
    g = torch.Generator().manual_seed(16)

    def lin(n_out, k_in):
        l = pkg.Int8TensorwiseOps.Linear(k_in, n_out, bias=True)
        return _load(l, {"weight": torch.randint(-127, 128, (n_out, k_in), dtype=torch.int8, generator=g),
                         "weight_scale": torch.rand(n_out, 1, generator=g) * 0.002 + 1e-3, "bias": (torch.randn(n_out, generator=g) * 0.1).bfloat16()})

    class Single(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.linear1, self.linear2 = lin(256 + 512, 256), lin(256, 256 + 512)

        def forward(self, x, gate):
            a, mlp = torch.split(self.linear1(x), [256, 512], dim=-1)
            return x + gate * self.linear2(torch.cat((a, F.gelu(mlp, approximate="tanh")), 2))

    m = Single().to(dev)
    x = torch.randn(2, 40, 256, generator=g).bfloat16().to(dev)
    gate = (torch.randn(2, 1, 256, generator=g) * 0.3).bfloat16().to(dev)
    seen = []

    def counting(gm, inputs):
        calls = [n for n in gm.graph.nodes if n.op == "call_function"]
        seen.append((sum("int8_linear_prologue" in str(n.target) for n in calls),
                     sum(n.kwargs.get("gate") is not None and n.kwargs.get("addend") is not None for n in calls),
                     sum(n.target in (operator.mul, operator.add, torch.mul, torch.add, torch.cat) or "gelu" in str(n.target) for n in calls)))
        from torch._dynamo.backends.registry import lookup_backend
        return lookup_backend("inductor")(gm, inputs)

    got = torch.compile(m, backend=pkg.compile_ops.backend(counting), fullgraph=True)(x, gate)
    assert seen == [(1, 1, 0)]
    a, mlp = torch.split(m.linear1(x), [256, 512], dim=-1)
    want = m.linear2(a, prologue=pkg._lib.PRO_CONCAT_GELU, mod_scale=mlp, gate=gate, residual=x)
    assert torch.equal(got, want)
    loose = m(x, gate)
    assert (got.float() - loose.float()).abs().max().item() <= 2.0**-6 * loose.float().abs().max().item()
    few = m.linear2(a[:, :4], prologue=pkg._lib.PRO_CONCAT_GELU, mod_scale=mlp[:, :4])     # 8 rows: torch concatenates, the small-batch path runs
    ref = m.linear2(torch.cat((a[:, :4], F.gelu(mlp[:, :4], approximate="tanh")), -1))
    assert torch.equal(few, ref)


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [48, 8])
@pytest.mark.parametrize("scalar_scale", [False, True])
def test_compiled_forward_equals_eager(pkg, dev, rows, scalar_scale):
    torch.manual_seed(3)
    lin = pkg.Int8TensorwiseOps.Linear(256, 128, bias=True)
    sd = {"weight": torch.randint(-127, 128, (128, 256), dtype=torch.int8), "bias": torch.randn(128).bfloat16(),
          "weight_scale": torch.tensor(0.004) if scalar_scale else torch.rand(128, 1) * 0.01 + 1e-3}
    _load(lin, sd)
    lin._use_quarot = True
    lin = lin.to(dev)
    x = torch.randn(rows, 256, device=dev).bfloat16()
    eager = lin(x)
    compiled = torch.compile(lin, backend="aot_eager", fullgraph=True)
    got = compiled(x)
    assert got.dtype == eager.dtype and torch.equal(got.view(torch.int16), eager.view(torch.int16))


@pytest.mark.gpu
def test_opcheck_int8_linear(pkg, dev):
    x = torch.randn(40, 256, device=dev).bfloat16()
    w = torch.randint(-127, 128, (64, 256), dtype=torch.int8, device=dev)
    ws = (torch.rand(64, 1, device=dev) * 0.01 + 1e-3)
    b = torch.randn(64, device=dev).bfloat16()
    torch.library.opcheck(torch.ops.i8f.int8_linear.default, (x, w, ws, 0.0, b, torch.bfloat16, True, 0),
                          test_utils=("test_schema", "test_faketensor"))
    q, s = torch.ops.i8f.quantize_rowwise(x, False)
    torch.library.opcheck(torch.ops.i8f.linear_w8a8.default, (q, s, w, None, 0.01, None, torch.float16, 1),
                          test_utils=("test_schema", "test_faketensor"))
