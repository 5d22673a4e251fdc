"""torch.library registration of the forward path: schemas and shape-only implementations on the CPU,
Dynamo tracing of Linear.forward without graph breaks, and (GPU) compiled == eager bit for bit."""
import pytest
import torch


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
