"""Host-side behaviour of the ComfyUI-facing layer that needs no GPU: state-dict loading rules,
scale bookkeeping, ModelPatcher hooks, LoRA scale slicing, delta reconstruction, Hadamard build."""
import numpy as np
import pytest
import torch


@pytest.fixture(autouse=True)
def reset_flags(pkg):
    ops = pkg.Int8TensorwiseOps
    saved = (list(ops.excluded_names), ops.dynamic_quantize, ops.enable_quarot, ops._is_prequantized)
    yield
    ops.excluded_names, ops.dynamic_quantize, ops.enable_quarot, ops._is_prequantized = saved


def load(layer, sd, prefix="blk.0.lin."):
    missing = []
    layer._load_from_state_dict(dict(sd), prefix, {}, True, missing, [], [])
    return missing


def test_prequantized_scalar_scale_becomes_python_float(pkg):
    lin = pkg.Int8TensorwiseOps.Linear(64, 32, bias=True)
    w = torch.randint(-128, 128, (32, 64), dtype=torch.int8)
    sd = {"blk.0.lin.weight": w, "blk.0.lin.weight_scale": torch.tensor(0.0125), "blk.0.lin.bias": torch.zeros(32),
          "blk.0.lin.input_scale": torch.tensor(1.0), "blk.0.lin.comfy_quant": torch.zeros(1)}
    assert load(lin, sd) == []
    assert lin._is_quantized and not lin._is_per_row and lin.weight_scale is None
    assert lin._weight_scale_scalar == pytest.approx(0.0125) and isinstance(lin._get_weight_scale(), float)
    assert lin.weight.dtype == torch.int8 and not lin.weight.requires_grad and torch.equal(lin.weight, w)
    assert lin.weight_comfy_model_dtype == torch.int8 and lin.bias_comfy_model_dtype == torch.float32
    assert pkg.Int8TensorwiseOps._is_prequantized


def test_prequantized_per_row_and_odd_scale_shapes(pkg):
    w = torch.zeros(32, 64, dtype=torch.int8)
    lin = pkg.Int8TensorwiseOps.Linear(64, 32, bias=False)
    load(lin, {"blk.0.lin.weight": w, "blk.0.lin.weight_scale": torch.rand(32, 1).half()})
    assert lin._is_per_row and lin.weight_scale.dtype == torch.float32 and lin.weight_scale.shape == (32, 1)
    assert lin._weight_scale_scalar is None and lin.bias is None
    lin2 = pkg.Int8TensorwiseOps.Linear(64, 32, bias=False)
    load(lin2, {"blk.0.lin.weight": w, "blk.0.lin.weight_scale": torch.rand(32)})   # not [N,1]: kept, treated as one scale
    assert lin2._is_quantized and not lin2._is_per_row and lin2.weight_scale.shape == (32,)
    lin3 = pkg.Int8TensorwiseOps.Linear(64, 32, bias=False)
    load(lin3, {"blk.0.lin.weight": w, "blk.0.lin.weight_scale": 0.5})
    assert lin3._weight_scale_scalar == 0.5


def test_float_weights_stay_float_unless_dynamic_quantize(pkg):
    ops = pkg.Int8TensorwiseOps
    w = torch.randn(32, 64).bfloat16()
    lin = ops.Linear(64, 32, bias=False)
    load(lin, {"blk.0.lin.weight": w})
    assert not lin._is_quantized and lin.weight.dtype == torch.bfloat16
    ops.dynamic_quantize = True
    ops.excluded_names = ["blk.0"]
    lin = ops.Linear(64, 32, bias=False)
    load(lin, {"blk.0.lin.weight": w})
    assert not lin._is_quantized                              # excluded by name
    ops.excluded_names = []
    lin = ops.Linear(64, 1, bias=False)
    load(lin, {"blk.0.lin.weight": torch.randn(1, 64)})
    assert not lin._is_quantized                              # a dimension of 1 is never quantised
    lin = ops.Linear(64, 32, bias=False)
    assert load(lin, {}) == ["blk.0.lin.weight"]              # missing key is reported
    if not torch.cuda.is_available():
        lin = ops.Linear(64, 32, bias=False)
        with pytest.raises(RuntimeError):                      # quantising needs the GPU library: no CPU path
            load(lin, {"blk.0.lin.weight": w})


def test_unquantized_layer_is_a_plain_linear(pkg):
    lin = pkg.Int8TensorwiseOps.Linear(16, 8, bias=True)
    w, b = torch.randn(8, 16), torch.randn(8)
    load(lin, {"blk.0.lin.weight": w, "blk.0.lin.bias": b})
    x = torch.randn(3, 5, 16)
    assert torch.allclose(lin(x), torch.nn.functional.linear(x, w, b))
    assert lin.convert_weight(w) is w


def test_model_patcher_hooks(pkg):
    lin = pkg.Int8TensorwiseOps.Linear(64, 32, bias=True)
    w = torch.randint(-128, 128, (32, 64), dtype=torch.int8)
    load(lin, {"blk.0.lin.weight": w, "blk.0.lin.weight_scale": torch.rand(32, 1), "blk.0.lin.bias": torch.zeros(32)})
    assert lin.convert_weight(torch.zeros(1)) is lin.weight               # int8 payload handed to the adapter
    w2 = torch.randint(-128, 128, (32, 64), dtype=torch.int8)
    assert lin.set_weight(w2, return_weight=True) is w2
    lin.set_weight(w2)
    assert torch.equal(lin.weight, w2) and isinstance(lin.weight, torch.nn.Parameter)
    w3 = torch.randint(-128, 128, (32, 64), dtype=torch.int8)
    keep = lin.weight
    lin.set_weight(w3, inplace_update=True)
    assert lin.weight is keep and torch.equal(lin.weight, w3)
    assert lin.set_bias(None) is None
    nb = torch.ones(32)
    lin.set_bias(nb)
    assert torch.equal(lin.bias, nb)
    lin.set_bias(torch.full((32,), 2.0), inplace_update=True)
    assert float(lin.bias[0]) == 2.0


def test_pass_through_layers_and_conv_nd(pkg):
    ops = pkg.Int8TensorwiseOps
    assert isinstance(ops.conv_nd(2, 3, 4, 3), ops.Conv2d) and isinstance(ops.conv_nd(3, 3, 4, 3), ops.Conv3d)
    with pytest.raises(ValueError):
        ops.conv_nd(1, 3, 4, 3)
    for name in ("GroupNorm", "LayerNorm", "ConvTranspose2d", "Embedding"):
        assert hasattr(ops, name)
    assert ops.use_triton is True and ops.excluded_names == []


def test_scale_slicing_rules_of_both_adapters(pkg):
    ws = torch.arange(96, dtype=torch.float32).reshape(96, 1)
    single = pkg.INT8LoRAPatchAdapter(set(), (None,) * 6, ws, seed=1)
    assert single._get_effective_scale(torch.zeros(32, 8), (0, 32, 32)).flatten().tolist() == list(range(32, 64))
    assert single._get_effective_scale(torch.zeros(96, 8), (0, 32, 32)).shape == (32, 1)   # offset wins even if rows match
    assert single._get_effective_scale(torch.zeros(32, 8), None).flatten().tolist() == list(range(32))
    assert single._get_effective_scale(torch.zeros(96, 8), None) is ws
    assert single._get_effective_scale(torch.zeros(32, 8), (0, 80, 32)).shape == (16, 1)   # clipped at the end
    assert pkg.INT8LoRAPatchAdapter(set(), (None,) * 6, 0.5)._get_effective_scale(torch.zeros(4, 4), (0, 1, 2)) == 0.5
    inner = pkg.INT8LoRAPatchAdapter({"k"}, (None,) * 6, ws)
    merged = pkg.INT8MergedLoRAPatchAdapter([(inner, 1.0)], ws, seed=2)
    assert merged.loaded_keys == {"k"} and merged.seed == 2
    assert merged._get_effective_scale(torch.zeros(32, 8), (0, 32, 32)).flatten().tolist() == list(range(32, 64))
    assert merged._get_effective_scale(torch.zeros(96, 8), (0, 32, 32)) is ws              # older rule: only on mismatch
    assert merged._get_effective_scale(torch.zeros(32, 8), (1, 0, 8)).flatten().tolist() == list(range(32))


def test_reconstruct_lora_diff_variants(pkg):
    f = pkg.int8_quant.reconstruct_lora_diff
    g = torch.Generator().manual_seed(0)
    up, down = torch.randn(12, 4, generator=g), torch.randn(4, 10, generator=g)
    d, s = f((up, down, 8.0, None, None, None), (12, 10), "cpu", torch.float32, 0.5)
    assert torch.allclose(d, up @ down) and s == pytest.approx(8.0 / 4 * 0.5)
    mid = torch.randn(4, 4, generator=g)
    d, s = f((up, down, None, mid, None, None), (12, 10), "cpu", torch.float32, 0.7)
    assert torch.allclose(d, up @ mid @ down, atol=1e-5) and s == 0.7
    w1a, w1b, w2a, w2b = (torch.randn(*sh, generator=g) for sh in [(12, 3), (3, 10), (12, 3), (3, 10)])
    d, s = f((w1a, w1b, 3.0, w2a, w2b, None, None, None), (12, 10), "cpu", torch.float32, 1.0)
    assert torch.allclose(d, (w1a @ w1b) * (w2a @ w2b)) and s == pytest.approx(1.0)
    k1, k2 = torch.randn(3, 2, generator=g), torch.randn(4, 5, generator=g)
    d, s = f((k1, k2, 1.0, None, None, None, None, None, None), (12, 10), "cpu", torch.float32, 2.0)
    assert torch.allclose(d, torch.kron(k1, k2)) and s == 2.0
    assert f((1, 2, 3), (1,), "cpu", torch.float32, 1.0) == (None, 1.0)


def test_build_hadamard(pkg):
    from scipy.linalg import hadamard

    H = pkg.quarot.build_hadamard(128)
    assert np.array_equal(H.numpy(), (torch.tensor(hadamard(128), dtype=torch.float32) / (128**0.5)).numpy())
    assert torch.allclose(H @ H.T, torch.eye(128), atol=1e-6) and torch.equal(H, H.T)
    assert pkg.quarot.build_hadamard(128) is H                         # cached
    Hb = pkg.quarot.build_hadamard(128, dtype=torch.bfloat16)
    assert Hb.dtype == torch.bfloat16 and float(Hb[0, 0]) == 0.08837890625
    with pytest.raises(ValueError):
        pkg.quarot.build_hadamard(96)
    with pytest.raises(ValueError):
        pkg.quarot.rotate_weight(torch.zeros(4, 100))
    with pytest.raises(ValueError):
        pkg.quarot.rotate_activation(torch.zeros(4, 256), None, 64)


def test_quantize_int8_given_scale_and_dequantize(pkg):
    x = torch.tensor([[0.5, -1.26, 100.0, -100.0, 0.024, 0.026]])
    q = pkg.quantize_int8(x, 0.05)
    assert q.tolist() == [[10, -25, 127, -128, 0, 1]]
    assert torch.allclose(pkg.dequantize(q, 0.05), torch.tensor([[0.5, -1.25, 6.35, -6.4, 0.0, 0.05]]))


def test_aliases_keep_the_reference_names(pkg):
    assert pkg.triton_quantize_rowwise is pkg.hip_quantize_rowwise
    assert pkg.triton_int8_linear is pkg.hip_int8_linear
    assert pkg.triton_int8_linear_per_row is pkg.hip_int8_linear_per_row
    with pytest.raises(ValueError):
        pkg.quantize_int8_axiswise(torch.zeros(4, 8), dim=0)
