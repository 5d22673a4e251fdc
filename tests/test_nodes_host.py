"""Graph nodes and the dynamic-LoRA hook, exercised without ComfyUI: the logic underneath the nodes
runs on plain torch modules, and the nodes themselves run against small stand-ins for
`folder_paths` and `comfy.*` that record what they were asked to do."""
import sys
import types

import pytest
import torch
from torch import nn


@pytest.fixture(autouse=True)
def reset_flags(pkg):
    ops = pkg.Int8TensorwiseOps
    saved = (list(ops.excluded_names), ops.dynamic_quantize, ops.enable_quarot, ops._is_prequantized, ops.use_triton)
    yield
    ops.excluded_names, ops.dynamic_quantize, ops.enable_quarot, ops._is_prequantized, ops.use_triton = saved


class FakeAdapter:
    def __init__(self, up, down, alpha=None, mid=None):
        self.loaded_keys = {"k"}
        self.weights = (up, down, alpha, mid, None, None)


def quantised_linear(pkg, n, k, per_row):
    lin = pkg.Int8TensorwiseOps.Linear(k, n, bias=False)
    scale = torch.rand(n, 1) * 0.01 + 0.001 if per_row else torch.tensor(0.004)
    lin._load_from_state_dict({"p.weight": torch.zeros(n, k, dtype=torch.int8), "p.weight_scale": scale}, "p.", {}, True, [], [], [])
    return lin


def toy_model(pkg):
    class Block(nn.Module):
        def __init__(self, per_row):
            super().__init__()
            self.qkv = quantised_linear(pkg, 24, 16, per_row)
            self.norm = nn.LayerNorm(16)

    class Toy(nn.Module):
        def __init__(self):
            super().__init__()
            self.blocks = nn.ModuleList([Block(False), Block(True)])
            self.img_in = nn.Linear(16, 16)

        def forward(self, x, timestep=None, context=None, transformer_options=None):
            return x

    return Toy()


# --------------------------------------------------------------------------- loader switches
def test_configure_ops_sets_switches_and_exclusions(pkg):
    nodes = pkg.nodes
    ops = nodes.configure_ops("flux2", True, True)
    assert ops is pkg.Int8TensorwiseOps and ops.dynamic_quantize and ops.enable_quarot and ops.use_triton
    assert not ops._is_prequantized
    assert "double_stream_modulation_img" in ops.excluded_names and "img_in" in ops.excluded_names
    ops = nodes.configure_ops("wan", False)
    assert ops.excluded_names == ["patch_embedding", "text_embedding", "time_embedding", "time_projection", "head", "img_emb"]
    assert not ops.dynamic_quantize and not ops.enable_quarot
    assert nodes.configure_ops("something-else", False).excluded_names == []
    assert set(nodes.MODEL_TYPES) == set(nodes.MODEL_EXCLUSIONS)


def test_node_ids_are_those_of_the_reference(pkg):
    assert set(pkg.NODE_CLASS_MAPPINGS) == {"OTUNetLoaderW8A8", "INT8LoraLoader", "INT8LoraLoaderStack",
                                            "INT8DynamicLoraLoader", "INT8DynamicLoraStack"}
    assert set(pkg.NODE_DISPLAY_NAME_MAPPINGS) == set(pkg.NODE_CLASS_MAPPINGS)
    for cls in pkg.NODE_CLASS_MAPPINGS.values():
        assert cls.RETURN_TYPES == ("MODEL",) and cls.CATEGORY == "loaders" and hasattr(cls, cls.FUNCTION)
    assert pkg.register_checkpoint_format() is False      # no ComfyUI in this environment


# --------------------------------------------------------------------------- patch upgrading
def test_resolve_module_spellings(pkg):
    model = toy_model(pkg)
    r = pkg.nodes.resolve_module
    assert r(model, "diffusion_model.blocks.1.qkv.weight") is model.blocks[1].qkv
    assert r(model, "blocks.0.qkv") is model.blocks[0].qkv
    assert r(model, ("diffusion_model.blocks.0.qkv.weight", (0, 8, 8))) is model.blocks[0].qkv
    with pytest.raises(AttributeError):
        r(model, "blocks.0.nothing.weight")


def test_upgrade_patches_only_touches_quantised_layers(pkg):
    model = toy_model(pkg)
    mk = lambda n, k: FakeAdapter(torch.randn(n, 4), torch.randn(4, k), 4.0)
    patches = {
        "diffusion_model.blocks.0.qkv.weight": mk(24, 16),
        ("diffusion_model.blocks.1.qkv.weight", (0, 8, 8)): mk(8, 16),
        "diffusion_model.img_in.weight": mk(16, 16),
        "diffusion_model.gone.weight": mk(16, 16),
    }
    out, n = pkg.nodes.upgrade_patches(model, patches, seed=7)
    assert n == 2 and set(out) == set(patches)
    a0 = out["diffusion_model.blocks.0.qkv.weight"]
    assert isinstance(a0, pkg.INT8LoRAPatchAdapter) and a0.seed == 7
    assert isinstance(a0.weight_scale, float) and a0.weight_scale == pytest.approx(0.004)
    assert a0.weights is patches["diffusion_model.blocks.0.qkv.weight"].weights
    a1 = out[("diffusion_model.blocks.1.qkv.weight", (0, 8, 8))]
    assert isinstance(a1, pkg.INT8LoRAPatchAdapter) and torch.equal(a1.weight_scale, model.blocks[1].qkv.weight_scale)
    assert out["diffusion_model.img_in.weight"] is patches["diffusion_model.img_in.weight"]
    assert out["diffusion_model.gone.weight"] is patches["diffusion_model.gone.weight"]


def test_stack_and_merge(pkg):
    model = toy_model(pkg)
    a, b = (FakeAdapter(torch.randn(24, 2), torch.randn(2, 16), 2.0) for _ in range(2))
    c = FakeAdapter(torch.randn(16, 2), torch.randn(2, 16), 4.0)
    layered = pkg.nodes.stack_patches([({"blocks.0.qkv.weight": a, "img_in.weight": c}, 0.5),
                                       ({"blocks.0.qkv.weight": b, "missing.weight": c}, -1.0)])
    assert layered["blocks.0.qkv.weight"] == [(a, 0.5), (b, -1.0)]
    merged, loose, quantised = pkg.nodes.merge_patch_stacks(model, layered, seed=3)
    assert quantised == 1 and set(merged) == {"blocks.0.qkv.weight", "img_in.weight"}
    m = merged["blocks.0.qkv.weight"]
    assert isinstance(m, pkg.INT8MergedLoRAPatchAdapter) and m.patches == [(a, 0.5), (b, -1.0)] and m.seed == 3
    assert m.weight_scale == pytest.approx(0.004) and merged["img_in.weight"].weight_scale == 1.0
    assert loose == [("missing.weight", c, -1.0)]
    # a float layer goes through the merged adapter in floating point: w + sum(strength * alpha/rank * up @ down)
    w = torch.randn(16, 16)
    got = merged["img_in.weight"].calculate_weight(w, "img_in.weight", 1.0, 1.0, None, None)
    assert torch.allclose(got, w + 0.5 * (4.0 / 2) * (c.weights[0] @ c.weights[1]), atol=1e-6)


def test_selected_loras_skips_empty_slots(pkg):
    kw = {"lora_1": "a.safetensors", "strength_1": 0.8, "lora_2": "None", "strength_2": 1.0,
          "lora_3": "c.safetensors", "strength_3": 0, "lora_5": "e.safetensors", "strength_5": -0.5}
    assert pkg.nodes.selected_loras(kw) == [("a.safetensors", 0.8), ("e.safetensors", -0.5)]


# --------------------------------------------------------------------------- dynamic LoRA hook
def test_dynamic_hook_composes_factors_and_caches(pkg):
    dl = pkg.dynamic_lora
    model = toy_model(pkg)
    up1, down1 = torch.randn(24, 4), torch.randn(4, 16)
    up2, down2 = torch.randn(24, 2), torch.randn(2, 16)
    p1 = {"diffusion_model.blocks.0.qkv.weight": FakeAdapter(up1, down1, 8.0)}
    p2 = {"diffusion_model.blocks.0.qkv.weight": FakeAdapter(up2, down2, None), "blocks.1.qkv.weight": FakeAdapter(up1, down1, 4.0)}
    options = {}
    dl.append_entry(options, "one", 0.5, p1)
    parent_list = options["transformer_options"][dl.OPTIONS_KEY]
    dl.append_entry(options, "two", 2.0, p2)
    assert len(parent_list) == 1 and len(options["transformer_options"][dl.OPTIONS_KEY]) == 2   # the parent's list is untouched

    hook = dl.DynamicLoRAHook.register(model)
    assert dl.DynamicLoRAHook.register(model) is hook                  # one hook per model
    model(torch.zeros(1, 16), transformer_options=options["transformer_options"])
    q0, q1 = model.blocks[0].qkv, model.blocks[1].qkv
    assert torch.equal(q0.lora_A, torch.cat([down1 * (8.0 / 4 * 0.5), down2 * 2.0]))
    assert torch.equal(q0.lora_B, torch.cat([up1, up2], dim=1)) and q0.lora_alpha is None
    assert torch.equal(q1.lora_A, down1 * (4.0 / 4 * 2.0)) and torch.equal(q1.lora_B, up1)
    # the same entries again: nothing is rebuilt
    kept = q0.lora_A
    model(torch.zeros(1, 16), transformer_options=options["transformer_options"])
    assert q0.lora_A is kept
    # transformer options inside the third positional argument, first LoRA only
    model(torch.zeros(1, 16), None, {"transformer_options": {dl.OPTIONS_KEY: parent_list}})
    assert torch.equal(q0.lora_A, down1 * (8.0 / 4 * 0.5)) and q1.lora_A is None
    # no entries: the factors are cleared
    model(torch.zeros(1, 16))
    assert q0.lora_A is None and q0.lora_B is None


def test_dynamic_hook_mid_factor(pkg):
    dl = pkg.dynamic_lora
    model = toy_model(pkg)
    up, down, mid = torch.randn(24, 4), torch.randn(4, 16), torch.randn(4, 4)
    dl.compose_into(model, [{"name": "x", "strength": 1.0, "patches": {"blocks.0.qkv.weight": FakeAdapter(up, down, None, mid)}}])
    assert torch.allclose(model.blocks[0].qkv.lora_A, mid @ down)


# --------------------------------------------------------------------------- nodes against stand-ins for ComfyUI
class FakePatcher:
    def __init__(self, model, options=None):
        self.model = types.SimpleNamespace(diffusion_model=model, model_type=types.SimpleNamespace(name="FLUX"))
        self.model_options = options if options is not None else {}
        self.added = []
        self.parent = None

    def clone(self):
        c = FakePatcher(self.model.diffusion_model, {k: dict(v) if isinstance(v, dict) else v for k, v in self.model_options.items()})
        c.parent = self
        return c

    def add_patches(self, patches, strength):
        self.added.append((dict(patches), strength))


@pytest.fixture
def fake_comfy(monkeypatch, pkg):
    calls = {}
    model = toy_model(pkg)
    lora_files = {
        "a.safetensors": {"diffusion_model.blocks.0.qkv.weight": FakeAdapter(torch.randn(24, 2), torch.randn(2, 16), 2.0),
                          "diffusion_model.img_in.weight": FakeAdapter(torch.randn(16, 2), torch.randn(2, 16), 2.0)},
        "b.safetensors": {"diffusion_model.blocks.0.qkv.weight": FakeAdapter(torch.randn(24, 2), torch.randn(2, 16), 2.0)},
    }
    fp = types.ModuleType("folder_paths")
    fp.get_filename_list = lambda kind: sorted(lora_files) if kind == "loras" else ["unet.safetensors"]
    fp.get_full_path = lambda kind, name: f"/models/{kind}/{name}"
    comfy = types.ModuleType("comfy")
    utils = types.ModuleType("comfy.utils")
    utils.load_torch_file = lambda path, safe_load=False: {"path": path, "safe": safe_load}
    lora = types.ModuleType("comfy.lora")
    lora.model_lora_keys_unet = lambda m, key_map: {"mapped": True}
    lora.load_lora = lambda state, key_map, log_missing=True: lora_files[state["path"].rsplit("/", 1)[1]]
    sd = types.ModuleType("comfy.sd")

    def load_diffusion_model(path, model_options=None):
        calls["load"] = (path, model_options)
        return "MODEL"

    sd.load_diffusion_model = load_diffusion_model
    comfy.utils, comfy.lora, comfy.sd = utils, lora, sd
    for name, mod in (("folder_paths", fp), ("comfy", comfy), ("comfy.utils", utils), ("comfy.lora", lora), ("comfy.sd", sd)):
        monkeypatch.setitem(sys.modules, name, mod)
    return types.SimpleNamespace(calls=calls, model=model, files=lora_files)


def test_loader_node_passes_the_ops_class(pkg, fake_comfy, monkeypatch):
    import torch._inductor.config as inductor_config
    monkeypatch.setattr(inductor_config, "pre_grad_custom_pass", None)       # (restored when the test ends)
    monkeypatch.setattr(pkg.compile_ops, "_installed", False)
    node = pkg.NODE_CLASS_MAPPINGS["OTUNetLoaderW8A8"]()
    inputs = node.INPUT_TYPES()["required"]
    assert inputs["unet_name"] == (["unet.safetensors"],) and inputs["model_type"][0][0] == "flux2"
    assert set(inputs) == {"unet_name", "weight_dtype", "model_type", "on_the_fly_quantization", "enable_quarot"}
    out = node.load_unet("unet.safetensors", "default", "qwen", True, enable_quarot=True)
    path, options = fake_comfy.calls["load"]
    assert out == ("MODEL",) and path == "/models/diffusion_models/unet.safetensors"
    assert options == {"custom_operations": pkg.Int8TensorwiseOps}
    assert pkg.Int8TensorwiseOps.excluded_names == ["time_text_embed", "img_in", "norm_out", "proj_out", "txt_in"]
    assert pkg.Int8TensorwiseOps.dynamic_quantize and pkg.Int8TensorwiseOps.enable_quarot
    # a model from this loader may be compiled later: inductor has been given the graph rewrites as its pre-grad pass
    assert inductor_config.pre_grad_custom_pass is not None and pkg.compile_ops._installed
    monkeypatch.setenv("I8F_NO_INDUCTOR_PASS", "1")
    monkeypatch.setattr(inductor_config, "pre_grad_custom_pass", None)
    monkeypatch.setattr(pkg.compile_ops, "_installed", False)
    node.load_unet("unet.safetensors", "default", "qwen", True)
    assert inductor_config.pre_grad_custom_pass is None


def test_lora_node_upgrades_and_registers(pkg, fake_comfy):
    node = pkg.NODE_CLASS_MAPPINGS["INT8LoraLoader"]()
    base = FakePatcher(fake_comfy.model)
    assert node.load_lora(base, "a.safetensors", 0) == (base,)            # strength 0: untouched, not even cloned
    (patched,) = node.load_lora(base, "a.safetensors", 0.75)
    assert patched.parent is base and base.added == []
    (patches, strength), = patched.added
    assert strength == 0.75
    assert isinstance(patches["diffusion_model.blocks.0.qkv.weight"], pkg.INT8LoRAPatchAdapter)
    assert patches["diffusion_model.blocks.0.qkv.weight"].seed == 318008
    assert patches["diffusion_model.img_in.weight"] is fake_comfy.files["a.safetensors"]["diffusion_model.img_in.weight"]


def test_lora_stack_node_merges(pkg, fake_comfy):
    node = pkg.NODE_CLASS_MAPPINGS["INT8LoraLoaderStack"]()
    opt = node.INPUT_TYPES()["optional"]
    assert len(opt) == 20 and opt["lora_1"] == (["None", "a.safetensors", "b.safetensors"],) and opt["strength_10"][1]["max"] == 10.0
    base = FakePatcher(fake_comfy.model)
    assert node.apply_stack(base, lora_1="None", strength_1=1.0) == (base,)
    (patched,) = node.apply_stack(base, lora_1="a.safetensors", strength_1=0.5, lora_2="b.safetensors", strength_2=-0.25)
    (patches, strength), = patched.added
    assert strength == 1.0
    m = patches["diffusion_model.blocks.0.qkv.weight"]
    assert isinstance(m, pkg.INT8MergedLoRAPatchAdapter) and [s for _, s in m.patches] == [0.5, -0.25]
    assert [s for _, s in patches["diffusion_model.img_in.weight"].patches] == [0.5]


def test_dynamic_nodes_register_hook_and_options(pkg, fake_comfy):
    dl = pkg.dynamic_lora
    base = FakePatcher(fake_comfy.model)
    stack = pkg.NODE_CLASS_MAPPINGS["INT8DynamicLoraStack"]()
    assert stack.INPUT_TYPES()["optional"]["strength_3"][1]["min"] == -20.0
    (patched,) = stack.apply_stack(base, lora_1="a.safetensors", strength_1=1.5, lora_2="b.safetensors", strength_2=0.5)
    entries = patched.model_options["transformer_options"][dl.OPTIONS_KEY]
    assert [(e["name"], e["strength"]) for e in entries] == [("a.safetensors", 1.5), ("b.safetensors", 0.5)]
    assert base.model_options == {}                                         # the input patcher is untouched
    assert isinstance(getattr(fake_comfy.model, dl.HOOK_ATTR), dl.DynamicLoRAHook)
    fake_comfy.model(torch.zeros(1, 16), transformer_options=patched.model_options["transformer_options"])
    assert fake_comfy.model.blocks[0].qkv.lora_A.shape == (4, 16) and fake_comfy.model.blocks[0].qkv.lora_B.shape == (24, 4)
