"""ComfyUI graph nodes of the INT8 path: the model loader and the LoRA loaders.

Same node ids, inputs and behaviour as the reference's nodes (int8_unet_loader.py:9-100,
int8_lora.py:7-210, int8_dynamic_lora.py:8-103, ids in __init__.py:90-104), so saved workflows load
unchanged.  The nodes hold no arithmetic: they set the switches of `Int8TensorwiseOps`, hand it to
ComfyUI's loader as `custom_operations`, and swap ComfyUI's LoRA adapters for the INT8 ones on
quantised layers.  ComfyUI modules (`folder_paths`, `comfy.*`) are imported when a node runs, not
when this module is imported, so that the logic underneath (`configure_ops`, `upgrade_patches`,
`merge_patch_stacks`) can be used and tested without ComfyUI.
"""
from __future__ import annotations

import logging
import os

import torch

from . import compile_ops
from .dynamic_lora import DynamicLoRAHook, append_entry
from .int8_quant import INT8LoRAPatchAdapter, INT8MergedLoRAPatchAdapter, Int8TensorwiseOps

DEFAULT_SEED = 318008
MAX_STACK = 10

# Layers that stay in floating point, by model family: a layer is excluded when its name contains
# one of the fragments (int8_unet_loader.py:53-95).
MODEL_EXCLUSIONS = {
    "flux2": ("img_in", "time_in", "guidance_in", "txt_in", "final_layer", "double_stream_modulation_img",
              "double_stream_modulation_txt", "single_stream_modulation"),
    "z-image": ("cap_embedder", "t_embedder", "x_embedder", "cap_pad_token", "context_refiner", "final_layer",
                "noise_refiner", "adaLN", "x_pad_token", "layers.0."),
    "chroma": ("distilled_guidance_layer", "final_layer", "img_in", "txt_in", "nerf_image_embedder", "nerf_blocks",
               "nerf_final_layer_conv", "__x0__"),
    "wan": ("patch_embedding", "text_embedding", "time_embedding", "time_projection", "head", "img_emb"),
    "ltx2": ("adaln_single", "audio_adaln_single", "audio_caption_projection", "audio_patchify_proj", "audio_proj_out",
             "audio_scale_shift_table", "av_ca_a2v_gate_adaln_single", "av_ca_audio_scale_shift_adaln_single",
             "av_ca_v2a_gate_adaln_single", "av_ca_video_scale_shift_adaln_single", "caption_projection",
             "patchify_proj", "proj_out", "scale_shift_table"),
    "qwen": ("time_text_embed", "img_in", "norm_out", "proj_out", "txt_in"),
    "ernie": ("time", "x_embedder", "adaLN", "final", "text_proj", "norm", "layers.0.", "layers.35"),
    "anima": ("embed", "llm", "blocks.0.", "blocks.1.", "blocks.2."),
}
MODEL_TYPES = ["flux2", "z-image", "chroma", "wan", "ltx2", "qwen", "ernie", "anima"]   # order of the node's menu


# --------------------------------------------------------------------------- logic without ComfyUI
def configure_ops(model_type: str, on_the_fly_quantization: bool, enable_quarot: bool = False):
    """Set the class-level switches that `Int8TensorwiseOps.Linear` reads while a state dict loads."""
    ops = Int8TensorwiseOps
    ops.excluded_names = list(MODEL_EXCLUSIONS.get(model_type, ()))
    ops.dynamic_quantize = bool(on_the_fly_quantization)
    ops.enable_quarot = bool(enable_quarot)
    ops.use_triton = True          # the fused kernel path; the reference forces it as well (int8_unet_loader.py:50)
    ops._is_prequantized = False
    return ops


def resolve_module(diffusion_model, patch_key):
    """The module a patch key names: 'diffusion_model.a.3.b.weight', 'a.3.b', or (name, offset) tuples."""
    name = patch_key[0] if isinstance(patch_key, tuple) else patch_key
    if name.endswith(".weight"):
        name = name[: -len(".weight")]
    parts = name.split(".")
    if parts and parts[0] == "diffusion_model":
        parts = parts[1:]
    module = diffusion_model
    for part in parts:
        module = module[int(part)] if part.isdigit() else getattr(module, part)
    return module


def _layer_scale(module):
    """The weight scale an adapter needs: a float for one scale, the [N,1] tensor for per-row scales."""
    scale = module._get_weight_scale()
    if isinstance(scale, torch.Tensor) and scale.numel() == 1:
        return scale.item()
    return scale


def _is_int8_layer(module) -> bool:
    return bool(getattr(module, "_is_quantized", False))


def upgrade_patches(diffusion_model, patch_dict: dict, seed: int = DEFAULT_SEED):
    """Replace the adapter of every patch that targets a quantised layer by `INT8LoRAPatchAdapter`.

    Returns (patches, number of upgraded patches).  Patches whose target cannot be resolved, or is
    not quantised, keep ComfyUI's adapter and are applied in floating point by ComfyUI."""
    out, upgraded = {}, 0
    for key, adapter in patch_dict.items():
        try:
            module = resolve_module(diffusion_model, key)
            if _is_int8_layer(module):
                out[key] = INT8LoRAPatchAdapter(adapter.loaded_keys, adapter.weights, _layer_scale(module), seed=seed)
                upgraded += 1
                continue
        except (AttributeError, KeyError, IndexError, TypeError, ValueError):
            pass
        out[key] = adapter
    return out, upgraded


def stack_patches(patch_dicts_with_strength):
    """[(patch_dict, strength), ...] -> key -> [(adapter, strength), ...] in stack order."""
    layered: dict = {}
    for patch_dict, strength in patch_dicts_with_strength:
        for key, adapter in patch_dict.items():
            layered.setdefault(key, []).append((adapter, strength))
    return layered


def merge_patch_stacks(diffusion_model, layered: dict, seed: int = DEFAULT_SEED):
    """One `INT8MergedLoRAPatchAdapter` per key: the deltas of a stack are summed in floating point and
    rounded stochastically once (int8_quant.py:364-402).

    Returns (merged patches, patches to apply one by one because their target did not resolve,
    number of quantised layers)."""
    merged, loose, quantised = {}, [], 0
    for key, patches in layered.items():
        try:
            module = resolve_module(diffusion_model, key)
            scale = 1.0
            if _is_int8_layer(module):
                scale = _layer_scale(module)
                quantised += 1
            merged[key] = INT8MergedLoRAPatchAdapter(patches, scale, seed=seed)
        except Exception:   # noqa: BLE001 - any failure falls back to ComfyUI's own sequential patching
            loose.extend((key, adapter, strength) for adapter, strength in patches)
    return merged, loose, quantised


def stack_inputs(strength_range: float):
    """The ten optional (lora_i, strength_i) inputs of a stack node."""
    import folder_paths

    names = ["None"] + folder_paths.get_filename_list("loras")
    optional = {}
    for i in range(1, MAX_STACK + 1):
        optional[f"lora_{i}"] = (names,)
        optional[f"strength_{i}"] = ("FLOAT", {"default": 1.0, "min": -strength_range, "max": strength_range, "step": 0.01})
    return {"required": {"model": ("MODEL",)}, "optional": optional}


def selected_loras(kwargs: dict):
    """(name, strength) of the filled slots of a stack node, in slot order."""
    picked = []
    for i in range(1, MAX_STACK + 1):
        name, strength = kwargs.get(f"lora_{i}"), kwargs.get(f"strength_{i}", 0)
        if name and name != "None" and strength != 0:
            picked.append((name, strength))
    return picked


# --------------------------------------------------------------------------- ComfyUI side
def _load_patch_dict(model_patcher, lora_name: str):
    import comfy.lora
    import comfy.utils
    import folder_paths

    state = comfy.utils.load_torch_file(folder_paths.get_full_path("loras", lora_name), safe_load=True)
    key_map = {}
    if model_patcher.model.model_type.name != "ModelType.CLIP":
        key_map = comfy.lora.model_lora_keys_unet(model_patcher.model, key_map)
    return comfy.lora.load_lora(state, key_map, log_missing=True)


class UNetLoaderINTW8A8:
    """Load a diffusion model with INT8 linears (pre-quantised checkpoint, or quantised while loading)."""

    RETURN_TYPES = ("MODEL",)
    FUNCTION = "load_unet"
    CATEGORY = "loaders"
    DESCRIPTION = "Load INT8 quantized diffusion models; linears run as W8A8 on the matrix cores."

    @classmethod
    def INPUT_TYPES(cls):
        import folder_paths

        return {"required": {
            "unet_name": (folder_paths.get_filename_list("diffusion_models"),),
            "weight_dtype": (["default", "fp8_e4m3fn", "fp16", "bf16"],),
            "model_type": (list(MODEL_TYPES),),
            "on_the_fly_quantization": ("BOOLEAN", {"default": False}),
            "enable_quarot": ("BOOLEAN", {"default": False, "tooltip": "Enable QuaRot (Hadamard rotation) for better quantization."}),
        }}

    def load_unet(self, unet_name, weight_dtype, model_type, on_the_fly_quantization, enable_quarot=False):
        import folder_paths
        from comfy.sd import load_diffusion_model

        ops = configure_ops(model_type, on_the_fly_quantization, enable_quarot)
        # a model loaded here may be handed to torch.compile later (ComfyUI's compile nodes use the inductor backend):
        # have inductor apply the graph rewrites to graphs that hold this package's operators
        if not os.environ.get("I8F_NO_INDUCTOR_PASS"):
            compile_ops.install_inductor_pass()
        path = folder_paths.get_full_path("diffusion_models", unet_name)
        return (load_diffusion_model(path, model_options={"custom_operations": ops}),)


class INT8LoraLoader:
    """Merge one LoRA into the INT8 weights with stochastic rounding, through ComfyUI's patch system."""

    RETURN_TYPES = ("MODEL",)
    FUNCTION = "load_lora"
    CATEGORY = "loaders"
    DESCRIPTION = "Loads LoRA for INT8 models with INT8-space patching and stochastic rounding."

    @classmethod
    def INPUT_TYPES(cls):
        import folder_paths

        return {"required": {
            "model": ("MODEL",),
            "lora_name": (folder_paths.get_filename_list("loras"),),
            "strength": ("FLOAT", {"default": 1.0, "min": -10.0, "max": 10.0, "step": 0.01}),
        }}

    def load_lora(self, model, lora_name, strength, seed=DEFAULT_SEED):
        if strength == 0:
            return (model,)
        patcher = model.clone()
        patch_dict = _load_patch_dict(patcher, lora_name)
        patches, upgraded = upgrade_patches(patcher.model.diffusion_model, patch_dict, seed)
        patcher.add_patches(patches, strength)
        logging.info("INT8 LoRA: '%s' at strength %.2f, %d quantized layers, %d others", lora_name, strength, upgraded,
                     len(patch_dict) - upgraded)
        return (patcher,)


class INT8LoraLoaderStack:
    """Merge up to ten LoRAs at once: their deltas are summed in floating point and rounded once."""

    RETURN_TYPES = ("MODEL",)
    FUNCTION = "apply_stack"
    CATEGORY = "loaders"
    DESCRIPTION = "Applies a stack of LoRAs to INT8 models with a single stochastic rounding."

    @classmethod
    def INPUT_TYPES(cls):
        return stack_inputs(10.0)

    def apply_stack(self, model, seed=DEFAULT_SEED, **kwargs):
        picked = selected_loras(kwargs)
        if not picked:
            return (model,)
        patcher = model.clone()
        layered = stack_patches((_load_patch_dict(patcher, name), strength) for name, strength in picked)
        merged, loose, quantised = merge_patch_stacks(patcher.model.diffusion_model, layered, seed)
        for key, adapter, strength in loose:
            patcher.add_patches({key: adapter}, strength)
        patcher.add_patches(merged, 1.0)   # the merged adapters carry the individual strengths
        logging.info("INT8 LoRA stack: %d LoRAs merged for %d quantized layers", len(picked), quantised)
        return (patcher,)


class INT8DynamicLoraLoader:
    """Attach one LoRA as a side branch of the INT8 linears (nothing is merged into the weights)."""

    RETURN_TYPES = ("MODEL",)
    FUNCTION = "load_lora"
    CATEGORY = "loaders"

    @classmethod
    def INPUT_TYPES(cls):
        import folder_paths

        return {"required": {
            "model": ("MODEL",),
            "lora_name": (folder_paths.get_filename_list("loras"),),
            "strength": ("FLOAT", {"default": 1.0, "min": -20.0, "max": 20.0, "step": 0.01}),
        }}

    def load_lora(self, model, lora_name, strength):
        if strength == 0:
            return (model,)
        patcher = model.clone()
        patch_dict = _load_patch_dict(patcher, lora_name)
        DynamicLoRAHook.register(patcher.model.diffusion_model)
        append_entry(patcher.model_options, lora_name, strength, patch_dict)
        return (patcher,)


class INT8DynamicLoraStack:
    """Up to ten dynamic LoRAs in one node."""

    RETURN_TYPES = ("MODEL",)
    FUNCTION = "apply_stack"
    CATEGORY = "loaders"

    @classmethod
    def INPUT_TYPES(cls):
        return stack_inputs(20.0)

    def apply_stack(self, model, **kwargs):
        loader = INT8DynamicLoraLoader()
        for name, strength in selected_loras(kwargs):
            (model,) = loader.load_lora(model, name, strength)
        return (model,)


NODE_CLASS_MAPPINGS = {
    "OTUNetLoaderW8A8": UNetLoaderINTW8A8,
    "INT8LoraLoader": INT8LoraLoader,
    "INT8LoraLoaderStack": INT8LoraLoaderStack,
    "INT8DynamicLoraLoader": INT8DynamicLoraLoader,
    "INT8DynamicLoraStack": INT8DynamicLoraStack,
}
NODE_DISPLAY_NAME_MAPPINGS = {
    "OTUNetLoaderW8A8": "Load Diffusion Model INT8 (W8A8)",
    "INT8LoraLoader": "Load LoRA INT8 (Stochastic)",
    "INT8LoraLoaderStack": "INT8 LoRA Stack (Stochastic)",
    "INT8DynamicLoraLoader": "Load LoRA INT8 (Dynamic)",
    "INT8DynamicLoraStack": "INT8 LoRA Stack (Dynamic)",
}
