"""Dynamic (un-merged) LoRA: factors attached to the quantised linears and applied as a side branch.

Mirrors `DynamicLoRAHook` of the reference (int8_quant.py:415-507).  A model patcher carries a list
`transformer_options["dynamic_loras"]` of `{"name", "strength", "patches"}` entries; a forward
pre-hook on the diffusion model turns the entries that are current for this call into two matrices
per layer,

    lora_A = concat_rows( strength_i * alpha_i / rank_i * down_i )      [sum of ranks, K]
    lora_B = concat_cols( up_i )                                        [N, sum of ranks]

and `Int8TensorwiseOps.Linear.forward` adds `(x @ lora_A.T) @ lora_B.T` to its result (the addition
itself runs inside the GEMM epilogue).  The composition is redone only when the set of entries
changes.  The reference marks this path as deprecated in favour of the merging loaders; it is kept
so that existing workflows run.
"""
from __future__ import annotations

import torch

OPTIONS_KEY = "dynamic_loras"
HOOK_ATTR = "_dynamic_lora_hook"


def _entries_signature(entries):
    """Identity of a set of entries: which patch dictionaries, at which strengths, in which order."""
    if not entries:
        return None
    return tuple((id(e["patches"]), float(e["strength"])) for e in entries)


def _factor_pair(adapter, strength):
    """(A, B) of one LoRA patch: A = scaled down-projection (through `mid` if present), B = up."""
    up, down, alpha, mid = adapter.weights[0], adapter.weights[1], adapter.weights[2], adapter.weights[3]
    rank = down.shape[0] if down.ndim >= 2 else 1
    scale = strength if alpha is None else (alpha / rank) * strength
    a = down
    if mid is not None:
        a = torch.mm(mid.flatten(1), down.flatten(1)).reshape(down.shape)
    return a * scale, up


def group_by_layer(entries):
    """patch key -> [(adapter, strength), ...] over all entries, in entry order."""
    grouped: dict = {}
    for entry in entries or ():
        for key, adapter in entry["patches"].items():
            grouped.setdefault(key, []).append((adapter, entry["strength"]))
    return grouped


def compose_into(diffusion_model, entries) -> int:
    """Set `lora_A` / `lora_B` on every module that has those attributes; returns how many got factors.

    A module is matched by `diffusion_model.<name>.weight` or `<name>.weight`, the two spellings
    ComfyUI's key maps produce (int8_quant.py:462-468)."""
    grouped = group_by_layer(entries)
    touched = 0
    for name, module in diffusion_model.named_modules():
        if not hasattr(module, "lora_A"):
            continue
        patches = grouped.get(f"diffusion_model.{name}.weight") or grouped.get(f"{name}.weight")
        if not patches:
            module.lora_A = module.lora_B = module.lora_alpha = None
            continue
        pairs = [_factor_pair(adapter, strength) for adapter, strength in patches]
        weight = getattr(module, "weight", None)
        device = weight.device if isinstance(weight, torch.Tensor) else torch.device("cpu")
        module.lora_A = torch.cat([a for a, _ in pairs], dim=0).to(device)
        module.lora_B = torch.cat([b for _, b in pairs], dim=1).to(device)
        module.lora_alpha = None   # the scaling is already inside lora_A
        touched += 1
    return touched


class DynamicLoRAHook:
    """Forward pre-hook that keeps the modules' factors in step with the caller's patcher."""

    def __init__(self):
        self.current_lora_id = None

    @staticmethod
    def _options(args, kwargs):
        options = kwargs.get("transformer_options") or {}
        if not options and len(args) > 2 and isinstance(args[2], dict):
            options = args[2].get("transformer_options", {})   # some models pass them inside the context
        return options

    def pre_forward(self, module, input_args, input_kwargs):
        entries = self._options(input_args, input_kwargs).get(OPTIONS_KEY, [])
        signature = _entries_signature(entries)
        if signature != self.current_lora_id:
            self.apply_composition(module, entries)
            self.current_lora_id = signature
        return None

    def apply_composition(self, diffusion_model, dynamic_loras):
        compose_into(diffusion_model, dynamic_loras)

    @classmethod
    def register(cls, diffusion_model):
        hook = getattr(diffusion_model, HOOK_ATTR, None)
        if hook is None:
            hook = cls()
            setattr(diffusion_model, HOOK_ATTR, hook)
            diffusion_model.register_forward_pre_hook(hook.pre_forward, with_kwargs=True)
        return hook


def append_entry(model_options: dict, name: str, strength: float, patches: dict) -> None:
    """Add one LoRA to a patcher's options without touching the list its parent patcher holds."""
    options = model_options.setdefault("transformer_options", {})
    options[OPTIONS_KEY] = list(options.get(OPTIONS_KEY, ())) + [{"name": name, "strength": strength, "patches": patches}]
