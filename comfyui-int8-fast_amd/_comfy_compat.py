"""ComfyUI base classes, or minimal stand-ins when ComfyUI is not importable.

The ops class and the LoRA adapters subclass ComfyUI types (comfy.ops.manual_cast,
comfy.weight_adapter.lora.LoRAAdapter).  Outside ComfyUI (unit tests, benchmarks)
the stand-ins below provide just what those subclasses use, with ComfyUI's
attribute names, so the same classes can be exercised.
"""
from __future__ import annotations

import torch
from torch import nn

try:  # pragma: no cover - depends on the host application
    from comfy.ops import cast_bias_weight, manual_cast, uncast_bias_weight

    HAVE_COMFY_OPS = True
except ImportError:
    HAVE_COMFY_OPS = False

    class _CastMixin:
        comfy_cast_weights = False
        weight_function: list = []
        bias_function: list = []

        def reset_parameters(self):
            return None

    class manual_cast:  # noqa: N801 - ComfyUI's name
        class Linear(_CastMixin, nn.Linear):
            pass

        class GroupNorm(_CastMixin, nn.GroupNorm):
            pass

        class LayerNorm(_CastMixin, nn.LayerNorm):
            pass

        class Conv2d(_CastMixin, nn.Conv2d):
            pass

        class Conv3d(_CastMixin, nn.Conv3d):
            pass

        class ConvTranspose2d(_CastMixin, nn.ConvTranspose2d):
            pass

        class Embedding(_CastMixin, nn.Embedding):
            pass

    def cast_bias_weight(s, input=None, dtype=None, device=None, bias_dtype=None, offloadable=False):
        if input is not None:
            dtype = dtype or input.dtype
            device = device or input.device
            bias_dtype = bias_dtype or dtype
        weight = s.weight.to(device=device, dtype=dtype)
        bias = None if s.bias is None else s.bias.to(device=device, dtype=bias_dtype)
        return weight, bias, None

    def uncast_bias_weight(s, weight, bias, offload_stream):
        return None


try:  # pragma: no cover
    from comfy.weight_adapter.lora import LoRAAdapter

    HAVE_COMFY_LORA = True
except ImportError:
    HAVE_COMFY_LORA = False

    class LoRAAdapter:
        """Stand-in with the two attributes the INT8 adapters read."""

        name = "lora"

        def __init__(self, loaded_keys, weights):
            self.loaded_keys = loaded_keys
            self.weights = weights


def compute_device() -> torch.device:
    """Where merges are computed: ComfyUI's device choice when available, else the current GPU."""
    try:  # pragma: no cover
        import comfy.model_management

        return comfy.model_management.get_torch_device()
    except ImportError:
        if not torch.cuda.is_available():
            raise RuntimeError("the INT8 engine needs a gfx950 GPU (no CPU path)") from None
        return torch.device("cuda", torch.cuda.current_device())
