"""MI355X-native INT8 linear engine for ComfyUI (gfx950 HIP kernels behind a C ABI).

The package replaces the W8A8 linear hot path of ComfyUI-INT8-Fast:

    int8_fused_kernel   quantise + GEMM + dequant pipeline   (HIP, was Triton)
    int8_quant          quantisation helpers, Int8TensorwiseOps, INT8 LoRA adapters
    quarot              128-block Hadamard rotation
    compile_ops         torch.library operators (namespace i8f) for torch.compile
    nodes               ComfyUI graph nodes (model loader, LoRA loaders); ComfyUI is imported when they run
    dynamic_lora        hook for un-merged LoRA side branches
    _lib                ctypes binding of libi8f_gfx950.so (include/i8f.h)
    build               hipcc build of the library

The directory name is ComfyUI's convention for custom nodes and is not a Python
identifier; ComfyUI imports such packages by path, and so do this repository's
tests (see `load_package` in __graft_entry__.py).  The node ids and the registration
of the `int8_tensorwise` checkpoint format are those of the reference
(__init__.py:19-104), so saved workflows and pre-quantised checkpoints load unchanged.
"""
import logging

import torch

from . import _lib, compile_ops, dynamic_lora, int8_fused_kernel, int8_quant, nodes, quarot  # noqa: F401
from .int8_fused_kernel import (  # noqa: F401
    hip_int8_linear,
    hip_int8_linear_pair,
    hip_int8_linear_per_row,
    hip_quantize_rowwise,
    triton_int8_linear,
    triton_int8_linear_per_row,
    triton_quantize_rowwise,
)
from .int8_quant import (  # noqa: F401
    INT8LoRAPatchAdapter,
    INT8MergedLoRAPatchAdapter,
    Int8TensorwiseOps,
    dequantize,
    forward_fanout,
    forward_pair,
    int8_forward_dynamic,
    int8_forward_dynamic_per_row,
    quantize_int8,
    quantize_int8_axiswise,
    quantize_int8_tensorwise,
    stochastic_round_int8_delta,
)

from .nodes import NODE_CLASS_MAPPINGS, NODE_DISPLAY_NAME_MAPPINGS  # noqa: E402,F401


def register_checkpoint_format() -> bool:
    """Tell ComfyUI's quantisation registry about checkpoints tagged `int8_tensorwise`
    (reference __init__.py:19-62): int8 storage, parameters `weight_scale` and `input_scale`
    (the latter is read so that loading does not complain, and ignored: activations are
    quantised per token at run time).  Returns False outside ComfyUI."""
    try:
        from comfy.quant_ops import QUANT_ALGOS, QuantizedLayout, register_layout_class
    except ImportError:
        return False

    class Int8TensorwiseLayout(QuantizedLayout):
        class Params:
            def __init__(self, scale=None, orig_dtype=None, orig_shape=None, **_):
                self.scale, self.orig_dtype, self.orig_shape = scale, orig_dtype, orig_shape

            def clone(self):
                scale = self.scale.clone() if isinstance(self.scale, torch.Tensor) else self.scale
                return type(self)(scale=scale, orig_dtype=self.orig_dtype, orig_shape=self.orig_shape)

        @classmethod
        def state_dict_tensors(cls, qdata, params):
            return {"": qdata, "weight_scale": params.scale}

        @classmethod
        def dequantize(cls, qdata, params):
            return qdata.float() * params.scale

    try:
        register_layout_class("Int8TensorwiseLayout", Int8TensorwiseLayout)
        QUANT_ALGOS.setdefault("int8_tensorwise", {"storage_t": torch.int8, "parameters": {"weight_scale", "input_scale"},
                                                   "comfy_tensor_layout": "Int8TensorwiseLayout"})
    except Exception as e:  # noqa: BLE001 - an older ComfyUI with another registry interface
        logging.error("INT8 Fast: could not register the int8_tensorwise layout: %s", e)
        return False
    return True


register_checkpoint_format()

__all__ = ["NODE_CLASS_MAPPINGS", "NODE_DISPLAY_NAME_MAPPINGS", "Int8TensorwiseOps"]
