"""MI355X-native INT8 linear engine for ComfyUI (gfx950 HIP kernels behind a C ABI).

The package replaces the W8A8 linear hot path of ComfyUI-INT8-Fast:

    int8_fused_kernel   quantise + GEMM + dequant pipeline   (HIP, was Triton)
    int8_quant          quantisation helpers, Int8TensorwiseOps, INT8 LoRA adapters
    quarot              128-block Hadamard rotation
    compile_ops         torch.library operators (namespace i8f) for torch.compile
    _lib                ctypes binding of libi8f_gfx950.so (include/i8f.h)
    build               hipcc build of the library

The directory name is ComfyUI's convention for custom nodes and is not a Python
identifier; ComfyUI imports such packages by path, and so do this repository's
tests (see `load_package` in __graft_entry__.py).  ComfyUI's graph nodes (loader,
LoRA loader nodes) are host-application glue and are not part of this package;
`Int8TensorwiseOps` is the object they would pass as `custom_operations`.
"""
from . import _lib, compile_ops, int8_fused_kernel, int8_quant, quarot  # noqa: F401
from .int8_fused_kernel import (  # noqa: F401
    hip_int8_linear,
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
    int8_forward_dynamic,
    int8_forward_dynamic_per_row,
    quantize_int8,
    quantize_int8_axiswise,
    quantize_int8_tensorwise,
    stochastic_round_int8_delta,
)

# No graph nodes are defined here (see the module docstring).
NODE_CLASS_MAPPINGS: dict = {}
NODE_DISPLAY_NAME_MAPPINGS: dict = {}

__all__ = ["NODE_CLASS_MAPPINGS", "NODE_DISPLAY_NAME_MAPPINGS", "Int8TensorwiseOps"]
