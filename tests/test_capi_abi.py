"""The C ABI: the library loads, exports everything include/i8f.h declares, and rejects bad
arguments on the host before anything is launched (so these run without a GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "i8f.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(i8f_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points(L):
    names = declared_functions()
    assert set(names) == set(L.EXPORTS)
    assert len(names) == 26


def test_library_exports_every_declared_symbol(L):
    lib = L.lib()
    for name in declared_functions():
        assert getattr(lib, name) is not None


def test_version_and_status_strings(L):
    lib = L.lib()
    header = open(os.path.join(ROOT, "include", "i8f.h")).read()
    assert lib.i8f_version() == int(re.search(r"#define I8F_VERSION (\d+)", header).group(1))
    assert lib.i8f_status_string(0) == b"ok"
    for code in (-1, -2, -3, -4):
        assert lib.i8f_status_string(code) not in (b"ok", b"unknown status")
    assert lib.i8f_status_string(-99) == b"unknown status"
    assert lib.i8f_last_hip_error() == 0


def test_bad_arguments_are_rejected_before_any_launch(L):
    lib = L.lib()
    null = ctypes.c_void_p(None)
    one = ctypes.c_void_p(16)   # never dereferenced: validation fails first
    INVALID, UNSUPPORTED = -1, -2
    # negative sizes, bad dtype, bad rotate block, rotation with K not a multiple of 128
    assert lib.i8f_quant_rowwise(one, L.BF16, -1, 8, 8, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise(one, 7, 4, 8, 8, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise(one, L.BF16, 4, 256, 256, 64, one, one, null) == UNSUPPORTED
    assert lib.i8f_quant_rowwise(one, L.BF16, 4, 200, 200, 128, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise(one, L.BF16, 4, 256, 128, 0, one, one, null) == INVALID     # ldx < K
    assert lib.i8f_quant_rowwise(null, L.BF16, 4, 256, 256, 0, one, one, null) == INVALID    # NULL input
    assert lib.i8f_quant_rowwise(null, L.BF16, 0, 256, 256, 0, null, null, null) == 0        # empty: nothing to do
    groups = (L._QuantGroup * 2)()
    groups[0].x, groups[0].M, groups[0].ldx, groups[0].q, groups[0].scale = 16, 4, 256, 16, 16
    groups[1].x, groups[1].M, groups[1].ldx, groups[1].q, groups[1].scale = 16, 4, 128, 16, 16    # ldx < K
    assert lib.i8f_quant_rowwise_grouped(ctypes.byref(groups), 2, L.BF16, 256, 0, null) == INVALID
    groups[1].ldx, groups[1].q = 256, None                                                          # NULL output
    assert lib.i8f_quant_rowwise_grouped(ctypes.byref(groups), 2, L.BF16, 256, 0, null) == INVALID
    assert lib.i8f_quant_rowwise_grouped(ctypes.byref(groups), 2, L.BF16, 200, 128, null) == INVALID
    assert lib.i8f_quant_rowwise_grouped(ctypes.byref(groups), 2, 9, 256, 0, null) == INVALID
    assert lib.i8f_quant_rowwise_grouped(null, 1, L.BF16, 256, 0, null) == INVALID
    assert lib.i8f_quant_rowwise_grouped(null, 0, L.BF16, 256, 0, null) == 0
    assert lib.i8f_rotate128(one, L.F32, 4, 100, 100, one, null) == INVALID
    # K-split workspace: too small, misaligned; the size is what the header says (16 MB + 4 KB)
    nbytes = lib.i8f_linear_w8a8_workspace_bytes()
    assert nbytes == 4096 + 256 * 128 * 128 * 4
    args = (one, one, one, one, 1.0, 0, null, 0, null, one, L.BF16, 4, 8, 16, 0)
    assert lib.i8f_linear_w8a8_splitk(*args, one, nbytes - 1, null) == INVALID
    assert lib.i8f_linear_w8a8_splitk(*args, ctypes.c_void_p(24), nbytes, null) == INVALID
    assert lib.i8f_linear_w8a8_splitk(one, one, one, one, 1.0, 0, null, 0, null, one, 9, 4, 8, 16, 0, one, nbytes, null) == INVALID  # bad dtype
    # quantiser with a prologue: unknown operation, modulation without its vectors or with a bad group size
    assert lib.i8f_quant_rowwise_prologue(one, L.BF16, 4, 256, 256, 7, null, null, 1, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_prologue(one, L.BF16, 4, 256, 256, L.PRO_MODULATE, null, one, 4, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_prologue(one, L.BF16, 4, 256, 256, L.PRO_MODULATE, one, one, 0, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_prologue(one, L.BF16, 4, 200, 200, L.PRO_GELU_TANH, null, null, 1, 128, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_prologue(null, L.BF16, 0, 256, 256, L.PRO_GELU_TANH, null, null, 1, 0, null, null, null) == 0
    # tensorwise quantiser: workspace missing or too small, tensor beyond the static scratch's limit
    need = lib.i8f_quant_tensorwise_workspace_bytes(1 << 20)
    assert 0 < need <= 4096 and lib.i8f_quant_tensorwise_workspace_bytes(1 << 40) == 4096
    assert lib.i8f_quant_tensorwise(one, L.BF16, 1 << 20, one, one, null, need, null) == INVALID
    assert lib.i8f_quant_tensorwise(one, L.BF16, 1 << 20, one, one, one, need - 4, null) == INVALID
    assert lib.i8f_quant_tensorwise(one, 9, 16, one, one, one, 4096, null) == INVALID
    assert lib.i8f_quant_tensorwise(null, L.BF16, 16, one, one, one, 4096, null) == INVALID
    assert lib.i8f_quant_tensorwise_static(one, L.BF16, (1 << 32) + 1, one, one, null) == UNSUPPORTED
    assert lib.i8f_quant_tensorwise_static(one, L.BF16, -1, one, one, null) == INVALID
    assert lib.i8f_gemm_i32(one, one, -1, 4, 4, one, null) == INVALID
    assert lib.i8f_gemm_i32(null, one, 4, 4, 4, one, null) == INVALID
    assert lib.i8f_gemm_i32(null, null, 0, 4, 4, null, null) == 0
    assert lib.i8f_linear_w8a8(one, one, one, null, 1.0, L.SCALE_ROW, null, 0, one, L.BF16, 4, 4, 4, 0, null) == INVALID  # row scales missing
    assert lib.i8f_linear_w8a8(one, one, one, one, 1.0, 5, null, 0, one, L.BF16, 4, 4, 4, 0, null) == INVALID             # bad scale mode
    assert lib.i8f_linear_w8a8(one, one, one, one, 1.0, 0, null, 0, one, L.BF16, 4, 4, 4, 9, null) == INVALID             # bad epilogue order
    # side branch in the epilogue: operands missing, binary32 output, rank not a multiple of 16 or above 64
    assert lib.i8f_linear_w8a8_lora(one, one, one, one, 1.0, 1, null, 0, null, one, 16, 0, 0.0, one, L.BF16, 32, 32, 128, 0, null) == INVALID
    assert lib.i8f_linear_w8a8_lora(one, one, one, one, 1.0, 1, null, 0, one, one, 16, 0, 0.0, one, L.F32, 32, 32, 128, 0, null) == UNSUPPORTED
    assert lib.i8f_linear_w8a8_lora(one, one, one, one, 1.0, 1, null, 0, one, one, 24, 0, 0.0, one, L.BF16, 32, 32, 128, 0, null) == UNSUPPORTED
    assert lib.i8f_linear_w8a8_lora(one, one, one, one, 1.0, 1, null, 0, one, one, 80, 0, 0.0, one, L.BF16, 32, 32, 128, 0, null) == UNSUPPORTED
    # normalising quantiser: operands missing, negative eps, binary32 rows
    assert lib.i8f_quant_rowwise_norm_modulate(one, L.BF16, 4, 256, 256, 1e-6, null, one, 4, 0, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_norm_modulate(one, L.BF16, 4, 256, 256, -1.0, one, one, 4, 0, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_norm_modulate(one, L.BF16, 4, 256, 256, 1e-6, one, one, 0, 0, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_norm_modulate(one, L.BF16, 4, 200, 200, 1e-6, one, one, 4, 0, 128, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_norm_modulate(null, L.BF16, 0, 256, 256, 1e-6, null, null, 1, 0, 0, null, null, null) == 0
    assert lib.i8f_quant_rowwise_rms_norm(one, L.BF16, 4, 256, 256, -1.0, null, null, null, 1, 0, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_rms_norm(one, L.BF16, 4, 256, 256, 1e-6, null, one, null, 0, 0, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_rms_norm(one, L.BF16, 4, 200, 200, 1e-6, null, null, null, 1, 0, 128, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_rms_norm(one, L.BF16, 4, 256, 128, 1e-6, null, null, null, 1, 0, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_rms_norm(null, L.BF16, 0, 256, 256, 1e-6, null, null, null, 1, 0, 0, null, null, null) == 0
    assert lib.i8f_quant_rowwise_prologue(one, L.BF16, 4, 256, 256, 9, null, null, 1, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_prologue(one, L.BF16, 4, 256, 256, 8, null, null, 1, 0, one, one, null) == INVALID   # fused modulation without vectors
    grp = (L._SmallMGroup * 2)()
    assert lib.i8f_linear_w8a16_small_m_grouped(grp, 0, L.BF16, 1, 0, null) == 0
    assert lib.i8f_linear_w8a16_small_m_grouped(null, 2, L.BF16, 1, 0, null) == INVALID
    assert lib.i8f_linear_w8a16_small_m_grouped(grp, 2, 9, 1, 0, null) == INVALID
    grp[0].M, grp[0].N, grp[0].K, grp[0].ldx = 17, 16, 16, 16
    assert lib.i8f_linear_w8a16_small_m_grouped(grp, 2, L.BF16, 1, 0, null) == UNSUPPORTED
    grp[0].M = 4
    assert lib.i8f_linear_w8a16_small_m_grouped(grp, 2, L.BF16, 1, 0, null) == INVALID   # no pointers
    assert lib.i8f_quant_rowwise_prologue(one, L.BF16, 4, 256, 256, L.PRO_NORM_MODULATE, one, one, 4, 0, one, one, null) == INVALID  # needs its own entry point: it carries eps
    # concatenating quantiser: negative widths, operands missing, a rotation block that would straddle the seam, binary32,
    # widths that are not whole runs of 16, more than 16384 columns
    assert lib.i8f_quant_rowwise_concat_gelu(one, L.BF16, 4, -16, 16, one, 16, 16, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_concat_gelu(one, L.BF16, 4, 16, 16, null, 16, 16, 0, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_concat_gelu(one, L.BF16, 4, 64, 64, one, 128, 128, 128, one, one, null) == INVALID
    assert lib.i8f_quant_rowwise_concat_gelu(one, L.F32, 4, 16, 16, one, 16, 16, 0, one, one, null) == UNSUPPORTED
    assert lib.i8f_quant_rowwise_concat_gelu(one, L.BF16, 4, 24, 24, one, 16, 16, 0, one, one, null) == UNSUPPORTED
    assert lib.i8f_quant_rowwise_concat_gelu(one, L.BF16, 4, 8192, 8192, one, 8208, 8208, 0, one, one, null) == UNSUPPORTED
    assert lib.i8f_quant_rowwise_concat_gelu(null, L.BF16, 0, 16, 16, null, 16, 16, 0, null, null, null) == 0
    # gated residual: a gate needs a positive row count per vector
    assert lib.i8f_linear_w8a8_gated(one, one, one, one, 1.0, 1, null, 0, one, 0, one, one, L.BF16, 4, 8, 16, 0, null, 0, null) == INVALID
    assert lib.i8f_linear_w8a8_gated(one, one, one, one, 1.0, 1, null, 0, one, 4, one, null, L.BF16, 4, 8, 16, 0, null, 0, null) == INVALID
    assert lib.i8f_linear_w8a8_gated(null, null, null, null, 1.0, 1, null, 0, null, 1, null, null, L.BF16, 0, 8, 16, 0, null, 0, null) == 0
    # grouped linear: no groups, a bad mode or dtype, too many groups, a group without output or without scales
    lg = (L._LinearGroup * 5)()
    for g in lg:
        g.a = g.a_scale = g.w = g.w_scale = g.out = one.value
        g.M = 4
    assert lib.i8f_linear_w8a8_grouped(null, 0, 1, L.BF16, L.BF16, 8, 16, 0, null, 0, null) == 0
    assert lib.i8f_linear_w8a8_grouped(null, 2, 1, L.BF16, L.BF16, 8, 16, 0, null, 0, null) == INVALID
    assert lib.i8f_linear_w8a8_grouped(ctypes.byref(lg), 2, 5, L.BF16, L.BF16, 8, 16, 0, null, 0, null) == INVALID
    assert lib.i8f_linear_w8a8_grouped(ctypes.byref(lg), 2, 1, L.BF16, 9, 8, 16, 0, null, 0, null) == INVALID
    assert lib.i8f_linear_w8a8_grouped(ctypes.byref(lg), 2, 1, L.BF16, L.BF16, 8, 16, 7, null, 0, null) == INVALID
    assert lib.i8f_linear_w8a8_grouped(ctypes.byref(lg), 2, 1, L.BF16, L.BF16, 8, 16, 0, one, 64, null) == INVALID      # workspace too small
    assert lib.i8f_linear_w8a8_grouped(ctypes.byref(lg), 5, 1, L.BF16, L.BF16, 8, 16, 0, null, 0, null) == UNSUPPORTED
    lg[1].gate, lg[1].rows_per_gate = one.value, 0       # a gate without a row count
    assert lib.i8f_linear_w8a8_grouped(ctypes.byref(lg), 2, 1, L.BF16, L.BF16, 8, 16, 0, null, 0, null) == INVALID
    lg[1].gate = None
    lg[1].out = None
    assert lib.i8f_linear_w8a8_grouped(ctypes.byref(lg), 2, 1, L.BF16, L.BF16, 8, 16, 0, null, 0, null) == INVALID
    lg[1].out, lg[1].w_scale = one.value, None
    assert lib.i8f_linear_w8a8_grouped(ctypes.byref(lg), 2, 1, L.BF16, L.BF16, 8, 16, 0, null, 0, null) == INVALID
    lg[1].M = 0   # an empty group is skipped, whatever its pointers
    lg[0].M = 0
    assert lib.i8f_linear_w8a8_grouped(ctypes.byref(lg), 2, 1, L.BF16, L.BF16, 8, 16, 0, null, 0, null) == 0
    assert lib.i8f_linear_w8a8(one, null, one, one, 1.0, 0, null, 0, one, L.BF16, 4, 4, 4, 0, null) == INVALID            # activation scales missing
    assert lib.i8f_linear_w8a8_add(one, one, one, one, 1.0, 0, null, 0, one, null, L.BF16, 4, 4, 4, 0, null) == INVALID   # no output
    assert lib.i8f_linear_w8a8_add(one, one, one, one, 1.0, 0, null, 0, one, one, 9, 4, 4, 4, 0, null) == INVALID         # bad output dtype
    assert lib.i8f_linear_w8a16_small_m(one, L.BF16, 17, 8, 8, one, one, 1.0, 0, null, 0, one, 4, null) == UNSUPPORTED    # M > 16
    assert lib.i8f_sr_quant_delta(null, one, 1.0, 0, one, 4, 4, one, null) == INVALID
    assert lib.i8f_lora_merge_sr(one, one, 1.0, 0, null, null, null, 8, 1.0, one, 4, 4, one, null) == INVALID             # neither delta nor factors
    assert lib.i8f_lora_merge_sr(one, one, 1.0, 0, null, one, one, 300, 1.0, one, 4, 4, one, null) == UNSUPPORTED         # rank > 256


def test_missing_library_is_a_loud_error(pkg, monkeypatch, tmp_path):
    monkeypatch.setattr(pkg._lib, "_lib", None)
    monkeypatch.setattr(pkg._lib, "LIB_PATH", str(tmp_path / "libi8f_gfx950.so"))
    with pytest.raises(RuntimeError, match="is missing"):
        pkg._lib.lib()


def test_cpu_tensors_are_refused_not_emulated(pkg):
    import torch

    x = torch.randn(32, 128).bfloat16()
    w = torch.zeros(16, 128, dtype=torch.int8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        pkg.hip_quantize_rowwise(x)
    with pytest.raises(RuntimeError, match="no CPU path"):
        pkg.int8_forward_dynamic(x, w, 0.01, None, torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        pkg._lib.gemm_i32(w, w)


def test_product_code_never_imports_the_oracle():
    pkg_dir = os.path.join(ROOT, "comfyui-int8-fast_amd")
    for dirpath, _, files in os.walk(pkg_dir):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"
                assert "_int_mm(" not in text, f"{f} calls torch._int_mm"


def test_gemm_tile_reports_the_configuration_of_the_benchmark_shapes(L):
    """Host-only: the tile choice is a function of the shape."""
    assert L.gemm_tile(4608, 3072, 3072) == (256, 256, 2)
    assert L.gemm_tile(4608, 12288, 3072) == (288, 256, 2)
    assert L.gemm_tile(4608, 3072, 12288) == (256, 256, 2)
    assert L.gemm_tile(512, 12288, 3072) == (256, 96, 3)
    assert L.gemm_tile(33, 64, 77) == (1, 1, 0)           # K % 16 != 0: the generic kernel
    assert L.lib().i8f_gemm_tile(0, 8, 16, None, None, None) == -1
