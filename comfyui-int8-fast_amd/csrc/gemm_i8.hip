// Entry points of the int8 GEMM (include/i8f.h) and the instantiations for bfloat16 outputs; the other
// output types are instantiated in gemm_i8_f16.hip and gemm_i8_wide.hip.
#include "gemm_i8_impl.hpp"

namespace i8f {
namespace gemm {
template int launch<OUT_BF16>(GemmArgs &, hipStream_t);
template int launch_group<OUT_BF16>(GemmArgs *, int, hipStream_t);
extern template int launch_group<OUT_F16>(GemmArgs *, int, hipStream_t);
extern template int launch_group<OUT_F32>(GemmArgs *, int, hipStream_t);
extern template int launch<OUT_F16>(GemmArgs &, hipStream_t);
extern template int launch<OUT_F32>(GemmArgs &, hipStream_t);
extern template int launch<OUT_I32>(GemmArgs &, hipStream_t);
}  // namespace gemm
}  // namespace i8f

extern "C" int i8f_gemm_i32(const int8_t *a, const int8_t *w, int64_t M, int64_t N, int64_t K, int32_t *acc,
                            void *stream) {
    using namespace i8f;
    using namespace i8f::gemm;
    if (int rc = validate(a, w, M, N, K, acc)) return rc;
    if (M == 0 || N == 0) return I8F_OK;
    if (int rc = check_device()) return rc;
    GemmArgs g{};
    g.x = a, g.w = w, g.M = (int)M, g.N = (int)N, g.K = (int)K, g.out = acc;
    return launch<OUT_I32>(g, (hipStream_t)stream);
}

extern "C" int64_t i8f_linear_w8a8_workspace_bytes(void) { return i8f::gemm::SPLITK_WORKSPACE_BYTES; }

extern "C" int i8f_linear_w8a8_add(const int8_t *a, const float *a_scale, const int8_t *w, const float *w_scale,
                                   float w_scale_host, int scale_mode, const void *bias, int bias_dtype,
                                   const void *addend, void *out, int out_dtype, int64_t M, int64_t N, int64_t K,
                                   int order, void *stream) {
    return i8f_linear_w8a8_splitk(a, a_scale, w, w_scale, w_scale_host, scale_mode, bias, bias_dtype, addend, out, out_dtype, M, N,
                                  K, order, nullptr, 0, stream);
}

extern "C" int i8f_linear_w8a8_splitk(const int8_t *a, const float *a_scale, const int8_t *w, const float *w_scale,
                                      float w_scale_host, int scale_mode, const void *bias, int bias_dtype,
                                      const void *addend, void *out, int out_dtype, int64_t M, int64_t N, int64_t K,
                                      int order, void *workspace, int64_t workspace_bytes, void *stream) {
    return i8f_linear_w8a8_gated(a, a_scale, w, w_scale, w_scale_host, scale_mode, bias, bias_dtype, nullptr, 1, addend, out, out_dtype,
                                 M, N, K, order, workspace, workspace_bytes, stream);
}

extern "C" int i8f_linear_w8a8_gated(const int8_t *a, const float *a_scale, const int8_t *w, const float *w_scale,
                                     float w_scale_host, int scale_mode, const void *bias, int bias_dtype, const void *gate,
                                     int64_t rows_per_gate, const void *residual, void *out, int out_dtype, int64_t M, int64_t N,
                                     int64_t K, int order, void *workspace, int64_t workspace_bytes, void *stream) {
    using namespace i8f;
    using namespace i8f::gemm;
    const void *addend = residual;
    if (gate && rows_per_gate <= 0) return I8F_ERR_INVALID;
    if (workspace && (workspace_bytes < SPLITK_WORKSPACE_BYTES || (uintptr_t)workspace % 16)) return I8F_ERR_INVALID;
    if (int rc = validate(a, w, M, N, K, out)) return rc;
    if (!valid_dtype(out_dtype) || (bias && !valid_dtype(bias_dtype))) return I8F_ERR_INVALID;
    if (scale_mode != I8F_SCALE_TENSOR && scale_mode != I8F_SCALE_ROW) return I8F_ERR_INVALID;
    if (order != I8F_EPI_TORCH && order != I8F_EPI_FUSED) return I8F_ERR_INVALID;
    if (M == 0 || N == 0) return I8F_OK;
    if (!a_scale) return I8F_ERR_INVALID;
    if (scale_mode == I8F_SCALE_ROW && !w_scale) return I8F_ERR_INVALID;
    if (int rc = check_device()) return rc;
    GemmArgs g{};
    g.x = a, g.w = w, g.M = (int)M, g.N = (int)N, g.K = (int)K, g.out = out;
    g.xs = a_scale, g.ws = w_scale, g.ws_host = w_scale_host, g.row_scale = scale_mode == I8F_SCALE_ROW;
    g.bias = bias, g.bias_dtype = bias_dtype, g.order = order, g.addend = addend;
    g.gate = gate, g.gate_rows = (int)(rows_per_gate < 0x7fffffff ? rows_per_gate : 0x7fffffff);  // (M itself is below 2^31)
    if (workspace) g.arrivals = (unsigned *)workspace, g.partials = (int *)((char *)workspace + SPLITK_COUNTER_BYTES);
    hipStream_t st = (hipStream_t)stream;
    switch (out_dtype) {
    case I8F_BF16: return launch<OUT_BF16>(g, st);
    case I8F_F16: return launch<OUT_F16>(g, st);
    default: return launch<OUT_F32>(g, st);
    }
}

extern "C" int i8f_linear_w8a8_lora(const int8_t *a, const float *a_scale, const int8_t *w, const float *w_scale,
                                    float w_scale_host, int scale_mode, const void *bias, int bias_dtype,
                                    const void *side_t, const void *side_b, int64_t rank, int has_alpha, float alpha,
                                    void *out, int out_dtype, int64_t M, int64_t N, int64_t K, int order, void *stream) {
    using namespace i8f;
    using namespace i8f::gemm;
    if (int rc = validate(a, w, M, N, K, out)) return rc;
    if (!valid_dtype(out_dtype) || (bias && !valid_dtype(bias_dtype))) return I8F_ERR_INVALID;
    if (scale_mode != I8F_SCALE_TENSOR && scale_mode != I8F_SCALE_ROW) return I8F_ERR_INVALID;
    if (order != I8F_EPI_TORCH && order != I8F_EPI_FUSED) return I8F_ERR_INVALID;
    if (rank <= 0 || !side_t || !side_b) return I8F_ERR_INVALID;
    if (M == 0 || N == 0) return I8F_OK;
    if (!a_scale) return I8F_ERR_INVALID;
    if (scale_mode == I8F_SCALE_ROW && !w_scale) return I8F_ERR_INVALID;
    // the matrix-core side product: 16-bit operands of the output dtype, rank a multiple of 16 up to 64
    if (out_dtype == I8F_F32 || rank % 16 || rank > 64 || K == 0) return I8F_ERR_UNSUPPORTED;
    if (int rc = check_device()) return rc;
    GemmArgs g{};
    g.x = a, g.w = w, g.M = (int)M, g.N = (int)N, g.K = (int)K, g.out = out;
    g.xs = a_scale, g.ws = w_scale, g.ws_host = w_scale_host, g.row_scale = scale_mode == I8F_SCALE_ROW;
    g.bias = bias, g.bias_dtype = bias_dtype, g.order = order, g.addend = nullptr;
    g.side_t = side_t, g.side_b = side_b, g.side_rank = (int)rank, g.side_has_alpha = has_alpha != 0, g.side_alpha = alpha;
    hipStream_t st = (hipStream_t)stream;
    return out_dtype == I8F_BF16 ? launch<OUT_BF16>(g, st) : launch<OUT_F16>(g, st);
}

extern "C" int i8f_linear_w8a8(const int8_t *a, const float *a_scale, const int8_t *w, const float *w_scale,
                               float w_scale_host, int scale_mode, const void *bias, int bias_dtype, void *out,
                               int out_dtype, int64_t M, int64_t N, int64_t K, int order, void *stream) {
    return i8f_linear_w8a8_add(a, a_scale, w, w_scale, w_scale_host, scale_mode, bias, bias_dtype, nullptr, out,
                               out_dtype, M, N, K, order, stream);
}

extern "C" int i8f_linear_w8a8_grouped(const i8f_linear_group *groups, int n_groups, int scale_mode, int bias_dtype, int out_dtype,
                                       int64_t N, int64_t K, int order, void *workspace, int64_t workspace_bytes, void *stream) {
    using namespace i8f;
    using namespace i8f::gemm;
    if (n_groups < 0 || (n_groups > 0 && !groups) || N < 0 || K < 0) return I8F_ERR_INVALID;
    if (workspace && (workspace_bytes < SPLITK_WORKSPACE_BYTES || (uintptr_t)workspace % 16)) return I8F_ERR_INVALID;
    if (!valid_dtype(out_dtype) || !valid_dtype(bias_dtype)) return I8F_ERR_INVALID;
    if (scale_mode != I8F_SCALE_TENSOR && scale_mode != I8F_SCALE_ROW) return I8F_ERR_INVALID;
    if (order != I8F_EPI_TORCH && order != I8F_EPI_FUSED) return I8F_ERR_INVALID;
    if (n_groups > I8F_MAX_LINEAR_GROUPS) return I8F_ERR_UNSUPPORTED;
    GemmArgs gs[I8F_MAX_LINEAR_GROUPS];
    int n = 0;
    for (int i = 0; i < n_groups; ++i) {
        const i8f_linear_group &p = groups[i];
        if (int rc = validate(p.a, p.w, p.M, N, K, p.out)) return rc;
        if (p.M == 0 || N == 0) continue;
        if (!p.a_scale || (scale_mode == I8F_SCALE_ROW && !p.w_scale)) return I8F_ERR_INVALID;
        GemmArgs g{};
        g.x = p.a, g.w = p.w, g.M = (int)p.M, g.N = (int)N, g.K = (int)K, g.out = p.out;
        g.xs = p.a_scale, g.ws = p.w_scale, g.ws_host = p.w_scale_host, g.row_scale = scale_mode == I8F_SCALE_ROW;
        g.bias = p.bias, g.bias_dtype = bias_dtype, g.order = order, g.addend = p.addend;
        if (p.gate && p.rows_per_gate <= 0) return I8F_ERR_INVALID;
        g.gate = p.gate, g.gate_rows = (int)(p.rows_per_gate < 0x7fffffff ? p.rows_per_gate : 0x7fffffff);
        if (workspace) g.arrivals = (unsigned *)workspace, g.partials = (int *)((char *)workspace + SPLITK_COUNTER_BYTES);
        gs[n++] = g;
    }
    if (n == 0) return I8F_OK;
    if (int rc = check_device()) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (out_dtype) {
    case I8F_BF16: return launch_group<OUT_BF16>(gs, n, st);
    case I8F_F16: return launch_group<OUT_F16>(gs, n, st);
    default: return launch_group<OUT_F32>(gs, n, st);
    }
}

extern "C" int i8f_gemm_tile(int64_t M, int64_t N, int64_t K, int *bm, int *bn, int *stages) {
    using namespace i8f;
    using namespace i8f::gemm;
    if (M <= 0 || N <= 0 || K < 0 || !bm || !bn || !stages) return I8F_ERR_INVALID;
    if (K % 16 || N % 8 || N * K >= (1ll << 31)) {  // such shapes take the one-thread-per-output kernel
        *bm = *bn = 1, *stages = 0;
        return I8F_OK;
    }
    if (M * K >= (1ll << 31)) M = (((1ll << 31) - 1) / K) / 256 * 256;  // launched in row blocks of this size
    switch (choose_tile(M, N)) {
    case TILE_BIG: tile_dims<CfgBig>(bm, bn, stages); break;
    case TILE_B192: tile_dims<CfgB192>(bm, bn, stages); break;
    case TILE_MID: tile_dims<CfgMid>(bm, bn, stages); break;
    case TILE_TALL: tile_dims<CfgTall>(bm, bn, stages); break;
    case TILE_WIDE: tile_dims<CfgWide>(bm, bn, stages); break;
    case TILE_W96: tile_dims<CfgW96>(bm, bn, stages); break;
    case TILE_MID_DEEP: tile_dims<CfgMidDeep>(bm, bn, stages); break;
    case TILE_M96_DEEP: tile_dims<CfgM96Deep>(bm, bn, stages); break;
    case TILE_S64_DEEP: tile_dims<CfgS64Deep>(bm, bn, stages); break;
    default: tile_dims<CfgT64Deep>(bm, bn, stages); break;
    }
    return I8F_OK;
}
