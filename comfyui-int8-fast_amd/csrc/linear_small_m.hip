// Small-batch (M <= 16) W8A16 linear: bandwidth-bound stream over the int8
// weight, dequantised in registers; the activations are not quantised.
//
//   out[m,n] = round( sum_k x[m,k] * round(float(w[n,k]) * ws[n]) + round(bias[n]) )
//
// with round() = rounding to x's dtype, which is where the reference rounds
// (Linear.forward, int8_quant.py:756-760: the dequantised weight and the bias
// are cast to x.dtype before F.linear).  The reference writes the whole
// dequantised weight to memory and reads it back on every call; here the weight
// is read once as int8.  One wavefront owns one output column n: 64 lanes x 16
// weights per step, partial sums as fmaf chains in binary32, then a butterfly
// reduction across the wavefront.
#include "i8f_common.hpp"

namespace i8f {
namespace {

struct SmallMArgs {
    const void *x;
    int64_t M, K, ldx, N;
    const int8_t *w;
    const float *ws;
    float ws_host;
    int row_scale;
    const void *bias;
    int bias_dtype;
    void *out;
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

template <int DT>
__device__ __forceinline__ void load16(const void *x, int64_t idx, float (&xf)[16]) {
    if constexpr (DT == I8F_F32) {
        const float4 *p = (const float4 *)((const float *)x + idx);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float4 t = p[j];
            xf[4 * j] = t.x, xf[4 * j + 1] = t.y, xf[4 * j + 2] = t.z, xf[4 * j + 3] = t.w;
        }
    } else {
        const uint4 *p = (const uint4 *)((const uint16_t *)x + idx);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint4 t = p[j];
            const uint32_t u[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if constexpr (DT == I8F_BF16) {
                    xf[8 * j + 2 * e] = bf16_bits_to_f32(u[e] & 0xffffu);
                    xf[8 * j + 2 * e + 1] = bf16_bits_to_f32(u[e] >> 16);
                } else {
                    xf[8 * j + 2 * e] = f16_bits_to_f32(u[e] & 0xffffu);
                    xf[8 * j + 2 * e + 1] = f16_bits_to_f32(u[e] >> 16);
                }
            }
        }
    }
}

template <int DT, bool VEC>
__global__ __launch_bounds__(256) void small_m_kernel(const SmallMArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t n = (int64_t)blockIdx.x * 4 + wave;
    if (n >= a.N) return;
    const float wsn = a.ws ? a.ws[a.row_scale ? n : 0] : a.ws_host;
    const int8_t *wr = a.w + n * a.K;
    const int M = (int)a.M;

    float acc[16];
#pragma unroll
    for (int m = 0; m < 16; ++m) acc[m] = 0.0f;

    if constexpr (VEC) {
        for (int64_t k0 = (int64_t)lane * 16; k0 < a.K; k0 += 1024) {
            const uint4 wq = *(const uint4 *)(wr + k0);
            const uint32_t u[4] = {wq.x, wq.y, wq.z, wq.w};
            float wf[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int b = (int)(int8_t)(u[e >> 2] >> (8 * (e & 3)));
                wf[e] = round_to_dtype<DT>((float)b * wsn);
            }
#pragma unroll
            for (int m = 0; m < 16; ++m) {
                if (m < M) {
                    float xf[16];
                    load16<DT>(a.x, (int64_t)m * a.ldx + k0, xf);
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[m] = fmaf(xf[e], wf[e], acc[m]);
                }
            }
        }
    } else {
        for (int64_t k = lane; k < a.K; k += 64) {
            const float wf = round_to_dtype<DT>((float)wr[k] * wsn);
#pragma unroll
            for (int m = 0; m < 16; ++m)
                if (m < M) acc[m] = fmaf(load_as_f32<DT>(a.x, (int64_t)m * a.ldx + k), wf, acc[m]);
        }
    }

    float b = 0.0f;
    if (a.bias) {
        if (a.bias_dtype == I8F_F32) b = ((const float *)a.bias)[n];
        else if (a.bias_dtype == I8F_BF16) b = bf16_bits_to_f32(((const uint16_t *)a.bias)[n]);
        else b = f16_bits_to_f32(((const uint16_t *)a.bias)[n]);
        b = round_to_dtype<DT>(b);
    }
#pragma unroll
    for (int m = 0; m < 16; ++m) {
        if (m < M) {
            const float s = wave_sum(acc[m]);
            if (lane == 0) store_from_f32<DT>(a.out, (int64_t)m * a.N + n, s + b);
        }
    }
}

template <int DT>
int launch(const SmallMArgs &a, hipStream_t st) {
    const size_t es = dtype_size(DT);
    const bool vec = a.K % 16 == 0 && (uintptr_t)a.w % 16 == 0 && (uintptr_t)a.x % 16 == 0 && (a.ldx * es) % 16 == 0;
    dim3 grid((unsigned)((a.N + 3) / 4));
    if (vec) hipLaunchKernelGGL((small_m_kernel<DT, true>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((small_m_kernel<DT, false>), grid, dim3(256), 0, st, a);
    return check_launch();
}

}  // namespace
}  // namespace i8f

extern "C" int i8f_linear_w8a16_small_m(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                        const int8_t *w, const float *w_scale, float w_scale_host, int scale_mode,
                                        const void *bias, int bias_dtype, void *out, int64_t N, void *stream) {
    using namespace i8f;
    if (M < 0 || N < 0 || K < 0 || !valid_dtype(x_dtype) || (bias && !valid_dtype(bias_dtype))) return I8F_ERR_INVALID;
    if (scale_mode != I8F_SCALE_TENSOR && scale_mode != I8F_SCALE_ROW) return I8F_ERR_INVALID;
    if (M > 16) return I8F_ERR_UNSUPPORTED;
    if (M == 0 || N == 0) return I8F_OK;
    if (!out || ldx < K) return I8F_ERR_INVALID;
    if (K > 0 && (!x || !w)) return I8F_ERR_INVALID;
    if (scale_mode == I8F_SCALE_ROW && !w_scale) return I8F_ERR_INVALID;
    if (N > 0x7fffffffll * 4) return I8F_ERR_UNSUPPORTED;
    if (int rc = check_device()) return rc;
    SmallMArgs a{};
    a.x = x, a.M = M, a.K = K, a.ldx = ldx, a.N = N, a.w = w, a.ws = w_scale, a.ws_host = w_scale_host;
    a.row_scale = scale_mode == I8F_SCALE_ROW, a.bias = bias, a.bias_dtype = bias_dtype, a.out = out;
    hipStream_t st = (hipStream_t)stream;
    switch (x_dtype) {
    case I8F_BF16: return launch<I8F_BF16>(a, st);
    case I8F_F16: return launch<I8F_F16>(a, st);
    default: return launch<I8F_F32>(a, st);
    }
}
