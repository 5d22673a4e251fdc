// One absmax scale for a whole tensor, then int8 quantisation: quantize_int8_tensorwise
// (int8_quant.py:23-26 of the reference) as two launches that use every CU.
//
//   pass 1  absmax_partial_kernel   each workgroup takes a contiguous slice of the tensor and writes
//                                   the largest |x| of its slice to partial[blockIdx.x]
//   pass 2  quant_tensor_kernel     every workgroup reduces the (at most 1024) partial maxima itself,
//                                   derives scale and reciprocal exactly as the row quantiser does, and
//                                   quantises its slice; workgroup 0 writes the scale
//
// The partial maxima are the only device memory beyond inputs and outputs.  They live either in a
// workspace of the caller (i8f_quant_tensorwise) or in a file-scope device array of this library
// (i8f_quant_tensorwise_static, for callers that cannot allocate).  Nothing has to be cleared between
// calls: pass 1 writes every slot that pass 2 of the same call reads.
#include <mutex>

#include "i8f_common.hpp"

namespace i8f {
namespace {

constexpr int MAX_PARTIALS = 1024;               // slots of the partial-maximum buffer
constexpr int TPB = 256;                         // threads per workgroup
constexpr int64_t SLICE_MIN = 16 * 1024;         // elements: below this a slice is not worth a workgroup
constexpr int64_t STATIC_MAX_ELEMS = 1ll << 32;  // limit of the allocation-free entry point

// The allocation-free entry point's scratch.  In host code this name is only a handle: the device
// address comes from hipGetSymbolAddress, once per device (each GPU holds its own copy).
static __device__ __align__(256) float scratch[MAX_PARTIALS];

template <int DT>
struct Vec {
    static constexpr int EPC = DT == I8F_F32 ? 4 : 8;  // elements per 16-byte chunk
};

template <int DT>
__device__ __forceinline__ void load_chunk(const char *p, float (&v)[Vec<DT>::EPC]) {
    const uint4 r = *(const uint4 *)p;
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
    if constexpr (DT == I8F_F32) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = __uint_as_float(w[j]);
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (DT == I8F_BF16) {
                v[2 * j] = bf16_bits_to_f32(w[j] & 0xffffu);
                v[2 * j + 1] = bf16_bits_to_f32(w[j] >> 16);
            } else {
                v[2 * j] = f16_bits_to_f32(w[j] & 0xffffu);
                v[2 * j + 1] = f16_bits_to_f32(w[j] >> 16);
            }
        }
    }
}

__device__ __forceinline__ float block_max(float v, float *red) {
    v = wave_max(v);
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    if (lane == 0) red[wv] = v;
    __syncthreads();
    v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    return v;
}

// slice [lo, hi) of workgroup b: whole 16-byte chunks, the last workgroup takes the tail
__device__ __forceinline__ void slice_of(int64_t n, int64_t per, int b, int64_t &lo, int64_t &hi) {
    lo = (int64_t)b * per;
    hi = lo + per < n ? lo + per : n;
    if (lo > n) lo = n;
}

template <int DT, bool ALIGNED>
__global__ __launch_bounds__(TPB) void absmax_partial_kernel(const void *__restrict__ x, int64_t n, int64_t per,
                                                              float *__restrict__ partial) {
    constexpr int EPC = Vec<DT>::EPC;
    __shared__ float red[4];
    int64_t lo, hi;
    slice_of(n, per, blockIdx.x, lo, hi);
    float amax = 0.0f;
    if constexpr (ALIGNED) {
        const int64_t c_hi = lo + (hi - lo) / EPC * EPC;  // `per` is a multiple of EPC, so lo is chunk-aligned
        for (int64_t i = lo + (int64_t)threadIdx.x * EPC; i < c_hi; i += (int64_t)TPB * EPC) {
            float v[EPC];
            load_chunk<DT>((const char *)x + i * (DT == I8F_F32 ? 4 : 2), v);
#pragma unroll
            for (int j = 0; j < EPC; ++j) amax = fmaxf(amax, fabsf(v[j]));
        }
        for (int64_t i = c_hi + threadIdx.x; i < hi; i += TPB) amax = fmaxf(amax, fabsf(load_as_f32<DT>(x, i)));
    } else {
        for (int64_t i = lo + threadIdx.x; i < hi; i += TPB) amax = fmaxf(amax, fabsf(load_as_f32<DT>(x, i)));
    }
    amax = block_max(amax, red);
    if (threadIdx.x == 0) partial[blockIdx.x] = amax;
}

template <int DT, bool ALIGNED>
__global__ __launch_bounds__(TPB) void quant_tensor_kernel(const void *__restrict__ x, int64_t n, int64_t per,
                                                            const float *__restrict__ partial, int nparts,
                                                            int8_t *__restrict__ q, float *__restrict__ scale) {
    constexpr int EPC = Vec<DT>::EPC;
    __shared__ float red[4];
    float amax = 0.0f;
    for (int i = threadIdx.x; i < nparts; i += TPB) amax = fmaxf(amax, partial[i]);
    amax = block_max(amax, red);
    // the arithmetic of quantize_int8_tensorwise + quantize_int8 (int8_quant.py:20-26)
    float s = amax / 127.0f;
    s = s < 1e-30f ? 1e-30f : s;
    const float inv = 1.0f / s;
    if (blockIdx.x == 0 && threadIdx.x == 0) *scale = s;

    int64_t lo, hi;
    slice_of(n, per, blockIdx.x, lo, hi);
    if constexpr (ALIGNED) {
        const int64_t c_hi = lo + (hi - lo) / EPC * EPC;
        for (int64_t i = lo + (int64_t)threadIdx.x * EPC; i < c_hi; i += (int64_t)TPB * EPC) {
            float v[EPC];
            load_chunk<DT>((const char *)x + i * (DT == I8F_F32 ? 4 : 2), v);
            uint32_t w[EPC / 4];
#pragma unroll
            for (int j = 0; j < EPC / 4; ++j) {
                w[j] = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[j] |= (uint32_t)(quant_i8(v[4 * j + e] * inv) & 0xff) << (8 * e);
            }
            if constexpr (EPC == 8) stream_store8(q + i, make_uint2(w[0], w[1]));
            else stream_store4(q + i, w[0]);
        }
        for (int64_t i = c_hi + threadIdx.x; i < hi; i += TPB) q[i] = (int8_t)quant_i8(load_as_f32<DT>(x, i) * inv);
    } else {
        for (int64_t i = lo + threadIdx.x; i < hi; i += TPB) q[i] = (int8_t)quant_i8(load_as_f32<DT>(x, i) * inv);
    }
}

int parts_for(int64_t n) {
    int64_t p = (n + SLICE_MIN - 1) / SLICE_MIN;
    return (int)(p < 1 ? 1 : (p > MAX_PARTIALS ? MAX_PARTIALS : p));
}

template <int DT>
int run(const void *x, int64_t n, int8_t *q, float *scale, float *partial, hipStream_t st) {
    const int parts = parts_for(n);
    int64_t per = (n + parts - 1) / parts;
    per = (per + 15) / 16 * 16;  // slices start on 16-byte boundaries of x and 8-byte boundaries of q
    const bool aligned = (uintptr_t)x % 16 == 0 && (uintptr_t)q % 8 == 0;
    if (aligned) {
        hipLaunchKernelGGL((absmax_partial_kernel<DT, true>), dim3(parts), dim3(TPB), 0, st, x, n, per, partial);
        hipLaunchKernelGGL((quant_tensor_kernel<DT, true>), dim3(parts), dim3(TPB), 0, st, x, n, per, partial, parts, q, scale);
    } else {
        hipLaunchKernelGGL((absmax_partial_kernel<DT, false>), dim3(parts), dim3(TPB), 0, st, x, n, per, partial);
        hipLaunchKernelGGL((quant_tensor_kernel<DT, false>), dim3(parts), dim3(TPB), 0, st, x, n, per, partial, parts, q, scale);
    }
    return check_launch();
}

int dispatch(const void *x, int x_dtype, int64_t n, int8_t *q, float *scale, float *partial, hipStream_t st) {
    switch (x_dtype) {
    case I8F_BF16: return run<I8F_BF16>(x, n, q, scale, partial, st);
    case I8F_F16: return run<I8F_F16>(x, n, q, scale, partial, st);
    default: return run<I8F_F32>(x, n, q, scale, partial, st);
    }
}

int validate(const void *x, int x_dtype, int64_t n, const int8_t *q, const float *scale) {
    if (n < 0 || !valid_dtype(x_dtype) || !scale) return I8F_ERR_INVALID;
    if (n > 0 && (!x || !q)) return I8F_ERR_INVALID;
    return I8F_OK;
}

// device address of `scratch` on the current device, looked up once per device
int static_scratch(float **out) {
    static std::mutex mu;
    static float *ptr_of_device[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        last_hip_error_slot() = (int)e;
        return I8F_ERR_HIP;
    }
    if (dev < 0 || dev >= 64) return I8F_ERR_DEVICE;
    std::lock_guard<std::mutex> lock(mu);
    if (!ptr_of_device[dev]) {
        float *p = nullptr;
        e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            last_hip_error_slot() = (int)e;
            return I8F_ERR_HIP;
        }
        ptr_of_device[dev] = p;
    }
    *out = ptr_of_device[dev];
    return I8F_OK;
}

}  // namespace
}  // namespace i8f

extern "C" int64_t i8f_quant_tensorwise_workspace_bytes(int64_t n) {
    return n < 0 ? 0 : (int64_t)i8f::parts_for(n) * (int64_t)sizeof(float);
}

extern "C" int i8f_quant_tensorwise(const void *x, int x_dtype, int64_t n, int8_t *q, float *scale, void *workspace,
                                    int64_t workspace_bytes, void *stream) {
    using namespace i8f;
    if (int rc = validate(x, x_dtype, n, q, scale)) return rc;
    if (!workspace || workspace_bytes < i8f_quant_tensorwise_workspace_bytes(n) || (uintptr_t)workspace % 4) return I8F_ERR_INVALID;
    if (int rc = check_device()) return rc;
    return dispatch(x, x_dtype, n, q, scale, (float *)workspace, (hipStream_t)stream);
}

extern "C" int i8f_quant_tensorwise_static(const void *x, int x_dtype, int64_t n, int8_t *q, float *scale,
                                           void *stream) {
    using namespace i8f;
    if (int rc = validate(x, x_dtype, n, q, scale)) return rc;
    if (n > STATIC_MAX_ELEMS) return I8F_ERR_UNSUPPORTED;  // the library's own scratch is sized for tensors up to this
    if (int rc = check_device()) return rc;
    float *partial = nullptr;
    if (int rc = static_scratch(&partial)) return rc;
    return dispatch(x, x_dtype, n, q, scale, partial, (hipStream_t)stream);
}
