// Shared device helpers of the gfx950 INT8 linear engine.
//
// All floating-point code in this library is compiled with -ffp-contract=off:
// a multiply followed by an add is two rounded operations unless the source
// says fmaf().  The bit-exact contracts of the quantiser, the epilogue and the
// LoRA merge depend on it.
#pragma once

// The numerical contract and some hand-scheduled assembly depend on how these sources are compiled, so a build with
// other flags must fail instead of producing a library that is subtly wrong: the build script passes
// -DI8F_BUILD_CONTRACT=1 together with -ffp-contract=off, -fno-fast-math, -fhip-fp32-correctly-rounded-divide-sqrt and
// the packed-FP32 feature switched off (the flags a macro cannot see); fast-math and finite-math are seen here.
#if !defined(I8F_BUILD_CONTRACT) || I8F_BUILD_CONTRACT != 1
#error "compile these sources with the flags of comfyui-int8-fast_amd/build.py (FLAGS): the results depend on them"
#endif
#if defined(__FAST_MATH__) || defined(__FINITE_MATH_ONLY__) && __FINITE_MATH_ONLY__
#error "fast-math changes the rounding of the quantiser, the epilogue and the merge: build without it"
#endif
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "this library is written for gfx950 only"
#endif

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/i8f.h"

namespace i8f {

// thread-local record of the last HIP error, read by i8f_last_hip_error()
int &last_hip_error_slot();

inline int check_launch() {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        last_hip_error_slot() = (int)e;
        return I8F_ERR_HIP;
    }
    return I8F_OK;
}

// I8F_OK if the current device is a gfx950, I8F_ERR_DEVICE otherwise (cached per device).
int check_device();

struct bf16_t {
    uint16_t bits;
};
struct f16_t {
    uint16_t bits;
};

// ---- widen -----------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}

// ---- round to nearest even ---------------------------------------------------
// bfloat16: the hardware conversion of gfx950 (v_cvt_pk_bf16_f32) rounds to
// nearest even and quiets NaNs, the same as torch's float -> bfloat16 cast.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float v) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)v);
}
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    f2 in = {lo, hi};
    bf2 o = __builtin_convertvector(in, bf2);
    return __builtin_bit_cast(uint32_t, o);
}
// The empty asm keeps the value opaque on its way into the conversion: without it the compiler
// folds a preceding binary32 multiply into v_fma_mixlo_f16, which rounds the exact product once
// to binary16 instead of first to binary32 and then to binary16, and the results differ on ties.
__device__ __forceinline__ uint32_t f32_to_f16_bits(float v) {
    asm("" : "+v"(v));
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)v);
}
__device__ __forceinline__ uint32_t f32x2_to_f16x2_bits(float lo, float hi) {
    return f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16);
}

// value rounded to the storage dtype and widened again
template <int DT>
__device__ __forceinline__ float round_to_dtype(float v) {
    // bfloat16: the packed conversion with a zero in the low half leaves the rounded value in the high half, which IS
    // its binary32 form: one instruction rounds and widens
    if constexpr (DT == I8F_BF16) return __uint_as_float(f32x2_to_bf16x2_bits(0.0f, v));
    else if constexpr (DT == I8F_F16) return f16_bits_to_f32(f32_to_f16_bits(v));
    else return v;
}

template <int DT>
__device__ __forceinline__ float load_as_f32(const void *p, int64_t i) {
    if constexpr (DT == I8F_BF16) return bf16_bits_to_f32(((const uint16_t *)p)[i]);
    else if constexpr (DT == I8F_F16) return f16_bits_to_f32(((const uint16_t *)p)[i]);
    else return ((const float *)p)[i];
}

template <int DT>
__device__ __forceinline__ void store_from_f32(void *p, int64_t i, float v) {
    if constexpr (DT == I8F_BF16) ((uint16_t *)p)[i] = (uint16_t)f32_to_bf16_bits(v);
    else if constexpr (DT == I8F_F16) ((uint16_t *)p)[i] = (uint16_t)f32_to_f16_bits(v);
    else ((float *)p)[i] = v;
}

// The entry of the normalised 128-point Hadamard matrix in each dtype:
// 1/sqrt(128) rounded to that dtype (0x3DB504F3 in binary32; 181/2048 in
// bfloat16 and binary16), as quarot.py:35-36 of the reference builds it.
template <int DT>
__device__ __forceinline__ float hadamard_entry() {
    if constexpr (DT == I8F_F32) return __uint_as_float(0x3DB504F3u);
    else return 0.08837890625f;
}

// round-to-nearest-even float -> int8 with saturation
__device__ __forceinline__ int quant_i8(float v) {
    float r = __builtin_rintf(v);
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return (int)r;
}

// Maximum over the 64 lanes of a wave, returned to every lane.  Lane exchanges are DPP operands of
// the max instructions (no LDS round trips: the butterfly through ds_bpermute costs six dependent
// LDS latencies): quads, half rows and rows of 16 first, then row 0 -> 1, 2 -> 3 and rows 0..1 -> 2..3
// by the row broadcasts, which leaves the result in lane 63.  One v_max_f32 with a DPP operand per
// step, from assembly (through the builtins the compiler makes a copy, a DPP move and a maximum of
// it).  A DPP read of a register needs two wait states after the vector write of it: the s_nop.  In
// the last two steps the rows that receive nothing are masked out of the write and keep their value.
__device__ __forceinline__ float wave_max(float v) {
    asm volatile("s_nop 1\n\tv_max_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
                 "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
                 "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
                 "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"   // every lane of a row of 16 holds the row's maximum
                 "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"  // into rows 1 and 3
                 "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"  // into rows 2 and 3
                 "s_nop 1"
                 : "+v"(v));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// ---- streaming stores and loads ------------------------------------------------------
// Results are written with non-temporal stores: they go out while the kernel runs instead of
// sitting dirty in the 8 per-XCD L2s until the write-back at the end of the kernel, which the next
// kernel on the stream has to wait for (a quarter of the time of a 10-microsecond kernel).  Nothing
// is lost: L2 is invalidated between kernels anyway, so the consumer never finds them there.
typedef unsigned v4u_t __attribute__((ext_vector_type(4)));
typedef unsigned v2u_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void stream_store16(void *p, uint4 v) {
    v4u_t t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, (v4u_t *)p);
}
__device__ __forceinline__ void stream_store8(void *p, uint2 v) {
    v2u_t t = {v.x, v.y};
    __builtin_nontemporal_store(t, (v2u_t *)p);
}
__device__ __forceinline__ void stream_store4(void *p, uint32_t v) { __builtin_nontemporal_store(v, (uint32_t *)p); }
inline size_t dtype_size(int dt) { return dt == I8F_F32 ? 4 : 2; }
inline bool valid_dtype(int dt) { return dt == I8F_BF16 || dt == I8F_F16 || dt == I8F_F32; }

}  // namespace i8f
