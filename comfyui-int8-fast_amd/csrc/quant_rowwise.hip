// Fused (block-Hadamard rotation +) per-row absmax int8 quantiser for gfx950.
//
// One pass over HBM: a row is read once with 16-byte loads, kept in registers,
// optionally rotated, reduced to its absolute maximum, scaled, rounded and
// written as int8 with its float scale.  The reference does this in two
// (quantise, int8_fused_kernel.py:10-73) or three (rotate first, quarot.py:99-102)
// separate passes.
//
// Arithmetic contract (bit-exact with the torch path int8_quant.py:20-31 on CPU):
//   amax  = max |v|                    v = x, or the rotated row rounded to x's dtype
//   scale = max(amax / 127.0f, 1e-30f) correctly rounded division
//   inv   = 1.0f / scale               correctly rounded division
//   q     = sat8(rint(v * inv))        ties to even
//
// Rotation: every aligned block of 128 elements is multiplied by the normalised
// Sylvester-Hadamard matrix of x's dtype.  It is evaluated as a 7-stage
// radix-2 butterfly in binary32 with strides 1,2,...,64, each pair (lo,hi)
// becoming (lo+hi, lo-hi), then one multiply by the matrix entry and one
// rounding to x's dtype.  Strides smaller than the per-lane chunk are done in
// registers, the rest across lanes; the order of operations does not depend on
// how the block is spread over lanes.
#include <cstdlib>

#include "i8f_common.hpp"

namespace i8f {
namespace {

template <int DT>
struct Elem {
    static constexpr int EPC = (DT == I8F_F32) ? 4 : 8;  // elements per 16-byte chunk
    static constexpr int LPB = 128 / EPC;                // lanes that share one 128-block
};

// ---- elementwise prologue --------------------------------------------------------------
// What the model computes on the activations right in front of a quantised linear can be applied
// while the row is read, which saves that operation's own pass over [M,K] (one write and one read):
//   I8F_PRO_MODULATE   v = (1 + s[k]) * x + t[k]      adaLN modulation; s, t one vector per group of
//                                                     rows_per_vec rows, in x's dtype.  Evaluated as
//                                                     torch evaluates the three tensor operations in
//                                                     x's dtype: each result rounded to that dtype.
//   I8F_PRO_SILU_GATE  v = silu(x) * g[k]             gated activation of a SwiGLU feed-forward; g like s above (one
//                                                     row of g per row of x when rows_per_vec = 1); silu in binary32
//                                                     rounded to x's dtype, then the product rounded to x's dtype.
//   I8F_PRO_GELU_TANH  v = gelu(x), tanh form         0.5 x (1 + tanh(b (x + 0.044715 x^3))), b = sqrt(2/pi),
//                                                     evaluated in binary32 and rounded once to x's dtype,
//                                                     tanh(u) = 1 - 2 / (exp(2u) + 1) on the hardware's
//                                                     exp2 and reciprocal (a few binary32 ulp).
//   I8F_PRO_GELU_ERF   v = gelu(x), exact form        0.5 x (1 + erf(x / sqrt(2))) = x Phi(x), in binary32, rounded once;
//                                                     erfc by a rational-exponential form good to 1.5e-7 of Phi.
//   I8F_PRO_RMS_NORM   v = x / rms(x) * w[k], then optionally (1 + s[k]) * v and + t[k]; w, s, t may each be absent.
struct Prologue {
    int kind;
    const void *s, *t;       // modulation vectors (MODULATE, NORM_MODULATE), gate operand (SILU_GATE)
    int64_t rows_per_vec;    // rows that share one pair of vectors
    float eps;               // NORM_MODULATE: added to the row's variance
    // CONCAT_GELU: the row is x's row (runs_a runs of 16 elements) followed by gelu(b's row); b [M, .] with its own stride
    const void *b;
    int64_t ldb_bytes;
    int runs_a;
    const void *w;           // RMS_NORM: the norm's weight vector [K] (or nullptr)
    int fused_add;           // the modulation's product and sum with ONE rounding, round((1 + s) * x + t): torch.addcmul
};

// the sum over the wave in a fixed order (the same in every lane)
__device__ __forceinline__ float wave_sum_all(float v) {
#pragma unroll
    for (int b = 1; b < 64; b <<= 1) v += __shfl_xor(v, b, 64);
    return v;
}

// 0.5 x (1 + tanh(u)), u = sqrt(2/pi) (x + 0.044715 x^3), written as x / (1 + exp(-2u)): five vector instructions and the
// hardware's exp2 and reciprocal.  exp(-2u) = exp2(x (c1 + c2 x^2)) with c1 = -2 log2(e) sqrt(2/pi), c2 = 0.044715 c1; an
// overflow to +inf gives x * 0, an underflow to 0 gives x.  No cancellation in the negative tail, unlike 1 + tanh.
__device__ __forceinline__ float gelu_tanh_f32(float x) {
    const float c1 = -2.302208198144325f, c2 = -0.1029432395800235f;
    const float a = x * __builtin_fmaf(x * x, c2, c1);
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(a));
}

// x / (1 + exp(-x)) on the hardware's exp2 and reciprocal (a few binary32 ulp); exp2 overflowing to +inf gives x * 0
__device__ __forceinline__ float silu_f32(float x) {
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

// x Phi(x) with Phi(x) = 1 - erfc(|x| / sqrt 2) / 2 for x >= 0 and erfc(|x| / sqrt 2) / 2 below, so that the negative tail
// is formed without cancellation; erfc(z) = t (a1 + t (a2 + t (a3 + t (a4 + t a5)))) exp(-z^2), t = 1 / (1 + p z)
// (Abramowitz & Stegun 7.1.26, |error| <= 1.5e-7), on the hardware's reciprocal and exp2; the halves are folded into
// the coefficients.  Thirteen vector instructions and the two transcendental ones.
__device__ __forceinline__ float gelu_erf_f32(float x) {
    const float z = fabsf(x) * 0.7071067811865476f;
    const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(z, 0.3275911f, 1.0f));
    float pl = __builtin_fmaf(t, 0.5307027145f, -0.7265760135f);
    pl = __builtin_fmaf(t, pl, 0.7107068705f);
    pl = __builtin_fmaf(t, pl, -0.142248368f);
    pl = __builtin_fmaf(t, pl, 0.127414796f);
    const float h = pl * t * __builtin_amdgcn_exp2f(z * z * -1.4426950408889634f);   // erfc(z) / 2
    return x * (x >= 0.0f ? 1.0f - h : h);
}

// (fused: torch.addcmul(t, x, 1 + s) -- the gain still a rounded tensor of its own, its product with x, exact in binary32
// for 16-bit operands, added to t and rounded once)
template <int DT, int PRO>
__device__ __forceinline__ float apply_prologue(float x, float s, float t, bool fused = false) {
    if constexpr (PRO == I8F_PRO_SILU_GATE) {
        return round_to_dtype<DT>(round_to_dtype<DT>(silu_f32(x)) * s);
    } else if constexpr (PRO == I8F_PRO_MODULATE || PRO == I8F_PRO_NORM_MODULATE) {
        const float a = round_to_dtype<DT>(1.0f + s);
        const float p = a * x;
        const float b = fused ? p : round_to_dtype<DT>(p);
        return round_to_dtype<DT>(b + t);
    } else if constexpr (PRO == I8F_PRO_GELU_TANH) {
        return round_to_dtype<DT>(gelu_tanh_f32(x));
    } else if constexpr (PRO == I8F_PRO_GELU_ERF) {
        return round_to_dtype<DT>(gelu_erf_f32(x));
    } else {
        return x;
    }
}

template <int DT>
__device__ __forceinline__ void load_chunk(const void *p, float (&v)[Elem<DT>::EPC]) {
    const uint4 u = *(const uint4 *)p;
    if constexpr (DT == I8F_F32) {
        v[0] = __uint_as_float(u.x);
        v[1] = __uint_as_float(u.y);
        v[2] = __uint_as_float(u.z);
        v[3] = __uint_as_float(u.w);
    } else if constexpr (DT == I8F_BF16) {
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = __uint_as_float(w[j] << 16);
            v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        }
    } else {
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = f16_bits_to_f32(w[j] & 0xffffu);
            v[2 * j + 1] = f16_bits_to_f32(w[j] >> 16);
        }
    }
}

// Rotate the chunk held by this lane; the LPB lanes of an aligned group hold one
// 128-block, lane g of the group holding elements [g*EPC, (g+1)*EPC).
template <int DT>
__device__ __forceinline__ void rotate_chunk(float (&v)[Elem<DT>::EPC], int lane) {
    constexpr int EPC = Elem<DT>::EPC;
    constexpr int LPB = Elem<DT>::LPB;
#pragma unroll
    for (int s = 1; s < EPC; s <<= 1) {
#pragma unroll
        for (int j = 0; j < EPC; ++j) {
            if ((j & s) == 0) {
                const float lo = v[j], hi = v[j + s];
                v[j] = lo + hi;
                v[j + s] = lo - hi;
            }
        }
    }
#pragma unroll
    for (int b = 1; b < LPB; b <<= 1) {
        const bool upper = (lane & b) != 0;
#pragma unroll
        for (int j = 0; j < EPC; ++j) {
            const float other = __shfl_xor(v[j], b, 64);
            v[j] = upper ? (other - v[j]) : (v[j] + other);
        }
    }
    const float h = hadamard_entry<DT>();
#pragma unroll
    for (int j = 0; j < EPC; ++j) v[j] = round_to_dtype<DT>(v[j] * h);
}

// binary32 rows: a 128-block is 32 chunks of 4 elements, held by an aligned group of 32 lanes.  Strides 1, 2 of the
// butterfly stay inside a lane; strides 4 ... 32 pair chunks c and c ^ 1, c ^ 2, c ^ 4, c ^ 8, which DPP reaches as lanes
// l ^ 1, l ^ 2 (quad permutes), l ^ 7 (mirror of 8 lanes) and l ^ 15 (mirror of a row of 16) if lane l holds chunk
//   c(l) = (l & 3) ^ (7 if bit 2 of l) ^ (12 if bit 3 of l)     (linear over GF(2): c(l ^ 7) = c(l) ^ 4, c(l ^ 15) = c(l) ^ 8)
// of its group of 16; stride 64 pairs the two rows of 16 of the group through one lane exchange.  As in rotate_run16 a
// DPP stage is own + sign * other (one fused multiply-add whose product is exact), which leaves the upper chunk of a
// pair with the negative of the butterfly's value; both lanes of every later pair carry the same accumulated sign, and
// the product of the four signs is folded into the final multiplication.  Same fixed-order butterfly, 4 of the 5
// cross-lane stages without an LDS round trip.
__device__ __forceinline__ int chunk_of_lane16(int l) { return (l & 3) ^ ((l & 4) ? 7 : 0) ^ ((l & 8) ? 12 : 0); }

#define I8F_DPP_FMAC4(ctrl)                                                                                              \
    asm volatile("s_nop 1\n\t"                                                                                           \
                 "v_fmac_f32_dpp %0, %0, %4 " ctrl " row_mask:0xf bank_mask:0xf bound_ctrl:0\n\t"                        \
                 "v_fmac_f32_dpp %1, %1, %4 " ctrl " row_mask:0xf bank_mask:0xf bound_ctrl:0\n\t"                        \
                 "v_fmac_f32_dpp %2, %2, %4 " ctrl " row_mask:0xf bank_mask:0xf bound_ctrl:0\n\t"                        \
                 "v_fmac_f32_dpp %3, %3, %4 " ctrl " row_mask:0xf bank_mask:0xf bound_ctrl:0\n\t"                        \
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3])                                                       \
                 : "v"(sign))
template <int STAGE>
__device__ __forceinline__ void dpp_fmac4(float (&v)[4], float sign) {
    if constexpr (STAGE == 0) I8F_DPP_FMAC4("quad_perm:[1,0,3,2]");
    else if constexpr (STAGE == 1) I8F_DPP_FMAC4("quad_perm:[2,3,0,1]");
    else if constexpr (STAGE == 2) I8F_DPP_FMAC4("row_half_mirror");
    else I8F_DPP_FMAC4("row_mirror");
}

// v: the chunk chunk_of_lane16(lane % 16) + 16 (lane / 16 % 2) of the lane's 128-block
__device__ __forceinline__ void rotate_chunk_f32(float (&v)[4], int lane) {
#pragma unroll
    for (int s = 1; s < 4; s <<= 1) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if ((j & s) == 0) {
                const float lo = v[j], hi = v[j + s];
                v[j] = lo + hi;
                v[j + s] = lo - hi;
            }
        }
    }
    const int c = chunk_of_lane16(lane & 15);
    const float s0 = (c & 1) ? -1.0f : 1.0f, s1 = (c & 2) ? -1.0f : 1.0f, s2 = (c & 4) ? -1.0f : 1.0f, s3 = (c & 8) ? -1.0f : 1.0f;
    dpp_fmac4<0>(v, s0);
    dpp_fmac4<1>(v, s1);
    dpp_fmac4<2>(v, s2);
    dpp_fmac4<3>(v, s3);
    const bool upper = (lane & 16) != 0;   // both lanes of this pair carry the same accumulated sign
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float other = __shfl_xor(v[j], 16, 64);
        v[j] = upper ? (other - v[j]) : (v[j] + other);
    }
    const float h = hadamard_entry<I8F_F32>() * (s0 * s1 * s2 * s3);
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = v[j] * h;
}

// TPR threads share a row (64, 256 or 1024); each holds NCH chunks of it.
template <int DT, bool ROT, int TPR, int NCH>
__global__ __launch_bounds__((TPR > 256 ? TPR : 256)) void quant_rows_kernel(
    const char *__restrict__ x, int64_t M, int64_t K, int64_t ldx_bytes, int8_t *__restrict__ q,
    float *__restrict__ scale) {
    constexpr int EPC = Elem<DT>::EPC;
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int ROWS = BLOCK / TPR;
    constexpr int WPR = TPR / 64;  // waves per row
    const int t = threadIdx.x % TPR;
    const int rb = threadIdx.x / TPR;
    const int64_t m = (int64_t)blockIdx.x * ROWS + rb;
    const bool row_ok = m < M;
    const int nchunks = (int)(K / EPC);
    const char *xrow = x + (row_ok ? m : 0) * ldx_bytes;
    // which chunk of its step a lane holds: its own, or (rotating binary32 rows) the one that lets DPP pair the lanes
    constexpr bool DPP32 = ROT && DT == I8F_F32;
    const int tc = DPP32 ? ((t & ~15) | chunk_of_lane16(t & 15)) : t;

    float v[NCH][EPC];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = i * TPR + tc;
        if (row_ok && c < nchunks) {
            load_chunk<DT>(xrow + (int64_t)c * 16, v[i]);
        } else {
#pragma unroll
            for (int j = 0; j < EPC; ++j) v[i][j] = 0.0f;
        }
    }

    if constexpr (ROT) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            if constexpr (DPP32) rotate_chunk_f32(v[i], t);
            else rotate_chunk<DT>(v[i], t);
        }
    }

    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int j = 0; j < EPC; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
    amax = wave_max(amax);
    if constexpr (WPR > 1) {
        __shared__ float red[ROWS][WPR];
        const int wv = t / 64;
        if ((t & 63) == 0) red[rb][wv] = amax;
        __syncthreads();
        amax = red[rb][0];
#pragma unroll
        for (int w = 1; w < WPR; ++w) amax = fmaxf(amax, red[rb][w]);
    }

    float s = amax / 127.0f;
    s = s < 1e-30f ? 1e-30f : s;
    const float inv = 1.0f / s;

    if (!row_ok) return;
    int8_t *qrow = q + m * K;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = i * TPR + tc;
        if (c < nchunks) {
            uint32_t packed[EPC / 4];
#pragma unroll
            for (int j = 0; j < EPC / 4; ++j) {
                uint32_t w = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    w |= ((uint32_t)quant_i8(v[i][4 * j + b] * inv) & 0xffu) << (8 * b);
                packed[j] = w;
            }
            if constexpr (EPC == 8) {
                stream_store8(qrow + (int64_t)c * 8, make_uint2(packed[0], packed[1]));
            } else {
                *(uint32_t *)(qrow + (int64_t)c * 4) = packed[0];
            }
        }
    }
    if (t == 0) scale[m] = s;
}

// ---- 16-bit inputs, the hot case -------------------------------------------------------
// A lane owns runs of 16 consecutive elements (32 bytes in, 16 bytes out): the int8 store is
// one fully coalesced 16-byte store per lane and run.  With the rotation a 128-block is 8 runs,
// held by an aligned group of 8 lanes: strides 1..8 of the butterfly stay inside a lane, strides
// 16, 32, 64 pair lanes through DPP (quad permutes and the 8-lane mirror).  The mirror flips all
// three low lane bits, so lanes 4..7 of a group hold runs 7,6,5,4: then "mirror" pairs exactly
// the runs that differ in bit 2.  The arithmetic is the same fixed-order butterfly as everywhere
// else; only the assignment of elements to lanes differs.
//
// Rounding to int8 uses the 1.5*2^23 trick: p + 12582912.0f is exact round-half-to-even of p for
// |p| < 2^22 and leaves the two's-complement integer in the low mantissa bits.  No clamp is
// needed: |v * inv| <= 127 * (1 + 2^-22) because inv = 1/fl(amax/127) and |v| <= amax.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xf, 0xf, true));
}

template <int DT>
__device__ __forceinline__ void expand16(const uint4 &a, const uint4 &b, float (&v)[16]) {
    const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        if constexpr (DT == I8F_BF16) {
            v[2 * j] = __uint_as_float(w[j] << 16);
            v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        } else {
            v[2 * j] = f16_bits_to_f32(w[j] & 0xffffu);
            v[2 * j + 1] = f16_bits_to_f32(w[j] >> 16);
        }
    }
}

// v[j] += sign * (v[j] of the partner lane) for 16 registers: v_fmac_f32 with a DPP source.  The
// compiler does not fold a DPP move into a fused multiply-add, hence the assembly.  A DPP read of a
// register needs two wait states after a vector write of it, which the compiler cannot see inside
// the block: the s_nop covers the instruction in front of it, and inside it every instruction
// touches another register.
#define I8F_DPP_FMAC(n, ctrl) "v_fmac_f32_dpp %" #n ", %" #n ", %16 " ctrl " row_mask:0xf bank_mask:0xf bound_ctrl:0\n\t"
#define I8F_DPP_FMAC16(ctrl)                                                                                       \
    asm volatile("s_nop 1\n\t" I8F_DPP_FMAC(0, ctrl) I8F_DPP_FMAC(1, ctrl) I8F_DPP_FMAC(2, ctrl) I8F_DPP_FMAC(3, ctrl)  \
                 I8F_DPP_FMAC(4, ctrl) I8F_DPP_FMAC(5, ctrl) I8F_DPP_FMAC(6, ctrl) I8F_DPP_FMAC(7, ctrl)             \
                 I8F_DPP_FMAC(8, ctrl) I8F_DPP_FMAC(9, ctrl) I8F_DPP_FMAC(10, ctrl) I8F_DPP_FMAC(11, ctrl)           \
                 I8F_DPP_FMAC(12, ctrl) I8F_DPP_FMAC(13, ctrl) I8F_DPP_FMAC(14, ctrl) I8F_DPP_FMAC(15, ctrl)         \
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]),  \
                   "+v"(v[8]), "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]), "+v"(v[14]),         \
                   "+v"(v[15])                                                                                     \
                 : "v"(sign))
template <int STAGE>
__device__ __forceinline__ void dpp_fmac16(float (&v)[16], float sign) {
    if constexpr (STAGE == 0) I8F_DPP_FMAC16("quad_perm:[1,0,3,2]");
    else if constexpr (STAGE == 1) I8F_DPP_FMAC16("quad_perm:[2,3,0,1]");
    else I8F_DPP_FMAC16("row_half_mirror");
}

template <int DT>
__device__ __forceinline__ void rotate_run16(float (&v)[16], float s0, float s1, float s2) {
#pragma unroll
    for (int s = 1; s < 16; s <<= 1) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            if ((j & s) == 0) {
                const float lo = v[j], hi = v[j + s];
                v[j] = lo + hi;
                v[j + s] = lo - hi;
            }
        }
    }
    // Across lanes a stage is own + sign * other: the lower lane gets own + other, the upper lane
    // own - other, which is the negative of the butterfly's other - own.  Negation is exact and
    // commutes with every rounding, both lanes of a later pair carry the same accumulated sign, and
    // the product of the three signs is folded into the final multiplication (hs = +-h).  One
    // fused multiply-add with a DPP operand per element and stage; the product by +-1 is exact, so
    // the sum is rounded once, as an addition would be.
    dpp_fmac16<0>(v, s0);   // quad_perm [1,0,3,2]
    dpp_fmac16<1>(v, s1);   // quad_perm [2,3,0,1]
    dpp_fmac16<2>(v, s2);   // row_half_mirror
    const float h = hadamard_entry<DT>() * (s0 * s1 * s2);
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const float a = v[j] * h;
        // bfloat16: the packed conversion with a zero in the low half leaves the rounded value in the high half, which
        // IS its binary32 form: one instruction rounds and widens (two values per conversion would need two more
        // instructions to pull them apart again)
        if constexpr (DT == I8F_BF16) v[j] = __uint_as_float(f32x2_to_bf16x2_bits(0.0f, a));
        else v[j] = round_to_dtype<DT>(a);
    }
}

__device__ __forceinline__ float max3_abs(float m, float a, float b) {
    float r;
    asm("v_max3_f32 %0, %1, |%2|, |%3|" : "=v"(r) : "v"(m), "v"(a), "v"(b));
    return r;
}

// scale = max(amax / 127, 1e-30) and inv = 1 / scale, both correctly rounded, for an amax that is a value of a 16-bit
// dtype, without the division sequence (22 instructions of a wave's fixed work become 8):
//   amax / 127 = fma(r, y, q) with y = RN(1 / 127), q = RN(amax y), r = amax - 127 q (exact): Markstein's correction,
//     which gives the correctly rounded quotient for every finite bfloat16 and binary16 amax whose quotient is not
//     below the 1e-30 floor (every such value is checked on the host by the test suite);
//   1 / scale = fma(e, y0, y0) with y0 the hardware reciprocal (1 ulp) and e = 1 - scale y0: correctly rounded unless
//     the significand of scale is all ones (Markstein), which takes the division.
__device__ __forceinline__ void scale_and_inverse16(float amax, float &scale, float &inv) {
    const float y = 0x1.020408p-7f;  // RN(1 / 127)
    const float q = amax * y;
    const float r = __builtin_fmaf(-127.0f, q, amax);
    float s = __builtin_fmaf(r, y, q);
    s = s < 1e-30f ? 1e-30f : s;
    const float y0 = __builtin_amdgcn_rcpf(s);
    const float e = __builtin_fmaf(-s, y0, 1.0f);
    float iv = __builtin_fmaf(e, y0, y0);
    // (every lane holds the same scale: a scalar test and a branch that is practically never taken)
    if (__builtin_expect((__builtin_amdgcn_readfirstlane(__float_as_uint(s)) & 0x7fffffu) == 0x7fffffu, 0)) iv = 1.0f / s;
    scale = s;
    inv = iv;
}

// Sixteen values of one run to sixteen int8 in four dwords.  p + 1.5 * 2^23 leaves the rounded integer in the low byte
// of the sum; the additions after the first of each dword write that byte straight into its place (an SDWA destination
// select with the other bytes preserved), so nothing is left to shuffle: 32 instructions per run instead of 44.  An
// instruction that writes part of a register must not be followed at once by a reader of that register: the four dwords
// are worked on in turn, which puts three instructions between any two that touch the same one.
__device__ __forceinline__ uint4 quant16_magic(const float (&v)[16], float inv) {
    float p[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) p[j] = v[j] * inv;
    const float M = 12582912.0f;
    uint32_t o0, o1, o2, o3;
#define I8F_SDWA_ADD(d, s, b) "v_add_f32_sdwa %" #d ", %" #s ", %20 dst_sel:BYTE_" #b " dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
    asm("v_add_f32 %0, %4, %20\n\tv_add_f32 %1, %8, %20\n\tv_add_f32 %2, %12, %20\n\tv_add_f32 %3, %16, %20\n\t"
        I8F_SDWA_ADD(0, 5, 1) I8F_SDWA_ADD(1, 9, 1) I8F_SDWA_ADD(2, 13, 1) I8F_SDWA_ADD(3, 17, 1)
        I8F_SDWA_ADD(0, 6, 2) I8F_SDWA_ADD(1, 10, 2) I8F_SDWA_ADD(2, 14, 2) I8F_SDWA_ADD(3, 18, 2)
        I8F_SDWA_ADD(0, 7, 3) I8F_SDWA_ADD(1, 11, 3) I8F_SDWA_ADD(2, 15, 3) I8F_SDWA_ADD(3, 19, 3)
        "s_nop 0"
        : "=&v"(o0), "=&v"(o1), "=&v"(o2), "=&v"(o3)
        : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7]), "v"(p[8]), "v"(p[9]),
          "v"(p[10]), "v"(p[11]), "v"(p[12]), "v"(p[13]), "v"(p[14]), "v"(p[15]), "v"(M));
#undef I8F_SDWA_ADD
    return make_uint4(o0, o1, o2, o3);
}

// WPR waves share a row (1 or 4); each lane holds RUNS runs of 16 elements; one row per wave or group of
// waves (walking several rows per wave with the next row's loads in flight measured slower at every size:
// fewer, longer-lived waves ramp up and drain more slowly).  FULL: every lane's runs exist and every row of
// the grid exists (K = 16 RUNS 64 WPR, M a multiple of the rows of a workgroup), so nothing is tested or
// zero-filled: 3 % at 4608 x 3072.
// SEG > 1 (with WPR = 1): a row is cut into SEG contiguous segments of whole 128-blocks, one wave each, which share
// only the row maximum: units of half a row, for rows that would otherwise leave some SIMDs with a whole row more
// than others.
template <int DT, bool ROT, int WPR, int RUNS, bool FULL, int PRO, int SEG>
__device__ __forceinline__ void quant16_body(const char *__restrict__ x, int64_t M, int64_t K, int64_t ldx_bytes,
                                             int8_t *__restrict__ q, float *__restrict__ scale, const Prologue &pro,
                                             int64_t first_row) {
    static_assert(SEG == 1 || WPR == 1, "segments are for the one-wave-per-row form");
    constexpr int TPR = 64 * WPR;
    constexpr int ROWS = 256 / (TPR * SEG);  // rows per workgroup
    const int t = threadIdx.x % TPR;
    const int unit = threadIdx.x / TPR;
    const int rb = unit / SEG, sg = unit % SEG;
    const int64_t m = first_row + rb;
    const int nruns = (int)(K / 16) / SEG;   // runs of this wave's segment (of the row if SEG == 1)
    const int64_t seg_run = (int64_t)sg * nruns;  // first run of the segment
    // run held by this lane inside its group of 8: lanes 4..7 take runs 7..4
    const int p = t ^ (((t >> 2) & 1) * 3);
    const float s0 = (p & 1) ? -1.0f : 1.0f, s1 = (p & 2) ? -1.0f : 1.0f, s2 = (p & 4) ? -1.0f : 1.0f;

    uint4 raw[RUNS][2];
    {
        const bool ok = FULL || m < M;
        const char *xrow = x + (ok ? m : 0) * ldx_bytes;
        [[maybe_unused]] const char *brow = nullptr;
        if constexpr (PRO == I8F_PRO_CONCAT_GELU) brow = (const char *)pro.b + (ok ? m : 0) * pro.ldb_bytes;
#pragma unroll
        for (int r = 0; r < RUNS; ++r) {
            const int R = r * TPR + p;
            if (FULL || (ok && R < nruns)) {
                const char *src = xrow + (seg_run + R) * 32;
                if constexpr (PRO == I8F_PRO_CONCAT_GELU) {   // the runs behind x's row come from b's
                    if (R >= pro.runs_a) src = brow + (int64_t)(R - pro.runs_a) * 32;
                }
                raw[r][0] = *(const uint4 *)src;
                raw[r][1] = *(const uint4 *)(src + 16);
            } else {
                raw[r][0] = make_uint4(0, 0, 0, 0);
                raw[r][1] = make_uint4(0, 0, 0, 0);
            }
        }
    }
    {
        float v[RUNS][16];
        float amax = 0.0f;
        // A row's sum for the normalising prologues: over the wave, then (four waves to a row) over the waves' partial
        // sums through LDS, always in the same order, so that launches agree bit for bit.  Two slots: the second sum
        // of a LayerNorm may be written while a slower wave still reads the first.
        [[maybe_unused]] __shared__ float row_sums[2][ROWS][WPR];
        [[maybe_unused]] auto row_sum = [&](float part, int slot) {
            part = wave_sum_all(part);
            if constexpr (WPR > 1) {
                if ((t & 63) == 0) row_sums[slot][rb][t / 64] = part;
                __syncthreads();
                part = row_sums[slot][rb][0];
#pragma unroll
                for (int w = 1; w < WPR; ++w) part += row_sums[slot][rb][w];
            }
            return part;
        };
        [[maybe_unused]] int64_t vrow = 0;  // the row's pair of modulation vectors (M < 2^31: a 32-bit division)
        if constexpr (PRO == I8F_PRO_MODULATE || PRO == I8F_PRO_SILU_GATE || PRO == I8F_PRO_NORM_MODULATE || PRO == I8F_PRO_RMS_NORM)
            vrow = (uint32_t)(FULL || m < M ? m : 0) / (uint32_t)pro.rows_per_vec;
        if constexpr (PRO == I8F_PRO_NORM_MODULATE) {
            // LayerNorm without affine over the row, which this wave holds whole: mean, then the variance of the
            // differences (two passes over registers), y = (x - mean) / sqrt(var + eps) rounded to the dtype.
            static_assert(SEG == 1, "the row's statistics are taken by the waves that hold it whole");
            float sum = 0.0f;
#pragma unroll
            for (int r = 0; r < RUNS; ++r) {
                expand16<DT>(raw[r][0], raw[r][1], v[r]);   // (runs beyond the row are zeros)
#pragma unroll
                for (int j = 0; j < 16; ++j) sum += v[r][j];
            }
            const float mean = row_sum(sum, 0) / (float)K;
            float ss = 0.0f;
#pragma unroll
            for (int r = 0; r < RUNS; ++r) {
                const bool in = FULL || r * TPR + p < nruns;
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const float d = v[r][j] - mean;
                    v[r][j] = d;
                    ss += in ? d * d : 0.0f;
                }
            }
            const float rstd = 1.0f / sqrtf(row_sum(ss, 1) / (float)K + pro.eps);
#pragma unroll
            for (int r = 0; r < RUNS; ++r)
#pragma unroll
                for (int j = 0; j < 16; ++j) v[r][j] = round_to_dtype<DT>(v[r][j] * rstd);
        }
        if constexpr (PRO == I8F_PRO_RMS_NORM) {
            // RMSNorm over the row, which this wave holds whole: y = x / sqrt(sum x^2 / K + eps) * w in binary32, rounded
            // once to the dtype (torch's rms_norm); then the modulation's operations, each rounded, where s / t exist.
            static_assert(SEG == 1, "the row's statistics are taken by the waves that hold it whole");
            float ss = 0.0f;
#pragma unroll
            for (int r = 0; r < RUNS; ++r) {
                expand16<DT>(raw[r][0], raw[r][1], v[r]);   // (runs beyond the row are zeros)
#pragma unroll
                for (int j = 0; j < 16; ++j) ss = __builtin_fmaf(v[r][j], v[r][j], ss);
            }
            const float rstd = 1.0f / sqrtf(row_sum(ss, 0) / (float)K + pro.eps);
#pragma unroll
            for (int r = 0; r < RUNS; ++r) {
                const int R = r * TPR + p;
                const bool in = FULL || R < nruns;
                const int64_t col = (in ? R : 0) * 32;   // byte offset of the run's columns in a vector
                float wv[16];
                if (pro.w) {
                    expand16<DT>(*(const uint4 *)((const char *)pro.w + col), *(const uint4 *)((const char *)pro.w + col + 16), wv);
#pragma unroll
                    for (int j = 0; j < 16; ++j) v[r][j] = round_to_dtype<DT>(v[r][j] * rstd * wv[j]);
                } else {
#pragma unroll
                    for (int j = 0; j < 16; ++j) v[r][j] = round_to_dtype<DT>(v[r][j] * rstd);
                }
                const int64_t off = vrow * K * 2 + col;
                if (pro.s) {
                    expand16<DT>(*(const uint4 *)((const char *)pro.s + off), *(const uint4 *)((const char *)pro.s + off + 16), wv);
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        const float pr = round_to_dtype<DT>(1.0f + wv[j]) * v[r][j];
                        v[r][j] = (pro.fused_add && pro.t) ? pr : round_to_dtype<DT>(pr);   // (fused: rounded with the sum below)
                    }
                }
                if (pro.t) {
                    expand16<DT>(*(const uint4 *)((const char *)pro.t + off), *(const uint4 *)((const char *)pro.t + off + 16), wv);
#pragma unroll
                    for (int j = 0; j < 16; ++j) v[r][j] = round_to_dtype<DT>(v[r][j] + wv[j]);
                }
                if (!in) {
#pragma unroll
                    for (int j = 0; j < 16; ++j) v[r][j] = 0.0f;
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RUNS; ++r) {
            if constexpr (PRO != I8F_PRO_NORM_MODULATE && PRO != I8F_PRO_RMS_NORM) expand16<DT>(raw[r][0], raw[r][1], v[r]);
            if constexpr (PRO == I8F_PRO_MODULATE || PRO == I8F_PRO_NORM_MODULATE) {
                // the vectors of this row's group, same 16 columns (they come from cache: every row of the group reads them)
                const int R = r * TPR + p;
                const int64_t off = (vrow * K + (seg_run + (FULL || R < nruns ? R : 0)) * 16) * 2;
                float sv[16], tv[16];
                expand16<DT>(*(const uint4 *)((const char *)pro.s + off), *(const uint4 *)((const char *)pro.s + off + 16), sv);
                expand16<DT>(*(const uint4 *)((const char *)pro.t + off), *(const uint4 *)((const char *)pro.t + off + 16), tv);
#pragma unroll
                for (int j = 0; j < 16; ++j) v[r][j] = FULL || R < nruns ? apply_prologue<DT, PRO>(v[r][j], sv[j], tv[j], pro.fused_add != 0) : 0.0f;
            } else if constexpr (PRO == I8F_PRO_SILU_GATE) {
                const int R = r * TPR + p;
                const int64_t off = (vrow * K + (seg_run + (FULL || R < nruns ? R : 0)) * 16) * 2;
                float gv[16];
                expand16<DT>(*(const uint4 *)((const char *)pro.s + off), *(const uint4 *)((const char *)pro.s + off + 16), gv);
#pragma unroll
                for (int j = 0; j < 16; ++j) v[r][j] = FULL || R < nruns ? apply_prologue<DT, PRO>(v[r][j], gv[j], 0.0f) : 0.0f;
            } else if constexpr (PRO == I8F_PRO_GELU_TANH || PRO == I8F_PRO_GELU_ERF) {
#pragma unroll
                for (int j = 0; j < 16; ++j) v[r][j] = apply_prologue<DT, PRO>(v[r][j], 0.0f, 0.0f);
            } else if constexpr (PRO == I8F_PRO_CONCAT_GELU) {
                const bool from_b = r * TPR + p >= pro.runs_a;   // (per lane: a wave's runs straddle the seam)
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const float act = apply_prologue<DT, I8F_PRO_GELU_TANH>(v[r][j], 0.0f, 0.0f);
                    v[r][j] = from_b ? act : v[r][j];
                }
            }
            if constexpr (ROT) rotate_run16<DT>(v[r], s0, s1, s2);
#pragma unroll
            for (int j = 0; j < 16; j += 2) amax = max3_abs(amax, v[r][j], v[r][j + 1]);
        }
        amax = wave_max(amax);
        if constexpr (WPR * SEG > 1) {
            __shared__ float red[ROWS][WPR * SEG];
            if ((t & 63) == 0) red[rb][sg * WPR + t / 64] = amax;
            __syncthreads();
            amax = red[rb][0];
#pragma unroll
            for (int w = 1; w < WPR * SEG; ++w) amax = fmaxf(amax, red[rb][w]);
        }

        float s, inv;
        scale_and_inverse16(amax, s, inv);

        if (FULL || m < M) {
            int8_t *qrow = q + m * K;
#pragma unroll
            for (int r = 0; r < RUNS; ++r) {
                const int R = r * TPR + p;
                if (FULL || R < nruns) {
                    stream_store16(qrow + (seg_run + R) * 16, quant16_magic(v[r], inv));
                }
            }
            if (t == 0 && sg == 0) scale[m] = s;
        }
    }
}

template <int DT, bool ROT, int WPR, int RUNS, bool FULL, int PRO = I8F_PRO_NONE>
__global__ __launch_bounds__(256) void quant16_kernel(const char *__restrict__ x, int64_t M, int64_t K,
                                                       int64_t ldx_bytes, int8_t *__restrict__ q,
                                                       float *__restrict__ scale, const Prologue pro) {
    quant16_body<DT, ROT, WPR, RUNS, FULL, PRO, 1>(x, M, K, ldx_bytes, q, scale, pro, (int64_t)blockIdx.x * (256 / (64 * WPR)));
}

// The rotating quantiser is bound by the vector ALUs of the SIMDs that get the most rows.  1 024 SIMDs take a multiple
// of 1 024 rows evenly, one wave per row; up to 512 rows beyond that would put a whole extra row on as many SIMDs
// while the others idle, so those rows go as half rows (two waves to a row, two rows to a workgroup): every SIMD gets
// at most half a row more.  One launch: the first main_blocks workgroups take four whole rows each, the others two
// rows in halves.
constexpr int TAIL_SEG = 2;  // (quarter rows measured the same as half rows: twice the waves, each with a wave's fixed work)
template <int DT, bool ROT, int RUNS>
__global__ __launch_bounds__(256) void quant16_tail_kernel(const char *__restrict__ x, int64_t M, int64_t K,
                                                            int64_t ldx_bytes, int8_t *__restrict__ q,
                                                            float *__restrict__ scale, int main_blocks) {
    const Prologue none{};
    if ((int)blockIdx.x < main_blocks)
        quant16_body<DT, ROT, 1, RUNS, true, I8F_PRO_NONE, 1>(x, M, K, ldx_bytes, q, scale, none, (int64_t)blockIdx.x * 4);
    else
        quant16_body<DT, ROT, 1, (RUNS + TAIL_SEG - 1) / TAIL_SEG, false, I8F_PRO_NONE, TAIL_SEG>(
            x, M, K, ldx_bytes, q, scale, none, (int64_t)main_blocks * 4 + ((int64_t)blockIdx.x - main_blocks) * (4 / TAIL_SEG));
}

// Several row blocks of one width in one launch (the image and the text tokens of a transformer block, each with
// its own tensors): workgroup b belongs to the group whose range of workgroups holds b.  Launches of a few
// microseconds cost as much in the gap between kernels as in the kernel, so two 5 us launches become one of 7.
constexpr int MAX_GROUPS = 8;
struct GroupedArgs {
    const char *x[MAX_GROUPS];
    int8_t *q[MAX_GROUPS];
    float *scale[MAX_GROUPS];
    int64_t M[MAX_GROUPS], ldx_bytes[MAX_GROUPS];
    int first_block[MAX_GROUPS + 1];   // first workgroup of each group; [n] = all workgroups
    int n;
};

// FULL: every group's rows fill its workgroups and K fills every lane's runs (no bounds tests, no zero fill)
template <int DT, bool ROT, int WPR, int RUNS, bool FULL>
__global__ __launch_bounds__(256) void quant16_grouped_kernel(const GroupedArgs g, int64_t K) {
    int grp = 0;
#pragma unroll
    for (int i = 1; i < MAX_GROUPS; ++i)
        if (i < g.n && (int)blockIdx.x >= g.first_block[i]) grp = i;
    grp = __builtin_amdgcn_readfirstlane(grp);
    const Prologue none{};
    quant16_body<DT, ROT, WPR, RUNS, FULL, I8F_PRO_NONE, 1>(g.x[grp], g.M[grp], K, g.ldx_bytes[grp], g.q[grp], g.scale[grp], none,
                                                            (int64_t)((int)blockIdx.x - g.first_block[grp]) * (256 / (64 * WPR)));
}

template <int DT, bool ROT, int WPR, int RUNS>
int launch16_grouped(const GroupedArgs &g, int64_t K, hipStream_t st) {
    constexpr int ROWS = 256 / (64 * WPR);
    bool full = K == (int64_t)RUNS * 64 * WPR * 16;
    for (int i = 0; i < g.n; ++i) full = full && g.M[i] % ROWS == 0;
    if (full)
        hipLaunchKernelGGL((quant16_grouped_kernel<DT, ROT, WPR, RUNS, true>), dim3((unsigned)g.first_block[g.n]), dim3(256), 0, st, g, K);
    else
        hipLaunchKernelGGL((quant16_grouped_kernel<DT, ROT, WPR, RUNS, false>), dim3((unsigned)g.first_block[g.n]), dim3(256), 0, st, g, K);
    return check_launch();
}

template <int DT, bool ROT, int WPR>
int pick_runs16_grouped(int runs, const GroupedArgs &g, int64_t K, hipStream_t st) {
    switch (runs) {
    case 1: return launch16_grouped<DT, ROT, WPR, 1>(g, K, st);
    case 2: return launch16_grouped<DT, ROT, WPR, 2>(g, K, st);
    case 3: return launch16_grouped<DT, ROT, WPR, 3>(g, K, st);
    default: return launch16_grouped<DT, ROT, WPR, 4>(g, K, st);
    }
}

template <int DT, bool ROT, int WPR, int RUNS, int PRO = I8F_PRO_NONE>
int launch16(const void *x, int64_t M, int64_t K, int64_t ldx, int8_t *q, float *scale, hipStream_t st, const Prologue &pro = Prologue{}) {
    constexpr int ROWS = 256 / (64 * WPR);
    const int64_t blocks = (M + ROWS - 1) / ROWS;
    if constexpr (ROT && PRO == I8F_PRO_NONE && WPR == 1) {  // (the quantiser without rotation is not bound by the vector ALUs: the split costs it 2 %)
        // whole rows for every SIMD, then the rest (at most half a row per SIMD) in half rows of whole 128-blocks
        const int64_t rest = M % 1024;
        if (K == (int64_t)RUNS * 64 * 16 && M % 4 == 0 && M >= 1024 && rest > 0 && rest <= 512 && (K / 16) % (8 * TAIL_SEG) == 0) {
            const int main_blocks = (int)((M - rest) / 4);
            hipLaunchKernelGGL((quant16_tail_kernel<DT, ROT, RUNS>), dim3((unsigned)(main_blocks + rest * TAIL_SEG / 4)), dim3(256), 0, st,
                               (const char *)x, M, K, ldx * 2, q, scale, main_blocks);
            return check_launch();
        }
    }
    if (PRO == I8F_PRO_NONE && K == (int64_t)RUNS * 64 * WPR * 16 && M % ROWS == 0)
        hipLaunchKernelGGL((quant16_kernel<DT, ROT, WPR, RUNS, PRO == I8F_PRO_NONE, PRO>), dim3((unsigned)blocks), dim3(ROWS * 64 * WPR), 0, st,
                           (const char *)x, M, K, ldx * 2, q, scale, pro);
    else
        hipLaunchKernelGGL((quant16_kernel<DT, ROT, WPR, RUNS, false, PRO>), dim3((unsigned)blocks), dim3(ROWS * 64 * WPR), 0, st,
                           (const char *)x, M, K, ldx * 2, q, scale, pro);
    return check_launch();
}

template <int DT, bool ROT, int WPR, int PRO = I8F_PRO_NONE>
int pick_runs16(int runs, const void *x, int64_t M, int64_t K, int64_t ldx, int8_t *q, float *scale, hipStream_t st, const Prologue &pro = Prologue{}) {
    switch (runs) {
    case 1: return launch16<DT, ROT, WPR, 1, PRO>(x, M, K, ldx, q, scale, st, pro);
    case 2: return launch16<DT, ROT, WPR, 2, PRO>(x, M, K, ldx, q, scale, st, pro);
    case 3: return launch16<DT, ROT, WPR, 3, PRO>(x, M, K, ldx, q, scale, st, pro);
    default: return launch16<DT, ROT, WPR, 4, PRO>(x, M, K, ldx, q, scale, st, pro);
    }
}

// ---- generic kernel: any K, any alignment; one 256-thread block per row, the row
// is read twice (the second time from cache) --------------------------------------
template <int DT>
__device__ __forceinline__ void rotate128_wave(float &e0, float &e1, int lane) {
    // the wave holds one 128-block: lane l has elements l (e0) and l + 64 (e1)
#pragma unroll
    for (int b = 1; b < 64; b <<= 1) {
        const bool upper = (lane & b) != 0;
        const float o0 = __shfl_xor(e0, b, 64);
        const float o1 = __shfl_xor(e1, b, 64);
        e0 = upper ? (o0 - e0) : (e0 + o0);
        e1 = upper ? (o1 - e1) : (e1 + o1);
    }
    const float lo = e0, hi = e1;
    e0 = lo + hi;
    e1 = lo - hi;
    const float h = hadamard_entry<DT>();
    e0 = round_to_dtype<DT>(e0 * h);
    e1 = round_to_dtype<DT>(e1 * h);
}

template <int DT, bool ROT, int PRO = I8F_PRO_NONE>
__global__ __launch_bounds__(256) void quant_rows_generic_kernel(const void *__restrict__ x, int64_t M,
                                                                  int64_t K, int64_t ldx,
                                                                  int8_t *__restrict__ q,
                                                                  float *__restrict__ scale, const Prologue pro) {
    const int64_t m = blockIdx.x;
    if (m >= M) return;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wv = tid >> 6;
    const int64_t base = m * ldx;
    __shared__ float red[4];
    // element k of this row after the prologue
    const int64_t vbase = (PRO == I8F_PRO_MODULATE || PRO == I8F_PRO_SILU_GATE) ? (m / pro.rows_per_vec) * K : 0;
    auto element = [&](int64_t k) {
        const float xv = load_as_f32<DT>(x, base + k);
        if constexpr (PRO == I8F_PRO_SILU_GATE) return apply_prologue<DT, PRO>(xv, load_as_f32<DT>(pro.s, vbase + k), 0.0f);
        else if constexpr (PRO == I8F_PRO_MODULATE) return apply_prologue<DT, PRO>(xv, load_as_f32<DT>(pro.s, vbase + k), load_as_f32<DT>(pro.t, vbase + k), pro.fused_add != 0);
        else return apply_prologue<DT, PRO>(xv, 0.0f, 0.0f);
    };

    float amax = 0.0f;
    if constexpr (ROT) {
        for (int64_t blk = wv; blk < K / 128; blk += 4) {
            float e0 = element(blk * 128 + lane);
            float e1 = element(blk * 128 + 64 + lane);
            rotate128_wave<DT>(e0, e1, lane);
            amax = fmaxf(amax, fmaxf(fabsf(e0), fabsf(e1)));
        }
    } else {
        for (int64_t k = tid; k < K; k += 256) amax = fmaxf(amax, fabsf(element(k)));
    }
    amax = wave_max(amax);
    if (lane == 0) red[wv] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));

    float s = amax / 127.0f;
    s = s < 1e-30f ? 1e-30f : s;
    const float inv = 1.0f / s;
    int8_t *qrow = q + m * K;
    if constexpr (ROT) {
        for (int64_t blk = wv; blk < K / 128; blk += 4) {
            float e0 = element(blk * 128 + lane);
            float e1 = element(blk * 128 + 64 + lane);
            rotate128_wave<DT>(e0, e1, lane);
            qrow[blk * 128 + lane] = (int8_t)quant_i8(e0 * inv);
            qrow[blk * 128 + 64 + lane] = (int8_t)quant_i8(e1 * inv);
        }
    } else {
        for (int64_t k = tid; k < K; k += 256) qrow[k] = (int8_t)quant_i8(element(k) * inv);
    }
    if (tid == 0) scale[m] = s;
}

// ---- rotation alone -------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ void store_chunk(void *p, const float (&v)[Elem<DT>::EPC]) {
    if constexpr (DT == I8F_F32) {
        *(float4 *)p = make_float4(v[0], v[1], v[2], v[3]);
    } else {
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (DT == I8F_BF16) w[j] = f32x2_to_bf16x2_bits(v[2 * j], v[2 * j + 1]);
            else w[j] = f32x2_to_f16x2_bits(v[2 * j], v[2 * j + 1]);
        }
        stream_store16(p, make_uint4(w[0], w[1], w[2], w[3]));
    }
}

// one thread per 16-byte chunk; an aligned group of LPB lanes holds one 128-block
template <int DT>
__global__ __launch_bounds__(256) void rotate_kernel(const char *x, int64_t M, int64_t K,
                                                      int64_t ldx_bytes, char *out) {
    constexpr int EPC = Elem<DT>::EPC;
    const int64_t nchunks = K / EPC;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool ok = idx < M * nchunks;
    const int64_t m = ok ? idx / nchunks : 0, c = ok ? idx % nchunks : 0;
    float v[EPC];
    if (ok) {
        load_chunk<DT>(x + m * ldx_bytes + c * 16, v);
    } else {
#pragma unroll
        for (int j = 0; j < EPC; ++j) v[j] = 0.0f;
    }
    rotate_chunk<DT>(v, threadIdx.x);
    if (ok) store_chunk<DT>(out + (m * nchunks + c) * 16, v);
}

// any alignment: one wavefront per 128-block
template <int DT>
__global__ __launch_bounds__(256) void rotate_generic_kernel(const void *x, int64_t M, int64_t K,
                                                              int64_t ldx, void *out) {
    const int lane = threadIdx.x & 63;
    const int64_t blk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t per_row = K / 128;
    if (blk >= M * per_row) return;
    const int64_t m = blk / per_row, b = blk % per_row;
    float e0 = load_as_f32<DT>(x, m * ldx + b * 128 + lane);
    float e1 = load_as_f32<DT>(x, m * ldx + b * 128 + 64 + lane);
    rotate128_wave<DT>(e0, e1, lane);
    store_from_f32<DT>(out, m * K + b * 128 + lane, e0);
    store_from_f32<DT>(out, m * K + b * 128 + 64 + lane, e1);
}

template <int DT>
int launch_rotate(const void *x, int64_t M, int64_t K, int64_t ldx, void *out, hipStream_t st) {
    constexpr int EPC = Elem<DT>::EPC;
    const size_t es = dtype_size(DT);
    const bool aligned = ((uintptr_t)x % 16 == 0) && ((ldx * es) % 16 == 0) && ((uintptr_t)out % 16 == 0);
    if (aligned) {
        const int64_t total = M * (K / EPC);
        hipLaunchKernelGGL((rotate_kernel<DT>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                           (const char *)x, M, K, ldx * (int64_t)es, (char *)out);
    } else {
        const int64_t blocks = M * (K / 128);
        hipLaunchKernelGGL((rotate_generic_kernel<DT>), dim3((unsigned)((blocks + 3) / 4)), dim3(256), 0, st, x, M,
                           K, ldx, out);
    }
    return check_launch();
}

template <int DT, bool ROT, int TPR, int NCH>
int launch_fast(const void *x, int64_t M, int64_t K, int64_t ldx, int8_t *q, float *scale,
                hipStream_t st) {
    constexpr int BLOCK = TPR > 256 ? TPR : 256;
    constexpr int ROWS = BLOCK / TPR;
    const int64_t blocks = (M + ROWS - 1) / ROWS;
    hipLaunchKernelGGL((quant_rows_kernel<DT, ROT, TPR, NCH>), dim3((unsigned)blocks), dim3(BLOCK), 0, st,
                       (const char *)x, M, K, ldx * (int64_t)dtype_size(DT), q, scale);
    return check_launch();
}

template <int DT, bool ROT, int TPR>
int pick_nch(int per_thread, const void *x, int64_t M, int64_t K, int64_t ldx, int8_t *q, float *scale,
             hipStream_t st) {
    if (per_thread <= 1) return launch_fast<DT, ROT, TPR, 1>(x, M, K, ldx, q, scale, st);
    if (per_thread <= 2) return launch_fast<DT, ROT, TPR, 2>(x, M, K, ldx, q, scale, st);
    if (per_thread <= 4) return launch_fast<DT, ROT, TPR, 4>(x, M, K, ldx, q, scale, st);
    if (per_thread <= 6) return launch_fast<DT, ROT, TPR, 6>(x, M, K, ldx, q, scale, st);
    return launch_fast<DT, ROT, TPR, 8>(x, M, K, ldx, q, scale, st);
}

template <int DT, bool ROT, int PRO = I8F_PRO_NONE>
int dispatch(const void *x, int64_t M, int64_t K, int64_t ldx, int8_t *q, float *scale, hipStream_t st, const Prologue &pro = Prologue{}) {
    constexpr int EPC = Elem<DT>::EPC;
    const size_t es = dtype_size(DT);
    bool aligned = ((uintptr_t)x % 16 == 0) && ((ldx * es) % 16 == 0) && (K % EPC == 0) && ((uintptr_t)q % 8 == 0);
    if constexpr (PRO == I8F_PRO_MODULATE || PRO == I8F_PRO_NORM_MODULATE) aligned = aligned && (uintptr_t)pro.s % 16 == 0 && (uintptr_t)pro.t % 16 == 0;
    if constexpr (PRO == I8F_PRO_RMS_NORM)   // (absent vectors are null pointers, which pass)
        aligned = aligned && (uintptr_t)pro.s % 16 == 0 && (uintptr_t)pro.t % 16 == 0 && (uintptr_t)pro.w % 16 == 0;
    if constexpr (PRO == I8F_PRO_SILU_GATE) aligned = aligned && (uintptr_t)pro.s % 16 == 0;
    if constexpr (PRO == I8F_PRO_CONCAT_GELU) aligned = aligned && (uintptr_t)pro.b % 16 == 0 && pro.ldb_bytes % 16 == 0;
    const int64_t nchunks = K / EPC;
    if constexpr (DT != I8F_F32) {
        const int64_t nruns = K / 16;
        if (aligned && K % 16 == 0 && (uintptr_t)q % 16 == 0 && nruns >= 1 && nruns <= 64 * 4 * 4) {
            if (nruns <= 64 * 4) return pick_runs16<DT, ROT, 1, PRO>((int)((nruns + 63) / 64), x, M, K, ldx, q, scale, st, pro);
            return pick_runs16<DT, ROT, 4, PRO>((int)((nruns + 255) / 256), x, M, K, ldx, q, scale, st, pro);
        }
    }
    // the normalising and the concatenating prologues exist where the row stays in registers: 16-bit rows of up to
    // 16384 aligned elements
    if constexpr (PRO == I8F_PRO_NORM_MODULATE || PRO == I8F_PRO_RMS_NORM || PRO == I8F_PRO_CONCAT_GELU) return I8F_ERR_UNSUPPORTED;
    else {
    if constexpr (PRO == I8F_PRO_NONE) {  // the chunked kernels have no prologue form: such shapes take the generic kernel
        if (aligned && nchunks <= 1024 * 8) {
            if (nchunks <= 64 * 8) return pick_nch<DT, ROT, 64>((int)((nchunks + 63) / 64), x, M, K, ldx, q, scale, st);
            if (nchunks <= 256 * 8) return pick_nch<DT, ROT, 256>((int)((nchunks + 255) / 256), x, M, K, ldx, q, scale, st);
            return pick_nch<DT, ROT, 1024>((int)((nchunks + 1023) / 1024), x, M, K, ldx, q, scale, st);
        }
    }
    hipLaunchKernelGGL((quant_rows_generic_kernel<DT, ROT, PRO>), dim3((unsigned)M), dim3(256), 0, st, x, M, K, ldx,
                       q, scale, pro);
    return check_launch();
    }
}

template <int DT>
int dispatch_rot(bool rot, const void *x, int64_t M, int64_t K, int64_t ldx, int8_t *q, float *scale,
                 hipStream_t st, const Prologue &pro = Prologue{}) {
    switch (pro.kind) {
    case I8F_PRO_MODULATE:
        return rot ? dispatch<DT, true, I8F_PRO_MODULATE>(x, M, K, ldx, q, scale, st, pro)
                   : dispatch<DT, false, I8F_PRO_MODULATE>(x, M, K, ldx, q, scale, st, pro);
    case I8F_PRO_GELU_TANH:
        return rot ? dispatch<DT, true, I8F_PRO_GELU_TANH>(x, M, K, ldx, q, scale, st, pro)
                   : dispatch<DT, false, I8F_PRO_GELU_TANH>(x, M, K, ldx, q, scale, st, pro);
    case I8F_PRO_GELU_ERF:
        return rot ? dispatch<DT, true, I8F_PRO_GELU_ERF>(x, M, K, ldx, q, scale, st, pro)
                   : dispatch<DT, false, I8F_PRO_GELU_ERF>(x, M, K, ldx, q, scale, st, pro);
    case I8F_PRO_RMS_NORM:
        if constexpr (DT == I8F_F32) return I8F_ERR_UNSUPPORTED;
        else return rot ? dispatch<DT, true, I8F_PRO_RMS_NORM>(x, M, K, ldx, q, scale, st, pro)
                        : dispatch<DT, false, I8F_PRO_RMS_NORM>(x, M, K, ldx, q, scale, st, pro);
    case I8F_PRO_SILU_GATE:
        return rot ? dispatch<DT, true, I8F_PRO_SILU_GATE>(x, M, K, ldx, q, scale, st, pro)
                   : dispatch<DT, false, I8F_PRO_SILU_GATE>(x, M, K, ldx, q, scale, st, pro);
    case I8F_PRO_CONCAT_GELU:
        if constexpr (DT == I8F_F32) return I8F_ERR_UNSUPPORTED;
        else return rot ? dispatch<DT, true, I8F_PRO_CONCAT_GELU>(x, M, K, ldx, q, scale, st, pro)
                        : dispatch<DT, false, I8F_PRO_CONCAT_GELU>(x, M, K, ldx, q, scale, st, pro);
    case I8F_PRO_NORM_MODULATE:
        if constexpr (DT == I8F_F32) return I8F_ERR_UNSUPPORTED;
        else return rot ? dispatch<DT, true, I8F_PRO_NORM_MODULATE>(x, M, K, ldx, q, scale, st, pro)
                        : dispatch<DT, false, I8F_PRO_NORM_MODULATE>(x, M, K, ldx, q, scale, st, pro);
    default: return rot ? dispatch<DT, true>(x, M, K, ldx, q, scale, st) : dispatch<DT, false>(x, M, K, ldx, q, scale, st);
    }
}

}  // namespace
}  // namespace i8f

extern "C" int i8f_quant_rowwise(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                                 int rotate_block, int8_t *q, float *scale, void *stream) {
    using namespace i8f;
    if (M < 0 || K < 0 || !valid_dtype(x_dtype)) return I8F_ERR_INVALID;
    if (rotate_block != 0 && rotate_block != 128) return I8F_ERR_UNSUPPORTED;
    if (rotate_block && K % rotate_block) return I8F_ERR_INVALID;
    if (M == 0) return I8F_OK;
    if (!scale || ldx < K) return I8F_ERR_INVALID;
    if (K > 0 && (!x || !q)) return I8F_ERR_INVALID;
    if (M > 0x7fffffff) return I8F_ERR_UNSUPPORTED;
    if (int rc = check_device()) return rc;
    hipStream_t st = (hipStream_t)stream;
    const bool rot = rotate_block != 0;
    switch (x_dtype) {
    case I8F_BF16: return dispatch_rot<I8F_BF16>(rot, x, M, K, ldx, q, scale, st);
    case I8F_F16: return dispatch_rot<I8F_F16>(rot, x, M, K, ldx, q, scale, st);
    default: return dispatch_rot<I8F_F32>(rot, x, M, K, ldx, q, scale, st);
    }
}

extern "C" int i8f_quant_rowwise_grouped(const i8f_quant_group *groups, int n_groups, int x_dtype, int64_t K,
                                         int rotate_block, void *stream) {
    using namespace i8f;
    if (n_groups < 0 || (n_groups > 0 && !groups) || K < 0 || !valid_dtype(x_dtype)) return I8F_ERR_INVALID;
    if (rotate_block != 0 && rotate_block != 128) return I8F_ERR_UNSUPPORTED;
    if (rotate_block && K % rotate_block) return I8F_ERR_INVALID;
    bool one_launch = x_dtype != I8F_F32 && n_groups >= 2 && n_groups <= MAX_GROUPS && K % 16 == 0 && K >= 16 && K <= 16 * 64 * 4 * 4;
    int64_t blocks = 0;
    const int wpr = K / 16 <= 64 * 4 ? 1 : 4;
    for (int i = 0; i < n_groups; ++i) {
        const i8f_quant_group &g = groups[i];
        if (g.M < 0 || (g.M > 0 && (!g.scale || g.ldx < K || (K > 0 && (!g.x || !g.q))))) return I8F_ERR_INVALID;
        if (g.M > 0x7fffffff) return I8F_ERR_UNSUPPORTED;
        one_launch = one_launch && (uintptr_t)g.x % 16 == 0 && (g.ldx * 2) % 16 == 0 && (uintptr_t)g.q % 16 == 0;
        blocks += (g.M + 4 / wpr - 1) / (4 / wpr);
    }
    if (!one_launch || blocks > 0x7fffffff) {  // shapes without a grouped kernel: one launch per group, same results
        for (int i = 0; i < n_groups; ++i)
            if (int rc = i8f_quant_rowwise(groups[i].x, x_dtype, groups[i].M, K, groups[i].ldx, rotate_block, groups[i].q,
                                           groups[i].scale, stream))
                return rc;
        return I8F_OK;
    }
    if (blocks == 0) return I8F_OK;
    if (int rc = check_device()) return rc;
    GroupedArgs ga{};
    ga.n = n_groups;
    int at = 0;
    for (int i = 0; i < n_groups; ++i) {
        ga.x[i] = (const char *)groups[i].x, ga.q[i] = groups[i].q, ga.scale[i] = groups[i].scale;
        ga.M[i] = groups[i].M, ga.ldx_bytes[i] = groups[i].ldx * 2;
        ga.first_block[i] = at;
        at += (int)((groups[i].M + 4 / wpr - 1) / (4 / wpr));
    }
    ga.first_block[n_groups] = at;
    hipStream_t st = (hipStream_t)stream;
    const bool rot = rotate_block != 0;
    const int64_t nruns = K / 16;
    const int runs = wpr == 1 ? (int)((nruns + 63) / 64) : (int)((nruns + 255) / 256);
#define I8F_GROUPED(DT)                                                                                              \
    (wpr == 1 ? (rot ? pick_runs16_grouped<DT, true, 1>(runs, ga, K, st) : pick_runs16_grouped<DT, false, 1>(runs, ga, K, st)) \
              : (rot ? pick_runs16_grouped<DT, true, 4>(runs, ga, K, st) : pick_runs16_grouped<DT, false, 4>(runs, ga, K, st)))
    return x_dtype == I8F_BF16 ? I8F_GROUPED(I8F_BF16) : I8F_GROUPED(I8F_F16);
#undef I8F_GROUPED
}

extern "C" int i8f_quant_rowwise_prologue(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx, int prologue,
                                          const void *mod_scale, const void *mod_shift, int64_t rows_per_vec,
                                          int rotate_block, int8_t *q, float *scale, void *stream) {
    using namespace i8f;
    if (prologue == I8F_PRO_NONE) return i8f_quant_rowwise(x, x_dtype, M, K, ldx, rotate_block, q, scale, stream);
    const bool fused_add = prologue == I8F_PRO_MODULATE_FUSED;   // the modulation with torch.addcmul's single rounding
    if (fused_add) prologue = I8F_PRO_MODULATE;
    if (prologue != I8F_PRO_MODULATE && prologue != I8F_PRO_GELU_TANH && prologue != I8F_PRO_SILU_GATE && prologue != I8F_PRO_GELU_ERF)
        return I8F_ERR_INVALID;
    if (fused_add && x_dtype == I8F_F32) return I8F_ERR_UNSUPPORTED;   // (a binary32 product is not exact: torch's result depends on contraction)
    if (M < 0 || K < 0 || !valid_dtype(x_dtype)) return I8F_ERR_INVALID;
    if (rotate_block != 0 && rotate_block != 128) return I8F_ERR_UNSUPPORTED;
    if (rotate_block && K % rotate_block) return I8F_ERR_INVALID;
    if (M == 0) return I8F_OK;
    if (!scale || ldx < K) return I8F_ERR_INVALID;
    if (K > 0 && (!x || !q)) return I8F_ERR_INVALID;
    if (prologue == I8F_PRO_MODULATE && (rows_per_vec <= 0 || (K > 0 && (!mod_scale || !mod_shift)))) return I8F_ERR_INVALID;
    if (prologue == I8F_PRO_SILU_GATE && (rows_per_vec <= 0 || (K > 0 && !mod_scale))) return I8F_ERR_INVALID;
    if (M > 0x7fffffff) return I8F_ERR_UNSUPPORTED;
    if (int rc = check_device()) return rc;
    if (rows_per_vec > 0x7fffffff) rows_per_vec = 0x7fffffff;  // M itself is below 2^31
    Prologue pro{prologue, mod_scale, mod_shift, rows_per_vec > 0 ? rows_per_vec : 1, 0.0f};
    pro.fused_add = fused_add ? 1 : 0;
    hipStream_t st = (hipStream_t)stream;
    const bool rot = rotate_block != 0;
    switch (x_dtype) {
    case I8F_BF16: return dispatch_rot<I8F_BF16>(rot, x, M, K, ldx, q, scale, st, pro);
    case I8F_F16: return dispatch_rot<I8F_F16>(rot, x, M, K, ldx, q, scale, st, pro);
    default: return dispatch_rot<I8F_F32>(rot, x, M, K, ldx, q, scale, st, pro);
    }
}

extern "C" int i8f_quant_rowwise_norm_modulate(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx, float eps,
                                               const void *mod_scale, const void *mod_shift, int64_t rows_per_vec, int modulate_fused,
                                               int rotate_block, int8_t *q, float *scale, void *stream) {
    using namespace i8f;
    if (M < 0 || K < 0 || !valid_dtype(x_dtype) || !(eps >= 0.0f)) return I8F_ERR_INVALID;
    if (rotate_block != 0 && rotate_block != 128) return I8F_ERR_UNSUPPORTED;
    if (rotate_block && K % rotate_block) return I8F_ERR_INVALID;
    if (M == 0) return I8F_OK;
    if (!scale || ldx < K || K == 0 || !x || !q || rows_per_vec <= 0 || !mod_scale || !mod_shift) return I8F_ERR_INVALID;
    if (M > 0x7fffffff) return I8F_ERR_UNSUPPORTED;
    if (int rc = check_device()) return rc;
    if (rows_per_vec > 0x7fffffff) rows_per_vec = 0x7fffffff;
    Prologue pro{I8F_PRO_NORM_MODULATE, mod_scale, mod_shift, rows_per_vec, eps};
    pro.fused_add = modulate_fused ? 1 : 0;
    hipStream_t st = (hipStream_t)stream;
    const bool rot = rotate_block != 0;
    switch (x_dtype) {
    case I8F_BF16: return dispatch_rot<I8F_BF16>(rot, x, M, K, ldx, q, scale, st, pro);
    case I8F_F16: return dispatch_rot<I8F_F16>(rot, x, M, K, ldx, q, scale, st, pro);
    default: return I8F_ERR_UNSUPPORTED;
    }
}

extern "C" int i8f_quant_rowwise_rms_norm(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx, float eps, const void *weight,
                                          const void *mod_scale, const void *mod_shift, int64_t rows_per_vec, int modulate_fused,
                                          int rotate_block, int8_t *q, float *scale, void *stream) {
    using namespace i8f;
    if (M < 0 || K < 0 || !valid_dtype(x_dtype) || !(eps >= 0.0f)) return I8F_ERR_INVALID;
    if (rotate_block != 0 && rotate_block != 128) return I8F_ERR_UNSUPPORTED;
    if (rotate_block && K % rotate_block) return I8F_ERR_INVALID;
    if (M == 0) return I8F_OK;
    if (!scale || ldx < K || K == 0 || !x || !q) return I8F_ERR_INVALID;
    if ((mod_scale || mod_shift) && rows_per_vec <= 0) return I8F_ERR_INVALID;
    if (M > 0x7fffffff) return I8F_ERR_UNSUPPORTED;
    if (int rc = check_device()) return rc;
    if (rows_per_vec > 0x7fffffff || rows_per_vec <= 0) rows_per_vec = 0x7fffffff;
    Prologue pro{I8F_PRO_RMS_NORM, mod_scale, mod_shift, rows_per_vec, eps, nullptr, 0, 0, weight, modulate_fused ? 1 : 0};
    hipStream_t st = (hipStream_t)stream;
    const bool rot = rotate_block != 0;
    switch (x_dtype) {
    case I8F_BF16: return dispatch_rot<I8F_BF16>(rot, x, M, K, ldx, q, scale, st, pro);
    case I8F_F16: return dispatch_rot<I8F_F16>(rot, x, M, K, ldx, q, scale, st, pro);
    default: return I8F_ERR_UNSUPPORTED;
    }
}

extern "C" int i8f_quant_rowwise_concat_gelu(const void *a, int dtype, int64_t M, int64_t Ka, int64_t lda, const void *b, int64_t Kb,
                                             int64_t ldb, int rotate_block, int8_t *q, float *scale, void *stream) {
    using namespace i8f;
    if (M < 0 || Ka < 0 || Kb < 0 || !valid_dtype(dtype)) return I8F_ERR_INVALID;
    if (rotate_block != 0 && rotate_block != 128) return I8F_ERR_UNSUPPORTED;
    const int64_t K = Ka + Kb;
    if (rotate_block && (Ka % rotate_block || Kb % rotate_block)) return I8F_ERR_INVALID;
    if (M == 0) return I8F_OK;
    if (!scale || lda < Ka || ldb < Kb || K == 0 || !q || (Ka > 0 && !a) || (Kb > 0 && !b)) return I8F_ERR_INVALID;
    if (M > 0x7fffffff) return I8F_ERR_UNSUPPORTED;
    // both parts in whole runs of 16 elements with 16-byte aligned rows
    if (dtype == I8F_F32 || Ka % 16 || Kb % 16 || lda % 8 || ldb % 8 || K > 16 * 64 * 4 * 4) return I8F_ERR_UNSUPPORTED;
    if (int rc = check_device()) return rc;
    Prologue pro{I8F_PRO_CONCAT_GELU, nullptr, nullptr, 1, 0.0f, b, ldb * 2, (int)(Ka / 16)};
    // (a part without elements: its pointer is never read, the other one stands in so that alignment checks pass)
    const void *x = Ka > 0 ? a : b;
    if (Kb == 0) pro.b = a;
    hipStream_t st = (hipStream_t)stream;
    const bool rot = rotate_block != 0;
    return dtype == I8F_BF16 ? dispatch_rot<I8F_BF16>(rot, x, M, K, lda, q, scale, st, pro) : dispatch_rot<I8F_F16>(rot, x, M, K, lda, q, scale, st, pro);
}

extern "C" int i8f_rotate128(const void *x, int dtype, int64_t M, int64_t K, int64_t ldx, void *out, void *stream) {
    using namespace i8f;
    if (M < 0 || K < 0 || !valid_dtype(dtype) || K % 128) return I8F_ERR_INVALID;
    if (M == 0 || K == 0) return I8F_OK;
    if (!x || !out || ldx < K) return I8F_ERR_INVALID;
    if (x == out && ldx != K) return I8F_ERR_INVALID;
    if (M * (K / 4) / 256 > 0x7fffffffll) return I8F_ERR_UNSUPPORTED;
    if (int rc = check_device()) return rc;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
    case I8F_BF16: return launch_rotate<I8F_BF16>(x, M, K, ldx, out, st);
    case I8F_F16: return launch_rotate<I8F_F16>(x, M, K, ldx, out, st);
    default: return launch_rotate<I8F_F32>(x, M, K, ldx, out, st);
    }
}
