/*
 * i8f_oracle.c -- CPU restatement of the W8A8 linear hot path of
 * ComfyUI-INT8-Fast, in plain C.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the
 * smoke check and the benchmark's "cpu_baseline" leg may load it, and only as
 * the checker the HIP library is compared against.  Nothing in the shipped
 * package links, imports or falls back to it.
 *
 * Every function names the lines of the reference it restates
 * (paths relative to the reference checkout).  The arithmetic is IEEE-754
 * binary32 with round-to-nearest-even and no contraction: build with
 * -ffp-contract=off and without -ffast-math (see the Makefile beside this
 * file).  The only fused multiply-add is the explicit fmaf() in
 * orc_lora_delta, where the fused definition is stated.
 *
 * Parity status of each function (what pins it is in tests/test_oracle_*.py):
 *   orc_quant_rowwise (no rotation)  pinned: torch CPU elementwise ops, closed
 *                                    forms, brute force in float64/fractions
 *   orc_quant_rowwise (rotation)     pinned up to summation order: dense
 *                                    product with scipy.linalg.hadamard, WHT
 *                                    invariants.  The reference's own rotation
 *                                    is a dense BLAS matmul whose summation
 *                                    order is unspecified, so bit-for-bit the
 *                                    target is THIS fixed butterfly order
 *   orc_gemm_i32                     pinned: torch._int_mm on CPU, int64 matmul
 *   orc_epilogue (torch order)       pinned: torch CPU elementwise ops
 *   orc_epilogue (fused order)       pinned: float64 closed form within 1 ulp
 *   orc_linear_w8a16                 pinned within tolerance: torch F.linear
 *   orc_sr_delta / orc_merge_i8      pinned: torch CPU elementwise ops, special
 *                                    cases (noise 0, noise -> 1, frac 0)
 *   orc_lora_delta                   pinned within tolerance: torch.mm (the
 *                                    reference's product has no fixed order)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_BF16 0
#define ORC_F16 1
#define ORC_F32 2

#define ORC_SCALE_TENSOR 0
#define ORC_SCALE_ROW 1

#define ORC_EPI_TORCH 0 /* order of int8_quant.py:84-87 / 115-118 */
#define ORC_EPI_FUSED 1 /* order of int8_fused_kernel.py:156-173 / 310-324 */

/* ------------------------------------------------------------------------- */
/* storage-format conversions                                                */
/* ------------------------------------------------------------------------- */

static inline float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

float orc_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* round-to-nearest-even, NaN -> quiet NaN (what torch's .to(bfloat16) does) */
uint16_t orc_f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0x1f) return bits_f32(sign | 0x7f800000u | (man << 13));
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal half: man * 2^-24, exact in binary32 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* round-to-nearest-even binary32 -> binary16 */
uint16_t orc_f32_to_f16(float f) {
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 -> inf */
    if (a < 0x38800000u) { /* below the smallest normal half: result is subnormal or 0 */
        /* value * 2^24 rounded to an integer with ties-to-even is the mantissa */
        float scaled = bits_f32(a) * 16777216.0f; /* exact scaling */
        float r = nearbyintf(scaled);
        return (uint16_t)(sign | (uint16_t)r);
    }
    uint32_t m = a - 0x38000000u; /* rebias exponent 127 -> 15 */
    m += 0xfffu + ((m >> 13) & 1u);
    return (uint16_t)(sign | (uint16_t)(m >> 13));
}

static inline float load_as_f32(const void *p, int dtype, size_t i) {
    switch (dtype) {
    case ORC_BF16: return orc_bf16_to_f32(((const uint16_t *)p)[i]);
    case ORC_F16: return orc_f16_to_f32(((const uint16_t *)p)[i]);
    default: return ((const float *)p)[i];
    }
}

/* value rounded to the storage dtype, returned as binary32 */
static inline float round_to_dtype(float v, int dtype) {
    switch (dtype) {
    case ORC_BF16: return orc_bf16_to_f32(orc_f32_to_bf16(v));
    case ORC_F16: return orc_f16_to_f32(orc_f32_to_f16(v));
    default: return v;
    }
}

static inline void store_from_f32(void *p, int dtype, size_t i, float v) {
    switch (dtype) {
    case ORC_BF16: ((uint16_t *)p)[i] = orc_f32_to_bf16(v); break;
    case ORC_F16: ((uint16_t *)p)[i] = orc_f32_to_f16(v); break;
    default: ((float *)p)[i] = v; break;
    }
}

/* ------------------------------------------------------------------------- */
/* QuaRot block rotation                                                     */
/* ------------------------------------------------------------------------- */

/*
 * The entry of the normalised 128-point Hadamard matrix in each dtype, as the
 * reference builds it: quarot.py:35-36 makes a +-1 tensor in `dtype` and divides
 * it by the Python float 128**0.5, so the entry is 1/sqrt(128) rounded to that
 * dtype: 0x3DB504F3 in binary32, 0x3DB5 in bfloat16, 0x2DA8 in binary16 (both
 * of the latter equal 0.08837890625 = 181/2048).
 */
float orc_hadamard_entry(int dtype) {
    if (dtype == ORC_F32) return bits_f32(0x3DB504F3u);
    return 0.08837890625f;
}

/*
 * In-place unnormalised Walsh-Hadamard transform of one block of n = 2^p
 * binary32 values in Sylvester (natural) order, i.e. v <- v @ H_n with
 * H_n[k][j] = (-1)^popcount(k&j), the matrix scipy.linalg.hadamard(n) returns
 * (quarot.py:35).  The summation order is FIXED: stages with stride 1, 2, 4,
 * ..., n/2; in each stage every pair (lo, hi = lo + stride) becomes
 * (lo + hi, lo - hi), each a single rounded binary32 operation.
 */
void orc_fwht_f32(float *v, int n) {
    for (int stride = 1; stride < n; stride <<= 1) {
        for (int base = 0; base < n; base += 2 * stride) {
            for (int j = base; j < base + stride; ++j) {
                float lo = v[j], hi = v[j + stride];
                v[j] = lo + hi;
                v[j + stride] = lo - hi;
            }
        }
    }
}

/*
 * rotate_activation (quarot.py:73-102, called at int8_quant.py:741-744) and
 * rotate_weight (quarot.py:42-70, called at int8_quant.py:602-607), both with
 * group_size 128: every aligned block of `block` consecutive elements of a row
 * is multiplied by the normalised Hadamard matrix of `dtype`, and the result
 * is returned in `dtype` (torch.matmul of two `dtype` tensors).  H is
 * symmetric, so "@ H" (activations) and "@ H.T" (weights) are the same map.
 *
 * Restated as: widen to binary32, fixed-order butterfly (orc_fwht_f32), one
 * multiply by the dtype's Hadamard entry, one rounding to `dtype`.
 * `row` holds K binary32 values and is overwritten with the rotated row, each
 * value already rounded to `dtype` (and widened again).
 */
void orc_rotate_row(float *row, int64_t K, int dtype, int block) {
    const float h = orc_hadamard_entry(dtype);
    for (int64_t b = 0; b + block <= K; b += block) {
        orc_fwht_f32(row + b, block);
        for (int j = 0; j < block; ++j) row[b + j] = round_to_dtype(row[b + j] * h, dtype);
    }
}

/* ------------------------------------------------------------------------- */
/* a1/a3/a4: (optional rotation +) per-row absmax int8 quantisation          */
/* ------------------------------------------------------------------------- */

/*
 * quantize_int8_axiswise(x, dim=-1) -> quantize_int8 (int8_quant.py:28-31 and
 * :20-21), preceded by the block rotation when rotate_block != 0.
 *
 *   amax  = max_k |x[m,k]|                      (exact, taken in x's dtype)
 *   scale = max(float(amax) / 127.0f, 1e-30f)   (true binary32 division)
 *   inv   = 1.0f / scale                        ("1.0 / scale" on a tensor is
 *                                                reciprocal(scale) * 1.0)
 *   q     = int8(clamp(rint(float(x) * inv), -128, 127))   (ties to even)
 *
 * x is M rows of K elements, row stride ldx elements, dtype ORC_BF16/F16/F32.
 * q is [M,K] int8 contiguous, scale is [M] binary32 (the reference's [M,1]).
 * rotate_block must be 0 or a power of two that divides K.
 * Returns 0, or -1 for a bad argument.
 */
int orc_quant_rowwise(const void *x, int dtype, int64_t M, int64_t K, int64_t ldx,
                      int rotate_block, int8_t *q, float *scale) {
    if (M < 0 || K < 0 || ldx < K) return -1;
    if (rotate_block != 0 &&
        (rotate_block < 2 || (rotate_block & (rotate_block - 1)) || K % rotate_block))
        return -1;
    int rc = 0;
#pragma omp parallel
    {
        float *row = (float *)malloc((size_t)(K > 0 ? K : 1) * sizeof(float));
#pragma omp for schedule(static)
        for (int64_t m = 0; m < M; ++m) {
            if (!row) { rc = -1; continue; }
            for (int64_t k = 0; k < K; ++k) row[k] = load_as_f32(x, dtype, (size_t)(m * ldx + k));
            if (rotate_block) orc_rotate_row(row, K, dtype, rotate_block);
            float amax = 0.0f;
            for (int64_t k = 0; k < K; ++k) {
                float a = fabsf(row[k]);
                if (a > amax) amax = a;
            }
            float s = amax / 127.0f;
            if (s < 1e-30f) s = 1e-30f;
            const float inv = 1.0f / s;
            for (int64_t k = 0; k < K; ++k) {
                float r = nearbyintf(row[k] * inv);
                if (r < -128.0f) r = -128.0f;
                if (r > 127.0f) r = 127.0f;
                q[m * K + k] = (int8_t)r;
            }
            scale[m] = s;
        }
        free(row);
    }
    return rc;
}

/*
 * The elementwise operation a model applies in front of a quantised linear, which
 * the reference's torch.compile path fuses into its quantiser (README.md:4,56;
 * the Triton quantiser int8_fused_kernel.py:10-53 is traceable).  Restated as
 * torch's eager kernels evaluate it on a tensor of `dtype`:
 *   kind 1  (1 + s[k]) * x + t[k]: three tensor operations, each computed in
 *           binary32 and rounded to dtype; s, t are [ceil(M / rows_per_vec), K],
 *           row m uses vector m / rows_per_vec
 *   kind 2  gelu(x, approximate="tanh") = 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))
 *           in binary32, rounded once to dtype (the tanh is the C library's: a
 *           tolerance reference in the last binary32 bits, not a bit pattern)
 *   kind 3  silu(x) * g[k]: x / (1 + exp(-x)) in binary32 rounded to dtype, then the
 *           product rounded to dtype (torch's silu and mul kernels; the gated activation of a
 *           SwiGLU feed-forward, e.g. the z-image family the loader names,
 *           int8_unet_loader.py:60-93); g is s, laid out like s of kind 1; expf is the C
 *           library's: a tolerance reference like kind 2
 *   kind 6  gelu(x) in its exact form, x * 0.5 * (1 + erf(x / sqrt 2)) in binary32 as torch's kernel writes it,
 *           rounded once to dtype (erff is the C library's: a tolerance reference)
 *   kind 8  torch.addcmul(t, x, 1 + s): the gain 1 + s rounded to dtype (a tensor of its own), then t + x * gain in
 *           binary32 (the product of two 16-bit values is exact there) rounded once to dtype
 * out is [M,K] of dtype, contiguous.  Followed by orc_quant_rowwise it is the
 * oracle of the fused quantiser.
 */
int orc_prologue(const void *x, int dtype, int64_t M, int64_t K, int64_t ldx, int kind,
                 const void *s, const void *t, int64_t rows_per_vec, void *out) {
    if (M < 0 || K < 0 || ldx < K || (kind != 1 && kind != 2 && kind != 3 && kind != 6 && kind != 8)) return -1;
    if ((kind == 1 || kind == 8) && (rows_per_vec <= 0 || !s || !t)) return -1;
    if (kind == 3 && (rows_per_vec <= 0 || !s)) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t k = 0; k < K; ++k) {
            const float xv = load_as_f32(x, dtype, (size_t)(m * ldx + k));
            float v;
            if (kind == 1 || kind == 8) {
                const size_t vi = (size_t)((m / rows_per_vec) * K + k);
                const float a = round_to_dtype(1.0f + load_as_f32(s, dtype, vi), dtype);
                const float p = a * xv;
                const float b = kind == 8 ? p : round_to_dtype(p, dtype);
                v = b + load_as_f32(t, dtype, vi);
            } else if (kind == 3) {
                /* silu(x) * g as two tensor operations: x / (1 + exp(-x)) in binary32, rounded to the dtype, then
                 * the product with the gate value, rounded again by the store below */
                const size_t vi = (size_t)((m / rows_per_vec) * K + k);
                const float a = round_to_dtype(xv / (1.0f + expf(-xv)), dtype);
                v = a * load_as_f32(s, dtype, vi);
            } else if (kind == 6) {
                v = xv * 0.5f * (1.0f + erff(xv * 0.70710678118654752440f));
            } else {
                const float kBeta = 0.7978845608028654f, kKappa = 0.044715f;
                const float x3 = xv * xv * xv;
                const float inner = kBeta * (xv + kKappa * x3);
                v = 0.5f * xv * (1.0f + tanhf(inner));
            }
            store_from_f32(out, dtype, (size_t)(m * K + k), v);
        }
    }
    return 0;
}

/*
 * RMSNorm, optionally followed by the modulation (the model's own torch operations in front of
 * Linear.forward, int8_quant.py:703, in the families the loader names that normalise with an RMSNorm,
 * int8_unet_loader.py:60-93):
 *   y = round(x * rstd * w),  rstd = 1 / sqrt(sum x^2 / K + eps)     (torch's rms_norm: binary32, one rounding; w optional)
 *   z = round(round(1 + s) * y)   if s,   z = round(z + t)   if t
 * The row's sum is taken in double (torch takes it in binary32 in its own order).
 */
int orc_rms_norm(const void *x, int dtype, int64_t M, int64_t K, int64_t ldx, float eps, const void *w,
                 const void *s, const void *t, int64_t rows_per_vec, int fused, void *out) {
    if (M < 0 || K <= 0 || ldx < K || ((s || t) && rows_per_vec <= 0)) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        double ss = 0.0;
        for (int64_t k = 0; k < K; ++k) {
            const double d = (double)load_as_f32(x, dtype, (size_t)(m * ldx + k));
            ss += d * d;
        }
        const float rstd = 1.0f / sqrtf((float)(ss / (double)K) + eps);
        for (int64_t k = 0; k < K; ++k) {
            const size_t vi = (s || t) ? (size_t)((m / rows_per_vec) * K + k) : 0;
            float y = load_as_f32(x, dtype, (size_t)(m * ldx + k)) * rstd;
            if (w) y = y * load_as_f32(w, dtype, (size_t)k);
            y = round_to_dtype(y, dtype);
            if (s) {
                y = round_to_dtype(1.0f + load_as_f32(s, dtype, vi), dtype) * y;
                if (!(fused && t)) y = round_to_dtype(y, dtype);   /* fused with a shift: torch.addcmul(t, y, 1 + s) */
            }
            if (t) y = y + load_as_f32(t, dtype, vi);
            store_from_f32(out, dtype, (size_t)(m * K + k), y);
        }
    }
    return 0;
}

/*
 * LayerNorm without affine parameters followed by the adaLN modulation, the producer of a DiT block's
 * qkv and MLP inputs (the model's own torch operations in front of Linear.forward, int8_quant.py:703):
 *   y = round((x - mean) * rstd),  mean = sum x / K,  rstd = 1 / sqrt(sum (x - mean)^2 / K + eps)
 *   z = round(round(round(1 + s) * y) + t)
 * The row's sums are taken in double (torch's kernels take them in binary32 in their own order; the
 * difference is far below a unit in the last place of a 16-bit dtype except at rounding boundaries),
 * mean and rstd are then binary32 values and the elementwise part runs in binary32 as torch's does.
 */
int orc_norm_modulate(const void *x, int dtype, int64_t M, int64_t K, int64_t ldx, float eps,
                      const void *s, const void *t, int64_t rows_per_vec, int fused, void *out) {
    if (M < 0 || K <= 0 || ldx < K || rows_per_vec <= 0 || !s || !t) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        double sum = 0.0, ss = 0.0;
        for (int64_t k = 0; k < K; ++k) sum += (double)load_as_f32(x, dtype, (size_t)(m * ldx + k));
        const float mean = (float)(sum / (double)K);
        for (int64_t k = 0; k < K; ++k) {
            const double d = (double)(load_as_f32(x, dtype, (size_t)(m * ldx + k)) - mean);
            ss += d * d;
        }
        const float var = (float)(ss / (double)K);
        const float rstd = 1.0f / sqrtf(var + eps);
        for (int64_t k = 0; k < K; ++k) {
            const size_t vi = (size_t)((m / rows_per_vec) * K + k);
            const float y = round_to_dtype((load_as_f32(x, dtype, (size_t)(m * ldx + k)) - mean) * rstd, dtype);
            const float a = round_to_dtype(1.0f + load_as_f32(s, dtype, vi), dtype);
            const float b = fused ? a * y : round_to_dtype(a * y, dtype);   /* fused: torch.addcmul(t, y, 1 + s), one rounding */
            store_from_f32(out, dtype, (size_t)(m * K + k), b + load_as_f32(t, dtype, vi));
        }
    }
    return 0;
}

/*
 * quantize_int8_tensorwise (int8_quant.py:23-26): one scale for the whole
 * tensor.  Used to prepare the tensorwise weights of BASELINE config 0.
 */
int orc_quant_tensorwise(const void *x, int dtype, int64_t n, int8_t *q, float *scale) {
    float amax = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
        float a = fabsf(load_as_f32(x, dtype, (size_t)i));
        if (a > amax) amax = a;
    }
    float s = amax / 127.0f;
    if (s < 1e-30f) s = 1e-30f;
    const float inv = 1.0f / s;
    for (int64_t i = 0; i < n; ++i) {
        float r = nearbyintf(load_as_f32(x, dtype, (size_t)i) * inv);
        if (r < -128.0f) r = -128.0f;
        if (r > 127.0f) r = 127.0f;
        q[i] = (int8_t)r;
    }
    *scale = s;
    return 0;
}

/* ------------------------------------------------------------------------- */
/* a5: int8 x int8 -> int32 "NT" product                                     */
/* ------------------------------------------------------------------------- */

/*
 * torch._int_mm(x8, weight.T) (int8_quant.py:80,110) and the tl.dot K-loop
 * (int8_fused_kernel.py:132-144): acc[m,n] = sum_k a[m,k] * w[n,k], exact in
 * int32 for K <= 131072.  a is [M,K], w is [N,K], both row-major int8.
 */
__attribute__((target_clones("arch=skylake-avx512", "avx2", "default")))
static void gemm_rows(const int8_t *a, const int8_t *w, int64_t m0, int64_t m1, int64_t N,
                      int64_t K, int32_t *acc) {
    for (int64_t m = m0; m < m1; ++m) {
        const int8_t *am = a + m * K;
        for (int64_t n = 0; n < N; ++n) {
            const int8_t *wn = w + n * K;
            int32_t s = 0;
            for (int64_t k = 0; k < K; ++k) s += (int32_t)am[k] * (int32_t)wn[k];
            acc[m * N + n] = s;
        }
    }
}

int orc_gemm_i32(const int8_t *a, const int8_t *w, int64_t M, int64_t N, int64_t K,
                 int32_t *acc) {
    if (M < 0 || N < 0 || K < 0) return -1;
    const int64_t RB = 8; /* rows per task: keeps a block of `a` in L1 while streaming w */
    const int64_t nblk = (M + RB - 1) / RB;
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t b = 0; b < nblk; ++b) {
        int64_t m0 = b * RB, m1 = m0 + RB < M ? m0 + RB : M;
        gemm_rows(a, w, m0, m1, N, K, acc);
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* a6/a7: dequantisation epilogue                                            */
/* ------------------------------------------------------------------------- */

/*
 * ORC_EPI_TORCH, the order of the torch path that BASELINE config 0 names:
 *   tensorwise (int8_quant.py:84-87):
 *       t = out_dtype( float(acc) * (float(ws) * xs[m]) )
 *   per-row   (int8_quant.py:115-118):
 *       t = out_dtype( (float(acc) * xs[m]) * ws[n] )
 *   then, with a bias:  y = out_dtype( float(t) + float(out_dtype(bias[n])) )
 *   (the sum of two out_dtype tensors is formed in binary32 and rounded once).
 *
 * ORC_EPI_FUSED, the order of the fused kernels
 * (int8_fused_kernel.py:156-173 and :310-324): one rounding at the store,
 *       y = out_dtype( float(acc) * (xs[m] * ws[n or 0]) + float(bias[n]) )
 *   with the product and the sum rounded separately in binary32 (no fma).
 *
 * acc [M,N] int32; xs [M]; ws [1] (ORC_SCALE_TENSOR) or [N] (ORC_SCALE_ROW);
 * bias NULL or [N] of bias_dtype; out [M,N] of out_dtype (ORC_F32 is allowed
 * for out_dtype as a debugging aid: the roundings to out_dtype are identities).
 */
int orc_epilogue(const int32_t *acc, const float *xs, const float *ws, int scale_mode,
                 const void *bias, int bias_dtype, void *out, int out_dtype, int64_t M,
                 int64_t N, int order) {
    if (M < 0 || N < 0) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        const float xsm = xs[m];
        for (int64_t n = 0; n < N; ++n) {
            const float a = (float)acc[m * N + n];
            const float wsn = scale_mode == ORC_SCALE_ROW ? ws[n] : ws[0];
            float y;
            if (order == ORC_EPI_TORCH) {
                float t;
                if (scale_mode == ORC_SCALE_ROW) {
                    t = a * xsm;
                    t = t * wsn;
                } else {
                    float sc = wsn * xsm;
                    t = a * sc;
                }
                y = round_to_dtype(t, out_dtype);
                if (bias) {
                    float b = round_to_dtype(load_as_f32(bias, bias_dtype, (size_t)n), out_dtype);
                    y = y + b;
                }
            } else {
                float sc = xsm * wsn;
                y = a * sc;
                if (bias) y = y + load_as_f32(bias, bias_dtype, (size_t)n);
            }
            store_from_f32(out, out_dtype, (size_t)(m * N + n), y);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* whole W8A8 linear (what the CPU baseline times)                            */
/* ------------------------------------------------------------------------- */

/*
 * int8_forward_dynamic / int8_forward_dynamic_per_row, torch path
 * (int8_quant.py:75-88, 106-119), preceded by the online rotation of
 * Linear.forward (int8_quant.py:741-744) when rotate_block != 0.
 * Scratch (q, xs, acc) is allocated here; returns -2 if that fails.
 */
int orc_linear_w8a8(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                    int rotate_block, const int8_t *w, const float *ws, int scale_mode,
                    const void *bias, int bias_dtype, void *out, int out_dtype, int64_t N,
                    int order) {
    int8_t *q = (int8_t *)malloc((size_t)(M * K > 0 ? M * K : 1));
    float *xs = (float *)malloc((size_t)(M > 0 ? M : 1) * sizeof(float));
    int32_t *acc = (int32_t *)malloc((size_t)(M * N > 0 ? M * N : 1) * sizeof(int32_t));
    int rc = -2;
    if (q && xs && acc) {
        rc = orc_quant_rowwise(x, x_dtype, M, K, ldx, rotate_block, q, xs);
        if (!rc) rc = orc_gemm_i32(q, w, M, N, K, acc);
        if (!rc) rc = orc_epilogue(acc, xs, ws, scale_mode, bias, bias_dtype, out, out_dtype, M, N, order);
    }
    free(q);
    free(xs);
    free(acc);
    return rc;
}

/*
 * The gated residual behind a linear layer of an adaLN-Zero block, x + gate * y, as torch's two tensor
 * operations compute it on tensors of one dtype (the model's own operations behind Linear.forward,
 * int8_quant.py:703-778):  out = round(residual + round(gate[m / rows_per_gate, n] * y[m, n])).
 * y, gate, residual and out are stored in `dtype`; gate or residual may be NULL (that operation is left out).
 */
int orc_gate_residual(const void *y, int dtype, int64_t M, int64_t N, const void *gate, int64_t rows_per_gate,
                      const void *residual, void *out) {
    if (M < 0 || N < 0 || (gate && rows_per_gate <= 0)) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t n = 0; n < N; ++n) {
            float t = load_as_f32(y, dtype, (size_t)(m * N + n));
            if (gate) t = round_to_dtype(t * load_as_f32(gate, dtype, (size_t)((m / rows_per_gate) * N + n)), dtype);
            if (residual) t = t + load_as_f32(residual, dtype, (size_t)(m * N + n));
            store_from_f32(out, dtype, (size_t)(m * N + n), t);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* a8: small-M (M <= 16) W8A16 path                                          */
/* ------------------------------------------------------------------------- */

/*
 * Linear.forward, rows <= 16 (int8_quant.py:756-760):
 *   w_float = (float(w) * ws).to(x.dtype);  y = F.linear(x, w_float, bias.to(x.dtype))
 * The activations are NOT quantised.  F.linear's summation order is the BLAS
 * library's, so this restatement is a tolerance reference, not a bit pattern:
 * it accumulates the products of the dtype-rounded operands in binary64, adds
 * the dtype-rounded bias and rounds once to x's dtype.
 */
int orc_linear_w8a16(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                     const int8_t *w, const float *ws, int scale_mode, const void *bias,
                     int bias_dtype, void *out, int64_t N) {
    if (M < 0 || N < 0 || K < 0) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const float wsn = scale_mode == ORC_SCALE_ROW ? ws[n] : ws[0];
        for (int64_t m = 0; m < M; ++m) {
            double s = 0.0;
            for (int64_t k = 0; k < K; ++k) {
                float wf = round_to_dtype((float)w[n * K + k] * wsn, x_dtype);
                s += (double)load_as_f32(x, x_dtype, (size_t)(m * ldx + k)) * (double)wf;
            }
            if (bias) s += (double)round_to_dtype(load_as_f32(bias, bias_dtype, (size_t)n), x_dtype);
            store_from_f32(out, x_dtype, (size_t)(m * N + n), (float)s);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* a9/a10/a11: stochastic-rounding LoRA merge                                */
/* ------------------------------------------------------------------------- */

/*
 * stochastic_round_int8_delta (int8_quant.py:36-62) with the uniform noise
 * SUPPLIED by the caller instead of drawn from a device generator:
 *   xs = x / scale (true binary32 division; scale is one value or one per row)
 *   f = floor(xs); frac = xs - f; r = noise
 *   dq = int8(clamp(r < frac ? f + 1 : f, -128, 127))
 * x, noise [N,K] binary32; scale [1] or [N]; dq [N,K] int8.
 */
int orc_sr_delta(const float *x, const float *scale, int scale_mode, const float *noise,
                 int64_t N, int64_t K, int8_t *dq) {
    if (N < 0 || K < 0) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const float sc = scale_mode == ORC_SCALE_ROW ? scale[n] : scale[0];
        for (int64_t k = 0; k < K; ++k) {
            float xs = x[n * K + k] / sc;
            float f = floorf(xs);
            float frac = xs - f;
            float r = noise[n * K + k] < frac ? f + 1.0f : f;
            if (r < -128.0f) r = -128.0f;
            if (r > 127.0f) r = 127.0f;
            dq[n * K + k] = (int8_t)r;
        }
    }
    return 0;
}

/*
 * Check of an arithmetic identity that the HIP quantiser for 16-bit inputs relies on (no counterpart in the reference,
 * which divides, int8_quant.py:21,29): with y = 1/127 correctly rounded, q = a*y followed by ONE correction
 * fma(fma(-127, q, a), y, q), clamped below at 1e-30, equals max(a / 127, 1e-30).  Returns how many of the n values
 * disagree (bit patterns compared) and stores the index of the first in *first_bad.
 */
int64_t orc_scale_by_127_mismatches(const float *a, int64_t n, int64_t *first_bad) {
    int64_t bad = 0;
    const float y = 1.0f / 127.0f;
    for (int64_t i = 0; i < n; ++i) {
        float q = a[i] * y;
        const float r = fmaf(-127.0f, q, a[i]);
        q = fmaf(r, y, q);
        if (q < 1e-30f) q = 1e-30f;
        float t = a[i] / 127.0f;
        if (t < 1e-30f) t = 1e-30f;
        if (memcmp(&q, &t, 4) != 0) {
            if (bad == 0 && first_bad) *first_bad = i;
            ++bad;
        }
    }
    return bad;
}

/*
 * Check of an arithmetic identity that the HIP merge kernels rely on (no counterpart in the reference, which
 * divides): with y = 1/b correctly rounded, q = a*y followed by two corrections q = fma(fma(-b, q, a), y, q)
 * is the correctly rounded a/b as long as nothing over- or underflows.  Returns how many of the n pairs
 * disagree with the division (bit patterns compared) and stores the index of the first in *first_bad.
 */
int64_t orc_quotient_by_reciprocal_mismatches(const float *a, const float *b, int64_t n, int64_t *first_bad) {
    int64_t bad = 0;
    for (int64_t i = 0; i < n; ++i) {
        const float y = 1.0f / b[i];
        float q = a[i] * y;
        float r = fmaf(-b[i], q, a[i]);
        q = fmaf(r, y, q);
        r = fmaf(-b[i], q, a[i]);
        q = fmaf(r, y, q);
        const float t = a[i] / b[i];
        if (memcmp(&q, &t, 4) != 0) {
            if (bad == 0 && first_bad) *first_bad = i;
            ++bad;
        }
    }
    return bad;
}

/*
 * int8-space merge (int8_quant.py:313-316 and :399-402):
 *   w' = int8(clamp(int32(w) + int32(dq), -128, 127))
 */
int orc_merge_i8(const int8_t *w, const int8_t *dq, int64_t n, int8_t *out) {
    for (int64_t i = 0; i < n; ++i) {
        int32_t s = (int32_t)w[i] + (int32_t)dq[i];
        if (s < -128) s = -128;
        if (s > 127) s = 127;
        out[i] = (int8_t)s;
    }
    return 0;
}

/*
 * Plain LoRA delta (reconstruct_lora_diff case 1, int8_quant.py:143-157, and
 * the scaling at :295):  delta_f = (up @ down) * scale, up [N,r], down [r,K].
 * The reference's product is torch.mm, whose order is unspecified; the fused
 * merge kernel and this restatement fix it as
 *   acc = 0;  for j in 0..r-1: acc = fmaf(up[n,j], down[j,k], acc)
 *   delta_f[n,k] = acc * scale
 */
int orc_lora_delta(const float *up, const float *down, int64_t N, int64_t K, int64_t r,
                   float scale, float *delta) {
    if (N < 0 || K < 0 || r < 0) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        for (int64_t k = 0; k < K; ++k) {
            float acc = 0.0f;
            for (int64_t j = 0; j < r; ++j) acc = fmaf(up[n * r + j], down[j * K + k], acc);
            delta[n * K + k] = acc * scale;
        }
    }
    return 0;
}

/*
 * calculate_weight, int8 branch (int8_quant.py:293-318) from delta_f onward:
 * stochastic rounding of the delta with the layer's weight scale, then the
 * saturating int8 add.  delta NULL means "build it from up/down" with
 * orc_lora_delta.
 */
int orc_lora_merge_sr(const int8_t *w, const float *w_scale, int scale_mode, const float *delta,
                      const float *up, const float *down, int64_t r, float lora_scale,
                      const float *noise, int64_t N, int64_t K, int8_t *out) {
    float *tmp = NULL;
    if (!delta) {
        tmp = (float *)malloc((size_t)(N * K > 0 ? N * K : 1) * sizeof(float));
        if (!tmp) return -2;
        orc_lora_delta(up, down, N, K, r, lora_scale, tmp);
        delta = tmp;
    }
    int8_t *dq = (int8_t *)malloc((size_t)(N * K > 0 ? N * K : 1));
    int rc = -2;
    if (dq) {
        rc = orc_sr_delta(delta, w_scale, scale_mode, noise, N, K, dq);
        if (!rc) rc = orc_merge_i8(w, dq, N * K, out);
    }
    free(dq);
    free(tmp);
    return rc;
}

void orc_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

int orc_num_threads(void) {
    int n = 1;
#ifdef _OPENMP
#pragma omp parallel
    {
#pragma omp master
        n = omp_get_num_threads();
    }
#endif
    return n;
}
