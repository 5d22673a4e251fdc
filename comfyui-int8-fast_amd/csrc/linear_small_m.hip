// Small-batch (M <= 16) W8A16 linear: bandwidth-bound stream over the int8
// weight, dequantised in registers; the activations are not quantised.
//
//   out[m,n] = round( sum_k x[m,k] * round(float(w[n,k]) * ws[n]) + round(bias[n]) )
//
// with round() = rounding to x's dtype, which is where the reference rounds
// (Linear.forward, int8_quant.py:756-760: the dequantised weight and the bias
// are cast to x.dtype before F.linear).  The reference writes the whole
// dequantised weight to memory and reads it back on every call; here the weight
// is read once as int8.  Two kernels: binary16/bfloat16 activations with
// 16-byte aligned rows go to the matrix cores (small_m_lds_kernel); anything
// else to small_m_kernel, where one wavefront owns one output column n (64 lanes
// x 16 weights per step, partial sums as fmaf chains in binary32, then a
// butterfly reduction across the wavefront).  The order of the binary32 sums
// differs between the two; the result is compared with a tolerance of one
// rounding step of the output type.
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

// ---- matrix-core variant (binary16 / bfloat16 activations, K % 16 == 0) ---------------------------
// The weight stream is the only traffic that counts (N*K bytes); the work per weight on the vector
// ALUs is what decides whether the stream runs at memory speed.  Here it is convert, scale, round
// (2.5 instructions per weight for bfloat16) and the multiply-adds go to v_mfma_f32_16x16x32: the
// dequantised weights of 16 output columns are the A operand, the (up to 16) activation rows the B
// operand, so the arithmetic costs the same for every M <= 16.  A wave owns NB blocks of 16 output
// columns and every WAVES-th 128-byte step along K.  Lane (r = lane % 16, g = lane / 16) feeds
// weight row r, bytes 32 j + 8 g .. + 8 of the step, to MFMA j = 0..3 and the activations of row r
// at the same k.  The
// WAVES partial sums meet in LDS and are added in wave order, so results do not depend on timing.
typedef float v4f_t __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));
typedef _Float16 v8h_t __attribute__((ext_vector_type(8)));

template <int DT>
__device__ __forceinline__ uint32_t dequant_pair(uint32_t word, int e, float ws) {
    const float a = (float)(int)(int8_t)(word >> (8 * e)) * ws;
    const float b = (float)(int)(int8_t)(word >> (8 * e + 8)) * ws;
    if constexpr (DT == I8F_BF16) return f32x2_to_bf16x2_bits(a, b);
    else return f32_to_f16_bits(a) | (f32_to_f16_bits(b) << 16);
}

template <int DT>
__device__ __forceinline__ v4f_t mma8(uint32_t wlo, uint32_t whi, v4u_t xk, float ws, v4f_t acc) {
    v4u_t a;
    a.x = dequant_pair<DT>(wlo, 0, ws);
    a.y = dequant_pair<DT>(wlo, 2, ws);
    a.z = dequant_pair<DT>(whi, 0, ws);
    a.w = dequant_pair<DT>(whi, 2, ws);
    if constexpr (DT == I8F_BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf_t, a), __builtin_bit_cast(v8bf_t, xk), acc, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h_t, a), __builtin_bit_cast(v8h_t, xk), acc, 0, 0, 0);
}

// The weight fetch is fully coalesced: a wave instruction reads 8 rows x 128 contiguous bytes
// (8 cache lines, adjacent lanes adjacent 16 bytes); the wave parks them in its own LDS tile and
// reads them back in the MFMA operand layout (8 bytes per lane and MFMA).  The tile is private to
// the wave, so no barrier is involved.  Fetching straight into the operand layout (16 rows per
// instruction, 16 or more cache lines) measured 12 % slower, and slower still the more lines an
// instruction touched.
// (The body is shared by the kernel of one layer and the kernel of several layers in one launch: `block` is the
// workgroup's number within its layer.)
template <int DT, int NB, int WAVES>
__device__ __forceinline__ void small_m_lds_body(const SmallMArgs &a, const int64_t block) {
    constexpr int COLS = NB * 16;
    constexpr int PITCH = 144;
    __shared__ float red[WAVES][COLS][16];
    __shared__ __attribute__((aligned(16))) char tiles[WAVES][COLS * PITCH];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int lr = lane >> 3, lc = lane & 7;   // fetch layout: row within 8, 16-byte column
    const int64_t n0 = block * COLS;
    const int K = (int)a.K;
    const int nsteps = (K + 127) / 128;
    const bool xrow = r < (int)a.M;
    const char *xp = (const char *)a.x + (int64_t)(xrow ? r : 0) * a.ldx * 2;
    char *tile = tiles[wave];

    const int8_t *frow[NB][2];
    float wsn[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            int64_t n = n0 + b * 16 + h * 8 + lr;
            n = n < a.N ? n : a.N - 1;
            frow[b][h] = a.w + n * a.K + lc * 16;
        }
        int64_t n = n0 + b * 16 + r;
        n = n < a.N ? n : a.N - 1;
        wsn[b] = a.ws ? a.ws[a.row_scale ? n : 0] : a.ws_host;
    }

    const v4u_t zero = {0u, 0u, 0u, 0u};
    v4u_t wq[2][NB][2], xq[2][4];
    auto fetch = [&](int t, int buf) __attribute__((always_inline)) {
        const int kw = t * 128;
        const bool wok = kw + lc * 16 + 16 <= K;
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int h = 0; h < 2; ++h) wq[buf][b][h] = wok ? *(const v4u_t *)(frow[b][h] + kw) : zero;
        // MFMA j takes k = kw + 32 j ... + 31, its lane group g the 8 values from 8 g on: the four groups of a row
        // read 64 contiguous bytes per instruction (with the groups 32 values apart every instruction touched twice
        // the cache lines, which is what M = 16 paid for: 21.7 -> 19.5 us at 18432 x 3072)
        const int k = kw + g * 8;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            xq[buf][j] = (xrow && k + 32 * j + 8 <= K) ? *(const v4u_t *)(xp + (int64_t)(k + 32 * j) * 2) : zero;
    };
    v4f_t acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[b] = v4f_t{0.f, 0.f, 0.f, 0.f};

    auto compute = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int h = 0; h < 2; ++h) *(v4u_t *)(tile + (b * 16 + h * 8 + lr) * PITCH + lc * 16) = wq[buf][b][h];
        // the tile is private to the wave, but a lane reads what other lanes wrote: fence the exchange
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        v2u_t wa[NB][4];
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int j = 0; j < 4; ++j) wa[b][j] = *(const v2u_t *)(tile + (b * 16 + r) * PITCH + j * 32 + 8 * g);
        __builtin_amdgcn_wave_barrier();  // every lane has its operands before the tile is overwritten
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[b] = mma8<DT>(wa[b][j].x, wa[b][j].y, xq[buf][j], wsn[b], acc[b]);
    };

    int t = wave;
    if (t < nsteps) fetch(t, 0);
    for (; t < nsteps; t += 2 * WAVES) {
        if (t + WAVES < nsteps) fetch(t + WAVES, 1);
        compute(0);
        if (t + WAVES < nsteps) {
            if (t + 2 * WAVES < nsteps) fetch(t + 2 * WAVES, 0);
            compute(1);
        }
    }

#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave][b * 16 + 4 * g + i][r] = acc[b][i];
    __syncthreads();
    for (int o = threadIdx.x; o < COLS * 16; o += WAVES * 64) {
        const int m = o / COLS, c = o % COLS;
        const int64_t n = n0 + c;
        if (m < (int)a.M && n < a.N) {
            float s = red[0][c][m];
#pragma unroll
            for (int w = 1; w < WAVES; ++w) s += red[w][c][m];
            float bv = 0.0f;
            if (a.bias) {
                if (a.bias_dtype == I8F_F32) bv = ((const float *)a.bias)[n];
                else if (a.bias_dtype == I8F_BF16) bv = bf16_bits_to_f32(((const uint16_t *)a.bias)[n]);
                else bv = f16_bits_to_f32(((const uint16_t *)a.bias)[n]);
                bv = round_to_dtype<DT>(bv);
            }
            store_from_f32<DT>(a.out, (int64_t)m * a.N + n, s + bv);
        }
    }
}

template <int DT, int NB, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void small_m_lds_kernel(const SmallMArgs a) {
    small_m_lds_body<DT, NB, WAVES>(a, (int64_t)blockIdx.x);
}

// Several layers in one launch (the modulation projections of the image and of the text stream of a double-stream
// block read the same conditioning vector through their own weights): a weight stream of 57 MB lasts 13 us, of which
// ramp-up and drain are a good part; two of them back to back in one grid keep the memory system busy through the seam.
constexpr int MAX_SMALL_M_GROUPS = 4;
struct SmallMGroups {
    SmallMArgs a[MAX_SMALL_M_GROUPS];
    int first_block[MAX_SMALL_M_GROUPS + 1];
    int n;
};

template <int DT, int NB, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void small_m_lds_grouped_kernel(const SmallMGroups gg) {
    int grp = 0;
#pragma unroll
    for (int i = 1; i < MAX_SMALL_M_GROUPS; ++i)
        if (i < gg.n && (int)blockIdx.x >= gg.first_block[i]) grp = i;
    // (selected with constant indices: the argument structure then stays in scalar registers)
    SmallMArgs a = gg.a[0];
#pragma unroll
    for (int i = 1; i < MAX_SMALL_M_GROUPS; ++i)
        if (grp == i) a = gg.a[i];
    small_m_lds_body<DT, NB, WAVES>(a, (int64_t)((int)blockIdx.x - gg.first_block[grp]));
}

template <int DT, int NB, int WAVES>
int launch_lds(const SmallMArgs &a, hipStream_t st) {
    const int64_t cols = NB * 16;
    hipLaunchKernelGGL((small_m_lds_kernel<DT, NB, WAVES>), dim3((unsigned)((a.N + cols - 1) / cols)), dim3(WAVES * 64), 0, st, a);
    return check_launch();
}

template <int DT>
int launch(const SmallMArgs &a, hipStream_t st) {
    const size_t es = dtype_size(DT);
    const bool vec = a.K % 16 == 0 && (uintptr_t)a.w % 16 == 0 && (uintptr_t)a.x % 16 == 0 && (a.ldx * es) % 16 == 0;
    if constexpr (DT != I8F_F32) {
        if (vec && a.K < (1ll << 30)) {
            // Workgroups of two 16-column blocks, unless that leaves CUs without one: then one block each, twice as
            // many workgroups (3072 x 12288: 192 instead of 96, 18.4 -> 13.1 us with the weight from HBM).  Beyond one
            // workgroup per CU the two-block form is the faster one at every size measured (it fetches the activations
            // once for both blocks).
            const int64_t blocks = (a.N + 15) / 16;
            // (Workgroups of 4 waves, which are all resident at once where 8-wave ones spill into a thin second round --
            // 18432 columns are 576 workgroups on 512 places -- measured no faster: 13.9 against 13.5 us.)
            if ((blocks + 1) / 2 < 256) return launch_lds<DT, 1, 8>(a, st);
            return launch_lds<DT, 2, 8>(a, st);
        }
    }
    dim3 grid((unsigned)((a.N + 3) / 4));
    if (vec) hipLaunchKernelGGL((small_m_kernel<DT, true>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((small_m_kernel<DT, false>), grid, dim3(256), 0, st, a);
    return check_launch();
}

// the layers of a group launch: all of them on the fast path, with the same block form
template <int DT>
int launch_grouped(const SmallMArgs *as, int n, hipStream_t st) {
    SmallMGroups gg{};
    gg.n = n;
    int64_t total_blocks16 = 0;
    for (int i = 0; i < n; ++i) total_blocks16 += (as[i].N + 15) / 16;
    const bool two = (total_blocks16 + 1) / 2 >= 256;     // as for one layer: two 16-column blocks per workgroup once every CU has one
    const int64_t cols = two ? 32 : 16;
    int64_t first = 0;
    for (int i = 0; i < n; ++i) {
        gg.a[i] = as[i];
        gg.first_block[i] = (int)first;
        first += (as[i].N + cols - 1) / cols;
    }
    for (int i = n; i <= MAX_SMALL_M_GROUPS; ++i) gg.first_block[i] = (int)first;
    if (first > 0x7fffffff) return I8F_ERR_UNSUPPORTED;
    if (two) hipLaunchKernelGGL((small_m_lds_grouped_kernel<DT, 2, 8>), dim3((unsigned)first), dim3(512), 0, st, gg);
    else hipLaunchKernelGGL((small_m_lds_grouped_kernel<DT, 1, 8>), dim3((unsigned)first), dim3(512), 0, st, gg);
    return check_launch();
}

}  // namespace
}  // namespace i8f

extern "C" int i8f_linear_w8a16_small_m_grouped(const i8f_small_m_group *groups, int n_groups, int x_dtype, int scale_mode,
                                                int bias_dtype, void *stream) {
    using namespace i8f;
    if (n_groups < 0 || (n_groups > 0 && !groups) || !valid_dtype(x_dtype)) return I8F_ERR_INVALID;
    if (scale_mode != I8F_SCALE_TENSOR && scale_mode != I8F_SCALE_ROW) return I8F_ERR_INVALID;
    bool one_launch = n_groups >= 2 && n_groups <= MAX_SMALL_M_GROUPS && x_dtype != I8F_F32;
    bool any_bias = false;
    for (int i = 0; i < n_groups; ++i) {
        const i8f_small_m_group &g = groups[i];
        if (g.M < 0 || g.N < 0 || g.K < 0) return I8F_ERR_INVALID;
        if (g.M > 16) return I8F_ERR_UNSUPPORTED;
        if (g.M > 0 && g.N > 0) {
            if (!g.out || g.ldx < g.K || (g.K > 0 && (!g.a || !g.w)) || (scale_mode == I8F_SCALE_ROW && !g.w_scale)) return I8F_ERR_INVALID;
        }
        any_bias = any_bias || g.bias;
        // what the fast kernel asks of a layer (as the single-layer entry point checks it)
        one_launch = one_launch && g.M > 0 && g.N > 0 && g.K % 16 == 0 && g.K > 0 && g.K < (1ll << 30) && (uintptr_t)g.w % 16 == 0 &&
                     (uintptr_t)g.a % 16 == 0 && (g.ldx * 2) % 16 == 0;
    }
    if (any_bias && !valid_dtype(bias_dtype)) return I8F_ERR_INVALID;
    if (!one_launch) {   // shapes without a grouped kernel: one launch per layer, same results
        for (int i = 0; i < n_groups; ++i) {
            const i8f_small_m_group &g = groups[i];
            if (int rc = i8f_linear_w8a16_small_m(g.a, x_dtype, g.M, g.K, g.ldx, g.w, g.w_scale, g.w_scale_host, scale_mode, g.bias,
                                                  bias_dtype, g.out, g.N, stream))
                return rc;
        }
        return I8F_OK;
    }
    if (int rc = check_device()) return rc;
    SmallMArgs as[MAX_SMALL_M_GROUPS];
    for (int i = 0; i < n_groups; ++i) {
        const i8f_small_m_group &g = groups[i];
        as[i] = SmallMArgs{};
        as[i].x = g.a, as[i].M = g.M, as[i].K = g.K, as[i].ldx = g.ldx, as[i].N = g.N, as[i].w = g.w, as[i].ws = g.w_scale;
        as[i].ws_host = g.w_scale_host, as[i].row_scale = scale_mode == I8F_SCALE_ROW, as[i].bias = g.bias, as[i].bias_dtype = bias_dtype;
        as[i].out = g.out;
    }
    hipStream_t st = (hipStream_t)stream;
    return x_dtype == I8F_BF16 ? launch_grouped<I8F_BF16>(as, n_groups, st) : launch_grouped<I8F_F16>(as, n_groups, st);
}

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
