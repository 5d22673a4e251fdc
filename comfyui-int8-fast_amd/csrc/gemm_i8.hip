// int8 x int8 -> int32 "NT" GEMM on the gfx950 matrix cores with the
// dequantisation epilogue fused in registers.
//
//   acc[m,n] = sum_k X[m,k] * W[n,k]         X [M,K] int8, W [N,K] int8 (K contiguous)
//   out[m,n] = epilogue(acc, xs[m], ws[n], bias[n])
//
// Structure of one workgroup (a BM x BN tile of the output):
//   * global -> LDS with buffer_load_dwordx4 ... lds (16 bytes per lane, no
//     VGPR round trip), STAGES tiles of BK bytes in flight; rows and K-tails
//     outside the matrices are zero-filled by the buffer bounds check.
//   * LDS rows keep the K-contiguous layout of the operands; the 16-byte chunk
//     index is XOR-swizzled with the row so that the 32 lanes reading one K
//     chunk of 32 different rows hit different banks.
//   * v_mfma_i32_32x32x32_i8, W fragments as the A operand and X fragments as
//     the B operand, so that a lane ends up with 4 consecutive n of one m:
//     integer sums do not depend on the order of k, so any k permutation that
//     is the same for both operands is allowed and none has to be undone.
//   * epilogue: scale/bias/round in registers, then a per-wave transpose
//     through LDS so that every global store is 16 bytes per lane and covers
//     whole 128-byte lines.
//   * workgroup id -> tile: consecutive ids go to different XCDs (hardware
//     round-robin), so ids are first regrouped per XCD and then walked in
//     GROUP_M-row panels, which keeps the X and W panels a single XCD touches
//     small enough for its own L2.
#include "i8f_common.hpp"

namespace i8f {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

enum { OUT_BF16 = 0, OUT_F16 = 1, OUT_F32 = 2, OUT_I32 = 3 };

struct GemmArgs {
    const int8_t *x;
    const int8_t *w;
    int M, N, K;
    const float *xs;
    const float *ws;
    float ws_host;
    int row_scale;  // 1: ws[n]; 0: one scale (ws[0] or ws_host when ws == nullptr)
    const void *bias;
    int bias_dtype;
    int order;
    void *out;
    int tiles_m, tiles_n;
};

template <int BM_, int BN_, int BK_, int WM_, int WN_, int STAGES_, int GROUP_M_>
struct Cfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, STAGES = STAGES_, GROUP_M = GROUP_M_;
    static constexpr int NW = WM * WN;
    static constexpr int NT = NW * 64;
    static constexpr int WTM = BM / WM, WTN = BN / WN;  // per-wave tile
    static constexpr int MI = WTM / 32, NI = WTN / 32;  // 32x32 MFMA blocks per wave
    static constexpr int CPR = BK / 16;                 // 16-byte chunks per LDS row
    static constexpr int X_BYTES = BM * BK, W_BYTES = BN * BK;
    static constexpr int STAGE_BYTES = X_BYTES + W_BYTES;
    static constexpr int X_LOADS = X_BYTES / 1024 / NW, W_LOADS = W_BYTES / 1024 / NW;
    static constexpr int LOADS = X_LOADS + W_LOADS;
    static constexpr int LDS_BYTES = STAGE_BYTES * STAGES;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert(X_BYTES % (1024 * NW) == 0 && W_BYTES % (1024 * NW) == 0, "tile must split into whole wave loads");
    static_assert(BK == 64 || BK == 128, "BK");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
};

// chunk swizzle: a function of the low 5 bits of the row only
template <int CPR>
__device__ __forceinline__ int swz(int r) {
    if constexpr (CPR == 4) return ((r >> 1) & 3) ^ ((r >> 3) & 1);
    else return (r ^ (r >> 3)) & 7;
}

__device__ __forceinline__ constexpr int waitcnt_vm(int n) {
    // gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]; others left at "no wait"
    return (n & 0xf) | (0x7 << 4) | (0xf << 8) | (((n >> 4) & 0x3) << 14);
}

typedef __attribute__((address_space(3))) void *lds_ptr_t;

template <int OUT>
struct OutElem {
    static constexpr int BYTES = (OUT == OUT_BF16 || OUT == OUT_F16) ? 2 : 4;
};

template <class C, int OUT>
__global__ __launch_bounds__(C::NT) void gemm_i8_kernel(const GemmArgs g) {
    constexpr int BM = C::BM, BN = C::BN, BK = C::BK, NW = C::NW, MI = C::MI, NI = C::NI, CPR = C::CPR;
    constexpr int S = C::STAGES;
    constexpr int OB = OutElem<OUT>::BYTES;
    __shared__ __attribute__((aligned(1024))) char smem[C::LDS_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / C::WN, wn = wave % C::WN;
    const int l32 = lane & 31, lhalf = lane >> 5;

    // ---- workgroup id -> output tile -------------------------------------------------
    int tile_m, tile_n;
    {
        const int T = g.tiles_m * g.tiles_n;
        const int bid = blockIdx.x;
        const int per = (T + 7) / 8;
        const int tall = (T % 8 == 0) ? 8 : (T % 8);
        const int xcd = bid % 8, loc = bid / 8;
        const int L = xcd < tall ? xcd * per + loc : tall * per + (xcd - tall) * (per - 1) + loc;
        const int in_group = C::GROUP_M * g.tiles_n;
        const int grp = L / in_group;
        const int first_m = grp * C::GROUP_M;
        const int gsz = min(g.tiles_m - first_m, C::GROUP_M);
        const int r = L % in_group;
        tile_m = first_m + r % gsz;
        tile_n = r / gsz;
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // ---- global -> LDS plan ------------------------------------------------------------
    const int K = g.K;
    __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)g.x, 0, (int)((int64_t)g.M * K), 0x00020000);
    __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc((void *)g.w, 0, (int)((int64_t)g.N * K), 0x00020000);
    const bool k_tail = (K % BK) != 0;
    const uint32_t OOB = 0x7ffffff0u;

    uint32_t xoff[C::X_LOADS], woff[C::W_LOADS];  // byte offset of this lane's chunk at k-tile 0
    int xck[C::X_LOADS], wck[C::W_LOADS];         // byte position of that chunk inside a k-tile
#pragma unroll
    for (int t = 0; t < C::X_LOADS; ++t) {
        const int gidx = (t * NW + wave) * 64 + lane;
        const int row = gidx / CPR, cl = gidx % CPR;
        xck[t] = (cl ^ swz<CPR>(row)) * 16;
        const int64_t grow = (int64_t)m0 + row;
        xoff[t] = grow < g.M ? (uint32_t)(grow * K + xck[t]) : OOB;
    }
#pragma unroll
    for (int t = 0; t < C::W_LOADS; ++t) {
        const int gidx = (t * NW + wave) * 64 + lane;
        const int row = gidx / CPR, cl = gidx % CPR;
        wck[t] = (cl ^ swz<CPR>(row)) * 16;
        const int64_t grow = (int64_t)n0 + row;
        woff[t] = grow < g.N ? (uint32_t)(grow * K + wck[t]) : OOB;
    }

    auto issue = [&](int kt) {
        char *st = smem + (kt % S) * C::STAGE_BYTES;
        const int kb = kt * BK;
#pragma unroll
        for (int t = 0; t < C::X_LOADS; ++t) {
            uint32_t vo = xoff[t] + (uint32_t)kb;
            if (k_tail && kb + xck[t] >= K) vo = OOB;
            if (xoff[t] == OOB) vo = OOB;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr_t)(st + (t * NW + wave) * 1024), 16, vo, 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < C::W_LOADS; ++t) {
            uint32_t vo = woff[t] + (uint32_t)kb;
            if (k_tail && kb + wck[t] >= K) vo = OOB;
            if (woff[t] == OOB) vo = OOB;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, (lds_ptr_t)(st + C::X_BYTES + (t * NW + wave) * 1024), 16, vo, 0, 0, 0);
        }
    };

    // ---- LDS -> register plan ----------------------------------------------------------
    const int sw = swz<CPR>(l32);
    int koff[BK / 32];
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) koff[ks] = ((ks * 2 + lhalf) ^ sw) * 16;
    const int xrow_off = (wm * C::WTM + l32) * BK;
    const int wrow_off = C::X_BYTES + (wn * C::WTN + l32) * BK;

    v16i acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const int KT = (K + BK - 1) / BK;

    // ---- prologue: S-1 tiles in flight ---------------------------------------------------
#pragma unroll
    for (int s = 0; s < S - 1; ++s)
        if (s < KT) issue(s);

    for (int kt = 0; kt < KT; ++kt) {
        // tile kt must have landed; tiles kt+1 .. kt+S-2 may still be in flight
        if (kt + S - 2 < KT) __builtin_amdgcn_s_waitcnt(waitcnt_vm((S - 2) * C::LOADS));
        else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
        // A bare barrier: __syncthreads() would add a fence that waits for ALL loads in flight.
        __builtin_amdgcn_s_barrier();  // everyone's part of tile kt is in LDS; everyone is done reading tile kt-1
        if (kt + S - 1 < KT) issue(kt + S - 1);  // overwrites the stage tile kt-1 was in

        const char *st = smem + (kt % S) * C::STAGE_BYTES;
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks) {
            v4i xf[MI], wf[NI];
#pragma unroll
            for (int i = 0; i < MI; ++i) xf[i] = *(const v4i *)(st + xrow_off + i * 32 * BK + koff[ks]);
#pragma unroll
            for (int j = 0; j < NI; ++j) wf[j] = *(const v4i *)(st + wrow_off + j * 32 * BK + koff[ks]);
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[j], xf[i], acc[i][j], 0, 0, 0);
        }
    }

    // ---- epilogue ----------------------------------------------------------------------
    __syncthreads();  // the stages are dead; reuse them as per-wave transpose buffers
    constexpr int ROW_BYTES = C::WTN * OB;
    constexpr int PITCH = ROW_BYTES + (OB == 2 ? 8 : 16);
    constexpr int WAVE_BYTES = 32 * PITCH;
    static_assert(WAVE_BYTES * NW <= C::LDS_BYTES, "epilogue buffer");
    char *ebuf = smem + wave * WAVE_BYTES;

    const bool has_bias = g.bias != nullptr;
    const float ws_one = g.ws ? (g.row_scale ? 0.0f : g.ws[0]) : g.ws_host;

#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int m = m0 + wm * C::WTM + i * 32 + l32;
        float xs = 0.0f;
        if (OUT != OUT_I32 && m < g.M) xs = g.xs[m];
#pragma unroll
        for (int j = 0; j < NI; ++j) {
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const int nl = j * 32 + qd * 8 + lhalf * 4;  // first of 4 consecutive n held by this lane
                const int n = n0 + wn * C::WTN + nl;
                if constexpr (OUT == OUT_I32) {
                    v4i o = {acc[i][j][4 * qd], acc[i][j][4 * qd + 1], acc[i][j][4 * qd + 2], acc[i][j][4 * qd + 3]};
                    *(v4i *)(ebuf + l32 * PITCH + nl * 4) = o;
                } else {
                    float wsv[4], bv[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        wsv[e] = ws_one;
                        bv[e] = 0.0f;
                    }
                    if (n < g.N) {  // N is a multiple of 8 here: the four n are all inside or all outside
                        if (g.row_scale) {
                            const float4 t = *(const float4 *)(g.ws + n);
                            wsv[0] = t.x, wsv[1] = t.y, wsv[2] = t.z, wsv[3] = t.w;
                        }
                        if (has_bias) {
                            if (g.bias_dtype == I8F_F32) {
                                const float4 t = *(const float4 *)((const float *)g.bias + n);
                                bv[0] = t.x, bv[1] = t.y, bv[2] = t.z, bv[3] = t.w;
                            } else {
                                const uint2 t = *(const uint2 *)((const uint16_t *)g.bias + n);
                                if (g.bias_dtype == I8F_BF16) {
                                    bv[0] = bf16_bits_to_f32(t.x & 0xffffu), bv[1] = bf16_bits_to_f32(t.x >> 16);
                                    bv[2] = bf16_bits_to_f32(t.y & 0xffffu), bv[3] = bf16_bits_to_f32(t.y >> 16);
                                } else {
                                    bv[0] = f16_bits_to_f32(t.x & 0xffffu), bv[1] = f16_bits_to_f32(t.x >> 16);
                                    bv[2] = f16_bits_to_f32(t.y & 0xffffu), bv[3] = f16_bits_to_f32(t.y >> 16);
                                }
                            }
                        }
                    }
                    float y[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float a = (float)acc[i][j][4 * qd + e];
                        constexpr int DT = OUT == OUT_BF16 ? I8F_BF16 : (OUT == OUT_F16 ? I8F_F16 : I8F_F32);
                        if (g.order == I8F_EPI_TORCH) {
                            float t;
                            if (g.row_scale) {
                                t = a * xs;
                                t = t * wsv[e];
                            } else {
                                const float sc = wsv[e] * xs;
                                t = a * sc;
                            }
                            t = round_to_dtype<DT>(t);
                            if (has_bias) t = t + round_to_dtype<DT>(bv[e]);
                            y[e] = t;
                        } else {
                            const float sc = xs * wsv[e];
                            float t = a * sc;
                            if (has_bias) t = t + bv[e];
                            y[e] = t;
                        }
                    }
                    if constexpr (OUT == OUT_BF16) {
                        *(uint2 *)(ebuf + l32 * PITCH + nl * 2) =
                            make_uint2(f32x2_to_bf16x2_bits(y[0], y[1]), f32x2_to_bf16x2_bits(y[2], y[3]));
                    } else if constexpr (OUT == OUT_F16) {
                        *(uint2 *)(ebuf + l32 * PITCH + nl * 2) =
                            make_uint2(f32x2_to_f16x2_bits(y[0], y[1]), f32x2_to_f16x2_bits(y[2], y[3]));
                    } else {
                        *(float4 *)(ebuf + l32 * PITCH + nl * 4) = make_float4(y[0], y[1], y[2], y[3]);
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
        // read the 32 x WTN strip back row-contiguously and store 16 bytes per lane
        constexpr int CPO = ROW_BYTES / 16;      // chunks per output row of the strip
        constexpr int EPCO = 16 / OB;            // output elements per chunk
        constexpr int PASSES = 32 * CPO / 64;
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int id = p * 64 + lane;
            const int row = id / CPO, cc = id % CPO;
            const uint4 val = *(const uint4 *)(ebuf + row * PITCH + cc * 16);
            const int mm = m0 + wm * C::WTM + i * 32 + row;
            const int nn = n0 + wn * C::WTN + cc * EPCO;
            if (mm < g.M && nn < g.N) *(uint4 *)((char *)g.out + ((int64_t)mm * g.N + nn) * OB) = val;
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// ---- slow but shape-agnostic kernel: one thread per output -----------------------------
template <int OUT>
__global__ __launch_bounds__(256) void gemm_i8_generic_kernel(const GemmArgs g) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)g.M * g.N) return;
    const int m = (int)(idx / g.N), n = (int)(idx % g.N);
    const int8_t *xr = g.x + (int64_t)m * g.K;
    const int8_t *wr = g.w + (int64_t)n * g.K;
    int acc = 0;
    for (int k = 0; k < g.K; ++k) acc += (int)xr[k] * (int)wr[k];
    if constexpr (OUT == OUT_I32) {
        ((int *)g.out)[idx] = acc;
    } else {
        constexpr int DT = OUT == OUT_BF16 ? I8F_BF16 : (OUT == OUT_F16 ? I8F_F16 : I8F_F32);
        const float xs = g.xs[m];
        const float ws = g.ws ? g.ws[g.row_scale ? n : 0] : g.ws_host;
        const float a = (float)acc;
        float b = 0.0f;
        if (g.bias) {
            if (g.bias_dtype == I8F_F32) b = ((const float *)g.bias)[n];
            else if (g.bias_dtype == I8F_BF16) b = bf16_bits_to_f32(((const uint16_t *)g.bias)[n]);
            else b = f16_bits_to_f32(((const uint16_t *)g.bias)[n]);
        }
        float t;
        if (g.order == I8F_EPI_TORCH) {
            if (g.row_scale) {
                t = a * xs;
                t = t * ws;
            } else {
                const float sc = ws * xs;
                t = a * sc;
            }
            t = round_to_dtype<DT>(t);
            if (g.bias) t = t + round_to_dtype<DT>(b);
        } else {
            const float sc = xs * ws;
            t = a * sc;
            if (g.bias) t = t + b;
        }
        store_from_f32<DT>(g.out, idx, t);
    }
}

// tile configurations
using CfgBig = Cfg<256, 256, 64, 2, 4, 4, 6>;    // 8 waves, 128 KB LDS, one workgroup per CU
using CfgMid = Cfg<128, 128, 64, 2, 2, 4, 8>;    // 4 waves, 64 KB LDS, two workgroups per CU

template <class C, int OUT>
int launch_cfg(GemmArgs &g, hipStream_t st) {
    g.tiles_m = (g.M + C::BM - 1) / C::BM;
    g.tiles_n = (g.N + C::BN - 1) / C::BN;
    const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
    hipLaunchKernelGGL((gemm_i8_kernel<C, OUT>), dim3((unsigned)tiles), dim3(C::NT), 0, st, g);
    return check_launch();
}

template <int OUT>
int launch(GemmArgs &g, hipStream_t st) {
    const int ob = OutElem<OUT>::BYTES;
    const bool fast = (g.K % 16 == 0) && (g.N % 8 == 0) && ((uintptr_t)g.x % 16 == 0) && ((uintptr_t)g.w % 16 == 0) &&
                      ((uintptr_t)g.out % 16 == 0) && ((int64_t)g.M * g.K < (1ll << 31)) &&
                      ((int64_t)g.N * g.K < (1ll << 31)) &&
                      (!g.ws || !g.row_scale || (uintptr_t)g.ws % 16 == 0) &&
                      (!g.bias || (uintptr_t)g.bias % 16 == 0);
    (void)ob;
    if (!fast) {
        const int64_t total = (int64_t)g.M * g.N;
        hipLaunchKernelGGL((gemm_i8_generic_kernel<OUT>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, g);
        return check_launch();
    }
    const int64_t big_tiles = (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256);
    if (big_tiles >= 128) return launch_cfg<CfgBig, OUT>(g, st);
    return launch_cfg<CfgMid, OUT>(g, st);
}

int validate(const int8_t *a, const int8_t *w, int64_t M, int64_t N, int64_t K, const void *out) {
    if (M < 0 || N < 0 || K < 0) return I8F_ERR_INVALID;
    if (M == 0 || N == 0) return I8F_OK;
    if (!out) return I8F_ERR_INVALID;
    if (K > 0 && (!a || !w)) return I8F_ERR_INVALID;
    if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return I8F_ERR_UNSUPPORTED;
    if (M * N >= (1ll << 40)) return I8F_ERR_UNSUPPORTED;
    return I8F_OK;
}

}  // namespace
}  // namespace i8f

extern "C" int i8f_gemm_i32(const int8_t *a, const int8_t *w, int64_t M, int64_t N, int64_t K, int32_t *acc,
                            void *stream) {
    using namespace i8f;
    if (int rc = validate(a, w, M, N, K, acc)) return rc;
    if (M == 0 || N == 0) return I8F_OK;
    if (int rc = check_device()) return rc;
    GemmArgs g{};
    g.x = a, g.w = w, g.M = (int)M, g.N = (int)N, g.K = (int)K, g.out = acc;
    return launch<OUT_I32>(g, (hipStream_t)stream);
}

extern "C" int i8f_linear_w8a8(const int8_t *a, const float *a_scale, const int8_t *w, const float *w_scale,
                               float w_scale_host, int scale_mode, const void *bias, int bias_dtype, void *out,
                               int out_dtype, int64_t M, int64_t N, int64_t K, int order, void *stream) {
    using namespace i8f;
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
    g.bias = bias, g.bias_dtype = bias_dtype, g.order = order;
    hipStream_t st = (hipStream_t)stream;
    switch (out_dtype) {
    case I8F_BF16: return launch<OUT_BF16>(g, st);
    case I8F_F16: return launch<OUT_F16>(g, st);
    default: return launch<OUT_F32>(g, st);
    }
}
