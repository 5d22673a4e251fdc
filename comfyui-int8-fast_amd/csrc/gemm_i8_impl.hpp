// int8 x int8 -> int32 "NT" GEMM on the gfx950 matrix cores with the
// dequantisation epilogue fused in registers.  (Kernel templates and launch logic; the translation
// units gemm_i8*.hip instantiate them per output type so that they compile side by side.)
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
//   * v_mfma_i32_16x16x64_i8 (or v_mfma_i32_32x32x32_i8, per configuration), W
//     fragments as the A operand and X fragments as the B operand, so that a
//     lane ends up with 4 consecutive n of one m: integer sums do not depend
//     on the order of k, so any k permutation that is the same for both
//     operands is allowed and none has to be undone.
//   * epilogue: scale/bias/round in registers, then a per-wave transpose
//     through LDS so that every global store is 16 bytes per lane and covers
//     whole 128-byte lines.
//   * workgroup id -> tile: consecutive ids go to different XCDs (hardware
//     round-robin), so ids are first regrouped per XCD and then walked in
//     GROUP_M-row panels, which keeps the X and W panels a single XCD touches
//     small enough for its own L2.
#include <type_traits>

#pragma once

#include "i8f_common.hpp"
#include "splitk_protocol.h"
#include <algorithm>
#include <atomic>

namespace i8f {
namespace gemm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

enum { OUT_BF16 = 0, OUT_F16 = 1, OUT_F32 = 2, OUT_I32 = 3 };

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf_t __attribute__((ext_vector_type(8)));
typedef _Float16 v8h_t __attribute__((ext_vector_type(8)));

// 32 x 32 x 16 product of two 16-bit fragments (8 values per lane each) into a binary32 block
template <int OUT>
__device__ __forceinline__ v16f side_mfma(v4i a, v4i b, v16f c) {
    if constexpr (OUT == OUT_BF16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf_t, a), __builtin_bit_cast(v8bf_t, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h_t, a), __builtin_bit_cast(v8h_t, b), c, 0, 0, 0);
}

// 16 x 16 x 16 product of two 16-bit fragments (4 values per lane each) into a binary32 block
typedef float v4f __attribute__((ext_vector_type(4)));
typedef short v4s_t __attribute__((ext_vector_type(4)));
typedef _Float16 v4h_t __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
template <int OUT>
__device__ __forceinline__ v4f side_mfma16(v2i a, v2i b, v4f c) {
    if constexpr (OUT == OUT_BF16)
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(v4s_t, a), __builtin_bit_cast(v4s_t, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(v4h_t, a), __builtin_bit_cast(v4h_t, b), c, 0, 0, 0);
}

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
    const void *addend;  // nullptr or [M,N] of the output dtype, added to the rounded result
    // nullptr or [ceil(M / gate_rows), N] of the output dtype: the rounded result (side branch included) is multiplied by
    // gate[m / gate_rows, n] and rounded before the addend is added (the gated residual of an adaLN-Zero block,
    // x + gate * linear(h), as torch's two tensor operations compute it)
    const void *gate;
    int gate_rows;
    // low-rank side branch, side[m,n] = sum_j side_t[m,j] * side_b[n,j] (operands of the output dtype, rank % 16 == 0),
    // rounded to that dtype, times side_alpha if side_has_alpha (rounded again), added to the rounded result
    const void *side_t, *side_b;
    int side_rank, side_has_alpha;
    float side_alpha;
    void *out;
    int tiles_m, tiles_n;
    // K split over `splits` workgroups per tile (1: none): partial sums and per-tile arrival counters in caller memory
    int splits;
    int *partials;          // [splits][tiles][BM * BN] int32, in the register order of the kernel
    unsigned *arrivals;     // [tiles] arrival words (splitk_protocol.h); any contents before the launch, zero after it
    unsigned splitk_tag;    // names this launch in the arrival words
};

// SPLIT_ (two-stage configurations): how a wave's loads of one K-tile are dealt over the phases that
// follow the barrier which frees their stage, one hex digit per phase, first phase in the top digit
// (0 = all of them in the first phase).
// MF_: the MFMA shape, 32 (v_mfma_i32_32x32x32_i8) or 16 (v_mfma_i32_16x16x64_i8).
// WSTAGES_: stages of the W tile if not STAGES_ (which the X tile always has): 160 KB of LDS hold two 256 x 128-byte
// X tiles and three W tiles but not three of each, and one operand a stage ahead of the other is enough to take the
// global->LDS latency out of the loop's critical path (the W refill then has two K-tiles of time to land, and the X
// refill, half the bytes of a whole stage, is issued first behind the barrier).
template <int BM_, int BN_, int BK_, int WM_, int WN_, int STAGES_, int GROUP_M_, int SPLIT_ = 0, int MF_ = 32, int WSTAGES_ = STAGES_>
struct Cfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, STAGES = STAGES_, GROUP_M = GROUP_M_;
    static constexpr int SPLIT = SPLIT_, MF = MF_, WSTAGES = WSTAGES_;
    static constexpr int NW = WM * WN;
    static constexpr int NT = NW * 64;
    static constexpr int WTM = BM / WM, WTN = BN / WN;  // per-wave tile
    // A wave's accumulators are blocks of 32 rows x CB columns: 32 x 32 with the 32x32x32 MFMA, 32 x 16 (two 16 x 16
    // products one above the other) with the 16x16x64 MFMA, whose wave tiles may therefore be 48 columns wide.
    static constexpr int CB = MF_ == 16 ? 16 : 32;
    static constexpr int MI = WTM / 32, NJ = WTN / CB;
    static constexpr int CPR = BK / 16;                 // 16-byte chunks per LDS row
    static constexpr int X_BYTES = BM * BK, W_BYTES = BN * BK;
    // every wave issues the same number of 1 KB loads per tile; a tile that does not split evenly
    // over the waves is rounded up, and the surplus loads are out of range (they move nothing)
    static constexpr int X_LOADS = (X_BYTES / 1024 + NW - 1) / NW, W_LOADS = (W_BYTES / 1024 + NW - 1) / NW;
    static constexpr int X_ALLOC = X_LOADS * NW * 1024, W_ALLOC = W_LOADS * NW * 1024;
    static constexpr int LOADS = X_LOADS + W_LOADS;
    // LDS: stages of an X tile followed by its W tile; with W a stage deeper, the X stages and then the W stages
    static constexpr int W_BASE = WSTAGES == STAGES ? X_ALLOC : X_ALLOC * STAGES;
    static constexpr int X_STRIDE = WSTAGES == STAGES ? X_ALLOC + W_ALLOC : X_ALLOC;
    static constexpr int W_STRIDE = WSTAGES == STAGES ? X_ALLOC + W_ALLOC : W_ALLOC;
    static constexpr int LDS_BYTES = X_ALLOC * STAGES + W_ALLOC * WSTAGES;
    static_assert(WSTAGES == STAGES || (STAGES == 2 && WSTAGES == 3), "W may be one stage ahead of a two-stage X");
    static_assert(WTM % 32 == 0 && WTN % CB == 0, "wave tile must be a multiple of 32 rows x CB columns");
    static_assert(X_BYTES % 1024 == 0 && W_BYTES % 1024 == 0, "tile must split into whole wave loads");
    static_assert(BK == 64 || BK == 128, "BK");
    static_assert(MF == 32 || (MF == 16 && BK == 128), "the 16x16x64 form takes 128-byte K-tiles");
};

// chunk swizzle: a function of the low 5 bits of the row only
template <int CPR>
__device__ __forceinline__ int swz(int r) {
    if constexpr (CPR == 4) return ((r >> 1) & 3) ^ ((r >> 3) & 1);
    else return (r ^ ((r >> 3) & 3)) & 7;
}

__device__ __forceinline__ constexpr int waitcnt_vm(int n) {
    // gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]; others left at "no wait"
    return (n & 0xf) | (0x7 << 4) | (0xf << 8) | (((n >> 4) & 0x3) << 14);
}

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// One wave-wide global -> LDS load of 16 bytes per lane (lane l lands at lds_base + 16 l), issued
// from inline assembly on purpose: the compiler knows nothing of an LDS write in flight, so it does
// not put a full vmcnt(0) wait in front of every later LDS read (it cannot prove that the reads
// touch another stage).  The waits for these loads are the explicit s_waitcnt of the main loop.
__device__ __forceinline__ void dma16(v4i rsrc, uint32_t lds_base, uint32_t voffset, int soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset)
                 : "memory", "m0");
}

__device__ __forceinline__ v4i make_rsrc(const void *p, uint32_t bytes) {
    const uint64_t a = (uint64_t)p;
    v4i r = {(int)(uint32_t)a, (int)((uint32_t)(a >> 32) & 0xffffu), (int)bytes, 0x00020000};
    return r;
}

template <int OUT>
struct OutElem {
    static constexpr int BYTES = (OUT == OUT_BF16 || OUT == OUT_F16) ? 2 : 4;
};

// One 4-element group of the epilogue, with the operation order, the scale mode and the bias
// fixed at compile time (a run-time test per value costs more than the arithmetic).
template <int OUT, int ORDER, bool ROW, bool BIAS, bool SIDE = false>
__device__ __forceinline__ void epilogue_quad(const int (&a4)[4], float xs, const float4 w4, const float4 b4,
                                              char *dst, const float *side4 = nullptr) {
    constexpr int DT = OUT == OUT_BF16 ? I8F_BF16 : (OUT == OUT_F16 ? I8F_F16 : I8F_F32);
    const float wsv[4] = {w4.x, w4.y, w4.z, w4.w};
    const float bv[4] = {b4.x, b4.y, b4.z, b4.w};
    float y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float a = (float)a4[e];
        float t;
        if constexpr (ORDER == I8F_EPI_TORCH) {
            if constexpr (ROW) {
                t = a * xs;
                t = t * wsv[e];
            } else {
                const float sc = wsv[e] * xs;
                t = a * sc;
            }
            t = round_to_dtype<DT>(t);
            if constexpr (BIAS) t = t + round_to_dtype<DT>(bv[e]);
        } else {
            const float sc = xs * wsv[e];
            t = a * sc;
            if constexpr (BIAS) t = t + bv[e];
        }
        // the side branch is added to the ROUNDED result, as a tensor addition would (y + side.to(y.dtype))
        if constexpr (SIDE) t = round_to_dtype<DT>(t) + side4[e];
        y[e] = t;
    }
    if constexpr (OUT == OUT_BF16) {
        *(uint2 *)dst = make_uint2(f32x2_to_bf16x2_bits(y[0], y[1]), f32x2_to_bf16x2_bits(y[2], y[3]));
    } else if constexpr (OUT == OUT_F16) {
        *(uint2 *)dst = make_uint2(f32x2_to_f16x2_bits(y[0], y[1]), f32x2_to_f16x2_bits(y[2], y[3]));
    } else {
        *(float4 *)dst = make_float4(y[0], y[1], y[2], y[3]);
    }
}

// Eight (or four) outputs of one 16-byte piece plus the addend's, rounded once more to the output
// dtype: what the reference's `y + side.to(y.dtype)` computes on its rounded tensors.
template <int OUT>
__device__ __forceinline__ uint4 add_rounded(uint4 y, uint4 s) {
    if constexpr (OUT == OUT_F32) {
        return make_uint4(__float_as_uint(__uint_as_float(y.x) + __uint_as_float(s.x)),
                          __float_as_uint(__uint_as_float(y.y) + __uint_as_float(s.y)),
                          __float_as_uint(__uint_as_float(y.z) + __uint_as_float(s.z)),
                          __float_as_uint(__uint_as_float(y.w) + __uint_as_float(s.w)));
    } else if constexpr (OUT == OUT_I32) {
        return y;
    } else {
        const uint32_t yv[4] = {y.x, y.y, y.z, y.w}, sv[4] = {s.x, s.y, s.z, s.w};
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (OUT == OUT_BF16) {
                const float lo = bf16_bits_to_f32(yv[e] & 0xffffu) + bf16_bits_to_f32(sv[e] & 0xffffu);
                const float hi = bf16_bits_to_f32(yv[e] >> 16) + bf16_bits_to_f32(sv[e] >> 16);
                o[e] = f32x2_to_bf16x2_bits(lo, hi);
            } else {
                const float lo = f16_bits_to_f32(yv[e] & 0xffffu) + f16_bits_to_f32(sv[e] & 0xffffu);
                const float hi = f16_bits_to_f32(yv[e] >> 16) + f16_bits_to_f32(sv[e] >> 16);
                o[e] = f32x2_to_f16x2_bits(lo, hi);
            }
        }
        return make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// Eight (or four) outputs of one 16-byte piece times the gate's, each product rounded to the output dtype: what
// `gate * y` computes on tensors of that dtype.
template <int OUT>
__device__ __forceinline__ uint4 mul_rounded(uint4 y, uint4 s) {
    if constexpr (OUT == OUT_F32) {
        return make_uint4(__float_as_uint(__uint_as_float(y.x) * __uint_as_float(s.x)),
                          __float_as_uint(__uint_as_float(y.y) * __uint_as_float(s.y)),
                          __float_as_uint(__uint_as_float(y.z) * __uint_as_float(s.z)),
                          __float_as_uint(__uint_as_float(y.w) * __uint_as_float(s.w)));
    } else if constexpr (OUT == OUT_I32) {
        return y;
    } else {
        const uint32_t yv[4] = {y.x, y.y, y.z, y.w}, sv[4] = {s.x, s.y, s.z, s.w};
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (OUT == OUT_BF16) {
                const float lo = bf16_bits_to_f32(yv[e] & 0xffffu) * bf16_bits_to_f32(sv[e] & 0xffffu);
                const float hi = bf16_bits_to_f32(yv[e] >> 16) * bf16_bits_to_f32(sv[e] >> 16);
                o[e] = f32x2_to_bf16x2_bits(lo, hi);
            } else {
                const float lo = f16_bits_to_f32(yv[e] & 0xffffu) * f16_bits_to_f32(sv[e] & 0xffffu);
                const float hi = f16_bits_to_f32(yv[e] >> 16) * f16_bits_to_f32(sv[e] >> 16);
                o[e] = f32x2_to_f16x2_bits(lo, hi);
            }
        }
        return make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// KTAIL: K is not a multiple of BK (the last tile is ragged); the common case is the other kernel.
// What the prologue needs (operand pointers, sizes, tile counts) comes first in the argument list: the
// first 16 dwords of the kernel arguments are preloaded into SGPRs at wave launch, the rest (epilogue
// operands) is fetched by scalar loads that have the whole main loop to land.
// (The body is shared by the kernel of one problem and the kernel of a group of problems: wg_id is the workgroup's
// number within its problem, gout / gaddend / ggate / ws_host that problem's output, addend, gate and host-side weight scale.)
template <class C, int OUT, bool KTAIL, bool SIDE = false, bool SPLITK = false>
__device__ __forceinline__ void gemm_i8_body(const int8_t *gx, const int8_t *gw, int gM, int gN, int gK, int tiles_m, int tiles_n,
                                             const float *gxs, const float *gws, const void *gbias, int flags, const GemmArgs &g,
                                             const int wg_id, void *gout, const void *gaddend, const float ws_host,
                                             const void *ggate, const int ggate_rows) {
    constexpr int BM = C::BM, BN = C::BN, BK = C::BK, NW = C::NW, MI = C::MI, NJ = C::NJ, CB = C::CB, CPR = C::CPR;
    constexpr int S = C::STAGES, WS = C::WSTAGES;
    constexpr bool ASYM = WS != S;  // the W tile one stage deeper than the X tile
    constexpr int OB = OutElem<OUT>::BYTES;
    constexpr int KS = BK / 32;  // phases per tile (a k-step of 32 each, or half a wave tile's share of a k-step of 64)
    static_assert(KS % 2 == 0, "fragment double-buffering alternates over an even number of k-steps");
    constexpr bool M16 = C::MF == 16;
    constexpr int QPB = M16 ? 2 : 4;  // quads (4 consecutive n of one m) a lane holds per block
    constexpr int NQ = M16 ? 1 : 4;   // distinct column positions among them
    // The epilogue stages EPI_STRIPS 32-row strips of a wave's tile at once (all of it for 2-byte
    // outputs), padded so that the transposing writes do not collide on banks.
    constexpr int ROW_BYTES = C::WTN * OB;
    constexpr int PITCH = ROW_BYTES + (OB == 2 ? 8 : 16);
    // (one strip at a time with a side branch, whose operands take the rest of the memory)
    constexpr int EPI_STRIPS = SIDE ? 1 : ((OB == 2 || MI == 1) ? MI : MI / 2);
    constexpr int WAVE_BYTES = EPI_STRIPS * 32 * PITCH;
    // The epilogue operands of the tile (token scales, weight scales, bias) are staged behind the waves' transpose
    // buffers, in memory that belongs to the K-tile stages while the main loop runs.
    constexpr int EPI_OPS_OFF = WAVE_BYTES * NW, EPI_OPS_BYTES = 4 * (BM + 2 * BN);
    // The side branch's operands of the tile, BM rows of side_t and then BN rows of side_b, up to SIDE_RMAX ranks of
    // 2 bytes per row at a pitch that keeps 16-byte pieces aligned and spreads the rows over the banks.
    constexpr int SIDE_RMAX = 64, SIDE_PITCH = SIDE_RMAX * 2 + 16;
    constexpr int SIDE_OFF = EPI_OPS_OFF + EPI_OPS_BYTES, SIDE_BYTES = SIDE ? (BM + BN) * SIDE_PITCH : 0;
    static_assert(SIDE_OFF % 16 == 0, "16-byte pieces");
    constexpr int SMEM_BYTES = C::LDS_BYTES > SIDE_OFF + SIDE_BYTES ? C::LDS_BYTES : SIDE_OFF + SIDE_BYTES;
    static_assert(SMEM_BYTES + (SPLITK ? 16 : 0) <= 160 * 1024, "LDS");
    __shared__ __attribute__((aligned(1024))) char smem[SMEM_BYTES];
    float *const s_xs = (float *)(smem + EPI_OPS_OFF), *const s_ws = s_xs + BM, *const s_bias = s_ws + BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: lets LDS bases live in SGPRs
    const int wm = wave / C::WN, wn = wave % C::WN;
    const int l32 = lane & 31, lhalf = lane >> 5;

    // ---- workgroup id -> output tile -------------------------------------------------
    int tile_m, tile_n;
    {
        const int T = tiles_m * tiles_n;
        const int bid = SPLITK ? __builtin_amdgcn_readfirstlane(wg_id % T) : wg_id;  // the K slices of a tile are T workgroup ids apart
        const int per = (T + 7) / 8;
        const int tall = (T % 8 == 0) ? 8 : (T % 8);
        const int xcd = bid % 8, loc = bid / 8;
        const int L = xcd < tall ? xcd * per + loc : tall * per + (xcd - tall) * (per - 1) + loc;
        const int in_group = C::GROUP_M * tiles_n;
        const int grp = L / in_group;
        const int first_m = grp * C::GROUP_M;
        const int gsz = min(tiles_m - first_m, C::GROUP_M);
        const int r = L % in_group;
        tile_m = first_m + r % gsz;
        tile_n = r / gsz;
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // ---- global -> LDS plan ------------------------------------------------------------
    // One wave load moves 64 x 16 bytes into 1 KB of LDS (lane l lands at offset 16*l).  The lane
    // decides WHICH global chunk it fetches, which is where the swizzle is applied.  The byte
    // offset of the K-tile travels in the scalar offset of the buffer instruction, so issuing a
    // load costs no vector arithmetic; rows beyond the matrix carry an out-of-range vector offset
    // and are zero-filled by the buffer bounds check (which looks at the vector offset only).
    const int K = gK;
    const v4i rx = make_rsrc(gx, (uint32_t)((int64_t)gM * K));
    const v4i rw = make_rsrc(gw, (uint32_t)((int64_t)gN * K));
    const uint32_t OOB = 0x7ffffff0u;

    uint32_t xoff[C::X_LOADS], woff[C::W_LOADS];  // byte offset of this lane's chunk at k-tile 0
    int xck[C::X_LOADS], wck[C::W_LOADS];         // byte position of that chunk inside a k-tile
#pragma unroll
    for (int t = 0; t < C::X_LOADS; ++t) {
        const int gidx = (t * NW + wave) * 64 + lane;
        const int row = gidx / CPR, cl = gidx % CPR;
        xck[t] = (cl ^ swz<CPR>(row)) * 16;
        const int64_t grow = (int64_t)m0 + row;
        xoff[t] = (row < BM && grow < gM) ? (uint32_t)(grow * K + xck[t]) : OOB;
    }
#pragma unroll
    for (int t = 0; t < C::W_LOADS; ++t) {
        const int gidx = (t * NW + wave) * 64 + lane;
        const int row = gidx / CPR, cl = gidx % CPR;
        wck[t] = (cl ^ swz<CPR>(row)) * 16;
        const int64_t grow = (int64_t)n0 + row;
        woff[t] = (row < BN && grow < gN) ? (uint32_t)(grow * K + wck[t]) : OOB;
    }

    // SPLITK: this workgroup multiplies k-tiles [kt_first, kt_first + KT) of its output tile only
    const int KT_all = (K + BK - 1) / BK;
    // (integer division runs on the vector ALUs: readfirstlane brings the quotients back to scalar registers, where the
    // K offset of the loads has to be)
    [[maybe_unused]] const int slice = SPLITK ? __builtin_amdgcn_readfirstlane(wg_id / (tiles_m * tiles_n)) : 0;
    const int kt_per = SPLITK ? __builtin_amdgcn_readfirstlane((KT_all + g.splits - 1) / g.splits) : KT_all;
    const int kt_first = slice * kt_per;
    const int KT = SPLITK ? max(min(kt_per, KT_all - kt_first), 0) : KT_all;

    // `live` false (a tile index past the end, at the tail of the loop) turns every lane's offset
    // out of range: the instruction is still issued, which keeps the loop body free of branches,
    // but moves no data.
    // load r of tile kt: r < X_LOADS fetches a piece of the X tile, the others a piece of the W tile
    const uint32_t smem_base = (uint32_t)(uintptr_t)smem;
    // (sx, sw: the stage of the X and of the W tile that receives tile kt)
    auto issue_to = [&](int kt, int sx, int sw, bool live, int r) {
        const bool is_x = r < C::X_LOADS;
        const int t = is_x ? r : r - C::X_LOADS;
        const uint32_t st = smem_base + (is_x ? sx * C::X_STRIDE : C::W_BASE + sw * C::W_STRIDE) + wave * 1024;
        const int kb = (kt_first + kt) * BK;
        uint32_t vo = live ? (is_x ? xoff[t] : woff[t]) : OOB;
        int so = kb;
        if constexpr (KTAIL) {  // chunks past K are forced out of range per lane
            vo = (kb + (is_x ? xck[t] : wck[t]) < K && vo != OOB) ? vo + (uint32_t)kb : OOB;
            so = 0;
        }
        dma16(is_x ? rx : rw, st + t * NW * 1024, vo, so);
    };
    auto issue_one = [&](int kt, bool live, int r) { issue_to(kt, kt % S, kt % WS, live, r); };  // (prologue: kt is a constant)
    auto issue = [&](int kt, bool live) {
#pragma unroll
        for (int r = 0; r < C::LOADS; ++r) issue_one(kt, live, r);
    };

    // ---- LDS -> register plan ----------------------------------------------------------
    const int sw = swz<CPR>(l32);
    int koff[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) koff[ks] = ((ks * 2 + lhalf) ^ sw) * 16;
    const int xrow_off = (wm * C::WTM + l32) * BK;
    const int wrow_off = (wn * C::WTN + l32) * BK;
    // 16x16x64 form: a fragment is 16 rows x 64 k; lane l fetches the 16 bytes of row l % 16 at k-chunk l / 16 of the
    // k-step (any k order will do as long as both operands use the same one).  The swizzle looks at the low five bits
    // of the row, so the odd 16-row groups have their own chunk offsets.  Which chunk a lane quarter takes is chosen so
    // that lane l touches the banks that lane l of the 32x32x32 form touches (lanes l and l + 32 read neighbouring
    // chunks of one row): quarters 0, 1, 2, 3 take chunks 0, 2, 1, 3.
    const int l16 = lane & 15, lq = lane >> 4;
    const int lchunk = ((lq & 1) << 1) | (lq >> 1);
    [[maybe_unused]] int koff16[2][2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int hp = 0; hp < 2; ++hp) koff16[kk][hp] = ((kk * 4 + lchunk) ^ swz<CPR>(hp * 16 + l16)) * 16;
    [[maybe_unused]] const int xrow16 = (wm * C::WTM + l16) * BK;
    [[maybe_unused]] const int wrow16 = (wn * C::WTN + l16) * BK;
    // (a wave tile of 48 columns starts on an odd 16-row group of the W tile in every other wave: its column fragments
    // then take the chunk offsets of the other parity)
    [[maybe_unused]] int koffw[2][2];
    {
        const bool odd = (C::WTN % 32 != 0) && ((wn * (C::WTN / 16)) & 1);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int hp = 0; hp < 2; ++hp) koffw[kk][hp] = odd ? koff16[kk][hp ^ 1] : koff16[kk][hp];
    }

    // accumulators: per block (32 rows x CB columns) QPB quads of 4 consecutive n per lane.
    //   32x32x32: quad qd holds n = 8 qd + 4 (lane / 32) + e of row m = lane % 32
    //   16x16x64: quad qd holds n = 4 (lane / 16) + e of row m = 16 qd + lane % 16
    v16i acc[M16 ? 1 : MI][M16 ? 1 : NJ];
    v4i acc16[M16 ? MI : 1][M16 ? NJ : 1][2];
    if constexpr (M16) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int qd = 0; qd < 2; ++qd) acc16[i][j][qd] = (v4i)0;
    } else {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    }
    // the lane's quad qd of block (i, j), and where it sits inside the block
    auto quad_of = [&](int i, int j, int qd) -> v4i {
        if constexpr (M16) return acc16[i][j][qd];
        else return v4i{acc[i][j][4 * qd], acc[i][j][4 * qd + 1], acc[i][j][4 * qd + 2], acc[i][j][4 * qd + 3]};
    };
    auto quad_add = [&](int i, int j, int qd, v4i v) {
        if constexpr (M16) acc16[i][j][qd] += v;
        else acc[i][j][4 * qd] += v.x, acc[i][j][4 * qd + 1] += v.y, acc[i][j][4 * qd + 2] += v.z, acc[i][j][4 * qd + 3] += v.w;
    };
    auto quad_m = [&](int qd) { return M16 ? qd * 16 + l16 : l32; };              // row inside the 32-row strip
    auto quad_n = [&](int qd) { return M16 ? lq * 4 : qd * 8 + lhalf * 4; };      // first column inside the block
    auto quad_c = [&](int qd) constexpr { return M16 ? 0 : qd; };                 // which of the NQ column positions

    // Fragment registers per phase.  32x32x32: MI + NJ fragments of one k-step of 32.  16x16x64: a phase is one half of
    // the wave tile's rows (MI fragments of 16 rows) against all NJ column fragments for a k-step of 64; phases 0, 1
    // share the column fragments of k-step 0, phases 2, 3 those of k-step 1.
    constexpr int XF = MI, WF = NJ;
    constexpr int MN = MI * NJ;  // MFMAs per phase
    auto load_x = [&](const char *st, int ph, v4i (&xf)[XF]) {
        if constexpr (M16) {
            const int h = ph & 1, kk = (ph >> 1) & 1;
#pragma unroll
            for (int t = 0; t < MI; ++t) {
                const int ii = h * MI + t;
                xf[t] = *(const v4i *)(st + xrow16 + ii * 16 * BK + koff16[kk][ii & 1]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < MI; ++i) xf[i] = *(const v4i *)(st + xrow_off + i * 32 * BK + koff[ph]);
        }
    };
    auto load_w = [&](const char *st, int ph, v4i (&wf)[WF]) {
        if constexpr (M16) {
            const int kk = (ph >> 1) & 1;
#pragma unroll
            for (int jj = 0; jj < WF; ++jj) wf[jj] = *(const v4i *)(st + wrow16 + jj * 16 * BK + koffw[kk][jj & 1]);
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) wf[j] = *(const v4i *)(st + wrow_off + j * 32 * BK + koff[ph]);
        }
    };
    auto load_frags = [&](const char *xst, const char *wst, int ph, v4i (&xf)[XF], v4i (&wf)[WF]) {
        load_w(wst, ph, wf);
        load_x(xst, ph, xf);
    };
    auto mma_one = [&](const v4i (&xf)[XF], const v4i (&wf)[WF], int ph, int r) {
        if constexpr (M16) {
            const int jj = r / MI, t = r % MI, ii = (ph & 1) * MI + t;  // a column fragment is done with after MI MFMAs
            v4i &a = acc16[ii >> 1][jj][ii & 1];
            a = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[jj], xf[t], a, 0, 0, 0);
        } else {
            const int i = r / NJ, j = r % NJ;
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[j], xf[i], acc[i][j], 0, 0, 0);
        }
    };

    // ---- prologue: S tiles in flight, fragments of the first k-step in registers --------------
    // Two ways to keep the stages full.  With two stages a stage is refilled right after the barrier
    // that frees it (tile kt+S from the last phase of iteration kt on), in one burst or, by the SPLIT
    // of the configuration, over that phase and the following ones of iteration kt+1.  With three
    // or more the refill of the stage freed by the PREVIOUS iteration is dealt out over the whole of
    // iteration kt (tile kt+S-1): a wave that issues many loads at once blocks on the load queue, and
    // while it is blocked it issues no MFMAs either.  Loads past the last tile are issued all the
    // same (they move nothing), so the number of loads in flight at any point is a constant.
    constexpr bool SPREAD_DMA = S >= 3;
    constexpr int PRE = SPREAD_DMA ? S - 1 : S;  // tiles issued before the loop
    // two stages: loads [cut(p), cut(p+1)) of a tile go out in the p-th phase after the barrier
    auto cut = [](int p) constexpr {
        if (C::SPLIT == 0) return p <= 0 ? 0 : C::LOADS;
        int c = 0;
        for (int q = 0; q < p && q < KS; ++q) c += (C::SPLIT >> (4 * (KS - 1 - q))) & 0xf;
        return c;
    };
    static_assert(SPREAD_DMA || cut(KS) == C::LOADS, "the split has to cover every load of a tile");
    // W one stage ahead: the X tile goes out first behind the barrier (all of it), the W tile, which has a K-tile more
    // to land, in the phases after; at any barrier the loads that may still be in flight are that one W tile's
    static_assert(!ASYM || (!SPREAD_DMA && cut(1) == C::X_LOADS), "X behind the barrier, W in the phases that follow");
#pragma unroll
    for (int s = 0; s < PRE; ++s) {
        if (!SPREAD_DMA && s == PRE - 1) {
#pragma unroll
            for (int r = 0; r < (ASYM ? C::LOADS : cut(1)); ++r) issue_one(s, s < KT, r);  // the rest follows inside the loop
        } else {
            issue(s, s < KT);
        }
    }
    // ---- epilogue operands: requested behind the first tiles, parked in registers until the main loop
    // is done.  Nothing looks at the results before the epilogue: indices are clamped instead of
    // predicated and the conversion happens after the loop, so no instruction in between waits for
    // them (the wait for tile 0 below counts them among the younger loads it may leave in flight, and
    // so waits for up to three loads of tile 1 more than it has to).
    constexpr int XS_PER = (BM + C::NT - 1) / C::NT, WS_PER = (BN + C::NT - 1) / C::NT;
    float xs_r[XS_PER], ws_r[WS_PER];
    uint32_t bias_r[WS_PER];
    float ws_one = 0.0f;
    const bool row_scale = flags & 1;
    const int bias_dtype = flags >> 1;
    if constexpr (OUT != OUT_I32) {
        if (gws && !row_scale) ws_one = gws[0];
#pragma unroll
        for (int u = 0; u < XS_PER; ++u) xs_r[u] = gxs[min(m0 + tid + u * C::NT, gM - 1)];
#pragma unroll
        for (int u = 0; u < WS_PER; ++u) {
            const int n = min(n0 + tid + u * C::NT, gN - 1);
            ws_r[u] = row_scale ? gws[n] : 0.0f;
            bias_r[u] = 0;
            if (gbias) {
                if (bias_dtype == I8F_F32) bias_r[u] = ((const uint32_t *)gbias)[n];
                else bias_r[u] = ((const uint16_t *)gbias)[n];
            }
        }
    }

    __builtin_amdgcn_s_waitcnt(waitcnt_vm(SPREAD_DMA ? (PRE - 1) * C::LOADS : (ASYM ? C::LOADS : cut(1))));  // younger tiles may be in flight
    __builtin_amdgcn_s_barrier();  // tile 0 is in LDS for everyone (no fence: nothing else has been written)

    // Fragments are double-buffered in registers: the LDS reads of k-step s+1 are issued before
    // the MFMAs of k-step s, so the matrix pipe does not wait for LDS.  There is one barrier per
    // K-tile, in front of its last MFMA group: by then every wave has finished reading tile kt
    // (its last fragments are in registers), so the stage of tile kt is refilled with tile kt+S
    // right away, and tile kt+1 is known to have landed, so its first fragments can be fetched.
    v4i xa[XF] = {}, wa[WF] = {}, xb[XF] = {}, wb[WF] = {};
    if (KT > 0) load_frags(smem, smem + C::W_BASE, 0, xa, wa);
    // Drain scalar loads (kernel arguments) here: a scalar load still pending at the loop header
    // would turn every LDS wait inside the loop into a full lgkmcnt(0).
    __builtin_amdgcn_s_waitcnt(0xC07F);

    int ix = 0, iw = 0;  // kt % S, kt % WS: the stages that hold tile kt
    for (int kt = 0; kt < KT; ++kt) {
        if constexpr (!ASYM) iw = ix;  // (one index: the W tile then sits at a constant distance from its X tile)
        const int ix1 = ix + 1 == S ? 0 : ix + 1, iw1 = ASYM ? (iw + 1 == WS ? 0 : iw + 1) : ix1;      // ... tile kt + 1
        const int ixp = ix == 0 ? S - 1 : ix - 1, iwp = ASYM ? (iw == 0 ? WS - 1 : iw - 1) : ixp;      // ... held tile kt - 1
        const char *xst = smem + ix * C::X_STRIDE, *xnx = smem + ix1 * C::X_STRIDE;
        const char *wst = ASYM ? smem + C::W_BASE + iw * C::W_STRIDE : xst + C::W_BASE;
        const char *wnx = ASYM ? smem + C::W_BASE + iw1 * C::W_STRIDE : xnx + C::W_BASE;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const bool last = ks == KS - 1;
            if (last) {
                // my part of tile kt+1 has landed and my LDS reads of tile kt have returned; what may
                // still be in flight are the younger tiles (and, spread, the part of the newest one
                // that the earlier phases of this iteration have issued)
                constexpr int YOUNGER = SPREAD_DMA ? (S - 3) * C::LOADS + (KS - 1) * C::LOADS / KS : (ASYM ? C::W_LOADS : 0);
                __builtin_amdgcn_s_waitcnt(waitcnt_vm(YOUNGER) & 0xF0FF);
                __builtin_amdgcn_s_barrier();
            }
            v4i(&xc)[XF] = (ks & 1) ? xb : xa;
            v4i(&xn)[XF] = (ks & 1) ? xa : xb;
            // (16x16x64: one set of column fragments, each replaced as soon as its last MFMA of a k-step has issued)
            v4i(&wc)[WF] = (!M16 && (ks & 1)) ? wb : wa;
            v4i(&wn_)[WF] = (M16 || (ks & 1)) ? wa : wb;
            // past the last tile the next-fragment reads fetch stale LDS that nobody uses
            const char *fx = last ? xnx : xst, *fw = last ? wnx : wst;
            const int fks = last ? 0 : ks + 1;
            // 32x32x32: the next phase's fragments are requested in front of this phase's MFMAs.  16x16x64: one fragment
            // behind each of the first MFMAs instead (a 16-cycle MFMA covers three or four other instructions, not a
            // burst of eight LDS reads with their address arithmetic, and the two waves of a SIMD run in step).
            if constexpr (!M16) load_frags(fx, fw, fks, xn, wn_);
            __builtin_amdgcn_sched_barrier(0);
            // the tile being fetched: two stages refill the stage that this iteration's barrier frees
            // (tile kt+2) from the last phase on and finish in the following phases of the next iteration
            // (the stage freed by the previous barrier, or from the last phase on by this iteration's: each operand's
            // tile is the one its stage count puts there)
            const bool behind = !SPREAD_DMA && last;
            const int ftx = kt + S - (behind ? 0 : 1), ftw = kt + WS - (behind ? 0 : 1);
            const int fsx = behind ? ix : ixp, fsw = behind ? iw : iwp;
            // this phase's share of its loads
            const int la = SPREAD_DMA ? ks * C::LOADS / KS : (last ? 0 : cut(ks + 1));
            const int lb = SPREAD_DMA ? (ks + 1) * C::LOADS / KS : (last ? cut(1) : cut(ks + 2));
            [[maybe_unused]] int frag = 0;  // row fragments of the next phase requested so far
#pragma unroll
            for (int r = 0; r < MN; ++r) {
                mma_one(xc, wc, ks, r);
                const int l0 = la + r * (lb - la) / MN, l1 = la + (r + 1) * (lb - la) / MN;
                if constexpr (M16) {
                    const int kk = (fks >> 1) & 1;
                    if ((ks & 1) && r % MI == MI - 1) {  // the k-step ends with this phase: the column fragment is free
                        const int jj = r / MI;
                        wn_[jj] = *(const v4i *)(fw + wrow16 + jj * 16 * BK + koffw[kk][jj & 1]);
                    } else if (l0 == l1 && frag < XF) {  // a slot with nothing else to issue takes a row fragment
                        const int ii = (fks & 1) * MI + frag;
                        xn[frag] = *(const v4i *)(fx + xrow16 + ii * 16 * BK + koff16[kk][ii & 1]);
                        ++frag;
                    }
                }
#pragma unroll
                for (int l = l0; l < l1; ++l) {
                    const int ft = l < C::X_LOADS ? ftx : ftw;
                    issue_to(ft, fsx, fsw, ft < KT, l);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (M16) {  // (a phase with fewer free slots than row fragments)
                const int kk = (fks >> 1) & 1;
#pragma unroll
                for (int f = 0; f < XF; ++f) {
                    if (f >= frag) {
                        const int ii = (fks & 1) * MI + f;
                        xn[f] = *(const v4i *)(fx + xrow16 + ii * 16 * BK + koff16[kk][ii & 1]);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        ix = ix1, iw = iw1;
    }

    // ---- epilogue ----------------------------------------------------------------------
    // The loads issued past the last tile move no data from memory but still zero-fill their LDS
    // destination: they must have landed before the stages are reused.
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __builtin_amdgcn_s_barrier();  // every wave is done with the stages: the epilogue operands may go where they were
    if constexpr (SPLITK) {
        // Every slice leaves its sums in memory (in register order: thread t of the workgroup writes 16 bytes at
        // 16 (q NT + t) of its block for its q-th group of four) and counts itself in; the slice that arrives
        // last adds the others' to its own and carries on into the epilogue, the others are done.  Integer sums:
        // the order of the slices changes nothing.  Nobody waits for anybody.
        // The sums travel with sc1 (agent-coherent) stores and loads, which go to the level where all eight L2s
        // agree, and the count is taken once this workgroup's stores are acknowledged: no cache-wide write-back or
        // invalidate, which a release/acquire fence pair at agent scope would cost every workgroup on the XCD.
        __shared__ unsigned s_arrived;
        const int T = tiles_m * tiles_n, tile = __builtin_amdgcn_readfirstlane(wg_id % T);
        constexpr int QUADS = MI * NJ * QPB;
        static_assert(QUADS % 4 == 0, "the partial sums are read back four quads at a time");
        int *mine = g.partials + ((int64_t)slice * T + tile) * (BM * BN);
#pragma unroll
        for (int qd = 0; qd < QUADS; ++qd) {
            const int i = qd / (NJ * QPB), j = qd / QPB % NJ;
            const v4i o = quad_of(i, j, qd % QPB);
            // (s_nop 1: a 16-byte store reads its data registers after it has issued, and the two wait states that keep a
            // following vector instruction from overwriting them are the compiler's job, which it cannot do for an
            // instruction it does not see)
            asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(mine + ((int64_t)qd * C::NT + tid) * 4), "v"(o) : "memory");
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            unsigned word = __hip_atomic_load(g.arrivals + tile, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), next;
            uint32_t before;
            do {
                next = splitk_arrive(word, g.splitk_tag, (uint32_t)g.splits, &before);
            } while (!__hip_atomic_compare_exchange_strong(g.arrivals + tile, &word, next, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                           __HIP_MEMORY_SCOPE_AGENT));
            s_arrived = before;
        }
        __syncthreads();
        if (s_arrived + 1 != (unsigned)g.splits) return;
        for (int o = 0; o < g.splits; ++o) {
            if (o == slice) continue;
            const int *theirs = g.partials + ((int64_t)o * T + tile) * (BM * BN);
#pragma unroll
            for (int q0 = 0; q0 < QUADS; q0 += 4) {
                v4i v[4];
                const int *p0 = theirs + ((int64_t)q0 * C::NT + tid) * 4;
                asm volatile("global_load_dwordx4 %0, %4, off sc1\n\tglobal_load_dwordx4 %1, %5, off sc1\n\t"
                             "global_load_dwordx4 %2, %6, off sc1\n\tglobal_load_dwordx4 %3, %7, off sc1\n\ts_waitcnt vmcnt(0)"
                             : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3])
                             : "v"(p0), "v"(p0 + C::NT * 4), "v"(p0 + 2 * C::NT * 4), "v"(p0 + 3 * C::NT * 4)
                             : "memory");
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int qd = q0 + u, i = qd / (NJ * QPB), j = qd / QPB % NJ;
                    quad_add(i, j, qd % QPB, v[u]);
                }
            }
        }
        if (tid == 0) __hip_atomic_store(g.arrivals + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    }
    if constexpr (OUT != OUT_I32) {
        if (!gws) ws_one = ws_host;
#pragma unroll
        for (int u = 0; u < XS_PER; ++u) {
            const int t = tid + u * C::NT;
            if (t < BM) s_xs[t] = (m0 + t < gM) ? xs_r[u] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < WS_PER; ++u) {
            const int t = tid + u * C::NT;
            if (t < BN) {
                const bool in = n0 + t < gN;
                float bv = 0.0f;
                if (gbias && in) {
                    if (bias_dtype == I8F_F32) bv = __uint_as_float(bias_r[u]);
                    else if (bias_dtype == I8F_BF16) bv = bf16_bits_to_f32(bias_r[u]);
                    else bv = f16_bits_to_f32(bias_r[u]);
                }
                s_ws[t] = row_scale ? (in ? ws_r[u] : 0.0f) : ws_one;
                s_bias[t] = bv;
            }
        }
    }
    if constexpr (SIDE) {
        // side_t rows m0 ... and side_b rows n0 ... of the tile, 16 bytes (8 ranks) per thread and step; rows beyond
        // the matrix repeat its last row (their outputs are not stored)
        const int cpr = g.side_rank >> 3;  // 16-byte pieces per row
        for (int c = tid; c < (BM + BN) * cpr; c += C::NT) {
            const int row = c / cpr, cc = c - row * cpr;
            const char *src = row < BM ? (const char *)g.side_t + (int64_t)min(m0 + row, gM - 1) * g.side_rank * 2
                                       : (const char *)g.side_b + (int64_t)min(n0 + row - BM, gN - 1) * g.side_rank * 2;
            *(uint4 *)(smem + SIDE_OFF + row * SIDE_PITCH + cc * 16) = *(const uint4 *)(src + cc * 16);
        }
    }
    __syncthreads();  // the stages are dead (reused as per-wave transpose buffers), the operands staged
    char *ebuf = smem + wave * WAVE_BYTES;
    [[maybe_unused]] const char *const s_side_t = smem + SIDE_OFF + (wm * C::WTM) * SIDE_PITCH;
    [[maybe_unused]] const char *const s_side_b = smem + SIDE_OFF + (BM + wn * C::WTN) * SIDE_PITCH;

    // scale, bias, round: the flags are wave-uniform, so the variant is chosen once
    // scale, bias, round.  The per-column operands (4 consecutive n per lane and MFMA block) are
    // fetched from LDS into registers once, in front of the strips: fetched inside, every group of
    // four values would wait for an LDS round trip.
    // the activation scales of the lane's rows of strip i: one row, or (16x16x64) one per 16-row half
    auto strip_scales = [&](int i, float (&xs2)[2]) {
        xs2[0] = s_xs[wm * C::WTM + i * 32 + quad_m(0)];
        xs2[1] = M16 ? s_xs[wm * C::WTM + i * 32 + quad_m(1)] : xs2[0];
    };
    auto convert_strip = [&](int i, char *dst_rows, const auto &wr, const auto &br, auto ORDER, auto ROW, auto BIAS) {
        float xs2[2];
        strip_scales(i, xs2);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
#pragma unroll
            for (int qd = 0; qd < QPB; ++qd) {
                const int nl = j * CB + quad_n(qd);  // first of 4 consecutive n held by this lane
                const v4i q4 = quad_of(i, j, qd);
                const int a4[4] = {q4.x, q4.y, q4.z, q4.w};
                epilogue_quad<OUT, decltype(ORDER)::value, decltype(ROW)::value, decltype(BIAS)::value>(
                    a4, xs2[M16 ? qd : 0], wr[j][quad_c(qd)], br[j][quad_c(qd)], dst_rows + quad_m(qd) * PITCH + nl * OB);
            }
        }
    };
    using T_ = std::true_type;
    using F_ = std::false_type;
    using O0 = std::integral_constant<int, I8F_EPI_TORCH>;
    using O1 = std::integral_constant<int, I8F_EPI_FUSED>;
    const int variant = (g.order == I8F_EPI_FUSED ? 4 : 0) | (row_scale ? 2 : 0) | (gbias ? 1 : 0);

    // The whole epilogue is instantiated once per variant and the variant is chosen ONCE, so that
    // the instructions a wave executes are contiguous in memory (the epilogue runs once per wave,
    // straight from a cold instruction cache).
    // With more than 8 waves a wave has fewer registers than the accumulators plus the operands of
    // all its columns need: the column operands are then fetched per column block, and a block is
    // converted for all staged strips before the next one is fetched.
    // (the variant with a low-rank side branch needs registers for its operands: per-block fetches as well)
    constexpr bool PRELOAD_ALL = C::NT <= 512 && !SIDE;
    auto run_epilogue = [&](auto ORDER, auto ROW, auto BIAS) {
        constexpr int NPRE = PRELOAD_ALL ? NJ : 1;
        float4 wr[NPRE][NQ], br[NPRE][NQ];
        auto fetch_cols = [&](int j, float4 (&wj)[NQ], float4 (&bj)[NQ]) __attribute__((always_inline)) {
#pragma unroll
            for (int c = 0; c < NQ; ++c) {
                const int nl = wn * C::WTN + j * CB + quad_n(c);
                if constexpr (decltype(ROW)::value) wj[c] = *(const float4 *)&s_ws[nl];
                else wj[c] = make_float4(s_ws[0], s_ws[0], s_ws[0], s_ws[0]);
                if constexpr (decltype(BIAS)::value) bj[c] = *(const float4 *)&s_bias[nl];
                else bj[c] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
        };
        if constexpr (OUT != OUT_I32 && PRELOAD_ALL) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) fetch_cols(j, wr[j], br[j]);
        }
#pragma unroll
        for (int i0 = 0; i0 < MI; i0 += EPI_STRIPS) {
#pragma unroll
            for (int is = 0; is < EPI_STRIPS; ++is) {
                const int i = i0 + is;
                char *rows = ebuf + is * 32 * PITCH;
                if constexpr (OUT == OUT_I32) {
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
#pragma unroll
                        for (int qd = 0; qd < QPB; ++qd) {
                            const int nl = j * CB + quad_n(qd);
                            *(v4i *)(rows + quad_m(qd) * PITCH + nl * 4) = quad_of(i, j, qd);
                        }
                } else if constexpr (PRELOAD_ALL) {
                    convert_strip(i, rows, wr, br, ORDER, ROW, BIAS);
                }
            }
            if constexpr (OUT != OUT_I32 && !PRELOAD_ALL) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    fetch_cols(j, wr[0], br[0]);
                    // side branch: the rank-r product of this block on the matrix cores, with the same
                    // operand roles as the main product (rows n from side_b, columns m from side_t), so that
                    // the result has the accumulators' layout
                    // (16x16x64 form: two 16 x 16 products per block, a lane's fragment being 4 ranks of one row)
                    constexpr int RMAX = 64;
                    [[maybe_unused]] v4i bfr[M16 ? 1 : RMAX / 16];
                    [[maybe_unused]] v2i bfr16[RMAX / 16];
                    if constexpr (SIDE && !M16) {
#pragma unroll
                        for (int ks = 0; ks < RMAX / 16; ++ks)
                            if (ks * 16 < g.side_rank)
                                bfr[ks] = *(const v4i *)(s_side_b + (j * 32 + l32) * SIDE_PITCH + (ks * 16 + lhalf * 8) * 2);
                    }
                    if constexpr (SIDE && M16) {
#pragma unroll
                        for (int ks = 0; ks < RMAX / 16; ++ks)
                            if (ks * 16 < g.side_rank)
                                bfr16[ks] = *(const v2i *)(s_side_b + (j * 16 + l16) * SIDE_PITCH + (ks * 16 + lq * 4) * 2);
                    }
#pragma unroll
                    for (int is = 0; is < EPI_STRIPS; ++is) {
                        const int i = i0 + is;
                        float xs2[2];
                        strip_scales(i, xs2);
                        [[maybe_unused]] float sd[16];
                        constexpr int SDT = OUT == OUT_F16 ? I8F_F16 : I8F_BF16;
                        if constexpr (SIDE && !M16) {
                            v16f sacc;
#pragma unroll
                            for (int r = 0; r < 16; ++r) sacc[r] = 0.0f;
#pragma unroll
                            for (int ks = 0; ks < RMAX / 16; ++ks) {
                                if (ks * 16 < g.side_rank) {
                                    const v4i tfr = *(const v4i *)(s_side_t + (i * 32 + l32) * SIDE_PITCH + (ks * 16 + lhalf * 8) * 2);
                                    sacc = side_mfma<OUT>(bfr[ks], tfr, sacc);
                                }
                            }
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                float v = round_to_dtype<SDT>(sacc[r]);
                                if (g.side_has_alpha) v = round_to_dtype<SDT>(v * g.side_alpha);
                                sd[r] = v;
                            }
                        }
                        if constexpr (SIDE && M16) {
#pragma unroll
                            for (int u = 0; u < 2; ++u) {
                                v4f sacc = (v4f)0.0f;
#pragma unroll
                                for (int ks = 0; ks < RMAX / 16; ++ks) {
                                    if (ks * 16 < g.side_rank) {
                                        const v2i tfr = *(const v2i *)(s_side_t + (i * 32 + u * 16 + l16) * SIDE_PITCH + (ks * 16 + lq * 4) * 2);
                                        sacc = side_mfma16<OUT>(bfr16[ks], tfr, sacc);
                                    }
                                }
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    float y = round_to_dtype<SDT>(sacc[e]);
                                    if (g.side_has_alpha) y = round_to_dtype<SDT>(y * g.side_alpha);
                                    sd[4 * u + e] = y;
                                }
                            }
                        }
#pragma unroll
                        for (int qd = 0; qd < QPB; ++qd) {
                            const int nl = j * CB + quad_n(qd);
                            const v4i q4 = quad_of(i, j, qd);
                            const int a4[4] = {q4.x, q4.y, q4.z, q4.w};
                            epilogue_quad<OUT, decltype(ORDER)::value, decltype(ROW)::value, decltype(BIAS)::value, SIDE>(
                                a4, xs2[M16 ? qd : 0], wr[0][quad_c(qd)], br[0][quad_c(qd)], ebuf + (is * 32 + quad_m(qd)) * PITCH + nl * OB,
                                SIDE ? &sd[4 * qd] : nullptr);
                        }
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
            // read the staged rows back row-contiguously and store 16 bytes per lane
            constexpr int CPO = ROW_BYTES / 16;      // chunks per output row
            constexpr int EPCO = 16 / OB;            // output elements per chunk
            constexpr int PASSES = EPI_STRIPS * 32 * CPO / 64;
#pragma unroll
            for (int p = 0; p < PASSES; ++p) {
                const int id = p * 64 + lane;
                const int row = id / CPO, cc = id % CPO;
                const uint4 val = *(const uint4 *)(ebuf + row * PITCH + cc * 16);
                const int mm = m0 + wm * C::WTM + i0 * 32 + row;
                const int nn = n0 + wn * C::WTN + cc * EPCO;
                if (mm < gM && nn < gN)
                {
                    const int64_t off = ((int64_t)mm * gN + nn) * OB;
                    uint4 v = val;
                    if (ggate)
                        v = mul_rounded<OUT>(v, *(const uint4 *)((const char *)ggate + ((int64_t)((uint32_t)mm / (uint32_t)ggate_rows) * gN + nn) * OB));
                    if (gaddend) v = add_rounded<OUT>(v, *(const uint4 *)((const char *)gaddend + off));
                    stream_store16((char *)gout + off, v);
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    };
    if constexpr (OUT == OUT_I32) {
        run_epilogue(O0{}, F_{}, F_{});
    } else {
        switch (variant) {
        case 0: run_epilogue(O0{}, F_{}, F_{}); break;
        case 1: run_epilogue(O0{}, F_{}, T_{}); break;
        case 2: run_epilogue(O0{}, T_{}, F_{}); break;
        case 3: run_epilogue(O0{}, T_{}, T_{}); break;
        case 4: run_epilogue(O1{}, F_{}, F_{}); break;
        case 5: run_epilogue(O1{}, F_{}, T_{}); break;
        case 6: run_epilogue(O1{}, T_{}, F_{}); break;
        default: run_epilogue(O1{}, T_{}, T_{}); break;
        }
    }
}

template <class C, int OUT, bool KTAIL, bool SIDE = false, bool SPLITK = false>
__global__ __launch_bounds__(C::NT) void gemm_i8_kernel(const int8_t *gx, const int8_t *gw, int gM, int gN, int gK, int tiles_m, int tiles_n,
                                                        const float *gxs, const float *gws, const void *gbias, int flags,
                                                        const GemmArgs g) {
    gemm_i8_body<C, OUT, KTAIL, SIDE, SPLITK>(gx, gw, gM, gN, gK, tiles_m, tiles_n, gxs, gws, gbias, flags, g, (int)blockIdx.x, g.out,
                                              g.addend, g.ws_host, g.gate, g.gate_rows);
}

// Several problems of one layer shape (N, K, scale mode, dtypes) with their own activations, weights and outputs in
// one launch: the tiles of a transformer block's image and text stream for the same projection.  Workgroup b
// belongs to the group whose range of tiles holds b and works as workgroup b - first_tile of that problem.  Where the
// small problem's tiles fit into the CUs that the large one's last round leaves idle (192 + 24 tiles of 256 x 256 for
// 4096 and 512 tokens into 3072 columns), the small problem costs nothing.
constexpr int MAX_GEMM_GROUPS = 4;
struct GemmGroups {
    const int8_t *x[MAX_GEMM_GROUPS], *w[MAX_GEMM_GROUPS];
    const float *xs[MAX_GEMM_GROUPS], *ws[MAX_GEMM_GROUPS];
    const void *bias[MAX_GEMM_GROUPS], *addend[MAX_GEMM_GROUPS], *gate[MAX_GEMM_GROUPS];
    void *out[MAX_GEMM_GROUPS];
    float ws_host[MAX_GEMM_GROUPS];
    int M[MAX_GEMM_GROUPS], tiles_m[MAX_GEMM_GROUPS], gate_rows[MAX_GEMM_GROUPS];
    int first_tile[MAX_GEMM_GROUPS + 1];  // [n] = all tiles
    int n;
};

template <class C, int OUT>
__global__ __launch_bounds__(C::NT) void gemm_i8_grouped_kernel(int gN, int gK, int tiles_n, int flags, const GemmGroups gg, const GemmArgs g) {
    int grp = 0;
#pragma unroll
    for (int i = 1; i < MAX_GEMM_GROUPS; ++i)
        if (i < gg.n && (int)blockIdx.x >= gg.first_tile[i]) grp = i;
    grp = __builtin_amdgcn_readfirstlane(grp);
    gemm_i8_body<C, OUT, false>(gg.x[grp], gg.w[grp], gg.M[grp], gN, gK, gg.tiles_m[grp], tiles_n, gg.xs[grp], gg.ws[grp], gg.bias[grp],
                                flags, g, (int)blockIdx.x - gg.first_tile[grp], gg.out[grp], gg.addend[grp], gg.ws_host[grp], gg.gate[grp],
                                gg.gate_rows[grp]);
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
        if (g.gate) t = round_to_dtype<DT>(t) * load_as_f32<DT>(g.gate, (int64_t)(m / g.gate_rows) * g.N + n);
        if (g.addend) t = round_to_dtype<DT>(t) + load_as_f32<DT>(g.addend, idx);
        store_from_f32<DT>(g.out, idx, t);
    }
}

// tile configurations.  The one-workgroup-per-CU tiles run on v_mfma_i32_16x16x64_i8: on realistic operands the chip is at
// its power limit, and the same multiply-accumulates cost less energy in that form than as v_mfma_i32_32x32x32_i8 (with
// nothing but MFMAs in a loop, operands in registers, the chip sustains 3.9 POP/s against 3.2; on all-zero operands both
// reach 4.9), so the clock settles higher.  The shorter instruction covers fewer other instructions, which is why that form
// deals its LDS reads out one by one; the 128 x 128 tile and the few-tile configurations (one wave per SIMD, bound by the
// global->LDS path) lose more to that than they gain and keep the 32x32x32 form.
#ifndef I8F_WST
#define I8F_WST 3
#endif
using CfgBig = Cfg<256, 256, 128, 2, 4, 2, 6, 0x4400, 16, I8F_WST>;  // 8 waves, 2 X and 3 W stages of 32 KB (all of the LDS), one workgroup per CU
using CfgB192 = Cfg<256, 192, 128, 4, 2, 2, 6, 0x4300, 16, I8F_WST>;  // 8 waves of 64 x 96, 2 x 32 + 3 x 24 KB: fills 256 CUs where 256 x 256 leaves a partial round
using CfgMid = Cfg<128, 128, 128, 2, 2, 2, 8>;   // 4 waves, 2 x 32 KB stages, two workgroups per CU (10 % slower with the 16x16x64 MFMA: 32x32x32)
using CfgTall = Cfg<288, 256, 128, 3, 4, 2, 8, 0, 16>;  // 12 waves of 96 x 64, 2 x 72 KB stages
using CfgWide = Cfg<256, 288, 128, 4, 3, 2, 8, 0, 16>;  // 12 waves of 64 x 96, the same transposed
// (Workgroups beyond the tile count that do nothing but touch, a few K-tiles ahead, the W lines the tiles of their XCD are
// about to request -- they land on the CUs a 216-tile launch leaves idle, since a workgroup of this kernel takes a CU's
// whole LDS -- were measured and are not kept: 39.8 us against 38.7 us at 4608 x 3072 x 3072, 130.3 against 125.2 us at
// K = 12288.  The misses they take off the busy CUs do not pay for what their requests add to the XCD's L2 queues.)
// (A 288 x 192 tile of twelve 96 x 48 waves, which covers 4608 x 3072 in exactly 256 workgroups, was measured and is not
// kept: 42.9 us against 37.7 us for the 216 tiles of 256 x 256.  It moves 11 % more bytes per multiply-accumulate through a
// load path that is already the bound, and with all 256 CUs multiplying the clock settles 8 % lower.)
// Outputs of few tiles: about one workgroup per CU, so nothing hides the latency of the global->LDS
// loads (the weight comes from HBM: a model's weights are far larger than the caches) but the loads in
// flight; four stages instead of two, and the largest tile that still gives 192 workgroups.
using CfgW96 = Cfg<256, 96, 128, 8, 1, 3, 8, 0, 16>;      // 8 waves of 32 x 96, 3 x 44 KB stages
using CfgMidDeep = Cfg<128, 128, 128, 2, 2, 4, 8>;
using CfgM96Deep = Cfg<128, 96, 128, 4, 1, 4, 8>;
using CfgS64Deep = Cfg<128, 64, 128, 2, 2, 4, 8>;
using CfgT64Deep = Cfg<64, 64, 128, 2, 2, 4, 8>;
template <class C, int OUT>
int launch_cfg(GemmArgs &g, hipStream_t st) {
    g.tiles_m = (g.M + C::BM - 1) / C::BM;
    g.tiles_n = (g.N + C::BN - 1) / C::BN;
    const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
    const int flags = (g.row_scale ? 1 : 0) | (g.bias_dtype << 1);  // what the prologue wants to know of the epilogue
    if (g.side_t) {  // validated by the entry point: K % BK == 0 here
        if constexpr (OUT == OUT_BF16 || OUT == OUT_F16) {
            hipLaunchKernelGGL((gemm_i8_kernel<C, OUT, false, true>), dim3((unsigned)tiles), dim3(C::NT), 0, st, g.x, g.w, g.M, g.N,
                               g.K, g.tiles_m, g.tiles_n, g.xs, g.ws, g.bias, flags, g);
            return check_launch();
        } else {
            return I8F_ERR_UNSUPPORTED;
        }
    }
    if constexpr (C::STAGES == 4) {  // the K split exists for the few-tile configurations
        if (g.splits > 1) {
            const unsigned wgs = (unsigned)(tiles * g.splits);
            if (g.K % C::BK)
                hipLaunchKernelGGL((gemm_i8_kernel<C, OUT, true, false, true>), dim3(wgs), dim3(C::NT), 0, st, g.x, g.w, g.M, g.N, g.K,
                                   g.tiles_m, g.tiles_n, g.xs, g.ws, g.bias, flags, g);
            else
                hipLaunchKernelGGL((gemm_i8_kernel<C, OUT, false, false, true>), dim3(wgs), dim3(C::NT), 0, st, g.x, g.w, g.M, g.N, g.K,
                                   g.tiles_m, g.tiles_n, g.xs, g.ws, g.bias, flags, g);
            return check_launch();
        }
    }
    if (g.K % C::BK)
        hipLaunchKernelGGL((gemm_i8_kernel<C, OUT, true>), dim3((unsigned)tiles), dim3(C::NT), 0, st, g.x, g.w, g.M, g.N, g.K,
                           g.tiles_m, g.tiles_n, g.xs, g.ws, g.bias, flags, g);
    else
        hipLaunchKernelGGL((gemm_i8_kernel<C, OUT, false>), dim3((unsigned)tiles), dim3(C::NT), 0, st, g.x, g.w, g.M, g.N, g.K,
                           g.tiles_m, g.tiles_n, g.xs, g.ws, g.bias, flags, g);
    return check_launch();
}

enum Tile { TILE_BIG, TILE_B192, TILE_MID, TILE_TALL, TILE_WIDE, TILE_W96, TILE_MID_DEEP, TILE_M96_DEEP, TILE_S64_DEEP, TILE_T64_DEEP };

// The tile configuration an M x N output takes (K does not enter).
inline Tile choose_tile(int64_t M, int64_t N) {
    // With 256-row tiles a CU holds one workgroup at a time, so a launch costs about
    // ceil(tiles / 256 CUs) rounds of one tile's work; per operation the 256 x 192 tile is about 8 %
    // dearer than 256 x 256 (more LDS and global->LDS traffic per MFMA) and the 288 x 256 tile of
    // twelve waves, or 256 x 288, about 2 % (they pay where they save a round: 4608 x 12288 takes 768
    // tiles of 288 x 256, three rounds, instead of 864 of 256 x 256, four; 4096 x 9216 takes 512 of
    // 256 x 288, two rounds).  Outputs of fewer than 128
    // such tiles take 128 x 128 tiles with two stages if that gives at least one workgroup per CU,
    // else the four-stage configurations above.
    const int64_t CUS = 256;
    auto rounds_cost = [&](int bm, int bn, int per_op_cost) {
        const int64_t tiles = (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
        return ((tiles + CUS - 1) / CUS) * (int64_t)bm * bn * per_op_cost;
    };
    const int64_t big_tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
    if (big_tiles < 128) {
        const int64_t mid_tiles = (int64_t)((M + 127) / 128) * ((N + 127) / 128);
        if (mid_tiles >= CUS) {
            // Two 128 x 128 tiles to a CU fetch 2 x 256 rows per K-step, one 256 x 96 tile 352: the
            // narrow tile wins where it still covers the output in one round (512 x 12288: 256 tiles).
            const int64_t w96_tiles = (int64_t)((M + 255) / 256) * ((N + 95) / 96);
            const int64_t f_w96 = ((w96_tiles + CUS - 1) / CUS) * (256 + 96);
            const int64_t f_mid2 = ((mid_tiles + 2 * CUS - 1) / (2 * CUS)) * 2 * (128 + 128);
            if (f_w96 < f_mid2) return TILE_W96;
            return TILE_MID;
        }
        // Few tiles: the global->LDS path of a CU is what bounds these shapes, so a configuration costs
        // the bytes its busiest CU has to fetch: (BM + BN) per K-step times the tiles that CU gets.
        // Ties go to the larger tile (less traffic in total).
        auto fetch_cost = [&](int bm, int bn) {
            const int64_t tiles = (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
            return ((tiles + CUS - 1) / CUS) * (bm + bn);
        };
        const int64_t f_mid = fetch_cost(128, 128), f_96 = fetch_cost(128, 96), f_s64 = fetch_cost(128, 64), f_t64 = fetch_cost(64, 64);
        const int64_t f_min = std::min(std::min(f_mid, f_96), std::min(f_s64, f_t64));
        if (f_mid == f_min) return TILE_MID_DEEP;
        if (f_96 == f_min) return TILE_M96_DEEP;
        if (f_s64 == f_min) return TILE_S64_DEEP;
        return TILE_T64_DEEP;
    }
    const int64_t c_big = rounds_cost(256, 256, 100), c_192 = rounds_cost(256, 192, 108);
    const int64_t c_tall = rounds_cost(288, 256, 102), c_wide = rounds_cost(256, 288, 102);
    // 128 x 128 tiles, two workgroups to a CU: 41 % dearer per operation, but nothing is wasted on a
    // ragged M (640 x 12288: one round of 480 of them against 192 tiles of 256 x 192)
    const int64_t mid_all = (int64_t)((M + 127) / 128) * ((N + 127) / 128);
    const int64_t c_mid = ((mid_all + 2 * CUS - 1) / (2 * CUS)) * 2 * 128 * 128 * 141;
    const int64_t c_min = std::min(std::min(std::min(c_big, c_192), std::min(c_tall, c_wide)), c_mid);
    if (c_big == c_min) return TILE_BIG;
    if (c_mid == c_min) return TILE_MID;
    if (c_tall == c_min) return TILE_TALL;
    if (c_wide == c_min) return TILE_WIDE;
    return TILE_B192;
}

// Workspace of the K split: arrival counters (one per tile, at most 1024), then the partial sums of at most 256
// workgroups of at most 128 x 128 outputs.
constexpr int64_t SPLITK_COUNTER_BYTES = 4096, SPLITK_WORKSPACE_BYTES = SPLITK_COUNTER_BYTES + 256ll * 128 * 128 * 4;

// Few tiles and a long K: the tile's K range is dealt over `splits` workgroups, which exchange their sums through
// memory (integer sums, so the result is the same).  It pays where it fills idle CUs and a slice still has a long
// loop: measured with weights from HBM, 512 x 3072 x 12288 42 -> 34 us, 256 x 3072 x 12288 33 -> 26 us,
// 64 x 3072 x 12288 33 -> 15 us, nothing at K = 6144.  A candidate costs what its busiest CU fetches,
// (K / splits) (BM + BN), plus 7 splits BM BN for the exchange (fitted to those measurements); one round of
// workgroups at most, slices of at least 2048.
inline void choose_split(int64_t M, int64_t N, int64_t K, Tile &t, int &splits) {
    splits = 1;
    if (K < 10240) return;
    if (t != TILE_MID_DEEP && t != TILE_M96_DEEP && t != TILE_S64_DEEP && t != TILE_T64_DEEP) return;
    const int64_t CUS = 256;
    struct Cand { Tile tile; int bm, bn; };
    const Cand cands[4] = {{TILE_MID_DEEP, 128, 128}, {TILE_M96_DEEP, 128, 96}, {TILE_S64_DEEP, 128, 64}, {TILE_T64_DEEP, 64, 64}};
    int64_t best = -1;
    for (const Cand &c : cands) {
        const int64_t tiles = ((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn);
        if (c.tile == t) {
            const int64_t cost = ((tiles + CUS - 1) / CUS) * K * (c.bm + c.bn);
            if (best < 0 || cost < best) best = cost, splits = 1;  // (t stays)
        }
    }
    Tile keep = t;
    for (const Cand &c : cands) {
        const int64_t tiles = ((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn);
        if (tiles > CUS / 2 || tiles > SPLITK_COUNTER_BYTES / 4) continue;
        int64_t sp = CUS / tiles;
        if (sp > 8) sp = 8;
        while (sp > 1 && K / sp < 2048) --sp;
        if (sp <= 1) continue;
        const int64_t cost = (K / sp) * (c.bm + c.bn) + 7 * sp * c.bm * c.bn;
        if (cost < best) best = cost, keep = c.tile, splits = (int)sp;
    }
    t = keep;
}

template <int OUT>
int launch_tile(Tile t, GemmArgs &g, hipStream_t st) {
    switch (t) {
    case TILE_BIG: return launch_cfg<CfgBig, OUT>(g, st);
    case TILE_B192: return launch_cfg<CfgB192, OUT>(g, st);
    case TILE_MID: return launch_cfg<CfgMid, OUT>(g, st);
    case TILE_TALL: return launch_cfg<CfgTall, OUT>(g, st);
    case TILE_WIDE: return launch_cfg<CfgWide, OUT>(g, st);
    case TILE_W96: return launch_cfg<CfgW96, OUT>(g, st);
    case TILE_MID_DEEP: return launch_cfg<CfgMidDeep, OUT>(g, st);
    case TILE_M96_DEEP: return launch_cfg<CfgM96Deep, OUT>(g, st);
    case TILE_S64_DEEP: return launch_cfg<CfgS64Deep, OUT>(g, st);
    default: return launch_cfg<CfgT64Deep, OUT>(g, st);
    }
}

template <class C>
void tile_dims(int *bm, int *bn, int *stages) {
    *bm = C::BM, *bn = C::BN, *stages = C::STAGES;
}

template <int OUT>
int launch(GemmArgs &g, hipStream_t st) {
    const int ob = OutElem<OUT>::BYTES;
    const bool aligned = (g.K % 16 == 0) && (g.N % 8 == 0) && ((uintptr_t)g.x % 16 == 0) && ((uintptr_t)g.w % 16 == 0) &&
                         ((uintptr_t)g.out % 16 == 0) && ((int64_t)g.N * g.K < (1ll << 31)) &&
                         (!g.ws || !g.row_scale || (uintptr_t)g.ws % 16 == 0) &&
                         (!g.bias || (uintptr_t)g.bias % 16 == 0) && (!g.addend || (uintptr_t)g.addend % 16 == 0) &&
                         (!g.gate || (uintptr_t)g.gate % 16 == 0);
    // The buffer descriptors address 2^31 bytes: more activations than that go in row blocks.
    if (aligned && (int64_t)g.M * g.K >= (1ll << 31) && (int64_t)256 * g.K < (1ll << 31)) {
        const int rows_per = (int)((((1ll << 31) - 1) / g.K) / 256 * 256);
        for (int64_t m0 = 0; m0 < g.M; m0 += rows_per) {
            GemmArgs sub = g;
            sub.M = (int)(g.M - m0 < rows_per ? g.M - m0 : rows_per);
            sub.x = g.x + m0 * g.K;
            if (g.xs) sub.xs = g.xs + m0;
            sub.out = (char *)g.out + m0 * g.N * ob;
            if (g.addend) sub.addend = (const char *)g.addend + m0 * g.N * ob;
            if (g.gate) {  // the row blocks must start on a gate boundary for the sub-problem to index its vectors from 0
                if (m0 % g.gate_rows) return I8F_ERR_UNSUPPORTED;
                sub.gate = (const char *)g.gate + (m0 / g.gate_rows) * g.N * ob;
            }
            if (g.side_t) sub.side_t = (const char *)g.side_t + m0 * g.side_rank * 2;
            if (int rc = launch<OUT>(sub, st)) return rc;
        }
        return I8F_OK;
    }
    const bool fast = aligned && ((int64_t)g.M * g.K < (1ll << 31));
    if (g.side_t && (!fast || g.K % 128 || (uintptr_t)g.side_t % 16 || (uintptr_t)g.side_b % 16)) return I8F_ERR_UNSUPPORTED;
    if (!fast) {
        const int64_t total = (int64_t)g.M * g.N;
        hipLaunchKernelGGL((gemm_i8_generic_kernel<OUT>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, g);
        return check_launch();
    }
    Tile t = choose_tile(g.M, g.N);
    int splits = 1;
    if (g.partials && !g.side_t) choose_split(g.M, g.N, g.K, t, splits);
    g.splits = splits;
    if (splits > 1) {
        static std::atomic<uint32_t> launches{0};
        g.splitk_tag = splitk_tag(launches.fetch_add(1, std::memory_order_relaxed));
    }
    return launch_tile<OUT>(t, g, st);
}

template <class C, int OUT>
int launch_cfg_grouped(const GemmArgs *gs, int n, hipStream_t st) {
    GemmGroups gg{};
    gg.n = n;
    const int tiles_n = (gs[0].N + C::BN - 1) / C::BN;
    int first = 0;
    for (int i = 0; i < n; ++i) {
        gg.x[i] = gs[i].x, gg.w[i] = gs[i].w, gg.xs[i] = gs[i].xs, gg.ws[i] = gs[i].ws, gg.bias[i] = gs[i].bias;
        gg.addend[i] = gs[i].addend, gg.out[i] = gs[i].out, gg.ws_host[i] = gs[i].ws_host, gg.M[i] = gs[i].M;
        gg.gate[i] = gs[i].gate, gg.gate_rows[i] = gs[i].gate ? gs[i].gate_rows : 1;
        gg.tiles_m[i] = (gs[i].M + C::BM - 1) / C::BM;
        gg.first_tile[i] = first;
        first += gg.tiles_m[i] * tiles_n;
    }
    for (int i = n; i <= MAX_GEMM_GROUPS; ++i) gg.first_tile[i] = first;
    const int flags = (gs[0].row_scale ? 1 : 0) | (gs[0].bias_dtype << 1);
    hipLaunchKernelGGL((gemm_i8_grouped_kernel<C, OUT>), dim3((unsigned)first), dim3(C::NT), 0, st, gs[0].N, gs[0].K, tiles_n, flags, gg, gs[0]);
    return check_launch();
}

// Estimated shader cycles of one launch, for the choice between one launch for a group of problems and one launch per
// problem; the constants are this kernel's measured figures.  A one-workgroup-per-CU tile costs its rounds over the 256
// CUs times K-tiles times the time of a K-tile (2 970 cycles for 256 x 256, the others in proportion to their area and
// their relative cost per operation, as choose_tile prices them); the few-tile configurations cost what their busiest
// CU fetches at 33 bytes per cycle (with the K split: the model of choose_split); every launch 12 000 cycles of launch,
// prologue and epilogue.
constexpr int64_t LAUNCH_CYCLES = 12000;
inline void tile_shape(Tile t, int *bm, int *bn) {
    int st = 0;
    switch (t) {
    case TILE_BIG: tile_dims<CfgBig>(bm, bn, &st); break;
    case TILE_B192: tile_dims<CfgB192>(bm, bn, &st); break;
    case TILE_MID: tile_dims<CfgMid>(bm, bn, &st); break;
    case TILE_TALL: tile_dims<CfgTall>(bm, bn, &st); break;
    case TILE_WIDE: tile_dims<CfgWide>(bm, bn, &st); break;
    case TILE_W96: tile_dims<CfgW96>(bm, bn, &st); break;
    case TILE_MID_DEEP: tile_dims<CfgMidDeep>(bm, bn, &st); break;
    case TILE_M96_DEEP: tile_dims<CfgM96Deep>(bm, bn, &st); break;
    case TILE_S64_DEEP: tile_dims<CfgS64Deep>(bm, bn, &st); break;
    default: tile_dims<CfgT64Deep>(bm, bn, &st); break;
    }
}
inline int64_t ktile_cycles(Tile t) {  // of one K-tile of one tile, one-workgroup-per-CU configurations
    int bm, bn;
    tile_shape(t, &bm, &bn);
    const int per_op = t == TILE_BIG ? 100 : (t == TILE_B192 ? 108 : 102);
    return 2970ll * bm * bn * per_op / (256 * 256 * 100);
}
inline int64_t launch_cycles(int64_t tiles, Tile t, int64_t K) { return (tiles + 255) / 256 * ((K + 127) / 128) * ktile_cycles(t) + LAUNCH_CYCLES; }
inline int64_t alone_cycles(int64_t M, int64_t N, int64_t K, bool has_workspace) {
    Tile t = choose_tile(M, N);
    int splits = 1;
    if (has_workspace) choose_split(M, N, K, t, splits);
    int bm, bn;
    tile_shape(t, &bm, &bn);
    const int64_t tiles = ((M + bm - 1) / bm) * ((N + bn - 1) / bn);
    if (t == TILE_BIG || t == TILE_B192 || t == TILE_TALL || t == TILE_WIDE) return launch_cycles(tiles, t, K);
    if (t == TILE_MID) return (tiles + 511) / 512 * 2 * ((K + 127) / 128) * (2970ll * 141 / 400) + LAUNCH_CYCLES;
    if (splits > 1) return ((K / splits) * (bm + bn) + 7ll * splits * bm * bn) / 33 + LAUNCH_CYCLES;
    return (tiles + 255) / 256 * K * (bm + bn) / 33 + LAUNCH_CYCLES;
}

// n problems that share N, K, the scale mode, the dtypes and the operation order (gs[i] differ in M and in their
// pointers).  One launch with the cheapest of the one-workgroup-per-CU tiles where that is estimated to cost less than
// one launch per problem (the small problems' tiles run on CUs that the large problem's last round would leave idle);
// else one launch per problem, as launch() would do it.  The results are the same either way.
template <int OUT>
int launch_group(GemmArgs *gs, int n, hipStream_t st) {
    bool together = n >= 2 && n <= MAX_GEMM_GROUPS;
    for (int i = 0; i < n && together; ++i) {
        const GemmArgs &g = gs[i];
        together = (g.K % 128 == 0) && (g.N % 8 == 0) && ((uintptr_t)g.x % 16 == 0) && ((uintptr_t)g.w % 16 == 0) &&
                   ((uintptr_t)g.out % 16 == 0) && ((int64_t)g.N * g.K < (1ll << 31)) && ((int64_t)g.M * g.K < (1ll << 31)) &&
                   (!g.ws || !g.row_scale || (uintptr_t)g.ws % 16 == 0) && (!g.bias || (uintptr_t)g.bias % 16 == 0) &&
                   (!g.addend || (uintptr_t)g.addend % 16 == 0) && (!g.gate || (uintptr_t)g.gate % 16 == 0) && !g.side_t;
    }
    Tile t = TILE_BIG;
    if (together) {
        const int64_t N = gs[0].N, K = gs[0].K;
        int64_t separate = 0;
        for (int i = 0; i < n; ++i) separate += alone_cycles(gs[i].M, N, K, gs[i].partials != nullptr);
        int64_t best = -1;
        for (Tile c : {TILE_BIG, TILE_B192, TILE_TALL, TILE_WIDE}) {
            int bm, bn;
            tile_shape(c, &bm, &bn);
            int64_t tiles = 0;
            for (int i = 0; i < n; ++i) tiles += ((gs[i].M + bm - 1) / bm) * ((N + bn - 1) / bn);
            const int64_t cost = launch_cycles(tiles, c, K);
            if (best < 0 || cost < best) best = cost, t = c;
        }
        together = best < separate;
    }
    if (!together) {
        for (int i = 0; i < n; ++i)
            if (int rc = launch<OUT>(gs[i], st)) return rc;
        return I8F_OK;
    }
    switch (t) {
    case TILE_BIG: return launch_cfg_grouped<CfgBig, OUT>(gs, n, st);
    case TILE_B192: return launch_cfg_grouped<CfgB192, OUT>(gs, n, st);
    case TILE_TALL: return launch_cfg_grouped<CfgTall, OUT>(gs, n, st);
    default: return launch_cfg_grouped<CfgWide, OUT>(gs, n, st);
    }
}

inline int validate(const int8_t *a, const int8_t *w, int64_t M, int64_t N, int64_t K, const void *out) {
    if (M < 0 || N < 0 || K < 0) return I8F_ERR_INVALID;
    if (M == 0 || N == 0) return I8F_OK;
    if (!out) return I8F_ERR_INVALID;
    if (K > 0 && (!a || !w)) return I8F_ERR_INVALID;
    if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return I8F_ERR_UNSUPPORTED;
    if (M * N >= (1ll << 40)) return I8F_ERR_UNSUPPORTED;
    return I8F_OK;
}

}  // namespace gemm
}  // namespace i8f
