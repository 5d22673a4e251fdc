// Stochastic-rounding LoRA merge into int8 weights, one pass over HBM.
//
//   xs  = delta_f / w_scale                 correctly rounded division (sr_row: how it is obtained)
//   f   = floor(xs);  frac = xs - f
//   dq  = sat8(noise < frac ? f + 1 : f)    strict compare, noise supplied
//   w'  = sat8(w + dq)
//
// (stochastic_round_int8_delta, int8_quant.py:36-62, and the int8 add of
// calculate_weight, :313-316.)  The reference runs this as about a dozen
// elementwise torch launches over [N,K] float/int32 temporaries.
//
// delta_f is either read (10 bytes per element in total) or rebuilt from the
// rank-r factors in registers (6 bytes per element):
//   acc = 0; for j < r: acc = fmaf(up[n,j], down[j,k], acc); delta_f = acc * lora_scale
// The factors are small (r*(N+K) floats) and stay in cache.
#include "i8f_common.hpp"

namespace i8f {
namespace {

struct MergeArgs {
    const int8_t *w;  // nullptr: write dq itself (stochastic_round_int8_delta alone)
    const float *ws;
    float ws_host;
    int row_scale;
    const float *delta;
    const float *up;
    const float *down;
    int rank;
    float lora_scale;
    const float *noise;
    int64_t N, K;
    int8_t *out;
};

// A weight row's scale with what the fast quotient below needs.
struct RowScale {
    float sc, rcp;
    bool fast;
};

__device__ __forceinline__ RowScale row_scale(float sc) {
    RowScale r;
    r.sc = sc;
    r.rcp = 1.0f / sc;                              // correctly rounded
    r.fast = sc >= 0x1p-20f && sc <= 0x1p+20f;      // false for NaN
    return r;
}

// Stochastic rounding of NE elements of one weight row: r[e] = sat8(noise < frac ? floor + 1 : floor) as a float.
//
// The quotient delta / sc is the correctly rounded one.  With y = RN(1/sc) computed once per row, q = delta * y followed by
// two corrections q += RN(delta - sc q) * y (each an fma pair) gives it in five instructions instead of the division's
// eleven: after the first correction q is within one ulp of the quotient, the remainder delta - sc q is then exact, and a
// correction of such a q with a correctly rounded reciprocal rounds correctly (Markstein's theorem) as long as nothing
// overflows or underflows: 2^-20 <= sc <= 2^20 and 2^-102 <= |delta| <= 2^80 make every intermediate a normal number.
// A zero delta gives a zero quotient on either route.  A smaller non-zero delta has |quotient| < 2^-82; whatever the
// corrections make of it (same sign or a zero of either sign, still tiny), floor and compare give the same result as
// for the true quotient when 2^-82 <= noise < 1, which is tested on the noise's bit pattern (so NaN and negative noise
// fail).  A NaN delta gives NaN on either route.  Lanes that fail a test redo their elements with the division.
struct SrGuard {
    float dmax = 0.0f;
    uint32_t nmin = 0xffffffffu, nmax = 0u;
    template <int NE>
    __device__ __forceinline__ void add(const float (&delta)[NE], const float (&noise)[NE]) {
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            dmax = fmaxf(dmax, fabsf(delta[e]));
            const uint32_t nb = __float_as_uint(noise[e]);
            nmin = min(nmin, nb), nmax = max(nmax, nb);
        }
    }
    __device__ __forceinline__ bool fast(const RowScale &rs) const {
        return rs.fast && dmax <= 0x1p+80f && nmin >= 0x16800000u /* 2^-82 */ && nmax < 0x3f800000u /* 1 */;
    }
};

__device__ __forceinline__ float fast_quotient(float delta, const RowScale &rs) {
    float q = delta * rs.rcp;
    float t = __builtin_fmaf(-rs.sc, q, delta);
    q = __builtin_fmaf(t, rs.rcp, q);
    t = __builtin_fmaf(-rs.sc, q, delta);
    return __builtin_fmaf(t, rs.rcp, q);
}

__device__ __forceinline__ float sr_round(float xs, float noise) {
    const float f = floorf(xs);
    const float frac = xs - f;
    const float v = noise < frac ? f + 1.0f : f;
    return fminf(fmaxf(v, -128.0f), 127.0f);  // NaN becomes -128
}

template <int NE>
__device__ __forceinline__ void sr_row(const float (&delta)[NE], const float (&noise)[NE], const RowScale &rs, float (&r)[NE]) {
    float xs[NE];
    SrGuard g;
    g.add(delta, noise);
#pragma unroll
    for (int e = 0; e < NE; ++e) xs[e] = fast_quotient(delta[e], rs);
    if (__builtin_expect(!g.fast(rs), 0)) {
#pragma unroll
        for (int e = 0; e < NE; ++e) xs[e] = delta[e] / rs.sc;
    }
#pragma unroll
    for (int e = 0; e < NE; ++e) r[e] = sr_round(xs[e], noise[e]);
}

__device__ __forceinline__ int sat8(int v) { return min(max(v, -128), 127); }

// sat8(w + r) for four int8 weights packed in wp and four integer-valued r in [-128, 127], packed again.  With both
// moved up by 128 the sum is a float in [0, 510] minus 128 and the saturating float-to-byte conversion does the clamp.
__device__ __forceinline__ uint32_t add_sat8_pack(uint32_t wp, const float (&r)[4]) {
    const uint32_t u = wp ^ 0x80808080u;
    uint32_t o = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float t = (float)((u >> (8 * e)) & 0xffu) + r[e];
        o = __builtin_amdgcn_cvt_pk_u8_f32(t, e, o);  // v_cvt_pk_u8_f32 clamps to 0..255
    }
    return o ^ 0x80808080u;
}

// VEC: 4 elements per thread with 16-byte loads when K % 4 == 0 and pointers are aligned, else 1
template <int VEC, bool FUSED>
__global__ __launch_bounds__(256) void lora_merge_kernel(const MergeArgs a) {
    const int64_t n = blockIdx.y;
    const int64_t k0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (k0 >= a.K) return;
    const float sc = a.ws ? a.ws[a.row_scale ? n : 0] : a.ws_host;
    const int64_t base = n * a.K + k0;

    float d[VEC], nz[VEC];
    if constexpr (FUSED) {
        float acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = 0.0f;
        const float *upr = a.up + n * a.rank;
        for (int j = 0; j < a.rank; ++j) {
            const float u = upr[j];
            if constexpr (VEC == 4) {
                const float4 dn = *(const float4 *)(a.down + (int64_t)j * a.K + k0);
                acc[0] = fmaf(u, dn.x, acc[0]);
                acc[1] = fmaf(u, dn.y, acc[1]);
                acc[2] = fmaf(u, dn.z, acc[2]);
                acc[3] = fmaf(u, dn.w, acc[3]);
            } else {
                acc[0] = fmaf(u, a.down[(int64_t)j * a.K + k0], acc[0]);
            }
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) d[e] = acc[e] * a.lora_scale;
    } else {
        if constexpr (VEC == 4) {
            const float4 t = *(const float4 *)(a.delta + base);
            d[0] = t.x, d[1] = t.y, d[2] = t.z, d[3] = t.w;
        } else {
            d[0] = a.delta[base];
        }
    }
    if constexpr (VEC == 4) {
        const float4 t = *(const float4 *)(a.noise + base);
        nz[0] = t.x, nz[1] = t.y, nz[2] = t.z, nz[3] = t.w;
    } else {
        nz[0] = a.noise[base];
    }

    float r[VEC];
    sr_row<VEC>(d, nz, row_scale(sc), r);

    if constexpr (VEC == 4) {
        stream_store4(a.out + base, add_sat8_pack(a.w ? *(const uint32_t *)(a.w + base) : 0u, r));
    } else {
        a.out[base] = (int8_t)sat8((a.w ? (int)a.w[base] : 0) + (int)r[0]);
    }
}

// Fused low-rank form on the vector ALUs (K not a multiple of 32).  A thread owns 4 consecutive columns and keeps the RANK x 4
// slice of `down` it needs in registers for the whole kernel; the block then walks a band of rows.
// Per row and thread that leaves 16 bytes of noise and 4 bytes of weight to read, 4 bytes to write,
// and the row of `up`, which is the same for every lane and comes through scalar loads.  (Indexing
// the other way round, every element re-reads its column of `down` from L2: 32 bytes of cache
// traffic per byte of weight.)  The sum over the rank is the same fma chain in increasing j.
// One row is fetched ahead; fetching further ahead costs registers, hence resident waves, and is
// slower: the kernel is bound by the fma chain, not by memory.
template <int RANK>
__global__ __launch_bounds__(256) void lora_merge_band_kernel(const MergeArgs a, int rows_per_block) {
    const int64_t k0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    const bool col_ok = k0 < a.K;  // K % 4 == 0 here
    float4 dn[RANK];
#pragma unroll
    for (int j = 0; j < RANK; ++j)
        dn[j] = col_ok ? *(const float4 *)(a.down + (int64_t)j * a.K + k0) : make_float4(0.f, 0.f, 0.f, 0.f);

    const int64_t n_begin = (int64_t)blockIdx.y * rows_per_block;
    const int64_t n_end = n_begin + rows_per_block < a.N ? n_begin + rows_per_block : a.N;
    if (n_begin >= n_end || !col_ok) return;

    float4 nz = *(const float4 *)(a.noise + n_begin * a.K + k0);
    uint32_t wp = *(const uint32_t *)(a.w + n_begin * a.K + k0);
    for (int64_t n = n_begin; n < n_end; ++n) {
        const float4 nz_cur = nz;
        const uint32_t wp_cur = wp;
        if (n + 1 < n_end) {  // next row's operands are in flight while this row is computed
            nz = *(const float4 *)(a.noise + (n + 1) * a.K + k0);
            wp = *(const uint32_t *)(a.w + (n + 1) * a.K + k0);
        }
        const float sc = a.ws ? a.ws[a.row_scale ? n : 0] : a.ws_host;
        const float *upr = a.up + n * RANK;
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < RANK; ++j) {
            const float u = upr[j];
            acc[0] = fmaf(u, dn[j].x, acc[0]);
            acc[1] = fmaf(u, dn[j].y, acc[1]);
            acc[2] = fmaf(u, dn[j].z, acc[2]);
            acc[3] = fmaf(u, dn[j].w, acc[3]);
        }
        const float nzv[4] = {nz_cur.x, nz_cur.y, nz_cur.z, nz_cur.w};
        float d[4], r[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) d[e] = acc[e] * a.lora_scale;
        sr_row<4>(d, nzv, row_scale(sc), r);
        stream_store4(a.out + n * a.K + k0, add_sat8_pack(wp_cur, r));
    }
}

// The same fused form on the matrix cores.  v_mfma_f32_32x32x2_f32 adds two products per output to
// its accumulator, the k = 0 product first and each with a single rounding, so a sequence of them
// over j = (0,1), (2,3), ... is the fma chain in increasing j of the definition above, bit for bit
// (the parity tests check this against a CPU fmaf chain).  The output block is computed transposed,
// D[k][n] = sum_j down[j][k] * up[n][j]: a lane then holds, for ONE weight row n, four groups of
// four consecutive k, so the rounding step works on 16-byte noise and 4-byte weight pieces.
//
// A workgroup of 8 waves owns 256 columns and walks blocks of 32 rows (every bands-th one).  The noise of a
// block goes from global memory straight into one of two LDS tiles (buffer_load ... lds: a wave
// instruction moves 1 KB of one noise row, no registers involved) while the block before it is
// worked on; weights and `up` travel through registers.  Every wave takes the 32 x 32 piece of its
// own 32 columns from the tiles in the layout above; results go back through the weight tile so that
// they leave in 256-byte runs.  Each wave keeps its slice of `down` in RANK/2 registers.
//
// The product of block i+1 is computed while block i is rounded: the matrix instructions (64 cycles
// each, one dependent chain) are dealt out between the vector instructions of the rounding, so a
// wave keeps both units busy instead of using them in turn.
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v4i_t __attribute__((ext_vector_type(4)));

template <int RANK>
struct MfmaMergeLds {
    static constexpr int WAVES = 8, COLS = WAVES * 32;
    static constexpr int NZ_PITCH = COLS * 4 + 16;   // 260 words: the column reads of 16 rows hit 16 different bank groups
    static constexpr int UP_PITCH = RANK * 4 + 4;
    static constexpr int WB_PITCH = COLS + 16;
    static constexpr int NZ_BYTES = 32 * NZ_PITCH;
    static constexpr int NZ = 0, UP = 2 * NZ_BYTES, WB = UP + ((32 * UP_PITCH + 15) / 16) * 16;
    static constexpr int BYTES = WB + 32 * WB_PITCH;
};

// Workgroup barrier for data exchanged through LDS only: waits for this wave's LDS operations and leaves its global
// loads and stores in flight (__syncthreads() would wait for those as well).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// One wave-wide load of 16 bytes per lane from a buffer straight into LDS: lane l lands at lds_base + 16 l.  Bytes
// beyond the buffer's size arrive as zeros.  The compiler does not see this load: what waits for it is an explicit
// s_waitcnt vmcnt in the caller.
__device__ __forceinline__ void buffer_to_lds16(v4i_t rsrc, uint32_t lds_base, uint32_t voffset, uint32_t soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset)
                 : "memory", "m0");
}

// p and bytes are the same in every lane; readfirstlane tells the compiler so (64-bit address arithmetic runs on the
// vector ALUs and would otherwise leave the descriptor in vector registers, where a buffer instruction cannot take it).
__device__ __forceinline__ v4i_t buffer_resource(const void *p, uint32_t bytes) {
    const uint64_t a = (uint64_t)p;
    v4i_t r = {__builtin_amdgcn_readfirstlane((int)(uint32_t)a), __builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu)),
               __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000};
    return r;
}

template <int RANK>
__global__ __launch_bounds__(512, 4) void lora_merge_mfma_kernel(const MergeArgs a, int bands) {
    using T = MfmaMergeLds<RANK>;
    constexpr int NT = 512, P = RANK / 2;
    __shared__ __attribute__((aligned(16))) char lds[T::BYTES];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;
    // Workgroup (band, column block) takes the row blocks band, band + bands, band + 2 bands, ... of its 256 columns,
    // so that the workgroups running at the same time read neighbouring rows.
    const int64_t nblocks = (a.N + 31) / 32;
    const int band = blockIdx.y;
    const int count = (int)((nblocks - band + bands - 1) / bands);
    if (count <= 0) return;
    auto block_of = [&](int it) { return band + (int64_t)it * bands; };

    const int64_t k0 = (int64_t)blockIdx.x * T::COLS;      // first column of the workgroup (K % 32 == 0 here)
    const int64_t kbase = k0 + wave * 32;                  // first column of this wave
    float da[P];
#pragma unroll
    for (int p = 0; p < P; ++p) da[p] = kbase < a.K ? a.down[(int64_t)(2 * p + half) * a.K + kbase + l32] : 0.0f;

    // Noise: wave w moves rows w, w + 8, w + 16, w + 24 of a block, lane l the 16 bytes at column 4 l.  The buffer
    // starts at the block's first row and the workgroup's first column and ends with the array, so rows past N
    // read as zeros (their results are not stored).
    const uint32_t row_bytes = (uint32_t)a.K * 4u;
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    auto fetch_noise = [&](int64_t nb, int buf) __attribute__((always_inline)) {
        const int64_t first = nb * 32 * a.K + k0;
        const int64_t left = (a.N * a.K - first) * 4;
        const v4i_t rsrc = buffer_resource(a.noise + first, left < 0xffffffffll ? (uint32_t)left : 0xffffffffu);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            buffer_to_lds16(rsrc, lds_base + T::NZ + buf * T::NZ_BYTES + (wave + 8 * i) * T::NZ_PITCH, (uint32_t)lane * 16u,
                            (uint32_t)(wave + 8 * i) * row_bytes);
    };
    // Weights (one 16-byte piece per thread: row tid / 16, column 16 (tid % 16)), the row scale and, threads below
    // 8 RANK, one 16-byte piece of the contiguous 32 x RANK block of `up`, through registers.
    constexpr int UP_THREADS = 32 * RANK / 4;
    static_assert(UP_THREADS <= NT, "one piece of the up block per thread");
    const int wb_row = tid >> 4, wb_col = tid & 15;
    const bool wb_col_ok = k0 + wb_col * 16 < a.K;
    auto clampn = [&](int64_t n) { return n < a.N ? n : a.N - 1; };  // rows past the end repeat the last one, unstored
    auto fetch_weights = [&](int64_t nb, v4u_t &wb, float &sc) __attribute__((always_inline)) {
        if (wb_col_ok) wb = *(const v4u_t *)(a.w + clampn(nb * 32 + wb_row) * a.K + k0 + wb_col * 16);
        sc = a.ws ? a.ws[a.row_scale ? clampn(nb * 32 + l32) : 0] : a.ws_host;
    };
    auto fetch_up = [&](int64_t nb, v4f &up) __attribute__((always_inline)) {
        if (tid < UP_THREADS) up = *(const v4f *)(a.up + clampn(nb * 32 + tid * 4 / RANK) * RANK + (tid * 4) % RANK);
    };
    auto park_up = [&](const v4f &up) __attribute__((always_inline)) {
        if (tid < UP_THREADS) {
            float *dst = (float *)(lds + T::UP + (tid * 4 / RANK) * T::UP_PITCH + ((tid * 4) % RANK) * 4);
            dst[0] = up.x, dst[1] = up.y, dst[2] = up.z, dst[3] = up.w;
        }
    };
    auto up_operand = [&](int p) __attribute__((always_inline)) {
        return *(const float *)(lds + T::UP + l32 * T::UP_PITCH + (2 * p + half) * 4);
    };

    v4f up_r = {};
    v4u_t wb_r = {};
    float sc_r = 1.0f;
    v16f acc_cur, acc_next;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc_cur[i] = 0.0f;
    // the first block's product; every later one is computed beside the rounding of its predecessor
    fetch_up(block_of(0), up_r);
    fetch_noise(block_of(0), 0);
    fetch_weights(block_of(0), wb_r, sc_r);
    park_up(up_r);
    fetch_up(block_of(1), up_r);
    lds_barrier();
#pragma unroll
    for (int p = 0; p < P; ++p) acc_cur = __builtin_amdgcn_mfma_f32_32x32x2f32(da[p], up_operand(p), acc_cur, 0, 0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the first block's noise is in its tile
    lds_barrier();

    for (int it = 0; it < count; ++it) {
        const int64_t nb = block_of(it);
        const int buf = it & 1;
        const char *nz_tile = lds + T::NZ + buf * T::NZ_BYTES;
        park_up(up_r);  // of the next block
        *(v4u_t *)(lds + T::WB + wb_row * T::WB_PITCH + wb_col * 16) = wb_r;
        const RowScale rs = row_scale(sc_r);
        lds_barrier();  // this block's noise landed before the last barrier of the block before (or of the prologue)
        if (it + 1 < count) {
            fetch_noise(block_of(it + 1), buf ^ 1);
            fetch_weights(block_of(it + 1), wb_r, sc_r);
        }
        if (it + 2 < count) fetch_up(block_of(it + 2), up_r);

        float d[16];
        uint32_t o[4];
        SrGuard guard;
        auto noise_quad = [&](int q, float (&nzv)[4]) __attribute__((always_inline)) {
            const v4f nz = *(const v4f *)(nz_tile + l32 * T::NZ_PITCH + wave * 128 + (2 * q + half) * 16);
            nzv[0] = nz.x, nzv[1] = nz.y, nzv[2] = nz.z, nzv[3] = nz.w;
        };
        auto weight_quad = [&](int q) __attribute__((always_inline)) {
            return *(const uint32_t *)(lds + T::WB + l32 * T::WB_PITCH + wave * 32 + 8 * q + 4 * half);
        };
#pragma unroll
        for (int q = 0; q < 4; ++q) {  // the noise is read again where it is used: sixteen registers fewer across the block
            float nzv[4], dq[4];
            noise_quad(q, nzv);
#pragma unroll
            for (int e = 0; e < 4; ++e) dq[e] = d[4 * q + e] = acc_cur[4 * q + e] * a.lora_scale;
            guard.add(dq, nzv);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) acc_next[i] = 0.0f;
        if (__builtin_amdgcn_ballot_w64(!guard.fast(rs)) == 0) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int p = q * P / 4; p < (q + 1) * P / 4; ++p)
                    acc_next = __builtin_amdgcn_mfma_f32_32x32x2f32(da[p], up_operand(p), acc_next, 0, 0, 0);
                float r[4], nzv[4];
                noise_quad(q, nzv);
#pragma unroll
                for (int e = 0; e < 4; ++e) r[e] = sr_round(fast_quotient(d[4 * q + e], rs), nzv[e]);
                o[q] = add_sat8_pack(weight_quad(q), r);
            }
#pragma unroll
            for (int i = 0; i < P; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);        // one matrix instruction
                __builtin_amdgcn_sched_group_barrier(0x002, 224 / P, 0);  // its share of the vector work
            }
        } else {  // some lane needs the division: every lane takes it
#pragma unroll
            for (int p = 0; p < P; ++p) acc_next = __builtin_amdgcn_mfma_f32_32x32x2f32(da[p], up_operand(p), acc_next, 0, 0, 0);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float r[4], nzv[4];
                noise_quad(q, nzv);
#pragma unroll
                for (int e = 0; e < 4; ++e) r[e] = sr_round(d[4 * q + e] / rs.sc, nzv[e]);
                o[q] = add_sat8_pack(weight_quad(q), r);
            }
        }
        acc_cur = acc_next;
        // results: back through the weight tile (each lane overwrites exactly the bytes it read),
        // then one 16-byte store per thread
#pragma unroll
        for (int q = 0; q < 4; ++q) *(uint32_t *)(lds + T::WB + l32 * T::WB_PITCH + wave * 32 + 8 * q + 4 * half) = o[q];
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the next block's noise is in its tile (and this wave's last store is out)
        lds_barrier();
        const v4u_t obv = *(const v4u_t *)(lds + T::WB + wb_row * T::WB_PITCH + wb_col * 16);
        const int64_t nrow = nb * 32 + wb_row;
        if (nrow < a.N && wb_col_ok) stream_store16(a.out + nrow * a.K + k0 + wb_col * 16, make_uint4(obv.x, obv.y, obv.z, obv.w));
        lds_barrier();  // the weight and `up` tiles are free for the next block
    }
}

template <int RANK>
int launch_mfma(const MergeArgs &a, hipStream_t st) {
    const int64_t col_blocks = (a.K + 255) / 256, nblocks = (a.N + 31) / 32;
    if (col_blocks > 0x7fffffffll) return I8F_ERR_UNSUPPORTED;
    // Two workgroups fit a CU (LDS), so 512 run at a time.  Bands are chosen for the fewest block steps on the busiest
    // CU: rounds of 512 workgroups times the blocks of a band, plus half a step for a workgroup's start (its first
    // product is not overlapped with anything); a tie goes to fewer rounds, then to more bands (more of the chip reading).
    constexpr int64_t SLOTS = 512;
    int64_t max_bands = 4 * SLOTS / col_blocks + 1;
    if (max_bands > nblocks) max_bands = nblocks;
    if (max_bands > 65535) max_bands = 65535;
    int64_t bands = 1, best = -1, best_rounds = 0;
    for (int64_t b = 1; b <= max_bands; ++b) {
        const int64_t rounds = (col_blocks * b + SLOTS - 1) / SLOTS, steps2 = 2 * ((nblocks + b - 1) / b) + 1;
        if (best < 0 || rounds * steps2 < best || (rounds * steps2 == best && rounds <= best_rounds))
            best = rounds * steps2, best_rounds = rounds, bands = b;
    }
    hipLaunchKernelGGL((lora_merge_mfma_kernel<RANK>), dim3((unsigned)col_blocks, (unsigned)bands), dim3(512), 0, st, a, (int)bands);
    return check_launch();
}

template <int RANK>
int launch_band(const MergeArgs &a, hipStream_t st) {
    const unsigned col_blocks = (unsigned)((a.K + 1023) / 1024);
    // enough row bands to fill the chip several times over, each long enough to amortise its slice of `down`
    int64_t bands = (256 * 12 + col_blocks - 1) / col_blocks;
    int64_t rows = (a.N + bands - 1) / bands;
    if (rows < 16) rows = 16;
    bands = (a.N + rows - 1) / rows;
    if (bands > 65535) return I8F_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((lora_merge_band_kernel<RANK>), dim3(col_blocks, (unsigned)bands), dim3(256), 0, st, a, (int)rows);
    return check_launch();
}

int run(MergeArgs &a, hipStream_t st) {
    if (a.N == 0 || a.K == 0) return I8F_OK;
    if (a.N > 65535 * 1024ll) return I8F_ERR_UNSUPPORTED;
    const bool fused = a.delta == nullptr;
    auto al = [](const void *p, int n) { return p == nullptr || (uintptr_t)p % n == 0; };
    const bool vec = a.K % 4 == 0 && al(a.w, 4) && al(a.out, 4) && al(a.noise, 16) && al(a.delta, 16) &&
                     (!fused || al(a.down, 16));
    // (K < 2^24: the 32 rows of a block are addressed with 32-bit byte offsets from the block's first element)
    if (fused && vec && a.w && a.N < (1ll << 31) && a.K % 32 == 0 && a.K < (1 << 24) && al(a.up, 16) && al(a.w, 16) && al(a.out, 16)) {
        switch (a.rank) {
        case 4: return launch_mfma<4>(a, st);
        case 8: return launch_mfma<8>(a, st);
        case 16: return launch_mfma<16>(a, st);
        case 32: return launch_mfma<32>(a, st);
        default: break;
        }
    }
    if (fused && vec && a.w && a.N < (1ll << 31)) {
        switch (a.rank) {
        case 4: return launch_band<4>(a, st);
        case 8: return launch_band<8>(a, st);
        case 16: return launch_band<16>(a, st);
        case 32: return launch_band<32>(a, st);
        default: break;  // other ranks take the per-element kernel below
        }
    }
    // grid.y is limited to 65535: fold larger N into several launches
    for (int64_t n0 = 0; n0 < a.N; n0 += 65535) {
        MergeArgs b = a;
        const int64_t rows = a.N - n0 < 65535 ? a.N - n0 : 65535;
        b.N = rows;
        if (b.w) b.w += n0 * a.K;
        b.out += n0 * a.K;
        b.noise += n0 * a.K;
        if (b.delta) b.delta += n0 * a.K;
        if (b.up) b.up += n0 * a.rank;
        if (b.ws && b.row_scale) b.ws += n0;
        const int per_block = 256 * (vec ? 4 : 1);
        dim3 grid((unsigned)((a.K + per_block - 1) / per_block), (unsigned)rows);
        if (vec) {
            if (fused) hipLaunchKernelGGL((lora_merge_kernel<4, true>), grid, dim3(256), 0, st, b);
            else hipLaunchKernelGGL((lora_merge_kernel<4, false>), grid, dim3(256), 0, st, b);
        } else {
            if (fused) hipLaunchKernelGGL((lora_merge_kernel<1, true>), grid, dim3(256), 0, st, b);
            else hipLaunchKernelGGL((lora_merge_kernel<1, false>), grid, dim3(256), 0, st, b);
        }
        if (int rc = check_launch()) return rc;
    }
    return I8F_OK;
}

}  // namespace
}  // namespace i8f

extern "C" int i8f_sr_quant_delta(const float *x, const float *scale, float scale_host, int scale_mode,
                                  const float *noise, int64_t N, int64_t K, int8_t *dq, void *stream) {
    using namespace i8f;
    if (N < 0 || K < 0) return I8F_ERR_INVALID;
    if (scale_mode != I8F_SCALE_TENSOR && scale_mode != I8F_SCALE_ROW) return I8F_ERR_INVALID;
    if (N == 0 || K == 0) return I8F_OK;
    if (!x || !noise || !dq) return I8F_ERR_INVALID;
    if (scale_mode == I8F_SCALE_ROW && !scale) return I8F_ERR_INVALID;
    if (int rc = check_device()) return rc;
    MergeArgs a{};
    a.ws = scale, a.ws_host = scale_host, a.row_scale = scale_mode == I8F_SCALE_ROW;
    a.delta = x, a.noise = noise, a.N = N, a.K = K, a.out = dq;
    return run(a, (hipStream_t)stream);
}

extern "C" int i8f_lora_merge_sr(const int8_t *w, const float *w_scale, float w_scale_host, int scale_mode,
                                 const float *delta, const float *up, const float *down, int64_t rank,
                                 float lora_scale, const float *noise, int64_t N, int64_t K, int8_t *w_out,
                                 void *stream) {
    using namespace i8f;
    if (N < 0 || K < 0) return I8F_ERR_INVALID;
    if (scale_mode != I8F_SCALE_TENSOR && scale_mode != I8F_SCALE_ROW) return I8F_ERR_INVALID;
    if (N == 0 || K == 0) return I8F_OK;
    if (!w || !noise || !w_out) return I8F_ERR_INVALID;
    if (scale_mode == I8F_SCALE_ROW && !w_scale) return I8F_ERR_INVALID;
    if (!delta) {
        if (!up || !down || rank < 0) return I8F_ERR_INVALID;
        if (rank > 256) return I8F_ERR_UNSUPPORTED;
    }
    if (int rc = check_device()) return rc;
    MergeArgs a{};
    a.w = w, a.ws = w_scale, a.ws_host = w_scale_host, a.row_scale = scale_mode == I8F_SCALE_ROW;
    a.delta = delta, a.up = up, a.down = down, a.rank = (int)rank, a.lora_scale = lora_scale;
    a.noise = noise, a.N = N, a.K = K, a.out = w_out;
    return run(a, (hipStream_t)stream);
}
