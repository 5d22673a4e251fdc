// Stochastic-rounding LoRA merge into int8 weights, one pass over HBM.
//
//   xs  = delta_f / w_scale                 correctly rounded division
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

__device__ __forceinline__ int sr_one(float delta, float sc, float noise) {
    const float xs = delta / sc;
    const float f = floorf(xs);
    const float frac = xs - f;
    float r = noise < frac ? f + 1.0f : f;
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return (int)r;
}

__device__ __forceinline__ int sat8(int v) { return min(max(v, -128), 127); }

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

    int q[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) q[e] = sr_one(d[e], sc, nz[e]);

    if constexpr (VEC == 4) {
        if (a.w) {
            const uint32_t wp = *(const uint32_t *)(a.w + base);
#pragma unroll
            for (int e = 0; e < 4; ++e) q[e] = sat8((int)(int8_t)(wp >> (8 * e)) + q[e]);
        }
        uint32_t o = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) o |= ((uint32_t)q[e] & 0xffu) << (8 * e);
        stream_store4(a.out + base, o);
    } else {
        if (a.w) q[0] = sat8((int)a.w[base] + q[0]);
        a.out[base] = (int8_t)q[0];
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
        uint32_t o = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int dq = sr_one(acc[e] * a.lora_scale, sc, nzv[e]);
            const int wv = (int)(int8_t)(wp_cur >> (8 * e));
            o |= ((uint32_t)sat8(wv + dq) & 0xffu) << (8 * e);
        }
        stream_store4(a.out + n * a.K + k0, o);
    }
}

// The same fused form on the matrix cores.  v_mfma_f32_32x32x2_f32 adds two products per output to
// its accumulator, the k = 0 product first and each with a single rounding, so a sequence of them
// over j = (0,1), (2,3), ... is the fma chain in increasing j of the definition above, bit for bit
// (the parity tests check this against a CPU fmaf chain).  The output block is computed transposed,
// D[k][n] = sum_j down[j][k] * up[n][j]: a lane then holds, for ONE weight row n, four groups of
// four consecutive k, so the rounding step works on 16-byte noise and 4-byte weight pieces.
//
// A workgroup of 8 waves owns 256 columns and walks a band of rows in blocks of 32.  Its threads
// fetch a block row by row (one wave instruction = 1 KB of one noise row) into an LDS tile, from
// which every wave takes the 32 x 32 piece of its own 32 columns in the layout above; results go
// back through the tile so that they leave in 256-byte runs.  Each wave keeps its slice of `down`
// in RANK/2 registers; `up` is fetched once per block for all eight waves.  The operands of the
// next block are in flight while this one is computed.
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

template <int RANK>
struct MfmaMergeLds {
    static constexpr int WAVES = 8, COLS = WAVES * 32;
    static constexpr int NZ_PITCH = COLS * 4 + 16;   // 260 words: the column reads of 16 rows hit 16 different bank groups
    static constexpr int UP_PITCH = RANK * 4 + 4;
    static constexpr int WB_PITCH = COLS + 16;
    static constexpr int NZ = 0, UP = NZ + 32 * NZ_PITCH, WB = UP + ((32 * UP_PITCH + 15) / 16) * 16;
    static constexpr int BYTES = WB + 32 * WB_PITCH;
};

template <int RANK>
__global__ __launch_bounds__(512) void lora_merge_mfma_kernel(const MergeArgs a, int blocks_per_band) {
    using T = MfmaMergeLds<RANK>;
    __shared__ __attribute__((aligned(16))) char lds[T::BYTES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int64_t k0 = (int64_t)blockIdx.x * T::COLS;     // first column of the workgroup (K % 32 == 0 here)
    const int64_t kbase = k0 + wave * 32;                  // first column of this wave
    const bool wave_live = kbase < a.K;
    float da[RANK / 2];
#pragma unroll
    for (int p = 0; p < RANK / 2; ++p) da[p] = wave_live ? a.down[(int64_t)(2 * p + half) * a.K + kbase + l32] : 0.0f;

    const int64_t nblocks = (a.N + 31) / 32;
    const int64_t nb_begin = (int64_t)blockIdx.y * blocks_per_band;
    const int64_t nb_end = nb_begin + blocks_per_band < nblocks ? nb_begin + blocks_per_band : nblocks;

    // what a thread fetches of a block: 4 pieces of noise (piece c = tid + 512 i: row c / 64, 16-byte
    // column c % 64), one 16-byte piece of weight (row tid / 16, column tid % 16) and, threads below
    // 8 RANK, one 16-byte piece of the contiguous 32 x RANK block of `up`
    constexpr int UP_THREADS = 32 * RANK / 4;
    const bool nz_col_ok = k0 + (tid & 63) * 4 < a.K, wb_col_ok = k0 + (tid & 15) * 16 < a.K;
    auto clampn = [&](int64_t n) { return n < a.N ? n : a.N - 1; };  // rows past the end repeat the last one, unstored
    auto fetch = [&](int64_t nb, v4f (&nz)[4], v4f &up, v4u_t &wb, float &sc) __attribute__((always_inline)) {
        const int64_t n0 = nb * 32;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (nz_col_ok) nz[i] = *(const v4f *)(a.noise + clampn(n0 + (tid >> 6) + 8 * i) * a.K + k0 + (tid & 63) * 4);
        if (tid < UP_THREADS) up = *(const v4f *)(a.up + clampn(n0 + tid * 4 / RANK) * RANK + (tid * 4) % RANK);
        if (wb_col_ok) wb = *(const v4u_t *)(a.w + clampn(n0 + (tid >> 4)) * a.K + k0 + (tid & 15) * 16);
        sc = a.ws ? a.ws[a.row_scale ? clampn(n0 + l32) : 0] : a.ws_host;
    };

    v4f nz_r[4] = {}, up_r = {};
    v4u_t wb_r = {};
    float sc_r = 1.0f;
    if (nb_begin < nb_end) fetch(nb_begin, nz_r, up_r, wb_r, sc_r);
    for (int64_t nb = nb_begin; nb < nb_end; ++nb) {
        // registers -> LDS tile; the same registers then receive the next block
#pragma unroll
        for (int i = 0; i < 4; ++i) *(v4f *)(lds + T::NZ + ((tid >> 6) + 8 * i) * T::NZ_PITCH + (tid & 63) * 16) = nz_r[i];
        if (tid < UP_THREADS) {
            float *dst = (float *)(lds + T::UP + (tid * 4 / RANK) * T::UP_PITCH + ((tid * 4) % RANK) * 4);
            dst[0] = up_r.x, dst[1] = up_r.y, dst[2] = up_r.z, dst[3] = up_r.w;
        }
        *(v4u_t *)(lds + T::WB + (tid >> 4) * T::WB_PITCH + (tid & 15) * 16) = wb_r;
        const float sc = sc_r;
        __syncthreads();
        if (nb + 1 < nb_end) fetch(nb + 1, nz_r, up_r, wb_r, sc_r);

        v16f acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
        for (int p = 0; p < RANK / 2; ++p) {
            const float u = *(const float *)(lds + T::UP + l32 * T::UP_PITCH + (2 * p + half) * 4);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(da[p], u, acc, 0, 0, 0);
        }
        uint32_t o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const v4f nz = *(const v4f *)(lds + T::NZ + l32 * T::NZ_PITCH + wave * 128 + (2 * q + half) * 16);
            const uint32_t wp = *(const uint32_t *)(lds + T::WB + l32 * T::WB_PITCH + wave * 32 + 8 * q + 4 * half);
            const float nzv[4] = {nz.x, nz.y, nz.z, nz.w};
            o[q] = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int dq = sr_one(acc[4 * q + e] * a.lora_scale, sc, nzv[e]);
                const int wv = (int)(int8_t)(wp >> (8 * e));
                o[q] |= ((uint32_t)sat8(wv + dq) & 0xffu) << (8 * e);
            }
        }
        // results: back through the weight tile (each lane overwrites exactly the bytes it read),
        // then one 16-byte store per thread
#pragma unroll
        for (int q = 0; q < 4; ++q) *(uint32_t *)(lds + T::WB + l32 * T::WB_PITCH + wave * 32 + 8 * q + 4 * half) = o[q];
        __syncthreads();
        const v4u_t obv = *(const v4u_t *)(lds + T::WB + (tid >> 4) * T::WB_PITCH + (tid & 15) * 16);
        const int64_t nrow = nb * 32 + (tid >> 4);
        if (nrow < a.N && wb_col_ok) stream_store16(a.out + nrow * a.K + k0 + (tid & 15) * 16, make_uint4(obv.x, obv.y, obv.z, obv.w));
        __syncthreads();  // the tile is free for the next block
    }
}

template <int RANK>
int launch_mfma(const MergeArgs &a, hipStream_t st) {
    const unsigned col_blocks = (unsigned)((a.K + 255) / 256);
    const int64_t nblocks = (a.N + 31) / 32;
    const int64_t target_wgs = 256 * 12;  // short bands: several workgroups per CU take turns at the barriers
    int64_t bands = (target_wgs + col_blocks - 1) / col_blocks;
    int64_t per = (nblocks + bands - 1) / bands;
    if (per < 2) per = 2;
    bands = (nblocks + per - 1) / per;
    if (bands > 65535) return I8F_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((lora_merge_mfma_kernel<RANK>), dim3(col_blocks, (unsigned)bands), dim3(512), 0, st, a, (int)per);
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
    if (fused && vec && a.w && a.N < (1ll << 31) && a.K % 32 == 0 && al(a.up, 16) && al(a.w, 16) && al(a.out, 16)) {
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
