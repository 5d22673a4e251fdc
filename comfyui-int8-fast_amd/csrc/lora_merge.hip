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

// Fused low-rank form, the fast kernel.  A thread owns 4 consecutive columns and keeps the RANK x 4
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
