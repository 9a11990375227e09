// Bandwidth-bound quantised GEMV on the int8 matrix cores (M <= 4 activation rows; I8, I4 and U4 weights) for gfx950.
//
//   out[m,n] = act((sum_k A[m,k]*q(W[n,k]))*scale[n] + zero[n]*sum_k A[m,k] + bias[n])
//   (gemm_batch_packed_simd + apply_affine_dot, src/backend/cpu/microkernels/gemm.rs:1982-2088,
//    src/backend/cpu/microkernels/mod.rs:283-295)
//
// Integer weights need no conversion at all to be a v_mfma_i32_16x16x64_i8 operand: an I8 lane load of 16 bytes IS
// the operand of one step (64 k-values of one weight row), a 4-bit word becomes two operands with two logic ops
// (even nibbles and odd nibbles moved to the high half of a byte: 16*q; unsigned nibbles stay as they are).  The f32
// activations are split exactly into four signed base-256 digits after a power-of-two scaling per slice of 512
// k-values: x = 2^e * (((d0*256 + d1)*256 + d2)*256 + d3), 30 bits below the slice maximum, so an activation 256 times
// smaller than the largest of its slice still keeps 22 bits (what the f16 hi + lo split of the other GEMV kernels
// keeps per element).  The four digit rows of an activation row sit in four of the 16 rows of the MFMA's activation
// operand, which a GEMV leaves empty anyway, so one MFMA per step yields the four exact i32 partial sums and the
// matrix core does twice the k-values per instruction of the f16 form, with no decode arithmetic on the vector ALU.
//
// Work split: a workgroup converts the activation rows ONCE into digit fragments in LDS and then walks row tiles of 16
// weight rows (tile = blockIdx.x, += gridDim.x): the grid is one workgroup per CU.  Wave w owns the K slices
// w, w + NW, ... of every tile; the packed bytes of a wave's next (tile, slice) are requested before it works on the
// current one, so a wave always has three slices in flight.  Per tile the waves' partial sums meet in LDS in a fixed
// order (double-buffered: one workgroup barrier per tile) and 16*M threads apply the affine / bias / activation
// epilogue.  Algorithmic bytes per launch: N*K*bits/8 + side tables + 4*M*(K+N).
#include "mfma.h"

namespace {

struct DotArgs {
    const uint32_t *words;
    const float *scales, *zeros, *a, *bias;
    float *out;
    int64_t m, n, k, kp;
    int act;
    int nslice;   // slices of 512 k-values covering K
    int spw;      // slices per wave and tile = ceil(nslice / NW)
    int ntiles;   // row tiles of 16
};

constexpr int SL = 512;   // k-values per slice
constexpr int NSTEP = 8;  // MFMA steps (64 k-values) per slice

// packed words of one lane load -> int8 operands
template <int DT>
struct Int8Op;
template <>
struct Int8Op<FNN_DT_I8> {
    static constexpr int LOADS = 8;      // 16-byte lane loads per slice: one per step
    static constexpr int PER_LOAD = 1;   // MFMA steps per load
    static constexpr float POST = 1.0f;
    __device__ static __forceinline__ i32x4 op(const uint32_t (&w)[4], int) { return i32x4{(int)w[0], (int)w[1], (int)w[2], (int)w[3]}; }
};
template <>
struct Int8Op<FNN_DT_I4> {
    static constexpr int LOADS = 4;      // a load covers 128 k-values: even nibbles are one step, odd nibbles the next
    static constexpr int PER_LOAD = 2;
    static constexpr float POST = 0.0625f;   // operands are 16*q
    __device__ static __forceinline__ i32x4 op(const uint32_t (&w)[4], int odd)
    {
        if (odd) return i32x4{(int)(w[0] & 0xF0F0F0F0u), (int)(w[1] & 0xF0F0F0F0u), (int)(w[2] & 0xF0F0F0F0u), (int)(w[3] & 0xF0F0F0F0u)};
        return i32x4{(int)((w[0] << 4) & 0xF0F0F0F0u), (int)((w[1] << 4) & 0xF0F0F0F0u), (int)((w[2] << 4) & 0xF0F0F0F0u),
                     (int)((w[3] << 4) & 0xF0F0F0F0u)};
    }
};
template <>
struct Int8Op<FNN_DT_U4> {
    static constexpr int LOADS = 4;
    static constexpr int PER_LOAD = 2;
    static constexpr float POST = 1.0f;
    __device__ static __forceinline__ i32x4 op(const uint32_t (&w)[4], int odd)
    {
        if (odd) return i32x4{(int)((w[0] >> 4) & 0x0F0F0F0Fu), (int)((w[1] >> 4) & 0x0F0F0F0Fu), (int)((w[2] >> 4) & 0x0F0F0F0Fu),
                              (int)((w[3] >> 4) & 0x0F0F0F0Fu)};
        return i32x4{(int)(w[0] & 0x0F0F0F0Fu), (int)(w[1] & 0x0F0F0F0Fu), (int)(w[2] & 0x0F0F0F0Fu), (int)(w[3] & 0x0F0F0F0Fu)};
    }
};

template <int DT, int MM, int NW>
__global__ void __launch_bounds__(NW * 64) qgemv_i8dot_kernel(DotArgs p)
{
    using W = Int8Op<DT>;
    constexpr int LOADS = W::LOADS, PER = W::PER_LOAD;
    constexpr int R4 = 4 * MM;               // digit rows kept in LDS per step: row m*4 + digit
    constexpr bool FOUR_BIT = PER == 2;

    // [slice][step][R4 rows][4 groups] 16-byte operand fragments, then [slice][MM] slice scales
    extern __shared__ __attribute__((aligned(16))) uint4 lds_dyn[];
    __shared__ float red[2][NW][MM][16];
    __shared__ float xred[NW][MM];

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int ln = lane & 15, g = lane >> 4;
    const int64_t K = p.k, N = p.n, kp = p.kp;
    const int mreal = (int)p.m;
    const int nslice = p.nslice, spw = p.spw;
    uint4 *frag = lds_dyn;
    float *cscale = reinterpret_cast<float *>(lds_dyn + (size_t)nslice * NSTEP * R4 * 4);

    // units of work of this wave: (tile, slice) pairs, tile-major
    const int my_tiles = ((int)blockIdx.x < p.ntiles) ? (p.ntiles - 1 - (int)blockIdx.x) / (int)gridDim.x + 1 : 0;
    const int nunits = my_tiles * spw;

    // this lane's group of 8 activations of every row for one slice (clamped address, masked afterwards)
    auto load_slice = [&](int slice, float (&xr)[MM][8]) {
        const int64_t kk = (int64_t)slice * SL + lane * 8;
        const int64_t kkc = kk < K ? kk : K - 8;   // K % 8 == 0
#pragma unroll
        for (int m = 0; m < MM; m++) {
            const int64_t mrow = m < mreal ? m : mreal - 1;
            const uint32_t keep = (m < mreal && kk < K) ? 0xffffffffu : 0u;
            const uint4 x0 = *reinterpret_cast<const uint4 *>(p.a + mrow * K + kkc);
            const uint4 x1 = *reinterpret_cast<const uint4 *>(p.a + mrow * K + kkc + 4);
            xr[m][0] = __uint_as_float(x0.x & keep); xr[m][1] = __uint_as_float(x0.y & keep);
            xr[m][2] = __uint_as_float(x0.z & keep); xr[m][3] = __uint_as_float(x0.w & keep);
            xr[m][4] = __uint_as_float(x1.x & keep); xr[m][5] = __uint_as_float(x1.y & keep);
            xr[m][6] = __uint_as_float(x1.z & keep); xr[m][7] = __uint_as_float(x1.w & keep);
        }
    };
    // lane (n, g), load l of a slice: words [slice*SL*bits/32 + l*16 + g*4, +4) of row n; a chunk past the end of the
    // row re-reads the row's last chunk (its activation digits are zero), a slice past K likewise
    uint32_t wq0[LOADS][4], wq1[LOADS][4], wq2[LOADS][4];
    auto request = [&](int unit, uint32_t (&dst)[LOADS][4]) {
        const int it = unit / spw, j = unit - it * spw;
        const int slice = wv + j * NW;
        int64_t row = ((int64_t)blockIdx.x + (int64_t)it * gridDim.x) * 16 + ln;
        if (row > N - 1) row = N - 1;
        const uint32_t *wrow = p.words + row * kp;
        const int64_t wbase = (int64_t)slice * (LOADS * 16);
#pragma unroll
        for (int l = 0; l < LOADS; l++) {
            const int64_t woff = wbase + l * 16 + g * 4;
            const uint4 v = *reinterpret_cast<const uint4 *>(wrow + (woff + 4 <= kp ? woff : kp - 4));   // kp % 4 == 0, kp >= 4
            dst[l][0] = v.x; dst[l][1] = v.y; dst[l][2] = v.z; dst[l][3] = v.w;
        }
    };

    // ---- requests first: the wave's first activation slice (oldest, so that its conversion does not wait for packed
    // bytes), then the packed bytes of its first three units; everything is in flight while the activations are converted
    float xr[MM][8];
    load_slice(wv < nslice ? wv : nslice - 1, xr);
    if (nunits > 0) request(0, wq0);
    if (nunits > 1) request(1, wq1);
    if (nunits > 2) request(2, wq2);
    __builtin_amdgcn_sched_barrier(0);

    // ---- activation rows -> digit fragments (wave w: slices w, w + NW, ..., the ones it multiplies with later, so no
    // workgroup barrier separates the two)
    float xsum[MM];
#pragma unroll
    for (int m = 0; m < MM; m++) xsum[m] = 0.0f;
    for (int slice = wv; slice < nslice; slice += NW) {
        if (slice != wv) load_slice(slice, xr);
#pragma unroll
        for (int m = 0; m < MM; m++) {
            const float *x = xr[m];
            float mx = fmaxf(fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3]))),
                             fmaxf(fmaxf(fabsf(x[4]), fabsf(x[5])), fmaxf(fabsf(x[6]), fabsf(x[7]))));
            mx = wave_max_uniform(mx);
            const float ssum = wave_sum_uniform(((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7])));
            xsum[m] += ssum;
            // power of two e with max*2^-e in [2^29, 2^30): |v| < 2^30, so the top digit stays within +-64
            int ex = (int)((__float_as_uint(mx) >> 23) & 0xff) - 127 - 29;
            if (mx == 0.0f) ex = 0;
            ex = ex < -100 ? -100 : (ex > 98 ? 98 : ex);
            const float inv = __uint_as_float((uint32_t)(127 - ex) << 23);
            // a NaN or an infinity among the slice's activations shows in their sum: the integer digits cannot carry
            // it, so the slice scale does (the row's outputs become NaN, as the float path's would be NaN or inf)
            const bool finite = fabsf(ssum) <= 3.4028234663852886e38f;
            if (lane == 0) cscale[slice * MM + m] = finite ? __uint_as_float((uint32_t)(127 + ex) << 23) : __uint_as_float(0x7fc00000u);
            // v = round(x * 2^-e), |v| < 2^30.  Its balanced base-256 digits (each in [-128, 127], v = sum d_j 256^j)
            // are the bytes of (v + 0x80808080) ^ 0x80808080: adding 128 to every digit gives the plain unsigned
            // base-256 form, flipping the top bit of every byte subtracts the 128 again.  Byte 3 is the top digit d0.
            uint32_t dg[8];
#pragma unroll
            for (int j = 0; j < 8; j++)
                dg[j] = ((uint32_t)(int)rintf(x[j] * inv) + 0x80808080u) ^ 0x80808080u;
            // digit rows: byte `dgt` of four activations side by side (4x4 byte transposes with v_perm_b32;
            // selector bytes 0-3 pick from the second operand, 4-7 from the first)
            auto transpose4 = [](uint32_t a, uint32_t b, uint32_t c, uint32_t d, uint32_t (&o)[4]) {
                const uint32_t ab_lo = __builtin_amdgcn_perm(b, a, 0x05010400u);   // a0 b0 a1 b1
                const uint32_t ab_hi = __builtin_amdgcn_perm(b, a, 0x07030602u);   // a2 b2 a3 b3
                const uint32_t cd_lo = __builtin_amdgcn_perm(d, c, 0x05010400u);
                const uint32_t cd_hi = __builtin_amdgcn_perm(d, c, 0x07030602u);
                o[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);           // a0 b0 c0 d0: lowest digit d3
                o[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);           // a1 b1 c1 d1
                o[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
                o[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);           // a3 b3 c3 d3: top digit d0
            };
            uint32_t t0[4], t1[4];   // [byte of v]: t[3] = top digit row d0 ... t[0] = lowest digit row d3
            // where this lane's 8 k-values sit in the operand fragments
            if constexpr (FOUR_BIT) {
                // word `lane` of the slice: load l = lane / 16, group (lane / 4) % 4, word lane % 4 of the 16 bytes;
                // even nibbles belong to step 2l, odd nibbles to step 2l + 1
                transpose4(dg[0], dg[2], dg[4], dg[6], t0);
                transpose4(dg[1], dg[3], dg[5], dg[7], t1);
                const int l = lane >> 4, gg = (lane >> 2) & 3, jw = lane & 3;
                uint32_t *f32w = reinterpret_cast<uint32_t *>(frag);
                const int base_e = (((slice * NSTEP + 2 * l) * R4 + m * 4) * 4 + gg) * 4 + jw;   // in 4-byte words
                const int base_o = base_e + R4 * 16;
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    f32w[base_e + d * 16] = t0[3 - d];
                    f32w[base_o + d * 16] = t1[3 - d];
                }
            } else {
                // bytes [lane*8, +8) of the slice: step lane / 8, group (lane / 2) % 4, half lane % 2 of the 16 bytes
                transpose4(dg[0], dg[1], dg[2], dg[3], t0);
                transpose4(dg[4], dg[5], dg[6], dg[7], t1);
                const int st = lane >> 3, gg = (lane >> 1) & 3, half = lane & 1;
                uint2 *f64w = reinterpret_cast<uint2 *>(frag);
                const int base = (((slice * NSTEP + st) * R4 + m * 4) * 4 + gg) * 2 + half;      // in 8-byte words
#pragma unroll
                for (int d = 0; d < 4; d++) f64w[base + d * 8] = uint2{t0[3 - d], t1[3 - d]};
            }
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int m = 0; m < MM; m++) xred[wv][m] = xsum[m];
    }
    // only this wave reads the fragments it wrote, and the LDS serves a wave's requests in order
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_sched_barrier(0);

    // the thread that finishes output (m, column c) of every tile: tid = m*16 + c
    const int e_m = tid >> 4, e_c = tid & 15;
    const bool finisher = tid < MM * 16 && e_m < mreal;

    // operand fragment this lane reads at a step: operand row ln = activation row ln / 4, digit ln % 4; rows past M
    // re-read row 0
    const uint4 *frd = frag + ((ln >> 2) < MM ? ln : 0) * 4 + g;
    const float *csc = cscale + (g < MM ? g : 0);     // this lane's accumulators belong to activation row g

    float tot = 0.0f;
    float e_scale = 0.0f, e_zero = 0.0f, e_bias = 0.0f, e_xs = 0.0f;
    int64_t e_n = 0;
    auto work = [&](int unit, const uint32_t (&cur)[LOADS][4]) {
        const int it = unit / spw, j = unit - it * spw;
        const int slice = wv + j * NW;
        const int64_t tile = (int64_t)blockIdx.x + (int64_t)it * gridDim.x;
        if (j == 0 && finisher) {   // epilogue operands of this tile: requested now, used after the tile's barrier
            e_n = tile * 16 + e_c;
            const int64_t nn = e_n < N ? e_n : N - 1;
            e_scale = p.scales[nn];
            e_zero = p.zeros[nn];
            e_bias = p.bias ? p.bias[nn] : 0.0f;
        }
        if (slice < nslice) {
            i32x4 acc = i32x4{0, 0, 0, 0};
            const uint4 *fs = frd + (size_t)slice * (NSTEP * R4 * 4);
#pragma unroll
            for (int l = 0; l < LOADS; l++)
#pragma unroll
                for (int q = 0; q < PER; q++) {
                    const i32x4 av = __builtin_bit_cast(i32x4, fs[(l * PER + q) * R4 * 4]);
                    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, W::op(cur[l], q), acc, 0, 0, 0);
                }
            // acc[i] = operand row g*4 + i = digit i of activation row g
            const float hi = fmaf((float)acc[0], 256.0f, (float)acc[1]), lo = fmaf((float)acc[2], 256.0f, (float)acc[3]);
            tot = fmaf(fmaf(hi, 65536.0f, lo), csc[slice * MM], tot);
        }
        if (j == spw - 1) {
            // the tile's partial sums of all waves meet in LDS (buffer it & 1); one barrier per tile
            const int par = it & 1;
            if (g < MM) red[par][wv][g][ln] = tot;
            tot = 0.0f;
            __syncthreads();
            if (finisher) {
                if (it == 0) {      // the waves' activation sums: written before the first tile's barrier
#pragma unroll
                    for (int w = 0; w < NW; w++) e_xs += xred[w][e_m];
                }
                if (e_n < N) {
                    float dot = 0.0f;
#pragma unroll
                    for (int w = 0; w < NW; w++) dot += red[par][w][e_m][e_c];
                    dot *= W::POST;
                    const float v = dot * e_scale + e_zero * e_xs;
                    p.out[(int64_t)e_m * N + e_n] = fnn_activation(p.bias ? v + e_bias : v, p.act);
                }
            }
        }
    };

    // three units in flight per wave: a buffer is requested again as soon as its unit is done
    for (int u = 0; u < nunits; u += 3) {
        work(u, wq0);
        if (u + 3 < nunits) request(u + 3, wq0);
        if (u + 1 < nunits) {
            work(u + 1, wq1);
            if (u + 4 < nunits) request(u + 4, wq1);
        }
        if (u + 2 < nunits) {
            work(u + 2, wq2);
            if (u + 5 < nunits) request(u + 5, wq2);
        }
    }
}

template <int DT, int MM, int NW>
hipError_t launch_nw(DotArgs p, int grid, hipStream_t s, bool *handled)
{
    p.nslice = (int)((p.k + SL - 1) / SL);
    p.spw = (p.nslice + NW - 1) / NW;
    p.ntiles = (int)((p.n + 15) / 16);
    const size_t lds = (size_t)p.nslice * NSTEP * 4 * MM * 4 * 16 + (size_t)p.nslice * MM * 4;
    if (lds > 128 * 1024) return hipSuccess;   // long K with several rows: left to the f16 kernels
    auto kern = qgemv_i8dot_kernel<DT, MM, NW>;
    if (lds > 48 * 1024) {
        static std::atomic<uint64_t> lds_raised{0};
        hipError_t e = fnn_raise_lds_limit(lds_raised, reinterpret_cast<const void *>(kern), 132 * 1024);
        if (e != hipSuccess) return e;
    }
    if (grid <= 0) grid = 256;                 // one workgroup per CU
    if (grid > p.ntiles) grid = p.ntiles;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NW * 64), lds, s, p);
    *handled = true;
    return hipGetLastError();
}

template <int DT>
hipError_t launch_dt(const DotArgs &p, int grid, hipStream_t s, bool *handled)
{
    const int mm = p.m <= 1 ? 1 : (p.m <= 2 ? 2 : 4);
    const bool shortk = p.k <= 4 * SL;   // K <= 2048: four waves, so that no wave idles
    if (mm == 1) return shortk ? launch_nw<DT, 1, 4>(p, grid, s, handled) : launch_nw<DT, 1, 8>(p, grid, s, handled);
    if (mm == 2) return shortk ? launch_nw<DT, 2, 4>(p, grid, s, handled) : launch_nw<DT, 2, 8>(p, grid, s, handled);
    return shortk ? launch_nw<DT, 4, 4>(p, grid, s, handled) : launch_nw<DT, 4, 8>(p, grid, s, handled);
}

}  // namespace

int fnn_i8dot_qgemv(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q, bool *handled)
{
    *handled = false;
    if (fnn_ctx_option(ctx, FNN_OPT_GEMV_INT8) == 0) return FNN_OK;
    if (w->dtype != FNN_DT_I8 && w->dtype != FNN_DT_I4 && w->dtype != FNN_DT_U4) return FNN_OK;
    if (q.m < 1 || q.m > 4 || q.n < 1) return FNN_OK;
    if (q.kp % 4 != 0 || q.k % 8 != 0 || q.k < 8) return FNN_OK;
    if ((reinterpret_cast<uintptr_t>(q.a) & 15) || (reinterpret_cast<uintptr_t>(q.words) & 15)) return FNN_OK;
    if (q.n > (int64_t)16 * 0x7fffffff / 2) return FNN_OK;
    DotArgs p;
    p.words = q.words; p.scales = q.scales; p.zeros = q.zeros; p.a = q.a; p.bias = q.bias; p.out = q.out;
    p.m = q.m; p.n = q.n; p.k = q.k; p.kp = q.kp; p.act = q.act;
    p.nslice = p.spw = p.ntiles = 0;
    const int grid = (int)fnn_ctx_option(ctx, FNN_OPT_GEMV_GRID);
    hipError_t e;
    switch (w->dtype) {
    case FNN_DT_I8: e = launch_dt<FNN_DT_I8>(p, grid, s, handled); break;
    case FNN_DT_I4: e = launch_dt<FNN_DT_I4>(p, grid, s, handled); break;
    default: e = launch_dt<FNN_DT_U4>(p, grid, s, handled); break;
    }
    if (e != hipSuccess) { *handled = false; return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e)); }
    return FNN_OK;
}
