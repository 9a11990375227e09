// Matrix-core quantised MatMul for gfx950: packed weights are streamed from HBM exactly
// once, decoded in registers to f16 (integer lanes, E4M3/E5M2 and E2M1 values are all exact
// in f16) and fed to v_mfma_f32_16x16x32_f16 against the activation tile held in LDS.
//
//   out[m,n] = act((sum_k A[m,k]*u(W[n,k]))*scale[n] + zero[n]*sum_k A[m,k] + bias[n])
//   (gemm_batch_packed_simd + apply_affine_dot, src/backend/cpu/microkernels/gemm.rs:1982-2088,
//    src/backend/cpu/microkernels/mod.rs:283-295)
//
// Activations stay f32-accurate: each row of a K-chunk is scaled by a power of two into
// f16 range and split into hi + lo f16 terms (two MFMAs per step, ~22 mantissa bits); the
// chunk's partial product is scaled back in f32.  FNN_FLAG_ACT_F16_SINGLE keeps hi only.
//
// Decomposition: a workgroup owns R*16 weight rows and all of K; its waves take turns on
// 128-byte row segments (lane (n,g) holds 32 contiguous packed bytes of row n); per wave the
// same A fragments serve R weight row tiles and MTL activation row tiles; wave partials are
// reduced through LDS in a fixed order and the affine/bias/activation epilogue is fused.
// Up to M = 16*MTL activation rows per launch; bandwidth-bound while M is small.
#include "mfma.h"
#include "dech.h"

#include <cstdlib>

namespace {

using namespace dech;

struct MfmaArgs {
    const uint32_t *words;
    const float *scales, *zeros, *a, *bias;
    float *out;
    int64_t m, n, k, kp;
    int act, kc, single;
};

constexpr int NLOAD = 2;  // 16-byte loads per lane and row tile: 32 contiguous bytes, 128 per row

template <int DT, int MTL, int R, int PF, int MAXT>
__global__ void __launch_bounds__(MAXT) qmm_mfma_kernel(MfmaArgs p)
{
    using D = DecH<DT>;
    constexpr int WPS = D::WPS;
    constexpr int SPT = NLOAD * 4 / WPS;   // MFMA steps per tile (8 for 4-bit, 4 for 8-bit types)
    constexpr int KT = 4 * SPT * 8;        // k-values per tile (256 / 128)
    constexpr int MR = MTL * 16;
    constexpr int MAXW = MAXT / 64;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int KC = p.kc;
    const int ngrp = KC / 8;                      // 16-byte A groups per row and chunk
    const int mr = p.m < MR ? (int)p.m : MR;      // activation rows held in LDS
    uint4 *a_hi = reinterpret_cast<uint4 *>(smem);
    uint4 *a_lo = a_hi + (size_t)ngrp * mr;
    float *fbase = reinterpret_cast<float *>(a_lo + (p.single ? 0 : (size_t)ngrp * mr));
    const int SEG = KC / 512;                     // 64-group segments per row
    float *pmax = fbase;                          // [MR*SEG]
    float *psum = pmax + MR * SEG;                // [MR*SEG]
    float *cscale = psum + MR * SEG;              // [MR]
    float *xtot = cscale + MR;                    // [MR]
    float *red = reinterpret_cast<float *>(smem); // reuses the A area after the last chunk

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = tid >> 6;
    const int nw = blockDim.x >> 6;
    const int ln = lane & 15;   // weight row / activation row within a 16-tile
    const int g = lane >> 4;    // k-group
    const int64_t K = p.k, N = p.n, M = p.m, kp = p.kp;
    const int64_t n0 = (int64_t)blockIdx.x * (R * 16);

    if (tid < MR) xtot[tid] = 0.0f;

    f32x4 tot[MTL][R];
#pragma unroll
    for (int mt = 0; mt < MTL; mt++)
#pragma unroll
        for (int r = 0; r < R; r++) tot[mt][r] = f32x4{0.f, 0.f, 0.f, 0.f};

    const uint32_t *wrow[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        int64_t row = n0 + r * 16 + ln;
        if (row > N - 1) row = N - 1;
        wrow[r] = p.words + row * kp;
    }

    // lane (n,g) of tile T: words [T*32 + g*8, +8) of its row, i.e. 32 contiguous packed bytes
    auto load_tile = [&](int64_t tglob, uint32_t(&wq)[R][NLOAD * 4]) {
        const int64_t woff = tglob * 32 + g * (NLOAD * 4);
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int q = 0; q < NLOAD; q++) {
                uint4 t = make_uint4(0, 0, 0, 0);
                if (woff + q * 4 + 4 <= kp) t = *reinterpret_cast<const uint4 *>(wrow[r] + woff + q * 4);
                wq[r][q * 4 + 0] = t.x; wq[r][q * 4 + 1] = t.y; wq[r][q * 4 + 2] = t.z; wq[r][q * 4 + 3] = t.w;
            }
    };
    // Single-chunk launches request the wave's first PF tiles before anything else, so the
    // HBM stream is in flight while the activations are converted.
    uint32_t pre[PF > 0 ? PF : 1][R][NLOAD * 4];
    if constexpr (PF > 0) {
#pragma unroll
        for (int i = 0; i < PF; i++) load_tile(wv + i * nw, pre[i]);
    }

    for (int64_t c0 = 0; c0 < K; c0 += KC) {
        // ---- pass 1: per-row max |x| of this chunk (64-group segments, one per wave turn)
        const int nwi = mr * SEG;
        for (int wi = wv; wi < nwi; wi += nw) {
            const int row = wi / SEG, seg = wi % SEG;
            float mx = 0.0f;
            if (row < M) {
                const int64_t kk = c0 + ((int64_t)seg * 64 + lane) * 8;
                if (kk < K) {  // K % 8 == 0: a group is entirely inside or outside
                    const float4 x0 = *reinterpret_cast<const float4 *>(p.a + row * K + kk);
                    const float4 x1 = *reinterpret_cast<const float4 *>(p.a + row * K + kk + 4);
                    mx = fmaxf(fmaxf(fmaxf(fabsf(x0.x), fabsf(x0.y)), fmaxf(fabsf(x0.z), fabsf(x0.w))),
                               fmaxf(fmaxf(fabsf(x1.x), fabsf(x1.y)), fmaxf(fabsf(x1.z), fabsf(x1.w))));
                }
            }
            mx = wave_max(mx);
            if (lane == 0) pmax[wi] = mx;
        }
        __syncthreads();
        // ---- pass 2: scale into f16 range, split hi/lo, store in fragment order
        for (int wi = wv; wi < nwi; wi += nw) {
            const int row = wi / SEG, seg = wi % SEG;
            float mx = 0.0f;
            for (int s2 = 0; s2 < SEG; s2++) mx = fmaxf(mx, pmax[row * SEG + s2]);
            // power of two e with max*2^-e in [2^14, 2^15); clamped so that 2^-e stays finite
            int ex = (int)((__float_as_uint(mx) >> 23) & 0xff) - 127 - 14;
            if (mx == 0.0f) ex = 0;
            ex = ex < -100 ? -100 : (ex > 120 ? 120 : ex);
            const float inv = __uint_as_float((uint32_t)(127 - ex) << 23);
            if (seg == 0 && lane == 0) cscale[row] = __uint_as_float((uint32_t)(127 + ex) << 23);
            const int kg = seg * 64 + lane;  // group index inside the chunk
            float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            const int64_t kk = c0 + (int64_t)kg * 8;
            if (row < M && kk < K) {
                const float4 x0 = *reinterpret_cast<const float4 *>(p.a + row * K + kk);
                const float4 x1 = *reinterpret_cast<const float4 *>(p.a + row * K + kk + 4);
                x[0] = x0.x; x[1] = x0.y; x[2] = x0.z; x[3] = x0.w;
                x[4] = x1.x; x[5] = x1.y; x[6] = x1.z; x[7] = x1.w;
            }
            float s = ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
            s = wave_sum(s);
            if (lane == 0) psum[wi] = s;
            _Float16 hi[8], lo[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int src = D::INTERLEAVED ? ((j >> 1) + 4 * (j & 1)) : j;
                const float v = x[src] * inv;
                hi[j] = (_Float16)v;
                lo[j] = (_Float16)(v - (float)hi[j]);
            }
            // group kg -> tile dt, k-group gg, step st; stored at ((dt*SPT + st)*mr + row)*4 + gg
            const int dt = kg / (KT / 8), rr = kg % (KT / 8);
            const int gg = rr / SPT, st = rr % SPT;
            const size_t dst = ((size_t)(dt * SPT + st) * mr + row) * 4 + gg;
            a_hi[dst] = __builtin_bit_cast(uint4, f16x8{hi[0], hi[1], hi[2], hi[3], hi[4], hi[5], hi[6], hi[7]});
            if (!p.single)
                a_lo[dst] = __builtin_bit_cast(uint4, f16x8{lo[0], lo[1], lo[2], lo[3], lo[4], lo[5], lo[6], lo[7]});
        }
        __syncthreads();
        if (tid < mr) {
            float s = 0.0f;
            for (int s2 = 0; s2 < SEG; s2++) s += psum[tid * SEG + s2];
            xtot[tid] += s;
        }

        // ---- MFMA phase: wave w takes tiles w, w+nw, ... of this chunk
        f32x4 acc[MTL][R];
#pragma unroll
        for (int mt = 0; mt < MTL; mt++)
#pragma unroll
            for (int r = 0; r < R; r++) acc[mt][r] = f32x4{0.f, 0.f, 0.f, 0.f};
        const int ntile = KC / KT;
        auto compute_tile = [&](int dt, uint32_t(&wq)[R][NLOAD * 4]) {
#pragma unroll
            for (int st = 0; st < SPT; st++) {
                f16x8 ah[MTL], al[MTL];
#pragma unroll
                for (int mt = 0; mt < MTL; mt++) {
                    const int row = mt * 16 + ln;
                    uint4 vh = make_uint4(0, 0, 0, 0), vl = make_uint4(0, 0, 0, 0);
                    if (row < M) {
                        const size_t src = ((size_t)(dt * SPT + st) * mr + row) * 4 + g;
                        vh = a_hi[src];
                        if (!p.single) vl = a_lo[src];
                    }
                    ah[mt] = __builtin_bit_cast(f16x8, vh);
                    al[mt] = __builtin_bit_cast(f16x8, vl);
                }
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const f16x8 b = D::step(&wq[r][st * WPS]);
#pragma unroll
                    for (int mt = 0; mt < MTL; mt++) {
                        // operands: first = activations (rows m), second = weights (cols n)
                        acc[mt][r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah[mt], b, acc[mt][r], 0, 0, 0);
                        if (!p.single)
                            acc[mt][r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al[mt], b, acc[mt][r], 0, 0, 0);
                    }
                }
            }
        };
        if constexpr (PF > 0) {
#pragma unroll
            for (int i = 0; i < PF; i++) {
                const int dt = wv + i * nw;
                if (dt < ntile && (int64_t)dt * 32 < kp) compute_tile(dt, pre[i]);
            }
        }
        for (int dt = wv + PF * nw; dt < ntile; dt += nw) {
            const int64_t tglob = c0 / KT + dt;
            if (tglob * 32 >= kp) continue;  // tile beyond the row end (wave-uniform)
            uint32_t wq[R][NLOAD * 4];
            load_tile(tglob, wq);
            compute_tile(dt, wq);
        }
        // chunk partial back to the activations' scale: acc[i] is row (g*4 + i) of the tile
#pragma unroll
        for (int mt = 0; mt < MTL; mt++) {
            float cs[4];
#pragma unroll
            for (int i = 0; i < 4; i++) cs[i] = (mt * 16 + g * 4 + i < mr) ? cscale[mt * 16 + g * 4 + i] : 1.0f;
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int i = 0; i < 4; i++) tot[mt][r][i] = fmaf(acc[mt][r][i], cs[i], tot[mt][r][i]);
        }
        __syncthreads();  // LDS is rewritten by the next chunk (or by the reduction below)
    }

    // ---- reduce the waves' partial tiles in a fixed order, fused epilogue
    __shared__ float xtot_s[MR];
    if (tid < MR) xtot_s[tid] = xtot[tid];
    __syncthreads();
#pragma unroll
    for (int mt = 0; mt < MTL; mt++)
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                red[(((size_t)wv * MTL + mt) * R + r) * 256 + i * 64 + lane] = tot[mt][r][i];
    __syncthreads();
    for (int idx = tid; idx < MTL * R * 256; idx += blockDim.x) {
        const int e = idx & 255, tr = idx >> 8;
        const int r = tr % R, mt = tr / R;
        const int l2 = e & 63, i = e >> 6;
        const int64_t mrow = mt * 16 + (l2 >> 4) * 4 + i;
        const int64_t ncol = n0 + r * 16 + (l2 & 15);
        if (mrow >= M || ncol >= N) continue;
        float dot = 0.0f;
        for (int w = 0; w < nw; w++) dot += red[(((size_t)w * MTL + mt) * R + r) * 256 + e];
        p.out[mrow * N + ncol] = fnn_epilogue(dot, p.scales[ncol], p.zeros[ncol], xtot_s[mrow], p.bias, ncol, p.act);
    }
    (void)MAXW;
}

int env_int(const char *name, int dflt)
{
    const char *s = getenv(name);
    return (s && *s) ? atoi(s) : dflt;
}

template <int DT, int MTL, int R, int PF>
hipError_t launch_cfg(const MfmaArgs &p0, int nw, hipStream_t s)
{
    constexpr int MAXT = 512;
    constexpr int MR = MTL * 16;
    MfmaArgs p = p0;
    // K-chunk: largest multiple of 512 whose hi/lo activation tiles fit the LDS budget
    const int64_t kpad = (p.k + 511) / 512 * 512;
    const size_t budget = 96 * 1024;
    const int mr = p.m < MR ? (int)p.m : MR;
    const size_t per_k = (size_t)mr * 2 * (p.single ? 1 : 2);
    int kc = 32768;
    while (kc > 512 && ((size_t)kc * per_k > budget || kc / 2 >= kpad)) kc /= 2;
    if (kc > kpad) kc = (int)kpad;
    if (PF > 0 && kc < kpad) return hipErrorInvalidValue;  // prefetching needs a single chunk
    p.kc = kc;
    size_t lds = (size_t)kc * per_k + (size_t)(2 * MR * (kc / 512) + 2 * MR) * 4 + 64;
    const size_t red = (size_t)nw * MTL * R * 256 * 4;
    if (red > lds) lds = red;
    auto kern = qmm_mfma_kernel<DT, MTL, R, PF, MAXT>;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 2048);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int64_t grid = (p.n + R * 16 - 1) / (R * 16);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(nw * 64), lds, s, p);
    return hipGetLastError();
}

// true when M x Kpad activations (hi+lo f16) fit one LDS chunk
inline bool single_chunk(const MfmaArgs &p, int mr)
{
    const int64_t kpad = (p.k + 511) / 512 * 512;
    return (size_t)kpad * mr * 2 * (p.single ? 1 : 2) <= 96 * 1024 && kpad <= 32768;
}

template <int DT, int MTL>
hipError_t launch_r(const MfmaArgs &p, hipStream_t s)
{
    static const int env_nw = env_int("FNN_MFMA_NW", 0);
    static const int env_r = env_int("FNN_MFMA_R", 0);
    static const int env_pf = env_int("FNN_MFMA_PF", -1);
    constexpr int KT = DecH<DT>::WPS == 1 ? 256 : 128;
    int nw = 8;
    int r = (MTL >= 2) ? 2 : 1;
    if (env_nw > 0) nw = env_nw > 8 ? 8 : env_nw;
    if (env_r > 0) r = env_r;
    if (MTL * r > 8) r = 8 / MTL;
    if constexpr (MTL == 1) {
        // GEMV regime (M <= 16): the whole activation fits one chunk for the usual K; request
        // every tile of the wave up front (2 or 4 tiles of 32 bytes per lane and row tile)
        const int mr = p.m < 16 ? (int)p.m : 16;
        const int64_t tiles_per_wave = ((p.k + KT - 1) / KT + nw - 1) / nw;
        int pf = 0;
        if (single_chunk(p, mr)) pf = tiles_per_wave <= 2 ? 2 : 4;
        if (env_pf >= 0) pf = env_pf;
        if (r == 1) {
            if (pf == 2) return launch_cfg<DT, 1, 1, 2>(p, nw, s);
            if (pf == 4) return launch_cfg<DT, 1, 1, 4>(p, nw, s);
            return launch_cfg<DT, 1, 1, 0>(p, nw, s);
        }
        if (pf == 2) return launch_cfg<DT, 1, 2, 2>(p, nw, s);
        return launch_cfg<DT, 1, 2, 0>(p, nw, s);
    } else {
        if (r == 1) return launch_cfg<DT, MTL, 1, 0>(p, nw, s);
        return launch_cfg<DT, MTL, 2, 0>(p, nw, s);
    }
}

template <int DT>
hipError_t launch_m(const MfmaArgs &p0, hipStream_t s)
{
    // up to 64 activation rows per launch; larger M runs in row slabs
    MfmaArgs p = p0;
    int64_t m0 = 0;
    while (m0 < p0.m) {
        int64_t mt = p0.m - m0;
        if (mt > 64) mt = 64;
        p.a = p0.a + m0 * p0.k;
        p.out = p0.out + m0 * p0.n;
        p.m = mt;
        hipError_t e;
        if (mt <= 16) e = launch_r<DT, 1>(p, s);
        else if (mt <= 32) e = launch_r<DT, 2>(p, s);
        else e = launch_r<DT, 4>(p, s);
        if (e != hipSuccess) return e;
        m0 += mt;
    }
    return hipSuccess;
}

}  // namespace

int fnn_mfma_qmatmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q,
                     int flags, bool *handled)
{
    *handled = false;
    if (w->dtype == FNN_DT_I4CB) return FNN_OK;                       // codebook type: FMA / generic kernels
    if (q.kp % 4 != 0 || q.k % 8 != 0) return FNN_OK;                 // 16-byte row pieces, whole k-groups
    if ((reinterpret_cast<uintptr_t>(q.a) & 15) || (reinterpret_cast<uintptr_t>(q.words) & 15)) return FNN_OK;
    MfmaArgs p;
    p.words = q.words; p.scales = q.scales; p.zeros = q.zeros; p.a = q.a; p.bias = q.bias; p.out = q.out;
    p.m = q.m; p.n = q.n; p.k = q.k; p.kp = q.kp; p.act = q.act; p.kc = 0;
    p.single = (flags & FNN_FLAG_ACT_F16_SINGLE) ? 1 : 0;
    hipError_t e;
    switch (w->dtype) {
    case FNN_DT_I8: e = launch_m<FNN_DT_I8>(p, s); break;
    case FNN_DT_I4: e = launch_m<FNN_DT_I4>(p, s); break;
    case FNN_DT_U8: e = launch_m<FNN_DT_U8>(p, s); break;
    case FNN_DT_U4: e = launch_m<FNN_DT_U4>(p, s); break;
    case FNN_DT_F8: e = launch_m<FNN_DT_F8>(p, s); break;
    case FNN_DT_F8R: e = launch_m<FNN_DT_F8R>(p, s); break;
    case FNN_DT_F4: e = launch_m<FNN_DT_F4>(p, s); break;
    default: return FNN_OK;
    }
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    *handled = true;
    return FNN_OK;
}

int fnn_mfma_qmatmul_i8act(fnn_hip_ctx *, hipStream_t, const fnn_hip_weight *, const I8ActArgs &, bool *handled)
{
    *handled = false;
    return FNN_OK;
}
