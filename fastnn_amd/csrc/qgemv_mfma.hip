// Bandwidth-bound quantised GEMV on the matrix cores (M <= 4 activation rows) for gfx950.
//
//   out[m,n] = act((sum_k A[m,k]*u(W[n,k]))*scale[n] + zero[n]*sum_k A[m,k] + bias[n])
//   (gemm_batch_packed_simd + apply_affine_dot, src/backend/cpu/microkernels/gemm.rs:1982-2088,
//    src/backend/cpu/microkernels/mod.rs:283-295)
//
// The f32 FMA form of this GEMV is VALU-bound for 4-bit weights (unpack + convert + FMA per
// element).  Here the packed words are turned into f16 operands with ~1 VALU op per
// element and v_mfma_f32_16x16x32_f16 does the multiply-accumulate, so the kernel runs at
// the speed the weights arrive from HBM.
//
// One workgroup = RT*16 weight rows x all of K, 8 waves.  Wave w owns the K slice
// [w*512, (w+1)*512) of every round of 4096 k-values:
//   1. it requests all of its packed bytes first (lane (n,g): row n, 16 bytes per tile);
//   2. while they are in flight it converts its own slice of the activations: one group of
//      8 floats per lane and row, scaled by a power of two taken from the slice maximum,
//      split into hi + lo f16 and written to the wave's LDS area in operand order;
//   3. MFMA steps, scale the slice partial back in f32;
//   4. partial 16x16 tiles and activation sums of the 8 waves are added in a fixed order
//      through LDS and the affine / bias / activation epilogue is applied.
// Algorithmic bytes per launch: N*K*bits/8 + side tables + 4*M*(K+N).
#include "dech.h"
#include "mfma.h"

#include <cstdlib>

namespace {

using namespace dech;

struct GemvArgs {
    const uint32_t *words;
    const float *scales, *zeros, *a, *bias;
    float *out;
    int64_t m, n, k, kp;
    int act, single;
};

constexpr int GV_NW = 8;        // waves per workgroup
constexpr int GV_SLICE = 512;   // k-values per wave and round (64 groups of 8: one per lane)
constexpr int GV_MMAX = 4;

template <int DT, int RT, int MM>
__global__ void __launch_bounds__(GV_NW * 64) qgemv_mfma_kernel(GemvArgs p)
{
    using D = DecH<DT>;
    constexpr int WPS = D::WPS;
    constexpr int SPT = 4 / WPS;            // MFMA steps per 16-byte lane load (4 / 2)
    constexpr int KT = 4 * SPT * 8;         // k-values per tile (128 / 64)
    constexpr int TPW = GV_SLICE / KT;      // tiles per wave and round (4 / 8)
    constexpr int NSTEP = TPW * SPT;        // MFMA steps per wave and round (16)

    // dynamic LDS: per wave [NSTEP][M][4 g] 16-byte fragments (hi plane, then lo plane)
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int frag_per_wave = NSTEP * MM * 4;
    uint4 *a_hi_w = reinterpret_cast<uint4 *>(smem) + (size_t)(threadIdx.x >> 6) * frag_per_wave;
    uint4 *a_lo_w = a_hi_w + (size_t)GV_NW * frag_per_wave;
    __shared__ float red[GV_NW][RT][64];
    __shared__ float xred[GV_NW][GV_MMAX];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = tid >> 6;
    const int ln = lane & 15;
    const int g = lane >> 4;
    const int64_t K = p.k, N = p.n, kp = p.kp;
    constexpr int M = MM;  // activation rows of this instantiation (1, 2 or 4; p.m <= MM)
    const int mreal = (int)p.m;
    const int64_t n0 = (int64_t)blockIdx.x * (RT * 16);

    const uint32_t *wrow[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) {
        int64_t row = n0 + r * 16 + ln;
        if (row > N - 1) row = N - 1;
        wrow[r] = p.words + row * kp;
    }

    f32x4 tot[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) tot[r] = f32x4{0.f, 0.f, 0.f, 0.f};
    float xsum[GV_MMAX] = {0.f, 0.f, 0.f, 0.f};

    const int64_t round_k = (int64_t)GV_NW * GV_SLICE;
    for (int64_t k0 = 0; k0 < K; k0 += round_k) {
        const int64_t ks = k0 + (int64_t)wv * GV_SLICE;  // first k of this wave's slice
        // ---- 0. this lane's group of 8 activations per row: requested ahead of the weight
        //         stream so that it does not queue behind it
        const int64_t kk = ks + (int64_t)lane * 8;
        float xr[MM][8];
#pragma unroll
        for (int m = 0; m < MM; m++) {
#pragma unroll
            for (int j = 0; j < 8; j++) xr[m][j] = 0.0f;
            if (m < mreal && kk < K) {  // K % 8 == 0
                const float4 x0 = *reinterpret_cast<const float4 *>(p.a + (int64_t)m * K + kk);
                const float4 x1 = *reinterpret_cast<const float4 *>(p.a + (int64_t)m * K + kk + 4);
                xr[m][0] = x0.x; xr[m][1] = x0.y; xr[m][2] = x0.z; xr[m][3] = x0.w;
                xr[m][4] = x1.x; xr[m][5] = x1.y; xr[m][6] = x1.z; xr[m][7] = x1.w;
            }
        }
        // ---- 1. request the packed bytes: tile t, lane (n,g): words [ (ks + t*KT)/EPW + g*4, +4 )
        uint32_t wq[RT][TPW * 4];
        const int64_t wbase = ks * 4 / (8 * SPT);         // word offset of the slice (ks * bits / 32)
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int t = 0; t < TPW; t++) {
                const int64_t woff = wbase + t * 16 + g * 4;
                uint4 v = make_uint4(0, 0, 0, 0);
                if (woff + 4 <= kp) v = *reinterpret_cast<const uint4 *>(wrow[r] + woff);
                wq[r][t * 4 + 0] = v.x; wq[r][t * 4 + 1] = v.y; wq[r][t * 4 + 2] = v.z; wq[r][t * 4 + 3] = v.w;
            }

        // ---- 2. this wave's activation slice -> f16 hi/lo fragments in its LDS area
        float csc[GV_MMAX] = {1.f, 1.f, 1.f, 1.f};
        {
            // group -> (tile, g, step) and fragment slot (step*M + m)*4 + g
            const int kl = lane * 8;
            const int t = kl / KT, rr = kl % KT;
            const int gg = rr / (SPT * 8), st = (rr % (SPT * 8)) / 8;
#pragma unroll
            for (int m = 0; m < MM; m++) {
                const float *x = xr[m];
                float mx = fmaxf(fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3]))),
                                 fmaxf(fmaxf(fabsf(x[4]), fabsf(x[5])), fmaxf(fabsf(x[6]), fabsf(x[7]))));
                mx = wave_max(mx);
                const float s = wave_sum(((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7])));
                xsum[m] += s;
                // power of two e with max*2^-e in [2^14, 2^15), clamped so that 2^-e is finite
                int ex = (int)((__float_as_uint(mx) >> 23) & 0xff) - 127 - 14;
                if (mx == 0.0f) ex = 0;
                ex = ex < -100 ? -100 : (ex > 120 ? 120 : ex);
                const float inv = __uint_as_float((uint32_t)(127 - ex) << 23);
                csc[m] = __uint_as_float((uint32_t)(127 + ex) << 23);
                _Float16 hi[8], lo[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int src = D::INTERLEAVED ? ((j >> 1) + 4 * (j & 1)) : j;
                    const float v = x[src] * inv;
                    hi[j] = (_Float16)v;
                    lo[j] = (_Float16)(v - (float)hi[j]);
                }
                const int dst = ((t * SPT + st) * M + m) * 4 + gg;
                a_hi_w[dst] = __builtin_bit_cast(uint4, f16x8{hi[0], hi[1], hi[2], hi[3], hi[4], hi[5], hi[6], hi[7]});
                if (!p.single)
                    a_lo_w[dst] = __builtin_bit_cast(uint4, f16x8{lo[0], lo[1], lo[2], lo[3], lo[4], lo[5], lo[6], lo[7]});
            }
        }
        __syncthreads();

        // ---- 3. MFMA over the slice
        f32x4 acc[RT], acl[RT];  // hi and lo terms keep separate dependency chains
#pragma unroll
        for (int r = 0; r < RT; r++) acc[r] = acl[r] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < TPW; t++)
#pragma unroll
            for (int st = 0; st < SPT; st++) {
                uint4 vh = make_uint4(0, 0, 0, 0), vl = make_uint4(0, 0, 0, 0);
                if (ln < M) {
                    const int src = ((t * SPT + st) * M + ln) * 4 + g;
                    vh = a_hi_w[src];
                    if (!p.single) vl = a_lo_w[src];
                }
                const f16x8 ah = __builtin_bit_cast(f16x8, vh);
                const f16x8 al = __builtin_bit_cast(f16x8, vl);
#pragma unroll
                for (int r = 0; r < RT; r++) {
                    const f16x8 b = D::step(&wq[r][t * 4 + st * WPS]);
                    acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, b, acc[r], 0, 0, 0);
                    if (!p.single) acl[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, b, acl[r], 0, 0, 0);
                }
            }
        // acc[i] is activation row g*4 + i: only g == 0 carries rows < 4
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int i = 0; i < 4; i++) tot[r][i] = fmaf(acc[r][i] + acl[r][i], csc[i], tot[r][i]);
        __syncthreads();  // the wave areas are rewritten by the next round
    }

    // ---- 4. fixed-order reduction over the waves, fused epilogue
    if (g == 0) {
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int i = 0; i < 4; i++) red[wv][r][i * 16 + ln] = tot[r][i];
    }
    if (lane == 0) {
#pragma unroll
        for (int m = 0; m < GV_MMAX; m++) xred[wv][m] = xsum[m];
    }
    __syncthreads();
    for (int idx = tid; idx < RT * 64; idx += GV_NW * 64) {
        const int r = idx >> 6, e = idx & 63;
        const int m = e >> 4;
        const int64_t n = n0 + r * 16 + (e & 15);
        if (m >= mreal || n >= N) continue;
        float dot = 0.0f, xs = 0.0f;
#pragma unroll
        for (int w = 0; w < GV_NW; w++) {
            dot += red[w][r][e];
            xs += xred[w][m];
        }
        p.out[(int64_t)m * N + n] = fnn_epilogue(dot, p.scales[n], p.zeros[n], xs, p.bias, n, p.act);
    }
}

template <int DT>
hipError_t launch_gemv(const GemvArgs &p, hipStream_t s)
{
    static const int env_rt = []() { const char *e = getenv("FNN_GEMV_MFMA_RT"); return (e && *e) ? atoi(e) : 0; }();
    int rt = (p.n >= 16384) ? 2 : 1;
    if (env_rt > 0) rt = env_rt;
    // hi (+ lo) fragment planes: 8 waves x 16 steps x M rows x 4 groups x 16 bytes
    const int mm = p.m <= 1 ? 1 : (p.m <= 2 ? 2 : 4);
    const size_t lds = (size_t)GV_NW * 16 * (size_t)mm * 4 * 16 * (p.single ? 1 : 2);
    const dim3 g1((unsigned)((p.n + 15) / 16)), g2((unsigned)((p.n + 31) / 32)), blk(GV_NW * 64);
    if (rt == 2) {
        if (mm == 1) hipLaunchKernelGGL((qgemv_mfma_kernel<DT, 2, 1>), g2, blk, lds, s, p);
        else if (mm == 2) hipLaunchKernelGGL((qgemv_mfma_kernel<DT, 2, 2>), g2, blk, lds, s, p);
        else hipLaunchKernelGGL((qgemv_mfma_kernel<DT, 2, 4>), g2, blk, lds, s, p);
    } else {
        if (mm == 1) hipLaunchKernelGGL((qgemv_mfma_kernel<DT, 1, 1>), g1, blk, lds, s, p);
        else if (mm == 2) hipLaunchKernelGGL((qgemv_mfma_kernel<DT, 1, 2>), g1, blk, lds, s, p);
        else hipLaunchKernelGGL((qgemv_mfma_kernel<DT, 1, 4>), g1, blk, lds, s, p);
    }
    return hipGetLastError();
}

}  // namespace

int fnn_mfma_qgemv(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q,
                   int flags, bool *handled)
{
    *handled = false;
    if (q.m < 1 || q.m > GV_MMAX || w->dtype == FNN_DT_I4CB) return FNN_OK;
    if (q.kp % 4 != 0 || q.k % 8 != 0) return FNN_OK;
    if ((reinterpret_cast<uintptr_t>(q.a) & 15) || (reinterpret_cast<uintptr_t>(q.words) & 15)) return FNN_OK;
    GemvArgs p;
    p.words = q.words; p.scales = q.scales; p.zeros = q.zeros; p.a = q.a; p.bias = q.bias; p.out = q.out;
    p.m = q.m; p.n = q.n; p.k = q.k; p.kp = q.kp; p.act = q.act;
    p.single = (flags & FNN_FLAG_ACT_F16_SINGLE) ? 1 : 0;
    hipError_t e;
    switch (w->dtype) {
    case FNN_DT_I8: e = launch_gemv<FNN_DT_I8>(p, s); break;
    case FNN_DT_I4: e = launch_gemv<FNN_DT_I4>(p, s); break;
    case FNN_DT_U8: e = launch_gemv<FNN_DT_U8>(p, s); break;
    case FNN_DT_U4: e = launch_gemv<FNN_DT_U4>(p, s); break;
    case FNN_DT_F8: e = launch_gemv<FNN_DT_F8>(p, s); break;
    case FNN_DT_F8R: e = launch_gemv<FNN_DT_F8R>(p, s); break;
    case FNN_DT_F4: e = launch_gemv<FNN_DT_F4>(p, s); break;
    default: return FNN_OK;
    }
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    *handled = true;
    return FNN_OK;
}
