// Bandwidth-bound quantised GEMV on the matrix cores (M <= 8 activation rows) for gfx950.
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
// One workgroup = RT*16 weight rows (RT = 1..3, chosen per shape) x all of K, 8 waves.  Wave w owns the K slice
// [w*512, (w+1)*512) of every round of 4096 k-values:
//   0. it requests its slice of the activations, then
//   1. all of its packed bytes (lane (n,g): row n, 16 bytes per tile); scheduling barriers pin this order
//      (left alone, the compiler sinks most of these requests below step 2 and puts step 3's waits into it);
//   2. while they are in flight it converts the activations: one group of 8 floats per lane
//      and row, scaled by a power of two taken from the slice maximum and split into hi + lo
//      f16 terms.  hi and lo occupy DIFFERENT ROWS of the 16-row MFMA operand (rows 0..M-1
//      and M..2M-1), so one MFMA per step yields both partial products;
//   3. MFMA steps; the slice partial is scaled back in f32;
//   4. partial tiles and activation sums of the 8 waves are added in a fixed order through
//      LDS (hi row + lo row), and the affine / bias / activation epilogue is applied.
// Operand rows >= 2M are never read back, so their lanes load a clamped (valid) row
// instead of zeros and no lane masking is needed in the inner loop.
// Algorithmic bytes per launch: N*K*bits/8 + side tables + 4*M*(K+N).
#include "dech.h"
#include "mfma.h"

#include <cstdlib>

namespace {

using namespace dech;

struct GemvArgs {
    const uint32_t *words;
    const float *scales, *zeros, *a, *bias;
    const float *umean;   // single-f16 mode: mean lane value per weight row, or null
    float *out;
    int64_t m, n, k, kp;
    int act;
    const uint32_t *words_tm;   // non-null: the words in blocks of 16 rows x 64 bytes ([row block][k block][row][64 bytes]),
    int64_t kb64;               // kb64 k blocks per row: a wave load is then one contiguous KB
};

constexpr int GV_NW = 8;        // waves per workgroup
constexpr int GV_SLICE = 512;   // k-values per wave and round (64 groups of 8: one per lane)
constexpr int GV_MMAX = 8;

// TMAJ: the packed words come from the tile-major copy (a wave load = the contiguous KB of one 16-row x 64-byte block)
template <int DT, int RT, int MM, bool SINGLE, int NW, bool TMAJ = false>
__global__ void __launch_bounds__(NW * 64) qgemv_mfma_kernel(GemvArgs p)
{
    using D = DecH<DT>;
    constexpr int WPS = D::WPS;
    constexpr int SPT = 4 / WPS;            // MFMA steps per 16-byte lane load (4 / 2)
    constexpr int KT = 4 * SPT * 8;         // k-values per tile (128 / 64)
    constexpr int TPW = GV_SLICE / KT;      // tiles per wave and round (4 / 8)
    constexpr int NSTEP = TPW * SPT;        // MFMA steps per wave and round (16)
    constexpr int ROWS = SINGLE ? MM : 2 * MM;  // operand rows in use: hi rows, then lo rows

    // per wave: [NSTEP][ROWS][4 g] 16-byte operand fragments
    extern __shared__ __attribute__((aligned(16))) uint4 frag_dyn[];  // GV_NW * NSTEP * ROWS * 4
    constexpr int RROWS = ROWS > 8 ? 16 : 8;   // operand rows kept for the reduction
    __shared__ float red[GV_NW][RT][RROWS][16];
    __shared__ float xred[GV_NW][GV_MMAX];
    __shared__ float ered[GV_NW][GV_MMAX];   // single-f16 mode: sum_k (hi - x) per activation row

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = tid >> 6;
    constexpr int nw = NW;                  // waves in this workgroup (compile time: 8, or 4 for K <= 2048)
    const int ln = lane & 15;
    const int g = lane >> 4;
    const int64_t K = p.k, N = p.n, kp = p.kp;
    const int mreal = (int)p.m;             // <= MM
    const int64_t n0 = (int64_t)blockIdx.x * (RT * 16);
    uint4 *fw = frag_dyn + wv * (NSTEP * ROWS * 4);

    const uint32_t *wrow[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) {
        int64_t row = n0 + r * 16 + ln;
        if (row > N - 1) row = N - 1;
        wrow[r] = TMAJ ? p.words_tm + ((row >> 4) * p.kb64) * 256 + (row & 15) * 16 : p.words + row * kp;
    }

    // epilogue operands of the output this thread will finish (idx = tid): requested now,
    // used after the last barrier, so their latency is off the critical path
    const int e_r = (tid / (MM * 16)) % RT, e_m = (tid % (MM * 16)) >> 4, e_c = tid & 15;
    int64_t e_n = n0 + e_r * 16 + e_c;
    const bool e_ok = tid < RT * MM * 16 && e_m < mreal && e_n < N;
    if (e_n > N - 1) e_n = N - 1;
    const float e_scale = p.scales[e_n], e_zero = p.zeros[e_n];
    const float e_bias = p.bias ? p.bias[e_n] : 0.0f;
    const float e_umean = (SINGLE && p.umean) ? p.umean[e_n] : 0.0f;

    f32x4 tot[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) tot[r] = f32x4{0.f, 0.f, 0.f, 0.f};
    float xsum[MM], xerr[MM];
#pragma unroll
    for (int m = 0; m < MM; m++) xsum[m] = xerr[m] = 0.0f;

    // operand fragment this lane reads at step s: row min(ln, ROWS-1), group g
    const int rsel = ln < ROWS ? ln : ROWS - 1;
    const uint4 *frd = fw + rsel * 4 + g;

    const int64_t round_k = (int64_t)nw * GV_SLICE;
    for (int64_t k0 = 0; k0 < K; k0 += round_k) {
        const int64_t ks = k0 + (int64_t)wv * GV_SLICE;  // first k of this wave's slice
        // ---- 0. this lane's group of 8 activations per row, ahead of the weight stream
        const int64_t kk = ks + (int64_t)lane * 8;
        // (loads go to clamped, always valid addresses and are masked afterwards: no branch sits
        //  between a load and the next one, so all of them are in flight together)
        float xr[MM][8];
        const int64_t kkc = kk < K ? kk : K - 8;  // K % 8 == 0
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
        // ---- 1. the packed bytes: tile t, lane (n,g): words [slice + t*16 + g*4, +4) of row n
        // (a chunk past the end of the row re-reads the row's last chunk instead: it only meets activations
        //  that are masked to zero, and the bytes belong to the same output row)
        uint32_t wq[RT][TPW * 4];
        const int64_t wbase = ks * 4 / (8 * SPT);         // word offset of the slice (ks * bits / 32)
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int t = 0; t < TPW; t++) {
                int64_t woff;
                if constexpr (TMAJ) {   // k block min(wbase/16 + t, kb64 - 1) of the row's blocks (1 KB apart), words g*4 of its 64 bytes
                    const int64_t kb = (wbase >> 4) + t;
                    woff = (kb < p.kb64 ? kb : p.kb64 - 1) * 256 + g * 4;
                } else {
                    woff = wbase + t * 16 + g * 4;
                    if (woff + 4 > kp) woff = kp - 4;     // kp % 4 == 0, kp >= 4
                }
                const uint4 v = *reinterpret_cast<const uint4 *>(wrow[r] + woff);
                wq[r][t * 4 + 0] = v.x; wq[r][t * 4 + 1] = v.y; wq[r][t * 4 + 2] = v.z; wq[r][t * 4 + 3] = v.w;
            }
        // every request of the round is issued before anything waits: the activations (oldest requests) are
        // converted while the packed bytes are still on their way
        __builtin_amdgcn_sched_barrier(0);

        // ---- 2. activation slice -> f16 hi/lo operand rows in this wave's LDS area
        float csc[MM];
        {
            // this lane's group -> (tile, g, step); fragment slot (step*ROWS + row)*4 + g
            const int kl = lane * 8;
            const int t = kl / KT, rr = kl % KT;
            const int gg = rr / (SPT * 8), st = (rr % (SPT * 8)) / 8;
            const int slot = (t * SPT + st) * ROWS * 4 + gg;
#pragma unroll
            for (int m = 0; m < MM; m++) {
                const float *x = xr[m];
                float mx = fmaxf(fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3]))),
                                 fmaxf(fmaxf(fabsf(x[4]), fabsf(x[5])), fmaxf(fabsf(x[6]), fabsf(x[7]))));
                mx = wave_max_uniform(mx);
                xsum[m] += wave_sum_uniform(((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7])));
                // power of two e with max*2^-e in [2^14, 2^15), clamped so that 2^-e is finite
                int ex = (int)((__float_as_uint(mx) >> 23) & 0xff) - 127 - 14;
                if (mx == 0.0f) ex = 0;
                ex = ex < -100 ? -100 : (ex > 120 ? 120 : ex);
                const float inv = __uint_as_float((uint32_t)(127 - ex) << 23);
                csc[m] = __uint_as_float((uint32_t)(127 + ex) << 23);
                _Float16 hi[8], lo[8];
                float rerr = 0.0f;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int src = D::INTERLEAVED ? ((j >> 1) + 4 * (j & 1)) : j;
                    const float v = x[src] * inv;
                    hi[j] = (_Float16)v;
                    lo[j] = (_Float16)(v - (float)hi[j]);
                    if (SINGLE) rerr += (float)hi[j] - v;
                }
                // single-f16 mode: the rounding of the row, in the units of x, for the first-order correction
                // dot -= mean_k u[n,k] * sum_k (hi - x)
                if (SINGLE) xerr[m] += csc[m] * wave_sum_uniform(rerr);
                fw[slot + m * 4] = __builtin_bit_cast(uint4, f16x8{hi[0], hi[1], hi[2], hi[3], hi[4], hi[5], hi[6], hi[7]});
                if (!SINGLE)
                    fw[slot + (MM + m) * 4] =
                        __builtin_bit_cast(uint4, f16x8{lo[0], lo[1], lo[2], lo[3], lo[4], lo[5], lo[6], lo[7]});
            }
        }
        // only this wave reads these fragments, and the LDS serves a wave's requests in order: no workgroup
        // barrier, just a point the compiler moves no memory operation across
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_sched_barrier(0);   // nothing of step 3 (it waits for the packed bytes) moves up into step 2

        // ---- 3. MFMA over the slice: straight-line, one MFMA per step and row tile
        f32x4 acc[RT];
#pragma unroll
        for (int r = 0; r < RT; r++) acc[r] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NSTEP; s++) {
            const f16x8 av = __builtin_bit_cast(f16x8, frd[s * ROWS * 4]);
#pragma unroll
            for (int r = 0; r < RT; r++) {
                const f16x8 b = D::step(&wq[r][s * WPS]);   // tile t = s / SPT, step s % SPT
                acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, b, acc[r], 0, 0, 0);
            }
        }
        // acc[i] is operand row g*4 + i, i.e. activation row (g*4 + i) % MM (hi or lo part)
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                // eight activation rows: operand row g*4 + i belongs to activation row (g & 1)*4 + i
                const float cs = MM == 8 ? ((g & 1) ? csc[(4 + i) % MM] : csc[i % MM]) : csc[i % MM];
                tot[r][i] = fmaf(acc[r][i], cs, tot[r][i]);
            }
        __builtin_amdgcn_wave_barrier();  // the wave's own area is rewritten by its next round
    }

    // ---- 4. fixed-order reduction over the waves (hi row + lo row), fused epilogue
    if (g * 4 < RROWS) {
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int i = 0; i < 4; i++) red[wv][r][g * 4 + i][ln] = tot[r][i];
    }
    if (lane == 0) {
#pragma unroll
        for (int m = 0; m < GV_MMAX; m++) {
            xred[wv][m] = m < MM ? xsum[m < MM ? m : 0] : 0.0f;
            ered[wv][m] = m < MM ? xerr[m < MM ? m : 0] : 0.0f;
        }
    }
    __syncthreads();
    if (e_ok) {  // RT*MM*16 <= 128 outputs: one per thread
        float dot = 0.0f, xs = 0.0f, es = 0.0f;
#pragma unroll
        for (int w = 0; w < GV_NW; w++) {   // all reads issued together; absent waves add 0
            const int ws = w < nw ? w : 0;
            float v = red[ws][e_r][e_m][e_c];
            if (!SINGLE) v += red[ws][e_r][MM + e_m][e_c];
            dot += w < nw ? v : 0.0f;
            xs += w < nw ? xred[ws][e_m] : 0.0f;
            if (SINGLE) es += w < nw ? ered[ws][e_m] : 0.0f;
        }
        if (SINGLE) dot = dot - e_umean * es;
        const float v = dot * e_scale + e_zero * xs + e_bias;   // fnn_epilogue with preloaded operands
        p.out[(int64_t)e_m * N + e_n] = fnn_activation(p.bias ? v : dot * e_scale + e_zero * xs, p.act);
    }
}

template <int DT, int RT, bool SINGLE, int NW, bool TMAJ = false>
void launch_rt(const GemvArgs &p, hipStream_t s)
{
    // the tile-major variants exist for the 8-bit types this kernel is the default for (hi + lo activations)
    if constexpr (!TMAJ && !SINGLE && (DT == FNN_DT_U8 || DT == FNN_DT_F8 || DT == FNN_DT_F8R)) {
        if (p.words_tm) return launch_rt<DT, RT, SINGLE, NW, true>(p, s);
    }
    const dim3 grid((unsigned)((p.n + RT * 16 - 1) / (RT * 16))), blk(NW * 64);
    // operand fragments: waves x 16 steps x rows x 4 groups x 16 bytes
    const int mm = p.m <= 1 ? 1 : (p.m <= 2 ? 2 : (p.m <= 4 ? 4 : 8));
    const size_t lds = (size_t)NW * 16 * (SINGLE ? mm : 2 * mm) * 4 * 16;
    if (mm == 1) hipLaunchKernelGGL((qgemv_mfma_kernel<DT, RT, 1, SINGLE, NW, TMAJ>), grid, blk, lds, s, p);
    else if (mm == 2) hipLaunchKernelGGL((qgemv_mfma_kernel<DT, RT, 2, SINGLE, NW, TMAJ>), grid, blk, lds, s, p);
    else if (mm == 4) {
        auto kern = qgemv_mfma_kernel<DT, RT, 4, SINGLE, NW, TMAJ>;
        static std::atomic<uint64_t> lds_raised{0};   // up to 64 KiB of dynamic LDS plus the static reduction buffers
        (void)fnn_raise_lds_limit(lds_raised, reinterpret_cast<const void *>(kern), 96 * 1024);
        hipLaunchKernelGGL(kern, grid, blk, lds, s, p);
    } else {
        auto kern = qgemv_mfma_kernel<DT, RT, 8, SINGLE, NW, TMAJ>;
        static std::atomic<uint64_t> lds_raised{0};   // up to 128 KiB of dynamic LDS: one workgroup per CU
        (void)fnn_raise_lds_limit(lds_raised, reinterpret_cast<const void *>(kern), 128 * 1024);
        hipLaunchKernelGGL(kern, grid, blk, lds, s, p);
    }
}

// Row tiles (of 16 weight rows) per workgroup.  A workgroup converts its activation slice once for all of its
// row tiles, so more tiles mean less repeated work (the larger M, the more it weighs), but the workgroups
// should still come in whole rounds over the 256 CUs: cost ~ rounds * (conversion + tiles).
// C2 (N = 11008): M=2 9.2 -> 8.2 us, M=4 12.3 -> 9.4 us with three tiles; at M=1 one tile is as fast or faster.
inline int gemv_row_tiles(int64_t n, int64_t m, int nw, int forced)
{
    if (m <= 1) return 1;   // one activation row: the conversion is cheap and more workgroups in flight win (measured)
    const int mm = m <= 2 ? 2 : (m <= 4 ? 4 : 8);
    if (forced >= 1 && forced <= 3 && forced * mm * 16 <= nw * 64) return forced;
    const double conv = 0.6 + 0.6 * mm;
    int best = 1;
    double best_cost = 1e30;
    for (int rt = 1; rt <= 3; rt++) {
        if (rt * mm * 16 > nw * 64) break;   // one output per thread in the epilogue
        const int64_t wgs = (n + rt * 16 - 1) / (rt * 16);
        const double cost = (double)((wgs + 255) / 256) * (conv + rt);
        if (cost < best_cost - 1e-9) { best_cost = cost; best = rt; }
    }
    return best;
}

template <int DT, bool SINGLE, int NW>
void launch_mm(const GemvArgs &p, int forced_rt, hipStream_t s)
{
    switch (gemv_row_tiles(p.n, p.m, NW, forced_rt)) {
    case 3: launch_rt<DT, 3, SINGLE, NW>(p, s); break;
    case 2: launch_rt<DT, 2, SINGLE, NW>(p, s); break;
    default: launch_rt<DT, 1, SINGLE, NW>(p, s); break;
    }
}

template <int DT>
hipError_t launch_gemv(const GemvArgs &p, bool single, int forced_rt, hipStream_t s)
{
    // 8 waves split K in slices of 512; short K (<= 2048) runs 4-wave workgroups so that no wave idles
    if (p.k <= 4 * GV_SLICE) {
        if (single) launch_mm<DT, true, 4>(p, forced_rt, s); else launch_mm<DT, false, 4>(p, forced_rt, s);
    } else {
        if (single) launch_mm<DT, true, 8>(p, forced_rt, s); else launch_mm<DT, false, 8>(p, forced_rt, s);
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
    const bool single = (flags & FNN_FLAG_ACT_F16_SINGLE) != 0;
    p.words_tm = nullptr; p.kb64 = 0;
    if (!single && (w->dtype == FNN_DT_U8 || w->dtype == FNN_DT_F8 || w->dtype == FNN_DT_F8R))
        if (int rc = fnn_tile_major_words(ctx, s, w, q, &p.words_tm, &p.kb64)) return rc;
    p.umean = nullptr;
    if (single) {
        int rc = fnn_row_means(ctx, s, w, &p.umean);
        if (rc) return rc;
    }
    const int rt = (int)fnn_ctx_option(ctx, FNN_OPT_GEMV_ROW_TILES);   // 0: by the cost model
    hipError_t e;
    switch (w->dtype) {
    case FNN_DT_I8: e = launch_gemv<FNN_DT_I8>(p, single, rt, s); break;
    case FNN_DT_I4: e = launch_gemv<FNN_DT_I4>(p, single, rt, s); break;
    case FNN_DT_U8: e = launch_gemv<FNN_DT_U8>(p, single, rt, s); break;
    case FNN_DT_U4: e = launch_gemv<FNN_DT_U4>(p, single, rt, s); break;
    case FNN_DT_F8: e = launch_gemv<FNN_DT_F8>(p, single, rt, s); break;
    case FNN_DT_F8R: e = launch_gemv<FNN_DT_F8R>(p, single, rt, s); break;
    case FNN_DT_F4: e = launch_gemv<FNN_DT_F4>(p, single, rt, s); break;
    default: return FNN_OK;
    }
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    *handled = true;
    return FNN_OK;
}
