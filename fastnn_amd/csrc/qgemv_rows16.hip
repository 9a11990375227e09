// Quantised MatMul for 9..16 activation rows on the matrix cores, organised like the GEMV
// (qgemv_mfma.hip): the packed weights are streamed once, every workgroup converts the whole
// activation block itself, no separate preparation or reduction launch.
//
//   out[m,n] = act((sum_k A[m,k]*u(W[n,k]))*scale[n] + zero[n]*sum_k A[m,k] + bias[n])
//   (gemm_batch_packed_simd + apply_affine_dot, src/backend/cpu/microkernels/gemm.rs:1982-2088,
//    src/backend/cpu/microkernels/mod.rs:283-295)
//
// The 16 rows of the v_mfma_f32_16x16x32_f16 activation operand are the 16 activation rows.
// Wave w owns the K slice [w*512, (w+1)*512) of every round:
//   0. it requests its activations: per weight tile (128 or 64 k-values) a pair of 16-byte loads per
//      lane covers 2 KB of contiguous row segments (4 or 8 rows), so every cache line is consumed by
//      neighbouring lanes of two adjacent instructions;
//   1. it requests all of its packed bytes; scheduling barriers pin "all requests first";
//   2. row maxima and sums of the slice by DPP over the 16 (or 8) lanes that share a row; each row is
//      scaled by a power of two (slice maximum into [2^14, 2^15));
//   3. tile by tile: the lane's groups of 8 values become hi + lo f16 operand fragments in a small LDS
//      buffer of the wave (reused for every tile, swizzled so that writes and reads are conflict-free),
//      then two MFMAs per step and row tile (hi and lo against the same decoded weights);
//   4. the slice partial is scaled back in f32; the partial tiles of the waves are added in a fixed
//      order through LDS and the affine / bias / activation epilogue is applied.
// Algorithmic bytes per launch: N*K*bits/8 + side tables + 4*M*(K+N).
#include "dech.h"
#include "mfma.h"

#include <cstdlib>

namespace {

using namespace dech;

struct Rows16Args {
    const uint32_t *words;
    const float *scales, *zeros, *a, *bias;
    const float *umean;   // single-f16 mode: mean lane value per weight row, or null
    float *out;
    int64_t m, n, k, kp;
    int act;
    const uint32_t *words_tm;   // non-null: the words in blocks of 16 rows x 64 bytes ([row block][k block][row][64 bytes]),
    int64_t kb64;               // kb64 k blocks per row: a wave load of packed bytes is then one contiguous KB
};

constexpr int R16_SLICE = 512;   // k-values per wave and round

// TMAJ: the packed words come from the tile-major copy (p.words_tm)
template <int DT, int RT, bool SINGLE, int NW, bool TMAJ = false>
__global__ void __launch_bounds__(NW * 64) qgemv_rows16_kernel(Rows16Args p)
{
    using D = DecH<DT>;
    constexpr int WPS = D::WPS;
    constexpr int SPT = 4 / WPS;            // MFMA steps per 16-byte lane load of weights (4 / 2)
    constexpr int KT = 4 * SPT * 8;         // k-values per weight tile (128 / 64)
    constexpr int TPW = R16_SLICE / KT;     // weight tiles per wave and round (4 / 8)
    constexpr int LPR = KT / 8;             // lanes that share an activation row in a load pair (16 / 8)
    constexpr int RPP = 64 / LPR;           // rows per load pair (4 / 8)
    constexpr int PPT = 16 / RPP;           // load pairs per tile (4 / 2)
    constexpr int ST_STRIDE = 32 * 64 + (SPT == 4 ? 64 : 128);   // bytes between the steps of the fragment buffer
    constexpr int FRAG_BYTES = SPT * ST_STRIDE;

    __shared__ __attribute__((aligned(16))) unsigned char frag[NW][FRAG_BYTES];
    __shared__ float red[NW][RT][16][16];
    __shared__ float xred[NW][16];
    __shared__ float cscs[NW][16];
    __shared__ float ered[NW][16];   // single-f16 mode: sum_k (hi - x) per activation row

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = tid >> 6;
    const int ln = lane & 15;               // MFMA: activation row (operand A) / weight row of the tile (operand B)
    const int g = lane >> 4;
    const int64_t K = p.k, N = p.n, kp = p.kp;
    const int mreal = (int)p.m;             // <= 16
    const int64_t n0 = (int64_t)blockIdx.x * (RT * 16);
    // loads: this lane's group of 8 k-values inside a tile, and its row inside a load pair
    const int grp = lane % LPR, lrow = lane / LPR;
    const int l_g = grp / SPT, l_st = grp % SPT;   // k inside the tile = l_g*SPT*8 + l_st*8 = grp*8

    const uint32_t *wrow[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) {
        int64_t row = n0 + r * 16 + ln;
        if (row > N - 1) row = N - 1;
        wrow[r] = TMAJ ? p.words_tm + ((row >> 4) * p.kb64) * 256 + (row & 15) * 16 : p.words + row * kp;
    }
    const float *arow[PPT];
    bool row_live[PPT];
    unsigned wr_off[PPT];                   // where this lane's fragments of pair j go (hi; lo is 16 rows further)
#pragma unroll
    for (int j = 0; j < PPT; j++) {
        const int row = j * RPP + lrow;
        row_live[j] = row < mreal;
        arow[j] = p.a + (int64_t)(row_live[j] ? row : mreal - 1) * K;
        wr_off[j] = l_st * ST_STRIDE + row * 64 + ((l_g ^ ((row >> 2) & 3)) * 16);
    }
    const unsigned char *fr = frag[wv];
    unsigned char *fwr = frag[wv];
    const unsigned rd_off = ln * 64 + ((g ^ ((ln >> 2) & 3)) * 16);   // operand fragment (row ln, group g) of a step

    f32x4 tot[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) tot[r] = f32x4{0.f, 0.f, 0.f, 0.f};
    float xsum[PPT], xerr[PPT];
#pragma unroll
    for (int j = 0; j < PPT; j++) xsum[j] = xerr[j] = 0.0f;

    const int64_t round_k = (int64_t)NW * R16_SLICE;
    for (int64_t k0 = 0; k0 < K; k0 += round_k) {
        const int64_t ks = k0 + (int64_t)wv * R16_SLICE;
        // ---- 0. activations (clamped, always valid addresses; masked afterwards)
        uint4 xa[TPW][PPT], xb[TPW][PPT];
        bool kok[TPW];
#pragma unroll
        for (int t = 0; t < TPW; t++) {
            const int64_t kk = ks + t * KT + grp * 8;
            kok[t] = kk < K;                // K % 8 == 0
            const int64_t kc = kok[t] ? kk : K - 8;
#pragma unroll
            for (int j = 0; j < PPT; j++) {
                xa[t][j] = *reinterpret_cast<const uint4 *>(arow[j] + kc);
                xb[t][j] = *reinterpret_cast<const uint4 *>(arow[j] + kc + 4);
            }
        }
        // ---- 1. the packed bytes: tile t, lane (n,g): words [slice + t*16 + g*4, +4) of row n
        //         (a chunk past the end of the row re-reads the row's last chunk: it only meets masked activations)
        uint32_t wq[RT][TPW * 4];
        const int64_t wbase = ks * 4 / (8 * SPT);
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
                    if (woff + 4 > kp) woff = kp - 4;
                }
                const uint4 v = *reinterpret_cast<const uint4 *>(wrow[r] + woff);
                wq[r][t * 4 + 0] = v.x; wq[r][t * 4 + 1] = v.y; wq[r][t * 4 + 2] = v.z; wq[r][t * 4 + 3] = v.w;
            }
        __builtin_amdgcn_sched_barrier(0);   // every request of the round is out before anything waits

        // ---- 2. row statistics of the slice
        float inv[PPT], csc[PPT];
#pragma unroll
        for (int j = 0; j < PPT; j++) {
            float mx = 0.0f, sum = 0.0f;
#pragma unroll
            for (int t = 0; t < TPW; t++) {
                const uint32_t keep = (kok[t] && row_live[j]) ? 0xffffffffu : 0u;
                xa[t][j].x &= keep; xa[t][j].y &= keep; xa[t][j].z &= keep; xa[t][j].w &= keep;
                xb[t][j].x &= keep; xb[t][j].y &= keep; xb[t][j].z &= keep; xb[t][j].w &= keep;
                const float x0 = __uint_as_float(xa[t][j].x), x1 = __uint_as_float(xa[t][j].y), x2 = __uint_as_float(xa[t][j].z), x3 = __uint_as_float(xa[t][j].w);
                const float x4 = __uint_as_float(xb[t][j].x), x5 = __uint_as_float(xb[t][j].y), x6 = __uint_as_float(xb[t][j].z), x7 = __uint_as_float(xb[t][j].w);
                mx = fmaxf(mx, fmaxf(fmaxf(fmaxf(fabsf(x0), fabsf(x1)), fmaxf(fabsf(x2), fabsf(x3))),
                                     fmaxf(fmaxf(fabsf(x4), fabsf(x5)), fmaxf(fabsf(x6), fabsf(x7)))));
                sum += ((x0 + x1) + (x2 + x3)) + ((x4 + x5) + (x6 + x7));
            }
            // over the LPR neighbouring lanes that hold the same row (every one of them ends with the result)
            mx = fmaxf(mx, dpp_f32<0xB1>(mx));  sum += dpp_f32<0xB1>(sum);    // quad_perm [1,0,3,2]
            mx = fmaxf(mx, dpp_f32<0x4E>(mx));  sum += dpp_f32<0x4E>(sum);    // quad_perm [2,3,0,1]
            mx = fmaxf(mx, dpp_f32<0x141>(mx)); sum += dpp_f32<0x141>(sum);   // row_half_mirror
            if (LPR == 16) { mx = fmaxf(mx, dpp_f32<0x140>(mx)); sum += dpp_f32<0x140>(sum); }   // row_mirror
            xsum[j] += sum;
            // power of two e with max*2^-e in [2^14, 2^15), clamped so that 2^-e is finite
            int ex = (int)((__float_as_uint(mx) >> 23) & 0xff) - 127 - 14;
            if (mx == 0.0f) ex = 0;
            ex = ex < -100 ? -100 : (ex > 120 ? 120 : ex);
            inv[j] = __uint_as_float((uint32_t)(127 - ex) << 23);
            csc[j] = __uint_as_float((uint32_t)(127 + ex) << 23);
            if (grp == 0) cscs[wv][j * RPP + lrow] = csc[j];
        }

        // ---- 3. tile by tile: operand fragments through the wave's LDS buffer, then the MFMA steps
        f32x4 acc[RT];
#pragma unroll
        for (int r = 0; r < RT; r++) acc[r] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < TPW; t++) {
#pragma unroll
            for (int j = 0; j < PPT; j++) {
                const float x[8] = {__uint_as_float(xa[t][j].x), __uint_as_float(xa[t][j].y), __uint_as_float(xa[t][j].z), __uint_as_float(xa[t][j].w),
                                    __uint_as_float(xb[t][j].x), __uint_as_float(xb[t][j].y), __uint_as_float(xb[t][j].z), __uint_as_float(xb[t][j].w)};
                f16x8 hi, lo;
                float rerr = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int src = D::INTERLEAVED ? ((e >> 1) + 4 * (e & 1)) : e;
                    const float v = x[src] * inv[j];
                    const _Float16 h = (_Float16)v;
                    hi[e] = h;
                    lo[e] = (_Float16)(v - (float)h);
                    if (SINGLE) rerr += (float)h - v;
                }
                if (SINGLE) xerr[j] += csc[j] * rerr;   // this lane's share; summed over the row's lanes at the end
                *reinterpret_cast<f16x8 *>(fwr + wr_off[j]) = hi;
                if (!SINGLE) *reinterpret_cast<f16x8 *>(fwr + wr_off[j] + 16 * 64) = lo;
            }
            __builtin_amdgcn_wave_barrier();   // only this wave uses the buffer; the LDS serves a wave in order
            if (t == 0) __builtin_amdgcn_sched_barrier(0);   // the waits for the packed bytes stay behind the statistics
#pragma unroll
            for (int st = 0; st < SPT; st++) {
                const f16x8 ahi = *reinterpret_cast<const f16x8 *>(fr + st * ST_STRIDE + rd_off);
                f16x8 alo;
                if (!SINGLE) alo = *reinterpret_cast<const f16x8 *>(fr + st * ST_STRIDE + rd_off + 16 * 64);
#pragma unroll
                for (int r = 0; r < RT; r++) {
                    const f16x8 b = D::step(&wq[r][(t * SPT + st) * WPS]);
                    acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, b, acc[r], 0, 0, 0);
                    if (!SINGLE) acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, b, acc[r], 0, 0, 0);
                }
            }
            __builtin_amdgcn_wave_barrier();   // the buffer is rewritten by the next tile
        }
        // acc[i] is activation row g*4 + i: scale it back with that row's factor
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float cs = cscs[wv][g * 4 + i];
#pragma unroll
            for (int r = 0; r < RT; r++) tot[r][i] = fmaf(acc[r][i], cs, tot[r][i]);
        }
        __builtin_amdgcn_wave_barrier();       // the wave's own factors are rewritten by its next round
    }

    // ---- 4. fixed-order reduction over the waves, fused epilogue
#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int i = 0; i < 4; i++) red[wv][r][g * 4 + i][ln] = tot[r][i];
    if (SINGLE) {
#pragma unroll
        for (int j = 0; j < PPT; j++) {   // over the LPR neighbouring lanes that hold the same row
            float v = xerr[j];
            v += dpp_f32<0xB1>(v);
            v += dpp_f32<0x4E>(v);
            v += dpp_f32<0x141>(v);
            if (LPR == 16) v += dpp_f32<0x140>(v);
            xerr[j] = v;
        }
    }
    if (grp == 0) {
#pragma unroll
        for (int j = 0; j < PPT; j++) {
            xred[wv][j * RPP + lrow] = xsum[j];
            ered[wv][j * RPP + lrow] = xerr[j];
        }
    }
    __syncthreads();
    for (int o = tid; o < RT * 256; o += NW * 64) {
        const int r = o >> 8, m = (o >> 4) & 15, c = o & 15;
        const int64_t n = n0 + r * 16 + c;
        if (m >= mreal || n >= N) continue;
        float dot = 0.0f, xs = 0.0f, es = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; w++) {
            dot += red[w][r][m][c];
            xs += xred[w][m];
            if (SINGLE) es += ered[w][m];
        }
        // single-f16 mode, first-order correction of the rounding: dot -= mean_k u[n,k] * sum_k (hi - x)
        if (SINGLE && p.umean) dot = dot - p.umean[n] * es;
        p.out[(int64_t)m * N + n] = fnn_epilogue(dot, p.scales[n], p.zeros[n], xs, p.bias, n, p.act);
    }
}

// row tiles per workgroup: the activation block is converted once per workgroup, so as many as the registers
// allow while the workgroups still cover the CUs
template <int DT>
inline int rows16_tiles(int64_t n, int forced)
{
    constexpr int max_rt = DecH<DT>::WPS == 1 ? 3 : 2;   // 8-bit types hold twice the packed words per tile
    if (forced >= 1 && forced <= max_rt) return forced;
    int best = 1;
    double best_cost = 1e30;
    for (int rt = 1; rt <= max_rt; rt++) {
        const int64_t wgs = (n + rt * 16 - 1) / (rt * 16);
        const double cost = (double)((wgs + 255) / 256) * (6.0 + rt);
        if (cost < best_cost - 1e-9) { best_cost = cost; best = rt; }
    }
    return best;
}

template <int DT, int RT, bool SINGLE, int NW, bool TMAJ = false>
void launch_rt(const Rows16Args &p, hipStream_t s)
{
    if constexpr (!TMAJ && !SINGLE) {   // (the tile-major variants exist for the default activation mode)
        if (p.words_tm) return launch_rt<DT, RT, SINGLE, NW, true>(p, s);
    }
    const dim3 grid((unsigned)((p.n + RT * 16 - 1) / (RT * 16))), blk(NW * 64);
    hipLaunchKernelGGL((qgemv_rows16_kernel<DT, RT, SINGLE, NW, TMAJ>), grid, blk, 0, s, p);
}

template <int DT, bool SINGLE, int NW>
void launch_nw(const Rows16Args &p, int forced_rt, hipStream_t s)
{
    const int rt = rows16_tiles<DT>(p.n, forced_rt);
    if constexpr (DecH<DT>::WPS == 1) {
        if (rt == 3) { launch_rt<DT, 3, SINGLE, NW>(p, s); return; }
    }
    if (rt == 2) launch_rt<DT, 2, SINGLE, NW>(p, s);
    else launch_rt<DT, 1, SINGLE, NW>(p, s);
}

template <int DT>
hipError_t launch_rows16(const Rows16Args &p, bool single, int forced_rt, hipStream_t s)
{
    // 8 waves split K in slices of 512; short K (<= 2048) runs 4-wave workgroups so that no wave idles
    if (p.k <= 4 * R16_SLICE) {
        if (single) launch_nw<DT, true, 4>(p, forced_rt, s); else launch_nw<DT, false, 4>(p, forced_rt, s);
    } else {
        if (single) launch_nw<DT, true, 8>(p, forced_rt, s); else launch_nw<DT, false, 8>(p, forced_rt, s);
    }
    return hipGetLastError();
}

}  // namespace

int fnn_mfma_rows16(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q,
                    int flags, bool *handled)
{
    *handled = false;
    const int64_t min_m = fnn_ctx_option(ctx, FNN_OPT_ROWS16_MIN_M);
    if (q.m < min_m || q.m > 16 || w->dtype == FNN_DT_I4CB) return FNN_OK;
    if (q.kp % 4 != 0 || q.k % 8 != 0) return FNN_OK;
    if ((reinterpret_cast<uintptr_t>(q.a) & 15) || (reinterpret_cast<uintptr_t>(q.words) & 15)) return FNN_OK;
    Rows16Args p;
    p.words = q.words; p.scales = q.scales; p.zeros = q.zeros; p.a = q.a; p.bias = q.bias; p.out = q.out;
    p.m = q.m; p.n = q.n; p.k = q.k; p.kp = q.kp; p.act = q.act;
    const bool single = (flags & FNN_FLAG_ACT_F16_SINGLE) != 0;
    p.umean = nullptr;
    p.words_tm = nullptr; p.kb64 = 0;
    if (single) {
        int rc = fnn_row_means(ctx, s, w, &p.umean);
        if (rc) return rc;
    } else if (int rc = fnn_tile_major_words(ctx, s, w, q, &p.words_tm, &p.kb64)) {
        return rc;
    }
    const int rt = (int)fnn_ctx_option(ctx, FNN_OPT_ROWS16_ROW_TILES);   // 0: by the cost model
    hipError_t e;
    switch (w->dtype) {
    case FNN_DT_I8: e = launch_rows16<FNN_DT_I8>(p, single, rt, s); break;
    case FNN_DT_I4: e = launch_rows16<FNN_DT_I4>(p, single, rt, s); break;
    case FNN_DT_U8: e = launch_rows16<FNN_DT_U8>(p, single, rt, s); break;
    case FNN_DT_U4: e = launch_rows16<FNN_DT_U4>(p, single, rt, s); break;
    case FNN_DT_F8: e = launch_rows16<FNN_DT_F8>(p, single, rt, s); break;
    case FNN_DT_F8R: e = launch_rows16<FNN_DT_F8R>(p, single, rt, s); break;
    case FNN_DT_F4: e = launch_rows16<FNN_DT_F4>(p, single, rt, s); break;
    default: return FNN_OK;
    }
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    *handled = true;
    return FNN_OK;
}
