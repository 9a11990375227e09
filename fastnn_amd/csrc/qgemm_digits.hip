// Quantised MatMul with f32 activations on the int8 matrix cores, M >= 17, I8 / I4 / U4 weights.
//
//   out[m,n] = act((sum_k A[m,k]*u(W[n,k]))*scale[n] + zero[n]*sum_k A[m,k] + bias[n])
//   (gemm_batch_packed_simd + apply_affine_dot, src/backend/cpu/microkernels/gemm.rs:1982-2088,
//    src/backend/cpu/microkernels/mod.rs:283-295)
//
// The integer lanes of these weight types are int8 operands as they are (I8) or after one mask per word
// (4-bit lanes), so the weight side needs no decode to f16.  The activations become exact integers first:
// row m is scaled by a power of two, v = rint(x * 2^e) with |v| < 2^30 (four planes) or 2^22 (three planes, the
// default wherever they measured faster: see fnn_digits_qmatmul), and written as balanced base-256
// digits, v = sum_j 256^j d_j with -128 <= d_j <= 127, one int8 plane per digit.
// v_mfma_i32_32x32x32_i8 multiplies every plane with the weight lanes exactly; the planes of an output meet in
// one lane (tile_kernel.h) and are recombined in f32 before the reference's affine epilogue.  Against the f16
// form (hi + lo f16 rows, weights decoded to f16 per MFMA step) this is the same matrix-core time (four planes at
// twice the f16 rate), a fraction of the vector instructions per stage, and a tighter result: the only rounding
// before the epilogue is rint() at 2^-30 (2^-22 with three planes) of the row's largest magnitude.
//
// Launches: digit_prep_kernel (once per call), qgemm_tile_kernel<int8, DIG>, and with K split over workgroups
// splitk_epilogue_kernel (partials added in split order: results do not depend on scheduling).
// A row holding a non-finite activation comes out as NaN in every column (the reference yields inf or NaN there
// depending on the weights' signs and zeros).
#include "mfma.h"
#include "dech.h"
#include "range_io.h"

#include <type_traits>

namespace {

using namespace dech;

constexpr float LO_UP = 2048.0f, LO_DOWN = 1.0f / 2048.0f;   // f16 mode of the shared kernel (unused here)
#include "tile_kernel.h"

constexpr int KB = 128;   // k-values (= bytes of one plane) per stage and operand row

struct DigitArgs {
    const float *a;
    int8_t *planes;    // [kpad/128][rows_pad][128]
    int *rexp;         // [m_pad] exponent applied to the row, INT_MIN for a row with a non-finite value
    float *xsum;       // [m_pad] sum_k A[m,k]
    int64_t m, k, kpad, rows_pad;
};

// 4x4 byte transpose: o[j] = byte j of a, b, c, d (selector bytes 0-3 pick from the second operand of v_perm_b32)
__device__ __forceinline__ void transpose4(uint32_t a, uint32_t b, uint32_t c, uint32_t d, uint32_t (&o)[4])
{
    const uint32_t ab_lo = __builtin_amdgcn_perm(b, a, 0x05010400u);   // a0 b0 a1 b1
    const uint32_t ab_hi = __builtin_amdgcn_perm(b, a, 0x07030602u);   // a2 b2 a3 b3
    const uint32_t cd_lo = __builtin_amdgcn_perm(d, c, 0x05010400u);
    const uint32_t cd_hi = __builtin_amdgcn_perm(d, c, 0x07030602u);
    o[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);
    o[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
    o[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
    o[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
}

// One workgroup per activation row slot: row statistics, then the DIG digit planes of the row in the tile-major
// operand layout.  Operand row of (activation row m, plane j): (m / RPB) * 32 + j * RPB + m % RPB, RPB = 32 / DIG, for
// two and four planes; with three planes ((m / 8) * 3 + j) * 8 + m % 8 (groups of 24 rows: 8 activation rows x 3 planes).
// IL: the nibble decoders deliver k = 0,2,4,6,1,3,5,7 of each 8, and the activations are stored in that order.
template <int DIG, bool IL>
__global__ void __launch_bounds__(256) digit_prep_kernel(DigitArgs p)
{
    constexpr int RPB = DIG == 3 ? 8 : 32 / DIG;
    constexpr uint32_t BIAS = DIG == 4 ? 0x80808080u : (DIG == 3 ? 0x00808080u : 0x00008080u);
    __shared__ float red[2][4];
    const int64_t m = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int64_t nchunks = p.kpad / 16;
    const int64_t row0 = DIG == 3 ? (m / 8) * 24 + m % 8 : (m / RPB) * 32 + m % RPB;
    auto chunk_at = [&](int j, int64_t c) { return p.planes + (((c >> 3) * p.rows_pad + row0 + j * RPB) * KB + (c & 7) * 16); };
    if (m >= p.m) {   // padding rows of the last tile
        const uint4 z = make_uint4(0, 0, 0, 0);
        for (int64_t c = tid; c < nchunks; c += 256)
#pragma unroll
            for (int j = 0; j < DIG; j++) *reinterpret_cast<uint4 *>(chunk_at(j, c)) = z;
        if (tid == 0) { p.rexp[m] = 0; p.xsum[m] = 0.0f; }
        return;
    }
    const float *x = p.a + m * p.k;
    const bool vec = (p.k % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    auto load16 = [&](int64_t c, float (&v)[16]) {
        const int64_t k0 = c * 16;
        if (vec && k0 + 16 <= p.k) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 t = *reinterpret_cast<const float4 *>(x + k0 + 4 * q);
                v[4 * q] = t.x; v[4 * q + 1] = t.y; v[4 * q + 2] = t.z; v[4 * q + 3] = t.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; i++) v[i] = (k0 + i < p.k) ? x[k0 + i] : 0.0f;
        }
    };
    const bool in_regs = nchunks <= 256;   // K <= 4096: the row stays in registers between the two passes
    float keep[16];
    float mx = 0.0f, sum = 0.0f;
    bool finite = true;
    auto stats = [&](const float (&v)[16]) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            mx = fmaxf(mx, fmaxf(fmaxf(fabsf(v[4 * q]), fabsf(v[4 * q + 1])), fmaxf(fabsf(v[4 * q + 2]), fabsf(v[4 * q + 3]))));
            sum += (v[4 * q] + v[4 * q + 1]) + (v[4 * q + 2] + v[4 * q + 3]);
        }
    };
    if (in_regs) {
#pragma unroll
        for (int i = 0; i < 16; i++) keep[i] = 0.0f;
        if (tid < nchunks) load16(tid, keep);
        stats(keep);
    } else {
        for (int64_t c = tid; c < nchunks; c += 256) {
            float v[16];
            load16(c, v);
            stats(v);
        }
    }
    // fmaxf drops NaN operands: the sum carries them (and +-inf), so test both
    finite = (mx < __builtin_huge_valf()) && (sum == sum) && (fabsf(sum) < __builtin_huge_valf());
    mx = wave_max(mx);
    sum = wave_sum(sum);
    if (lane == 0) { red[0][wv] = mx; red[1][wv] = sum; }
    const int all_finite = __syncthreads_and(finite ? 1 : 0);
    mx = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
    sum = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
    int e = 0;
    if (mx > 0.0f) {
        int ex;
        (void)frexpf(mx, &ex);            // mx = f * 2^ex, f in [0.5, 1)
        e = (DIG == 4 ? 30 : (DIG == 3 ? 22 : 14)) - ex;    // |x * 2^e| < 2^30 (2^22 with three planes, 2^14 with two)
    }
    auto convert = [&](int64_t c, const float (&v)[16]) {
        uint32_t t[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int vi = all_finite ? (int)rintf(ldexpf(v[i], e)) : 0;
            t[i] = ((uint32_t)vi + BIAS) ^ BIAS;    // byte j = digit j as a signed byte
        }
        uint32_t w[4][4];   // w[word of the chunk][plane]
        if (IL) {
            transpose4(t[0], t[2], t[4], t[6], w[0]);
            transpose4(t[1], t[3], t[5], t[7], w[1]);
            transpose4(t[8], t[10], t[12], t[14], w[2]);
            transpose4(t[9], t[11], t[13], t[15], w[3]);
        } else {
            transpose4(t[0], t[1], t[2], t[3], w[0]);
            transpose4(t[4], t[5], t[6], t[7], w[1]);
            transpose4(t[8], t[9], t[10], t[11], w[2]);
            transpose4(t[12], t[13], t[14], t[15], w[3]);
        }
#pragma unroll
        for (int j = 0; j < DIG; j++)
            *reinterpret_cast<uint4 *>(chunk_at(j, c)) = make_uint4(w[0][j], w[1][j], w[2][j], w[3][j]);
    };
    if (in_regs) {
        if (tid < nchunks) convert(tid, keep);
    } else {
        for (int64_t c = tid; c < nchunks; c += 256) {
            float v[16];
            load16(c, v);
            convert(c, v);
        }
    }
    if (tid == 0) {
        p.rexp[m] = all_finite ? e : INT_MIN;
        p.xsum[m] = sum;
    }
}

template <int DT, int WGM, int WGN, int TM, int TN, int NS, int DIG>
hipError_t launch_digit_tile(const TileArgs &p, hipStream_t s)
{
    constexpr int WC = 2 * DecI<DT>::WPS;
    constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
    constexpr size_t lds = (size_t)NS * (BM * 128 + BN * WC * 16);
    if constexpr (lds > 160 * 1024) {
        return hipErrorInvalidValue;   // (not reachable: the caller picks ring depths that fit)
    } else {
    auto kern = qgemm_tile_kernel<DT, WGM, WGN, TM, TN, false, NS, true, DIG>;
    static std::atomic<uint64_t> lds_raised{0};
    hipError_t e = fnn_raise_lds_limit(lds_raised, reinterpret_cast<const void *>(kern), (int)lds);
    if (e != hipSuccess) return e;
    const unsigned total = (unsigned)p.mtiles * p.ntiles * p.splits;
    hipLaunchKernelGGL(kern, dim3(total), dim3(WGM * WGN * 64), lds, s, p);
    return hipGetLastError();
    }
}

template <int DT, int DIG>
int run_digits(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q)
{
    constexpr int RPB = 32 / DIG;
    constexpr bool IL = DecI<DT>::INTERLEAVED;
    const int64_t M = q.m, N = q.n, K = q.k;
    const int64_t kpad = (K + KB - 1) / KB * KB;
    const int64_t meff = (M + RPB - 1) / RPB * 32;
    // tile shapes (operand rows x weight rows):
    //   0 = 128 x 128, 4 waves of 64 x 64 (4-bit weights: two workgroups per CU)   1 = 256 x 128, 4 waves of 128 x 64
    //   2 = 256 x 128, 8 waves of 64 x 64 (two waves per SIMD)                      3 = 256 x 256, 8 waves of 128 x 64 (4-bit weights)
    //   4 = 256 x 192, 8 waves of 64 x 96 (4-bit weights): for N where 256-wide tiles leave CUs idle
    // Shape and K split minimise a small cost model in microseconds: rounds of workgroups over the CU slots x
    // (stages per workgroup x time per stage + a fixed cost per workgroup; resident workgroups share the CU), plus
    // the write and read of the partial tiles and the extra launch.  The stage times are measured on 4096 x 11008
    // (4-bit) and 4096 x 4096 (8-bit) at M = 64 ... 1024; shape 1 never won there and is only reachable by option.
    constexpr bool W4 = DecI<DT>::WPS == 2;
    const int iters = (int)(kpad / KB);
    const double part_us = (double)M * (double)N * 8.0 / 3.0e6;
    struct Plan { int cfg, splits, mtiles, ntiles, bm; double cost; };
    auto plan_for = [&](int cfg) {
        Plan pl;
        pl.cfg = cfg;
        pl.bm = cfg == 0 ? 128 : 256;
        const int bn = cfg == 3 ? 256 : (cfg == 4 ? 192 : 128);
        const int per_cu = (cfg == 0 && W4) ? 2 : 1;    // resident workgroups per CU (LDS)
        const double t_stage = cfg == 4 ? 1.5 : (cfg == 3 ? 1.9 : (cfg == 2 ? 1.35 : (cfg == 1 ? 1.2 : (W4 ? 0.55 : 0.8))));
        pl.mtiles = (int)((meff + pl.bm - 1) / pl.bm);
        pl.ntiles = (int)((N + bn - 1) / bn);
        const int base = pl.mtiles * pl.ntiles;
        pl.splits = 1;
        pl.cost = 1e30;
        for (int sp = 1; sp <= 32 && sp <= (iters / 2 > 0 ? iters / 2 : 1); sp++) {
            const int per = (iters + sp - 1) / sp;
            const double rounds = (double)(int64_t)(((double)base * sp + 256.0 * per_cu - 1) / (256.0 * per_cu));
            const double cost = rounds * per_cu * (per * t_stage + 1.0) + (sp > 1 ? sp * part_us + 3.0 : 0.0);
            if (cost < pl.cost * 0.995) { pl.cost = cost; pl.splits = sp; }
        }
        return pl;
    };
    Plan pl = plan_for(0);
    {
        const Plan big = plan_for(W4 ? 3 : 2);
        if (big.cost < pl.cost) pl = big;
        if (W4) {
            const Plan mid = plan_for(4);
            if (mid.cost < pl.cost) pl = mid;
        }
    }
    const int64_t opt_cfg = fnn_ctx_option(ctx, FNN_OPT_TILE_SHAPE);
    if (opt_cfg >= 0 && opt_cfg <= 4) pl = plan_for((opt_cfg >= 3 && !W4) ? 2 : (int)opt_cfg);   // (wider stages of 8-bit weights do not fit the LDS)
    const int cfg = pl.cfg, mtiles = pl.mtiles, ntiles = pl.ntiles;
    int splits = pl.splits;
    const int64_t rows_pad = (int64_t)mtiles * pl.bm;
    const int64_t m_pad = rows_pad / 32 * RPB;
    const int opt_split = (int)fnn_ctx_option(ctx, FNN_OPT_TILE_SPLIT);
    if (opt_split > 0) splits = opt_split;
    if (splits > iters) splits = iters;
    const int ips = (iters + splits - 1) / splits;
    splits = (iters + ips - 1) / ips;   // no empty split

    const size_t a_bytes = (size_t)rows_pad * kpad;
    const size_t meta_off = (a_bytes + 255) / 256 * 256;
    void *ws0 = nullptr, *ws1 = nullptr;
    int rc;
    if ((rc = fnn_ctx_ensure_tmp(ctx, 0, meta_off + (size_t)m_pad * 8 + 256, &ws0))) return rc;
    if (splits > 1 && (rc = fnn_ctx_ensure_tmp(ctx, 1, (size_t)splits * M * N * 4, &ws1))) return rc;

    DigitArgs d;
    d.a = q.a;
    d.planes = (int8_t *)ws0;
    d.rexp = (int *)((char *)ws0 + meta_off);
    d.xsum = (float *)(d.rexp + m_pad);
    d.m = M; d.k = K; d.kpad = kpad; d.rows_pad = rows_pad;
    hipLaunchKernelGGL((digit_prep_kernel<DIG, IL>), dim3((unsigned)m_pad), dim3(256), 0, s, d);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));

    TileArgs t = {};
    t.words = q.words;
    if constexpr (DecI<DT>::WPS == 2) {   // 4-bit weights: 64 bytes per row and stage, one block of the tile-major copy
        if (int rc = fnn_tile_major_words(ctx, s, w, q, &t.words_tm, &t.kb64)) return rc;
    }
    t.zero_chunk = q.words + w->rows * q.kp;    // the zeroed margin behind the last row
    t.scales = q.scales; t.zeros = q.zeros; t.bias = q.bias;
    t.ap = reinterpret_cast<const _Float16 *>(d.planes);
    t.rexp = d.rexp; t.xsum = d.xsum;
    t.out = q.out; t.part = (float *)ws1;
    if (FnnResidualIo *res = fnn_ctx_residual_io(ctx); splits > 1 && res->residual && res->of_out == q.out && res->elems == (uint64_t)(M * N)) {
        t.residual = res->residual; t.sum_out = res->sum_out;
        res->used = 1;
    }
    t.m = M; t.n = N; t.kp = q.kp; t.kpad = kpad; t.rows_pad = rows_pad;
    t.act = q.act; t.splits = splits; t.iters = iters; t.ips = ips; t.mtiles = mtiles; t.ntiles = ntiles;
    // ring depth: a stage is requested NS - 2 stages before it is consumed, and what is in flight has to cover the
    // memory latency at the rate the matrix cores consume stages; 160 KB of LDS bound it
    constexpr int WC = 2 * DecI<DT>::WPS;
    constexpr int NS0 = (160 * 1024) / (128 * 128 + 128 * WC * 16) >= 6 ? 6 : 5;   // 128 x 128 tiles: 6 (4-bit), 5 (8-bit)
    constexpr int NS1 = (160 * 1024) / (256 * 128 + 128 * WC * 16) >= 4 ? 4 : 3;   // 256 x 128 tiles: 4 (4-bit), 3 (8-bit)
    const int opt_ns = (int)fnn_ctx_option(ctx, FNN_OPT_TILE_STAGES);
    if (cfg == 4) {
        if constexpr (W4) e = launch_digit_tile<DT, 4, 2, 2, 3, 3, DIG>(t, s);
        else e = hipErrorInvalidValue;
    } else if (cfg == 3) {
        if constexpr (W4) e = launch_digit_tile<DT, 2, 4, 4, 2, 3, DIG>(t, s);
        else e = hipErrorInvalidValue;
    } else if (cfg == 2) e = launch_digit_tile<DT, 4, 2, 2, 2, 3, DIG>(t, s);
    else if (cfg == 1) e = opt_ns == 3 ? launch_digit_tile<DT, 2, 2, 4, 2, 3, DIG>(t, s) : launch_digit_tile<DT, 2, 2, 4, 2, NS1, DIG>(t, s);
    else if (opt_ns == 3 || (opt_ns == 0 && W4)) e = launch_digit_tile<DT, 2, 2, 2, 2, 3, DIG>(t, s);
    else if (opt_ns == 4 || opt_ns == 0) e = launch_digit_tile<DT, 2, 2, 2, 2, 4, DIG>(t, s);
    else e = launch_digit_tile<DT, 2, 2, 2, 2, NS0, DIG>(t, s);
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    if (splits > 1) {
        const int64_t colb = (N + 255) / 256;
        int64_t rowb = (2048 + colb - 1) / colb;   // about 2048 workgroups
        if (rowb > M) rowb = M;
        if (rowb > 65535) rowb = 65535;
        hipLaunchKernelGGL(splitk_epilogue_kernel, dim3((unsigned)colb, (unsigned)rowb), dim3(256), 0, s, t, 0);
        e = hipGetLastError();
        if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    }
    return FNN_OK;
}


// Three digit planes: rint(x * 2^e) with |v| < 2^22 per row.  A quarter less matrix-core work and activation operand
// traffic than four planes for 2e-5 of max|ref| stated (about 3e-6 measured on rows with 200x outliers; the four-plane
// form holds 4e-6).  Operand rows come in groups of 24, so a wave owns three MFMA blocks: tiles of 192 operand rows
// (64 activation rows) x 128 weight rows on four waves, x 256 on eight for 4-bit weights with many column tiles.
template <int DT>
int run_digits3(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q)
{
    constexpr bool IL = DecI<DT>::INTERLEAVED;
    constexpr bool W4 = DecI<DT>::WPS == 2;
    const int64_t M = q.m, N = q.n, K = q.k;
    const int64_t kpad = (K + KB - 1) / KB * KB;
    const int iters = (int)(kpad / KB);
    const int bm = 192, act_rows = 64;
    // tile forms: 0 = 192 x 128 on four waves, 1 = 192 x 256 on eight (4-bit weights), 2 = 192 x 128 on eight (twice the
    // waves requesting the operands).  By shape: 4-bit weights take the wide tiles while those still cover the chip.
    // ... or where they save a round of workgroups (a wide tile takes about 1.4 times as long as a narrow one:
    // 4096 x 4096 at M = 513, 144 wide tiles against 288 narrow ones; 4096 x 11008 at M = 129 ... 192, 129 against 258)
    int form = 2;
    if (W4) {
        const int64_t mt = (M + 63) / 64, wide_tiles = (N + 255) / 256 * mt, narrow_tiles = (N + 127) / 128 * mt;
        if (wide_tiles >= 160 || 1.4 * (double)((wide_tiles + 255) / 256) < (double)((narrow_tiles + 255) / 256)) form = 1;
    }
    const int64_t opt_cfg = fnn_ctx_option(ctx, FNN_OPT_TILE_SHAPE);
    if (opt_cfg >= 0 && opt_cfg <= 2 && (opt_cfg != 1 || W4)) form = (int)opt_cfg;
    const int wide = form == 1;
    const int bn = wide ? 256 : 128;
    const int mtiles = (int)((M + act_rows - 1) / act_rows), ntiles = (int)((N + bn - 1) / bn);
    const int64_t tiles = (int64_t)mtiles * ntiles;
    // K split: as many workgroups as fit one round over the 256 CUs, never more (4096 x 11008 at M = 256, 172 tiles:
    // 47 us unsplit, 66 us in two splits; 4096 x 4096 at M = 128, 64 tiles: 23 us in four splits, 31 us unsplit)
    int splits = (int)(256 / tiles);
    if (splits > iters / 4) splits = iters / 4;   // four stages or more per workgroup
    if (splits < 1) splits = 1;
    const int opt_split = (int)fnn_ctx_option(ctx, FNN_OPT_TILE_SPLIT);
    if (opt_split > 0) splits = opt_split;
    if (splits > iters) splits = iters;
    const int ips = (iters + splits - 1) / splits;
    splits = (iters + ips - 1) / ips;   // no empty split
    const int64_t rows_pad = (int64_t)mtiles * bm, m_pad = (int64_t)mtiles * act_rows;

    const size_t a_bytes = (size_t)rows_pad * kpad;
    const size_t meta_off = (a_bytes + 255) / 256 * 256;
    void *ws0 = nullptr, *ws1 = nullptr;
    int rc;
    if ((rc = fnn_ctx_ensure_tmp(ctx, 0, meta_off + (size_t)m_pad * 8 + 256, &ws0))) return rc;
    if (splits > 1 && (rc = fnn_ctx_ensure_tmp(ctx, 1, (size_t)splits * M * N * 4, &ws1))) return rc;

    DigitArgs d;
    d.a = q.a;
    d.planes = (int8_t *)ws0;
    d.rexp = (int *)((char *)ws0 + meta_off);
    d.xsum = (float *)(d.rexp + m_pad);
    d.m = M; d.k = K; d.kpad = kpad; d.rows_pad = rows_pad;
    hipLaunchKernelGGL((digit_prep_kernel<3, IL>), dim3((unsigned)m_pad), dim3(256), 0, s, d);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));

    TileArgs t = {};
    t.words = q.words;
    if constexpr (DecI<DT>::WPS == 2) {   // 4-bit weights: 64 bytes per row and stage, one block of the tile-major copy
        if (int rc = fnn_tile_major_words(ctx, s, w, q, &t.words_tm, &t.kb64)) return rc;
    }
    t.zero_chunk = q.words + w->rows * q.kp;    // the zeroed margin behind the last row
    t.scales = q.scales; t.zeros = q.zeros; t.bias = q.bias;
    t.ap = reinterpret_cast<const _Float16 *>(d.planes);
    t.rexp = d.rexp; t.xsum = d.xsum;
    t.out = q.out; t.part = (float *)ws1;
    if (FnnResidualIo *res = fnn_ctx_residual_io(ctx); splits > 1 && res->residual && res->of_out == q.out && res->elems == (uint64_t)(M * N)) {
        t.residual = res->residual; t.sum_out = res->sum_out;
        res->used = 1;
    }
    t.m = M; t.n = N; t.kp = q.kp; t.kpad = kpad; t.rows_pad = rows_pad;
    t.act = q.act; t.splits = splits; t.iters = iters; t.ips = ips; t.mtiles = mtiles; t.ntiles = ntiles;
    // ring depth: four stages (24 KB of planes + 8 or 16 KB of weights each; the 8-bit and the wide forms fill the LDS)
    if (form == 1) {
        if constexpr (W4) e = launch_digit_tile<DT, 2, 4, 3, 2, 4, 3>(t, s);
        else e = hipErrorInvalidValue;
    } else if (form == 2) e = launch_digit_tile<DT, 2, 4, 3, 1, 4, 3>(t, s);
    else e = launch_digit_tile<DT, 2, 2, 3, 2, 4, 3>(t, s);
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    if (splits > 1) {
        const int64_t colb = (N + 255) / 256;
        int64_t rowb = (2048 + colb - 1) / colb;   // about 2048 workgroups
        if (rowb > M) rowb = M;
        if (rowb > 65535) rowb = 65535;
        hipLaunchKernelGGL(splitk_epilogue_kernel, dim3((unsigned)colb, (unsigned)rowb), dim3(256), 0, s, t, 0);
        e = hipGetLastError();
        if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    }
    return FNN_OK;
}

}  // namespace

int fnn_digits_qmatmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q, int flags, bool *handled)
{
    *handled = false;
    if (fnn_ctx_option(ctx, FNN_OPT_GEMM_INT8) == 0) return FNN_OK;
    if (q.m < fnn_ctx_option(ctx, FNN_OPT_GEMM_INT8_MIN_M)) return FNN_OK;
    const int dt = w->dtype;
    if (dt != FNN_DT_I8 && dt != FNN_DT_I4 && dt != FNN_DT_U4) return FNN_OK;
    // exact i32 sums: |digit| <= 128, |lane| <= 128 (16*q for 4-bit signed lanes) -> K * 2^14 < 2^31
    if (q.m > (1 << 22) || q.n > (1 << 24) || q.k > (1 << 16)) return FNN_OK;
    if (q.words != w->words) return FNN_OK;   // (a row slice of a weight: the zero margin behind the last row is not behind the slice)
    QMatmulArgs qa = q;
    int rc;
    if ((rc = fnn_aligned_rows(ctx, s, w, &qa.words, &qa.kp))) return rc;
    if (qa.kp % 4 != 0 || (reinterpret_cast<uintptr_t>(qa.words) & 15)) return FNN_OK;
    // The single-rounding mode stays with the f16 tiles: two digit planes (15 bits below the row maximum) were 15 %
    // faster than one f16 row but measured 1.9e-3 on rows with a few 200x outliers, where a float rounding per
    // element keeps 2.4e-4; three planes cost what the f16 row costs.
    if (flags & FNN_FLAG_ACT_F16_SINGLE) return FNN_OK;
    // Small weights stay with the f16 tiles as well (by rule; FNN_OPT_DIGIT_PLANES = 3 or 4 or FNN_OPT_GEMM_INT8_MIN_M
    // below its default still bring them here): 1024 x 1024 I4 at M = 48 / 256 / 1024 14.6 / 16.2 / 22.3 us here against 12.9 / 13.6 / 15.9 there, 2048 x 2048 I8
    // at M = 64 / 512 16.4 / 26.6 against 15.1 / 22.0; from 3072 x 3072 and 8192 x 1024 on this path is ahead
    int64_t planes = fnn_ctx_option(ctx, FNN_OPT_DIGIT_PLANES);
    if (planes != 3 && planes != 4 && q.n * q.k <= (int64_t)2048 * 2048 && fnn_ctx_option(ctx, FNN_OPT_GEMM_INT8_MIN_M) >= 17) return FNN_OK;
    // Planes by shape: three wherever they measured faster than four, i.e. 4-bit weights at every M (4096 x 11008: M = 64
    // 26.3 against 29.3 us, M = 128 30.9 against 40.2, M = 256 47.2 against 54.9, M = 1024 139 against 168) and 8-bit
    // weights from M = 96 (4096 x 4096: M = 64 21.6 against 19.1, M = 128 23.1 against 24.2, M = 512 40.7 against 49.7).
    if (planes != 3 && planes != 4) planes = (dt == FNN_DT_I8 && q.m < 96) ? 4 : 3;
    // 8-bit weights decode to f16 with one permute per pair, so at four planes the int8 form only ties the f16 tiles
    // (hi + lo rows) and falls 4-5 % behind them from M = 1024 on (4096 x 4096: 93 vs 89 us, M = 2048: 172 vs 164); at
    // three planes it stays ahead (M = 1024: 70 against 86 us, M = 2048: 128 against 160)
    if (planes == 4 && dt == FNN_DT_I8 && q.m >= 768 && fnn_ctx_option(ctx, FNN_OPT_GEMM_INT8_MIN_M) <= 17) return FNN_OK;
    if (planes == 3) {
        switch (dt) {
        case FNN_DT_I8: rc = run_digits3<FNN_DT_I8>(ctx, s, w, qa); break;
        case FNN_DT_I4: rc = run_digits3<FNN_DT_I4>(ctx, s, w, qa); break;
        default: rc = run_digits3<FNN_DT_U4>(ctx, s, w, qa); break;
        }
        if (rc) return rc;
        *handled = true;
        return FNN_OK;
    }
    switch (dt) {
    case FNN_DT_I8: rc = run_digits<FNN_DT_I8, 4>(ctx, s, w, qa); break;
    case FNN_DT_I4: rc = run_digits<FNN_DT_I4, 4>(ctx, s, w, qa); break;
    default: rc = run_digits<FNN_DT_U4, 4>(ctx, s, w, qa); break;
    }
    if (rc) return rc;
    *handled = true;
    return FNN_OK;
}
