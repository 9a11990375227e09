// The tiled matrix-core GEMM kernel shared by the f16 path (f32 activations x packed weights,
// qgemm_tiled.hip) and the int8 path (I8 activations / quantised conv, qgemm_i8.hip).
// Included inside an anonymous namespace after dech.h and the LO_UP / LO_DOWN constants; see
// qgemm_tiled.hip for the design.
#pragma once
#include <climits>

struct TileArgs {
    const uint32_t *words;
    // non-null (weight types with 64 bytes per row and stage only): the words in blocks of 16 rows x 64 bytes,
    // [row block][k block][row][64 bytes], kb64 k blocks per row: a wave's 64 chunk loads of a stage are one contiguous KB
    const uint32_t *words_tm = nullptr;
    int64_t kb64 = 0;
    const uint32_t *zero_chunk;   // 16 zero bytes: source of weight chunks past the end of a row
    const float *scales, *zeros, *umean, *bias;
    const _Float16 *ap;
    const int *rexp;
    const float *xsum, *esum;
    float *out, *part;
    const float *residual;        // split-K reduction only: non-null = sum_out[m,n] = out[m,n] + residual[m,n] as well
    float *sum_out;
    int32_t *c_i32;               // int8 mode: raw accumulators [m][ldc]
    int64_t ldc;
    int64_t m, n, kp, kpad, rows_pad;
    int act, splits, iters, ips, mtiles, ntiles;
    int a_wrap;   // > 0: the activation operand has a_wrap k blocks and is swept again after them (weights = [hi | lo])
    // codebook weights decoded in the kernel (DT = FNN_DT_I4CB): block scales [n][bpr] (one per 32 k-values), the 16
    // table values, and the power of two the table is scaled by before it is split into f16 hi + lo
    const float *bscales;
    const float *codebook;
    int64_t bpr;
    // quantised Conv2d epilogue inside the int8 kernel (CONV): scales / zeros / bias above are those of the group's
    // channels; y and acc_out start at the group's first channel of image 0
    struct Conv {
        float *y;                  // [B, OC, np]
        int32_t *acc_out;          // same shape, or null
        const float *actq;         // [B*groups][4]: activation scale, zero, 1/scale, unused
        const int32_t *qsum;       // [nq][rows_pad]: partial sums of q_a per im2col row
        const int32_t *row_qsum;   // [channels of the group]: sum of q_w
        int64_t oc;
        uint32_t np;
        int nq, groups, g, kk;
        int vec4;                  // np % 4 == 0 and 16-byte aligned outputs: four pixels per store
        // non-null (only with np >= rows of a tile, so that a tile meets at most two images): partial (min, max)
        // pairs of the values this launch stores, [image][range_stride][2]; the tile (mt, nt) fills pair
        // nt * (np / BM + 2) + (mt - first tile of the image) of every image it meets, (np / BM + 2) * ntiles pairs per image
        float *range_out;
        int range_stride;
        // non-null: sum_out = y + residual as well (same layout as y); range_out then describes the sums
        const float *residual;
        float *sum_out;
    } cv;
};

// HBM -> LDS without passing registers: lane i of the wave stores its 16 bytes at
// LDS address m0 + 16*i.  The compiler does not see these loads: waits are placed by hand.
__device__ __forceinline__ void load_to_lds16(const void *gptr, unsigned lds_wave_base)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_wave_base), "v"(gptr) : "memory");
}
// Up to four such loads behind one M0 write: load i lands at m0 + 1024*i + 16*lane.  The instruction offset moves
// the LDS address and the memory address alike, so the pointers passed in are biased by -1024*i bytes.
template <int N>
__device__ __forceinline__ void load_group_to_lds16(const void *g0, const void *g1, const void *g2, const void *g3, unsigned lds_wave_base)
{
    static_assert(N >= 1 && N <= 4, "1..4 loads per M0 value");
    if constexpr (N == 1)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_wave_base), "v"(g0) : "memory");
    else if constexpr (N == 2)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\tglobal_load_lds_dwordx4 %2, off offset:1024"
                     ::"s"(lds_wave_base), "v"(g0), "v"(g1) : "memory");
    else if constexpr (N == 3)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\tglobal_load_lds_dwordx4 %2, off offset:1024\n\t"
                     "global_load_lds_dwordx4 %3, off offset:2048" ::"s"(lds_wave_base), "v"(g0), "v"(g1), "v"(g2) : "memory");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\tglobal_load_lds_dwordx4 %2, off offset:1024\n\t"
                     "global_load_lds_dwordx4 %3, off offset:2048\n\tglobal_load_lds_dwordx4 %4, off offset:3072"
                     ::"s"(lds_wave_base), "v"(g0), "v"(g1), "v"(g2), "v"(g3) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_loads_but()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// INT8 = false: f16 operands, v_mfma_f32_32x32x16_f16, 64 k-values per stage, float epilogue.
// INT8 = true:  int8 operands, v_mfma_i32_32x32x32_i8, 128 k-values per stage (the same 128 bytes
//               per activation row), accumulators stored as they are (4-bit weights enter as
//               16*q in the high nibble of a byte and the sum is shifted back).
// DIG > 0 (with INT8): the activation operand holds DIG balanced base-256 digit planes of f32 activations
//               scaled per row by 2^rexp: a 32-row MFMA block = 32/DIG activation rows x DIG planes (plane j in
//               block rows [j*32/DIG, (j+1)*32/DIG)), so a lane holds every plane's exact i32 sum of its outputs
//               and recombines them, sum_j 256^j * acc_j, before the float epilogue.  DIG = 3: eight activation
//               rows x 3 planes form a group of 24 operand rows (plane j in rows [8j, 8j + 8) of the group); the
//               8-row slabs of a lane's accumulators then alternate plane by plane, three MFMA blocks per four groups.
// CONV (with INT8, DIG = 0): the rows are im2col rows (image, pixel); the accumulators are turned into the
//               convolution's outputs here (conv_dequant) and stored NCHW, four consecutive pixels of a channel
//               per lane and store where the image size allows.
// FP8 (with INT8, DT = FNN_DT_I8, DIG = 0, no CONV): the bytes of both operands are OCP E4M3 values; the same pipeline
//               with two v_mfma_f32_32x32x16_fp8_fp8 per step (the low and the high 8 bytes of a lane's 16) and f32
//               accumulators, whose bits are stored where the int8 mode stores its integers.
template <int DT, int WGM, int WGN, int TM, int TN, bool PRECISE, int NS, bool INT8 = false, int DIG = 0, bool CONV = false, bool CRNG = false,
          bool FP8 = false>
__global__ void __launch_bounds__(WGM * WGN * 64) qgemm_tile_kernel(TileArgs p)
{
    static_assert(!FP8 || (INT8 && DT == FNN_DT_I8 && DIG == 0 && !CONV), "the fp8 mode rides on the plain byte pipeline");
    static_assert(DIG == 0 || (INT8 && (DIG == 2 || DIG == 3 || DIG == 4)), "digit planes ride on the int8 operands");
    static_assert(DIG != 3 || TM % 3 == 0, "three planes: a wave's rows are whole groups of 24 operand rows (8 activation rows x 3 planes)");
    static_assert(!CONV || (INT8 && DIG == 0), "the conv epilogue belongs to the plain int8 kernel");
    static_assert(!CRNG || CONV, "output ranges come from the conv epilogue");   // CRNG: p.cv.range_out is set
    // Codebook weights (w[n,k] = bscale[n, k/32] * table[nibble], src/packed_tensor.rs:469-521) are decoded here:
    // the nibble looks up an (f16 hi, f16 lo) pair of the scaled table value in LDS, two MFMAs per step (hi, lo)
    // add into a per-block accumulator, and after the two steps of a 32-value block the accumulator is folded into
    // the running sum with the block's scale: sum_blk s_blk * sum_k table[q]*a, the reference's association.
    constexpr bool CB = !INT8 && DT == FNN_DT_I4CB;
    using D = typename std::conditional<INT8, DecI<DT>, DecH<DT>>::type;
    static_assert(!(INT8 && PRECISE), "int8 operands have no hi/lo rows");
    constexpr int WPS = D::WPS;          // words per 8 k-values
    constexpr int WC = 2 * WPS;          // 16-byte weight chunks per row and stage (32, 64 or 128 bytes)
    constexpr int WQW = CB ? 8 : 4 * WPS; // weight words a lane holds per stage and 32-row block
    constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
    constexpr int A_BYTES = BM * 128, W_BYTES = BN * WC * 16, STAGE = A_BYTES + W_BYTES;
    constexpr int NWV = WGM * WGN;                  // waves per workgroup: 4, or 8 (two per SIMD)
    constexpr int A_LPW = BM / (8 * NWV);           // activation load instructions per wave and stage
    // weight load instructions per wave and stage.  When the stage's weight chunks do not divide evenly over the
    // waves (W_WAVES < NWV), the first W_WAVES waves take W_LPW loads each and the others none: the waits below
    // count per wave.
    constexpr int W_LOADS = BN * WC / 64;
    constexpr int W_LPW = (W_LOADS + NWV - 1) / NWV;
    constexpr int W_WAVES = W_LOADS / W_LPW;
    constexpr int LPS = A_LPW + W_LPW;
    static_assert(NWV == 4 || NWV == 8, "4 or 8 waves");
    static_assert(BM % (8 * NWV) == 0 && BN * WC % 64 == 0 && W_LOADS % W_LPW == 0 && NS >= 3 && NS <= 8, "stage shape");
    const bool w_on = W_WAVES == NWV || (int)(threadIdx.x >> 6) < W_WAVES;   // wave-uniform

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)smem;

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int wm = wv / WGN, wn = wv % WGN;
    const int lr = lane & 31, h = lane >> 5;
    __shared__ uint32_t cbt[16];   // codebook mode: (hi | lo << 16) per table entry
    int cb_exp = 0;
    if constexpr (CB) {
        cb_exp = codebook_exp(p.codebook);
        if (tid < 16) {
            const float v = ldexpf(p.codebook[tid], cb_exp);
            const _Float16 hi = (_Float16)v;
            const _Float16 lo = (_Float16)(v - (float)hi);
            cbt[tid] = (uint32_t)__builtin_bit_cast(uint16_t, hi) | ((uint32_t)__builtin_bit_cast(uint16_t, lo) << 16);
        }
        // (the barrier before the first operand read orders this store)
    }

    // workgroup id -> tile, row tile fastest.  Ids are dealt round-robin over the 8 XCDs (each with
    // its own L2), so an XCD keeps meeting the same few row tiles of the activations, the operand
    // with the most bytes per MAC, while the packed weights stream through.
    const unsigned L = blockIdx.x;
    const int mt = L % p.mtiles;
    const unsigned rest = L / p.mtiles;
    const int z = rest % p.splits;
    const int nt = rest / p.splits;
    const int64_t n0 = (int64_t)nt * BN;
    const int it0 = z * p.ips;
    const int it1 = (it0 + p.ips < p.iters) ? it0 + p.ips : p.iters;

    // conv epilogue: per-row constants of the tile (activation scale / zero of the row's image, sum of q_a, NCHW
    // offset of the pixel), requested now so that their latency hides behind the K loop
    constexpr int CV_PARTS = CONV ? (WGM * WGN * 64) / (WGM * TM * 32) : 1;
    __shared__ float cv_sa[CONV ? WGM * TM * 32 : 1], cv_za[CONV ? WGM * TM * 32 : 1];
    __shared__ int cv_qs[CV_PARTS > 0 ? CV_PARTS : 1][CONV ? WGM * TM * 32 : 1];
    __shared__ int64_t cv_off[CONV ? WGM * TM * 32 : 1];
    __shared__ unsigned char cv_img[CRNG ? WGM * TM * 32 : 1];   // 0: the image of the tile's first row, 1: the next one
    __shared__ float cv_red[CRNG ? WGM * WGN : 1][4];
    if constexpr (CONV) {
        constexpr int BM_ = WGM * TM * 32;
        static_assert((WGM * WGN * 64) % BM_ == 0 && CV_PARTS >= 1, "whole row groups per workgroup");
        const int row = threadIdx.x % BM_, part = threadIdx.x / BM_;
        const int64_t r = (int64_t)mt * BM_ + row;
        int qs = 0;
        if (r < p.m)
            for (int y = part; y < p.cv.nq; y += CV_PARTS) qs += p.cv.qsum[(int64_t)y * p.rows_pad + r];
        cv_qs[part][row] = qs;
        if (part == 0) {
            float sa = 0.0f, za = 0.0f;
            int64_t off = 0;
            unsigned char second = 0;
            if (r < p.m) {
                const uint32_t nn = (uint32_t)r / p.cv.np, px = (uint32_t)r - nn * p.cv.np;
                const int bg = (int)nn * p.cv.groups + p.cv.g;
                sa = p.cv.actq[bg * 4 + 0];
                za = p.cv.actq[bg * 4 + 1];
                off = (int64_t)nn * p.cv.oc * p.cv.np + px;
                if constexpr (CRNG) second = (uint32_t)(r - row) / p.cv.np != nn;   // (r - row = the tile's first row)
            }
            cv_sa[row] = sa; cv_za[row] = za; cv_off[row] = off;
            if constexpr (CRNG) cv_img[row] = second;
        }
    }
    // output ranges: which pair of which image this tile fills (32-bit arithmetic: rows < 2^31), worked out before the
    // K loop.  Pair (tile - first tile of the image) * ntiles + nt; a tile that holds the last row of its first
    // image also fills that image's unused pairs, up to np / BM + 2 per column tile.
    uint32_t rng_img = 0;
    int rng_slot = 0, rng_fill = 0, rng_per_m = 0;
    bool rng_two = false, rng_plain = false;
    if constexpr (CRNG) {
        constexpr uint32_t BM_ = WGM * TM * 32;
        const uint32_t np = p.cv.np, row_a = (uint32_t)mt * BM_;
        const uint32_t last = (uint32_t)p.m - 1, row_z = row_a + BM_ - 1 < last ? row_a + BM_ - 1 : last;
        rng_img = row_a / np;
        const uint32_t img_end = (rng_img + 1) * np - 1;           // last row of that image
        rng_slot = (int)((uint32_t)mt - (rng_img * np) / BM_);
        rng_two = row_z > img_end;
        rng_per_m = (int)(np / BM_) + 2;
        rng_fill = row_z >= img_end ? rng_slot + 1 : rng_per_m;
        rng_plain = !rng_two && row_a + BM_ - 1 <= last;
    }
    // ... and this lane's channel constants (scale, zero, scale * sum q_w, bias)
    float cv_sw[CONV ? TN : 1], cv_zw[CONV ? TN : 1], cv_wt[CONV ? TN : 1], cv_bi[CONV ? TN : 1];
    if constexpr (CONV) {
#pragma unroll
        for (int tn = 0; tn < TN; tn++) {
            const int64_t n = (int64_t)nt * (WGN * TN * 32) + (((threadIdx.x >> 6) % WGN) * TN + tn) * 32 + (threadIdx.x & 31);
            const bool ok = n < p.n;
            cv_sw[tn] = ok ? p.scales[n] : 0.0f;
            cv_zw[tn] = ok ? p.zeros[n] : 0.0f;
            cv_wt[tn] = ok ? cv_sw[tn] * (float)p.cv.row_qsum[n] : 0.0f;
            cv_bi[tn] = (ok && p.bias) ? p.bias[n] : 0.0f;
        }
    }

    // ---- what this lane fetches per stage.  LDS slot s of a region = 16-byte chunk s.
    // The LDS has 64 banks of 4 bytes: a 128-bit read is conflict-free when every 16 lanes cover
    // all sixteen 16-byte slots of a 256-byte window, hence the row-dependent XOR of the chunk index.
    // activations: chunk (row, g) lives at slot row*8 + (g ^ ((row >> 1) & 7))
    const _Float16 *a_src[A_LPW];
#pragma unroll
    for (int j = 0; j < A_LPW; j++) {
        const int slot = (wv * A_LPW + j) * 64 + lane;
        const int row = slot >> 3, g = (slot & 7) ^ ((row >> 1) & 7);
        a_src[j] = p.ap + ((int64_t)mt * BM + row) * 64 + g * 8 - (j & 3) * 512;   // (biased: see load_group_to_lds16)
    }
    // weights: chunk (row, c) lives at slot row*WC + (c ^ swz(row)); rows past N repeat the last row
    // tile-major copy: 64 bytes per row and stage = one block per stage (WC == 4); 32 bytes = half a block (WC == 2)
    const bool tmaj = (WC == 4 || WC == 2) && !CB && p.words_tm != nullptr;   // (uniform)
    const uint32_t *w_src[W_LPW];
    int w_chunk[W_LPW];
#pragma unroll
    for (int j = 0; j < W_LPW; j++) {
        const int slot = (wv * W_LPW + j) * 64 + lane;
        const int row = slot / WC;
        const int sw = (WC == 2) ? ((row >> 3) & 1) : (WC == 4 ? ((row >> 2) & 3) : ((row >> 1) & 7));
        const int c = (slot % WC) ^ sw;
        int64_t grow = n0 + row;
        if (grow > p.n - 1) grow = p.n - 1;
        w_src[j] = p.words + grow * p.kp + c * 4 - (j & 3) * 256;                  // (biased likewise)
        if (tmaj) w_src[j] = p.words_tm + (((grow >> 4) * p.kb64) << 8) + ((grow & 15) << 4) + c * 4 - (j & 3) * 256;
        w_chunk[j] = c * 4;
    }
    const int w_stride = tmaj ? 256 : WC * 4;   // words between consecutive stages of a row (tile-major, WC == 4: one block on)
    const int64_t a_step = p.rows_pad * 64;   // elements between consecutive k blocks
    const unsigned a_dst = __builtin_amdgcn_readfirstlane(lds0 + wv * A_LPW * 1024);
    const unsigned w_dst = __builtin_amdgcn_readfirstlane(lds0 + A_BYTES + wv * W_LPW * 1024);

    // dense f16 weights ([hi | lo] halves): rows are whole stages long and the activations are swept twice;
    // packed weights: one sweep, and the last stage of a row may be partly past its end
    constexpr bool DENSE = !INT8 && D::WPS == 4;
    // running source pointers: advanced after every stage, frozen once the K range is exhausted
    // (the extra requests of the last iterations re-read the final stage and are never consumed)
#pragma unroll
    for (int j = 0; j < A_LPW; j++) a_src[j] += (int64_t)(DENSE ? it0 % p.a_wrap : it0) * a_step;
#pragma unroll
    for (int j = 0; j < W_LPW; j++) w_src[j] += (tmaj && WC == 2) ? (int64_t)(it0 >> 1) * 256 + (it0 & 1) * 8 : (int64_t)it0 * w_stride;
    int a_pos = DENSE ? it0 % p.a_wrap : 0;       // position inside the activation sweep
    const bool ragged = !DENSE && (p.kp % (WC * 4)) != 0;
    bool w_past[W_LPW];   // this lane's chunk of the last stage lies behind the end of the row
#pragma unroll
    for (int j = 0; j < W_LPW; j++) w_past[j] = (int64_t)(p.iters - 1) * (WC * 4) + w_chunk[j] + 4 > p.kp;
    auto issue = [&](int it, int buf) {
        const unsigned sb = buf * STAGE;
        const bool last_ragged = ragged && it >= p.iters - 1;   // wave-uniform; folded into selects, no branch
        const void *wp[W_LPW];
#pragma unroll
        for (int j = 0; j < W_LPW; j++) {
            // both addresses are read into values first: a select between the memory locations
            // would keep the pointer array in scratch memory
            const uint64_t wa = reinterpret_cast<uint64_t>(w_src[j]);
            const uint64_t za = reinterpret_cast<uint64_t>(p.zero_chunk) - (uint64_t)((j & 3) * 1024);
            const uint64_t mask = (last_ragged && w_past[j]) ? ~0ull : 0ull;
            wp[j] = reinterpret_cast<const void *>((wa & ~mask) | (za & mask));
        }
#pragma unroll
        for (int g = 0; g < W_LPW; g += 4) {
            if (!w_on) break;
            const int n = W_LPW - g >= 4 ? 4 : W_LPW - g;
            const unsigned base = w_dst + sb + g * 1024;
            if (n == 4) load_group_to_lds16<4>(wp[g], wp[g + 1 < W_LPW ? g + 1 : g], wp[g + 2 < W_LPW ? g + 2 : g], wp[g + 3 < W_LPW ? g + 3 : g], base);
            else if (n == 3) load_group_to_lds16<3>(wp[g], wp[g + 1 < W_LPW ? g + 1 : g], wp[g + 2 < W_LPW ? g + 2 : g], nullptr, base);
            else if (n == 2) load_group_to_lds16<2>(wp[g], wp[g + 1 < W_LPW ? g + 1 : g], nullptr, nullptr, base);
            else load_group_to_lds16<1>(wp[g], nullptr, nullptr, nullptr, base);
        }
#pragma unroll
        for (int g = 0; g < A_LPW; g += 4) {
            const int n = A_LPW - g >= 4 ? 4 : A_LPW - g;
            const unsigned base = a_dst + sb + g * 1024;
            if (n == 4) load_group_to_lds16<4>(a_src[g], a_src[g + 1 < A_LPW ? g + 1 : g], a_src[g + 2 < A_LPW ? g + 2 : g], a_src[g + 3 < A_LPW ? g + 3 : g], base);
            else if (n == 3) load_group_to_lds16<3>(a_src[g], a_src[g + 1 < A_LPW ? g + 1 : g], a_src[g + 2 < A_LPW ? g + 2 : g], nullptr, base);
            else if (n == 2) load_group_to_lds16<2>(a_src[g], a_src[g + 1 < A_LPW ? g + 1 : g], nullptr, nullptr, base);
            else load_group_to_lds16<1>(a_src[g], nullptr, nullptr, nullptr, base);
        }
        const bool more = it + 1 < it1;           // wave-uniform
        int64_t astep = more ? a_step : 0;
        if (DENSE && more && ++a_pos == p.a_wrap) {   // second sweep over the activations
            a_pos = 0;
            astep = -(int64_t)(p.a_wrap - 1) * a_step;
        }
        // (half blocks: from the even half to the odd half of a block 32 bytes, from there to the next block 1024 - 32)
        const int wstep = !more ? 0 : ((tmaj && WC == 2) ? ((it & 1) ? 248 : 8) : w_stride);
#pragma unroll
        for (int j = 0; j < A_LPW; j++) a_src[j] += astep;
#pragma unroll
        for (int j = 0; j < W_LPW; j++) w_src[j] += wstep;
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[tm][tn][i] = 0.0f;

    // operand read offsets inside a stage
    int a_off[TM], w_off[TN];
#pragma unroll
    for (int tm = 0; tm < TM; tm++) a_off[tm] = ((wm * TM + tm) * 32 + lr) * 128;
#pragma unroll
    for (int tn = 0; tn < TN; tn++) {
        const int row = (wn * TN + tn) * 32 + lr;
        if constexpr (CB) w_off[tn] = A_BYTES + row * 32;   // both chunks of the row are read
        else if constexpr (WC == 2) w_off[tn] = A_BYTES + (row * 2 + (h ^ ((row >> 3) & 1))) * 16;
        else w_off[tn] = A_BYTES + row * (WC * 16);   // chunk index added per read
    }
    const int asw = (lr >> 1) & 7;   // (row >> 1) & 7 of every activation row this lane reads

    if (it0 < it1) {
        // ---- main loop: a flat software pipeline over the MFMA steps (4 per stage).
        //  - activation fragments are requested from LDS two steps ahead (ring of 4 register sets),
        //  - weight words are decoded one step ahead,
        //  - the stage hand-over (wait for the next stage, barrier, request of a further stage)
        //    sits between steps 1 and 2; steps 2 and 3 already read the next stage's operands,
        // so the matrix cores never wait for a whole LDS round trip.
        auto read_w = [&](const unsigned char *sbase, uint32_t(&wq)[TN][WQW]) {
#pragma unroll
            for (int tn = 0; tn < TN; tn++) {
                if constexpr (CB) {
                    // the 8 words (64 nibbles) of the row's stage; MFMA step s takes word 2s + h
                    const int row = (wn * TN + tn) * 32 + lr;
                    const int sw = (row >> 3) & 1;
                    const u32x4 t0 = *reinterpret_cast<const u32x4 *>(sbase + w_off[tn] + (0 ^ sw) * 16);
                    const u32x4 t1 = *reinterpret_cast<const u32x4 *>(sbase + w_off[tn] + (1 ^ sw) * 16);
                    wq[tn][0] = t0[0]; wq[tn][1] = t0[1]; wq[tn][2] = t0[2]; wq[tn][3] = t0[3];
                    wq[tn][4] = t1[0]; wq[tn][5] = t1[1]; wq[tn][6] = t1[2]; wq[tn][7] = t1[3];
                } else if constexpr (WC == 2) {
                    const u32x4 t = *reinterpret_cast<const u32x4 *>(sbase + w_off[tn]);
                    wq[tn][0] = t[0]; wq[tn][1] = t[1]; wq[tn][2] = t[2]; wq[tn][3] = t[3];
                } else {
                    constexpr int CPH = WC / 2;   // chunks per lane half: 2 (8-bit types) or 4 (f16)
                    const int row = (wn * TN + tn) * 32 + lr;
                    const int sw = (WC == 4) ? ((row >> 2) & 3) : ((row >> 1) & 7);
#pragma unroll
                    for (int c = 0; c < CPH; c++) {
                        const u32x4 t = *reinterpret_cast<const u32x4 *>(sbase + w_off[tn] + (((CPH * h + c) ^ sw) * 16));
                        wq[tn][4 * c + 0] = t[0]; wq[tn][4 * c + 1] = t[1]; wq[tn][4 * c + 2] = t[2]; wq[tn][4 * c + 3] = t[3];
                    }
                }
            }
        };
        auto read_a = [&](const unsigned char *sbase, int s, f16x8(&af)[TM]) {
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
                af[tm] = *reinterpret_cast<const f16x8 *>(sbase + a_off[tm] + (((CB ? 2 * s + h : 4 * h + s) ^ asw) * 16));
        };
        f32x16 accb[CB ? TM : 1][CB ? TN : 1];   // codebook mode: sum over the current 32-value block
        float bs_cur[TN][2], bs_nxt[TN][2];         // ... and the block scales of this lane's columns (this / next stage)
        auto load_bscales = [&](int it, float(&bs)[TN][2]) {
#pragma unroll
            for (int tn = 0; tn < TN; tn++) {
                int64_t n = n0 + (wn * TN + tn) * 32 + lr;
                if (n > p.n - 1) n = p.n - 1;
#pragma unroll
                for (int b = 0; b < 2; b++) {
                    int64_t blk = 2 * (int64_t)it + b;
                    if (blk > p.bpr - 1) blk = p.bpr - 1;   // past K: the activations are zero there
                    bs[tn][b] = p.bscales[n * p.bpr + blk];
                }
            }
        };
        auto decode = [&](const uint32_t(&wq)[TN][WQW], int s, f16x8(&bf)[TN], f16x8(&bl)[CB ? TN : 1]) {
#pragma unroll
            for (int tn = 0; tn < TN; tn++) {
                if constexpr (CB) {
                    const uint32_t w = h ? wq[tn][2 * s + 1] : wq[tn][2 * s];
                    uint32_t d[8];
                    d[0] = cbt[w & 15u];
#pragma unroll
                    for (int j = 1; j < 8; j++) d[j] = cbt[(w >> (4 * j)) & 15u];
                    uint32_t hi4[4], lo4[4];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        hi4[j] = __builtin_amdgcn_perm(d[2 * j + 1], d[2 * j], 0x05040100u);   // low halves: hi parts
                        lo4[j] = __builtin_amdgcn_perm(d[2 * j + 1], d[2 * j], 0x07060302u);   // high halves: lo parts
                    }
                    bf[tn] = pack8(hi4[0], hi4[1], hi4[2], hi4[3]);
                    bl[tn] = pack8(lo4[0], lo4[1], lo4[2], lo4[3]);
                } else {
                    bf[tn] = D::step(&wq[tn][s * WPS]);
                }
            }
        };
        // s = step inside the stage (codebook mode: steps 0,1 are one block, steps 2,3 the next)
        auto mfmas = [&](const f16x8(&af)[TM], const f16x8(&bf)[TN], const f16x8(&bl)[CB ? TN : 1], int s) {
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int tn = 0; tn < TN; tn++)
                    if constexpr (FP8) {
                        typedef long i64x2 __attribute__((ext_vector_type(2)));
                        const i64x2 a2 = __builtin_bit_cast(i64x2, af[tm]), b2 = __builtin_bit_cast(i64x2, bf[tn]);
                        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a2[0], b2[0], acc[tm][tn], 0, 0, 0);
                        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a2[1], b2[1], acc[tm][tn], 0, 0, 0);
                    } else if constexpr (INT8) {
                        acc[tm][tn] = __builtin_bit_cast(f32x16, __builtin_amdgcn_mfma_i32_32x32x32_i8(
                                                                     __builtin_bit_cast(i32x4, af[tm]), __builtin_bit_cast(i32x4, bf[tn]),
                                                                     __builtin_bit_cast(i32x16, acc[tm][tn]), 0, 0, 0));
                    } else if constexpr (CB) {
                        f32x16 c0 = accb[tm][tn];
                        if ((s & 1) == 0) {
#pragma unroll
                            for (int i = 0; i < 16; i++) c0[i] = 0.0f;
                        }
                        c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[tm], bf[tn], c0, 0, 0, 0);
                        accb[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[tm], bl[tn], c0, 0, 0, 0);
                        if (s & 1) {
                            const float sc = bs_cur[tn][s >> 1];
#pragma unroll
                            for (int i = 0; i < 16; i++) acc[tm][tn][i] = fmaf(sc, accb[tm][tn][i], acc[tm][tn][i]);
                        }
                    } else {
                        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[tm], bf[tn], acc[tm][tn], 0, 0, 0);
                    }
        };

        // With a ring of three a hand-over waits for every outstanding load, so stages past the K range need not be
        // requested to keep the wait counts right: a short K range (the first conv layers: one or two stages)
        // then moves no byte twice and needs one LDS buffer per stage it has (the launcher sizes LDS to that).
        // Deeper rings keep requesting (re-reads of the final stage that nothing consumes).
        constexpr bool EXACT = NS == 3;
        const bool one_stage = EXACT && it1 - it0 == 1;   // (workgroup-uniform)
        if (one_stage) {
            issue(it0, 0);
        } else {
#pragma unroll
            for (int st = 0; st < NS - 1; st++) issue(it0 + st, st);
        }
        uint32_t wq[TN][WQW], wqn[TN][WQW];
        f16x8 af[4][TM], bfr[2][TN], bfl[2][CB ? TN : 1];
        if constexpr (CB) load_bscales(it0, bs_cur);
        // first stage: this wave's part has landed
        if (one_stage) wait_loads_but<0>();
        else if (w_on) wait_loads_but<(NS - 2) * LPS>();
        else wait_loads_but<(NS - 2) * A_LPW>();
        __syncthreads();                    // ... and everybody else's
        read_w(smem, wq);
        read_a(smem, 0, af[0]);
        read_a(smem, 1, af[1]);
        decode(wq, 0, bfr[0], bfl[0]);
        // The loop body is one straight-line block (no branches), so the compiler can interleave LDS
        // reads, decode and MFMAs across the whole stage; the last stage, which has no successor to
        // hand over to, is peeled off.
        int buf = 0;
        for (int it = it0; it < it1 - 1; it++) {
            const unsigned char *sbase = smem + buf * STAGE;
            const int nbuf = (buf + 1 == NS) ? 0 : buf + 1;
            const unsigned char *nbase = smem + nbuf * STAGE;
            if constexpr (CB) load_bscales(it + 1, bs_nxt);
            // step 0
            read_a(sbase, 2, af[2]);
            decode(wq, 1, bfr[1], bfl[1]);
            mfmas(af[0], bfr[0], bfl[0], 0);
            // step 1
            read_a(sbase, 3, af[3]);
            decode(wq, 2, bfr[0], bfl[0]);
            mfmas(af[1], bfr[1], bfl[1], 1);
            // hand-over
            // this wave's part of the next stage has landed
            if (w_on) wait_loads_but<(NS - 3) * LPS>();
            else wait_loads_but<(NS - 3) * A_LPW>();
            __syncthreads();                    // everybody's; the stage before the current one is free
            int fb = buf + NS - 1;
            if (fb >= NS) fb -= NS;
            if (!EXACT || it + NS - 1 < it1) issue(it + NS - 1, fb);
            // step 2, with the first reads of the next stage
            read_w(nbase, wqn);
            read_a(nbase, 0, af[0]);
            decode(wq, 3, bfr[1], bfl[1]);
            mfmas(af[2], bfr[0], bfl[0], 2);
            // step 3
            read_a(nbase, 1, af[1]);
            decode(wqn, 0, bfr[0], bfl[0]);
            mfmas(af[3], bfr[1], bfl[1], 3);
#pragma unroll
            for (int tn = 0; tn < TN; tn++)
#pragma unroll
                for (int q = 0; q < WQW; q++) wq[tn][q] = wqn[tn][q];
            if constexpr (CB) {
#pragma unroll
                for (int tn = 0; tn < TN; tn++) { bs_cur[tn][0] = bs_nxt[tn][0]; bs_cur[tn][1] = bs_nxt[tn][1]; }
            }
            buf = nbuf;
        }
        {   // last stage
            const unsigned char *sbase = smem + buf * STAGE;
            read_a(sbase, 2, af[2]);
            decode(wq, 1, bfr[1], bfl[1]);
            mfmas(af[0], bfr[0], bfl[0], 0);
            read_a(sbase, 3, af[3]);
            decode(wq, 2, bfr[0], bfl[0]);
            mfmas(af[1], bfr[1], bfl[1], 1);
            decode(wq, 3, bfr[1], bfl[1]);
            mfmas(af[2], bfr[0], bfl[0], 2);
            mfmas(af[3], bfr[1], bfl[1], 3);
        }
        wait_loads_but<0>();   // nothing may still be writing LDS when the workgroup retires
    }



    // ---- epilogue.  acc[i] of a 32x32 block: row (i/4)*8 + h*4 + i%4, column lr.  With hi/lo
    // operands a block holds 16 output rows: hi in rows 0..15 (i < 8), lo in rows 16..31 (i + 8).
    if constexpr (INT8 && DIG == 3) {
        // slab q of the wave (operand rows 8q .. 8q + 7, q = tm*4 + i/4) = plane q % 3 of the activation rows
        // 8 (q/3) .. + 7; a lane holds rows 4h + t of every slab in acc[q / 4][tn][(q % 4) * 4 + t]
        constexpr int SHIFT = (DT == FNN_DT_I4) ? 4 : 0;   // 4-bit signed lanes entered as 16*q
        constexpr int GR = TM * 4 / 3;                      // groups of 8 activation rows per wave
        const int64_t mrow0 = ((int64_t)mt * BM + wm * TM * 32) / 3;
        const bool split = p.splits > 1;
        float sc[TN], zp[TN], bi[TN];
#pragma unroll
        for (int tn = 0; tn < TN; tn++) {
            const int64_t n = n0 + (wn * TN + tn) * 32 + lr;
            const bool ok = n < p.n && !split;
            sc[tn] = ok ? p.scales[n] : 0.0f;
            zp[tn] = ok ? p.zeros[n] : 0.0f;
            bi[tn] = (ok && p.bias) ? p.bias[n] : 0.0f;
        }
        int rexp[GR][4];
        float rxs[GR][4];
#pragma unroll
        for (int u = 0; u < GR; u++)
#pragma unroll
            for (int t = 0; t < 4; t++) {
                int64_t m = mrow0 + u * 8 + h * 4 + t;
                if (m > p.m - 1) m = p.m - 1;
                rexp[u][t] = p.rexp[m];
                rxs[u][t] = split ? 0.0f : p.xsum[m];
            }
#pragma unroll
        for (int u = 0; u < GR; u++)
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int64_t m = mrow0 + u * 8 + h * 4 + t;
                if (m >= p.m) continue;
                const int e = rexp[u][t];
                const bool bad = e == INT_MIN;      // the row holds a non-finite activation
#pragma unroll
                for (int tn = 0; tn < TN; tn++) {
                    const int64_t n = n0 + (wn * TN + tn) * 32 + lr;
                    if (n >= p.n) continue;
                    float v = 0.0f;
#pragma unroll
                    for (int j = 2; j >= 0; j--) {
                        const int q = 3 * u + j;
                        v = fmaf(v, 256.0f, (float)__float_as_int(acc[q >> 2][tn][(q & 3) * 4 + t]));
                    }
                    const float d = bad ? __builtin_nanf("") : ldexpf(v, -e - SHIFT);
                    if (split) {
                        p.part[((int64_t)z * p.m + m) * p.n + n] = d;
                    } else {
                        float o = d * sc[tn] + zp[tn] * rxs[u][t];
                        if (p.bias) o = o + bi[tn];
                        p.out[m * p.n + n] = fnn_activation(o, p.act);
                    }
                }
            }
        return;
    } else if constexpr (INT8 && DIG > 0) {
        constexpr int RPB = 32 / DIG;        // activation rows per 32-row block
        constexpr int NR = RPB / 2;          // ... of which a lane holds NR (the other half belongs to lanes h ^ 1)
        constexpr int SHIFT = (DT == FNN_DT_I4) ? 4 : 0;   // 4-bit signed lanes entered as 16*q
        const int64_t mrow0 = ((int64_t)mt * (BM / 32) + wm * TM) * RPB;
        const bool split = p.splits > 1;
        float sc[TN], zp[TN], bi[TN];
#pragma unroll
        for (int tn = 0; tn < TN; tn++) {
            const int64_t n = n0 + (wn * TN + tn) * 32 + lr;
            const bool ok = n < p.n && !split;
            sc[tn] = ok ? p.scales[n] : 0.0f;
            zp[tn] = ok ? p.zeros[n] : 0.0f;
            bi[tn] = (ok && p.bias) ? p.bias[n] : 0.0f;
        }
        // acc index of (row r of the lane, plane j): block row j*RPB + (r/4)*8 + h*4 + r%4 = (i/4)*8 + h*4 + i%4
        int rexp[TM][NR];
        float rxs[TM][NR];
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
#pragma unroll
            for (int r = 0; r < NR; r++) {
                int64_t m = mrow0 + tm * RPB + (r / 4) * 8 + h * 4 + (r % 4);
                if (m > p.m - 1) m = p.m - 1;
                rexp[tm][r] = p.rexp[m];
                rxs[tm][r] = split ? 0.0f : p.xsum[m];
            }
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
#pragma unroll
            for (int r = 0; r < NR; r++) {
                const int64_t m = mrow0 + tm * RPB + (r / 4) * 8 + h * 4 + (r % 4);
                if (m >= p.m) continue;
                const int e = rexp[tm][r];
                const bool bad = e == INT_MIN;      // the row holds a non-finite activation
#pragma unroll
                for (int tn = 0; tn < TN; tn++) {
                    const int64_t n = n0 + (wn * TN + tn) * 32 + lr;
                    if (n >= p.n) continue;
                    float v = 0.0f;
#pragma unroll
                    for (int j = DIG - 1; j >= 0; j--) {
                        const int i = j * (RPB / 8) * 4 + (r / 4) * 4 + (r % 4);
                        const float bits = acc[tm][tn][i];
                        v = fmaf(v, 256.0f, (float)__float_as_int(bits));
                    }
                    float d = bad ? __builtin_nanf("") : ldexpf(v, -e - SHIFT);
                    if (split) {
                        p.part[((int64_t)z * p.m + m) * p.n + n] = d;
                    } else {
                        float o = d * sc[tn] + zp[tn] * rxs[tm][r];
                        if (p.bias) o = o + bi[tn];
                        p.out[m * p.n + n] = fnn_activation(o, p.act);
                    }
                }
            }
        return;
    } else if constexpr (INT8 && CONV) {
        __syncthreads();   // the row tables
        const float *sw = cv_sw, *zw = cv_zw, *wt = cv_wt, *bi = cv_bi;
        const bool has_bias = p.bias != nullptr;
        const int64_t np = p.cv.np;
        float mn0 = INFINITY, mx0 = -INFINITY, mn1 = INFINITY, mx1 = -INFINITY;   // of the stored values, per image
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
#pragma unroll
            for (int ig = 0; ig < 4; ig++) {
                const int rr0 = (wm * TM + tm) * 32 + ig * 8 + h * 4;   // four consecutive rows of the tile
                const int64_t r0 = (int64_t)mt * BM + rr0;
                if (r0 >= p.m) continue;
                float sa[4], za[4], rs[4];
                bool second[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    second[j] = (CRNG && rng_two) ? cv_img[rr0 + j] != 0 : false;
                    int qs = 0;
#pragma unroll
                    for (int y = 0; y < CV_PARTS; y++) qs += cv_qs[y][rr0 + j];
                    sa[j] = cv_sa[rr0 + j];
                    za[j] = cv_za[rr0 + j];
                    rs[j] = sa[j] * (float)qs;
                }
#pragma unroll
                for (int tn = 0; tn < TN; tn++) {
                    const int64_t n = n0 + (wn * TN + tn) * 32 + lr;
                    if (n >= p.n) continue;
                    float v[4];
                    int av[4], bq[4];
                    // the rounded bias depends on (image, channel) only: one division for the four rows when they
                    // share an image
                    bq[0] = has_bias ? conv_bias_q(bi[tn], sa[0], sw[tn]) : 0;
#pragma unroll
                    for (int j = 1; j < 4; j++) bq[j] = (p.cv.vec4 || !has_bias) ? bq[0] : conv_bias_q(bi[tn], sa[j], sw[tn]);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const float bits = acc[tm][tn][ig * 4 + j];
                        int a = __float_as_int(bits);
                        if constexpr (DT == FNN_DT_I4) a >>= 4;
                        v[j] = conv_affine(a, sa[j], za[j], rs[j], sw[tn], zw[tn], wt[tn], bq[j], p.cv.kk, &av[j]);
                    }
                    conv_act4(v, p.act);
                    if (p.cv.vec4) {
                        const int64_t o = cv_off[rr0] + n * np;
                        *reinterpret_cast<float4 *>(p.cv.y + o) = make_float4(v[0], v[1], v[2], v[3]);
                        if (p.cv.acc_out) *reinterpret_cast<int4 *>(p.cv.acc_out + o) = make_int4(av[0], av[1], av[2], av[3]);
                        if (p.cv.residual) {   // the Add behind this convolution: v becomes the sums (their ranges travel on)
                            const float4 r4 = *reinterpret_cast<const float4 *>(p.cv.residual + o);
                            v[0] = v[0] + r4.x; v[1] = v[1] + r4.y; v[2] = v[2] + r4.z; v[3] = v[3] + r4.w;
                            *reinterpret_cast<float4 *>(p.cv.sum_out + o) = make_float4(v[0], v[1], v[2], v[3]);
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            if (r0 + j >= p.m) continue;
                            const int64_t o = cv_off[rr0 + j] + n * np;
                            p.cv.y[o] = v[j];
                            if (p.cv.acc_out) p.cv.acc_out[o] = av[j];
                            if (p.cv.residual) {
                                v[j] = v[j] + p.cv.residual[o];
                                p.cv.sum_out[o] = v[j];
                            }
                        }
                    }
                    if constexpr (CRNG) {
                        if (rng_plain) {   // (workgroup-uniform) every row of the tile exists and lies in one image
                            mn0 = fminf(fminf(mn0, fminf(v[0], v[1])), fminf(v[2], v[3]));
                            mx0 = fmaxf(fmaxf(mx0, fmaxf(v[0], v[1])), fmaxf(v[2], v[3]));
                        } else {
#pragma unroll
                            for (int j = 0; j < 4; j++) {
                                if (r0 + j >= p.m) continue;
                                if (second[j]) { mn1 = fminf(mn1, v[j]); mx1 = fmaxf(mx1, v[j]); }
                                else { mn0 = fminf(mn0, v[j]); mx0 = fmaxf(mx0, v[j]); }
                            }
                        }
                    }
                }
            }
        if (CRNG && (int64_t)mt * BM < p.m) {   // (workgroup-uniform)
            mn0 = wave_min(mn0); mx0 = wave_max(mx0);
            if (rng_two) { mn1 = wave_min(mn1); mx1 = wave_max(mx1); }
            if (lane == 0) { cv_red[wv][0] = mn0; cv_red[wv][1] = mx0; cv_red[wv][2] = mn1; cv_red[wv][3] = mx1; }
            __syncthreads();
            if (tid == 0) {
#pragma unroll
                for (int w2 = 1; w2 < NWV; w2++) {
                    mn0 = fminf(mn0, cv_red[w2][0]); mx0 = fmaxf(mx0, cv_red[w2][1]);
                    mn1 = fminf(mn1, cv_red[w2][2]); mx1 = fmaxf(mx1, cv_red[w2][3]);
                }
                // (the pairs of a column tile lie together: a reader of some of the channels takes its tiles' pairs)
                float *row = p.cv.range_out + (int64_t)rng_img * p.cv.range_stride * 2 + (int64_t)nt * rng_per_m * 2;
                float *dst = row + (int64_t)rng_slot * 2;
                dst[0] = mn0; dst[1] = mx0;
                if (rng_two) {   // the next image starts in this tile: its pair 0
                    float *d1 = row + (int64_t)p.cv.range_stride * 2;
                    d1[0] = mn1; d1[1] = mx1;
                }
                for (int j = rng_fill; j < rng_per_m; j++) {   // the image of the first row ends here: its unused pairs
                    float *d2 = row + (int64_t)j * 2;
                    d2[0] = INFINITY; d2[1] = -INFINITY;
                }
            }
        }
        return;
    } else if constexpr (INT8) {
        const int64_t mrow = ((int64_t)mt * (BM / 32) + wm * TM) * 32;
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int64_t m = mrow + tm * 32 + (i / 4) * 8 + h * 4 + (i % 4);
                if (m >= p.m) continue;
#pragma unroll
                for (int tn = 0; tn < TN; tn++) {
                    const int64_t n = n0 + (wn * TN + tn) * 32 + lr;
                    if (n >= p.n) continue;
                    const float bits = acc[tm][tn][i];   // (bit_cast on a vector element would read element 0)
                    int v = __float_as_int(bits);
                    if constexpr (DT == FNN_DT_I4) v >>= 4;
                    p.c_i32[((int64_t)z * p.m + m) * p.ldc + n] = v;   // (K split: one exact partial matrix per split)
                }
            }
        return;
    }
    constexpr int RPB = PRECISE ? 16 : 32;           // output rows per block
    constexpr int NI = PRECISE ? 8 : 16;
    const int64_t mrow0 = ((int64_t)mt * (BM / 32) + wm * TM) * RPB;
    float sc[TN], zp[TN], bi[TN], um[TN];
    const bool split = p.splits > 1;
#pragma unroll
    for (int tn = 0; tn < TN; tn++) {
        const int64_t n = n0 + (wn * TN + tn) * 32 + lr;
        const bool ok = n < p.n && !split;
        if constexpr (CB) {   // block scales are applied in the loop; what is left is the table's power of two
            sc[tn] = ok ? ldexpf(1.0f, -cb_exp) : 0.0f;
            zp[tn] = 0.0f;
        } else {
            sc[tn] = ok ? p.scales[n] : 0.0f;
            zp[tn] = ok ? p.zeros[n] : 0.0f;
        }
        bi[tn] = (ok && p.bias) ? p.bias[n] : 0.0f;
        um[tn] = (!PRECISE && ok && p.umean) ? p.umean[n] : 0.0f;
    }
    // row constants of every output row this lane holds, requested together (clamped rows, masked
    // later) so that their latencies overlap instead of chaining behind the stores
    int rexp[TM][NI];
    float rxs[TM][NI], rcorr[TM][NI];
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
#pragma unroll
        for (int i = 0; i < NI; i++) {
            int64_t m = mrow0 + tm * RPB + (i / 4) * 8 + h * 4 + (i % 4);
            if (m > p.m - 1) m = p.m - 1;
            rexp[tm][i] = p.rexp[m];
            rxs[tm][i] = split ? 0.0f : p.xsum[m];
            rcorr[tm][i] = (!PRECISE && !split) ? p.esum[m] : 0.0f;
        }
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const int64_t m = mrow0 + tm * RPB + (i / 4) * 8 + h * 4 + (i % 4);
            if (m >= p.m) continue;
            const int e = rexp[tm][i];
            const float xs = rxs[tm][i];
            float corr = 0.0f;
            if constexpr (!PRECISE) corr = ldexpf(rcorr[tm][i], -e);
#pragma unroll
            for (int tn = 0; tn < TN; tn++) {
                const int64_t n = n0 + (wn * TN + tn) * 32 + lr;
                if (n >= p.n) continue;
                float v;
                if constexpr (PRECISE) v = acc[tm][tn][i] + acc[tm][tn][i + 8] * LO_DOWN;
                else v = acc[tm][tn][i];
                float d = ldexpf(v, -e);   // this workgroup's share of sum_k A[m,k]*u(W[n,k])
                if (split) {
                    p.part[((int64_t)z * p.m + m) * p.n + n] = d;
                } else {
                    if constexpr (!PRECISE) d = d - um[tn] * corr;
                    float o = d * sc[tn] + zp[tn] * xs;
                    if (p.bias) o = o + bi[tn];
                    p.out[m * p.n + n] = fnn_activation(o, p.act);
                }
            }
        }
}

// sum of the K-split partial tiles in split order + affine / bias / activation epilogue.  A thread owns one
// output column (its constants stay in registers) and walks rows blockIdx.y, +gridDim.y, ...; the partial tiles
// of an element are requested four at a time and added in split order.
__global__ void __launch_bounds__(256) splitk_epilogue_kernel(TileArgs p, int single)
{
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (n >= p.n) return;
    const int64_t total = p.m * p.n;
    const float sc = p.codebook ? ldexpf(1.0f, -codebook_exp(p.codebook)) : p.scales[n];   // (codebook weights decoded in the tile kernel)
    const float zr = p.codebook ? 0.0f : p.zeros[n];
    const float bs = p.bias ? p.bias[n] : 0.0f;
    const bool comp = single && p.umean;
    const float um = comp ? p.umean[n] : 0.0f;
    for (int64_t m = blockIdx.y; m < p.m; m += gridDim.y) {
        const int64_t idx = m * p.n + n;
        const float *pp = p.part + idx;
        float d = 0.0f;
        int zz = 0;
        for (; zz + 4 <= p.splits; zz += 4) {
            const float v0 = pp[(int64_t)zz * total], v1 = pp[(int64_t)(zz + 1) * total];
            const float v2 = pp[(int64_t)(zz + 2) * total], v3 = pp[(int64_t)(zz + 3) * total];
            d = (((d + v0) + v1) + v2) + v3;
        }
        for (; zz < p.splits; zz++) d += pp[(int64_t)zz * total];
        if (comp) d = d - um * ldexpf(p.esum[m], -p.rexp[m]);
        float o = d * sc + zr * p.xsum[m];
        if (p.bias) o = o + bs;
        o = fnn_activation(o, p.act);
        p.out[idx] = o;
        if (p.residual) p.sum_out[idx] = o + p.residual[idx];
    }
}
