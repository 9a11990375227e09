// Quantised MatMul for up to 32 activation rows (17..32 by default) in ONE launch on the matrix cores (gfx950): the packed weights are
// streamed straight into the registers that are the MFMA's weight operand, the f32 activations are converted inside
// the kernel, K is split over workgroups and the split is reduced inside the same launch.
//
//   out[m,n] = act((sum_k A[m,k]*u(W[n,k]))*scale[n] + zero[n]*sum_k A[m,k] + bias[n])
//   (gemm_batch_packed_simd + apply_affine_dot, src/backend/cpu/microkernels/gemm.rs:1982-2088,
//    src/backend/cpu/microkernels/mod.rs:283-295)
//
// These calls are bound by the weight bytes (at most 128 flop per byte), so the organisation is the GEMV's, not the
// tile GEMM's: no preparation launch, no weight bytes through LDS, no reduction launch.
//
// Work split.  A workgroup of 8 waves owns 8*RT*16 weight rows x a K range of `rounds` x KR values (grid = column
// tiles x splits).  Per round:
//   1. every wave requests its packed bytes (16 rows x KR values per row tile, raw buffer loads: rows past N and
//      bytes past the buffer read as zero) and its share of the activation block (16*MB rows x KR values, split in
//      units of 16 rows x one lane load of weights; the four lanes of a row load 64 contiguous bytes per
//      instruction, and step 3 scatters each register to the fragment of the lane that multiplies it);
//   2. row maxima and row sums of the round meet in LDS; every row gets one power-of-two scale per round;
//   3. the units are converted into MFMA operand fragments in LDS, laid out so that a fragment is 64 lanes x 16
//      contiguous bytes (conflict-free reads, no swizzle):
//        I8 / I4 / U4 weights: three exact balanced base-256 digit planes of rint(x * 2^-e), |v| < 2^22, for
//          v_mfma_i32_16x16x64_i8 against the packed bytes as they are (4-bit lanes: one mask / shift-mask per word);
//        U8 / F8 / F8R / F4 weights: f16 hi + lo of x * 2^-e (about 22 mantissa bits) for v_mfma_f32_16x16x32_f16
//          against the weights decoded to f16 in registers (exact for every one of these types);
//        codebook weights (blocks of 32 values with an f32 scale each, 16 table values): the same activation halves
//          against the f16 hi and lo of the table value (scaled by one power of two) that a nibble looks up in a
//          16-word LDS table; one MFMA step is one block, its sum is folded into the running sum with the block's
//          scale: sum_blk s_blk * sum_k table[q] * a, the reference's association (src/packed_tensor.rs:469-521);
//   4. every wave multiplies its row tiles with all MB activation blocks; integer plane sums are exact and are
//      recombined in f32 once per round.
// Split K: a workgroup stores its partial accumulator registers and row sums with agent-scope (write-through)
// stores, waits for them, and counts itself on the column tile's counter.  The workgroup that finds the count
// complete adds the partials of all splits in split order (agent-scope loads, so the sum does not depend on which
// workgroup arrives last), resets the counter and runs the epilogue.  Nobody waits for anybody: there is no spinning.
// Algorithmic bytes per launch: N*K*bits/8 + side tables + 4*M*(K+N).
#pragma once
#include "dech.h"
#include "mfma.h"
#include "qgemm_stream.h"

#include <climits>

namespace {

using namespace dech;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int NW = FNN_STREAM_NW;

// which matrix core a weight type runs on here, and the geometry of one 16-byte lane load of its packed words
template <int DT>
struct StreamType;
template <> struct StreamType<FNN_DT_I8> { static constexpr int BITS = 8; static constexpr bool INT8 = true; static constexpr float POST = 1.0f; };
template <> struct StreamType<FNN_DT_I4> { static constexpr int BITS = 4; static constexpr bool INT8 = true; static constexpr float POST = 0.0625f; };
template <> struct StreamType<FNN_DT_U4> { static constexpr int BITS = 4; static constexpr bool INT8 = true; static constexpr float POST = 1.0f; };
template <> struct StreamType<FNN_DT_U8> { static constexpr int BITS = 8; static constexpr bool INT8 = false; static constexpr float POST = 1.0f; };
template <> struct StreamType<FNN_DT_F8> { static constexpr int BITS = 8; static constexpr bool INT8 = false; static constexpr float POST = 1.0f; };
template <> struct StreamType<FNN_DT_F8R> { static constexpr int BITS = 8; static constexpr bool INT8 = false; static constexpr float POST = 1.0f; };
template <> struct StreamType<FNN_DT_F4> { static constexpr int BITS = 4; static constexpr bool INT8 = false; static constexpr float POST = 1.0f; };
template <> struct StreamType<FNN_DT_I4CB> { static constexpr int BITS = 4; static constexpr bool INT8 = false; static constexpr float POST = 1.0f; };

// int8 operand of one MFMA from the four words of a lane load (4-bit types: even nibbles, then odd nibbles)
template <int DT>
__device__ __forceinline__ i32x4 int8_operand(const u32x4 &w, int odd)
{
    if constexpr (DT == FNN_DT_I8) {
        return i32x4{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    } else if constexpr (DT == FNN_DT_I4) {   // 16*q in the high nibble of a byte
        if (odd) return i32x4{(int)(w[0] & 0xF0F0F0F0u), (int)(w[1] & 0xF0F0F0F0u), (int)(w[2] & 0xF0F0F0F0u), (int)(w[3] & 0xF0F0F0F0u)};
        return i32x4{(int)((w[0] << 4) & 0xF0F0F0F0u), (int)((w[1] << 4) & 0xF0F0F0F0u), (int)((w[2] << 4) & 0xF0F0F0F0u),
                     (int)((w[3] << 4) & 0xF0F0F0F0u)};
    } else {                                  // unsigned nibbles fit a signed byte as they are
        if (odd) return i32x4{(int)((w[0] >> 4) & 0x0F0F0F0Fu), (int)((w[1] >> 4) & 0x0F0F0F0Fu), (int)((w[2] >> 4) & 0x0F0F0F0Fu),
                              (int)((w[3] >> 4) & 0x0F0F0F0Fu)};
        return i32x4{(int)(w[0] & 0x0F0F0F0Fu), (int)(w[1] & 0x0F0F0F0Fu), (int)(w[2] & 0x0F0F0F0Fu), (int)(w[3] & 0x0F0F0F0Fu)};
    }
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t raw_buffer(const void *base, uint64_t bytes)
{
    const uint32_t n = bytes > 0xffffffffull ? 0xffffffffu : (uint32_t)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n, 0x00020000);
}

// Stores and loads that other workgroups of the same launch must see / be seen by: agent scope, so they go through
// to memory instead of staying in (or being answered from) the L2 of one XCD.
__device__ __forceinline__ void agent_store(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float agent_load(const float *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// byte `d` of four values side by side (4x4 byte transpose with v_perm_b32; selector bytes 0-3 pick from the second
// operand, 4-7 from the first): o[d] = {a.d, b.d, c.d, d.d}
__device__ __forceinline__ void transpose4(uint32_t a, uint32_t b, uint32_t c, uint32_t d, uint32_t (&o)[4])
{
    const uint32_t ab_lo = __builtin_amdgcn_perm(b, a, 0x05010400u);
    const uint32_t ab_hi = __builtin_amdgcn_perm(b, a, 0x07030602u);
    const uint32_t cd_lo = __builtin_amdgcn_perm(d, c, 0x05010400u);
    const uint32_t cd_hi = __builtin_amdgcn_perm(d, c, 0x07030602u);
    o[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);
    o[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
    o[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
    o[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
}

// MB: blocks of 16 activation rows (M <= 16*MB); RT: row tiles of 16 weight rows per wave; KR: k-values per round
// TMAJ: the packed words come from the tile-major copy (p.words_tm)
template <int DT, int MB, int RT, int KR, bool TMAJ = false>
__global__ void __launch_bounds__(NW * 64) qgemm_stream_kernel(StreamArgs p)
{
    using T = StreamType<DT>;
    constexpr bool INT8 = T::INT8;
    constexpr bool CB = DT == FNN_DT_I4CB;           // nibbles look up a 16-entry table; one f32 scale per 32 values
    constexpr int BITS = T::BITS;
    constexpr int LOADS = KR * BITS / 8 / 64;        // 16-byte lane loads per weight row tile and round
    constexpr int FPL = 128 / BITS;                  // activations a lane converts per unit: those its 16 weight bytes meet
    constexpr int CHUNK = 4 * FPL;                   // k-values per lane load over the four k groups of a wave
    constexpr int PAR = BITS == 4 ? 2 : 1;           // int8: MFMAs per lane load (even / odd nibbles)
    constexpr int SPL = FPL / 8;                     // f16: MFMA steps per lane load
    constexpr int SUB = INT8 ? PAR * 3 : SPL * 2;    // fragments per (lane load, activation block)
    constexpr int UNITS = LOADS * MB;                // conversion units of a round
    constexpr int UPW = (UNITS + NW - 1) / NW;       // ... per wave
    constexpr int ROWS = 16 * MB;
    constexpr int NT = NW * RT * 16;                 // weight rows of a workgroup
    constexpr int SLOTS = MB * RT * 4;               // accumulator registers per thread
    static_assert(LOADS >= 1 && KR % CHUNK == 0, "a round is whole lane loads");
    if constexpr (!INT8 && !CB) static_assert(!DecH<DT>::INTERLEAVED, "operand order of the f16 decoders used here is the memory order");

    extern __shared__ __attribute__((aligned(16))) uint4 frag[];   // [LOADS][SUB][MB][64 lanes]
    __shared__ float pmax[LOADS][ROWS], psum[LOADS][ROWS];
    __shared__ float csc[ROWS];      // f16 path: 2^e per row of the round
    __shared__ int cse[ROWS];        // int8 path: e per row, INT_MIN marks a row with a non-finite activation
    __shared__ float xs[ROWS];       // row sums over the workgroup's K range (over all of K after the reduction)
    __shared__ int last_flag;
    __shared__ uint32_t cbt[16];     // codebook weights: f16 hi | f16 lo << 16 of table value * 2^cb_exp

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int ln = lane & 15, g = lane >> 4;
    const int64_t K = p.k, N = p.n, kp = p.kp;
    const int mreal = (int)p.m;
    const int nt = blockIdx.x / p.splits, ks = blockIdx.x % p.splits;
    const int64_t n0 = (int64_t)nt * NT;
    const int64_t kbeg = (int64_t)ks * p.rounds * KR;

    const __amdgpu_buffer_rsrc_t wbuf = TMAJ ? raw_buffer(p.words_tm + (n0 / 16) * p.kb64 * 256, (uint64_t)((N + 15) / 16 - n0 / 16) * (uint64_t)p.kb64 * 1024)
                                             : raw_buffer(p.words + n0 * kp, (uint64_t)(N - n0) * (uint64_t)kp * 4);
    const __amdgpu_buffer_rsrc_t abuf = raw_buffer(p.a, (uint64_t)mreal * (uint64_t)K * 4);
    const uint32_t wlane = TMAJ ? (uint32_t)(wv * RT) * (uint32_t)p.kb64 * 1024 + (uint32_t)ln * 64 + (uint32_t)g * 16
                                : (uint32_t)(wv * RT * 16 + ln) * (uint32_t)kp * 4 + (uint32_t)g * 16;

    // codebook weights: the block scales of the workgroup's rows, [row][bpr]; the table
    const __amdgpu_buffer_rsrc_t sbuf = raw_buffer(CB ? p.scales + n0 * p.bpr : p.scales, CB ? (uint64_t)(N - n0) * (uint64_t)p.bpr * 4 : 0);
    int cb_exp = 0;
    if constexpr (CB) {
        cb_exp = codebook_exp(p.codebook);
        if (tid < 16) {
            const float v = ldexpf(p.codebook[tid], cb_exp);
            const _Float16 h = (_Float16)v, l = (_Float16)(v - (float)h);
            cbt[tid] = (uint32_t)__builtin_bit_cast(uint16_t, h) | ((uint32_t)__builtin_bit_cast(uint16_t, l) << 16);
        }
        // (the first barrier of the first round orders these writes before the first look-up)
    }

    float e_scale[RT], e_zero[RT], e_bias[RT];   // epilogue operands of this lane's columns
    float tot[MB][RT][4];
#pragma unroll
    for (int b = 0; b < MB; b++)
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int i = 0; i < 4; i++) tot[b][r][i] = 0.0f;
    float rowsum = 0.0f;   // thread t < ROWS: sum of activation row t over the rounds so far

    for (int round = 0; round < p.rounds; round++) {
        const int64_t k0 = kbeg + (int64_t)round * KR;
        // ---- 1. requests: this wave's activation units first (they come from the L2 and their conversion must not
        // wait for the packed bytes behind them: loads return in order), then the packed bytes, the long pole
        // Load j of a unit covers, for every row, 64 contiguous bytes with the four lanes of the row (lane (ln, g): the
        // four values k = chunk + 16 j + 4 g ..), so neighbouring lanes consume neighbouring pieces of a line; the values a
        // lane converts are therefore not the ones its own weight bytes meet, and the conversion below writes every
        // register's digits (or halves) where the lane that multiplies them will read them.
        u32x4 xr[UPW][FPL / 4];
#pragma unroll
        for (int u = 0; u < UPW; u++) {
            const int unit = wv + u * NW;
            const int c = unit % LOADS, b = unit / LOADS;
            const int row = b * 16 + ln;
            const int64_t kk = k0 + c * CHUNK + g * 4;
#pragma unroll
            for (int j = 0; j < FPL / 4; j++) {
                // K % 8 == 0: a 16-byte piece lies wholly inside or wholly past K; past K (or past the units of the
                // round) the offset leaves the buffer and the load returns zero
                const bool ok = unit < UNITS && row < mreal && kk + j * 16 < K;
                const uint32_t off = ok ? (uint32_t)(((int64_t)row * K + kk + j * 16) * 4) : 0xFFFFFF00u;
                xr[u][j] = __builtin_amdgcn_raw_buffer_load_b128(abuf, off, 0, 0);
            }
        }
        u32x4 wq[RT][LOADS];
        const uint32_t wk = (uint32_t)(k0 * BITS / 8);
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int l = 0; l < LOADS; l++) {
                // a lane load wholly past K leaves the buffer and reads as zero (a row's bytes past K would be the next
                // row's); the f16 types require K % CHUNK == 0, so no load of theirs straddles K, and the int8 types
                // meet zero digits there
                const uint32_t off = !(k0 + l * CHUNK < K) ? 0xFFFFFF00u
                                     : TMAJ ? wlane + ((uint32_t)r * (uint32_t)p.kb64 + (wk >> 6) + l) * 1024
                                            : wlane + (uint32_t)r * 16 * (uint32_t)kp * 4 + wk + l * 64;
                wq[r][l] = __builtin_amdgcn_raw_buffer_load_b128(wbuf, off, 0, 0);
            }
        // codebook weights: the scales of the four blocks a lane load of a row covers (the four lanes of a row ask for
        // the same 16 bytes)
        u32x4 bsq[CB ? RT : 1][CB ? LOADS : 1];
        if constexpr (CB) {
#pragma unroll
            for (int r = 0; r < RT; r++)
#pragma unroll
                for (int l = 0; l < LOADS; l++) {
                    const uint32_t off = !(k0 + l * CHUNK < K) ? 0xFFFFFF00u
                                                               : (uint32_t)((wv * RT + r) * 16 + ln) * (uint32_t)p.bpr * 4 + (uint32_t)((k0 >> 5) + l * 4) * 4;
                    bsq[r][l] = __builtin_amdgcn_raw_buffer_load_b128(sbuf, off, 0, 0);
                }
        }
        __builtin_amdgcn_sched_barrier(0);

        if (round == 0) {   // requested behind the first round's operands: needed last, and loads return in order
#pragma unroll
            for (int r = 0; r < RT; r++) {
                const int64_t n = n0 + (wv * RT + r) * 16 + ln;
                const bool ok = n < N;
                e_scale[r] = CB ? ldexpf(1.0f, -cb_exp) : p.scales[ok ? n : 0];   // (block scales are applied in the loop)
                e_zero[r] = CB ? 0.0f : p.zeros[ok ? n : 0];
                e_bias[r] = p.bias ? p.bias[ok ? n : 0] : 0.0f;
            }
        }
        // ---- 2. row maxima and sums of the units
#pragma unroll
        for (int u = 0; u < UPW; u++) {
            const int unit = wv + u * NW;
            float mx = 0.0f, sm = 0.0f;
#pragma unroll
            for (int j = 0; j < FPL / 4; j++) {
                const float x0 = __uint_as_float(xr[u][j][0]), x1 = __uint_as_float(xr[u][j][1]);
                const float x2 = __uint_as_float(xr[u][j][2]), x3 = __uint_as_float(xr[u][j][3]);
                mx = fmaxf(mx, fmaxf(fmaxf(fabsf(x0), fabsf(x1)), fmaxf(fabsf(x2), fabsf(x3))));
                sm += (x0 + x1) + (x2 + x3);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            sm += __shfl_xor(sm, 16, 64);
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            sm += __shfl_xor(sm, 32, 64);
            if (unit < UNITS && g == 0) {
                pmax[unit % LOADS][(unit / LOADS) * 16 + ln] = mx;
                psum[unit % LOADS][(unit / LOADS) * 16 + ln] = sm;
            }
        }
        __syncthreads();

        // ---- 3. one scale per row and round; operand fragments
        if (tid < ROWS) {
            float mx = 0.0f, sm = 0.0f;
#pragma unroll
            for (int c = 0; c < LOADS; c++) { mx = fmaxf(mx, pmax[c][tid]); sm += psum[c][tid]; }
            rowsum += sm;
            int ex = (int)((__float_as_uint(mx) >> 23) & 0xff) - 127;
            if (INT8) {
                ex = mx == 0.0f ? 0 : ex - 21;
                // a NaN or an infinity among the row's activations shows in their sum: integer digits cannot carry it,
                // so the row's scale does (its outputs become NaN, as the float path's would be NaN or inf)
                cse[tid] = fabsf(sm) <= 3.4028234663852886e38f ? ex : INT_MIN;
            } else {
                ex = mx == 0.0f ? 0 : ex - 14;
                ex = ex < -100 ? -100 : (ex > 120 ? 120 : ex);
                csc[tid] = __uint_as_float((uint32_t)(127 + ex) << 23);
            }
        }
#pragma unroll
        for (int u = 0; u < UPW; u++) {
            const int unit = wv + u * NW;
            if (unit >= UNITS) continue;
            const int c = unit % LOADS, b = unit / LOADS;
            float mx = 0.0f;
#pragma unroll
            for (int cc = 0; cc < LOADS; cc++) mx = fmaxf(mx, pmax[cc][b * 16 + ln]);
            int ex = (int)((__float_as_uint(mx) >> 23) & 0xff) - 127;
            // register j holds the values f0 .. f0 + 3 of the unit's chunk, f0 = 16 j + 4 g: they belong to the k group
            // f0 / FPL of the row (the lane (ln, f0 / FPL) of the MFMA operand), local index f0 % FPL
            unsigned char *fbase = reinterpret_cast<unsigned char *>(frag + ((size_t)(c * SUB) * MB + b) * 64);   // fragment `sub` MB * 1024 bytes further
            if constexpr (INT8) {
                ex = mx == 0.0f ? 0 : ex - 21;
                // v = rint(x * 2^-e), |v| < 2^22.  Its balanced base-256 digits (each in [-128, 127], v = sum d_j 256^j,
                // j < 3) are the low three bytes of (v + 0x808080) ^ 0x808080.
                // Rounding by addition: x * 2^-e + 1.5 * 2^23 has the integer rint(x * 2^-e) in its low mantissa bits (two's
                // complement, |v| < 2^22), so subtracting the bits of 1.5 * 2^23 leaves v; that subtraction and the digit
                // offset are one constant.  2^-e is applied as an exact factor in two steps (e spans -148 .. 106).
                const int e1 = -ex / 2, e2 = -ex - e1;
                const float f1 = __uint_as_float((uint32_t)(127 + e1) << 23), f2 = __uint_as_float((uint32_t)(127 + e2) << 23);
#pragma unroll
                for (int j = 0; j < FPL / 4; j++) {
                    uint32_t dg[4];
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        dg[e] = (__float_as_uint(__builtin_fmaf(__uint_as_float(xr[u][j][e]) * f1, f2, 12582912.0f)) + (0x00808080u - 0x4B400000u)) ^ 0x00808080u;
                    const int f0 = j * 16 + g * 4, owner = f0 / FPL, li = f0 % FPL;
                    unsigned char *dl = fbase + (owner * 16 + ln) * 16;
                    if constexpr (PAR == 1) {
                        // bytes 4w .. 4w + 3 of the owner's lane load are k = 4w .. 4w + 3: word w = li / 4 of each plane
                        uint32_t t[4];
                        transpose4(dg[0], dg[1], dg[2], dg[3], t);
#pragma unroll
                        for (int pln = 0; pln < 3; pln++) *reinterpret_cast<uint32_t *>(dl + (size_t)pln * MB * 1024 + (li / 4) * 4) = t[pln];
                    } else {
                        // word w = li / 8 of the owner's lane load holds k = 8w .. 8w + 7, low nibbles the even, high nibbles the
                        // odd ones: these four values are elements (li % 8) / 2 and + 1 of the word's even and of its odd operand
                        const int wbyte = (li / 8) * 4 + ((li % 8) / 2);
#pragma unroll
                        for (int pln = 0; pln < 3; pln++) {
                            const uint32_t sel = 0x0c0c0400u + 0x0101u * pln;   // byte `pln` of the second, then of the first operand
                            const uint32_t ev = __builtin_amdgcn_perm(dg[2], dg[0], sel), od = __builtin_amdgcn_perm(dg[3], dg[1], sel);
                            *reinterpret_cast<uint16_t *>(dl + (size_t)pln * MB * 1024 + wbyte) = (uint16_t)ev;
                            *reinterpret_cast<uint16_t *>(dl + (size_t)(3 + pln) * MB * 1024 + wbyte) = (uint16_t)od;
                        }
                    }
                }
            } else {
                ex = mx == 0.0f ? 0 : ex - 14;
                ex = ex < -100 ? -100 : (ex > 120 ? 120 : ex);
                const float inv = __uint_as_float((uint32_t)(127 - ex) << 23);
#pragma unroll
                for (int j = 0; j < FPL / 4; j++) {
                    typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
                    f16x4 hi, lo;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float v = __uint_as_float(xr[u][j][e]) * inv;
                        const _Float16 h = (_Float16)v;
                        hi[e] = h;
                        lo[e] = (_Float16)(v - (float)h);
                    }
                    // MFMA step li / 8 of the owner's lane load, halves (li % 8) .. + 3 of its hi and of its lo fragment
                    // (codebook weights: a step is one block of 32 values, the owner holds its values 8 * owner ..)
                    const int f0 = j * 16 + g * 4;
                    const int owner = CB ? (f0 % 32) / 8 : f0 / FPL, step = CB ? f0 / 32 : (f0 % FPL) / 8;
                    unsigned char *dl = fbase + (owner * 16 + ln) * 16 + (f0 % 8) * 2;
                    *reinterpret_cast<f16x4 *>(dl + (size_t)(step * 2) * MB * 1024) = hi;
                    *reinterpret_cast<f16x4 *>(dl + (size_t)(step * 2 + 1) * MB * 1024) = lo;
                }
            }
        }
        __syncthreads();

        // ---- 4. the matrix cores.  The fragments of the whole round are walked in one fixed order through a small
        // ring of registers: fragment i + DEPTH is requested before fragment i is multiplied, so the LDS latency is paid
        // once per round and not once per MFMA.
        const uint4 *frd = frag + lane;
        if constexpr (INT8) {
            constexpr int ITEMS = LOADS * PAR * 3 * MB;   // (lane load, parity, plane, activation block), block fastest
            constexpr int DEPTH = ITEMS < 6 ? ITEMS : 6;
            i32x4 acc[3][MB][RT];
#pragma unroll
            for (int j = 0; j < 3; j++)
#pragma unroll
                for (int b = 0; b < MB; b++)
#pragma unroll
                    for (int r = 0; r < RT; r++) acc[j][b][r] = i32x4{0, 0, 0, 0};
            uint4 ring[DEPTH];
#pragma unroll
            for (int i = 0; i < DEPTH; i++) ring[i] = frd[i * 64];   // item i lives at fragment index i: ((l*SUB + q*3 + j)*MB + b)
            i32x4 bw[RT];
#pragma unroll
            for (int i = 0; i < ITEMS; i++) {
                const int b = i % MB, j = (i / MB) % 3, q = (i / (MB * 3)) % PAR, l = i / (MB * 3 * PAR);
                if (b == 0 && j == 0) {
#pragma unroll
                    for (int r = 0; r < RT; r++) bw[r] = int8_operand<DT>(wq[r][l], q);
                }
                const i32x4 av = __builtin_bit_cast(i32x4, ring[i % DEPTH]);
                if (i + DEPTH < ITEMS) ring[i % DEPTH] = frd[(i + DEPTH) * 64];
#pragma unroll
                for (int r = 0; r < RT; r++) acc[j][b][r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bw[r], acc[j][b][r], 0, 0, 0);
            }
            // acc[.][b][r][i]: activation row b*16 + g*4 + i, weight row (wv*RT + r)*16 + ln; |plane sum| <= KR * 2^14 < 2^24
#pragma unroll
            for (int b = 0; b < MB; b++) {
                const int4 e4 = *reinterpret_cast<const int4 *>(&cse[b * 16 + g * 4]);
                const int ee[4] = {e4.x, e4.y, e4.z, e4.w};
#pragma unroll
                for (int r = 0; r < RT; r++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float v = fmaf(fmaf((float)acc[2][b][r][i], 256.0f, (float)acc[1][b][r][i]), 256.0f, (float)acc[0][b][r][i]);
                        tot[b][r][i] += ee[i] == INT_MIN ? __uint_as_float(0x7fc00000u) : ldexpf(v, ee[i]);
                    }
            }
        } else if constexpr (CB) {
            // A lane load holds the four words of ONE block of its row, lane (ln, g) that of block 4 l + g; an MFMA step
            // must be one block over all four k groups, so the words are transposed across the groups: afterwards word s
            // of lane (ln, g) is word g (values 8 g .. 8 g + 7) of block 4 l + s.
#pragma unroll
            for (int r = 0; r < RT; r++)
#pragma unroll
                for (int l = 0; l < LOADS; l++) {
                    // rows 2, 3 of the first operand <-> rows 0, 1 of the second; then odd rows <-> even rows (a row: 16 lanes)
                    const auto s02 = __builtin_amdgcn_permlane32_swap(wq[r][l][0], wq[r][l][2], false, false);
                    const auto s13 = __builtin_amdgcn_permlane32_swap(wq[r][l][1], wq[r][l][3], false, false);
                    const auto t01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
                    const auto t23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
                    wq[r][l] = u32x4{t01[0], t01[1], t23[0], t23[1]};
                }
            constexpr int ITEMS = LOADS * SPL * MB;       // (lane load, block, activation block): a hi and a lo fragment each
            constexpr int DEPTH = ITEMS < 3 ? ITEMS : 3;
            f32x4 acc[MB][RT];
#pragma unroll
            for (int b = 0; b < MB; b++)
#pragma unroll
                for (int r = 0; r < RT; r++) acc[b][r] = f32x4{0.f, 0.f, 0.f, 0.f};
            uint4 rhi[DEPTH], rlo[DEPTH];
#pragma unroll
            for (int i = 0; i < DEPTH; i++) {
                const int b = i % MB, ls = i / MB;
                rhi[i] = frd[((ls * 2) * MB + b) * 64];
                rlo[i] = frd[((ls * 2 + 1) * MB + b) * 64];
            }
            f16x8 bwh[RT], bwl[RT];
            float bsc[RT];
#pragma unroll
            for (int i = 0; i < ITEMS; i++) {
                const int b = i % MB, ls = i / MB, sidx = ls % SPL, l = ls / SPL;
                if (b == 0) {
#pragma unroll
                    for (int r = 0; r < RT; r++) {
                        const uint32_t w = wq[r][l][sidx];
                        uint32_t d[8];
                        d[0] = cbt[w & 15u];
#pragma unroll
                        for (int j = 1; j < 8; j++) d[j] = cbt[(w >> (4 * j)) & 15u];
                        uint32_t h4[4], l4[4];
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            h4[j] = __builtin_amdgcn_perm(d[2 * j + 1], d[2 * j], 0x05040100u);   // low halves: hi parts
                            l4[j] = __builtin_amdgcn_perm(d[2 * j + 1], d[2 * j], 0x07060302u);   // high halves: lo parts
                        }
                        bwh[r] = __builtin_bit_cast(f16x8, u32x4{h4[0], h4[1], h4[2], h4[3]});
                        bwl[r] = __builtin_bit_cast(f16x8, u32x4{l4[0], l4[1], l4[2], l4[3]});
                        bsc[r] = __uint_as_float(bsq[r][l][sidx]);
                    }
                }
                const f16x8 ahi = __builtin_bit_cast(f16x8, rhi[i % DEPTH]);
                const f16x8 alo = __builtin_bit_cast(f16x8, rlo[i % DEPTH]);
                if (i + DEPTH < ITEMS) {
                    const int nb = (i + DEPTH) % MB, nls = (i + DEPTH) / MB;
                    rhi[i % DEPTH] = frd[((nls * 2) * MB + nb) * 64];
                    rlo[i % DEPTH] = frd[((nls * 2 + 1) * MB + nb) * 64];
                }
#pragma unroll
                for (int r = 0; r < RT; r++) {
                    // the block's sum (the lo x lo product is below 2^-22 of the terms), then the block scale
                    f32x4 blk = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, bwh[r], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    blk = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, bwl[r], blk, 0, 0, 0);
                    blk = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, bwh[r], blk, 0, 0, 0);
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[b][r][e] = fmaf(bsc[r], blk[e], acc[b][r][e]);
                }
            }
#pragma unroll
            for (int b = 0; b < MB; b++) {
                const float4 c4 = *reinterpret_cast<const float4 *>(&csc[b * 16 + g * 4]);
                const float cc[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
                for (int r = 0; r < RT; r++)
#pragma unroll
                    for (int i = 0; i < 4; i++) tot[b][r][i] = fmaf(acc[b][r][i], cc[i], tot[b][r][i]);
            }
        } else {
            using D = DecH<DT>;
            constexpr int ITEMS = LOADS * SPL * MB;       // (lane load, step, activation block): a hi and a lo fragment each
            constexpr int DEPTH = ITEMS < 3 ? ITEMS : 3;
            f32x4 acc[MB][RT];
#pragma unroll
            for (int b = 0; b < MB; b++)
#pragma unroll
                for (int r = 0; r < RT; r++) acc[b][r] = f32x4{0.f, 0.f, 0.f, 0.f};
            // item i = ((l*SPL + s)*MB + b): hi at fragment ((l*SUB + 2s)*MB + b), lo MB fragments further
            uint4 rhi[DEPTH], rlo[DEPTH];
#pragma unroll
            for (int i = 0; i < DEPTH; i++) {
                const int b = i % MB, ls = i / MB;
                rhi[i] = frd[((ls * 2) * MB + b) * 64];
                rlo[i] = frd[((ls * 2 + 1) * MB + b) * 64];
            }
            f16x8 bw[RT];
#pragma unroll
            for (int i = 0; i < ITEMS; i++) {
                const int b = i % MB, ls = i / MB, sidx = ls % SPL, l = ls / SPL;
                if (b == 0) {
#pragma unroll
                    for (int r = 0; r < RT; r++) {
                        const uint32_t w4[4] = {wq[r][l][0], wq[r][l][1], wq[r][l][2], wq[r][l][3]};
                        bw[r] = D::step(&w4[sidx * D::WPS]);
                    }
                }
                const f16x8 ahi = __builtin_bit_cast(f16x8, rhi[i % DEPTH]);
                const f16x8 alo = __builtin_bit_cast(f16x8, rlo[i % DEPTH]);
                if (i + DEPTH < ITEMS) {
                    const int nb = (i + DEPTH) % MB, nls = (i + DEPTH) / MB;
                    rhi[i % DEPTH] = frd[((nls * 2) * MB + nb) * 64];
                    rlo[i % DEPTH] = frd[((nls * 2 + 1) * MB + nb) * 64];
                }
#pragma unroll
                for (int r = 0; r < RT; r++) {
                    acc[b][r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, bw[r], acc[b][r], 0, 0, 0);
                    acc[b][r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, bw[r], acc[b][r], 0, 0, 0);
                }
            }
#pragma unroll
            for (int b = 0; b < MB; b++) {
                const float4 c4 = *reinterpret_cast<const float4 *>(&csc[b * 16 + g * 4]);
                const float cc[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
                for (int r = 0; r < RT; r++)
#pragma unroll
                    for (int i = 0; i < 4; i++) tot[b][r][i] = fmaf(acc[b][r][i], cc[i], tot[b][r][i]);
            }
        }
        // (the next round writes pmax / psum before its first barrier and fragments, csc / cse after it: by then every
        // wave has left this round's MFMA loop and read its scales)
    }

    // ---- split K: partials out, count, and the last workgroup of the column tile adds them in split order
    if (p.splits > 1) {
        constexpr int WGF = SLOTS * NW * 64 + ROWS;   // floats a workgroup leaves
        float *mine = p.part + ((size_t)ks * p.ntiles + nt) * WGF;
#pragma unroll
        for (int b = 0; b < MB; b++)
#pragma unroll
            for (int r = 0; r < RT; r++)
#pragma unroll
                for (int i = 0; i < 4; i++) agent_store(mine + ((b * RT + r) * 4 + i) * (NW * 64) + tid, tot[b][r][i]);
        if (tid < ROWS) agent_store(mine + SLOTS * NW * 64 + tid, rowsum);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);   // every store of this wave has been acknowledged
        __syncthreads();
        if (tid == 0) {
            const uint32_t before = __hip_atomic_fetch_add(p.count + nt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_flag = before == (uint32_t)p.splits - 1 ? 1 : 0;
        }
        __syncthreads();
        if (!last_flag) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (tid == 0) __hip_atomic_store(p.count + nt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
#pragma unroll
        for (int b = 0; b < MB; b++)
#pragma unroll
            for (int r = 0; r < RT; r++)
#pragma unroll
                for (int i = 0; i < 4; i++) tot[b][r][i] = 0.0f;
        rowsum = 0.0f;
        // several splits' registers are requested before the first is added (the adds stay in split order)
        constexpr int BATCH = SLOTS >= 16 ? 2 : (SLOTS >= 8 ? 4 : 8);
        for (int s0 = 0; s0 < p.splits; s0 += BATCH) {
            float v[BATCH][SLOTS], rs[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; j++) {
                const int sj = s0 + j < p.splits ? s0 + j : p.splits - 1;   // (past the end: a valid address, value unused)
                const float *theirs = p.part + ((size_t)sj * p.ntiles + nt) * WGF;
#pragma unroll
                for (int q = 0; q < SLOTS; q++) v[j][q] = agent_load(theirs + q * (NW * 64) + tid);
                rs[j] = agent_load(theirs + SLOTS * NW * 64 + (tid < ROWS ? tid : 0));
            }
#pragma unroll
            for (int j = 0; j < BATCH; j++) {
                if (s0 + j < p.splits) {
#pragma unroll
                    for (int b = 0; b < MB; b++)
#pragma unroll
                        for (int r = 0; r < RT; r++)
#pragma unroll
                            for (int i = 0; i < 4; i++) tot[b][r][i] += v[j][(b * RT + r) * 4 + i];
                    rowsum += rs[j];
                }
            }
        }
    }
    if (tid < ROWS) xs[tid] = rowsum;
    __syncthreads();

    // ---- epilogue: lane (ln, g) holds activation rows b*16 + g*4 + i of weight row (column) n
    float res[MB][RT][4];
    if (p.sum_out) {   // the residual values are requested together, before the first store
#pragma unroll
        for (int b = 0; b < MB; b++)
#pragma unroll
            for (int r = 0; r < RT; r++) {
                const int64_t n = n0 + (wv * RT + r) * 16 + ln;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int m = b * 16 + g * 4 + i;
                    const bool ok = m < mreal && n < N;
                    res[b][r][i] = p.residual[ok ? (int64_t)m * N + n : 0];
                }
            }
    }
#pragma unroll
    for (int b = 0; b < MB; b++) {
        const float4 x4 = *reinterpret_cast<const float4 *>(&xs[b * 16 + g * 4]);
        const float xx[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
        for (int r = 0; r < RT; r++) {
            const int64_t n = n0 + (wv * RT + r) * 16 + ln;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float dot = tot[b][r][i] * T::POST;
                v[i] = CB ? dot * e_scale[r] : dot * e_scale[r] + e_zero[r] * xx[i];
                if (p.bias) v[i] = v[i] + e_bias[r];
                v[i] = fnn_activation(v[i], p.act);
            }
            if (n < N) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int m = b * 16 + g * 4 + i;
                    if (m < mreal) {
                        const int64_t o = (int64_t)m * N + n;
                        p.out[o] = v[i];
                        if (p.sum_out) p.sum_out[o] = v[i] + res[b][r][i];
                    }
                }
            }
        }
    }
}

template <int DT, int MB, int RT, int KR>
size_t stream_lds_bytes()
{
    using T = StreamType<DT>;
    constexpr int LOADS = KR * T::BITS / 8 / 64, FPL = 128 / T::BITS;
    constexpr int SUB = T::INT8 ? (T::BITS == 4 ? 2 : 1) * 3 : (FPL / 8) * 2;
    return (size_t)LOADS * SUB * MB * 64 * 16;
}

template <int DT, int MB, int RT, int KR, bool TMAJ = false>
hipError_t launch_stream(const StreamArgs &p, hipStream_t s)
{
    if constexpr (!TMAJ) {
        if (p.words_tm) return launch_stream<DT, MB, RT, KR, true>(p, s);
    }
    static std::atomic<uint64_t> raised{0};
    const size_t lds = stream_lds_bytes<DT, MB, RT, KR>();
    if (lds > 48 * 1024) {
        hipError_t e = fnn_raise_lds_limit(raised, (const void *)qgemm_stream_kernel<DT, MB, RT, KR, TMAJ>, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((qgemm_stream_kernel<DT, MB, RT, KR, TMAJ>), dim3((unsigned)(p.ntiles * p.splits)), dim3(NW * 64), lds, s, p);
    return hipGetLastError();
}

template <int DT, int MB>
hipError_t launch_mb(const StreamPlan &pl, const StreamArgs &p, hipStream_t s)
{
    using T = StreamType<DT>;
    constexpr int kTiles = T::INT8 ? 4 : (DT == FNN_DT_I4CB ? 6 : 8);   // MB * RT accumulator tiles (x 3 planes on the int8 path) that fit the registers
    if (pl.rt == 2) {
        if constexpr (MB * 2 <= kTiles) {
            if (pl.kr == 512) return launch_stream<DT, MB, 2, 512>(p, s);
            return launch_stream<DT, MB, 2, 256>(p, s);
        } else {
            return hipErrorInvalidValue;
        }
    }
    if (pl.kr == 512) return launch_stream<DT, MB, 1, 512>(p, s);
    return launch_stream<DT, MB, 1, 256>(p, s);
}

template <int DT>
hipError_t launch_dt(const StreamPlan &pl, const StreamArgs &p, hipStream_t s)
{
    switch (pl.mb) {   // (three and four blocks measured slower than the tiled path for every per-channel type: built for the codebook type only)
    case 1: return launch_mb<DT, 1>(pl, p, s);
    case 2: return launch_mb<DT, 2>(pl, p, s);
    case 3: if constexpr (DT == FNN_DT_I4CB) return launch_mb<DT, 3>(pl, p, s); else return hipErrorInvalidValue;
    case 4: if constexpr (DT == FNN_DT_I4CB) return launch_mb<DT, 4>(pl, p, s); else return hipErrorInvalidValue;
    default: return hipErrorInvalidValue;
    }
}

}  // namespace
