// Bandwidth-bound quantised GEMV on the int8 matrix cores (M <= 16 activation rows; I8, I4 and U4 weights) for gfx950.
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
// Work split (the organisation of the f16 GEMV kernel): one workgroup = 16 weight rows x all of K; wave w owns the K
// slices w, w + NW, ...; it requests its activation slice and its packed bytes, converts the activations into digit
// fragments in its own LDS area while the bytes are on their way, multiplies, and the waves' partial sums meet in LDS
// in a fixed order for the fused affine / bias / activation epilogue.  All global reads are raw buffer loads: an
// address past the end of the weight tile, of K or of the activation rows reads as zero, so no lane clamps or masks.
// 5 <= M <= 16: the activation rows are taken in chunks of four against the same packed bytes, which stay in
// registers: chunk c + 1 is requested while chunk c is converted and multiplied.  Each further chunk costs about
// 2.7 us (N = 11008, K = 4096: M = 4 7.7 us, M = 5..8 10.1-10.7 against 11.9 for the f16 kernel, M = 12 14.0 against
// 13.9, M = 16 16.2 against 14.2), so M <= 8 is the default range.
// Algorithmic bytes per launch: N*K*bits/8 + side tables + 4*M*(K+N).
#include "mfma.h"

#include <climits>

namespace {

struct DotArgs {
    const uint32_t *words;
    const float *scales, *zeros, *a, *bias;
    float *out;
    int64_t m, n, k, kp;
    int act;
    int nslice;   // slices of 512 k-values covering K
    int ntiles;   // row tiles of 16
    const uint32_t *words_tm;   // non-null: the same words in blocks of 16 rows x 64 bytes, [row block][k block][row][64 bytes]
    int64_t kb64;               // ... k blocks per row
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

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Raw buffer descriptor over [base, base + bytes): loads past the end return zero instead of faulting, so no lane
// clamps or masks its address (rows past N, slices past K, activation rows past M).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t raw_buffer(const void *base, uint64_t bytes)
{
    const uint32_t n = bytes > 0xffffffffull ? 0xffffffffu : (uint32_t)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n, 0x00020000);
}

// MM activation rows per chunk (1, 2, 4), MC chunks (MC > 1 only with MM = 4): M <= MM * MC
// TMAJ: the packed words come from the tile-major copy (a wave load = the contiguous KB of one 16-row x 64-byte block)
template <int DT, int MM, int NW, int RT, int MC = 1, bool TMAJ = false>
__global__ void __launch_bounds__(NW * 64) qgemv_i8dot_kernel(DotArgs p)
{
    using W = Int8Op<DT>;
    constexpr int LOADS = W::LOADS, PER = W::PER_LOAD;
    constexpr int R4 = 4 * MM;               // digit rows per step: row m*4 + digit, digit 0 the most significant
    constexpr bool FOUR_BIT = PER == 2;
    constexpr int MT = MM * MC;              // activation rows in all
    constexpr int OUTS = RT * MT * 16;       // outputs of the workgroup
    constexpr int OPT = (OUTS + NW * 64 - 1) / (NW * 64);   // ... per thread in the epilogue
    static_assert(MC == 1 || MM == 4, "chunks are four rows");

    // per wave: [step][R4 rows][4 groups] 16-byte operand fragments of the slice it is working on
    extern __shared__ __attribute__((aligned(16))) uint4 lds_dyn[];
    __shared__ float red[NW][RT][MT][16];
    __shared__ float xred[NW][MT];

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int ln = lane & 15, g = lane >> 4;
    const int64_t K = p.k, N = p.n, kp = p.kp;
    const int mreal = (int)p.m;
    const int64_t n0 = (int64_t)blockIdx.x * (16 * RT);
    uint4 *frag = lds_dyn + wv * (NSTEP * R4 * 4);

    // the tile's 16 weight rows (rows past N read as zero) and the activation rows (rows past M read as zero)
    const __amdgpu_buffer_rsrc_t wbuf = TMAJ ? raw_buffer(p.words_tm + (n0 / 16) * p.kb64 * 256, (uint64_t)((N + 15) / 16 - n0 / 16) * (uint64_t)p.kb64 * 1024)
                                             : raw_buffer(p.words + n0 * kp, (uint64_t)(N - n0) * (uint64_t)kp * 4);
    // one descriptor over the M activation rows: row m starts at byte m*K*4 (below 4 GiB, checked on the host)
    const __amdgpu_buffer_rsrc_t abuf = raw_buffer(p.a, (uint64_t)mreal * (uint64_t)K * 4);
    const uint32_t arow = (uint32_t)K * 4;
    const uint32_t wlane = TMAJ ? (uint32_t)ln * 64 + (uint32_t)g * 16
                                : (uint32_t)ln * (uint32_t)kp * 4 + (uint32_t)g * 16;   // 16 rows of kp words: below 4 GiB (checked on the host)

    // the thread that finishes output (row tile r, m, column c): tid = (r*MM + m)*16 + c; its epilogue operands are
    // requested first
    int e_r[OPT], e_m[OPT], e_c[OPT];
    int64_t e_n[OPT];
    bool finisher[OPT];
    float e_scale[OPT], e_zero[OPT], e_bias[OPT];
#pragma unroll
    for (int o = 0; o < OPT; o++) {
        const int idx = tid + o * NW * 64;
        e_r[o] = idx / (MT * 16); e_m[o] = (idx >> 4) % MT; e_c[o] = idx & 15;
        e_n[o] = n0 + e_r[o] * 16 + e_c[o];
        finisher[o] = idx < OUTS && e_m[o] < mreal && e_n[o] < N;
        e_scale[o] = e_zero[o] = e_bias[o] = 0.0f;
        if (finisher[o]) {
            e_scale[o] = p.scales[e_n[o]];
            e_zero[o] = p.zeros[e_n[o]];
            e_bias[o] = p.bias ? p.bias[e_n[o]] : 0.0f;
        }
    }

    // operand fragment this lane reads at a step: operand row ln = activation row ln / 4, digit ln % 4 (rows past M: row 0)
    const uint4 *frd = frag + ((ln >> 2) < MM ? ln : 0) * 4 + g;

    float tot[MC][RT];     // lanes with g < MM: partial dot of (activation row c*MM + g, weight row n0 + r*16 + ln)
#pragma unroll
    for (int c = 0; c < MC; c++)
#pragma unroll
        for (int r = 0; r < RT; r++) tot[c][r] = 0.0f;
    float xsum[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) xsum[m] = 0.0f;

    for (int slice = wv; slice < p.nslice; slice += NW) {
        // ---- requests: this lane's 8 activations per row (oldest: their conversion does not wait for packed bytes),
        // then the slice's packed bytes; lane (n, g), load l: words [slice*SL*bits/32 + l*16 + g*4, +4) of row n.
        // Bytes past the end of a row belong to the next row or read as zero: their activation digits are zero.
        u32x4 xa[MM][2], xn[MM][2];
        // (a lane's 8 values lie wholly inside or wholly past K: K % 8 == 0; past K the offset leaves the buffer and
        // the load returns zero instead of the next row's values)
        const bool past_k = (int64_t)slice * SL + lane * 8 >= K;
        const uint32_t aoff = past_k ? 0xFFFFFF00u : ((uint32_t)slice * SL + (uint32_t)lane * 8) * 4;
        const uint32_t astep = past_k ? 0u : arow;
#pragma unroll
        for (int m = 0; m < MM; m++) {
            xa[m][0] = __builtin_amdgcn_raw_buffer_load_b128(abuf, aoff + (uint32_t)m * astep, 0, 0);
            xa[m][1] = __builtin_amdgcn_raw_buffer_load_b128(abuf, aoff + (uint32_t)m * astep + 16, 0, 0);
        }
        u32x4 wq[RT][LOADS];
        // (tile-major: k block slice * LOADS + l of row block r; a slice past K lands in the next row block or past the
        // buffer, and its activation digits are zero)
        const uint32_t woff = TMAJ ? wlane + (uint32_t)slice * (LOADS * 1024) : wlane + (uint32_t)slice * (LOADS * 64);
        const uint32_t rstep = TMAJ ? (uint32_t)p.kb64 * 1024 : 16 * (uint32_t)kp * 4, lstep = TMAJ ? 1024 : 64;
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int l = 0; l < LOADS; l++)
                wq[r][l] = __builtin_amdgcn_raw_buffer_load_b128(wbuf, woff + (uint32_t)r * rstep + l * lstep, 0, 0);
        __builtin_amdgcn_sched_barrier(0);

#pragma unroll
        for (int ck = 0; ck < MC; ck++) {
            if (ck + 1 < MC) {   // the next chunk's rows are on their way while this one is converted and multiplied
#pragma unroll
                for (int m = 0; m < MM; m++) {
                    const uint32_t ro = aoff + (uint32_t)((ck + 1) * MM + m) * astep;
                    xn[m][0] = __builtin_amdgcn_raw_buffer_load_b128(abuf, ro, 0, 0);
                    xn[m][1] = __builtin_amdgcn_raw_buffer_load_b128(abuf, ro + 16, 0, 0);
                }
            }
            // ---- activation slice -> four digit rows per activation row in this wave's LDS area
            int cs[MM];      // slice exponent per row; INT_MIN marks a slice with a non-finite activation
#pragma unroll
            for (int m = 0; m < MM; m++) {
                float x[8];
#pragma unroll
                for (int j = 0; j < 4; j++) { x[j] = __uint_as_float(xa[m][0][j]); x[4 + j] = __uint_as_float(xa[m][1][j]); }
                float mx = fmaxf(fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3]))),
                                 fmaxf(fmaxf(fabsf(x[4]), fabsf(x[5])), fmaxf(fabsf(x[6]), fabsf(x[7]))));
                mx = wave_max_uniform(mx);
                const float ssum = wave_sum_uniform(((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7])));
                xsum[ck * MM + m] += ssum;
                // power of two e with max*2^-e in [2^29, 2^30): |v| < 2^30, so the top digit stays within +-64
                int ex = (int)((__float_as_uint(mx) >> 23) & 0xff) - 127 - 29;
                if (mx == 0.0f) ex = 0;
                // (-156 for subnormal maxima up to 98: applied with ldexp, whose exponent argument has no such limits
                // as a power-of-two factor would)
                // a NaN or an infinity among the slice's activations shows in their sum: the integer digits cannot carry
                // it, so the slice scale does (the row's outputs become NaN, as the float path's would be NaN or inf)
                const bool finite = fabsf(ssum) <= 3.4028234663852886e38f;
                cs[m] = finite ? ex : INT_MIN;
                // v = trunc(x * 2^-e), |v| < 2^30.  Its balanced base-256 digits (each in [-128, 127], v = sum d_j 256^j)
                // are the bytes of (v + 0x80808080) ^ 0x80808080: adding 128 to every digit gives the plain unsigned
                // base-256 form, flipping the top bit of every byte subtracts the 128 again.  Byte 3 is the top digit.
                uint32_t dg[8];
#pragma unroll
                for (int j = 0; j < 8; j++) dg[j] = ((uint32_t)(int)ldexpf(x[j], -ex) + 0x80808080u) ^ 0x80808080u;
                // digit rows: byte `d` of four activations side by side (4x4 byte transposes with v_perm_b32; selector
                // bytes 0-3 pick from the second operand, 4-7 from the first)
                auto transpose4 = [](uint32_t a, uint32_t b, uint32_t c, uint32_t d, uint32_t (&o)[4]) {
                    const uint32_t ab_lo = __builtin_amdgcn_perm(b, a, 0x05010400u);   // a0 b0 a1 b1
                    const uint32_t ab_hi = __builtin_amdgcn_perm(b, a, 0x07030602u);   // a2 b2 a3 b3
                    const uint32_t cd_lo = __builtin_amdgcn_perm(d, c, 0x05010400u);
                    const uint32_t cd_hi = __builtin_amdgcn_perm(d, c, 0x07030602u);
                    o[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);           // a0 b0 c0 d0: lowest digit
                    o[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
                    o[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
                    o[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);           // a3 b3 c3 d3: top digit
                };
                uint32_t t0[4], t1[4];
                if constexpr (FOUR_BIT) {
                    // word `lane` of the slice: load lane / 16, group (lane / 4) % 4, word lane % 4 of the lane's 16 bytes;
                    // even nibbles belong to step 2l, odd nibbles to step 2l + 1
                    transpose4(dg[0], dg[2], dg[4], dg[6], t0);
                    transpose4(dg[1], dg[3], dg[5], dg[7], t1);
                    uint32_t *f32w = reinterpret_cast<uint32_t *>(frag);
                    const int base_e = ((2 * (lane >> 4) * R4 + m * 4) * 4 + ((lane >> 2) & 3)) * 4 + (lane & 3);   // 4-byte words
#pragma unroll
                    for (int d = 0; d < 4; d++) {
                        f32w[base_e + d * 16] = t0[3 - d];
                        f32w[base_e + R4 * 16 + d * 16] = t1[3 - d];
                    }
                } else {
                    // bytes [lane*8, +8) of the slice: step lane / 8, group (lane / 2) % 4, half lane % 2 of the 16 bytes
                    transpose4(dg[0], dg[1], dg[2], dg[3], t0);
                    transpose4(dg[4], dg[5], dg[6], dg[7], t1);
                    uint2 *f64w = reinterpret_cast<uint2 *>(frag);
                    const int base = (((lane >> 3) * R4 + m * 4) * 4 + ((lane >> 1) & 3)) * 2 + (lane & 1);         // 8-byte words
#pragma unroll
                    for (int d = 0; d < 4; d++) f64w[base + d * 8] = uint2{t0[3 - d], t1[3 - d]};
                }
            }
            // only this wave reads the fragments it wrote, and the LDS serves a wave's requests in order
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_sched_barrier(0);

            // ---- integer MFMA over the slice
            i32x4 acc[RT];
#pragma unroll
            for (int r = 0; r < RT; r++) acc[r] = i32x4{0, 0, 0, 0};
#pragma unroll
            for (int l = 0; l < LOADS; l++)
#pragma unroll
                for (int q = 0; q < PER; q++) {
                    const i32x4 av = __builtin_bit_cast(i32x4, frd[(l * PER + q) * R4 * 4]);
#pragma unroll
                    for (int r = 0; r < RT; r++) {
                        const uint32_t w4[4] = {wq[r][l][0], wq[r][l][1], wq[r][l][2], wq[r][l][3]};
                        acc[r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, W::op(w4, q), acc[r], 0, 0, 0);
                    }
                }
            // acc[i] = operand row g*4 + i = digit i of activation row g
            int csm = cs[0];
#pragma unroll
            for (int m = 1; m < MM; m++) csm = g == m ? cs[m] : csm;
#pragma unroll
            for (int r = 0; r < RT; r++) {
                const float hi = fmaf((float)acc[r][0], 256.0f, (float)acc[r][1]), lo = fmaf((float)acc[r][2], 256.0f, (float)acc[r][3]);
                tot[ck][r] += csm == INT_MIN ? __uint_as_float(0x7fc00000u) : ldexpf(fmaf(hi, 65536.0f, lo), csm);
            }
            __builtin_amdgcn_wave_barrier();   // the wave's LDS area is rewritten by its next chunk or slice
            if (ck + 1 < MC) {
#pragma unroll
                for (int m = 0; m < MM; m++) { xa[m][0] = xn[m][0]; xa[m][1] = xn[m][1]; }
            }
        }
    }

    // ---- the waves' partial sums in a fixed order, fused epilogue
    if (g < MM) {
#pragma unroll
        for (int c = 0; c < MC; c++)
#pragma unroll
            for (int r = 0; r < RT; r++) red[wv][r][c * MM + g][ln] = tot[c][r];
    }
    if (lane == 0) {
#pragma unroll
        for (int m = 0; m < MT; m++) xred[wv][m] = xsum[m];
    }
    __syncthreads();
#pragma unroll
    for (int o = 0; o < OPT; o++) {
        if (finisher[o]) {
            float dot = 0.0f, xs = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; w++) { dot += red[w][e_r[o]][e_m[o]][e_c[o]]; xs += xred[w][e_m[o]]; }
            dot *= W::POST;
            const float v = dot * e_scale[o] + e_zero[o] * xs;
            p.out[(int64_t)e_m[o] * N + e_n[o]] = fnn_activation(p.bias ? v + e_bias[o] : v, p.act);
        }
    }
}

template <int DT, int MM, int NW, int RT, int MC = 1>
hipError_t launch_rt(DotArgs p, hipStream_t s, bool *handled)
{
    p.nslice = (int)((p.k + SL - 1) / SL);
    p.ntiles = (int)((p.n + 16 * RT - 1) / (16 * RT));
    const size_t lds = (size_t)NW * NSTEP * 4 * MM * 4 * 16;    // 2 KiB per wave and activation row of a chunk
    if (p.words_tm) hipLaunchKernelGGL((qgemv_i8dot_kernel<DT, MM, NW, RT, MC, true>), dim3((unsigned)p.ntiles), dim3(NW * 64), lds, s, p);
    else hipLaunchKernelGGL((qgemv_i8dot_kernel<DT, MM, NW, RT, MC>), dim3((unsigned)p.ntiles), dim3(NW * 64), lds, s, p);
    *handled = true;
    return hipGetLastError();
}

template <int DT, int MM, int NW, int MC = 1>
hipError_t launch_nw(const DotArgs &p, int rt, hipStream_t s, bool *handled)
{
    if (rt == 3 && (MC > 1 || MM * 48 <= NW * 64)) return launch_rt<DT, MM, NW, 3, MC>(p, s, handled);
    if (rt >= 2 && (MC > 1 || MM * 32 <= NW * 64)) return launch_rt<DT, MM, NW, 2, MC>(p, s, handled);
    return launch_rt<DT, MM, NW, 1, MC>(p, s, handled);
}

template <int DT>
hipError_t launch_dt(const DotArgs &p, int rt, hipStream_t s, bool *handled)
{
    const bool shortk = p.k <= 4 * SL;   // K <= 2048: four waves, so that no wave idles
    if (p.m > 12) return shortk ? launch_nw<DT, 4, 4, 4>(p, rt, s, handled) : launch_nw<DT, 4, 8, 4>(p, rt, s, handled);
    if (p.m > 8) return shortk ? launch_nw<DT, 4, 4, 3>(p, rt, s, handled) : launch_nw<DT, 4, 8, 3>(p, rt, s, handled);
    if (p.m > 4) return shortk ? launch_nw<DT, 4, 4, 2>(p, rt, s, handled) : launch_nw<DT, 4, 8, 2>(p, rt, s, handled);
    const int mm = p.m <= 1 ? 1 : (p.m <= 2 ? 2 : 4);
    if (mm == 1) return shortk ? launch_nw<DT, 1, 4>(p, rt, s, handled) : launch_nw<DT, 1, 8>(p, rt, s, handled);
    if (mm == 2) return shortk ? launch_nw<DT, 2, 4>(p, rt, s, handled) : launch_nw<DT, 2, 8>(p, rt, s, handled);
    return shortk ? launch_nw<DT, 4, 4>(p, rt, s, handled) : launch_nw<DT, 4, 8>(p, rt, s, handled);
}

// row-major packed words -> blocks of 16 rows x 64 bytes; one thread per 16-byte piece of the destination
__global__ void __launch_bounds__(256) tile_major_kernel(const uint32_t *src, int64_t rows, int64_t kp, int64_t kb64, u32x4 *dst)
{
    const int64_t total = (rows + 15) / 16 * kb64 * 64;   // 16-byte pieces
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t blk = i >> 6, rb = blk / kb64, kb = blk % kb64;
        const int ln = (int)((i >> 2) & 15), g = (int)(i & 3);
        const int64_t row = rb * 16 + ln;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (row < rows) v = *reinterpret_cast<const u32x4 *>(src + row * kp + kb * 16 + g * 4);
        dst[i] = v;
    }
}

}  // namespace

// The tile-major copy of a weight's packed words (FNN_OPT_GEMV_TILE_MAJOR) for the GEMV kernels: *words_tm = null where it
// does not apply (option off, rows that are not whole 64-byte blocks, a call on part of a weight, or the copy does not
// exist yet and this call may not allocate), else the copy (built here on first use) and *kb64 = 64-byte blocks per row.
int fnn_tile_major_words(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q, const uint32_t **words_tm, int64_t *kb64)
{
    *words_tm = nullptr;
    *kb64 = 0;
    if (fnn_ctx_option(ctx, FNN_OPT_GEMV_TILE_MAJOR) != 1 || q.words != w->words || q.kp != w->kp || q.kp % 16 != 0 || q.n != w->rows) return FNN_OK;
    fnn_hip_weight *wm = const_cast<fnn_hip_weight *>(w);
    if (!wm->words_tm && !fnn_ctx_no_alloc(ctx)) {
        const int64_t nwords = (w->rows + 15) / 16 * 16 * w->kp;
        if (hipMalloc((void **)&wm->words_tm, (size_t)nwords * 4 + 256) != hipSuccess)
            return fnn_ctx_fail(ctx, FNN_ERR_MEMORY, "out of device memory (tile-major weight rows)");
        int64_t blocks = (nwords / 4 + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(tile_major_kernel, dim3((unsigned)blocks), dim3(256), 0, s, w->words, w->rows, w->kp, w->kp / 16,
                           reinterpret_cast<u32x4 *>(wm->words_tm));
        if (hipGetLastError() != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, "building the tile-major weight rows failed");
    }
    if (wm->words_tm) { *words_tm = wm->words_tm; *kb64 = w->kp / 16; }
    return FNN_OK;
}

int fnn_i8dot_qgemv(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q, bool *handled)
{
    *handled = false;
    if (fnn_ctx_option(ctx, FNN_OPT_GEMV_INT8) == 0) return FNN_OK;
    if (w->dtype != FNN_DT_I8 && w->dtype != FNN_DT_I4 && w->dtype != FNN_DT_U4) return FNN_OK;
    if (q.m < 1 || q.m > fnn_ctx_option(ctx, FNN_OPT_GEMV_INT8_MAX_M) || q.m > 16 || q.n < 1) return FNN_OK;
    if (q.kp % 4 != 0 || q.k % 8 != 0 || q.k < 8) return FNN_OK;
    if ((reinterpret_cast<uintptr_t>(q.a) & 15) || (reinterpret_cast<uintptr_t>(q.words) & 15)) return FNN_OK;
    if (q.n > (int64_t)16 * 0x7fffffff / 2 || q.kp * 4 * 48 >= (int64_t)1 << 31 || q.k >= (int64_t)1 << 29 ||
        q.m * q.k * 4 >= (int64_t)0xFFFFFF00) return FNN_OK;   // 32-bit buffer offsets
    DotArgs p;
    p.words = q.words; p.scales = q.scales; p.zeros = q.zeros; p.a = q.a; p.bias = q.bias; p.out = q.out;
    p.m = q.m; p.n = q.n; p.k = q.k; p.kp = q.kp; p.act = q.act;
    p.nslice = p.ntiles = 0;
    p.words_tm = nullptr; p.kb64 = 0;
    if (int rc = fnn_tile_major_words(ctx, s, w, q, &p.words_tm, &p.kb64)) return rc;
    // Row tiles (of 16 weight rows) per workgroup: a workgroup converts the activation rows once for all of its tiles,
    // and the workgroups should come in whole rounds over the 256 CUs: cost ~ rounds * (rows to convert + tiles).
    // Measured on N = 11008, K = 4096 (I4): M = 1 6.8 / 7.7 / 6.8 us with 1 / 2 / 3 tiles, M = 2 8.0 / 8.3 / 6.8,
    // M = 4 10.4 / 9.5 / 7.5; on N = 4096 one tile (256 workgroups) is best for every M.
    int rt = (int)fnn_ctx_option(ctx, FNN_OPT_GEMV_ROW_TILES);
    if (rt == 0) {
        const int mm = q.m <= 1 ? 1 : (q.m <= 2 ? 2 : (int)((q.m + 3) / 4 * 4));
        const int nw = q.k <= 4 * SL ? 4 : 8;
        int64_t best = -1;
        for (int c = 1; c <= 3; c++) {
            if (q.m <= 4 && mm * 16 * c > nw * 64) break;   // (M <= 4: one output per thread in the epilogue)
            const int64_t wgs = (q.n + 16 * c - 1) / (16 * c);
            const int64_t cost = ((wgs + 255) / 256) * (mm + c);
            if (best < 0 || cost < best) { best = cost; rt = c; }
        }
    }
    hipError_t e;
    switch (w->dtype) {
    case FNN_DT_I8: e = launch_dt<FNN_DT_I8>(p, rt, s, handled); break;
    case FNN_DT_I4: e = launch_dt<FNN_DT_I4>(p, rt, s, handled); break;
    default: e = launch_dt<FNN_DT_U4>(p, rt, s, handled); break;
    }
    if (e != hipSuccess) { *handled = false; return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e)); }
    return FNN_OK;
}
