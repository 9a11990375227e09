// Tiled matrix-core quantised MatMul for gfx950, M >= 5 activation rows.
//
//   out[m,n] = act((sum_k A[m,k]*u(W[n,k]))*scale[n] + zero[n]*sum_k A[m,k] + bias[n])
//   (gemm_batch_packed_simd + apply_affine_dot, src/backend/cpu/microkernels/gemm.rs:1982-2088,
//    src/backend/cpu/microkernels/mod.rs:283-295)
//
// Launches:
//  1. act_prep_kernel turns the f32 activations into f16 MFMA operands once per call (not
//     once per workgroup): each row is scaled by a power of two so that max|x| lands in
//     [2^14, 2^15) and written as hi = f16(x') and, in the default mode, lo = f16((x'-hi)*2^11),
//     so that hi + lo*2^-11 carries ~22 mantissa bits.  The 16 hi rows and the 16 lo rows of
//     16 activation rows form one 32-row MFMA block: same MFMAs, different operand rows.  Row sums
//     (for the zero-point term) are accumulated in f32 in a fixed order.
//  2. qgemm_tile_kernel: a workgroup of 4 waves owns a BM x BN output tile and a K range.
//     Both operands travel HBM -> LDS with global_load_lds_dwordx4 (no registers in between)
//     through a ring of NS stages of 64 k-values, so several stages are in flight while one
//     is consumed; 16-byte chunks are placed with an XOR swizzle that keeps the 128-bit LDS
//     reads of the MFMA operands free of bank conflicts.  The packed weights are decoded to
//     f16 in registers (integer lanes, E4M3/E5M2/E2M1 values are exact in f16) and multiplied
//     with v_mfma_f32_32x32x16_f16.
//  3. With K split over several workgroups (few activation rows: not enough tiles to fill
//     the chip) the partial tiles go to a workspace and splitk_epilogue_kernel adds them in
//     split order, so results do not depend on scheduling.  Asked to (a plan whose next instruction is the MatMul
//     that reads this result: FnnResidualIo / FnnPrepIo in range_io.h), that kernel also stores the sum with a
//     residual, and splitk_prep_epilogue_kernel, one workgroup per output row, leaves the operand of step 1 for that
//     next MatMul, which then starts at step 2.
//
// FNN_FLAG_ACT_F16_SINGLE keeps hi only and removes the first-order effect of the rounding
// on rows with a non-zero mean lane value: dot -= mean_k(u[n,k]) * sum_k (hi - x').
#include "mfma.h"
#include "dech.h"
#include "range_io.h"

#include <cstdlib>
#include <type_traits>

namespace {

using namespace dech;

// internal operand type: weights already expanded to f16 (8 k-values = 4 words), no decode
constexpr int DT_F16_DENSE = 64;
}  // namespace
namespace dech {
template <>
struct DecH<64> {
    static constexpr int WPS = 4;
    static constexpr bool INTERLEAVED = false;
    __device__ static __forceinline__ f16x8 step(const uint32_t *w) { return pack8(w[0], w[1], w[2], w[3]); }
};
}  // namespace dech
namespace {
// the lo activation term is stored scaled by 2^11 so that it stays in the normal f16 range
constexpr float LO_UP = 2048.0f, LO_DOWN = 1.0f / 2048.0f;
constexpr int BK = 64;          // k-values per main-loop iteration

struct PrepArgs {
    const float *a;
    _Float16 *ap;     // [kpad/64][rows_pad][64]: the rows of one 64-wide k block are contiguous
    int64_t rows_pad;
    int *rexp;        // [m_pad] power-of-two exponent applied to the row
    float *xsum;      // [m_pad] sum_k A[m,k]
    float *esum;      // [m_pad] sum_k (hi - x') (single mode)
    int64_t m, k, kpad;
    int precise, interleaved;
};

// effective operand row of activation row m: a 32-row MFMA block holds 16 hi rows, then their 16 lo rows
__device__ __host__ inline int64_t eff_row(int64_t m, int precise, int lo)
{
    if (!precise) return m;
    return (m / 16) * 32 + lo * 16 + m % 16;
}

constexpr int PREP_RG = 4;   // 8-value groups of a row a thread can keep in registers: rows of up to 8192 values

// Statistics and conversion of activation row m held in registers: thread tid has the groups tid + 256 r (8 values
// each, zeros past the row) in keep[r]; writes the hi (+ lo) operand rows, the row's exponent, sum and rounding sum.
// Called by all 256 threads of a workgroup; red: shared scratch.
__device__ __forceinline__ void prep_row_from_regs(const PrepArgs &p, int64_t m, const float4 (&keep)[PREP_RG][2], float (&red)[3][4])
{
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int64_t ngroups = p.kpad / 8;
    _Float16 *hi_row = p.ap + eff_row(m, p.precise, 0) * 64;
    _Float16 *lo_row = p.precise ? p.ap + eff_row(m, 1, 1) * 64 : nullptr;
    const int64_t kb_stride = p.rows_pad * 64;
    auto group_at = [&](_Float16 *row, int64_t g) { return row + (g >> 3) * kb_stride + (g & 7) * 8; };
    float mx = 0.0f, sum = 0.0f;
#pragma unroll
    for (int r = 0; r < PREP_RG; r++)
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const float4 v = keep[r][q];
            mx = fmaxf(mx, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
            sum += (v.x + v.y) + (v.z + v.w);
        }
    mx = wave_max(mx);
    sum = wave_sum(sum);
    if (lane == 0) { red[0][wv] = mx; red[1][wv] = sum; }
    __syncthreads();
    mx = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
    sum = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
    int e = 0;
    if (mx > 0.0f && mx < __builtin_huge_valf()) {
        int ex;
        (void)frexpf(mx, &ex);  // mx = f * 2^ex, f in [0.5, 1)
        e = 15 - ex;            // mx * 2^e in [2^14, 2^15)
    }
    float err = 0.0f;
#pragma unroll
    for (int r = 0; r < PREP_RG; r++) {
        const int64_t g = tid + 256 * r;
        if (g < ngroups) {
            const float v[8] = {keep[r][0].x, keep[r][0].y, keep[r][0].z, keep[r][0].w,
                                keep[r][1].x, keep[r][1].y, keep[r][1].z, keep[r][1].w};
            f16x8 h, l;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                // operand slot j holds k = 0,4,1,5,2,6,3,7 for the nibble decoders
                const int src = p.interleaved ? ((j & 1) * 4 + (j >> 1)) : j;
                const float xs = ldexpf(v[src], e);
                const _Float16 hh = (_Float16)xs;
                h[j] = hh;
                const float rr = xs - (float)hh;
                l[j] = (_Float16)(rr * LO_UP);
                err -= rr;
            }
            *reinterpret_cast<f16x8 *>(group_at(hi_row, g)) = h;
            if (lo_row) *reinterpret_cast<f16x8 *>(group_at(lo_row, g)) = l;
        }
    }
    err = wave_sum(err);
    if (lane == 0) red[2][wv] = err;
    __syncthreads();
    if (tid == 0) {
        p.rexp[m] = e;
        p.xsum[m] = sum;
        p.esum[m] = (red[2][0] + red[2][1]) + (red[2][2] + red[2][3]);
    }
}

// zero operands for a padding row of the last tile
__device__ __forceinline__ void prep_zero_row(const PrepArgs &p, int64_t m)
{
    const int tid = threadIdx.x;
    const int64_t ngroups = p.kpad / 8;
    _Float16 *hi_row = p.ap + eff_row(m, p.precise, 0) * 64;
    _Float16 *lo_row = p.precise ? p.ap + eff_row(m, 1, 1) * 64 : nullptr;
    const int64_t kb_stride = p.rows_pad * 64;
    auto group_at = [&](_Float16 *row, int64_t g) { return row + (g >> 3) * kb_stride + (g & 7) * 8; };
    const uint4 z = make_uint4(0, 0, 0, 0);
    for (int64_t g = tid; g < ngroups; g += 256) {
        *reinterpret_cast<uint4 *>(group_at(hi_row, g)) = z;
        if (lo_row) *reinterpret_cast<uint4 *>(group_at(lo_row, g)) = z;
    }
    if (tid == 0) { p.rexp[m] = 0; p.xsum[m] = 0.0f; p.esum[m] = 0.0f; }
}

__global__ void __launch_bounds__(256) act_prep_kernel(PrepArgs p)
{
    __shared__ float red[3][4];
    const int64_t m = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int64_t K = p.k, ngroups = p.kpad / 8;
    if (m >= p.m) {  // padding rows of the last tile: zero operands
        prep_zero_row(p, m);
        return;
    }
    const float *x = p.a + m * K;
    const bool vec = (K % 8 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    const bool in_regs = vec && ngroups <= 256 * PREP_RG && p.kpad == K;
    if (in_regs) {
        // one trip to memory: the row stays in registers between the statistics and the conversion
        float4 keep[PREP_RG][2];
#pragma unroll
        for (int r = 0; r < PREP_RG; r++) {
            const int64_t g = tid + 256 * r;
            keep[r][0] = keep[r][1] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (g < ngroups) {
                keep[r][0] = *reinterpret_cast<const float4 *>(x + g * 8);
                keep[r][1] = *reinterpret_cast<const float4 *>(x + g * 8 + 4);
            }
        }
        prep_row_from_regs(p, m, keep, red);
        return;
    }
    // 16-byte group g of a row: k block g/8, position g%8 inside the block's 128-byte row
    _Float16 *hi_row = p.ap + eff_row(m, p.precise, 0) * 64;
    _Float16 *lo_row = p.precise ? p.ap + eff_row(m, 1, 1) * 64 : nullptr;
    const int64_t kb_stride = p.rows_pad * 64;
    auto group_at = [&](_Float16 *row, int64_t g) { return row + (g >> 3) * kb_stride + (g & 7) * 8; };
    float mx = 0.0f, sum = 0.0f;
    if (vec) {
        for (int64_t i = tid; i < K / 4; i += 256) {
            const float4 v = reinterpret_cast<const float4 *>(x)[i];
            mx = fmaxf(mx, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
            sum += (v.x + v.y) + (v.z + v.w);
        }
    } else {
        for (int64_t i = tid; i < K; i += 256) {
            mx = fmaxf(mx, fabsf(x[i]));
            sum += x[i];
        }
    }
    mx = wave_max(mx);
    sum = wave_sum(sum);
    if (lane == 0) { red[0][wv] = mx; red[1][wv] = sum; }
    __syncthreads();
    mx = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
    sum = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
    int e = 0;
    if (mx > 0.0f && mx < __builtin_huge_valf()) {
        int ex;
        (void)frexpf(mx, &ex);  // mx = f * 2^ex, f in [0.5, 1)
        e = 15 - ex;            // mx * 2^e in [2^14, 2^15)
    }
    float err = 0.0f;
    auto convert = [&](int64_t g, const float(&v)[8]) {
        f16x8 h, l;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            // operand slot j holds k = 0,4,1,5,2,6,3,7 for the nibble decoders
            const int src = p.interleaved ? ((j & 1) * 4 + (j >> 1)) : j;
            const float xs = ldexpf(v[src], e);
            const _Float16 hh = (_Float16)xs;
            h[j] = hh;
            const float r = xs - (float)hh;
            l[j] = (_Float16)(r * LO_UP);
            err -= r;
        }
        *reinterpret_cast<f16x8 *>(group_at(hi_row, g)) = h;
        if (lo_row) *reinterpret_cast<f16x8 *>(group_at(lo_row, g)) = l;
    };
    for (int64_t g = tid; g < ngroups; g += 256) {
        float v[8];
        const int64_t k0 = g * 8;
        if (vec && k0 + 8 <= K) {
            const float4 a0 = *reinterpret_cast<const float4 *>(x + k0);
            const float4 a1 = *reinterpret_cast<const float4 *>(x + k0 + 4);
            v[0] = a0.x; v[1] = a0.y; v[2] = a0.z; v[3] = a0.w;
            v[4] = a1.x; v[5] = a1.y; v[6] = a1.z; v[7] = a1.w;
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = (k0 + j < K) ? x[k0 + j] : 0.0f;
        }
        convert(g, v);
    }
    err = wave_sum(err);
    if (lane == 0) red[2][wv] = err;
    __syncthreads();
    if (tid == 0) {
        p.rexp[m] = e;
        p.xsum[m] = sum;
        p.esum[m] = (red[2][0] + red[2][1]) + (red[2][2] + red[2][3]);
    }
}

// mean lane value per weight row (single mode compensation); one wave per row
template <int DT>
__global__ void __launch_bounds__(64) row_umean_kernel(const uint32_t *words, int64_t rows, int64_t kp, int64_t k, float *umean)
{
    const int64_t r = blockIdx.x;
    if (r >= rows) return;
    constexpr int EPW = Codec<DT>::EPW;
    float s = 0.0f;
    for (int64_t i = threadIdx.x; i < kp; i += 64) {
        float v[EPW];
        Codec<DT>::decode(words[r * kp + i], v);
#pragma unroll
        for (int j = 0; j < EPW; j++)
            if (i * EPW + j < k) s += v[j];
    }
    s = wave_sum(s);
    if (threadIdx.x == 0) umean[r] = s / (float)k;
}

#include "tile_kernel.h"

// Split-K reduction that also prepares the operand of the MatMul reading this one's result (a plan's next layer):
// workgroup m owns output row m whole.  Thread (r, tid) of its RW * 256 threads owns the columns 8 * (tid + 256 r),
// the group that thread tid of act_prep_kernel holds in keep[r]: it adds the partial tiles in split order and applies
// the epilogue exactly as splitk_epilogue_kernel does, stores its eight values (and their sums with a residual), and
// converts what the next MatMul reads, `use_sum` ? the sums : the values, as prep_row_from_regs would: the row
// maximum is order-free, and the row sum and the rounding sum are formed by the threads r == 0 from the other
// threads' terms in the order of act_prep_kernel's loops, so every word left behind equals what act_prep_kernel
// writes for the same row.  n % 64 == 0, n <= 2048 * RW, no codebook scales; rows m >= p.m are the padding rows of
// the next operand.
template <int RW>
__global__ void __launch_bounds__(256 * RW) splitk_prep_epilogue_kernel(TileArgs p, PrepArgs next, int single, int use_sum)
{
    constexpr int NWV = 4 * RW;
    __shared__ float red_mx[NWV];
    __shared__ float red[3][4];
    __shared__ float s_sum[RW][2][256];
    __shared__ float s_rr[RW][8][256];
    const int64_t m = blockIdx.x;
    const int t = threadIdx.x, tid = t & 255, r = t >> 8, lane = t & 63, wv = t >> 6;
    const int64_t ngroups = p.n / 8;
    _Float16 *hi_row = next.ap + eff_row(m, next.precise, 0) * 64;
    _Float16 *lo_row = next.precise ? next.ap + eff_row(m, 1, 1) * 64 : nullptr;
    const int64_t kb_stride = next.rows_pad * 64;
    auto group_at = [&](_Float16 *row, int64_t g) { return row + (g >> 3) * kb_stride + (g & 7) * 8; };
    if (m >= p.m) {
        const uint4 z = make_uint4(0, 0, 0, 0);
        for (int64_t g = t; g < ngroups; g += 256 * RW) {
            *reinterpret_cast<uint4 *>(group_at(hi_row, g)) = z;
            if (lo_row) *reinterpret_cast<uint4 *>(group_at(lo_row, g)) = z;
        }
        if (t == 0) { next.rexp[m] = 0; next.xsum[m] = 0.0f; next.esum[m] = 0.0f; }
        return;
    }
    const int64_t total = p.m * p.n;
    const bool comp = single && p.umean;
    const int64_t g = tid + 256 * r;
    const bool mine = g < ngroups;
    float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};   // what the next MatMul reads in these columns
    if (mine) {
        const int64_t n0 = g * 8, idx = m * p.n + n0;
        const float xs = p.xsum[m];
        const float cterm = comp ? ldexpf(p.esum[m], -p.rexp[m]) : 0.0f;
        float d[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const float *pp = p.part + idx;
        int zz = 0;
        for (; zz + 4 <= p.splits; zz += 4) {
            float4 v[4][2];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                v[u][0] = *reinterpret_cast<const float4 *>(pp + (int64_t)(zz + u) * total);
                v[u][1] = *reinterpret_cast<const float4 *>(pp + (int64_t)(zz + u) * total + 4);
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                d[0] += v[u][0].x; d[1] += v[u][0].y; d[2] += v[u][0].z; d[3] += v[u][0].w;
                d[4] += v[u][1].x; d[5] += v[u][1].y; d[6] += v[u][1].z; d[7] += v[u][1].w;
            }
        }
        for (; zz < p.splits; zz++) {
            const float4 v0 = *reinterpret_cast<const float4 *>(pp + (int64_t)zz * total);
            const float4 v1 = *reinterpret_cast<const float4 *>(pp + (int64_t)zz * total + 4);
            d[0] += v0.x; d[1] += v0.y; d[2] += v0.z; d[3] += v0.w;
            d[4] += v1.x; d[5] += v1.y; d[6] += v1.z; d[7] += v1.w;
        }
        float sc[8], zr[8];
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const float4 a = *reinterpret_cast<const float4 *>(p.scales + n0 + 4 * q);
            const float4 b = *reinterpret_cast<const float4 *>(p.zeros + n0 + 4 * q);
            sc[4 * q] = a.x; sc[4 * q + 1] = a.y; sc[4 * q + 2] = a.z; sc[4 * q + 3] = a.w;
            zr[4 * q] = b.x; zr[4 * q + 1] = b.y; zr[4 * q + 2] = b.z; zr[4 * q + 3] = b.w;
        }
        float o[8], sm[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            float dj = d[j];
            if (comp) dj = dj - p.umean[n0 + j] * cterm;
            float v = dj * sc[j] + zr[j] * xs;
            if (p.bias) v = v + p.bias[n0 + j];
            o[j] = fnn_activation(v, p.act);
            sm[j] = p.residual ? o[j] + p.residual[idx + j] : o[j];
        }
        *reinterpret_cast<float4 *>(p.out + idx) = make_float4(o[0], o[1], o[2], o[3]);
        *reinterpret_cast<float4 *>(p.out + idx + 4) = make_float4(o[4], o[5], o[6], o[7]);
        if (p.residual) {
            *reinterpret_cast<float4 *>(p.sum_out + idx) = make_float4(sm[0], sm[1], sm[2], sm[3]);
            *reinterpret_cast<float4 *>(p.sum_out + idx + 4) = make_float4(sm[4], sm[5], sm[6], sm[7]);
        }
#pragma unroll
        for (int j = 0; j < 8; j++) x[j] = use_sum ? sm[j] : o[j];
    }
    // ---- row statistics in act_prep_kernel's order
    float mx = fmaxf(fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3]))),
                     fmaxf(fmaxf(fabsf(x[4]), fabsf(x[5])), fmaxf(fabsf(x[6]), fabsf(x[7]))));
    mx = wave_max(mx);
    if (lane == 0) red_mx[wv] = mx;
    s_sum[r][0][tid] = (x[0] + x[1]) + (x[2] + x[3]);
    s_sum[r][1][tid] = (x[4] + x[5]) + (x[6] + x[7]);
    __syncthreads();
    mx = red_mx[0];
#pragma unroll
    for (int w2 = 1; w2 < NWV; w2++) mx = fmaxf(mx, red_mx[w2]);
    if (r == 0) {
        float sum = 0.0f;
#pragma unroll
        for (int r2 = 0; r2 < RW; r2++) { sum += s_sum[r2][0][tid]; sum += s_sum[r2][1][tid]; }
        sum = wave_sum(sum);
        if (lane == 0) red[1][wv] = sum;
    }
    int e = 0;
    if (mx > 0.0f && mx < __builtin_huge_valf()) {
        int ex;
        (void)frexpf(mx, &ex);
        e = 15 - ex;
    }
    if (mine) {
        f16x8 h, l;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int src = next.interleaved ? ((j & 1) * 4 + (j >> 1)) : j;
            const float xs2 = ldexpf(x[src], e);
            const _Float16 hh = (_Float16)xs2;
            h[j] = hh;
            const float rr = xs2 - (float)hh;
            l[j] = (_Float16)(rr * LO_UP);
            s_rr[r][j][tid] = rr;
        }
        *reinterpret_cast<f16x8 *>(group_at(hi_row, g)) = h;
        if (lo_row) *reinterpret_cast<f16x8 *>(group_at(lo_row, g)) = l;
    }
    __syncthreads();
    if (r == 0) {
        float err = 0.0f;
#pragma unroll
        for (int r2 = 0; r2 < RW; r2++) {
            if (tid + 256 * r2 < ngroups) {
#pragma unroll
                for (int j = 0; j < 8; j++) err -= s_rr[r2][j][tid];
            }
        }
        err = wave_sum(err);
        if (lane == 0) red[2][wv] = err;
    }
    __syncthreads();
    if (t == 0) {
        next.rexp[m] = e;
        next.xsum[m] = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
        next.esum[m] = (red[2][0] + red[2][1]) + (red[2][2] + red[2][3]);
    }
}

template <int DT, int WGM, int WGN, int TM, int TN, bool PRECISE, int NS>
hipError_t launch_tile(const TileArgs &p, hipStream_t s)
{
    constexpr int WC = 2 * DecH<DT>::WPS;
    constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
    constexpr size_t lds = (size_t)NS * (BM * 128 + BN * WC * 16);
    auto kern = qgemm_tile_kernel<DT, WGM, WGN, TM, TN, PRECISE, NS>;
    static std::atomic<uint64_t> lds_raised{0};
    hipError_t e = fnn_raise_lds_limit(lds_raised, reinterpret_cast<const void *>(kern), (int)lds);
    if (e != hipSuccess) return e;
    const unsigned total = (unsigned)p.mtiles * p.ntiles * p.splits;
    hipLaunchKernelGGL(kern, dim3(total), dim3(WGM * WGN * 64), lds, s, p);
    return hipGetLastError();
}

template <int DT>
hipError_t launch_umean(const fnn_hip_weight *w, float *umean, hipStream_t s)
{
    hipLaunchKernelGGL(row_umean_kernel<DT>, dim3((unsigned)w->rows), dim3(64), 0, s, w->words, w->rows, w->kp, w->inner, umean);
    return hipGetLastError();
}

// weights expanded beforehand to f16 [N][2*kpad] = [hi | lo] (codebook type): replaces the packed operand
struct DenseOperand {
    const uint32_t *words;
    const float *row_scale, *row_zero;
};

// Shape of the prepared activation operand and of the tiles for an [M, K] x [N, K]^T product
struct TileLayout {
    bool precise;
    int cfg, bm, mtiles, ntiles;
    int64_t kpad, meff, rows_pad, m_pad;
    size_t ap_bytes, meta_off, ws_bytes;
};

template <int DT>
TileLayout tile_layout(fnn_hip_ctx *ctx, int64_t M, int64_t N, int64_t K, int flags, bool dense)
{
    TileLayout L;
    const bool precise = !(flags & FNN_FLAG_ACT_F16_SINGLE);
    const int64_t kpad = (K + BK - 1) / BK * BK;
    const int64_t meff = precise ? (M + 15) / 16 * 32 : (M + 31) / 32 * 32;
    // tile shape by effective row count
    // 0: 128x128 (2x2 waves of 64x64), 1: 64x128 (4 waves of 64x32), 2: 32x128 (4 waves of 32x32)
    // (measured: with at most 128 tiles of 128x128 the 64-row tiles win, they need a smaller K split or none:
    //  C1 M=64 24.1 -> 20.6 us, M=256 39.2 -> 36.7 us, FP8 2048->8192 M=64 23.5 -> 19.9 us; the dense codebook
    //  operand, swept twice, is the exception)
    int cfg;
    if (meff > 64) cfg = (!dense && ((meff + 127) / 128) * ((N + 127) / 128) <= 128) ? 1 : 0;
    else if (meff == 64) cfg = 1;
    else cfg = 2;
    // ... unless the 32-row tiles fill the chip in one round without a K split (192..256 of them: no reduction launch,
    // no partial tiles).  FP8 2048 -> 8192: M = 33 19.0 -> 17.0 us, M = 64 19.4 -> 17.6; FP4: 17.9 -> 14.4, 18.4 -> 14.9;
    // with fewer or more tiles than that the 64-row tiles and their split stay ahead (4096 x 4096 at M = 64: 19.7 against
    // 21.6 us; 2048 -> 8192 at M = 96: 21.6 against 25.5).
    // codebook weights decoded in the kernel: the 64-row tiles at every size (their loop is bound by the vector ALU, and
    // four waves of 64 x 32 share it better than four of 64 x 64: M = 512 109.6 against 131.6 us, M = 1024 204 against 231)
    if (DT == FNN_DT_I4CB && meff > 64) cfg = 1;
    if (cfg == 1 && !dense && meff <= 128 && DT != FNN_DT_I4CB) {   // (measured for up to 64 activation rows; the codebook decode wants the larger tiles)
        const int64_t small_tiles = ((meff + 31) / 32) * ((N + 127) / 128);
        if (small_tiles >= 192 && small_tiles <= 256) cfg = 2;
    }
    // the dense (expanded codebook) operand: 256 x 128 tiles on eight waves (twice the waves that fetch a stage's bytes,
    // and half the weight bytes per row tile) where they need fewer rounds of workgroups.  In units of a 128 x 128 tile's
    // sweep over K: rounds of 256 workgroups x the share of K per workgroup, a 256 x 128 tile 1.36 of it, plus 0.13 / 0.35
    // for the partial tiles of a K split (the rules further down).  us, 128 x 128 / 256 x 128 tiles, 4096 x 4096:
    // M = 256 57 / 86, 384 80 / 92, 512 91 / 92, 640 225 / 137, 1024 225 / 155, 2048 436 / 289, 4096 871 / 562;
    // 4096 x 11008: M = 192 211 / 151, 256 228 / 152, 384 307 / 230, 512 335 / 247; 11008 x 4096: M = 256 154 / 219; 8192 x 8192: M = 256
    // 188 / 185, 384 473 / 295, 512 478 / 318, 1024 910 / 607
    if (dense && meff > 128) {
        const int64_t nt = (N + 127) / 128, t0 = ((meff + 127) / 128) * nt, t3 = ((meff + 255) / 256) * nt;
        const int64_t s0 = t0 >= 256 ? 1 : 256 / t0;
        const double c0 = (double)((t0 * s0 + 255) / 256) / (double)s0 + (s0 > 1 ? 0.13 : 0.0);
        const double r1 = (double)((t3 + 255) / 256), r2 = (double)((2 * t3 + 255) / 256) / 2.0 + 0.1;
        const int64_t s3 = r2 < r1 ? 2 : 1;
        const double c3 = 1.36 * (double)((t3 * s3 + 255) / 256) / (double)s3 + (s3 > 1 ? 0.35 : 0.0);
        if (c3 < c0) cfg = 3;
    }
    const int64_t opt_cfg = fnn_ctx_option(ctx, FNN_OPT_TILE_SHAPE);
    // 3 (by option only): 256x128 with 8 waves of 64x64, two waves per SIMD.  Measured on FP8 4096 x 4096 and 2048 -> 8192
    // at M = 128 ... 1024: 0-30 % slower than the automatic choice, except where it turns the tile count into one whole
    // round (2048 -> 8192, M = 1024, single rounding: 84 -> 57 us).  Deeper rings (8 stages) for the 64- and 32-row
    // tiles changed nothing either: a wave's HBM -> LDS loads complete at about 3.7 bytes per clock however many are
    // in flight, so four waves deliver ~15 bytes per clock and CU, eight ~30, twelve ~41.
    // For 17 <= M <= 128 neither helps: 64 x 256 and 128 x 256 tiles with eight waves side by side along N (every
    // wave loading) measured 10-40 % slower than the 4-wave tiles at every K split; these calls are bound by their
    // three dependent launches (activation preparation, tiles, split-K reduction), not by delivery.
    if (opt_cfg >= 0 && opt_cfg <= 3) cfg = (int)opt_cfg;
    if (cfg == 3 && DecH<DT>::WPS < 2) cfg = 0;  // (8-bit weights only: a stage of 4-bit rows has too few 16-byte chunks for 8 waves)
    L.precise = precise; L.cfg = cfg;
    L.bm = cfg == 3 ? 256 : (cfg == 0 ? 128 : (cfg == 1 ? 64 : 32));
    L.mtiles = (int)((meff + L.bm - 1) / L.bm);
    L.ntiles = (int)((N + 127) / 128);
    L.kpad = kpad; L.meff = meff;
    L.rows_pad = (int64_t)L.mtiles * L.bm;
    L.m_pad = precise ? L.rows_pad / 2 : L.rows_pad;
    L.ap_bytes = (size_t)L.rows_pad * kpad * 2;
    L.meta_off = (L.ap_bytes + 255) / 256 * 256;
    L.ws_bytes = L.meta_off + (size_t)L.m_pad * 12 + 256;
    return L;
}

// the same for a weight whose type is known at run time; false: that type does not run through run_tiled's packed form
bool tile_layout_of(fnn_hip_ctx *ctx, int dtype, int64_t M, int64_t N, int64_t K, int flags, TileLayout *L, int *interleaved)
{
    switch (dtype) {
    case FNN_DT_U8: *L = tile_layout<FNN_DT_U8>(ctx, M, N, K, flags, false); *interleaved = DecH<FNN_DT_U8>::INTERLEAVED; return true;
    case FNN_DT_F8: *L = tile_layout<FNN_DT_F8>(ctx, M, N, K, flags, false); *interleaved = DecH<FNN_DT_F8>::INTERLEAVED; return true;
    case FNN_DT_F8R: *L = tile_layout<FNN_DT_F8R>(ctx, M, N, K, flags, false); *interleaved = DecH<FNN_DT_F8R>::INTERLEAVED; return true;
    case FNN_DT_F4: *L = tile_layout<FNN_DT_F4>(ctx, M, N, K, flags, false); *interleaved = DecH<FNN_DT_F4>::INTERLEAVED; return true;
    default: return false;
    }
}

template <int DT>
int run_tiled(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q, int flags,
              const DenseOperand *dense = nullptr)
{
    const int64_t M = q.m, N = q.n, K = q.k;
    const TileLayout L = tile_layout<DT>(ctx, M, N, K, flags, dense != nullptr);
    const bool precise = L.precise;
    const int cfg = L.cfg;
    const int64_t kpad = L.kpad, rows_pad = L.rows_pad, m_pad = L.m_pad;
    const int mtiles = L.mtiles, ntiles = L.ntiles;
    const int passes = dense ? 2 : 1;
    const int iters = (int)(kpad / BK) * passes;
    // Split K over workgroups when the tiles alone do not fill the 256 CUs.  The factor minimises a
    // small cost model in microseconds, fitted to sweeps over the split factor on the benchmark shapes:
    // stages per workgroup x time a CU needs per stage x workgroups per CU (a CU gets through
    // stages at the same rate with one or several workgroups resident, but a lone workgroup cannot
    // hide its load latency: factor 1.5), plus, for s > 1, the write + read of s partial [M,N] tiles.
    const int env_split = (int)fnn_ctx_option(ctx, FNN_OPT_TILE_SPLIT);
    const int base = mtiles * ntiles;
    // (codebook weights decoded in the kernel: two MFMAs per step and the table look-ups)
    const double t_bits = DT == FNN_DT_I4CB ? 0.9 : (DecH<DT>::WPS == 1 ? 0.4 : (DecH<DT>::WPS == 2 ? 0.7 : 1.0));
    const double t_stage = t_bits * (cfg == 3 ? 2.0 : (cfg == 0 ? 1.0 : (cfg == 1 ? 0.5 : 0.25)));
    const double part_us = (double)M * (double)N * 8.0 / 3.0e6;
    int splits = 1;
    double best = 1e30;
    for (int sp = 1; sp <= 32 && sp <= (iters / 4 > 0 ? iters / 4 : 1); sp++) {
        const int per = (iters + sp - 1) / sp;
        const double r = (double)base * sp / 256.0;
        // (the dense operand's 128x128 stages take 96 KB of LDS: one workgroup per CU, rounds do not overlap)
        const double wgs = (dense && cfg == 0) ? 1.5 * (double)(int64_t)(r + 0.999)
                                               : (r <= 1.0 ? 1.5 : (double)(int64_t)(r + 0.95));
        const double cost = per * t_stage * wgs + (sp > 1 ? 2.0 * sp * part_us : 0.0);
        if (cost < best * 0.995) { best = cost; splits = sp; }   // on a tie the coarser split wins
    }
    // the dense operand (128 x 128 tiles, one workgroup per CU): as many splits as fill one round, no more (measured on
    // 4096 x 4096: 96 tiles 58.0 us with 2 splits against 71.6 with the model's choice, 192 tiles 82.1 with none against 110)
    if (dense && cfg == 0) splits = base >= 256 ? 1 : 256 / base;
    // ... and on its 256 x 128 tiles: two splits only where they save a round of workgroups (M = 1536: 245 against 265 us;
    // M = 1024, 2048, 4096: one split 155 / 289 / 562 against 169 / 316 / 640)
    if (dense && cfg == 3) {
        const double r1 = (double)((base + 255) / 256), r2 = (double)((2 * base + 255) / 256) / 2.0 + 0.1;
        splits = r2 < r1 ? 2 : 1;
    }
    if (env_split > 0) splits = env_split;
    if (splits > iters / 4) splits = iters / 4 > 0 ? iters / 4 : 1;
    int ips = (iters + splits - 1) / splits;
    splits = (iters + ips - 1) / ips;   // no empty split

    // workspace: operands + row tables; partial tiles.  The operand may be in place already: the MatMul call before
    // this one can have prepared it (FnnPrepIo), in which case nothing may touch that buffer before the tiles run.
    const size_t meta_off = L.meta_off;
    FnnPrepIo *pio = fnn_ctx_prep_io(ctx);
    FnnPreparedOperand *have = fnn_ctx_prepared(ctx);
    constexpr int kInterleaved = DecH<DT>::INTERLEAVED ? 1 : 0;
    const bool handed = pio->offered && !dense && have->buffer && have->a == q.a && have->m == M && have->k == K && have->kpad == kpad &&
                        have->rows_pad == rows_pad && have->precise == (precise ? 1 : 0) && have->interleaved == kInterleaved;
    const int own_slot = handed ? have->slot : 0;
    void *ws0 = handed ? have->buffer : nullptr, *ws1 = nullptr;
    int rc;
    if (!handed && (rc = fnn_ctx_ensure_tmp(ctx, 0, L.ws_bytes, &ws0))) return rc;
    if (splits > 1 && (rc = fnn_ctx_ensure_tmp(ctx, 1, (size_t)splits * M * N * 4, &ws1))) return rc;
    *have = FnnPreparedOperand{};   // (whatever was there is used by this call or stale)
    pio->consumed = handed ? 1 : 0;

    fnn_hip_weight *wm = const_cast<fnn_hip_weight *>(w);
    const bool want_umean = !precise && !dense && (DT == FNN_DT_I8 || DT == FNN_DT_I4 || DT == FNN_DT_U8 || DT == FNN_DT_U4 || DT == FNN_DT_F4);
    if constexpr (DT != DT_F16_DENSE && DT != FNN_DT_I4CB) if (want_umean && !wm->umean) {
        if (fnn_ctx_no_alloc(ctx)) return fnn_ctx_fail(ctx, FNN_ERR_MEMORY, "first single-pass use of a weight while allocation is not allowed (graph capture, fnn_hip_qmatmul_static)");
        if (hipMalloc((void **)&wm->umean, (size_t)w->rows * 4 + 64) != hipSuccess)
            return fnn_ctx_fail(ctx, FNN_ERR_MEMORY, "out of device memory (row means)");
        hipError_t e = launch_umean<DT>(w, wm->umean, s);
        if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    }

    PrepArgs pa;
    pa.a = q.a;
    pa.ap = (_Float16 *)ws0;
    pa.rexp = (int *)((char *)ws0 + meta_off);
    pa.xsum = (float *)(pa.rexp + m_pad);
    pa.esum = pa.xsum + m_pad;
    pa.m = M; pa.k = K; pa.kpad = kpad; pa.rows_pad = rows_pad;
    pa.precise = precise ? 1 : 0;
    pa.interleaved = DecH<DT>::INTERLEAVED ? 1 : 0;
    hipError_t e = hipSuccess;
    if (!handed) {
        hipLaunchKernelGGL(act_prep_kernel, dim3((unsigned)m_pad), dim3(256), 0, s, pa);
        e = hipGetLastError();
        if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    }

    TileArgs t = {};
    t.words = q.words;
    if constexpr (DT != DT_F16_DENSE && DT != FNN_DT_I4CB && (DecH<DT>::WPS == 2 || DecH<DT>::WPS == 1)) {   // 64 (8-bit types) or 32 bytes (4-bit) per row and stage: a block or half a block of the tile-major copy
        if (!dense)
            if (int rc2 = fnn_tile_major_words(ctx, s, w, q, &t.words_tm, &t.kb64)) return rc2;
    }
    t.zero_chunk = q.words + w->rows * q.kp;    // the zeroed margin behind the last row
    t.scales = q.scales; t.zeros = q.zeros; t.umean = want_umean ? wm->umean : nullptr; t.bias = q.bias;
    t.ap = pa.ap; t.rexp = pa.rexp; t.xsum = pa.xsum; t.esum = pa.esum;
    t.out = q.out; t.part = (float *)ws1;
    t.residual = nullptr; t.sum_out = nullptr;
    if (FnnResidualIo *res = fnn_ctx_residual_io(ctx); splits > 1 && res->residual && res->of_out == q.out && res->elems == (uint64_t)(M * N)) {
        t.residual = res->residual; t.sum_out = res->sum_out;
        res->used = 1;
    }
    t.m = M; t.n = N; t.kp = q.kp; t.kpad = kpad; t.rows_pad = rows_pad;
    t.a_wrap = 0;
    t.bscales = nullptr; t.codebook = nullptr; t.bpr = 0;
    if constexpr (DT == FNN_DT_I4CB) {
        t.bscales = q.scales; t.codebook = q.codebook; t.bpr = q.bpr;
        t.scales = nullptr; t.zeros = nullptr;
    }
    if (dense) {
        t.words = dense->words; t.zero_chunk = dense->words;
        t.scales = dense->row_scale; t.zeros = dense->row_zero;
        t.kp = kpad;                      // words per row: 2*kpad f16
        t.a_wrap = (int)(kpad / BK);
    }
    t.act = q.act; t.splits = splits; t.iters = iters; t.ips = ips; t.mtiles = mtiles; t.ntiles = ntiles;
    const int env_ns = (int)fnn_ctx_option(ctx, FNN_OPT_TILE_STAGES);
    const bool deep = cfg == 0 && (env_ns == 5 || (env_ns == 0 && base * splits <= 256));
    constexpr int WCX = 2 * DecH<DT>::WPS;
    if (cfg == 3) {
        if constexpr (WCX >= 4 && 3 * (256 * 128 + 128 * WCX * 16) <= 160 * 1024)
            e = precise ? launch_tile<DT, 4, 2, 2, 2, true, 3>(t, s) : launch_tile<DT, 4, 2, 2, 2, false, 3>(t, s);
        else e = hipErrorInvalidValue;
    } else if (deep) e = precise ? launch_tile<DT, 2, 2, 2, 2, true, 5>(t, s) : launch_tile<DT, 2, 2, 2, 2, false, 5>(t, s);
    else if (precise) {
        if (cfg == 0) e = launch_tile<DT, 2, 2, 2, 2, true, 3>(t, s);
        else if (cfg == 1) e = launch_tile<DT, 1, 4, 2, 1, true, 4>(t, s);
        else e = launch_tile<DT, 1, 4, 1, 1, true, 6>(t, s);
    } else {
        if (cfg == 0) e = launch_tile<DT, 2, 2, 2, 2, false, 3>(t, s);
        else if (cfg == 1) e = launch_tile<DT, 1, 4, 2, 1, false, 4>(t, s);
        else e = launch_tile<DT, 1, 4, 1, 1, false, 6>(t, s);
    }
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    if (splits > 1) {
        // The reduction can leave the prepared operand of the MatMul that reads this result (a request in FnnPrepIo):
        // whole rows per workgroup, in the other operand buffer than the one this call's own row tables live in.
        TileLayout NL;
        int n_il = 0;
        const bool may_prepare = pio->next_w && !dense && !t.codebook && !fnn_ctx_static_mode(ctx) && M >= 17 && N % 64 == 0 && N <= 2048 * PREP_RG &&
                                 (pio->next_a == q.out || (t.residual && pio->next_a == t.sum_out)) &&
                                 pio->next_w->inner == N && tile_layout_of(ctx, pio->next_w->dtype, M, pio->next_w->rows, N, pio->next_flags, &NL, &n_il) &&
                                 NL.kpad == N && !((reinterpret_cast<uintptr_t>(t.scales) | reinterpret_cast<uintptr_t>(t.zeros) | reinterpret_cast<uintptr_t>(t.out) |
                                                    reinterpret_cast<uintptr_t>(t.sum_out) | reinterpret_cast<uintptr_t>(t.part)) & 15);
        void *nb = nullptr;
        const int next_slot = own_slot == 0 ? 4 : 0;
        if (may_prepare && fnn_ctx_ensure_tmp(ctx, next_slot, NL.ws_bytes, &nb) == FNN_OK && nb) {
            PrepArgs np;
            np.a = nullptr;
            np.ap = (_Float16 *)nb;
            np.rexp = (int *)((char *)nb + NL.meta_off);
            np.xsum = (float *)(np.rexp + NL.m_pad);
            np.esum = np.xsum + NL.m_pad;
            np.m = M; np.k = N; np.kpad = NL.kpad; np.rows_pad = NL.rows_pad;
            np.precise = NL.precise ? 1 : 0;
            np.interleaved = n_il;
            const int use_sum = pio->next_a == q.out ? 0 : 1;
            if (N > 4096) hipLaunchKernelGGL(splitk_prep_epilogue_kernel<4>, dim3((unsigned)NL.m_pad), dim3(1024), 0, s, t, np, precise ? 0 : 1, use_sum);
            else if (N > 2048) hipLaunchKernelGGL(splitk_prep_epilogue_kernel<2>, dim3((unsigned)NL.m_pad), dim3(512), 0, s, t, np, precise ? 0 : 1, use_sum);
            else hipLaunchKernelGGL(splitk_prep_epilogue_kernel<1>, dim3((unsigned)NL.m_pad), dim3(256), 0, s, t, np, precise ? 0 : 1, use_sum);
            e = hipGetLastError();
            if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
            have->a = pio->next_a; have->buffer = nb; have->slot = next_slot;
            have->m = M; have->k = N; have->kpad = NL.kpad; have->rows_pad = NL.rows_pad;
            have->precise = np.precise; have->interleaved = n_il;
            pio->produced = 1;
            return FNN_OK;
        }
        const int64_t colb = (N + 255) / 256;
        int64_t rowb = (2048 + colb - 1) / colb;   // about 2048 workgroups
        if (rowb > M) rowb = M;
        if (rowb > 65535) rowb = 65535;
        hipLaunchKernelGGL(splitk_epilogue_kernel, dim3((unsigned)colb, (unsigned)rowb), dim3(256), 0, s, t, precise ? 0 : 1);
        e = hipGetLastError();
        if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    }
    return FNN_OK;
}

// Codebook type: w[n,k] = scales[n, k/qblock] * codebook[nibble]  (to_f32_vec_codebook,
// src/packed_tensor.rs:469-521).  Expanded per call into a transient f16 operand: the row is scaled
// by a power of two (max |w| of the row into [2^14, 2^15)) and each value written as hi = f16(w'),
// lo = f16(w' - hi); hi and lo follow each other along K and the GEMM runs over both with the same
// activations, so the product keeps ~22 mantissa bits of the f32 weight.
__global__ void __launch_bounds__(256) expand_codebook_kernel(const uint32_t *words, const float *scales, const float *codebook,
                                                              int64_t rows, int64_t inner, int64_t kp, int64_t bpr, int qblock,
                                                              int64_t kpad, _Float16 *out, float *row_scale, float *row_zero)
{
    __shared__ float cb[16];
    __shared__ float red[4];
    const int64_t r = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    if (tid < 16) cb[tid] = codebook[tid];
    __syncthreads();
    float cbmax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) cbmax = fmaxf(cbmax, fabsf(cb[i]));
    float smax = 0.0f;
    for (int64_t b = tid; b < bpr; b += 256) smax = fmaxf(smax, fabsf(scales[r * bpr + b]));
    smax = wave_max(smax);
    if (lane == 0) red[wv] = smax;
    __syncthreads();
    const float mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])) * cbmax;   // bound of |w| on the row
    int e = 0;
    if (mx > 0.0f && mx < __builtin_huge_valf()) {
        int ex;
        (void)frexpf(mx, &ex);
        e = 15 - ex;
    }
    _Float16 *hi = out + r * 2 * kpad, *lo = hi + kpad;
    for (int64_t g = tid; g < kpad / 8; g += 256) {
        f16x8 h8, l8;
        const uint32_t wd = g < kp ? words[r * kp + g] : 0u;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int64_t k = g * 8 + j;
            float v = 0.0f;
            if (k < inner) v = scales[r * bpr + k / qblock] * cb[(wd >> (4 * j)) & 0xf];
            const float vs = ldexpf(v, e);
            const _Float16 hh = (_Float16)vs;
            h8[j] = hh;
            l8[j] = (_Float16)(vs - (float)hh);
        }
        *reinterpret_cast<f16x8 *>(hi + g * 8) = h8;
        *reinterpret_cast<f16x8 *>(lo + g * 8) = l8;
    }
    if (tid == 0) {
        row_scale[r] = ldexpf(1.0f, -e);
        row_zero[r] = 0.0f;
    }
}

int run_tiled_codebook(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q, int flags)
{
    const int64_t kpad = (q.k + BK - 1) / BK * BK;
    const size_t op_bytes = (size_t)q.n * 2 * kpad * 2;
    const size_t tab_off = (op_bytes + 255) / 256 * 256;
    const size_t total = tab_off + (size_t)q.n * 8 + 256;
    // The expansion is kept with the weight (eight times the packed bytes, what the CPU path spends on its
    // cached f32 copy); with FNN_OPT_CODEBOOK_CACHE = 0 a call expands into a workspace instead.
    const bool keep = fnn_ctx_option(ctx, FNN_OPT_CODEBOOK_CACHE) != 0;
    fnn_hip_weight *wm = const_cast<fnn_hip_weight *>(w);
    void *ws = keep && q.words == w->words ? wm->dense16 : nullptr;
    bool expand = true;
    if (ws) {
        expand = false;
    } else if (keep && q.words == w->words && !fnn_ctx_no_alloc(ctx)) {
        if (hipMalloc(&wm->dense16, total) != hipSuccess)
            return fnn_ctx_fail(ctx, FNN_ERR_MEMORY, "out of device memory (expanded codebook weight)");
        ws = wm->dense16;
    } else {
        int rc = fnn_ctx_ensure_tmp(ctx, 3, total, &ws);
        if (rc) return rc;
    }
    _Float16 *op = (_Float16 *)ws;
    float *row_scale = (float *)((char *)ws + tab_off), *row_zero = row_scale + q.n;
    if (expand) {
        hipLaunchKernelGGL(expand_codebook_kernel, dim3((unsigned)q.n), dim3(256), 0, s, q.words, q.scales, q.codebook, q.n, q.k,
                           q.kp, q.bpr, q.qblock, kpad, op, row_scale, row_zero);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    }
    DenseOperand d{(const uint32_t *)op, row_scale, row_zero};
    return run_tiled<DT_F16_DENSE>(ctx, s, w, q, flags, &d);
}

}  // namespace

// Mean lane value per weight row, built on the first single-f16 use of a weight whose lanes have a non-zero mean
// (asymmetric integer types, FP4): *umean stays null for the other types.
int fnn_row_means(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const float **umean)
{
    *umean = nullptr;
    const int dt = w->dtype;
    if (dt != FNN_DT_I8 && dt != FNN_DT_I4 && dt != FNN_DT_U8 && dt != FNN_DT_U4 && dt != FNN_DT_F4) return FNN_OK;
    fnn_hip_weight *wm = const_cast<fnn_hip_weight *>(w);
    if (!wm->umean) {
        if (fnn_ctx_no_alloc(ctx)) return fnn_ctx_fail(ctx, FNN_ERR_MEMORY, "first single-pass use of a weight while allocation is not allowed (graph capture, fnn_hip_qmatmul_static)");
        if (hipMalloc((void **)&wm->umean, (size_t)w->rows * 4 + 64) != hipSuccess)
            return fnn_ctx_fail(ctx, FNN_ERR_MEMORY, "out of device memory (row means)");
        hipError_t e;
        switch (dt) {
        case FNN_DT_I8: e = launch_umean<FNN_DT_I8>(w, wm->umean, s); break;
        case FNN_DT_I4: e = launch_umean<FNN_DT_I4>(w, wm->umean, s); break;
        case FNN_DT_U8: e = launch_umean<FNN_DT_U8>(w, wm->umean, s); break;
        case FNN_DT_U4: e = launch_umean<FNN_DT_U4>(w, wm->umean, s); break;
        default: e = launch_umean<FNN_DT_F4>(w, wm->umean, s); break;
        }
        if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    }
    *umean = wm->umean;
    return FNN_OK;
}

int fnn_tiled_qmatmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q, int flags, bool *handled)
{
    *handled = false;
    const int64_t min_m = fnn_ctx_option(ctx, FNN_OPT_TILE_MIN_M);
    if (q.m < min_m) return FNN_OK;
    if (w->dtype == FNN_DT_I4CB) {
        if (q.as_written || q.qblock <= 0 || q.n > (1 << 24) || q.m > (1 << 22)) return FNN_OK;
        // blocks of 32 values: nibbles decoded inside the tile kernel (4 bits per value cross the memory system instead
        // of the 32 of the expanded f16 hi + lo operand, and no expansion is kept with the weight); other block
        // sizes, or by option, the expanded operand.  Measured on 4096 x 4096 (us, in-kernel / expanded): M = 5 ... 16
        // 19-20 / 23-26, M = 32 23.3 / 24.5, M = 64 30.5 / 31.5, M = 128 41.2 / 42.4, M = 256 65.8 / 58.4, M = 1024
        // 191 / 207 (155 on the 256 x 128 tiles the expanded operand takes from M = 513 on; M = 640: 142 / 137, M = 2048:
        // 372 / 289); single rounding: M <= 16 20 / 24-27, M = 64 30.1 / 27.2, M = 256 48.3 / 46.2, M = 1024 119 / 99
        // (the per-block fold of the accumulator, 2 x 64 FMAs per wave and stage, and the look-ups make the loop
        // vector-ALU bound; the expanded operand's loop is the plain f16 one).
        const int64_t opt_exp = fnn_ctx_option(ctx, FNN_OPT_CODEBOOK_EXPANDED);
        const bool precise = !(flags & FNN_FLAG_ACT_F16_SINGLE);
        const bool in_kernel = opt_exp == 0 ? (precise ? q.m < 192 : q.m <= 16) : opt_exp == 2;
        if (q.qblock == 32 && in_kernel) {
            QMatmulArgs qa = q;
            int rc;
            if (q.words == w->words && (rc = fnn_aligned_rows(ctx, s, w, &qa.words, &qa.kp))) return rc;
            if (qa.kp % 4 == 0 && !(reinterpret_cast<uintptr_t>(qa.words) & 15)) {
                rc = run_tiled<FNN_DT_I4CB>(ctx, s, w, qa, flags);
                if (rc) return rc;
                *handled = true;
                return FNN_OK;
            }
        }
        int rc = run_tiled_codebook(ctx, s, w, q, flags);
        if (rc) return rc;
        *handled = true;
        return FNN_OK;
    }
    if (w->dtype < FNN_DT_I8 || w->dtype > FNN_DT_F4) return FNN_OK;
    if (q.m > (1 << 22) || q.n > (1 << 24)) return FNN_OK;      // 32-bit tile counts
    // the kernel fetches 16-byte pieces of a weight row: rows whose length is not a multiple of four words
    // are read from a re-strided copy (made once per weight)
    QMatmulArgs qa = q;
    int rc;
    if (q.words == w->words && (rc = fnn_aligned_rows(ctx, s, w, &qa.words, &qa.kp))) return rc;
    if (qa.kp % 4 != 0 || (reinterpret_cast<uintptr_t>(qa.words) & 15)) return FNN_OK;
    switch (w->dtype) {
    case FNN_DT_I8: rc = run_tiled<FNN_DT_I8>(ctx, s, w, qa, flags); break;
    case FNN_DT_I4: rc = run_tiled<FNN_DT_I4>(ctx, s, w, qa, flags); break;
    case FNN_DT_U8: rc = run_tiled<FNN_DT_U8>(ctx, s, w, qa, flags); break;
    case FNN_DT_U4: rc = run_tiled<FNN_DT_U4>(ctx, s, w, qa, flags); break;
    case FNN_DT_F8: rc = run_tiled<FNN_DT_F8>(ctx, s, w, qa, flags); break;
    case FNN_DT_F8R: rc = run_tiled<FNN_DT_F8R>(ctx, s, w, qa, flags); break;
    case FNN_DT_F4: rc = run_tiled<FNN_DT_F4>(ctx, s, w, qa, flags); break;
    default: return FNN_OK;
    }
    if (rc) return rc;
    *handled = true;
    return FNN_OK;
}
