// Bandwidth-bound fused dequant GEMV (M <= 4 activation rows) for gfx950.
//
// out[m,n] = act((sum_k A[m,k]*u(W[n,k]))*scale[n] + zero[n]*sum_k A[m,k] + bias[n])
// (gemm_batch_packed_simd + apply_affine_dot, src/backend/cpu/microkernels/gemm.rs:1982-2088,
//  src/backend/cpu/microkernels/mod.rs:283-295), weights in fastnn's row-major packed layout.
//
// Work decomposition (one workgroup = RB consecutive weight rows, all of K):
//   * a wave is 4 DPP rows of 16 lanes; DPP row `sub` works on weight row 4*rg+sub,
//     lane c of the DPP row owns 16 packed bytes at K offset c*EPL of the current chunk,
//     so one wave load instruction fetches four contiguous 256-byte row segments;
//   * K is cut into chunks of 16*EPL elements, chunk j belongs to wave j % NW: the
//     workgroup's waves split K, every packed byte is requested exactly once and the
//     activation slice a lane needs (EPL floats) is loaded once per chunk and reused
//     for all RG row groups;
//   * partial dots are reduced over the 16 lanes with DPP, then over waves through LDS
//     in a fixed order (deterministic), and the affine/bias/activation epilogue is fused.
// Algorithmic bytes per launch: N*K*bits/8 + side tables + 4*M*(K+N).
#include "common.h"

#include <cstdlib>

namespace {

template <int DT, int MT, int RG, int MAXT>
__global__ void __launch_bounds__(MAXT) qgemv_kernel(QMatmulArgs p)
{
    using C = Codec<DT>;
    constexpr int EPW = C::EPW;
    constexpr int EPL = 4 * EPW;   // elements behind one 16-byte lane load
    constexpr int CK = 16 * EPL;   // elements per chunk (one DPP row of 16 lanes)
    constexpr int RB = RG * 4;     // weight rows per workgroup
    constexpr int MAXW = MAXT / 64;

    __shared__ float part[MAXW][MT][RB];
    __shared__ float xpart[MAXW][MT];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = tid >> 6;
    const int nw = blockDim.x >> 6;
    const int sub = lane >> 4;
    const int c = lane & 15;
    const int64_t n0 = (int64_t)blockIdx.x * RB;
    const int64_t K = p.k, N = p.n, kp = p.kp;

    float acc[MT][RG];
    float xs[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) {
        xs[m] = 0.0f;
#pragma unroll
        for (int rg = 0; rg < RG; rg++) acc[m][rg] = 0.0f;
    }

    const int64_t nchunks = (K + CK - 1) / CK;
    for (int64_t j = wv; j < nchunks; j += nw) {
        const int64_t k0 = j * CK + (int64_t)c * EPL;
        const bool kvalid = k0 < K;  // K % EPL == 0: a lane's 16 bytes are all inside the row or all outside

        uint4 wr[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const int64_t row = n0 + rg * 4 + sub;
            wr[rg] = make_uint4(0, 0, 0, 0);
            if (kvalid && row < N) wr[rg] = *reinterpret_cast<const uint4 *>(p.words + row * kp + k0 / EPW);
        }

        float xv[MT][EPL];
#pragma unroll
        for (int m = 0; m < MT; m++) {
#pragma unroll
            for (int q = 0; q < EPL / 4; q++) {
                float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
                if (kvalid) t = *reinterpret_cast<const float4 *>(p.a + (int64_t)m * K + k0 + q * 4);
                xv[m][q * 4 + 0] = t.x;
                xv[m][q * 4 + 1] = t.y;
                xv[m][q * 4 + 2] = t.z;
                xv[m][q * 4 + 3] = t.w;
            }
            float s = 0.0f;
#pragma unroll
            for (int e = 0; e < EPL; e++) s += xv[m][e];
            xs[m] += s;
        }

#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const uint32_t w4[4] = {wr[rg].x, wr[rg].y, wr[rg].z, wr[rg].w};
            float dot[MT];
#pragma unroll
            for (int m = 0; m < MT; m++) dot[m] = 0.0f;
#pragma unroll
            for (int wd = 0; wd < 4; wd++) {
                float wf[EPW];
                C::decode(w4[wd], wf);
#pragma unroll
                for (int m = 0; m < MT; m++)
#pragma unroll
                    for (int e = 0; e < EPW; e++) dot[m] = fmaf(wf[e], xv[m][wd * EPW + e], dot[m]);
            }
#pragma unroll
            for (int m = 0; m < MT; m++) acc[m][rg] += dot[m];
        }
    }

#pragma unroll
    for (int m = 0; m < MT; m++) {
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            float v = row16_sum(acc[m][rg]);
            if (c == 0) part[wv][m][rg * 4 + sub] = v;
        }
        float v = row16_sum(xs[m]);
        if (lane == 0) xpart[wv][m] = v;
    }
    __syncthreads();

    for (int t = tid; t < MT * RB; t += blockDim.x) {
        const int m = t / RB, r = t % RB;
        const int64_t n = n0 + r;
        if (n >= N) continue;
        float dot = 0.0f, xsum = 0.0f;
        for (int w = 0; w < nw; w++) {
            dot += part[w][m][r];
            xsum += xpart[w][m];
        }
        const float res = fnn_epilogue(dot, p.scales[n], p.zeros[n], xsum, p.bias, n, p.act);
        p.out[(int64_t)m * N + n] = res;
    }
}

// Codebook weights (I4 indices, one 16-entry f32 codebook, one f32 scale per block of 32 k-values):
//   out[m,n] = act(sum_blk scales[n,blk] * sum_{k in blk} A[m,k]*codebook[idx(n,k)] + bias[n])
//   (PackedTensor::get_or_init_f32_weights, src/packed_tensor.rs:469-521, then the f32 MatMul)
// The table lookup costs what it costs (two address operations and one LDS read per element), so the kernel is
// organised around keeping many of them in flight: lane (sub, c) owns one block of row 4*rg + sub per chunk of 512
// k-values (its 16 bytes), all 32 lookups of a block are issued before the first is used and feed four independent
// accumulators.  The 16-entry table sits in 16 consecutive LDS banks: lanes that read the same entry share one
// broadcast, different entries never meet in a bank.  The chunk's activations are fetched once per wave (coalesced,
// 32 bytes per lane) and handed to the lanes through a wave-local LDS area laid out so that the 16 lanes of a DPP row
// read consecutive 16-byte pieces; wave w owns chunks w, w + NW, ...
template <int MT, int RG, int NW>
__global__ void __launch_bounds__(NW * 64) qgemv_codebook_kernel(QMatmulArgs p)
{
    constexpr int CK = 512;        // k-values per chunk: 16 lanes x one block of 32
    constexpr int RB = RG * 4;
    __shared__ float cb_s[16];
    __shared__ __attribute__((aligned(16))) float4 xs_s[NW][MT][128];   // [q][c] pieces: lane c's q-th float4 at q*16 + c
    __shared__ float part[NW][MT][RB];

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int sub = lane >> 4, c = lane & 15;
    const int64_t n0 = (int64_t)blockIdx.x * RB;
    const int64_t K = p.k, N = p.n, kp = p.kp;
    const int mreal = (int)p.m;

    if (tid < 16) cb_s[tid] = p.codebook[tid];
    __syncthreads();

    float acc[MT][RG];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int rg = 0; rg < RG; rg++) acc[m][rg] = 0.0f;

    const int64_t nchunks = (K + CK - 1) / CK;
    for (int64_t j = wv; j < nchunks; j += NW) {
        // ---- requests: this lane's 8 activations per row (clamped address, masked), then blocks and block scales
        const int64_t ka = j * CK + lane * 8;
        const int64_t kac = ka < K ? ka : K - 8;               // K % 32 == 0
        uint4 xa[MT][2];
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const int64_t mrow = m < mreal ? m : mreal - 1;
            const uint32_t keep = (m < mreal && ka < K) ? 0xffffffffu : 0u;
            xa[m][0] = *reinterpret_cast<const uint4 *>(p.a + mrow * K + kac);
            xa[m][1] = *reinterpret_cast<const uint4 *>(p.a + mrow * K + kac + 4);
            xa[m][0].x &= keep; xa[m][0].y &= keep; xa[m][0].z &= keep; xa[m][0].w &= keep;
            xa[m][1].x &= keep; xa[m][1].y &= keep; xa[m][1].z &= keep; xa[m][1].w &= keep;
        }
        const int64_t k0 = j * CK + (int64_t)c * 32;
        const int64_t k0c = k0 < K ? k0 : K - 32;              // a block past K re-reads the last block: its activations are 0
        uint4 wr[RG];
        float bs[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            int64_t row = n0 + rg * 4 + sub;
            if (row > N - 1) row = N - 1;
            wr[rg] = *reinterpret_cast<const uint4 *>(p.words + row * kp + k0c / 8);
            bs[rg] = p.scales[row * p.bpr + k0c / 32];
        }
        // ---- activations through the wave's LDS area: float4 f = 2*lane + h of the chunk belongs to lane c = f / 8 as its
        // q = f % 8 th piece
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int f = 2 * lane + h;
                xs_s[wv][m][(f & 7) * 16 + (f >> 3)] = __builtin_bit_cast(float4, xa[m][h]);
            }
        __builtin_amdgcn_wave_barrier();
        float xv[MT][32];
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const float4 t = xs_s[wv][m][q * 16 + c];
                xv[m][q * 4 + 0] = t.x; xv[m][q * 4 + 1] = t.y; xv[m][q * 4 + 2] = t.z; xv[m][q * 4 + 3] = t.w;
            }
        // ---- blocks: 32 lookups in flight, four accumulators per activation row
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const uint32_t w4[4] = {wr[rg].x, wr[rg].y, wr[rg].z, wr[rg].w};
            float wf[32];
#pragma unroll
            for (int wd = 0; wd < 4; wd++)
#pragma unroll
                for (int i = 0; i < 8; i++) wf[wd * 8 + i] = cb_s[(w4[wd] >> (4 * i)) & 0xf];
#pragma unroll
            for (int m = 0; m < MT; m++) {
                float d0 = 0.0f, d1 = 0.0f, d2 = 0.0f, d3 = 0.0f;
#pragma unroll
                for (int e = 0; e < 32; e += 4) {
                    d0 = fmaf(wf[e], xv[m][e], d0);
                    d1 = fmaf(wf[e + 1], xv[m][e + 1], d1);
                    d2 = fmaf(wf[e + 2], xv[m][e + 2], d2);
                    d3 = fmaf(wf[e + 3], xv[m][e + 3], d3);
                }
                acc[m][rg] = fmaf((d0 + d1) + (d2 + d3), bs[rg], acc[m][rg]);
            }
        }
        __builtin_amdgcn_wave_barrier();   // the wave's LDS area is rewritten by its next chunk
    }

#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const float v = row16_sum(acc[m][rg]);
            if (c == 0) part[wv][m][rg * 4 + sub] = v;
        }
    __syncthreads();
    for (int t = tid; t < MT * RB; t += NW * 64) {
        const int m = t / RB, r = t % RB;
        const int64_t n = n0 + r;
        if (n >= N || m >= mreal) continue;
        float dot = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; w++) dot += part[w][m][r];
        if (p.bias) dot = dot + p.bias[n];
        p.out[(int64_t)m * N + n] = fnn_activation(dot, p.act);
    }
}

template <int MT>
hipError_t launch_codebook(const QMatmulArgs &p, hipStream_t s)
{
    // 8 rows per workgroup while that leaves at most four workgroups per CU (measured on 4096 x 4096 at M = 1:
    // 4 rows 5.9 us, 8 rows 5.4 us, 16 rows 5.8 us, 32 rows 7.8 us), else 16; short K (<= 2048) runs four waves so that
    // none idles
    const bool wide = p.n > 8 * 1024;
    const unsigned grid = (unsigned)(wide ? (p.n + 15) / 16 : (p.n + 7) / 8);
    if (p.k <= 2048) {
        if (wide) hipLaunchKernelGGL((qgemv_codebook_kernel<MT, 4, 4>), dim3(grid), dim3(256), 0, s, p);
        else hipLaunchKernelGGL((qgemv_codebook_kernel<MT, 2, 4>), dim3(grid), dim3(256), 0, s, p);
    } else {
        if (wide) hipLaunchKernelGGL((qgemv_codebook_kernel<MT, 4, 8>), dim3(grid), dim3(512), 0, s, p);
        else hipLaunchKernelGGL((qgemv_codebook_kernel<MT, 2, 8>), dim3(grid), dim3(512), 0, s, p);
    }
    return hipGetLastError();
}

template <int DT, int MT, int RG, int MAXT>
hipError_t launch_one(const QMatmulArgs &p, int nw, hipStream_t s)
{
    constexpr int RB = RG * 4;
    const int64_t grid = (p.n + RB - 1) / RB;
    if (nw * 64 > MAXT) nw = MAXT / 64;
    hipLaunchKernelGGL((qgemv_kernel<DT, MT, RG, MAXT>), dim3((unsigned)grid), dim3(nw * 64), 0, s, p);
    return hipGetLastError();
}

template <int DT, int MT>
hipError_t launch_rg(const QMatmulArgs &p, hipStream_t s)
{
    constexpr int EPL = 4 * Codec<DT>::EPW;
    constexpr int CK = 16 * EPL;
    const int64_t nchunks = (p.k + CK - 1) / CK;
    // 4-bit lanes keep 32 activations per row in registers: cap the block at 8 waves there.
    constexpr int MAXT = (EPL * MT <= 32) ? 1024 : 512;
    int nw = (int)(nchunks < MAXT / 64 ? nchunks : MAXT / 64);
    if (nw < 1) nw = 1;
    // rows per workgroup: enough workgroups to give every CU (256) a few.
    int rg = (p.n >= 16384) ? 8 : 4;
    if (p.n <= 1024) rg = 2;
    switch (rg) {
    case 2: return launch_one<DT, MT, 2, MAXT>(p, nw, s);
    case 8: return launch_one<DT, MT, 8, MAXT>(p, nw, s);
    default: return launch_one<DT, MT, 4, MAXT>(p, nw, s);
    }
}

template <int DT>
hipError_t launch_dt(const QMatmulArgs &p0, hipStream_t s)
{
    // 4-bit types hold 32 activations per lane and row: at most 2 rows per pass; 8-bit: 4.
    constexpr int MTMAX = (Codec<DT>::EPW == 8) ? 2 : 4;
    QMatmulArgs p = p0;
    int64_t m0 = 0;
    while (m0 < p0.m) {
        int64_t mt = p0.m - m0;
        if (mt > MTMAX) mt = MTMAX;
        p.a = p0.a + m0 * p0.k;
        p.out = p0.out + m0 * p0.n;
        p.m = mt;
        hipError_t e;
        if (mt == 1) e = launch_rg<DT, 1>(p, s);
        else if (mt == 2) e = launch_rg<DT, 2>(p, s);
        else if constexpr (MTMAX >= 4) {
            if (mt == 3) e = launch_rg<DT, 3>(p, s);
            else e = launch_rg<DT, 4>(p, s);
        } else e = hipErrorInvalidValue;
        if (e != hipSuccess) return e;
        m0 += mt;
    }
    return hipSuccess;
}

}  // namespace

// Takes the call when the layout allows 16-byte lane loads: every row a multiple of
// 16 bytes (kp % 4 == 0), K a multiple of the lane's element count, 16-byte aligned
// activation rows, block size 32 for the codebook type.  *handled = false otherwise.
hipError_t launch_qgemv(int dtype, const QMatmulArgs &p, hipStream_t s, bool *handled)
{
    *handled = false;
    if (p.m < 1 || p.m > 4 || p.as_written) return hipSuccess;
    const int epw = (dtype == FNN_DT_I8 || dtype == FNN_DT_U8 || dtype == FNN_DT_F8 ||
                     dtype == FNN_DT_F8R) ? 4 : 8;
    const int epl = 4 * epw;
    if (p.kp % 4 != 0 || p.k % epl != 0 || p.k % 4 != 0) return hipSuccess;
    if ((reinterpret_cast<uintptr_t>(p.a) & 15) || (reinterpret_cast<uintptr_t>(p.words) & 15))
        return hipSuccess;
    if (dtype == FNN_DT_I4CB && p.qblock != 32) return hipSuccess;
    *handled = true;
    switch (dtype) {
    case FNN_DT_I8: return launch_dt<FNN_DT_I8>(p, s);
    case FNN_DT_I4: return launch_dt<FNN_DT_I4>(p, s);
    case FNN_DT_U8: return launch_dt<FNN_DT_U8>(p, s);
    case FNN_DT_U4: return launch_dt<FNN_DT_U4>(p, s);
    case FNN_DT_F8: return launch_dt<FNN_DT_F8>(p, s);
    case FNN_DT_F8R: return launch_dt<FNN_DT_F8R>(p, s);
    case FNN_DT_F4: return launch_dt<FNN_DT_F4>(p, s);
    case FNN_DT_I4CB: {
        // up to four activation rows in one pass: the looked-up block values are used by every row (a lane keeps 32
        // activations per row in registers: 128 at four rows)
        const hipError_t e = p.m == 1 ? launch_codebook<1>(p, s) : (p.m == 2 ? launch_codebook<2>(p, s) : (p.m == 3 ? launch_codebook<3>(p, s) : launch_codebook<4>(p, s)));
        if (e != hipSuccess) return e;
        return hipSuccess;
    }
    default: *handled = false; return hipSuccess;
    }
}
