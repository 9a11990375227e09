// Shape-agnostic quantised MatMul and dequantise kernels for gfx950.
//
// The generic MatMul takes any K (ragged tail words, rows that are not 16-byte
// multiples), any codebook block size and the as-written codebook variant; it is the
// fallback behind the vectorised GEMV and the MFMA GEMM.  One wave per weight row and
// tile of 4 activation rows; lanes stride over the row's packed words.
#include "common.h"

namespace {

constexpr int GEN_MT = 4;

template <int DT>
__global__ void __launch_bounds__(256) qgemm_generic_kernel(QMatmulArgs p)
{
    using C = Codec<DT>;
    constexpr int EPW = C::EPW;
    constexpr bool CB = (DT == FNN_DT_I4CB);
    __shared__ float cb_s[16];
    if (CB) {
        if (threadIdx.x < 16) cb_s[threadIdx.x] = p.codebook[threadIdx.x];
        __syncthreads();
    }
    const int lane = threadIdx.x & 63;
    const int64_t n = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t m0 = (int64_t)blockIdx.y * GEN_MT;
    if (n >= p.n) return;
    const int64_t K = p.k;
    float acc[GEN_MT], xs[GEN_MT];
#pragma unroll
    for (int m = 0; m < GEN_MT; m++) acc[m] = xs[m] = 0.0f;

    for (int64_t wd = lane; wd < p.kp; wd += 64) {
        float wf[EPW];
        if constexpr (CB) {
            if (p.as_written) {
                // the [N,K] dequantised buffer read as a row-major [K,N] matrix:
                // B[k][n] = deq_flat[k*N + n]; this lane covers k = wd*8 .. wd*8+7 of column n
#pragma unroll
                for (int e = 0; e < EPW; e++) {
                    int64_t kk = wd * EPW + e;
                    wf[e] = 0.0f;
                    if (kk < K) {
                        int64_t flat = kk * p.n + n;  // K == N enforced by the caller
                        int64_t r = flat / K, cc = flat % K;
                        uint32_t w = p.words[r * p.kp + cc / 8];
                        wf[e] = p.scales[r * p.bpr + cc / p.qblock] * cb_s[(w >> (4 * (cc % 8))) & 0xf];
                    }
                }
            } else {
                const uint32_t w = p.words[n * p.kp + wd];
#pragma unroll
                for (int e = 0; e < EPW; e++) {
                    int64_t kk = wd * EPW + e;
                    float sc = (kk < K) ? p.scales[n * p.bpr + kk / p.qblock] : 0.0f;
                    wf[e] = sc * cb_s[(w >> (4 * e)) & 0xf];
                }
            }
        } else {
            C::decode(p.words[n * p.kp + wd], wf);
        }
#pragma unroll
        for (int e = 0; e < EPW; e++) {
            const int64_t kk = wd * EPW + e;
            if (kk < K) {
#pragma unroll
                for (int m = 0; m < GEN_MT; m++) {
                    if (m0 + m < p.m) {
                        float x = p.a[(m0 + m) * K + kk];
                        acc[m] = fmaf(wf[e], x, acc[m]);
                        xs[m] += x;
                    }
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < GEN_MT; m++) {
        float d = wave_sum(acc[m]);
        float s = wave_sum(xs[m]);
        if (lane == 0 && m0 + m < p.m) {
            float res;
            if constexpr (CB) {
                float v = d;
                if (p.bias) v = v + p.bias[n];
                res = fnn_activation(v, p.act);
            } else {
                res = fnn_epilogue(d, p.scales[n], p.zeros[n], s, p.bias, n, p.act);
            }
            p.out[(m0 + m) * p.n + n] = res;
        }
    }
}

// out[r, c] = u(W[r,c]) * scale[r] + zero[r]   (one IEEE multiply and one add, not fused)
template <int DT>
__global__ void __launch_bounds__(256)
dequant_kernel(const uint32_t *words, const float *scales, const float *zeros,
               const float *codebook, int64_t rows, int64_t inner, int64_t kp, int64_t bpr,
               int qblock, float *out)
{
    using C = Codec<DT>;
    constexpr int EPW = C::EPW;
    const int64_t total = rows * kp;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / kp, wd = i % kp;
        const uint32_t w = words[i];
        float wf[EPW];
        if constexpr (DT == FNN_DT_I4CB) {
#pragma unroll
            for (int e = 0; e < EPW; e++) {
                int64_t cc = wd * EPW + e;
                if (cc < inner) out[r * inner + cc] = scales[r * bpr + cc / qblock] * codebook[(w >> (4 * e)) & 0xf];
            }
        } else {
            C::decode(w, wf);
            const float s = scales[r], z = zeros[r];
#pragma unroll
            for (int e = 0; e < EPW; e++) {
                int64_t cc = wd * EPW + e;
                if (cc < inner) out[r * inner + cc] = wf[e] * s + z;
            }
        }
    }
}

template <int DT>
hipError_t launch_generic_dt(const QMatmulArgs &p, hipStream_t s)
{
    const int wpb = 4;
    dim3 grid((unsigned)((p.n + wpb - 1) / wpb), (unsigned)((p.m + GEN_MT - 1) / GEN_MT));
    hipLaunchKernelGGL((qgemm_generic_kernel<DT>), grid, dim3(wpb * 64), 0, s, p);
    return hipGetLastError();
}

template <int DT>
hipError_t launch_dequant_dt(const fnn_hip_weight *w, float *out, hipStream_t s)
{
    int64_t total = w->rows * w->kp;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65535) blocks = 65535;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL((dequant_kernel<DT>), dim3((unsigned)blocks), dim3(256), 0, s, w->words,
                       w->scales, w->zeros, w->codebook, w->rows, w->inner, w->kp, w->bpr,
                       w->qblock, out);
    return hipGetLastError();
}

}  // namespace

#define FNN_DISPATCH_DT(dt, CALL)                                   \
    switch (dt) {                                                   \
    case FNN_DT_I8: return CALL(FNN_DT_I8);                         \
    case FNN_DT_I4: return CALL(FNN_DT_I4);                         \
    case FNN_DT_U8: return CALL(FNN_DT_U8);                         \
    case FNN_DT_U4: return CALL(FNN_DT_U4);                         \
    case FNN_DT_F8: return CALL(FNN_DT_F8);                         \
    case FNN_DT_F8R: return CALL(FNN_DT_F8R);                       \
    case FNN_DT_F4: return CALL(FNN_DT_F4);                         \
    case FNN_DT_I4CB: return CALL(FNN_DT_I4CB);                     \
    default: return hipErrorInvalidValue;                           \
    }

hipError_t launch_qgemm_generic(int dtype, const QMatmulArgs &p, hipStream_t s)
{
#define CALL_GEN(D) launch_generic_dt<D>(p, s)
    FNN_DISPATCH_DT(dtype, CALL_GEN)
#undef CALL_GEN
}

hipError_t launch_dequant(const fnn_hip_weight *w, float *out, hipStream_t s)
{
#define CALL_DQ(D) launch_dequant_dt<D>(w, out, s)
    FNN_DISPATCH_DT(w->dtype, CALL_DQ)
#undef CALL_DQ
}
