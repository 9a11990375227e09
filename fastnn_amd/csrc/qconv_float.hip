// Conv2d for the weight types that have no integer kernel (U8, U4, F8, F8R, F4, 4-bit codebook):
// the CPU backend dequantises such weights once and runs an f32 im2col convolution
// (src/backend/cpu/mod.rs:4204-4257, src/backend/cpu/microkernels/conv.rs:509-660).  Here the
// im2col matrix [B*Ho*Wo, C/g*KH*KW] is written as f32 rows, the fused-dequant MatMul kernels
// multiply it with the packed weight rows (bias and activation in their epilogue), and the
// [pixel, channel] result is turned into NCHW.
#include "common.h"

namespace {

// col[r, e] = x[b, g*cg + ic, oh*s + i*d - pad, ow*s + j*d - pad] (0 outside), r = b*np + oh*wo + ow,
// e = (ic*KH + i)*KW + j (src/backend/cpu/im2col.rs:32-52).  Consecutive lanes take consecutive e.
__global__ void __launch_bounds__(256) im2col_f32_kernel(const float *x, float *col, int64_t rows, int64_t np, int64_t wo,
                                                         int64_t c, int64_t cg, int g, int64_t h, int64_t w, int kh, int kw,
                                                         int stride, int pad, int dil, int64_t kk)
{
    const int64_t total = rows * kk;
    const int khw = kh * kw;
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int64_t r = idx / kk;
        const int e = (int)(idx - r * kk);
        const int64_t nn = r / np, p = r - nn * np;
        const int64_t oh = p / wo, ow = p - oh * wo;
        const int ic = e / khw, rem = e - ic * khw;
        const int i = rem / kw, j = rem - i * kw;
        const int64_t ih = oh * stride + (int64_t)i * dil - pad, iw = ow * stride + (int64_t)j * dil - pad;
        float v = 0.0f;
        if (ih >= 0 && ih < h && iw >= 0 && iw < w) v = x[((nn * c + (int64_t)g * cg + ic) * h + ih) * w + iw];
        col[idx] = v;
    }
}

// y[b, ch0 + f, p] = rows_out[(b*np + p)*ocg + f]: 32x32 tiles through LDS so that both sides coalesce
__global__ void __launch_bounds__(256) rows_to_nchw_kernel(const float *src, float *y, int64_t np, int64_t oc, int64_t ch0, int64_t ocg)
{
    __shared__ float tile[32][33];
    const int64_t nn = blockIdx.z;
    const int64_t p0 = (int64_t)blockIdx.x * 32, f0 = (int64_t)blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int64_t p = p0 + ty + 8 * k, f = f0 + tx;
        tile[ty + 8 * k][tx] = (p < np && f < ocg) ? src[(nn * np + p) * ocg + f] : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int64_t f = f0 + ty + 8 * k, p = p0 + tx;
        if (f < ocg && p < np) y[(nn * oc + ch0 + f) * np + p] = tile[tx][ty + 8 * k];
    }
}

}  // namespace

hipError_t launch_im2col_f32(const float *x, float *col, int64_t b, int64_t c, int groups, int g, int64_t h, int64_t w,
                             int64_t ho, int64_t wo, int kh, int kw, int stride, int pad, int dil, hipStream_t s)
{
    const int64_t cg = c / groups, kk = cg * kh * kw, np = ho * wo, rows = b * np;
    int64_t blocks = (rows * kk + 255) / 256;
    if (blocks > 65535 * 16) blocks = 65535 * 16;
    if (blocks < 1) return hipSuccess;
    hipLaunchKernelGGL(im2col_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, s, x, col, rows, np, wo, c, cg, g, h, w, kh, kw,
                       stride, pad, dil, kk);
    return hipGetLastError();
}

hipError_t launch_rows_to_nchw(const float *src, float *y, int64_t b, int64_t np, int64_t oc, int64_t ch0, int64_t ocg, hipStream_t s)
{
    if (b < 1 || np < 1 || ocg < 1) return hipSuccess;
    if (b > 65535 || (ocg + 31) / 32 > 65535) return hipErrorInvalidValue;
    const dim3 grid((unsigned)((np + 31) / 32), (unsigned)((ocg + 31) / 32), (unsigned)b);
    hipLaunchKernelGGL(rows_to_nchw_kernel, grid, dim3(256), 0, s, src, y, np, oc, ch0, ocg);
    return hipGetLastError();
}
