// f32 kernels that sit between quantised layers in a plan: elementwise
// ("add_f32", "relu_f32", "gelu_f32", "silu_f32"; src/backend/cpu/mod.rs:2699-2751) and data movement
// ("concat" :4267-4324, "slice_f32" :4721-4760, "pool_f32" max :4362-4397 with
// microkernels/ops.rs:104-158, "upsample_nearest2d" :5496-5535 with microkernels/misc.rs:338-364).
#include "common.h"

#include "../../include/fastnn_hip_backend.h"

namespace {
__global__ void __launch_bounds__(256) eltwise_kernel(int op, const float *a, const float *b, uint64_t nb, float *out, uint64_t n)
{
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
        float v = a[i];
        if (op == 0) v = v + b[i % nb];
        else v = fnn_activation(v, op);
        out[i] = v;
    }
}
__global__ void __launch_bounds__(256) fill_kernel(float *dst, uint64_t n, float value)
{
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) dst[i] = value;
}
// height rows of width values: dst[r*dst_pitch + c] = src[r*src_pitch + c], clamped to both lengths
// (the block copies of "concat" and "slice_f32")
__global__ void __launch_bounds__(256) copy2d_kernel(float *dst, uint64_t dst_pitch, uint64_t dst_len, const float *src,
                                                     uint64_t src_pitch, uint64_t src_len, uint64_t width, uint64_t height)
{
    const uint64_t total = width * height;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t r = i / width, c = i - r * width;
        const uint64_t si = r * src_pitch + c, di = r * dst_pitch + c;
        if (si < src_len && di < dst_len) dst[di] = src[si];
    }
}

// window maximum from -inf with a strict `>` (a NaN never wins), taps in the padding skipped
// indices (nullable): window position kh*kernel + kw of the first strict maximum in (kh, kw) order, 0 when no tap
// lies inside the image; an output position is visited when it lies inside the value slice or the index slice
__global__ void __launch_bounds__(256) maxpool2d_kernel(const float *x, uint64_t in_len, float *y, uint64_t out_len, uint64_t c,
                                                        uint64_t h, uint64_t w, uint64_t ho, uint64_t wo, int kernel, int stride, int pad,
                                                        int64_t *indices, uint64_t idx_len)
{
    const uint64_t total = out_len > idx_len ? out_len : idx_len;
    for (uint64_t o = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t ww = o % wo, t = o / wo, hh = t % ho, nc = t / ho;   // nc = n*c + channel
        float val = -INFINITY;
        int best = 0;
        for (int kh = 0; kh < kernel; kh++) {
            const int64_t hi = (int64_t)(hh * stride) + kh - pad;
            if (hi < 0 || hi >= (int64_t)h) continue;
            for (int kw = 0; kw < kernel; kw++) {
                const int64_t wi = (int64_t)(ww * stride) + kw - pad;
                if (wi < 0 || wi >= (int64_t)w) continue;
                const uint64_t idx = (nc * h + (uint64_t)hi) * w + (uint64_t)wi;
                if (idx < in_len) {
                    const float v = x[idx];
                    if (v > val) { val = v; best = kh * kernel + kw; }
                }
            }
        }
        if (o < out_len) y[o] = val;
        if (o < idx_len) indices[o] = best;
    }
    (void)c;
}

// window mean over the taps inside the image (padding taps neither add nor count), summed in (kh, kw) order
__global__ void __launch_bounds__(256) avgpool2d_kernel(const float *x, uint64_t in_len, float *y, uint64_t out_len,
                                                        uint64_t h, uint64_t w, uint64_t ho, uint64_t wo, int kernel, int stride, int pad)
{
    for (uint64_t o = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; o < out_len; o += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t ww = o % wo, t = o / wo, hh = t % ho, nc = t / ho;
        float val = 0.0f;
        int count = 0;
        for (int kh = 0; kh < kernel; kh++) {
            const int64_t hi = (int64_t)(hh * stride) + kh - pad;
            if (hi < 0 || hi >= (int64_t)h) continue;
            for (int kw = 0; kw < kernel; kw++) {
                const int64_t wi = (int64_t)(ww * stride) + kw - pad;
                if (wi < 0 || wi >= (int64_t)w) continue;
                const uint64_t idx = (nc * h + (uint64_t)hi) * w + (uint64_t)wi;
                if (idx < in_len) {
                    val += x[idx];
                    count++;
                }
            }
        }
        if (count > 0) val /= (float)count;
        y[o] = val;
    }
}

__global__ void __launch_bounds__(256) upsample_nearest2d_kernel(const float *x, float *y, uint64_t total, uint64_t h, uint64_t w, int sh, int sw)
{
    const uint64_t wo = w * sw, ho = h * sh;
    for (uint64_t o = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t ow = o % wo, t = o / wo, oh = t % ho, nc = t / ho;
        y[o] = x[(nc * h + oh / sh) * w + ow / sw];
    }
}
}  // namespace

static unsigned grid_for(uint64_t n)
{
    uint64_t blocks = (n + 255) / 256;
    return (unsigned)(blocks > 8192 ? 8192 : (blocks < 1 ? 1 : blocks));
}

hipError_t launch_copy2d(float *dst, uint64_t dst_pitch, uint64_t dst_len, const float *src, uint64_t src_pitch, uint64_t src_len,
                         uint64_t width, uint64_t height, hipStream_t s)
{
    if (width == 0 || height == 0) return hipSuccess;
    hipLaunchKernelGGL(copy2d_kernel, dim3(grid_for(width * height)), dim3(256), 0, s, dst, dst_pitch, dst_len, src, src_pitch, src_len, width, height);
    return hipGetLastError();
}

hipError_t launch_maxpool2d(const float *x, uint64_t in_len, float *y, uint64_t out_len, uint64_t c, uint64_t h, uint64_t w,
                            uint64_t ho, uint64_t wo, int kernel, int stride, int pad, int64_t *indices, uint64_t idx_len, hipStream_t s)
{
    if (!indices) idx_len = 0;
    const uint64_t total = out_len > idx_len ? out_len : idx_len;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(maxpool2d_kernel, dim3(grid_for(total)), dim3(256), 0, s, x, in_len, y, out_len, c, h, w, ho, wo, kernel, stride, pad,
                       indices, idx_len);
    return hipGetLastError();
}

hipError_t launch_avgpool2d(const float *x, uint64_t in_len, float *y, uint64_t out_len, uint64_t h, uint64_t w,
                            uint64_t ho, uint64_t wo, int kernel, int stride, int pad, hipStream_t s)
{
    if (out_len == 0) return hipSuccess;
    hipLaunchKernelGGL(avgpool2d_kernel, dim3(grid_for(out_len)), dim3(256), 0, s, x, in_len, y, out_len, h, w, ho, wo, kernel, stride, pad);
    return hipGetLastError();
}

hipError_t launch_upsample_nearest2d(const float *x, float *y, uint64_t nc, uint64_t h, uint64_t w, int sh, int sw, hipStream_t s)
{
    const uint64_t total = nc * h * sh * w * sw;
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(upsample_nearest2d_kernel, dim3(grid_for(total)), dim3(256), 0, s, x, y, total, h, w, sh, sw);
    return hipGetLastError();
}

hipError_t launch_fill(float *dst, uint64_t n, float value, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    uint64_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks), dim3(256), 0, s, dst, n, value);
    return hipGetLastError();
}

hipError_t launch_eltwise(int op, const float *a, const float *b, uint64_t nb, float *out, uint64_t n, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    uint64_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(eltwise_kernel, dim3((unsigned)blocks), dim3(256), 0, s, op, a, b, nb, out, n);
    return hipGetLastError();
}
