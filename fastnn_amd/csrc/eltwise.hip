// f32 kernels that sit between quantised layers in a plan: elementwise
// ("add_f32", "relu_f32", "gelu_f32", "silu_f32"; src/backend/cpu/mod.rs:2699-2751) and data movement
// ("concat" :4267-4324, "slice_f32" :4721-4760, "pool_f32" max :4362-4397 with
// microkernels/ops.rs:104-158, "upsample_nearest2d" :5496-5535 with microkernels/misc.rs:338-364).
#include "common.h"
#include "range_io.h"

#include "../../include/fastnn_hip_backend.h"

namespace {
// Partial value ranges of what a launch writes, for the quantised Conv2d that reads the tensor next (range_io.h): with
// a table the grid is (blocks, images), block (x, y) walks the values of image y only and leaves their (min, max) in
// pair slot0 + x of that image; without one the grid is (blocks, 1) and the whole output counts as one image.
struct RangeEmit {
    float *table;           // [images][stride][2], or null
    uint64_t image_elems;   // output values per image
    int stride, slot0;
};

__device__ __forceinline__ void emit_range(const RangeEmit &re, float mn, float mx)
{
    __shared__ float smn[4], smx[4];
    mn = wave_min(mn);
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) { smn[threadIdx.x >> 6] = mn; smx[threadIdx.x >> 6] = mx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float *d = re.table + ((uint64_t)blockIdx.y * re.stride + re.slot0 + blockIdx.x) * 2;
        d[0] = fminf(fminf(smn[0], smn[1]), fminf(smn[2], smn[3]));
        d[1] = fmaxf(fmaxf(smx[0], smx[1]), fmaxf(smx[2], smx[3]));
    }
}

__global__ void __launch_bounds__(256) eltwise_kernel(int op, const float *a, const float *b, uint64_t nb, float *out, uint64_t n)
{
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
        float v = a[i];
        if (op == 0) v = v + b[nb >= n ? i : i % nb];   // (the usual residual add has operands of one length: no division)
        else v = fnn_activation(v, op);
        out[i] = v;
    }
}
// The same with ranges: block (x, y) takes 1024 * U consecutive values of image y, every thread requests its 4 * U
// operands before it uses the first one.
template <int U>
__global__ void __launch_bounds__(256) eltwise_ranges_kernel(int op, const float *a, const float *b, uint64_t nb, float *out, uint64_t n, RangeEmit re)
{
    const uint64_t base = (uint64_t)blockIdx.y * re.image_elems, j0 = (uint64_t)blockIdx.x * (1024 * U) + threadIdx.x;
    float va[4 * U], vb[4 * U];
#pragma unroll
    for (int k = 0; k < 4 * U; k++) {
        const uint64_t j = j0 + (uint64_t)k * 256;
        const bool in = j < re.image_elems;
        va[k] = in ? a[base + j] : 0.0f;
        vb[k] = (in && op == 0) ? b[nb >= n ? base + j : (base + j) % nb] : 0.0f;
    }
    float mn = INFINITY, mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < 4 * U; k++) {
        const uint64_t j = j0 + (uint64_t)k * 256;
        if (j >= re.image_elems) continue;
        const float v = op == 0 ? va[k] + vb[k] : fnn_activation(va[k], op);
        out[base + j] = v;
        mn = fminf(mn, v);
        mx = fmaxf(mx, v);
    }
    if (re.table) emit_range(re, mn, mx);
}
__global__ void __launch_bounds__(256) fill_kernel(float *dst, uint64_t n, float value)
{
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) dst[i] = value;
}
// height rows of width values: dst[r*dst_pitch + c] = src[r*src_pitch + c], clamped to both lengths
// (the block copies of "concat" and "slice_f32").
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
// The same with ranges, one image per row, nothing clipped: block (x, y) takes 1024 * U consecutive values of row y,
// every thread requests its 4 * U values before it stores the first one (V4: as U 16-byte accesses, for rows that
// start on 16-byte boundaries and hold a multiple of four values).
template <int U, bool V4>
__global__ void __launch_bounds__(256) copy2d_ranges_kernel(float *dst, uint64_t dst_pitch, const float *src, uint64_t src_pitch, uint64_t width,
                                                            RangeEmit re)
{
    const float *s = src + (uint64_t)blockIdx.y * src_pitch;
    float *d = dst + (uint64_t)blockIdx.y * dst_pitch;
    float mn = INFINITY, mx = -INFINITY;
    if constexpr (V4) {
        const uint64_t c0 = ((uint64_t)blockIdx.x * (256 * U) + threadIdx.x) * 4;
        float4 v[U];
#pragma unroll
        for (int k = 0; k < U; k++) {
            const uint64_t c = c0 + (uint64_t)k * 1024;
            v[k] = c < width ? *reinterpret_cast<const float4 *>(s + c) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int k = 0; k < U; k++) {
            const uint64_t c = c0 + (uint64_t)k * 1024;
            if (c >= width) continue;
            *reinterpret_cast<float4 *>(d + c) = v[k];
            mn = fminf(fminf(mn, fminf(v[k].x, v[k].y)), fminf(v[k].z, v[k].w));
            mx = fmaxf(fmaxf(mx, fmaxf(v[k].x, v[k].y)), fmaxf(v[k].z, v[k].w));
        }
    } else {
        const uint64_t c0 = (uint64_t)blockIdx.x * (1024 * U) + threadIdx.x;
        float v[4 * U];
#pragma unroll
        for (int k = 0; k < 4 * U; k++) {
            const uint64_t c = c0 + (uint64_t)k * 256;
            v[k] = c < width ? s[c] : 0.0f;
        }
#pragma unroll
        for (int k = 0; k < 4 * U; k++) {
            const uint64_t c = c0 + (uint64_t)k * 256;
            if (c >= width) continue;
            d[c] = v[k];
            mn = fminf(mn, v[k]);
            mx = fmaxf(mx, v[k]);
        }
    }
    if (re.table) emit_range(re, mn, mx);
}

// "concat" along a middle axis in one launch: part j contributes `width[j]` values per outer position, stored at
// offset off[j] of the destination's row; grid (blocks of 1024 values, outer positions, parts), blocks past a part's
// width leave at once.  With ranges (one image per outer position) part j's pairs start at pair blk0[j].
constexpr int CONCAT_MAX_PARTS = 8;
struct ConcatArgs {
    const float *src[CONCAT_MAX_PARTS];
    uint64_t width[CONCAT_MAX_PARTS], off[CONCAT_MAX_PARTS];
    uint32_t blk0[CONCAT_MAX_PARTS];
};
template <bool V4>
__global__ void __launch_bounds__(256) concat_kernel(float *dst, uint64_t dst_pitch, ConcatArgs a, RangeEmit re)
{
    const int part = blockIdx.z;
    const uint64_t width = a.width[part];
    if ((uint64_t)blockIdx.x * 1024 >= width) return;   // (workgroup-uniform)
    const float *s = a.src[part] + (uint64_t)blockIdx.y * width;
    float *d = dst + (uint64_t)blockIdx.y * dst_pitch + a.off[part];
    float mn = INFINITY, mx = -INFINITY;
    if constexpr (V4) {
        const uint64_t c = ((uint64_t)blockIdx.x * 256 + threadIdx.x) * 4;
        if (c < width) {
            const float4 v = *reinterpret_cast<const float4 *>(s + c);
            *reinterpret_cast<float4 *>(d + c) = v;
            mn = fminf(fminf(v.x, v.y), fminf(v.z, v.w));
            mx = fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w));
        }
    } else {
        const uint64_t c0 = (uint64_t)blockIdx.x * 1024 + threadIdx.x;
        float v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = c0 + k * 256 < width ? s[c0 + k * 256] : 0.0f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            if (c0 + k * 256 >= width) continue;
            d[c0 + k * 256] = v[k];
            mn = fminf(mn, v[k]);
            mx = fmaxf(mx, v[k]);
        }
    }
    if (re.table) {
        re.slot0 += (int)a.blk0[part];
        emit_range(re, mn, mx);
    }
}

// window maximum from -inf with a strict `>` (a NaN never wins), taps in the padding skipped
// indices (nullable): window position kh*kernel + kw of the first strict maximum in (kh, kw) order, 0 when no tap
// lies inside the image; an output position is visited when it lies inside the value slice or the index slice
__global__ void __launch_bounds__(256) maxpool2d_kernel(const float *x, uint64_t in_len, float *y, uint64_t out_len, uint64_t c,
                                                        uint64_t h, uint64_t w, uint64_t ho, uint64_t wo, int kernel, int stride, int pad,
                                                        int64_t *indices, uint64_t idx_len, RangeEmit re)
{
    const uint64_t total = out_len > idx_len ? out_len : idx_len;
    const uint64_t ie = re.table ? re.image_elems : total, base = (uint64_t)blockIdx.y * ie;
    float mn = INFINITY, mx = -INFINITY;
    for (uint64_t j = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; j < ie && base + j < total; j += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t o = base + j;
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
        if (o < out_len) {
            y[o] = val;
            mn = fminf(mn, val);
            mx = fmaxf(mx, val);
        }
        if (o < idx_len) indices[o] = best;
    }
    if (re.table) emit_range(re, mn, mx);
    (void)c;
}

// The same for tensors below 2^31 values: 32-bit index arithmetic, divisions by multiplication.
__global__ void __launch_bounds__(256) maxpool2d_small_kernel(const float *x, uint32_t in_len, float *y, uint32_t out_len, uint32_t h, uint32_t w,
                                                              FastDiv ho, FastDiv wo, int kernel, int stride, int pad, int64_t *indices,
                                                              uint32_t idx_len, RangeEmit re)
{
    const uint32_t total = out_len > idx_len ? out_len : idx_len;
    const uint32_t ie = re.table ? (uint32_t)re.image_elems : total, base = blockIdx.y * ie;
    float mn = INFINITY, mx = -INFINITY;
    for (uint32_t j = blockIdx.x * 256 + threadIdx.x; j < ie && base + j < total; j += gridDim.x * 256) {
        const uint32_t o = base + j;
        const uint32_t t = wo.div(o), ww = o - t * wo.d, nc = ho.div(t), hh = t - nc * ho.d;
        const int h0 = (int)(hh * stride) - pad, w0 = (int)(ww * stride) - pad;
        const uint64_t chan0 = (uint64_t)nc * h * w;   // this channel's first value
        float val = -INFINITY;
        int best = 0;
        for (int kh = 0; kh < kernel; kh++) {
            const int hi = h0 + kh;
            if ((unsigned)hi >= h) continue;
            for (int kw = 0; kw < kernel; kw++) {
                const int wi = w0 + kw;
                if ((unsigned)wi >= w) continue;
                const uint64_t idx = chan0 + (uint32_t)hi * w + (uint32_t)wi;
                if (idx < in_len) {
                    const float v = x[idx];
                    if (v > val) { val = v; best = kh * kernel + kw; }
                }
            }
        }
        if (o < out_len) {
            y[o] = val;
            mn = fminf(mn, val);
            mx = fmaxf(mx, val);
        }
        if (o < idx_len) indices[o] = best;
    }
    if (re.table) emit_range(re, mn, mx);
}

// The same without indices for K x K windows that always meet the image (pad < K): the K * K taps are requested at once
// from clamped coordinates.  A clamped tap repeats a value of the window, which leaves its maximum as it is; the
// values meet in (kh, kw) order under the same comparison as above.
template <int K>
__global__ void __launch_bounds__(256) maxpool2d_window_kernel(const float *x, float *y, uint32_t out_len, uint32_t h, uint32_t w, FastDiv ho,
                                                               FastDiv wo, int stride, int pad, RangeEmit re)
{
    const uint32_t ie = re.table ? (uint32_t)re.image_elems : out_len, base = blockIdx.y * ie;
    float mn = INFINITY, mx = -INFINITY;
    for (uint32_t j = blockIdx.x * 256 + threadIdx.x; j < ie && base + j < out_len; j += gridDim.x * 256) {
        const uint32_t o = base + j;
        const uint32_t t = wo.div(o), ww = o - t * wo.d, nc = ho.div(t), hh = t - nc * ho.d;
        const int h0 = (int)(hh * stride) - pad, w0 = (int)(ww * stride) - pad;
        const float *ch = x + (uint64_t)nc * h * w;
        uint32_t ro[K], co[K];
#pragma unroll
        for (int k = 0; k < K; k++) {
            ro[k] = (uint32_t)min(max(h0 + k, 0), (int)h - 1) * w;
            co[k] = (uint32_t)min(max(w0 + k, 0), (int)w - 1);
        }
        float v[K][K];
#pragma unroll
        for (int kh = 0; kh < K; kh++)
#pragma unroll
            for (int kw = 0; kw < K; kw++) v[kh][kw] = ch[ro[kh] + co[kw]];
        float val = -INFINITY;
#pragma unroll
        for (int kh = 0; kh < K; kh++)
#pragma unroll
            for (int kw = 0; kw < K; kw++) val = v[kh][kw] > val ? v[kh][kw] : val;
        y[o] = val;
        mn = fminf(mn, val);
        mx = fmaxf(mx, val);
    }
    if (re.table) emit_range(re, mn, mx);
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

__global__ void __launch_bounds__(256) upsample_nearest2d_kernel(const float *x, float *y, uint64_t total, uint64_t h, uint64_t w, int sh, int sw,
                                                                 RangeEmit re)
{
    const uint64_t wo = w * sw, ho = h * sh;
    const uint64_t ie = re.table ? re.image_elems : total, base = (uint64_t)blockIdx.y * ie;
    float mn = INFINITY, mx = -INFINITY;
    for (uint64_t j = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; j < ie && base + j < total; j += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t o = base + j;
        const uint64_t ow = o % wo, t = o / wo, oh = t % ho, nc = t / ho;
        const float v = x[(nc * h + oh / sh) * w + ow / sw];
        y[o] = v;
        mn = fminf(mn, v);
        mx = fmaxf(mx, v);
    }
    if (re.table) emit_range(re, mn, mx);
}
__global__ void __launch_bounds__(256) upsample_nearest2d_small_kernel(const float *x, float *y, uint32_t total, uint32_t h, uint32_t w, FastDiv ho,
                                                                       FastDiv wo, FastDiv sh, FastDiv sw, RangeEmit re)
{
    const uint32_t ie = re.table ? (uint32_t)re.image_elems : total, base = blockIdx.y * ie;
    float mn = INFINITY, mx = -INFINITY;
    for (uint32_t j = blockIdx.x * 256 + threadIdx.x; j < ie && base + j < total; j += gridDim.x * 256) {
        const uint32_t o = base + j;
        const uint32_t t = wo.div(o), ow = o - t * wo.d, nc = ho.div(t), oh = t - nc * ho.d;
        const float v = x[((size_t)nc * h + sh.div(oh)) * w + sw.div(ow)];
        y[o] = v;
        mn = fminf(mn, v);
        mx = fmaxf(mx, v);
    }
    if (re.table) emit_range(re, mn, mx);
}
// ... four consecutive outputs of a row per thread (output rows of a multiple of four values, 16-byte aligned y)
__global__ void __launch_bounds__(256) upsample_nearest2d_v4_kernel(const float *x, float *y, uint32_t total, uint32_t h, uint32_t w, FastDiv ho,
                                                                    FastDiv wo4, FastDiv sh, FastDiv sw, RangeEmit re)
{
    const uint32_t ie = (re.table ? (uint32_t)re.image_elems : total) / 4, base = blockIdx.y * ie;   // in groups of four
    float mn = INFINITY, mx = -INFINITY;
    for (uint32_t j = blockIdx.x * 256 + threadIdx.x; j < ie && base + j < total / 4; j += gridDim.x * 256) {
        const uint32_t o4 = base + j;
        const uint32_t t = wo4.div(o4), ow = (o4 - t * wo4.d) * 4, nc = ho.div(t), oh = t - nc * ho.d;
        const float *row = x + ((size_t)nc * h + sh.div(oh)) * w;
        const float4 v = make_float4(row[sw.div(ow)], row[sw.div(ow + 1)], row[sw.div(ow + 2)], row[sw.div(ow + 3)]);
        *reinterpret_cast<float4 *>(y + (size_t)o4 * 4) = v;
        mn = fminf(fminf(mn, fminf(v.x, v.y)), fminf(v.z, v.w));
        mx = fmaxf(fmaxf(mx, fmaxf(v.x, v.y)), fmaxf(v.z, v.w));
    }
    if (re.table) emit_range(re, mn, mx);
}
}  // namespace

static unsigned grid_for(uint64_t n)
{
    uint64_t blocks = (n + 255) / 256;
    return (unsigned)(blocks > 8192 ? 8192 : (blocks < 1 ? 1 : blocks));
}

// Launch shape and table slice for the next call's range request (range_io.h): `per_image` values per image in
// `images` images.  Without a usable request: one image, as many blocks as `n` values want.
struct RangePlan {
    RangeEmit re;
    dim3 grid;
    int parts;
};
static RangePlan range_plan(FnnRangeIo *rio, uint64_t n, uint64_t per_image, uint64_t images, unsigned flat_blocks)
{
    RangePlan rp;
    rp.re = RangeEmit{nullptr, 0, 0, 0};
    rp.grid = dim3(flat_blocks);
    rp.parts = 0;
    if (!rio || !rio->out_table) return rp;
    uint64_t blocks = (per_image + 2047) / 2048;
    if (blocks > 512) blocks = 512;
    if (blocks < 1) blocks = 1;
    if (per_image == 0 || images == 0 || images > 65535 || rio->out_images != images || per_image * images != n ||
        (uint64_t)rio->out_parts + blocks > (uint64_t)rio->out_stride) {   // (out_parts: pairs already in place)
        rio->out_failed = 1;
        return rp;
    }
    rp.re = RangeEmit{rio->out_table, per_image, rio->out_stride, rio->out_parts};
    rp.grid = dim3((unsigned)blocks, (unsigned)images);
    rp.parts = (int)blocks;
    return rp;
}

// The same for the kernels that give a block 1024 * U consecutive values of an image: the smallest U in 1, 2, 4, 8
// whose pairs fit the table.
static RangePlan range_plan_chunks(FnnRangeIo *rio, uint64_t n, uint64_t per_image, uint64_t images, int *unroll)
{
    RangePlan rp;
    rp.re = RangeEmit{nullptr, 0, 0, 0};
    rp.grid = dim3(1);
    rp.parts = 0;
    *unroll = 1;
    if (!rio || !rio->out_table) return rp;
    uint64_t blocks = 0;
    int u = 1;
    for (; u <= 8; u *= 2) {
        blocks = (per_image + 1024 * u - 1) / (1024 * u);
        if ((uint64_t)rio->out_parts + blocks <= (uint64_t)rio->out_stride) break;
    }
    if (u > 8 || per_image == 0 || images == 0 || images > 65535 || rio->out_images != images || per_image * images != n) {
        rio->out_failed = 1;
        return rp;
    }
    rp.re = RangeEmit{rio->out_table, per_image, rio->out_stride, rio->out_parts};
    rp.grid = dim3((unsigned)blocks, (unsigned)images);
    rp.parts = (int)blocks;
    *unroll = u;
    return rp;
}

hipError_t launch_copy2d(float *dst, uint64_t dst_pitch, uint64_t dst_len, const float *src, uint64_t src_pitch, uint64_t src_len,
                         uint64_t width, uint64_t height, hipStream_t s, FnnRangeIo *rio)
{
    if (width == 0 || height == 0) return hipSuccess;
    // a copy clipped by either length keeps the kernel that checks every index (and leaves no ranges: it has not
    // seen every value of the destination)
    const bool whole = dst_len >= (height - 1) * dst_pitch + width && src_len >= (height - 1) * src_pitch + width;
    // ranges: one image per row of the destination, so the rows must be the reader's images
    const bool wanted = rio && rio->out_table;
    const bool ranges = wanted && whole && rio->out_image_elems == dst_pitch;
    if (wanted && !ranges) rio->out_failed = 1;
    if (!whole || height > 65535) {
        if (ranges) rio->out_failed = 1;
        hipLaunchKernelGGL(copy2d_kernel, dim3(grid_for(width * height)), dim3(256), 0, s, dst, dst_pitch, dst_len, src, src_pitch, src_len, width, height);
        return hipGetLastError();
    }
    int u = 1;
    RangePlan rp = range_plan_chunks(ranges ? rio : nullptr, width * height, width, height, &u);
    if (!rp.re.table) {   // no table (none wanted, or no room in it): the same kernel, one block per 1024 values of a row
        u = 1;
        rp.grid = dim3((unsigned)((width + 1023) / 1024), (unsigned)height);
    }
    const bool v4 = width % 4 == 0 && dst_pitch % 4 == 0 && src_pitch % 4 == 0 && ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15) == 0;
    auto go = [&](auto kern) { hipLaunchKernelGGL(kern, rp.grid, dim3(256), 0, s, dst, dst_pitch, src, src_pitch, width, rp.re); };
    if (u == 1) v4 ? go(copy2d_ranges_kernel<1, true>) : go(copy2d_ranges_kernel<1, false>);
    else if (u == 2) v4 ? go(copy2d_ranges_kernel<2, true>) : go(copy2d_ranges_kernel<2, false>);
    else if (u == 4) v4 ? go(copy2d_ranges_kernel<4, true>) : go(copy2d_ranges_kernel<4, false>);
    else v4 ? go(copy2d_ranges_kernel<8, true>) : go(copy2d_ranges_kernel<8, false>);
    if (rp.re.table) rio->out_parts += rp.parts;
    return hipGetLastError();
}

// every part unclipped: dst holds height * dst_pitch values, part j holds height * width[j]
hipError_t launch_concat(float *dst, uint64_t dst_pitch, int n_parts, const float *const *srcs, const uint64_t *widths, uint64_t height,
                         hipStream_t s, FnnRangeIo *rio, bool *done)
{
    *done = false;
    if (n_parts < 1 || n_parts > CONCAT_MAX_PARTS || height == 0 || height > 65535) return hipSuccess;
    ConcatArgs a = {};
    uint64_t off = 0, blocks = 0, max_blocks = 0;
    bool v4 = dst_pitch % 4 == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
    for (int j = 0; j < n_parts; j++) {
        const uint64_t b = (widths[j] + 1023) / 1024;
        a.src[j] = srcs[j]; a.width[j] = widths[j]; a.off[j] = off; a.blk0[j] = (uint32_t)blocks;
        v4 = v4 && widths[j] % 4 == 0 && off % 4 == 0 && (reinterpret_cast<uintptr_t>(srcs[j]) & 15) == 0;
        off += widths[j];
        blocks += b;
        if (b > max_blocks) max_blocks = b;
    }
    if (off > dst_pitch || max_blocks == 0 || max_blocks > (1u << 30)) return hipSuccess;
    RangeEmit re{nullptr, 0, 0, 0};
    if (rio && rio->out_table) {
        if (rio->out_images == height && rio->out_image_elems == dst_pitch && off == dst_pitch &&
            (uint64_t)rio->out_parts + blocks <= (uint64_t)rio->out_stride)
            re = RangeEmit{rio->out_table, dst_pitch, rio->out_stride, rio->out_parts};
        else
            rio->out_failed = 1;
    }
    const dim3 grid((unsigned)max_blocks, (unsigned)height, (unsigned)n_parts);
    if (v4) hipLaunchKernelGGL(concat_kernel<true>, grid, dim3(256), 0, s, dst, dst_pitch, a, re);
    else hipLaunchKernelGGL(concat_kernel<false>, grid, dim3(256), 0, s, dst, dst_pitch, a, re);
    if (re.table) rio->out_parts += (int)blocks;
    *done = true;
    return hipGetLastError();
}

hipError_t launch_maxpool2d(const float *x, uint64_t in_len, float *y, uint64_t out_len, uint64_t c, uint64_t h, uint64_t w,
                            uint64_t ho, uint64_t wo, int kernel, int stride, int pad, int64_t *indices, uint64_t idx_len, hipStream_t s,
                            FnnRangeIo *rio)
{
    if (!indices) idx_len = 0;
    const uint64_t total = out_len > idx_len ? out_len : idx_len;
    if (total == 0) return hipSuccess;
    const bool images_match = idx_len <= out_len && rio && rio->out_image_elems == c * ho * wo;
    if (!images_match && rio && rio->out_table) rio->out_failed = 1;
    RangePlan rp = range_plan(images_match ? rio : nullptr, out_len, c * ho * wo, c * ho * wo ? out_len / (c * ho * wo) : 0, grid_for(total));
    const uint64_t chans = ho * wo ? (out_len + ho * wo - 1) / (ho * wo) : 0;
    const bool window = idx_len == 0 && (kernel == 2 || kernel == 3 || kernel == 5) && pad >= 0 && pad < kernel && stride >= 1 && h >= 1 && w >= 1 &&
                        ho >= 1 && wo >= 1 && (int64_t)(ho - 1) * stride - pad <= (int64_t)h - 1 && (int64_t)(wo - 1) * stride - pad <= (int64_t)w - 1 &&
                        chans * h * w <= in_len && in_len < (1ull << 31) && out_len < (1ull << 31);
    if (window) {
        const FastDiv dh = fast_div((uint32_t)ho), dw = fast_div((uint32_t)wo);
        if (kernel == 2) hipLaunchKernelGGL(maxpool2d_window_kernel<2>, rp.grid, dim3(256), 0, s, x, y, (uint32_t)out_len, (uint32_t)h, (uint32_t)w, dh, dw, stride, pad, rp.re);
        else if (kernel == 3) hipLaunchKernelGGL(maxpool2d_window_kernel<3>, rp.grid, dim3(256), 0, s, x, y, (uint32_t)out_len, (uint32_t)h, (uint32_t)w, dh, dw, stride, pad, rp.re);
        else hipLaunchKernelGGL(maxpool2d_window_kernel<5>, rp.grid, dim3(256), 0, s, x, y, (uint32_t)out_len, (uint32_t)h, (uint32_t)w, dh, dw, stride, pad, rp.re);
    } else if (in_len < (1ull << 31) && total < (1ull << 31) && h * w < (1ull << 31))
        hipLaunchKernelGGL(maxpool2d_small_kernel, rp.grid, dim3(256), 0, s, x, (uint32_t)in_len, y, (uint32_t)out_len, (uint32_t)h, (uint32_t)w,
                           fast_div((uint32_t)ho), fast_div((uint32_t)wo), kernel, stride, pad, indices, (uint32_t)idx_len, rp.re);
    else
        hipLaunchKernelGGL(maxpool2d_kernel, rp.grid, dim3(256), 0, s, x, in_len, y, out_len, c, h, w, ho, wo, kernel, stride, pad,
                           indices, idx_len, rp.re);
    if (rio) rio->out_parts += rp.parts;
    return hipGetLastError();
}

hipError_t launch_avgpool2d(const float *x, uint64_t in_len, float *y, uint64_t out_len, uint64_t h, uint64_t w,
                            uint64_t ho, uint64_t wo, int kernel, int stride, int pad, hipStream_t s)
{
    if (out_len == 0) return hipSuccess;
    hipLaunchKernelGGL(avgpool2d_kernel, dim3(grid_for(out_len)), dim3(256), 0, s, x, in_len, y, out_len, h, w, ho, wo, kernel, stride, pad);
    return hipGetLastError();
}

hipError_t launch_upsample_nearest2d(const float *x, float *y, uint64_t nc, uint64_t h, uint64_t w, int sh, int sw, hipStream_t s, FnnRangeIo *rio)
{
    const uint64_t total = nc * h * sh * w * sw;
    if (total == 0) return hipSuccess;
    const uint64_t per_image = rio && rio->out_table ? rio->out_image_elems : 0;
    RangePlan rp = range_plan(rio, total, per_image, per_image ? total / per_image : 0, grid_for(total));
    if (total < (1ull << 31) && sh >= 1 && sw >= 1 && (w * sw) % 4 == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 &&
        (!rp.re.table || rp.re.image_elems % 4 == 0)) {
        const dim3 grid(rp.re.table ? rp.grid.x : grid_for(total / 4), rp.grid.y);
        hipLaunchKernelGGL(upsample_nearest2d_v4_kernel, grid, dim3(256), 0, s, x, y, (uint32_t)total, (uint32_t)h, (uint32_t)w,
                           fast_div((uint32_t)(h * sh)), fast_div((uint32_t)(w * sw / 4)), fast_div((uint32_t)sh), fast_div((uint32_t)sw), rp.re);
    } else if (total < (1ull << 31) && sh >= 1 && sw >= 1)
        hipLaunchKernelGGL(upsample_nearest2d_small_kernel, rp.grid, dim3(256), 0, s, x, y, (uint32_t)total, (uint32_t)h, (uint32_t)w,
                           fast_div((uint32_t)(h * sh)), fast_div((uint32_t)(w * sw)), fast_div((uint32_t)sh), fast_div((uint32_t)sw), rp.re);
    else
        hipLaunchKernelGGL(upsample_nearest2d_kernel, rp.grid, dim3(256), 0, s, x, y, total, h, w, sh, sw, rp.re);
    if (rio) rio->out_parts += rp.parts;
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

hipError_t launch_eltwise(int op, const float *a, const float *b, uint64_t nb, float *out, uint64_t n, hipStream_t s, FnnRangeIo *rio)
{
    if (n == 0) return hipSuccess;
    const uint64_t per_image = rio && rio->out_table ? rio->out_image_elems : 0;
    int u = 1;
    RangePlan rp = range_plan_chunks(rio, n, per_image, per_image ? n / per_image : 0, &u);
    if (rp.re.table) {
        if (u == 1) hipLaunchKernelGGL(eltwise_ranges_kernel<1>, rp.grid, dim3(256), 0, s, op, a, b, nb ? nb : 1, out, n, rp.re);
        else if (u == 2) hipLaunchKernelGGL(eltwise_ranges_kernel<2>, rp.grid, dim3(256), 0, s, op, a, b, nb ? nb : 1, out, n, rp.re);
        else if (u == 4) hipLaunchKernelGGL(eltwise_ranges_kernel<4>, rp.grid, dim3(256), 0, s, op, a, b, nb ? nb : 1, out, n, rp.re);
        else hipLaunchKernelGGL(eltwise_ranges_kernel<8>, rp.grid, dim3(256), 0, s, op, a, b, nb ? nb : 1, out, n, rp.re);
        rio->out_parts += rp.parts;
        return hipGetLastError();
    }
    if (n <= (1ull << 40)) {   // no table: the same kernel over the whole tensor as one image (all operands of a thread requested first)
        const RangeEmit none{nullptr, n, 0, 0};
        hipLaunchKernelGGL(eltwise_ranges_kernel<1>, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, s, op, a, b, nb ? nb : 1, out, n, none);
        return hipGetLastError();
    }
    uint64_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(eltwise_kernel, dim3((unsigned)blocks), dim3(256), 0, s, op, a, b, nb, out, n);
    return hipGetLastError();
}
