// Quantised Conv2d (I8 or I4 weights, f32 NCHW activations) for gfx950:
// conv2d_packed_i8x4 = im2col + per-(image,group) dynamic int8 activation quantisation +
// integer GEMM with the fused 4-term dequantise, bias and activation
// (src/backend/cpu/packed_conv.rs:125-232,444-625,1118-1196);
// conv2d_packed_i4x8 = the same with 4-bit weights and activations quantised to 16 levels
// (packed_conv.rs:236-283,659-841,1202-1280).
//
// The im2col matrix is never materialised: its (min,max) scan and the activation
// quantisation are evaluated from the NCHW input through the index formula
//   col[p, c*KH*KW + i*KW + j] = x[c, oh*s + i*d - pad, ow*s + j*d - pad]  (0 outside),
// so the HBM traffic is the input, the weights and the output only.
#include "common.h"

#include "i8act.h"

namespace {

__device__ __forceinline__ float col_value(const float *xg, int64_t h, int64_t w, int kh, int kw,
                                           int stride, int pad, int dil, int64_t wo, int64_t p,
                                           int64_t e)
{
    const int64_t khw = (int64_t)kh * kw;
    const int64_t ic = e / khw;
    const int rem = (int)(e % khw);
    const int i = rem / kw, j = rem % kw;
    const int64_t oh = p / wo, ow = p % wo;
    const int64_t ih = oh * stride + (int64_t)i * dil - pad;
    const int64_t iw = ow * stride + (int64_t)j * dil - pad;
    if (ih < 0 || ih >= h || iw < 0 || iw >= w) return 0.0f;
    return xg[(ic * h + ih) * w + iw];
}

// min/max over the whole im2col matrix of one (image, group), padding zeros included
// (src/backend/cpu/im2col.rs:496-507).
__global__ void __launch_bounds__(256) conv_minmax_kernel(QConvArgs a)
{
    __shared__ float smn[4], smx[4];
    const int bg = blockIdx.y;
    const int64_t nn = bg / a.groups, g = bg % a.groups;
    const int64_t cg = a.c / a.groups;
    const int64_t kk = cg * a.kh * a.kw;
    const int64_t np = a.ho * a.wo;
    const float *xg = a.x + (nn * a.c + g * cg) * a.h * a.w;
    float mn = INFINITY, mx = -INFINITY;
    const int64_t total = np * kk;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        // pixel-fastest order keeps neighbouring lanes on neighbouring input columns
        const int64_t e = idx / np, p = idx % np;
        const float v = col_value(xg, a.h, a.w, a.kh, a.kw, a.stride, a.pad, a.dil, a.wo, p, e);
        mn = fminf(mn, v);
        mx = fmaxf(mx, v);
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) { smn[threadIdx.x >> 6] = mn; smx[threadIdx.x >> 6] = mx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float *dst = a.minmax_partial + ((int64_t)bg * QCONV_NPART + blockIdx.x) * 2;
        dst[0] = fminf(fminf(smn[0], smn[1]), fminf(smn[2], smn[3]));
        dst[1] = fmaxf(fmaxf(smx[0], smx[1]), fmaxf(smx[2], smx[3]));
    }
}

// The same min/max without walking the im2col matrix: an input pixel (ih, iw) appears in it iff some
// tap reaches it, which factorises into a row condition and a column condition; the zero of the
// padding takes part iff some tap falls outside.  min/max do not depend on order or multiplicity,
// so the result is identical to the scan above.
__global__ void __launch_bounds__(256) conv_minmax_cover_kernel(QConvArgs a, int pad_touched)
{
    extern __shared__ unsigned char cov[];   // [h] rows reached, then [w] columns reached
    __shared__ float smn[4], smx[4];
    unsigned char *cov_h = cov, *cov_w = cov + a.h;
    for (int64_t t = threadIdx.x; t < a.h + a.w; t += blockDim.x) {
        const bool is_h = t < a.h;
        const int64_t pos = is_h ? t : t - a.h;
        const int taps = is_h ? a.kh : a.kw;
        const int64_t outs = is_h ? a.ho : a.wo;
        unsigned char hit = 0;
        for (int i = 0; i < taps; i++) {
            const int64_t num = pos + a.pad - (int64_t)i * a.dil;   // = o * stride
            if (num >= 0 && num % a.stride == 0 && num / a.stride < outs) hit = 1;
        }
        cov[t] = hit;
    }
    __syncthreads();
    const int bg = blockIdx.y;
    const int64_t nn = bg / a.groups, g = bg % a.groups;
    const int64_t cg = a.c / a.groups;
    const float *xg = a.x + (nn * a.c + g * cg) * a.h * a.w;
    float mn = pad_touched ? 0.0f : INFINITY, mx = pad_touched ? 0.0f : -INFINITY;
    // A wave takes a chunk of whole image rows (channel, ih) at a time, consecutive lanes on consecutive
    // elements (16 bytes per lane when the row length allows): rows and columns no tap reaches are skipped by
    // two table lookups, and the index arithmetic is per 16 bytes, not per element.
    const int64_t nrows = cg * a.h;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6), nwaves = (int64_t)gridDim.x * 4;
    const bool vec4 = (a.w % 4 == 0) && ((reinterpret_cast<uintptr_t>(xg) & 15) == 0);
    const int per_lane = vec4 ? 4 : 1;
    const int64_t span = 64 * per_lane;                              // elements a wave covers per step
    const int64_t rows_per_chunk = a.w >= span ? 1 : span / a.w;     // whole rows per chunk
    const int64_t steps = a.w >= span ? (a.w + span - 1) / span : 1; // steps per chunk (long rows)
    const int64_t chunks = (nrows + rows_per_chunk - 1) / rows_per_chunk;
    for (int64_t ch = wave; ch < chunks; ch += nwaves) {
        const int64_t row0 = ch * rows_per_chunk;
        for (int64_t st = 0; st < steps; st++) {
            const int64_t e = st * span + (int64_t)lane * per_lane;   // element inside the chunk
            const int64_t sub = e / a.w, iw = e - sub * a.w;
            const int64_t row = row0 + sub;
            if (sub >= rows_per_chunk || row >= nrows || iw >= a.w) continue;
            if (!cov_h[row % a.h]) continue;
            const float *src = xg + row * a.w + iw;
            if (vec4) {
                const float4 v = *reinterpret_cast<const float4 *>(src);
                if (cov_w[iw + 0]) { mn = fminf(mn, v.x); mx = fmaxf(mx, v.x); }
                if (cov_w[iw + 1]) { mn = fminf(mn, v.y); mx = fmaxf(mx, v.y); }
                if (cov_w[iw + 2]) { mn = fminf(mn, v.z); mx = fmaxf(mx, v.z); }
                if (cov_w[iw + 3]) { mn = fminf(mn, v.w); mx = fmaxf(mx, v.w); }
            } else if (cov_w[iw]) {
                const float v = *src;
                mn = fminf(mn, v);
                mx = fmaxf(mx, v);
            }
        }
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) { smn[threadIdx.x >> 6] = mn; smx[threadIdx.x >> 6] = mx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float *dst = a.minmax_partial + ((int64_t)bg * QCONV_NPART + blockIdx.x) * 2;
        dst[0] = fminf(fminf(smn[0], smn[1]), fminf(smn[2], smn[3]));
        dst[1] = fmaxf(fmaxf(smx[0], smx[1]), fmaxf(smx[2], smx[3]));
    }
}

// Every input row and column is reached by some tap (the usual case: stride <= kernel extent) and the slab of the
// (image, group) is 16-byte aligned: a plain min/max over the contiguous slab, four 16-byte loads in flight per lane.
__global__ void __launch_bounds__(256) conv_minmax_flat_kernel(QConvArgs a, int pad_touched)
{
    __shared__ float smn[4], smx[4];
    const int bg = blockIdx.y;
    const int64_t nn = bg / a.groups, g = bg % a.groups;
    const int64_t cg = a.c / a.groups;
    const float4 *x4 = reinterpret_cast<const float4 *>(a.x + (nn * a.c + g * cg) * a.h * a.w);
    const int64_t n4 = (cg * a.h * a.w) >> 2;
    float mn = pad_touched ? 0.0f : INFINITY, mx = pad_touched ? 0.0f : -INFINITY;
    const int64_t stride = (int64_t)gridDim.x * 256;
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + 3 * stride < n4; i += 4 * stride) {
        const float4 v0 = x4[i], v1 = x4[i + stride], v2 = x4[i + 2 * stride], v3 = x4[i + 3 * stride];
        mn = fminf(fminf(fminf(mn, fminf(v0.x, v0.y)), fminf(fminf(v0.z, v0.w), fminf(v1.x, v1.y))),
                   fminf(fminf(fminf(v1.z, v1.w), fminf(v2.x, v2.y)), fminf(fminf(v2.z, v2.w), fminf(fminf(v3.x, v3.y), fminf(v3.z, v3.w)))));
        mx = fmaxf(fmaxf(fmaxf(mx, fmaxf(v0.x, v0.y)), fmaxf(fmaxf(v0.z, v0.w), fmaxf(v1.x, v1.y))),
                   fmaxf(fmaxf(fmaxf(v1.z, v1.w), fmaxf(v2.x, v2.y)), fmaxf(fmaxf(v2.z, v2.w), fmaxf(fmaxf(v3.x, v3.y), fmaxf(v3.z, v3.w)))));
    }
    for (; i < n4; i += stride) {
        const float4 v = x4[i];
        mn = fminf(fminf(mn, fminf(v.x, v.y)), fminf(v.z, v.w));
        mx = fmaxf(fmaxf(mx, fmaxf(v.x, v.y)), fmaxf(v.z, v.w));
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) { smn[threadIdx.x >> 6] = mn; smx[threadIdx.x >> 6] = mx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float *dst = a.minmax_partial + ((int64_t)bg * QCONV_NPART + blockIdx.x) * 2;
        dst[0] = fminf(fminf(smn[0], smn[1]), fminf(smn[2], smn[3]));
        dst[1] = fmaxf(fmaxf(smx[0], smx[1]), fmaxf(smx[2], smx[3]));
    }
}

// 8-bit: scale = range/255 (1 if range <= 0), zero = mn + 128*scale (0 if range <= 0), inv = 1/scale
// (src/backend/cpu/packed_conv.rs:149-156); 4-bit: scale = range/15 (1 if range <= 0),
// zero = mn + 8*scale in either case (packed_conv.rs:260-263)
__global__ void __launch_bounds__(64) conv_actq_kernel(QConvArgs a, int nparts)
{
    const int bg = blockIdx.x;
    float mn = a.range_zero ? 0.0f : INFINITY, mx = a.range_zero ? 0.0f : -INFINITY;
    for (int i = threadIdx.x; i < nparts; i += 64) {
        mn = fminf(mn, a.minmax_partial[((int64_t)bg * a.part_stride + i) * 2]);
        mx = fmaxf(mx, a.minmax_partial[((int64_t)bg * a.part_stride + i) * 2 + 1]);
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    if (threadIdx.x == 0) {
        const float range = mx - mn;
        float scale, zero;
        if (a.wbits == 4) {
            scale = (range > 0.0f) ? range / 15.0f : 1.0f;
            zero = mn + 8.0f * scale;
        } else {
            scale = (range > 0.0f) ? range / 255.0f : 1.0f;
            zero = (range > 0.0f) ? mn + 128.0f * scale : 0.0f;
        }
        const float inv = (scale != 0.0f) ? 1.0f / scale : 0.0f;
        a.actq[bg * 4 + 0] = scale;
        a.actq[bg * 4 + 1] = zero;
        a.actq[bg * 4 + 2] = inv;
        a.actq[bg * 4 + 3] = 0.0f;
    }
}

constexpr int CONV_OCT = 8;  // output channels per thread

// One thread = one output pixel x CONV_OCT output channels of one (image, group).
// acc = bias_q + sum q_a*q_w (i32, exact);
// val = acc*sab + zw*(sa*sum q_a) + za*(sw*qb) + (za*zw)*K, left to right
// (src/backend/cpu/packed_conv.rs:469-505).
__global__ void __launch_bounds__(256) conv_i8_kernel(QConvArgs a)
{
    const int bg = blockIdx.z;
    const int64_t nn = bg / a.groups, g = bg % a.groups;
    const int64_t cg = a.c / a.groups, ocg = a.oc / a.groups;
    const int64_t kk = cg * a.kh * a.kw;
    const int64_t np = a.ho * a.wo;
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t f0 = (int64_t)blockIdx.y * CONV_OCT;
    if (p >= np) return;
    const float *xg = a.x + (nn * a.c + g * cg) * a.h * a.w;
    const float sa = a.actq[bg * 4 + 0], za = a.actq[bg * 4 + 1], inv = a.actq[bg * 4 + 2];
    int acc[CONV_OCT];
#pragma unroll
    for (int t = 0; t < CONV_OCT; t++) acc[t] = 0;
    int qasum = 0;
    const int8_t *wb = reinterpret_cast<const int8_t *>(a.words);
    const float qlo = a.wbits == 4 ? -8.0f : -128.0f, qhi = a.wbits == 4 ? 7.0f : 127.0f;
    for (int64_t e = 0; e < kk; e++) {
        const float v = col_value(xg, a.h, a.w, a.kh, a.kw, a.stride, a.pad, a.dil, a.wo, p, e);
        const float t = roundf((v - za) * inv);
        const int q = (t != t) ? 0 : (int)fminf(fmaxf(t, qlo), qhi);
        qasum += q;
#pragma unroll
        for (int t2 = 0; t2 < CONV_OCT; t2++) {
            const int64_t f = f0 + t2;
            if (f >= ocg) continue;
            int qw;
            if (a.wbits == 4) qw = ((int)(a.words[(g * ocg + f) * a.kp + e / 8] << (28 - 4 * (int)(e % 8)))) >> 28;
            else qw = (int)wb[((g * ocg + f) * a.kp) * 4 + e];
            acc[t2] += q * qw;
        }
    }
    const float r = sa * (float)qasum;
#pragma unroll
    for (int t2 = 0; t2 < CONV_OCT; t2++) {
        const int64_t f = f0 + t2;
        if (f >= ocg) continue;
        const int64_t ch = g * ocg + f;
        const float sw = a.scales[ch], zw = a.zeros[ch];
        const float sab = sa * sw;
        int bias_q = 0;
        if (a.bias) {
            const float bq = roundf(a.bias[ch] / sab);
            bias_q = (bq != bq) ? 0 : (bq >= 2147483648.0f ? 2147483647 : (bq <= -2147483648.0f ? (-2147483647 - 1) : (int)bq));
        }
        const int accv = acc[t2] + bias_q;
        const float w_term = sw * (float)a.row_qsum[ch];
        const float zp_prod = za * zw;
        float val = (float)accv * sab;
        val = val + zw * r;
        val = val + za * w_term;
        val = val + zp_prod * (float)kk;
        if (a.act == FNN_ACT_RELU) val = fmaxf(val, 0.0f);
        else if (a.act == FNN_ACT_SILU) val = val / (1.0f + expf(-val));
        else if (a.act == FNN_ACT_GELU)
            val = val * 0.5f * (1.0f + tanhf(val * 0.7978846f * (1.0f + 0.044715f * val * val)));
        const int64_t o = (nn * a.oc + ch) * np + p;
        a.y[o] = val;
        if (a.acc_out) a.acc_out[o] = accv;
    }
}

template <int BITS>
__global__ void __launch_bounds__(256) row_qsum_kernel(const uint32_t *words, int64_t rows, int64_t kp, int32_t *out)
{
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    int s = 0;
    for (int64_t wd = lane; wd < kp; wd += 64) {
        const uint32_t w = words[r * kp + wd];
        if (BITS == 8) {
            s += (int)(int8_t)(w & 0xff) + (int)(int8_t)((w >> 8) & 0xff) + (int)(int8_t)((w >> 16) & 0xff) + ((int)w >> 24);
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) s += ((int)(w << (28 - 4 * i))) >> 28;
        }
    }
    s = wave_sum_i32(s);
    if (lane == 0) out[r] = s;
}

}  // namespace

hipError_t launch_row_qsum(const fnn_hip_weight *w, int32_t *out, hipStream_t s)
{
    dim3 grid((unsigned)((w->rows + 3) / 4));
    if (w->dtype == FNN_DT_I8)
        hipLaunchKernelGGL((row_qsum_kernel<8>), grid, dim3(256), 0, s, w->words, w->rows, w->kp, out);
    else if (w->dtype == FNN_DT_I4)
        hipLaunchKernelGGL((row_qsum_kernel<4>), grid, dim3(256), 0, s, w->words, w->rows, w->kp, out);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

__global__ void __launch_bounds__(256) conv_actq_from_payload_kernel(const uint8_t *payload, float *actq, int nbg)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= nbg) return;
    const float *hdr = reinterpret_cast<const float *>(payload);
    actq[i * 4 + 0] = hdr[0];
    actq[i * 4 + 1] = hdr[1];
    actq[i * 4 + 2] = 0.0f;
    actq[i * 4 + 3] = 0.0f;
}

hipError_t launch_conv_actq_from_payload(const uint8_t *payload, float *actq, int nbg, hipStream_t s)
{
    hipLaunchKernelGGL(conv_actq_from_payload_kernel, dim3((unsigned)((nbg + 255) / 256)), dim3(256), 0, s, payload, actq, nbg);
    return hipGetLastError();
}

// does any tap fall into the padding (rows and columns separately), and is every input row and column reached by
// some tap?  With both known, min / max of the im2col matrix are those of the input slab, plus zero if padded.
void fnn_conv_coverage(const QConvArgs &p, int *pad_touched_out, bool *every_input_reached)
{
    int pad_touched = 0;
    for (int64_t o = 0; o < p.ho && !pad_touched; o++)
        for (int i = 0; i < p.kh; i++) {
            const int64_t ih = o * p.stride + (int64_t)i * p.dil - p.pad;
            if (ih < 0 || ih >= p.h) { pad_touched = 1; break; }
        }
    for (int64_t o = 0; o < p.wo && !pad_touched; o++)
        for (int i = 0; i < p.kw; i++) {
            const int64_t iw = o * p.stride + (int64_t)i * p.dil - p.pad;
            if (iw < 0 || iw >= p.w) { pad_touched = 1; break; }
        }
    auto all_reached = [&](int64_t len, int taps, int64_t outs) {
        for (int64_t pos = 0; pos < len; pos++) {
            bool hit = false;
            for (int i = 0; i < taps && !hit; i++) {
                const int64_t num = pos + p.pad - (int64_t)i * p.dil;
                hit = num >= 0 && num % p.stride == 0 && num / p.stride < outs;
            }
            if (!hit) return false;
        }
        return true;
    };
    *pad_touched_out = pad_touched;
    *every_input_reached = p.h + p.w <= 32768 && all_reached(p.h, p.kh, p.ho) && all_reached(p.w, p.kw, p.wo);
}

hipError_t launch_qconv2d_i8(const QConvArgs &p, hipStream_t s, int phase, int *nparts_io)
{
    const int64_t bg = p.b * p.groups;
    const int64_t cg = p.c / p.groups, ocg = p.oc / p.groups;
    const int64_t np = p.ho * p.wo;
    const int64_t total = np * cg * p.kh * p.kw;
    if (bg == 0 || np == 0) return hipSuccess;
    int64_t nparts = (total + 256 * 16 - 1) / (256 * 16);
    if (nparts > QCONV_NPART) nparts = QCONV_NPART;
    if (nparts < 1) nparts = 1;
    if (phase == 4) {
        hipLaunchKernelGGL(conv_actq_kernel, dim3((unsigned)bg), dim3(64), 0, s, p, nparts_io ? *nparts_io : 1);
        return hipGetLastError();
    }
    if (phase != 2) {
        if (p.h + p.w <= 32768 && cg > 0) {
            int pad_touched = 0;
            bool reached = false;
            fnn_conv_coverage(p, &pad_touched, &reached);
            const int64_t elems = cg * p.h * p.w;
            const bool flat = elems % 4 == 0 && (reinterpret_cast<uintptr_t>(p.x) & 15) == 0 && reached;
            nparts = (elems + 256 * 4 - 1) / (256 * 4);
            const int64_t cap = 4096 / bg > 32 ? 4096 / bg : 32;   // about 4096 workgroups over all images
            if (nparts > cap) nparts = cap;
            if (nparts > QCONV_NPART) nparts = QCONV_NPART;
            if (nparts < 1) nparts = 1;
            if (flat) hipLaunchKernelGGL(conv_minmax_flat_kernel, dim3((unsigned)nparts, (unsigned)bg), dim3(256), 0, s, p, pad_touched);
            else hipLaunchKernelGGL(conv_minmax_cover_kernel, dim3((unsigned)nparts, (unsigned)bg), dim3(256), (size_t)(p.h + p.w), s, p, pad_touched);
        } else
            hipLaunchKernelGGL(conv_minmax_kernel, dim3((unsigned)nparts, (unsigned)bg), dim3(256), 0, s, p);
        if (nparts_io) *nparts_io = (int)nparts;
        if (phase != 3) hipLaunchKernelGGL(conv_actq_kernel, dim3((unsigned)bg), dim3(64), 0, s, p, (int)nparts);
    }
    if (phase == 1 || phase == 3) return hipGetLastError();
    dim3 grid((unsigned)((np + 255) / 256), (unsigned)((ocg + CONV_OCT - 1) / CONV_OCT), (unsigned)bg);
    hipLaunchKernelGGL(conv_i8_kernel, grid, dim3(256), 0, s, p);
    return hipGetLastError();
}
