// Launch interfaces of the I8-activation and quantised-conv kernels.
#pragma once
#include "common.h"

struct I8ActArgs {
    const uint32_t *words;
    const float *scales;    // [N]
    const float *zeros;     // [N]
    const uint8_t *payload; // [scale f32][zp f32][M*K i8]
    float *out;             // [M,N]
    int32_t *acc_out;       // [M,N] or null
    int64_t m, n, k, kp;
    // the activation-quantised mode of the f32-activation MatMul (FNN_FLAG_ACT_QUANT): bias + activation behind the
    // I8-activation formula, as the instruction chain matmul_i8_i8 -> add -> act would apply them
    const float *bias = nullptr;
    int act = 0;
};

struct QConvArgs {
    const uint32_t *words;   // [OC, kp] I8 or I4 words
    const float *scales;     // [OC]
    const float *zeros;      // [OC]
    const int32_t *row_qsum; // [OC] sum of q_w per output channel
    const float *x;          // [B,C,H,W]
    const float *bias;       // [OC] or null
    float *y;                // [B,OC,Ho,Wo]
    int32_t *acc_out;        // same shape as y, or null
    float *minmax_partial;   // [B*G][NPART][2]
    float *actq;             // [B*G][4]: sa, za, inv, unused
    int64_t b, c, h, w, oc, ho, wo, kp;
    int kh, kw, stride, pad, dil, groups, act;
    int wbits;               // 8: I8 weights, activations quantised to 256 levels; 4: I4 weights, 16 levels
    const int8_t *x8;        // non-null: the input is already int8 [B,C,H,W] (an activation payload's data)
                             // with one (scale, zero) for the whole tensor in actq; padding taps are the integer 0
    int payload_i4;          // with x8 and I4 weights: the matmul_i4_i8 formula and a float bias
    int nparts;              // > 0: actq is not filled yet; the operand kernel reduces the nparts partial ranges of
                             // its images itself (and stores actq for the epilogue); 0: actq holds the scales
    int part_stride;         // pairs per (image, group) minmax_partial has room for
    int range_zero;          // the partial ranges are those of the input tensor as its producer left them: the zero of
                             // the padding still has to join them
    float *range_out;        // non-null: partial (min, max) pairs of y per image go here, [B][range_out_stride][2]
    int range_out_stride;
    // a plan's Add behind this convolution (range_io.h, FnnResidualIo): sum_out = y + residual, same shape as y, stored
    // by the kernels whose epilogue holds the outputs in registers; the partial ranges are then those of the sums
    const float *residual = nullptr;
    float *sum_out = nullptr;
};
constexpr int QCONV_NPART = 512;
// divisors of the im2col index arithmetic: pixels per image, output width, kernel area, kernel width
struct ConvDivs { FastDiv np, wo, khw, kw; };

// One output of the quantised Conv2d: acc = acc_in + bias_q; val = acc*sab + zw*(sa*sum q_a) + za*(sw*sum q_w)
// + (za*zw)*K, left to right, then the activation (src/backend/cpu/packed_conv.rs:469-505,571,604-606).
// rsum = sa * sum q_a of the row, wt = sw * sum q_w of the channel.
// bias_q = round(bias / (sa*sw)) half away from zero, saturated: trunc(x + copysign(0.49999997, x)) equals roundf(x)
// wherever the result fits an i32, and the conversion saturates and maps NaN to 0
__device__ __forceinline__ int conv_bias_q(float bias, float sa, float sw)
{
    const float x = bias / (sa * sw);
    return (int)(x + __builtin_copysignf(0.49999997f, x));
}
// (the affine part alone; the activation follows, conv_act / conv_act4)
__device__ __forceinline__ float conv_affine(int acc_in, float sa, float za, float rsum, float sw, float zw, float wt,
                                             int bias_q, int kk, int *acc_out)
{
    const float sab = sa * sw;
    const int accv = acc_in + bias_q;
    const float zp_prod = za * zw;
    float val = (float)accv * sab;
    val = val + zw * rsum;
    val = val + za * wt;
    val = val + zp_prod * (float)kk;
    *acc_out = accv;
    return val;
}
__device__ __forceinline__ float conv_act(float val, int act)
{
    if (act == FNN_ACT_RELU) val = fmaxf(val, 0.0f);
    else if (act == FNN_ACT_SILU) val = fnn_sigmoid_times(val, val);
    else if (act == FNN_ACT_GELU) val = fnn_sigmoid_times(val, 2.0f * (val * 0.7978846f * (1.0f + 0.044715f * val * val)));   // = 0.5 v (1 + tanh(.))
    return val;
}
// the same on four outputs with one test of the (uniform) activation code
__device__ __forceinline__ void conv_act4(float (&v)[4], int act)
{
    if (act == FNN_ACT_RELU) {
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = fmaxf(v[j], 0.0f);
    } else if (act == FNN_ACT_SILU) {
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = fnn_sigmoid_times(v[j], v[j]);
    } else if (act == FNN_ACT_GELU) {
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = fnn_sigmoid_times(v[j], 2.0f * (v[j] * 0.7978846f * (1.0f + 0.044715f * v[j] * v[j])));
    }
}
__device__ __forceinline__ float conv_dequant(int acc_in, float sa, float za, float rsum, float sw, float zw, float wt,
                                              int bias_q, int kk, int act, int *acc_out)
{
    return conv_act(conv_affine(acc_in, sa, za, rsum, sw, zw, wt, bias_q, kk, acc_out), act);
}

// min / max over nparts (min, max) pairs at part (16-byte aligned) by the nthr threads of a workgroup, folded into
// this thread's mn / mx: up to eight pairs per thread are requested before the first is used
__device__ __forceinline__ void conv_fold_partial_ranges(const float *part, int nparts, int tid, int nthr, float &mn, float &mx)
{
    const float4 *p4 = reinterpret_cast<const float4 *>(part);
    const int n4 = nparts >> 1;
    float4 t[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int i = tid + k * nthr;
        t[k] = i < n4 ? p4[i] : make_float4(INFINITY, -INFINITY, INFINITY, -INFINITY);
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
        mn = fminf(mn, fminf(t[k].x, t[k].z));
        mx = fmaxf(mx, fmaxf(t[k].y, t[k].w));
    }
    for (int i = tid + 4 * nthr; i < n4; i += nthr) {
        const float4 u = p4[i];
        mn = fminf(mn, fminf(u.x, u.z));
        mx = fmaxf(mx, fmaxf(u.y, u.w));
    }
    if ((nparts & 1) && tid == 0) {
        mn = fminf(mn, part[(nparts - 1) * 2]);
        mx = fmaxf(mx, part[(nparts - 1) * 2 + 1]);
    }
}

hipError_t launch_quantize_activations(const float *x, int64_t numel, float scale, float zp,
                                       uint8_t *payload, float *scratch_partial, hipStream_t s);
hipError_t launch_dequantize_activations(const uint8_t *payload, uint64_t payload_len, float *out, uint64_t n, hipStream_t s);
// per-channel payloads ([nc u32][chunk u32][scales][zero points][chunk code bytes], chunk = numel / nc); scales and
// zero_points are host arrays of nc values, the header is at most 4 GiB (checked by the caller)
constexpr uint32_t PC_HEADER_VALS = 128;   // header values per launch of the header kernel
hipError_t launch_quantize_activations_per_channel(const float *x, uint64_t x_len, uint64_t numel, uint32_t nc, const float *scales,
                                                   const float *zero_points, uint8_t *payload, uint64_t payload_len, hipStream_t s);
hipError_t launch_dequantize_activations_per_channel(const uint8_t *payload, uint64_t payload_len, float *out, uint64_t out_len, hipStream_t s);
hipError_t launch_qgemm_i8act_generic(int dtype, const I8ActArgs &p, hipStream_t s);
hipError_t launch_row_qsum(const fnn_hip_weight *w, int32_t *out, hipStream_t s);
// phase 0: everything with the direct kernel; 1: range scan + scales; 2: the direct kernel only (scales present);
// 3: range scan only (*nparts = partial ranges per image and group); 4: scales from *nparts partial ranges
hipError_t launch_qconv2d_i8(const QConvArgs &p, hipStream_t s, int phase, int *nparts);
void fnn_conv_coverage(const QConvArgs &p, int *pad_touched, bool *every_input_reached);
// actq[i] = (scale, zero, 0, 0) of an activation payload's header, for i < nbg
hipError_t launch_conv_actq_from_payload(const uint8_t *payload, float *actq, int nbg, hipStream_t s);
