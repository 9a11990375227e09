// Shared declarations of libfastnn_hip: weight handle, codecs, epilogue, wave helpers.
// gfx950 only: 64-lane wavefronts, DPP row operations, hardware FP8/BF8/FP4 converts.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fastnn_hip.h"

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// A registered weight: the packed words of fastnn's PackedTensor (row-major,
// row r at word r*kp, lane i of a word at bits [i*w,(i+1)*w)) plus its side tables.
struct fnn_hip_weight {
    uint64_t key;
    int dtype;
    int64_t rows;       // N (MatMul) or OC (Conv2d)
    int64_t inner;      // K or IC/g*KH*KW
    int items;          // lanes per word: 4 or 8
    int64_t kp;         // words per row = ceil(inner/items)
    uint32_t *words;    // device; rows*kp words followed by zeroed padding
    float *scales;      // device; [rows] (grouped/scalar scales are expanded) or [rows*bpr] for I4CB
    float *zeros;       // device; [rows]
    float *codebook;    // device; 16 floats (I4CB) or nullptr
    int32_t *row_qsum;  // device; [rows] sum of integer lanes per row (I8/I4), for the conv epilogue
    float *umean;       // device; [rows] mean lane value per row, built on first single-pass GEMM use
    uint32_t *words4;   // device; rows re-strided to kp4 = ceil4(kp) words (+16 zero words) when kp % 4 != 0,
    int64_t kp4;        //         built on first use by a kernel that fetches 16-byte pieces of a row
    uint32_t *words_tm; // device; the packed words in blocks of 16 rows x 64 bytes (row block major, then k block), rows padded to
                        // whole blocks with zeros: the int8 GEMV's wave loads are one contiguous KB each; built on first use
    void *dense16;      // device; codebook type: rows expanded to f16 [hi(K) | lo(K)] + per-row scale tables, built on the
                        //         first MatMul with M >= 5 and kept (the CPU path keeps an f32 copy: packed_tensor.rs:469-521)
    int qblock;         // I4CB block length along inner
    int64_t bpr;        // blocks per row
    struct fnn_hip_ctx *ctx;
};

// ---------------------------------------------------------------------------
// wave helpers
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}

// Sum over each DPP row of 16 lanes; every lane of the row ends with the total.
__device__ __forceinline__ float row16_sum(float v)
{
    v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);  // row_half_mirror
    v += dpp_f32<0x140>(v);  // row_mirror
    return v;
}
__device__ __forceinline__ int row16_sum_i32(int v)
{
    v += dpp_i32<0xB1>(v);
    v += dpp_i32<0x4E>(v);
    v += dpp_i32<0x141>(v);
    v += dpp_i32<0x140>(v);
    return v;
}

// Sum over the whole 64-lane wave; every lane ends with the total.
__device__ __forceinline__ float wave_sum(float v)
{
    v = row16_sum(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
__device__ __forceinline__ int wave_sum_i32(int v)
{
    v = row16_sum_i32(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
__device__ __forceinline__ float wave_min(float v)
{
    v = fminf(v, dpp_f32<0xB1>(v));
    v = fminf(v, dpp_f32<0x4E>(v));
    v = fminf(v, dpp_f32<0x141>(v));
    v = fminf(v, dpp_f32<0x140>(v));
    v = fminf(v, __shfl_xor(v, 16, 64));
    v = fminf(v, __shfl_xor(v, 32, 64));
    return v;
}
__device__ __forceinline__ float wave_max(float v)
{
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    v = fmaxf(v, dpp_f32<0x140>(v));
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

// The same reductions with a wave-uniform result (scalar registers): rows of 16 lanes by DPP, then the four row
// results are read with v_readlane instead of two round trips through the LDS permute path.
__device__ __forceinline__ float wave_max_uniform(float v)
{
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    v = fmaxf(v, dpp_f32<0x140>(v));
    const int b = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0)), r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32)), r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}
__device__ __forceinline__ float wave_sum_uniform(float v)
{
    v = row16_sum(v);
    const int b = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0)), r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32)), r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}

// ---------------------------------------------------------------------------
// word codecs: raw lane value u(w) as f32, before scale/zero
// (src/dtypes/{i8x4,i4x8,u8x4,u4x8,f8x4,f8x4r,f4x8}.rs unpack_to_f32).
// The F8 words held on the device have every exponent-15 byte rewritten to
// 0x7F/0xFF, and the F4 words every 0x8 nibble rewritten to 0x0, so that the
// hardware OCP converts give exactly the reference's values (NaN, +0.0).
// ---------------------------------------------------------------------------
template <int DT>
struct Codec;

template <>
struct Codec<FNN_DT_I8> {
    static constexpr int EPW = 4;
    __device__ static __forceinline__ void decode(uint32_t w, float *o)
    {
        o[0] = (float)(int)(int8_t)(w & 0xff);
        o[1] = (float)(int)(int8_t)((w >> 8) & 0xff);
        o[2] = (float)(int)(int8_t)((w >> 16) & 0xff);
        o[3] = (float)((int)w >> 24);
    }
};
template <>
struct Codec<FNN_DT_U8> {
    static constexpr int EPW = 4;
    __device__ static __forceinline__ void decode(uint32_t w, float *o)
    {
        o[0] = (float)(w & 0xff);
        o[1] = (float)((w >> 8) & 0xff);
        o[2] = (float)((w >> 16) & 0xff);
        o[3] = (float)(w >> 24);
    }
};
template <>
struct Codec<FNN_DT_I4> {
    static constexpr int EPW = 8;
    __device__ static __forceinline__ void decode(uint32_t w, float *o)
    {
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = (float)(((int)(w << (28 - 4 * i))) >> 28);
    }
};
template <>
struct Codec<FNN_DT_U4> {
    static constexpr int EPW = 8;
    __device__ static __forceinline__ void decode(uint32_t w, float *o)
    {
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = (float)((w >> (4 * i)) & 0xf);
    }
};
template <>
struct Codec<FNN_DT_F8> {
    static constexpr int EPW = 4;
    __device__ static __forceinline__ void decode(uint32_t w, float *o)
    {
        f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
        f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
        o[0] = lo[0]; o[1] = lo[1]; o[2] = hi[0]; o[3] = hi[1];
    }
};
template <>
struct Codec<FNN_DT_F8R> {
    static constexpr int EPW = 4;
    __device__ static __forceinline__ void decode(uint32_t w, float *o)
    {
        f32x2 lo = __builtin_amdgcn_cvt_pk_f32_bf8((int)w, false);
        f32x2 hi = __builtin_amdgcn_cvt_pk_f32_bf8((int)w, true);
        o[0] = lo[0]; o[1] = lo[1]; o[2] = hi[0]; o[3] = hi[1];
    }
};
template <>
struct Codec<FNN_DT_F4> {
    static constexpr int EPW = 8;
    __device__ static __forceinline__ void decode(uint32_t w, float *o)
    {
        f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0);
        f32x2 b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1);
        f32x2 c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2);
        f32x2 d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3);
        o[0] = a[0]; o[1] = a[1]; o[2] = b[0]; o[3] = b[1];
        o[4] = c[0]; o[5] = c[1]; o[6] = d[0]; o[7] = d[1];
    }
};
// I4CB: lanes are codebook indices; decode() needs the table (in LDS).
template <>
struct Codec<FNN_DT_I4CB> {
    static constexpr int EPW = 8;
    __device__ static __forceinline__ void decode_cb(uint32_t w, const float *cb, float *o)
    {
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = cb[(w >> (4 * i)) & 0xf];
    }
};

// ---------------------------------------------------------------------------
// epilogue: apply_affine_dot (src/backend/cpu/microkernels/mod.rs:292-295)
// then bias add and activation (src/backend/cpu/microkernels/activations.rs:557-593)
// ---------------------------------------------------------------------------
// x / (1 + exp(-x)) on the hardware exponential and reciprocal (v_exp_f32 of -x*log2(e), v_rcp_f32, one ulp each; the
// rounded product adds |x| * 6e-8 to the exponential's relative error, which reaches the result scaled by
// e/(1+e)): a few ulp of the result for x > -4 and below 1e-8 in absolute terms for smaller x, where the result
// itself vanishes; about 6 instructions against ~35 for expf and an IEEE division.
__device__ __forceinline__ float fnn_sigmoid_times(float x, float arg)   // x * sigmoid(arg)
{
    const float e = __builtin_amdgcn_exp2f(arg * -1.44269504f);   // exp(-arg); inf for arg < -88.7, 0 for arg > 103
    return x * __builtin_amdgcn_rcpf(1.0f + e);                    // x * 0 where e = inf, as x / inf
}
__device__ __forceinline__ float fnn_activation(float v, int act)
{
    if (act == FNN_ACT_RELU) return v > 0.0f ? v : 0.0f;
    if (act == FNN_ACT_GELU) {
        // 0.5 * v * (1 + tanh(t)) = v * sigmoid(2t), t = 0.7978846 * (v + 0.044715 * v^3): the same function without
        // the cancellation of 1 + tanh for negative v
        float x3 = v * v * v;
        float t = 0.7978846f * (v + 0.044715f * x3);
        return fnn_sigmoid_times(v, 2.0f * t);
    }
    if (act == FNN_ACT_SILU) return fnn_sigmoid_times(v, v);
    return v;
}

__device__ __forceinline__ float fnn_epilogue(float dot, float scale, float zero, float xsum,
                                              const float *bias, int64_t n, int act)
{
    float v = dot * scale + zero * xsum;
    if (bias) v = v + bias[n];
    return fnn_activation(v, act);
}

// n / d for 0 <= n < 2^31 by one multiplication (d >= 1 fixed per launch): mul = ceil(2^(31 + ceil(log2 d)) / d)
struct FastDiv {
    uint32_t d, mul, shr;
    __device__ __forceinline__ uint32_t div(uint32_t n) const { return d == 1 ? n : __umulhi(n, mul) >> shr; }
};
static inline FastDiv fast_div(uint32_t d)
{
    FastDiv f = {d, 0, 0};
    if (d <= 1) { f.d = 1; return f; }
    uint32_t lg = 0;
    while ((1ull << lg) < d) lg++;
    const uint64_t p2 = 1ull << (31 + lg);
    f.mul = (uint32_t)((p2 + d - 1) / d);
    f.shr = lg - 1;
    return f;
}

// ---------------------------------------------------------------------------
// launch parameter blocks
// ---------------------------------------------------------------------------
struct QMatmulArgs {
    const uint32_t *words;
    const float *scales;   // [N] or block scales [N*bpr] (I4CB)
    const float *zeros;    // [N]
    const float *codebook; // I4CB
    const float *a;        // [M,K]
    const float *bias;     // [N] or null
    float *out;            // [M,N]
    int64_t m, n, k, kp, bpr;
    int qblock;
    int act;
    int as_written;        // I4CB: treat the [N,K] dequantised buffer as [K,N]
};

// launchers implemented in the kernel translation units
hipError_t launch_qgemv(int dtype, const QMatmulArgs &p, hipStream_t s, bool *handled);
hipError_t launch_qgemm_generic(int dtype, const QMatmulArgs &p, hipStream_t s);
hipError_t launch_dequant(const fnn_hip_weight *w, float *out, hipStream_t s);
