// I8-activation path for gfx950: the "quantize_activations" kernel and the
// "matmul_i8_i8" / "matmul_i4_i8" GEMMs with exact i32 accumulators
// (src/backend/cpu/mod.rs:6928-7008, src/backend/cpu/microkernels/gemm.rs:1641-1975).
#include "common.h"

#include "i8act.h"

namespace {

__global__ void __launch_bounds__(256) absmax_partial_kernel(const float *x, int64_t numel, float *partial)
{
    __shared__ float sm[4];
    float v = 0.0f;
    // (the maximum does not depend on the order: whole 16-byte groups first, the ragged end value by value)
    const bool vec = (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    const int64_t n4 = vec ? numel / 4 : 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        const float4 t = reinterpret_cast<const float4 *>(x)[i];
        v = fmaxf(v, fmaxf(fmaxf(fabsf(t.x), fabsf(t.y)), fmaxf(fabsf(t.z), fabsf(t.w))));  // fmaxf ignores NaN like f32::max
    }
    for (int64_t i = n4 * 4 + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < numel; i += (int64_t)gridDim.x * blockDim.x)
        v = fmaxf(v, fabsf(x[i]));
    v = wave_max(v);
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0) partial[blockIdx.x] = fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3]));
}

// payload = [scale][zp][q...]; q = clamp(round((x - zp)/scale), -128, 127)
__global__ void __launch_bounds__(256)
quantize_act_kernel(const float *x, int64_t numel, const float *partial, int npartial, float scale_in,
                    float zp, uint8_t *payload)
{
    __shared__ float s_scale;
    // the first 16-byte group of every thread is requested before the scale is formed (its latency and that of the
    // partial maxima overlap)
    const bool vec = ((reinterpret_cast<uintptr_t>(x) & 15) | (reinterpret_cast<uintptr_t>(payload) & 3)) == 0;
    const int64_t n4 = vec ? numel / 4 : 0;
    const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    float4 t0 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (first < n4) t0 = reinterpret_cast<const float4 *>(x)[first];
    if (threadIdx.x < 64) {
        float scale = scale_in;
        if (partial) {
            float v = 0.0f;
            for (int i = threadIdx.x; i < npartial; i += 64) v = fmaxf(v, partial[i]);
            v = wave_max(v);
            scale = (v == 0.0f) ? 1.0f : v / 127.0f;
        }
        if (threadIdx.x == 0) s_scale = scale;
    }
    __syncthreads();
    const float scale = s_scale;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        reinterpret_cast<float *>(payload)[0] = scale;
        reinterpret_cast<float *>(payload)[1] = zp;
    }
    int8_t *q = reinterpret_cast<int8_t *>(payload + 8);
    auto code = [&](float xv) {
        const float t = roundf((xv - zp) / scale);
        // clamp keeps NaN and the saturating cast maps NaN to 0
        return (t != t) ? 0 : (int)fminf(fmaxf(t, -128.0f), 127.0f);
    };
    // four values per thread where the input allows 16-byte loads (the payload is 4-byte aligned): one load, one store
    for (int64_t i = first; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        const float4 t = i == first ? t0 : reinterpret_cast<const float4 *>(x)[i];
        const uint32_t w = (uint32_t)(uint8_t)code(t.x) | ((uint32_t)(uint8_t)code(t.y) << 8) | ((uint32_t)(uint8_t)code(t.z) << 16) |
                           ((uint32_t)(uint8_t)code(t.w) << 24);
        reinterpret_cast<uint32_t *>(q)[i] = w;
    }
    for (int64_t i = n4 * 4 + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < numel; i += (int64_t)gridDim.x * blockDim.x)
        q[i] = (int8_t)code(x[i]);
}

template <int DT>
__device__ __forceinline__ void decode_int(uint32_t w, int *o)
{
    if constexpr (DT == FNN_DT_I8) {
        o[0] = (int)(int8_t)(w & 0xff);
        o[1] = (int)(int8_t)((w >> 8) & 0xff);
        o[2] = (int)(int8_t)((w >> 16) & 0xff);
        o[3] = (int)w >> 24;
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = ((int)(w << (28 - 4 * i))) >> 28;
    }
}

constexpr int I8_MT = 4;

// One wave per weight row and tile of 4 activation rows; lanes stride over packed words.
template <int DT>
__global__ void __launch_bounds__(256) qgemm_i8act_generic_kernel(I8ActArgs p)
{
    constexpr int EPW = (DT == FNN_DT_I8) ? 4 : 8;
    const int lane = threadIdx.x & 63;
    const int64_t n = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t m0 = (int64_t)blockIdx.y * I8_MT;
    if (n >= p.n) return;
    const float sa = reinterpret_cast<const float *>(p.payload)[0];
    const float za = reinterpret_cast<const float *>(p.payload)[1];
    const int8_t *qa = reinterpret_cast<const int8_t *>(p.payload + 8);
    const int64_t K = p.k;
    int acc[I8_MT], qs[I8_MT];
    float facc[I8_MT], fsum[I8_MT];
#pragma unroll
    for (int m = 0; m < I8_MT; m++) { acc[m] = qs[m] = 0; facc[m] = fsum[m] = 0.0f; }
    const bool affine = (za != 0.0f);
    for (int64_t wd = lane; wd < p.kp; wd += 64) {
        int wq[EPW];
        decode_int<DT>(p.words[n * p.kp + wd], wq);
#pragma unroll
        for (int e = 0; e < EPW; e++) {
            const int64_t kk = wd * EPW + e;
            if (kk < K) {
#pragma unroll
                for (int m = 0; m < I8_MT; m++) {
                    if (m0 + m < p.m) {
                        int q = qa[(m0 + m) * K + kk];
                        if (affine) {
                            float a = (float)q * sa + za;
                            facc[m] += a * (float)wq[e];
                            fsum[m] += a;
                        } else {
                            acc[m] += wq[e] * q;
                            qs[m] += q;
                        }
                    }
                }
            }
        }
    }
    const float sw = p.scales[n], zw = p.zeros[n];
#pragma unroll
    for (int m = 0; m < I8_MT; m++) {
        if (m0 + m >= p.m) continue;
        float res;
        int a_tot = 0;
        if (affine) {
            float d = wave_sum(facc[m]);
            float s = wave_sum(fsum[m]);
            res = d * sw + zw * s;
        } else {
            a_tot = wave_sum_i32(acc[m]);
            int q_tot = wave_sum_i32(qs[m]);
            float dot = (float)a_tot * sa;
            float input_sum = (float)q_tot * sa + (float)K * za;
            res = dot * sw + zw * input_sum;
        }
        if (lane == 0) {
            if (p.bias) res = res + p.bias[n];
            res = fnn_activation(res, p.act);
            p.out[(m0 + m) * p.n + n] = res;
            if (p.acc_out) p.acc_out[(m0 + m) * p.n + n] = a_tot;
        }
    }
}

// out[i] = q[i]*scale + zp, two roundings as the CPU loop has them (no contraction);
// values past the payload read as q = 0
__global__ void __launch_bounds__(256) dequantize_act_kernel(const uint8_t *payload, uint64_t payload_len, float *out, uint64_t n)
{
    const float scale = payload_len >= 4 ? reinterpret_cast<const float *>(payload)[0] : 1.0f;
    const float zp = payload_len >= 8 ? reinterpret_cast<const float *>(payload)[1] : 0.0f;
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) {
        const int q = (8 + i < payload_len) ? (int)(int8_t)payload[8 + i] : 0;
        out[i] = __fadd_rn(__fmul_rn((float)q, scale), zp);
    }
}

// ---- per-channel payloads, as the reference's loops write and read them (src/backend/cpu/mod.rs:6941-6975,
// 7026-7061): header [num_channels u32][chunk u32][scale f32 x nc][zero point f32 x nc], chunk = numel / nc, and ONE
// block of chunk code bytes behind it that every channel's loop addresses from its start (byte `local` of channel ch
// is the code of x[ch * chunk + local]).  The quantiser's channels run in ascending order, so a byte keeps the code
// of the last channel that has an element at that position; the dequantiser reads the same block for every channel.

struct HeaderVals { float v[PC_HEADER_VALS]; };

// scales [first, first + count) and their zero points into the header (values travel as kernel arguments)
__global__ void __launch_bounds__(PC_HEADER_VALS) pc_header_kernel(uint8_t *payload, uint32_t nc, uint32_t chunk, uint32_t first,
                                                                  uint32_t count, HeaderVals sc, HeaderVals zp)
{
    const uint32_t t = threadIdx.x;
    if (first == 0 && t == 0) {
        reinterpret_cast<uint32_t *>(payload)[0] = nc;
        reinterpret_cast<uint32_t *>(payload)[1] = chunk;
    }
    if (t < count) {
        reinterpret_cast<float *>(payload + 8)[first + t] = sc.v[t];
        reinterpret_cast<float *>(payload + 8 + (size_t)nc * 4)[first + t] = zp.v[t];
    }
}

__global__ void __launch_bounds__(256) quantize_act_pc_kernel(const float *x, uint64_t x_len, uint32_t nc, uint64_t chunk, uint8_t *payload,
                                                              uint64_t payload_len)
{
    const uint64_t header = 8 + (uint64_t)nc * 8;
    const float *sc = reinterpret_cast<const float *>(payload + 8), *zps = sc + nc;
    for (uint64_t local = (uint64_t)blockIdx.x * 256 + threadIdx.x; local < chunk; local += (uint64_t)gridDim.x * 256) {
        if (header + local >= payload_len || local >= x_len) break;   // no room for the byte / no channel has the element
        uint64_t ch = (x_len - 1 - local) / chunk;   // the last channel whose element `local` lies inside the input
        if (ch > nc - 1) ch = nc - 1;
        const float scale = sc[ch], zp = zps[ch];
        int qi = 0;
        if (scale != 0.0f) {
            const float t = roundf((x[ch * chunk + local] - zp) / scale);
            qi = (t != t) ? 0 : (int)fminf(fmaxf(t, -128.0f), 127.0f);   // (a NaN casts to 0)
        }
        payload[header + local] = (uint8_t)(int8_t)qi;
    }
}

__global__ void __launch_bounds__(256) dequantize_act_pc_kernel(const uint8_t *payload, uint64_t payload_len, float *out, uint64_t out_len)
{
    if (payload_len < 8) return;
    const uint64_t nc = reinterpret_cast<const uint32_t *>(payload)[0], chunk = reinterpret_cast<const uint32_t *>(payload)[1];
    const uint64_t data = 8 + nc * 8;
    if (data > payload_len || chunk == 0) return;   // (a header that does not fit its payload: nothing is written)
    const float *sc = reinterpret_cast<const float *>(payload + 8), *zps = sc + nc;
    const uint64_t total = nc * chunk < out_len ? nc * chunk : out_len;
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (uint64_t)gridDim.x * 256) {
        const uint64_t ch = i / chunk, di = data + (i - ch * chunk);
        const int q = di < payload_len ? (int)(int8_t)payload[di] : 0;
        out[i] = __fadd_rn(__fmul_rn((float)q, sc[ch]), zps[ch]);
    }
}

}  // namespace

hipError_t launch_quantize_activations_per_channel(const float *x, uint64_t x_len, uint64_t numel, uint32_t nc, const float *scales,
                                                   const float *zero_points, uint8_t *payload, uint64_t payload_len, hipStream_t s)
{
    const uint64_t chunk = numel / nc;
    for (uint32_t first = 0; first < nc; first += PC_HEADER_VALS) {
        const uint32_t count = nc - first < PC_HEADER_VALS ? nc - first : PC_HEADER_VALS;
        HeaderVals sc, zp;
        for (uint32_t i = 0; i < PC_HEADER_VALS; i++) {
            sc.v[i] = i < count ? scales[first + i] : 0.0f;
            zp.v[i] = i < count ? zero_points[first + i] : 0.0f;
        }
        hipLaunchKernelGGL(pc_header_kernel, dim3(1), dim3(PC_HEADER_VALS), 0, s, payload, nc, (uint32_t)chunk, first, count, sc, zp);
    }
    if (chunk > 0) {
        uint64_t blocks = (chunk + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(quantize_act_pc_kernel, dim3((unsigned)blocks), dim3(256), 0, s, x, x_len, nc, chunk, payload, payload_len);
    }
    return hipGetLastError();
}

hipError_t launch_dequantize_activations_per_channel(const uint8_t *payload, uint64_t payload_len, float *out, uint64_t out_len, hipStream_t s)
{
    if (out_len == 0) return hipSuccess;
    uint64_t blocks = (out_len + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(dequantize_act_pc_kernel, dim3((unsigned)blocks), dim3(256), 0, s, payload, payload_len, out, out_len);
    return hipGetLastError();
}

hipError_t launch_dequantize_activations(const uint8_t *payload, uint64_t payload_len, float *out, uint64_t n, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    uint64_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(dequantize_act_kernel, dim3((unsigned)blocks), dim3(256), 0, s, payload, payload_len, out, n);
    return hipGetLastError();
}

hipError_t launch_quantize_activations(const float *x, int64_t numel, float scale, float zp,
                                       uint8_t *payload, float *scratch_partial, hipStream_t s)
{
    int64_t blocks = (numel + 255) / 256;
    if (blocks > 1024) blocks = 1024;
    if (blocks < 1) blocks = 1;
    int64_t pblocks = blocks;
    const float *partial = nullptr;
    if (!(scale > 0.0f)) {
        // (at most 256 partial maxima: every workgroup of the quantiser reduces them again before its first code)
        if (pblocks > 256) pblocks = 256;
        hipLaunchKernelGGL(absmax_partial_kernel, dim3((unsigned)pblocks), dim3(256), 0, s, x, numel,
                           scratch_partial);
        partial = scratch_partial;
        zp = 0.0f;
    }
    hipLaunchKernelGGL(quantize_act_kernel, dim3((unsigned)blocks), dim3(256), 0, s, x, numel, partial,
                       (int)pblocks, scale, zp, payload);
    return hipGetLastError();
}

hipError_t launch_qgemm_i8act_generic(int dtype, const I8ActArgs &p, hipStream_t s)
{
    const int wpb = 4;
    dim3 grid((unsigned)((p.n + wpb - 1) / wpb), (unsigned)((p.m + I8_MT - 1) / I8_MT));
    if (dtype == FNN_DT_I8)
        hipLaunchKernelGGL((qgemm_i8act_generic_kernel<FNN_DT_I8>), grid, dim3(wpb * 64), 0, s, p);
    else if (dtype == FNN_DT_I4)
        hipLaunchKernelGGL((qgemm_i8act_generic_kernel<FNN_DT_I4>), grid, dim3(wpb * 64), 0, s, p);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}
