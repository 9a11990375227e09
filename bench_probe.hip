// Device-ceiling probes, built by bench.py as a library of their own (libbench_probe.so): not part of the product ABI.
// A plain streaming read and a plain copy of a known number of bytes give (a) the bandwidth one launch of a
// given size can reach on this device, the ceiling a bandwidth-bound kernel of that size is judged against,
// and (b) a kernel of known traffic to scale hardware byte counters with.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

// A workgroup of 256 lanes walks chunks of 256*U consecutive 16-byte pieces; a lane has U independent loads
// in flight (addresses past the end are clamped to the last piece and their values masked).
template <int U>
__global__ void __launch_bounds__(256) probe_read_kernel(const uint4 *__restrict__ src, size_t n16, uint32_t *sink)
{
    const size_t nchunks = (n16 + 256 * U - 1) / (256 * U);
    uint32_t acc = 0;
    for (size_t chunk = blockIdx.x; chunk < nchunks; chunk += gridDim.x) {
        const size_t base = chunk * 256 * U + threadIdx.x;
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t i = base + (size_t)u * 256;
            v[u] = src[i < n16 ? i : n16 - 1];
        }
#pragma unroll
        for (int u = 0; u < U; u++) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;  // practically never true: keeps the loads alive
}

// The read pattern of the int8 GEMV kernel and nothing else: a workgroup of 8 waves owns RT * 16 consecutive rows
// of row_bytes bytes; wave w owns the byte columns [w * seg, (w + 1) * seg) of them (seg = 256: a slice of 512 4-bit
// values); lane (row ln = lane & 15, group g = lane >> 4) requests bytes [l * 64 + g * 16, +16) of its segment in
// every row tile, l = 0 .. seg / 64 - 1: RT * seg / 64 loads of 16 bytes per lane, each wave-load 16 rows x 64 bytes.
template <int RT>
__global__ void __launch_bounds__(512) probe_gemv_pattern_kernel(const unsigned char *__restrict__ src, size_t rows, size_t row_bytes,
                                                                 uint32_t *sink)
{
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, ln = lane & 15, g = lane >> 4;
    const size_t n0 = (size_t)blockIdx.x * (16 * RT);
    uint32_t acc = 0;
    for (size_t seg0 = (size_t)wv * 256; seg0 < row_bytes; seg0 += 8 * 256) {
        uint4 v[RT][4];
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int l = 0; l < 4; l++) {
                size_t row = n0 + r * 16 + ln;
                if (row >= rows) row = rows - 1;
                v[r][l] = *reinterpret_cast<const uint4 *>(src + row * row_bytes + seg0 + l * 64 + g * 16);
            }
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int l = 0; l < 4; l++) acc += v[r][l].x ^ v[r][l].y ^ v[r][l].z ^ v[r][l].w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;
}

template <int U>
__global__ void __launch_bounds__(256) probe_copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n16)
{
    const size_t nchunks = (n16 + 256 * U - 1) / (256 * U);
    for (size_t chunk = blockIdx.x; chunk < nchunks; chunk += gridDim.x) {
        const size_t base = chunk * 256 * U + threadIdx.x;
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t i = base + (size_t)u * 256;
            v[u] = src[i < n16 ? i : n16 - 1];
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t i = base + (size_t)u * 256;
            if (i < n16) dst[i] = v[u];
        }
    }
}

// Matrix-core ceiling: every wave issues nothing but MFMAs on ACCS independent accumulator tiles (operands are
// pseudo-random register values, so that the datapath toggles as it does on real data), `iters` rounds of ACCS
// instructions; no memory traffic inside the loop.  What a launch of this kernel sustains is what the matrix cores
// of this device deliver under their power limit, with nothing else in the way.
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

template <bool INT8, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) probe_mfma_kernel(int iters, uint32_t seed, uint32_t *sink)
{
    constexpr int ACCS = 4;
    uint32_t x = seed ^ (threadIdx.x * 2654435761u) ^ (blockIdx.x * 40503u);
    auto next = [&]() { x ^= x << 13; x ^= x >> 17; x ^= x << 5; return x; };
    i32x4 a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        if (INT8) {
            a[i] = i32x4{(int)next(), (int)next(), (int)next(), (int)next()};
            b[i] = i32x4{(int)next(), (int)next(), (int)next(), (int)next()};
        } else {   // f16 values of moderate size: exponent bits 01110/01111, random mantissas and signs
            auto h2 = [&]() { return (int)((next() & 0x83FF83FFu) | 0x38003C00u); };
            a[i] = i32x4{h2(), h2(), h2(), h2()};
            b[i] = i32x4{h2(), h2(), h2(), h2()};
        }
    }
    f32x16 acc[ACCS];
#pragma unroll
    for (int t = 0; t < ACCS; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[t][i] = 0.0f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int t = 0; t < ACCS; t++) {
            if constexpr (INT8)
                acc[t] = __builtin_bit_cast(f32x16, __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t & 1], b[(t >> 1) & 1],
                                                                                        __builtin_bit_cast(i32x16, acc[t]), 0, 0, 0));
            else
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[t & 1]), __builtin_bit_cast(f16x8, b[(t >> 1) & 1]),
                                                              acc[t], 0, 0, 0);
        }
    }
    uint32_t r = 0;
#pragma unroll
    for (int t = 0; t < ACCS; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) r ^= __float_as_uint(acc[t][i]);
    if (r == 0x9e3779b9u) sink[0] = r;   // practically never true: keeps the accumulators alive
}

// HBM / L2 -> LDS delivery: every wave of a workgroup issues LPW `global_load_lds_dwordx4` (1 KB each) per stage into
// a ring of NS stages, one workgroup barrier per stage, no other work.  The source is a small region re-read by all
// workgroups (L2 hits), so the figure is what the load path into the LDS delivers per CU for a given number of waves.
template <int WAVES, int LPW, int NS>
__global__ void __launch_bounds__(WAVES * 64) probe_lds_kernel(const uint4 *src, size_t region16, int iters, uint32_t *sink)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)smem;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    constexpr int STAGE = WAVES * LPW * 1024;
    const uint4 *base = src + (size_t)(blockIdx.x % 64) * region16;
    uint32_t acc = 0;
    auto issue = [&](int it, int buf) {
#pragma unroll
        for (int j = 0; j < LPW; j++) {
            const size_t idx = ((size_t)it * WAVES * LPW + wv * LPW + j) * 64 + lane;
            const uint4 *g = base + (idx % region16);
            const unsigned dst = __builtin_amdgcn_readfirstlane(lds0 + buf * STAGE + (wv * LPW + j) * 1024);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(g) : "memory");
        }
    };
    for (int s = 0; s < NS - 1; s++) issue(s, s);
    int buf = 0;
    for (int it = 0; it < iters; it++) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 2) * LPW) : "memory");
        __syncthreads();
        int fb = buf + NS - 1;
        if (fb >= NS) fb -= NS;
        issue(it + NS - 1, fb);
        acc ^= reinterpret_cast<const uint32_t *>(smem + buf * STAGE)[tid * 4];
        buf = buf + 1 == NS ? 0 : buf + 1;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // nothing may still be writing LDS when the workgroup retires
    __syncthreads();
    if (acc == 0x9e3779b9u) sink[0] = acc;
}

template <int WAVES, int LPW, int NS>
hipError_t launch_lds(const void *src, size_t region16, int workgroups, int iters, uint32_t *sink, hipStream_t s)
{
    constexpr size_t lds = (size_t)NS * WAVES * LPW * 1024;
    auto kern = probe_lds_kernel<WAVES, LPW, NS>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)workgroups), dim3(WAVES * 64), lds, s, reinterpret_cast<const uint4 *>(src), region16, iters, sink);
    return hipGetLastError();
}

template <int U>
hipError_t launch(const void *src, void *dst, size_t n16, unsigned grid, uint32_t *sink, hipStream_t s)
{
    if (dst)
        hipLaunchKernelGGL(probe_copy_kernel<U>, dim3(grid), dim3(256), 0, s, reinterpret_cast<const uint4 *>(src),
                           reinterpret_cast<uint4 *>(dst), n16);
    else
        hipLaunchKernelGGL(probe_read_kernel<U>, dim3(grid), dim3(256), 0, s, reinterpret_cast<const uint4 *>(src), n16, sink);
    return hipGetLastError();
}

}  // namespace

// One launch on `stream` (a hipStream_t) that reads `bytes` from src_dev, and writes them to dst_dev unless that
// is NULL.  loads_per_lane: 1, 2, 4 or 8 independent 16-byte loads per lane and trip; workgroups: 0 = one per
// chunk (everything requested at once), else a fixed grid walking the chunks.  sink_dev: 4 writable bytes.
// Returns 0 or the hipError_t value.
extern "C" int fnn_probe_stream(void *stream, const void *src_dev, void *dst_dev, size_t bytes, int loads_per_lane,
                                int workgroups, void *sink_dev)
{
    if (!src_dev || !sink_dev) return (int)hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(src_dev) & 15) || (reinterpret_cast<uintptr_t>(dst_dev) & 15)) return (int)hipErrorInvalidValue;
    const size_t n16 = bytes / 16;
    if (n16 == 0) return 0;
    const int u = loads_per_lane;
    if (u != 1 && u != 2 && u != 4 && u != 8) return (int)hipErrorInvalidValue;
    const size_t nchunks = (n16 + 256 * (size_t)u - 1) / (256 * (size_t)u);
    size_t grid = workgroups > 0 ? (size_t)workgroups : nchunks;
    if (grid > nchunks) grid = nchunks;
    if (grid > 0x7fffffffu) grid = 0x7fffffffu;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    uint32_t *sink = reinterpret_cast<uint32_t *>(sink_dev);
    switch (u) {
    case 1: return (int)launch<1>(src_dev, dst_dev, n16, (unsigned)grid, sink, s);
    case 2: return (int)launch<2>(src_dev, dst_dev, n16, (unsigned)grid, sink, s);
    case 4: return (int)launch<4>(src_dev, dst_dev, n16, (unsigned)grid, sink, s);
    default: return (int)launch<8>(src_dev, dst_dev, n16, (unsigned)grid, sink, s);
    }
}

// One launch on `stream` that reads rows x row_bytes bytes (row_bytes a multiple of 2048) in the int8 GEMV kernel's
// order: workgroups of 8 waves over row_tiles * 16 rows (row_tiles 1, 2 or 3).  Returns 0 or the hipError_t value.
extern "C" int fnn_probe_gemv_pattern(void *stream, const void *src_dev, size_t rows, size_t row_bytes, int row_tiles, void *sink_dev)
{
    if (!src_dev || !sink_dev || rows < 1 || row_bytes < 2048 || row_bytes % 2048 || row_tiles < 1 || row_tiles > 3) return (int)hipErrorInvalidValue;
    if (reinterpret_cast<uintptr_t>(src_dev) & 15) return (int)hipErrorInvalidValue;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    uint32_t *sink = reinterpret_cast<uint32_t *>(sink_dev);
    const unsigned char *src = reinterpret_cast<const unsigned char *>(src_dev);
    const dim3 grid((unsigned)((rows + 16 * row_tiles - 1) / (16 * row_tiles)));
    if (row_tiles == 1) hipLaunchKernelGGL(probe_gemv_pattern_kernel<1>, grid, dim3(512), 0, s, src, rows, row_bytes, sink);
    else if (row_tiles == 2) hipLaunchKernelGGL(probe_gemv_pattern_kernel<2>, grid, dim3(512), 0, s, src, rows, row_bytes, sink);
    else hipLaunchKernelGGL(probe_gemv_pattern_kernel<3>, grid, dim3(512), 0, s, src, rows, row_bytes, sink);
    return (int)hipGetLastError();
}

// One launch on `stream` of a kernel that only issues matrix-core instructions: kind 0 = v_mfma_f32_32x32x16_f16
// (32768 flop each), 1 = v_mfma_i32_32x32x32_i8 (65536 op each); `workgroups` workgroups of `waves` (4 or 8) waves,
// each wave 4 * iters instructions.  sink_dev: 4 writable bytes.  Returns 0 or the hipError_t value.
extern "C" int fnn_probe_mfma(void *stream, int kind, int workgroups, int waves, int iters, void *sink_dev)
{
    if (!sink_dev || workgroups < 1 || iters < 1 || (waves != 4 && waves != 8) || (kind != 0 && kind != 1)) return (int)hipErrorInvalidValue;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    uint32_t *sink = reinterpret_cast<uint32_t *>(sink_dev);
    const dim3 grid((unsigned)workgroups);
    if (kind == 0 && waves == 4) hipLaunchKernelGGL((probe_mfma_kernel<false, 4>), grid, dim3(256), 0, s, iters, 0x1234567u, sink);
    else if (kind == 0) hipLaunchKernelGGL((probe_mfma_kernel<false, 8>), grid, dim3(512), 0, s, iters, 0x1234567u, sink);
    else if (waves == 4) hipLaunchKernelGGL((probe_mfma_kernel<true, 4>), grid, dim3(256), 0, s, iters, 0x1234567u, sink);
    else hipLaunchKernelGGL((probe_mfma_kernel<true, 8>), grid, dim3(512), 0, s, iters, 0x1234567u, sink);
    return (int)hipGetLastError();
}

// One launch on `stream` of the LDS delivery loop: `workgroups` workgroups of `waves` waves (4, 8 or 16; 4 loads of
// 1 KB per wave and stage for 4 and 8 waves, 2 for 16), ring of `stages` (3 or 6) stages, `iters` stages per workgroup;
// src_dev: at least 8 MiB (64 regions of 128 KiB, re-read by all workgroups).  *bytes_out = bytes delivered into LDS by
// the launch.  Returns 0 or the hipError_t value.
extern "C" int fnn_probe_lds_delivery(void *stream, const void *src_dev, int waves, int stages, int workgroups, int iters,
                                      void *sink_dev, double *bytes_out)
{
    if (!src_dev || !sink_dev || workgroups < 1 || iters < 1) return (int)hipErrorInvalidValue;
    if ((waves != 4 && waves != 8 && waves != 16) || (stages != 3 && stages != 6) || (waves == 16 && stages == 6)) return (int)hipErrorInvalidValue;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    uint32_t *sink = reinterpret_cast<uint32_t *>(sink_dev);
    const size_t region16 = 8192;
    const int lpw = (waves == 16 || (waves == 8 && stages == 6)) ? 2 : 4;
    if (bytes_out) *bytes_out = (double)workgroups * (iters + stages - 1) * waves * lpw * 1024.0;
    if (waves == 4 && stages == 3) return (int)launch_lds<4, 4, 3>(src_dev, region16, workgroups, iters, sink, s);
    if (waves == 4) return (int)launch_lds<4, 4, 6>(src_dev, region16, workgroups, iters, sink, s);
    if (waves == 8 && stages == 3) return (int)launch_lds<8, 4, 3>(src_dev, region16, workgroups, iters, sink, s);
    if (waves == 8) return (int)launch_lds<8, 2, 6>(src_dev, region16, workgroups, iters, sink, s);
    return (int)launch_lds<16, 2, 3>(src_dev, region16, workgroups, iters, sink, s);
}
