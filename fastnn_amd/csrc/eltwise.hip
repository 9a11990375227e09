// f32 elementwise kernels that sit between quantised layers in a plan
// ("add_f32", "relu_f32", "gelu_f32", "silu_f32"; src/backend/cpu/mod.rs:2699-2751).
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
}  // namespace

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
