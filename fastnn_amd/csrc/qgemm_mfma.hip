// MFMA GEMM path (placeholder until the matrix-core kernels land).
#include "mfma.h"

int fnn_mfma_qmatmul(fnn_hip_ctx *, hipStream_t, const fnn_hip_weight *, const QMatmulArgs &, int, bool *handled)
{
    *handled = false;
    return FNN_OK;
}

int fnn_mfma_qmatmul_i8act(fnn_hip_ctx *, hipStream_t, const fnn_hip_weight *, const I8ActArgs &, bool *handled)
{
    *handled = false;
    return FNN_OK;
}
