// One-launch streaming MatMul, codebook weights with blocks of 32 values (kernels: qgemm_stream_impl.h).
#include "qgemm_stream_impl.h"

hipError_t fnn_stream_launch_i4cb(const StreamPlan &pl, const StreamArgs &p, hipStream_t s) { return launch_dt<FNN_DT_I4CB>(pl, p, s); }
