// One-launch streaming MatMul, I4 weights (kernels: qgemm_stream_impl.h).
#include "qgemm_stream_impl.h"

hipError_t fnn_stream_launch_i4(const StreamPlan &pl, const StreamArgs &p, hipStream_t s) { return launch_dt<FNN_DT_I4>(pl, p, s); }
