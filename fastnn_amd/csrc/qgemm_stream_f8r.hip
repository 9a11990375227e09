// One-launch streaming MatMul, F8R weights (kernels: qgemm_stream_impl.h).
#include "qgemm_stream_impl.h"

hipError_t fnn_stream_launch_f8r(const StreamPlan &pl, const StreamArgs &p, hipStream_t s) { return launch_dt<FNN_DT_F8R>(pl, p, s); }
