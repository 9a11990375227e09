// Shared declarations of the one-launch streaming MatMul (qgemm_stream.hip, qgemm_stream_impl.h).
#pragma once
#include "common.h"

struct StreamArgs {
    const uint32_t *words;
    const float *scales, *zeros, *a, *bias;   // codebook weights: scales = block scales [n][bpr], zeros unused
    const float *codebook;   // codebook weights: the 16 table values
    int64_t bpr;             // ... blocks of 32 values per row
    float *out;
    const float *residual;   // a plan's Add behind this MatMul: sum_out[i] = out[i] + residual[i], or null
    float *sum_out;
    float *part;             // splits > 1: [split][column tile][slot][thread] partial registers, then row sums
    uint32_t *count;         // splits > 1: one arrival counter per column tile, zero between launches
    int64_t m, n, k, kp;
    int act, splits, rounds, ntiles;
    const uint32_t *words_tm;   // non-null: the words in blocks of 16 rows x 64 bytes ([row block][k block][row][64 bytes]),
    int64_t kb64;               // kb64 k blocks per row: a wave load is one contiguous KB
};

constexpr int FNN_STREAM_NW = 8;   // waves per workgroup

// Shape of a launch: blocks of 16 activation rows, row tiles of 16 weight rows per wave, k-values per round, K splits,
// rounds per workgroup, column tiles
struct StreamPlan { int mb, rt, kr, splits, rounds, ntiles; };

// one translation unit per weight type (qgemm_stream_<type>.hip)
hipError_t fnn_stream_launch_i8(const StreamPlan &pl, const StreamArgs &p, hipStream_t s);
hipError_t fnn_stream_launch_i4(const StreamPlan &pl, const StreamArgs &p, hipStream_t s);
hipError_t fnn_stream_launch_u4(const StreamPlan &pl, const StreamArgs &p, hipStream_t s);
hipError_t fnn_stream_launch_u8(const StreamPlan &pl, const StreamArgs &p, hipStream_t s);
hipError_t fnn_stream_launch_f8(const StreamPlan &pl, const StreamArgs &p, hipStream_t s);
hipError_t fnn_stream_launch_f8r(const StreamPlan &pl, const StreamArgs &p, hipStream_t s);
hipError_t fnn_stream_launch_f4(const StreamPlan &pl, const StreamArgs &p, hipStream_t s);
hipError_t fnn_stream_launch_i4cb(const StreamPlan &pl, const StreamArgs &p, hipStream_t s);
