// Value ranges that travel with an f32 tensor from the call that writes it to the quantised Conv2d that reads it:
// the convolution's dynamic activation quantiser needs min / max of its input per image
// (src/backend/cpu/im2col.rs:496-507), and a producer that has every value in registers anyway can leave partial
// (min, max) pairs per image behind, which saves the consumer its scan of the tensor.
//
// A table is [images][stride][2] floats; a producer fills `parts` pairs per image (unused ones hold +inf, -inf).
// The side channel below belongs to one context and to the NEXT call on it: the caller states what it wants
// before the call and reads what happened after it.
#pragma once
#include <cstdint>

struct fnn_hip_ctx;

struct FnnRangeIo {
    // request to the next call that writes an f32 tensor: leave partial ranges of the output, split in images of
    // image_elems values, in out_table (room for out_stride pairs per image)
    float *out_table = nullptr;
    int out_stride = 0;
    uint64_t out_image_elems = 0, out_images = 0;
    int out_parts = 0;        // pairs per image in place: a call appends behind them (a tensor written by several calls,
                              // e.g. the parts of a concat) and adds what it wrote; 0 after a single call: none
    int out_failed = 0;       // answer: a call wrote values of the tensor without leaving their ranges
    // answer of a convolution: the pairs it left are grouped by blocks of output channels, out_tile_pairs pairs per
    // block and image, block after block; a block is out_tile_elems values of an image (channels x pixels).  A reader
    // of whole blocks of a ONE-image tensor takes just their pairs.  0: not grouped
    uint64_t out_tile_elems = 0;
    int out_tile_pairs = 0;
    // offer to the next quantised Conv2d: partial ranges of its input, one image per batch entry
    const float *in_table = nullptr;
    int in_stride = 0, in_parts = 0;
    int in_used = 0;          // answer: the convolution took them instead of scanning its input
};

FnnRangeIo *fnn_ctx_range_io(fnn_hip_ctx *ctx);
bool fnn_ctx_capturing(fnn_hip_ctx *ctx);   // a HIP graph is being recorded on the context's stream: no allocation

// A residual that travels with a MatMul or quantised Conv2d call: a plan's MatMul (Conv2d) followed by an Add of its
// output and another tensor can finish as one call.  The caller states the other operand and where the sum goes before the MatMul call (which
// still writes its own output); `used` tells afterwards whether the call's last kernel stored the sum as well (then
// sum_out[i] = out[i] + residual[i], the same f32 addition the Add would have done), else the caller runs the Add.
struct FnnResidualIo {
    const float *residual = nullptr;
    float *sum_out = nullptr;
    const float *of_out = nullptr;   // the MatMul (Conv2d) output the request is about
    uint64_t elems = 0;              // M * N (B * OC * HO * WO)
    int used = 0;
};
FnnResidualIo *fnn_ctx_residual_io(fnn_hip_ctx *ctx);

// A prepared MatMul operand that travels from one MatMul call to the next: at 17 <= M the f16 matrix-core path
// first turns its f32 activations into scaled f16 hi + lo operand rows (a launch of its own).  When the caller knows
// that the next call on the context is the MatMul reading this one's result, the split-K reduction of this call can
// leave that operand behind (it has the whole result row in registers), and the next call skips its preparation.
// The conversion code is the same, so results are identical.
struct fnn_hip_weight;
struct FnnPrepIo {
    // request to the next MatMul call: also prepare the operand of a MatMul with weight next_w and flags next_flags
    // that reads next_a (this call's output, or the sum it stores for a residual)
    const fnn_hip_weight *next_w = nullptr;
    int next_flags = 0;
    const float *next_a = nullptr;
    int produced = 0;        // answer: done
    // offer to the next MatMul call: no call has touched the context since the one that produced its operand
    int offered = 0;
    int consumed = 0;        // answer: the call used it
};
FnnPrepIo *fnn_ctx_prep_io(fnn_hip_ctx *ctx);
// what a producing call left behind (library-private record, checked field by field by the consuming call)
struct FnnPreparedOperand {
    const float *a = nullptr;       // the f32 tensor the operand was made from
    void *buffer = nullptr;         // operand rows + row tables
    int slot = -1;                  // workspace slot of buffer
    long long m = 0, k = 0, kpad = 0, rows_pad = 0;
    int precise = 0, interleaved = 0;
};
FnnPreparedOperand *fnn_ctx_prepared(fnn_hip_ctx *ctx);
