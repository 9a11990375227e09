// Matrix-core kernel entry points.
#pragma once
#include "common.h"
#include "i8act.h"

// context services implemented beside the C ABI
int fnn_ctx_ensure_tmp(fnn_hip_ctx *ctx, int which, size_t bytes, void **ptr);
int fnn_ctx_fail(fnn_hip_ctx *ctx, int code, const char *msg);
bool fnn_ctx_capturing(fnn_hip_ctx *ctx);

// M >= 5: activations prepared once as f16 operands, 4-wave output tiles with the
// activations staged through LDS and optional split of K (deterministic reduction).
int fnn_tiled_qmatmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &p,
                      int flags, bool *handled);

// single-f16 activation mode: mean lane value per weight row (null for types whose lanes have zero mean)
int fnn_row_means(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const float **umean);

// M <= 8: bandwidth-bound GEMV on the matrix cores (weights requested before anything else).
int fnn_mfma_qgemv(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &p,
                   int flags, bool *handled);

// 9 <= M <= 16: the same organisation with the 16 activation rows as the MFMA operand rows, loaded straight
// into registers (no preparation or reduction launch).
int fnn_mfma_rows16(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &p,
                    int flags, bool *handled);

// I8 activations x I8/I4 weights and the quantised Conv2d on int8 MFMA tiles with i32 accumulators.
int fnn_i8_tiled_matmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const I8ActArgs &p, bool *handled);
// p.actq must already hold the (image, group) activation scales.
int fnn_i8_tiled_conv(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QConvArgs &p, bool *handled);

// Weight rows as 16-byte addressable pieces: the registered words, or (when kp % 4 != 0) a copy with the
// rows re-strided to a multiple of four words, zero-filled, made on first use and kept with the weight.
int fnn_aligned_rows(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const uint32_t **words, int64_t *kp);
