// Matrix-core kernel entry points.
#pragma once
#include <atomic>

#include "common.h"
#include "i8act.h"

// context services implemented beside the C ABI
int fnn_ctx_ensure_tmp(fnn_hip_ctx *ctx, int which, size_t bytes, void **ptr);
int fnn_ctx_fail(fnn_hip_ctx *ctx, int code, const char *msg);
bool fnn_ctx_capturing(fnn_hip_ctx *ctx);
// true while device memory must not be allocated: graph capture, or a call through fnn_hip_qmatmul_static
bool fnn_ctx_no_alloc(fnn_hip_ctx *ctx);
bool fnn_ctx_static_mode(fnn_hip_ctx *ctx);
// value of a per-context option (FNN_OPT_*, set through fnn_hip_set_option)
int64_t fnn_ctx_option(const fnn_hip_ctx *ctx, int option);

// Raises a kernel's dynamic LDS limit once per device.  `done` is a bit mask of devices (one static per kernel
// instantiation); safe from several threads, and a second device gets its own call.
inline hipError_t fnn_raise_lds_limit(std::atomic<uint64_t> &done, const void *kernel, int bytes)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return e;
}

// M >= 5: activations prepared once as f16 operands, 4-wave output tiles with the
// activations staged through LDS and optional split of K (deterministic reduction).
// 17 <= M <= 32: one launch, weights streamed into the MFMA operand registers, activations converted in the kernel,
// K split over workgroups and reduced by the last one to arrive (qgemm_stream.hip)
int fnn_stream_qmatmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &p, int flags, bool *handled);
// arrival counters of that kernel's column tiles: FNN_STREAM_COUNTERS words of device memory, zero between launches
constexpr int FNN_STREAM_COUNTERS = 4096;
uint32_t *fnn_ctx_stream_counters(fnn_hip_ctx *ctx);
// int8 matrix-core GEMM over exact activation digit planes (qgemm_digits.hip): M >= 17, I8 / I4 / U4 weights
int fnn_digits_qmatmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &p, int flags, bool *handled);
int fnn_tiled_qmatmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &p,
                      int flags, bool *handled);
// FNN_FLAG_ACT_QUANT with F8 weights: activations rounded to E4M3 (one power-of-two scale per row), fp8 matrix cores
int fnn_fp8_actquant_qmatmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &p, bool *handled);

int64_t fnn_conv_operand_workgroups(const QConvArgs &p);
// the implicit-GEMM convolution (qconv_implicit.hip): rows of one of its workgroups for this shape, and the call
bool fnn_implicit_conv_takes(const fnn_hip_weight *w, const QConvArgs &p, int option, int *wg_rows, int64_t *wgs);
int fnn_i8_implicit_conv(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QConvArgs &p, bool *handled);

// single-f16 activation mode: mean lane value per weight row (null for types whose lanes have zero mean)
int fnn_row_means(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const float **umean);

// M <= 8: bandwidth-bound GEMV on the matrix cores (weights requested before anything else).
int fnn_mfma_qgemv(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &p,
                   int flags, bool *handled);

// M <= 4, integer weights (I8, I4, U4): int8 matrix cores, activations as three exact base-256 digit rows, one
// workgroup per CU walking the row tiles (no decode arithmetic, activations converted once per workgroup).
int fnn_i8dot_qgemv(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &p, bool *handled);
// tile-major copy of the packed words for the GEMV kernels (blocks of 16 rows x 64 bytes), null where it does not apply
int fnn_tile_major_words(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q, const uint32_t **words_tm, int64_t *kb64);

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
