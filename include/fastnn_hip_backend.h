/*
 * fastnn_hip_backend.h -- C view of the host-side HipBackend: the instruction-level
 * contract fastnn's executor hands a backend (src/backend/mod.rs:27-131), consumed here
 * without Rust.  A plan is a list of WriteConst / CallKernel / Fill / MemCopy
 * instructions over one byte arena; fnn_backend_dispatch() walks it sequentially the way
 * CpuBackend::dispatch does (src/backend/cpu/mod.rs:2644-2683), running the quantised
 * MatMul / Conv2d kernels (and the few f32 elementwise kernels found between them) on
 * the GPU against a device-resident arena.  A kernel name it does not implement returns
 * FNN_ERR_UNSUPPORTED_OP, which a Rust HipBackend answers by running that single
 * instruction on CpuBackend (as WgpuBackend does, src/backend/wgpu/mod.rs:162-239).
 */
#ifndef FASTNN_HIP_BACKEND_H
#define FASTNN_HIP_BACKEND_H

#include "fastnn_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct fnn_backend fnn_backend;
typedef struct fnn_plan fnn_plan;

/* BufferSlice, src/backend/mod.rs:27-38 */
typedef struct {
    uint64_t offset;
    uint64_t size;
} fnn_slice;

/* QuantizedWeightMeta, src/backend/mod.rs:40-58.  codebooks: n_codebooks x 16 floats (Vec<[f32; 16]>), 0 = no
 * codebook.  Like every decode of the reference (src/packed_tensor.rs:398, 489, 586) the kernels read
 * codebooks[0] only, whatever n_codebooks is. */
typedef struct {
    uint64_t bit_width;
    const float *scales;
    uint64_t n_scales;
    const float *zero_points;
    uint64_t n_zero_points;
    const uint64_t *shape;
    uint64_t n_shape;
    uint64_t quant_block_size;
    const float *codebooks;
    uint64_t n_codebooks;
} fnn_weight_meta;

/* Backend::name / allocate_arena / write_arena / read_arena, src/backend/mod.rs:152-254 */
int fnn_backend_create(int device, fnn_backend **out);
void fnn_backend_destroy(fnn_backend *b);
const char *fnn_backend_name(const fnn_backend *b);
/* FNN_FLAG_* bits OR-ed into every quantised MatMul / Conv2d call the backend makes from now on (no
 * counterpart in fastnn): FNN_FLAG_ACT_F16_SINGLE trades the default 2e-5 agreement for 1e-3 and about a third
 * less time at M >= 64; FNN_FLAG_FORCE_GENERIC / FNN_FLAG_PREFER_FMA select kernels for testing.  Other bits
 * are refused.  Plans captured before the change are captured again. */
int fnn_backend_set_kernel_flags(fnn_backend *b, int flags);
/* Resident plans replay as one HIP graph (default, enabled != 0) or run instruction by instruction on every
 * dispatch (enabled == 0); no counterpart in fastnn. */
int fnn_backend_set_graph_replay(fnn_backend *b, int enabled);
/* fnn_hip_set_option on the backend's context (FNN_OPT_*); plans captured before the change are captured again. */
int fnn_backend_set_option(fnn_backend *b, int option, int64_t value);
const char *fnn_backend_last_error(const fnn_backend *b);
int fnn_backend_allocate_arena(fnn_backend *b, uint64_t total_bytes);
int fnn_backend_write_arena(fnn_backend *b, uint64_t offset, const void *data, uint64_t size);
int fnn_backend_read_arena(fnn_backend *b, uint64_t offset, void *out, uint64_t size);

/* ExecutablePlan / Instruction, src/backend/mod.rs:60-107 */
int fnn_plan_create(uint64_t arena_size, fnn_plan **out);
void fnn_plan_destroy(fnn_plan *p);
int fnn_plan_add_write_const(fnn_plan *p, fnn_slice dst, const void *data, uint64_t len);
int fnn_plan_add_fill(fnn_plan *p, fnn_slice dst, float value);
int fnn_plan_add_memcopy(fnn_plan *p, fnn_slice dst, fnn_slice src);
/* kernel_name as CpuBackend::compile emits it (src/backend/cpu/mod.rs:415-495, 815-865);
 * a quantised MatMul may carry the epilogue the fusion pass attached as a suffix
 * "_relu" | "_gelu" | "_silu" and a third input slice for the bias.
 * secondary_output: CallKernel.secondary_output_slice (src/backend/mod.rs:66-67), NULL for None; "pool_f32" with
 * is_max = 1 writes the i64 window position kh*kernel + kw of each maximum there
 * (src/backend/cpu/mod.rs:4402-4410, src/backend/cpu/microkernels/ops.rs:150-155); other kernels ignore it.
 * params are resolved values: a caller with symbolic dims (param_dims + ShapeEnv,
 * src/backend/cpu/params.rs:11-39) resolves them before building the plan. */
int fnn_plan_add_call_kernel(fnn_plan *p, const char *kernel_name, const fnn_slice *inputs,
                             uint64_t n_inputs, fnn_slice output, const fnn_slice *secondary_output,
                             const uint64_t *params, uint64_t n_params, const fnn_weight_meta *meta);
uint64_t fnn_plan_len(const fnn_plan *p);
uint64_t fnn_plan_arena_size(const fnn_plan *p);

/* CallKernel.param_dims (src/backend/mod.rs:72-78): the symbolic form of `params`, one DimExpr
 * (src/ir/node.rs:163-167) per parameter.  kind 0 = Known(value), 1 = Symbol(symbol), 2 = Bounded { sym: symbol,
 * max: value }.  A quantised MatMul with param_dims takes [M, K, N] from them at dispatch time, evaluated in the
 * dispatch's shape environment exactly as resolve_params does (src/backend/cpu/params.rs:11-39,
 * DimExpr::evaluate_with_env, src/ir/node.rs:511-531): a Symbol must be bound, a Bounded dim falls back to its max
 * and refuses a larger binding; error texts are the reference's.  The other kernels of this backend take their
 * params as stored, like their CPU arms. */
typedef struct {
    uint32_t kind;
    uint64_t value;
    const char *symbol;   /* NULL for kind 0 */
} fnn_dim_expr;
int fnn_plan_set_param_dims(fnn_plan *p, uint64_t instruction, const fnn_dim_expr *dims, uint64_t n_dims);

/* ExecutablePlan::load / save (src/backend/mod.rs:117-131): the serde layout of ExecutablePlan, Instruction,
 * BufferSlice, QuantizedWeightMeta and DimExpr under bincode 1.3's default options (little endian, usize / u64 as 8
 * bytes, enum variant index as u32, Vec / String length as u64, Option as one tag byte, [f32; 16] without a length,
 * Arc<T> as T).  from_bincode refuses truncated input, trailing bytes, unknown variants and lengths the remaining
 * bytes cannot hold (FNN_ERR_COMPILATION, message with the byte offset).  node_id and levels are kept and written
 * back unchanged.  to_bincode: *needed receives the size; buf may be NULL to ask for it. */
int fnn_plan_from_bincode(const void *bytes, uint64_t len, fnn_plan **out);
int fnn_plan_to_bincode(const fnn_plan *p, void *buf, uint64_t cap, uint64_t *needed);
/* One instruction as a line of JSON (no counterpart in fastnn: for tools and tests). */
int fnn_plan_describe(const fnn_plan *p, uint64_t instruction, char *buf, uint64_t cap);

/* Backend::dispatch, src/backend/mod.rs:167-176.  Synchronises before returning.
 * The first dispatch of a plan uploads its WriteConst payloads and runs instruction by
 * instruction; while the constants stay in place (fnn_backend_write_arena elsewhere in the arena
 * does not disturb them, and neither does what another plan dispatched on this backend wrote) later
 * dispatches skip the uploads and replay the instruction stream as one HIP graph, the static-shape plan
 * reuse of src/backend/executor.rs:639-667 (see fnn_backend_set_graph_replay). */
int fnn_backend_dispatch(fnn_backend *b, fnn_plan *p);
/* Backend::dispatch with its ShapeEnv argument (src/backend/mod.rs:167-176, src/ir/node.rs:347-391): n_symbols
 * (name, value) bindings, valid for this dispatch; fnn_backend_dispatch is the same with an empty environment.  A
 * name bound twice to different values is refused, as ShapeEnv::bind does.  A resident plan replays its graph only
 * under the environment the graph was recorded with. */
int fnn_backend_dispatch_env(fnn_backend *b, fnn_plan *p, const char *const *names, const uint64_t *values,
                             uint64_t n_symbols);
/* Dispatch in segments, for a caller that runs kernels this library does not implement somewhere else, one
 * instruction at a time, the way WgpuBackend falls back to CpuBackend (src/backend/wgpu/mod.rs:162-239): runs the
 * instructions from index `first` on.  An instruction that is FNN_ERR_UNSUPPORTED_OP ends the segment with that
 * status, its index in *stopped_at and nothing of it executed (the message is the kernel name); the caller runs it
 * (fnn_backend_read_arena / fnn_backend_write_arena) and calls again with first = *stopped_at + 1.  FNN_OK means the
 * end of the plan was reached (*stopped_at = fnn_plan_len).  Such a plan is never replayed as a graph; its constants
 * still stay resident between passes. */
int fnn_backend_dispatch_from(fnn_backend *b, fnn_plan *p, const char *const *names, const uint64_t *values,
                              uint64_t n_symbols, uint64_t first, uint64_t *stopped_at);
/* 1 when the last dispatch of the plan ran as a graph replay, else 0 (no counterpart in fastnn:
 * lets tests and tools see which path ran). */
int fnn_plan_replayed(const fnn_plan *p);
/* Quantised Conv2d instructions of the plan that, on its last pass (or in its recorded graph), took the activation
 * ranges the instruction before them left instead of scanning their input (FNN_OPT_CONV_RANGES; no counterpart in
 * fastnn: lets tests and tools see which path ran). */
uint64_t fnn_plan_ranges_used(const fnn_plan *p);
/* add_f32 instructions of the plan that, on its last pass (or in its recorded graph), did not run as a launch of
 * their own because the MatMul or Conv2d before them stored the sum (FNN_OPT_FUSE_RESIDUAL; no counterpart in fastnn). */
uint64_t fnn_plan_residuals_fused(const fnn_plan *p);
/* MatMul instructions of the plan that, on its last pass (or in its recorded graph), found their activation operand
 * prepared by the split-K reduction of the MatMul before them (FNN_OPT_FUSE_PREP; no counterpart in fastnn). */
uint64_t fnn_plan_operands_handed(const fnn_plan *p);
/* Backend::dispatch_profile, src/backend/mod.rs:178-211: elapsed_ns[i] per instruction */
int fnn_backend_dispatch_profile(fnn_backend *b, fnn_plan *p, uint64_t *elapsed_ns, uint64_t n);
/* The same under the ShapeEnv the trait method is handed (symbolic param_dims are resolved against it, as
 * Backend::dispatch_profile's default does through dispatch, src/backend/mod.rs:178-211); the form without an
 * environment runs under an empty one. */
int fnn_backend_dispatch_profile_env(fnn_backend *b, fnn_plan *p, const char *const *names, const uint64_t *values,
                                     uint64_t n_symbols, uint64_t *elapsed_ns, uint64_t n);

/* f32 elementwise kernels found between quantised layers ("add_f32" with the second operand
 * broadcast by index modulo its length, "relu_f32", "gelu_f32", "silu_f32";
 * src/backend/cpu/mod.rs:2699-2751).  op: 0 add, 1 relu, 2 gelu, 3 silu.  Device pointers. */
int fnn_hip_elementwise(fnn_hip_ctx *ctx, int op, const float *a, const float *b, uint64_t nb,
                        float *out, uint64_t n);

/* f32 data movement between quantised convolutions, device pointers, lengths in elements:
 *  copy2d: `height` rows of `width` values, dst[r*dst_pitch + c] = src[r*src_pitch + c], dropped where either
 *    index leaves its buffer: the block copies of "concat" (src/backend/cpu/mod.rs:4267-4324) and "slice_f32"
 *    (:4721-4760);
 *  concat: the parts of one "concat" (:4267-4324) in one call: part j holds `height` rows of widths[j] values
 *    (src_lens[j] values in all) and lands at the sum of the widths before it in each row of dst (dst_pitch values
 *    per row); one launch when nothing is clipped and there are at most 8 parts, else a copy2d per part;
 *  maxpool2d: "pool_f32" with is_max = 1 (:4362-4397, src/backend/cpu/microkernels/ops.rs:104-158), output
 *    Ho = sat_sub(H + 2*pad, kernel)/stride + 1, writes past out_len dropped; indices (nullable, idx_len i64
 *    entries) receives kh*kernel + kw of the first strict maximum in (kh, kw) order, 0 for an empty window;
 *  avgpool2d: "pool_f32" with is_max != 1 (:4398-4470, ops.rs:162-210): the mean over the taps inside the image
 *    (padding taps are not counted), summed in (kh, kw) order;
 *  upsample_nearest2d: "upsample_nearest2d" (:5496-5535, src/backend/cpu/microkernels/misc.rs:338-364). */
int fnn_hip_copy2d_f32(fnn_hip_ctx *ctx, float *dst, uint64_t dst_pitch, uint64_t dst_len, const float *src,
                       uint64_t src_pitch, uint64_t src_len, uint64_t width, uint64_t height);
int fnn_hip_concat_f32(fnn_hip_ctx *ctx, float *dst, uint64_t dst_pitch, uint64_t dst_len, uint64_t n_parts,
                       const float *const *srcs, const uint64_t *widths, const uint64_t *src_lens, uint64_t height);
int fnn_hip_maxpool2d_f32(fnn_hip_ctx *ctx, const float *x, uint64_t in_len, float *y, uint64_t out_len,
                          uint64_t n, uint64_t c, uint64_t h, uint64_t w, uint64_t kernel, uint64_t stride,
                          uint64_t pad, int64_t *indices, uint64_t idx_len);
int fnn_hip_avgpool2d_f32(fnn_hip_ctx *ctx, const float *x, uint64_t in_len, float *y, uint64_t out_len,
                          uint64_t n, uint64_t c, uint64_t h, uint64_t w, uint64_t kernel, uint64_t stride,
                          uint64_t pad);
int fnn_hip_upsample_nearest2d_f32(fnn_hip_ctx *ctx, const float *x, float *y, uint64_t nc, uint64_t h,
                                   uint64_t w, uint64_t sh, uint64_t sw);

/* Instruction::Fill (f32 elements) and Instruction::MemCopy on device memory
 * (src/backend/mod.rs:92-106); both only enqueue on the context's stream. */
int fnn_hip_fill_f32(fnn_hip_ctx *ctx, float *dst, uint64_t n, float value);
int fnn_hip_copy(fnn_hip_ctx *ctx, void *dst_dev, const void *src_dev, uint64_t bytes);

#ifdef __cplusplus
}
#endif
#endif
