/*
 * fastnn_hip.h -- C ABI of libfastnn_hip.so: fastnn's weight-quantised MatMul
 * path (fused dequant GEMV/GEMM, I8-activation GEMM, quantised Conv2d) as
 * hand-written HIP kernels for gfx950 (MI355X).
 *
 * These are the entry points a `HipBackend: Backend` in fastnn binds through
 * FFI.  Each declaration names the fastnn interface it replaces (paths are
 * relative to the fastnn source tree).
 *
 * Conventions
 *   - every function returns an fnn_status; nothing throws or aborts across
 *     the boundary (every entry point catches C++ exceptions: std::bad_alloc
 *     becomes FNN_ERR_MEMORY, anything else FNN_ERR_DISPATCH); the message of
 *     the last failure on a context is returned by fnn_hip_last_error();
 *   - one context = one device + one HIP stream; a context is not re-entrant,
 *     matching the single-threaded dispatch contract of
 *     src/backend/cpu/mod.rs:176-188;
 *   - pointers are host pointers unless FNN_FLAG_DEVICE_PTRS is given; with
 *     host pointers a call copies in, runs, copies out and synchronises; with
 *     device pointers a call only enqueues work on the context's stream.
 */
#ifndef FASTNN_HIP_H
#define FASTNN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* BackendError variants of src/backend/mod.rs:6-12. */
typedef enum {
    FNN_OK = 0,
    FNN_ERR_DISPATCH = 1,
    FNN_ERR_MEMORY = 2,
    FNN_ERR_UNSUPPORTED_OP = 3,
    FNN_ERR_COMPILATION = 4
} fnn_status;

/* PackedWord types of src/dtypes/mod.rs:11-19; I4CB is I4x8 with a codebook
 * (QuantizedWeightMeta.codebooks non-empty, src/backend/mod.rs:42-58). */
typedef enum {
    FNN_DT_I8 = 0,
    FNN_DT_I4 = 1,
    FNN_DT_U8 = 2,
    FNN_DT_U4 = 3,
    FNN_DT_F8 = 4,
    FNN_DT_F8R = 5,
    FNN_DT_F4 = 6,
    FNN_DT_I4CB = 7
} fnn_dtype;

/* activation_type of src/backend/cpu/mod.rs:408-413 */
typedef enum { FNN_ACT_NONE = 0, FNN_ACT_RELU = 1, FNN_ACT_GELU = 2, FNN_ACT_SILU = 3 } fnn_act;

enum {
    FNN_FLAG_DEVICE_PTRS = 1 << 0,    /* activations / outputs / bias live in device memory      */
    FNN_FLAG_I4CB_AS_WRITTEN = 1 << 1,/* codebook MatMul multiplies by reshape(deq,[K,N]) the way */
                                      /* src/backend/cpu/matmul.rs:206-212 does (K == N only)     */
    FNN_FLAG_ACT_F16_SINGLE = 1 << 2, /* MFMA path: round activations to f16 once (default keeps  */
                                      /* a second f16 residual term, i.e. ~22 mantissa bits)      */
    FNN_FLAG_FORCE_GENERIC = 1 << 3,  /* take the shape-agnostic kernel (testing aid)             */
    FNN_FLAG_PREFER_FMA = 1 << 4,     /* M <= 4: take the f32 FMA GEMV instead of the MFMA kernel */
    FNN_FLAG_ACT_QUANT = 1 << 5       /* fnn_hip_qmatmul, opt-in fast mode, NOT the result of matmul_i8 / matmul_i4 /   */
                                      /* matmul_f8: the f32 activations are quantised on the way in.  I8 / I4 weights:  */
                                      /* the reference's own chain quantize_activations (dynamic, one scale per tensor, */
                                      /* src/backend/cpu/mod.rs:6928-7008) -> matmul_i8_i8 / matmul_i4_i8               */
                                      /* (src/backend/cpu/microkernels/gemm.rs:1641-1975) -> + bias -> activation, one   */
                                      /* int8 matrix-core plane, integer accumulators bit-exact against that chain.      */
                                      /* F8 weights: activations rounded to E4M3 with one power-of-two scale per row,    */
                                      /* fp8 matrix cores, f32 accumulation; within 5e-2 of max|ref| (3 mantissa bits).  */
                                      /* Other weight types refuse the flag (FNN_ERR_UNSUPPORTED_OP).                    */
};

typedef struct fnn_hip_ctx fnn_hip_ctx;
typedef struct fnn_hip_weight fnn_hip_weight;
typedef struct fnn_hip_graph fnn_hip_graph;

/* ---- context: Backend::name / allocate_arena, src/backend/mod.rs:152-158 ---- */
int fnn_hip_device_count(void);
int fnn_hip_create(int device, fnn_hip_ctx **out);
void fnn_hip_destroy(fnn_hip_ctx *ctx);
/* message of the last failing call on ctx (ctx may be NULL for create failures) */
const char *fnn_hip_last_error(fnn_hip_ctx *ctx);
int fnn_hip_sync(fnn_hip_ctx *ctx);

/* device arena: Backend::allocate_arena / write_arena / read_arena,
 * src/backend/mod.rs:157,245-253 */
int fnn_hip_malloc(fnn_hip_ctx *ctx, size_t bytes, void **dptr);
int fnn_hip_free(fnn_hip_ctx *ctx, void *dptr);
int fnn_hip_upload(fnn_hip_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
int fnn_hip_download(fnn_hip_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);

/* Per-context options (no counterpart in fastnn, whose CPU kernels read tuning values from the environment once per
 * process): kernel selection for measurements and tests.  Defaults give the automatic choice.  Unknown options and
 * values out of range are refused with FNN_ERR_DISPATCH; graphs captured earlier keep the choice of their capture. */
enum {
    FNN_OPT_CODEBOOK_CACHE = 1,   /* 1 (default): a codebook weight keeps its f16 expansion (8x the packed bytes)   */
                                  /* after its first MatMul with M >= 5; 0: a call expands into a workspace         */
    FNN_OPT_GEMV_ROW_TILES = 2,   /* M <= 8 kernels: 16-row tiles per workgroup, 1..3; 0 (default) = cost model     */
    FNN_OPT_ROWS16_ROW_TILES = 3, /* 9 <= M <= 16 kernel: the same                                                  */
    FNN_OPT_ROWS16_MIN_M = 4,     /* smallest M the 16-row kernel takes (default 9; 17 switches it off)             */
    FNN_OPT_TILE_SHAPE = 5,       /* tiled GEMMs, tile shape; -1 (default) = by shape.  f16 tiles: 0 = 128x128, 1 = 64x128, */
                                  /* 2 = 32x128, 3 = 256x128 with 8 waves (8-bit weights); int8 digit-plane tiles:       */
                                  /* 0 = 128x128, 1 = 256x128, 2 = 256x128 / 8 waves, 3 = 256x256, 4 = 256x192 (8 waves, 4-bit) */
                                  /* int8-activation GEMMs (matmul_*_i8, FNN_FLAG_ACT_QUANT): 0 = 128x128 on four waves,  */
                                  /* 1 = 128x128 on eight, 2 = 256x128 on eight (whole 256-row tiles only)                */
    FNN_OPT_TILE_SPLIT = 6,       /* tiled GEMM: K split over this many workgroups; 0 (default) = cost model        */
    FNN_OPT_TILE_STAGES = 7,      /* tiled GEMMs: LDS ring depth where the shape has variants (3..6); 0 (default) = by shape */
    FNN_OPT_TILE_MIN_M = 8,       /* smallest M the tiled GEMM takes (default 5)                                    */
    FNN_OPT_GEMV_INT8 = 9,        /* 1 (default): M <= 8 with I8 / I4 / U4 weights runs on the int8 matrix cores        */
                                  /* (activations as four exact base-256 digit rows, integer sums, no weight decode);  */
                                  /* 0: the f16 GEMV kernel takes them too                                             */
    FNN_OPT_GEMM_INT8 = 10,       /* 1 (default): M >= FNN_OPT_GEMM_INT8_MIN_M with I8 / I4 / U4 weights runs as an int8  */
                                  /* matrix-core GEMM over three or four exact activation digit planes (not in the single-rounding */
                                  /* mode, and by rule not weights of up to 2048 x 2048 elements, which the f16 tiles    */
                                  /* serve faster: FNN_OPT_DIGIT_PLANES = 3 / 4 or a smaller MIN_M brings them here);     */
                                  /* 0: the f16 tiled GEMM takes them too                                                 */
    FNN_OPT_GEMM_INT8_MIN_M = 11, /* smallest M of that path (default 17)                                                 */
    FNN_OPT_CODEBOOK_EXPANDED = 12, /* codebook weights with blocks of 32 at M >= 5: 0 (default) = by M (the streaming       */
                                  /* MatMul up to M = 64, beyond it decoded inside the tiled GEMM where that measured      */
                                  /* faster), 1 = always the tiled GEMM on the expanded f16 hi + lo operand                */
                                  /* (FNN_OPT_CODEBOOK_CACHE), 2 = always decoded inside the tiled GEMM                    */
    FNN_OPT_GEMV_INT8_MAX_M = 13, /* largest M the int8 GEMV kernel takes, 1..16 (default 8: beyond that the f16 16-row      */
                                  /* kernel measured faster, the activation chunks being converted one after the other)   */
    FNN_OPT_CONV_EPILOGUE = 14,   /* quantised Conv2d (I8 / I4 weights) on the int8 matrix cores: 0 (default) = by size,      */
                                  /* 1 = dequantise + bias + activation + NCHW stores inside the GEMM kernel, 2 = as a kernel */
                                  /* of its own after it, 3 = as 1 on 128-row tiles whatever the size (1 takes 64 x 64 tiles */
                                  /* while those leave CUs idle)                                                           */
    FNN_OPT_CONV_RANGES = 15,     /* plans: 1 (default) = the instruction that writes the input of a quantised Conv2d leaves   */
                                  /* partial (min, max) pairs per image behind and the convolution does not scan its input; 0 = */
                                  /* every convolution scans                                                               */
    FNN_OPT_CONV_IMPLICIT = 16,   /* quantised Conv2d (I8 / I4 weights, f32 input): 1 = one implicit-GEMM kernel (im2col taps    */
                                  /* fetched and quantised in the GEMM's operand registers, no int8 operand in memory), 2 = the */
                                  /* operand kernel + GEMM pair, 3 = the fused kernel (a workgroup quantises 32 pixels once     */
                                  /* into LDS and runs all output channels against them; K up to 1280), 0 (default) = by shape  */
    FNN_OPT_FUSE_RESIDUAL = 17,   /* plans: 1 (default) = a MatMul or quantised Conv2d whose output the next instruction adds to  */
                                  /* another tensor stores that sum from its own last kernel where it can (the Add instruction   */
                                  /* is then skipped; same f32 addition, identical results), 0 = every Add runs as its own launch */
    FNN_OPT_FUSE_PREP = 18,       /* plans: 1 (default) = a MatMul at 17 <= M whose result the next instruction multiplies (f16    */
                                  /* matrix-core weight types) leaves that MatMul's prepared activation operand behind, which  */
                                  /* then skips its own preparation launch (same conversion code, identical results); 0 = off  */
    FNN_OPT_STREAM_MIN_M = 19,    /* smallest and largest M of the one-launch streaming MatMul (weights straight into the      */
    FNN_OPT_STREAM_MAX_M = 20,    /* matrix-core operand registers, activations converted in the kernel, K split reduced by the  */
                                  /* last workgroup to arrive): defaults 17 and 32, 1..32; MAX_M = 0 switches it off.  By rule   */
                                  /* it declines shapes with more column tiles x K splits than the chip holds at once.           */
                                  /* Codebook weights with blocks of 32 (K % 128 == 0): with MAX_M at 32 the kernel takes        */
                                  /* min(MIN_M, 5) <= M <= 64 (a smaller MAX_M is taken as it is).  A long K over few output     */
                                  /* columns, with MIN_M not above its default: from M = 9 where K >= 4 N (K >= 2 N from         */
                                  /* K = 8192 on), from M = 5 where N <= 2048, K >= 4 N and K >= 8192 (16384 for I8 / I4 / U4);  */
                                  /* from M = 9 also where K / 512 fills the last of two or more rounds of eight at most half    */
    FNN_OPT_STREAM_SHAPE = 21,    /* its launch shape: 0 (default) = by rule, else (splits << 8) | (row tiles per wave << 4) |   */
                                  /* (k-values per round / 256), splits = 0 meaning one round per workgroup                      */
    FNN_OPT_DIGIT_PLANES = 22,    /* int8 matrix-core GEMM (M >= 17, I8 / I4 / U4 weights): activation digit planes, 3 (22 bits     */
                                  /* below the row maximum, 2e-5 of max|ref| stated) or 4 (30 bits, 4e-6, a third more matrix-core */
                                  /* work and operand traffic); 0 (default) = three wherever they measured faster                  */
    FNN_OPT_GEMV_TILE_MAJOR = 23, /* the kernels that stream the packed words straight into matrix-core operand registers (M <= 8: */
                                  /* I8 / I4 / U4 / U8 / F8 / F8R weights; 9 <= M <= 32: every per-channel type)                   */
                                  /* and the tile kernels of the types with 64 or 32 bytes per row and stage (I4 / U4 digit        */
                                  /* planes, U8 / F8 / F8R / F4):                                                                  */
                                  /* 1 (default) = read them from a second device copy laid out in blocks of 16 rows x 64 bytes    */
                                  /* (one contiguous KB per wave load: same bits, C1 M=1 5.97 -> 5.15 us, C2 6.70 -> 6.41, FP8     */
                                  /* 4096 x 4096 5.90 -> 5.40), built on the weight's first such call and kept with it (once more  */
                                  /* the packed bytes; rows of whole 64-byte blocks only; a call that may not allocate uses the    */
                                  /* row-major words until the copy exists); 0 = row-major words only                              */
    FNN_OPT_COUNT = 24
};
int fnn_hip_set_option(fnn_hip_ctx *ctx, int option, int64_t value);
int fnn_hip_get_option(fnn_hip_ctx *ctx, int option, int64_t *value);
/* The context's hipStream_t as an opaque pointer, for callers that enqueue work of their own in order with the
 * library's (no counterpart in fastnn). */
void *fnn_hip_stream(fnn_hip_ctx *ctx);

/* ---- weights: get_or_cache_packed + packed_tensor_from_meta,
 * src/backend/cpu/mod.rs:62-89, src/backend/cpu/matmul.rs:81-152.
 * Uploads the packed words once; `key` identifies the weight the way the CPU
 * cache keys (offset,size).  words: rows*ceil(inner/ITEMS) u32 (a trailing
 * 16-word margin may be present and is ignored).  shape is [rows, inner] =
 * [N, K] for MatMul, [OC, IC/g*KH*KW] for Conv2d.  n_zeros may be 0 (zeros
 * are then 0.0).  codebook16 non-NULL selects the codebook type. */
int fnn_hip_weight_register(fnn_hip_ctx *ctx, uint64_t key, int dtype, const uint32_t *words,
                            size_t n_words, int64_t rows, int64_t inner, const float *scales,
                            size_t n_scales, const float *zeros, size_t n_zeros,
                            int quant_block_size, const float *codebook16, fnn_hip_weight **out);
int fnn_hip_weight_lookup(fnn_hip_ctx *ctx, uint64_t key, fnn_hip_weight **out);
int fnn_hip_weight_release(fnn_hip_ctx *ctx, fnn_hip_weight *w);

/* PackedTensor::get_or_init_f32_weights, src/packed_tensor.rs:469-521:
 * out[rows*inner] = unpack*scale + zero, or scales[blk]*codebook[nibble]. */
int fnn_hip_dequant(fnn_hip_ctx *ctx, const fnn_hip_weight *w, float *out, int flags);

/* ---- quantised MatMul with f32 activations:
 * dispatch arms "matmul_i8|i4|u8|u4|f8|f8r|f4" (src/backend/cpu/mod.rs:3192-3315)
 * -> quantized_matmul_dispatch (src/backend/cpu/matmul.rs:165-225)
 * -> gemm_batch_packed_simd (src/backend/cpu/microkernels/gemm.rs:1982-2088);
 * fused with the bias add and ReLU/GELU/SiLU that the MatMulAdd{Relu,Gelu,Silu}
 * and Op{Relu,Gelu,Silu} fusions stand for
 * (src/compiler/passes/fusion/matmul_add_relu.rs:92-110).
 *   out[m,n] = act( (sum_k A[m,k]*u(W[n,k]))*scale[n] + zero[n]*sum_k A[m,k] + bias[n] )
 * A: [M,K] f32 row-major; out: [M,N] f32 row-major; bias: [N] or NULL. */
int fnn_hip_qmatmul(fnn_hip_ctx *ctx, const fnn_hip_weight *w, const float *a, int64_t m,
                    const float *bias, int act, float *out, int flags);

/* fnn_hip_qmatmul for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  No counterpart in fastnn.  Same kernels and the same result as
 * fnn_hip_qmatmul with FNN_FLAG_DEVICE_PTRS (a, bias, out are device pointers; the call only enqueues work on the
 * context's stream), but the workspaces of the M >= 17 path (prepared activation operands, split-K partial tiles)
 * come from a 32 MiB array inside the library's device image instead of hipMalloc, and the call makes no
 * allocation of any kind.  Limits, refused with FNN_ERR_MEMORY and a message that names them:
 *   - M <= FNN_STATIC_MAX_M;
 *   - operand workspace 2*ceil16(M)*ceil64(K)*2 + 12*M bytes <= 8 MiB (M = 256 at K = 4096 uses 4 MiB; half of
 *     that with FNN_FLAG_ACT_F16_SINGLE), split-K partials splits*M*N*4 bytes <= 24 MiB;
 *   - per-weight side tables that fnn_hip_qmatmul builds on first use (the f16 expansion of a codebook weight at
 *     M >= 5, row means for FNN_FLAG_ACT_F16_SINGLE, re-strided rows when ceil(K/ITEMS) % 4 != 0) must exist
 *     already: call fnn_hip_qmatmul once per weight and flag combination beforehand.
 * Every GPU the library runs on holds its copy of the array until the process ends, and every call on a GPU, from
 * any context, uses that one copy: calls that overlap in time on one GPU (two contexts, two threads) race; calls
 * on one context are ordered by its stream.  Nothing in the array needs to start at zero. */
#define FNN_STATIC_MAX_M 4096
int fnn_hip_qmatmul_static(fnn_hip_ctx *ctx, const fnn_hip_weight *w, const float *a_dev, int64_t m,
                           const float *bias_dev, int act, float *out_dev, int flags);

/* ---- I8 activations: kernel "quantize_activations"
 * (src/backend/cpu/mod.rs:6928-7008): payload = [scale f32][zp f32][numel x i8].
 * scale <= 0 selects the dynamic mode (scale = max|x|/127, zp = 0). */
int fnn_hip_quantize_activations(fnn_hip_ctx *ctx, const float *x, int64_t numel, float scale,
                                 float zp, uint8_t *payload, int flags);

/* kernel "dequantize_activations", per-tensor form (src/backend/cpu/mod.rs:7009-7088):
 * out[i] = q[i]*scale + zero for i < n, q = 0 where the payload ends early.  Device pointers;
 * the call is queued on the context's stream. */
int fnn_hip_dequantize_activations(fnn_hip_ctx *ctx, const uint8_t *payload, uint64_t payload_len,
                                   float *out, uint64_t n);

/* kernels "quantize_activations" / "dequantize_activations", per-channel form (src/backend/cpu/mod.rs:6941-6975,
 * 7026-7061), with the results those loops produce as written.  payload = [num_channels u32][chunk u32]
 * [scale f32 x nc][zero point f32 x nc][chunk x i8], chunk = numel / num_channels: every channel's loop addresses the
 * ONE block of chunk code bytes from its start, in ascending channel order, so byte `local` ends as the code of
 * x[ch*chunk + local] under (scale[ch], zero[ch]) of the last channel ch with ch*chunk + local < x_len (code 0 where
 * that scale is 0); bytes at or past payload_len are not written.  The dequantiser takes nc and chunk from the header
 * and writes out[ch*chunk + local] = code[local]*scale[ch] + zero[ch] for ch*chunk + local < out_len (code 0 past the
 * payload's end); a header that does not fit its payload (the reference panics) leaves `out` untouched.
 * x_dev / payload_dev / out_dev are device pointers (4-byte aligned), scales / zero_points host arrays of num_channels
 * values (passed on by value, so the call may be captured); x_len = f32 values readable at x_dev, out_len = f32 values
 * writable at out_dev.  Queued on the context's stream.  FNN_ERR_DISPATCH: num_channels == 0, a payload too small for
 * its header (the reference panics on both), chunk >= 2^32. */
int fnn_hip_quantize_activations_per_channel(fnn_hip_ctx *ctx, const float *x_dev, uint64_t x_len, uint64_t numel,
                                             uint32_t num_channels, const float *scales, const float *zero_points,
                                             uint8_t *payload_dev, uint64_t payload_len);
int fnn_hip_dequantize_activations_per_channel(fnn_hip_ctx *ctx, const uint8_t *payload_dev, uint64_t payload_len,
                                               float *out_dev, uint64_t out_len);

/* "matmul_i8_i8" / "matmul_i4_i8": gemm_cpu_flat_i8_i8x4 / gemm_cpu_flat_i8_i4x8
 * (src/backend/cpu/microkernels/gemm.rs:1641-1975).  acc_out (nullable, [M,N]
 * i32) receives the exact integer accumulators sum q_w*q_a when zp_a == 0. */
int fnn_hip_qmatmul_i8act(fnn_hip_ctx *ctx, const fnn_hip_weight *w, const uint8_t *payload,
                          int64_t m, float *out, int32_t *acc_out, int flags);

/* ---- quantised Conv2d, f32 NCHW activations, the "conv2d_*" arm of CpuBackend::dispatch
 * (src/backend/cpu/mod.rs:4100-4266), selected by the type of the registered weight:
 *  I8: conv2d_packed_i8x4 (src/backend/cpu/packed_conv.rs:1118-1196) = im2col + per-(image,group)
 *      dynamic int8 activation quantisation (packed_conv.rs:125-232) + gemm_packed_i8x4_fused_raw
 *      (packed_conv.rs:444-625);
 *  I4: conv2d_packed_i4x8 (packed_conv.rs:1202-1280): the same with 4-bit weights and activations
 *      quantised to 16 levels (packed_conv.rs:236-283, 659-841);
 *  U8, U4, F8, F8R, F4, I4CB: weights dequantised, f32 convolution conv2d_f32_im2col_gemm
 *      (src/backend/cpu/mod.rs:4204-4257, src/backend/cpu/microkernels/conv.rs:509-660).
 * acc_out (nullable, same shape as y; I8 and I4 only) receives the i32 accumulators incl. bias_q. */
int fnn_hip_qconv2d(fnn_hip_ctx *ctx, const fnn_hip_weight *w, const float *x, int64_t b,
                    int64_t c, int64_t h, int64_t wd, int kh, int kw, int stride, int pad,
                    int dil, int groups, const float *bias, int act, float *y, int32_t *acc_out,
                    int flags);

/* "conv2d_i8_i8[_act]" / "conv2d_i4_i8[_act]" (src/backend/cpu/mod.rs:3848-4098): the input is an
 * I8 activation payload [scale f32][zero f32][B*C*H*W x i8] (NCHW) as fnn_hip_quantize_activations
 * writes it; the int8 values are gathered with im2col_i8 (src/backend/cpu/packed_conv.rs:69-115,
 * padding taps are the integer 0), then
 *  I8 weights: gemm_packed_i8x4_fused_raw with the payload's (scale, zero)
 *      (packed_conv.rs:444-625, bias rounded to the accumulator grid);
 *  I4 weights: gemm_cpu_flat_i8_i4x8 (src/backend/cpu/microkernels/gemm.rs:1795-1975), then the bias
 *      added in f32 and the activation (mod.rs:4002-4032).
 * y is f32 NCHW.  A device payload pointer must be 4-byte aligned. */
int fnn_hip_qconv2d_i8act(fnn_hip_ctx *ctx, const fnn_hip_weight *w, const uint8_t *payload,
                          int64_t b, int64_t c, int64_t h, int64_t wd, int kh, int kw, int stride,
                          int pad, int dil, int groups, const float *bias, int act, float *y,
                          int flags);

/* ---- stream timing (Backend::dispatch_profile, src/backend/mod.rs:178-211):
 * HIP events recorded on the context's stream. */
int fnn_hip_timer_start(fnn_hip_ctx *ctx);
int fnn_hip_timer_stop(fnn_hip_ctx *ctx, float *elapsed_ms);

/* ---- HIP graphs over device-pointer calls: capture a dispatch sequence once,
 * replay it with one launch (a static-shape plan, src/backend/executor.rs:639-667). */
int fnn_hip_graph_begin(fnn_hip_ctx *ctx);
int fnn_hip_graph_end(fnn_hip_ctx *ctx, fnn_hip_graph **out);
int fnn_hip_graph_launch(fnn_hip_ctx *ctx, fnn_hip_graph *g);
int fnn_hip_graph_destroy(fnn_hip_ctx *ctx, fnn_hip_graph *g);
/* Counts how often the context re-allocated one of its internal workspaces (no counterpart in
 * fastnn).  A captured graph holds the workspace addresses of its capture: when the count has
 * changed since, the graph is stale and must be captured again instead of launched. */
uint64_t fnn_hip_workspace_epoch(const fnn_hip_ctx *ctx);

/* ---- host-side weight quantisers (no GPU needed): the packers the
 * quantisation pass calls (src/compiler/passes/quantization.rs:170-260,
 * 281-495): from_f32_per_channel_asymmetric (I8/I4/U8/U4/F4,
 * src/packed_tensor.rs:834-1049), from_f32_per_channel (F8/F8R, :661-742),
 * from_f32_per_block_codebook (I4CB, :1209-1313).  w_nk is the transposed
 * [N,K] matrix; words must hold fnn_packed_words() entries. */
size_t fnn_packed_words(int dtype, int64_t rows, int64_t inner);
int fnn_quantize_weights(int dtype, const float *w_nk, int64_t rows, int64_t inner,
                         int quant_block_size, uint32_t *words, float *scales, float *zeros,
                         float *codebook16);
/* [K,N] -> [N,K] (quantization.rs:144-156) */
void fnn_transpose_kn_to_nk(const float *w_kn, int64_t k, int64_t n, float *w_nk);

const char *fnn_hip_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FASTNN_HIP_H */
