// C ABI of libfastnn_hip.so: context, device arena helpers, weight registry and the
// entry points that enqueue the quantised MatMul / Conv2d kernels on the context's stream.
// No exception or abort crosses this boundary; every failure becomes a status code plus a
// message kept on the context.
#include "common.h"

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

#include "i8act.h"
#include "range_io.h"
#include "mfma.h"
#include "../../include/fastnn_hip_backend.h"

hipError_t launch_im2col_f32(const float *x, float *col, int64_t b, int64_t c, int groups, int g, int64_t h, int64_t w,
                             int64_t ho, int64_t wo, int kh, int kw, int stride, int pad, int dil, hipStream_t s);
hipError_t launch_rows_to_nchw(const float *src, float *y, int64_t b, int64_t np, int64_t oc, int64_t ch0, int64_t ocg, hipStream_t s);
hipError_t launch_fill(float *dst, uint64_t n, float value, hipStream_t s);
hipError_t launch_eltwise(int op, const float *a, const float *b, uint64_t nb, float *out, uint64_t n, hipStream_t s, FnnRangeIo *rio);
hipError_t launch_copy2d(float *dst, uint64_t dst_pitch, uint64_t dst_len, const float *src, uint64_t src_pitch, uint64_t src_len,
                         uint64_t width, uint64_t height, hipStream_t s, FnnRangeIo *rio);
hipError_t launch_concat(float *dst, uint64_t dst_pitch, int n_parts, const float *const *srcs, const uint64_t *widths, uint64_t height,
                         hipStream_t s, FnnRangeIo *rio, bool *done);
hipError_t launch_avgpool2d(const float *x, uint64_t in_len, float *y, uint64_t out_len, uint64_t h, uint64_t w,
                            uint64_t ho, uint64_t wo, int kernel, int stride, int pad, hipStream_t s);
hipError_t launch_maxpool2d(const float *x, uint64_t in_len, float *y, uint64_t out_len, uint64_t c, uint64_t h, uint64_t w,
                            uint64_t ho, uint64_t wo, int kernel, int stride, int pad, int64_t *indices, uint64_t idx_len, hipStream_t s,
                            FnnRangeIo *rio);
hipError_t launch_upsample_nearest2d(const float *x, float *y, uint64_t nc, uint64_t h, uint64_t w, int sh, int sw, hipStream_t s, FnnRangeIo *rio);

struct fnn_hip_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

struct Staging {
    void *ptr = nullptr;
    size_t cap = 0;
};

struct fnn_hip_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    char err[1024] = {0};      // fixed storage: recording a failure never allocates
    std::unordered_map<uint64_t, fnn_hip_weight *> weights;
    Staging st_a, st_out, st_bias, st_acc, st_tmp, st_tmp2, st_tmp3, st_tmp4, st_col, st_rows;
    int64_t options[FNN_OPT_COUNT];
    float *scratch = nullptr;  // small reduction scratch (partials)
    uint32_t *stream_counters = nullptr;   // arrival counters of the streaming MatMul's column tiles (zero between launches)
    bool capturing = false;
    uint64_t ws_epoch = 0;     // bumped whenever a staging buffer is re-allocated (captured graphs go stale)
    unsigned char *static_ws = nullptr;   // this device's copy of the library's static workspace
    bool static_mode = false;             // inside fnn_hip_qmatmul_static: workspaces come from static_ws, nothing allocates
    FnnRangeIo range;                     // value ranges handed from one call to the next (range_io.h)
    FnnResidualIo residual;               // a residual addition handed to the next MatMul call (range_io.h)
    FnnPrepIo prep;                       // a prepared operand handed from one MatMul call to the next (range_io.h)
    FnnPreparedOperand prepared;
};

// Workspace of fnn_hip_qmatmul_static, part of the library's device image: every GPU the library runs on holds one
// copy (32 MiB) until the process ends.  Region 0: prepared activation operands + row tables; region 1: split-K
// partial tiles.  Host code never passes the array's name to a kernel: the device address of each GPU's copy is
// looked up once per device (static_workspace_of) and kept.
constexpr size_t kStaticOperandBytes = 8u << 20;
constexpr size_t kStaticPartialBytes = 24u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticOperandBytes + kStaticPartialBytes];

namespace {

thread_local char g_err[1024] = {0};  // failures without a context

// device address of `scratch` on the current device; looked up on the first context of each device
hipError_t static_workspace_of(int device, unsigned char **out)
{
    static std::mutex mu;
    static unsigned char *ptrs[64] = {nullptr};
    std::lock_guard<std::mutex> lock(mu);
    unsigned char *&slot = ptrs[device & 63];
    if (!slot) {
        void *p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        slot = static_cast<unsigned char *>(p);
    }
    *out = slot;
    return hipSuccess;
}

int fail(fnn_hip_ctx *ctx, int code, const char *fmt, ...) noexcept
{
    char *buf = ctx ? ctx->err : g_err;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, 1024, fmt, ap);
    va_end(ap);
    return code;
}

// Every extern "C" body runs inside this: a C++ exception (std::bad_alloc from a container, std::length_error, ...)
// becomes a status code and a message instead of unwinding into the caller's language.
template <class F>
int guarded(fnn_hip_ctx *ctx, const char *fn, F &&body) noexcept
{
    try {
        return body();
    } catch (const std::bad_alloc &) {
        return fail(ctx, FNN_ERR_MEMORY, "%s: out of host memory", fn);
    } catch (const std::exception &e) {
        return fail(ctx, FNN_ERR_DISPATCH, "%s: %s", fn, e.what());
    } catch (...) {
        return fail(ctx, FNN_ERR_DISPATCH, "%s: unknown C++ exception", fn);
    }
}

// option defaults, and the range fnn_hip_set_option accepts
struct OptionSpec { int64_t dflt, lo, hi; };
const OptionSpec kOptions[FNN_OPT_COUNT] = {
    {0, 0, 0},        // (unused index 0)
    {1, 0, 1},        // FNN_OPT_CODEBOOK_CACHE
    {0, 0, 3},        // FNN_OPT_GEMV_ROW_TILES
    {0, 0, 3},        // FNN_OPT_ROWS16_ROW_TILES
    {9, 1, 17},       // FNN_OPT_ROWS16_MIN_M
    {-1, -1, 4},      // FNN_OPT_TILE_SHAPE
    {0, 0, 32},       // FNN_OPT_TILE_SPLIT
    {0, 0, 6},        // FNN_OPT_TILE_STAGES
    {5, 1, 1 << 20},  // FNN_OPT_TILE_MIN_M
    {1, 0, 1},        // FNN_OPT_GEMV_INT8
    {1, 0, 1},        // FNN_OPT_GEMM_INT8
    {17, 1, 1 << 20}, // FNN_OPT_GEMM_INT8_MIN_M
    {0, 0, 2},        // FNN_OPT_CODEBOOK_EXPANDED
    {8, 1, 16},       // FNN_OPT_GEMV_INT8_MAX_M
    {0, 0, 3},        // FNN_OPT_CONV_EPILOGUE
    {1, 0, 1},        // FNN_OPT_CONV_RANGES
    {0, 0, 3},        // FNN_OPT_CONV_IMPLICIT
    {1, 0, 1},        // FNN_OPT_FUSE_RESIDUAL
    {1, 0, 1},        // FNN_OPT_FUSE_PREP
    {17, 1, 32},      // FNN_OPT_STREAM_MIN_M
    {32, 0, 32},      // FNN_OPT_STREAM_MAX_M
    {0, 0, 0xffff},   // FNN_OPT_STREAM_SHAPE
    {0, 0, 4},        // FNN_OPT_DIGIT_PLANES
    {1, 0, 1},        // FNN_OPT_GEMV_TILE_MAJOR
};

#define HIP_TRY(ctx, code, expr)                                                              \
    do {                                                                                      \
        hipError_t e__ = (expr);                                                              \
        if (e__ != hipSuccess)                                                                \
            return fail(ctx, code, "%s failed: %s", #expr, hipGetErrorString(e__));           \
    } while (0)

int ensure(fnn_hip_ctx *ctx, Staging &s, size_t bytes)
{
    if (bytes <= s.cap && s.ptr) return FNN_OK;
    if (ctx->capturing) return fail(ctx, FNN_ERR_MEMORY, "staging growth during graph capture");
    if (ctx->static_mode) return fail(ctx, FNN_ERR_MEMORY, "fnn_hip_qmatmul_static: this call would allocate %zu bytes of staging", bytes);
    if (s.ptr) {
        HIP_TRY(ctx, FNN_ERR_MEMORY, hipStreamSynchronize(ctx->stream));
        HIP_TRY(ctx, FNN_ERR_MEMORY, hipFree(s.ptr));
        s.ptr = nullptr;
        s.cap = 0;
    }
    size_t cap = bytes < 4096 ? 4096 : bytes;
    HIP_TRY(ctx, FNN_ERR_MEMORY, hipMalloc(&s.ptr, cap));
    s.cap = cap;
    ctx->ws_epoch++;
    return FNN_OK;
}

int items_of(int dt)
{
    switch (dt) {
    case FNN_DT_I8: case FNN_DT_U8: case FNN_DT_F8: case FNN_DT_F8R: return 4;
    case FNN_DT_I4: case FNN_DT_U4: case FNN_DT_F4: case FNN_DT_I4CB: return 8;
    default: return 0;
    }
}

const char *kernel_name_of(int dt)
{
    switch (dt) {
    case FNN_DT_I8: return "matmul_i8";
    case FNN_DT_I4: return "matmul_i4";
    case FNN_DT_U8: return "matmul_u8";
    case FNN_DT_U4: return "matmul_u4";
    case FNN_DT_F8: return "matmul_f8";
    case FNN_DT_F8R: return "matmul_f8r";
    case FNN_DT_F4: return "matmul_f4";
    case FNN_DT_I4CB: return "matmul_i4";
    default: return "matmul_?";
    }
}

void free_weight(fnn_hip_weight *w)
{
    if (!w) return;
    if (w->words) (void)hipFree(w->words);
    if (w->scales) (void)hipFree(w->scales);
    if (w->zeros) (void)hipFree(w->zeros);
    if (w->codebook) (void)hipFree(w->codebook);
    if (w->row_qsum) (void)hipFree(w->row_qsum);
    if (w->umean) (void)hipFree(w->umean);
    if (w->words4) (void)hipFree(w->words4);
    if (w->words_tm) (void)hipFree(w->words_tm);
    if (w->dense16) (void)hipFree(w->dense16);
    delete w;
}

}  // namespace

extern "C" {

const char *fnn_hip_version(void) { return "fastnn-hip 0.1 (gfx950)"; }

int fnn_hip_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int fnn_hip_create(int device, fnn_hip_ctx **out)
{
    return guarded(nullptr, "fnn_hip_create", [&]() -> int {
        if (!out) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_hip_create: out is NULL");
        *out = nullptr;
        int n = 0;
        hipError_t e = hipGetDeviceCount(&n);
        if (e != hipSuccess || n <= 0)
            return fail(nullptr, FNN_ERR_MEMORY, "fnn_hip_create: no HIP device (%s)",
                        e == hipSuccess ? "count 0" : hipGetErrorString(e));
        if (device < 0 || device >= n)
            return fail(nullptr, FNN_ERR_DISPATCH, "fnn_hip_create: device %d out of range [0,%d)", device, n);
        fnn_hip_ctx *ctx = new (std::nothrow) fnn_hip_ctx();
        if (!ctx) return fail(nullptr, FNN_ERR_MEMORY, "fnn_hip_create: out of host memory");
        ctx->device = device;
        for (int i = 0; i < FNN_OPT_COUNT; i++) ctx->options[i] = kOptions[i].dflt;
        if ((e = hipSetDevice(device)) != hipSuccess ||
            (e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking)) != hipSuccess ||
            (e = hipEventCreate(&ctx->ev0)) != hipSuccess || (e = hipEventCreate(&ctx->ev1)) != hipSuccess ||
            (e = hipMalloc((void **)&ctx->scratch, 64 * 1024)) != hipSuccess ||
            (e = hipMalloc((void **)&ctx->stream_counters, FNN_STREAM_COUNTERS * 4)) != hipSuccess ||
            (e = hipMemsetAsync(ctx->stream_counters, 0, FNN_STREAM_COUNTERS * 4, ctx->stream)) != hipSuccess ||
        (e = static_workspace_of(device, &ctx->static_ws)) != hipSuccess) {
            int rc = fail(nullptr, FNN_ERR_MEMORY, "fnn_hip_create: %s", hipGetErrorString(e));
            fnn_hip_destroy(ctx);
            return rc;
        }
        *out = ctx;
        return FNN_OK;
    });
}

void fnn_hip_destroy(fnn_hip_ctx *ctx)
{
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    for (auto &kv : ctx->weights) free_weight(kv.second);
    for (Staging *s : {&ctx->st_a, &ctx->st_out, &ctx->st_bias, &ctx->st_acc, &ctx->st_tmp, &ctx->st_tmp2, &ctx->st_tmp3, &ctx->st_tmp4, &ctx->st_col, &ctx->st_rows})
        if (s->ptr) (void)hipFree(s->ptr);
    if (ctx->scratch) (void)hipFree(ctx->scratch);
    if (ctx->stream_counters) (void)hipFree(ctx->stream_counters);
    if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
    if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

const char *fnn_hip_last_error(fnn_hip_ctx *ctx) { return ctx ? ctx->err : g_err; }

int fnn_hip_sync(fnn_hip_ctx *ctx)
{
    return guarded(ctx, "fnn_hip_sync", [&]() -> int {
        if (!ctx) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_hip_sync: NULL context");
        HIP_TRY(ctx, FNN_ERR_DISPATCH, hipStreamSynchronize(ctx->stream));
        return FNN_OK;
    });
}

int fnn_hip_set_option(fnn_hip_ctx *ctx, int option, int64_t value)
{
    return guarded(ctx, "fnn_hip_set_option", [&]() -> int {
        if (!ctx) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_hip_set_option: NULL context");
        if (option <= 0 || option >= FNN_OPT_COUNT) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_set_option: unknown option %d", option);
        const OptionSpec &o = kOptions[option];
        if (value < o.lo || value > o.hi)
            return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_set_option: value %lld of option %d outside [%lld, %lld]", (long long)value,
                        option, (long long)o.lo, (long long)o.hi);
        if (ctx->capturing) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_set_option: graph capture active");
        ctx->options[option] = value;
        return FNN_OK;
    });
}

int fnn_hip_get_option(fnn_hip_ctx *ctx, int option, int64_t *value)
{
    return guarded(ctx, "fnn_hip_get_option", [&]() -> int {
        if (!ctx || !value) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_get_option: NULL argument");
        if (option <= 0 || option >= FNN_OPT_COUNT) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_get_option: unknown option %d", option);
        *value = ctx->options[option];
        return FNN_OK;
    });
}

void *fnn_hip_stream(fnn_hip_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int fnn_hip_malloc(fnn_hip_ctx *ctx, size_t bytes, void **dptr)
{
    return guarded(ctx, "fnn_hip_malloc", [&]() -> int {
        if (!ctx || !dptr) return fail(ctx, FNN_ERR_MEMORY, "fnn_hip_malloc: NULL argument");
        *dptr = nullptr;
        HIP_TRY(ctx, FNN_ERR_MEMORY, hipSetDevice(ctx->device));
        HIP_TRY(ctx, FNN_ERR_MEMORY, hipMalloc(dptr, bytes ? bytes : 1));
        return FNN_OK;
    });
}

int fnn_hip_free(fnn_hip_ctx *ctx, void *dptr)
{
    return guarded(ctx, "fnn_hip_free", [&]() -> int {
        if (!ctx) return fail(nullptr, FNN_ERR_MEMORY, "fnn_hip_free: NULL context");
        if (!dptr) return FNN_OK;
        HIP_TRY(ctx, FNN_ERR_MEMORY, hipStreamSynchronize(ctx->stream));
        HIP_TRY(ctx, FNN_ERR_MEMORY, hipFree(dptr));
        return FNN_OK;
    });
}

int fnn_hip_upload(fnn_hip_ctx *ctx, void *dst, const void *src, size_t bytes)
{
    return guarded(ctx, "fnn_hip_upload", [&]() -> int {
        if (!ctx || (bytes && (!dst || !src))) return fail(ctx, FNN_ERR_MEMORY, "fnn_hip_upload: NULL argument");
        if (!bytes) return FNN_OK;
        HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
        HIP_TRY(ctx, FNN_ERR_MEMORY, hipStreamSynchronize(ctx->stream));
        return FNN_OK;
    });
}

int fnn_hip_download(fnn_hip_ctx *ctx, void *dst, const void *src, size_t bytes)
{
    return guarded(ctx, "fnn_hip_download", [&]() -> int {
        if (!ctx || (bytes && (!dst || !src))) return fail(ctx, FNN_ERR_MEMORY, "fnn_hip_download: NULL argument");
        if (!bytes) return FNN_OK;
        HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(ctx, FNN_ERR_MEMORY, hipStreamSynchronize(ctx->stream));
        return FNN_OK;
    });
}

// Validation mirrors packed_tensor_from_meta (src/backend/cpu/matmul.rs:81-152).
int fnn_hip_weight_register(fnn_hip_ctx *ctx, uint64_t key, int dtype, const uint32_t *words,
                            size_t n_words, int64_t rows, int64_t inner, const float *scales,
                            size_t n_scales, const float *zeros, size_t n_zeros,
                            int quant_block_size, const float *codebook16, fnn_hip_weight **out)
{
    return guarded(ctx, "fnn_hip_weight_register", [&]() -> int {
        if (!ctx) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_hip_weight_register: NULL context");
        if (out) *out = nullptr;
        if (codebook16 && dtype == FNN_DT_I4) dtype = FNN_DT_I4CB;
        const int items = items_of(dtype);
        const char *kn = kernel_name_of(dtype);
        if (!items) return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "unsupported packed dtype %d", dtype);
        if (rows <= 0 || inner <= 0)
            return fail(ctx, FNN_ERR_DISPATCH, "%s: invalid weight shape [%lld, %lld]", kn, (long long)rows, (long long)inner);
        if (!scales || n_scales == 0)
            return fail(ctx, FNN_ERR_DISPATCH, "%s: quantized weight metadata missing scales", kn);
        if (n_zeros != 0 && n_zeros != n_scales && dtype != FNN_DT_I4CB)
            return fail(ctx, FNN_ERR_DISPATCH,
                        "%s: quantized weight metadata length mismatch: %zu scales vs %zu zero_points", kn,
                        n_scales, n_zeros);
        if (n_zeros != 0 && !zeros)
            return fail(ctx, FNN_ERR_DISPATCH, "%s: zero_points pointer is NULL", kn);
        const size_t urows = (size_t)rows;
        const bool valid_len = n_scales == 1 || n_scales == urows ||
                               (n_scales > 1 && urows > n_scales && urows % n_scales == 0) ||
                               (quant_block_size > 0 && n_scales > urows && n_scales % urows == 0);
        if (!valid_len)
            return fail(ctx, FNN_ERR_DISPATCH,
                        "%s: quantized weight metadata length %zu incompatible with shape [%lld, %lld] "
                        "(expected 1, %lld, or a divisor of %lld)",
                        kn, n_scales, (long long)rows, (long long)inner, (long long)rows, (long long)rows);
        const int64_t kp = (inner + items - 1) / items;
        const size_t expected = (size_t)(rows * kp);
        if (!words || n_words < expected)
            return fail(ctx, FNN_ERR_DISPATCH,
                        "%s: quantized weight payload too short: got %zu packed words for shape [%lld, %lld], "
                        "expected at least %zu",
                        kn, words ? n_words : (size_t)0, (long long)rows, (long long)inner, expected);
        int64_t bpr = 0;
        if (dtype == FNN_DT_I4CB) {
            if (!codebook16) return fail(ctx, FNN_ERR_DISPATCH, "%s: codebook weight without codebook", kn);
            if (quant_block_size <= 0)
                return fail(ctx, FNN_ERR_DISPATCH, "%s: codebook weight needs quant_block_size > 0", kn);
            bpr = (inner + quant_block_size - 1) / quant_block_size;
            if (n_scales < (size_t)(rows * bpr))
                return fail(ctx, FNN_ERR_DISPATCH, "%s: codebook weight needs %lld block scales, got %zu", kn,
                            (long long)(rows * bpr), n_scales);
        } else if (quant_block_size > 0 && n_scales > urows) {
            return fail(ctx, FNN_ERR_UNSUPPORTED_OP,
                        "%s: per-block scales without a codebook are not produced by the quantisation pass", kn);
        }
        if (ctx->weights.count(key))
            return fail(ctx, FNN_ERR_DISPATCH, "weight key %llu already registered", (unsigned long long)key);

        HIP_TRY(ctx, FNN_ERR_MEMORY, hipSetDevice(ctx->device));
        fnn_hip_weight *w = new (std::nothrow) fnn_hip_weight();
        if (!w) return fail(ctx, FNN_ERR_MEMORY, "out of host memory");
        memset(w, 0, sizeof(*w));
        w->key = key; w->dtype = dtype; w->rows = rows; w->inner = inner; w->items = items; w->kp = kp;
        w->qblock = (dtype == FNN_DT_I4CB) ? quant_block_size : 0;
        w->bpr = bpr; w->ctx = ctx;

        // device copy of the words, with the two value-preserving canonicalisations that let
        // the hardware converts stand for the reference's decode tables:
        //   F8: every exponent-15 byte decodes to NaN (src/dtypes/f8x4.rs:36) -> OCP NaN 0x7F/0xFF;
        //   F4: nibble 0x8 decodes to +0.0 (src/dtypes/f4x8.rs:31-35) -> 0x0.
        std::vector<uint32_t> host(expected);
        memcpy(host.data(), words, expected * sizeof(uint32_t));
        if (dtype == FNN_DT_F8) {
            for (auto &x : host)
                for (int i = 0; i < 4; i++)
                    if (((x >> (8 * i)) & 0x78u) == 0x78u) x |= (0x7Fu << (8 * i));
        } else if (dtype == FNN_DT_F4) {
            for (auto &x : host)
                for (int i = 0; i < 8; i++)
                    if (((x >> (4 * i)) & 0xFu) == 0x8u) x &= ~(0xFu << (4 * i));
        }
        const size_t pad = 256;
        hipError_t e;
        auto bail = [&](const char *what) {
            int rc = fail(ctx, FNN_ERR_MEMORY, "%s: %s", what, hipGetErrorString(e));
            free_weight(w);
            return rc;
        };
        if ((e = hipMalloc((void **)&w->words, expected * 4 + pad)) != hipSuccess) return bail("hipMalloc(words)");
        if ((e = hipMemsetAsync(w->words, 0, expected * 4 + pad, ctx->stream)) != hipSuccess) return bail("hipMemset(words)");
        if ((e = hipMemcpyAsync(w->words, host.data(), expected * 4, hipMemcpyHostToDevice, ctx->stream)) != hipSuccess)
            return bail("hipMemcpy(words)");

        // scales / zeros expanded to one entry per row (scale_for_row / zero_for_row,
        // src/packed_tensor.rs:438-462; group rule src/backend/cpu/matmul.rs:147-149)
        std::vector<float> sc, zr;
        if (dtype == FNN_DT_I4CB) {
            sc.assign(scales, scales + rows * bpr);
            zr.assign((size_t)rows, 0.0f);
        } else {
            sc.resize((size_t)rows);
            zr.resize((size_t)rows);
            const size_t group = (n_scales > 1 && urows > n_scales) ? urows / n_scales : 1;
            for (size_t r = 0; r < urows; r++) {
                const size_t idx = (n_scales == 1) ? 0 : r / group;
                sc[r] = scales[idx];
                zr[r] = n_zeros ? zeros[idx] : 0.0f;
            }
        }
        if ((e = hipMalloc((void **)&w->scales, sc.size() * 4 + 64)) != hipSuccess) return bail("hipMalloc(scales)");
        if ((e = hipMalloc((void **)&w->zeros, zr.size() * 4 + 64)) != hipSuccess) return bail("hipMalloc(zeros)");
        if ((e = hipMemcpyAsync(w->scales, sc.data(), sc.size() * 4, hipMemcpyHostToDevice, ctx->stream)) != hipSuccess)
            return bail("hipMemcpy(scales)");
        if ((e = hipMemcpyAsync(w->zeros, zr.data(), zr.size() * 4, hipMemcpyHostToDevice, ctx->stream)) != hipSuccess)
            return bail("hipMemcpy(zeros)");
        if (dtype == FNN_DT_I4CB) {
            if ((e = hipMalloc((void **)&w->codebook, 64)) != hipSuccess) return bail("hipMalloc(codebook)");
            if ((e = hipMemcpyAsync(w->codebook, codebook16, 64, hipMemcpyHostToDevice, ctx->stream)) != hipSuccess)
                return bail("hipMemcpy(codebook)");
        }
        if ((e = hipStreamSynchronize(ctx->stream)) != hipSuccess) return bail("hipStreamSynchronize");
        ctx->weights[key] = w;
        if (out) *out = w;
        return FNN_OK;
    });
}

int fnn_hip_weight_lookup(fnn_hip_ctx *ctx, uint64_t key, fnn_hip_weight **out)
{
    return guarded(ctx, "fnn_hip_weight_lookup", [&]() -> int {
        if (!ctx || !out) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_weight_lookup: NULL argument");
        auto it = ctx->weights.find(key);
        *out = (it == ctx->weights.end()) ? nullptr : it->second;
        if (!*out) return fail(ctx, FNN_ERR_DISPATCH, "weight key %llu not registered", (unsigned long long)key);
        return FNN_OK;
    });
}

int fnn_hip_weight_release(fnn_hip_ctx *ctx, fnn_hip_weight *w)
{
    return guarded(ctx, "fnn_hip_weight_release", [&]() -> int {
        if (!ctx || !w) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_weight_release: NULL argument");
        auto it = ctx->weights.find(w->key);
        if (it == ctx->weights.end() || it->second != w)
            return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_weight_release: weight does not belong to this context");
        HIP_TRY(ctx, FNN_ERR_DISPATCH, hipStreamSynchronize(ctx->stream));
        ctx->weights.erase(it);
        free_weight(w);
        return FNN_OK;
    });
}

int fnn_hip_dequant(fnn_hip_ctx *ctx, const fnn_hip_weight *w, float *out, int flags)
{
    return guarded(ctx, "fnn_hip_dequant", [&]() -> int {
        if (!ctx || !w || !out) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_dequant: NULL argument");
        const size_t bytes = (size_t)(w->rows * w->inner) * 4;
        float *dout = out;
        if (!(flags & FNN_FLAG_DEVICE_PTRS)) {
            int rc = ensure(ctx, ctx->st_out, bytes);
            if (rc) return rc;
            dout = (float *)ctx->st_out.ptr;
        }
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_dequant(w, dout, ctx->stream));
        if (!(flags & FNN_FLAG_DEVICE_PTRS)) {
            HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(out, dout, bytes, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(ctx, FNN_ERR_DISPATCH, hipStreamSynchronize(ctx->stream));
        }
        return FNN_OK;
    });
}

int fnn_hip_qmatmul(fnn_hip_ctx *ctx, const fnn_hip_weight *w, const float *a, int64_t m,
                    const float *bias, int act, float *out, int flags)
{
    return guarded(ctx, "fnn_hip_qmatmul", [&]() -> int {
        if (!ctx || !w) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_qmatmul: NULL context or weight");
        const char *kn = kernel_name_of(w->dtype);
        if (m < 0) return fail(ctx, FNN_ERR_DISPATCH, "%s: expected params [M,K,N], got M=%lld", kn, (long long)m);
        if (m == 0) return FNN_OK;
        if (!a || !out) return fail(ctx, FNN_ERR_DISPATCH, "%s: NULL activation or output pointer", kn);
        if (act < FNN_ACT_NONE || act > FNN_ACT_SILU)
            return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "%s: unknown activation %d", kn, act);
        if ((flags & FNN_FLAG_I4CB_AS_WRITTEN) && w->dtype != FNN_DT_I4CB)
            return fail(ctx, FNN_ERR_DISPATCH, "%s: as-written mode applies to codebook weights only", kn);
        const int64_t n = w->rows, k = w->inner;
        const bool dev = (flags & FNN_FLAG_DEVICE_PTRS) != 0;
        const float *da = a, *dbias = bias;
        float *dout = out;
        if (!dev) {
            int rc;
            if ((rc = ensure(ctx, ctx->st_a, (size_t)(m * k) * 4))) return rc;
            if ((rc = ensure(ctx, ctx->st_out, (size_t)(m * n) * 4))) return rc;
            HIP_TRY(ctx, FNN_ERR_MEMORY,
                    hipMemcpyAsync(ctx->st_a.ptr, a, (size_t)(m * k) * 4, hipMemcpyHostToDevice, ctx->stream));
            da = (const float *)ctx->st_a.ptr;
            dout = (float *)ctx->st_out.ptr;
            if (bias) {
                if ((rc = ensure(ctx, ctx->st_bias, (size_t)n * 4))) return rc;
                HIP_TRY(ctx, FNN_ERR_MEMORY,
                        hipMemcpyAsync(ctx->st_bias.ptr, bias, (size_t)n * 4, hipMemcpyHostToDevice, ctx->stream));
                dbias = (const float *)ctx->st_bias.ptr;
            }
        }
        QMatmulArgs p;
        p.words = w->words; p.scales = w->scales; p.zeros = w->zeros; p.codebook = w->codebook;
        p.a = da; p.bias = dbias; p.out = dout;
        p.m = m; p.n = n; p.k = k; p.kp = w->kp; p.bpr = w->bpr; p.qblock = w->qblock; p.act = act;
        p.as_written = (flags & FNN_FLAG_I4CB_AS_WRITTEN) ? 1 : 0;

        if (flags & FNN_FLAG_ACT_QUANT) {
            if (ctx->static_mode) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_qmatmul_static: flag not available here");
            if (w->dtype != FNN_DT_I8 && w->dtype != FNN_DT_I4 && w->dtype != FNN_DT_F8)
                return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "%s: FNN_FLAG_ACT_QUANT applies to I8, I4 and F8 weights", kn);
            if (w->dtype == FNN_DT_F8) {
                bool done = false;
                int rc = fnn_fp8_actquant_qmatmul(ctx, ctx->stream, w, p, &done);
                if (rc) return rc;
                if (!done) return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "%s: FNN_FLAG_ACT_QUANT needs K %% 128 == 0 and 16-byte aligned operands for F8 weights", kn);
            } else {
                // quantize_activations (dynamic: scale = max|x| / 127, zero 0) into a transient payload, then the
                // I8-activation MatMul with the bias and the activation behind its formula
                void *pl = nullptr;
                int rc = fnn_ctx_ensure_tmp(ctx, 2, (size_t)(m * k) + 8 + 16, &pl);
                if (rc) return rc;
                HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_quantize_activations(da, m * k, 0.0f, 0.0f, (uint8_t *)pl, ctx->scratch, ctx->stream));
                I8ActArgs q8;
                q8.words = w->words; q8.scales = w->scales; q8.zeros = w->zeros; q8.payload = (const uint8_t *)pl; q8.out = dout;
                q8.acc_out = nullptr; q8.m = m; q8.n = n; q8.k = k; q8.kp = w->kp;
                q8.bias = dbias; q8.act = act;
                bool done = false;
                if (!(flags & FNN_FLAG_FORCE_GENERIC)) {
                    rc = fnn_i8_tiled_matmul(ctx, ctx->stream, w, q8, &done);
                    if (rc) return rc;
                }
                if (!done) HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_qgemm_i8act_generic(w->dtype, q8, ctx->stream));
            }
            if (!dev) {
                HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(out, dout, (size_t)(m * n) * 4, hipMemcpyDeviceToHost, ctx->stream));
                HIP_TRY(ctx, FNN_ERR_DISPATCH, hipStreamSynchronize(ctx->stream));
            }
            return FNN_OK;
        }

        // kernel choice: matrix-core kernel for every M (bandwidth-bound at small M); the FMA GEMV
        // serves the codebook type at M <= 4 and any weight when FNN_FLAG_PREFER_FMA asks for it;
        // the shape-agnostic kernel takes what is left (ragged rows, unaligned pointers).
        bool handled = false;
        if (!(flags & FNN_FLAG_FORCE_GENERIC)) {
            const bool fma_first = (flags & FNN_FLAG_PREFER_FMA) || w->dtype == FNN_DT_I4CB;
            if (fma_first) HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_qgemv(w->dtype, p, ctx->stream, &handled));
            if (!handled) {   // (17 <= M <= 32 and, for a long K over few columns, from M = 9 or 5)
                int rc = fnn_stream_qmatmul(ctx, ctx->stream, w, p, flags, &handled);
                if (rc) return rc;
            }
            if (!handled && !(flags & FNN_FLAG_ACT_F16_SINGLE)) {
                int rc = fnn_i8dot_qgemv(ctx, ctx->stream, w, p, &handled);
                if (rc) return rc;
            }
            if (!handled) {
                int rc = fnn_mfma_qgemv(ctx, ctx->stream, w, p, flags, &handled);
                if (rc) return rc;
            }
            if (!handled) {
                int rc = fnn_mfma_rows16(ctx, ctx->stream, w, p, flags, &handled);
                if (rc) return rc;
            }
            if (!handled) {
                int rc = fnn_digits_qmatmul(ctx, ctx->stream, w, p, flags, &handled);
                if (rc) return rc;
            }
            if (!handled) {
                int rc = fnn_tiled_qmatmul(ctx, ctx->stream, w, p, flags, &handled);
                if (rc) return rc;
            }
            if (!handled && !fma_first) HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_qgemv(w->dtype, p, ctx->stream, &handled));
        }
        if (!handled) HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_qgemm_generic(w->dtype, p, ctx->stream));
        if (!dev) {
            HIP_TRY(ctx, FNN_ERR_MEMORY,
                    hipMemcpyAsync(out, dout, (size_t)(m * n) * 4, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(ctx, FNN_ERR_DISPATCH, hipStreamSynchronize(ctx->stream));
        }
        return FNN_OK;
    });
}

int fnn_hip_qmatmul_static(fnn_hip_ctx *ctx, const fnn_hip_weight *w, const float *a_dev, int64_t m,
                           const float *bias_dev, int act, float *out_dev, int flags)
{
    if (!ctx || !w) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_qmatmul_static: NULL context or weight");
    if (m > FNN_STATIC_MAX_M)
        return fail(ctx, FNN_ERR_MEMORY, "fnn_hip_qmatmul_static: M = %lld exceeds the limit of %d rows: use fnn_hip_qmatmul",
                    (long long)m, FNN_STATIC_MAX_M);
    if (flags & ~(FNN_FLAG_DEVICE_PTRS | FNN_FLAG_ACT_F16_SINGLE | FNN_FLAG_FORCE_GENERIC | FNN_FLAG_PREFER_FMA))
        return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_qmatmul_static: flag not available here");
    // device pointers only (host pointers would need staging buffers); workspaces come from the static array for the
    // duration of the call, and everything that would allocate fails instead
    struct Mode {
        fnn_hip_ctx *c;
        explicit Mode(fnn_hip_ctx *c_) : c(c_) { c->static_mode = true; }
        ~Mode() { c->static_mode = false; }
    } mode(ctx);
    return fnn_hip_qmatmul(ctx, w, a_dev, m, bias_dev, act, out_dev, flags | FNN_FLAG_DEVICE_PTRS);
}

int fnn_hip_quantize_activations(fnn_hip_ctx *ctx, const float *x, int64_t numel, float scale,
                                 float zp, uint8_t *payload, int flags)
{
    return guarded(ctx, "fnn_hip_quantize_activations", [&]() -> int {
        if (!ctx || !x || !payload || numel < 0)
            return fail(ctx, FNN_ERR_DISPATCH, "quantize_activations: NULL or invalid argument");
        const bool dev = (flags & FNN_FLAG_DEVICE_PTRS) != 0;
        const float *dx = x;
        uint8_t *dp = payload;
        if (!dev) {
            int rc;
            if ((rc = ensure(ctx, ctx->st_a, (size_t)numel * 4 + 16))) return rc;
            if ((rc = ensure(ctx, ctx->st_out, (size_t)numel + 16))) return rc;
            HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(ctx->st_a.ptr, x, (size_t)numel * 4, hipMemcpyHostToDevice, ctx->stream));
            dx = (const float *)ctx->st_a.ptr;
            dp = (uint8_t *)ctx->st_out.ptr;
        }
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_quantize_activations(dx, numel, scale, zp, dp, ctx->scratch, ctx->stream));
        if (!dev) {
            HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(payload, dp, (size_t)numel + 8, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(ctx, FNN_ERR_DISPATCH, hipStreamSynchronize(ctx->stream));
        }
        return FNN_OK;
    });
}

int fnn_hip_dequantize_activations(fnn_hip_ctx *ctx, const uint8_t *payload, uint64_t payload_len, float *out, uint64_t n)
{
    return guarded(ctx, "fnn_hip_dequantize_activations", [&]() -> int {
        if (!ctx || ((!payload || !out) && n)) return fail(ctx, FNN_ERR_DISPATCH, "dequantize_activations: NULL argument");
        if (reinterpret_cast<uintptr_t>(payload) & 3) return fail(ctx, FNN_ERR_DISPATCH, "dequantize_activations: payload must be 4-byte aligned");
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_dequantize_activations(payload, payload_len, out, n, ctx->stream));
        return FNN_OK;
    });
}

int fnn_hip_quantize_activations_per_channel(fnn_hip_ctx *ctx, const float *x_dev, uint64_t x_len, uint64_t numel, uint32_t num_channels,
                                             const float *scales, const float *zero_points, uint8_t *payload_dev, uint64_t payload_len)
{
    return guarded(ctx, "fnn_hip_quantize_activations_per_channel", [&]() -> int {
        if (!ctx || !x_dev || !payload_dev || !scales || !zero_points)
            return fail(ctx, FNN_ERR_DISPATCH, "quantize_activations (per channel): NULL argument");
        if (num_channels == 0) return fail(ctx, FNN_ERR_DISPATCH, "quantize_activations (per channel): no channels");
        if ((reinterpret_cast<uintptr_t>(payload_dev) & 3) || (reinterpret_cast<uintptr_t>(x_dev) & 3))
            return fail(ctx, FNN_ERR_DISPATCH, "quantize_activations (per channel): the input and the payload must be 4-byte aligned");
        const uint64_t header = 8 + (uint64_t)num_channels * 8;
        if (payload_len < header)
            return fail(ctx, FNN_ERR_DISPATCH, "quantize_activations (per channel): the payload holds %llu bytes, the header of %u channels takes %llu",
                        (unsigned long long)payload_len, num_channels, (unsigned long long)header);
        if (numel / num_channels > 0xffffffffull)
            return fail(ctx, FNN_ERR_DISPATCH, "quantize_activations (per channel): %llu elements per channel do not fit the header's u32",
                        (unsigned long long)(numel / num_channels));
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_quantize_activations_per_channel(x_dev, x_len, numel, num_channels, scales, zero_points, payload_dev,
                                                                              payload_len, ctx->stream));
        return FNN_OK;
    });
}

int fnn_hip_dequantize_activations_per_channel(fnn_hip_ctx *ctx, const uint8_t *payload_dev, uint64_t payload_len, float *out_dev, uint64_t out_len)
{
    return guarded(ctx, "fnn_hip_dequantize_activations_per_channel", [&]() -> int {
        if (!ctx || ((!payload_dev || !out_dev) && out_len)) return fail(ctx, FNN_ERR_DISPATCH, "dequantize_activations (per channel): NULL argument");
        if (reinterpret_cast<uintptr_t>(payload_dev) & 3) return fail(ctx, FNN_ERR_DISPATCH, "dequantize_activations (per channel): payload must be 4-byte aligned");
        if (payload_len < 8) return fail(ctx, FNN_ERR_DISPATCH, "dequantize_activations (per channel): a payload of %llu bytes has no header", (unsigned long long)payload_len);
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_dequantize_activations_per_channel(payload_dev, payload_len, out_dev, out_len, ctx->stream));
        return FNN_OK;
    });
}

int fnn_hip_qmatmul_i8act(fnn_hip_ctx *ctx, const fnn_hip_weight *w, const uint8_t *payload,
                          int64_t m, float *out, int32_t *acc_out, int flags)
{
    return guarded(ctx, "fnn_hip_qmatmul_i8act", [&]() -> int {
        if (!ctx || !w) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_qmatmul_i8act: NULL context or weight");
        if (w->dtype != FNN_DT_I8 && w->dtype != FNN_DT_I4)
            return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "matmul_*_i8: weight dtype %d has no I8-activation kernel", w->dtype);
        const char *kn = (w->dtype == FNN_DT_I8) ? "matmul_i8_i8" : "matmul_i4_i8";
        if (m < 0) return fail(ctx, FNN_ERR_DISPATCH, "%s: expected params [M,K,N]", kn);
        if (m == 0) return FNN_OK;
        if (!payload || !out) return fail(ctx, FNN_ERR_DISPATCH, "%s: NULL payload or output pointer", kn);
        const int64_t n = w->rows, k = w->inner;
        const bool dev = (flags & FNN_FLAG_DEVICE_PTRS) != 0;
        const uint8_t *dp = payload;
        float *dout = out;
        int32_t *dacc = acc_out;
        if (!dev) {
            int rc;
            if ((rc = ensure(ctx, ctx->st_a, (size_t)(m * k) + 8 + 16))) return rc;
            if ((rc = ensure(ctx, ctx->st_out, (size_t)(m * n) * 4))) return rc;
            HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(ctx->st_a.ptr, payload, (size_t)(m * k) + 8, hipMemcpyHostToDevice, ctx->stream));
            dp = (const uint8_t *)ctx->st_a.ptr;
            dout = (float *)ctx->st_out.ptr;
            if (acc_out) {
                if ((rc = ensure(ctx, ctx->st_acc, (size_t)(m * n) * 4))) return rc;
                dacc = (int32_t *)ctx->st_acc.ptr;
            }
        }
        I8ActArgs p;
        p.words = w->words; p.scales = w->scales; p.zeros = w->zeros; p.payload = dp; p.out = dout;
        p.acc_out = dacc; p.m = m; p.n = n; p.k = k; p.kp = w->kp;
        bool handled = false;
        if (!(flags & FNN_FLAG_FORCE_GENERIC)) {
            int rc = fnn_i8_tiled_matmul(ctx, ctx->stream, w, p, &handled);
            if (rc) return rc;
        }
        if (!handled) HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_qgemm_i8act_generic(w->dtype, p, ctx->stream));
        if (!dev) {
            HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(out, dout, (size_t)(m * n) * 4, hipMemcpyDeviceToHost, ctx->stream));
            if (acc_out)
                HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(acc_out, dacc, (size_t)(m * n) * 4, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(ctx, FNN_ERR_DISPATCH, hipStreamSynchronize(ctx->stream));
        }
        return FNN_OK;
    });
}

int fnn_hip_qconv2d(fnn_hip_ctx *ctx, const fnn_hip_weight *w, const float *x, int64_t b, int64_t c,
                    int64_t h, int64_t wd, int kh, int kw, int stride, int pad, int dil, int groups,
                    const float *bias, int act, float *y, int32_t *acc_out, int flags)
{
    return guarded(ctx, "fnn_hip_qconv2d", [&]() -> int {
        if (!ctx) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_hip_qconv2d: NULL context");
        if (!w) return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8: missing weight_meta for quantized weight");
        const bool integer_kernel = w->dtype == FNN_DT_I8 || w->dtype == FNN_DT_I4;
        if (!integer_kernel && acc_out)
            return fail(ctx, FNN_ERR_DISPATCH, "conv2d: weight type %d runs as an f32 convolution and has no i32 accumulators", w->dtype);
        if (groups <= 0) return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8: groups must be > 0");
        if (b < 0 || c <= 0 || h <= 0 || wd <= 0 || kh <= 0 || kw <= 0 || stride <= 0 || dil <= 0 || pad < 0)
            return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8: invalid geometry");
        if (c % groups || w->rows % groups)
            return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8: channels (%lld in, %lld out) not divisible by groups %d",
                        (long long)c, (long long)w->rows, groups);
        if (w->inner != (c / groups) * kh * kw)
            return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8: weight inner dim %lld != C/g*KH*KW = %lld", (long long)w->inner,
                        (long long)((c / groups) * kh * kw));
        if (act < FNN_ACT_NONE || act > FNN_ACT_SILU) return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "conv2d_i8: unknown activation %d", act);
        auto osz = [](int64_t in, int k, int s, int p, int d) -> int64_t {
            int64_t dk = (int64_t)(k - 1) * d + 1;
            return (in + 2 * p >= dk) ? (in + 2 * p - dk) / s + 1 : 0;
        };
        const int64_t ho = osz(h, kh, stride, pad, dil), wo = osz(wd, kw, stride, pad, dil);
        const int64_t oc = w->rows;
        if (b == 0 || ho == 0 || wo == 0) return FNN_OK;
        if (!x || !y) return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8: NULL input or output pointer");
        if (b * groups > 65535) return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "conv2d_i8: batch*groups > 65535");
        const bool dev = (flags & FNN_FLAG_DEVICE_PTRS) != 0;
        fnn_hip_weight *wm = const_cast<fnn_hip_weight *>(w);
        if (integer_kernel && !wm->row_qsum) {
            if (ctx->capturing) return fail(ctx, FNN_ERR_MEMORY, "conv2d_i8: first use of a weight during graph capture");
            HIP_TRY(ctx, FNN_ERR_MEMORY, hipMalloc((void **)&wm->row_qsum, (size_t)oc * 4 + 64));
            HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_row_qsum(w, wm->row_qsum, ctx->stream));
        }
        const size_t xin = (size_t)(b * c * h * wd) * 4, yout = (size_t)(b * oc * ho * wo) * 4;
        const float *dx = x, *dbias = bias;
        float *dy = y;
        int32_t *dacc = acc_out;
        int rc;
        if (!dev) {
            if ((rc = ensure(ctx, ctx->st_a, xin))) return rc;
            if ((rc = ensure(ctx, ctx->st_out, yout))) return rc;
            HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(ctx->st_a.ptr, x, xin, hipMemcpyHostToDevice, ctx->stream));
            dx = (const float *)ctx->st_a.ptr;
            dy = (float *)ctx->st_out.ptr;
            if (bias) {
                if ((rc = ensure(ctx, ctx->st_bias, (size_t)oc * 4))) return rc;
                HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(ctx->st_bias.ptr, bias, (size_t)oc * 4, hipMemcpyHostToDevice, ctx->stream));
                dbias = (const float *)ctx->st_bias.ptr;
            }
            if (acc_out) {
                if ((rc = ensure(ctx, ctx->st_acc, yout))) return rc;
                dacc = (int32_t *)ctx->st_acc.ptr;
            }
        }
        if (!integer_kernel) {
            // f32 convolution with dequantised weights (src/backend/cpu/mod.rs:4204-4257): im2col rows,
            // fused-dequant MatMul per group (bias and activation in its epilogue), [pixel, channel] -> NCHW
            const int64_t cg = c / groups, ocg = oc / groups, kk = cg * kh * kw, np = ho * wo, rows = b * np;
            if (rows > (1ll << 31) || b > 65535) return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "conv2d: %lld output pixels exceed the f32 path's limit", (long long)rows);
            if ((rc = ensure(ctx, ctx->st_col, (size_t)rows * kk * 4 + 256))) return rc;
            if ((rc = ensure(ctx, ctx->st_rows, (size_t)rows * ocg * 4 + 256))) return rc;
            float *col = (float *)ctx->st_col.ptr, *rows_out = (float *)ctx->st_rows.ptr;
            for (int g = 0; g < groups; g++) {
                HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_im2col_f32(dx, col, b, c, groups, g, h, wd, ho, wo, kh, kw, stride, pad, dil, ctx->stream));
                if (groups == 1) {
                    if ((rc = fnn_hip_qmatmul(ctx, w, col, rows, dbias, act, rows_out, FNN_FLAG_DEVICE_PTRS | (flags & (FNN_FLAG_FORCE_GENERIC | FNN_FLAG_ACT_F16_SINGLE))))) return rc;
                } else {
                    // a slice of the weight rows: the shape-agnostic kernel takes the offset pointers as they are
                    QMatmulArgs q;
                    q.words = w->words + (size_t)g * ocg * w->kp;
                    q.scales = w->dtype == FNN_DT_I4CB ? w->scales + (size_t)g * ocg * w->bpr : w->scales + (size_t)g * ocg;
                    q.zeros = w->zeros ? w->zeros + (size_t)g * ocg : nullptr;
                    q.codebook = w->codebook;
                    q.a = col; q.bias = dbias ? dbias + (size_t)g * ocg : nullptr; q.out = rows_out;
                    q.m = rows; q.n = ocg; q.k = kk; q.kp = w->kp; q.bpr = w->bpr; q.qblock = w->qblock; q.act = act;
                    q.as_written = 0;
                    HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_qgemm_generic(w->dtype, q, ctx->stream));
                }
                HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_rows_to_nchw(rows_out, dy, b, np, oc, (int64_t)g * ocg, ocg, ctx->stream));
            }
            if (!dev) {
                HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(y, dy, yout, hipMemcpyDeviceToHost, ctx->stream));
                HIP_TRY(ctx, FNN_ERR_DISPATCH, hipStreamSynchronize(ctx->stream));
            }
            return FNN_OK;
        }
        if ((rc = ensure(ctx, ctx->st_tmp, (size_t)(b * groups) * (QCONV_NPART * 2 + 4) * 4))) return rc;
        QConvArgs p;
        p.words = w->words; p.scales = w->scales; p.zeros = w->zeros; p.row_qsum = wm->row_qsum;
        p.x = dx; p.bias = dbias; p.y = dy; p.acc_out = dacc;
        p.minmax_partial = (float *)ctx->st_tmp.ptr;
        p.actq = p.minmax_partial + (size_t)(b * groups) * QCONV_NPART * 2;
        p.b = b; p.c = c; p.h = h; p.w = wd; p.oc = oc; p.ho = ho; p.wo = wo; p.kp = w->kp;
        p.kh = kh; p.kw = kw; p.stride = stride; p.pad = pad; p.dil = dil; p.groups = groups; p.act = act;
        p.wbits = w->dtype == FNN_DT_I4 ? 4 : 8;
        p.x8 = nullptr; p.payload_i4 = 0; p.nparts = 0;
        p.part_stride = QCONV_NPART; p.range_zero = 0; p.range_out = nullptr; p.range_out_stride = 0;
        FnnRangeIo &rio = ctx->range;
        rio.in_used = 0;
        if (flags & FNN_FLAG_FORCE_GENERIC) {
            if (rio.out_table) rio.out_failed = 1;
            HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_qconv2d_i8(p, ctx->stream, 0, nullptr));
        } else {
            // an Add of the plan rides along (range_io.h): the kernels whose epilogue holds y in registers store the sum
            // as well and say so; the ranges they leave are then those of the sum
            if (const FnnResidualIo &res = ctx->residual; dev && res.residual && res.sum_out && res.of_out == dy && res.elems == (uint64_t)(b * oc * ho * wo)) {
                p.residual = res.residual; p.sum_out = res.sum_out;
            }
            // the caller asks for partial ranges of y (range_io.h): the epilogue inside the GEMM kernel leaves them.
            // Pairs already in place (y is one part of a one-image tensor that several calls write): behind them.
            const int range_base = rio.out_parts;
            const bool want_out = rio.out_table && dev && (range_base == 0 || (b == 1 && range_base < rio.out_stride));
            rio.out_parts = 0;
            if (want_out && rio.out_images == (uint64_t)b && rio.out_image_elems == (uint64_t)(oc * ho * wo)) {
                p.range_out = rio.out_table + 2 * (size_t)range_base; p.range_out_stride = rio.out_stride - range_base;
            }
            // Activation ranges: from the partial pairs the producer of x left (usable when the im2col matrix holds
            // every input value, i.e. every input row and column is reached by some tap, and the group is the whole
            // image; the zero of the padding joins them), else from a scan of x.
            int nparts = 0;
            int pad_touched = 0;
            bool all_reached = false;
            if (rio.in_table && dev && groups == 1 && rio.in_parts > 0) fnn_conv_coverage(p, &pad_touched, &all_reached);
            if (all_reached) {
                p.minmax_partial = const_cast<float *>(rio.in_table);
                p.part_stride = rio.in_stride; p.range_zero = pad_touched;
                nparts = rio.in_parts;
                rio.in_used = 1;
            } else {
                HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_qconv2d_i8(p, ctx->stream, 3, &nparts));
            }
            // One implicit-GEMM kernel where it is ahead, else the operand kernel and the int8 GEMM.  Either forms
            // the scales itself when its workgroups' rows touch at most two images and they are few enough for the
            // repeated reduction to be cheaper than a launch.
            int wg_rows = 64;
            int64_t wgs = 0;
            // Many groups (depthwise convolutions): the matrix-core paths are one or two launches per group on a few
            // channels each; the direct kernel covers all groups in one launch (64 groups of one channel at 80 x 80:
            // 0.25 ms against 0.86-1.14 ms per call from host memory, 8 groups: equal, 4 groups: 0.35 against 0.22).
            const bool many_groups = groups >= 16;
            const bool implicit = !many_groups && fnn_implicit_conv_takes(w, p, ctx->options[FNN_OPT_CONV_IMPLICIT], &wg_rows, &wgs);
            if (!implicit) { wg_rows = 64; wgs = fnn_conv_operand_workgroups(p); }
            const bool fused_scales = !many_groups && ho * wo >= wg_rows && nparts <= 4 * QCONV_NPART && wgs <= 8192;
            if (fused_scales) p.nparts = nparts;
            else HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_qconv2d_i8(p, ctx->stream, 4, &nparts));
            bool handled = false;
            int rc2 = many_groups ? FNN_OK : (implicit ? fnn_i8_implicit_conv(ctx, ctx->stream, w, p, &handled) : fnn_i8_tiled_conv(ctx, ctx->stream, w, p, &handled));
            if (rc2) return rc2;
            if (implicit && !handled) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, "the implicit convolution kernel declined a shape it had accepted");
            if (!handled) {
                if (fused_scales) HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_qconv2d_i8(p, ctx->stream, 4, &nparts));
                p.nparts = 0;
                HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_qconv2d_i8(p, ctx->stream, 2, nullptr));
            }
            if (rio.out_table && dev && rio.out_parts == 0) rio.out_failed = 1;   // y is written, its ranges are not
            rio.out_parts += range_base;
        }
        if (!dev) {
            HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(y, dy, yout, hipMemcpyDeviceToHost, ctx->stream));
            if (acc_out) HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(acc_out, dacc, yout, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(ctx, FNN_ERR_DISPATCH, hipStreamSynchronize(ctx->stream));
        }
        return FNN_OK;
    });
}

int fnn_hip_qconv2d_i8act(fnn_hip_ctx *ctx, const fnn_hip_weight *w, const uint8_t *payload, int64_t b, int64_t c,
                          int64_t h, int64_t wd, int kh, int kw, int stride, int pad, int dil, int groups,
                          const float *bias, int act, float *y, int flags)
{
    return guarded(ctx, "fnn_hip_qconv2d_i8act", [&]() -> int {
        if (!ctx) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_hip_qconv2d_i8act: NULL context");
        if (!w) return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8_i8: missing weight_meta for quantized weight");
        if (w->dtype != FNN_DT_I8 && w->dtype != FNN_DT_I4)
            return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "conv2d_i8_i8: weight type %d has no I8-activation kernel", w->dtype);
        if (groups <= 0) return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8_i8: groups must be > 0");
        if (b < 0 || c <= 0 || h <= 0 || wd <= 0 || kh <= 0 || kw <= 0 || stride <= 0 || dil <= 0 || pad < 0)
            return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8_i8: invalid geometry");
        if (c % groups || w->rows % groups)
            return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8_i8: channels (%lld in, %lld out) not divisible by groups %d",
                        (long long)c, (long long)w->rows, groups);
        if (w->inner != (c / groups) * kh * kw)
            return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8_i8: weight inner dim %lld != C/g*KH*KW = %lld", (long long)w->inner,
                        (long long)((c / groups) * kh * kw));
        if (act < FNN_ACT_NONE || act > FNN_ACT_SILU) return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "conv2d_i8_i8: unknown activation %d", act);
        auto osz = [](int64_t in, int k, int s, int p, int d) -> int64_t {
            int64_t dk = (int64_t)(k - 1) * d + 1;
            return (in + 2 * p >= dk) ? (in + 2 * p - dk) / s + 1 : 0;
        };
        const int64_t ho = osz(h, kh, stride, pad, dil), wo = osz(wd, kw, stride, pad, dil);
        const int64_t oc = w->rows;
        if (b == 0 || ho == 0 || wo == 0) return FNN_OK;
        if (!payload || !y) return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8_i8: NULL input or output pointer");
        if (b * groups > 65535) return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "conv2d_i8_i8: batch*groups > 65535");
        const bool dev = (flags & FNN_FLAG_DEVICE_PTRS) != 0;
        if (dev && (reinterpret_cast<uintptr_t>(payload) & 3))
            return fail(ctx, FNN_ERR_DISPATCH, "conv2d_i8_i8: activation payload must be 4-byte aligned");
        fnn_hip_weight *wm = const_cast<fnn_hip_weight *>(w);
        if (!wm->row_qsum) {
            if (ctx->capturing) return fail(ctx, FNN_ERR_MEMORY, "conv2d_i8_i8: first use of a weight during graph capture");
            HIP_TRY(ctx, FNN_ERR_MEMORY, hipMalloc((void **)&wm->row_qsum, (size_t)oc * 4 + 64));
            HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_row_qsum(w, wm->row_qsum, ctx->stream));
        }
        const size_t xin = (size_t)(b * c * h * wd) + 8, yout = (size_t)(b * oc * ho * wo) * 4;
        const uint8_t *dp = payload;
        const float *dbias = bias;
        float *dy = y;
        int rc;
        if (!dev) {
            if ((rc = ensure(ctx, ctx->st_a, xin))) return rc;
            if ((rc = ensure(ctx, ctx->st_out, yout))) return rc;
            HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(ctx->st_a.ptr, payload, xin, hipMemcpyHostToDevice, ctx->stream));
            dp = (const uint8_t *)ctx->st_a.ptr;
            dy = (float *)ctx->st_out.ptr;
            if (bias) {
                if ((rc = ensure(ctx, ctx->st_bias, (size_t)oc * 4))) return rc;
                HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(ctx->st_bias.ptr, bias, (size_t)oc * 4, hipMemcpyHostToDevice, ctx->stream));
                dbias = (const float *)ctx->st_bias.ptr;
            }
        }
        if ((rc = ensure(ctx, ctx->st_tmp, (size_t)(b * groups) * (QCONV_NPART * 2 + 4) * 4))) return rc;
        QConvArgs p;
        p.words = w->words; p.scales = w->scales; p.zeros = w->zeros; p.row_qsum = wm->row_qsum;
        p.x = nullptr; p.bias = dbias; p.y = dy; p.acc_out = nullptr;
        p.minmax_partial = (float *)ctx->st_tmp.ptr;
        p.actq = p.minmax_partial + (size_t)(b * groups) * QCONV_NPART * 2;
        p.b = b; p.c = c; p.h = h; p.w = wd; p.oc = oc; p.ho = ho; p.wo = wo; p.kp = w->kp;
        p.kh = kh; p.kw = kw; p.stride = stride; p.pad = pad; p.dil = dil; p.groups = groups; p.act = act;
        p.wbits = w->dtype == FNN_DT_I4 ? 4 : 8;
        p.x8 = reinterpret_cast<const int8_t *>(dp + 8);
        p.payload_i4 = w->dtype == FNN_DT_I4; p.nparts = 0;
        p.part_stride = QCONV_NPART; p.range_zero = 0; p.range_out = nullptr; p.range_out_stride = 0;
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_conv_actq_from_payload(dp, p.actq, (int)(b * groups), ctx->stream));
        bool handled = false;
        if ((rc = fnn_i8_tiled_conv(ctx, ctx->stream, w, p, &handled))) return rc;
        if (!handled) return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "conv2d_i8_i8: shape outside the integer GEMM's limits");
        if (!dev) {
            HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(y, dy, yout, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(ctx, FNN_ERR_DISPATCH, hipStreamSynchronize(ctx->stream));
        }
        return FNN_OK;
    });
}

int fnn_hip_elementwise(fnn_hip_ctx *ctx, int op, const float *a, const float *b, uint64_t nb, float *out, uint64_t n)
{
    return guarded(ctx, "fnn_hip_elementwise", [&]() -> int {
        if (!ctx || !a || !out) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_elementwise: NULL argument");
        if (op < 0 || op > 3) return fail(ctx, FNN_ERR_UNSUPPORTED_OP, "fnn_hip_elementwise: unknown op %d", op);
        if (op == 0 && (!b || nb == 0)) return fail(ctx, FNN_ERR_DISPATCH, "add_f32: missing second operand");
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_eltwise(op, a, b, nb, out, n, ctx->stream, &ctx->range));
        return FNN_OK;
    });
}

int fnn_hip_fill_f32(fnn_hip_ctx *ctx, float *dst, uint64_t n, float value)
{
    return guarded(ctx, "fnn_hip_fill_f32", [&]() -> int {
        if (!ctx || (!dst && n)) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_fill_f32: NULL argument");
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_fill(dst, n, value, ctx->stream));
        return FNN_OK;
    });
}

int fnn_hip_copy(fnn_hip_ctx *ctx, void *dst_dev, const void *src_dev, uint64_t bytes)
{
    return guarded(ctx, "fnn_hip_copy", [&]() -> int {
        if (!ctx || ((!dst_dev || !src_dev) && bytes)) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_copy: NULL argument");
        if (bytes == 0) return FNN_OK;
        HIP_TRY(ctx, FNN_ERR_MEMORY, hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, ctx->stream));
        return FNN_OK;
    });
}

int fnn_hip_copy2d_f32(fnn_hip_ctx *ctx, float *dst, uint64_t dst_pitch, uint64_t dst_len, const float *src, uint64_t src_pitch,
                       uint64_t src_len, uint64_t width, uint64_t height)
{
    return guarded(ctx, "fnn_hip_copy2d_f32", [&]() -> int {
        if (!ctx || ((!dst || !src) && width && height)) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_copy2d_f32: NULL argument");
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_copy2d(dst, dst_pitch, dst_len, src, src_pitch, src_len, width, height, ctx->stream, &ctx->range));
        return FNN_OK;
    });
}

int fnn_hip_concat_f32(fnn_hip_ctx *ctx, float *dst, uint64_t dst_pitch, uint64_t dst_len, uint64_t n_parts, const float *const *srcs,
                       const uint64_t *widths, const uint64_t *src_lens, uint64_t height)
{
    return guarded(ctx, "fnn_hip_concat_f32", [&]() -> int {
        if (!ctx || !dst || (n_parts && (!srcs || !widths || !src_lens))) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_concat_f32: NULL argument");
        // one launch when nothing is clipped and the parts are few; else part by part
        bool whole = height > 0 && dst_len >= height * dst_pitch && n_parts <= 8;
        for (uint64_t j = 0; j < n_parts && whole; j++) whole = srcs[j] && src_lens[j] >= height * widths[j] && widths[j] > 0;
        bool done = false;
        if (whole) HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_concat(dst, dst_pitch, (int)n_parts, srcs, widths, height, ctx->stream, &ctx->range, &done));
        if (done) return FNN_OK;
        uint64_t off = 0;
        for (uint64_t j = 0; j < n_parts; j++) {
            if (off < dst_len && widths[j] && srcs[j])
                HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_copy2d(dst + off, dst_pitch, dst_len - off, srcs[j], widths[j], src_lens[j], widths[j], height, ctx->stream, &ctx->range));
            off += widths[j];
        }
        return FNN_OK;
    });
}

int fnn_hip_maxpool2d_f32(fnn_hip_ctx *ctx, const float *x, uint64_t in_len, float *y, uint64_t out_len, uint64_t n, uint64_t c,
                          uint64_t h, uint64_t w, uint64_t kernel, uint64_t stride, uint64_t pad, int64_t *indices, uint64_t idx_len)
{
    return guarded(ctx, "fnn_hip_maxpool2d_f32", [&]() -> int {
        if (!ctx || !x || !y) return fail(ctx, FNN_ERR_DISPATCH, "pool_f32: NULL argument");
        if (kernel == 0 || stride == 0 || kernel > 1024 || pad > 1024) return fail(ctx, FNN_ERR_DISPATCH, "pool_f32: invalid kernel, stride or padding");
        const uint64_t hp = h + 2 * pad, wp = w + 2 * pad;
        const uint64_t ho = (hp > kernel ? hp - kernel : 0) / stride + 1, wo = (wp > kernel ? wp - kernel : 0) / stride + 1;
        uint64_t total = n * c * ho * wo;
        if (total > out_len) total = out_len;   // writes past the output slice are dropped (ops.rs:147-149)
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_maxpool2d(x, in_len, y, total, c, h, w, ho, wo, (int)kernel, (int)stride, (int)pad, indices,
                                                         indices ? (idx_len < n * c * ho * wo ? idx_len : n * c * ho * wo) : 0, ctx->stream, &ctx->range));
        return FNN_OK;
    });
}

int fnn_hip_avgpool2d_f32(fnn_hip_ctx *ctx, const float *x, uint64_t in_len, float *y, uint64_t out_len, uint64_t n, uint64_t c,
                          uint64_t h, uint64_t w, uint64_t kernel, uint64_t stride, uint64_t pad)
{
    return guarded(ctx, "fnn_hip_avgpool2d_f32", [&]() -> int {
        if (!ctx || !x || !y) return fail(ctx, FNN_ERR_DISPATCH, "pool_f32: NULL argument");
        if (kernel == 0 || stride == 0 || kernel > 1024 || pad > 1024) return fail(ctx, FNN_ERR_DISPATCH, "pool_f32: invalid kernel, stride or padding");
        const uint64_t hp = h + 2 * pad, wp = w + 2 * pad;
        const uint64_t ho = (hp > kernel ? hp - kernel : 0) / stride + 1, wo = (wp > kernel ? wp - kernel : 0) / stride + 1;
        uint64_t total = n * c * ho * wo;
        if (total > out_len) total = out_len;   // writes past the output slice are dropped (ops.rs:203-205)
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_avgpool2d(x, in_len, y, total, h, w, ho, wo, (int)kernel, (int)stride, (int)pad, ctx->stream));
        return FNN_OK;
    });
}

int fnn_hip_upsample_nearest2d_f32(fnn_hip_ctx *ctx, const float *x, float *y, uint64_t nc, uint64_t h, uint64_t w, uint64_t sh, uint64_t sw)
{
    return guarded(ctx, "fnn_hip_upsample_nearest2d_f32", [&]() -> int {
        if (!ctx || !x || !y) return fail(ctx, FNN_ERR_DISPATCH, "upsample_nearest2d: NULL argument");
        if (sh > 1024 || sw > 1024) return fail(ctx, FNN_ERR_DISPATCH, "upsample_nearest2d: scale too large");
        HIP_TRY(ctx, FNN_ERR_DISPATCH, launch_upsample_nearest2d(x, y, nc, h, w, (int)sh, (int)sw, ctx->stream, &ctx->range));
        return FNN_OK;
    });
}

int fnn_hip_timer_start(fnn_hip_ctx *ctx)
{
    return guarded(ctx, "fnn_hip_timer_start", [&]() -> int {
        if (!ctx) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_hip_timer_start: NULL context");
        HIP_TRY(ctx, FNN_ERR_DISPATCH, hipEventRecord(ctx->ev0, ctx->stream));
        return FNN_OK;
    });
}

int fnn_hip_timer_stop(fnn_hip_ctx *ctx, float *ms)
{
    return guarded(ctx, "fnn_hip_timer_stop", [&]() -> int {
        if (!ctx || !ms) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_timer_stop: NULL argument");
        HIP_TRY(ctx, FNN_ERR_DISPATCH, hipEventRecord(ctx->ev1, ctx->stream));
        HIP_TRY(ctx, FNN_ERR_DISPATCH, hipEventSynchronize(ctx->ev1));
        HIP_TRY(ctx, FNN_ERR_DISPATCH, hipEventElapsedTime(ms, ctx->ev0, ctx->ev1));
        return FNN_OK;
    });
}

int fnn_hip_graph_begin(fnn_hip_ctx *ctx)
{
    return guarded(ctx, "fnn_hip_graph_begin", [&]() -> int {
        if (!ctx) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_hip_graph_begin: NULL context");
        if (ctx->capturing) return fail(ctx, FNN_ERR_DISPATCH, "graph capture already active");
        HIP_TRY(ctx, FNN_ERR_DISPATCH, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
        ctx->capturing = true;
        return FNN_OK;
    });
}

int fnn_hip_graph_end(fnn_hip_ctx *ctx, fnn_hip_graph **out)
{
    return guarded(ctx, "fnn_hip_graph_end", [&]() -> int {
        if (!ctx || !out) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_graph_end: NULL argument");
        if (!ctx->capturing) return fail(ctx, FNN_ERR_DISPATCH, "no graph capture active");
        *out = nullptr;
        // the stream leaves capture mode first, whatever fails afterwards
        hipGraph_t graph = nullptr;
        hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
        ctx->capturing = false;
        if (e != hipSuccess) return fail(ctx, FNN_ERR_DISPATCH, "graph capture failed: %s", hipGetErrorString(e));
        fnn_hip_graph *g = new (std::nothrow) fnn_hip_graph();
        if (!g) {
            (void)hipGraphDestroy(graph);
            return fail(ctx, FNN_ERR_MEMORY, "out of host memory");
        }
        g->graph = graph;
        e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
        if (e != hipSuccess) {
            (void)hipGraphDestroy(g->graph);
            delete g;
            return fail(ctx, FNN_ERR_DISPATCH, "graph instantiation failed: %s", hipGetErrorString(e));
        }
        *out = g;
        return FNN_OK;
    });
}

int fnn_hip_graph_launch(fnn_hip_ctx *ctx, fnn_hip_graph *g)
{
    return guarded(ctx, "fnn_hip_graph_launch", [&]() -> int {
        if (!ctx || !g) return fail(ctx, FNN_ERR_DISPATCH, "fnn_hip_graph_launch: NULL argument");
        HIP_TRY(ctx, FNN_ERR_DISPATCH, hipGraphLaunch(g->exec, ctx->stream));
        return FNN_OK;
    });
}

uint64_t fnn_hip_workspace_epoch(const fnn_hip_ctx *ctx) { return ctx ? ctx->ws_epoch : 0; }

int fnn_hip_graph_destroy(fnn_hip_ctx *ctx, fnn_hip_graph *g)
{
    return guarded(ctx, "fnn_hip_graph_destroy", [&]() -> int {
        if (!g) return FNN_OK;
        if (ctx && ctx->stream) (void)hipStreamSynchronize(ctx->stream);
        if (g->exec) (void)hipGraphExecDestroy(g->exec);
        if (g->graph) (void)hipGraphDestroy(g->graph);
        delete g;
        return FNN_OK;
    });
}

}  // extern "C"

// staging access for the matrix-core translation units
int fnn_ctx_ensure_tmp(fnn_hip_ctx *ctx, int which, size_t bytes, void **ptr)
{
    if (ctx->static_mode) {
        // fnn_hip_qmatmul_static: fixed regions of the static workspace, nothing grows
        const size_t off = which == 0 ? 0 : kStaticOperandBytes;
        const size_t cap = which == 0 ? kStaticOperandBytes : (which == 1 ? kStaticPartialBytes : 0);
        if (bytes > cap)
            return fail(ctx, FNN_ERR_MEMORY,
                        "fnn_hip_qmatmul_static: this shape needs %zu bytes of %s workspace, the static buffer holds %zu: use fnn_hip_qmatmul",
                        bytes, which == 0 ? "operand" : (which == 1 ? "split-K" : "weight expansion"), cap);
        *ptr = ctx->static_ws + off;
        return FNN_OK;
    }
    // 0: prepared operands, 1: partial tiles / accumulators, 2 and 3: conv operand, transient weight expansion,
    // 4: the prepared operand one MatMul call leaves for the next
    Staging &s = which == 0 ? ctx->st_tmp : (which == 1 ? ctx->st_tmp2 : (which == 4 ? ctx->st_tmp4 : ctx->st_tmp3));
    int rc = ensure(ctx, s, bytes);
    if (rc) return rc;
    *ptr = s.ptr;
    return FNN_OK;
}

bool fnn_ctx_capturing(fnn_hip_ctx *ctx) { return ctx->capturing; }

bool fnn_ctx_no_alloc(fnn_hip_ctx *ctx) { return ctx->capturing || ctx->static_mode; }

int fnn_ctx_fail(fnn_hip_ctx *ctx, int code, const char *msg) { return fail(ctx, code, "%s", msg); }

int64_t fnn_ctx_option(const fnn_hip_ctx *ctx, int option) { return ctx->options[option]; }
uint32_t *fnn_ctx_stream_counters(fnn_hip_ctx *ctx) { return ctx->stream_counters; }
FnnRangeIo *fnn_ctx_range_io(fnn_hip_ctx *ctx) { return &ctx->range; }
FnnResidualIo *fnn_ctx_residual_io(fnn_hip_ctx *ctx) { return &ctx->residual; }
FnnPrepIo *fnn_ctx_prep_io(fnn_hip_ctx *ctx) { return &ctx->prep; }
FnnPreparedOperand *fnn_ctx_prepared(fnn_hip_ctx *ctx) { return &ctx->prepared; }
bool fnn_ctx_static_mode(fnn_hip_ctx *ctx) { return ctx->static_mode; }
