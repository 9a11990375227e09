// Host-side HipBackend: walks fastnn's instruction stream (src/backend/mod.rs:60-131)
// over a device-resident arena and routes the quantised MatMul / Conv2d kernels to
// libfastnn_hip's C ABI.  Plain C++ on top of that ABI: no HIP types appear here.
//
// Follows CpuBackend::dispatch (src/backend/cpu/mod.rs:2644-2683) for instruction order
// and slice handling, quantized_matmul_dispatch (src/backend/cpu/matmul.rs:165-225) for
// the [activation, weight] / [M,K,N] convention, and the conv2d arm
// (src/backend/cpu/mod.rs:4106-4260) for the nine Conv2d params.  A kernel name that has
// no GPU implementation yields FNN_ERR_UNSUPPORTED_OP naming the kernel, so that a
// caller can run that one instruction elsewhere (src/backend/wgpu/mod.rs:162-239).
#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <exception>
#include <map>
#include <new>
#include <string>
#include <vector>

#include "../../include/fastnn_hip_backend.h"

namespace {

enum InstrKind { K_WRITE_CONST, K_CALL, K_FILL, K_MEMCOPY };

struct Meta {
    bool present = false;
    uint64_t bit_width = 0;
    std::vector<float> scales, zeros, codebook;
    std::vector<uint64_t> shape;
    uint64_t qblock = 0;
};

struct Instr {
    InstrKind kind;
    fnn_slice dst{0, 0}, src{0, 0};
    std::vector<uint8_t> data;
    float value = 0.0f;
    std::string kernel;
    bool has_secondary = false;   // CallKernel.secondary_output_slice (MaxPool indices)
    fnn_slice secondary{0, 0};
    std::vector<fnn_slice> inputs;
    std::vector<uint64_t> params;
    Meta meta;
    bool clobbered = false;  // WriteConst only: another instruction of the plan writes into dst
};

bool overlaps(const fnn_slice &a, const fnn_slice &b)
{
    return a.size && b.size && a.offset < b.offset + b.size && b.offset < a.offset + a.size;
}

struct KernelName {
    std::string base;
    int act = FNN_ACT_NONE;
};

// "matmul_i4_silu" -> {"matmul_i4", SILU}; names without an epilogue tag pass through.
KernelName split_activation(const std::string &name)
{
    KernelName r{name, FNN_ACT_NONE};
    static const struct { const char *suffix; int act; } tags[] = {
        {"_relu", FNN_ACT_RELU}, {"_gelu", FNN_ACT_GELU}, {"_silu", FNN_ACT_SILU}};
    for (const auto &t : tags) {
        size_t n = strlen(t.suffix);
        if (name.size() > n && name.compare(name.size() - n, n, t.suffix) == 0) {
            r.base = name.substr(0, name.size() - n);
            r.act = t.act;
            return r;
        }
    }
    return r;
}

int matmul_dtype(const std::string &base)
{
    if (base == "matmul_i8") return FNN_DT_I8;
    if (base == "matmul_i4") return FNN_DT_I4;
    if (base == "matmul_u8") return FNN_DT_U8;
    if (base == "matmul_u4") return FNN_DT_U4;
    if (base == "matmul_f8") return FNN_DT_F8;
    if (base == "matmul_f8r") return FNN_DT_F8R;
    if (base == "matmul_f4") return FNN_DT_F4;
    return -1;
}

}  // namespace

struct fnn_plan {
    uint64_t arena_size = 0;
    std::vector<Instr> instrs;
    uint64_t uid = 0;                 // never reused within the process
    uint64_t revision = 0;            // bumped whenever an instruction is added
    bool analysed = false;
    std::vector<fnn_slice> writes;    // union of every byte range the plan writes, as disjoint sorted intervals
    bool uploads_every_run = false;   // some WriteConst target is overwritten by the plan itself
    // WriteConst payloads stay valid in the arena of this backend (by unique id) at this generation
    uint64_t resident_uid = 0;
    uint64_t resident_generation = 0;
    uint64_t resident_seq = 0;        // host writes up to this sequence number are accounted for
    // HIP graph of the instruction stream, captured on a dispatch that found everything resident;
    // valid while the backend, its arena, its cached weights and the context's workspaces are the same
    fnn_hip_graph *graph = nullptr;
    uint64_t graph_uid = 0, graph_generation = 0, graph_weights_epoch = 0, graph_ws_epoch = 0, graph_scratch_epoch = 0;
    int graph_failures = 0;           // captures that did not go through; after two the plan stays eager
    bool last_replayed = false;
};

struct fnn_backend {
    fnn_hip_ctx *ctx = nullptr;
    uint8_t *arena = nullptr;
    uint64_t arena_bytes = 0;
    uint64_t uid = 0;         // never reused within the process
    uint64_t generation = 1;  // bumped when the arena is re-allocated or the write log overflows
    // Writes into the arena that a plan cannot know of: host writes (write_arena) and everything another plan's
    // dispatch wrote.  One entry per distinct byte range, with the sequence number of the latest write to it, so the
    // usual cycle (same input ranges every forward, the same few plans taking turns) keeps the log at a fixed size.
    // A plan's constants stay resident across writes that touch none of them.
    uint64_t write_seq = 0;
    std::vector<std::pair<uint64_t, fnn_slice>> host_writes;
    uint64_t last_plan_uid = 0, last_plan_revision = 0;   // the plan whose write set was logged last
    bool graph_replay = true;    // resident plans replay as one HIP graph (fnn_backend_set_graph_replay)
    uint64_t weights_epoch = 0;  // bumped whenever a cached device weight is created or released
    int kernel_flags = 0;        // extra FNN_FLAG_* bits for every MatMul / Conv2d call
    char err[1024] = {0};        // fixed storage: recording a failure never allocates
    std::map<std::pair<uint64_t, uint64_t>, fnn_hip_weight *> weights;  // (offset,size) like get_or_cache_packed
    std::vector<uint8_t> stage;
    uint8_t *scratch = nullptr;   // device copy of an input that overlaps its output
    uint64_t scratch_bytes = 0, scratch_epoch = 0;
};

namespace {

thread_local char g_err[1024] = {0};   // failures without a backend (create, plan building)

int fail(fnn_backend *b, int code, const char *fmt, ...) noexcept
{
    char *buf = b ? b->err : g_err;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, 1024, fmt, ap);
    va_end(ap);
    return code;
}

int lift(fnn_backend *b, int st) noexcept
{
    if (st != FNN_OK) {
        const char *m = fnn_hip_last_error(b->ctx);
        snprintf(b->err, sizeof b->err, "%s", m && *m ? m : "libfastnn_hip call failed");
    }
    return st;
}

// Every extern "C" body runs inside this: a C++ exception (std::bad_alloc from a container that copies a weight
// payload, std::length_error, ...) becomes a status code and a message instead of unwinding into the caller.
template <class F>
int guarded(fnn_backend *b, const char *fn, F &&body) noexcept
{
    try {
        return body();
    } catch (const std::bad_alloc &) {
        return fail(b, FNN_ERR_MEMORY, "%s: out of host memory", fn);
    } catch (const std::exception &e) {
        return fail(b, FNN_ERR_DISPATCH, "%s: %s", fn, e.what());
    } catch (...) {
        return fail(b, FNN_ERR_DISPATCH, "%s: unknown C++ exception", fn);
    }
}

// One more write to `s` that plans must notice: the entry of the same range takes the new sequence number, a new
// range is appended.  Past 4096 distinct ranges the log is dropped and every plan uploads its constants again.
void log_write(fnn_backend *b, const fnn_slice &s)
{
    if (s.size == 0) return;
    for (auto &e : b->host_writes)
        if (e.second.offset == s.offset && e.second.size == s.size) { e.first = b->write_seq; return; }
    if (b->host_writes.size() >= 4096) {
        b->host_writes.clear();
        b->generation++;
        return;
    }
    b->host_writes.emplace_back(b->write_seq, s);
}

bool in_arena(const fnn_backend *b, const fnn_slice &s)
{
    return s.offset <= b->arena_bytes && s.size <= b->arena_bytes - s.offset;
}

void drop_weights(fnn_backend *b)
{
    for (auto &kv : b->weights) fnn_hip_weight_release(b->ctx, kv.second);
    b->weights.clear();
    b->weights_epoch++;
}

void drop_weights_overlapping(fnn_backend *b, const fnn_slice &s)
{
    for (auto it = b->weights.begin(); it != b->weights.end();) {
        fnn_slice w{it->first.first, it->first.second};
        if (overlaps(w, s)) {
            fnn_hip_weight_release(b->ctx, it->second);
            it = b->weights.erase(it);
            b->weights_epoch++;
        } else {
            ++it;
        }
    }
}

// get_or_cache_packed + packed_tensor_from_meta: the packed words are taken from the
// arena bytes of w_slice once and kept as a registered device weight.
int weight_for(fnn_backend *b, const fnn_slice &ws, int dtype, const Meta &meta, uint64_t rows,
               uint64_t inner, const char *kernel, fnn_hip_weight **out)
{
    auto key = std::make_pair(ws.offset, ws.size);
    auto it = b->weights.find(key);
    if (it != b->weights.end()) {
        *out = it->second;
        return FNN_OK;
    }
    if (ws.size % 4) return fail(b, FNN_ERR_DISPATCH, "%s: weight slice of %llu bytes is not whole u32 words", kernel, (unsigned long long)ws.size);
    b->stage.resize(ws.size);
    int st = lift(b, fnn_hip_download(b->ctx, b->stage.data(), b->arena + ws.offset, ws.size));
    if (st) return st;
    static const float one = 1.0f, zero = 0.0f;
    const float *sc = &one, *zp = &zero;
    size_t nsc = 1, nzp = 1;
    int qb = 0;
    const float *cb = nullptr;
    if (meta.present) {
        sc = meta.scales.data(); nsc = meta.scales.size();
        zp = meta.zeros.data(); nzp = meta.zeros.size();
        qb = (int)meta.qblock;
        if (!meta.codebook.empty()) cb = meta.codebook.data();
    }
    fnn_hip_weight *w = nullptr;
    uint64_t id = ws.offset * 0x9E3779B97F4A7C15ull ^ ws.size;
    st = lift(b, fnn_hip_weight_register(b->ctx, id, dtype, (const uint32_t *)b->stage.data(), ws.size / 4,
                                         (int64_t)rows, (int64_t)inner, sc, nsc, zp, nzp, qb, cb, &w));
    if (st) return st;
    b->weights[key] = w;
    b->weights_epoch++;
    *out = w;
    return FNN_OK;
}

int run_matmul(fnn_backend *b, const Instr &in, const KernelName &kn, int dtype)
{
    const char *name = in.kernel.c_str();
    if (in.inputs.size() < 2) return FNN_OK;  // the CPU arm ignores a malformed slice list
    if (in.params.size() < 3) return fail(b, FNN_ERR_DISPATCH, "%s: expected params [M,K,N]", name);
    uint64_t m = in.params[0], k = in.params[1], n = in.params[2];
    const fnn_slice &as = in.inputs[0], &ws = in.inputs[1];
    if (as.size < m * k * 4) return fail(b, FNN_ERR_DISPATCH, "%s: activation slice holds %llu bytes, M*K*4 = %llu", name, (unsigned long long)as.size, (unsigned long long)(m * k * 4));
    if (in.dst.size < m * n * 4) return fail(b, FNN_ERR_DISPATCH, "%s: output slice holds %llu bytes, M*N*4 = %llu", name, (unsigned long long)in.dst.size, (unsigned long long)(m * n * 4));
    if (in.meta.present && !in.meta.codebook.empty()) {
        if (dtype != FNN_DT_I4) return fail(b, FNN_ERR_DISPATCH, "%s: a codebook needs 4-bit indices", name);
        dtype = FNN_DT_I4CB;
    }
    const float *bias = nullptr;
    if (in.inputs.size() >= 3 && in.inputs[2].size) {
        if (in.inputs[2].size < n * 4) return fail(b, FNN_ERR_DISPATCH, "%s: bias slice holds %llu bytes, N*4 = %llu", name, (unsigned long long)in.inputs[2].size, (unsigned long long)(n * 4));
        bias = (const float *)(b->arena + in.inputs[2].offset);
    }
    fnn_hip_weight *w = nullptr;
    int st = weight_for(b, ws, dtype, in.meta, n, k, name, &w);
    if (st) return st;
    if (m == 0 || n == 0) return FNN_OK;
    return lift(b, fnn_hip_qmatmul(b->ctx, w, (const float *)(b->arena + as.offset), (int64_t)m, bias, kn.act,
                                   (float *)(b->arena + in.dst.offset), FNN_FLAG_DEVICE_PTRS | b->kernel_flags));
}

int run_matmul_i8act(fnn_backend *b, const Instr &in, int dtype)
{
    const char *name = in.kernel.c_str();
    if (in.inputs.size() != 2) return FNN_OK;
    if (in.params.size() < 3) return fail(b, FNN_ERR_DISPATCH, "%s: expected params [M,K,N]", name);
    uint64_t m = in.params[0], k = in.params[1], n = in.params[2];
    const fnn_slice &as = in.inputs[0], &ws = in.inputs[1];
    if (as.size < 8 + m * k) return fail(b, FNN_ERR_DISPATCH, "%s: activation payload holds %llu bytes, 8+M*K = %llu", name, (unsigned long long)as.size, (unsigned long long)(8 + m * k));
    if (in.dst.size < m * n * 4) return fail(b, FNN_ERR_DISPATCH, "%s: output slice holds %llu bytes, M*N*4 = %llu", name, (unsigned long long)in.dst.size, (unsigned long long)(m * n * 4));
    fnn_hip_weight *w = nullptr;
    int st = weight_for(b, ws, dtype, in.meta, n, k, name, &w);
    if (st) return st;
    if (m == 0 || n == 0) return FNN_OK;
    return lift(b, fnn_hip_qmatmul_i8act(b->ctx, w, b->arena + as.offset, (int64_t)m, (float *)(b->arena + in.dst.offset),
                                         nullptr, FNN_FLAG_DEVICE_PTRS));
}

int run_quantize_activations(fnn_backend *b, const Instr &in)
{
    uint64_t numel = in.params.empty() ? 0 : in.params[0];
    bool per_channel = in.params.size() > 1 && in.params[1] == 1 && in.params.size() > 2 && in.params[2] > 0;
    if (per_channel) return fail(b, FNN_ERR_UNSUPPORTED_OP, "quantize_activations: per-channel payloads are not implemented on the GPU");
    if (in.inputs.empty()) return FNN_OK;
    const fnn_slice &xs = in.inputs[0];
    if (in.dst.size < 8) return fail(b, FNN_ERR_DISPATCH, "quantize_activations: output slice has no room for the header");
    uint64_t cap = in.dst.size - 8;
    if (numel > cap) numel = cap;  // min(out_bytes.len() - header, numel)
    if (xs.size < numel * 4) return fail(b, FNN_ERR_DISPATCH, "quantize_activations: input slice holds %llu bytes, numel*4 = %llu", (unsigned long long)xs.size, (unsigned long long)(numel * 4));
    float scale = 0.0f, zp = 0.0f;  // scale <= 0: dynamic max|x|/127
    if (in.params.size() >= 5) {
        uint32_t sb = (uint32_t)in.params[3], zb = (uint32_t)in.params[4];
        memcpy(&scale, &sb, 4);
        memcpy(&zp, &zb, 4);
        if (!(scale > 0.0f)) return fail(b, FNN_ERR_UNSUPPORTED_OP, "quantize_activations: calibrated scale %g is not positive", (double)scale);
    }
    return lift(b, fnn_hip_quantize_activations(b->ctx, (const float *)(b->arena + xs.offset), (int64_t)numel, scale, zp,
                                                b->arena + in.dst.offset, FNN_FLAG_DEVICE_PTRS));
}

// "dequantize_activations": params [numel, is_per_channel, num_channels] (src/backend/cpu/mod.rs:7009-7088)
int run_dequantize_activations(fnn_backend *b, const Instr &in)
{
    uint64_t numel = in.params.empty() ? 0 : in.params[0];
    bool per_channel = in.params.size() > 2 && in.params[1] == 1 && in.params[2] > 0;
    if (per_channel) return fail(b, FNN_ERR_UNSUPPORTED_OP, "dequantize_activations: per-channel payloads are not implemented on the GPU");
    if (in.inputs.empty()) return FNN_OK;
    const uint64_t out_len = in.dst.size / 4;
    if (numel > out_len) numel = out_len;   // out_f32.len().min(numel)
    return lift(b, fnn_hip_dequantize_activations(b->ctx, b->arena + in.inputs[0].offset, in.inputs[0].size,
                                                  (float *)(b->arena + in.dst.offset), numel));
}

int run_conv2d_i8(fnn_backend *b, const Instr &in, const KernelName &kn)
{
    const char *name = in.kernel.c_str();
    if (in.inputs.size() < 2) return FNN_OK;
    if (in.params.size() < 9)
        return fail(b, FNN_ERR_DISPATCH, "%s: expected at least 9 params [stride, padding, dilation, groups, input_c, input_h, input_w, kernel_h, kernel_w]", name);
    const uint64_t *p = in.params.data();
    uint64_t stride = p[0], pad = p[1], dil = p[2], groups = p[3], c = p[4], h = p[5], wd = p[6], kh = p[7], kw = p[8];
    if (groups == 0) return fail(b, FNN_ERR_DISPATCH, "%s: groups=0", name);
    if (!in.meta.present) return fail(b, FNN_ERR_DISPATCH, "%s: missing weight_meta", name);
    if (in.meta.shape.empty()) return fail(b, FNN_ERR_DISPATCH, "%s: weight_meta has no shape", name);
    uint64_t oc = in.meta.shape[0], inner = 1;
    for (size_t i = 1; i < in.meta.shape.size(); i++) inner *= in.meta.shape[i];
    uint64_t chw = c * h * wd;
    uint64_t batch = (in.inputs[0].size / 4) / (chw ? chw : 1);
    const float *bias = nullptr;
    if (in.inputs.size() >= 3 && in.inputs[2].size) {
        if (in.inputs[2].size < oc * 4) return fail(b, FNN_ERR_DISPATCH, "%s: bias slice holds %llu bytes, OC*4 = %llu", name, (unsigned long long)in.inputs[2].size, (unsigned long long)(oc * 4));
        bias = (const float *)(b->arena + in.inputs[2].offset);
    }
    if (stride == 0 || dil == 0) return fail(b, FNN_ERR_DISPATCH, "%s: stride and dilation must be positive", name);
    uint64_t eh = dil * (kh - 1) + 1, ew = dil * (kw - 1) + 1;
    if (h + 2 * pad < eh || wd + 2 * pad < ew) return fail(b, FNN_ERR_DISPATCH, "%s: kernel larger than padded input", name);
    uint64_t oh = (h + 2 * pad - eh) / stride + 1, ow = (wd + 2 * pad - ew) / stride + 1;
    if (in.dst.size < batch * oc * oh * ow * 4) return fail(b, FNN_ERR_DISPATCH, "%s: output slice holds %llu bytes, needs %llu", name, (unsigned long long)in.dst.size, (unsigned long long)(batch * oc * oh * ow * 4));
    // weight type as the CPU arm decides it (src/backend/cpu/mod.rs:4248-4264): by name for the types that run
    // as an f32 convolution with dequantised weights, else by bit width (codebook weights: f32 path as well)
    int dtype;
    if (kn.base == "conv2d_u4") dtype = FNN_DT_U4;
    else if (kn.base == "conv2d_u8") dtype = FNN_DT_U8;
    else if (kn.base == "conv2d_f4") dtype = FNN_DT_F4;
    else if (kn.base == "conv2d_f8r") dtype = FNN_DT_F8R;
    else if (kn.base == "conv2d_f8") dtype = FNN_DT_F8;
    else if (in.meta.bit_width == 4) dtype = in.meta.codebook.empty() ? FNN_DT_I4 : FNN_DT_I4CB;
    else dtype = FNN_DT_I8;
    fnn_hip_weight *w = nullptr;
    int st = weight_for(b, in.inputs[1], dtype, in.meta, oc, inner, name, &w);
    if (st) return st;
    if (batch == 0) return FNN_OK;
    return lift(b, fnn_hip_qconv2d(b->ctx, w, (const float *)(b->arena + in.inputs[0].offset), (int64_t)batch, (int64_t)c,
                                   (int64_t)h, (int64_t)wd, (int)kh, (int)kw, (int)stride, (int)pad, (int)dil, (int)groups,
                                   bias, kn.act, (float *)(b->arena + in.dst.offset), nullptr, FNN_FLAG_DEVICE_PTRS | b->kernel_flags));
}

// "conv2d_i8_i8" / "conv2d_i4_i8" (src/backend/cpu/mod.rs:3848-4098): input 0 is an activation payload
// [scale][zero][i8 NCHW]; the weight kernel is picked by weight_meta.bit_width
int run_conv2d_i8act(fnn_backend *b, const Instr &in, const KernelName &kn)
{
    const char *name = in.kernel.c_str();
    if (in.inputs.size() < 2) return FNN_OK;
    if (in.params.size() < 9)
        return fail(b, FNN_ERR_DISPATCH, "%s: expected at least 9 params [stride, padding, dilation, groups, input_c, input_h, input_w, kernel_h, kernel_w]", name);
    const uint64_t *p = in.params.data();
    uint64_t stride = p[0], pad = p[1], dil = p[2], groups = p[3], c = p[4], h = p[5], wd = p[6], kh = p[7], kw = p[8];
    if (groups == 0) return fail(b, FNN_ERR_DISPATCH, "%s: groups=0", name);
    if (!in.meta.present) return fail(b, FNN_ERR_DISPATCH, "%s: missing weight_meta", name);
    if (in.meta.shape.empty()) return fail(b, FNN_ERR_DISPATCH, "%s: weight_meta has no shape", name);
    if (in.inputs[0].size < 8) return fail(b, FNN_ERR_DISPATCH, "%s: activation payload holds %llu bytes, the header alone is 8", name, (unsigned long long)in.inputs[0].size);
    if (in.inputs[0].offset & 3) return fail(b, FNN_ERR_DISPATCH, "%s: activation payload must be 4-byte aligned", name);
    uint64_t oc = in.meta.shape[0], inner = 1;
    for (size_t i = 1; i < in.meta.shape.size(); i++) inner *= in.meta.shape[i];
    uint64_t chw = c * h * wd;
    uint64_t batch = (in.inputs[0].size - 8) / (chw ? chw : 1);
    const float *bias = nullptr;
    if (in.inputs.size() >= 3 && in.inputs[2].size) {
        if (in.inputs[2].size < oc * 4) return fail(b, FNN_ERR_DISPATCH, "%s: bias slice holds %llu bytes, OC*4 = %llu", name, (unsigned long long)in.inputs[2].size, (unsigned long long)(oc * 4));
        bias = (const float *)(b->arena + in.inputs[2].offset);
    }
    if (stride == 0 || dil == 0) return fail(b, FNN_ERR_DISPATCH, "%s: stride and dilation must be positive", name);
    uint64_t eh = dil * (kh - 1) + 1, ew = dil * (kw - 1) + 1;
    if (h + 2 * pad < eh || wd + 2 * pad < ew) return fail(b, FNN_ERR_DISPATCH, "%s: kernel larger than padded input", name);
    uint64_t oh = (h + 2 * pad - eh) / stride + 1, ow = (wd + 2 * pad - ew) / stride + 1;
    if (in.dst.size < batch * oc * oh * ow * 4) return fail(b, FNN_ERR_DISPATCH, "%s: output slice holds %llu bytes, needs %llu", name, (unsigned long long)in.dst.size, (unsigned long long)(batch * oc * oh * ow * 4));
    if (in.meta.bit_width == 4 && !in.meta.codebook.empty())
        return fail(b, FNN_ERR_UNSUPPORTED_OP, "%s: codebook weights have no I8-activation kernel", name);
    const int dtype = in.meta.bit_width == 4 ? FNN_DT_I4 : FNN_DT_I8;
    fnn_hip_weight *w = nullptr;
    int st = weight_for(b, in.inputs[1], dtype, in.meta, oc, inner, name, &w);
    if (st) return st;
    if (batch == 0) return FNN_OK;
    return lift(b, fnn_hip_qconv2d_i8act(b->ctx, w, b->arena + in.inputs[0].offset, (int64_t)batch, (int64_t)c, (int64_t)h, (int64_t)wd,
                                         (int)kh, (int)kw, (int)stride, (int)pad, (int)dil, (int)groups, bias, kn.act,
                                         (float *)(b->arena + in.dst.offset), FNN_FLAG_DEVICE_PTRS | b->kernel_flags));
}

int run_elementwise(fnn_backend *b, const Instr &in, int op)
{
    const char *name = in.kernel.c_str();
    if (in.inputs.empty()) return FNN_OK;
    uint64_t n = in.dst.size / 4;
    const fnn_slice &a = in.inputs[0];
    if (a.size / 4 < n) n = a.size / 4;
    const float *bp = nullptr;
    uint64_t nb = 0;
    if (op == 0) {
        if (in.inputs.size() < 2 || in.inputs[1].size < 4) return fail(b, FNN_ERR_DISPATCH, "%s: expected two inputs", name);
        bp = (const float *)(b->arena + in.inputs[1].offset);
        nb = in.inputs[1].size / 4;
    }
    return lift(b, fnn_hip_elementwise(b->ctx, op, (const float *)(b->arena + a.offset), bp, nb,
                                       (float *)(b->arena + in.dst.offset), n));
}

// An f32 op that reads `in` and writes `out` elementwise-unrelated positions must not alias: the CPU arms copy
// the input first when the slices overlap (src/backend/cpu/arena.rs:14-60).  Here: one device copy into the
// backend's scratch buffer.
int staged_input(fnn_backend *b, const fnn_slice &in, const fnn_slice &out, const float **src)
{
    *src = (const float *)(b->arena + in.offset);
    if (!overlaps(in, out)) return FNN_OK;
    if (b->scratch_bytes < in.size) {
        if (b->scratch) fnn_hip_free(b->ctx, b->scratch);
        b->scratch = nullptr;
        b->scratch_bytes = 0;
        void *d = nullptr;
        int st = lift(b, fnn_hip_malloc(b->ctx, in.size + 64, &d));
        if (st) return st;
        b->scratch = (uint8_t *)d;
        b->scratch_bytes = in.size;
        b->scratch_epoch++;
    }
    int st = lift(b, fnn_hip_copy(b->ctx, b->scratch, b->arena + in.offset, in.size));
    *src = (const float *)b->scratch;
    return st;
}

// "concat": params [axis, inner_stride, outer_count] (src/backend/cpu/mod.rs:4267-4324)
int run_concat(fnn_backend *b, const Instr &in)
{
    if (in.inputs.empty()) return FNN_OK;
    const uint64_t out_len = in.dst.size / 4;
    float *out = (float *)(b->arena + in.dst.offset);
    for (const auto &s : in.inputs)
        if (overlaps(s, in.dst)) return fail(b, FNN_ERR_DISPATCH, "concat: an input overlaps the output");
    if (in.params.size() >= 3) {
        const uint64_t outer = in.params[2] ? in.params[2] : 1;
        uint64_t pitch = 0;
        for (const auto &s : in.inputs) pitch += (s.size / 4) / outer;
        uint64_t off = 0;
        for (const auto &s : in.inputs) {
            const uint64_t len = s.size / 4, bs = len / outer;
            if (len % outer) return fail(b, FNN_ERR_DISPATCH, "concat: input of %llu elements does not split into %llu outer positions", (unsigned long long)len, (unsigned long long)outer);
            if (off < out_len) {
                int st = lift(b, fnn_hip_copy2d_f32(b->ctx, out + off, pitch, out_len - off, (const float *)(b->arena + s.offset), bs, len, bs, in.params[2]));
                if (st) return st;
            }
            off += bs;
        }
        return FNN_OK;
    }
    uint64_t off = 0;   // legacy form without axis information: inputs one after the other
    for (const auto &s : in.inputs) {
        const uint64_t len = s.size / 4;
        if (off < out_len) {
            int st = lift(b, fnn_hip_copy2d_f32(b->ctx, out + off, len, out_len - off, (const float *)(b->arena + s.offset), len, len, len, 1));
            if (st) return st;
        }
        off += len;
    }
    return FNN_OK;
}

// "slice_f32": params [dim, start, end, stride] (src/backend/cpu/mod.rs:4721-4760)
int run_slice(fnn_backend *b, const Instr &in)
{
    if (in.inputs.empty()) return FNN_OK;
    if (in.params.size() != 4) return fail(b, FNN_ERR_DISPATCH, "slice_f32: expected params [dim, start, end, stride]");
    const uint64_t start = in.params[1], end = in.params[2], stride = in.params[3];
    const uint64_t in_len = in.inputs[0].size / 4, out_len = in.dst.size / 4;
    uint64_t range_len = end > start ? end - start : 0;
    if (range_len < 1) range_len = 1;
    const uint64_t dim_size = out_len ? (in_len * range_len) / out_len : 0;
    const uint64_t outer = (dim_size > 0 && stride > 0) ? in_len / dim_size / stride : 1;
    const uint64_t slice_elems = range_len * stride;
    const uint64_t first = start * stride;
    if (first >= in_len || slice_elems == 0) return FNN_OK;
    const float *src = nullptr;
    int st = staged_input(b, in.inputs[0], in.dst, &src);
    if (st) return st;
    return lift(b, fnn_hip_copy2d_f32(b->ctx, (float *)(b->arena + in.dst.offset), slice_elems, out_len, src + first, dim_size * stride,
                                      in_len - first, slice_elems, outer));
}

// "pool_f32": params [kernel, stride, padding, is_max, N, C, H, W] (src/backend/cpu/mod.rs:4362-4470)
int run_pool(fnn_backend *b, const Instr &in)
{
    if (in.inputs.empty()) return FNN_OK;
    if (in.params.size() != 8) return fail(b, FNN_ERR_DISPATCH, "pool_f32: expected params [kernel, stride, padding, is_max, N, C, H, W]");
    const uint64_t *p = in.params.data();
    const float *src = nullptr;
    int st = staged_input(b, in.inputs[0], in.dst, &src);
    if (st) return st;
    if (p[3] != 1)   // pool_avg_f32_scalar (src/backend/cpu/microkernels/ops.rs:162-210)
        return lift(b, fnn_hip_avgpool2d_f32(b->ctx, src, in.inputs[0].size / 4, (float *)(b->arena + in.dst.offset), in.dst.size / 4, p[4],
                                             p[5], p[6], p[7], p[0], p[1], p[2]));
    // secondary output: i64 window position kh*kernel + kw of the maximum (MaxPool indices)
    int64_t *indices = nullptr;
    uint64_t idx_len = 0;
    if (in.has_secondary && in.secondary.size >= 8) {
        if (in.secondary.offset & 7) return fail(b, FNN_ERR_DISPATCH, "pool_f32: secondary output slice must be 8-byte aligned");
        if (overlaps(in.secondary, in.dst) || overlaps(in.secondary, in.inputs[0])) return fail(b, FNN_ERR_DISPATCH, "pool_f32: secondary output overlaps another slice");
        indices = (int64_t *)(b->arena + in.secondary.offset);
        idx_len = in.secondary.size / 8;
    }
    return lift(b, fnn_hip_maxpool2d_f32(b->ctx, src, in.inputs[0].size / 4, (float *)(b->arena + in.dst.offset), in.dst.size / 4, p[4], p[5],
                                         p[6], p[7], p[0], p[1], p[2], indices, idx_len));
}

// "upsample_nearest2d": params [scale_h, scale_w, h_in, w_in], defaults 2, 2, 1, 1 (src/backend/cpu/mod.rs:5496-5535)
int run_upsample(fnn_backend *b, const Instr &in)
{
    if (in.inputs.empty()) return FNN_OK;
    const uint64_t sh = in.params.size() > 0 ? in.params[0] : 2, sw = in.params.size() > 1 ? in.params[1] : 2;
    const uint64_t h = in.params.size() > 2 ? in.params[2] : 1, w = in.params.size() > 3 ? in.params[3] : 1;
    const uint64_t hw = h * w, in_len = in.inputs[0].size / 4;
    if (!(sh > 0 && sw > 0 && hw > 0 && in_len > 0 && in_len % hw == 0)) return FNN_OK;   // the CPU arm does nothing either
    const uint64_t nc = in_len / hw;
    if (in.dst.size / 4 < nc * hw * sh * sw) return fail(b, FNN_ERR_DISPATCH, "upsample_nearest2d: output slice holds %llu values, needs %llu", (unsigned long long)(in.dst.size / 4), (unsigned long long)(nc * hw * sh * sw));
    const float *src = nullptr;
    int st = staged_input(b, in.inputs[0], in.dst, &src);
    if (st) return st;
    return lift(b, fnn_hip_upsample_nearest2d_f32(b->ctx, src, (float *)(b->arena + in.dst.offset), nc, h, w, sh, sw));
}

int run_call(fnn_backend *b, const Instr &in)
{
    for (const auto &s : in.inputs)
        if (!in_arena(b, s)) return fail(b, FNN_ERR_DISPATCH, "%s: input slice [%llu,+%llu) outside the arena of %llu bytes", in.kernel.c_str(), (unsigned long long)s.offset, (unsigned long long)s.size, (unsigned long long)b->arena_bytes);
    if (!in_arena(b, in.dst)) return fail(b, FNN_ERR_DISPATCH, "%s: output slice [%llu,+%llu) outside the arena of %llu bytes", in.kernel.c_str(), (unsigned long long)in.dst.offset, (unsigned long long)in.dst.size, (unsigned long long)b->arena_bytes);
    if (in.has_secondary && !in_arena(b, in.secondary)) return fail(b, FNN_ERR_DISPATCH, "%s: secondary output slice [%llu,+%llu) outside the arena of %llu bytes", in.kernel.c_str(), (unsigned long long)in.secondary.offset, (unsigned long long)in.secondary.size, (unsigned long long)b->arena_bytes);
    const std::string &name = in.kernel;
    if (name == "quantize_activations") return run_quantize_activations(b, in);
    if (name == "dequantize_activations") return run_dequantize_activations(b, in);
    if (name == "matmul_i8_i8") return run_matmul_i8act(b, in, FNN_DT_I8);
    if (name == "matmul_i4_i8") return run_matmul_i8act(b, in, FNN_DT_I4);
    if (name == "add_f32") return run_elementwise(b, in, 0);
    if (name == "relu_f32") return run_elementwise(b, in, 1);
    if (name == "gelu_f32") return run_elementwise(b, in, 2);
    if (name == "silu_f32") return run_elementwise(b, in, 3);
    if (name == "concat") return run_concat(b, in);
    if (name == "slice_f32") return run_slice(b, in);
    if (name == "pool_f32") return run_pool(b, in);
    if (name == "upsample_nearest2d") return run_upsample(b, in);
    KernelName kn = split_activation(name);
    int dt = matmul_dtype(kn.base);
    if (dt >= 0) return run_matmul(b, in, kn, dt);
    if (kn.base == "conv2d_i8" || kn.base == "conv2d_i4" || kn.base == "conv2d_u8" || kn.base == "conv2d_u4" ||
        kn.base == "conv2d_f8" || kn.base == "conv2d_f8r" || kn.base == "conv2d_f4")
        return run_conv2d_i8(b, in, kn);
    if (kn.base == "conv2d_i8_i8" || kn.base == "conv2d_i4_i8") return run_conv2d_i8act(b, in, kn);
    return fail(b, FNN_ERR_UNSUPPORTED_OP, "%s", name.c_str());
}

void analyse(fnn_plan *p)
{
    for (auto &c : p->instrs) {
        if (c.kind != K_WRITE_CONST) continue;
        c.clobbered = false;
        for (const auto &o : p->instrs) {
            if (&o == &c) continue;
            if (overlaps(o.dst, c.dst) || (o.has_secondary && overlaps(o.secondary, c.dst))) { c.clobbered = true; break; }
        }
        if (c.clobbered && !c.data.empty()) p->uploads_every_run = true;
    }
    // the plan's write set as disjoint intervals (touching ranges are joined, gaps are never bridged)
    std::vector<fnn_slice> w;
    for (const auto &o : p->instrs) {
        if (o.dst.size) w.push_back(o.dst);
        if (o.has_secondary && o.secondary.size) w.push_back(o.secondary);
    }
    std::sort(w.begin(), w.end(), [](const fnn_slice &a, const fnn_slice &b) { return a.offset < b.offset; });
    p->writes.clear();
    for (const auto &r : w) {
        if (!p->writes.empty() && r.offset <= p->writes.back().offset + p->writes.back().size) {
            const uint64_t end = std::max(p->writes.back().offset + p->writes.back().size, r.offset + r.size);
            p->writes.back().size = end - p->writes.back().offset;
        } else {
            p->writes.push_back(r);
        }
    }
    p->analysed = true;
}

// After a dispatch of `p`: what it wrote is news to every other plan of this backend.  Logged when the plan (or its
// instruction list) differs from the one logged last; repeated dispatches of one plan add nothing.
void note_dispatched(fnn_backend *b, fnn_plan *p)
{
    if (b->last_plan_uid != p->uid || b->last_plan_revision != p->revision) {
        b->write_seq++;
        for (const auto &r : p->writes) log_write(b, r);
        b->last_plan_uid = p->uid;
        b->last_plan_revision = p->revision;
    }
    p->resident_uid = b->uid;
    p->resident_generation = b->generation;
    p->resident_seq = b->write_seq;
}

int run_instr(fnn_backend *b, fnn_plan *p, Instr &in, bool consts_resident)
{
    switch (in.kind) {
    case K_WRITE_CONST: {
        fnn_slice d{in.dst.offset, in.data.size()};
        if (!in_arena(b, d)) return fail(b, FNN_ERR_MEMORY, "WriteConst: %llu bytes at %llu outside the arena of %llu bytes", (unsigned long long)d.size, (unsigned long long)d.offset, (unsigned long long)b->arena_bytes);
        if (consts_resident && !in.clobbered) return FNN_OK;  // bytes already in place and never overwritten
        if (d.size == 0) return FNN_OK;
        drop_weights_overlapping(b, d);
        return lift(b, fnn_hip_upload(b->ctx, b->arena + d.offset, in.data.data(), d.size));
    }
    case K_FILL:
        if (!in_arena(b, in.dst)) return fail(b, FNN_ERR_MEMORY, "Fill: slice outside the arena");
        return lift(b, fnn_hip_fill_f32(b->ctx, (float *)(b->arena + in.dst.offset), in.dst.size / 4, in.value));
    case K_MEMCOPY: {
        if (!in_arena(b, in.dst) || !in_arena(b, in.src)) return fail(b, FNN_ERR_MEMORY, "MemCopy: slice outside the arena");
        uint64_t n = in.dst.size < in.src.size ? in.dst.size : in.src.size;
        if (n == 0 || in.dst.offset == in.src.offset) return FNN_OK;
        fnn_slice d{in.dst.offset, n}, s{in.src.offset, n};
        if (overlaps(d, s)) return fail(b, FNN_ERR_DISPATCH, "MemCopy: source and destination overlap");
        return lift(b, fnn_hip_copy(b->ctx, b->arena + d.offset, b->arena + s.offset, n));
    }
    case K_CALL:
        return run_call(b, in);
    }
    (void)p;
    return FNN_OK;
}

int dispatch_impl(fnn_backend *b, fnn_plan *p, uint64_t *elapsed_ns, uint64_t n_elapsed)
{
    if (!b || !p) return fail(b, FNN_ERR_DISPATCH, "dispatch: NULL argument");
    if (!b->arena) return fail(b, FNN_ERR_MEMORY, "dispatch: no arena allocated");
    if (p->arena_size > b->arena_bytes) return fail(b, FNN_ERR_MEMORY, "dispatch: plan needs an arena of %llu bytes, backend holds %llu", (unsigned long long)p->arena_size, (unsigned long long)b->arena_bytes);
    if (elapsed_ns && n_elapsed < p->instrs.size()) return fail(b, FNN_ERR_DISPATCH, "dispatch_profile: room for %llu timings, plan has %llu instructions", (unsigned long long)n_elapsed, (unsigned long long)p->instrs.size());
    if (!p->analysed) analyse(p);
    bool resident = p->resident_uid == b->uid && p->resident_generation == b->generation;
    if (resident && p->resident_seq != b->write_seq) {
        // the host wrote into the arena since: still resident unless a constant was hit
        for (const auto &hw : b->host_writes) {
            if (hw.first <= p->resident_seq) continue;
            for (const auto &c : p->instrs)
                if (c.kind == K_WRITE_CONST && overlaps(c.dst, hw.second)) { resident = false; break; }
            if (!resident) break;
        }
        if (resident) p->resident_seq = b->write_seq;
    }

    // Replay: a plan whose constants are in place, whose weights are all cached and whose
    // workspaces have their final size launches as one HIP graph (the executor's static-shape
    // plan, src/backend/executor.rs:639-667).  Profiling, re-uploaded constants and anything
    // that fails under capture keep the instruction-by-instruction path.
    const bool may_replay = b->graph_replay && !elapsed_ns && resident && !p->uploads_every_run && p->graph_failures < 2;
    if (p->graph && !(may_replay && p->graph_uid == b->uid && p->graph_generation == b->generation &&
                      p->graph_weights_epoch == b->weights_epoch && p->graph_ws_epoch == fnn_hip_workspace_epoch(b->ctx) &&
                      p->graph_scratch_epoch == b->scratch_epoch)) {
        fnn_hip_graph_destroy(p->graph_uid == b->uid ? b->ctx : nullptr, p->graph);
        p->graph = nullptr;
    }
    if (may_replay && !p->graph) {
        const uint64_t w0 = b->weights_epoch, s0 = fnn_hip_workspace_epoch(b->ctx), c0 = b->scratch_epoch;
        if (fnn_hip_graph_begin(b->ctx) == FNN_OK) {
            int st = FNN_OK;
            for (size_t i = 0; i < p->instrs.size() && st == FNN_OK; i++) st = run_instr(b, p, p->instrs[i], true);
            fnn_hip_graph *g = nullptr;
            int en = fnn_hip_graph_end(b->ctx, &g);
            if (st == FNN_OK && en == FNN_OK && g && w0 == b->weights_epoch && s0 == fnn_hip_workspace_epoch(b->ctx) && c0 == b->scratch_epoch) {
                p->graph = g;
                p->graph_uid = b->uid; p->graph_generation = b->generation;
                p->graph_weights_epoch = w0; p->graph_ws_epoch = s0; p->graph_scratch_epoch = c0;
            } else {
                if (g) fnn_hip_graph_destroy(b->ctx, g);
                p->graph_failures++;
                b->err[0] = 0;
            }
        } else {
            p->graph_failures++;
        }
    }
    p->last_replayed = false;
    if (p->graph) {
        int st = lift(b, fnn_hip_graph_launch(b->ctx, p->graph));
        if (st == FNN_OK) st = lift(b, fnn_hip_sync(b->ctx));
        p->last_replayed = st == FNN_OK;
        if (st == FNN_OK) note_dispatched(b, p);
        return st;
    }

    for (size_t i = 0; i < p->instrs.size(); i++) {
        auto t0 = std::chrono::steady_clock::now();
        int st = run_instr(b, p, p->instrs[i], resident);
        if (st == FNN_OK && elapsed_ns) st = lift(b, fnn_hip_sync(b->ctx));
        if (st != FNN_OK) {
            fnn_hip_sync(b->ctx);
            // what ran before the failure has written: other plans must see it
            b->write_seq++;
            for (const auto &r : p->writes) log_write(b, r);
            b->last_plan_uid = 0;
            p->resident_uid = 0;
            return st;
        }
        if (elapsed_ns) elapsed_ns[i] = (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - t0).count();
    }
    int st = lift(b, fnn_hip_sync(b->ctx));
    if (st == FNN_OK) note_dispatched(b, p);
    return st;
}

}  // namespace

extern "C" {

int fnn_backend_create(int device, fnn_backend **out)
{
    return guarded(nullptr, "fnn_backend_create", [&]() -> int {
        if (!out) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_backend_create: out is NULL");
        *out = nullptr;
        fnn_hip_ctx *ctx = nullptr;
        int st = fnn_hip_create(device, &ctx);
        if (st) {
            snprintf(g_err, sizeof g_err, "%s", fnn_hip_last_error(nullptr));
            return st;
        }
        static std::atomic<uint64_t> next_uid{1};
        fnn_backend *b = new (std::nothrow) fnn_backend();
        if (!b) {
            fnn_hip_destroy(ctx);
            return fail(nullptr, FNN_ERR_MEMORY, "fnn_backend_create: out of host memory");
        }
        b->uid = next_uid++;
        b->ctx = ctx;
        *out = b;
        return FNN_OK;
    });
}

void fnn_backend_destroy(fnn_backend *b)
{
    if (!b) return;
    drop_weights(b);
    if (b->arena) fnn_hip_free(b->ctx, b->arena);
    if (b->scratch) fnn_hip_free(b->ctx, b->scratch);
    fnn_hip_destroy(b->ctx);
    delete b;
}

const char *fnn_backend_name(const fnn_backend *) { return "hip"; }

int fnn_backend_set_kernel_flags(fnn_backend *b, int flags)
{
    if (!b) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_backend_set_kernel_flags: NULL backend");
    if (flags & ~(FNN_FLAG_ACT_F16_SINGLE | FNN_FLAG_FORCE_GENERIC | FNN_FLAG_PREFER_FMA))
        return fail(b, FNN_ERR_DISPATCH, "set_kernel_flags: only ACT_F16_SINGLE, FORCE_GENERIC and PREFER_FMA can be set per backend");
    if (flags != b->kernel_flags) b->weights_epoch++;   // captured graphs hold the old kernel choice
    b->kernel_flags = flags;
    return FNN_OK;
}

int fnn_backend_set_graph_replay(fnn_backend *b, int enabled)
{
    if (!b) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_backend_set_graph_replay: NULL backend");
    b->graph_replay = enabled != 0;
    return FNN_OK;
}

int fnn_backend_set_option(fnn_backend *b, int option, int64_t value)
{
    if (!b) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_backend_set_option: NULL backend");
    int st = lift(b, fnn_hip_set_option(b->ctx, option, value));
    if (st == FNN_OK) b->weights_epoch++;   // captured graphs hold the old kernel choice
    return st;
}

const char *fnn_backend_last_error(const fnn_backend *b) { return b ? b->err : g_err; }

int fnn_backend_allocate_arena(fnn_backend *b, uint64_t total_bytes)
{
    return guarded(b, "fnn_backend_allocate_arena", [&]() -> int {
        if (!b) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_backend_allocate_arena: NULL backend");
        drop_weights(b);
        if (b->arena) {
            fnn_hip_free(b->ctx, b->arena);
            b->arena = nullptr;
            b->arena_bytes = 0;
        }
        b->generation++;
        b->host_writes.clear();
        // CpuBuffer::new zero-fills; keep 64 bytes of slack so that vector loads at the end stay inside
        void *d = nullptr;
        uint64_t padded = ((total_bytes + 63) / 64) * 64 + 64;
        int st = lift(b, fnn_hip_malloc(b->ctx, padded, &d));
        if (st) return st;
        b->arena = (uint8_t *)d;
        b->arena_bytes = total_bytes;
        st = lift(b, fnn_hip_fill_f32(b->ctx, (float *)d, padded / 4, 0.0f));
        if (st) return st;
        return lift(b, fnn_hip_sync(b->ctx));
    });
}

int fnn_backend_write_arena(fnn_backend *b, uint64_t offset, const void *data, uint64_t size)
{
    return guarded(b, "fnn_backend_write_arena", [&]() -> int {
        if (!b) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_backend_write_arena: NULL backend");
        fnn_slice s{offset, size};
        if (!b->arena || !in_arena(b, s)) return fail(b, FNN_ERR_MEMORY, "write_arena: %llu bytes at %llu outside the arena of %llu bytes", (unsigned long long)size, (unsigned long long)offset, (unsigned long long)b->arena_bytes);
        if (size == 0) return FNN_OK;
        if (!data) return fail(b, FNN_ERR_DISPATCH, "write_arena: NULL data");
        drop_weights_overlapping(b, s);
        b->write_seq++;
        log_write(b, s);
        return lift(b, fnn_hip_upload(b->ctx, b->arena + offset, data, size));
    });
}

int fnn_backend_read_arena(fnn_backend *b, uint64_t offset, void *out, uint64_t size)
{
    return guarded(b, "fnn_backend_read_arena", [&]() -> int {
        if (!b) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_backend_read_arena: NULL backend");
        fnn_slice s{offset, size};
        if (!b->arena || !in_arena(b, s)) return fail(b, FNN_ERR_MEMORY, "read_arena: %llu bytes at %llu outside the arena of %llu bytes", (unsigned long long)size, (unsigned long long)offset, (unsigned long long)b->arena_bytes);
        if (size == 0) return FNN_OK;
        if (!out) return fail(b, FNN_ERR_DISPATCH, "read_arena: NULL destination");
        return lift(b, fnn_hip_download(b->ctx, out, b->arena + offset, size));
    });
}

int fnn_plan_create(uint64_t arena_size, fnn_plan **out)
{
    return guarded(nullptr, "fnn_plan_create", [&]() -> int {
        if (!out) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_create: out is NULL");
        static std::atomic<uint64_t> next_uid{1};
        *out = new fnn_plan();
        (*out)->arena_size = arena_size;
        (*out)->uid = next_uid++;
        return FNN_OK;
    });
}

void fnn_plan_destroy(fnn_plan *p)
{
    if (!p) return;
    if (p->graph) fnn_hip_graph_destroy(nullptr, p->graph);   // every dispatch ends with a sync: nothing in flight
    delete p;
}

uint64_t fnn_plan_len(const fnn_plan *p) { return p ? p->instrs.size() : 0; }

int fnn_plan_replayed(const fnn_plan *p) { return p && p->last_replayed ? 1 : 0; }

static void touched(fnn_plan *p)
{
    p->analysed = false;
    p->uploads_every_run = false;
    p->resident_uid = 0;
    p->revision++;
    if (p->graph) {
        fnn_hip_graph_destroy(nullptr, p->graph);
        p->graph = nullptr;
    }
}

int fnn_plan_add_write_const(fnn_plan *p, fnn_slice dst, const void *data, uint64_t len)
{
    return guarded(nullptr, "fnn_plan_add_write_const", [&]() -> int {
        if (!p || (!data && len)) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_add_write_const: NULL argument");
        Instr in;
        in.kind = K_WRITE_CONST;
        in.dst = fnn_slice{dst.offset, len};
        in.data.assign((const uint8_t *)data, (const uint8_t *)data + len);
        p->instrs.push_back(std::move(in));
        touched(p);
        return FNN_OK;
    });
}

int fnn_plan_add_fill(fnn_plan *p, fnn_slice dst, float value)
{
    return guarded(nullptr, "fnn_plan_add_fill", [&]() -> int {
        if (!p) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_add_fill: NULL plan");
        Instr in;
        in.kind = K_FILL;
        in.dst = dst;
        in.value = value;
        p->instrs.push_back(std::move(in));
        touched(p);
        return FNN_OK;
    });
}

int fnn_plan_add_memcopy(fnn_plan *p, fnn_slice dst, fnn_slice src)
{
    return guarded(nullptr, "fnn_plan_add_memcopy", [&]() -> int {
        if (!p) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_add_memcopy: NULL plan");
        Instr in;
        in.kind = K_MEMCOPY;
        in.dst = dst;
        in.src = src;
        p->instrs.push_back(std::move(in));
        touched(p);
        return FNN_OK;
    });
}

int fnn_plan_add_call_kernel(fnn_plan *p, const char *kernel_name, const fnn_slice *inputs, uint64_t n_inputs,
                             fnn_slice output, const fnn_slice *secondary_output, const uint64_t *params,
                             uint64_t n_params, const fnn_weight_meta *meta)
{
    return guarded(nullptr, "fnn_plan_add_call_kernel", [&]() -> int {
        if (!p || !kernel_name || (!inputs && n_inputs) || (!params && n_params))
            return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_add_call_kernel: NULL argument");
        Instr in;
        in.kind = K_CALL;
        in.kernel = kernel_name;
        in.inputs.assign(inputs, inputs + n_inputs);
        in.dst = output;
        if (secondary_output) {
            in.has_secondary = true;
            in.secondary = *secondary_output;
        }
        in.params.assign(params, params + n_params);
        if (meta) {
            // QuantizedWeightMeta.codebooks is a Vec<[f32; 16]>.  The quantisation pass emits one codebook per weight
            // (src/packed_tensor.rs:1310) and every decode of the reference reads codebooks[0] only
            // (src/packed_tensor.rs:398, 489, 586), whatever the vector's length: so does this backend.
            if (meta->n_codebooks >= 1 && !meta->codebooks)
                return fail(nullptr, FNN_ERR_DISPATCH, "%s: weight_meta.n_codebooks = %llu with a NULL codebooks pointer", kernel_name,
                            (unsigned long long)meta->n_codebooks);
            in.meta.present = true;
            in.meta.bit_width = meta->bit_width;
            if (meta->scales) in.meta.scales.assign(meta->scales, meta->scales + meta->n_scales);
            if (meta->zero_points) in.meta.zeros.assign(meta->zero_points, meta->zero_points + meta->n_zero_points);
            if (meta->shape) in.meta.shape.assign(meta->shape, meta->shape + meta->n_shape);
            in.meta.qblock = meta->quant_block_size;
            if (meta->n_codebooks >= 1) in.meta.codebook.assign(meta->codebooks, meta->codebooks + 16);
        }
        p->instrs.push_back(std::move(in));
        touched(p);
        return FNN_OK;
    });
}

int fnn_backend_dispatch(fnn_backend *b, fnn_plan *p)
{
    return guarded(b, "fnn_backend_dispatch", [&]() -> int { return dispatch_impl(b, p, nullptr, 0); });
}

int fnn_backend_dispatch_profile(fnn_backend *b, fnn_plan *p, uint64_t *elapsed_ns, uint64_t n)
{
    return guarded(b, "fnn_backend_dispatch_profile", [&]() -> int {
        if (!elapsed_ns) return fail(b, FNN_ERR_DISPATCH, "dispatch_profile: NULL timings");
        return dispatch_impl(b, p, elapsed_ns, n);
    });
}

}  // extern "C"
