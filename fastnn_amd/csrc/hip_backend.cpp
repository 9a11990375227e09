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
#include "range_io.h"

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
    // CallKernel.param_dims (src/backend/mod.rs:72-78): symbolic forms of `params`, resolved at dispatch time
    struct Dim {
        uint32_t kind = 0;      // 0 Known(value), 1 Symbol(sym), 2 Bounded{sym, max: value}
        uint64_t value = 0;
        std::string sym;
    };
    bool has_param_dims = false;
    std::vector<Dim> param_dims;
    bool has_node_id = false;   // CallKernel.node_id: carried through load / save, not used by dispatch
    uint64_t node_id = 0;
    Meta meta;
    bool clobbered = false;  // WriteConst only: another instruction of the plan writes into dst
    int add_operand = -1;    // MatMul whose output the next instruction (an add_f32) adds to a tensor: index (0 / 1) of that
                             // tensor among the Add's inputs, found by analyse(); -1: nothing to fuse
    bool add_is_conv = false;   // ... the same for a quantised Conv2d (the sum's value ranges then come from its kernel)
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
    std::vector<uint64_t> levels;     // ExecutablePlan.levels: carried through load / save (dispatch is sequential)
    std::string graph_env;            // shape environment the captured graph was recorded under
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
    bool has_unsupported = false;     // a segmented dispatch stopped at a kernel without a GPU implementation
    bool segment_resident = false;    // residency as the first segment of the pass in progress found it
    bool last_replayed = false;
    uint64_t ranges_used = 0;         // convolutions of the last host-side pass that took their ranges from a table
    size_t add_done = (size_t)-1;     // index of an Add whose sum the MatMul before it has already stored
    uint64_t residuals_fused = 0;     // such Adds in the last host-side pass
    size_t prep_ready = (size_t)-1;   // index of a MatMul whose operand the call before it has prepared
    uint64_t operands_handed = 0;     // such MatMuls in the last host-side pass
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
    std::vector<std::pair<std::string, uint64_t>> shape_env;   // ShapeEnv of the dispatch in progress
    std::string shape_env_sig;   // the same as one string: graphs recorded under another environment are stale
    char err[1024] = {0};        // fixed storage: recording a failure never allocates
    std::map<std::pair<uint64_t, uint64_t>, fnn_hip_weight *> weights;  // (offset,size) like get_or_cache_packed
    std::vector<uint8_t> stage;
    uint8_t *scratch = nullptr;   // device copy of an input that overlaps its output
    uint64_t scratch_bytes = 0, scratch_epoch = 0;
    // Value ranges handed from the instruction that writes an f32 tensor to the quantised Conv2d that reads it
    // (range_io.h).  Tables are device memory kept per (plan, instruction); a live entry says that the bytes of
    // `slice` are exactly what the table describes, and lasts until something writes into the slice or the dispatch
    // pass ends.
    struct RangeTable { float *dev = nullptr; uint64_t images = 0; };
    // (tile_elems > 0: the pairs come in groups of tile_pairs, one group per tile_elems values of the slice, in order)
    struct LiveRange { fnn_slice slice; const float *table; int parts; uint64_t image_elems, images; uint64_t tile_elems = 0; int tile_pairs = 0; };
    // A one-image tensor that several instructions write part by part (producers that store straight into the slot of
    // a later Concat's result): each leaves its pairs behind those of the parts before it; the entry becomes a live
    // range once disjoint parts cover the whole slice, and is void as soon as anything else writes into it.
    struct PendingRange { fnn_slice slice; float *table; int parts; std::vector<fnn_slice> written; bool failed; uint64_t image_elems; };
    std::map<std::pair<uint64_t, uint64_t>, RangeTable> range_tables;
    std::vector<LiveRange> live_ranges;
    std::vector<PendingRange> pending_ranges;
};
constexpr int kRangeStride = 2048;   // pairs per image a table has room for

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

// resolve_params (src/backend/cpu/params.rs:11-39): with param_dims present the first `expected` parameters are the
// dims evaluated in the dispatch's shape environment (DimExpr::evaluate_with_env, src/ir/node.rs:511-531), else the
// stored params as they are.
int resolve_params(fnn_backend *b, const Instr &in, size_t expected, std::vector<uint64_t> &out)
{
    if (!in.has_param_dims) {
        out = in.params;
        return FNN_OK;
    }
    if (in.param_dims.size() < expected)
        return fail(b, FNN_ERR_DISPATCH, "resolve_params: param_dims has %zu elements but expected %zu", in.param_dims.size(), expected);
    out.clear();
    for (size_t i = 0; i < expected; i++) {
        const Instr::Dim &d = in.param_dims[i];
        if (d.kind == 0) { out.push_back(d.value); continue; }
        const uint64_t *bound = nullptr;
        for (const auto &kv : b->shape_env)
            if (kv.first == d.sym) { bound = &kv.second; break; }
        if (d.kind == 2) {
            if (bound && *bound > d.value)
                return fail(b, FNN_ERR_DISPATCH, "resolve_params: DimExpr::Bounded: symbol '%s' resolved to %llu, exceeds bound %llu",
                            d.sym.c_str(), (unsigned long long)*bound, (unsigned long long)d.value);
            out.push_back(bound ? *bound : d.value);
        } else {
            if (!bound) return fail(b, FNN_ERR_DISPATCH, "resolve_params: DimExpr::Symbol '%s' is not bound in the ShapeEnv", d.sym.c_str());
            out.push_back(*bound);
        }
    }
    return FNN_OK;
}

// M, K, N of a MatMul instruction when they do not depend on the dispatch's ShapeEnv: the stored params of an
// instruction without param_dims, or param_dims whose first three entries are all DimExpr::Known, which is what
// CpuBackend::compile emits for every MatMul of a static graph (src/backend/cpu/mod.rs:601-613) and what
// resolve_params would return under any environment.
bool static_mkn(const Instr &in, uint64_t *mkn)
{
    if (!in.has_param_dims) {
        if (in.params.size() < 3) return false;
        for (int i = 0; i < 3; i++) mkn[i] = in.params[i];
        return true;
    }
    if (in.param_dims.size() < 3) return false;
    for (int i = 0; i < 3; i++) {
        if (in.param_dims[i].kind != 0) return false;
        mkn[i] = in.param_dims[i].value;
    }
    return true;
}

int run_matmul(fnn_backend *b, const Instr &in, const KernelName &kn, int dtype)
{
    const char *name = in.kernel.c_str();
    if (in.inputs.size() < 2) return FNN_OK;  // the CPU arm ignores a malformed slice list
    std::vector<uint64_t> par;
    int rs = resolve_params(b, in, 3, par);
    if (rs) return rs;
    if (par.size() < 3) return fail(b, FNN_ERR_DISPATCH, "%s: expected params [M,K,N]", name);
    uint64_t m = par[0], k = par[1], n = par[2];
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
    std::vector<uint64_t> par;
    int rs = resolve_params(b, in, 3, par);
    if (rs) return rs;
    if (par.size() < 3) return fail(b, FNN_ERR_DISPATCH, "%s: expected params [M,K,N]", name);
    uint64_t m = par[0], k = par[1], n = par[2];
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
    if (in.inputs.empty()) return FNN_OK;
    const fnn_slice &xs = in.inputs[0];
    if (per_channel) {
        // params [numel, 1, nc, scale bits x nc, zero-point bits x nc] (src/backend/cpu/mod.rs:2335-2350)
        const uint64_t nc = in.params[2];
        if (nc > 0xffffffffull || in.params.size() < 3 + 2 * nc)
            return fail(b, FNN_ERR_DISPATCH, "quantize_activations: %llu channels need %llu params, the instruction has %llu",
                        (unsigned long long)nc, (unsigned long long)(3 + 2 * nc), (unsigned long long)in.params.size());
        std::vector<float> sc(nc), zp(nc);
        for (uint64_t c = 0; c < nc; c++) {
            const uint32_t sb = (uint32_t)in.params[3 + c], zb = (uint32_t)in.params[3 + nc + c];
            memcpy(&sc[c], &sb, 4);
            memcpy(&zp[c], &zb, 4);
        }
        return lift(b, fnn_hip_quantize_activations_per_channel(b->ctx, (const float *)(b->arena + xs.offset), xs.size / 4, numel, (uint32_t)nc,
                                                                sc.data(), zp.data(), b->arena + in.dst.offset, in.dst.size));
    }
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
    if (in.inputs.empty()) return FNN_OK;
    if (per_channel)   // (channel count, chunk and the scales come from the payload's header, as in the reference)
        return lift(b, fnn_hip_dequantize_activations_per_channel(b->ctx, b->arena + in.inputs[0].offset, in.inputs[0].size,
                                                                  (float *)(b->arena + in.dst.offset), in.dst.size / 4));
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
        std::vector<const float *> srcs;
        std::vector<uint64_t> widths, lens;
        for (const auto &s : in.inputs) {
            const uint64_t len = s.size / 4;
            if (len % outer) return fail(b, FNN_ERR_DISPATCH, "concat: input of %llu elements does not split into %llu outer positions", (unsigned long long)len, (unsigned long long)outer);
            srcs.push_back((const float *)(b->arena + s.offset));
            widths.push_back(len / outer);
            lens.push_back(len);
        }
        return lift(b, fnn_hip_concat_f32(b->ctx, out, pitch, out_len, srcs.size(), srcs.data(), widths.data(), lens.data(), in.params[2]));
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

// ---- value ranges between instructions -------------------------------------------------------------------------
// Geometry of a quantised Conv2d instruction that takes its activation ranges from a table: integer weights, one
// group (the range of a group's channels is not that of the image).
struct ConvInput { uint64_t image_elems, images; };
bool ranged_conv_input(const Instr &in, ConvInput *g)
{
    if (in.kind != K_CALL || in.inputs.size() < 2 || in.params.size() < 9 || !in.meta.present) return false;
    const KernelName kn = split_activation(in.kernel);
    if (kn.base != "conv2d_i8" && kn.base != "conv2d_i4") return false;
    if (!in.meta.codebook.empty() || in.params[3] != 1) return false;
    const uint64_t chw = in.params[4] * in.params[5] * in.params[6];
    if (chw == 0 || in.inputs[0].size % (chw * 4) != 0 || in.inputs[0].size == 0) return false;
    g->image_elems = chw;
    g->images = in.inputs[0].size / (chw * 4);
    return true;
}

// can the kernel behind this instruction leave ranges of what it writes?
bool leaves_ranges(const Instr &in)
{
    if (in.kind != K_CALL) return false;
    const std::string &n = in.kernel;
    if (n == "add_f32" || n == "relu_f32" || n == "gelu_f32" || n == "silu_f32" || n == "concat" || n == "slice_f32" ||
        n == "upsample_nearest2d")
        return true;
    if (n == "pool_f32") return in.params.size() == 8 && in.params[3] == 1;
    const KernelName kn = split_activation(n);
    return (kn.base == "conv2d_i8" || kn.base == "conv2d_i4") && in.meta.present && in.meta.codebook.empty();
}

// (`contributes_to`: the pending entry that the write into `s` adds its own pairs to, which it does not void)
void drop_ranges_overlapping(fnn_backend *b, const fnn_slice &s, int contributes_to = -1)
{
    if (!s.size) return;
    auto &v = b->live_ranges;
    v.erase(std::remove_if(v.begin(), v.end(), [&](const fnn_backend::LiveRange &r) { return overlaps(r.slice, s); }), v.end());
    for (size_t q = 0; q < b->pending_ranges.size(); q++)
        if ((int)q != contributes_to && overlaps(b->pending_ranges[q].slice, s)) b->pending_ranges[q].failed = true;
}

void clear_ranges(fnn_backend *b)
{
    b->live_ranges.clear();
    b->pending_ranges.clear();
}

// a device table of `images` x kRangeStride pairs under `key` (null: none can be had right now)
float *range_table(fnn_backend *b, fnn_plan *p, std::pair<uint64_t, uint64_t> key, uint64_t images)
{
    if (b->range_tables.size() > 1024 && !fnn_ctx_capturing(b->ctx)) {
        // plans come and go on a long-lived backend: the tables of the others are dropped (they get new
        // ones on their next pass)
        for (auto it = b->range_tables.begin(); it != b->range_tables.end();) {
            if (it->first.first == p->uid) { ++it; continue; }
            if (it->second.dev) fnn_hip_free(b->ctx, it->second.dev);
            it = b->range_tables.erase(it);
        }
        b->weights_epoch++;   // captured graphs may hold a dropped table
    }
    auto &t = b->range_tables[key];
    if (t.dev && t.images < images && !fnn_ctx_capturing(b->ctx)) {
        fnn_hip_free(b->ctx, t.dev);
        t.dev = nullptr;
        b->weights_epoch++;   // a captured graph may hold the old table
    }
    if (!t.dev && !fnn_ctx_capturing(b->ctx)) {
        void *d = nullptr;
        if (fnn_hip_malloc(b->ctx, (size_t)images * kRangeStride * 8, &d) == FNN_OK) { t.dev = (float *)d; t.images = images; }
    }
    return (t.dev && t.images >= images) ? t.dev : nullptr;
}

// If a later convolution of the plan reads what instruction `idx` writes (from the first byte of its output slice,
// before anything overwrites it), asks the next call on the context for the partial ranges that convolution
// needs; *covered = the convolution's input slice.  If a later convolution of ONE image reads a slice of which `idx`
// writes a part (the slot of a Concat result that its producers fill in place), the request is for the part, behind
// the pairs of the parts before it; *pending = the entry that collects them (-1: none).  The pairs of a part also
// serve a convolution that reads just that part (note_ranges), so this form goes first.
void request_ranges(fnn_backend *b, fnn_plan *p, size_t idx, fnn_slice *covered, int *pending)
{
    const Instr &in = p->instrs[idx];
    FnnRangeIo *rio = fnn_ctx_range_io(b->ctx);
    *pending = -1;
    if (!in.dst.size) return;
    size_t exact = (size_t)-1, whole = (size_t)-1;
    bool some = false;   // a convolution of one image reads some of what `idx` writes (one half of a Split that is a view)
    ConvInput ce{0, 0}, cw{0, 0};
    for (size_t j = idx + 1; j < p->instrs.size() && whole == (size_t)-1; j++) {
        const Instr &nx = p->instrs[j];
        ConvInput cj;
        if (ranged_conv_input(nx, &cj)) {
            const fnn_slice &cs = nx.inputs[0];
            if (exact == (size_t)-1 && cs.offset == in.dst.offset && cs.size <= in.dst.size && cj.images <= 65535) { exact = j; ce = cj; }
            if (cj.images == 1 && in.dst.size % 4 == 0 && in.dst.size < cs.size && in.dst.offset >= cs.offset &&
                in.dst.offset + in.dst.size <= cs.offset + cs.size) { whole = j; cw = cj; }
            if (cj.images == 1 && cs.size < in.dst.size && cs.offset >= in.dst.offset && cs.offset + cs.size <= in.dst.offset + in.dst.size) some = true;
        }
        if (overlaps(nx.dst, in.dst) || (nx.has_secondary && overlaps(nx.secondary, in.dst))) break;
    }
    // (a reader of the first bytes only is served like any reader of some of them)
    if (exact != (size_t)-1 && ce.images == 1 && ce.image_elems * 4 < in.dst.size) exact = (size_t)-1;
    if (whole != (size_t)-1 && (exact == (size_t)-1 || ce.images == 1)) {
        const fnn_slice &cs = p->instrs[whole].inputs[0];
        int at = -1;
        for (size_t q = 0; q < b->pending_ranges.size(); q++)
            if (b->pending_ranges[q].slice.offset == cs.offset && b->pending_ranges[q].slice.size == cs.size) at = (int)q;
        if (at < 0) {
            // (keyed by the consumer, apart from the producers' tables: bit 63)
            if (float *t = range_table(b, p, {p->uid, (uint64_t)whole | (1ull << 63)}, 1)) {
                b->pending_ranges.push_back(fnn_backend::PendingRange{cs, t, 0, {}, false, cw.image_elems});
                at = (int)b->pending_ranges.size() - 1;
            }
        }
        if (at >= 0) {
            auto &pr = b->pending_ranges[(size_t)at];
            for (const auto &w : pr.written)
                if (overlaps(w, in.dst)) pr.failed = true;   // a part written twice: the pairs of the first are stale
            if (!pr.failed && pr.parts < kRangeStride) {
                rio->out_table = pr.table; rio->out_stride = kRangeStride; rio->out_parts = pr.parts;
                rio->out_image_elems = in.dst.size / 4; rio->out_images = 1;
                *covered = in.dst;
                *pending = at;
                return;
            }
        }
    }
    if (exact != (size_t)-1) {
        if (float *t = range_table(b, p, {p->uid, idx}, ce.images)) {
            rio->out_table = t; rio->out_stride = kRangeStride;
            rio->out_image_elems = ce.image_elems; rio->out_images = ce.images;
            *covered = p->instrs[exact].inputs[0];
        }
    } else if (some && in.dst.size % 4 == 0) {
        // the whole result as one image: a producer that groups its pairs by channel block serves the readers of blocks
        if (float *t = range_table(b, p, {p->uid, idx}, 1)) {
            rio->out_table = t; rio->out_stride = kRangeStride;
            rio->out_image_elems = in.dst.size / 4; rio->out_images = 1;
            *covered = in.dst;
        }
    }
}

void note_ranges(fnn_backend *b, const fnn_slice &covered, int pending)
{
    FnnRangeIo *rio = fnn_ctx_range_io(b->ctx);
    if (pending >= 0 && (size_t)pending < b->pending_ranges.size()) {
        auto &pr = b->pending_ranges[(size_t)pending];
        if (!rio->out_table || rio->out_failed || rio->out_parts <= pr.parts) { pr.failed = true; return; }
        // the part's own pairs describe it to a convolution that reads just the part
        b->live_ranges.push_back(fnn_backend::LiveRange{covered, pr.table + 2 * (size_t)pr.parts, rio->out_parts - pr.parts, covered.size / 4, 1,
                                                        rio->out_tile_elems, rio->out_tile_pairs});
        pr.parts = rio->out_parts;
        pr.written.push_back(covered);
        uint64_t bytes = 0;
        for (const auto &w : pr.written) bytes += w.size;   // (disjoint: checked when each was requested)
        if (bytes == pr.slice.size) {
            b->live_ranges.push_back(fnn_backend::LiveRange{pr.slice, pr.table, pr.parts, pr.image_elems, 1});
            b->pending_ranges.erase(b->pending_ranges.begin() + pending);
        }
        return;
    }
    if (rio->out_table && rio->out_parts > 0 && !rio->out_failed)
        b->live_ranges.push_back(fnn_backend::LiveRange{covered, rio->out_table, rio->out_parts, rio->out_image_elems, rio->out_images,
                                                        rio->out_images == 1 ? rio->out_tile_elems : 0, rio->out_tile_pairs});
}

int run_call_with_ranges(fnn_backend *b, fnn_plan *p, size_t idx)
{
    Instr &in = p->instrs[idx];
    FnnRangeIo *rio = fnn_ctx_range_io(b->ctx);
    *rio = FnnRangeIo{};
    int64_t enabled = 1;
    fnn_hip_get_option(b->ctx, FNN_OPT_CONV_RANGES, &enabled);
    FnnResidualIo *res = fnn_ctx_residual_io(b->ctx);
    const bool for_sum = in.add_is_conv && res->residual != nullptr;
    if (!enabled) {
        if (for_sum) drop_ranges_overlapping(b, p->instrs[idx + 1].dst);
        return run_call(b, in);
    }
    // consumer: a convolution whose input slice is described by a live table
    ConvInput ci;
    if (ranged_conv_input(in, &ci)) {
        const fnn_slice &xs = in.inputs[0];
        for (const auto &r : b->live_ranges)
            if (r.slice.offset == xs.offset && r.slice.size == xs.size && r.image_elems == ci.image_elems && r.images == ci.images) {
                rio->in_table = r.table; rio->in_stride = kRangeStride; rio->in_parts = r.parts;
                break;
            }
        // ... or whole channel blocks of a one-image tensor whose producer grouped its pairs by channel block (one half
        // of a Split that is a view into the convolution output it splits)
        if (!rio->in_table && ci.images == 1)
            for (const auto &r : b->live_ranges) {
                const uint64_t tb = r.tile_elems * 4;
                if (r.images != 1 || tb == 0 || r.tile_pairs <= 0 || xs.offset < r.slice.offset || xs.offset + xs.size > r.slice.offset + r.slice.size) continue;
                const uint64_t at = xs.offset - r.slice.offset;
                if (at % tb || xs.size % tb || xs.size != ci.image_elems * 4) continue;
                const uint64_t t0 = at / tb, nt = xs.size / tb;
                if ((t0 + nt) * (uint64_t)r.tile_pairs > (uint64_t)r.parts) continue;
                rio->in_table = r.table + 2 * t0 * (uint64_t)r.tile_pairs; rio->in_stride = kRangeStride; rio->in_parts = (int)(nt * (uint64_t)r.tile_pairs);
                break;
            }
    }
    // producer: some later convolution reads exactly what this instruction writes, before anything overwrites it.  A
    // convolution that carries the Add behind it asks on the Add's behalf: a kernel that stores the sum leaves the
    // sum's ranges (one that does not leaves those of its own output, which are then of no use: the Add runs and
    // asks again)
    fnn_slice covered{0, 0};
    int pending = -1;
    if (for_sum) request_ranges(b, p, idx + 1, &covered, &pending);
    else if (leaves_ranges(in)) request_ranges(b, p, idx, &covered, &pending);
    drop_ranges_overlapping(b, in.dst, for_sum ? -1 : pending);
    if (in.has_secondary) drop_ranges_overlapping(b, in.secondary);
    if (for_sum) drop_ranges_overlapping(b, p->instrs[idx + 1].dst, pending);
    const int st = run_call(b, in);
    if (st == FNN_OK && rio->in_used) p->ranges_used++;
    // (a convolution that did not take the Add along has written nothing into the sum's slot: the Add runs next and
    // leaves the sum's pairs itself)
    if (st == FNN_OK && (!for_sum || res->used)) note_ranges(b, covered, pending);
    *rio = FnnRangeIo{};
    return st;
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
    // MatMul (or quantised Conv2d with integer weights) followed by an Add of its whole output and another tensor of
    // the same size: candidates for one call.  A MatMul not when a quantised Conv2d reads the sum (the Add then leaves
    // that convolution's activation ranges; a Conv2d that stores the sum leaves them itself); neither when the sum
    // overlaps the call's own output or any of its inputs (workgroups still read them while others store sums), or
    // partly overlaps the other operand.
    for (size_t i = 0; i + 1 < p->instrs.size(); i++) {
        Instr &mm = p->instrs[i];
        const Instr &ad = p->instrs[i + 1];
        mm.add_operand = -1;
        mm.add_is_conv = false;
        if (mm.kind != K_CALL || ad.kind != K_CALL || ad.kernel != "add_f32" || ad.inputs.size() != 2) continue;
        const KernelName kn = split_activation(mm.kernel);
        uint64_t mkn[3];
        uint64_t bytes = 0;
        const bool is_conv = (kn.base == "conv2d_i8" || kn.base == "conv2d_i4") && mm.meta.present && mm.meta.codebook.empty();
        if (is_conv) bytes = mm.dst.size;
        else if (matmul_dtype(kn.base) >= 0 && static_mkn(mm, mkn)) bytes = mkn[0] * mkn[2] * 4;
        else continue;
        if (bytes == 0 || mm.dst.size != bytes || ad.dst.size != bytes) continue;
        int other = -1;
        for (int k = 0; k < 2; k++)
            if (ad.inputs[k].offset == mm.dst.offset && ad.inputs[k].size == bytes && ad.inputs[1 - k].size == bytes) other = 1 - k;
        if (other < 0) continue;
        const fnn_slice &res = ad.inputs[other];
        if (overlaps(res, mm.dst) || overlaps(ad.dst, mm.dst)) continue;
        if (overlaps(ad.dst, res) && ad.dst.offset != res.offset) continue;
        if (ad.dst.offset % 4 || res.offset % 4) continue;
        bool reads_sum_slot = false;
        for (const auto &mi : mm.inputs) reads_sum_slot = reads_sum_slot || overlaps(mi, ad.dst);
        if (reads_sum_slot) continue;
        bool feeds_conv = false;
        for (size_t j = i + 2; j < p->instrs.size() && !feeds_conv && !is_conv; j++) {
            ConvInput cj;
            feeds_conv = ranged_conv_input(p->instrs[j], &cj) && overlaps(p->instrs[j].inputs[0], ad.dst);
        }
        if (!feeds_conv) { mm.add_operand = other; mm.add_is_conv = is_conv; }
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

int run_instr(fnn_backend *b, fnn_plan *p, size_t idx, bool consts_resident)
{
    Instr &in = p->instrs[idx];
    if (idx == p->add_done) {   // the call before this Add has stored the sum already
        p->add_done = (size_t)-1;
        // (a convolution dropped the stale ranges of the sum's slot before it ran and may have noted the sum's own)
        if (!p->instrs[idx - 1].add_is_conv) drop_ranges_overlapping(b, in.dst);
        return FNN_OK;
    }
    p->add_done = (size_t)-1;
    const bool offered_here = p->prep_ready == idx;   // the call before this one prepared this MatMul's operand
    p->prep_ready = (size_t)-1;
    if (in.kind != K_CALL && in.kind != K_MEMCOPY) drop_ranges_overlapping(b, in.kind == K_WRITE_CONST ? fnn_slice{in.dst.offset, in.data.size()} : in.dst);
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
        // a copy that feeds a quantised Conv2d (a Split of a one-image batch) runs as a kernel that leaves the ranges
        FnnRangeIo *rio = fnn_ctx_range_io(b->ctx);
        *rio = FnnRangeIo{};
        int64_t ranges_on = 1;
        fnn_hip_get_option(b->ctx, FNN_OPT_CONV_RANGES, &ranges_on);
        fnn_slice covered{0, 0};
        int pending = -1;
        if (ranges_on && n == in.dst.size && n % 4 == 0 && d.offset % 4 == 0 && s.offset % 4 == 0) request_ranges(b, p, idx, &covered, &pending);
        drop_ranges_overlapping(b, in.dst, pending);
        if (rio->out_table && covered.size == n) {
            const uint64_t per = rio->out_image_elems, imgs = rio->out_images;
            int st = lift(b, fnn_hip_copy2d_f32(b->ctx, (float *)(b->arena + d.offset), per, n / 4, (const float *)(b->arena + s.offset), per, n / 4, per, imgs));
            if (st == FNN_OK) note_ranges(b, covered, pending);
            *rio = FnnRangeIo{};
            return st;
        }
        *rio = FnnRangeIo{};
        return lift(b, fnn_hip_copy(b->ctx, b->arena + d.offset, b->arena + s.offset, n));
    }
    case K_CALL: {
        int64_t fuse = 1, hand = 1;
        fnn_hip_get_option(b->ctx, FNN_OPT_FUSE_RESIDUAL, &fuse);
        fnn_hip_get_option(b->ctx, FNN_OPT_FUSE_PREP, &hand);
        // the Add behind this MatMul (Conv2d) rides along: the call's last kernel stores the sum too where it can
        bool with_res = in.add_operand >= 0 && fuse && idx + 1 < p->instrs.size();
        if (with_res) {
            const Instr &ad = p->instrs[idx + 1];
            with_res = in_arena(b, ad.inputs[in.add_operand]) && in_arena(b, ad.dst);   // (else the Add reports it)
        }
        FnnResidualIo *res = fnn_ctx_residual_io(b->ctx);
        *res = FnnResidualIo{};
        if (with_res) {
            const Instr &ad = p->instrs[idx + 1];
            res->residual = (const float *)(b->arena + ad.inputs[in.add_operand].offset);
            res->sum_out = (float *)(b->arena + ad.dst.offset);
            res->of_out = (const float *)(b->arena + in.dst.offset);
            res->elems = in.dst.size / 4;
        }
        // ... and when the next call on the context is the MatMul that reads this one's result (or that sum), this
        // call's reduction prepares its operand
        FnnPrepIo *pio = fnn_ctx_prep_io(b->ctx);
        *pio = FnnPrepIo{};
        size_t consumer = (size_t)-1;
        const KernelName kn = split_activation(in.kernel);
        uint64_t mkn[3] = {0, 0, 0}, nmkn[3] = {0, 0, 0};
        const bool plain_matmul = matmul_dtype(kn.base) >= 0 && static_mkn(in, mkn) && in.meta.codebook.empty();
        if (hand && plain_matmul) {
            pio->offered = offered_here ? 1 : 0;
            const size_t j = idx + (with_res ? 2 : 1);
            const uint64_t m = mkn[0], n = mkn[2];
            const fnn_slice &feeds = with_res ? p->instrs[idx + 1].dst : in.dst;
            if (j < p->instrs.size() && in.dst.size == m * n * 4) {
                const Instr &nx = p->instrs[j];
                const KernelName kx = nx.kind == K_CALL ? split_activation(nx.kernel) : KernelName{};
                const int dx = nx.kind == K_CALL ? matmul_dtype(kx.base) : -1;
                if (dx >= 0 && static_mkn(nx, nmkn) && nx.inputs.size() >= 2 && nx.meta.codebook.empty() &&
                    nmkn[0] == m && nmkn[1] == n && nx.inputs[0].offset == feeds.offset && nx.inputs[0].size == m * n * 4 &&
                    in_arena(b, nx.inputs[0]) && in_arena(b, nx.inputs[1])) {
                    fnn_hip_weight *wn = nullptr;
                    if (weight_for(b, nx.inputs[1], dx, nx.meta, nmkn[2], nmkn[1], nx.kernel.c_str(), &wn) == FNN_OK && wn) {
                        pio->next_w = wn;
                        pio->next_flags = FNN_FLAG_DEVICE_PTRS | b->kernel_flags;
                        pio->next_a = (const float *)(b->arena + feeds.offset);
                        consumer = j;
                    }
                }
            }
        }
        const int st = run_call_with_ranges(b, p, idx);
        if (st == FNN_OK && res->used) {
            p->add_done = idx + 1;
            p->residuals_fused++;
        }
        if (st == FNN_OK && pio->consumed) p->operands_handed++;
        if (st == FNN_OK && pio->produced && consumer != (size_t)-1 && (consumer == idx + 1 || p->add_done == idx + 1)) p->prep_ready = consumer;
        *res = FnnResidualIo{};
        *pio = FnnPrepIo{};
        return st;
    }
    }
    return FNN_OK;
}

// first / stopped_at: a caller that runs unsupported kernels elsewhere dispatches in segments.  With stopped_at given,
// an instruction that returns FNN_ERR_UNSUPPORTED_OP ends the segment (index in *stopped_at, nothing of it has run)
// and the caller resumes at the next index; a plan that ever stopped this way is not replayed as a graph.
int dispatch_impl(fnn_backend *b, fnn_plan *p, uint64_t *elapsed_ns, uint64_t n_elapsed, uint64_t first = 0, uint64_t *stopped_at = nullptr)
{
    if (!b || !p) return fail(b, FNN_ERR_DISPATCH, "dispatch: NULL argument");
    if (first > p->instrs.size()) return fail(b, FNN_ERR_DISPATCH, "dispatch: first instruction %llu of %zu", (unsigned long long)first, p->instrs.size());
    if (!b->arena) return fail(b, FNN_ERR_MEMORY, "dispatch: no arena allocated");
    if (p->arena_size > b->arena_bytes) return fail(b, FNN_ERR_MEMORY, "dispatch: plan needs an arena of %llu bytes, backend holds %llu", (unsigned long long)p->arena_size, (unsigned long long)b->arena_bytes);
    if (elapsed_ns && n_elapsed < p->instrs.size()) return fail(b, FNN_ERR_DISPATCH, "dispatch_profile: room for %llu timings, plan has %llu instructions", (unsigned long long)n_elapsed, (unsigned long long)p->instrs.size());
    if (!p->analysed) analyse(p);
    bool resident = p->resident_uid == b->uid && p->resident_generation == b->generation;
    if (first > 0) resident = p->segment_resident;   // later segment of one pass: as the first segment found it
    else if (resident && p->resident_seq != b->write_seq) {
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
    if (first == 0) p->segment_resident = resident;
    const bool may_replay = b->graph_replay && !elapsed_ns && first == 0 && !p->has_unsupported && resident && !p->uploads_every_run && p->graph_failures < 2;
    if (p->graph && !(may_replay && p->graph_env == b->shape_env_sig && p->graph_uid == b->uid && p->graph_generation == b->generation &&
                      p->graph_weights_epoch == b->weights_epoch && p->graph_ws_epoch == fnn_hip_workspace_epoch(b->ctx) &&
                      p->graph_scratch_epoch == b->scratch_epoch)) {
        fnn_hip_graph_destroy(p->graph_uid == b->uid ? b->ctx : nullptr, p->graph);
        p->graph = nullptr;
    }
    if (may_replay && !p->graph) {
        const uint64_t w0 = b->weights_epoch, s0 = fnn_hip_workspace_epoch(b->ctx), c0 = b->scratch_epoch;
        if (fnn_hip_graph_begin(b->ctx) == FNN_OK) {
            int st = FNN_OK;
            clear_ranges(b);
            p->ranges_used = 0;
            p->residuals_fused = 0;
            p->operands_handed = 0;
            p->add_done = (size_t)-1;
            p->prep_ready = (size_t)-1;
            for (size_t i = 0; i < p->instrs.size() && st == FNN_OK; i++) st = run_instr(b, p, i, true);
            clear_ranges(b);
            fnn_hip_graph *g = nullptr;
            int en = fnn_hip_graph_end(b->ctx, &g);
            if (st == FNN_OK && en == FNN_OK && g && w0 == b->weights_epoch && s0 == fnn_hip_workspace_epoch(b->ctx) && c0 == b->scratch_epoch) {
                p->graph = g;
                p->graph_uid = b->uid; p->graph_generation = b->generation;
                p->graph_weights_epoch = w0; p->graph_ws_epoch = s0; p->graph_scratch_epoch = c0;
                p->graph_env = b->shape_env_sig;
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

    clear_ranges(b);   // ranges never outlive a pass: between passes anyone may write into the arena
    if (first == 0) { p->ranges_used = 0; p->residuals_fused = 0; p->operands_handed = 0; }
    p->add_done = (size_t)-1;
    p->prep_ready = (size_t)-1;
    for (size_t i = (size_t)first; i < p->instrs.size(); i++) {
        auto t0 = std::chrono::steady_clock::now();
        int st = run_instr(b, p, i, resident);
        if (st == FNN_OK && elapsed_ns) st = lift(b, fnn_hip_sync(b->ctx));
        if (st == FNN_ERR_UNSUPPORTED_OP && stopped_at) {
            // the caller runs this instruction itself and comes back with first = i + 1
            fnn_hip_sync(b->ctx);
            *stopped_at = i;
            p->has_unsupported = true;
            if (b->last_plan_uid != p->uid || b->last_plan_revision != p->revision) {
                b->write_seq++;
                for (const auto &r : p->writes) log_write(b, r);
                b->last_plan_uid = p->uid;
                b->last_plan_revision = p->revision;
            }
            return st;
        }
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
    for (auto &t : b->range_tables)
        if (t.second.dev) fnn_hip_free(b->ctx, t.second.dev);
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

uint64_t fnn_plan_ranges_used(const fnn_plan *p) { return p ? p->ranges_used : 0; }
uint64_t fnn_plan_residuals_fused(const fnn_plan *p) { return p ? p->residuals_fused : 0; }
uint64_t fnn_plan_operands_handed(const fnn_plan *p) { return p ? p->operands_handed : 0; }

static void touched(fnn_plan *p)
{
    p->analysed = false;
    p->has_unsupported = false;
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
            if (meta->n_codebooks >= 1) in.meta.codebook.assign(meta->codebooks, meta->codebooks + 16 * meta->n_codebooks);
        }
        p->instrs.push_back(std::move(in));
        touched(p);
        return FNN_OK;
    });
}

int fnn_plan_set_param_dims(fnn_plan *p, uint64_t instruction, const fnn_dim_expr *dims, uint64_t n_dims)
{
    return guarded(nullptr, "fnn_plan_set_param_dims", [&]() -> int {
        if (!p || (!dims && n_dims)) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_set_param_dims: NULL argument");
        if (instruction >= p->instrs.size() || p->instrs[instruction].kind != K_CALL)
            return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_set_param_dims: instruction %llu is not a CallKernel", (unsigned long long)instruction);
        std::vector<Instr::Dim> v;
        for (uint64_t i = 0; i < n_dims; i++) {
            Instr::Dim d;
            d.kind = dims[i].kind;
            d.value = dims[i].value;
            if (d.kind > 2) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_set_param_dims: unknown DimExpr kind %u", d.kind);
            if (d.kind != 0) {
                if (!dims[i].symbol) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_set_param_dims: symbolic dim without a name");
                d.sym = dims[i].symbol;
            }
            v.push_back(std::move(d));
        }
        p->instrs[instruction].param_dims = std::move(v);
        p->instrs[instruction].has_param_dims = true;
        touched(p);
        return FNN_OK;
    });
}

static int set_shape_env(fnn_backend *b, const char *const *names, const uint64_t *values, uint64_t n)
{
    b->shape_env.clear();
    b->shape_env_sig.clear();
    for (uint64_t i = 0; i < n; i++) {
        if (!names[i]) return fail(b, FNN_ERR_DISPATCH, "dispatch: NULL symbol name in the shape environment");
        for (const auto &kv : b->shape_env)   // ShapeEnv::bind: one value per symbol
            if (kv.first == names[i] && kv.second != values[i])
                return fail(b, FNN_ERR_DISPATCH, "ShapeEnv: symbol '%s' bound to %llu then inconsistently to %llu", names[i],
                            (unsigned long long)kv.second, (unsigned long long)values[i]);
        b->shape_env.emplace_back(names[i], values[i]);
        b->shape_env_sig += names[i];
        b->shape_env_sig += '=';
        b->shape_env_sig += std::to_string(values[i]);
        b->shape_env_sig += ';';
    }
    return FNN_OK;
}

int fnn_backend_dispatch(fnn_backend *b, fnn_plan *p)
{
    return guarded(b, "fnn_backend_dispatch", [&]() -> int {
        if (b) { b->shape_env.clear(); b->shape_env_sig.clear(); }
        return dispatch_impl(b, p, nullptr, 0);
    });
}

int fnn_backend_dispatch_from(fnn_backend *b, fnn_plan *p, const char *const *names, const uint64_t *values, uint64_t n_symbols,
                              uint64_t first, uint64_t *stopped_at)
{
    return guarded(b, "fnn_backend_dispatch_from", [&]() -> int {
        if (!b || !stopped_at) return fail(b, FNN_ERR_DISPATCH, "dispatch: NULL argument");
        if ((!names || !values) && n_symbols) return fail(b, FNN_ERR_DISPATCH, "dispatch: NULL shape environment");
        int st = set_shape_env(b, names, values, n_symbols);
        if (st) return st;
        *stopped_at = p ? p->instrs.size() : 0;
        return dispatch_impl(b, p, nullptr, 0, first, stopped_at);
    });
}

int fnn_backend_dispatch_env(fnn_backend *b, fnn_plan *p, const char *const *names, const uint64_t *values, uint64_t n_symbols)
{
    return guarded(b, "fnn_backend_dispatch_env", [&]() -> int {
        if (!b) return fail(nullptr, FNN_ERR_DISPATCH, "dispatch: NULL argument");
        if ((!names || !values) && n_symbols) return fail(b, FNN_ERR_DISPATCH, "dispatch: NULL shape environment");
        int st = set_shape_env(b, names, values, n_symbols);
        if (st) return st;
        return dispatch_impl(b, p, nullptr, 0);
    });
}

// ---- ExecutablePlan::save / load (src/backend/mod.rs:117-131): bincode 1.3 with its default options, i.e. little
// endian, fixed-width integers (usize and u64 as 8 bytes, enum variant index as u32), sequence and string lengths as
// u64, Option as one tag byte, f32 as 4 bytes, fixed-size arrays without a length, Arc<T> as T.
namespace {

struct Reader {
    const uint8_t *p;
    uint64_t left;
    bool ok = true;
    bool take(void *dst, uint64_t n)
    {
        if (!ok || n > left) { ok = false; return false; }
        memcpy(dst, p, n);
        p += n;
        left -= n;
        return true;
    }
    uint64_t u64() { uint64_t v = 0; take(&v, 8); return v; }
    uint32_t u32() { uint32_t v = 0; take(&v, 4); return v; }
    uint8_t u8() { uint8_t v = 0; take(&v, 1); return v; }
    float f32() { float v = 0; take(&v, 4); return v; }
    // a length that the remaining bytes can hold at `elem` bytes per element (refuses absurd lengths before allocating)
    uint64_t len(uint64_t elem)
    {
        const uint64_t n = u64();
        if (ok && elem && n > left / elem) ok = false;
        return ok ? n : 0;
    }
    std::string str()
    {
        const uint64_t n = len(1);
        std::string s((size_t)n, '\0');
        if (n) take(&s[0], n);
        return s;
    }
    fnn_slice slice() { fnn_slice s; s.offset = u64(); s.size = u64(); return s; }
};

struct Writer {
    std::vector<uint8_t> out;
    void put(const void *src, size_t n) { const uint8_t *b = (const uint8_t *)src; out.insert(out.end(), b, b + n); }
    void u64(uint64_t v) { put(&v, 8); }
    void u32(uint32_t v) { put(&v, 4); }
    void u8(uint8_t v) { put(&v, 1); }
    void f32(float v) { put(&v, 4); }
    void str(const std::string &s) { u64(s.size()); put(s.data(), s.size()); }
    void slice(const fnn_slice &s) { u64(s.offset); u64(s.size); }
};

}  // namespace

int fnn_plan_from_bincode(const void *bytes, uint64_t len, fnn_plan **out)
{
    return guarded(nullptr, "fnn_plan_from_bincode", [&]() -> int {
        if (!out || (!bytes && len)) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_from_bincode: NULL argument");
        *out = nullptr;
        Reader r{(const uint8_t *)bytes, len};
        fnn_plan *p = nullptr;
        int st = fnn_plan_create(0, &p);
        if (st) return st;
        auto bad = [&](const char *what, uint64_t index) {
            const uint64_t at = len - r.left;
            fnn_plan_destroy(p);
            return fail(nullptr, FNN_ERR_COMPILATION, "fnn_plan_from_bincode: %s (instruction %llu, byte %llu of %llu)", what,
                        (unsigned long long)index, (unsigned long long)at, (unsigned long long)len);
        };
        // ExecutablePlan { instructions: Vec<Instruction>, arena_size: usize, levels: Vec<usize> }
        const uint64_t n_instr = r.len(4);
        for (uint64_t i = 0; i < n_instr; i++) {
            Instr in;
            const uint32_t variant = r.u32();   // enum Instruction { CallKernel, MemCopy, Fill, WriteConst }
            if (!r.ok) return bad("truncated", i);
            switch (variant) {
            case 0: {
                in.kind = K_CALL;
                in.kernel = r.str();                                  // kernel_name: String
                const uint64_t n_in = r.len(16);                      // input_slices: Vec<BufferSlice>
                for (uint64_t k = 0; k < n_in; k++) in.inputs.push_back(r.slice());
                in.dst = r.slice();                                   // output_slice: BufferSlice
                const uint8_t has_sec = r.u8();                       // secondary_output_slice: Option<BufferSlice>
                if (has_sec > 1) return bad("Option tag is neither 0 nor 1 (secondary_output_slice)", i);
                if (has_sec) { in.has_secondary = true; in.secondary = r.slice(); }
                const uint64_t n_par = r.len(8);                      // params: Vec<usize>
                for (uint64_t k = 0; k < n_par; k++) in.params.push_back(r.u64());
                const uint8_t has_node = r.u8();                      // node_id: Option<NodeId = usize>
                if (has_node > 1) return bad("Option tag is neither 0 nor 1 (node_id)", i);
                if (has_node) { in.has_node_id = true; in.node_id = r.u64(); }
                const uint8_t has_dims = r.u8();                      // param_dims: Option<Vec<DimExpr>>
                if (has_dims > 1) return bad("Option tag is neither 0 nor 1 (param_dims)", i);
                if (has_dims) {
                    in.has_param_dims = true;
                    const uint64_t n_d = r.len(4);
                    for (uint64_t k = 0; k < n_d && r.ok; k++) {
                        Instr::Dim d;
                        d.kind = r.u32();                             // enum DimExpr { Known(u64), Symbol(String), Bounded { sym, max } }
                        if (d.kind == 0) d.value = r.u64();
                        else if (d.kind == 1) d.sym = r.str();
                        else if (d.kind == 2) { d.sym = r.str(); d.value = r.u64(); }
                        else return bad("unknown DimExpr variant", i);
                        in.param_dims.push_back(std::move(d));
                    }
                }
                const uint8_t has_meta = r.u8();                      // weight_meta: Option<Arc<QuantizedWeightMeta>>
                if (has_meta > 1) return bad("Option tag is neither 0 nor 1 (weight_meta)", i);
                if (has_meta) {
                    in.meta.present = true;
                    in.meta.bit_width = r.u64();                      // bit_width: usize
                    const uint64_t n_sc = r.len(4);                   // scales: Vec<f32>
                    for (uint64_t k = 0; k < n_sc; k++) in.meta.scales.push_back(r.f32());
                    const uint64_t n_zp = r.len(4);                   // zero_points: Vec<f32>
                    for (uint64_t k = 0; k < n_zp; k++) in.meta.zeros.push_back(r.f32());
                    const uint64_t n_sh = r.len(8);                   // shape: Vec<usize>
                    for (uint64_t k = 0; k < n_sh; k++) in.meta.shape.push_back(r.u64());
                    in.meta.qblock = r.u64();                         // quant_block_size: usize
                    const uint64_t n_cb = r.len(64);                  // codebooks: Vec<[f32; 16]>
                    for (uint64_t k = 0; k < n_cb * 16; k++) in.meta.codebook.push_back(r.f32());
                }
                break;
            }
            case 1: in.kind = K_MEMCOPY; in.dst = r.slice(); in.src = r.slice(); break;    // MemCopy { dst, src }
            case 2: in.kind = K_FILL; in.dst = r.slice(); in.value = r.f32(); break;        // Fill { dst, value: f32 }
            case 3: {                                                                       // WriteConst { dst, data: Vec<u8> }
                in.kind = K_WRITE_CONST;
                in.dst = r.slice();
                const uint64_t n = r.len(1);
                in.data.resize((size_t)n);
                if (n) r.take(in.data.data(), n);
                in.dst.size = in.data.size();   // the dispatcher copies data.len() bytes to dst.offset (src/backend/cpu/mod.rs:7111-7121)
                break;
            }
            default: return bad("unknown Instruction variant", i);
            }
            if (!r.ok) return bad("truncated", i);
            p->instrs.push_back(std::move(in));
        }
        p->arena_size = r.u64();
        const uint64_t n_lv = r.len(8);
        for (uint64_t k = 0; k < n_lv; k++) p->levels.push_back(r.u64());
        if (!r.ok) return bad("truncated after the instructions", n_instr);
        if (r.left) return bad("trailing bytes", n_instr);
        touched(p);
        *out = p;
        return FNN_OK;
    });
}

int fnn_plan_to_bincode(const fnn_plan *p, void *buf, uint64_t cap, uint64_t *needed)
{
    return guarded(nullptr, "fnn_plan_to_bincode", [&]() -> int {
        if (!p || !needed) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_to_bincode: NULL argument");
        Writer w;
        w.u64(p->instrs.size());
        for (const Instr &in : p->instrs) {
            switch (in.kind) {
            case K_CALL:
                w.u32(0);
                w.str(in.kernel);
                w.u64(in.inputs.size());
                for (const auto &s : in.inputs) w.slice(s);
                w.slice(in.dst);
                w.u8(in.has_secondary ? 1 : 0);
                if (in.has_secondary) w.slice(in.secondary);
                w.u64(in.params.size());
                for (uint64_t v : in.params) w.u64(v);
                w.u8(in.has_node_id ? 1 : 0);
                if (in.has_node_id) w.u64(in.node_id);
                w.u8(in.has_param_dims ? 1 : 0);
                if (in.has_param_dims) {
                    w.u64(in.param_dims.size());
                    for (const auto &d : in.param_dims) {
                        w.u32(d.kind);
                        if (d.kind == 0) w.u64(d.value);
                        else if (d.kind == 1) w.str(d.sym);
                        else { w.str(d.sym); w.u64(d.value); }
                    }
                }
                w.u8(in.meta.present ? 1 : 0);
                if (in.meta.present) {
                    w.u64(in.meta.bit_width);
                    w.u64(in.meta.scales.size());
                    for (float v : in.meta.scales) w.f32(v);
                    w.u64(in.meta.zeros.size());
                    for (float v : in.meta.zeros) w.f32(v);
                    w.u64(in.meta.shape.size());
                    for (uint64_t v : in.meta.shape) w.u64(v);
                    w.u64(in.meta.qblock);
                    w.u64(in.meta.codebook.size() / 16);
                    for (float v : in.meta.codebook) w.f32(v);
                }
                break;
            case K_MEMCOPY: w.u32(1); w.slice(in.dst); w.slice(in.src); break;
            case K_FILL: w.u32(2); w.slice(in.dst); w.f32(in.value); break;
            case K_WRITE_CONST:
                w.u32(3);
                w.slice(in.dst);
                w.u64(in.data.size());
                w.put(in.data.data(), in.data.size());
                break;
            }
        }
        w.u64(p->arena_size);
        // levels: as loaded; a plan built through fnn_plan_add_* is sequential (level i for instruction i)
        if (p->levels.size() == p->instrs.size()) {
            w.u64(p->levels.size());
            for (uint64_t v : p->levels) w.u64(v);
        } else {
            w.u64(p->instrs.size());
            for (uint64_t i = 0; i < p->instrs.size(); i++) w.u64(i);
        }
        *needed = w.out.size();
        if (buf && cap >= w.out.size()) memcpy(buf, w.out.data(), w.out.size());
        else if (buf) return fail(nullptr, FNN_ERR_MEMORY, "fnn_plan_to_bincode: buffer of %llu bytes, plan needs %llu", (unsigned long long)cap, (unsigned long long)w.out.size());
        return FNN_OK;
    });
}

uint64_t fnn_plan_arena_size(const fnn_plan *p) { return p ? p->arena_size : 0; }

int fnn_plan_describe(const fnn_plan *p, uint64_t instruction, char *buf, uint64_t cap)
{
    return guarded(nullptr, "fnn_plan_describe", [&]() -> int {
        if (!p || !buf || cap == 0) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_describe: NULL argument");
        if (instruction >= p->instrs.size()) return fail(nullptr, FNN_ERR_DISPATCH, "fnn_plan_describe: instruction %llu of %zu", (unsigned long long)instruction, p->instrs.size());
        const Instr &in = p->instrs[instruction];
        std::string s;
        auto sl = [](const fnn_slice &x) { return "[" + std::to_string(x.offset) + "," + std::to_string(x.size) + "]"; };
        switch (in.kind) {
        case K_WRITE_CONST: s = "{\"op\":\"WriteConst\",\"dst\":" + sl(in.dst) + ",\"len\":" + std::to_string(in.data.size()) + "}"; break;
        case K_FILL: {
            char v[64];
            snprintf(v, sizeof v, "%.9g", (double)in.value);
            s = "{\"op\":\"Fill\",\"dst\":" + sl(in.dst) + ",\"value\":" + v + "}";
            break;
        }
        case K_MEMCOPY: s = "{\"op\":\"MemCopy\",\"dst\":" + sl(in.dst) + ",\"src\":" + sl(in.src) + "}"; break;
        case K_CALL: {
            s = "{\"op\":\"CallKernel\",\"kernel\":\"" + in.kernel + "\",\"inputs\":[";
            for (size_t i = 0; i < in.inputs.size(); i++) s += (i ? "," : "") + sl(in.inputs[i]);
            s += "],\"output\":" + sl(in.dst);
            s += ",\"secondary\":" + (in.has_secondary ? sl(in.secondary) : std::string("null"));
            s += ",\"params\":[";
            for (size_t i = 0; i < in.params.size(); i++) s += (i ? "," : "") + std::to_string(in.params[i]);
            s += "],\"node_id\":" + (in.has_node_id ? std::to_string(in.node_id) : std::string("null"));
            s += ",\"param_dims\":";
            if (!in.has_param_dims) s += "null";
            else {
                s += "[";
                for (size_t i = 0; i < in.param_dims.size(); i++) {
                    const auto &d = in.param_dims[i];
                    s += i ? "," : "";
                    if (d.kind == 0) s += std::to_string(d.value);
                    else if (d.kind == 1) s += "\"" + d.sym + "\"";
                    else s += "{\"sym\":\"" + d.sym + "\",\"max\":" + std::to_string(d.value) + "}";
                }
                s += "]";
            }
            s += ",\"meta\":";
            if (!in.meta.present) s += "null";
            else {
                s += "{\"bit_width\":" + std::to_string(in.meta.bit_width) + ",\"n_scales\":" + std::to_string(in.meta.scales.size()) +
                     ",\"n_zero_points\":" + std::to_string(in.meta.zeros.size()) + ",\"shape\":[";
                for (size_t i = 0; i < in.meta.shape.size(); i++) s += (i ? "," : "") + std::to_string(in.meta.shape[i]);
                s += "],\"quant_block_size\":" + std::to_string(in.meta.qblock) + ",\"n_codebooks\":" + std::to_string(in.meta.codebook.size() / 16) + "}";
            }
            s += "}";
            break;
        }
        }
        if (s.size() + 1 > cap) return fail(nullptr, FNN_ERR_MEMORY, "fnn_plan_describe: needs %zu bytes", s.size() + 1);
        memcpy(buf, s.c_str(), s.size() + 1);
        return FNN_OK;
    });
}

int fnn_backend_dispatch_profile(fnn_backend *b, fnn_plan *p, uint64_t *elapsed_ns, uint64_t n)
{
    return guarded(b, "fnn_backend_dispatch_profile", [&]() -> int {
        if (!elapsed_ns) return fail(b, FNN_ERR_DISPATCH, "dispatch_profile: NULL timings");
        if (b) { b->shape_env.clear(); b->shape_env_sig.clear(); }   // an empty ShapeEnv, not the previous dispatch's
        return dispatch_impl(b, p, elapsed_ns, n);
    });
}

int fnn_backend_dispatch_profile_env(fnn_backend *b, fnn_plan *p, const char *const *names, const uint64_t *values, uint64_t n_symbols,
                                     uint64_t *elapsed_ns, uint64_t n)
{
    return guarded(b, "fnn_backend_dispatch_profile_env", [&]() -> int {
        if (!b) return fail(nullptr, FNN_ERR_DISPATCH, "dispatch_profile: NULL argument");
        if (!elapsed_ns) return fail(b, FNN_ERR_DISPATCH, "dispatch_profile: NULL timings");
        if ((!names || !values) && n_symbols) return fail(b, FNN_ERR_DISPATCH, "dispatch_profile: NULL shape environment");
        int st = set_shape_env(b, names, values, n_symbols);
        if (st) return st;
        return dispatch_impl(b, p, elapsed_ns, n);
    });
}

}  // extern "C"
