// Host side of the one-launch streaming MatMul for up to 32 activation rows (kernels: qgemm_stream_impl.h, one
// translation unit per weight type): which calls it takes, the shape of the launch, the split-K workspace.
#include "mfma.h"
#include "qgemm_stream.h"
#include "range_io.h"

namespace {

// RT, KR, splits and rounds from FNN_OPT_STREAM_SHAPE or by rule (MB follows from M).  The phases of a round (requests,
// conversion, matrix cores) follow one another inside a workgroup, so a workgroup does one round where it can: one row
// tile per wave, K / KR splits, and KR = 512 while that still gives the 256 CUs a workgroup each.
bool plan_stream(int bits, int max_tiles, int max_mb, int64_t m, int64_t n, int64_t k, int64_t forced, StreamPlan *out)
{
    const int mb = (int)((m + 15) / 16);
    if (mb < 1 || mb > max_mb) return false;
    int rt = 1, kr = 512;
    const int64_t nt1 = (n + FNN_STREAM_NW * 16 - 1) / (FNN_STREAM_NW * 16);
    if (nt1 * ((k + 511) / 512) < 224) kr = 256;
    int64_t splits = 0;
    if (forced > 0) {
        rt = (int)((forced >> 4) & 15);
        kr = (int)(forced & 15) * 256;
        splits = forced >> 8;
        if (rt < 1 || rt > 2 || (kr != 256 && kr != 512)) return false;
    }
    if (mb * rt > max_tiles) return false;   // accumulator tiles that fit the registers
    const int64_t kr_total = (k + kr - 1) / kr;   // rounds over all of K
    if (splits == 0) splits = kr_total > 64 ? 64 : kr_total;
    if (splits > kr_total || splits > 64) return false;
    const int64_t rounds = (kr_total + splits - 1) / splits;
    if ((splits - 1) * rounds >= kr_total) return false;   // an empty split
    const int64_t ntiles = (n + FNN_STREAM_NW * rt * 16 - 1) / (FNN_STREAM_NW * rt * 16);
    // By rule the kernel takes a call only where it measured faster than preparation + tiles + reduction as three
    // launches: no more workgroups than the chip holds at once (a second wave of
    // workgroups repeats every phase).  4096 x 4096 at M = 32: 14.4 against 17.9 us; 2048 -> 8192 FP8: 13.3 against 17.4;
    // 4096 x 11008 (688 workgroups): 25.0 against 23.5; M = 64 on 4096 x 4096: 21.3 against 20.0.
    if (forced == 0 && ntiles * splits > 320) {
        // Wide outputs: two row tiles per wave (256 weight rows per workgroup) and as few rounds per workgroup as keep the
        // launch within one round of workgroups (one workgroup of this form per CU: at most 256).  4096 x 11008 (43 column tiles): 4 splits x 2 rounds of 512, 172 workgroups,
        // M = 17 19.2 us against 23.0 on the tiled path, M = 32 21.3 against 23.9 (8 splits x 1 round, 344 workgroups: 25.5).
        if (mb * 2 > max_tiles) return false;
        const int64_t ntiles2 = (n + FNN_STREAM_NW * 2 * 16 - 1) / (FNN_STREAM_NW * 2 * 16);
        const int64_t total512 = (k + 511) / 512;
        for (int64_t r2 = 1; r2 <= 4; r2++) {
            const int64_t s2 = (total512 + r2 - 1) / r2;
            if (s2 > 64 || (s2 - 1) * r2 >= total512) continue;   // (no empty split)
            if (ntiles2 * s2 > 256) continue;   // (one workgroup of this form per CU: 270 workgroups on 5120 x 13824 ran 33.7 us against 28.0 on the tiled path)
            if (ntiles2 * s2 < 128) break;                        // (too few workgroups: the tiled path is ahead)
            *out = StreamPlan{mb, 2, 512, (int)s2, (int)r2, (int)ntiles2};
            return true;
        }
        return false;
    }
    *out = StreamPlan{mb, rt, kr, (int)splits, (int)rounds, (int)ntiles};
    return true;
}

}  // namespace

int fnn_stream_qmatmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q, int flags, bool *handled)
{
    *handled = false;
    int64_t lo = fnn_ctx_option(ctx, FNN_OPT_STREAM_MIN_M), hi = fnn_ctx_option(ctx, FNN_OPT_STREAM_MAX_M);
    const int dt = w->dtype;
    const bool cb = dt == FNN_DT_I4CB;
    // Per-channel types: up to two blocks of 16 activation rows (three and four measured slower than the tiled path).
    // Codebook weights: the tiled path decodes them on the vector ALU inside its loop and is far from the memory bound,
    // so the range is wider, 5 <= M <= 64 with the options at their defaults.
    if (cb) { lo = lo < 5 ? lo : 5; hi = hi >= 32 ? 64 : hi; }
    // A long K over few output columns (the down projection of an MLP): the one-launch kernels for M <= 16 give every
    // workgroup whole rows -- few workgroups, each converting M x K activations -- while this kernel splits K over the
    // chip and its time hardly depends on M.  From M = 9 where K >= 4 N, or K >= 2 N from K = 8192 on (11008 -> 4096 I4:
    // 16.7-17.2 against 22.1-23.6 us; 4096 -> 1024 I8: 8.7 against 9.5; but 4096 -> 2048: 10.6 against 9.7, left out);
    // from M = 5 only where N <= 2048 and K >= 4 N with K >= 8192 (f16 types: 8192 -> 2048 FP8 12.0-12.2 against
    // 13.0-13.3 us) or K >= 16384 (types of the int8 GEMV, which is the better kernel below that: 16384 -> 1024 I4 13.7
    // against 20.2-20.8 us, 8192 -> 1024 I4 13.2 against 11.4).  Not when the option was raised above its default.
    const bool int_type = dt == FNN_DT_I8 || dt == FNN_DT_I4 || dt == FNN_DT_U4;
    if (!cb && lo <= 17) {
        // ... and from M = 9 where K leaves the eight waves of the kernel for 9 <= M <= 16 a ragged last round (its waves
        // take slices of 512 k-values in turn: 9, 10 or 12 slices are two rounds with half of the waves idle in the
        // second).  5120 x 13824 I4: 18.0-19.0 against 32.7-34.0 us; 5120 x 5120: 13.4-13.7 against 17.0; 6144 x 6144: 14.4-14.9
        // against 17.1-17.5; 3072 (six slices, one round) stays: 9.8 against 10.8-11.2.
        const int64_t nsl = (q.k + 511) / 512, rnds = (nsl + 7) / 8;
        if (rnds >= 2 && nsl * 4 <= rnds * 8 * 3) lo = lo < 9 ? lo : 9;
        if (q.k >= 4 * q.n || (q.k >= 2 * q.n && q.k >= 8192)) lo = lo < 9 ? lo : 9;
        if (q.n <= 2048 && q.k >= 4 * q.n && q.k >= (int_type ? 16384 : 8192)) lo = lo < 5 ? lo : 5;
    }
    if (q.m < lo || q.m > hi || q.m > (cb ? 64 : 32) || q.n < 1) return FNN_OK;
    if (flags & FNN_FLAG_ACT_F16_SINGLE) return FNN_OK;
    if (cb && fnn_ctx_option(ctx, FNN_OPT_CODEBOOK_EXPANDED) != 0) return FNN_OK;   // (the option names a form of the tiled path)
    if (cb && (q.as_written || q.qblock != 32 || q.k % 128 != 0 || q.bpr != q.k / 32 || (reinterpret_cast<uintptr_t>(q.scales) & 15) ||
               q.bpr * 4 * 256 >= (int64_t)1 << 31)) return FNN_OK;
    if (dt < FNN_DT_I8 || (dt > FNN_DT_F4 && !cb)) return FNN_OK;
    if (int_type && fnn_ctx_option(ctx, FNN_OPT_GEMM_INT8) == 0) return FNN_OK;
    if (q.kp % 4 != 0 || q.k % 8 != 0 || q.k < 8) return FNN_OK;
    // the f16 types multiply whatever bytes a lane load holds: every load must lie wholly inside or wholly past K
    if (!int_type && q.k % (dt == FNN_DT_F4 ? 128 : 64) != 0) return FNN_OK;
    if ((reinterpret_cast<uintptr_t>(q.a) & 15) || (reinterpret_cast<uintptr_t>(q.words) & 15)) return FNN_OK;
    // 32-bit buffer offsets: a column tile of 256 rows, the activation block
    if (q.kp * 4 * 256 >= (int64_t)1 << 31 || q.m * q.k * 4 >= (int64_t)0xFFFFFF00 || q.k >= (int64_t)1 << 28) return FNN_OK;
    StreamPlan pl;
    const int64_t forced = fnn_ctx_option(ctx, FNN_OPT_STREAM_SHAPE);
    const int bits = (dt == FNN_DT_I4 || dt == FNN_DT_U4 || dt == FNN_DT_F4 || cb) ? 4 : 8;
    if (!plan_stream(bits, int_type ? 4 : (cb ? 6 : 8), cb ? 4 : 2, q.m, q.n, q.k, forced, &pl)) return FNN_OK;
    if (pl.ntiles > FNN_STREAM_COUNTERS) return FNN_OK;
    StreamArgs p;
    p.words = q.words; p.scales = q.scales; p.zeros = q.zeros; p.a = q.a; p.bias = q.bias; p.out = q.out;
    p.codebook = cb ? q.codebook : nullptr; p.bpr = cb ? q.bpr : 0;
    p.residual = nullptr; p.sum_out = nullptr;
    p.part = nullptr; p.count = fnn_ctx_stream_counters(ctx);
    p.m = q.m; p.n = q.n; p.k = q.k; p.kp = q.kp;
    p.act = q.act; p.splits = pl.splits; p.rounds = pl.rounds; p.ntiles = pl.ntiles;
    if (int rc = fnn_tile_major_words(ctx, s, w, q, &p.words_tm, &p.kb64)) return rc;
    if (pl.splits > 1) {
        const size_t wgf = (size_t)pl.mb * pl.rt * 4 * FNN_STREAM_NW * 64 + 16 * pl.mb;
        void *ws = nullptr;
        int rc = fnn_ctx_ensure_tmp(ctx, 1, (size_t)pl.splits * pl.ntiles * wgf * 4, &ws);
        if (rc) return rc;
        p.part = (float *)ws;
    }
    if (FnnResidualIo *res = fnn_ctx_residual_io(ctx); res->residual && res->of_out == q.out && res->elems == (uint64_t)(q.m * q.n)) {
        p.residual = res->residual; p.sum_out = res->sum_out;
        res->used = 1;
    }
    hipError_t e;
    switch (dt) {
    case FNN_DT_I8: e = fnn_stream_launch_i8(pl, p, s); break;
    case FNN_DT_I4: e = fnn_stream_launch_i4(pl, p, s); break;
    case FNN_DT_U4: e = fnn_stream_launch_u4(pl, p, s); break;
    case FNN_DT_U8: e = fnn_stream_launch_u8(pl, p, s); break;
    case FNN_DT_F8: e = fnn_stream_launch_f8(pl, p, s); break;
    case FNN_DT_F8R: e = fnn_stream_launch_f8r(pl, p, s); break;
    case FNN_DT_I4CB: e = fnn_stream_launch_i4cb(pl, p, s); break;
    default: e = fnn_stream_launch_f4(pl, p, s); break;
    }
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    *handled = true;
    return FNN_OK;
}
