// Host-side weight packers of libfastnn_hip: the quantisers fastnn's compiler pass
// applies to constant MatMul / Conv weights before a backend sees them
// (src/compiler/passes/quantization.rs:170-260, 281-495).  Results are bit-identical to
// fastnn's: strict binary32 arithmetic in the reference's evaluation order (this file is
// compiled with FMA contraction off); only order-independent work is spread over threads.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

#include "../../include/fastnn_hip.h"

namespace {

constexpr size_t kMargin = 16;  // SIMD_MARGIN words after the last row (src/packed_tensor.rs:980-982)

inline int lanes_of(int dt)
{
    switch (dt) {
    case FNN_DT_I8: case FNN_DT_U8: case FNN_DT_F8: case FNN_DT_F8R: return 4;
    case FNN_DT_I4: case FNN_DT_U4: case FNN_DT_F4: case FNN_DT_I4CB: return 8;
    default: return 0;
    }
}

inline float clamp_keep_nan(float x, float lo, float hi) { return x < lo ? lo : (x > hi ? hi : x); }

// `as iN` after clamp+round: value already in range, NaN becomes 0
inline int32_t to_int(float f) { return std::isnan(f) ? 0 : (int32_t)f; }

// ---- single-lane encoders (pack_from_f32 of each PackedWord) -----------------------

struct EncI8 {  // src/dtypes/i8x4.rs:34-43
    static constexpr int kBits = 8;
    static uint32_t enc(float v) { return (uint32_t)(uint8_t)(int8_t)to_int(std::round(clamp_keep_nan(v, -128.f, 127.f))); }
};
struct EncI4 {  // src/dtypes/i4x8.rs:34-42
    static constexpr int kBits = 4;
    static uint32_t enc(float v) { return (uint32_t)(uint8_t)(int8_t)to_int(std::round(clamp_keep_nan(v, -8.f, 7.f))) & 0xFu; }
};
struct EncU8 {  // src/dtypes/u8x4.rs:33-40
    static constexpr int kBits = 8;
    static uint32_t enc(float v) { return (uint32_t)to_int(std::round(clamp_keep_nan(v, 0.f, 255.f))) & 0xFFu; }
};
struct EncU4 {  // src/dtypes/u4x8.rs:34-41
    static constexpr int kBits = 4;
    static uint32_t enc(float v) { return (uint32_t)to_int(std::round(clamp_keep_nan(v, 0.f, 15.f))) & 0xFu; }
};

// Minifloat encoder shared by E4M3 (src/dtypes/f8x4.rs:41-77) and E5M2
// (src/dtypes/f8x4r.rs:48-88): mantissa rounded half away from zero, carry into the
// exponent, saturation at `max_code`, subnormals scaled by `sub_mul`.
template <int MBITS, int BIAS, int EMAX>
uint32_t enc_minifloat(float v, float max_val, float sub_limit, float sub_mul, uint32_t max_code, bool has_inf)
{
    if (std::isnan(v)) return 0x7F;
    const uint32_t sign = (v < 0.0f) ? 0x80u : 0u;
    float a = std::fabs(v);
    if (a == 0.0f) return std::signbit(v) ? 0x80u : 0u;
    if (has_inf && std::isinf(v)) return v > 0.0f ? 0x7Cu : 0xFCu;
    a = std::min(a, max_val);
    constexpr int MONE = 1 << MBITS;
    if (a < sub_limit) {
        float r = std::round(a * sub_mul);
        int m = r >= 255.0f ? 255 : (int)r;
        if (m >= MONE) return sign | (uint32_t)MONE;
        return sign | (uint32_t)m;
    }
    int ex;
    (void)std::frexp(a, &ex);
    const int e = ex - 1;  // floor(log2 a); see the oracle's note on why this equals log2().floor() here
    const int biased = e + BIAS;
    const float normalized = a / std::ldexp(1.0f, e);
    float r = std::round((normalized - 1.0f) * (float)MONE);
    int mant = std::isnan(r) ? 0 : (r <= 0.0f ? 0 : (r >= 255.0f ? 255 : (int)r));
    if (mant >= MONE) {
        const int nb = biased + 1;
        if (nb >= EMAX) return sign | max_code;
        return sign | (uint32_t)(nb << MBITS);
    }
    if (biased >= EMAX) return sign | max_code;
    return sign | (uint32_t)(biased << MBITS) | (uint32_t)mant;
}

struct EncF8 {
    static constexpr int kBits = 8;
    static uint32_t enc(float v) { return enc_minifloat<3, 7, 15>(v, 240.0f, 0.015625f, 512.0f, 0x7Bu, false); }
};
struct EncF8R {
    static constexpr int kBits = 8;
    static uint32_t enc(float v) { return enc_minifloat<2, 15, 31>(v, 57344.0f, 1.0f / 16384.0f, 16384.0f, 0x7Cu, true); }
};
struct EncF4 {  // src/dtypes/f4x8.rs:49-70
    static constexpr int kBits = 4;
    static uint32_t enc(float v)
    {
        static const float mag[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
        if (std::isnan(v)) return 0;
        const float a = std::fabs(v);
        uint32_t best = 0;
        float best_d = a;
        for (uint32_t i = 0; i < 8; i++) {
            const float d = std::fabs(a - mag[i]);
            if (d < best_d) { best_d = d; best = i; }
        }
        return (std::signbit(v) && best != 0) ? (best | 0x8u) : best;
    }
};

// Pack one row: lane value f(x); lanes past the row end are the value 0.0
// (src/packed_tensor.rs:993-1003).
template <class Enc, class F>
void pack_row(const float *row, int64_t inner, uint32_t *dst, F f)
{
    constexpr int items = 32 / Enc::kBits;
    const int64_t kp = (inner + items - 1) / items;
    for (int64_t wd = 0; wd < kp; wd++) {
        uint32_t w = 0;
        for (int i = 0; i < items; i++) {
            const int64_t e = wd * items + i;
            const float lane = (e < inner) ? f(row[e]) : 0.0f;
            w |= Enc::enc(lane) << (Enc::kBits * i);
        }
        dst[wd] = w;
    }
}

template <class Fn>
void parallel_rows(int64_t rows, int64_t work_per_row, Fn fn)
{
    unsigned hw = std::thread::hardware_concurrency();
    int64_t nt = hw ? (int64_t)hw : 4;
    if (nt > 16) nt = 16;
    if (rows * work_per_row < (1 << 18)) nt = 1;
    if (nt > rows) nt = rows > 0 ? rows : 1;
    if (nt <= 1) { fn(0, rows); return; }
    std::vector<std::thread> th;
    const int64_t per = (rows + nt - 1) / nt;
    for (int64_t t = 0; t < nt; t++) {
        const int64_t r0 = t * per, r1 = std::min(rows, r0 + per);
        if (r0 >= r1) break;
        th.emplace_back([=] { fn(r0, r1); });
    }
    for (auto &t : th) t.join();
}

// from_f32_per_channel_asymmetric, group_size 0 (src/packed_tensor.rs:852-1049)
template <class Enc, bool FP4>
void quant_asym(const float *w, int64_t rows, int64_t inner, uint32_t *words, float *scales, float *zeros)
{
    constexpr int items = 32 / Enc::kBits;
    const int64_t kp = (inner + items - 1) / items;
    const float umax = (float)((1u << Enc::kBits) - 1u);
    const float sbias = (float)(1u << (Enc::kBits - 1));
    parallel_rows(rows, inner, [=](int64_t r0, int64_t r1) {
        for (int64_t r = r0; r < r1; r++) {
            const float *row = w + r * inner;
            float mn = 3.40282347e+38f, mx = -3.40282347e+38f;
            for (int64_t i = 0; i < inner; i++) { mn = std::fmin(mn, row[i]); mx = std::fmax(mx, row[i]); }
            const float range = mx - mn;
            float scale, zero;
            if (range == 0.0f) {
                scale = 1.0f; zero = 0.0f;
            } else if (FP4) {
                float sum = 0.0f;
                for (int64_t i = 0; i < inner; i++) sum += row[i];
                const float mean = sum / (float)inner;
                const float dev = std::fmax(std::fabs(mean - mn), std::fabs(mx - mean));
                scale = (dev == 0.0f ? 1e-10f : dev) / 4.0f;
                zero = mean;
            } else {
                const float init = range / umax;
                const float lo = mn - init, hi = mx + init;
                scale = (hi - lo) / umax;
                zero = lo + sbias * scale;
            }
            scales[r] = scale;
            zeros[r] = zero;
            const float inv = (scale != 0.0f) ? 1.0f / scale : 0.0f;
            pack_row<Enc>(row, inner, words + r * kp, [=](float x) { return (x - zero) * inv; });
        }
    });
}

// from_f32_per_channel (src/packed_tensor.rs:661-742)
template <class Enc>
void quant_sym(const float *w, int64_t rows, int64_t inner, float max_val, uint32_t *words, float *scales, float *zeros)
{
    constexpr int items = 32 / Enc::kBits;
    const int64_t kp = (inner + items - 1) / items;
    parallel_rows(rows, inner, [=](int64_t r0, int64_t r1) {
        for (int64_t r = r0; r < r1; r++) {
            const float *row = w + r * inner;
            float max_abs = 0.0f;
            for (int64_t i = 0; i < inner; i++) max_abs = std::fmax(max_abs, std::fabs(row[i]));
            const float scale = (max_abs == 0.0f) ? 1.0f : max_abs / max_val;
            scales[r] = scale;
            zeros[r] = 0.0f;
            const float inv = (scale != 1.0f) ? 1.0f / scale : 1.0f;
            pack_row<Enc>(row, inner, words + r * kp, [=](float x) { return x * inv; });
        }
    });
}

inline uint32_t nearest16(float v, const float *cb)
{
    float best_d = std::fabs(v - cb[0]);
    uint32_t best = 0;
    for (uint32_t i = 1; i < 16; i++) {
        const float d = std::fabs(v - cb[i]);
        if (d < best_d) { best_d = d; best = i; }
    }
    return best;
}

// kmeans_16 (src/packed_tensor.rs:18-75).  The assignment step is independent per value
// and runs on threads; the f32 cluster sums must follow data order and stay sequential.
bool kmeans16(const std::vector<float> &vals, int iters, float *c)
{
    const size_t n = vals.size();
    std::fill(c, c + 16, 0.0f);
    if (n == 0) return true;
    if (n == 1) { std::fill(c, c + 16, vals[0]); return true; }
    for (float v : vals) if (std::isnan(v)) return false;  // the reference panics on NaN
    {
        std::vector<float> sorted(vals);
        // stable, with -0.0 == +0.0, like sort_by(partial_cmp)
        std::stable_sort(sorted.begin(), sorted.end(), [](float a, float b) { return a < b; });
        for (int i = 0; i < 16; i++) {
            const float pct = ((float)i + 0.5f) / 16.0f;
            size_t idx = (size_t)(pct * (float)n);
            c[i] = sorted[std::min(idx, n - 1)];
        }
    }
    std::vector<uint8_t> assign(n);
    for (int it = 0; it < iters; it++) {
        float cc[16];
        std::memcpy(cc, c, sizeof(cc));
        parallel_rows((int64_t)n, 16, [&](int64_t i0, int64_t i1) {
            for (int64_t i = i0; i < i1; i++) assign[(size_t)i] = (uint8_t)nearest16(vals[(size_t)i], cc);
        });
        size_t counts[16] = {0};
        float sums[16] = {0};
        for (size_t i = 0; i < n; i++) { counts[assign[i]]++; sums[assign[i]] += vals[i]; }
        for (int k = 0; k < 16; k++) if (counts[k] > 0) c[k] = sums[k] / (float)counts[k];
    }
    std::stable_sort(c, c + 16, [](float a, float b) { return a < b; });
    return true;
}

// from_f32_per_block_codebook (src/packed_tensor.rs:1209-1313)
int quant_codebook(const float *w, int64_t rows, int64_t inner, int64_t qb, uint32_t *words, float *bscales, float *cb)
{
    const int64_t bpr = (inner + qb - 1) / qb, kp = (inner + 7) / 8;
    std::vector<float> norm((size_t)(rows * inner));
    parallel_rows(rows, inner, [&](int64_t r0, int64_t r1) {
        for (int64_t r = r0; r < r1; r++)
            for (int64_t b = 0; b < bpr; b++) {
                const int64_t base = r * inner + b * qb, end = std::min(base + qb, (r + 1) * inner);
                float mx = 0.0f;
                for (int64_t i = base; i < end; i++) mx = std::fmax(mx, std::fabs(w[i]));
                bscales[r * bpr + b] = mx;
                if (mx > 0.0f) {
                    const float inv = 1.0f / mx;
                    for (int64_t i = base; i < end; i++) norm[(size_t)i] = w[i] * inv;
                } else {
                    for (int64_t i = base; i < end; i++) norm[(size_t)i] = 0.0f;
                }
            }
    });
    // block order of the reference's normalised list == element order (blocks tile each row)
    if (!kmeans16(norm, 30, cb)) return FNN_ERR_COMPILATION;
    parallel_rows(rows, inner, [&](int64_t r0, int64_t r1) {
        for (int64_t r = r0; r < r1; r++)
            for (int64_t b = 0; b < bpr; b++) {
                const float s = bscales[r * bpr + b];
                const float inv = s > 0.0f ? 1.0f / s : 0.0f;
                const int64_t base = r * inner + b * qb, end = std::min(base + qb, (r + 1) * inner);
                for (int64_t eb = 0; eb < end - base; eb += 8) {
                    uint32_t word = 0;
                    for (int i = 0; i < 8; i++) {
                        const int64_t e = base + eb + i;
                        if (e < end) word |= nearest16(w[e] * inv, cb) << (4 * i);
                    }
                    words[r * kp + (b * qb + eb) / 8] = word;  // a straddling word keeps the later block's value
                }
            }
    });
    return FNN_OK;
}

}  // namespace

extern "C" {

size_t fnn_packed_words(int dtype, int64_t rows, int64_t inner)
{
    const int items = lanes_of(dtype);
    if (!items || rows < 0 || inner < 0) return 0;
    return (size_t)(rows * ((inner + items - 1) / items)) + kMargin;
}

void fnn_transpose_kn_to_nk(const float *w_kn, int64_t k, int64_t n, float *w_nk)
{
    constexpr int64_t T = 32;
    for (int64_t k0 = 0; k0 < k; k0 += T)
        for (int64_t n0 = 0; n0 < n; n0 += T)
            for (int64_t kk = k0; kk < std::min(k, k0 + T); kk++)
                for (int64_t nn = n0; nn < std::min(n, n0 + T); nn++) w_nk[nn * k + kk] = w_kn[kk * n + nn];
}

int fnn_quantize_weights(int dtype, const float *w, int64_t rows, int64_t inner, int qblock,
                         uint32_t *words, float *scales, float *zeros, float *codebook16)
{
    const int items = lanes_of(dtype);
    if (!items || !w || !words || !scales || rows <= 0 || inner <= 0) return FNN_ERR_COMPILATION;
    if (dtype != FNN_DT_I4CB && !zeros) return FNN_ERR_COMPILATION;
    std::memset(words, 0, fnn_packed_words(dtype, rows, inner) * sizeof(uint32_t));
    switch (dtype) {
    case FNN_DT_I8: quant_asym<EncI8, false>(w, rows, inner, words, scales, zeros); return FNN_OK;
    case FNN_DT_I4: quant_asym<EncI4, false>(w, rows, inner, words, scales, zeros); return FNN_OK;
    case FNN_DT_U8: quant_asym<EncU8, false>(w, rows, inner, words, scales, zeros); return FNN_OK;
    case FNN_DT_U4: quant_asym<EncU4, false>(w, rows, inner, words, scales, zeros); return FNN_OK;
    case FNN_DT_F4: quant_asym<EncF4, true>(w, rows, inner, words, scales, zeros); return FNN_OK;
    case FNN_DT_F8: quant_sym<EncF8>(w, rows, inner, 240.0f, words, scales, zeros); return FNN_OK;
    case FNN_DT_F8R: quant_sym<EncF8R>(w, rows, inner, 57344.0f, words, scales, zeros); return FNN_OK;
    case FNN_DT_I4CB:
        if (qblock <= 0 || !codebook16) return FNN_ERR_COMPILATION;
        return quant_codebook(w, rows, inner, qblock, words, scales, codebook16);
    default: return FNN_ERR_COMPILATION;
    }
}

}  // extern "C"
