/*
 * fnn_oracle.c -- CPU restatement of fastnn's weight-quantised MatMul path.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels.  It is never
 * linked into, imported by or called from the shipped package.
 *
 * Written from the text of the reference sources; every function names the
 * reference lines it follows (paths relative to the fastnn source tree).
 * Build with strict IEEE-754 semantics:
 *     gcc -O2 -std=c11 -ffp-contract=off -fno-fast-math
 *
 * Pinning status (what each part is checked against in tests/):
 *   word codecs ............ literals of src/dtypes/{i8x4,i4x8,f8x4,f4x8}.rs tests,
 *                            exhaustive closed forms, OCP E4M3/E5M2/E2M1 tables
 *   integer lane dots ...... literals of src/backend/cpu/swar.rs tests, brute force
 *   asymmetric quantiser ... FP4 scale/zero literals packed_tensor.rs:1972-2014,
 *                            |deq-x| <= scale invariant (:1009-1036), f64 re-derivation
 *   FP8 quantiser .......... closed form scale = max|row|/240, max -> code 0x77
 *   codebook quantiser ..... fixture packed_tensor.rs:2016-2115 (max err < 2),
 *                            argmin/sortedness invariants, brute force k-means on tiny input
 *   dequant ................ one IEEE multiply(+add) per element
 *   f32 MatMul ............. closed-form literals microkernels/tests.rs:369-763,
 *                            seeded end-to-end bounds tests/cpu_reference_oracle.rs
 *   I8-activation MatMul ... exact integers; literals microkernels/tests.rs:369-678
 *   per-channel activation payloads ... hand-worked byte images (a later channel overwrites an earlier one's
 *                            codes), the closed form "codes of the last channel in range", the per-tensor functions on
 *                            one channel
 *   conv lowering .......... (I8 and I4 weights) equals float conv of dequantised operands; integer
 *                            accumulators exact; brute-force direct convolution; activation
 *                            quantiser re-derived in f32; flat-input special cases
 *   conv on I8 payloads .... f64 convolution of the dequantised int8 activations (torch unfold on the
 *                            exact integers, padding taps = integer 0) with the dequantised weights;
 *                            bias on the accumulator grid (8-bit) or in f32 (4-bit); zero = 0 and != 0
 *   conv, other types ...... torch.nn.functional.conv2d in f64 on the dequantised weights
 *   concat / slice / max pool / nearest upsample ... numpy concatenate, slicing, repeat and
 *                            torch max_pool2d / interpolate (bit-identical data movement)
 *   What only an execution of the Rust crate could pin tighter: the last-bit
 *   value of its AVX/Rayon f32 summation order (tolerance-only by design).
 */
#include "fnn_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#if defined(__x86_64__)
#include <immintrin.h>
#endif

/* ------------------------------------------------------------------------ */
/* helpers                                                                    */
/* ------------------------------------------------------------------------ */

static inline size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }

/* Rust `x.clamp(lo, hi)`: NaN stays NaN. */
static inline float clampf(float x, float lo, float hi)
{
    if (x < lo) return lo;
    if (x > hi) return hi;
    return x;
}

/* Rust `f as i8` / `as u8` / `as i32`: saturating, NaN -> 0. */
static inline int32_t sat_i32(float f, int32_t lo, int32_t hi)
{
    if (f != f) return 0;
    if (f <= (float)lo) return lo;
    if (f >= (float)hi) return hi;
    return (int32_t)f;
}

/* ------------------------------------------------------------------------ */
/* word codecs                                                                */
/* ------------------------------------------------------------------------ */

/* src/dtypes/<type>.rs: ITEMS / BIT_WIDTH constants of each PackedWord impl. */
int fnn_or_items(int dt)
{
    switch (dt) {
    case FNN_OR_I8: case FNN_OR_U8: case FNN_OR_F8: case FNN_OR_F8R: return 4;
    case FNN_OR_I4: case FNN_OR_U4: case FNN_OR_F4: case FNN_OR_I4CB: return 8;
    default: return 0;
    }
}

int fnn_or_bit_width(int dt)
{
    int it = fnn_or_items(dt);
    return it ? 32 / it : 0;
}

/* src/dtypes/f8x4.rs:23-38 -- E4M3, bias 7; exp 0 subnormal; exp 15 always NaN. */
float fnn_or_e4m3_to_f32(uint8_t b)
{
    float sign = (b & 0x80) ? -1.0f : 1.0f;
    int e = (b >> 3) & 0x0F;
    float mant = (float)(b & 0x07);
    if (e == 0) {
        if (mant == 0.0f) return 0.0f * sign;
        return sign * ldexpf(1.0f, 1 - 7) * (mant / 8.0f);
    }
    if (e == 0x0F) return NAN;
    return sign * ldexpf(1.0f, e - 7) * (1.0f + mant / 8.0f);
}

/* floor(log2(x)) for finite positive normal-or-subnormal x.  The reference uses
 * `abs_v.log2().floor()` (f8x4.rs:62); if libm rounds log2 up to an integer for
 * x a few ulp below a power of two, (normalized-1)*8 is a tiny negative number
 * that rounds to -0 -> 0, which encodes the same byte as the mantissa carry
 * taken from the exact exponent, so the exact exponent is equivalent. */
static inline int floor_log2f(float x)
{
    int e;
    (void)frexpf(x, &e); /* x = f * 2^e, f in [0.5,1) */
    return e - 1;
}

/* src/dtypes/f8x4.rs:41-77 */
uint8_t fnn_or_f32_to_e4m3(float v)
{
    if (v != v) return 0x7F;
    uint8_t sign_bit = (v < 0.0f) ? 0x80 : 0x00;
    float abs_v = fabsf(v);
    if (abs_v == 0.0f) return signbit(v) ? 0x80 : 0x00;
    if (abs_v > 240.0f) abs_v = 240.0f;
    if (abs_v < 0.015625f) {
        int m = sat_i32(roundf(abs_v * 512.0f), 0, 255);
        if (m >= 8) return sign_bit | 0x08;
        if (m == 0) return sign_bit;
        return sign_bit | (uint8_t)m;
    }
    int e = floor_log2f(abs_v);
    int biased = e + 7;
    float normalized = abs_v / ldexpf(1.0f, e);
    int mant = sat_i32(roundf((normalized - 1.0f) * 8.0f), 0, 255);
    if (mant >= 8) {
        int nb = biased + 1;
        if (nb >= 15) return sign_bit | 0x7B;
        return sign_bit | (uint8_t)(nb << 3);
    }
    if (biased >= 15) return sign_bit | 0x7B;
    return sign_bit | (uint8_t)(biased << 3) | (uint8_t)mant;
}

/* src/dtypes/f8x4r.rs:24-45 -- E5M2, bias 15, exp 31: mant 0 = inf else NaN. */
float fnn_or_e5m2_to_f32(uint8_t b)
{
    float sign = (b & 0x80) ? -1.0f : 1.0f;
    int e = (b >> 2) & 0x1F;
    float mant = (float)(b & 0x03);
    if (e == 0) {
        if (mant == 0.0f) return 0.0f * sign;
        return sign * ldexpf(1.0f, 1 - 15) * (mant / 4.0f);
    }
    if (e == 0x1F) return (mant == 0.0f) ? sign * INFINITY : NAN;
    return sign * ldexpf(1.0f, e - 15) * (1.0f + mant / 4.0f);
}

/* src/dtypes/f8x4r.rs:48-88 */
uint8_t fnn_or_f32_to_e5m2(float v)
{
    if (v != v) return 0x7F;
    uint8_t sign_bit = (v < 0.0f) ? 0x80 : 0x00;
    float abs_v = fabsf(v);
    if (abs_v == 0.0f) return signbit(v) ? 0x80 : 0x00;
    if (isinf(v)) return (v > 0.0f) ? 0x7C : 0xFC;
    if (abs_v > 57344.0f) abs_v = 57344.0f;
    if (abs_v < (1.0f / 16384.0f)) {
        int m = sat_i32(roundf(abs_v * 16384.0f), 0, 255);
        if (m >= 4) return sign_bit | 0x04;
        if (m == 0) return sign_bit;
        return sign_bit | (uint8_t)m;
    }
    int e = floor_log2f(abs_v);
    int biased = e + 15;
    float normalized = abs_v / ldexpf(1.0f, e);
    int mant = sat_i32(roundf((normalized - 1.0f) * 4.0f), 0, 255);
    if (mant >= 4) {
        int nb = biased + 1;
        if (nb >= 31) return sign_bit | 0x7C;
        return sign_bit | (uint8_t)(nb << 2);
    }
    if (biased >= 31) return sign_bit | 0x7C;
    return sign_bit | (uint8_t)(biased << 2) | (uint8_t)mant;
}

/* src/dtypes/f4x8.rs:21 */
static const float FP4_MAG[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};

/* src/dtypes/f4x8.rs:25-39 -- code 0x8 decodes to +0.0. */
float fnn_or_fp4_to_f32(uint8_t code)
{
    float mag = FP4_MAG[code & 7];
    if ((code & 8) && (code & 7)) return -mag;
    return mag;
}

/* src/dtypes/f4x8.rs:49-70 -- nearest magnitude, strict '<' so lower index wins. */
uint8_t fnn_or_f32_to_fp4(float v)
{
    if (v != v) return 0;
    int sign = signbit(v) ? 1 : 0;
    float a = fabsf(v);
    uint8_t best_i = 0;
    float best_d = a;
    for (int i = 0; i < 8; i++) {
        float d = fabsf(a - FP4_MAG[i]);
        if (d < best_d) { best_d = d; best_i = (uint8_t)i; }
    }
    if (sign && best_i != 0) return best_i | 0x8;
    return best_i;
}

/* unpack_to_f32 of each PackedWord impl:
 * i8x4.rs:24-31, i4x8.rs:23-31, u8x4.rs, u4x8.rs:22-31, f8x4.rs:120-128,
 * f8x4r.rs, f4x8.rs:118-131.  Lane i sits at bits [i*w, (i+1)*w). */
void fnn_or_unpack_word(int dt, uint32_t w, float *out)
{
    switch (dt) {
    case FNN_OR_I8:
        for (int i = 0; i < 4; i++) out[i] = (float)(int8_t)((w >> (8 * i)) & 0xFF);
        break;
    case FNN_OR_U8:
        for (int i = 0; i < 4; i++) out[i] = (float)((w >> (8 * i)) & 0xFF);
        break;
    case FNN_OR_I4:
    case FNN_OR_I4CB:
        for (int i = 0; i < 8; i++) {
            int32_t nib = (int32_t)((w >> (4 * i)) & 0xF);
            out[i] = (float)(nib >= 8 ? nib - 16 : nib);
        }
        break;
    case FNN_OR_U4:
        for (int i = 0; i < 8; i++) out[i] = (float)((w >> (4 * i)) & 0xF);
        break;
    case FNN_OR_F8:
        for (int i = 0; i < 4; i++) out[i] = fnn_or_e4m3_to_f32((uint8_t)(w >> (8 * i)));
        break;
    case FNN_OR_F8R:
        for (int i = 0; i < 4; i++) out[i] = fnn_or_e5m2_to_f32((uint8_t)(w >> (8 * i)));
        break;
    case FNN_OR_F4:
        for (int i = 0; i < 8; i++) out[i] = fnn_or_fp4_to_f32((uint8_t)((w >> (4 * i)) & 0xF));
        break;
    default: break;
    }
}

/* pack_from_f32 of each PackedWord impl: integer types clamp THEN round half
 * away from zero (i8x4.rs:34-43, i4x8.rs:34-42, u8x4.rs:33-40, u4x8.rs:34-41). */
uint32_t fnn_or_pack_word(int dt, const float *v)
{
    uint32_t w = 0;
    switch (dt) {
    case FNN_OR_I8:
        for (int i = 0; i < 4; i++) {
            int32_t q = sat_i32(roundf(clampf(v[i], -128.0f, 127.0f)), -128, 127);
            w |= ((uint32_t)(uint8_t)(int8_t)q) << (8 * i);
        }
        break;
    case FNN_OR_U8:
        for (int i = 0; i < 4; i++) {
            int32_t q = sat_i32(roundf(clampf(v[i], 0.0f, 255.0f)), -2147483647, 2147483647);
            w |= ((uint32_t)q & 0xFF) << (8 * i);
        }
        break;
    case FNN_OR_I4:
    case FNN_OR_I4CB:
        for (int i = 0; i < 8; i++) {
            int32_t q = sat_i32(roundf(clampf(v[i], -8.0f, 7.0f)), -128, 127);
            w |= ((uint32_t)(uint8_t)(int8_t)q & 0xF) << (4 * i);
        }
        break;
    case FNN_OR_U4:
        for (int i = 0; i < 8; i++) {
            int32_t q = sat_i32(roundf(clampf(v[i], 0.0f, 15.0f)), -2147483647, 2147483647);
            w |= ((uint32_t)q & 0xF) << (4 * i);
        }
        break;
    case FNN_OR_F8:
        for (int i = 0; i < 4; i++) w |= ((uint32_t)fnn_or_f32_to_e4m3(v[i])) << (8 * i);
        break;
    case FNN_OR_F8R:
        for (int i = 0; i < 4; i++) w |= ((uint32_t)fnn_or_f32_to_e5m2(v[i])) << (8 * i);
        break;
    case FNN_OR_F4:
        for (int i = 0; i < 8; i++) w |= ((uint32_t)fnn_or_f32_to_fp4(v[i])) << (4 * i);
        break;
    default: break;
    }
    return w;
}

/* ------------------------------------------------------------------------ */
/* integer lane dots                                                          */
/* ------------------------------------------------------------------------ */

/* src/backend/cpu/swar.rs:15-38 */
int32_t fnn_or_i8x4_dot(uint32_t a, uint32_t b)
{
    int32_t s = 0;
    for (int i = 0; i < 4; i++)
        s += (int32_t)(int8_t)(a >> (8 * i)) * (int32_t)(int8_t)(b >> (8 * i));
    return s;
}

/* src/backend/cpu/swar.rs:41-48 */
int32_t fnn_or_i8x4_sum(uint32_t w)
{
    int32_t s = 0;
    for (int i = 0; i < 4; i++) s += (int32_t)(int8_t)(w >> (8 * i));
    return s;
}

static inline int32_t nib_s(uint32_t w, int i)
{
    int32_t n = (int32_t)((w >> (4 * i)) & 0xF);
    return n >= 8 ? n - 16 : n;
}

/* src/backend/cpu/swar.rs:61-90 */
int32_t fnn_or_i4x8_dot(uint32_t a, uint32_t b)
{
    int32_t s = 0;
    for (int i = 0; i < 8; i++) s += nib_s(a, i) * nib_s(b, i);
    return s;
}

/* src/backend/cpu/swar.rs:51-59 */
int32_t fnn_or_i4x8_sum(uint32_t w)
{
    int32_t s = 0;
    for (int i = 0; i < 8; i++) s += nib_s(w, i);
    return s;
}

/* src/dtypes/f4x8.rs:73-106 -- sum of round(4*a*b) over the 8 lanes; the LUT
 * there uses -0.0 for code 8, whose products round to 0 all the same. */
int32_t fnn_or_f4x8_dot(uint32_t a, uint32_t b)
{
    static const float vals[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                   0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
    int32_t s = 0;
    for (int i = 0; i < 8; i++) {
        float p = 4.0f * vals[(a >> (4 * i)) & 0xF] * vals[(b >> (4 * i)) & 0xF];
        s += (int32_t)roundf(p);
    }
    return s;
}

/* ------------------------------------------------------------------------ */
/* packers / quantisers                                                       */
/* ------------------------------------------------------------------------ */

/* packed_tensor.rs:223-227,978-982: rows*ceil(inner/ITEMS) words + 16 margin. */
size_t fnn_or_packed_words(int dt, size_t rows, size_t inner)
{
    return rows * ceil_div(inner, (size_t)fnn_or_items(dt)) + FNN_OR_SIMD_MARGIN;
}

/* Pack one row given a per-element transform (x - zero) * inv; tail lanes are
 * the value 0.0 before packing (packed_tensor.rs:995-1003, 234-242). */
static void pack_row_affine(int dt, const float *row, size_t inner, float zero, float inv,
                            int apply, uint32_t *dst)
{
    size_t items = (size_t)fnn_or_items(dt);
    size_t kp = ceil_div(inner, items);
    float lane[8];
    for (size_t wd = 0; wd < kp; wd++) {
        for (size_t i = 0; i < items; i++) {
            size_t e = wd * items + i;
            if (e < inner)
                lane[i] = apply ? (row[e] - zero) * inv : row[e];
            else
                lane[i] = 0.0f;
        }
        dst[wd] = fnn_or_pack_word(dt, lane);
    }
}

/* packed_tensor.rs:205-273 -- from_f32_slice with one scalar (scale, zero). */
void fnn_or_from_f32_slice(int dt, const float *data, size_t rows, size_t inner, float scale,
                           float zero, uint32_t *words)
{
    size_t kp = ceil_div(inner, (size_t)fnn_or_items(dt));
    memset(words, 0, (rows * kp + FNN_OR_SIMD_MARGIN) * sizeof(uint32_t));
    int apply = (scale != 1.0f || zero != 0.0f);
    float inv = 1.0f / scale;
    for (size_t r = 0; r < rows; r++)
        pack_row_affine(dt, data + r * inner, inner, zero, inv, apply, words + r * kp);
}

/* packed_tensor.rs:852-1049 (group_size == 0 branch :945-975, packing :984-1005).
 * Integer types: range==0 -> (1,0); else init=range/U, lo=mn-init, hi=mx+init,
 * scale=(hi-lo)/U, zero=lo+B*scale.  FP4 (IS_FLOAT && MAX_REPRESENTABLE < B):
 * zero = sequential f32 row sum / inner, scale = max(|zero-mn|,|mx-zero|)/4. */
void fnn_or_quant_per_channel_asym(int dt, const float *data, size_t rows, size_t inner,
                                   uint32_t *words, float *scales, float *zeros)
{
    int bits = fnn_or_bit_width(dt);
    size_t kp = ceil_div(inner, (size_t)fnn_or_items(dt));
    float unsigned_max = (float)((1u << bits) - 1u);
    float signed_bias = (float)(1u << (bits - 1));
    int is_fp4 = (dt == FNN_OR_F4); /* MAX_REPRESENTABLE 6 < 8; F8 240 >= 128 is not */
    memset(words, 0, (rows * kp + FNN_OR_SIMD_MARGIN) * sizeof(uint32_t));
    for (size_t r = 0; r < rows; r++) {
        const float *row = data + r * inner;
        float mn = 3.40282347e+38f, mx = -3.40282347e+38f; /* f32::MAX, f32::MIN */
        for (size_t i = 0; i < inner; i++) {
            mn = fminf(mn, row[i]);
            mx = fmaxf(mx, row[i]);
        }
        float range = mx - mn;
        float scale, zero;
        if (range == 0.0f || unsigned_max == 0.0f) {
            scale = 1.0f;
            zero = 0.0f;
        } else if (is_fp4) {
            float sum = 0.0f;
            for (size_t i = 0; i < inner; i++) sum += row[i];
            float mean = sum / (float)inner;
            float dev = fmaxf(fabsf(mean - mn), fabsf(mx - mean));
            float max_dev = (dev == 0.0f) ? 1e-10f : dev;
            scale = max_dev / 4.0f;
            zero = mean;
        } else {
            float init_scale = range / unsigned_max;
            float lo = mn - init_scale;
            float hi = mx + init_scale;
            scale = (hi - lo) / unsigned_max;
            zero = lo + signed_bias * scale;
        }
        scales[r] = scale;
        zeros[r] = zero;
        float inv = (scale != 0.0f) ? 1.0f / scale : 0.0f;
        pack_row_affine(dt, row, inner, zero, inv, 1, words + r * kp);
    }
}

/* packed_tensor.rs:661-742 -- symmetric per-row: scale = max|row|/MAX_REPRESENTABLE
 * (all-zero row -> 1), lane = x * (1/scale) (inv = 1 when scale == 1), zeros = 0. */
void fnn_or_quant_per_channel_sym(int dt, const float *data, size_t rows, size_t inner,
                                  uint32_t *words, float *scales, float *zeros)
{
    float max_val;
    switch (dt) {
    case FNN_OR_I8: max_val = 127.0f; break;
    case FNN_OR_I4: max_val = 7.0f; break;
    case FNN_OR_U8: max_val = 255.0f; break;
    case FNN_OR_U4: max_val = 15.0f; break;
    case FNN_OR_F8: max_val = 240.0f; break;
    case FNN_OR_F8R: max_val = 57344.0f; break;
    default: max_val = 6.0f; break;
    }
    size_t kp = ceil_div(inner, (size_t)fnn_or_items(dt));
    memset(words, 0, (rows * kp + FNN_OR_SIMD_MARGIN) * sizeof(uint32_t));
    for (size_t r = 0; r < rows; r++) {
        const float *row = data + r * inner;
        float max_abs = 0.0f;
        for (size_t i = 0; i < inner; i++) max_abs = fmaxf(max_abs, fabsf(row[i]));
        float scale = (max_abs == 0.0f) ? 1.0f : max_abs / max_val;
        scales[r] = scale;
        zeros[r] = 0.0f;
        float inv = (scale != 1.0f) ? 1.0f / scale : 1.0f;
        /* lane = x * inv: (x - 0.0) * inv is the same value for every x */
        size_t items = (size_t)fnn_or_items(dt);
        float lane[8];
        for (size_t wd = 0; wd < kp; wd++) {
            for (size_t i = 0; i < items; i++) {
                size_t e = wd * items + i;
                lane[i] = (e < inner) ? row[e] * inv : 0.0f;
            }
            words[r * kp + wd] = fnn_or_pack_word(dt, lane);
        }
    }
}

/* Stable ascending order of f32 under partial_cmp (-0.0 == +0.0 keep input
 * order), as `sort_by(partial_cmp)` gives (packed_tensor.rs:35-36).  LSD radix
 * sort on a monotone key in which both zeros share one key. */
static int stable_sort_f32(const float *in, size_t n, float *out)
{
    uint32_t *keys = (uint32_t *)malloc(n * sizeof(uint32_t));
    uint32_t *idx_a = (uint32_t *)malloc(n * sizeof(uint32_t));
    uint32_t *idx_b = (uint32_t *)malloc(n * sizeof(uint32_t));
    if (!keys || !idx_a || !idx_b) { free(keys); free(idx_a); free(idx_b); return -1; }
    for (size_t i = 0; i < n; i++) {
        if (in[i] != in[i]) { free(keys); free(idx_a); free(idx_b); return -2; }
        uint32_t b;
        memcpy(&b, &in[i], 4);
        if (b == 0x80000000u) b = 0;
        keys[i] = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
        idx_a[i] = (uint32_t)i;
    }
    for (int pass = 0; pass < 4; pass++) {
        size_t count[257];
        memset(count, 0, sizeof(count));
        int sh = pass * 8;
        for (size_t i = 0; i < n; i++) count[((keys[idx_a[i]] >> sh) & 0xFF) + 1]++;
        for (int c = 0; c < 256; c++) count[c + 1] += count[c];
        for (size_t i = 0; i < n; i++) {
            uint32_t id = idx_a[i];
            idx_b[count[(keys[id] >> sh) & 0xFF]++] = id;
        }
        uint32_t *t = idx_a; idx_a = idx_b; idx_b = t;
    }
    for (size_t i = 0; i < n; i++) out[i] = in[idx_a[i]];
    free(keys); free(idx_a); free(idx_b);
    return 0;
}

/* packed_tensor.rs:18-75 -- 1-D k-means, 16 centroids, percentile init on the
 * sorted data, `iters` Lloyd steps with f32 sums in data order, final ascending
 * sort.  Returns -2 if a value is NaN (the reference panics on unwrap). */
int fnn_or_kmeans16(const float *values, size_t n, int iters, float *c)
{
    for (int i = 0; i < 16; i++) c[i] = 0.0f;
    if (n == 0) return 0;
    if (n == 1) {
        for (int i = 0; i < 16; i++) c[i] = values[0];
        return 0;
    }
    float *sorted = (float *)malloc(n * sizeof(float));
    if (!sorted) return -1;
    int rc = stable_sort_f32(values, n, sorted);
    if (rc) { free(sorted); return rc; }
    for (int i = 0; i < 16; i++) {
        float percentile = ((float)i + 0.5f) / 16.0f;
        float pos = percentile * (float)n;
        size_t idx = (size_t)pos; /* `as usize` truncates; pos >= 0 */
        if (idx > n - 1) idx = n - 1;
        c[i] = sorted[idx];
    }
    free(sorted);
    uint8_t *assign = (uint8_t *)malloc(n);
    if (!assign) return -1;
    for (int it = 0; it < iters; it++) {
        for (size_t vi = 0; vi < n; vi++) {
            float v = values[vi];
            float best_d = fabsf(v - c[0]);
            int best_c = 0;
            for (int ci = 1; ci < 16; ci++) {
                float d = fabsf(v - c[ci]);
                if (d < best_d) { best_d = d; best_c = ci; }
            }
            assign[vi] = (uint8_t)best_c;
        }
        size_t counts[16];
        float sums[16];
        for (int ci = 0; ci < 16; ci++) { counts[ci] = 0; sums[ci] = 0.0f; }
        for (size_t vi = 0; vi < n; vi++) {
            counts[assign[vi]] += 1;
            sums[assign[vi]] += values[vi];
        }
        for (int ci = 0; ci < 16; ci++)
            if (counts[ci] > 0) c[ci] = sums[ci] / (float)counts[ci];
    }
    free(assign);
    /* sort_unstable_by(partial_cmp) on 16 values: insertion sort; only the
     * relative order of equal keys (identical values, or -0/+0) could differ. */
    for (int i = 1; i < 16; i++) {
        float x = c[i];
        int j = i - 1;
        while (j >= 0 && c[j] > x) { c[j + 1] = c[j]; j--; }
        c[j + 1] = x;
    }
    return 0;
}

/* packed_tensor.rs:77-88 */
static inline uint32_t nearest_cb(float v, const float *cb)
{
    float best_d = fabsf(v - cb[0]);
    uint32_t best_i = 0;
    for (uint32_t ci = 1; ci < 16; ci++) {
        float d = fabsf(v - cb[ci]);
        if (d < best_d) { best_d = d; best_i = ci; }
    }
    return best_i;
}

/* packed_tensor.rs:1209-1313 -- per-block max-abs scales, one global codebook
 * learnt on block-normalised values, nibble = nearest centroid.  A word that
 * straddles two blocks (qblock % 8 != 0) is overwritten by the later block,
 * exactly as `packed[chunk_idx] = default; *word = w` does there. */
int fnn_or_quant_codebook(const float *data, size_t rows, size_t inner, size_t qblock,
                          uint32_t *words, float *block_scales, float *codebook)
{
    if (qblock == 0) return -3;
    size_t bpr = ceil_div(inner, qblock);
    size_t nblocks = rows * bpr;
    size_t numel = rows * inner;
    size_t kp = ceil_div(inner, 8);
    float *norm = (float *)malloc((numel + 1) * sizeof(float));
    if (!norm) return -1;
    size_t nn = 0;
    for (size_t blk = 0; blk < nblocks; blk++) {
        size_t row = blk / bpr, bir = blk % bpr;
        size_t base = row * inner + bir * qblock;
        size_t end = base + qblock;
        if (end > (row + 1) * inner) end = (row + 1) * inner;
        float max_abs = 0.0f;
        for (size_t i = base; i < end; i++) max_abs = fmaxf(max_abs, fabsf(data[i]));
        block_scales[blk] = max_abs;
        if (max_abs > 0.0f) {
            float inv = 1.0f / max_abs;
            for (size_t i = base; i < end; i++) norm[nn++] = data[i] * inv;
        } else {
            for (size_t i = base; i < end; i++) norm[nn++] = 0.0f;
        }
    }
    int rc = fnn_or_kmeans16(norm, nn, 30, codebook);
    free(norm);
    if (rc) return rc;
    memset(words, 0, (rows * kp + FNN_OR_SIMD_MARGIN) * sizeof(uint32_t));
    for (size_t row = 0; row < rows; row++) {
        for (size_t blk = 0; blk < bpr; blk++) {
            float s = block_scales[row * bpr + blk];
            float inv = (s > 0.0f) ? 1.0f / s : 0.0f;
            size_t base = row * inner + blk * qblock;
            size_t end = base + qblock;
            if (end > (row + 1) * inner) end = (row + 1) * inner;
            size_t blen = end - base;
            for (size_t eb = 0; eb < blen; eb += 8) {
                size_t word_in_row = (blk * qblock + eb) / 8;
                uint32_t w = 0;
                for (size_t i = 0; i < 8; i++) {
                    size_t e = base + eb + i;
                    if (e >= end || e >= numel) continue;
                    w |= nearest_cb(data[e] * inv, codebook) << (4 * i);
                }
                words[row * kp + word_in_row] = w;
            }
        }
    }
    return 0;
}

/* compiler/passes/quantization.rs:144-156 -- [K,N] row-major -> [N,K]. */
void fnn_or_transpose(const float *src, size_t k, size_t n, float *dst)
{
    for (size_t kk = 0; kk < k; kk++)
        for (size_t nn = 0; nn < n; nn++) dst[nn * k + kk] = src[kk * n + nn];
}

/* ------------------------------------------------------------------------ */
/* dequantise                                                                 */
/* ------------------------------------------------------------------------ */

/* packed_tensor.rs:438-462 scale_for_row / zero_for_row with the group rule
 * of backend/cpu/matmul.rs:147-149 (group = rows / n_scales when fewer). */
static inline float per_row(const float *v, size_t n, size_t rows, size_t row, float dflt)
{
    if (n == 0) return dflt;
    if (n == 1) return v[0];
    if (rows > n) return v[row / (rows / n)];
    return v[row];
}

/* packed_tensor.rs:469-521 get_or_init_f32_weights: `unpacked * scale + zero`
 * for per-row types, `scales[row*bpr + col/qb] * codebook[nibble]` for the
 * codebook type (also :367-403). */
int fnn_or_dequant(int dt, const uint32_t *words, size_t rows, size_t inner,
                   const float *scales, size_t n_scales, const float *zeros, size_t n_zeros,
                   size_t qblock, const float *codebook, float *out)
{
    size_t items = (size_t)fnn_or_items(dt);
    if (!items) return -1;
    size_t kp = ceil_div(inner, items);
    float lane[8];
    if (dt == FNN_OR_I4CB) {
        if (!codebook || qblock == 0) return -3;
        size_t bpr = ceil_div(inner, qblock);
        if (n_scales < rows * bpr) return -4;
        for (size_t r = 0; r < rows; r++)
            for (size_t c = 0; c < inner; c++) {
                uint32_t w = words[r * kp + c / 8];
                uint32_t nib = (w >> (4 * (c % 8))) & 0xF;
                out[r * inner + c] = scales[r * bpr + c / qblock] * codebook[nib];
            }
        return 0;
    }
    for (size_t r = 0; r < rows; r++) {
        float s = per_row(scales, n_scales, rows, r, 1.0f);
        float z = per_row(zeros, n_zeros, rows, r, 0.0f);
        for (size_t wd = 0; wd < kp; wd++) {
            fnn_or_unpack_word(dt, words[r * kp + wd], lane);
            for (size_t i = 0; i < items; i++) {
                size_t c = wd * items + i;
                if (c < inner) out[r * inner + c] = lane[i] * s + z;
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* f32-activation quantised MatMul                                            */
/* ------------------------------------------------------------------------ */

/* microkernels/mod.rs:273-280 fma_f32_scalar */
static float dot_scalar(const float *a, const float *b, size_t len)
{
    float acc = 0.0f;
    for (size_t i = 0; i < len; i++) acc += a[i] * b[i];
    return acc;
}

static double dot_f64(const float *a, const float *b, size_t len)
{
    double acc = 0.0;
    for (size_t i = 0; i < len; i++) acc += (double)a[i] * (double)b[i];
    return acc;
}

#if defined(__x86_64__)
/* microkernels/mod.rs:340-383 fma_f32_avx2 and :240-251 hsum256_ps: four 8-lane
 * fused-multiply-add accumulators over 32-element steps, then 8-element steps
 * on acc0, pairwise combine, horizontal sum, scalar tail. */
__attribute__((target("avx2,fma"))) static float dot_avx2(const float *a, const float *b,
                                                          size_t len)
{
    __m256 acc0 = _mm256_setzero_ps(), acc1 = _mm256_setzero_ps();
    __m256 acc2 = _mm256_setzero_ps(), acc3 = _mm256_setzero_ps();
    size_t i = 0;
    for (; i + 32 <= len; i += 32) {
        acc0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i), _mm256_loadu_ps(b + i), acc0);
        acc1 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 8), _mm256_loadu_ps(b + i + 8), acc1);
        acc2 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 16), _mm256_loadu_ps(b + i + 16), acc2);
        acc3 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 24), _mm256_loadu_ps(b + i + 24), acc3);
    }
    for (; i + 8 <= len; i += 8)
        acc0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i), _mm256_loadu_ps(b + i), acc0);
    __m256 comb = _mm256_add_ps(_mm256_add_ps(acc0, acc1), _mm256_add_ps(acc2, acc3));
    __m128 hi = _mm256_extractf128_ps(comb, 1);
    __m128 lo = _mm256_castps256_ps128(comb);
    __m128 s = _mm_add_ps(lo, hi);
    __m128 sh = _mm_shuffle_ps(s, s, 0x0E);
    __m128 s2 = _mm_add_ps(s, sh);
    __m128 sh2 = _mm_shuffle_ps(s2, s2, 0x01);
    float total = _mm_cvtss_f32(_mm_add_ss(s2, sh2));
    for (; i < len; i++) total += a[i] * b[i];
    return total;
}
#endif

static float dot_order(const float *a, const float *b, size_t len, int order)
{
#if defined(__x86_64__)
    if (order == 1 && __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma"))
        return dot_avx2(a, b, len);
#endif
    (void)order;
    return dot_scalar(a, b, len);
}

/* Intended codebook MatMul: out = A . deq(W)^T with deq the [N,K] matrix of
 * packed_tensor.rs:476-495.  As written, backend/cpu/matmul.rs:206-212 hands
 * that [N,K] buffer to a row-major [K,N] SGEMM (blas.rs:29-31), i.e. it
 * multiplies by reshape(deq,[K,N]); i4cb_as_written reproduces that. */
static int qmatmul_codebook(const uint32_t *words, size_t n, size_t k, const float *scales,
                            size_t n_scales, size_t qblock, const float *codebook,
                            const float *a, size_t m, float *out, int order, int as_written)
{
    float *deq = (float *)malloc((n * k + 1) * sizeof(float));
    if (!deq) return -1;
    int rc = fnn_or_dequant(FNN_OR_I4CB, words, n, k, scales, n_scales, NULL, 0, qblock, codebook,
                            deq);
    if (rc) { free(deq); return rc; }
    if (as_written) {
        for (size_t mi = 0; mi < m; mi++)
            for (size_t ni = 0; ni < n; ni++) {
                double acc = 0.0;
                float accf = 0.0f;
                for (size_t ki = 0; ki < k; ki++) {
                    float wv = deq[ki * n + ni];
                    acc += (double)a[mi * k + ki] * (double)wv;
                    accf += a[mi * k + ki] * wv;
                }
                out[mi * n + ni] = (order == 2) ? (float)acc : accf;
            }
    } else {
        for (size_t mi = 0; mi < m; mi++)
            for (size_t ni = 0; ni < n; ni++) {
                if (order == 2)
                    out[mi * n + ni] = (float)dot_f64(a + mi * k, deq + ni * k, k);
                else
                    out[mi * n + ni] = dot_order(a + mi * k, deq + ni * k, k, order);
            }
    }
    free(deq);
    return 0;
}

/* microkernels/gemm.rs:1982-2088 gemm_batch_packed_simd with the epilogue of
 * microkernels/mod.rs:283-295:
 *   for each K-tile: for each weight row n: unpack the tile to f32, then for
 *   every batch row m: out[m,n] += dot(unpacked, a[m, tile]);
 *   finally out[m,n] = out[m,n]*scale[n] + zero[n]*sum_k a[m,k] (sequential sum).
 * k_tile is the reference's k_block_size() (gemm.rs:23-32: 4096..65536). */
int fnn_or_qmatmul(int dt, const uint32_t *words, size_t n, size_t k, const float *scales,
                   size_t n_scales, const float *zeros, size_t n_zeros, size_t qblock,
                   const float *codebook, const float *a, size_t m, float *out, int order,
                   size_t k_tile, int i4cb_as_written)
{
    size_t items = (size_t)fnn_or_items(dt);
    if (!items) return -1;
    if (dt == FNN_OR_I4CB)
        return qmatmul_codebook(words, n, k, scales, n_scales, qblock, codebook, a, m, out, order,
                                i4cb_as_written);
    if (k_tile == 0) k_tile = 65536;
    size_t kp = ceil_div(k, items);
    size_t tile_alloc = (k_tile < k ? k_tile : k) + 8;
    float *buf = (float *)malloc(tile_alloc * sizeof(float));
    double *acc64 = NULL;
    if (!buf) return -1;
    if (order == 2) {
        acc64 = (double *)calloc(m * n + 1, sizeof(double));
        if (!acc64) { free(buf); return -1; }
    }
    for (size_t i = 0; i < m * n; i++) out[i] = 0.0f;
    float lane[8];
    for (size_t k0 = 0; k0 < k; k0 += k_tile) {
        size_t k1 = (k0 + k_tile < k) ? k0 + k_tile : k;
        size_t klen = k1 - k0;
        size_t p0 = k0 / items, p1 = ceil_div(k1, items);
        for (size_t row = 0; row < n; row++) {
            for (size_t p = p0; p < p1; p++) {
                fnn_or_unpack_word(dt, words[row * kp + p], lane);
                for (size_t j = 0; j < items; j++) {
                    size_t idx = p * items + j;
                    if (idx >= k0 && idx < k1) buf[idx - k0] = lane[j];
                }
            }
            for (size_t bi = 0; bi < m; bi++) {
                const float *act = a + bi * k + k0;
                if (order == 2)
                    acc64[bi * n + row] += dot_f64(buf, act, klen);
                else
                    out[bi * n + row] += dot_order(buf, act, klen, order);
            }
        }
    }
    for (size_t bi = 0; bi < m; bi++) {
        const float *act = a + bi * k;
        if (order == 2) {
            double s = 0.0;
            for (size_t i = 0; i < k; i++) s += (double)act[i];
            for (size_t row = 0; row < n; row++) {
                double sc = per_row(scales, n_scales, n, row, 1.0f);
                double z = per_row(zeros, n_zeros, n, row, 0.0f);
                out[bi * n + row] = (float)(acc64[bi * n + row] * sc + z * s);
            }
        } else {
            float s = 0.0f;
            for (size_t i = 0; i < k; i++) s += act[i];
            for (size_t row = 0; row < n; row++) {
                float sc = per_row(scales, n_scales, n, row, 1.0f);
                float z = per_row(zeros, n_zeros, n, row, 0.0f);
                out[bi * n + row] = out[bi * n + row] * sc + z * s;
            }
        }
    }
    free(buf);
    free(acc64);
    return 0;
}

/* microkernels/activations.rs:557-562 (GELU, tanh form), :591-593 (SiLU);
 * ReLU is max(x, 0). */
float fnn_or_act(float x, int act)
{
    switch (act) {
    case FNN_OR_ACT_RELU: return x > 0.0f ? x : 0.0f;
    case FNN_OR_ACT_GELU: {
        float x3 = x * x * x;
        float t = 0.7978846f * (x + 0.044715f * x3);
        return 0.5f * x * (1.0f + tanhf(t));
    }
    case FNN_OR_ACT_SILU: return x / (1.0f + expf(-x));
    default: return x;
    }
}

/* The unfused chain matmul_q -> add_f32 (bias broadcast over rows) -> act that a
 * MatMul+Add+Act pattern means (compiler/passes/fusion/matmul_add_relu.rs:92-110;
 * f32 form `act(out + bias[i % n])` at backend/cpu/matmul.rs:64-72). */
void fnn_or_bias_act(float *out, size_t m, size_t n, const float *bias, int act)
{
    for (size_t i = 0; i < m * n; i++) {
        float v = out[i];
        if (bias) v = v + bias[i % n];
        out[i] = fnn_or_act(v, act);
    }
}

/* ------------------------------------------------------------------------ */
/* I8-activation MatMul                                                       */
/* ------------------------------------------------------------------------ */

/* "dequantize_activations", per-tensor form (backend/cpu/mod.rs:7063-7086): header scale
 * (1.0 if absent) and zero (0.0 if absent), out[i] = (q as f32)*scale + zp, q = 0 past the data. */
void fnn_or_dequantize_activations(const uint8_t *payload, size_t payload_len, float *out, size_t n)
{
    float scale = 1.0f, zp = 0.0f;
    if (payload_len >= 4) memcpy(&scale, payload, 4);
    if (payload_len >= 8) memcpy(&zp, payload + 4, 4);
    for (size_t i = 0; i < n; i++) {
        int8_t q = (8 + i < payload_len) ? (int8_t)payload[8 + i] : 0;
        volatile float prod = (float)q * scale;   /* two roundings, no contraction */
        out[i] = prod + zp;
    }
}

/* backend/cpu/mod.rs:6987-7007 -- dynamic per-tensor mode: scale = max|x|/127
 * (1 when all zero), zp = 0, q = clamp(round((x - zp)/scale), -128, 127);
 * payload = [scale f32 LE][zp f32 LE][numel x i8]. */
void fnn_or_quantize_activations(const float *x, size_t numel, uint8_t *payload)
{
    float max_abs = 0.0f;
    for (size_t i = 0; i < numel; i++) max_abs = fmaxf(max_abs, fabsf(x[i]));
    float scale = (max_abs == 0.0f) ? 1.0f : max_abs / 127.0f;
    fnn_or_quantize_activations_calibrated(x, numel, scale, 0.0f, payload);
}

/* backend/cpu/mod.rs:6978-6986,6994-7006 -- calibrated per-tensor (scale, zp). */
void fnn_or_quantize_activations_calibrated(const float *x, size_t numel, float scale, float zp,
                                            uint8_t *payload)
{
    memcpy(payload, &scale, 4);
    memcpy(payload + 4, &zp, 4);
    for (size_t i = 0; i < numel; i++) {
        float q = clampf(roundf((x[i] - zp) / scale), -128.0f, 127.0f);
        payload[8 + i] = (uint8_t)(int8_t)sat_i32(q, -128, 127);
    }
}

/* "quantize_activations", per-channel form (backend/cpu/mod.rs:6941-6975), loop for loop as written there:
 * the header, then for every channel in ascending order its chunk of codes, each chunk written from the first
 * byte behind the header (`header_offset + local`), so a later channel overwrites an earlier one.  x_len = length of
 * the f32 input view, payload_len = length of the output byte view; bytes the loops do not reach keep their value.
 * Returns -1 where the reference would panic on a slice index (header does not fit), else 0. */
int fnn_or_quantize_activations_per_channel(const float *x, size_t x_len, size_t numel, size_t num_channels,
                                            const float *scales, const float *zero_points, uint8_t *payload,
                                            size_t payload_len)
{
    if (num_channels == 0) return -1;
    size_t chunk_size = numel / num_channels;
    size_t header_offset = 4 + 4 + num_channels * 8;
    if (payload_len < header_offset) return -1;
    uint32_t nc32 = (uint32_t)num_channels, chunk32 = (uint32_t)chunk_size;
    memcpy(payload, &nc32, 4);
    memcpy(payload + 4, &chunk32, 4);
    size_t scale_start = 8, zp_start = 8 + num_channels * 4;
    for (size_t ch = 0; ch < num_channels; ch++) {
        float scale = scales[ch], zp = zero_points[ch];
        memcpy(payload + scale_start + ch * 4, &scale, 4);
        memcpy(payload + zp_start + ch * 4, &zp, 4);
        size_t ch_start = ch * chunk_size;
        size_t ch_end = ch_start + chunk_size < x_len ? ch_start + chunk_size : x_len;
        for (size_t i = ch_start; i < ch_end; i++) {
            size_t local = i - ch_start;
            if (header_offset + local < payload_len) {
                int8_t q = 0;
                if (scale != 0.0f)
                    q = (int8_t)sat_i32(clampf(roundf((x[i] - zp) / scale), -128.0f, 127.0f), -128, 127);
                payload[header_offset + local] = (uint8_t)q;
            }
        }
    }
    return 0;
}

/* "dequantize_activations", per-channel form (backend/cpu/mod.rs:7026-7061): channel count and chunk from the
 * header, out[ch*chunk + local] = (q[local] as f32)*scale[ch] + zp[ch], every channel reading the block behind the
 * header from its start, q = 0 past the payload.  Returns -1 where the reference would panic (header slices past
 * the payload), else 0. */
int fnn_or_dequantize_activations_per_channel(const uint8_t *payload, size_t payload_len, float *out, size_t out_len)
{
    if (payload_len < 8) return -1;
    uint32_t nc32, chunk32;
    memcpy(&nc32, payload, 4);
    memcpy(&chunk32, payload + 4, 4);
    size_t nc = nc32, chunk_size = chunk32;
    size_t data_start = 8 + nc * 8;
    if (data_start > payload_len) return -1;
    for (size_t ch = 0; ch < nc; ch++) {
        float scale, zp;
        memcpy(&scale, payload + 8 + ch * 4, 4);
        memcpy(&zp, payload + 8 + nc * 4 + ch * 4, 4);
        size_t ch_start = ch * chunk_size;
        size_t ch_end = ch_start + chunk_size < out_len ? ch_start + chunk_size : out_len;
        for (size_t i = ch_start; i < ch_end; i++) {
            size_t di = data_start + (i - ch_start);
            int8_t q = di < payload_len ? (int8_t)payload[di] : 0;
            volatile float prod = (float)q * scale;   /* two roundings, no contraction */
            out[i] = prod + zp;
        }
    }
    return 0;
}

/* microkernels/gemm.rs:1641-1788 (I8 weights) and :1795-1975 (I4 weights),
 * payload parsing microkernels/mod.rs:316-337.
 * zp_a == 0: acc = sum q_w*q_a exactly (i32 in the scalar build; the AVX2 and
 * the I4 scalar builds sum the same integers in f32, exact below 2^24);
 *   out = (acc*sa)*sw + zw*(qsum*sa + K*za).
 * zp_a != 0: per-lane f32: a = q*sa + za; acc += a*q_w; asum += a (in k order);
 *   out = acc*sw + zw*asum. */
int fnn_or_qmatmul_i8act(int dt, const uint32_t *words, size_t n, size_t k, const float *scales,
                         size_t n_scales, const float *zeros, size_t n_zeros,
                         const uint8_t *payload, size_t payload_len, size_t m, float *out,
                         int32_t *acc_out)
{
    if (dt != FNN_OR_I8 && dt != FNN_OR_I4) return -1;
    size_t items = (size_t)fnn_or_items(dt);
    size_t kp = ceil_div(k, items);
    float sa = 1.0f, za = 0.0f;
    if (payload_len >= 4) memcpy(&sa, payload, 4);
    if (payload_len >= 8) memcpy(&za, payload + 4, 4);
    if (payload_len < 8 + m * k) return -2;
    const int8_t *qa = (const int8_t *)(payload + 8);
    for (size_t bi = 0; bi < m; bi++) {
        for (size_t row = 0; row < n; row++) {
            float sw = per_row(scales, n_scales, n, row, 1.0f);
            float zw = per_row(zeros, n_zeros, n, row, 0.0f);
            if (za != 0.0f) {
                float acc = 0.0f, asum = 0.0f;
                for (size_t kk = 0; kk < k; kk++) {
                    uint32_t w = words[row * kp + kk / items];
                    float qw = (dt == FNN_OR_I8)
                                   ? (float)(int8_t)(w >> (8 * (kk % 4)))
                                   : (float)nib_s(w, (int)(kk % 8));
                    float av = (float)qa[bi * k + kk] * sa + za;
                    if (dt == FNN_OR_I8) acc += av * qw; else acc += qw * av;
                    asum += av;
                }
                out[bi * n + row] = acc * sw + zw * asum;
                if (acc_out) acc_out[bi * n + row] = 0;
                continue;
            }
            int32_t acc = 0, qsum = 0;
            for (size_t kk = 0; kk < k; kk++) {
                uint32_t w = words[row * kp + kk / items];
                int32_t qw = (dt == FNN_OR_I8) ? (int32_t)(int8_t)(w >> (8 * (kk % 4)))
                                               : nib_s(w, (int)(kk % 8));
                int32_t q = qa[bi * k + kk];
                acc += qw * q;
                qsum += q;
            }
            if (acc_out) acc_out[bi * n + row] = acc;
            float dot = (float)acc * sa;
            float input_sum = (float)qsum * sa + (float)k * za;
            out[bi * n + row] = dot * sw + zw * input_sum;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* quantised Conv2d (I8 weights)                                              */
/* ------------------------------------------------------------------------ */

/* packed_conv.rs:49-62 */
size_t fnn_or_conv_out_size(size_t input, size_t kernel, size_t stride, size_t padding,
                            size_t dilation)
{
    size_t dk = (kernel - 1) * dilation + 1;
    if (input + 2 * padding >= dk) return (input + 2 * padding - dk) / stride + 1;
    return 0;
}

/* The algorithm packed_conv.rs evidently intends (its im2col_pack_i8x4 as
 * written appends words after a zero-filled buffer, :159,211-228, so the
 * as-written activations are mostly zero; that defect is not reproduced):
 *   per image and group (packed_conv.rs:1142-1195):
 *     col[p, c*KH*KW + i*KW + j] = x[c, oh*s + i*d - pad, ow*s + j*d - pad] or 0
 *         (im2col.rs:32-52), p = oh*Wout + ow;
 *     (mn, mx) over the whole col matrix incl. padding zeros (im2col.rs:496-507);
 *     sa = (mx-mn)/255 (1 if range <= 0), za = mn + 128*sa (0 if range <= 0),
 *     q_a = clamp(round((x - za)*(1/sa)), -128, 127)          (packed_conv.rs:149-156,199-201);
 *   per output channel (packed_conv.rs:469-484): qb = sum q_w, sab = sa*sw,
 *     bias_q = round(bias/sab) as i32, w_term = sw*qb, zp_prod = za*zw;
 *   per pixel (:492-505): r = sa*sum q_a; acc = bias_q + sum q_a*q_w (i32);
 *     val = acc*sab + zw*r + za*w_term + zp_prod*K, left to right in f32;
 *   activation (:571,604-606: SiLU x/(1+exp(-x)); GELU val*0.5*(1+tanh(val*0.7978846*(1+0.044715*val*val))));
 *   y[b, oc, p] = val                                          (:1176-1188). */
static int qconv2d_int(int bits, const float *x, size_t b, size_t c, size_t h, size_t w,
                       const uint32_t *words, size_t oc, const float *scales, size_t n_scales,
                       const float *zeros, size_t n_zeros, const float *bias, size_t kh, size_t kw,
                       size_t stride, size_t pad, size_t dil, size_t groups, int act, float *y,
                       int32_t *acc_out, float *act_scale_out, float *act_zero_out)
{
    const size_t items = (bits == 4) ? 8 : 4;
    if (groups == 0 || c % groups || oc % groups) return -1;
    size_t cg = c / groups, ocg = oc / groups;
    size_t ho = fnn_or_conv_out_size(h, kh, stride, pad, dil);
    size_t wo = fnn_or_conv_out_size(w, kw, stride, pad, dil);
    size_t np = ho * wo;
    size_t kk = cg * kh * kw;
    size_t kp = ceil_div(kk, items);
    float *col = (float *)malloc((np * kk + 1) * sizeof(float));
    int8_t *qa = (int8_t *)malloc(np * kk + 1);
    if (!col || !qa) { free(col); free(qa); return -2; }
    for (size_t nn = 0; nn < b; nn++) {
        for (size_t g = 0; g < groups; g++) {
            const float *xin = x + nn * c * h * w + g * cg * h * w;
            float mn = INFINITY, mx = -INFINITY;
            for (size_t oh = 0; oh < ho; oh++)
                for (size_t ow = 0; ow < wo; ow++) {
                    size_t p = oh * wo + ow;
                    for (size_t ic = 0; ic < cg; ic++)
                        for (size_t i = 0; i < kh; i++)
                            for (size_t j = 0; j < kw; j++) {
                                size_t ih = oh * stride + i * dil - pad; /* wraps when < 0 */
                                size_t iw = ow * stride + j * dil - pad;
                                float v = 0.0f;
                                if (ih < h && iw < w) v = xin[(ic * h + ih) * w + iw];
                                col[p * kk + ic * kh * kw + i * kw + j] = v;
                            }
                }
            for (size_t i = 0; i < np * kk; i++) {
                mn = fminf(mn, col[i]);
                mx = fmaxf(mx, col[i]);
            }
            float range = mx - mn;
            float sa, za;
            if (bits == 4) { /* packed_conv.rs:260-263: the zero point is formed in either case */
                sa = (range > 0.0f) ? range / 15.0f : 1.0f;
                za = mn + 8.0f * sa;
            } else {
                sa = (range > 0.0f) ? range / 255.0f : 1.0f;
                za = (range > 0.0f) ? mn + 128.0f * sa : 0.0f;
            }
            const float qlo = (bits == 4) ? -8.0f : -128.0f, qhi = (bits == 4) ? 7.0f : 127.0f;
            float inv = (sa != 0.0f) ? 1.0f / sa : 0.0f;
            if (act_scale_out) act_scale_out[nn * groups + g] = sa;
            if (act_zero_out) act_zero_out[nn * groups + g] = za;
            for (size_t i = 0; i < np * kk; i++)
                qa[i] = (int8_t)sat_i32(clampf(roundf((col[i] - za) * inv), qlo, qhi), (int32_t)qlo,
                                        (int32_t)qhi);
            for (size_t f = 0; f < ocg; f++) {
                size_t ch = g * ocg + f;
                const uint32_t *wrow = words + ch * kp;
                int32_t qb = 0;
                for (size_t p = 0; p < kp; p++)
                    qb += (bits == 4) ? fnn_or_i4x8_sum(wrow[p]) : fnn_or_i8x4_sum(wrow[p]);
                float sw = (n_scales > 1) ? scales[ch] : scales[0];
                float zw = (n_zeros > 1) ? zeros[ch] : (n_zeros ? zeros[0] : 0.0f);
                float sab = sa * sw;
                int32_t bias_q = 0;
                if (bias) bias_q = sat_i32(roundf(bias[ch] / sab), -2147483647 - 1, 2147483647);
                float w_term = sw * (float)qb;
                float zp_prod = za * zw;
                for (size_t p = 0; p < np; p++) {
                    const int8_t *arow = qa + p * kk;
                    int32_t qasum = 0;
                    int32_t acc = bias_q;
                    for (size_t e = 0; e < kk; e++) {
                        int32_t qw = (bits == 4) ? nib_s(wrow[e / 8], (int)(e % 8))
                                                 : (int32_t)(int8_t)(wrow[e / 4] >> (8 * (e % 4)));
                        qasum += arow[e];
                        acc += arow[e] * qw;
                    }
                    float r = sa * (float)qasum;
                    float val = (float)acc * sab + zw * r + za * w_term + zp_prod * (float)kk;
                    if (act == FNN_OR_ACT_RELU) {
                        val = fmaxf(val, 0.0f);
                    } else if (act == FNN_OR_ACT_SILU) {
                        val = val / (1.0f + expf(-val));
                    } else if (act == FNN_OR_ACT_GELU) {
                        val = val * 0.5f *
                              (1.0f + tanhf(val * 0.7978846f * (1.0f + 0.044715f * val * val)));
                    }
                    size_t oidx = (nn * oc + ch) * np + p;
                    y[oidx] = val;
                    if (acc_out) acc_out[oidx] = acc;
                }
            }
        }
    }
    free(col);
    free(qa);
    return 0;
}

int fnn_or_qconv2d_i8(const float *x, size_t b, size_t c, size_t h, size_t w,
                      const uint32_t *words, size_t oc, const float *scales, size_t n_scales,
                      const float *zeros, size_t n_zeros, const float *bias, size_t kh, size_t kw,
                      size_t stride, size_t pad, size_t dil, size_t groups, int act, float *y,
                      int32_t *acc_out, float *act_scale_out, float *act_zero_out)
{
    return qconv2d_int(8, x, b, c, h, w, words, oc, scales, n_scales, zeros, n_zeros, bias, kh, kw,
                       stride, pad, dil, groups, act, y, acc_out, act_scale_out, act_zero_out);
}

/* conv2d_packed_i4x8 (packed_conv.rs:1202-1280): the same lowering with I4x8 weights and the
 * im2col matrix quantised to 16 levels, sa = range/15 (1 if range <= 0), za = mn + 8*sa,
 * q_a = clamp(round((x - za)*(1/sa)), -8, 7) (im2col_pack_i4x8, :236-283, which fills its
 * words in place, so the as-written and the intended algorithm coincide); per channel and per
 * pixel exactly the four-term formula of the 8-bit kernel (gemm_packed_i4x8_fused_raw, :659-841). */
int fnn_or_qconv2d_i4(const float *x, size_t b, size_t c, size_t h, size_t w,
                      const uint32_t *words, size_t oc, const float *scales, size_t n_scales,
                      const float *zeros, size_t n_zeros, const float *bias, size_t kh, size_t kw,
                      size_t stride, size_t pad, size_t dil, size_t groups, int act, float *y,
                      int32_t *acc_out, float *act_scale_out, float *act_zero_out)
{
    return qconv2d_int(4, x, b, c, h, w, words, oc, scales, n_scales, zeros, n_zeros, bias, kh, kw,
                       stride, pad, dil, groups, act, y, acc_out, act_scale_out, act_zero_out);
}

/* "conv2d_i8_i8" / "conv2d_i4_i8" (backend/cpu/mod.rs:3848-4098): the activation arrives as an I8 payload
 * [scale f32][zero f32][B*C*H*W x i8] (quantize_activations); per image and group the int8 values
 * are gathered with im2col_i8 (packed_conv.rs:69-115, padding taps are the integer 0), then
 *   I8 weights: gemm_packed_i8x4_fused_raw with (sa, za) of the payload, i.e. the four-term
 *     formula of conv2d_packed_i8x4 incl. the integer bias (packed_conv.rs:444-625);
 *   I4 weights: gemm_cpu_flat_i8_i4x8 (microkernels/gemm.rs:1795-1975) on [sa][za][col],
 *     then `+ bias` in f32 and the activation (mod.rs:4002-4032);
 * results go to NCHW. */
int fnn_or_qconv2d_i8payload(int dt, const uint8_t *payload, size_t payload_len, size_t c, size_t h,
                             size_t w, const uint32_t *words, size_t oc, const float *scales,
                             size_t n_scales, const float *zeros, size_t n_zeros, const float *bias,
                             size_t kh, size_t kw, size_t stride, size_t pad, size_t dil,
                             size_t groups, int act, float *y)
{
    if (dt != FNN_OR_I8 && dt != FNN_OR_I4) return -1;
    if (groups == 0 || c % groups || oc % groups || payload_len < 8) return -1;
    float sa, za;
    memcpy(&sa, payload, 4);
    memcpy(&za, payload + 4, 4);
    const int8_t *x8 = (const int8_t *)(payload + 8);
    size_t chw = c * h * w;
    size_t b = chw ? (payload_len - 8) / chw : 0;
    size_t cg = c / groups, ocg = oc / groups;
    size_t ho = fnn_or_conv_out_size(h, kh, stride, pad, dil);
    size_t wo = fnn_or_conv_out_size(w, kw, stride, pad, dil);
    size_t np = ho * wo, kk = cg * kh * kw;
    size_t items = (dt == FNN_OR_I4) ? 8 : 4, kp = ceil_div(kk, items);
    uint8_t *pl = (uint8_t *)malloc(8 + np * kk + 1);
    float *tmp = (float *)malloc((np * ocg + 1) * sizeof(float));
    if (!pl || !tmp) { free(pl); free(tmp); return -2; }
    memcpy(pl, payload, 8);
    int8_t *col = (int8_t *)(pl + 8);
    for (size_t nn = 0; nn < b; nn++)
        for (size_t g = 0; g < groups; g++) {
            const int8_t *xin = x8 + nn * chw + g * cg * h * w;
            for (size_t oh = 0; oh < ho; oh++)
                for (size_t ow = 0; ow < wo; ow++)
                    for (size_t ic = 0; ic < cg; ic++)
                        for (size_t i = 0; i < kh; i++)
                            for (size_t j = 0; j < kw; j++) {
                                size_t ih = oh * stride + i * dil, iw = ow * stride + j * dil;
                                int8_t v = 0;
                                if (ih < h + pad && iw < w + pad && ih >= pad && iw >= pad)
                                    v = xin[(ic * h + (ih - pad)) * w + (iw - pad)];
                                col[(oh * wo + ow) * kk + ic * kh * kw + i * kw + j] = v;
                            }
            const uint32_t *wg = words + g * ocg * kp;
            const float *sg = (n_scales > 1) ? scales + g * ocg : scales;
            const float *zg = (n_zeros > 1) ? zeros + g * ocg : zeros;
            if (dt == FNN_OR_I4) {
                int rc = fnn_or_qmatmul_i8act(dt, wg, ocg, kk, sg, n_scales > 1 ? ocg : n_scales, zg,
                                              n_zeros > 1 ? ocg : n_zeros, pl, 8 + np * kk, np, tmp, NULL);
                if (rc) { free(pl); free(tmp); return rc; }
                for (size_t p = 0; p < np; p++)
                    for (size_t f = 0; f < ocg; f++) {
                        float val = tmp[p * ocg + f];
                        if (bias) val += bias[g * ocg + f];
                        if (act == FNN_OR_ACT_RELU) val = fmaxf(val, 0.0f);
                        else if (act == FNN_OR_ACT_SILU) val = val / (1.0f + expf(-val));
                        else if (act == FNN_OR_ACT_GELU)
                            val = val * 0.5f * (1.0f + tanhf(val * 0.7978846f * (1.0f + 0.044715f * val * val)));
                        y[(nn * oc + g * ocg + f) * np + p] = val;
                    }
                continue;
            }
            for (size_t f = 0; f < ocg; f++) {
                size_t ch = g * ocg + f;
                const uint32_t *wrow = wg + f * kp;
                int32_t qb = 0;
                for (size_t p = 0; p < kp; p++) qb += fnn_or_i8x4_sum(wrow[p]);
                float sw = (n_scales > 1) ? sg[f] : sg[0];
                float zw = (n_zeros > 1) ? zg[f] : (n_zeros ? zg[0] : 0.0f);
                float sab = sa * sw;
                int32_t bias_q = 0;
                if (bias) bias_q = sat_i32(roundf(bias[ch] / sab), -2147483647 - 1, 2147483647);
                float w_term = sw * (float)qb, zp_prod = za * zw;
                for (size_t p = 0; p < np; p++) {
                    const int8_t *arow = col + p * kk;
                    int32_t qasum = 0, acc = bias_q;
                    for (size_t e = 0; e < kk; e++) {
                        qasum += arow[e];
                        acc += arow[e] * (int32_t)(int8_t)(wrow[e / 4] >> (8 * (e % 4)));
                    }
                    float r = sa * (float)qasum;
                    float val = (float)acc * sab + zw * r + za * w_term + zp_prod * (float)kk;
                    if (act == FNN_OR_ACT_RELU) val = fmaxf(val, 0.0f);
                    else if (act == FNN_OR_ACT_SILU) val = val / (1.0f + expf(-val));
                    else if (act == FNN_OR_ACT_GELU)
                        val = val * 0.5f * (1.0f + tanhf(val * 0.7978846f * (1.0f + 0.044715f * val * val)));
                    y[(nn * oc + ch) * np + p] = val;
                }
            }
        }
    free(pl);
    free(tmp);
    return 0;
}

/* Conv2d for the weight types without an integer kernel (U8, U4, F8, F8R, F4 and 4-bit codebook
 * weights; backend/cpu/mod.rs:4204-4257): the weights are dequantised to f32 once
 * (get_or_init_f32_weights, packed_tensor.rs:469-521) and conv2d_f32_im2col_gemm
 * (microkernels/conv.rs:509-660) runs an ordinary f32 convolution:
 *   y[b, oc, p] = act( sum_e W[oc, e] * col[p, e] + bias[oc] ),
 * col as in the integer lowering (im2col.rs:32-52), bias and activation applied after the GEMM
 * (conv_gemm.rs:26-47,154-235; GELU in its tanh form with the cubic term, :121-143).
 * The GEMM is a third-party SGEMM (crate gemm 0.19 / matrixmultiply): its summation order is not
 * part of the contract, so the sum is taken in double here and results are compared by tolerance. */
int fnn_or_qconv2d_float(int dt, const float *x, size_t b, size_t c, size_t h, size_t w,
                         const uint32_t *words, size_t oc, const float *scales, size_t n_scales,
                         const float *zeros, size_t n_zeros, size_t qblock, const float *codebook,
                         const float *bias, size_t kh, size_t kw, size_t stride, size_t pad,
                         size_t dil, size_t groups, int act, float *y)
{
    if (groups == 0 || c % groups || oc % groups) return -1;
    size_t cg = c / groups, ocg = oc / groups;
    size_t ho = fnn_or_conv_out_size(h, kh, stride, pad, dil);
    size_t wo = fnn_or_conv_out_size(w, kw, stride, pad, dil);
    size_t np = ho * wo;
    size_t kk = cg * kh * kw;
    float *wf = (float *)malloc((oc * kk + 1) * sizeof(float));
    if (!wf) return -2;
    int rc = fnn_or_dequant(dt, words, oc, kk, scales, n_scales, zeros, n_zeros, qblock, codebook, wf);
    if (rc) { free(wf); return rc; }
    for (size_t nn = 0; nn < b; nn++)
        for (size_t g = 0; g < groups; g++) {
            const float *xin = x + nn * c * h * w + g * cg * h * w;
            for (size_t f = 0; f < ocg; f++) {
                size_t ch = g * ocg + f;
                const float *wrow = wf + ch * kk;
                for (size_t oh = 0; oh < ho; oh++)
                    for (size_t ow = 0; ow < wo; ow++) {
                        double acc = 0.0;
                        for (size_t ic = 0; ic < cg; ic++)
                            for (size_t i = 0; i < kh; i++)
                                for (size_t j = 0; j < kw; j++) {
                                    size_t ih = oh * stride + i * dil - pad; /* wraps when < 0 */
                                    size_t iw = ow * stride + j * dil - pad;
                                    if (ih < h && iw < w)
                                        acc += (double)wrow[(ic * kh + i) * kw + j] *
                                               (double)xin[(ic * h + ih) * w + iw];
                                }
                        float v = (float)acc;
                        if (bias) v = v + bias[ch];
                        y[(nn * oc + ch) * np + oh * wo + ow] = fnn_or_act(v, act);
                    }
            }
        }
    free(wf);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* f32 data-movement ops found between quantised convolutions                 */
/* ------------------------------------------------------------------------ */

/* "concat" (backend/cpu/mod.rs:4267-4324): params [axis, inner_stride, outer_count]; every input
 * contributes blocks of elems/max(outer_count,1) values; for each outer position the blocks of
 * all inputs follow each other in the output.  Copies are clamped to the input and output lengths
 * and the output position advances by the (input-clamped) length.  Returns values written. */
size_t fnn_or_concat(const float *const *inputs, const size_t *lens, size_t n_inputs,
                     size_t outer_count, float *out, size_t out_len)
{
    size_t off = 0;
    for (size_t o = 0; o < outer_count; o++)
        for (size_t si = 0; si < n_inputs; si++) {
            size_t bs = lens[si] / (outer_count ? outer_count : 1);
            size_t src = o * bs;
            size_t end = src + bs < lens[si] ? src + bs : lens[si];
            size_t copy_len = end > src ? end - src : 0;
            size_t dst_end = off + copy_len < out_len ? off + copy_len : out_len;
            size_t actual = dst_end > off ? dst_end - off : 0;
            memcpy(out + off, inputs[si] + src, actual * sizeof(float));
            off += copy_len;
        }
    return off;
}

/* "slice_f32" (backend/cpu/mod.rs:4721-4760): params [dim, start, end, stride] where stride is the
 * number of elements per index of the sliced dimension; dim_size = in_len*range/out_len,
 * outer = in_len/dim_size/stride, each outer position copies range*stride values from
 * i*dim_size*stride + start*stride. */
void fnn_or_slice(const float *in, size_t in_len, size_t start, size_t end, size_t stride,
                  float *out, size_t out_len)
{
    size_t range_len = end > start ? end - start : 0;
    if (range_len < 1) range_len = 1;
    size_t dim_size = out_len ? (in_len * range_len) / out_len : 0;
    size_t outer = (dim_size > 0 && stride > 0) ? in_len / dim_size / stride : 1;
    size_t slice_elems = range_len * stride;
    for (size_t i = 0; i < outer; i++) {
        size_t src = i * dim_size * stride + start * stride;
        size_t dst = i * slice_elems;
        size_t room = in_len > src ? in_len - src : 0;
        size_t copy_len = slice_elems < room ? slice_elems : room;
        if (copy_len > 0) memcpy(out + dst, in + src, copy_len * sizeof(float));
    }
}

/* "pool_f32" with is_max = 1 (backend/cpu/mod.rs:4362-4397, microkernels/ops.rs:104-158):
 * params [kernel, stride, padding, is_max, N, C, H, W]; Ho = sat_sub(H + 2p, kernel)/stride + 1;
 * the window maximum starts at -inf and is replaced on a strict `>`; taps in the padding are skipped.
 * indices (nullable, the CallKernel's secondary output; ops.rs:110-155): best_kh*kernel + best_kw of the
 * tap that last replaced the maximum, (0, 0) when none did. */
void fnn_or_maxpool2d(const float *in, size_t in_len, size_t n, size_t c, size_t h, size_t w,
                      size_t kernel, size_t stride, size_t pad, float *out, size_t out_len,
                      int64_t *indices, size_t idx_len)
{
    size_t hp = h + 2 * pad, wp = w + 2 * pad;
    size_t ho = (hp > kernel ? hp - kernel : 0) / stride + 1;
    size_t wo = (wp > kernel ? wp - kernel : 0) / stride + 1;
    for (size_t nn = 0; nn < n; nn++)
        for (size_t cc = 0; cc < c; cc++)
            for (size_t hh = 0; hh < ho; hh++)
                for (size_t ww = 0; ww < wo; ww++) {
                    float val = -INFINITY;
                    size_t best_kh = 0, best_kw = 0;
                    for (size_t kh = 0; kh < kernel; kh++)
                        for (size_t kw = 0; kw < kernel; kw++) {
                            size_t hi = hh * stride + kh, wi = ww * stride + kw;
                            if (hi < pad || wi < pad) continue;
                            hi -= pad;
                            wi -= pad;
                            if (hi >= h || wi >= w) continue;
                            size_t idx = nn * (c * h * w) + cc * (h * w) + hi * w + wi;
                            if (idx < in_len && in[idx] > val) {
                                val = in[idx];
                                best_kh = kh;
                                best_kw = kw;
                            }
                        }
                    size_t o = nn * (c * ho * wo) + cc * (ho * wo) + hh * wo + ww;
                    if (o < out_len) out[o] = val;
                    if (indices && o < idx_len) indices[o] = (int64_t)(best_kh * kernel + best_kw);
                }
}

/* "pool_f32" with is_max != 1 (backend/cpu/mod.rs:4398-4470, microkernels/ops.rs:162-210; the AVX2
 * form ops.rs:425-560 sums interior windows in the same (kh, kw) order and divides by kernel^2, which
 * is the tap count there): mean over the taps inside the image, padding taps are not counted. */
void fnn_or_avgpool2d(const float *in, size_t in_len, size_t n, size_t c, size_t h, size_t w,
                      size_t kernel, size_t stride, size_t pad, float *out, size_t out_len)
{
    size_t hp = h + 2 * pad, wp = w + 2 * pad;
    size_t ho = (hp > kernel ? hp - kernel : 0) / stride + 1;
    size_t wo = (wp > kernel ? wp - kernel : 0) / stride + 1;
    for (size_t nn = 0; nn < n; nn++)
        for (size_t cc = 0; cc < c; cc++)
            for (size_t hh = 0; hh < ho; hh++)
                for (size_t ww = 0; ww < wo; ww++) {
                    float val = 0.0f;
                    size_t count = 0;
                    for (size_t kh = 0; kh < kernel; kh++)
                        for (size_t kw = 0; kw < kernel; kw++) {
                            size_t hi = hh * stride + kh, wi = ww * stride + kw;
                            if (hi < pad || wi < pad) continue;
                            hi -= pad;
                            wi -= pad;
                            if (hi >= h || wi >= w) continue;
                            size_t idx = nn * (c * h * w) + cc * (h * w) + hi * w + wi;
                            if (idx < in_len) { val += in[idx]; count++; }
                        }
                    if (count > 0) val /= (float)count;
                    size_t o = nn * (c * ho * wo) + cc * (ho * wo) + hh * wo + ww;
                    if (o < out_len) out[o] = val;
                }
}

/* "upsample_nearest2d" (backend/cpu/mod.rs:5496-5535, microkernels/misc.rs:338-364):
 * params [scale_h, scale_w, h_in, w_in]; nc = in_len/(h_in*w_in); every input value fills a
 * scale_h x scale_w block of the output. */
void fnn_or_upsample_nearest2d(const float *in, size_t nc, size_t h, size_t w, size_t sh, size_t sw,
                               float *out)
{
    size_t hw = h * w, orow = w * sw;
    for (size_t i = 0; i < nc; i++)
        for (size_t hi = 0; hi < h; hi++)
            for (size_t wi = 0; wi < w; wi++) {
                float v = in[i * hw + hi * w + wi];
                for (size_t a = 0; a < sh; a++)
                    for (size_t b = 0; b < sw; b++)
                        out[i * hw * sh * sw + (hi * sh + a) * orow + wi * sw + b] = v;
            }
}

/* ------------------------------------------------------------------------ */
/* generators                                                                 */
/* ------------------------------------------------------------------------ */

/* tests/cpu_reference_oracle.rs:18-36 -- xorshift64 (<<13, >>7, <<17);
 * value = ((state>>32) as i32 % 2049 - 1024)/256 + {-.75,-.25,0,.25,.75}[i%5]. */
void fnn_or_seeded_values(uint64_t seed, size_t len, float *out)
{
    static const float bias[5] = {-0.75f, -0.25f, 0.0f, 0.25f, 0.75f};
    uint64_t state = seed;
    for (size_t i = 0; i < len; i++) {
        state ^= state << 13;
        state ^= state >> 7;
        state ^= state << 17;
        int32_t hi = (int32_t)(uint32_t)(state >> 32);
        float centered = (float)(hi % 2049 - 1024) / 256.0f;
        out[i] = centered + bias[i % 5];
    }
}
