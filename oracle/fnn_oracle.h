/*
 * fnn_oracle.h -- CPU restatement of fastnn's weight-quantised MatMul path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP kernels are
 * compared against.  Nothing in the shipped package may include, link or call
 * it; only tests, the smoke check and the benchmark's cpu_baseline leg do.
 *
 * Every function restates, in plain C with strict IEEE-754 binary32
 * arithmetic (no FMA contraction, no reassociation), the behaviour of the
 * fastnn source lines cited next to its definition in fnn_oracle.c.
 */
#ifndef FNN_ORACLE_H
#define FNN_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Packed weight formats (same numbering as the product's public header). */
enum {
    FNN_OR_I8 = 0,   /* I8x4  : 4 signed bytes per word             */
    FNN_OR_I4 = 1,   /* I4x8  : 8 signed nibbles per word           */
    FNN_OR_U8 = 2,   /* U8x4  : 4 unsigned bytes per word           */
    FNN_OR_U4 = 3,   /* U4x8  : 8 unsigned nibbles per word         */
    FNN_OR_F8 = 4,   /* F8x4  : E4M3, bias 7, exp 15 = NaN          */
    FNN_OR_F8R = 5,  /* F8x4R : E5M2, bias 15                       */
    FNN_OR_F4 = 6,   /* F4x8  : E2M1 sign-magnitude                 */
    FNN_OR_I4CB = 7  /* I4x8 nibbles indexing a 16-entry codebook   */
};

enum { FNN_OR_ACT_NONE = 0, FNN_OR_ACT_RELU = 1, FNN_OR_ACT_GELU = 2, FNN_OR_ACT_SILU = 3 };

#define FNN_OR_SIMD_MARGIN 16

/* ---- word codecs ------------------------------------------------------- */
int      fnn_or_items(int dt);
int      fnn_or_bit_width(int dt);
void     fnn_or_unpack_word(int dt, uint32_t w, float *out);
uint32_t fnn_or_pack_word(int dt, const float *vals);
float    fnn_or_e4m3_to_f32(uint8_t b);
uint8_t  fnn_or_f32_to_e4m3(float v);
float    fnn_or_e5m2_to_f32(uint8_t b);
uint8_t  fnn_or_f32_to_e5m2(float v);
float    fnn_or_fp4_to_f32(uint8_t code);
uint8_t  fnn_or_f32_to_fp4(float v);

/* ---- integer lane dots -------------------------------------------------- */
int32_t fnn_or_i8x4_dot(uint32_t a, uint32_t b);
int32_t fnn_or_i8x4_sum(uint32_t w);
int32_t fnn_or_i4x8_dot(uint32_t a, uint32_t b);
int32_t fnn_or_i4x8_sum(uint32_t w);
int32_t fnn_or_f4x8_dot(uint32_t a, uint32_t b);

/* ---- packers / quantisers ----------------------------------------------- */
size_t fnn_or_packed_words(int dt, size_t rows, size_t inner); /* incl. margin */
void   fnn_or_from_f32_slice(int dt, const float *data, size_t rows, size_t inner,
                             float scale, float zero, uint32_t *words);
void   fnn_or_quant_per_channel_asym(int dt, const float *data, size_t rows, size_t inner,
                                     uint32_t *words, float *scales, float *zeros);
void   fnn_or_quant_per_channel_sym(int dt, const float *data, size_t rows, size_t inner,
                                    uint32_t *words, float *scales, float *zeros);
int    fnn_or_kmeans16(const float *values, size_t n, int iters, float *out16);
int    fnn_or_quant_codebook(const float *data, size_t rows, size_t inner, size_t qblock,
                             uint32_t *words, float *block_scales, float *codebook16);
void   fnn_or_transpose(const float *src_kn, size_t k, size_t n, float *dst_nk);

/* ---- dequantise ---------------------------------------------------------- */
int fnn_or_dequant(int dt, const uint32_t *words, size_t rows, size_t inner,
                   const float *scales, size_t n_scales, const float *zeros, size_t n_zeros,
                   size_t qblock, const float *codebook16, float *out);

/* ---- f32-activation quantised MatMul ------------------------------------ */
/* order: 0 = scalar sequential f32, 1 = AVX2 lane order f32 (4x8 partial sums),
 *        2 = binary64 accumulation (tolerance reference). */
int fnn_or_qmatmul(int dt, const uint32_t *words, size_t n, size_t k,
                   const float *scales, size_t n_scales, const float *zeros, size_t n_zeros,
                   size_t qblock, const float *codebook16,
                   const float *a, size_t m, float *out, int order, size_t k_tile,
                   int i4cb_as_written);
void fnn_or_bias_act(float *out, size_t m, size_t n, const float *bias, int act);
float fnn_or_act(float x, int act);

/* ---- I8-activation MatMul ------------------------------------------------ */
void fnn_or_quantize_activations(const float *x, size_t numel, uint8_t *payload);
/* "dequantize_activations", per-tensor form (backend/cpu/mod.rs:7063-7086) */
void fnn_or_dequantize_activations(const uint8_t *payload, size_t payload_len, float *out, size_t n);
int fnn_or_quantize_activations_per_channel(const float *x, size_t x_len, size_t numel, size_t num_channels,
                                            const float *scales, const float *zero_points, uint8_t *payload,
                                            size_t payload_len);
int fnn_or_dequantize_activations_per_channel(const uint8_t *payload, size_t payload_len, float *out, size_t out_len);
void fnn_or_quantize_activations_calibrated(const float *x, size_t numel, float scale, float zp,
                                            uint8_t *payload);
int  fnn_or_qmatmul_i8act(int dt, const uint32_t *words, size_t n, size_t k,
                          const float *scales, size_t n_scales, const float *zeros, size_t n_zeros,
                          const uint8_t *payload, size_t payload_len, size_t m,
                          float *out, int32_t *acc_out);

/* ---- quantised Conv2d (I8 weights, f32 NCHW activations) ----------------- */
size_t fnn_or_conv_out_size(size_t input, size_t kernel, size_t stride, size_t padding,
                            size_t dilation);
int fnn_or_qconv2d_i8(const float *x, size_t b, size_t c, size_t h, size_t w,
                      const uint32_t *words, size_t oc, const float *scales, size_t n_scales,
                      const float *zeros, size_t n_zeros, const float *bias,
                      size_t kh, size_t kw, size_t stride, size_t pad, size_t dil, size_t groups,
                      int act, float *y, int32_t *acc_out, float *act_scale_out,
                      float *act_zero_out);

/* I4x8 weights, activations quantised to 16 levels (packed_conv.rs:236-283,659-841,1202-1280) */
int fnn_or_qconv2d_i4(const float *x, size_t b, size_t c, size_t h, size_t w,
                      const uint32_t *words, size_t oc, const float *scales, size_t n_scales,
                      const float *zeros, size_t n_zeros, const float *bias,
                      size_t kh, size_t kw, size_t stride, size_t pad, size_t dil, size_t groups,
                      int act, float *y, int32_t *acc_out, float *act_scale_out,
                      float *act_zero_out);

/* "conv2d_i8_i8" / "conv2d_i4_i8": I8 activation payload, integer im2col (backend/cpu/mod.rs:3848-4098) */
int fnn_or_qconv2d_i8payload(int dt, const uint8_t *payload, size_t payload_len, size_t c, size_t h,
                             size_t w, const uint32_t *words, size_t oc, const float *scales,
                             size_t n_scales, const float *zeros, size_t n_zeros, const float *bias,
                             size_t kh, size_t kw, size_t stride, size_t pad, size_t dil,
                             size_t groups, int act, float *y);

/* weight types without an integer kernel: dequantise once, f32 convolution
 * (backend/cpu/mod.rs:4204-4257, microkernels/conv.rs:509-660) */
int fnn_or_qconv2d_float(int dt, const float *x, size_t b, size_t c, size_t h, size_t w,
                         const uint32_t *words, size_t oc, const float *scales, size_t n_scales,
                         const float *zeros, size_t n_zeros, size_t qblock, const float *codebook,
                         const float *bias, size_t kh, size_t kw, size_t stride, size_t pad,
                         size_t dil, size_t groups, int act, float *y);

/* ---- f32 data-movement ops between quantised convolutions ---------------- */
size_t fnn_or_concat(const float *const *inputs, const size_t *lens, size_t n_inputs,
                     size_t outer_count, float *out, size_t out_len);
void fnn_or_slice(const float *in, size_t in_len, size_t start, size_t end, size_t stride,
                  float *out, size_t out_len);
void fnn_or_avgpool2d(const float *in, size_t in_len, size_t n, size_t c, size_t h, size_t w,
                      size_t kernel, size_t stride, size_t pad, float *out, size_t out_len);
void fnn_or_maxpool2d(const float *in, size_t in_len, size_t n, size_t c, size_t h, size_t w,
                      size_t kernel, size_t stride, size_t pad, float *out, size_t out_len,
                      int64_t *indices, size_t idx_len);
void fnn_or_upsample_nearest2d(const float *in, size_t nc, size_t h, size_t w, size_t sh, size_t sw,
                               float *out);

/* ---- generators used by the reference's own tests ------------------------ */
void fnn_or_seeded_values(uint64_t seed, size_t len, float *out);

#ifdef __cplusplus
}
#endif
#endif
