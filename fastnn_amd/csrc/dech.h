// Register decoders packed weight -> f16 MFMA operand (shared by the matrix-core kernels).
#pragma once
#include "common.h"

namespace dech {

__device__ __forceinline__ f16x2 as_h2(uint32_t u) { return __builtin_bit_cast(f16x2, u); }
__device__ __forceinline__ uint32_t as_u(f16x2 h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ f16x2 h2(float v) { return f16x2{(_Float16)v, (_Float16)v}; }

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f16x8 pack8(uint32_t a, uint32_t b, uint32_t c, uint32_t d)
{
    return __builtin_bit_cast(f16x8, u32x4{a, b, c, d});
}

// power of two that brings the largest table magnitude into [2^14, 2^15): the f16 hi + lo split of the scaled table
// then carries ~22 bits of every entry (every thread computes the same value from the 16 cached floats)
__device__ __forceinline__ int codebook_exp(const float *cb)
{
    float mx = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) mx = fmaxf(mx, fabsf(cb[i]));
    if (!(mx > 0.0f) || !(mx < __builtin_huge_valf())) return 0;
    int ex;
    (void)frexpf(mx, &ex);
    return 15 - ex;
}

// Decoders: one MFMA step = 8 k-values of one weight row as f16x8.  `w` points at the
// lane's packed words for the step (1 word for 4-bit types, 2 for 8-bit types).
// PERM tells in which order the 8 k-values land in the operand (the activation fragments
// are stored in LDS in the same order).
template <int DT>
struct DecH;

// 1024 + v is exact in f16 for 0 <= v < 1024: OR-ing a small integer into the mantissa of
// 0x6400 builds it without a convert; 1024 + 16 v likewise for the upper nibble of a byte.
// (u & mask) ^ bits in one v_bitop3_b32 (truth table of (s0 & s1) ^ s2)
__device__ __forceinline__ uint32_t and_xor(uint32_t u, uint32_t mask, uint32_t bits)
{
    return __builtin_amdgcn_bitop3_b32(u, mask, bits, 0x6A);
}
template <>
struct DecH<FNN_DT_I4> {
    static constexpr int WPS = 1;
    static constexpr bool INTERLEAVED = true;  // operand order k = 0,4,1,5,2,6,3,7
    __device__ static __forceinline__ f16x8 step(const uint32_t *w)
    {
        // nibble q -> q + 8 (flip its top bit) inside the mantissa of 1024.0: one logic op per pair
        const uint32_t u = w[0];
        const uint32_t v = u >> 8;
        f16x2 r0 = as_h2(and_xor(u, 0x000F000Fu, 0x64086408u)) + h2(-1032.0f);
        f16x2 r1 = __builtin_elementwise_fma(as_h2(and_xor(u, 0x00F000F0u, 0x64806480u)), h2(0.0625f), h2(-72.0f));
        f16x2 r2 = as_h2(and_xor(v, 0x000F000Fu, 0x64086408u)) + h2(-1032.0f);
        f16x2 r3 = __builtin_elementwise_fma(as_h2(and_xor(v, 0x00F000F0u, 0x64806480u)), h2(0.0625f), h2(-72.0f));
        return pack8(as_u(r0), as_u(r1), as_u(r2), as_u(r3));
    }
};
template <>
struct DecH<FNN_DT_U4> {
    static constexpr int WPS = 1;
    static constexpr bool INTERLEAVED = true;
    __device__ static __forceinline__ f16x8 step(const uint32_t *w)
    {
        const uint32_t u = w[0];
        const uint32_t v = u >> 8;
        f16x2 r0 = as_h2(and_xor(u, 0x000F000Fu, 0x64006400u)) + h2(-1024.0f);
        f16x2 r1 = __builtin_elementwise_fma(as_h2(and_xor(u, 0x00F000F0u, 0x64006400u)), h2(0.0625f), h2(-64.0f));
        f16x2 r2 = as_h2(and_xor(v, 0x000F000Fu, 0x64006400u)) + h2(-1024.0f);
        f16x2 r3 = __builtin_elementwise_fma(as_h2(and_xor(v, 0x00F000F0u, 0x64006400u)), h2(0.0625f), h2(-64.0f));
        return pack8(as_u(r0), as_u(r1), as_u(r2), as_u(r3));
    }
};
template <>
struct DecH<FNN_DT_I8> {
    static constexpr int WPS = 2;
    static constexpr bool INTERLEAVED = false;
    __device__ static __forceinline__ f16x8 step(const uint32_t *w)
    {
        const uint32_t u0 = w[0] ^ 0x80808080u, u1 = w[1] ^ 0x80808080u;  // byte q -> q + 128
        f16x2 r0 = as_h2(__builtin_amdgcn_perm(0x64646464u, u0, 0x04010400u)) + h2(-1152.0f);
        f16x2 r1 = as_h2(__builtin_amdgcn_perm(0x64646464u, u0, 0x04030402u)) + h2(-1152.0f);
        f16x2 r2 = as_h2(__builtin_amdgcn_perm(0x64646464u, u1, 0x04010400u)) + h2(-1152.0f);
        f16x2 r3 = as_h2(__builtin_amdgcn_perm(0x64646464u, u1, 0x04030402u)) + h2(-1152.0f);
        return pack8(as_u(r0), as_u(r1), as_u(r2), as_u(r3));
    }
};
template <>
struct DecH<FNN_DT_U8> {
    static constexpr int WPS = 2;
    static constexpr bool INTERLEAVED = false;
    __device__ static __forceinline__ f16x8 step(const uint32_t *w)
    {
        f16x2 r0 = as_h2(__builtin_amdgcn_perm(0x64646464u, w[0], 0x04010400u)) + h2(-1024.0f);
        f16x2 r1 = as_h2(__builtin_amdgcn_perm(0x64646464u, w[0], 0x04030402u)) + h2(-1024.0f);
        f16x2 r2 = as_h2(__builtin_amdgcn_perm(0x64646464u, w[1], 0x04010400u)) + h2(-1024.0f);
        f16x2 r3 = as_h2(__builtin_amdgcn_perm(0x64646464u, w[1], 0x04030402u)) + h2(-1024.0f);
        return pack8(as_u(r0), as_u(r1), as_u(r2), as_u(r3));
    }
};
template <>
struct DecH<FNN_DT_F8> {
    static constexpr int WPS = 2;
    static constexpr bool INTERLEAVED = false;
    __device__ static __forceinline__ f16x8 step(const uint32_t *w)
    {
        f16x2 r0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[0], 1.0f, false);
        f16x2 r1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[0], 1.0f, true);
        f16x2 r2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[1], 1.0f, false);
        f16x2 r3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[1], 1.0f, true);
        return pack8(as_u(r0), as_u(r1), as_u(r2), as_u(r3));
    }
};
template <>
struct DecH<FNN_DT_F8R> {
    static constexpr int WPS = 2;
    static constexpr bool INTERLEAVED = false;
    // an E5M2 byte is the upper byte of the f16 with the same value (incl. inf/NaN)
    __device__ static __forceinline__ f16x8 step(const uint32_t *w)
    {
        uint32_t r0 = __builtin_amdgcn_perm(0u, w[0], 0x010C000Cu);
        uint32_t r1 = __builtin_amdgcn_perm(0u, w[0], 0x030C020Cu);
        uint32_t r2 = __builtin_amdgcn_perm(0u, w[1], 0x010C000Cu);
        uint32_t r3 = __builtin_amdgcn_perm(0u, w[1], 0x030C020Cu);
        return pack8(r0, r1, r2, r3);
    }
};
template <>
struct DecH<FNN_DT_F4> {
    static constexpr int WPS = 1;
    static constexpr bool INTERLEAVED = false;
    __device__ static __forceinline__ f16x8 step(const uint32_t *w)
    {
        f16x2 r0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w[0], 1.0f, 0);
        f16x2 r1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w[0], 1.0f, 1);
        f16x2 r2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w[0], 1.0f, 2);
        f16x2 r3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w[0], 1.0f, 3);
        return pack8(as_u(r0), as_u(r1), as_u(r2), as_u(r3));
    }
};

// codebook nibbles are looked up by the tile kernel itself (a table in LDS); only the word geometry is used
template <>
struct DecH<FNN_DT_I4CB> {
    static constexpr int WPS = 1;
    static constexpr bool INTERLEAVED = false;
    __device__ static __forceinline__ f16x8 step(const uint32_t *w) { return pack8(w[0], w[0], w[0], w[0]); }
};

// ---- int8 operands for v_mfma_i32_32x32x32_i8: one MFMA step = 16 k-values of a weight row (4 words).
template <int DT>
struct DecI;
template <>
struct DecI<FNN_DT_I8> {
    static constexpr int WPS = 4;              // words per step
    static constexpr bool INTERLEAVED = false;
    __device__ static __forceinline__ f16x8 step(const uint32_t *w) { return pack8(w[0], w[1], w[2], w[3]); }
};
// 4-bit lanes become 16*q: the nibble moved to (or left in) the high half of a byte is the signed
// byte 16*q.  Low nibbles (even k) and high nibbles (odd k) of a word form two operand words, so the
// operand order inside 8 k-values is 0,2,4,6,1,3,5,7; the activations are stored in the same order.
template <>
struct DecI<FNN_DT_I4> {
    static constexpr int WPS = 2;
    static constexpr bool INTERLEAVED = true;
    __device__ static __forceinline__ f16x8 step(const uint32_t *w)
    {
        return pack8((w[0] << 4) & 0xF0F0F0F0u, w[0] & 0xF0F0F0F0u, (w[1] << 4) & 0xF0F0F0F0u, w[1] & 0xF0F0F0F0u);
    }
};
// unsigned 4-bit lanes fit a signed byte as they are (0..15): low nibbles in place, high nibbles shifted down
template <>
struct DecI<FNN_DT_U4> {
    static constexpr int WPS = 2;
    static constexpr bool INTERLEAVED = true;
    __device__ static __forceinline__ f16x8 step(const uint32_t *w)
    {
        return pack8(w[0] & 0x0F0F0F0Fu, (w[0] >> 4) & 0x0F0F0F0Fu, w[1] & 0x0F0F0F0Fu, (w[1] >> 4) & 0x0F0F0F0Fu);
    }
};

}  // namespace dech
