// Quantised Conv2d (I8 or I4 weights, f32 NCHW activations) as one implicit GEMM on the int8 matrix cores:
// conv2d_packed_i8x4 / conv2d_packed_i4x8 (src/backend/cpu/packed_conv.rs:125-283,444-841) without an im2col
// operand in memory.  A wave owns 32 output pixels and TN x 32 output channels.  Per step of 32 k-values a lane
// (pixel lane & 31, k half lane >> 5) fetches its 16 im2col taps straight from the NCHW input, quantises them with the
// image's scale (q = clamp(round((v - za) * inv)), exactly the operand kernel's arithmetic) and packs them into the
// A operand of v_mfma_i32_32x32x32_i8; the weight rows come as 16-byte loads in operand order.  KW waves of a
// workgroup split the K range of the same pixels and add their exact i32 accumulators through LDS; the first of them
// applies the reference's float formula (conv_dequant) and stores NCHW, four pixels of a channel per store.
// Layers with many output channels run as conv_fused_kernel (below): the pixels quantised once into LDS, the waves
// of a workgroup sharing the channel blocks.
#include "mfma.h"
#include "dech.h"
#include "range_io.h"

namespace {

using namespace dech;

struct ImplicitArgs {
    QConvArgs a;
    ConvDivs dv;
    int g, kk, vec4;
    int rng_blocks;   // conv_fused_kernel: > 1 = that many channel blocks, one per wave, each with its own range pairs
};

constexpr int TAP_TABLE = 2048;   // taps (K rounded up to whole steps of 32) whose geometry is tabulated once per workgroup

// TAB: K (rounded up to whole steps) fits the tap table
template <int DT, int TN, int PW, int KW, bool RNG, bool TAB>
__global__ void __launch_bounds__(64 * PW * KW, TAB ? 4 : 2) conv_implicit_kernel(ImplicitArgs p)   // (TAB: four waves per SIMD, at most 128 registers)
{
    constexpr int NW = PW * KW;
    constexpr bool W4 = DT == FNN_DT_I4;
    constexpr int WBYTES = W4 ? 8 : 16;          // packed bytes of 16 k-values of a weight row
    const QConvArgs &a = p.a;
    extern __shared__ int red[];                 // [PW][KW - 1][TN * 16 + 1][64]: accumulators and q sums of the other K slices
    __shared__ float s_mm[2][2][NW];
    __shared__ float s_q[2][3];
    __shared__ float r_sa[PW][32], r_za[PW][32];
    __shared__ int r_qs[PW][32];
    __shared__ int64_t r_off[PW][32];
    __shared__ float s_rng[PW][4];
    __shared__ int s_cnt;
    __shared__ int r_img[PW][32];
    // offset inside the slab and validity bits needed per tap, where K fits
    __shared__ __attribute__((aligned(16))) uint32_t tap_offs[TAB ? TAP_TABLE : 4], tap_needs[TAB ? TAP_TABLE : 4];

    const int tid = threadIdx.x, lane = tid & 63;
    if constexpr (RNG) {
        if (tid == 0) s_cnt = 0;
        __syncthreads();
    }
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6), pw = wv / KW, kw = wv % KW;
    const int lr = lane & 31, hf = lane >> 5;
    const int g = p.g, kk = p.kk;
    const uint32_t np = (uint32_t)(a.ho * a.wo), wo = (uint32_t)a.wo;
    const int64_t rows = a.b * (int64_t)np;
    // (quotients of launch constants: kept in scalar registers, so that what is built from them -- the buffer
    // descriptors above all -- needs no per-lane check)
    const int cg = __builtin_amdgcn_readfirstlane((int)a.c / a.groups), ocg = __builtin_amdgcn_readfirstlane((int)(a.oc / a.groups));
    const int64_t r_first = (int64_t)blockIdx.x * (32 * PW);
    const int64_t n0 = (int64_t)blockIdx.y * (TN * 32);
    const uint32_t nn0 = p.dv.np.div((uint32_t)(r_first < rows ? r_first : 0));   // image of the workgroup's first row

    // ---- activation scales: from the partial ranges (a.nparts > 0: the workgroup's rows meet at most two images) or
    // from actq, as in the operand kernel of the explicit path
    const bool own_scales = a.nparts > 0 && r_first < rows;
    int bg_a = 0;
    if (own_scales) {
        const int64_t r_last = r_first + 32 * PW - 1 < rows ? r_first + 32 * PW - 1 : rows - 1;
        bg_a = (int)nn0 * a.groups + g;
        const int bg_b = (int)p.dv.np.div((uint32_t)r_last) * a.groups + g;
        const int nimg = bg_b != bg_a ? 2 : 1;
        for (int w = 0; w < nimg; w++) {
            const float *part = a.minmax_partial + (int64_t)(w ? bg_b : bg_a) * a.part_stride * 2;
            float mn = a.range_zero ? 0.0f : INFINITY, mx = a.range_zero ? 0.0f : -INFINITY;
            conv_fold_partial_ranges(part, a.nparts, tid, 64 * NW, mn, mx);
            mn = wave_min(mn);
            mx = wave_max(mx);
            if (lane == 0) { s_mm[w][0][wv] = mn; s_mm[w][1][wv] = mx; }
        }
        __syncthreads();
        if (tid < nimg) {
            float mn = s_mm[tid][0][0], mx = s_mm[tid][1][0];
#pragma unroll
            for (int w2 = 1; w2 < NW; w2++) { mn = fminf(mn, s_mm[tid][0][w2]); mx = fmaxf(mx, s_mm[tid][1][w2]); }
            const float range = mx - mn;
            float scale, zero;
            if (W4) {
                scale = (range > 0.0f) ? range / 15.0f : 1.0f;
                zero = mn + 8.0f * scale;
            } else {
                scale = (range > 0.0f) ? range / 255.0f : 1.0f;
                zero = (range > 0.0f) ? mn + 128.0f * scale : 0.0f;
            }
            const float inv = (scale != 0.0f) ? 1.0f / scale : 0.0f;
            s_q[tid][0] = scale; s_q[tid][1] = zero; s_q[tid][2] = inv;
        }
        __syncthreads();
    }

    // ---- this lane's pixel
    const int64_t r = r_first + pw * 32 + lr;
    const bool live = r < rows;
    const uint32_t ru = live ? (uint32_t)r : 0u;
    const uint32_t nn = p.dv.np.div(ru), px = ru - nn * np;
    const uint32_t oh = p.dv.wo.div(px), ow = px - oh * wo;
    const int bg = (int)nn * a.groups + g;
    float sa = 1.0f, za = 0.0f, inv = 0.0f;
    if (a.nparts <= 0) {
        sa = a.actq[bg * 4 + 0]; za = a.actq[bg * 4 + 1]; inv = a.actq[bg * 4 + 2];
    } else if (own_scales) {
        const int w = bg != bg_a ? 1 : 0;
        sa = s_q[w][0]; za = s_q[w][1]; inv = s_q[w][2];
    }
    // one buffer descriptor per workgroup over the input from the group's slab of image nn0 on: a tap outside the
    // image, past K or of a row past the last one gets the offset ~0, which the range check answers with zero
    const int64_t img = a.c * a.h * a.w;
    const int64_t slab0 = ((int64_t)nn0 * a.c + (int64_t)g * cg) * a.h * a.w;
    const int64_t left = (a.b * img - slab0) * 4;
    const __amdgpu_buffer_rsrc_t xbuf = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(a.x + slab0), 0, (int)(uint32_t)(left > 0xfffffff0ll ? 0xfffffff0ll : left), 0x00020000);
    const int hh = (int)a.h, ww = (int)a.w;
    constexpr int qlo = W4 ? -8 : -128, qhi = W4 ? 7 : 127;
    const int ih0 = (int)oh * a.stride - a.pad, iw0 = (int)ow * a.stride - a.pad;
    uint32_t okbits = 0;   // kernel rows (bits 0..14) and columns (16..30) inside the image for this pixel
    for (int i = 0; i < a.kh; i++) okbits |= ((unsigned)(ih0 + i * a.dil) < (unsigned)hh ? 1u : 0u) << i;
    for (int j = 0; j < a.kw; j++) okbits |= ((unsigned)(iw0 + j * a.dil) < (unsigned)ww ? 0x10000u : 0u) << j;
    if (!live) okbits = 0;
    const uint32_t lane_base = ((uint32_t)(nn - nn0) * (uint32_t)img + (uint32_t)(ih0 * ww + iw0)) * 4;   // (mod 2^32)

    // ---- weights: rows n0 + tn*32 + lr of the group, 16 k-values from byte (32*s + 16*hf) * bits / 8 of the row
    const int64_t wrow0 = (int64_t)g * ocg + n0;
    const int64_t wleft = ((int64_t)a.oc - wrow0) * a.kp * 4 + 256;   // (the zeroed margin behind the last row)
    const __amdgpu_buffer_rsrc_t wbuf = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t *>(a.words + wrow0 * a.kp), 0, (int)(uint32_t)(wleft > 0xfffffff0ll ? 0xfffffff0ll : wleft), 0x00020000);
    uint32_t wlane[TN];
#pragma unroll
    for (int tn = 0; tn < TN; tn++) {
        const int64_t n = n0 + tn * 32 + lr;
        wlane[tn] = n < ocg ? (uint32_t)((tn * 32 + lr) * a.kp * 4 + hf * WBYTES) : ~0u;   // rows past the group: zero weights
    }

    const int nsteps = (kk + 31) / 32;
    const uint32_t bperm = (uint32_t)(hf * 16) * 4;   // this lane's 16 taps sit in lanes 16*hf .. 16*hf + 15 of the geometry
    // The geometry of a tap does not depend on the pixel: with K up to TAP_TABLE taps it is worked out once per
    // workgroup; a lane then reads its 16 taps of a step from the table (two addresses per wave: broadcast reads).
    // A wave all of whose pixels exist and have every kernel row and column inside the image skips the validity test.
    if constexpr (TAB) {
        for (int e0 = tid; e0 < nsteps * 32; e0 += 64 * NW) {
            const uint32_t e = (uint32_t)e0;
            const uint32_t ic = p.dv.khw.div(e), rem = e - ic * (uint32_t)(a.kh * a.kw);
            const uint32_t i = p.dv.kw.div(rem), j = rem - i * (uint32_t)a.kw;
            tap_offs[e0] = ((ic * (uint32_t)hh + i * (uint32_t)a.dil) * (uint32_t)ww + j * (uint32_t)a.dil) * 4;
            tap_needs[e0] = (int)e < kk ? ((1u << i) | (0x10000u << j)) : 0x80000000u;
        }
        __syncthreads();
    }
    const uint32_t all_bits = ((1u << a.kh) - 1u) | (((1u << a.kw) - 1u) << 16);
    const bool inside = __builtin_amdgcn_ballot_w64(okbits != all_bits) == 0;   // (wave-uniform)
    i32x16 acc[TN];
#pragma unroll
    for (int tn = 0; tn < TN; tn++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[tn][i] = 0;
    int qs = 0;

    // tap geometry of a step: lane l & 31 works out tap 32*s + (l & 31): offset inside the slab and the validity bits
    // it needs (bit 31, never set in okbits, for taps past K)
    auto geometry = [&](int s, uint32_t &tap_off, uint32_t &tap_need) {
        const uint32_t e = (uint32_t)(32 * s + lr);
        const uint32_t ic = p.dv.khw.div(e), rem = e - ic * (uint32_t)(a.kh * a.kw);
        const uint32_t i = p.dv.kw.div(rem), j = rem - i * (uint32_t)a.kw;
        tap_off = ((ic * (uint32_t)hh + i * (uint32_t)a.dil) * (uint32_t)ww + j * (uint32_t)a.dil) * 4;
        tap_need = (int)e < kk ? ((1u << i) | (0x10000u << j)) : 0x80000000u;
    };
    auto fetch = [&](int s, float(&v)[16], u32x4(&wq)[TN]) {
        if constexpr (TAB) {
            // the lane's 16 taps are 64 contiguous bytes of either table: four 16-byte reads (two addresses per wave)
            const u32x4 *po = reinterpret_cast<const u32x4 *>(tap_offs + 32 * s + 16 * hf);
            if (inside && 32 * s + 32 <= kk) {
#pragma unroll
                for (int t4 = 0; t4 < 4; t4++) {
                    const u32x4 o4 = po[t4];
#pragma unroll
                    for (int t = 0; t < 4; t++)
                        v[t4 * 4 + t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xbuf, lane_base + o4[t], 0, 0));
                }
            } else {
                const u32x4 *pn = reinterpret_cast<const u32x4 *>(tap_needs + 32 * s + 16 * hf);
#pragma unroll
                for (int t4 = 0; t4 < 4; t4++) {
                    const u32x4 o4 = po[t4], n4 = pn[t4];
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        const uint32_t vo = (okbits & n4[t]) == n4[t] ? lane_base + o4[t] : ~0u;
                        v[t4 * 4 + t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xbuf, vo, 0, 0));
                    }
                }
            }
        } else {
            uint32_t tap_off, tap_need;
            geometry(s, tap_off, tap_need);
#pragma unroll
            for (int t = 0; t < 16; t++) {
                const uint32_t soff = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(bperm + 4 * t), (int)tap_off);
                const uint32_t need = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(bperm + 4 * t), (int)tap_need);
                const uint32_t vo = (okbits & need) == need ? lane_base + soff : ~0u;
                v[t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xbuf, vo, 0, 0));
            }
        }
#pragma unroll
        for (int tn = 0; tn < TN; tn++) {
            const uint32_t wo_ = wlane[tn] == ~0u ? ~0u : wlane[tn] + (uint32_t)s * (2 * WBYTES);
            if (W4) {
                const auto t2 = __builtin_amdgcn_raw_buffer_load_b64(wbuf, wo_, 0, 0);
                wq[tn][0] = t2[0]; wq[tn][1] = t2[1]; wq[tn][2] = 0; wq[tn][3] = 0;
            } else {
                wq[tn] = __builtin_amdgcn_raw_buffer_load_b128(wbuf, wo_, 0, 0);
            }
        }
    };
    auto consume = [&](int s, const float(&v)[16], const u32x4(&wq)[TN]) {
        int q[16];
#pragma unroll
        for (int t = 0; t < 16; t++) {
            // round half away from zero, then clamp: trunc(x + copysign(0.49999997, x)) equals roundf(x) after the
            // clamp for every float (the conversion truncates, saturates and maps NaN to 0)
            const float x = (v[t] - za) * inv;
            const int qi = (int)(x + __builtin_copysignf(0.49999997f, x));
            q[t] = max(qlo, min(qi, qhi));
        }
        // operand byte `pos` holds tap (pos & 8) + k(pos & 7): the order the weight decoder delivers
        i32x4 af;
#pragma unroll
        for (int wi = 0; wi < 4; wi++) {
            int tp[4];
#pragma unroll
            for (int bq = 0; bq < 4; bq++) {
                const int pos = wi * 4 + bq, sl = pos & 7;
                tp[bq] = (pos & 8) + (W4 ? ((sl & 3) * 2 + (sl >> 2)) : sl);
            }
            const uint32_t lo = __builtin_amdgcn_perm((uint32_t)q[tp[1]], (uint32_t)q[tp[0]], 0x0c0c0400u);
            const uint32_t hi = __builtin_amdgcn_perm((uint32_t)q[tp[3]], (uint32_t)q[tp[2]], 0x04000c0cu);
            af[wi] = (int)(lo | hi);
        }
        const int past = 32 * s + 16 * hf + 16 - kk;   // taps of this lane past K: their bytes are cleared
        if (past > 0) {
#pragma unroll
            for (int wi = 0; wi < 4; wi++) {
                uint32_t keep = 0;
#pragma unroll
                for (int bq = 0; bq < 4; bq++) {
                    const int pos = wi * 4 + bq, sl = pos & 7;
                    const int tpp = (pos & 8) + (W4 ? ((sl & 3) * 2 + (sl >> 2)) : sl);
                    keep |= (tpp < 16 - past) ? (0xffu << (8 * bq)) : 0u;
                }
                af[wi] &= (int)keep;
            }
        }
#pragma unroll
        for (int wi = 0; wi < 4; wi++) qs = __builtin_amdgcn_sdot4(af[wi], 0x01010101, qs, false);
#pragma unroll
        for (int tn = 0; tn < TN; tn++) {
            const uint32_t w4[4] = {wq[tn][0], wq[tn][1], wq[tn][2], wq[tn][3]};
            const f16x8 bf = DecI<DT>::step(w4);
            acc[tn] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, __builtin_bit_cast(i32x4, bf), acc[tn], 0, 0, 0);
        }
    };

    // ---- K loop of this wave: steps kw, kw + KW, ...; the next step's loads are requested before this one is used
    {
        float v0[16], v1[16];
        u32x4 w0[TN], w1[TN];
        int s = kw;
        if (s < nsteps) fetch(s, v0, w0);
        for (; s < nsteps; s += 2 * KW) {
            if (s + KW < nsteps) fetch(s + KW, v1, w1);
            consume(s, v0, w0);
            if (s + KW < nsteps) {
                if (s + 2 * KW < nsteps) fetch(s + 2 * KW, v0, w0);
                consume(s + KW, v1, w1);
            }
        }
    }

    // this lane's channel constants: requested when the K loop is done (not earlier: they would take registers the
    // loop's loads in flight need), so that they travel while the K slices meet
    // Up to 16 channels in a 32-channel column block: the lanes of channels 16 .. 31 would sit out the epilogue, so
    // they take over half of the pixels of the lane 16 below (`share`: lane lr works on channel lr & 15).
    const bool share = TN == 1 && ocg <= 16;   // (uniform)
    const int lch = share ? (lr & 15) : lr;
    float sw[TN], zw[TN], bi[TN];
    int wq_[TN];
#pragma unroll
    for (int tn = 0; tn < TN; tn++) {
        const int64_t n = n0 + tn * 32 + lch;
        const bool ok = kw == 0 && n < ocg;
        const int64_t ch = (int64_t)g * ocg + (ok ? n : 0);
        sw[tn] = ok ? a.scales[ch] : 0.0f;
        zw[tn] = ok ? a.zeros[ch] : 0.0f;
        wq_[tn] = ok ? a.row_qsum[ch] : 0;
        bi[tn] = (ok && a.bias) ? a.bias[ch] : 0.0f;
    }

    // ---- the K slices of a pixel block meet in LDS (exact integers: any order)
    constexpr int SLOT = (TN * 16 + 1) * 64;
    if (KW > 1) {
        if (kw > 0) {
            int *dst = red + (pw * (KW - 1) + (kw - 1)) * SLOT + lane;
#pragma unroll
            for (int tn = 0; tn < TN; tn++)
#pragma unroll
                for (int i = 0; i < 16; i++) dst[(tn * 16 + i) * 64] = acc[tn][i];
            dst[TN * 16 * 64] = qs;
        }
        __syncthreads();
#pragma unroll
        for (int k2 = 0; kw == 0 && k2 < KW - 1; k2++) {
            const int *src = red + (pw * (KW - 1) + k2) * SLOT + lane;
#pragma unroll
            for (int tn = 0; tn < TN; tn++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[tn][i] += src[(tn * 16 + i) * 64];
            qs += src[TN * 16 * 64];
        }
    }
    qs += __shfl_xor(qs, 32, 64);   // the two k halves of a pixel

    // ---- epilogue: row constants through this wave's LDS rows, then acc[tn][i] = pixel (i/4)*8 + hf*4 + i%4 of the
    // block, channel n0 + tn*32 + lr
    // output ranges (RNG): the workgroup (block of 32 * PW pixels, column tile) fills pair
    // (block - first block of the image) * column tiles + tile of every image it meets, (np / (32 * PW) + 2) * tiles
    // pairs per image; the block that holds the last pixel of its first image also fills that image's unused pairs
    float mn0 = INFINITY, mx0 = -INFINITY, mn1 = INFINITY, mx1 = -INFINITY;
    bool rng_two = false, rng_plain = false;
    if constexpr (RNG) {
        const uint32_t row_z = (uint32_t)(r_first + 32 * PW - 1 < rows ? r_first + 32 * PW - 1 : rows - 1);
        rng_two = r_first < rows && row_z > (nn0 + 1) * np - 1;
        rng_plain = !rng_two && r_first + 32 * PW <= rows;
    }
    if (kw == 0) {
        if (hf == 0) {
            r_sa[pw][lr] = sa; r_za[pw][lr] = za; r_qs[pw][lr] = qs;
            r_off[pw][lr] = (int64_t)nn * a.oc * np + px;
            if (RNG) r_img[pw][lr] = nn != nn0;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const bool has_bias = a.bias != nullptr;
        float *y = a.y + (int64_t)g * ocg * np;
        int32_t *acc_out = a.acc_out ? a.acc_out + (int64_t)g * ocg * np : nullptr;
        const float *residual = a.residual ? a.residual + (int64_t)g * ocg * np : nullptr;
        float *sum_out = a.sum_out + (int64_t)g * ocg * np;
        if constexpr (TN == 1) {
            if (share) {
                // rows of 16 lanes: (k half 0, channels 0-15), (0, 16-31), (1, 0-15), (1, 16-31).  Registers 8 .. 15 (pixel
                // groups 2 and 3) of the even rows move into registers 0 .. 7 of the odd rows above them
#pragma unroll
                for (int i = 0; i < 8; i++)
                    acc[0][i] = (int)__builtin_amdgcn_permlane16_swap((uint32_t)acc[0][i], (uint32_t)acc[0][i + 8], false, false)[0];
            }
        }
#pragma unroll
        for (int igl = 0; igl < 4; igl++) {
            if (share && igl >= 2) break;
            const int ig = share ? igl + 2 * (lr >> 4) : igl;   // pixel group of registers 4 igl .. 4 igl + 3
            const int rr0 = ig * 8 + hf * 4;
            const int64_t r0 = r_first + pw * 32 + rr0;
            if (r0 >= rows) continue;
            float rsa[4], rza[4], rs[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                rsa[j] = r_sa[pw][rr0 + j];
                rza[j] = r_za[pw][rr0 + j];
                rs[j] = rsa[j] * (float)r_qs[pw][rr0 + j];
            }
#pragma unroll
            for (int tn = 0; tn < TN; tn++) {
                const int64_t n = n0 + tn * 32 + lch;
                if (n >= ocg) continue;
                float v[4];
                int av[4], bq[4];
                bq[0] = has_bias ? conv_bias_q(bi[tn], rsa[0], sw[tn]) : 0;
#pragma unroll
                for (int j = 1; j < 4; j++) bq[j] = (p.vec4 || !has_bias) ? bq[0] : conv_bias_q(bi[tn], rsa[j], sw[tn]);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    int ai = acc[tn][igl * 4 + j];
                    if (W4) ai >>= 4;
                    v[j] = conv_affine(ai, rsa[j], rza[j], rs[j], sw[tn], zw[tn], sw[tn] * (float)wq_[tn], bq[j], kk, &av[j]);
                }
                conv_act4(v, a.act);
                // a.residual: the Add behind this convolution; v becomes the sums, whose ranges travel on instead of y's
                if (p.vec4) {
                    const int64_t o = r_off[pw][rr0] + n * np;
                    if constexpr (TN > 1) {   // stored below, channel by channel
#pragma unroll
                        for (int j = 0; j < 4; j++) acc[tn][igl * 4 + j] = __float_as_int(v[j]);
                    } else {
                        *reinterpret_cast<float4 *>(y + o) = make_float4(v[0], v[1], v[2], v[3]);
                    }
                    if (acc_out) *reinterpret_cast<int4 *>(acc_out + o) = make_int4(av[0], av[1], av[2], av[3]);
                    if (residual) {
                        const float4 r4 = *reinterpret_cast<const float4 *>(residual + o);
                        v[0] = v[0] + r4.x; v[1] = v[1] + r4.y; v[2] = v[2] + r4.z; v[3] = v[3] + r4.w;
                        *reinterpret_cast<float4 *>(sum_out + o) = make_float4(v[0], v[1], v[2], v[3]);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        if (r0 + j >= rows) continue;
                        const int64_t o = r_off[pw][rr0 + j] + n * np;
                        y[o] = v[j];
                        if (acc_out) acc_out[o] = av[j];
                        if (residual) {
                            v[j] = v[j] + residual[o];
                            sum_out[o] = v[j];
                        }
                    }
                }
                if constexpr (RNG) {
                    if (rng_plain) {   // (workgroup-uniform) every pixel of the block exists and lies in one image
                        mn0 = fminf(fminf(mn0, fminf(v[0], v[1])), fminf(v[2], v[3]));
                        mx0 = fmaxf(fmaxf(mx0, fmaxf(v[0], v[1])), fmaxf(v[2], v[3]));
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            if (r0 + j >= rows) continue;
                            if (rng_two && r_img[pw][rr0 + j]) { mn1 = fminf(mn1, v[j]); mx1 = fmaxf(mx1, v[j]); }
                            else { mn0 = fminf(mn0, v[j]); mx0 = fmaxf(mx0, v[j]); }
                        }
                    }
                }
            }
        }
        // several channel blocks per wave: the four stores that fill a channel's 128-byte line follow each other
        if constexpr (TN > 1) {
            if (p.vec4) {
#pragma unroll
                for (int tn = 0; tn < TN; tn++) {
                    const int64_t n = n0 + tn * 32 + lr;
                    if (n >= ocg) continue;
#pragma unroll
                    for (int ig = 0; ig < 4; ig++) {
                        const int rr0 = ig * 8 + hf * 4;
                        if (r_first + pw * 32 + rr0 >= rows) continue;
                        const int64_t o = r_off[pw][rr0] + n * np;
                        *reinterpret_cast<float4 *>(y + o) = make_float4(__int_as_float(acc[tn][ig * 4]), __int_as_float(acc[tn][ig * 4 + 1]),
                                                                          __int_as_float(acc[tn][ig * 4 + 2]), __int_as_float(acc[tn][ig * 4 + 3]));
                    }
                }
            }
        }
    }
    if constexpr (RNG) {
        if (r_first >= rows) return;   // (workgroup-uniform)
        if (kw != 0) return;
        // the pixel blocks' waves leave their pairs in LDS and count themselves; the last to arrive combines them (no
        // barrier: a wave that is done retires)
        mn0 = wave_min(mn0); mx0 = wave_max(mx0);
        if (rng_two) { mn1 = wave_min(mn1); mx1 = wave_max(mx1); }
        int arrived = 0;
        if (lane == 0) {
            s_rng[pw][0] = mn0; s_rng[pw][1] = mx0; s_rng[pw][2] = mn1; s_rng[pw][3] = mx1;
            __threadfence_block();
            arrived = atomicAdd(&s_cnt, 1);
            __threadfence_block();
        }
        if (lane == 0 && arrived == PW - 1) {
            mn0 = s_rng[0][0]; mx0 = s_rng[0][1]; mn1 = s_rng[0][2]; mx1 = s_rng[0][3];
#pragma unroll
            for (int w2 = 1; w2 < PW; w2++) {
                mn0 = fminf(mn0, s_rng[w2][0]); mx0 = fmaxf(mx0, s_rng[w2][1]);
                mn1 = fminf(mn1, s_rng[w2][2]); mx1 = fmaxf(mx1, s_rng[w2][3]);
            }
            constexpr uint32_t BM = 32 * PW;
            const uint32_t row_z = (uint32_t)(r_first + BM - 1 < rows ? r_first + BM - 1 : rows - 1);
            const uint32_t img_end = (nn0 + 1) * np - 1;
            const int nt = (int)blockIdx.y;
            const int slot = (int)(blockIdx.x - (nn0 * np) / BM), per_m = (int)(np / BM) + 2;
            const int fill = row_z >= img_end ? slot + 1 : per_m;
            // (the pairs of a channel block lie together: a reader of some of the channels takes its blocks' pairs)
            float *row = a.range_out + (int64_t)nn0 * a.range_out_stride * 2 + (int64_t)nt * per_m * 2;
            float *dst = row + (int64_t)slot * 2;
            dst[0] = mn0; dst[1] = mx0;
            if (rng_two) {   // the next image starts in this block: its pair 0
                float *d1 = row + (int64_t)a.range_out_stride * 2;
                d1[0] = mn1; d1[1] = mx1;
            }
            for (int j = fill; j < per_m; j++) {
                float *d2 = row + (int64_t)j * 2;
                d2[0] = INFINITY; d2[1] = -INFINITY;
            }
        }
    }
}

// The same convolution for layers with many output channels: a workgroup of four waves owns 32 output pixels and ALL
// output channels of the group.  Phase 1: the waves share the K steps, fetch and quantise the pixels' im2col taps
// once (the code of the kernel above) and leave the packed A operands of all steps in LDS (1 KB per step).  Phase 2:
// the waves share the blocks of TN x 32 channels; a wave runs the whole K range of its block from LDS against the
// weight rows streamed in operand order, and finishes it with the same epilogue.  No K slices to add, no operand in
// memory, no second fetch of the pixels per channel block.
constexpr int FUSED_MAX_STEPS = 40;   // A operands of a workgroup in LDS: 40 KB beside the 16 KB tap table

template <int DT, int TN, bool RNG>
__global__ void __launch_bounds__(256) conv_fused_kernel(ImplicitArgs p)
{
    constexpr int NW = 4;
    constexpr bool W4 = DT == FNN_DT_I4;
    constexpr int WBYTES = W4 ? 8 : 16;          // packed bytes of 16 k-values of a weight row
    const QConvArgs &a = p.a;
    extern __shared__ __attribute__((aligned(16))) unsigned char a_lds[];   // [steps][64 lanes][16 bytes]
    __shared__ float s_mm[2][2][NW];
    __shared__ float s_q[2][3];
    __shared__ float r_sa[32], r_za[32];
    __shared__ int r_qsw[NW][32];
    __shared__ int64_t r_off[32];
    __shared__ float s_rng[NW][4];
    __shared__ int s_cnt;
    __shared__ int r_img[32];
    __shared__ __attribute__((aligned(16))) uint32_t tap_offs[TAP_TABLE], tap_needs[TAP_TABLE];

    const int tid = threadIdx.x, lane = tid & 63;
    if constexpr (RNG) {
        if (tid == 0) s_cnt = 0;
    }
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 31, hf = lane >> 5;
    const int g = p.g, kk = p.kk;
    const uint32_t np = (uint32_t)(a.ho * a.wo), wo = (uint32_t)a.wo;
    const int64_t rows = a.b * (int64_t)np;
    // (quotients of launch constants: kept in scalar registers, so that what is built from them -- the buffer
    // descriptors above all -- needs no per-lane check)
    const int cg = __builtin_amdgcn_readfirstlane((int)a.c / a.groups), ocg = __builtin_amdgcn_readfirstlane((int)(a.oc / a.groups));
    const int64_t r_first = (int64_t)blockIdx.x * 32;
    const uint32_t nn0 = p.dv.np.div((uint32_t)(r_first < rows ? r_first : 0));   // image of the workgroup's first row

    // ---- activation scales (as above)
    const bool own_scales = a.nparts > 0 && r_first < rows;
    int bg_a = 0;
    if (own_scales) {
        const int64_t r_last = r_first + 31 < rows ? r_first + 31 : rows - 1;
        bg_a = (int)nn0 * a.groups + g;
        const int bg_b = (int)p.dv.np.div((uint32_t)r_last) * a.groups + g;
        const int nimg = bg_b != bg_a ? 2 : 1;
        for (int w = 0; w < nimg; w++) {
            const float *part = a.minmax_partial + (int64_t)(w ? bg_b : bg_a) * a.part_stride * 2;
            float mn = a.range_zero ? 0.0f : INFINITY, mx = a.range_zero ? 0.0f : -INFINITY;
            conv_fold_partial_ranges(part, a.nparts, tid, 64 * NW, mn, mx);
            mn = wave_min(mn);
            mx = wave_max(mx);
            if (lane == 0) { s_mm[w][0][wv] = mn; s_mm[w][1][wv] = mx; }
        }
        __syncthreads();
        if (tid < nimg) {
            float mn = s_mm[tid][0][0], mx = s_mm[tid][1][0];
#pragma unroll
            for (int w2 = 1; w2 < NW; w2++) { mn = fminf(mn, s_mm[tid][0][w2]); mx = fmaxf(mx, s_mm[tid][1][w2]); }
            const float range = mx - mn;
            float scale, zero;
            if (W4) {
                scale = (range > 0.0f) ? range / 15.0f : 1.0f;
                zero = mn + 8.0f * scale;
            } else {
                scale = (range > 0.0f) ? range / 255.0f : 1.0f;
                zero = (range > 0.0f) ? mn + 128.0f * scale : 0.0f;
            }
            const float inv = (scale != 0.0f) ? 1.0f / scale : 0.0f;
            s_q[tid][0] = scale; s_q[tid][1] = zero; s_q[tid][2] = inv;
        }
        __syncthreads();
    }

    // ---- this lane's pixel (the same 32 pixels in every wave)
    const int64_t r = r_first + lr;
    const bool live = r < rows;
    const uint32_t ru = live ? (uint32_t)r : 0u;
    const uint32_t nn = p.dv.np.div(ru), px = ru - nn * np;
    const uint32_t oh = p.dv.wo.div(px), ow = px - oh * wo;
    const int bg = (int)nn * a.groups + g;
    float sa = 1.0f, za = 0.0f, inv = 0.0f;
    if (a.nparts <= 0) {
        sa = a.actq[bg * 4 + 0]; za = a.actq[bg * 4 + 1]; inv = a.actq[bg * 4 + 2];
    } else if (own_scales) {
        const int w = bg != bg_a ? 1 : 0;
        sa = s_q[w][0]; za = s_q[w][1]; inv = s_q[w][2];
    }
    const int64_t img = a.c * a.h * a.w;
    const int64_t slab0 = ((int64_t)nn0 * a.c + (int64_t)g * cg) * a.h * a.w;
    const int64_t left = (a.b * img - slab0) * 4;
    const __amdgpu_buffer_rsrc_t xbuf = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(a.x + slab0), 0, (int)(uint32_t)(left > 0xfffffff0ll ? 0xfffffff0ll : left), 0x00020000);
    const int hh = (int)a.h, ww = (int)a.w;
    constexpr int qlo = W4 ? -8 : -128, qhi = W4 ? 7 : 127;
    const int ih0 = (int)oh * a.stride - a.pad, iw0 = (int)ow * a.stride - a.pad;
    uint32_t okbits = 0;
    for (int i = 0; i < a.kh; i++) okbits |= ((unsigned)(ih0 + i * a.dil) < (unsigned)hh ? 1u : 0u) << i;
    for (int j = 0; j < a.kw; j++) okbits |= ((unsigned)(iw0 + j * a.dil) < (unsigned)ww ? 0x10000u : 0u) << j;
    if (!live) okbits = 0;
    const uint32_t lane_base = ((uint32_t)(nn - nn0) * (uint32_t)img + (uint32_t)(ih0 * ww + iw0)) * 4;   // (mod 2^32)

    const int nsteps = (kk + 31) / 32;   // <= FUSED_MAX_STEPS, and nsteps * 32 <= TAP_TABLE (the host checks)
    for (int e0 = tid; e0 < nsteps * 32; e0 += 64 * NW) {
        const uint32_t e = (uint32_t)e0;
        const uint32_t ic = p.dv.khw.div(e), rem = e - ic * (uint32_t)(a.kh * a.kw);
        const uint32_t i = p.dv.kw.div(rem), j = rem - i * (uint32_t)a.kw;
        tap_offs[e0] = ((ic * (uint32_t)hh + i * (uint32_t)a.dil) * (uint32_t)ww + j * (uint32_t)a.dil) * 4;
        tap_needs[e0] = (int)e < kk ? ((1u << i) | (0x10000u << j)) : 0x80000000u;
    }
    __syncthreads();
    const uint32_t all_bits = ((1u << a.kh) - 1u) | (((1u << a.kw) - 1u) << 16);
    const bool inside = __builtin_amdgcn_ballot_w64(okbits != all_bits) == 0;   // (wave-uniform)

    // ---- phase 1: steps wv, wv + 4, ...: taps -> quantised A operand in LDS
    int qs = 0;
    auto fetch = [&](int s, float(&v)[16]) {
        const u32x4 *po = reinterpret_cast<const u32x4 *>(tap_offs + 32 * s + 16 * hf);
        if (inside && 32 * s + 32 <= kk) {
#pragma unroll
            for (int t4 = 0; t4 < 4; t4++) {
                const u32x4 o4 = po[t4];
#pragma unroll
                for (int t = 0; t < 4; t++)
                    v[t4 * 4 + t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xbuf, lane_base + o4[t], 0, 0));
            }
        } else {
            const u32x4 *pn = reinterpret_cast<const u32x4 *>(tap_needs + 32 * s + 16 * hf);
#pragma unroll
            for (int t4 = 0; t4 < 4; t4++) {
                const u32x4 o4 = po[t4], n4 = pn[t4];
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const uint32_t vo = (okbits & n4[t]) == n4[t] ? lane_base + o4[t] : ~0u;
                    v[t4 * 4 + t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xbuf, vo, 0, 0));
                }
            }
        }
    };
    auto quantise = [&](int s, const float(&v)[16]) {
        int q[16];
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const float x = (v[t] - za) * inv;
            const int qi = (int)(x + __builtin_copysignf(0.49999997f, x));
            q[t] = max(qlo, min(qi, qhi));
        }
        i32x4 af;
#pragma unroll
        for (int wi = 0; wi < 4; wi++) {
            int tp[4];
#pragma unroll
            for (int bq = 0; bq < 4; bq++) {
                const int pos = wi * 4 + bq, sl = pos & 7;
                tp[bq] = (pos & 8) + (W4 ? ((sl & 3) * 2 + (sl >> 2)) : sl);
            }
            const uint32_t lo = __builtin_amdgcn_perm((uint32_t)q[tp[1]], (uint32_t)q[tp[0]], 0x0c0c0400u);
            const uint32_t hi = __builtin_amdgcn_perm((uint32_t)q[tp[3]], (uint32_t)q[tp[2]], 0x04000c0cu);
            af[wi] = (int)(lo | hi);
        }
        const int past = 32 * s + 16 * hf + 16 - kk;   // taps of this lane past K: their bytes are cleared
        if (past > 0) {
#pragma unroll
            for (int wi = 0; wi < 4; wi++) {
                uint32_t keep = 0;
#pragma unroll
                for (int bq = 0; bq < 4; bq++) {
                    const int pos = wi * 4 + bq, sl = pos & 7;
                    const int tpp = (pos & 8) + (W4 ? ((sl & 3) * 2 + (sl >> 2)) : sl);
                    keep |= (tpp < 16 - past) ? (0xffu << (8 * bq)) : 0u;
                }
                af[wi] &= (int)keep;
            }
        }
#pragma unroll
        for (int wi = 0; wi < 4; wi++) qs = __builtin_amdgcn_sdot4(af[wi], 0x01010101, qs, false);
        *reinterpret_cast<i32x4 *>(a_lds + ((size_t)s * 64 + lane) * 16) = af;
    };
    {
        float v0[16], v1[16];
        int s = wv;
        if (s < nsteps) fetch(s, v0);
        for (; s < nsteps; s += 2 * NW) {
            if (s + NW < nsteps) fetch(s + NW, v1);
            quantise(s, v0);
            if (s + NW < nsteps) {
                if (s + 2 * NW < nsteps) fetch(s + 2 * NW, v0);
                quantise(s + NW, v1);
            }
        }
    }
    qs += __shfl_xor(qs, 32, 64);   // the two k halves of a pixel
    if (hf == 0) r_qsw[wv][lr] = qs;
    if (wv == 0 && hf == 0) {
        r_sa[lr] = sa; r_za[lr] = za;
        r_off[lr] = (int64_t)nn * a.oc * np + px;
        if (RNG) r_img[lr] = nn != nn0;
    }
    __syncthreads();

    // ---- phase 2: channel blocks wv, wv + 4, ... over the whole K range
    const int64_t wleft = ((int64_t)a.oc - (int64_t)g * ocg) * a.kp * 4 + 256;   // (the zeroed margin behind the last row)
    const __amdgpu_buffer_rsrc_t wbuf = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t *>(a.words + (int64_t)g * ocg * a.kp), 0, (int)(uint32_t)(wleft > 0xfffffff0ll ? 0xfffffff0ll : wleft), 0x00020000);
    float mn0 = INFINITY, mx0 = -INFINITY, mn1 = INFINITY, mx1 = -INFINITY;
    bool rng_two = false, rng_plain = false;
    if constexpr (RNG) {
        const uint32_t row_z = (uint32_t)(r_first + 31 < rows ? r_first + 31 : rows - 1);
        rng_two = r_first < rows && row_z > (nn0 + 1) * np - 1;
        rng_plain = !rng_two && r_first + 32 <= rows;
    }
    const bool has_bias = a.bias != nullptr;
    float *y = a.y + (int64_t)g * ocg * np;
    int32_t *acc_out = a.acc_out ? a.acc_out + (int64_t)g * ocg * np : nullptr;
    const float *residual = a.residual ? a.residual + (int64_t)g * ocg * np : nullptr;
    float *sum_out = a.sum_out + (int64_t)g * ocg * np;
    const int nblocks = (ocg + TN * 32 - 1) / (TN * 32);
    for (int cb = wv; cb < nblocks; cb += NW) {
        const int n0 = cb * (TN * 32);
        uint32_t wlane[TN];
        float sw[TN], zw[TN], bi[TN];
        int wq_[TN];
#pragma unroll
        for (int tn = 0; tn < TN; tn++) {
            const int n = n0 + tn * 32 + lr;
            const bool ok = n < ocg;
            wlane[tn] = ok ? (uint32_t)n * (uint32_t)a.kp * 4 + (uint32_t)(hf * WBYTES) : ~0u;   // rows past the group: zero weights
            const int64_t ch = (int64_t)g * ocg + (ok ? n : 0);
            sw[tn] = ok ? a.scales[ch] : 0.0f;
            zw[tn] = ok ? a.zeros[ch] : 0.0f;
            wq_[tn] = ok ? a.row_qsum[ch] : 0;
            bi[tn] = (ok && a.bias) ? a.bias[ch] : 0.0f;
        }
        i32x16 acc[TN];
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[tn][i] = 0;
        auto wfetch = [&](int s, u32x4(&wq)[TN]) {
#pragma unroll
            for (int tn = 0; tn < TN; tn++) {
                const uint32_t wo_ = wlane[tn] == ~0u ? ~0u : wlane[tn] + (uint32_t)s * (2 * WBYTES);
                if (W4) {
                    const auto t2 = __builtin_amdgcn_raw_buffer_load_b64(wbuf, wo_, 0, 0);
                    wq[tn][0] = t2[0]; wq[tn][1] = t2[1]; wq[tn][2] = 0; wq[tn][3] = 0;
                } else {
                    wq[tn] = __builtin_amdgcn_raw_buffer_load_b128(wbuf, wo_, 0, 0);
                }
            }
        };
        auto multiply = [&](int s, const u32x4(&wq)[TN]) {
            const i32x4 af = *reinterpret_cast<const i32x4 *>(a_lds + ((size_t)s * 64 + lane) * 16);
#pragma unroll
            for (int tn = 0; tn < TN; tn++) {
                const uint32_t w4[4] = {wq[tn][0], wq[tn][1], wq[tn][2], wq[tn][3]};
                const f16x8 bf = DecI<DT>::step(w4);
                acc[tn] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, __builtin_bit_cast(i32x4, bf), acc[tn], 0, 0, 0);
            }
        };
        {   // four steps' weights in flight (a ring of eight measured slower: registers, fewer waves per SIMD)
            u32x4 w0[TN], w1[TN], w2[TN], w3[TN];
            wfetch(0, w0);
            if (1 < nsteps) wfetch(1, w1);
            if (2 < nsteps) wfetch(2, w2);
            for (int s = 0; s < nsteps; s += 4) {
                if (s + 3 < nsteps) wfetch(s + 3, w3);
                multiply(s, w0);
                if (s + 1 < nsteps) {
                    if (s + 4 < nsteps) wfetch(s + 4, w0);
                    multiply(s + 1, w1);
                }
                if (s + 2 < nsteps) {
                    if (s + 5 < nsteps) wfetch(s + 5, w1);
                    multiply(s + 2, w2);
                }
                if (s + 3 < nsteps) {
                    if (s + 6 < nsteps) wfetch(s + 6, w2);
                    multiply(s + 3, w3);
                }
            }
        }
        // ---- epilogue of the block: acc[tn][i] = pixel (i/4)*8 + hf*4 + i%4, channel n0 + tn*32 + lr
#pragma unroll
        for (int ig = 0; ig < 4; ig++) {
            const int rr0 = ig * 8 + hf * 4;
            const int64_t r0 = r_first + rr0;
            if (r0 >= rows) continue;
            float rsa[4], rza[4], rs[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                rsa[j] = r_sa[rr0 + j];
                rza[j] = r_za[rr0 + j];
                rs[j] = rsa[j] * (float)(r_qsw[0][rr0 + j] + r_qsw[1][rr0 + j] + r_qsw[2][rr0 + j] + r_qsw[3][rr0 + j]);
            }
#pragma unroll
            for (int tn = 0; tn < TN; tn++) {
                const int64_t n = n0 + tn * 32 + lr;
                if (n >= ocg) continue;
                float v[4];
                int av[4], bq[4];
                bq[0] = has_bias ? conv_bias_q(bi[tn], rsa[0], sw[tn]) : 0;
#pragma unroll
                for (int j = 1; j < 4; j++) bq[j] = (p.vec4 || !has_bias) ? bq[0] : conv_bias_q(bi[tn], rsa[j], sw[tn]);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    int ai = acc[tn][ig * 4 + j];
                    if (W4) ai >>= 4;
                    v[j] = conv_affine(ai, rsa[j], rza[j], rs[j], sw[tn], zw[tn], sw[tn] * (float)wq_[tn], bq[j], kk, &av[j]);
                }
                conv_act4(v, a.act);
                // a.residual: the Add behind this convolution; v becomes the sums, whose ranges travel on instead of y's
                if (p.vec4) {
                    const int64_t o = r_off[rr0] + n * np;
                    *reinterpret_cast<float4 *>(y + o) = make_float4(v[0], v[1], v[2], v[3]);
                    if (acc_out) *reinterpret_cast<int4 *>(acc_out + o) = make_int4(av[0], av[1], av[2], av[3]);
                    if (residual) {
                        const float4 r4 = *reinterpret_cast<const float4 *>(residual + o);
                        v[0] = v[0] + r4.x; v[1] = v[1] + r4.y; v[2] = v[2] + r4.z; v[3] = v[3] + r4.w;
                        *reinterpret_cast<float4 *>(sum_out + o) = make_float4(v[0], v[1], v[2], v[3]);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        if (r0 + j >= rows) continue;
                        const int64_t o = r_off[rr0 + j] + n * np;
                        y[o] = v[j];
                        if (acc_out) acc_out[o] = av[j];
                        if (residual) {
                            v[j] = v[j] + residual[o];
                            sum_out[o] = v[j];
                        }
                    }
                }
                if constexpr (RNG) {
                    if (rng_plain) {   // (workgroup-uniform) every pixel of the block exists and lies in one image
                        mn0 = fminf(fminf(mn0, fminf(v[0], v[1])), fminf(v[2], v[3]));
                        mx0 = fmaxf(fmaxf(mx0, fmaxf(v[0], v[1])), fmaxf(v[2], v[3]));
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            if (r0 + j >= rows) continue;
                            if (rng_two && r_img[rr0 + j]) { mn1 = fminf(mn1, v[j]); mx1 = fmaxf(mx1, v[j]); }
                            else { mn0 = fminf(mn0, v[j]); mx0 = fmaxf(mx0, v[j]); }
                        }
                    }
                }
            }
        }
    }
    if constexpr (RNG) {
        if (r_first >= rows) return;   // (workgroup-uniform)
        // one pair per workgroup (block of 32 pixels) and channel group: pair (block - first block of the image) of
        // every image the block meets, np / 32 + 2 pairs per image and group; the waves leave theirs in LDS, the last to
        // arrive writes
        mn0 = wave_min(mn0); mx0 = wave_max(mx0);
        if (rng_two) { mn1 = wave_min(mn1); mx1 = wave_max(mx1); }
        int arrived = 0;
        if (lane == 0) {
            s_rng[wv][0] = mn0; s_rng[wv][1] = mx0; s_rng[wv][2] = mn1; s_rng[wv][3] = mx1;
            __threadfence_block();
            arrived = atomicAdd(&s_cnt, 1);
            __threadfence_block();
        }
        if (lane == 0 && arrived == NW - 1) {
            constexpr uint32_t BM = 32;
            const uint32_t row_z = (uint32_t)(r_first + BM - 1 < rows ? r_first + BM - 1 : rows - 1);
            const uint32_t img_end = (nn0 + 1) * np - 1;
            const int slot = (int)(blockIdx.x - (nn0 * np) / BM), per_m = (int)(np / BM) + 2;
            const int fill = row_z >= img_end ? slot + 1 : per_m;
            // p.rng_blocks > 1 (at most one channel block per wave): wave w's pair is that of channel block w, and the
            // pairs of a block lie together (a reader of some of the channels takes its blocks' pairs); else one pair
            // for all channels
            const int groups = p.rng_blocks > 1 ? p.rng_blocks : 1;
            for (int gq = 0; gq < groups; gq++) {
                float m0 = s_rng[gq][0], x0 = s_rng[gq][1], m1 = s_rng[gq][2], x1 = s_rng[gq][3];
                if (groups == 1) {
#pragma unroll
                    for (int w2 = 1; w2 < NW; w2++) {
                        m0 = fminf(m0, s_rng[w2][0]); x0 = fmaxf(x0, s_rng[w2][1]);
                        m1 = fminf(m1, s_rng[w2][2]); x1 = fmaxf(x1, s_rng[w2][3]);
                    }
                }
                float *row = a.range_out + (int64_t)nn0 * a.range_out_stride * 2 + (int64_t)gq * per_m * 2;
                float *dst = row + (int64_t)slot * 2;
                dst[0] = m0; dst[1] = x0;
                if (rng_two) {   // the next image starts in this block: its pair 0
                    float *d1 = row + (int64_t)a.range_out_stride * 2;
                    d1[0] = m1; d1[1] = x1;
                }
                for (int j = fill; j < per_m; j++) {
                    float *d2 = row + (int64_t)j * 2;
                    d2[0] = INFINITY; d2[1] = -INFINITY;
                }
            }
        }
    }
}

template <int DT, int TN>
hipError_t launch_fused(const ImplicitArgs &p, int64_t rows, hipStream_t s)
{
    const size_t lds = (size_t)((p.kk + 31) / 32) * 1024;
    const dim3 grid((unsigned)((rows + 31) / 32));
    if (p.a.range_out) hipLaunchKernelGGL((conv_fused_kernel<DT, TN, true>), grid, dim3(256), lds, s, p);
    else hipLaunchKernelGGL((conv_fused_kernel<DT, TN, false>), grid, dim3(256), lds, s, p);
    return hipGetLastError();
}

template <int DT, int TN, int PW, int KW>
hipError_t launch_implicit(const ImplicitArgs &p, int64_t rows, int64_t ocg, hipStream_t s)
{
    constexpr size_t lds = (size_t)PW * (KW - 1) * (TN * 16 + 1) * 64 * 4;
    static_assert(lds <= 48 * 1024, "the K slices meet in the default LDS allowance");
    const dim3 grid((unsigned)((rows + 32 * PW - 1) / (32 * PW)), (unsigned)((ocg + TN * 32 - 1) / (TN * 32)));
    const bool tab = (p.kk + 31) / 32 * 32 <= TAP_TABLE;
    if (p.a.range_out) {
        if (tab) hipLaunchKernelGGL((conv_implicit_kernel<DT, TN, PW, KW, true, true>), grid, dim3(64 * PW * KW), lds, s, p);
        else hipLaunchKernelGGL((conv_implicit_kernel<DT, TN, PW, KW, true, false>), grid, dim3(64 * PW * KW), lds, s, p);
    } else {
        if (tab) hipLaunchKernelGGL((conv_implicit_kernel<DT, TN, PW, KW, false, true>), grid, dim3(64 * PW * KW), lds, s, p);
        else hipLaunchKernelGGL((conv_implicit_kernel<DT, TN, PW, KW, false, false>), grid, dim3(64 * PW * KW), lds, s, p);
    }
    return hipGetLastError();
}

template <int DT>
hipError_t run_implicit(const ImplicitArgs &p, int64_t rows, int64_t ocg, int tn, int kw, hipStream_t s)
{
    if (tn == 2) {
        if (kw == 4) return launch_implicit<DT, 2, 1, 4>(p, rows, ocg, s);
        if (kw == 2) return launch_implicit<DT, 2, 2, 2>(p, rows, ocg, s);
        return launch_implicit<DT, 2, 4, 1>(p, rows, ocg, s);
    }
    if (kw == 4) return launch_implicit<DT, 1, 1, 4>(p, rows, ocg, s);
    if (kw == 2) return launch_implicit<DT, 1, 2, 2>(p, rows, ocg, s);
    return launch_implicit<DT, 1, 4, 1>(p, rows, ocg, s);
}

// shape of the launch: channels per wave (tn * 32), K slices per pixel block, pixels of a workgroup
void implicit_shape(const QConvArgs &p, int *tn_out, int *kw_out, int *wg_rows)
{
    const int64_t np = p.ho * p.wo, rows = p.b * np;
    const int64_t ocg = p.oc / p.groups, kk = (p.c / p.groups) * p.kh * p.kw;
    const int tn = ocg > 32 ? 2 : 1;
    const int64_t ntn = (ocg + tn * 32 - 1) / (tn * 32);
    const int64_t steps = (kk + 31) / 32;
    // K slices per pixel block: more of them while the launch would leave CUs idle and a slice keeps a few steps
    int kw = 1;
    if (((rows + 127) / 128) * ntn < 512 && steps >= 4) kw = 2;
    if (((rows + 63) / 64) * ntn < 256 && steps >= 8) kw = 4;
    *tn_out = tn; *kw_out = kw; *wg_rows = 128 / kw;   // four waves: 4, 2 or 1 pixel blocks of 32
}

}  // namespace

namespace {

// Which one-launch form runs this convolution: 0 = none (operand kernel + GEMM), 1 = conv_implicit_kernel, 2 =
// conv_fused_kernel.  option: FNN_OPT_CONV_IMPLICIT (0: by shape, where each measured faster; 1: the implicit kernel
// wherever it can run; 2: neither; 3: the fused kernel wherever it can run).
int implicit_form(const fnn_hip_weight *w, const QConvArgs &p, int option)
{
    if (option == 2) return 0;
    if ((w->dtype != FNN_DT_I8 && w->dtype != FNN_DT_I4) || p.x8 || p.payload_i4) return 0;
    const int64_t np = p.ho * p.wo, rows = p.b * np;
    const int64_t cg = p.c / p.groups, ocg = p.oc / p.groups, kk = cg * p.kh * p.kw;
    if (rows < 1 || rows > (1ll << 28) || kk > (1 << 20) || ocg < 1) return 0;
    if (cg * p.h * p.w >= (1ll << 29) || np >= (1ll << 31)) return 0;
    int tn, kw, wr;
    implicit_shape(p, &tn, &kw, &wr);
    const int64_t span = p.b < (wr - 1) / np + 2 ? p.b : (wr - 1) / np + 2;   // images under one buffer descriptor
    if (p.kh > 15 || p.kw > 15 || span * p.c * p.h * p.w * 4 > 0xfffffff0ll) return 0;
    if (p.pad > 32767 || p.dil > 32767 || p.stride > 32767) return 0;
    if (ocg * p.kp * 4 > 0x7fffffffll) return 0;   // 32-bit byte offsets inside the group's weight rows
    const bool fused_fits = (kk + 31) / 32 <= FUSED_MAX_STEPS && (kk + 31) / 32 * 32 <= TAP_TABLE;
    if (option == 1) return 1;
    if (option == 3) return fused_fits ? 2 : 0;
    // By shape, from YOLOv8n-shaped layers at 640 x 640, one image and sixteen (us, implicit / pair / fused).
    // The implicit kernel passes over the pixels once per 32 * tn channels: ahead while the channels fit one MFMA
    // column block (409 600 pixels, 16 -> 16 3x3: 38 / 72 / 66; 6400 pixels, 32 -> 32 3x3: 8.6 / 11.8 / 8.7) or two and
    // the pixels fill the chip several times (102 400 pixels, 64 channels: 18.3 / 28.1 / 23.0).
    if (ocg <= 32 && rows >= 2048) return 1;
    if (ocg <= 64 && rows >= 65536) return 1;
    // ... or, whatever the channels, a K of one or two steps under many pixels: nothing to save by quantising once
    // (25 088 pixels, 64 -> 256 1x1: 20.8 / 26.6 / 23.9)
    if (kk <= 64 && rows >= 12800) return 1;
    // The fused kernel quantises once for all channels: ahead from 33 channels on where its workgroups (32 pixels each)
    // fill half the chip (25 600 pixels: 64 -> 64 3x3 18.6 / 20.9 / 15.7, 384 -> 128 1x1 23.3 / 25.3 / 18.9, 64 -> 128 3x3
    // stride 2 38.1 / 32.0 / 25.5; not 128 -> 256 3x3 at 6400 pixels: 46 / 25 / 28), and with fewer workgroups while a
    // wave's chain of steps stays short (1600 pixels: 128 -> 128 1x1 10.9 / 10.7 / 7.3, 64 -> 64 3x3 13.9 / 12.6 / 12.1;
    // 400 pixels: 256 -> 128 1x1 11.8 / 10.5 / 8.1, 128 -> 256 3x3 22 / 15.6 / 28).
    if (fused_fits) {
        const int64_t wgs = (rows + 31) / 32, nsteps = (kk + 31) / 32, passes = (ocg + 127) / 128;
        if (wgs >= 128) {
            if (!(ocg > 128 && nsteps > 18)) return 2;
        } else if (nsteps * passes <= 12 || (wgs >= 96 && nsteps * passes <= 20)) {   // (3136 pixels, 64 -> 64 3x3: 14.6 / 14.9 / 12.9)
            return 2;
        }
    }
    if (ocg <= 64 && rows >= 12800) return 1;
    return 0;
}

}  // namespace

// Does a one-launch kernel take this convolution?  *wg_rows = pixels of one of its workgroups, *wgs = their number (the
// caller decides with them whether the kernel forms the activation scales itself: a workgroup's rows must meet at
// most two images).
bool fnn_implicit_conv_takes(const fnn_hip_weight *w, const QConvArgs &p, int option, int *wg_rows, int64_t *wgs)
{
    const int form = implicit_form(w, p, option);
    if (form == 0) return false;
    const int64_t rows = p.b * p.ho * p.wo, ocg = p.oc / p.groups;
    int tn, kw, wr;
    implicit_shape(p, &tn, &kw, &wr);
    if (form == 2) wr = 32;   // (one workgroup per 32 pixels, whatever the channels)
    if (wg_rows) *wg_rows = wr;
    if (wgs) *wgs = ((rows + wr - 1) / wr) * (form == 2 ? 1 : (ocg + tn * 32 - 1) / (tn * 32));
    return true;
}

// p.range_out: the partial ranges of y are left when a workgroup meets at most two images and the pairs fit
// (ctx's out_parts says so), as by the fused epilogue of the explicit path
int fnn_i8_implicit_conv(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QConvArgs &p, bool *handled)
{
    *handled = false;
    const int form = implicit_form(w, p, (int)fnn_ctx_option(ctx, FNN_OPT_CONV_IMPLICIT));
    if (form == 0) return FNN_OK;
    const int64_t np = p.ho * p.wo, rows = p.b * np;
    const int64_t cg = p.c / p.groups, ocg = p.oc / p.groups, kk = cg * p.kh * p.kw;
    int tn, kw, wg_rows;
    implicit_shape(p, &tn, &kw, &wg_rows);
    ImplicitArgs ia;
    ia.a = p;
    ia.dv = ConvDivs{fast_div((uint32_t)np), fast_div((uint32_t)p.wo), fast_div((uint32_t)(p.kh * p.kw)), fast_div((uint32_t)p.kw)};
    ia.kk = (int)kk;
    const bool with_sum = p.residual && p.sum_out;
    if (!with_sum) ia.a.residual = nullptr;
    ia.vec4 = (np % 4 == 0 && (reinterpret_cast<uintptr_t>(p.y) & 15) == 0 && (!p.acc_out || (reinterpret_cast<uintptr_t>(p.acc_out) & 15) == 0) &&
               (!with_sum || ((reinterpret_cast<uintptr_t>(p.residual) | reinterpret_cast<uintptr_t>(p.sum_out)) & 15) == 0)) ? 1 : 0;
    if (form == 2) wg_rows = 32;
    // range pairs: per channel block (of the implicit form's column tiles; of the fused form's waves when every wave
    // has at most one block), np / wg_rows + 2 pairs per image and block
    const int block_ch = form == 2 ? (ocg > 128 ? 64 : 32) : tn * 32;
    const int64_t nblocks = (ocg + block_ch - 1) / block_ch;
    ia.rng_blocks = (form == 2 && nblocks <= 4 && (np / wg_rows + 2) * nblocks <= p.range_out_stride) ? (int)nblocks : 1;   // (else one pair for all channels)
    const int64_t groups_of_pairs = form == 2 ? ia.rng_blocks : nblocks;
    const int64_t parts = (np / wg_rows + 2) * groups_of_pairs;
    if (p.range_out && p.groups == 1 && np >= wg_rows && parts <= p.range_out_stride) {
        FnnRangeIo *rio = fnn_ctx_range_io(ctx);
        rio->out_parts = (int)parts;
        if (groups_of_pairs == nblocks) { rio->out_tile_elems = (uint64_t)block_ch * (uint64_t)np; rio->out_tile_pairs = (int)(np / wg_rows + 2); }
    } else {
        ia.a.range_out = nullptr;
    }
    for (int g = 0; g < p.groups; g++) {
        ia.g = g;
        hipError_t e;
        if (form == 2) {
            // two blocks of 32 channels per wave from 256 channels on: four waves then cover them in one pass
            if (w->dtype == FNN_DT_I8) e = ocg > 128 ? launch_fused<FNN_DT_I8, 2>(ia, rows, s) : launch_fused<FNN_DT_I8, 1>(ia, rows, s);
            else e = ocg > 128 ? launch_fused<FNN_DT_I4, 2>(ia, rows, s) : launch_fused<FNN_DT_I4, 1>(ia, rows, s);
        } else {
            e = w->dtype == FNN_DT_I8 ? run_implicit<FNN_DT_I8>(ia, rows, ocg, tn, kw, s) : run_implicit<FNN_DT_I4>(ia, rows, ocg, tn, kw, s);
        }
        if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    }
    if (with_sum) fnn_ctx_residual_io(ctx)->used = 1;   // the epilogue stored y + residual as well
    *handled = true;
    return FNN_OK;
}
