// Integer matrix-core path for gfx950: I8 activations x I8/I4 weights with exact i32 accumulators
// on v_mfma_i32_32x32x32_i8, serving
//   - "matmul_i8_i8" / "matmul_i4_i8" (gemm_cpu_flat_i8_i8x4 / gemm_cpu_flat_i8_i4x8,
//     src/backend/cpu/microkernels/gemm.rs:1641-1975), and
//   - the quantised Conv2d lowering conv2d_packed_i8x4 (im2col + per-(image,group) int8 activation
//     quantisation + integer GEMM + 4-term dequantise, src/backend/cpu/packed_conv.rs:125-232,444-625).
// An operand kernel writes the int8 activation matrix in the tile-major layout of the GEMM kernel (for conv it
// evaluates im2col and the quantisation on the fly) and leaves sum_k q_a per row; the shared tiled GEMM kernel
// produces the i32 accumulators.  MatMul: an epilogue kernel applies the reference's float formula to them.
// Conv: the same formula, the activation and the NCHW stores run inside the GEMM kernel (or, by option and for
// the matmul-form epilogue of 4-bit weights on an int8 payload, as a kernel of their own).
#include "mfma.h"
#include "dech.h"
#include "range_io.h"

#include <type_traits>

namespace {

using namespace dech;

constexpr float LO_UP = 2048.0f, LO_DOWN = 1.0f / 2048.0f;   // f16 mode of the shared kernel (unused here)
#include "tile_kernel.h"

constexpr int KB = 128;   // k-values (= bytes) per stage and activation row

// position of k inside its group of 8 in the operand: identity, or 0,2,4,6,1,3,5,7 for nibble weights
__device__ __forceinline__ int slot_of(int j, int interleaved) { return interleaved ? ((j & 1) * 4 + (j >> 1)) : j; }

// ---- I8-activation MatMul operand: payload rows -> tile-major int8 [kpad/128][rows_pad][128] + sum q_a per row.
// Whole 16-byte chunks of 8-byte aligned rows are moved as two 8-byte loads (a byte permutation for the
// interleaved operand of the nibble decoders, a 4-way dot with ones for the row sum); ragged ends byte by byte.
template <bool IL>
__global__ void __launch_bounds__(256) i8_rows_operand_kernel(const int8_t *qa, int64_t m, int64_t k, int64_t kpad,
                                                              int64_t rows_pad, int8_t *a8, int32_t *qsum)
{
    __shared__ int red[4];
    const int64_t r = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const bool rows_aligned = (k % 8 == 0) && ((reinterpret_cast<uintptr_t>(qa) & 7) == 0);
    int s = 0;
    for (int64_t c = tid; c < kpad / 16; c += 256) {   // 16-byte chunk c of the row
        uint32_t out[4] = {0, 0, 0, 0};
        if (r < m) {
            if (rows_aligned && c * 16 + 16 <= k) {
                const uint2 lo = *reinterpret_cast<const uint2 *>(qa + r * k + c * 16);
                const uint2 hi = *reinterpret_cast<const uint2 *>(qa + r * k + c * 16 + 8);
                s += __builtin_amdgcn_sdot4((int)lo.x, 0x01010101, 0, false) + __builtin_amdgcn_sdot4((int)lo.y, 0x01010101, 0, false) +
                     __builtin_amdgcn_sdot4((int)hi.x, 0x01010101, 0, false) + __builtin_amdgcn_sdot4((int)hi.y, 0x01010101, 0, false);
                if (IL) {   // operand slot order k = 0,2,4,6,1,3,5,7 of each 8
                    out[0] = __builtin_amdgcn_perm(lo.y, lo.x, 0x06040200u);
                    out[1] = __builtin_amdgcn_perm(lo.y, lo.x, 0x07050301u);
                    out[2] = __builtin_amdgcn_perm(hi.y, hi.x, 0x06040200u);
                    out[3] = __builtin_amdgcn_perm(hi.y, hi.x, 0x07050301u);
                } else {
                    out[0] = lo.x; out[1] = lo.y; out[2] = hi.x; out[3] = hi.y;
                }
            } else {
#pragma unroll
                for (int g8 = 0; g8 < 2; g8++)
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const int64_t kk = c * 16 + g8 * 8 + j;
                        const int q = kk < k ? (int)qa[r * k + kk] : 0;
                        s += q;
                        const int pos = g8 * 8 + slot_of(j, IL);
                        out[pos >> 2] |= (uint32_t)(uint8_t)q << (8 * (pos & 3));
                    }
            }
        }
        const int64_t kb = c >> 3, cc = c & 7;
        *reinterpret_cast<uint4 *>(a8 + (kb * rows_pad + r) * KB + cc * 16) = make_uint4(out[0], out[1], out[2], out[3]);
    }
    s = wave_sum_i32(s);
    if (lane == 0) red[wv] = s;
    __syncthreads();
    if (tid == 0) qsum[r] = (red[0] + red[1]) + (red[2] + red[3]);
}

// res = dot*sw + zw*input_sum with dot = acc*sa, input_sum = sum(q_a)*sa + K*za
// (gemm.rs:1641-1975).  With za != 0 the reference multiplies per lane in f32; the same quantity is
// formed here from the integer sums: sum (q_a*sa + za)*q_w = sa*acc + za*sum_k q_w.
__global__ void __launch_bounds__(256) i8_matmul_epilogue_kernel(const int32_t *c, const uint8_t *payload, const int32_t *qsum,
                                                                 const int32_t *wsum, const float *scales, const float *zeros,
                                                                 int64_t m, int64_t n, int64_t k, float *out, int32_t *acc_out, int splits,
                                                                 const float *bias, int act)
{
    // a thread owns one output column (its weight constants stay in registers) and walks rows blockIdx.y, +gridDim.y, ...
    const float sa = reinterpret_cast<const float *>(payload)[0];
    const float za = reinterpret_cast<const float *>(payload)[1];
    const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (col >= n) return;
    const float sw = scales[col], zw = zeros[col];
    const float zwsum = za * (float)wsum[col];
    const float kza = (float)k * za;
    const float bs = bias ? bias[col] : 0.0f;
    for (int64_t r = blockIdx.y; r < m; r += gridDim.y) {
        const int64_t idx = r * n + col;
        int acc = c[idx];
        for (int z = 1; z < splits; z++) acc += c[(int64_t)z * m * n + idx];   // exact whatever the order
        const float input_sum = (float)qsum[r] * sa + kza;
        const float dot = (za != 0.0f) ? (float)acc * sa + zwsum : (float)acc * sa;
        float v = dot * sw + zw * input_sum;
        if (bias) v = v + bs;
        out[idx] = fnn_activation(v, act);
        if (acc_out) acc_out[idx] = (za != 0.0f) ? 0 : acc;
    }
}

// ---- conv operand: im2col row (image nn, pixel p) of group g, quantised with the (image, group) scale:
// q = clamp(round((v - za) * inv), -128, 127)  (packed_conv.rs:149-232); for an input that is already int8
// (X8) the values are taken as they are and padding taps are the integer 0 (packed_conv.rs:69-115).
// A workgroup owns 64 consecutive rows and CONV_CPB * NC 16-value chunks of them: wave `slot` takes NC consecutive
// chunks, so the (channel, tap) geometry is the same for the whole wave and lives in scalar registers, neighbouring
// lanes = neighbouring pixels (the NCHW reads coalesce), and what a lane works out about its pixel (image, position,
// which kernel rows and columns fall inside the image) is paid once per NC * 16 taps.  All loads of a wave are
// requested before the first value is used.
constexpr int CONV_CPB = 4;   // waves per workgroup, each with its own chunks


template <bool X8, bool W4, int NC>   // X8: int8 input; W4: 4-bit weights (16 activation levels unless X8, interleaved operand)
                                      // NC <= 4: a wave's taps are worked out one per lane
__global__ void __launch_bounds__(256) conv_operand_kernel(QConvArgs a, int g, int kk, int64_t kpad, int64_t rows_pad,
                                                           int8_t *a8, int32_t *qsum, ConvDivs dv)
{
    __shared__ int part[4][64];
    const int tid = threadIdx.x, rr = tid & 63;
    const int slot = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave index: the chunk geometry stays in scalar registers
    const uint32_t np = (uint32_t)(a.ho * a.wo), wo = (uint32_t)a.wo;
    const int64_t r = (int64_t)blockIdx.x * 64 + rr;
    const int64_t rows = a.b * (int64_t)np;   // < 2^31 (checked on the host)
    const int cg = (int)a.c / a.groups;
    const int live_chunks = (kk + 15) / 16;
    const bool live = r < rows;
    const int c0 = ((int)blockIdx.y * CONV_CPB + slot) * NC;   // this wave's first chunk
    // Scales not formed yet (a.nparts > 0): every workgroup reduces the partial ranges of the (at most two) images
    // its 64 rows belong to and derives scale, zero and 1/scale exactly as conv_actq_kernel does; the workgroups of
    // the first chunk group also store them for the epilogue.
    __shared__ float s_mm[2][2][4];
    __shared__ float s_q[2][3];
    const int64_t r_first = (int64_t)blockIdx.x * 64;
    const bool own_scales = !X8 && a.nparts > 0 && r_first < rows;
    const uint32_t nn0 = dv.np.div((uint32_t)(r_first < rows ? r_first : 0));   // image of the workgroup's first row
    int bg_a = 0;
    if (own_scales) {
        const int64_t r_last = r_first + 63 < rows ? r_first + 63 : rows - 1;
        bg_a = (int)nn0 * a.groups + g;
        const int bg_b = (int)dv.np.div((uint32_t)r_last) * a.groups + g;
        const int nimg = bg_b != bg_a ? 2 : 1;
        for (int w = 0; w < nimg; w++) {
            const float *part = a.minmax_partial + (int64_t)(w ? bg_b : bg_a) * a.part_stride * 2;
            float mn = a.range_zero ? 0.0f : INFINITY, mx = a.range_zero ? 0.0f : -INFINITY;
            conv_fold_partial_ranges(part, a.nparts, tid, 256, mn, mx);
            mn = wave_min(mn);
            mx = wave_max(mx);
            if (rr == 0) { s_mm[w][0][tid >> 6] = mn; s_mm[w][1][tid >> 6] = mx; }
        }
        __syncthreads();
        if (tid < nimg) {
            const float mn = fminf(fminf(s_mm[tid][0][0], s_mm[tid][0][1]), fminf(s_mm[tid][0][2], s_mm[tid][0][3]));
            const float mx = fmaxf(fmaxf(s_mm[tid][1][0], s_mm[tid][1][1]), fmaxf(s_mm[tid][1][2], s_mm[tid][1][3]));
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
            if (blockIdx.y == 0) {
                float *dst = a.actq + (tid ? bg_b : bg_a) * 4;
                dst[0] = scale; dst[1] = zero; dst[2] = inv; dst[3] = 0.0f;
            }
        }
        __syncthreads();
    }
    int s = 0;
    if (r < rows_pad && c0 < live_chunks) {
        const uint32_t ru = live ? (uint32_t)r : 0u;
        const uint32_t nn = dv.np.div(ru), p = ru - nn * np;
        const uint32_t oh = dv.wo.div(p), ow = p - oh * wo;
        const int bg = (int)nn * a.groups + g;
        float za, inv;
        if (X8 || a.nparts <= 0) {
            za = a.actq[bg * 4 + 1]; inv = a.actq[bg * 4 + 2];
        } else {
            const int w = (own_scales && bg != bg_a) ? 1 : 0;
            za = own_scales ? s_q[w][1] : 0.0f; inv = own_scales ? s_q[w][2] : 0.0f;
        }
        // One buffer descriptor per wave, from the group's slab in the image of the workgroup's first row to the end
        // of the tensor: a lane's byte offset is (images further on) * image size + pixel offset + tap offset, and a
        // tap outside the image (or past K, or of a row past the last one) gets the offset ~0, which the buffer
        // range check answers with zero: no branch, no select on the loaded value (the host checked that the offsets
        // of one workgroup fit 32 bits).
        constexpr uint32_t ESZ = X8 ? 1 : 4;
        const int64_t img = a.c * a.h * a.w;
        const int64_t slab0 = ((int64_t)nn0 * a.c + (int64_t)g * cg) * a.h * a.w;
        const void *base = X8 ? (const void *)(a.x8 + slab0) : (const void *)(a.x + slab0);
        const int64_t left = (a.b * img - slab0) * ESZ;   // bytes from there to the end of the tensor
        const __amdgpu_buffer_rsrc_t xbuf = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<void *>(base), 0, (int)(uint32_t)(left > 0xfffffff0ll ? 0xfffffff0ll : left), 0x00020000);
        const int hh = (int)a.h, ww = (int)a.w;
        constexpr int qlo = W4 ? -8 : -128, qhi = W4 ? 7 : 127;
        constexpr int interleaved = W4;   // the 4-bit weight decoder delivers k = 0,2,4,6,1,3,5,7 of each 8
        const int ih0 = (int)oh * a.stride - a.pad, iw0 = (int)ow * a.stride - a.pad;
        // which kernel rows (bits 0..14) and columns (bits 16..30) land inside the image for this pixel; bit 31 stays
        // clear: taps past K ask for it
        uint32_t okbits = 0;
        for (int i = 0; i < a.kh; i++) okbits |= ((unsigned)(ih0 + i * a.dil) < (unsigned)hh ? 1u : 0u) << i;
        for (int j = 0; j < a.kw; j++) okbits |= ((unsigned)(iw0 + j * a.dil) < (unsigned)ww ? 0x10000u : 0u) << j;
        if (!live) okbits = 0;
        const uint32_t lane_base = ((uint32_t)(nn - nn0) * (uint32_t)img + (uint32_t)(ih0 * ww + iw0)) * ESZ;   // (mod 2^32)
        // Tap geometry: lane t works out tap e0 + t of this wave (channel, kernel row, kernel column -> offset inside
        // the slab and the two bits the tap needs), and the unrolled loop below reads each tap's pair into scalar
        // registers: no per-tap index arithmetic on either unit.
        const int e0 = c0 * 16;
        uint32_t tap_off, tap_need;
        {
            const uint32_t e = (uint32_t)(e0 + rr);
            const uint32_t ic = dv.khw.div(e), rem = e - ic * (uint32_t)(a.kh * a.kw);
            const uint32_t i = dv.kw.div(rem), j = rem - i * (uint32_t)a.kw;
            tap_off = ((ic * (uint32_t)hh + i * (uint32_t)a.dil) * (uint32_t)ww + j * (uint32_t)a.dil) * ESZ;
            tap_need = (int)e < kk ? ((1u << i) | (0x10000u << j)) : 0x80000000u;
        }
        float v[NC][16];
        int v8[NC][16];
#pragma unroll
        for (int cc = 0; cc < NC; cc++)
#pragma unroll
            for (int t = 0; t < 16; t++) {
                const uint32_t soff = (uint32_t)__builtin_amdgcn_readlane((int)tap_off, cc * 16 + t);
                const uint32_t need = (uint32_t)__builtin_amdgcn_readlane((int)tap_need, cc * 16 + t);
                const uint32_t vo = (okbits & need) == need ? lane_base + soff : ~0u;
                if (X8) v8[cc][t] = (int)(int8_t)__builtin_amdgcn_raw_buffer_load_b8(xbuf, vo, 0, 0);
                else v[cc][t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xbuf, vo, 0, 0));
            }
#pragma unroll
        for (int cc = 0; cc < NC; cc++) {
            const int c = c0 + cc;
            if (c >= live_chunks) break;   // (wave-uniform)
            int q[16];
#pragma unroll
            for (int t = 0; t < 16; t++) {
                if (X8) {
                    q[t] = v8[cc][t];
                } else {
                    // round half away from zero, then clamp: trunc(x + copysign(0.49999997, x)) equals roundf(x)
                    // after the clamp for every float (the conversion truncates, saturates and maps NaN to 0)
                    const float x = (v[cc][t] - za) * inv;
                    const int qi = (int)(x + __builtin_copysignf(0.49999997f, x));
                    q[t] = max(qlo, min(qi, qhi));
                }
            }
            // byte `pos` of the 16 holds tap (pos & 8) + k(pos & 7), k = the inverse of slot_of; the row sum is a
            // 4-way dot with ones
            uint32_t out[4];
            int tp[16];
#pragma unroll
            for (int pos = 0; pos < 16; pos++) {
                const int sl = pos & 7;
                tp[pos] = (pos & 8) + (interleaved ? ((sl & 3) * 2 + (sl >> 2)) : sl);
            }
#pragma unroll
            for (int wi = 0; wi < 4; wi++) {
                const uint32_t lo = __builtin_amdgcn_perm((uint32_t)q[tp[wi * 4 + 1]], (uint32_t)q[tp[wi * 4 + 0]], 0x0c0c0400u);
                const uint32_t hi = __builtin_amdgcn_perm((uint32_t)q[tp[wi * 4 + 3]], (uint32_t)q[tp[wi * 4 + 2]], 0x04000c0cu);
                out[wi] = lo | hi;
            }
            if (c * 16 + 16 > kk) {   // (wave-uniform) the chunk K ends in: bytes of taps past K are cleared
#pragma unroll
                for (int wi = 0; wi < 4; wi++) {
                    uint32_t keep = 0;
#pragma unroll
                    for (int bq = 0; bq < 4; bq++) keep |= (c * 16 + tp[wi * 4 + bq] < kk) ? (0xffu << (8 * bq)) : 0u;
                    out[wi] &= keep;
                }
            }
#pragma unroll
            for (int wi = 0; wi < 4; wi++) s = __builtin_amdgcn_sdot4((int)out[wi], 0x01010101, s, false);
            *reinterpret_cast<uint4 *>(a8 + ((int64_t)(c >> 3) * rows_pad + r) * KB + (c & 7) * 16) = make_uint4(out[0], out[1], out[2], out[3]);
        }
    }
    part[slot][rr] = s;
    // Chunks past the data (k >= K rounded up to 16) are not written: the weight operand is zero there
    // (rows end in zero lanes and reads past a row go to the zero chunk), and an int8 product with zero is
    // zero whatever the activation byte holds.
    __syncthreads();
    // one partial sum per chunk group; the epilogue adds them
    const int64_t qrow = (int64_t)blockIdx.x * 64 + tid;
    if (tid < 64 && qrow < rows_pad) qsum[(int64_t)blockIdx.y * rows_pad + qrow] = (part[0][tid] + part[1][tid]) + (part[2][tid] + part[3][tid]);
}

// acc = bias_q + sum q_a*q_w; val = acc*sab + zw*(sa*sum q_a) + za*(sw*sum q_w) + (za*zw)*K, left to right,
// then the activation (packed_conv.rs:469-505,571,604-606).  A workgroup takes 64 rows of C (read along the
// channels, as stored), turns the tile in LDS and writes NCHW with consecutive lanes on consecutive pixels.
constexpr int EPI_CH = 32;   // channels per epilogue workgroup

__global__ void __launch_bounds__(256) conv_epilogue_kernel(QConvArgs a, int g, int kk, const int32_t *c, int ocg,
                                                            const int32_t *qsum, int nq, int64_t rows_pad)
{
    __shared__ float tile[EPI_CH * 65];   // [channel of the block][row], padded
    __shared__ int itile[EPI_CH * 65];    // accumulators incl. bias_q, same shape
    __shared__ int r_part[4][64];                            // partial sums of q_a per row
    __shared__ float r_sa[64], r_za[64], r_sum[64];          // per row: activation scale / zero of its image, sa * sum q_a
    __shared__ float c_sw[EPI_CH], c_zw[EPI_CH], c_wt[EPI_CH], c_bias[EPI_CH];   // per channel
    const uint32_t np = (uint32_t)(a.ho * a.wo);
    const int64_t rows = a.b * (int64_t)np;
    const int64_t row0 = (int64_t)blockIdx.x * 64;
    const int f0 = blockIdx.y * EPI_CH;
    const int fb = ocg - f0 < EPI_CH ? ocg - f0 : EPI_CH;   // channels of this block
    const int tid = threadIdx.x;
    {
        // sum q_a of a row: its nq partial sums are split over the four waves and read four at a time
        const int part = tid >> 6, rr = tid & 63;
        const int64_t r = row0 + rr;
        int qs = 0;
        if (r < rows) {
            const int32_t *q = qsum + r;
            int y = part;
            for (; y + 12 < nq; y += 16) {
                const int q0 = q[(int64_t)y * rows_pad], q1 = q[(int64_t)(y + 4) * rows_pad];
                const int q2 = q[(int64_t)(y + 8) * rows_pad], q3 = q[(int64_t)(y + 12) * rows_pad];
                qs += (q0 + q1) + (q2 + q3);
            }
            for (; y < nq; y += 4) qs += q[(int64_t)y * rows_pad];
        }
        r_part[part][rr] = qs;
        if (tid < 64) {
            if (r < rows) {
                const int bg = (int)((uint32_t)r / np) * a.groups + g;
                r_sa[tid] = a.actq[bg * 4 + 0];
                r_za[tid] = a.actq[bg * 4 + 1];
            }
        } else if (tid < 64 + fb) {
            const int fl = tid - 64;
            const int64_t ch = (int64_t)g * ocg + f0 + fl;
            const float sw = a.scales[ch];
            c_sw[fl] = sw;
            c_zw[fl] = a.zeros[ch];
            c_wt[fl] = sw * (float)a.row_qsum[ch];
            c_bias[fl] = a.bias ? a.bias[ch] : 0.0f;
        }
    }
    __syncthreads();
    if (tid < 64) r_sum[tid] = r_sa[tid] * (float)((r_part[0][tid] + r_part[1][tid]) + (r_part[2][tid] + r_part[3][tid]));
    __syncthreads();
    auto element = [&](int rr, int fl, int acc_in) {
        const float sa = r_sa[rr], za = r_za[rr];
        const float sw = c_sw[fl], zw = c_zw[fl];
        int accv;
        float val;
        if (a.payload_i4) {
            // gemm_cpu_flat_i8_i4x8 on the gathered rows, then `+ bias` in f32 (mod.rs:3975-4032);
            // for za != 0 the dot of the dequantised activations is formed from the integer sums
            accv = acc_in;
            const float dot = (za != 0.0f) ? (float)accv * sa + za * (float)a.row_qsum[(int64_t)g * ocg + f0 + fl] : (float)accv * sa;
            const float input_sum = r_sum[rr] + (float)kk * za;
            val = dot * sw + zw * input_sum;
            if (a.bias) val += c_bias[fl];
            if (a.act == FNN_ACT_RELU) val = fmaxf(val, 0.0f);
            else if (a.act == FNN_ACT_SILU) val = val / (1.0f + expf(-val));
            else if (a.act == FNN_ACT_GELU) val = val * 0.5f * (1.0f + tanhf(val * 0.7978846f * (1.0f + 0.044715f * val * val)));
        } else {
            val = conv_dequant(acc_in, sa, za, r_sum[rr], sw, zw, c_wt[fl], a.bias ? conv_bias_q(c_bias[fl], sa, sw) : 0, kk, a.act, &accv);
        }
        tile[fl * 65 + rr] = val;
        itile[fl * 65 + rr] = accv;
    };
    // consecutive threads on consecutive channels of a row of C (as stored); for the usual block widths the
    // (row, channel) of a thread comes from shifts and all of its accumulators are requested together
    if (fb == 32 || fb == 16) {
        const int sh = fb == 32 ? 5 : 4;
        const int fl = tid & (fb - 1), rbase = tid >> sh, rstep = 256 >> sh, n_it = 64 / rstep;   // 8 or 4 rows per thread
        int accs[8];
#pragma unroll
        for (int it = 0; it < 8; it++) {
            const int64_t r = row0 + rbase + it * rstep;
            accs[it] = (it < n_it && r < rows) ? c[r * ocg + f0 + fl] : 0;
        }
#pragma unroll
        for (int it = 0; it < 8; it++) {
            const int rr = rbase + it * rstep;
            if (it < n_it && row0 + rr < rows) element(rr, fl, accs[it]);
        }
    } else {
        for (int idx = tid; idx < 64 * fb; idx += 256) {
            const int rr = idx / fb, fl = idx - rr * fb;
            const int64_t r = row0 + rr;
            if (r < rows) element(rr, fl, c[r * ocg + f0 + fl]);
        }
    }
    __syncthreads();
    // NCHW stores: consecutive lanes on consecutive pixels
    const int rr = tid & 63;
    const int64_t r = row0 + rr;
    if (r < rows) {
        const uint32_t nn = (uint32_t)r / np, p = (uint32_t)r - nn * np;
        for (int fl = tid >> 6; fl < fb; fl += 4) {
            const int64_t o = ((int64_t)nn * a.oc + (int64_t)g * ocg + f0 + fl) * np + p;
            a.y[o] = tile[fl * 65 + rr];
            if (a.acc_out) a.acc_out[o] = itile[fl * 65 + rr];
        }
    }
}

template <int DT, int WGM, int WGN, int TM, int TN, int NS, bool CONV = false, bool CRNG = false, bool FP8 = false>
hipError_t launch_i8_tile(const TileArgs &p, hipStream_t s)
{
    if constexpr (CONV && !CRNG) {
        if (p.cv.range_out) return launch_i8_tile<DT, WGM, WGN, TM, TN, NS, true, true>(p, s);
    }
    constexpr int WC = 2 * DecI<DT>::WPS;
    constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
    constexpr size_t lds = (size_t)NS * (BM * 128 + BN * WC * 16);
    auto kern = qgemm_tile_kernel<DT, WGM, WGN, TM, TN, false, NS, true, 0, CONV, CRNG, FP8>;
    static std::atomic<uint64_t> lds_raised{0};
    hipError_t e = fnn_raise_lds_limit(lds_raised, reinterpret_cast<const void *>(kern), (int)lds);
    if (e != hipSuccess) return e;
    // (a ring of three requests only the stages its K range has: one LDS buffer per stage, at most three)
    const int bufs = (NS == 3 && p.ips < NS) ? p.ips : NS;
    hipLaunchKernelGGL(kern, dim3((unsigned)p.mtiles * p.ntiles * p.splits), dim3(WGM * WGN * 64), lds / NS * bufs, s, p);
    return hipGetLastError();
}

__global__ void __launch_bounds__(256) restride_rows_kernel(const uint32_t *src, int64_t rows, int64_t kp, int64_t kp4, uint32_t *dst)
{
    const int64_t total = rows * kp4 + 16;   // + zero margin
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t r = i / kp4, c = i % kp4;
        dst[i] = (r < rows && c < kp) ? src[r * kp + c] : 0u;
    }
}

}  // namespace

// weight rows as 16-byte addressable pieces: the registered words, or a re-strided copy when kp % 4 != 0
int fnn_aligned_rows(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const uint32_t **words, int64_t *kp)
{
    if (w->kp % 4 == 0) { *words = w->words; *kp = w->kp; return FNN_OK; }
    fnn_hip_weight *wm = const_cast<fnn_hip_weight *>(w);
    if (!wm->words4) {
        if (fnn_ctx_no_alloc(ctx)) return fnn_ctx_fail(ctx, FNN_ERR_MEMORY, "first use of re-strided weight rows while allocation is not allowed (graph capture, fnn_hip_qmatmul_static)");
        const int64_t kp4 = (w->kp + 3) / 4 * 4;
        if (hipMalloc((void **)&wm->words4, (size_t)(w->rows * kp4 + 16) * 4) != hipSuccess)
            return fnn_ctx_fail(ctx, FNN_ERR_MEMORY, "out of device memory (re-strided weight rows)");
        wm->kp4 = kp4;
        int64_t blocks = (w->rows * kp4 + 16 + 255) / 256;
        if (blocks > 2048) blocks = 2048;
        hipLaunchKernelGGL(restride_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, s, w->words, w->rows, w->kp, kp4, wm->words4);
        if (hipGetLastError() != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, "re-striding weight rows failed");
    }
    *words = wm->words4; *kp = wm->kp4;
    return FNN_OK;
}

namespace {

// C[m][n] = sum_k A8[m][k] * q_w[n0 + n][k] for `n` weight rows starting at row n0 (rows of kp words, 16-byte aligned)
// `conv` (optional): the conv epilogue runs inside the kernel (scales / zeros / bias / act in it are the group's) and c is not written
template <int DT>
hipError_t run_i8_gemm(const uint32_t *words, int64_t kp, int64_t rows_total, int64_t n0, int64_t n, const int8_t *a8, int64_t m,
                       int64_t rows_pad, int64_t kpad, int32_t *c, int64_t ldc, hipStream_t s, int splits = 1, const TileArgs *conv = nullptr,
                       bool small_tiles = false, int form = 0)
{
    TileArgs t = {};
    if (conv) { t.cv = conv->cv; t.scales = conv->scales; t.zeros = conv->zeros; t.bias = conv->bias; t.act = conv->act; }
    t.words = words + n0 * kp;
    t.zero_chunk = words + rows_total * kp;   // the zeroed margin behind the last row
    t.ap = reinterpret_cast<const _Float16 *>(a8);
    t.c_i32 = c; t.ldc = ldc;
    t.m = m; t.n = n; t.kp = kp; t.kpad = kpad; t.rows_pad = rows_pad;
    t.iters = (int)(kpad / KB);
    t.ips = (t.iters + splits - 1) / splits;
    t.splits = (t.iters + t.ips - 1) / t.ips;   // (no empty split; the caller sized c for `splits` partial matrices)
    t.mtiles = (int)(rows_pad / 128); t.a_wrap = 0;
    if (conv && small_tiles) {   // few rows: 64 x 64 tiles put the epilogue's arithmetic on four times as many waves
        t.mtiles = (int)(rows_pad / 64);
        t.ntiles = (int)((n + 63) / 64);
        return launch_i8_tile<DT, 2, 2, 1, 1, 3, true>(t, s);
    }
    if (n <= 64) {   // narrow outputs (early conv layers): 128 x 64 tiles, four waves stacked along M
        t.ntiles = (int)((n + 63) / 64);
        return conv ? launch_i8_tile<DT, 4, 1, 1, 2, 3, true>(t, s) : launch_i8_tile<DT, 4, 1, 1, 2, 3>(t, s);
    }
    t.ntiles = (int)((n + 127) / 128);
    if (!conv && form == 1) return launch_i8_tile<DT, 2, 4, 2, 1, 3>(t, s);      // 128 x 128 on eight waves of 64 x 32
    if (!conv && form == 2) {                                                    // 256 x 128 on eight waves of 64 x 64
        t.mtiles = (int)((rows_pad + 255) / 256);
        return launch_i8_tile<DT, 4, 2, 2, 2, 3>(t, s);
    }
    return conv ? launch_i8_tile<DT, 2, 2, 2, 2, 3, true>(t, s) : launch_i8_tile<DT, 2, 2, 2, 2, 3>(t, s);
}

}  // namespace

// ---- FNN_FLAG_ACT_QUANT with F8 weights: f32 activations rounded to E4M3, fp8 matrix cores.
// Row m is scaled by a power of two that brings its largest magnitude into [128, 256) (E4M3 reaches 448) and rounded
// to nearest-even E4M3 by v_cvt_pk_fp8_f32; the bytes go into the tile-major operand layout of the int8 kernels.
// No counterpart in fastnn (it has no fp8 activation quantiser): a fast mode with a stated tolerance.
namespace {

__global__ void __launch_bounds__(256) fp8_rows_operand_kernel(const float *a, int64_t m, int64_t k, int64_t kpad, int64_t rows_pad,
                                                               int8_t *a8, float *rscale)
{
    __shared__ float red[4];
    const int64_t r = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    float mx = 0.0f;
    const bool vec = (k % 4 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15) == 0);   // rows start on 16-byte boundaries
    if (r < m) {
        if (vec) {
            for (int64_t i = tid; i < k / 4; i += 256) {
                const float4 t = reinterpret_cast<const float4 *>(a + r * k)[i];
                mx = fmaxf(mx, fmaxf(fmaxf(fabsf(t.x), fabsf(t.y)), fmaxf(fabsf(t.z), fabsf(t.w))));
            }
        } else {
            for (int64_t i = tid; i < k; i += 256) mx = fmaxf(mx, fabsf(a[r * k + i]));
        }
    }
    mx = wave_max(mx);
    if (lane == 0) red[wv] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    int ex = (int)((__float_as_uint(mx) >> 23) & 0xff) - 127 - 7;   // mx * 2^-ex in [128, 256)
    if (mx == 0.0f) ex = 0;
    ex = ex < -100 ? -100 : (ex > 120 ? 120 : ex);
    const float inv = __uint_as_float((uint32_t)(127 - ex) << 23);
    for (int64_t c = tid; c < kpad / 16; c += 256) {   // 16-byte chunk c of the row
        uint32_t out[4] = {0, 0, 0, 0};
        if (r < m) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                float v[4];
                const int64_t k0 = c * 16 + q * 4;
                if (vec && k0 + 4 <= k) {
                    const float4 t = *reinterpret_cast<const float4 *>(a + r * k + k0);
                    v[0] = t.x * inv; v[1] = t.y * inv; v[2] = t.z * inv; v[3] = t.w * inv;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) v[j] = k0 + j < k ? a[r * k + k0 + j] * inv : 0.0f;
                }
                int w = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], 0, false);
                w = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], w, true);
                out[q] = (uint32_t)w;
            }
        }
        const int64_t kb = c >> 3, cc = c & 7;
        *reinterpret_cast<uint4 *>(a8 + (kb * rows_pad + r) * KB + cc * 16) = make_uint4(out[0], out[1], out[2], out[3]);
    }
    if (tid == 0 && r < m) rscale[r] = __uint_as_float((uint32_t)(127 + ex) << 23);
}

// out[m,n] = act((sum over splits of the f32 partial sums) * 2^e[m] * scale[n] + bias[n]), partials added in split order
__global__ void __launch_bounds__(256) fp8_matmul_epilogue_kernel(const float *c, const float *rscale, const float *scales, const float *bias,
                                                                  int64_t m, int64_t n, float *out, int splits, int act)
{
    // a thread owns four consecutive columns (16-byte loads and stores where n % 4 == 0 and the buffers are aligned)
    const int64_t col0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (col0 >= n) return;
    const bool vec = col0 + 4 <= n && n % 4 == 0 && ((reinterpret_cast<uintptr_t>(c) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    float sw[4], bs[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const bool ok = col0 + j < n;
        sw[j] = ok ? scales[col0 + j] : 0.0f;
        bs[j] = (ok && bias) ? bias[col0 + j] : 0.0f;
    }
    for (int64_t r0 = (int64_t)blockIdx.y * 2; r0 < m; r0 += (int64_t)gridDim.y * 2) {   // two rows per trip, loads first
        float acc[2][4] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
        float rs[2] = {0.0f, 0.0f};
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const int64_t r = r0 + t;
            if (r >= m) break;
            const int64_t idx = r * n + col0;
            rs[t] = rscale[r];
            if (vec) {
                const float4 v0 = *reinterpret_cast<const float4 *>(c + idx);
                acc[t][0] = v0.x; acc[t][1] = v0.y; acc[t][2] = v0.z; acc[t][3] = v0.w;
                for (int z = 1; z < splits; z++) {
                    const float4 u = *reinterpret_cast<const float4 *>(c + (int64_t)z * m * n + idx);
                    acc[t][0] += u.x; acc[t][1] += u.y; acc[t][2] += u.z; acc[t][3] += u.w;
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (col0 + j < n) {
                        acc[t][j] = c[idx + j];
                        for (int z = 1; z < splits; z++) acc[t][j] += c[(int64_t)z * m * n + idx + j];
                    }
            }
        }
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const int64_t r = r0 + t;
            if (r >= m) break;
            const int64_t idx = r * n + col0;
            float o[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float v = (acc[t][j] * rs[t]) * sw[j];
                if (bias) v = v + bs[j];
                o[j] = fnn_activation(v, act);
            }
            if (vec) *reinterpret_cast<float4 *>(out + idx) = make_float4(o[0], o[1], o[2], o[3]);
            else {
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (col0 + j < n) out[idx + j] = o[j];
            }
        }
    }
}

}  // namespace

int fnn_fp8_actquant_qmatmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QMatmulArgs &q, bool *handled)
{
    *handled = false;
    if (w->dtype != FNN_DT_F8) return FNN_OK;
    if ((reinterpret_cast<uintptr_t>(q.words) & 15) || q.kp % 4 != 0) return FNN_OK;
    if (q.m < 1 || q.m > (1 << 22) || q.n > (1 << 24) || q.k > (1 << 20)) return FNN_OK;
    const int64_t kpad = (q.k + KB - 1) / KB * KB;
    const int64_t rows_pad = (q.m + 127) / 128 * 128;
    const size_t a_bytes = (size_t)rows_pad * kpad;
    const size_t r_off = (a_bytes + 255) / 256 * 256;
    const int64_t tiles = (rows_pad / 128) * ((q.n + 127) / 128);
    const int iters = (int)(kpad / KB);
    int splits = (int)(256 / (tiles > 0 ? tiles : 1));
    if (splits > iters / 4) splits = iters / 4;
    if (splits > 4) splits = 4;   // (more partial matrices cost more than the idle CUs they fill)
    if (splits < 1) splits = 1;
    void *ws0 = nullptr, *ws1 = nullptr;
    int rc;
    if ((rc = fnn_ctx_ensure_tmp(ctx, 0, r_off + (size_t)rows_pad * 4 + 256, &ws0))) return rc;
    if ((rc = fnn_ctx_ensure_tmp(ctx, 1, (size_t)splits * q.m * q.n * 4 + 256, &ws1))) return rc;
    int8_t *a8 = (int8_t *)ws0;
    float *rscale = (float *)((char *)ws0 + r_off);
    hipLaunchKernelGGL(fp8_rows_operand_kernel, dim3((unsigned)rows_pad), dim3(256), 0, s, q.a, q.m, q.k, kpad, rows_pad, a8, rscale);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    TileArgs t = {};
    t.words = q.words;
    t.zero_chunk = q.words + w->rows * q.kp;   // the zeroed margin behind the last row
    t.ap = reinterpret_cast<const _Float16 *>(a8);
    t.c_i32 = (int32_t *)ws1; t.ldc = q.n;
    t.m = q.m; t.n = q.n; t.kp = q.kp; t.kpad = kpad; t.rows_pad = rows_pad;
    t.iters = iters;
    t.ips = (iters + splits - 1) / splits;
    t.splits = (iters + t.ips - 1) / t.ips;
    t.mtiles = (int)(rows_pad / 128);
    t.ntiles = (int)((q.n + 127) / 128);
    e = launch_i8_tile<FNN_DT_I8, 2, 4, 2, 1, 3, false, false, true>(t, s);   // 128 x 128 on eight waves (every wave loads)
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    const int64_t colb = (q.n + 1023) / 1024;   // (four columns per thread)
    int64_t rowb = (4096 + colb - 1) / colb;
    if (rowb > (q.m + 1) / 2) rowb = (q.m + 1) / 2;   // (two rows per thread and trip)
    if (rowb > 65535) rowb = 65535;
    hipLaunchKernelGGL(fp8_matmul_epilogue_kernel, dim3((unsigned)colb, (unsigned)rowb), dim3(256), 0, s, (const float *)ws1, rscale, q.scales,
                       q.bias, q.m, q.n, q.out, t.splits, q.act);
    e = hipGetLastError();
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    *handled = true;
    return FNN_OK;
}

int fnn_i8_tiled_matmul(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const I8ActArgs &p, bool *handled)
{
    *handled = false;
    if (w->dtype != FNN_DT_I8 && w->dtype != FNN_DT_I4) return FNN_OK;
    if (reinterpret_cast<uintptr_t>(p.words) & 15) return FNN_OK;
    if (p.m < 1 || p.m > (1 << 22) || p.n > (1 << 24) || p.k > (1 << 20)) return FNN_OK;
    const int64_t kpad = (p.k + KB - 1) / KB * KB;
    const int64_t rows_pad = (p.m + 127) / 128 * 128;
    const size_t a_bytes = (size_t)rows_pad * kpad;
    const size_t q_off = (a_bytes + 255) / 256 * 256;
    void *ws0 = nullptr, *ws1 = nullptr;
    int rc;
    // K split over workgroups while the tiles alone leave CUs idle: the partial matrices are exact integers, so the
    // epilogue adds them in any order (4096 x 4096 at M = 256: 64 tiles, 31 -> 24 us with four K ranges)
    const int64_t tiles = (rows_pad / 128) * (p.n <= 64 ? (p.n + 63) / 64 : (p.n + 127) / 128);
    const int iters = (int)(kpad / KB);
    int splits = (int)(256 / (tiles > 0 ? tiles : 1));
    // Tile form: 128 x 128 on eight waves of 64 x 32 (every wave issues loads: 4096 x 4096 at M = 256 25.7 -> 24.3 us, M = 128
    // 21.9 -> 20.5), 256 x 128 on eight waves of 64 x 64 once those fill the chip unsplit (M = 2048: 90.6 -> 70.1 us);
    // FNN_OPT_TILE_SHAPE 0 / 1 / 2 picks the four-wave tiles / either of these.
    int form = (int)fnn_ctx_option(ctx, FNN_OPT_TILE_SHAPE);
    if (form < 0 || form > 2) form = (rows_pad % 256 == 0 && (rows_pad / 256) * ((p.n + 127) / 128) >= 256) ? 2 : 1;
    if (p.n <= 64) form = 0;
    if (form == 2 && rows_pad % 256) form = 1;
    if (form == 2) splits *= 2;
    if (splits > 4) splits = 4;   // (more partial matrices cost more than the idle CUs they fill: M = 128 23.8 -> 20.5 us)
    if (const int64_t forced = fnn_ctx_option(ctx, FNN_OPT_TILE_SPLIT); forced > 0) splits = (int)forced;
    if (splits > iters / 4) splits = iters / 4;
    if (splits > 16) splits = 16;
    if (splits < 1) splits = 1;
    if ((rc = fnn_ctx_ensure_tmp(ctx, 0, q_off + (size_t)rows_pad * 4 + 256, &ws0))) return rc;
    if ((rc = fnn_ctx_ensure_tmp(ctx, 1, (size_t)splits * p.m * p.n * 4 + 256, &ws1))) return rc;
    fnn_hip_weight *wm = const_cast<fnn_hip_weight *>(w);
    if (!wm->row_qsum) {
        if (fnn_ctx_no_alloc(ctx)) return fnn_ctx_fail(ctx, FNN_ERR_MEMORY, "first use of re-strided weight rows while allocation is not allowed (graph capture, fnn_hip_qmatmul_static)");
        if (hipMalloc((void **)&wm->row_qsum, (size_t)w->rows * 4 + 64) != hipSuccess)
            return fnn_ctx_fail(ctx, FNN_ERR_MEMORY, "out of device memory (row sums)");
        hipError_t e = launch_row_qsum(w, wm->row_qsum, s);
        if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    }
    const uint32_t *words;
    int64_t kp;
    if ((rc = fnn_aligned_rows(ctx, s, w, &words, &kp))) return rc;
    int8_t *a8 = (int8_t *)ws0;
    int32_t *qsum = (int32_t *)((char *)ws0 + q_off);
    int32_t *c = (int32_t *)ws1;
    const int interleaved = w->dtype == FNN_DT_I4 ? 1 : 0;
    if (interleaved)
        hipLaunchKernelGGL(i8_rows_operand_kernel<true>, dim3((unsigned)rows_pad), dim3(256), 0, s,
                           reinterpret_cast<const int8_t *>(p.payload + 8), p.m, p.k, kpad, rows_pad, a8, qsum);
    else
        hipLaunchKernelGGL(i8_rows_operand_kernel<false>, dim3((unsigned)rows_pad), dim3(256), 0, s,
                           reinterpret_cast<const int8_t *>(p.payload + 8), p.m, p.k, kpad, rows_pad, a8, qsum);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess)
        e = w->dtype == FNN_DT_I8 ? run_i8_gemm<FNN_DT_I8>(words, kp, w->rows, 0, p.n, a8, p.m, rows_pad, kpad, c, p.n, s, splits, nullptr, false, form)
                                  : run_i8_gemm<FNN_DT_I4>(words, kp, w->rows, 0, p.n, a8, p.m, rows_pad, kpad, c, p.n, s, splits, nullptr, false, form);
    if (e == hipSuccess) {
        const int ips = (iters + splits - 1) / splits;
        splits = (iters + ips - 1) / ips;   // as run_i8_gemm rounds it
        const int64_t colb = (p.n + 255) / 256;
        int64_t rowb = (4096 + colb - 1) / colb;   // about 4096 workgroups
        if (rowb > p.m) rowb = p.m;
        if (rowb > 65535) rowb = 65535;
        hipLaunchKernelGGL(i8_matmul_epilogue_kernel, dim3((unsigned)colb, (unsigned)rowb), dim3(256), 0, s, c, p.payload, qsum, wm->row_qsum,
                           p.scales, p.zeros, p.m, p.n, p.k, p.out, p.acc_out, splits, p.bias, p.act);
        e = hipGetLastError();
    }
    if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    *handled = true;
    return FNN_OK;
}

namespace {
// chunks per wave of the operand kernel: more of them spread a lane's per-pixel set-up over more taps, fewer keep the
// launch wide
int conv_chunks_per_wave(int64_t rows_pad, int64_t chunks)
{
    const int64_t wg1 = (rows_pad / 64) * ((chunks + CONV_CPB - 1) / CONV_CPB);   // workgroups with one chunk per wave
    if (wg1 < 2048) return 1;
    // enough workgroups left: the fewest chunk groups of at most 4 chunks per wave, evenly filled
    const int64_t groups_max = (chunks + CONV_CPB * 4 - 1) / (CONV_CPB * 4);
    return (int)((chunks + CONV_CPB * groups_max - 1) / (CONV_CPB * groups_max));
}
}  // namespace

// workgroups the operand kernel of this convolution launches per group (each reduces the partial activation ranges of
// its images itself when the scales are not formed yet)
int64_t fnn_conv_operand_workgroups(const QConvArgs &p)
{
    const int64_t rows = p.b * p.ho * p.wo, rows_pad = (rows + 127) / 128 * 128;
    const int64_t chunks = ((p.c / p.groups) * p.kh * p.kw + 15) / 16;
    const int nc = conv_chunks_per_wave(rows_pad, chunks);
    return (rows_pad / 64) * ((chunks + CONV_CPB * nc - 1) / (CONV_CPB * nc));
}

// after the (image, group) activation scales are known (p.actq): operand, integer GEMM and epilogue per group
int fnn_i8_tiled_conv(fnn_hip_ctx *ctx, hipStream_t s, const fnn_hip_weight *w, const QConvArgs &p, bool *handled)
{
    *handled = false;
    if ((w->dtype != FNN_DT_I8 && w->dtype != FNN_DT_I4) || (reinterpret_cast<uintptr_t>(p.words) & 15)) return FNN_OK;
    const int64_t np = p.ho * p.wo, rows = p.b * np;
    const int64_t cg = p.c / p.groups, ocg = p.oc / p.groups, kk = cg * p.kh * p.kw;
    if (rows < 1 || rows > (1ll << 28) || kk > (1 << 20) || ocg < 1) return FNN_OK;
    if (cg * p.h * p.w >= (1ll << 31) || p.ho * p.wo >= (1ll << 31)) return FNN_OK;   // 32-bit offsets inside an image slab
    // the operand kernel keeps one validity bit per kernel row / column (15 of each) and addresses the images a workgroup's 64
    // rows touch with 32-bit byte offsets from the first of them
    const int64_t span = p.b < 63 / np + 2 ? p.b : 63 / np + 2;
    if (p.kh > 15 || p.kw > 15 || span * p.c * p.h * p.w * 4 > 0xfffffff0ll) return FNN_OK;
    if (p.pad > 32767 || p.dil > 32767 || p.stride > 32767) return FNN_OK;   // (its 32-bit pixel and tap offsets)
    const int64_t kpad = (kk + KB - 1) / KB * KB;
    const int64_t rows_pad = (rows + 127) / 128 * 128;
    const size_t a_bytes = (size_t)rows_pad * kpad;
    const size_t q_off = (a_bytes + 255) / 256 * 256;
    void *ws1 = nullptr, *ws3 = nullptr;
    int rc;
    const int64_t chunks = (kk + 15) / 16;
    const int nc = conv_chunks_per_wave(rows_pad, chunks);
    const int nq = (int)((chunks + CONV_CPB * nc - 1) / (CONV_CPB * nc));   // partial row sums per row
    if (nq > 65535) return FNN_OK;
    if ((rc = fnn_ctx_ensure_tmp(ctx, 3, q_off + (size_t)rows_pad * 4 * nq + 256, &ws3))) return rc;   // 0 holds the scales
    if ((rc = fnn_ctx_ensure_tmp(ctx, 1, (size_t)rows * ocg * 4 + 256, &ws1))) return rc;
    const uint32_t *words;
    int64_t kp;
    if ((rc = fnn_aligned_rows(ctx, s, w, &words, &kp))) return rc;
    int8_t *a8 = (int8_t *)ws3;
    int32_t *qsum = (int32_t *)((char *)ws3 + q_off);
    int32_t *c = (int32_t *)ws1;
    if (ocg > 65535 * EPI_CH) return FNN_OK;
    // the epilogue inside the GEMM kernel (one launch and the accumulator matrix's trip through memory less) or as a
    // kernel of its own; the matmul-form epilogue of 4-bit weights on an int8 payload exists only as a kernel
    const int opt_fused = fnn_ctx_option(ctx, FNN_OPT_CONV_EPILOGUE);
    const bool fused = !p.payload_i4 && opt_fused != 2;
    const int64_t tiles128 = (rows_pad / 128) * (ocg <= 64 ? 1 : (ocg + 127) / 128);
    const bool small_tiles = tiles128 <= 256 && opt_fused != 3;   // less than one 128-row tile per CU
    const bool with_sum = fused && p.residual && p.sum_out;   // (the epilogue kernel of its own leaves the Add to its caller)
    const bool vec4 = np % 4 == 0 && (reinterpret_cast<uintptr_t>(p.y) & 15) == 0 && (!p.acc_out || (reinterpret_cast<uintptr_t>(p.acc_out) & 15) == 0) &&
                      (!with_sum || ((reinterpret_cast<uintptr_t>(p.residual) | reinterpret_cast<uintptr_t>(p.sum_out)) & 15) == 0);
    for (int g = 0; g < p.groups; g++) {
        const dim3 grid((unsigned)(rows_pad / 64), (unsigned)nq);
        const bool w4 = p.wbits == 4;
        const ConvDivs dv = {fast_div((uint32_t)np), fast_div((uint32_t)p.wo), fast_div((uint32_t)(p.kh * p.kw)), fast_div((uint32_t)p.kw)};
        auto launch = [&](auto kern) { hipLaunchKernelGGL(kern, grid, dim3(256), 0, s, p, g, (int)kk, kpad, rows_pad, a8, qsum, dv); };
        auto pick = [&](auto x8c, auto w4c) {
            constexpr bool X8 = decltype(x8c)::value, W4 = decltype(w4c)::value;
            if (nc == 4) launch(conv_operand_kernel<X8, W4, 4>);
            else if (nc == 3) launch(conv_operand_kernel<X8, W4, 3>);
            else if (nc == 2) launch(conv_operand_kernel<X8, W4, 2>);
            else launch(conv_operand_kernel<X8, W4, 1>);
        };
        if (p.x8 && w4) pick(std::true_type{}, std::true_type{});
        else if (p.x8) pick(std::true_type{}, std::false_type{});
        else if (w4) pick(std::false_type{}, std::true_type{});
        else pick(std::false_type{}, std::false_type{});
        hipError_t e = hipGetLastError();
        TileArgs cv = {};
        if (fused) {
            cv.scales = p.scales + g * ocg; cv.zeros = p.zeros + g * ocg; cv.bias = p.bias ? p.bias + g * ocg : nullptr; cv.act = p.act;
            cv.cv.y = p.y + g * ocg * np; cv.cv.acc_out = p.acc_out ? p.acc_out + g * ocg * np : nullptr;
            cv.cv.actq = p.actq; cv.cv.qsum = qsum; cv.cv.row_qsum = p.row_qsum + g * ocg;
            cv.cv.oc = p.oc; cv.cv.np = (uint32_t)np; cv.cv.nq = nq; cv.cv.groups = p.groups; cv.cv.g = g; cv.cv.kk = (int)kk;
            cv.cv.vec4 = vec4 ? 1 : 0;
            if (with_sum) { cv.cv.residual = p.residual + g * ocg * np; cv.cv.sum_out = p.sum_out + g * ocg * np; }
            // partial ranges of y (of the sums, with a residual) for the next convolution: one group, and tiles that meet at most two images
            const int64_t bm = small_tiles ? 64 : 128;
            const int64_t ntl = small_tiles ? (ocg + 63) / 64 : (ocg <= 64 ? 1 : (ocg + 127) / 128);
            const int64_t parts = (np / bm + 2) * ntl;
            if (p.range_out && p.groups == 1 && np >= bm && parts <= p.range_out_stride) {
                cv.cv.range_out = p.range_out; cv.cv.range_stride = p.range_out_stride;
                FnnRangeIo *rio = fnn_ctx_range_io(ctx);
                rio->out_parts = (int)parts;
                rio->out_tile_elems = (uint64_t)(small_tiles || ocg <= 64 ? 64 : 128) * (uint64_t)np;   // (the pairs of a column tile lie together)
                rio->out_tile_pairs = (int)(np / bm + 2);
            }
        }
        if (e == hipSuccess)
            e = w->dtype == FNN_DT_I8 ? run_i8_gemm<FNN_DT_I8>(words, kp, w->rows, g * ocg, ocg, a8, rows, rows_pad, kpad, c, ocg, s, 1, fused ? &cv : nullptr, small_tiles)
                                      : run_i8_gemm<FNN_DT_I4>(words, kp, w->rows, g * ocg, ocg, a8, rows, rows_pad, kpad, c, ocg, s, 1, fused ? &cv : nullptr, small_tiles);
        if (e == hipSuccess && !fused) {
            hipLaunchKernelGGL(conv_epilogue_kernel, dim3((unsigned)((rows + 63) / 64), (unsigned)((ocg + EPI_CH - 1) / EPI_CH)), dim3(256), 0, s, p, g,
                               (int)kk, c, (int)ocg, qsum, nq, rows_pad);
            e = hipGetLastError();
        }
        if (e != hipSuccess) return fnn_ctx_fail(ctx, FNN_ERR_DISPATCH, hipGetErrorString(e));
    }
    if (with_sum) fnn_ctx_residual_io(ctx)->used = 1;
    *handled = true;
    return FNN_OK;
}
