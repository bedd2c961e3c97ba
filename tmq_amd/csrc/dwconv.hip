// Depthwise ternary convolution (groups == channels) on 2-bit packed weights, gfx950.
//
//   y[p][c] = epilogue( sum_t x(p, t, c) * T[c][t] ),   t = (i, j) over the ky x kx taps
//
// The weight tensor [C][1][ky][kx] is packed by the reference as words[t][ceil(C/16)]
// (tmq/tmq_native.cpp:279-294 with one input channel): word (t, q) holds the codes of channels
// 16 q .. 16 q + 15 at tap t, first channel in bits 31:30. The kernels read that format directly.
//
// One multiply-add per input element: the op is bound by HBM traffic (2 B in / output element and
// tap on a cold cache, far less with the taps' overlap served from L2), not by arithmetic. A thread
// owns 8 consecutive channels of one output position -- 16-byte fp16 loads, neighbouring threads on
// neighbouring channel groups -- and applies a weight as two selects on the sign / nonzero bits.
//
// Two sources of x:
//   * NHWC image (tmq_ternary_dwconv2d): taps are gathered on the fly, padding reads as zero;
//   * unfolded patches [P][T][C] fp32, the calling convention of the reference's
//     ternary_dwconv_cuda (tmq/tmq_cuda.cu:166-238, host 607-642; caller tmq/tmq.py:849-853).
//
// Depthwise transposed convolution, y[b][oh][ow][c] = sum over (ih, i), (iw, j) with
// oh = ih sy - py + i dy, ow = iw sx - px + j dx of x[b][ih][iw][c] * T[c][i][j], in the same two forms:
//   * NHWC image (tmq_ternary_dwconvtrans2d): each output position gathers the inputs that reach it
//     (no columns, no col2im scatter);
//   * columns: y[b][c T + t][p] = x[b][p][c] * T[c][t], the calling convention of the reference's
//     ternary_dwconvtrans_cuda (tmq/tmq_cuda.cu:118-162, host 645-686; caller tmq/tmq.py:1026-1029),
//     whose result the caller scatters with F.fold. Pure data movement: 4 B in, 4 T B out per element.
#include <type_traits>

#include "common.h"
#include "mfma.h"

namespace tmq {
namespace {

struct DwEpilogue {
    const float *scale, *bias;
    const void *residual;
    void *y;
    int relu, y_f16;
};

// codes of 8 consecutive channels starting at c0 (a multiple of 8) from the word that holds them:
// returns them left-aligned, channel c0 in bits 31:30
__device__ __forceinline__ uint32_t codes8(const uint32_t *__restrict__ words, int64_t Q, int t, int64_t c0) {
    const uint32_t w = words[(int64_t)t * Q + (c0 >> 4)];
    return (c0 & 8) ? (w << 16) : w;
}

// value * {+1, -1, 0} for the code in bits 31:30 of `codes` (01 -> +1, 10 -> -1, 00 / 11 -> 0)
__device__ __forceinline__ float apply_code(float v, uint32_t codes) {
    const uint32_t c = codes >> 30;
    return c == 1u ? v : (c == 2u ? -v : 0.0f);
}

__device__ __forceinline__ void store8(const DwEpilogue &ep, int64_t o, int64_t c0, int64_t C, float (&acc)[8], int vec) {
#pragma unroll
    for (int e = 0; e < 8; e++) {
        if (c0 + e >= C) break;
        float v = acc[e];
        if (ep.scale) v *= ep.scale[c0 + e];
        if (ep.bias) v += ep.bias[c0 + e];
        if (ep.residual)
            v += ep.y_f16 ? (float)static_cast<const _Float16 *>(ep.residual)[o + e] : static_cast<const float *>(ep.residual)[o + e];
        if (ep.relu) v = v < 0.f ? 0.f : v;
        acc[e] = v;
    }
    if (vec == 2 && ep.y_f16) {                                    // a whole group whose pixel starts on 8 bytes
        half4 lo, hi;
#pragma unroll
        for (int e = 0; e < 4; e++) { lo[e] = (_Float16)acc[e]; hi[e] = (_Float16)acc[4 + e]; }
        *reinterpret_cast<half4 *>(static_cast<_Float16 *>(ep.y) + o) = lo;
        *reinterpret_cast<half4 *>(static_cast<_Float16 *>(ep.y) + o + 4) = hi;
    } else if (vec) {
        if (ep.y_f16) {
            half8 h;
#pragma unroll
            for (int e = 0; e < 8; e++) h[e] = (_Float16)acc[e];
            *reinterpret_cast<half8 *>(static_cast<_Float16 *>(ep.y) + o) = h;
        } else {
            float *yp = static_cast<float *>(ep.y) + o;
            *reinterpret_cast<floatx4 *>(yp) = floatx4{acc[0], acc[1], acc[2], acc[3]};
            *reinterpret_cast<floatx4 *>(yp + 4) = floatx4{acc[4], acc[5], acc[6], acc[7]};
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            if (c0 + e >= C) break;
            if (ep.y_f16) static_cast<_Float16 *>(ep.y)[o + e] = (_Float16)acc[e];
            else static_cast<float *>(ep.y)[o + e] = acc[e];
        }
    }
}

// The same epilogue as store8 for whole groups of 8 channels with 16-byte aligned tensors: scale and bias
// come in as two 16-byte loads each (once per thread), residual and result move 16 bytes at a time. Same
// operations in the same order as store8.
struct ChannelConstants {
    floatx4 sc[2], bi[2];
};

__device__ __forceinline__ ChannelConstants load_channel_constants(const DwEpilogue &ep, int64_t c0) {
    ChannelConstants cc;
    cc.sc[0] = cc.sc[1] = floatx4{1.f, 1.f, 1.f, 1.f};
    cc.bi[0] = cc.bi[1] = floatx4{0.f, 0.f, 0.f, 0.f};
    if (ep.scale) { cc.sc[0] = *reinterpret_cast<const floatx4 *>(ep.scale + c0); cc.sc[1] = *reinterpret_cast<const floatx4 *>(ep.scale + c0 + 4); }
    if (ep.bias) { cc.bi[0] = *reinterpret_cast<const floatx4 *>(ep.bias + c0); cc.bi[1] = *reinterpret_cast<const floatx4 *>(ep.bias + c0 + 4); }
    return cc;
}

__device__ __forceinline__ void store8_vec(const DwEpilogue &ep, const ChannelConstants &cc, int64_t o, const float (&acc)[8]) {
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        v[e] = acc[e];
        if (ep.scale) v[e] *= cc.sc[e >> 2][e & 3];
        if (ep.bias) v[e] += cc.bi[e >> 2][e & 3];
    }
    if (ep.residual) {
        if (ep.y_f16) {
            const half8 rs = *reinterpret_cast<const half8 *>(static_cast<const _Float16 *>(ep.residual) + o);
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] += (float)rs[e];
        } else {
            const floatx4 r0 = *reinterpret_cast<const floatx4 *>(static_cast<const float *>(ep.residual) + o);
            const floatx4 r1 = *reinterpret_cast<const floatx4 *>(static_cast<const float *>(ep.residual) + o + 4);
#pragma unroll
            for (int e = 0; e < 4; e++) { v[e] += r0[e]; v[4 + e] += r1[e]; }
        }
    }
    if (ep.relu) {
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = v[e] < 0.f ? 0.f : v[e];
    }
    if (ep.y_f16) {
        half8 h;
#pragma unroll
        for (int e = 0; e < 8; e++) h[e] = (_Float16)v[e];
        *reinterpret_cast<half8 *>(static_cast<_Float16 *>(ep.y) + o) = h;
    } else {
        float *yp = static_cast<float *>(ep.y) + o;
        *reinterpret_cast<floatx4 *>(yp) = floatx4{v[0], v[1], v[2], v[3]};
        *reinterpret_cast<floatx4 *>(yp + 4) = floatx4{v[4], v[5], v[6], v[7]};
    }
}

// NHWC fp16 image. grid.x covers P * ceil(C / 8) threads.
__global__ __launch_bounds__(256) void dwconv_image_kernel(const _Float16 *__restrict__ x, const uint32_t *__restrict__ words,
                                                           int B, int C, int H, int W, int Ho, int Wo, int ky, int kx,
                                                           int sy, int sx, int py, int px, int dy, int dx, int vec,
                                                           DwEpilogue ep) {
    const int64_t G = (C + 7) / 8, Q = (C + 15) / 16;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x, total = (int64_t)B * Ho * Wo * G;
    if (id >= total) return;
    int cg, ow, oh;
    const int64_t p = div_rem(id, (int)G, cg), c0 = (int64_t)cg * 8;
    const int64_t r = div_rem(p, Wo, ow);
    const int b = (int)div_rem(r, Ho, oh);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // Groups of 8 channels in 16- or 8-byte loads. With 8-byte pixels (vec & 4) the last, partial group of a pixel
    // reads on into the next pixel -- values that meet weight codes of zero and sums that are never stored -- except at
    // the tensor's last pixel, which goes element by element.
    const bool fast = (vec & 3) || (vec & 4);
    const int64_t last_pixel = (int64_t)B * H * W - 1;
    for (int i = 0; i < ky; i++) {
        const int ih = oh * sy - py + i * dy;
        if (ih < 0 || ih >= H) continue;
        for (int j = 0; j < kx; j++) {
            const int iw = ow * sx - px + j * dx;
            if (iw < 0 || iw >= W) continue;
            const int64_t pixel = ((int64_t)b * H + ih) * W + iw;
            const _Float16 *src = x + pixel * C + c0;
            uint32_t codes = codes8(words, Q, i * kx + j, c0);
            if (fast && ((vec & 3) || c0 + 8 <= C || pixel < last_pixel)) {
                // the codes as fp16 +-2.0 operands, two per register (see dwconv_square_image_kernel): the sums run at
                // twice their value and are halved below. (vec & 4: pixels start on 8 bytes only -- C a multiple of 4 --
                // and a whole group of 8 channels comes as two 8-byte loads.)
                half8 v;
                if (vec & 3) {
                    v = *reinterpret_cast<const half8 *>(src);
                } else {
                    const half4 lo = *reinterpret_cast<const half4 *>(src), hi = *reinterpret_cast<const half4 *>(src + 4);
                    v = half8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                }
                codes ^= (codes >> 1) & 0x55555555u;
                const uint32_t t = (codes & 0xFF000000u) | ((codes >> 8) & 0x0000FF00u);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const half2v w = __builtin_bit_cast(half2v, (t << (2 * e)) & 0xC000C000u);
                    acc[e] = __builtin_fmaf((float)v[e], (float)w[1], acc[e]);
                    acc[4 + e] = __builtin_fmaf((float)v[4 + e], (float)w[0], acc[4 + e]);
                }
            } else {
                // (fast: the sums run at twice their value, so this tap counts twice as well)
#pragma unroll
                for (int e = 0; e < 8; e++)
                    if (c0 + e < C) acc[e] += (fast ? 2.f : 1.f) * apply_code((float)src[e], codes << (2 * e));
            }
        }
    }
    if (fast) {
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] *= 0.5f;                 // exact: the weights were +-2
    }
    if (vec & 2) store8_vec(ep, load_channel_constants(ep, c0), p * C + c0, acc);
    else store8(ep, p * C + c0, c0, C, acc, (vec & 1) ? 1 : (((vec & 8) && c0 + 8 <= C) ? 2 : 0));
}

// The common cases -- windows of ky rows x KS columns (KS of 1 .. 5 or 7, any ky), horizontal stride 1 or 2 and
// dilation DX of 1 or 2, any vertical stride and dilation, whole groups of 8 channels, fewer than 2^31 threads. A
// thread owns 8 channels of PX horizontally adjacent output positions: the columns their windows share are loaded once
// (for stride 1, PX + KS - 1 columns per row instead of KS PX), the 8 weights of a tap are expanded to fp16 operands
// once for all PX positions, and the index arithmetic is multiply-high (FastDiv). All loads of a row are in
// flight together; taps outside the image read the clamped pixel and are replaced by zero. Per output the
// taps are accumulated in the same order as in dwconv_image_kernel (fp32, every product exact). Workgroups are taken
// in an order that keeps one XCD on neighbouring pieces of the image (the input rows that vertically adjacent
// outputs share then come from that XCD's L2: batch 64, 128 channels, 56 x 56, 3 x 3: 32.8 -> 28.4 us).
// KY: the window's rows when they equal KS and neither direction is dilated (the square windows of the common
// depthwise layers keep a compile-time row count), 0: ky and dy from the arguments.
template <int KS, int PX, int SX, int DX = 1, int KY = 0>
__global__ __launch_bounds__(256) void dwconv_square_image_kernel(const _Float16 *__restrict__ x, const uint32_t *__restrict__ words,
                                                              uint32_t total, int C, int H, int W, int Wo, FastDiv by_g,
                                                              FastDiv by_wg, FastDiv by_ho, int ky, int sy, int py, int px,
                                                              int dy, DwEpilogue ep) {
    constexpr int NC = (PX - 1) * SX + (KS - 1) * DX + 1;          // input columns the PX windows cover
    // workgroups of one XCD take neighbouring pieces of the image: the rows that vertically adjacent outputs share
    // are then found in that XCD's L2
    const uint32_t id = (uint32_t)xcd_contiguous((int)blockIdx.x, (int)gridDim.x) * 256u + threadIdx.x;
    if (id >= total) return;
    int cg, wg, oh;
    const uint32_t p = by_g.divmod(id, cg);                         // channel group fastest: neighbours share a pixel
    const uint32_t r = by_wg.divmod(p, wg);
    const int b = (int)by_ho.divmod(r, oh);
    const int c0 = cg * 8, ow0 = wg * PX, iw0 = ow0 * SX - px;
    const int64_t Q = (C + 15) / 16;
    const _Float16 *img = x + (int64_t)b * H * W * C + c0;

    float acc[PX][8];
#pragma unroll
    for (int q = 0; q < PX; q++)
#pragma unroll
        for (int e = 0; e < 8; e++) acc[q][e] = 0.f;

    const int rows = KY ? KY : ky, step = KY ? 1 : dy;
#pragma unroll 1
    for (int i = 0; i < rows; i++) {                               // one row at a time: its NC loads in flight, few registers
        const int ih = oh * sy - py + i * step;
        const bool row_in = (unsigned)ih < (unsigned)H;
        const int ihc = ih < 0 ? 0 : (ih >= H ? H - 1 : ih);
        const _Float16 *row = img + (int64_t)ihc * W * C;
        // a column is needed when some window reads it: c = q SX + j DX (with stride and dilation both 2, every other one)
        constexpr auto used = [](int c) {
            for (int q = 0; q < PX; q++)
                for (int j = 0; j < KS; j++)
                    if (q * SX + j * DX == c) return true;
            return false;
        };
        half8 v[NC];
#pragma unroll
        for (int c = 0; c < NC; c++) {
            if (!used(c)) continue;
            const int iw = iw0 + c, iwc = iw < 0 ? 0 : (iw >= W ? W - 1 : iw);
            v[c] = *reinterpret_cast<const half8 *>(row + (int64_t)iwc * C);
        }
#pragma unroll
        for (int c = 0; c < NC; c++) {
            if (!used(c)) continue;
            const int iw = iw0 + c;
            if (!(row_in && (unsigned)iw < (unsigned)W)) v[c] = half8{0, 0, 0, 0, 0, 0, 0, 0};
        }
#pragma unroll
        for (int j = 0; j < KS; j++) {
            // The 8 codes as fp16 operands, two per register: 01 / 10 / 11 become 01 / 11 / 10 (an fp16's 2.0 bit and
            // sign: +2, -2, -0), channels 4 .. 7 move 8 bits down, and (t << 2 e) & 0xC000C000 is channel e's weight in
            // the high half and channel e + 4's in the low half -- 15 operations per tap instead of 32, and every
            // product one v_fma_mix_f32 on two fp16 sources. The sums run at exactly twice their value.
            uint32_t codes = codes8(words, Q, i * KS + j, c0);
            codes ^= (codes >> 1) & 0x55555555u;
            const uint32_t t = (codes & 0xFF000000u) | ((codes >> 8) & 0x0000FF00u);
            half2v w[4];
#pragma unroll
            for (int e = 0; e < 4; e++) w[e] = __builtin_bit_cast(half2v, (t << (2 * e)) & 0xC000C000u);
#pragma unroll
            for (int q = 0; q < PX; q++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    acc[q][e] = __builtin_fmaf((float)v[q * SX + j * DX][e], (float)w[e][1], acc[q][e]);
                    acc[q][4 + e] = __builtin_fmaf((float)v[q * SX + j * DX][4 + e], (float)w[e][0], acc[q][4 + e]);
                }
        }
    }
    // epilogue: the 8 channels' scale and bias once for all PX positions, 16-byte accesses throughout
    const ChannelConstants cc = load_channel_constants(ep, c0);
#pragma unroll
    for (int q = 0; q < PX; q++) {
        if (ow0 + q >= Wo) break;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[q][e] *= 0.5f;             // exact: the weights were +-2
        store8_vec(ep, cc, ((int64_t)(r * (uint32_t)Wo) + ow0 + q) * C + c0, acc[q]);
    }
}

// Unfolded patches [P][T][C], fp32 (the reference's calling convention) or fp16.
template <typename T>
__global__ __launch_bounds__(256) void dwconv_patches_kernel(const T *__restrict__ x, const uint32_t *__restrict__ words,
                                                             int64_t P, int taps, int64_t C, int vec, DwEpilogue ep) {
    const int64_t G = (C + 7) / 8, Q = (C + 15) / 16;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= P * G) return;
    int cg;
    const int64_t p = div_rem(id, (int)G, cg), c0 = (int64_t)cg * 8;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int t = 0; t < taps; t++) {
        const T *src = x + (p * taps + t) * C + c0;
        const uint32_t codes = codes8(words, Q, t, c0);
        float v[8];
        if (vec) {
            if constexpr (sizeof(T) == 4) {
                const floatx4 a = *reinterpret_cast<const floatx4 *>(src), b = *reinterpret_cast<const floatx4 *>(src + 4);
#pragma unroll
                for (int e = 0; e < 4; e++) { v[e] = a[e]; v[4 + e] = b[e]; }
            } else {
                const half8 h = *reinterpret_cast<const half8 *>(src);
#pragma unroll
                for (int e = 0; e < 8; e++) v[e] = (float)h[e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] = c0 + e < C ? (float)src[e] : 0.f;
        }
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] += apply_code(v[e], codes << (2 * e));
    }
    store8(ep, p * C + c0, c0, C, acc, vec);
}

// Transposed depthwise convolution on an NHWC fp16 image: a thread owns 8 channels of one OUTPUT
// position and visits the taps whose source coordinate (oh + py - i dy) / sy is integral and inside.
__global__ __launch_bounds__(256) void dwconvtrans_image_kernel(const _Float16 *__restrict__ x,
                                                                const uint32_t *__restrict__ words, int B, int C, int H,
                                                                int W, int Ho, int Wo, int ky, int kx, int sy, int sx,
                                                                int py, int px, int dy, int dx, int vec, DwEpilogue ep) {
    const int64_t G = (C + 7) / 8, Q = (C + 15) / 16;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x, total = (int64_t)B * Ho * Wo * G;
    if (id >= total) return;
    int cg, ow, oh;
    const int64_t p = div_rem(id, (int)G, cg), c0 = (int64_t)cg * 8;
    const int64_t r = div_rem(p, Wo, ow);
    const int b = (int)div_rem(r, Ho, oh);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    auto tap = [&](int i, int j, int ih, int iw) {
        const _Float16 *src = x + (((int64_t)b * H + ih) * W + iw) * C + c0;
        const uint32_t codes = codes8(words, Q, i * kx + j, c0);
        if (vec) {
            // the codes as fp16 +-2.0 operands, two per register (see dwconv_square_image_kernel): the sums run at twice
            // their value and are halved below
            const half8 v = *reinterpret_cast<const half8 *>(src);
            const uint32_t fixed = codes ^ ((codes >> 1) & 0x55555555u);
            const uint32_t t = (fixed & 0xFF000000u) | ((fixed >> 8) & 0x0000FF00u);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const half2v w = __builtin_bit_cast(half2v, (t << (2 * e)) & 0xC000C000u);
                acc[e] = __builtin_fmaf((float)v[e], (float)w[1], acc[e]);
                acc[4 + e] = __builtin_fmaf((float)v[4 + e], (float)w[0], acc[4 + e]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (c0 + e < C) acc[e] += apply_code((float)src[e], codes << (2 * e));
        }
    };
    if (dy == 1 && dx == 1) {
        // undilated: the taps that reach this position are i = (oh + py) % sy, + sy, ... (source row (oh + py - i) / sy,
        // one lower per step), and the same along x -- no divisibility test per tap, ceil(ky / sy) ceil(kx / sx) visits
        const int ty = oh + py, tx = ow + px, j0 = tx % sx;
        for (int i = ty % sy, ih = ty / sy; i < ky && ih >= 0; i += sy, ih--) {
            if (ih >= H) continue;
            for (int j = j0, iw = tx / sx; j < kx && iw >= 0; j += sx, iw--)
                if (iw < W) tap(i, j, ih, iw);
        }
    } else {
        for (int i = 0; i < ky; i++) {
            const int ny = oh + py - i * dy;
            if (ny < 0 || ny % sy) continue;
            const int ih = ny / sy;
            if (ih >= H) continue;
            for (int j = 0; j < kx; j++) {
                const int nx = ow + px - j * dx;
                if (nx < 0 || nx % sx) continue;
                const int iw = nx / sx;
                if (iw < W) tap(i, j, ih, iw);
            }
        }
    }
    if (vec) {
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] *= 0.5f;                 // exact: the weights were +-2
    }
    if (vec & 2) store8_vec(ep, load_channel_constants(ep, c0), p * C + c0, acc);
    else store8(ep, p * C + c0, c0, C, acc, vec);
}

// Column form. A workgroup transposes a 64-patch x 64-channel tile of one batch entry through LDS:
// reads run along channels, writes along patches (256 contiguous bytes per (channel, tap) row).
// The product is formed as x * {+1, -1, 0} in fp32 like the reference's (a zero weight keeps the sign
// of x in the zero it writes).
__global__ __launch_bounds__(256) void dwconvtrans_cols_kernel(const float *__restrict__ x, const uint32_t *__restrict__ words,
                                                               int64_t P, int taps, int64_t C, float *__restrict__ y) {
    __shared__ float tile[64][65];
    const int64_t p0 = (int64_t)blockIdx.x * 64, c0 = (int64_t)blockIdx.y * 64, b = blockIdx.z;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const float *xb = x + b * P * C;
    for (int r = wv; r < 64; r += 4) {
        const int64_t p = p0 + r, c = c0 + lane;
        tile[r][lane] = (p < P && c < C) ? xb[p * C + c] : 0.f;
    }
    __syncthreads();
    const int64_t Q = (C + 15) / 16;
    float *yb = y + b * C * taps * P;
    const int64_t p = p0 + lane;
    const int nc = (int)((C - c0) < 64 ? (C - c0) : 64);
    for (int pair = wv; pair < nc * taps; pair += 4) {       // (channel, tap) rows, dealt to the 4 wavefronts
        const int cc = pair / taps, t = pair - cc * taps;
        const int64_t c = c0 + cc;
        const uint32_t code = (words[(int64_t)t * Q + (c >> 4)] >> (30 - 2 * (int)(c & 15))) & 3u;
        const float coef = code == 1u ? 1.0f : (code == 2u ? -1.0f : 0.0f);
        if (p < P) yb[(c * taps + t) * P + p] = tile[lane][cc] * coef;
    }
}

bool aligned_for(const void *p, size_t bytes) { return (reinterpret_cast<uintptr_t>(p) % bytes) == 0; }

}  // namespace
}  // namespace tmq

using namespace tmq;

extern "C" {

int tmq_ternary_dwconv2d(const void *x, const tmq_conv_shape *s, const uint32_t *words, const tmq_epilogue *epilogue,
                         void *y, void *stream) {
    if (!s || !x || !words || !y) return TMQ_ERR_INVALID_ARG;
    if (s->N != s->C) return TMQ_ERR_INVALID_ARG;                 // depthwise: one filter per channel
    tmq_epilogue e = {nullptr, nullptr, nullptr, 0, TMQ_F32};
    if (epilogue) e = *epilogue;
    if (e.y_dtype != TMQ_F16 && e.y_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
    int32_t ho, wo;
    int rc = tmq_conv2d_out_hw(s, &ho, &wo);
    if (rc != TMQ_OK) return rc;
    if (s->B < 0 || s->C <= 0 || s->H <= 0 || s->W <= 0 || ho <= 0 || wo <= 0) return TMQ_ERR_INVALID_ARG;
    const int64_t total = (int64_t)s->B * ho * wo * ((s->C + 7) / 8), blocks = (total + 255) / 256;
    if (total == 0) return TMQ_OK;
    if (blocks > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    const int y_f16 = e.y_dtype == TMQ_F16;
    const size_t ya = y_f16 ? 16 : 16;
    int vec = (s->C % 8 == 0) && aligned_for(x, 16) && aligned_for(y, ya) && (!e.residual || aligned_for(e.residual, ya));
    if (vec && aligned_for(e.scale, 16) && aligned_for(e.bias, 16)) vec |= 2;       // the 16-byte epilogue as well
    DwEpilogue ep{e.scale, e.bias, e.residual, y, e.relu, y_f16};
    const bool columns = (s->kx >= 1 && s->kx <= 5) || s->kx == 7;
    if ((vec & 2) && columns && (s->dx == 1 || s->dx == 2) && (s->sx == 1 || s->sx == 2) && total < (int64_t)0x7FFFFFFF &&
        (int64_t)s->B * ho * wo < (int64_t)0x7FFFFFFF) {
        // output positions per thread, measured on square windows: 4 except at stride 2 with fewer than 7 columns (the
        // windows then share few columns, and 4 positions would hold 9 or 11 columns of a row in registers); dilated
        // windows: 4 while that keeps at most 11 columns of a row in registers
        const int px_per_thread = s->dx == 1 ? ((s->sx == 1 || s->kx == 7) ? 4 : 2) : (s->kx <= (s->sx == 1 ? 4 : 3) ? 4 : 2);
        const int64_t wgroups = (wo + px_per_thread - 1) / px_per_thread, G = s->C / 8;
        const int64_t threads = (int64_t)s->B * ho * wgroups * G, nblocks = (threads + 255) / 256;
        const FastDiv by_g((uint32_t)G), by_wg((uint32_t)wgroups), by_ho((uint32_t)ho);
        auto go = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, dim3((uint32_t)nblocks), dim3(256), 0, as_stream(stream),
                               static_cast<const _Float16 *>(x), words, (uint32_t)threads, s->C, s->H, s->W, wo, by_g, by_wg,
                               by_ho, s->ky, s->sy, s->py, s->px, s->dy, ep);
            return check_launch();
        };
        auto by_positions = [&](auto ks, auto sx, auto dx) {
            constexpr int KS = decltype(ks)::value, SX = decltype(sx)::value, DX = decltype(dx)::value;
            if constexpr (DX == 1 && (KS == 3 || KS == 5 || KS == 7)) {
                if (s->ky == KS && s->dy == 1)
                    return px_per_thread == 4 ? go(dwconv_square_image_kernel<KS, 4, SX, 1, KS>) : go(dwconv_square_image_kernel<KS, 2, SX, 1, KS>);
            }
            return px_per_thread == 4 ? go(dwconv_square_image_kernel<KS, 4, SX, DX>) : go(dwconv_square_image_kernel<KS, 2, SX, DX>);
        };
        auto by_step = [&](auto ks) {
            using one = std::integral_constant<int, 1>;
            using two = std::integral_constant<int, 2>;
            if (s->sx == 1) return s->dx == 1 ? by_positions(ks, one{}, one{}) : by_positions(ks, one{}, two{});
            return s->dx == 1 ? by_positions(ks, two{}, one{}) : by_positions(ks, two{}, two{});
        };
        switch (s->kx) {
            case 1: return by_step(std::integral_constant<int, 1>{});
            case 2: return by_step(std::integral_constant<int, 2>{});
            case 3: return by_step(std::integral_constant<int, 3>{});
            case 4: return by_step(std::integral_constant<int, 4>{});
            case 5: return by_step(std::integral_constant<int, 5>{});
            default: return by_step(std::integral_constant<int, 7>{});
        }
    }
    if (!vec && s->C % 4 == 0 && aligned_for(x, 8)) {              // pixels on 8 bytes: whole channel groups as two 8-byte loads
        vec = 4;
        if (aligned_for(y, 16) && (!e.residual || y_f16)) vec |= 8;   // ... and stores (fp32 pixels then start on 16 bytes)
    }
    hipLaunchKernelGGL(dwconv_image_kernel, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream),
                       static_cast<const _Float16 *>(x), words, s->B, s->C, s->H, s->W, ho, wo, s->ky, s->kx, s->sy, s->sx,
                       s->py, s->px, s->dy, s->dx, vec, ep);
    return check_launch();
}

int tmq_ternary_dwconv_patches(const void *x, int x_dtype, int64_t P, int32_t taps, int64_t C, const uint32_t *words,
                               float *y, void *stream) {
    if (P < 0 || taps <= 0 || C <= 0) return TMQ_ERR_INVALID_ARG;
    if (P == 0) return TMQ_OK;
    if (!x || !words || !y) return TMQ_ERR_INVALID_ARG;
    if (x_dtype != TMQ_F32 && x_dtype != TMQ_F16) return TMQ_ERR_UNSUPPORTED;
    const int64_t total = P * ((C + 7) / 8), blocks = (total + 255) / 256;
    if (blocks > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    const int vec = (C % 8 == 0) && aligned_for(x, 16) && aligned_for(y, 16);
    DwEpilogue ep{nullptr, nullptr, nullptr, y, 0, 0};
    if (x_dtype == TMQ_F32)
        hipLaunchKernelGGL(dwconv_patches_kernel<float>, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const float *>(x), words, P, (int)taps, C, vec, ep);
    else
        hipLaunchKernelGGL(dwconv_patches_kernel<_Float16>, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const _Float16 *>(x), words, P, (int)taps, C, vec, ep);
    return check_launch();
}

int tmq_convtranspose2d_out_hw(const tmq_conv_shape *s, int32_t out_pad_y, int32_t out_pad_x, int32_t *ho, int32_t *wo) {
    if (!s || !ho || !wo) return TMQ_ERR_INVALID_ARG;
    if (s->ky <= 0 || s->kx <= 0 || s->sy <= 0 || s->sx <= 0 || s->dy <= 0 || s->dx <= 0 || s->py < 0 || s->px < 0 ||
        out_pad_y < 0 || out_pad_x < 0 || s->H <= 0 || s->W <= 0)
        return TMQ_ERR_INVALID_ARG;
    const int64_t h = ((int64_t)s->H - 1) * s->sy - 2 * (int64_t)s->py + (int64_t)s->dy * (s->ky - 1) + 1 + out_pad_y;
    const int64_t w = ((int64_t)s->W - 1) * s->sx - 2 * (int64_t)s->px + (int64_t)s->dx * (s->kx - 1) + 1 + out_pad_x;
    if (h <= 0 || w <= 0 || h > 0x7FFFFFFF || w > 0x7FFFFFFF) return TMQ_ERR_INVALID_ARG;
    *ho = (int32_t)h;
    *wo = (int32_t)w;
    return TMQ_OK;
}

int tmq_ternary_dwconvtrans2d(const void *x, const tmq_conv_shape *s, int32_t out_pad_y, int32_t out_pad_x,
                              const uint32_t *words, const tmq_epilogue *epilogue, void *y, void *stream) {
    if (!s || !x || !words || !y) return TMQ_ERR_INVALID_ARG;
    if (s->N != s->C || s->C <= 0 || s->B < 0) return TMQ_ERR_INVALID_ARG;
    tmq_epilogue e = {nullptr, nullptr, nullptr, 0, TMQ_F32};
    if (epilogue) e = *epilogue;
    if (e.y_dtype != TMQ_F16 && e.y_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
    int32_t ho, wo;
    int rc = tmq_convtranspose2d_out_hw(s, out_pad_y, out_pad_x, &ho, &wo);
    if (rc != TMQ_OK) return rc;
    const int64_t total = (int64_t)s->B * ho * wo * ((s->C + 7) / 8), blocks = (total + 255) / 256;
    if (total == 0) return TMQ_OK;
    if (blocks > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    const int y_f16 = e.y_dtype == TMQ_F16;
    int vec = (s->C % 8 == 0) && aligned_for(x, 16) && aligned_for(y, 16) && (!e.residual || aligned_for(e.residual, 16));
    if (vec && aligned_for(e.scale, 16) && aligned_for(e.bias, 16)) vec |= 2;       // the 16-byte epilogue as well
    DwEpilogue ep{e.scale, e.bias, e.residual, y, e.relu, y_f16};
    hipLaunchKernelGGL(dwconvtrans_image_kernel, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream),
                       static_cast<const _Float16 *>(x), words, s->B, s->C, s->H, s->W, ho, wo, s->ky, s->kx, s->sy, s->sx,
                       s->py, s->px, s->dy, s->dx, vec, ep);
    return check_launch();
}

int tmq_ternary_dwconvtrans_cols(const float *x, int64_t B, int64_t P, int32_t taps, int64_t C, const uint32_t *words,
                                 float *y, void *stream) {
    if (B < 0 || P < 0 || taps <= 0 || C <= 0) return TMQ_ERR_INVALID_ARG;
    if (B == 0 || P == 0) return TMQ_OK;
    if (!x || !words || !y) return TMQ_ERR_INVALID_ARG;
    const int64_t gx = (P + 63) / 64, gy = (C + 63) / 64;
    if (gx > 0x7FFFFFFF || gy > 65535 || B > 65535) return TMQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL(dwconvtrans_cols_kernel, dim3((uint32_t)gx, (uint32_t)gy, (uint32_t)B), dim3(256), 0, as_stream(stream),
                       x, words, P, (int)taps, C, y);
    return check_launch();
}

}  // extern "C"
