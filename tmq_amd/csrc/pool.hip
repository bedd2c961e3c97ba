// Memory-bound companions of the ternary convolutions for fp16 NHWC feature maps, gfx950: max-pool,
// global average pool, and the NCHW -> NHWC repack of a few-channel network input. Each is one pass
// with 16-byte accesses (8 fp16 channels per thread); arithmetic is negligible, the bound is HBM.
// The reference has no kernels for these: its ResNet sample (samples/resnet_test.py:91-118) runs
// torchvision's NCHW fp32 model and so uses PyTorch's pooling.
#include "common.h"
#include "mfma.h"

namespace tmq {
namespace {

// y[b][oh][ow][c] = max over the window of x[b][oh sy - py + i][ow sx - px + j][c]; taps outside the
// image do not take part (PyTorch's implicit -inf padding). Thread = 8 channels of one output pixel.
// NaN inputs: the packed fp16 maximum returns the other operand (IEEE maxNum), where PyTorch would
// propagate the NaN.
__global__ __launch_bounds__(256) void maxpool_nhwc_kernel(const _Float16 *__restrict__ x, int B, int C, int H, int W, int Ho,
                                                           int Wo, int ky, int kx, int sy, int sx, int py, int px, int vec,
                                                           _Float16 *__restrict__ y) {
    const int64_t G = (C + 7) / 8;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x, total = (int64_t)B * Ho * Wo * G;
    if (id >= total) return;
    int cg, ow, oh;
    const int64_t p = div_rem(id, (int)G, cg), c0 = (int64_t)cg * 8;
    const int64_t r = div_rem(p, Wo, ow);
    const int b = (int)div_rem(r, Ho, oh);
    const _Float16 ninf = (_Float16)(-__builtin_inff());
    half8 best = {ninf, ninf, ninf, ninf, ninf, ninf, ninf, ninf};
    for (int i = 0; i < ky; i++) {
        const int ih = oh * sy - py + i;
        if (ih < 0 || ih >= H) continue;
        for (int j = 0; j < kx; j++) {
            const int iw = ow * sx - px + j;
            if (iw < 0 || iw >= W) continue;
            const _Float16 *src = x + (((int64_t)b * H + ih) * W + iw) * C + c0;
            half8 v = best;
            if (vec) {
                v = *reinterpret_cast<const half8 *>(src);
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++)
                    if (c0 + e < C) v[e] = src[e];
            }
            best = __builtin_elementwise_max(best, v);
        }
    }
    _Float16 *dst = y + p * C + c0;
    if (vec) {
        *reinterpret_cast<half8 *>(dst) = best;
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++)
            if (c0 + e < C) dst[e] = best[e];
    }
}

// The common case -- a 3 x 3 window, whole groups of 8 channels, fewer than 2^31 threads: the index
// arithmetic by multiply-high (FastDiv) and all nine loads in flight at once. Taps outside the image read
// the clamped pixel and are replaced by -inf afterwards, so no load depends on a branch.
__global__ __launch_bounds__(256) void maxpool3x3_nhwc_kernel(const _Float16 *__restrict__ x, uint32_t total, int C, int H, int W,
                                                              FastDiv by_g, FastDiv by_wo, FastDiv by_ho, int sy, int sx,
                                                              int py, int px, _Float16 *__restrict__ y) {
    const uint32_t id = blockIdx.x * 256u + threadIdx.x;
    if (id >= total) return;
    int cg, ow, oh;
    const uint32_t p = by_g.divmod(id, cg);
    const uint32_t r = by_wo.divmod(p, ow);
    const int b = (int)by_ho.divmod(r, oh);
    const _Float16 ninf = (_Float16)(-__builtin_inff());
    const half8 none = {ninf, ninf, ninf, ninf, ninf, ninf, ninf, ninf};
    const _Float16 *img = x + (int64_t)b * H * W * C + cg * 8;
    half8 v[9];
    bool in[9];
#pragma unroll
    for (int i = 0; i < 3; i++) {
        const int ih = oh * sy - py + i, ihc = ih < 0 ? 0 : (ih >= H ? H - 1 : ih);
#pragma unroll
        for (int j = 0; j < 3; j++) {
            const int iw = ow * sx - px + j, iwc = iw < 0 ? 0 : (iw >= W ? W - 1 : iw);
            in[i * 3 + j] = (ih == ihc) & (iw == iwc);
            v[i * 3 + j] = *reinterpret_cast<const half8 *>(img + ((int64_t)ihc * W + iwc) * C);
        }
    }
    half8 best = none;
#pragma unroll
    for (int t = 0; t < 9; t++) best = __builtin_elementwise_max(best, in[t] ? v[t] : none);
    *reinterpret_cast<half8 *>(y + (int64_t)p * C + cg * 8) = best;
}

// y[b][c] = mean over the HW positions of x[b][.][c], fp32 accumulation. A workgroup = one image x 64
// groups of 8 channels; its four wavefronts take every fourth position each (loads of a wavefront are
// one contiguous KiB, several in flight), then the four partial sums are added in wavefront order.
__global__ __launch_bounds__(256) void avgpool_global_nhwc_kernel(const _Float16 *__restrict__ x, int64_t B, int64_t HW, int64_t C,
                                                                  int vec, void *__restrict__ y, int y_f16) {
    __shared__ float part[4][64][9];
    const int64_t G = (C + 7) / 8, GB = (G + 63) / 64;
    const int64_t b = (uint32_t)blockIdx.x / (uint32_t)GB, cg = (int64_t)((uint32_t)blockIdx.x % (uint32_t)GB) * 64 + (threadIdx.x & 63);
    const int lane = threadIdx.x & 63, slice = threadIdx.x >> 6;
    const int64_t c0 = cg * 8;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (cg < G) {
        const _Float16 *src = x + b * HW * C + c0;
        if (vec) {
            int64_t p = slice;
            for (; p + 12 < HW; p += 16) {             // four loads in flight
                half8 v[4];
#pragma unroll
                for (int u = 0; u < 4; u++) v[u] = *reinterpret_cast<const half8 *>(src + (p + 4 * u) * C);
#pragma unroll
                for (int u = 0; u < 4; u++)
#pragma unroll
                    for (int e = 0; e < 8; e++) acc[e] += (float)v[u][e];
            }
            for (; p < HW; p += 4) {
                const half8 v = *reinterpret_cast<const half8 *>(src + p * C);
#pragma unroll
                for (int e = 0; e < 8; e++) acc[e] += (float)v[e];
            }
        } else {
            for (int64_t p = slice; p < HW; p += 4)
#pragma unroll
                for (int e = 0; e < 8; e++)
                    if (c0 + e < C) acc[e] += (float)src[p * C + e];
        }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) part[slice][lane][e] = acc[e];
    __syncthreads();
    if (slice != 0 || cg >= G) return;
    const float inv = 1.0f / (float)HW;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        if (c0 + e >= C) break;
        const float m = (((part[0][lane][e] + part[1][lane][e]) + part[2][lane][e]) + part[3][lane][e]) * inv;
        if (y_f16) static_cast<_Float16 *>(y)[b * C + c0 + e] = (_Float16)m;
        else static_cast<float *>(y)[b * C + c0 + e] = m;
    }
}

// A network's head in one launch: the global average pool of an image (avgpool_global_nhwc_kernel's arithmetic, the
// means rounded to fp16 as that kernel stores them) followed by the classifier's ternary product on those means.
// One workgroup per image (C <= 512: 64 groups of 8 channels); the means stay in LDS, the four wavefronts share the
// classifier's 16-channel blocks, and the row of means is row 0 of the MFMA's activation operand (the other 15 rows
// are zero: at one row per image the instruction's idle rows cost nothing that matters next to a saved launch).
__global__ __launch_bounds__(256) void avgpool_linear_kernel(const _Float16 *__restrict__ x, int64_t HW, int64_t C,
                                                             const u32x4 *__restrict__ native, int64_t N, int Nb, int Kb,
                                                             const float *__restrict__ scale, const float *__restrict__ bias,
                                                             int relu, void *__restrict__ y, int y_f16) {
    __shared__ float part[4][64][9];
    __shared__ __attribute__((aligned(16))) _Float16 means[512];
    const int64_t b = blockIdx.x, G = C / 8;
    const int lane = threadIdx.x & 63, slice = threadIdx.x >> 6;
    const int64_t c0 = (int64_t)lane * 8;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (lane < G) {
        const _Float16 *src = x + b * HW * C + c0;
        int64_t p = slice;
        for (; p + 12 < HW; p += 16) {             // four loads in flight
            half8 v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = *reinterpret_cast<const half8 *>(src + (p + 4 * u) * C);
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int e = 0; e < 8; e++) acc[e] += (float)v[u][e];
        }
        for (; p < HW; p += 4) {
            const half8 v = *reinterpret_cast<const half8 *>(src + p * C);
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] += (float)v[e];
        }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) part[slice][lane][e] = acc[e];
    __syncthreads();
    if (slice == 0) {
        const float inv = 1.0f / (float)HW;
        half8 m;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            // the mean is rounded to fp32 and then to fp16, as the pooling kernel stores it; without the empty asm the
            // compiler folds product and conversion into v_fma_mixlo_f16, which rounds once and differs on fp16 ties
            float mean = (((part[0][lane][e] + part[1][lane][e]) + part[2][lane][e]) + part[3][lane][e]) * inv;
            asm volatile("" : "+v"(mean));
            m[e] = lane < G ? (_Float16)mean : (_Float16)0;
        }
        *reinterpret_cast<half8 *>(&means[lane * 8]) = m;      // channels past C: zero (the weights there are zero too)
    }
    __syncthreads();
    const int j = lane & 15, g = lane >> 4;
    for (int nb = slice; nb < Nb; nb += 4) {
        floatx4 d = {0.f, 0.f, 0.f, 0.f};
        for (int kb = 0; kb < Kb; kb++) {
            const u32x4 w = native[((int64_t)nb * Kb + kb) * 64 + lane];
#pragma unroll
            for (int ks = 0; ks < 8; ks++) {
                half8 a = {0, 0, 0, 0, 0, 0, 0, 0};
                if (j == 0) a = *reinterpret_cast<const half8 *>(&means[kb * 256 + ks * 32 + g * 8]);
                d = mfma16(a, decode_step(w[ks >> 1], ks & 1), d);
            }
        }
        // row 0 of the result: element 0 of the lanes with g == 0, column j
        const int64_t n = (int64_t)nb * 16 + j;
        if (g == 0 && n < N) {
            float v = d[0] * ((scale ? scale[n] : 1.0f) * (1.0f / kWeightUnit)) + (bias ? bias[n] : 0.0f);
            if (relu && v < 0.f) v = 0.f;
            if (y_f16) static_cast<_Float16 *>(y)[b * N + n] = (_Float16)v;
            else static_cast<float *>(y)[b * N + n] = v;
        }
    }
}

// NCHW (fp16 or fp32, C <= 4) -> NHWC fp16 with 4 channels, the missing ones zero.
// Thread = 4 neighbouring pixels of one row (W % 4 == 0): reads along W, writes 32 contiguous bytes.
template <typename T>
__global__ __launch_bounds__(256) void nchw_to_nhwc4_kernel(const T *__restrict__ x, int64_t B, int C, int64_t H, int64_t W,
                                                            _Float16 *__restrict__ y) {
    const int64_t W4 = W / 4;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= B * H * W4) return;
    int wq, hh;
    const int64_t bh = div_rem(id, (int)W4, wq), w0 = (int64_t)wq * 4;
    const int64_t b = div_rem(bh, (int)H, hh), h = hh;
    _Float16 px[4][4];
#pragma unroll
    for (int c = 0; c < 4; c++) {
        if (c < C) {
            const T *src = x + ((b * C + c) * H + h) * W + w0;
#pragma unroll
            for (int q = 0; q < 4; q++) px[q][c] = (_Float16)src[q];
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) px[q][c] = (_Float16)0;
        }
    }
    half8 lo = {px[0][0], px[0][1], px[0][2], px[0][3], px[1][0], px[1][1], px[1][2], px[1][3]};
    half8 hi = {px[2][0], px[2][1], px[2][2], px[2][3], px[3][0], px[3][1], px[3][2], px[3][3]};
    half8 *dst = reinterpret_cast<half8 *>(y + ((b * H + h) * W + w0) * 4);
    dst[0] = lo;
    dst[1] = hi;
}

}  // namespace
}  // namespace tmq

using namespace tmq;

extern "C" {

int tmq_maxpool2d_nhwc(const void *x, int32_t B, int32_t C, int32_t H, int32_t W, int32_t ky, int32_t kx, int32_t sy,
                       int32_t sx, int32_t py, int32_t px, void *y, void *stream) {
    if (B < 0 || C <= 0 || H <= 0 || W <= 0 || ky <= 0 || kx <= 0 || sy <= 0 || sx <= 0 || py < 0 || px < 0)
        return TMQ_ERR_INVALID_ARG;
    if (2 * py > ky || 2 * px > kx) return TMQ_ERR_INVALID_ARG;          // PyTorch's rule: pad at most half the window
    const int64_t ho = ((int64_t)H + 2 * py - ky) / sy + 1, wo = ((int64_t)W + 2 * px - kx) / sx + 1;
    if ((int64_t)H + 2 * py < ky || (int64_t)W + 2 * px < kx) return TMQ_ERR_INVALID_ARG;
    if (B == 0) return TMQ_OK;
    if (!x || !y) return TMQ_ERR_INVALID_ARG;
    const int64_t total = (int64_t)B * ho * wo * ((C + 7) / 8), blocks = (total + 255) / 256;
    if (blocks > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    const int vec = (C % 8 == 0) && aligned16(x) && aligned16(y);
    if (vec && ky == 3 && kx == 3 && total < (int64_t)0x7FFFFFFF) {
        hipLaunchKernelGGL(maxpool3x3_nhwc_kernel, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const _Float16 *>(x), (uint32_t)total, C, H, W, FastDiv((uint32_t)(C / 8)),
                           FastDiv((uint32_t)wo), FastDiv((uint32_t)ho), sy, sx, py, px, static_cast<_Float16 *>(y));
        return check_launch();
    }
    hipLaunchKernelGGL(maxpool_nhwc_kernel, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream),
                       static_cast<const _Float16 *>(x), B, C, H, W, (int)ho, (int)wo, ky, kx, sy, sx, py, px, vec,
                       static_cast<_Float16 *>(y));
    return check_launch();
}

int tmq_avgpool_global_nhwc(const void *x, int64_t B, int64_t HW, int64_t C, void *y, int y_dtype, void *stream) {
    if (B < 0 || HW <= 0 || C <= 0) return TMQ_ERR_INVALID_ARG;
    if (y_dtype != TMQ_F16 && y_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
    if (B == 0) return TMQ_OK;
    if (!x || !y) return TMQ_ERR_INVALID_ARG;
    const int64_t blocks = B * (((C + 7) / 8 + 63) / 64);
    if (blocks > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    const int vec = (C % 8 == 0) && aligned16(x);
    hipLaunchKernelGGL(avgpool_global_nhwc_kernel, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream),
                       static_cast<const _Float16 *>(x), B, HW, C, vec, y, y_dtype == TMQ_F16 ? 1 : 0);
    return check_launch();
}

int tmq_avgpool_linear(const void *x, int64_t B, int64_t HW, int64_t C, const void *native, int64_t N,
                       const tmq_epilogue *epilogue, void *y, void *stream) {
    if (B < 0 || HW <= 0 || C <= 0 || N <= 0) return TMQ_ERR_INVALID_ARG;
    tmq_epilogue e = {nullptr, nullptr, nullptr, 0, TMQ_F32};
    if (epilogue) e = *epilogue;
    if (e.y_dtype != TMQ_F16 && e.y_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
    // one workgroup per image holds all channel means: at most 512 channels in whole groups of 8, no residual
    if (C > 512 || C % 8 != 0 || e.residual || !aligned16(x) || B > 0x7FFFFFFF || native_blocks_n(N) > 0x7FFFFFFF) return TMQ_ERR_UNSUPPORTED;
    if (B == 0) return TMQ_OK;
    if (!x || !native || !y || !aligned16(native)) return TMQ_ERR_INVALID_ARG;
    hipLaunchKernelGGL(avgpool_linear_kernel, dim3((uint32_t)B), dim3(256), 0, as_stream(stream),
                       static_cast<const _Float16 *>(x), HW, C, static_cast<const u32x4 *>(native), N, (int)native_blocks_n(N),
                       (int)native_blocks_k(C), e.scale, e.bias, e.relu, y, e.y_dtype == TMQ_F16 ? 1 : 0);
    return check_launch();
}

int tmq_nchw_to_nhwc4(const void *x, int x_dtype, int64_t B, int32_t C, int64_t H, int64_t W, void *y, void *stream) {
    if (B < 0 || C <= 0 || C > 4 || H <= 0 || W <= 0 || W % 4 != 0) return TMQ_ERR_INVALID_ARG;
    if (x_dtype != TMQ_F16 && x_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
    if (H > 0x7FFFFFFF || W > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    if (B == 0) return TMQ_OK;
    if (!x || !y || !aligned16(y)) return TMQ_ERR_INVALID_ARG;
    const int64_t total = B * H * (W / 4), blocks = (total + 255) / 256;
    if (blocks > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    if (x_dtype == TMQ_F16)
        hipLaunchKernelGGL(nchw_to_nhwc4_kernel<_Float16>, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const _Float16 *>(x), B, (int)C, H, W, static_cast<_Float16 *>(y));
    else
        hipLaunchKernelGGL(nchw_to_nhwc4_kernel<float>, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream),
                           static_cast<const float *>(x), B, (int)C, H, W, static_cast<_Float16 *>(y));
    return check_launch();
}

}  // extern "C"
