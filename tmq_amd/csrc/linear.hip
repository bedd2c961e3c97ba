// Ternary linear layers on gfx950: y[m][n] = scale[n] * sum_k x[m][k] * T[k][n] + bias[n].
//
//   prepack_kernel : reference packing words[K][ceil(N/16)] -> kernel-native blocks (mfma.h)
//   skinny_kernel  : M <= 64 (GEMV and small batches). Bound by streaming the 2-bit weights:
//                    every wavefront fetches 1 KiB weight blocks with one coalesced dwordx4 load,
//                    expands them in registers to exact +-2/0 fp16 MFMA operands (two VALU ops
//                    per register), and contracts with the activations on
//                    v_mfma_f32_16x16x32_f16 (fp32 accumulate). K is split over the wavefronts
//                    of a workgroup and reduced through LDS in a fixed order (deterministic).
//   The MFMA-bound large-M kernel lives in gemm.hip.
#include "common.h"
#include "mfma.h"

namespace tmq {
namespace {

// ---- prepack ------------------------------------------------------------------------------------
// One thread per native dword. For convolution weights the reduction index is reordered from the
// reference's (c, y, x) to (y, x, c) so that an im2col row is contiguous in NHWC memory.
__global__ __launch_bounds__(256) void prepack_kernel(const uint32_t *__restrict__ words, uint32_t *__restrict__ native,
                                                      int64_t N, int64_t K, int64_t C, int64_t ky, int64_t kx,
                                                      int64_t Kb, int64_t total) {
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= total) return;
    const int d = (int)(id & 3), lane = (int)((id >> 2) & 63);
    const int64_t blk = id >> 8, kb = blk % Kb, nb = blk / Kb;
    const int nl = lane & 15, g = lane >> 4;
    const int64_t Q = (N + 15) / 16, n = nb * 16 + nl;
    uint32_t out = 0;
    if (n < N) {
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int64_t kn = kb * kKB + d * 64 + s * 32 + g * 8 + e;
                if (kn >= K) continue;
                int64_t kr = kn;
                if (ky * kx > 1) {
                    const int64_t c = kn % C, yx = kn / C;
                    kr = (c * ky + yx / kx) * kx + yx % kx;
                }
                const uint32_t code = (words[kr * Q + nb] >> (30 - 2 * nl)) & 3u;
                const uint32_t field = code == 1u ? 1u : (code == 2u ? 3u : 0u);
                const int f = 4 * s + (e >> 1);
                out |= field << ((e & 1 ? 16 : 0) + 14 - 2 * f);
            }
    }
    native[id] = out;
}

// ---- activation operand ---------------------------------------------------------------------------
// Lane (j = lane % 16, g = lane / 16) needs x[m][k0 + 8g .. k0 + 8g + 7] as 8 fp16. fp32
// activations are split into hi = fp16(x) and lo = fp16(x - hi); two MFMAs then carry ~22 bits.
template <bool X32>
struct XFrag {
    half8 hi, lo;
};

template <bool X32, bool VEC>
__device__ __forceinline__ XFrag<X32> load_x(const void *x, int64_t m, int64_t M, int64_t K, int64_t k) {
    XFrag<X32> f;
    f.hi = half8{0, 0, 0, 0, 0, 0, 0, 0};
    f.lo = f.hi;
    if (m >= M || k >= K) return f;
    if constexpr (!X32) {
        const _Float16 *p = static_cast<const _Float16 *>(x) + m * K + k;
        if (VEC && k + 8 <= K) {
            f.hi = *reinterpret_cast<const half8 *>(p);
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (k + e < K) f.hi[e] = p[e];
        }
    } else {
        const float *p = static_cast<const float *>(x) + m * K + k;
        float v[8];
        if (VEC && k + 8 <= K) {
            floatx4 a = *reinterpret_cast<const floatx4 *>(p), b = *reinterpret_cast<const floatx4 *>(p + 4);
#pragma unroll
            for (int e = 0; e < 4; e++) { v[e] = a[e]; v[4 + e] = b[e]; }
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] = (k + e < K) ? p[e] : 0.f;
        }
#pragma unroll
        for (int e = 0; e < 8; e++) {
            _Float16 h = (_Float16)v[e];
            f.hi[e] = h;
            f.lo[e] = (_Float16)(v[e] - (float)h);
        }
    }
    return f;
}

// ---- skinny kernel --------------------------------------------------------------------------------
// grid.x = ceil(N/16); blockDim.x = 64 * waves; wave w owns the weight blocks kb = w, w + waves, ...
// MT = number of 16-row activation tiles (M <= 16 MT). D[n][m]: weights are the A operand.
template <int MT, bool X32, bool VEC>
__global__ __launch_bounds__(1024) void skinny_kernel(const void *__restrict__ x, int64_t M, int64_t K,
                                                      const u32x4 *__restrict__ native, int64_t Kb, int64_t N,
                                                      const float *__restrict__ scale, const float *__restrict__ bias,
                                                      const void *__restrict__ residual, int relu, void *__restrict__ y,
                                                      int y_f16) {
    extern __shared__ float red[];   // [waves][MT][64][4]
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int64_t nb = blockIdx.x;
    floatx4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

    for (int64_t kb = wv; kb < Kb; kb += waves) {
        const u32x4 wq = __builtin_nontemporal_load(native + (nb * Kb + kb) * 64 + lane);
#pragma unroll
        for (int d = 0; d < 4; d++) {
#pragma unroll
            for (int s = 0; s < 2; s++) {
                const int64_t k0 = kb * kKB + d * 64 + s * 32;
                if (k0 >= K) continue;   // wave-uniform
                const half8 a = decode_step(wq[d], s);
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const XFrag<X32> xf = load_x<X32, VEC>(x, t * 16 + j, M, K, k0 + g * 8);
                    acc[t] = mfma16(a, xf.hi, acc[t]);
                    if constexpr (X32) acc[t] = mfma16(a, xf.lo, acc[t]);
                }
            }
        }
    }
    // cross-wave reduction in wave order, then epilogue: lane slot (t, lane) holds
    // y[m = 16 t + j][n = 16 nb + 4 g + r], r = 0..3.
    floatx4 *slot = reinterpret_cast<floatx4 *>(red);
#pragma unroll
    for (int t = 0; t < MT; t++) slot[(wv * MT + t) * 64 + lane] = acc[t];
    __syncthreads();
    for (int id = threadIdx.x; id < MT * 64; id += blockDim.x) {
        const int t = id >> 6, l = id & 63, jj = l & 15, gg = l >> 4;
        floatx4 s = slot[id];
        for (int w = 1; w < waves; w++) {
            const floatx4 p = slot[(w * MT + t) * 64 + l];
            s[0] += p[0]; s[1] += p[1]; s[2] += p[2]; s[3] += p[3];
        }
        const int64_t m = t * 16 + jj, n0 = nb * 16 + gg * 4;
        if (m >= M) continue;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t n = n0 + r;
            if (n < N) {
                const float sc = (scale ? scale[n] : 1.0f) * (1.0f / kWeightUnit);
                float v = s[r] * sc;
                if (bias) v += bias[n];
                const int64_t o = m * N + n;
                if (y_f16) {
                    if (residual) v += (float)static_cast<const _Float16 *>(residual)[o];
                    if (relu) v = v > 0.f ? v : 0.f;
                    static_cast<_Float16 *>(y)[o] = (_Float16)v;
                } else {
                    if (residual) v += static_cast<const float *>(residual)[o];
                    if (relu) v = v > 0.f ? v : 0.f;
                    static_cast<float *>(y)[o] = v;
                }
            }
        }
    }
}

template <int MT, bool X32>
int launch_skinny(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const tmq_epilogue &ep,
                  void *y, void *stream) {
    const float *scale = ep.scale, *bias = ep.bias;
    const void *residual = ep.residual;
    const int relu = ep.relu, y_f16 = ep.y_dtype == TMQ_F16;
    const int64_t Nb = native_blocks_n(N), Kb = native_blocks_k(K);
    int waves = 16;
    while (waves > 1 && (waves > Kb || waves * MT > 32)) waves >>= 1;
    const size_t lds = (size_t)waves * MT * 64 * sizeof(floatx4);
    const bool vec = (K % 8 == 0) && aligned16(x);
    if (Nb > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    dim3 grid((uint32_t)Nb), block(64 * waves);
    const u32x4 *nat = static_cast<const u32x4 *>(native);
    if (vec)
        hipLaunchKernelGGL((skinny_kernel<MT, X32, true>), grid, block, lds, as_stream(stream), x, M, K, nat, Kb, N, scale,
                           bias, residual, relu, y, y_f16);
    else
        hipLaunchKernelGGL((skinny_kernel<MT, X32, false>), grid, block, lds, as_stream(stream), x, M, K, nat, Kb, N,
                           scale, bias, residual, relu, y, y_f16);
    return check_launch();
}

template <bool X32>
int skinny_rows(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const tmq_epilogue &ep, void *y,
                void *stream) {
    switch ((int)((M + 15) / 16)) {
        case 1: return launch_skinny<1, X32>(x, M, K, native, N, ep, y, stream);
        case 2: return launch_skinny<2, X32>(x, M, K, native, N, ep, y, stream);
        case 3: return launch_skinny<3, X32>(x, M, K, native, N, ep, y, stream);
        default: return launch_skinny<4, X32>(x, M, K, native, N, ep, y, stream);
    }
}

}  // namespace

// gemm.hip: the MFMA-bound tile kernel for large M (fp16 activations).
int launch_gemm_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                      const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream);

}  // namespace tmq

using namespace tmq;

extern "C" {

size_t tmq_native_weight_bytes(int64_t N, int64_t K) {
    if (N <= 0 || K <= 0) return 0;
    return (size_t)native_blocks_n(N) * (size_t)native_blocks_k(K) * 1024u;
}

int tmq_prepack_weights(const uint32_t *words, int64_t N, int64_t C, int64_t ky, int64_t kx, void *native,
                        void *stream) {
    if (N <= 0 || C <= 0 || ky <= 0 || kx <= 0) return TMQ_ERR_INVALID_ARG;
    if (!words || !native || !aligned16(native)) return TMQ_ERR_INVALID_ARG;
    const int64_t K = C * ky * kx, Kb = native_blocks_k(K);
    const int64_t total = native_blocks_n(N) * Kb * 256;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL(prepack_kernel, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream), words,
                       static_cast<uint32_t *>(native), N, K, C, ky, kx, Kb, total);
    return check_launch();
}

int tmq_ternary_linear(const void *x, int x_dtype, int64_t M, int64_t K, const void *native, int64_t N,
                       const tmq_epilogue *epilogue, void *y, void *stream) {
    if (M < 0 || K <= 0 || N <= 0) return TMQ_ERR_INVALID_ARG;
    if (M == 0) return TMQ_OK;
    if (!x || !native || !y || !aligned16(native)) return TMQ_ERR_INVALID_ARG;
    if (x_dtype != TMQ_F16 && x_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
    tmq_epilogue ep = {nullptr, nullptr, nullptr, 0, TMQ_F32};
    if (epilogue) ep = *epilogue;
    if (ep.y_dtype != TMQ_F16 && ep.y_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
    const bool x32 = x_dtype == TMQ_F32;
    if (M <= 64) return x32 ? skinny_rows<true>(x, M, K, native, N, ep, y, stream)
                            : skinny_rows<false>(x, M, K, native, N, ep, y, stream);
    if (!x32)
        return launch_gemm_dense(x, M, K, native, N, ep.scale, ep.bias, ep.residual, ep.relu, y,
                                 ep.y_dtype == TMQ_F16, stream);
    // fp32 activations with M > 64: 64-row slabs through the two-term skinny kernel (keeps fp32
    // accuracy; the fp16 tile kernel is the fast path).
    const size_t ysz = ep.y_dtype == TMQ_F16 ? 2 : 4;
    for (int64_t m0 = 0; m0 < M; m0 += 64) {
        const int64_t mm = M - m0 < 64 ? M - m0 : 64;
        tmq_epilogue e2 = ep;
        if (ep.residual) e2.residual = static_cast<const char *>(ep.residual) + (size_t)m0 * N * ysz;
        int rc = skinny_rows<true>(static_cast<const char *>(x) + (size_t)m0 * K * 4, mm, K, native, N, e2,
                                   static_cast<char *>(y) + (size_t)m0 * N * ysz, stream);
        if (rc != TMQ_OK) return rc;
    }
    return TMQ_OK;
}

}  // extern "C"
