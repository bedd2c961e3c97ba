// MFMA-bound ternary GEMM / implicit-GEMM convolution for gfx950.
//
//   Y[m][n] = epilogue( sum_k A[m][k] * T[k][n] ),   A = activations (fp16), T = ternary weights
//
// Work split: a workgroup owns a BM x BN output tile; its WGM x WGN wavefronts each own
// (16 WM) x (16 WN) of it as WM x WN accumulators of v_mfma_f32_16x16x32_f16 (fp32 accumulate).
//   * Activations: staged global -> registers -> LDS one 64-wide k-tile ahead of the math (the
//     next tile's global loads are in flight while the current one is multiplied); LDS rows are
//     padded to 144 bytes so the 16-byte operand reads of a wavefront are conflict-free. The A
//     tile is shared by every wavefront of the workgroup.
//   * Weights: never touch LDS. Each lane loads the dword of the kernel-native layout (mfma.h)
//     that holds exactly its own operand bits and expands it in two VALU ops per register to
//     +-2/0 fp16. The 2-bit weights are a few hundred KiB per workgroup and stay in L2.
//   * The loader is a template: a dense row-major matrix, or an im2col view of an NHWC tensor
//     (implicit GEMM, no materialised patches); the reduction index of a convolution is ordered
//     (ky, kx, c) so that 8 consecutive k are 16 contiguous bytes.
//   * Workgroup ids are remapped so that the workgroups resident on one XCD (ids congruent
//     mod 8) cover neighbouring tiles and share activation rows in that XCD's L2.
#include "common.h"
#include "mfma.h"

namespace tmq {
namespace {

constexpr int kBK = 64;          // k-tile
constexpr int kPitch = 72;       // LDS row pitch in halfs (64 + 8 pad = 144 bytes)

struct Epilogue {
    const float *scale;      // [N] or null
    const float *bias;       // [N] or null
    const void *residual;    // same shape/dtype as y, or null
    void *y;
    int relu;
    int y_f16;
};

// ---- loaders ------------------------------------------------------------------------------------------
// A loader hands every thread CH 16-byte chunks (8 fp16) of the BM x 64 activation tile:
// chunk i of thread t is row (t / 8 + i * T / 8), k offset (t % 8) * 8.
struct DenseLoader {
    const _Float16 *x;
    int64_t M, K;
    int vec;   // rows are 16-byte aligned (K % 8 == 0 and aligned base)

    template <int CH, int T>
    struct State {
        const _Float16 *row[CH];
        int kc;
    };
    template <int CH, int T>
    __device__ __forceinline__ void init(State<CH, T> &st, int64_t m0, int tid) const {
        st.kc = (tid & 7) * 8;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const int64_t m = m0 + (tid >> 3) + i * (T / 8);
            st.row[i] = m < M ? x + m * K : nullptr;
        }
    }
    template <int CH, int T>
    __device__ __forceinline__ void fetch(State<CH, T> &st, int64_t k0, u32x4 (&out)[CH]) const {
        const int64_t k = k0 + st.kc;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (st.row[i] && k < K) {
                if (vec && k + 8 <= K) {
                    v = *reinterpret_cast<const u32x4 *>(st.row[i] + k);
                } else {
                    half8 h = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        if (k + e < K) h[e] = st.row[i][k + e];
                    v = __builtin_bit_cast(u32x4, h);
                }
            }
            out[i] = v;
        }
    }
    template <int CH, int T>
    __device__ __forceinline__ void advance(State<CH, T> &) const {}
};

// im2col view of an NHWC fp16 tensor: row m = (b, oh, ow), k = (i * kx + j) * C + c.
struct ConvLoader {
    const _Float16 *x;
    int64_t M, K;
    int B, C, H, W, Ho, Wo, ky, kx, sy, sx, py, px, dy, dx;
    int vec;   // C % 8 == 0 and aligned base: a chunk is 8 channels of one tap

    template <int CH, int T>
    struct State {
        const _Float16 *img[CH];   // batch base pointer or null
        int ih0[CH], iw0[CH];
        int i, j, c;               // tap and channel of this thread's chunk in the current k-tile
    };
    template <int CH, int T>
    __device__ __forceinline__ void init(State<CH, T> &st, int64_t m0, int tid) const {
        const int k = (tid & 7) * 8;
        st.c = k % C;
        const int tap = k / C;
        st.j = tap % kx;
        st.i = tap / kx;
#pragma unroll
        for (int q = 0; q < CH; q++) {
            const int64_t m = m0 + (tid >> 3) + q * (T / 8);
            if (m < M) {
                const int ow = (int)(m % Wo);
                const int64_t t = m / Wo;
                const int oh = (int)(t % Ho);
                const int64_t b = t / Ho;
                st.img[q] = x + b * (int64_t)H * W * C;
                st.ih0[q] = oh * sy - py;
                st.iw0[q] = ow * sx - px;
            } else {
                st.img[q] = nullptr;
                st.ih0[q] = 0;
                st.iw0[q] = 0;
            }
        }
    }
    __device__ __forceinline__ _Float16 at(const _Float16 *img, int ih0, int iw0, int64_t k) const {
        if (k >= K) return (_Float16)0;
        const int c = (int)(k % C), tap = (int)(k / C), j = tap % kx, i = tap / kx;
        const int ih = ih0 + i * dy, iw = iw0 + j * dx;
        if (ih < 0 || ih >= H || iw < 0 || iw >= W) return (_Float16)0;
        return img[((int64_t)ih * W + iw) * C + c];
    }
    template <int CH, int T>
    __device__ __forceinline__ void fetch(State<CH, T> &st, int64_t k0, u32x4 (&out)[CH]) const {
        const int64_t k = k0 + (threadIdx.x & 7) * 8;
#pragma unroll
        for (int q = 0; q < CH; q++) {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (st.img[q] && k < K) {
                if (vec) {
                    const int ih = st.ih0[q] + st.i * dy, iw = st.iw0[q] + st.j * dx;
                    if (ih >= 0 && ih < H && iw >= 0 && iw < W)
                        v = *reinterpret_cast<const u32x4 *>(st.img[q] + ((int64_t)ih * W + iw) * C + st.c);
                } else {
                    half8 h;
#pragma unroll
                    for (int e = 0; e < 8; e++) h[e] = at(st.img[q], st.ih0[q], st.iw0[q], k + e);
                    v = __builtin_bit_cast(u32x4, h);
                }
            }
            out[q] = v;
        }
    }
    template <int CH, int T>
    __device__ __forceinline__ void advance(State<CH, T> &st) const {   // next k-tile: k += 64
        st.c += kBK;
        while (st.c >= C) {
            st.c -= C;
            if (++st.j == kx) { st.j = 0; ++st.i; }
        }
    }
};

// ---- the tile kernel ---------------------------------------------------------------------------------
template <int WM, int WN, int WGM, int WGN, class Loader>
__global__ __launch_bounds__(64 * WGM * WGN) void tile_kernel(Loader ld, const uint32_t *__restrict__ native,
                                                              int64_t M, int64_t K, int64_t N, int64_t Kb, int64_t Nb,
                                                              Epilogue ep, int tiles_m, int tiles_n) {
    constexpr int T = 64 * WGM * WGN, BM = 16 * WM * WGM, BN = 16 * WN * WGN, CH = BM * 8 / T;
    static_assert(BM * 8 % T == 0, "chunks must divide evenly");
    __shared__ __attribute__((aligned(16))) _Float16 As[BM * kPitch];

    // XCD-aware tile order: workgroup ids go round-robin over the 8 XCDs; give each XCD a
    // contiguous run of tiles, n fastest, so its L2 sees the same activation rows.
    int id = blockIdx.x;
    const int G = tiles_m * tiles_n;
    if ((G & 7) == 0) id = (id & 7) * (G >> 3) + (id >> 3);
    const int tm = id / tiles_n, tn = id % tiles_n;
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int wm = wv / WGN, wn = wv % WGN;
    const int r16 = lane & 15, g = lane >> 4;

    typename Loader::template State<CH, T> st;
    ld.template init<CH, T>(st, m0, tid);

    floatx4 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; i++)
#pragma unroll
        for (int j = 0; j < WN; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    // per n-fragment pointer into the native layout (dword index lane * 4 + d inside a block)
    const uint32_t *wptr[WN];
#pragma unroll
    for (int j = 0; j < WN; j++) {
        const int64_t nb = n0 / 16 + wn * WN + j;
        wptr[j] = nb < Nb ? native + (nb * Kb) * 256 + lane * 4 : nullptr;
    }
    const int KT = (int)((K + kBK - 1) / kBK);

    u32x4 stage[CH];
    uint32_t wcur[WN], wnext[WN];
    ld.template fetch<CH, T>(st, 0, stage);
#pragma unroll
    for (int j = 0; j < WN; j++) wcur[j] = wptr[j] ? wptr[j][0] : 0u;

    const int srow = tid >> 3, scol = (tid & 7) * 8;
    for (int kt = 0; kt < KT; kt++) {
        __syncthreads();   // every wave is done reading the previous tile
#pragma unroll
        for (int i = 0; i < CH; i++)
            *reinterpret_cast<u32x4 *>(&As[(srow + i * (T / 8)) * kPitch + scol]) = stage[i];
        __syncthreads();
        if (kt + 1 < KT) {
            ld.template advance<CH, T>(st);
            ld.template fetch<CH, T>(st, (int64_t)(kt + 1) * kBK, stage);
            const int kn = kt + 1;
#pragma unroll
            for (int j = 0; j < WN; j++) wnext[j] = wptr[j] ? wptr[j][(int64_t)(kn >> 2) * 256 + (kn & 3)] : 0u;
        }
#pragma unroll
        for (int s = 0; s < 2; s++) {
            half8 b[WN];
#pragma unroll
            for (int j = 0; j < WN; j++) b[j] = decode_step(wcur[j], s);
#pragma unroll
            for (int i = 0; i < WM; i++) {
                const half8 a = *reinterpret_cast<const half8 *>(
                    &As[(wm * WM * 16 + i * 16 + r16) * kPitch + s * 32 + g * 8]);
#pragma unroll
                for (int j = 0; j < WN; j++) acc[i][j] = mfma16(a, b[j], acc[i][j]);
            }
        }
#pragma unroll
        for (int j = 0; j < WN; j++) wcur[j] = wnext[j];
    }

    // epilogue: lane holds rows m = .. + 4g + r (r = 0..3), column n = .. + r16
#pragma unroll
    for (int j = 0; j < WN; j++) {
        const int64_t n = n0 + (wn * WN + j) * 16 + r16;
        if (n >= N) continue;
        const float sc = (ep.scale ? ep.scale[n] : 1.0f) * (1.0f / kWeightUnit);
        const float bi = ep.bias ? ep.bias[n] : 0.0f;
#pragma unroll
        for (int i = 0; i < WM; i++) {
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int64_t m = m0 + (wm * WM + i) * 16 + g * 4 + r;
                if (m >= M) continue;
                float v = acc[i][j][r] * sc + bi;
                const int64_t o = m * N + n;
                if (ep.y_f16) {
                    if (ep.residual) v += (float)static_cast<const _Float16 *>(ep.residual)[o];
                    if (ep.relu) v = v > 0.f ? v : 0.f;
                    static_cast<_Float16 *>(ep.y)[o] = (_Float16)v;
                } else {
                    if (ep.residual) v += static_cast<const float *>(ep.residual)[o];
                    if (ep.relu) v = v > 0.f ? v : 0.f;
                    static_cast<float *>(ep.y)[o] = v;
                }
            }
        }
    }
}

template <int WM, int WN, int WGM, int WGN, class Loader>
int launch_tile(const Loader &ld, const void *native, int64_t M, int64_t K, int64_t N, const Epilogue &ep,
                void *stream) {
    constexpr int BM = 16 * WM * WGM, BN = 16 * WN * WGN;
    const int64_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    if (tm * tn > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL((tile_kernel<WM, WN, WGM, WGN, Loader>), dim3((uint32_t)(tm * tn)), dim3(64 * WGM * WGN), 0,
                       as_stream(stream), ld, static_cast<const uint32_t *>(native), M, K, N, native_blocks_k(K),
                       native_blocks_n(N), ep, (int)tm, (int)tn);
    return check_launch();
}

// Tile choice: the largest tile that still yields at least ~2 workgroups per CU, else smaller.
template <class Loader>
int dispatch_tile(const Loader &ld, const void *native, int64_t M, int64_t K, int64_t N, const Epilogue &ep,
                  void *stream) {
    auto wgs = [&](int bm, int bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    if (N > 128 && wgs(256, 256) >= 256) return launch_tile<8, 4, 2, 4>(ld, native, M, K, N, ep, stream);
    if (N > 64 && wgs(256, 128) >= 384) return launch_tile<8, 4, 2, 2>(ld, native, M, K, N, ep, stream);
    if (N > 64 && wgs(128, 128) >= 256) return launch_tile<4, 4, 2, 2>(ld, native, M, K, N, ep, stream);
    if (wgs(128, 64) >= 512) return launch_tile<4, 4, 2, 1>(ld, native, M, K, N, ep, stream);
    return launch_tile<2, 4, 2, 1>(ld, native, M, K, N, ep, stream);
}

}  // namespace

int launch_gemm_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                      const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream) {
    DenseLoader ld{static_cast<const _Float16 *>(x), M, K, (K % 8 == 0) && aligned16(x) ? 1 : 0};
    Epilogue ep{scale, bias, residual, y, relu, y_f16};
    return dispatch_tile(ld, native, M, K, N, ep, stream);
}

}  // namespace tmq

using namespace tmq;

extern "C" {

int tmq_conv2d_out_hw(const tmq_conv_shape *s, int32_t *ho, int32_t *wo) {
    if (!s || !ho || !wo || s->sy <= 0 || s->sx <= 0 || s->dy <= 0 || s->dx <= 0 || s->ky <= 0 || s->kx <= 0)
        return TMQ_ERR_INVALID_ARG;
    *ho = (s->H + 2 * s->py - s->dy * (s->ky - 1) - 1) / s->sy + 1;
    *wo = (s->W + 2 * s->px - s->dx * (s->kx - 1) - 1) / s->sx + 1;
    return TMQ_OK;
}

int tmq_ternary_conv2d(const void *x, const tmq_conv_shape *s, const void *native, const tmq_epilogue *epilogue,
                       void *y, void *stream) {
    if (!s || !x || !native || !y || !aligned16(native)) return TMQ_ERR_INVALID_ARG;
    tmq_epilogue e = {nullptr, nullptr, nullptr, 0, TMQ_F32};
    if (epilogue) e = *epilogue;
    const float *scale = e.scale, *bias = e.bias;
    const void *residual = e.residual;
    const int relu = e.relu, y_dtype = e.y_dtype;
    if (y_dtype != TMQ_F16 && y_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
    int32_t ho, wo;
    int rc = tmq_conv2d_out_hw(s, &ho, &wo);
    if (rc != TMQ_OK) return rc;
    if (s->B < 0 || s->C <= 0 || s->H <= 0 || s->W <= 0 || s->N <= 0 || s->py < 0 || s->px < 0) return TMQ_ERR_INVALID_ARG;
    if (ho <= 0 || wo <= 0) return TMQ_ERR_INVALID_ARG;
    const int64_t M = (int64_t)s->B * ho * wo, K = (int64_t)s->C * s->ky * s->kx;
    if (M == 0) return TMQ_OK;
    ConvLoader ld{static_cast<const _Float16 *>(x), M, K, s->B, s->C, s->H, s->W, ho, wo, s->ky, s->kx, s->sy, s->sx,
                  s->py, s->px, s->dy, s->dx, (s->C % 8 == 0) && aligned16(x) ? 1 : 0};
    Epilogue ep{scale, bias, residual, y, relu, y_dtype == TMQ_F16 ? 1 : 0};
    return dispatch_tile(ld, native, M, K, s->N, ep, stream);
}

}  // extern "C"
