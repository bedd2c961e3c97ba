// 2-bit ternary pack / unpack on the GPU (gfx950).
//
// Format (tmq/tmq_native.cpp:152-208): a weight matrix W[N][K] (N output channels, K = fan-in,
// for a convolution K = C*ky*kx in that order) becomes words[K][ceil(N/16)]; word (k,q) holds
// the codes of W[16q+j][k], j = 0..15, first element in bits 31:30; 0 -> 00, +1 -> 01, -1 -> 10.
//
// The layout is a transpose, so the kernels tile it: a workgroup owns 64 k x 256 n. Lane = k,
// which makes every global fp32 access a coalesced 256-byte row segment of W; each lane builds
// (or splits) whole words in registers; words cross between the "lane = k" and the "16 words
// per row" arrangements through a 4 KiB LDS tile so that the packed side moves 64-byte segments.
// Both directions are bound by the fp32 side: 4 B/weight + 1/8 B/weight.
#include "common.h"

namespace tmq {
namespace {

constexpr int kTileK = 64;   // lanes of one wave
constexpr int kTileQ = 16;   // words per tile row (256 output channels); 4 per wave
constexpr int kThreads = 256;

// float -> code with the reference's semantics: roundf (half away from zero), then the x86
// float->int conversion (NaN and |v| >= 2^31 become INT_MIN), then clamp to [-1, 1].
// On the bits u of v: +1 exactly for 0.5 <= v < 2^31, i.e. 0x3F000000 <= u < 0x4F000000 (one unsigned range check);
// -1 for every other value of magnitude >= 0.5, which takes in negative numbers, +-Inf and NaN (their magnitude bits
// exceed 0x7F800000 >= 0x3F000000); 0 otherwise.
__device__ __forceinline__ uint32_t code_of(float v) {
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    const bool plus = (u - 0x3F000000u) < 0x10000000u;
    const bool nonzero = (u & 0x7FFFFFFFu) >= 0x3F000000u;
    return plus ? 1u : (nonzero ? 2u : 0u);
}
__device__ __forceinline__ uint32_t code_of(int32_t v) { return v > 0 ? 1u : (v < 0 ? 2u : 0u); }
__device__ __forceinline__ uint32_t code_of(int8_t v) { return v > 0 ? 1u : (v < 0 ? 2u : 0u); }

template <typename T>
__global__ __launch_bounds__(kThreads) void pack_kernel(const T *__restrict__ w, uint32_t *__restrict__ out, int64_t N,
                                                        int64_t K, int64_t Q) {
    __shared__ uint32_t tile[kTileK][kTileQ + 1];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t k0 = (int64_t)blockIdx.x * kTileK, q0 = (int64_t)blockIdx.y * kTileQ;
    const int64_t k = k0 + lane;
#pragma unroll
    for (int qi = 0; qi < 4; qi++) {
        const int ql = wv * 4 + qi;
        const int64_t nbase = (q0 + ql) * 16;
        uint32_t word = 0;
        if (k < K && nbase < N) {
            T v[16];
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = (nbase + j < N) ? w[(nbase + j) * K + k] : T(0);
#pragma unroll
            for (int j = 0; j < 16; j++) word = (word << 2) | code_of(v[j]);
        }
        tile[lane][ql] = word;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int row = i * 16 + (threadIdx.x >> 4), col = threadIdx.x & 15;
        if (k0 + row < K && q0 + col < Q) out[(k0 + row) * Q + q0 + col] = tile[row][col];
    }
}

__global__ __launch_bounds__(kThreads) void unpack_kernel(const uint32_t *__restrict__ in, float *__restrict__ w,
                                                          int64_t N, int64_t K, int64_t Q) {
    __shared__ uint32_t tile[kTileK][kTileQ + 1];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t k0 = (int64_t)blockIdx.x * kTileK, q0 = (int64_t)blockIdx.y * kTileQ;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int row = i * 16 + (threadIdx.x >> 4), col = threadIdx.x & 15;
        tile[row][col] = (k0 + row < K && q0 + col < Q) ? in[(k0 + row) * Q + q0 + col] : 0u;
    }
    __syncthreads();
    const int64_t k = k0 + lane;
    if (k >= K) return;
#pragma unroll
    for (int qi = 0; qi < 4; qi++) {
        const int ql = wv * 4 + qi;
        const int64_t nbase = (q0 + ql) * 16;
        if (nbase >= N) break;
        const uint32_t word = tile[lane][ql];
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const uint32_t c = (word >> (30 - 2 * j)) & 3u;
            const float v = c == 1u ? 1.0f : (c == 2u ? -1.0f : 0.0f);   // 11 decodes to 0
            if (nbase + j < N) w[(nbase + j) * K + k] = v;
        }
    }
}

// ---- 4-wide variants ----------------------------------------------------------------------------------
// Same tile with four k per thread: every global access on the unpacked side is a 16-byte (fp32 /
// int32) or 4-byte (int8) vector. Need K % 4 == 0 and a base address aligned to four elements;
// anything else takes the scalar kernels above.
template <typename T>
struct alignas(sizeof(T) * 4) Vec4 {
    T v[4];
};

template <typename T>
__global__ __launch_bounds__(kThreads) void pack4_kernel(const T *__restrict__ w, uint32_t *__restrict__ out, int64_t N,
                                                         int64_t K, int64_t Q) {
    // 64 k x 256 n per workgroup as in the scalar kernel; thread = (4 consecutive k, one word column):
    // 16 neighbouring lanes read 256 contiguous bytes of a row, a thread has 16 vector loads in flight
    __shared__ uint32_t tile[kTileK][kTileQ + 1];
    const int kq = threadIdx.x & 15, ql = threadIdx.x >> 4;
    const int64_t k0 = (int64_t)blockIdx.x * kTileK, q0 = (int64_t)blockIdx.y * kTileQ;
    const int64_t k = k0 + kq * 4, nbase = (q0 + ql) * 16;
    uint32_t word[4] = {0u, 0u, 0u, 0u};
    if (k < K && nbase < N) {
        Vec4<T> v[16];
#pragma unroll
        for (int j = 0; j < 16; j++) {
            if (nbase + j < N) v[j] = *reinterpret_cast<const Vec4<T> *>(w + (nbase + j) * K + k);
            else v[j] = Vec4<T>{{T(0), T(0), T(0), T(0)}};
        }
#pragma unroll
        for (int j = 0; j < 16; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) word[e] = (word[e] << 2) | code_of(v[j].v[e]);
    }
#pragma unroll
    for (int e = 0; e < 4; e++) tile[kq * 4 + e][ql] = word[e];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int row = i * 16 + (threadIdx.x >> 4), col = threadIdx.x & 15;
        if (k0 + row < K && q0 + col < Q) out[(k0 + row) * Q + q0 + col] = tile[row][col];
    }
}

__global__ __launch_bounds__(kThreads) void unpack4_kernel(const uint32_t *__restrict__ in, float *__restrict__ w,
                                                           int64_t N, int64_t K, int64_t Q) {
    __shared__ uint32_t tile[kTileK][kTileQ + 1];
    const int kq = threadIdx.x & 15, ql = threadIdx.x >> 4;
    const int64_t k0 = (int64_t)blockIdx.x * kTileK, q0 = (int64_t)blockIdx.y * kTileQ;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int row = i * 16 + (threadIdx.x >> 4), col = threadIdx.x & 15;
        tile[row][col] = (k0 + row < K && q0 + col < Q) ? in[(k0 + row) * Q + q0 + col] : 0u;
    }
    __syncthreads();
    const int64_t k = k0 + kq * 4, nbase = (q0 + ql) * 16;
    if (k >= K || nbase >= N) return;
    uint32_t word[4];
#pragma unroll
    for (int e = 0; e < 4; e++) word[e] = tile[kq * 4 + e][ql];
#pragma unroll
    for (int j = 0; j < 16; j++) {
        Vec4<float> v;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t c = (word[e] >> (30 - 2 * j)) & 3u;
            v.v[e] = c == 1u ? 1.0f : (c == 2u ? -1.0f : 0.0f);   // 11 decodes to 0
        }
        if (nbase + j < N) *reinterpret_cast<Vec4<float> *>(w + (nbase + j) * K + k) = v;
    }
}

// ---- wide variants: 256 k per workgroup ------------------------------------------------------------------
// A wavefront owns one word column (16 output channels) over 256 consecutive k: lane l holds k = 4 l .. 4 l + 3,
// so every access on the unpacked side is a whole contiguous KiB of one row of W per instruction, like a plain
// copy; a lane has all 16 rows in flight at once. The WAVES word columns of a workgroup meet in LDS
// (column-major, one conflict-free 16-byte access per lane on that side), so that the packed side moves
// 4 WAVES contiguous bytes per k. Same preconditions as the 4-wide kernels.
constexpr int kWideK = 256, kWidePitch = kWideK + 4;
constexpr int kPackWaves = 4, kUnpackWaves = 8;   // word columns per workgroup (measured, see the launches)
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

template <typename T, int WQ, int WK>
__global__ __launch_bounds__(64 * WQ * WK) void pack_wide_kernel(const T *__restrict__ w, uint32_t *__restrict__ out,
                                                                 int64_t N, int64_t K, int64_t Q) {
    constexpr int TK = kWideK * WK;
    __shared__ __attribute__((aligned(16))) uint32_t tile[WQ][TK + 4];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, wq = wv / WK, wk = wv % WK;
    const int64_t k0 = (int64_t)blockIdx.x * TK, q0 = (int64_t)blockIdx.y * WQ;
    const int64_t k = k0 + wk * kWideK + lane * 4, nbase = (q0 + wq) * 16;
    uint32_t word[4] = {0u, 0u, 0u, 0u};
    if (k < K && nbase < N) {
        typedef T vec4 __attribute__((ext_vector_type(4)));
        vec4 v[16];
        if (nbase + 16 <= N) {
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = __builtin_nontemporal_load(reinterpret_cast<const vec4 *>(w + (nbase + j) * K + k));
        } else {
#pragma unroll
            for (int j = 0; j < 16; j++) {
                if (nbase + j < N) v[j] = *reinterpret_cast<const vec4 *>(w + (nbase + j) * K + k);
                else v[j] = vec4{T(0), T(0), T(0), T(0)};
            }
        }
#pragma unroll
        for (int j = 0; j < 16; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) word[e] = (word[e] << 2) | code_of((T)v[j][e]);
    }
    *reinterpret_cast<u32x4_t *>(&tile[wq][wk * kWideK + lane * 4]) = u32x4_t{word[0], word[1], word[2], word[3]};
    __syncthreads();
    if (WQ == 4 && Q % 4 == 0 && q0 + 4 <= Q && (reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
        // a thread per k: the four words of its row as one 16-byte store
        for (int row = threadIdx.x; row < TK; row += 64 * WQ * WK)
            if (k0 + row < K)
                *reinterpret_cast<u32x4_t *>(out + (k0 + row) * Q + q0) = u32x4_t{tile[0][row], tile[1 % WQ][row], tile[2 % WQ][row], tile[3 % WQ][row]};
        return;
    }
    for (int idx = threadIdx.x; idx < TK * WQ; idx += 64 * WQ * WK) {
        const int row = idx / WQ, col = idx % WQ;
        if (k0 + row < K && q0 + col < Q) out[(k0 + row) * Q + q0 + col] = tile[col][row];
    }
}

template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) void unpack_wide_kernel(const uint32_t *__restrict__ in, float *__restrict__ w,
                                                                 int64_t N, int64_t K, int64_t Q) {
    __shared__ __attribute__((aligned(16))) uint32_t tile[WAVES][kWidePitch];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t k0 = (int64_t)blockIdx.x * kWideK, q0 = (int64_t)blockIdx.y * WAVES;
    for (int idx = threadIdx.x; idx < kWideK * WAVES; idx += 64 * WAVES) {
        const int row = idx / WAVES, col = idx % WAVES;
        tile[col][row] = (k0 + row < K && q0 + col < Q) ? in[(k0 + row) * Q + q0 + col] : 0u;
    }
    __syncthreads();
    const int64_t k = k0 + lane * 4, nbase = (q0 + wv) * 16;
    if (k >= K || nbase >= N) return;
    const u32x4_t word = *reinterpret_cast<const u32x4_t *>(&tile[wv][lane * 4]);
#pragma unroll
    for (int j = 0; j < 16; j++) {
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t c = (word[e] >> (30 - 2 * j)) & 3u;
            v[e] = c == 1u ? 1.0f : (c == 2u ? -1.0f : 0.0f);   // 11 decodes to 0
        }
        if (nbase + j < N) __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(w + (nbase + j) * K + k));
    }
}

template <typename T>
bool vec4_ok(const void *p, int64_t K) {
    return K % 4 == 0 && (reinterpret_cast<uintptr_t>(p) % (4 * sizeof(T))) == 0;
}

template <typename T>
void launch_pack(const void *w, int64_t N, int64_t K, int64_t Q, uint32_t *words, void *stream) {
    const bool wide = vec4_ok<T>(w, K);
    if (wide && K >= kWideK) {
        // Four word columns x 256 k per workgroup measured best (K = N = 4096: 14.3 us; sixteen columns 17.4, two
        // columns x 512 k 16.0, one column x 1024 k 17.7): small independent workgroups overlap one another's loads,
        // coding and stores, and the packed side still leaves in 16-byte pieces.
        dim3 wgrid((uint32_t)((K + kWideK - 1) / kWideK), (uint32_t)((Q + kPackWaves - 1) / kPackWaves));
        hipLaunchKernelGGL((pack_wide_kernel<T, kPackWaves, 1>), wgrid, dim3(64 * kPackWaves), 0, as_stream(stream),
                           static_cast<const T *>(w), words, N, K, Q);
        return;
    }
    dim3 grid((uint32_t)((K + kTileK - 1) / kTileK), (uint32_t)((Q + kTileQ - 1) / kTileQ)), block(kThreads);
    if (wide)
        hipLaunchKernelGGL(pack4_kernel<T>, grid, block, 0, as_stream(stream), static_cast<const T *>(w), words, N, K, Q);
    else
        hipLaunchKernelGGL(pack_kernel<T>, grid, block, 0, as_stream(stream), static_cast<const T *>(w), words, N, K, Q);
}

}  // namespace
}  // namespace tmq

using namespace tmq;

extern "C" {

int tmq_pack_ternary(const void *w, int dtype, int64_t N, int64_t K, uint32_t *words, void *stream) {
    if (N < 0 || K < 0) return TMQ_ERR_INVALID_ARG;
    if (N == 0 || K == 0) return TMQ_OK;
    if (!w || !words) return TMQ_ERR_INVALID_ARG;
    const int64_t Q = (N + 15) / 16;
    const int64_t gx = (K + kTileK - 1) / kTileK, gy = (Q + kTileQ - 1) / kTileQ;
    if (gx > 0x7FFFFFFF || gy > 65535 || (Q + kPackWaves - 1) / kPackWaves > 65535) return TMQ_ERR_TOO_LARGE;
    switch (dtype) {
        case TMQ_F32: launch_pack<float>(w, N, K, Q, words, stream); break;
        case TMQ_I32: launch_pack<int32_t>(w, N, K, Q, words, stream); break;
        case TMQ_I8: launch_pack<int8_t>(w, N, K, Q, words, stream); break;
        default: return TMQ_ERR_UNSUPPORTED;
    }
    return check_launch();
}

int tmq_unpack_ternary(const uint32_t *words, int64_t N, int64_t K, float *w, void *stream) {
    if (N < 0 || K < 0) return TMQ_ERR_INVALID_ARG;
    if (N == 0 || K == 0) return TMQ_OK;
    if (!w || !words) return TMQ_ERR_INVALID_ARG;
    const int64_t Q = (N + 15) / 16;
    const int64_t gx = (K + kTileK - 1) / kTileK, gy = (Q + kTileQ - 1) / kTileQ;
    if (gx > 0x7FFFFFFF || gy > 65535 || (Q + kUnpackWaves - 1) / kUnpackWaves > 65535) return TMQ_ERR_TOO_LARGE;
    if (vec4_ok<float>(w, K) && K >= kWideK) {
        hipLaunchKernelGGL(unpack_wide_kernel<kUnpackWaves>,
                           dim3((uint32_t)((K + kWideK - 1) / kWideK), (uint32_t)((Q + kUnpackWaves - 1) / kUnpackWaves)),
                           dim3(64 * kUnpackWaves), 0, as_stream(stream), words, w, N, K, Q);
    } else if (vec4_ok<float>(w, K))
        hipLaunchKernelGGL(unpack4_kernel, dim3((uint32_t)gx, (uint32_t)gy), dim3(kThreads), 0, as_stream(stream), words, w,
                           N, K, Q);
    else
        hipLaunchKernelGGL(unpack_kernel, dim3((uint32_t)gx, (uint32_t)gy), dim3(kThreads), 0, as_stream(stream), words,
                           w, N, K, Q);
    return check_launch();
}

}  // extern "C"
