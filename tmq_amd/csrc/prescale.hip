// fp32 activations for the fp16 MFMA kernels: the power-of-two prescale that brings a tensor into fp16's
// range, and the split of (prescaled) values into fp16 terms.
//
// The ternary kernels multiply fp16 operands. fp32 activations are carried as hi = fp16(x), lo = fp16(x - hi)
// (22 significant bits), which only works while x sits inside fp16's exponent range: above 65504 hi
// overflows, below ~6e-5 the terms are subnormal and lose their bits. The reference multiplies in fp32
// (tmq/tmq_cuda.cu:242-427) and has no such limit. So a caller first scales the tensor by the power of two s
// that puts max|x| into [1024, 2048) -- exact, whatever the magnitude -- and folds 1/s into the
// per-channel scale of the epilogue; elements more than 2^14 below the maximum keep an absolute
// precision of 2^-35 of that maximum, which is below the rounding of the fp32 accumulation.
#include "common.h"
#include "mfma.h"

#include <math.h>

namespace tmq {
namespace {

constexpr int kPartials = 1024;           // partial maxima of the multi-block scan
constexpr int64_t kSingleMax = 1 << 16;   // up to here one workgroup does everything in one launch

__device__ __forceinline__ float finite_abs(float v) {
    const float a = __builtin_fabsf(v);
    return a < INFINITY ? a : 0.f;          // NaN and Inf take no part in the maximum (they propagate anyway)
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// maximum over the workgroup, valid in every thread
__device__ __forceinline__ float block_max(float v, float *lds /* >= 17 floats */) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    if (lane == 0) lds[wv] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
        for (int i = 0; i < nw; i++) t = fmaxf(t, lds[i]);
        lds[16] = t;
    }
    __syncthreads();
    return lds[16];
}

// s = 2^(11 - e) for amax in [2^(e-1), 2^e), kept inside the normal range together with its reciprocal.
__device__ __forceinline__ void make_prescale(float amax, float &s, float &inv) {
    s = 1.f;
    inv = 1.f;
    if (!(amax > 0.f)) return;
    int e;
    (void)frexpf(amax, &e);
    int p = 11 - e;
    p = p > 126 ? 126 : (p < -126 ? -126 : p);
    s = ldexpf(1.f, p);
    inv = ldexpf(1.f, -p);
}

__device__ __forceinline__ float scan_abs_max(const float *__restrict__ x, int64_t n, int64_t first, int64_t stride, bool vec) {
    float m = 0.f;
    if (vec) {
        const int64_t n4 = n / 4;
        for (int64_t i = first; i < n4; i += stride) {
            const floatx4 v = *reinterpret_cast<const floatx4 *>(x + 4 * i);
            m = fmaxf(fmaxf(m, fmaxf(finite_abs(v[0]), finite_abs(v[1]))), fmaxf(finite_abs(v[2]), finite_abs(v[3])));
        }
        for (int64_t i = 4 * n4 + first; i < n; i += stride) m = fmaxf(m, finite_abs(x[i]));
    } else {
        for (int64_t i = first; i < n; i += stride) m = fmaxf(m, finite_abs(x[i]));
    }
    return m;
}

__device__ __forceinline__ void write_scale(const float *scale_in, float *scale_out, int64_t channels, float inv) {
    if (!scale_out) return;
    for (int64_t c = threadIdx.x; c < channels; c += blockDim.x) scale_out[c] = (scale_in ? scale_in[c] : 1.f) * inv;
}

// Small tensors: one workgroup scans, derives the prescale, writes the scaled copy and the adjusted
// per-channel scale -- one launch in front of a GEMV.
__global__ __launch_bounds__(1024) void prescale_single_kernel(const float *__restrict__ x, int64_t n, float *prescale,
                                                               float *__restrict__ xs, const float *scale_in,
                                                               float *scale_out, int64_t channels, int vec) {
    __shared__ float lds[17];
    const float amax = block_max(scan_abs_max(x, n, threadIdx.x, blockDim.x, vec != 0), lds);
    float s, inv;
    make_prescale(amax, s, inv);
    if (threadIdx.x == 0) {
        prescale[0] = s;
        prescale[1] = inv;
    }
    if (xs) {
        if (vec) {
            const int64_t n4 = n / 4;
            for (int64_t i = threadIdx.x; i < n4; i += blockDim.x)
                *reinterpret_cast<floatx4 *>(xs + 4 * i) = *reinterpret_cast<const floatx4 *>(x + 4 * i) * s;
            for (int64_t i = 4 * n4 + threadIdx.x; i < n; i += blockDim.x) xs[i] = x[i] * s;
        } else {
            for (int64_t i = threadIdx.x; i < n; i += blockDim.x) xs[i] = x[i] * s;
        }
    }
    write_scale(scale_in, scale_out, channels, inv);
}

__global__ __launch_bounds__(256) void absmax_partial_kernel(const float *__restrict__ x, int64_t n, float *partials, int vec) {
    __shared__ float lds[17];
    const float m = block_max(scan_abs_max(x, n, (int64_t)blockIdx.x * 256 + threadIdx.x, (int64_t)gridDim.x * 256, vec != 0), lds);
    if (threadIdx.x == 0) partials[blockIdx.x] = m;
}

__global__ __launch_bounds__(1024) void prescale_finalize_kernel(const float *partials, int count, float *prescale,
                                                                 const float *scale_in, float *scale_out, int64_t channels) {
    __shared__ float lds[17];
    const float amax = block_max((int)threadIdx.x < count ? partials[threadIdx.x] : 0.f, lds);
    float s, inv;
    make_prescale(amax, s, inv);
    if (threadIdx.x == 0) {
        prescale[0] = s;
        prescale[1] = inv;
    }
    write_scale(scale_in, scale_out, channels, inv);
}

__global__ __launch_bounds__(256) void scale_copy_kernel(const float *__restrict__ x, const float *prescale,
                                                         float *__restrict__ xs, int64_t n, int vec) {
    const float s = prescale[0];
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i0 >= n) return;
    if (vec && i0 + 4 <= n) {
        *reinterpret_cast<floatx4 *>(xs + i0) = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(x + i0)) * s;
    } else {
        for (int64_t i = i0; i < n && i < i0 + 4; i++) xs[i] = x[i] * s;
    }
}

// x s = hi + lo with hi = fp16(x s), lo = fp16(x s - hi): 22 significant bits in two fp16 values (s = 1 without
// a prescale; lo may be left out). 8 elements per thread (two 16-byte loads, a 16-byte store per term) when
// the pointers allow it.
template <bool LO, bool SCALED>
__global__ __launch_bounds__(256) void split_terms_kernel(const float *__restrict__ x, const float *prescale,
                                                          _Float16 *__restrict__ hi, _Float16 *__restrict__ lo, int64_t n,
                                                          int vec) {
    float s = 1.f;
    if constexpr (SCALED) s = prescale[0];
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i0 >= n) return;
    if (vec && i0 + 8 <= n) {
        floatx4 a = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(x + i0));
        floatx4 b = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(x + i0 + 4));
        if constexpr (SCALED) {
            a *= s;
            b *= s;
        }
        half8 h, l;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            h[e] = (_Float16)a[e];
            h[4 + e] = (_Float16)b[e];
            l[e] = (_Float16)(a[e] - (float)h[e]);
            l[4 + e] = (_Float16)(b[e] - (float)h[4 + e]);
        }
        *reinterpret_cast<half8 *>(hi + i0) = h;
        if constexpr (LO) *reinterpret_cast<half8 *>(lo + i0) = l;
    } else {
        for (int64_t i = i0; i < n && i < i0 + 8; i++) {
            const float v = SCALED ? x[i] * s : x[i];
            const _Float16 h = (_Float16)v;
            hi[i] = h;
            if constexpr (LO) lo[i] = (_Float16)(v - (float)h);
        }
    }
}

// A few fp32 rows as fp16 row pairs, each row with a prescale of its own: one workgroup per row finds the row's
// largest finite |x|, scales by the power of two s that brings it into [1024, 2048) and writes hi = fp16(s x) and
// lo = fp16(s x - hi) to x16, 1 / s to row_scale[m]. The rows go in groups of `group` (the last may be shorter):
// group g occupies x16 rows 2 g group onwards, its hi rows first, then its lo rows. The fp16 rows have Kp >= K values
// (a multiple of 8), zeros behind the K-th. vec: K a multiple of 4 and x 16-byte aligned (whole float4s).
__global__ __launch_bounds__(1024) void split_rows_kernel(const float *__restrict__ x, int64_t K, int64_t Kp, int rows, int group,
                                                          _Float16 *__restrict__ x16, float *__restrict__ row_scale, int vec) {
    __shared__ float lds[17];
    const int m = blockIdx.x;
    const int g = m / group, w = m - g * group, in_group = rows - g * group < group ? rows - g * group : group;
    const float *row = x + (int64_t)m * K;
    const float amax = block_max(scan_abs_max(row, K, threadIdx.x, 1024, vec != 0), lds);
    float s, inv;
    make_prescale(amax, s, inv);
    if (threadIdx.x == 0) row_scale[m] = inv;
    _Float16 *hi = x16 + (int64_t)(2 * g * group + w) * Kp, *lo = hi + (int64_t)in_group * Kp;
    for (int64_t i0 = (int64_t)threadIdx.x * 8; i0 < Kp; i0 += 8192) {
        floatx4 a = {0.f, 0.f, 0.f, 0.f}, b = {0.f, 0.f, 0.f, 0.f};
        if (vec) {
            if (i0 < K) a = *reinterpret_cast<const floatx4 *>(row + i0) * s;
            if (i0 + 4 < K) b = *reinterpret_cast<const floatx4 *>(row + i0 + 4) * s;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                if (i0 + e < K) a[e] = row[i0 + e] * s;
                if (i0 + 4 + e < K) b[e] = row[i0 + 4 + e] * s;
            }
        }
        half8 h, l;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            h[e] = (_Float16)a[e];
            h[4 + e] = (_Float16)b[e];
            l[e] = (_Float16)(a[e] - (float)h[e]);
            l[4 + e] = (_Float16)(b[e] - (float)h[4 + e]);
        }
        *reinterpret_cast<half8 *>(hi + i0) = h;
        *reinterpret_cast<half8 *>(lo + i0) = l;
    }
}

// Largest finite |x| of 4096 values per workgroup and round (four 16-byte loads per thread in flight), one partial
// per workgroup. x 16-byte aligned; the n % 4 values at the end go to workgroup 0.
__global__ __launch_bounds__(256) void absmax_wide_kernel(const float *__restrict__ x, int64_t n, float *partials) {
    __shared__ float lds[17];
    const int64_t n4 = n / 4;
    float m = 0.f;
    for (int64_t base = (int64_t)blockIdx.x * 1024; base < n4; base += (int64_t)gridDim.x * 1024) {
        floatx4 v[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int64_t at = base + i * 256 + threadIdx.x;
            v[i] = at < n4 ? __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(x) + at) : floatx4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
            m = fmaxf(fmaxf(m, fmaxf(finite_abs(v[i][0]), finite_abs(v[i][1]))), fmaxf(finite_abs(v[i][2]), finite_abs(v[i][3])));
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) m = fmaxf(m, finite_abs(x[4 * n4 + threadIdx.x]));
    m = block_max(m, lds);
    if (threadIdx.x == 0) partials[blockIdx.x] = m;
}

// hi = fp16(s x) for the whole tensor in the launch after absmax_wide_kernel: every workgroup asks for its 8192 values
// first, reduces the partial maxima itself while they are on their way (at most 1024 floats), derives s, converts, and
// writes its slice of the per-channel scale divided by s; workgroup 0 also writes the prescale.
__global__ __launch_bounds__(256) void convert_prescaled_kernel(const float *__restrict__ x, int64_t n,
                                                                const float *__restrict__ partials, int count,
                                                                _Float16 *__restrict__ hi, float *prescale,
                                                                const float *scale_in, float *scale_out, int64_t channels,
                                                                int vec) {
    __shared__ float lds[17];
    constexpr int kQuads = 8;                                      // float4s per thread
    const int64_t n4 = n / 4, base = (int64_t)blockIdx.x * (256 * kQuads);
    floatx4 v[kQuads];
    if (vec) {
#pragma unroll
        for (int i = 0; i < kQuads; i++) {
            const int64_t at = base + i * 256 + threadIdx.x;
            v[i] = at < n4 ? __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(x) + at) : floatx4{0.f, 0.f, 0.f, 0.f};
        }
    }
    float pm = 0.f;
    for (int i = threadIdx.x; i < count; i += 256) pm = fmaxf(pm, partials[i]);
    const float amax = block_max(pm, lds);
    float s, inv;
    make_prescale(amax, s, inv);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        prescale[0] = s;
        prescale[1] = inv;
    }
    if (scale_out)
        for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < channels; c += (int64_t)gridDim.x * 256)
            scale_out[c] = (scale_in ? scale_in[c] : 1.f) * inv;
    if (vec) {
#pragma unroll
        for (int i = 0; i < kQuads; i++) {
            const int64_t at = base + i * 256 + threadIdx.x;
            if (at >= n4) continue;
            const floatx4 a = v[i] * s;
            *reinterpret_cast<half4 *>(hi + 4 * at) = half4{(_Float16)a[0], (_Float16)a[1], (_Float16)a[2], (_Float16)a[3]};
        }
        if (blockIdx.x == 0 && threadIdx.x < (n & 3)) hi[4 * n4 + threadIdx.x] = (_Float16)(x[4 * n4 + threadIdx.x] * s);
    } else {
        for (int64_t i = base * 4 + threadIdx.x; i < n && i < (base + 256 * kQuads) * 4; i += 256) hi[i] = (_Float16)(x[i] * s);
    }
}

// Many fp32 rows as fp16 row pairs in groups of eight, every group under a power of two s of its own: a workgroup
// of 1024 takes the group's 8 K values -- float4 number 1024 i + t to thread t, up to NQ of them in
// registers and all asked for at once (a single trip to memory; longer rows are read a second time) -- finds the
// largest finite |x|, and writes hi = fp16(s x) of row m to x16 row 16 (m / 8) + m % 8, lo = fp16(s x - hi) eight rows
// further on (rows past M of the last group: zeros) and 1 / s to group_scale[m / 8]. K a multiple of 4.
template <int NQ>
__global__ __launch_bounds__(1024) void split_groups_kernel(const float *__restrict__ x, int64_t M, int64_t K,
                                                            _Float16 *__restrict__ x16, float *__restrict__ group_scale) {
    __shared__ float lds[17];
    const int64_t g = blockIdx.x, q_row = K / 4, quads = 8 * q_row;              // float4s per row / per group
    const float *src = x + g * 8 * K;
    int64_t live = (M - g * 8) * q_row;                                            // float4s that exist
    if (live > quads) live = quads;
    const bool held = quads <= (int64_t)NQ * 1024;
    floatx4 q[NQ];
    float amax = 0.f;
    if (held) {
#pragma unroll
        for (int i = 0; i < NQ; i++) {
            const int64_t at = (int64_t)i * 1024 + threadIdx.x;
            q[i] = at < live ? __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(src) + at) : floatx4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int i = 0; i < NQ; i++)
            amax = fmaxf(fmaxf(amax, fmaxf(finite_abs(q[i][0]), finite_abs(q[i][1]))), fmaxf(finite_abs(q[i][2]), finite_abs(q[i][3])));
    } else {
        for (int64_t at = threadIdx.x; at < live; at += 1024) {
            const floatx4 v = *(reinterpret_cast<const floatx4 *>(src) + at);
            amax = fmaxf(fmaxf(amax, fmaxf(finite_abs(v[0]), finite_abs(v[1]))), fmaxf(finite_abs(v[2]), finite_abs(v[3])));
        }
    }
    amax = block_max(amax, lds);
    float s, inv;
    make_prescale(amax, s, inv);
    if (threadIdx.x == 0 && blockIdx.y == 0) group_scale[g] = inv;
    // gridDim.y workgroups (a power of two) share a group: each takes the whole group for the maximum -- one CU pulls
    // ~40 GB/s, and the idle CUs are free -- and converts every gridDim.y-th run of 1024 float4s
    const int share = gridDim.y - 1, mine = blockIdx.y;
    _Float16 *dst = x16 + g * 16 * K;                                              // the group's hi rows, then its lo rows
    auto emit = [&](int64_t at, floatx4 v) {
        v *= s;
        half4 h, l;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            h[e] = (_Float16)v[e];
            l[e] = (_Float16)(v[e] - (float)h[e]);
        }
        *reinterpret_cast<half4 *>(dst + 4 * at) = h;                              // row at / q_row of the group, same position
        *reinterpret_cast<half4 *>(dst + 8 * K + 4 * at) = l;
    };
    if (held) {
#pragma unroll
        for (int i = 0; i < NQ; i++) {
            const int64_t at = (int64_t)i * 1024 + threadIdx.x;
            if ((i & share) == mine && at < quads) emit(at, q[i]);
        }
    } else {
        for (int64_t at = (int64_t)mine * 1024 + threadIdx.x; at < quads; at += (int64_t)(share + 1) * 1024)
            emit(at, at < live ? *(reinterpret_cast<const floatx4 *>(src) + at) : floatx4{0.f, 0.f, 0.f, 0.f});
    }
}

}  // namespace

// The same split for rows of any length and alignment, written as rows of Kp >= K values (Kp a multiple of 8) with
// zeros behind the K-th: one workgroup per group of eight rows, element-wise reads, one 16-byte piece of a hi row and
// of its lo row per thread and step. The second pass over the group's 32 K bytes comes from L2. With few groups,
// gridDim.y workgroups share one: each finds the group's maximum itself and writes every gridDim.y-th run of pieces.
// VEC: K is a multiple of 4 and x 16-byte aligned -- whole float4s, two per piece (K a multiple of 8: never across the end).
template <bool VEC>
__global__ __launch_bounds__(1024) void split_groups_padded_kernel(const float *__restrict__ x, int64_t M, int K, int Kp,
                                                                   FastDiv by_row, _Float16 *__restrict__ x16,
                                                                   float *__restrict__ group_scale) {
    __shared__ float lds[17];
    const int64_t g = blockIdx.x;
    const float *src = x + g * 8 * (int64_t)K;
    const int rows = M - g * 8 < 8 ? (int)(M - g * 8) : 8;
    float amax = 0.f;
    if constexpr (VEC) {
        for (int at = threadIdx.x; at < rows * (K / 4); at += 1024) {
            const floatx4 v = *(reinterpret_cast<const floatx4 *>(src) + at);
            amax = fmaxf(fmaxf(amax, fmaxf(finite_abs(v[0]), finite_abs(v[1]))), fmaxf(finite_abs(v[2]), finite_abs(v[3])));
        }
    } else {
        for (int at = threadIdx.x; at < rows * K; at += 1024) amax = fmaxf(amax, finite_abs(src[at]));
    }
    amax = block_max(amax, lds);
    float s, inv;
    make_prescale(amax, s, inv);
    if (threadIdx.x == 0 && blockIdx.y == 0) group_scale[g] = inv;
    _Float16 *dst = x16 + g * 16 * (int64_t)Kp;                    // the group's hi rows, then its lo rows
    const uint32_t pieces = 8u * (uint32_t)(Kp / 8);
    for (uint32_t p = blockIdx.y * 1024u + threadIdx.x; p < pieces; p += 1024u * gridDim.y) {
        int c;
        const int r = (int)by_row.divmod(p, c);
        const int k0 = c * 8;
        half8 h = {0, 0, 0, 0, 0, 0, 0, 0}, l = {0, 0, 0, 0, 0, 0, 0, 0};
        if (r < rows) {
            if constexpr (VEC) {
#pragma unroll
                for (int q = 0; q < 2; q++)
                    if (k0 + 4 * q < K) {
                        const floatx4 f = *reinterpret_cast<const floatx4 *>(src + (int64_t)r * K + k0 + 4 * q);
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float v = s * f[e];
                            h[4 * q + e] = (_Float16)v;
                            l[4 * q + e] = (_Float16)(v - (float)h[4 * q + e]);
                        }
                    }
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++)
                    if (k0 + e < K) {
                        const float v = s * src[(int64_t)r * K + k0 + e];
                        h[e] = (_Float16)v;
                        l[e] = (_Float16)(v - (float)h[e]);
                    }
            }
        }
        *reinterpret_cast<half8 *>(dst + (int64_t)r * Kp + k0) = h;
        *reinterpret_cast<half8 *>(dst + (int64_t)(8 + r) * Kp + k0) = l;
    }
}

// x16: 16 ceil(M / 8) rows of Kp fp16 values (Kp >= K, a multiple of 8; zeros behind the K-th), 16-byte aligned;
// group_scale: ceil(M / 8) floats. Whole float4s of 16-byte aligned rows and Kp == K take the kernel above.
int launch_split_groups(const float *x, int64_t M, int64_t K, int64_t Kp, void *x16, float *group_scale, void *stream) {
    const int64_t groups = (M + 7) / 8, quads = 8 * (K / 4);
    if (groups > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    if (Kp != K || K % 4 != 0 || !aligned16(x)) {
        if (8 * Kp > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
        // few groups: up to eight workgroups each (M = 17, K = 4000: 3 workgroups -> 12)
        const int64_t runs = (Kp + 1023) / 1024;
        const uint32_t share = groups > 64 ? 1 : (uint32_t)(runs < 1 ? 1 : runs > 8 ? 8 : runs);
        auto padded = K % 4 == 0 && aligned16(x) ? split_groups_padded_kernel<true> : split_groups_padded_kernel<false>;
        hipLaunchKernelGGL(padded, dim3((uint32_t)groups, share), dim3(1024), 0, as_stream(stream), x, M, (int)K,
                           (int)Kp, FastDiv((uint32_t)(Kp / 8)), static_cast<_Float16 *>(x16), group_scale);
        return check_launch();
    }
    auto kernel = quads <= 2 * 1024 ? split_groups_kernel<2> : quads <= 4 * 1024 ? split_groups_kernel<4>
                : quads <= 8 * 1024 ? split_groups_kernel<8> : split_groups_kernel<16>;
    // up to 64 groups share a group among up to four workgroups (M = 32 at K = 4096: 14.5 -> 13.4 us in all, M = 512
    // 42.4 -> 40.8; M = 1024, where the CUs are busy anyway, 62.0 -> 63.1)
    const uint32_t share = groups > 64 || quads <= 1024 ? 1 : quads <= 2048 ? 2 : 4;
    hipLaunchKernelGGL(kernel, dim3((uint32_t)groups, share), dim3(1024), 0, as_stream(stream), x, M, K,
                       static_cast<_Float16 *>(x16), group_scale);
    return check_launch();
}

// Rows of K fp16 values copied to rows of Kp >= K values (Kp a multiple of 8), zeros behind the K-th: a thread moves
// one 16-byte piece of the destination (vec: K % 8 == 0 and x 16-byte aligned, so the piece is one load as well).
__global__ __launch_bounds__(256) void pad_rows_kernel(const _Float16 *__restrict__ x, uint32_t pieces, int K, FastDiv by_row,
                                                       _Float16 *__restrict__ out, int vec) {
    const uint32_t id = blockIdx.x * 256u + threadIdx.x;
    if (id >= pieces) return;
    int c;
    const uint32_t m = by_row.divmod(id, c);
    const int k0 = c * 8;
    const _Float16 *src = x + (int64_t)m * K + k0;
    half8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (vec) {
        if (k0 < K) v = *reinterpret_cast<const half8 *>(src);
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++)
            if (k0 + e < K) v[e] = src[e];
    }
    *reinterpret_cast<half8 *>(out + (int64_t)id * 8) = v;
}

// out: M rows of Kp fp16 values, 16-byte aligned; Kp % 8 == 0, M Kp < 2^31.
int launch_pad_rows(const void *x, int64_t M, int64_t K, int64_t Kp, void *out, void *stream) {
    const int64_t pieces = M * (Kp / 8);
    if (pieces <= 0 || pieces > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL(pad_rows_kernel, dim3((uint32_t)((pieces + 255) / 256)), dim3(256), 0, as_stream(stream),
                       static_cast<const _Float16 *>(x), (uint32_t)pieces, (int)K, FastDiv((uint32_t)(Kp / 8)),
                       static_cast<_Float16 *>(out), (K % 8 == 0 && aligned16(x)) ? 1 : 0);
    return check_launch();
}

// x16: 2 M rows of Kp >= K fp16 values (Kp % 8 == 0, zeros behind the K-th), 16-byte aligned; row_scale: M floats.
int launch_split_rows(const float *x, int64_t M, int64_t K, int64_t Kp, int64_t group, void *x16, float *row_scale, void *stream) {
    hipLaunchKernelGGL(split_rows_kernel, dim3((uint32_t)M), dim3(1024), 0, as_stream(stream), x, K, Kp, (int)M, (int)group,
                       static_cast<_Float16 *>(x16), row_scale, (K % 4 == 0 && aligned16(x)) ? 1 : 0);
    return check_launch();
}

}  // namespace tmq

using namespace tmq;

extern "C" {

size_t tmq_f32_prescale_workspace_bytes(int64_t n) { return n > kSingleMax ? kPartials * sizeof(float) : 0; }

int tmq_f32_prescale(const float *x, int64_t n, float *prescale, float *xs, const float *scale_in, float *scale_out,
                     int64_t channels, void *workspace, void *stream) {
    if (n <= 0 || !x || !prescale || channels < 0 || (scale_out && channels == 0)) return TMQ_ERR_INVALID_ARG;
    const int vec = aligned16(x) && (!xs || aligned16(xs));
    if (n <= kSingleMax) {
        hipLaunchKernelGGL(prescale_single_kernel, dim3(1), dim3(1024), 0, as_stream(stream), x, n, prescale, xs, scale_in,
                           scale_out, channels, vec);
        return check_launch();
    }
    if (!workspace) return TMQ_ERR_INVALID_ARG;
    float *partials = static_cast<float *>(workspace);
    int64_t blocks = (n + 8191) / 8192;                    // 32 values per thread and more
    if (blocks > kPartials) blocks = kPartials;
    hipLaunchKernelGGL(absmax_partial_kernel, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream), x, n, partials,
                       (int)aligned16(x));
    int rc = check_launch();
    if (rc != TMQ_OK) return rc;
    hipLaunchKernelGGL(prescale_finalize_kernel, dim3(1), dim3(1024), 0, as_stream(stream), partials, (int)blocks, prescale,
                       scale_in, scale_out, channels);
    rc = check_launch();
    if (rc != TMQ_OK || !xs) return rc;
    const int64_t cblocks = (n + 1023) / 1024;
    if (cblocks > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL(scale_copy_kernel, dim3((uint32_t)cblocks), dim3(256), 0, as_stream(stream), x, prescale, xs, n, vec);
    return check_launch();
}

int tmq_split_f32_scaled(const float *x, const float *prescale, void *hi, void *lo, int64_t n, void *stream) {
    if (n < 0 || (n > 0 && (!x || !hi))) return TMQ_ERR_INVALID_ARG;
    if (n == 0) return TMQ_OK;
    const int64_t blocks = (n + 2047) / 2048;
    if (blocks > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    const int vec = aligned16(x) && aligned16(hi) && aligned16(lo);
    auto kernel = lo ? (prescale ? split_terms_kernel<true, true> : split_terms_kernel<true, false>)
                     : (prescale ? split_terms_kernel<false, true> : split_terms_kernel<false, false>);
    hipLaunchKernelGGL(kernel, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream), x, prescale,
                       static_cast<_Float16 *>(hi), static_cast<_Float16 *>(lo), n, vec);
    return check_launch();
}

size_t tmq_f32_to_f16_prescaled_workspace_bytes(int64_t n) { return n > 0 ? kPartials * sizeof(float) : 0; }

int tmq_f32_to_f16_prescaled(const float *x, int64_t n, float *prescale, void *hi, const float *scale_in, float *scale_out,
                             int64_t channels, void *workspace, void *stream) {
    if (n <= 0 || !x || !prescale || !hi || !workspace || channels < 0 || (scale_out && channels == 0)) return TMQ_ERR_INVALID_ARG;
    float *partials = static_cast<float *>(workspace);
    const int vec = aligned16(x) && (reinterpret_cast<uintptr_t>(hi) & 7u) == 0;
    int64_t blocks = (n + 4095) / 4096;                    // 16 values per thread and round
    if (blocks > kPartials) blocks = kPartials;
    if (vec) {
        hipLaunchKernelGGL(absmax_wide_kernel, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream), x, n, partials);
    } else {
        blocks = (n + 8191) / 8192;
        if (blocks > kPartials) blocks = kPartials;
        hipLaunchKernelGGL(absmax_partial_kernel, dim3((uint32_t)blocks), dim3(256), 0, as_stream(stream), x, n, partials, 0);
    }
    if (int rc = check_launch()) return rc;
    const int64_t groups = (n + 8191) / 8192;
    if (groups > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL(convert_prescaled_kernel, dim3((uint32_t)groups), dim3(256), 0, as_stream(stream), x, n, partials, (int)blocks,
                       static_cast<_Float16 *>(hi), prescale, scale_in, scale_out, channels, vec);
    return check_launch();
}

int tmq_split_f32(const float *x, void *hi, void *lo, int64_t n, void *stream) {
    if (n > 0 && !lo) return TMQ_ERR_INVALID_ARG;
    return tmq_split_f32_scaled(x, nullptr, hi, lo, n, stream);
}

}  // extern "C"
