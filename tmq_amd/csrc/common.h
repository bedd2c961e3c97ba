// Shared host/device helpers of libtmq_hip (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tmq_hip.h"

namespace tmq {

// Records the failing hipError_t for tmq_last_hip_error() and maps it to TMQ_ERR_LAUNCH.
int note_hip_error(hipError_t e);

inline int check_launch() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? TMQ_OK : note_hip_error(e);
}

// A kernel that wants more than 64 KiB of dynamic LDS has to opt in once per device
// (hipFuncAttributeMaxDynamicSharedMemorySize). Remembers the largest size granted per kernel and device, so
// the runtime call is made the first time only (and again if a later launch asks for more); callable from
// any thread, with the launch's device current. TMQ_OK or TMQ_ERR_LAUNCH.
int allow_dynamic_lds(const void *kernel, size_t bytes);

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int kWave = 64;

// Whether a GEMM of M x N outputs over K reduction indices goes to the split-reduction kernels (mid.hip)
// rather than the big-tile kernel. Measured crossovers: with K >= 512 the split reduction wins up to two
// tiles of 64 x 64 per CU, which 64 x 128 tiles still cover in one pass (beyond that its second pass runs
// partly empty: M = 4608, K = 4096, N = 512 takes 52 us there and 31 us on the big-tile kernel); with shorter
// reductions its per-tile cost shows earlier (K = 256: up to ~128 tiles, K = 128: ~64). Long reductions over
// wide layers keep it a little longer (M = 576, K = 8192, N = 4096: 50 us against 58 us).
inline bool split_reduction_pays(int64_t M, int64_t K, int64_t N) {
    const int64_t tiles64 = ((M + 63) / 64) * ((N + 63) / 64);
    return K >= 512 ? tiles64 <= ((K >= 8192 && N >= 2048) ? 640 : 512) : tiles64 <= K / 2;
}

// 16 bytes per lane from global memory straight into LDS through a buffer resource: lane l's 16 bytes at byte
// `offset` of the buffer go to byte 16 l of the (uniform) destination; a lane whose offset lies past the end of
// the buffer gets zeros. The padding taps of a convolution then cost a select of the offset instead of a select
// between two 64-bit addresses. The host pass does not know the builtins and only sees empty bodies.
constexpr uint32_t kPastTheEnd = 0xFFFFFFF0u;   // beyond any buffer these kernels wrap (hosts check: < 2^32 - 32 bytes)
#if defined(__HIP_DEVICE_COMPILE__)
typedef __amdgpu_buffer_rsrc_t BufferResource;
#else
struct BufferResource {};
#endif
__device__ __forceinline__ BufferResource make_buffer_resource(const void *base, uint32_t bytes) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);   // raw buffer, 32-bit elements
#else
    return {};
#endif
}
__device__ __forceinline__ void buffer_to_lds(BufferResource rsrc, uint32_t offset, unsigned char *dst) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef __attribute__((address_space(3))) void *lds_ptr;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr)dst, 16, offset, 0, 0, 0);
#endif
}

// Workgroup ids are dealt round-robin over the 8 XCDs, each with an L2 of its own. Position of workgroup `id` of `G`
// in an order where the workgroups of one XCD are consecutive, so that a kernel can give them neighbouring tiles.
// XCDs below G % 8 (all of them when that is 0) hold ceil(G / 8) workgroups, the others one fewer.
__device__ __forceinline__ int xcd_contiguous(int id, int G) {
    const int xcd = id & 7, per = (G + 7) >> 3, rem = G & 7;
    return xcd * per - ((rem != 0 && xcd > rem) ? xcd - rem : 0) + (id >> 3);
}

// Division of 0 <= n < 2^31 by a divisor known on the host (an image extent): q = umulhi(n, mul) >> shift,
// two instructions instead of the ~25 of a 32-bit division. With s = ceil(log2 d) and mul = ceil(2^(31 + s) / d)
// (< 2^32), n mul / 2^(31 + s) exceeds n / d by less than 2^-s <= 1 / d, so the floor is the same.
struct FastDiv {
    uint32_t mul, shift, d;
    FastDiv() : mul(0), shift(0), d(1) {}
    explicit FastDiv(uint32_t div) : mul(0), shift(0), d(div) {
        if (div > 1) {
            uint32_t s = 0;
            while ((uint64_t(1) << s) < div) s++;
            mul = (uint32_t)(((uint64_t(1) << (31 + s)) + div - 1) / div);
            shift = s - 1;
        }
    }
#if defined(__HIPCC__)
    __device__ __forceinline__ uint32_t divmod(uint32_t n, int &rem) const {
        const uint32_t q = d > 1 ? __umulhi(n, mul) >> shift : n;
        rem = (int)(n - q * d);
        return q;
    }
#endif
};

// Where the rows of an implicit-GEMM convolution go when they are not consecutive in y. Row m is position
// (b, oh, ow) of the computed output grid; the kept positions (h0 <= oh < h0 + h_cnt, the same along w) go to pixel
// b sb + (oh - h0) sh + (ow - w0) sw of the destination (a pixel is the N contiguous channels of one position),
// the others are dropped. A phase of a transposed convolution writes its share of the interleaved output this way.
struct NoMap {                          // rows are consecutive: row m is pixel m (an empty member of the epilogue structs)
    static constexpr bool kDrops = false;   // pixel() never returns -1
    static constexpr bool kPairs = false;   // rows r and r ^ 8 of a 16-row fragment are not added
#if defined(__HIPCC__)
    __device__ __forceinline__ int64_t pixel(int64_t m) const { return m; }
#endif
};

struct RowMap {
    static constexpr bool kDrops = true;
    static constexpr bool kPairs = false;
    FastDiv hw, w;                     // computed positions per image / per image row
    int32_t h0 = 0, w0 = 0, h_cnt = 0, w_cnt = 0;
    int64_t sb = 0, sh = 0, sw = 0;    // in pixels
#if defined(__HIPCC__)
    __device__ __forceinline__ int64_t pixel(int64_t m) const {      // -1: dropped
        int rem, ow;
        const uint32_t b = hw.divmod((uint32_t)m, rem);
        const int oh = (int)w.divmod((uint32_t)rem, ow) - h0;
        ow -= w0;
        if ((uint32_t)oh >= (uint32_t)h_cnt || (uint32_t)ow >= (uint32_t)w_cnt) return -1;
        return (int64_t)b * sb + (int64_t)oh * sh + (int64_t)ow * sw;
    }
#endif
};

// fp32 rows carried as two fp16 rows each (hi = fp16(s x), lo = fp16(s x - hi)), eight rows at a time: rows
// 16 q .. 16 q + 7 of the fp16 matrix are the hi terms of output rows 8 q .. 8 q + 7, rows 16 q + 8 .. 16 q + 15 their
// lo terms -- a pair always sits in one 16-row MFMA fragment, whatever the tile. Every group of eight rows has a power
// of two s of its own. The epilogues add rows r and r ^ 8 of a fragment where they read it back from LDS (kPairs) and
// multiply by the group's 1 / s (group_scale[m / 16]) before the per-channel scale; the lo rows are dropped and row m
// goes to output row 8 (m / 16) + m % 8.
struct PairMap {
    static constexpr bool kDrops = true;
    static constexpr bool kPairs = true;
    int64_t rows_out = 0;
    const float *group_scale = nullptr;     // ceil(rows_out / 8) floats
#if defined(__HIPCC__)
    __device__ __forceinline__ int64_t pixel(int64_t m) const {
        const int64_t o = ((m >> 4) << 3) + (m & 7);
        return (m & 8) || o >= rows_out ? -1 : o;
    }
    // 1 / s of the fragment that starts at row m16 (a multiple of 16); fragments past the last group: 0
    __device__ __forceinline__ float fragment_scale(int64_t m16) const {
        return (m16 >> 1) < rows_out ? group_scale[m16 >> 4] : 0.f;
    }
#endif
};

#if defined(__HIPCC__)
// a / b and a % b for 0 <= a, 0 < b. The GPU has no integer divider: a 64-bit division expands to
// ~100 instructions, a 32-bit one to ~20, and index arithmetic (pixel -> batch, row, column) sits in
// the prologue of every workgroup -- so take the 32-bit route whenever the dividend fits.
__device__ __forceinline__ int64_t div_rem(int64_t a, int b, int &rem) {
    if (a < ((int64_t)1 << 32)) {
        const uint32_t q = (uint32_t)a / (uint32_t)b;
        rem = (int)((uint32_t)a - q * (uint32_t)b);
        return q;
    }
    const int64_t q = a / b;
    rem = (int)(a - q * b);
    return q;
}

// Sum over the 64 lanes of a wavefront with DPP row operations (no LDS traffic): butterfly
// inside each row of 16 lanes, then the four row sums are fetched with v_readlane.
__device__ __forceinline__ float wave_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false));  // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false));  // row_mirror
    const int iv = __builtin_bit_cast(int, v);
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
    return (r0 + r1) + (r2 + r3);
}

// Block-wide sum (blockDim.x a multiple of 64, at most 1024): wave_sum, then one LDS slot per
// wave, then the first wave adds the slots. The result is valid in thread 0.
__device__ __forceinline__ float block_sum(float v, float *lds /* >= 16 floats */) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    if (lane == 0) lds[wv] = v;
    __syncthreads();
    float t = 0.f;
    if (threadIdx.x == 0)
        for (int i = 0; i < nw; i++) t += lds[i];
    return t;
}
#endif

}  // namespace tmq
