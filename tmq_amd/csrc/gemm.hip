// MFMA-bound ternary GEMM / implicit-GEMM convolution for gfx950.
//
//   Y[m][n] = epilogue( sum_k A[m][k] * T[k][n] ),   A = activations (fp16), T = ternary weights
//
// Work split: a workgroup owns a BM x BN output tile; its WGM x WGN wavefronts each own
// (16 WM) x (16 WN) of it as WM x WN accumulators of v_mfma_f32_16x16x32_f16 (fp32 accumulate).
//   * Activations: one 64-wide k-tile ahead of the math in LDS, shared by every wavefront of the
//     workgroup. Aligned shapes (dense rows with K % 64 == 0, convolutions with 8, 16, 32 or a
//     multiple of 64 channels) are loaded global -> LDS directly (tile_dma_kernel); everything else
//     goes global -> registers -> LDS with per-element guards (tile_kernel). LDS rows are 128 bytes,
//     chunks XOR-swizzled so the 16-byte operand reads of a wavefront are conflict-free.
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
#include "tile_epilogue.h"
#include <type_traits>
#include <utility>

namespace tmq {

// mid.hip: split-reduction kernel for outputs of a few hundred 64 x 64 tiles
bool mid_conv_ok(const void *x, const tmq_conv_shape *s);
int launch_mid_conv(const void *x, const tmq_conv_shape *s, int ho, int wo, const void *native, const float *scale,
                    const float *bias, const void *residual, int relu, void *y, int y_f16, const RowMap *map, void *stream);

namespace {

constexpr int kBK = 64;          // k-tile
__device__ u32x4 kZeroChunk;              // zero-initialised, never written: what loads of padding taps / k-tiles past K are redirected to

constexpr int kPitch = 64;       // LDS row pitch in halfs: 128 bytes = 8 chunks of 16 bytes, no padding.
// Chunk c of row r is stored at position c ^ (r & 7): a wavefront's stores cover whole rows
// (contiguous kilobytes) and the operand reads of 8 consecutive rows at one k offset land in 8
// different 16-byte bank groups.

// ---- loaders ------------------------------------------------------------------------------------------
// A loader hands every thread CH 16-byte chunks (8 fp16) of the BM x 64 activation tile: chunk i of
// thread t belongs to row (t / 8 + i * T / 8). Two kinds:
//   * register loaders (fetch): any shape; values pass through registers, guards in the loop. The
//     thread's chunk sits at k offset (t % 8) * 8.
//   * direct loaders (addr): rows are 16-byte aligned and a chunk never straddles the end of K or of a
//     tap, so a chunk is one address -- the zero chunk for padding -- and can be loaded straight into
//     LDS. The kernel tells init() which of the row's 8 chunks the thread fetches.

// Dense rows, any K / alignment. VEC: K is a multiple of 8 and x 16-byte aligned, so a chunk is 16 aligned bytes that
// lie wholly inside or wholly outside the row: one unconditional load, of zeros for what does not exist.
template <bool VEC>
struct DenseLoader {
    static constexpr bool kDirect = false;
    [[maybe_unused]] static constexpr bool kConv = false;
    [[maybe_unused]] static constexpr bool kBuffer = false;
    const _Float16 *x;
    int64_t M, K;

    template <int CH, int T>
    struct State {
        const _Float16 *row[CH];
        bool live[CH];
        int kc;
    };
    template <int CH, int T>
    __device__ __forceinline__ void init(State<CH, T> &st, int64_t m0, int tid) const {
        st.kc = (tid & 7) * 8;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const int64_t m = m0 + (tid >> 3) + i * (T / 8);
            st.live[i] = m < M;
            st.row[i] = x + (m < M ? m : M - 1) * K;
        }
    }
    template <int CH, int T>
    __device__ __forceinline__ void fetch(State<CH, T> &st, int64_t k0, u32x4 (&out)[CH]) const {
        const int64_t k = k0 + st.kc;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            if constexpr (VEC) {
                const bool in = st.live[i] & (k < K);
                const _Float16 *src = in ? st.row[i] + k : reinterpret_cast<const _Float16 *>(&kZeroChunk);
                out[i] = *reinterpret_cast<const u32x4 *>(src);
            } else {
                half8 h = {0, 0, 0, 0, 0, 0, 0, 0};
                if (st.live[i]) {
#pragma unroll
                    for (int e = 0; e < 8; e++)
                        if (k + e < K) h[e] = st.row[i][k + e];
                }
                out[i] = __builtin_bit_cast(u32x4, h);
            }
        }
    }
    template <int CH, int T>
    __device__ __forceinline__ void advance(State<CH, T> &) const {}
};

// Dense rows, 16-byte aligned, K a multiple of the k-tile. Rows past M are clamped to the last row
// (their results are never stored); k-tiles past K, which the pipeline prefetches and never multiplies,
// re-read the last tile.
struct DenseDirect {
    static constexpr bool kDirect = true;
    [[maybe_unused]] static constexpr bool kConv = false;
    [[maybe_unused]] static constexpr bool kBuffer = false;
    const _Float16 *x;
    int64_t M, K;

    template <int CH, int T>
    struct State {
        const _Float16 *row[CH];
        int kc;
    };
    template <int CH, int T>
    __device__ __forceinline__ void init(State<CH, T> &st, int64_t m0, int tid, int chunk) const {
        st.kc = chunk * 8;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const int64_t m = m0 + (tid >> 3) + i * (T / 8);
            st.row[i] = x + (m < M ? m : M - 1) * K;
        }
    }
    template <int CH, int T>
    __device__ __forceinline__ const void *addr(const State<CH, T> &st, int64_t k0, int i) const {
        return st.row[i] + ((k0 >= K ? K - kBK : k0) + st.kc);
    }
    template <int CH, int T>
    __device__ __forceinline__ void advance(State<CH, T> &) const {}
};

// The same rows fetched through a buffer resource over x (fewer than 2^32 - 32 bytes): a chunk is a 32-bit
// byte offset, and the loads are buffer instructions. The compiler keeps exact wait counts next to those; one
// pending global-to-LDS load makes it wait for every outstanding load and LDS read at each use (it treats that
// instruction like a flat access that may touch both memories). k-tiles past K deliver zeros.
struct DenseBuffer {
    [[maybe_unused]] static constexpr bool kDirect = true;
    [[maybe_unused]] static constexpr bool kConv = false;
    [[maybe_unused]] static constexpr bool kBuffer = true;
    const _Float16 *x;
    int64_t M, K;

    template <int CH, int T>
    struct State {
        uint32_t row[CH];   // byte offset of the row + this thread's chunk
        uint32_t k2;        // uniform: byte offset of the current k-tile inside a row
    };
    template <int CH, int T>
    __device__ __forceinline__ void init(State<CH, T> &st, int64_t m0, int tid, int chunk) const {
        st.k2 = 0;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const int64_t m = m0 + (tid >> 3) + i * (T / 8);
            st.row[i] = (uint32_t)((m < M ? m : M - 1) * K * 2) + chunk * 16;
        }
    }
    template <int CH, int T>
    __device__ __forceinline__ uint32_t offset(const State<CH, T> &st, int i) const {
        return st.k2 < (uint32_t)(K * 2) ? st.row[i] + st.k2 : kPastTheEnd;
    }
    __device__ __forceinline__ uint32_t bytes() const { return (uint32_t)(M * K * 2); }
    template <int CH, int T>
    __device__ __forceinline__ void advance(State<CH, T> &st) const { st.k2 += kBK * 2; }
};

// im2col view of an NHWC fp16 tensor: row m = (b, oh, ow), k = (i * kx + j) * C + c.
// VEC = C is a multiple of 8 and the base is 16-byte aligned: a chunk is 8 channels of one tap.
template <bool VEC>
struct ConvLoader {
    static constexpr bool kDirect = false;
    [[maybe_unused]] static constexpr bool kConv = true;
    [[maybe_unused]] static constexpr bool kBuffer = false;
    const _Float16 *x;
    int64_t M, K;
    int B, C, H, W, Ho, Wo, ky, kx, sy, sx, py, px, dy, dx;
    int quads = 0;                 // !VEC: C is a multiple of 4 and x 8-byte aligned -- a chunk is two 8-byte loads

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
                int ow, oh;
                const int64_t t = div_rem(m, Wo, ow);
                const int64_t b = div_rem(t, Ho, oh);
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
    template <int CH, int T>
    __device__ __forceinline__ void fetch(State<CH, T> &st, int64_t k0, u32x4 (&out)[CH]) const {
        const int64_t k = k0 + (threadIdx.x & 7) * 8;
#pragma unroll
        for (int q = 0; q < CH; q++) {
            u32x4 v = {0u, 0u, 0u, 0u};
            if constexpr (VEC) {
                // one unconditional load: chunks outside the image, past K or of rows past M read 16 bytes of zeros
                // (conditions joined without short circuit -- as branches they are an exec-mask round trip per chunk)
                const int ih = st.ih0[q] + st.i * dy, iw = st.iw0[q] + st.j * dx;
                const bool in = (st.img[q] != nullptr) & (k < K) & ((unsigned)ih < (unsigned)H) & ((unsigned)iw < (unsigned)W);
                const _Float16 *src = in ? st.img[q] + ((int64_t)ih * W + iw) * C + st.c
                                         : reinterpret_cast<const _Float16 *>(&kZeroChunk);
                v = *reinterpret_cast<const u32x4 *>(src);
            } else if (quads) {
                // two halves of four channels, each inside one tap (the second may be the next tap's first four); what
                // does not exist is read from 16 bytes of zeros
                typedef uint32_t u32x2v __attribute__((ext_vector_type(2)));
                int i = st.i, j = st.j, c = st.c;
                u32x2v half[2];
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int ih = st.ih0[q] + i * dy, iw = st.iw0[q] + j * dx;
                    const bool in = (st.img[q] != nullptr) & (k + 4 * h < K) & ((unsigned)ih < (unsigned)H) & ((unsigned)iw < (unsigned)W);
                    const _Float16 *src = in ? st.img[q] + ((int64_t)ih * W + iw) * C + c
                                             : reinterpret_cast<const _Float16 *>(&kZeroChunk);
                    half[h] = *reinterpret_cast<const u32x2v *>(src);
                    c += 4;
                    if (c == C) {
                        c = 0;
                        if (++j == kx) { j = 0; ++i; }
                    }
                }
                v = u32x4{half[0][0], half[0][1], half[1][0], half[1][1]};
            } else if (st.img[q] && k < K) {
                // element by element from the chunk's tap and channel onwards (a chunk may run over into the next tap)
                half8 h = {0, 0, 0, 0, 0, 0, 0, 0};
                int i = st.i, j = st.j, c = st.c;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int ih = st.ih0[q] + i * dy, iw = st.iw0[q] + j * dx;
                    if (k + e < K && (unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W)
                        h[e] = st.img[q][((int64_t)ih * W + iw) * C + c];
                    if (++c == C) {
                        c = 0;
                        if (++j == kx) { j = 0; ++i; }
                    }
                }
                v = __builtin_bit_cast(u32x4, h);
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

// im2col view for C % 64 == 0 (fewer than 2^31 elements): a 64-wide k-tile is
// 64 consecutive channels of ONE filter tap, so tap and channel offset are the same for the whole
// workgroup and live in scalar registers. Per row the loader keeps one 32-bit element offset and the
// window's top-left coordinate; a fetch is two unsigned compares, one add and the load.
// Bit t set when 0 <= x0 + t d < limit, for the taps t = 0 .. n - 1 (n <= 15) of one axis of a window that starts at x0.
// Without dilation the taps inside are a run lo .. hi, built from two shifts; dilated windows test tap by tap.
__device__ __forceinline__ uint32_t taps_inside(int x0, int n, int d, int limit) {
    if (d == 1) {
        const int lo = x0 < 0 ? -x0 : 0, hi = (limit - x0 < n ? limit - x0 : n) - 1;      // first and last tap inside
        return hi >= lo ? ((2u << hi) - 1u) & ~((1u << lo) - 1u) : 0u;
    }
    uint32_t bits = 0;
    for (int t = 0; t < n; t++) bits |= ((unsigned)(x0 + t * d) < (unsigned)limit) ? (1u << t) : 0u;
    return bits;
}

struct ConvLoader64 {
    static constexpr bool kDirect = true;
    [[maybe_unused]] static constexpr bool kConv = true;
    [[maybe_unused]] static constexpr bool kBuffer = true;
    const _Float16 *x;
    int64_t M, K;
    int B, C, H, W, Ho, Wo, ky, kx, sy, sx, py, px, dy, dx;
    FastDiv by_wo, by_ho;      // set by with_divisors(); M < 2^31

    // A row's window is tested against the image once: bit i of `taps` says that tap row i lies inside it, bit
    // 16 + j the same for tap column j (ky, kx <= 15, checked by the host). A k-tile's test is then one AND and one
    // compare against the tile's two bits instead of two additions, two compares and the scalar mask logic between them.
    template <int CH, int T>
    struct State {
        uint32_t off0[CH];         // byte offset of (b, ih0, iw0, channel kc); wraps below zero for padding
        uint32_t taps[CH];         // valid tap rows / columns of the row's window (rows past M: none)
        int i, j, c0;              // uniform: tap and first channel of the current k-tile
        uint32_t delta;            // uniform: byte offset of (tap, c0) relative to off0
        uint32_t want;             // uniform: the current tap's two bits; bit 15 (never set in taps) past the last tap
    };
    template <int CH, int T>
    __device__ __forceinline__ void init(State<CH, T> &st, int64_t m0, int tid, int chunk) const {
        st.i = st.j = st.c0 = 0;
        st.delta = 0;
        st.want = 1u | (1u << 16);
        const int kc = chunk * 8;
#pragma unroll
        for (int q = 0; q < CH; q++) {
            const int64_t m = m0 + (tid >> 3) + q * (T / 8);
            st.off0[q] = 0;
            st.taps[q] = 0;
            if (m < M) {
                int ow, oh;
                const uint32_t t = by_wo.divmod((uint32_t)m, ow);
                const int b = (int)by_ho.divmod(t, oh);
                const int ih0 = oh * sy - py, iw0 = ow * sx - px;
                st.off0[q] = (uint32_t)(((b * H + ih0) * W + iw0) * C + kc) * 2u;
                st.taps[q] = taps_inside(ih0, ky, dy, H) | (taps_inside(iw0, kx, dx, W) << 16);
            }
        }
    }
    template <int CH, int T>
    __device__ __forceinline__ const void *addr(const State<CH, T> &st, int64_t, int q) const {
        const bool in = (st.taps[q] & st.want) == st.want;
        return in ? static_cast<const void *>(reinterpret_cast<const unsigned char *>(x) + (st.off0[q] + st.delta))
                  : static_cast<const void *>(&kZeroChunk);
    }
    // The same chunk as a byte offset into a buffer resource over x; padding taps and the K tail get an
    // offset past its end, for which the load delivers zeros.
    template <int CH, int T>
    __device__ __forceinline__ uint32_t offset(const State<CH, T> &st, int q) const {
        return (st.taps[q] & st.want) == st.want ? st.off0[q] + st.delta : kPastTheEnd;
    }
    __device__ __forceinline__ uint32_t bytes() const { return (uint32_t)((int64_t)B * H * W * C * 2); }
    template <int CH, int T>
    __device__ __forceinline__ void advance(State<CH, T> &st) const {   // next k-tile: 64 channels on
        st.c0 += kBK;
        if (st.c0 == C) {
            st.c0 = 0;
            if (++st.j == kx) { st.j = 0; ++st.i; }   // past the last tap only in the zero-padded K tail: i >= ky
        }
        st.delta = (uint32_t)((st.i * dy * W + st.j * dx) * C + st.c0) * 2u;
        st.want = st.i < ky ? (1u << st.i) | (0x10000u << st.j) : 0x8000u;
    }
};

// im2col view for few channels (C = 8, 16 or 32; fewer than 2^31 elements): a
// 16-byte chunk is 8 channels of one tap and a 64-wide k-tile covers 64 / C taps. A thread's chunk
// keeps its channel offset for the whole reduction and its tap advances by 64 / C per k-tile, so the
// loader carries its tap (i, j) per thread, one 32-bit offset and the window's top-left coordinate per row.
struct ConvLoaderFewC {
    static constexpr bool kDirect = true;
    [[maybe_unused]] static constexpr bool kConv = true;
    [[maybe_unused]] static constexpr bool kBuffer = true;
    const _Float16 *x;
    int64_t M, K;
    int B, C, H, W, Ho, Wo, ky, kx, sy, sx, py, px, dy, dx;
    FastDiv by_wo, by_ho;      // set by with_divisors(); M < 2^31

    template <int CH, int T>
    struct State {
        int32_t off0[CH];          // element offset of (b, ih0, iw0, this thread's channel offset)
        int32_t ih0[CH], iw0[CH];  // top-left input coordinate of the row's window (rows past M: far outside)
        int i, j;                  // this thread's tap in the current k-tile
    };
    template <int CH, int T>
    __device__ __forceinline__ void init(State<CH, T> &st, int64_t m0, int tid, int chunk) const {
        const int kc = chunk * 8, tap = kc / C;
        st.i = tap / kx;
        st.j = tap - st.i * kx;
#pragma unroll
        for (int q = 0; q < CH; q++) {
            const int64_t m = m0 + (tid >> 3) + q * (T / 8);
            st.off0[q] = 0;
            st.ih0[q] = st.iw0[q] = INT32_MIN / 2;
            if (m < M) {
                int ow, oh;
                const uint32_t t = by_wo.divmod((uint32_t)m, ow);
                const int b = (int)by_ho.divmod(t, oh);
                st.ih0[q] = oh * sy - py;
                st.iw0[q] = ow * sx - px;
                st.off0[q] = ((b * H + st.ih0[q]) * W + st.iw0[q]) * C + kc % C;
            }
        }
    }
    template <int CH, int T>
    __device__ __forceinline__ const void *addr(const State<CH, T> &st, int64_t, int q) const {
        const int di = st.i * dy, dj = st.j * dx;
        const bool in = (st.i < ky) & ((unsigned)(st.ih0[q] + di) < (unsigned)H) & ((unsigned)(st.iw0[q] + dj) < (unsigned)W);
        return in ? static_cast<const void *>(x + (st.off0[q] + (di * W + dj) * C)) : static_cast<const void *>(&kZeroChunk);
    }
    template <int CH, int T>
    __device__ __forceinline__ uint32_t offset(const State<CH, T> &st, int q) const {
        const int di = st.i * dy, dj = st.j * dx;
        const bool in = (st.i < ky) & ((unsigned)(st.ih0[q] + di) < (unsigned)H) & ((unsigned)(st.iw0[q] + dj) < (unsigned)W);
        return in ? (uint32_t)(st.off0[q] + (di * W + dj) * C) * 2u : kPastTheEnd;
    }
    __device__ __forceinline__ uint32_t bytes() const { return (uint32_t)((int64_t)B * H * W * C * 2); }
    template <int CH, int T>
    __device__ __forceinline__ void advance(State<CH, T> &st) const {   // next k-tile: 64 / C taps on
        st.j += kBK / C;
        while (st.j >= kx) { st.j -= kx; ++st.i; }
    }
};

// ---- the tile kernel ---------------------------------------------------------------------------------
template <int WM, int WN, int WGM, int WGN, int D, class Loader, class Ep>
__global__ __launch_bounds__(64 * WGM * WGN, 2) void tile_kernel(Loader ld, const uint32_t *__restrict__ native,
                                                              int64_t M, int64_t K, int64_t N, int64_t Kb, int64_t Nb,
                                                              Ep ep, int tiles_m, int tiles_n) {
    constexpr int T = 64 * WGM * WGN, BM = 16 * WM * WGM, BN = 16 * WN * WGN, CH = BM * 8 / T;
    static_assert(BM * 8 % T == 0, "chunks must divide evenly");
    // two stages: the next k-tile is written while the current one is multiplied (one barrier per tile)
    __shared__ __attribute__((aligned(16))) _Float16 As[2][BM * kPitch];

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

    // per n-fragment pointer into the native layout (dword index lane * 4 + d inside a block);
    // fragments past N read block 0 of the last valid fragment (finite bits, never stored)
    const uint32_t *wptr[WN];
#pragma unroll
    for (int j = 0; j < WN; j++) {
        int64_t nb = n0 / 16 + wn * WN + j;
        if (nb >= Nb) nb = Nb - 1;
        wptr[j] = native + (nb * Kb) * 256 + lane * 4;
    }
    const int KT = (int)((K + kBK - 1) / kBK);

    // Register prefetch, D k-tiles deep: while tile kt is multiplied out of LDS, tiles kt + 1 .. kt + D
    // are in flight from global memory (D = 1: fetched at the top of a pass, stored at its end); a
    // 64-wide k-tile of MFMA work is far shorter than a trip to L2 when the tile is small.
    u32x4 stage[D][CH];
    uint32_t wcur[WN], wq[D][WN];
    const int srow = tid >> 3;
    const int scol = (((tid & 7) ^ (srow & 7)) * 8);   // (T / 8) is a multiple of 8, so row & 7 == srow & 7 for every chunk
    auto wload = [&](uint32_t (&w)[WN], int kn) {
        if (kn >= KT) kn = KT - 1;
#pragma unroll
        for (int j = 0; j < WN; j++) w[j] = wptr[j][(int64_t)(kn >> 2) * 256 + (kn & 3)];
    };
    auto lds_store = [&](int buf, const u32x4 (&v)[CH]) {
#pragma unroll
        for (int i = 0; i < CH; i++) *reinterpret_cast<u32x4 *>(&As[buf][(srow + i * (T / 8)) * kPitch + scol]) = v[i];
    };
    wload(wcur, 0);
    ld.template fetch<CH, T>(st, 0, stage[0]);
    lds_store(0, stage[0]);
#pragma unroll
    for (int d = 0; d + 1 < D; d++) {   // the last set is filled by the first pass of the loop
        ld.template advance<CH, T>(st);
        ld.template fetch<CH, T>(st, (int64_t)(d + 1) * kBK, stage[d]);
        wload(wq[d], d + 1);
    }
    __syncthreads();

    // per-column epilogue constants, fetched now so their latency hides behind the main loop
    const int64_t nw0 = n0 + (int64_t)wn * WN * 16;        // first column of this wave
    ColumnConstants cc;
    load_scale_bias<WN>(ep, lane, nw0, N, cc);

    const int arow = (wm * WM * 16 + r16) * kPitch;
    // operand read of m-fragment i, k-step s: chunk (4 s + g) of row (.. + 16 i + r16); 16 i keeps row & 7
    auto swz = [&](int i, int s) { return i * 16 * kPitch + (((4 * s + g) ^ (r16 & 7)) * 8); };
    // one k-tile; `slot` (static) is the register set that holds tile kt + 1
    auto body = [&](int kt, auto slot_tag) {
        constexpr int slot = decltype(slot_tag)::value, freed = (slot + D - 1) % D;
        // the set written to LDS in the previous pass is refilled with tile kt + D; issued ahead of
        // the matrix work so that address arithmetic and load issue overlap with it
        ld.template advance<CH, T>(st);
        ld.template fetch<CH, T>(st, (int64_t)(kt + D) * kBK, stage[freed]);
        wload(wq[freed], kt + D);
        const int cur = kt & 1;
        const _Float16 *abase = &As[cur][arow];
        // Software pipeline over the 2 WM operand reads of the tile (fragment i, k-step s): kAhead reads
        // are in flight ahead of the MFMAs that consume them, so LDS latency hides behind matrix
        // work of this wave. sched_barrier pins the order; the compiler only adds the waits.
        constexpr int NQ = 2 * WM, kAhead = NQ < 4 ? NQ : 4;
        half8 a[NQ];
        half8 bfr[2][WN];
#pragma unroll
        for (int q = 0; q < kAhead; q++) a[q] = *reinterpret_cast<const half8 *>(abase + swz(q >> 1, q & 1));
#pragma unroll
        for (int j = 0; j < WN; j++) bfr[0][j] = decode_step(wcur[j], 0);
#pragma unroll
        for (int j = 0; j < WN; j++) bfr[1][j] = decode_step(wcur[j], 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int q = 0; q < NQ; q++) {
#pragma unroll
            for (int j = 0; j < WN; j++) acc[q >> 1][j] = mfma16(a[q], bfr[q & 1][j], acc[q >> 1][j]);
            if (q + kAhead < NQ)
                a[q + kAhead] = *reinterpret_cast<const half8 *>(abase + swz((q + kAhead) >> 1, (q + kAhead) & 1));
            __builtin_amdgcn_sched_barrier(0);
        }
        // tile kt + 1 goes to the other LDS buffer
        lds_store(cur ^ 1, stage[slot]);
        // (a real move, pinned here: left to the compiler the copy drifts to the loop header and
        // then waits for loads that are still in flight)
#pragma unroll
        for (int j = 0; j < WN; j++) {
            if constexpr (D > 1) asm volatile("v_mov_b32 %0, %1" : "=v"(wcur[j]) : "v"(wq[slot][j]));
            else wcur[j] = wq[slot][j];
        }
        __syncthreads();
    };
    // enter the loop with nothing outstanding: the conditional loads above would otherwise make the
    // compiler wait for every load at each use inside the loop
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    int kt = 0;
    for (; kt + D <= KT; kt += D) {
        body(kt, std::integral_constant<int, 0>{});
        if constexpr (D > 1) body(kt + 1, std::integral_constant<int, 1>{});
        if constexpr (D > 2) body(kt + 2, std::integral_constant<int, 2>{});
    }
    if constexpr (D > 1) {
        if (kt < KT) body(kt++, std::integral_constant<int, 0>{});
    }
    if constexpr (D > 2) {
        if (kt < KT) body(kt++, std::integral_constant<int, 1>{});
    }

    // the k-loop is over: its LDS buffers become the epilogue's transpose slabs
    constexpr int kEP = 16 * WN + 4;
    static_assert(WGM * WGN * 16 * kEP * 4 <= 2 * BM * kPitch * 2, "epilogue slab does not fit the LDS buffer");
    write_tile<WM, WN>(reinterpret_cast<float *>(&As[0][0]) + wv * 16 * kEP, acc, cc, lane, m0 + (int64_t)wm * WM * 16,
                       nw0, M, N, ep);
}

// ---- the tile kernel with direct-to-LDS activation loads ----------------------------------------------
// Same tiling and arithmetic as tile_kernel; the activation tiles go global -> LDS without passing
// through registers (global_load_lds_dwordx4). That removes the staging registers and the LDS store
// instructions. The load writes lane l of a wavefront to byte 16 l of its destination, which is
// exactly "row tid / 8, position tid % 8" of the 128-byte rows; the XOR swizzle is applied on the
// global side (the thread at position p of row r fetches chunk p ^ (r % 8)).
// A pass multiplies P k-tiles out of one half of a ring of 2 P buffers while the next P tiles (and
// their weight dwords) are on their way into the other half. The compiler does not order these loads
// against the operand reads: each pass starts with a hand-written s_waitcnt vmcnt(0) -- everything the
// previous pass issued has landed -- followed by the pass's one barrier.
// 16 bytes per lane from global memory straight into LDS (the host pass does not know the builtin).
__device__ __forceinline__ void load_to_lds(const void *src, unsigned char *dst) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef __attribute__((address_space(3))) void *lds_ptr;
    __builtin_amdgcn_global_load_lds(src, (lds_ptr)dst, 16, 0, 0);
#endif
}

template <int WM, int WN, int WGM, int WGN, int P, class Loader, class Ep>
__global__ __launch_bounds__(64 * WGM * WGN, WGM * WGN > 4 ? 1 : 2) void tile_dma_kernel(Loader ld, const uint32_t *__restrict__ native,
                                                                  int64_t M, int64_t K, int64_t N, int64_t Kb,
                                                                  int64_t Nb, Ep ep, int tiles_m, int tiles_n) {
    // BL: rows per tile as loaded -- BM rounded up to whole chunk rounds of the workgroup (a 112-row tile of four
    // wavefronts is loaded as 128 rows: the 16 extra rows are the next tile's, fetched and never read)
    constexpr int T = 64 * WGM * WGN, BM = 16 * WM * WGM, BN = 16 * WN * WGN, BL = (BM * 8 + T - 1) / T * T / 8;
    constexpr int CH = BL * 8 / T, S = 2 * P;
    constexpr int kTileBytes = BL * kPitch * 2;
    static_assert(P >= 1 && P <= 2, "geometry");
    __shared__ __attribute__((aligned(16))) _Float16 As[S][BL * kPitch];

    int id = blockIdx.x;
    const int G = tiles_m * tiles_n;
    if ((G & 7) == 0) id = (id & 7) * (G >> 3) + (id >> 3);
    const int tm = id / tiles_n, tn = id % tiles_n;
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

    const int tid = threadIdx.x, lane = tid & 63, wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wv / WGN, wn = wv % WGN;
    const int r16 = lane & 15, g = lane >> 4;

    typename Loader::template State<CH, T> st;
    ld.template init<CH, T>(st, m0, tid, (tid & 7) ^ ((tid >> 3) & 7));

    floatx4 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; i++)
#pragma unroll
        for (int j = 0; j < WN; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    const uint32_t *wptr[WN];
#pragma unroll
    for (int j = 0; j < WN; j++) {
        int64_t nb = n0 / 16 + wn * WN + j;
        if (nb >= Nb) nb = Nb - 1;
        wptr[j] = native + (nb * Kb) * 256 + lane * 4;
    }
    const int KT = (int)((K + kBK - 1) / kBK);

    // Weights: a lane's dwords of a whole native block (4 k-tiles) per n-fragment in one 16-byte load,
    // fetched one block ahead -- one vector-memory instruction per k-tile instead of WN.
    const int KB = (KT + 3) >> 2;
    u32x4 wblk[WN], wnext[WN];
    auto wload = [&](u32x4 (&w)[WN], int kb) {
        if (kb >= KB) kb = KB - 1;
#pragma unroll
        for (int j = 0; j < WN; j++) w[j] = *reinterpret_cast<const u32x4 *>(wptr[j] + (int64_t)kb * 256);
    };
    // tile `kn` -> ring buffer `slot`; the loader's state moves on to the next tile (tiles past K, which
    // the last pass prefetches and nobody multiplies, read whatever the loader substitutes)
    unsigned char *const lds0 = reinterpret_cast<unsigned char *>(&As[0][0]) + wv * 1024;
    BufferResource rsrc;
    if constexpr (Loader::kBuffer) rsrc = make_buffer_resource(ld.x, ld.bytes());
    auto fill = [&](int kn, int slot) {
        unsigned char *dst = lds0 + slot * kTileBytes;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            if constexpr (Loader::kBuffer) buffer_to_lds(rsrc, ld.template offset<CH, T>(st, i), dst + i * (T * 16));
            else load_to_lds(ld.template addr<CH, T>(st, (int64_t)kn * kBK, i), dst + i * (T * 16));
        }
        ld.template advance<CH, T>(st);
    };

    // the first tiles are requested before anything else waits on memory
#pragma unroll
    for (int i = 0; i < P; i++) fill(i, i);
    wload(wblk, 0);
    const int64_t nw0 = n0 + (int64_t)wn * WN * 16;
    ColumnConstants cc;
    load_scale_bias<WN>(ep, lane, nw0, N, cc);
    __builtin_amdgcn_sched_barrier(0);

    const int arow = (wm * WM * 16 + r16) * kPitch;
    auto swz = [&](int i, int s) { return i * 16 * kPitch + (((4 * s + g) ^ (r16 & 7)) * 8); };
    // one k-tile out of ring buffer `slot`: operand reads four ahead of the MFMAs that use them
    auto multiply = [&](int slot, const uint32_t (&w)[WN]) {
        const _Float16 *abase = &As[0][0] + slot * (BL * kPitch) + arow;
        constexpr int NQ = 2 * WM, kAhead = NQ < 4 ? NQ : 4;
        half8 a[NQ];
        half8 bfr[2][WN];
#pragma unroll
        for (int q = 0; q < kAhead; q++) a[q] = *reinterpret_cast<const half8 *>(abase + swz(q >> 1, q & 1));
#pragma unroll
        for (int j = 0; j < WN; j++) bfr[0][j] = decode_step(w[j], 0);
#pragma unroll
        for (int j = 0; j < WN; j++) bfr[1][j] = decode_step(w[j], 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int q = 0; q < NQ; q++) {
#pragma unroll
            for (int j = 0; j < WN; j++) acc[q >> 1][j] = mfma16(a[q], bfr[q & 1][j], acc[q >> 1][j]);
            if (q + kAhead < NQ)
                a[q + kAhead] = *reinterpret_cast<const half8 *>(abase + swz((q + kAhead) >> 1, (q + kAhead) & 1));
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    int half = 0;                                    // which half of the ring is being multiplied
    for (int kb = 0; kb < KB; kb++) {
#pragma unroll
        for (int q = 0; q < 4; q += P) {             // the passes over this block's k-tiles
            const int kt = kb * 4 + q;
            if (kt < KT) {
                __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this thread's part of tiles kt .. kt + P - 1 is in LDS
                __syncthreads();                      // ... and everybody's; the other half of the ring is free
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < P; i++) fill(kt + P + i, (half ^ 1) * P + i);
                if (q == 0) wload(wnext, kb + 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < P; i++)
                    if (i == 0 || kt + i < KT) {
                        uint32_t w[WN];
#pragma unroll
                        for (int j = 0; j < WN; j++) w[j] = wblk[j][q + i];
                        multiply(half * P + i, w);
                    }
                half ^= 1;
            }
        }
#pragma unroll
        for (int j = 0; j < WN; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) asm volatile("v_mov_b32 %0, %1" : "=v"(wblk[j][e]) : "v"(wnext[j][e]));
    }
    // drain the prefetches past K before the buffers are reused as transpose slabs
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();

    constexpr int kEP = 16 * WN + 4;
    static_assert(WGM * WGN * 16 * kEP * 4 <= S * kTileBytes, "epilogue slab does not fit the LDS buffer");
    write_tile<WM, WN>(reinterpret_cast<float *>(&As[0][0]) + wv * 16 * kEP, acc, cc, lane, m0 + (int64_t)wm * WM * 16,
                       nw0, M, N, ep);
}

// ---- one workgroup per CU: everything a wavefront does besides MFMAs goes between its MFMAs -----------------
// With a single wavefront per SIMD nothing covers what the wavefront itself does not overlap. Measured with
// the cycle counter on a 128 x 256 tile (per 64-wide k-tile and wavefront: 64 MFMAs = 1 024 cycles): the
// expansion of the weight words costs 217 cycles when it sits in front of the MFMAs, issuing the tile's loads
// 155 (a wavefront-wide 16-byte load occupies the issue slot for ~30 cycles, in a burst or not), a barrier
// with its waits ~250. So here:
//   * the operands of a k-tile's second 32-wide step are expanded between the MFMA groups of its first step,
//     and the next tile's first-step operands between the groups of the second (VALU work issues while the
//     matrix pipe is busy): the MFMA order is step-major, all row fragments of step 0, then all of step 1;
//   * the loads -- the tile chunks of the pass two ahead and, once per weight block, the next block's
//     words -- are issued one at a time between MFMA groups;
//   * a pass is two k-tiles (one barrier per 128 reduction indices) and the ring holds three passes: what pass
//     p requests has all of pass p + 1 to land in. The wait at the start of a pass leaves exactly the previous
//     pass's loads outstanding (s_waitcnt vmcnt(n), n from the issue order: loads return in order).
// Registers: up to 512 per lane at this occupancy (the accumulators may live in AGPRs). Needs a buffer loader
// (exact wait counts, see DenseBuffer).
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N_, class F>
__device__ __forceinline__ void static_for(F &&f) {   // f(integral_constant<int, 0>) ... f(integral_constant<int, N_ - 1>)
    static_for_impl(f, std::make_integer_sequence<int, N_>{});
}

template <int N_>
__device__ __forceinline__ void wait_vmcnt() {   // s_waitcnt vmcnt(N_), the other counters left alone
    static_assert(N_ >= 0 && N_ < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N_ & 15) | ((N_ >> 4) << 14));
}

template <int WM, int WN, int WGM, int WGN, int P, class Loader, class Ep>
__global__ __launch_bounds__(64 * WGM * WGN, 1) void tile_solo_kernel(Loader ld, const uint32_t *__restrict__ native,
                                                                   int64_t M, int64_t K, int64_t N, int64_t Kb,
                                                                   int64_t Nb, Ep ep, int tiles_m, int tiles_n) {
    constexpr int WG = WGM * WGN, T = 64 * WG, BM = 16 * WM * WGM, BN = 16 * WN * WGN, CH = BM * 8 / T;
    constexpr int kTileBytes = BM * kPitch * 2, kRing = 3;                 // passes in the ring, P tiles each
    static_assert(BM * 8 % T == 0 && WM >= WN && (P == 1 || P == 2) && Loader::kBuffer, "geometry");
    extern __shared__ __attribute__((aligned(16))) unsigned char ring_bytes[];

    int id = blockIdx.x;
    const int G = tiles_m * tiles_n;
    if ((G & 7) == 0) id = (id & 7) * (G >> 3) + (id >> 3);
    const int tm = id / tiles_n, tn = id % tiles_n;
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

    const int tid = threadIdx.x, lane = tid & 63, wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wv / WGN, wn = wv % WGN;
    const int r16 = lane & 15, g = lane >> 4;

    typename Loader::template State<CH, T> st;
    ld.template init<CH, T>(st, m0, tid, (tid & 7) ^ ((tid >> 3) & 7));

    floatx4 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; i++)
#pragma unroll
        for (int j = 0; j < WN; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    const uint32_t *wptr[WN];
#pragma unroll
    for (int j = 0; j < WN; j++) {
        int64_t nb = n0 / 16 + wn * WN + j;
        if (nb >= Nb) nb = Nb - 1;
        wptr[j] = native + (nb * Kb) * 256 + lane * 4;
    }
    const int KT = (int)((K + kBK - 1) / kBK), KB = (KT + 3) >> 2, KBfull = KT >> 2;
    u32x4 wblk[WN], wnext[WN];

    unsigned char *const lds0 = ring_bytes + wv * 1024;
    const BufferResource rsrc = make_buffer_resource(ld.x, ld.bytes());
    auto chunk = [&](int tslot, int i) {   // chunk i of the loader's current tile -> tile slot of the ring
        buffer_to_lds(rsrc, ld.template offset<CH, T>(st, i), lds0 + tslot * kTileBytes + i * (T * 16));
    };

    // the first two passes and the first weight block, before anything waits on memory
#pragma unroll
    for (int t = 0; t < (kRing - 1) * P; t++) {
#pragma unroll
        for (int i = 0; i < CH; i++) chunk(t, i);
        ld.template advance<CH, T>(st);
    }
#pragma unroll
    for (int j = 0; j < WN; j++) wblk[j] = *reinterpret_cast<const u32x4 *>(wptr[j]);
    const int64_t nw0 = n0 + (int64_t)wn * WN * 16;
    ColumnConstants cc;
    load_scale_bias<WN>(ep, lane, nw0, N, cc);
    __builtin_amdgcn_sched_barrier(0);

    const int arow = (wm * WM * 16 + r16) * kPitch;
    auto swz = [&](int i, int s) { return i * 16 * kPitch + (((4 * s + g) ^ (r16 & 7)) * 8); };
    constexpr int NQ = 2 * WM, kAhead = 4;
    half8 b0[2][WN], b1[WN];        // expanded operands: step 0 of the tiles of even / odd parity, step 1

    // One k-tile out of tile slot `tslot`, MFMA group p = step p / WM, row fragment p % WM. Its step-0 operands
    // are in b0[PAR]; its step-1 operands are expanded from `w` during step 0, the next tile's step-0 operands
    // from `wn` during step 1, and after group p `between(p)` may issue one load.
    auto multiply = [&](int tslot, auto par, const uint32_t (&w)[WN], const uint32_t (&wn_)[WN], auto between) {
        constexpr int PAR = decltype(par)::value;
        const _Float16 *abase = reinterpret_cast<const _Float16 *>(ring_bytes) + tslot * (BM * kPitch) + arow;
        half8 a[NQ];
#pragma unroll
        for (int q = 0; q < kAhead; q++) a[q] = *reinterpret_cast<const half8 *>(abase + swz(q % WM, q / WM));
        __builtin_amdgcn_sched_barrier(0);
        static_for<NQ>([&](auto qc) {
                constexpr int Q = decltype(qc)::value, fi = Q % WM, fs = Q / WM;
#pragma unroll
                for (int j = 0; j < WN; j++) acc[fi][j] = mfma16(a[Q], fs == 0 ? b0[PAR][j] : b1[j], acc[fi][j]);
                if constexpr (Q + kAhead < NQ)
                    a[Q + kAhead] = *reinterpret_cast<const half8 *>(abase + swz((Q + kAhead) % WM, (Q + kAhead) / WM));
                if constexpr (fs == 0 && fi < WN) b1[fi] = decode_step(w[fi], 1);
                if constexpr (fs == 1 && fi < WN) b0[PAR ^ 1][fi] = decode_step(wn_[fi], 0);
                between(std::integral_constant<int, Q>{});
                // issue order inside the group: two VALU operations behind every MFMA (they issue while the
                // matrix pipe is busy; in one block behind the MFMAs they would delay the next group)
#pragma unroll
                for (int j = 0; j < WN; j++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);       // MFMA
                    __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);       // VALU
                }
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);           // DS read
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);           // VMEM read
                __builtin_amdgcn_sched_barrier(0);
        });
    };

    // everything the prologue asked for has landed: the counted waits start from nothing outstanding
    __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
    for (int j = 0; j < WN; j++) b0[0][j] = decode_step(wblk[j][0], 0);
    int cur = 0;                                     // ring slot of the pass being multiplied
    // Pass H of weight block kb: tiles 4 kb + H P .. + P - 1. It requests the tiles of the pass two ahead (ring
    // slot cur + 2) and, when H == 0, the next weight block.
    auto pass = [&](int kb, auto hc) {
        constexpr int H = decltype(hc)::value;
        // this thread's chunks of the pass are in LDS: all it has asked for except what the last pass issued
        wait_vmcnt<P * CH + ((H + 4 / P - 1) % (4 / P) == 0 ? WN : 0)>();
        __builtin_amdgcn_s_waitcnt(0xC07F);           // (lgkmcnt(0): and its operand reads of the last pass are done)
        __builtin_amdgcn_s_barrier();                 // ... and everybody's; the slot multiplied last is free
        __builtin_amdgcn_sched_barrier(0);
        const int ahead = cur == 0 ? kRing - 1 : cur - 1;     // = (cur + kRing - 1) % kRing
        static_for<P>([&](auto ec) {
                constexpr int E = decltype(ec)::value;
                constexpr int q = P * H + E;          // position of the tile in its weight block
                constexpr int kItems = CH + ((H == 0 && E == 0) ? WN : 0);
                uint32_t w[WN], wn_[WN];
#pragma unroll
                for (int j = 0; j < WN; j++) {
                    w[j] = wblk[j][q];
                    wn_[j] = q < 3 ? wblk[j][q < 3 ? q + 1 : 0] : wnext[j][0];
                }
                multiply(cur * P + E, std::integral_constant<int, q & 1>{}, w, wn_, [&](auto gc) {
                    constexpr int grp = decltype(gc)::value;
#pragma unroll
                    for (int t = 0; t < kItems; t++)      // item t goes out after group t NQ / kItems
                        if (t * NQ / kItems == grp) {
                            if (t < CH) chunk(ahead * P + E, t);
                            else {
                                int nb = kb + 1;
                                if (nb >= KB) nb = KB - 1;
                                wnext[t - CH] = *reinterpret_cast<const u32x4 *>(wptr[t - CH] + (int64_t)nb * 256);
                            }
                        }
                });
                ld.template advance<CH, T>(st);
        });
        cur = cur == kRing - 1 ? 0 : cur + 1;
    };
    for (int kb = 0; kb < KBfull; kb++) {
        pass(kb, std::integral_constant<int, 0>{});
        pass(kb, std::integral_constant<int, 1>{});
        if constexpr (P == 1) {
            pass(kb, std::integral_constant<int, 2>{});
            pass(kb, std::integral_constant<int, 3>{});
        }
#pragma unroll
        for (int j = 0; j < WN; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) asm volatile("v_mov_b32 %0, %1" : "=v"(wblk[j][e]) : "v"(wnext[j][e]));
    }
    // The last, partial weight block (1 .. 3 tiles): plain tiles, operands expanded in front of the MFMAs. The
    // loop has requested the first (kRing - 1) P of them; a further one is fetched here, into the slot of the
    // pass multiplied last.
    for (int kt = KBfull * 4; kt < KT; kt++) {
        const int e = kt & 3;
        int ps = cur + e / P;
        if (ps >= kRing) ps -= kRing;
        const int tslot = ps * P + e % P;
        if (e >= (kRing - 1) * P) {
            __syncthreads();
#pragma unroll
            for (int i = 0; i < CH; i++) chunk(tslot, i);
            ld.template advance<CH, T>(st);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        const _Float16 *abase = reinterpret_cast<const _Float16 *>(ring_bytes) + tslot * (BM * kPitch) + arow;
        half8 bfr[2][WN];
#pragma unroll
        for (int j = 0; j < WN; j++) {
            const uint32_t w = e == 0 ? wblk[j][0] : e == 1 ? wblk[j][1] : wblk[j][2];
            bfr[0][j] = decode_step(w, 0);
            bfr[1][j] = decode_step(w, 1);
        }
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            const half8 a = *reinterpret_cast<const half8 *>(abase + swz(q >> 1, q & 1));
#pragma unroll
            for (int j = 0; j < WN; j++) acc[q >> 1][j] = mfma16(a, bfr[q & 1][j], acc[q >> 1][j]);
        }
    }
    // drain the requests past K before the ring is reused as transpose slabs
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    constexpr int kEP = 16 * WN + 4;
    static_assert(WG * 16 * kEP * 4 <= kRing * P * kTileBytes, "epilogue slab does not fit the ring");
    write_tile<WM, WN>(reinterpret_cast<float *>(ring_bytes) + wv * 16 * kEP, acc, cc, lane, m0 + (int64_t)wm * WM * 16,
                       nw0, M, N, ep);
}

template <int WM, int WN, int WGM, int WGN, int P, class Loader, class Ep>
int launch_tile_solo(const Loader &ld, const void *native, int64_t M, int64_t K, int64_t N, const Ep &ep,
                     void *stream) {
    constexpr int BM = 16 * WM * WGM, BN = 16 * WN * WGN, kLds = 3 * P * BM * kPitch * 2;
    const int64_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    if (tm * tn > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    auto kernel = tile_solo_kernel<WM, WN, WGM, WGN, P, Loader, Ep>;
    if constexpr (kLds > 64 * 1024) {
        if (int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), kLds)) return st;
    }
    hipLaunchKernelGGL(kernel, dim3((uint32_t)(tm * tn)), dim3(64 * WGM * WGN), kLds, as_stream(stream), ld,
                       static_cast<const uint32_t *>(native), M, K, N, native_blocks_k(K), native_blocks_n(N), ep, (int)tm,
                       (int)tn);
    return check_launch();
}

template <int WM, int WN, int WGM, int WGN, int P, class Loader, class Ep>
int launch_tile_dma(const Loader &ld, const void *native, int64_t M, int64_t K, int64_t N, const Ep &ep,
                    void *stream) {
    constexpr int BM = 16 * WM * WGM, BN = 16 * WN * WGN;
    const int64_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    if (tm * tn > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL((tile_dma_kernel<WM, WN, WGM, WGN, P, Loader, Ep>), dim3((uint32_t)(tm * tn)), dim3(64 * WGM * WGN), 0,
                       as_stream(stream), ld, static_cast<const uint32_t *>(native), M, K, N, native_blocks_k(K),
                       native_blocks_n(N), ep, (int)tm, (int)tn);
    return check_launch();
}

template <int WM, int WN, int WGM, int WGN, int D, class Loader, class Ep>
int launch_tile(const Loader &ld, const void *native, int64_t M, int64_t K, int64_t N, const Ep &ep,
                void *stream) {
    constexpr int BM = 16 * WM * WGM, BN = 16 * WN * WGN;
    const int64_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    if (tm * tn > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL((tile_kernel<WM, WN, WGM, WGN, D, Loader, Ep>), dim3((uint32_t)(tm * tn)), dim3(64 * WGM * WGN), 0,
                       as_stream(stream), ld, static_cast<const uint32_t *>(native), M, K, N, native_blocks_k(K),
                       native_blocks_n(N), ep, (int)tm, (int)tn);
    return check_launch();
}

// Tile choice, from a sweep over M x K x N (4096^2 weights at M = 768 .. 4096 and the ResNet-18 layer
// shapes): 128 x 256 once it gives 1.5 workgroups per CU, 128 x 128 down to one per CU, else
// 64 x 64. Larger tiles (256 x 256, 256 x 128) and 128 x 64 never won.
// How a tile is dealt to its wavefronts matters as much: every wavefront expands the weights of its own
// columns (2 VALU operations per operand register), so the small tiles give each wavefront all rows and a
// slice of the columns -- 64 x 32 of a 64 x 64 tile, 128 x 32 of a 128 x 128 tile -- instead of a square:
// half the expansions per MFMA for twice the (cheap) operand reads from LDS. 3 x 3 convolution 64 -> 64 at
// 56 x 56, batch 64: 31.4 -> 26.1 us (counters had shown 1500 VALU instructions per wavefront next to 144
// MFMAs). Dense 128 x 128 tiles with two workgroups per CU are the exception (M = 2048 at K = N = 4096:
// 51 -> 57 us, the LDS reads then cost more than the expansions save) and keep the square split.
template <class Loader>
Loader with_divisors(Loader ld) {
    ld.by_wo = FastDiv((uint32_t)ld.Wo);
    ld.by_ho = FastDiv((uint32_t)ld.Ho);
    return ld;
}

template <class Loader, class Ep>
int dispatch_tile(const Loader &ld, const void *native, int64_t M, int64_t K, int64_t N, const Ep &ep,
                  void *stream) {
    auto wgs = [&](int bm, int bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    if constexpr (Loader::kDirect) {
        // Tiles per pass: two (half the barriers, a whole extra tile of time for the loads to land) pay
        // on long reductions when the doubled ring does not cost residency -- the 128 x 256 tile, which
        // runs two workgroups per CU either way, and 128 x 128 when there is at most one per CU
        // (measured at K = 4096: M = 4096 100 -> 93.5 us, M = 1024 52.5 -> 46.6, but M = 2048, two
        // 128 x 128 tiles per CU, 59 -> 64; every 64 x 64 case loses).
        const bool two = K >= 2048;
        // A chip full of 128 x 512 tiles, eight wavefronts of 128 rows x 64 channels (one workgroup per CU): every
        // activation row is read N / 512 times instead of N / 256 (M = K = N = 4096: 98.9 -> 93.8 us, M = 8192
        // 196 -> 188, 8192^3 709 -> 693; with ragged tiles, N = 11008, it loses 1 %)
        if (!Loader::kConv && two && N % 512 == 0 && wgs(128, 512) >= 256)
            return launch_tile_dma<8, 4, 1, 8, 2>(ld, native, M, K, N, ep, stream);
        if (N > 128 && wgs(128, 256) >= 384)
            return two ? launch_tile_dma<8, 4, 1, 4, 2>(ld, native, M, K, N, ep, stream)
                       : launch_tile_dma<8, 4, 1, 4, 1>(ld, native, M, K, N, ep, stream);
        // Convolutions whose 128 x 128 tiles come to between one and two per CU (all resident at once, two workgroups
        // per CU): 112-row tiles, while those are all resident too, leave every workgroup an eighth less to do for the
        // same number of rounds -- 128 -> 128 channels on 28 x 28 at batch 64 (392 tiles -> 448) 24.2 -> 22.7 us, the
        // strided 64 -> 128 before it 16.9 -> 16.5; 96-row tiles (523) would need a third round.
        if constexpr (std::is_same<Loader, ConvLoader64>::value) {
            if (N % 128 == 0 && wgs(128, 128) > 256 && wgs(112, 128) <= 512)
                return launch_tile_dma<7, 2, 1, 4, 1>(ld, native, M, K, N, ep, stream);
        }
        if (N > 64 && wgs(128, 128) >= 256) {
            const bool one = wgs(128, 128) <= 256;      // at most one workgroup per CU
            if (Loader::kConv || one)
                return two && one ? launch_tile_dma<8, 2, 1, 4, 2>(ld, native, M, K, N, ep, stream)
                                  : launch_tile_dma<8, 2, 1, 4, 1>(ld, native, M, K, N, ep, stream);
            return launch_tile_dma<4, 4, 2, 2, 1>(ld, native, M, K, N, ep, stream);
        }
        return launch_tile_dma<4, 2, 1, 2, 1>(ld, native, M, K, N, ep, stream);
    } else {
        // Register prefetch depth: the big tile has a k-tile of work long enough to cover a trip to L2
        // (and no registers to spare); the smaller ones fetch two tiles ahead once the reduction is
        // long enough to pay for the extra tile in the prologue.
        const bool deep = K >= 16 * kBK;
        if (N > 128 && wgs(128, 256) >= 384) return launch_tile<8, 4, 1, 4, 1>(ld, native, M, K, N, ep, stream);
        if (N > 64 && wgs(128, 128) >= 256)
            return deep ? launch_tile<4, 4, 2, 2, 2>(ld, native, M, K, N, ep, stream)
                        : launch_tile<4, 4, 2, 2, 1>(ld, native, M, K, N, ep, stream);
        return deep ? launch_tile<4, 2, 1, 2, 2>(ld, native, M, K, N, ep, stream)
                    : launch_tile<4, 2, 1, 2, 1>(ld, native, M, K, N, ep, stream);
    }
}

}  // namespace

template <class Ep>
static int gemm_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const Ep &ep, void *stream) {
    // Dense rows through a buffer resource: the kernel that puts its expansion and loads between the MFMAs.
    //  * A chip full of 128 x 512 tiles (N a multiple of 512), eight wavefronts of 128 rows x 64 channels, one k-tile
    //    per pass: every activation row is read N / 512 times from L2. Against 128 x 256 tiles with two workgroups
    //    per CU: M = K = N = 4096 98.9 -> 93.0 us, M = 8192 196 -> 186, M = 6144 171 -> 163.5, 4096 x 8192 x 8192
    //    349 -> 340 (the same tiles in tile_dma_kernel: 93.8, 188, 171, 349).
    //  * 192 .. 256 tiles of 64 x 512, eight wavefronts: M = 2048 53.0 -> 50.7 us, M = 1536 47.1 -> 43.9.
    //  * A few hundred 64 x 256 tiles, four wavefronts, one or two workgroups per CU: M = 768 32.0 -> 29.4 us,
    //    M = 1024 36.1 -> 30.2, M = 3072 84.8 -> 75.9; from 1024 such tiles on the 128 x 256 tiles of
    //    tile_dma_kernel, two workgroups per CU, win (N = 11008 at M = 4096).
    if ((K % kBK == 0) && aligned16(x) && K >= 1024 && N > 128 && M * K * 2 < (int64_t)kPastTheEnd - 16) {
        const DenseBuffer ld{static_cast<const _Float16 *>(x), M, K};
        if (N % 512 == 0) {
            const int64_t t128 = ((M + 127) / 128) * (N / 512), t64 = ((M + 63) / 64) * (N / 512);
            if (K >= 2048 && t128 >= 256) return launch_tile_solo<8, 4, 1, 8, 1>(ld, native, M, K, N, ep, stream);
            if (t64 >= 192 && t64 <= 256) return launch_tile_solo<4, 4, 1, 8, 2>(ld, native, M, K, N, ep, stream);
        }
        const int64_t t64 = ((M + 63) / 64) * ((N + 255) / 256);
        if (t64 >= 192 && t64 < 1024) return launch_tile_solo<4, 4, 1, 4, 2>(ld, native, M, K, N, ep, stream);
    }
    if ((K % kBK == 0) && aligned16(x))
        return dispatch_tile(DenseDirect{static_cast<const _Float16 *>(x), M, K}, native, M, K, N, ep, stream);
    if constexpr (decltype(ep.map)::kPairs) return TMQ_ERR_UNSUPPORTED;      // row pairs are made aligned
    else if (K % 8 == 0 && aligned16(x))
        return dispatch_tile(DenseLoader<true>{static_cast<const _Float16 *>(x), M, K}, native, M, K, N, ep, stream);
    else return dispatch_tile(DenseLoader<false>{static_cast<const _Float16 *>(x), M, K}, native, M, K, N, ep, stream);
}

int launch_gemm_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                      const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream) {
    return gemm_dense(x, M, K, native, N, Epilogue{scale, bias, residual, y, relu, y_f16}, stream);
}

// The same on M16 fp16 rows that are the hi / lo terms of rows_out fp32 rows in groups of eight (PairMap).
int launch_gemm_dense_pairs(const void *x16, int64_t M16, int64_t K, const void *native, int64_t N, const float *scale,
                            const float *bias, const void *residual, int relu, void *y, int y_f16, int64_t rows_out,
                            const float *group_scale, void *stream) {
    return gemm_dense(x16, M16, K, native, N, PairEpilogue{scale, bias, residual, y, relu, y_f16, PairMap{rows_out, group_scale}}, stream);
}

// Adds the slices of a reduction that was cut across workgroups in slice order (deterministic) and applies the
// epilogue. partial holds `slices` fp32 matrices [M][N] with the weight unit already divided out.
namespace {
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ partial, int slices, int64_t M, int64_t N,
                                                            Epilogue ep) {
    const int64_t MN = M * N;
    const bool vec = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(ep.y) | reinterpret_cast<uintptr_t>(ep.residual) |
                                       reinterpret_cast<uintptr_t>(ep.scale) | reinterpret_cast<uintptr_t>(ep.bias)) & 15u) == 0;
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= MN) return;
    if (vec) {
        floatx4 v = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(partial + i));
        for (int s = 1; s < slices; s++) v += __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(partial + s * MN + i));
        const int64_t n = i % N;
        if (ep.scale) v *= *reinterpret_cast<const floatx4 *>(ep.scale + n);
        if (ep.bias) v += *reinterpret_cast<const floatx4 *>(ep.bias + n);
        if (ep.residual) {
            if (ep.y_f16) {
                const half4 r = *reinterpret_cast<const half4 *>(static_cast<const _Float16 *>(ep.residual) + i);
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] += (float)r[e];
            } else {
                v += *reinterpret_cast<const floatx4 *>(static_cast<const float *>(ep.residual) + i);
            }
        }
        if (ep.relu) {
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = v[e] < 0.f ? 0.f : v[e];
        }
        if (ep.y_f16) {
            half4 h;
#pragma unroll
            for (int e = 0; e < 4; e++) h[e] = (_Float16)v[e];
            *reinterpret_cast<half4 *>(static_cast<_Float16 *>(ep.y) + i) = h;
        } else {
            *reinterpret_cast<floatx4 *>(static_cast<float *>(ep.y) + i) = v;
        }
        return;
    }
    for (int e = 0; e < 4 && i + e < MN; e++) {
        const int64_t o = i + e, n = o % N;
        float f = partial[o];
        for (int s = 1; s < slices; s++) f += partial[s * MN + o];
        if (ep.scale) f *= ep.scale[n];
        if (ep.bias) f += ep.bias[n];
        if (ep.residual) f += ep.y_f16 ? (float)static_cast<const _Float16 *>(ep.residual)[o] : static_cast<const float *>(ep.residual)[o];
        if (ep.relu) f = f < 0.f ? 0.f : f;
        if (ep.y_f16) static_cast<_Float16 *>(ep.y)[o] = (_Float16)f;
        else static_cast<float *>(ep.y)[o] = f;
    }
}
}  // namespace

int launch_splitk_reduce(const float *partial, int slices, int64_t M, int64_t N, const Epilogue &ep, void *stream) {
    const int64_t groups = (M * N + 1023) / 1024;
    if (groups > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((uint32_t)groups), dim3(256), 0, as_stream(stream), partial, slices, M, N, ep);
    return check_launch();
}

// rows.hip: 17 .. 32 rows over a very large layer, the reduction cut across workgroups
int rows_split_slices(const void *x, int64_t M, int64_t K, int64_t N);
int launch_rows_split(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const Epilogue &ep, float *partial,
                      int slices, void *stream);

// Two to sixteen fp32 rows over whole weight blocks: split once into fp16 row pairs (prescale.hip), then one pass of
// the fp16 weight-stream kernel over twice the rows (mid.hip; two passes of about half the rows each from nine rows)
// -- against the kernel that splits every block's activations on the fly in each workgroup: 8192^2, 4 rows
// 17.4 -> 10.8 us, 8 rows 25.5 -> 11.7 us; and on short reductions against a prescale launch in front of the skinny
// kernels: K = 1024, N = 4096, 4 rows 7.9 -> 6.0 us, 8 rows 9.5 -> 6.4, 16 rows 12.3 -> 9.4.
int launch_split_rows(const float *x, int64_t M, int64_t K, int64_t Kp, int64_t group, void *x16, float *row_scale, void *stream);
inline int64_t padded_blocks(int64_t K) { return (K + kKB - 1) / kKB * kKB; }   // the weight stream wants whole 256-index blocks
int launch_stream_pairs(const void *x16, int64_t M, int64_t K, const void *native, int64_t N, const float *row_scale,
                        const float *scale, const float *bias, const void *residual, int relu, void *y, int y_f16,
                        void *stream);
bool gemv8_dense32_ok(const void *x, int64_t M, int64_t K, int64_t N);
inline bool row_pairs_ok(const void *x, int64_t M, int64_t K, int64_t N) {
    if (gemv8_dense32_ok(x, M, K, N)) return false;               // two rows over a small layer: one launch (gemv8.hip)
    // (a ragged length is written zero-padded to whole blocks, rows of any alignment are read element-wise)
    return M >= 1 && M <= 16 && K >= 1 && 2 * M * padded_blocks(K) < (int64_t)0x7FFFFFFF;
}
inline size_t row_pairs_bytes(int64_t M, int64_t K) { return 256 + (size_t)(2 * M * padded_blocks(K)) * sizeof(_Float16); }

// Seventeen fp16 rows or more whose reduction length is no multiple of 64: the kernels with direct global -> LDS
// loads want whole 64-index tiles of 16-byte aligned rows, and the register-staged kernel that takes everything else
// guards every load (K = 4000 against 4096 at M = 1024, N = 4096: 261 us against 35). With a workspace the rows are
// copied once to rows of the next multiple of 64, zeros behind (the native weights are padded with zeros to whole
// 256-index blocks anyway), and take the aligned kernels: 261 -> 39 us, K = 784, M = 128, N = 1024 24.4 -> 6 us.
int launch_pad_rows(const void *x, int64_t M, int64_t K, int64_t Kp, void *out, void *stream);
inline int64_t padded_k(int64_t K) { return (K + 63) / 64 * 64; }
inline bool pad_rows_ok(int64_t M, int64_t K) { return M >= 17 && K % 64 != 0 && M * padded_k(K) < (int64_t)0x7FFFFFFF; }
inline size_t pad_rows_bytes(int64_t M, int64_t K) { return (size_t)(M * padded_k(K)) * sizeof(_Float16); }

// Seventeen fp32 rows or more over K a multiple of 64: one launch splits them into fp16 row pairs in groups of eight,
// every group scaled by a power of two of its own (PairMap); the fp16 kernels then run once over 16 ceil(M / 8) rows
// and their epilogues add each pair and undo the group's scale. Against the kernels that split on the fly, or two
// fp16 passes chained through the residual.
int launch_split_groups(const float *x, int64_t M, int64_t K, int64_t Kp, void *x16, float *group_scale, void *stream);
int launch_mid_dense_pairs(const void *x16, int64_t M16, int64_t K, const void *native, int64_t N, const float *scale,
                           const float *bias, const void *residual, int relu, void *y, int y_f16, int64_t rows_out,
                           const float *group_scale, void *stream);
inline int64_t pair_rows16(int64_t M) { return (M + 7) / 8 * 16; }
inline bool pair_rows_ok(const void *x, int64_t M, int64_t K, int64_t N) {
    (void)x;                                                       // rows of any alignment: the splitter reads them element-wise if it must
    return M >= 17 && K >= 1 && pair_rows16(M) * padded_k(K) < (int64_t)0x7FFFFFFF;
}
// the workspace: the groups' 1 / s (padded to 256 bytes), then the fp16 rows
inline size_t pair_scale_bytes(int64_t M) { return ((size_t)((M + 7) / 8) * sizeof(float) + 255) & ~(size_t)255; }
inline size_t pair_rows_bytes(int64_t M, int64_t K, int64_t N) {
    return pair_scale_bytes(M) + (size_t)(pair_rows16(M) * padded_k(K)) * sizeof(_Float16);
}

}  // namespace tmq

namespace tmq {
namespace {

// The tile kernels behind tmq_ternary_conv2d for an epilogue with consecutive rows (Epilogue) or rows scattered into a
// strided destination (ViewEpilogue).
template <class Ep>
int conv_tiles(const void *x, const tmq_conv_shape *s, int ho, int wo, const void *native, const Ep &ep, void *stream) {
    const int64_t M = (int64_t)s->B * ho * wo, K = (int64_t)s->C * s->ky * s->kx;
    const _Float16 *xp = static_cast<const _Float16 *>(x);
    const bool small = (int64_t)s->B * s->H * s->W * s->C < (int64_t)0x7FFFFFF0 && M < (int64_t)0x7FFFFFFF;   // 32-bit offsets and rows
    // 129 .. 256 output channels over at least 128 tiles of 64 rows: one 64 x 256 tile per workgroup, eight
    // wavefronts of 64 rows x 32 channels -- an im2col tile is then fetched once instead of once per 64 channels
    // (the four such 3 x 3 convolutions of ResNet-18 at batch 64: 18.9 / 25.8 / 23.3 / 23.2 -> 14.4 / 21.4 / 21.3 / 22.0 us;
    // the 1 x 1 downsample beside them, two k-tiles, is faster on the small tiles: 5.4 against 7.9 us)
    if ((s->C % kBK == 0) && s->ky <= 15 && s->kx <= 15 && aligned16(x) && small && s->N > 128 && s->N <= 256 && M >= 128 * 64 && K >= 8 * kBK)
        return launch_tile_solo<4, 2, 1, 8, 1>(with_divisors(ConvLoader64{xp, M, K, s->B, s->C, s->H, s->W, ho, wo, s->ky, s->kx,
                                                                          s->sy, s->sx, s->py, s->px, s->dy, s->dx, {}, {}}),
                                               native, M, K, s->N, ep, stream);
    if ((s->C % kBK == 0) && s->ky <= 15 && s->kx <= 15 && aligned16(x) && small)
        return dispatch_tile(with_divisors(ConvLoader64{xp, M, K, s->B, s->C, s->H, s->W, ho, wo, s->ky, s->kx, s->sy,
                                                        s->sx, s->py, s->px, s->dy, s->dx, {}, {}}), native, M, K, s->N, ep, stream);
    if ((s->C == 8 || s->C == 16 || s->C == 32) && aligned16(x) && small)
        return dispatch_tile(with_divisors(ConvLoaderFewC{xp, M, K, s->B, s->C, s->H, s->W, ho, wo, s->ky, s->kx, s->sy,
                                                          s->sx, s->py, s->px, s->dy, s->dx, {}, {}}), native, M, K, s->N, ep, stream);
    if ((s->C % 8 == 0) && aligned16(x))
        return dispatch_tile(ConvLoader<true>{xp, M, K, s->B, s->C, s->H, s->W, ho, wo, s->ky, s->kx, s->sy, s->sx,
                                              s->py, s->px, s->dy, s->dx}, native, M, K, s->N, ep, stream);
    return dispatch_tile(ConvLoader<false>{xp, M, K, s->B, s->C, s->H, s->W, ho, wo, s->ky, s->kx, s->sy, s->sx, s->py,
                                           s->px, s->dy, s->dx, (s->C % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 7u) == 0) ? 1 : 0},
                         native, M, K, s->N, ep, stream);
}

}  // namespace
}  // namespace tmq

using namespace tmq;

extern "C" {

size_t tmq_ternary_linear_workspace_bytes(int x_dtype, int64_t M, int64_t K, int64_t N) {
    if (M <= 0 || K <= 0 || N <= 0) return 0;
    if (x_dtype == TMQ_F32)
        return row_pairs_ok(nullptr, M, K, N) ? row_pairs_bytes(M, K) : pair_rows_ok(nullptr, M, K, N) ? pair_rows_bytes(M, K, N) : 0;
    if (x_dtype != TMQ_F16) return 0;
    static const _Float16 *const aligned = nullptr;              // the plan assumes 16-byte aligned rows; _ws checks the real pointer
    const int slices = rows_split_slices(aligned, M, K, N);
    if (slices) return (size_t)slices * (size_t)M * (size_t)N * sizeof(float);
    return pad_rows_ok(M, K) ? pad_rows_bytes(M, K) : 0;
}

int tmq_ternary_linear_ws(const void *x, int x_dtype, int64_t M, int64_t K, const void *native, int64_t N,
                          const tmq_epilogue *epilogue, void *y, void *workspace, size_t workspace_bytes, void *stream) {
    if (x && native && y && x_dtype == TMQ_F32 && N > 0 && workspace && aligned16(workspace) && aligned16(native) &&
        row_pairs_ok(x, M, K, N) && workspace_bytes >= row_pairs_bytes(M, K)) {
        tmq_epilogue e = {nullptr, nullptr, nullptr, 0, TMQ_F32};
        if (epilogue) e = *epilogue;
        if (e.y_dtype != TMQ_F16 && e.y_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
        // the rows' 1 / s first (256 bytes), then the 2 M fp16 rows
        float *row_scale = static_cast<float *>(workspace);
        void *x16 = static_cast<unsigned char *>(workspace) + 256;
        // up to eight rows make one pass of sixteen fp16 rows; nine to sixteen go as two groups of about equal size
        const int64_t group = M <= 8 ? M : (M + 1) / 2;
        const int64_t Kp = padded_blocks(K);
        if (int st = launch_split_rows(static_cast<const float *>(x), M, K, Kp, group, x16, row_scale, stream)) return st;
        const size_t out_elt = e.y_dtype == TMQ_F16 ? 2 : 4;
        for (int64_t m0 = 0; m0 < M; m0 += group) {
            const int64_t rows = M - m0 < group ? M - m0 : group;
            const unsigned char *res = static_cast<const unsigned char *>(e.residual);
            const int st = launch_stream_pairs(static_cast<const _Float16 *>(x16) + 2 * m0 * Kp, rows, Kp, native, N, row_scale + m0,
                                               e.scale, e.bias, res ? res + (size_t)(m0 * N) * out_elt : nullptr, e.relu,
                                               static_cast<unsigned char *>(y) + (size_t)(m0 * N) * out_elt,
                                               e.y_dtype == TMQ_F16 ? 1 : 0, stream);
            if (st) return st;
        }
        return TMQ_OK;
    }
    if (x && native && y && x_dtype == TMQ_F32 && N > 0 && workspace && aligned16(workspace) && aligned16(native) &&
        !row_pairs_ok(x, M, K, N) && pair_rows_ok(x, M, K, N) && workspace_bytes >= pair_rows_bytes(M, K, N)) {
        tmq_epilogue e = {nullptr, nullptr, nullptr, 0, TMQ_F32};
        if (epilogue) e = *epilogue;
        if (e.y_dtype != TMQ_F16 && e.y_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
        float *group_scale = static_cast<float *>(workspace);
        void *x16 = static_cast<unsigned char *>(workspace) + pair_scale_bytes(M);
        // (a length that is no multiple of 64: rows of the next multiple, zeros behind -- the native weights are padded
        // with zeros to whole 256-index blocks)
        const int64_t Kp = padded_k(K);
        if (int st = launch_split_groups(static_cast<const float *>(x), M, K, Kp, x16, group_scale, stream)) return st;
        const int64_t M16 = pair_rows16(M);
        const int y_f16 = e.y_dtype == TMQ_F16 ? 1 : 0;
        if (split_reduction_pays(M16, Kp, N))
            return launch_mid_dense_pairs(x16, M16, Kp, native, N, e.scale, e.bias, e.residual, e.relu, y, y_f16, M, group_scale, stream);
        return launch_gemm_dense_pairs(x16, M16, Kp, native, N, e.scale, e.bias, e.residual, e.relu, y, y_f16, M, group_scale, stream);
    }
    if (x && native && y && x_dtype == TMQ_F16 && M > 0 && K > 0 && N > 0 && workspace && aligned16(workspace) && aligned16(native)) {
        const int slices = rows_split_slices(x, M, K, N);
        if (slices && workspace_bytes >= (size_t)slices * (size_t)M * (size_t)N * sizeof(float)) {
            tmq_epilogue e = {nullptr, nullptr, nullptr, 0, TMQ_F32};
            if (epilogue) e = *epilogue;
            if (e.y_dtype != TMQ_F16 && e.y_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
            const Epilogue ep{e.scale, e.bias, e.residual, y, e.relu, e.y_dtype == TMQ_F16 ? 1 : 0};
            return launch_rows_split(x, M, K, native, N, ep, static_cast<float *>(workspace), slices, stream);
        }
        if (!slices && pad_rows_ok(M, K) && workspace_bytes >= pad_rows_bytes(M, K)) {
            if (int st = launch_pad_rows(x, M, K, padded_k(K), workspace, stream)) return st;
            return tmq_ternary_linear(workspace, TMQ_F16, M, padded_k(K), native, N, epilogue, y, stream);
        }
    }
    return tmq_ternary_linear(x, x_dtype, M, K, native, N, epilogue, y, stream);
}

int64_t tmq_selfcheck_fastdiv(uint32_t divisor, const uint32_t *n, int64_t count) {
    if (divisor == 0 || divisor >= 0x80000000u || !n || count < 0) return -1;
    const FastDiv f(divisor);
    int64_t bad = 0;
    for (int64_t i = 0; i < count; i++) {
        const uint32_t q = divisor > 1 ? (uint32_t)(((uint64_t)n[i] * f.mul) >> 32) >> f.shift : n[i];   // = FastDiv::divmod
        if (n[i] >= 0x80000000u || q != n[i] / divisor) bad++;
    }
    return bad;
}

int tmq_conv2d_out_hw(const tmq_conv_shape *s, int32_t *ho, int32_t *wo) {
    if (!s || !ho || !wo || s->sy <= 0 || s->sx <= 0 || s->dy <= 0 || s->dx <= 0 || s->ky <= 0 || s->kx <= 0)
        return TMQ_ERR_INVALID_ARG;
    if (s->py < 0 || s->px < 0 || s->py_end < 0 || s->px_end < 0) return TMQ_ERR_INVALID_ARG;
    const int32_t eh = s->H + s->py + s->py_end - s->dy * (s->ky - 1) - 1;
    const int32_t ew = s->W + s->px + s->px_end - s->dx * (s->kx - 1) - 1;
    *ho = eh < 0 ? 0 : eh / s->sy + 1;
    *wo = ew < 0 ? 0 : ew / s->sx + 1;
    return TMQ_OK;
}

int tmq_ternary_conv2d(const void *x, const tmq_conv_shape *s, const void *native, const tmq_epilogue *epilogue,
                       void *y, void *stream) {
    return tmq_ternary_conv2d_view(x, s, native, epilogue, y, nullptr, stream);
}

int tmq_ternary_conv2d_view(const void *x, const tmq_conv_shape *s, const void *native, const tmq_epilogue *epilogue,
                            void *y, const tmq_output_view *view, void *stream) {
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
    RowMap map;
    if (view) {
        // the kept part of the computed grid must lie inside it; rows are decomposed with 32-bit arithmetic
        if (view->h0 < 0 || view->w0 < 0 || view->h_cnt < 0 || view->w_cnt < 0 || view->h0 + (int64_t)view->h_cnt > ho ||
            view->w0 + (int64_t)view->w_cnt > wo || view->stride_b < 0 || view->stride_h < 0 || view->stride_w < 0)
            return TMQ_ERR_INVALID_ARG;
        if (M >= (int64_t)0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
        if (view->h_cnt == 0 || view->w_cnt == 0) return TMQ_OK;
        map.hw = FastDiv((uint32_t)ho * (uint32_t)wo);
        map.w = FastDiv((uint32_t)wo);
        map.h0 = view->h0; map.w0 = view->w0; map.h_cnt = view->h_cnt; map.w_cnt = view->w_cnt;
        map.sb = view->stride_b; map.sh = view->stride_h; map.sw = view->stride_w;
    }
    const int y_f16 = y_dtype == TMQ_F16 ? 1 : 0;
    // few output tiles: split the reduction inside the workgroup (mid.hip)
    if (mid_conv_ok(x, s) && split_reduction_pays(M, K, s->N))
        return launch_mid_conv(x, s, ho, wo, native, scale, bias, residual, relu, y, y_f16, view ? &map : nullptr, stream);
    if (view) return conv_tiles(x, s, ho, wo, native, ViewEpilogue{scale, bias, residual, y, relu, y_f16, map}, stream);
    return conv_tiles(x, s, ho, wo, native, Epilogue{scale, bias, residual, y, relu, y_f16, {}}, stream);
}

}  // extern "C"
