// Ternary GEMM / implicit-GEMM convolution for outputs too small to fill the chip with big tiles
// (a few hundred 64 x 64 tiles): the reduction is split over the wavefronts of a workgroup.
//
// A workgroup of WAVES wavefronts owns a (16 WM) x (16 WN) output tile; wavefront kg multiplies the
// whole tile over the "pairs" (64 reduction indices each) kg, kg + WAVES, ... and the partial tiles
// are summed through LDS in wavefront order, so the result does not depend on scheduling and needs
// no workspace. Every wavefront runs on its own: there is no workgroup barrier inside the loop, and
// one wavefront expands each weight word for 64 rows (the expansion costs two VALU operations per
// operand register whatever the number of rows).
//
//   * Weights: the dword of the kernel-native layout (mfma.h) a lane needs, straight from global
//     memory (the blocks stay in L1 / L2 between the four dword loads), expanded in two VALU ops
//     per operand register.
//   * Activations: an MFMA operand wants 16 bytes of row (lane % 16) in every lane -- loaded
//     directly, 16 neighbouring lanes would touch 16 different rows and cost the texture path one
//     cache line each. Instead a wavefront fetches whole 128-byte row pieces (8 lanes per row, 8
//     rows per instruction) with global_load_lds_dwordx4 straight into a private LDS window and
//     reads them back in operand order. The load writes lane l to byte 16 l of its destination, so
//     the bank swizzle is applied on the global side: lane (row r, position p) fetches chunk
//     p ^ ((r / 2) % 8) of its row piece; the reader undoes it. Operand reads of 16 rows then fall
//     into 16 different 16-byte bank groups.
//   * Pipeline unit: a "pair" = 64 reduction indices = one dword of every weight block = two MFMA
//     steps. While pair p is multiplied out of one LDS slot, the loads of pair p + 1 fill the
//     other. The window belongs to one wavefront: no workgroup barrier inside the loop.
//   * Rows: a dense row-major matrix, or the im2col view of an NHWC tensor with C % 64 == 0 (a pair
//     is then 64 consecutive channels of one filter tap; taps outside the image and reduction
//     indices past K read a zero chunk instead).
#include "common.h"
#include "mfma.h"
#include <type_traits>

namespace tmq {
namespace {

__device__ const u32x4 kZeroChunk[8] = {};   // 128 zero bytes: the source of padding taps / the K tail

template <class Map>
struct MidEpilogueT {
    const float *scale, *bias;
    const void *residual;
    void *y;
    int relu, y_f16;
    [[no_unique_address]] Map map;   // where row m goes: pixel m (NoMap, no bytes) or a strided destination (RowMap)
};
using MidEpilogue = MidEpilogueT<NoMap>;
static_assert(sizeof(MidEpilogue) == 40, "the dense epilogue carries no map");

// Row providers. `prepare` fixes what a lane needs for its 2 WM row pieces (load c of fragment mi
// covers rows 8 c .. 8 c + 7; the lane's row is R = 8 c + lane / 8); `source` returns the address
// of the lane's 16-byte chunk of pair starting at reduction index k0 (uniform).
struct DenseRows {
    static constexpr bool kBuffer = false;
    const _Float16 *x;
    int64_t M, K;

    template <int WM>
    struct State {
        uint32_t off[WM][2];     // element offset of the row + swizzled chunk (host: M K < 2^31)
    };
    template <int WM>
    __device__ __forceinline__ void prepare(State<WM> &st, int64_t m0, int lane) const {
#pragma unroll
        for (int mi = 0; mi < WM; mi++)
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const int R = c * 8 + (lane >> 3);
                int64_t m = m0 + mi * 16 + R;
                if (m >= M) m = M - 1;                      // rows past M: finite data, never stored
                st.off[mi][c] = (uint32_t)(m * K) + (((lane & 7) ^ ((R >> 1) & 7)) * 8);
            }
    }
    struct Pair { int64_t k0; bool live; };
    __device__ __forceinline__ Pair pair(int64_t k0) const { return {k0, k0 < K}; }
    template <int WM>
    __device__ __forceinline__ const void *source(const State<WM> &st, const Pair &p, int mi, int c, int lane) const {
        return p.live ? static_cast<const void *>(x + (p.k0 + st.off[mi][c]))
                      : static_cast<const void *>(kZeroChunk + (lane & 7));
    }
};

struct ConvRows {
    static constexpr bool kBuffer = true;      // chunks are fetched through a buffer resource over x
    const _Float16 *x;
    int64_t M, K;
    int B, C, H, W, Ho, Wo, ky, kx, sy, sx, py, px, dy, dx;
    FastDiv by_wo, by_ho;      // M < 2^31
    FastDiv by_c, by_kx;       // K < 2^31

    template <int WM>
    struct State {
        int32_t off[WM][2];      // element offset of (b, ih0, iw0, swizzled chunk); may be negative
        int32_t ih0[WM][2], iw0[WM][2];
    };
    template <int WM>
    __device__ __forceinline__ void prepare(State<WM> &st, int64_t m0, int lane) const {
#pragma unroll
        for (int mi = 0; mi < WM; mi++)
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const int R = c * 8 + (lane >> 3);
                int64_t m = m0 + mi * 16 + R;
                if (m >= M) m = M - 1;
                int ow, oh;
                const uint32_t t = by_wo.divmod((uint32_t)m, ow);
                const int b = (int)by_ho.divmod(t, oh);
                st.ih0[mi][c] = oh * sy - py;
                st.iw0[mi][c] = ow * sx - px;
                st.off[mi][c] = ((b * H + st.ih0[mi][c]) * W + st.iw0[mi][c]) * C + (((lane & 7) ^ ((R >> 1) & 7)) * 8);
            }
    }
    struct Pair { int di, dj, delta; bool live; };
    __device__ __forceinline__ Pair pair(int64_t k0) const {       // uniform
        int c0, j;                                                  // multiply-high: no division sequence per pair
        const uint32_t tap = by_c.divmod((uint32_t)k0, c0);         // K < 2^31
        const int i = (int)by_kx.divmod(tap, j);
        return {i * dy, j * dx, (i * dy * W + j * dx) * C + c0, k0 < K};
    }
    template <int WM>
    __device__ __forceinline__ const void *source(const State<WM> &st, const Pair &p, int mi, int c, int lane) const {
        const bool in = p.live && (unsigned)(st.ih0[mi][c] + p.di) < (unsigned)H &&
                        (unsigned)(st.iw0[mi][c] + p.dj) < (unsigned)W;
        return in ? static_cast<const void *>(x + (st.off[mi][c] + p.delta))
                  : static_cast<const void *>(kZeroChunk + (lane & 7));
    }
    // the same chunk as a byte offset into the buffer; padding taps and the K tail: past its end (zeros)
    // (The three conditions are joined without short circuit: as branches they cost an exec-mask round trip per chunk
    // -- 512 -> 512 channels on 7 x 7, batch 64: 25.9 -> 24.8 us. One bit per tap row and tap column, tested with one
    // AND and one compare as in the tile kernels' loader, measured slower here: 25.4, and its set-up costs the short
    // reductions 4 %.)
    template <int WM>
    __device__ __forceinline__ uint32_t offset(const State<WM> &st, const Pair &p, int mi, int c) const {
        const bool in = p.live & ((unsigned)(st.ih0[mi][c] + p.di) < (unsigned)H) &
                        ((unsigned)(st.iw0[mi][c] + p.dj) < (unsigned)W);
        return in ? (uint32_t)(st.off[mi][c] + p.delta) * 2u : kPastTheEnd;
    }
    __device__ __forceinline__ uint32_t bytes() const { return (uint32_t)((int64_t)B * H * W * C * 2); }
};

// 16 bytes per lane from global memory straight into LDS: lane l lands at dst + 16 l (dst uniform).
// The host pass of the compiler does not know the builtin and would drop every kernel that uses it,
// so it only sees an empty body.
__device__ __forceinline__ void load_to_lds(const void *src, unsigned char *dst) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef __attribute__((address_space(3))) void *lds_ptr;
    __builtin_amdgcn_global_load_lds(src, (lds_ptr)dst, 16, 0, 0);
#endif
}

// Scale (already divided by the weight unit) and bias of a thread's four output columns in the epilogue
// below. Fetched before the main loop where registers allow: asked for only after it, the two loads are a
// trip to memory that nothing overlaps.
struct ThreadColumns {
    floatx4 sc, bi;
};

template <class Ep>
__device__ __forceinline__ bool epilogue_vectorised(int64_t N, const Ep &ep) {
    return (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(ep.y) | reinterpret_cast<uintptr_t>(ep.residual) |
                             reinterpret_cast<uintptr_t>(ep.scale) | reinterpret_cast<uintptr_t>(ep.bias)) & 15u) == 0;
}

template <int WN, class Ep>
__device__ __forceinline__ ThreadColumns load_column_constants(int64_t n0, int64_t N, const Ep &ep) {
    const int64_t n = n0 + (int)(threadIdx.x % (4 * WN)) * 4;
    ThreadColumns c{{1.f, 1.f, 1.f, 1.f}, {0.f, 0.f, 0.f, 0.f}};
    if (n < N) {
        if (epilogue_vectorised(N, ep)) {
            if (ep.scale) c.sc = *reinterpret_cast<const floatx4 *>(ep.scale + n);
            if (ep.bias) c.bi = *reinterpret_cast<const floatx4 *>(ep.bias + n);
        } else {
#pragma unroll
            for (int r = 0; r < 4; r++)
                if (n + r < N) {
                    if (ep.scale) c.sc[r] = ep.scale[n + r];
                    if (ep.bias) c.bi[r] = ep.bias[n + r];
                }
        }
    }
    c.sc *= 1.0f / kWeightUnit;
    return c;
}

// Epilogue of the split-reduction kernels. Lane (j, g) of fragment (mi, nj) holds
// y[16 mi + j][16 nj + 4 g + r], r = 0..3. Every wavefront parks its fragments in LDS (the windows are
// dead by now) with the four g of a row next to each other; then the whole workgroup walks the tile row
// by row: 16 consecutive threads own one row (4 columns each), add the WAVES partial sums in wavefront
// order -- so the result does not depend on scheduling -- and write 128 or 256 contiguous bytes per row.
// A thread keeps its columns for all its rows. Its residual values are asked for before the fragments go
// to LDS, so that they arrive while the workgroup synchronises (and before any store of this thread: the
// residual may be the output buffer).
//
// Pairs: fp32 rows carried as two fp16 rows each (hi = fp16(s x), lo = fp16(s x - hi), row m and row m + pair of the
// tile, s the row's own power of two). With RowPairs the two rows' sums are added -- hi's partial sums in wavefront
// order, then lo's -- and multiplied by row_scale[m] = 1 / s before the per-channel scale; M counts output rows.
struct NoPairs {
    static constexpr bool kOn = false;
};
struct RowPairs {
    static constexpr bool kOn = true;
    int pair;
    const float *row_scale;
};

template <int WM, int WN, int WAVES, class Ep, class Pairs = NoPairs>
__device__ __forceinline__ void reduce_and_store(unsigned char *smem, const floatx4 (&acc)[WM][WN], int kg, int lane,
                                                 int64_t m0, int64_t n0, int64_t M, int64_t N, const Ep &ep,
                                                 const ThreadColumns &cc, const Pairs &pairs = Pairs{}) {
    constexpr int NF = WM * WN;
    const int j = lane & 15, g = lane >> 4;
    constexpr int kFragPitch = 1024 + 64;                       // bytes; +64 spreads the nj over the banks
    constexpr int T = 64 * WAVES, kC4 = 4 * WN;                 // threads; float4 columns per row
    static_assert(T % kC4 == 0, "a thread must keep its columns");
    constexpr int kSweep = T / kC4, kIter = (16 * WM + kSweep - 1) / kSweep;   // rows per sweep of the workgroup; sweeps
    const int tid = threadIdx.x, c4 = tid % kC4, row0 = tid / kC4;
    const int64_t n = n0 + c4 * 4;
    const bool vec = epilogue_vectorised(N, ep);

    half4 res16[kIter];
    floatx4 res32[kIter];
    if (vec && ep.residual && n < N) {
#pragma unroll
        for (int it = 0; it < kIter; it++) {
            const int row = row0 + it * kSweep;
            const int64_t m = m0 + row;
            if (row < 16 * WM && m < M) {
                const int64_t px = ep.map.pixel(m);
                if (decltype(ep.map)::kDrops && px < 0) continue;
                if (ep.y_f16) res16[it] = *reinterpret_cast<const half4 *>(static_cast<const _Float16 *>(ep.residual) + px * N + n);
                else res32[it] = *reinterpret_cast<const floatx4 *>(static_cast<const float *>(ep.residual) + px * N + n);
            }
        }
    }

    if constexpr (WAVES > 1) __syncthreads();
    else __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int mi = 0; mi < WM; mi++)
#pragma unroll
        for (int nj = 0; nj < WN; nj++)
            *reinterpret_cast<floatx4 *>(smem + (size_t)(kg * NF + mi * WN + nj) * kFragPitch + (j * 4 + (g ^ ((j >> 2) & 3))) * 16) = acc[mi][nj];
    if constexpr (WAVES > 1) __syncthreads();
    else __builtin_amdgcn_wave_barrier();

    if (n >= N) return;
    const floatx4 sc = cc.sc, bi = cc.bi;
    auto row_sums = [&](int row) {
        const unsigned char *src = smem + (size_t)((row >> 4) * WN + (c4 >> 2)) * kFragPitch + ((row & 15) * 4 + ((c4 & 3) ^ ((row >> 2) & 3))) * 16;
        floatx4 v = *reinterpret_cast<const floatx4 *>(src);
#pragma unroll
        for (int q = 1; q < WAVES; q++) v += *reinterpret_cast<const floatx4 *>(src + (size_t)q * NF * kFragPitch);
        return v;
    };
    auto partial_sums = [&](int row) {
        floatx4 v = row_sums(row);
        if constexpr (Pairs::kOn) v = (v + row_sums(row + pairs.pair)) * pairs.row_scale[m0 + row];
        if constexpr (decltype(ep.map)::kPairs)                                  // the hi row's sums, then its lo row's, / s
            v = (v + row_sums(row ^ 8)) * ep.map.fragment_scale((m0 + row) & ~(int64_t)15);
        return v * sc + bi;
    };
    if (vec) {
#pragma unroll
        for (int it = 0; it < kIter; it++) {
            const int row = row0 + it * kSweep;
            const int64_t m = m0 + row;
            if (row >= 16 * WM || m >= M) break;
            const int64_t px = ep.map.pixel(m);
            if (decltype(ep.map)::kDrops && px < 0) continue;
            floatx4 v = partial_sums(row);
            const int64_t o = px * N + n;
            if (ep.y_f16) {
                if (ep.residual) {
#pragma unroll
                    for (int r = 0; r < 4; r++) v[r] += (float)res16[it][r];
                }
                half4 h;
#pragma unroll
                for (int r = 0; r < 4; r++) h[r] = (_Float16)((ep.relu && v[r] < 0.f) ? 0.f : v[r]);
                *reinterpret_cast<half4 *>(static_cast<_Float16 *>(ep.y) + o) = h;
            } else {
                if (ep.residual) v += res32[it];
                if (ep.relu) {
#pragma unroll
                    for (int r = 0; r < 4; r++) v[r] = v[r] < 0.f ? 0.f : v[r];
                }
                *reinterpret_cast<floatx4 *>(static_cast<float *>(ep.y) + o) = v;
            }
        }
        return;
    }
    for (int row = row0; row < 16 * WM; row += kSweep) {
        const int64_t m = m0 + row;
        if (m >= M) break;
        const int64_t px = ep.map.pixel(m);
        if (decltype(ep.map)::kDrops && px < 0) continue;
        const floatx4 v = partial_sums(row);
        const int64_t o = px * N + n;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            if (n + r >= N) break;
            float f = v[r];
            if (ep.y_f16) {
                if (ep.residual) f += (float)static_cast<const _Float16 *>(ep.residual)[o + r];
                static_cast<_Float16 *>(ep.y)[o + r] = (_Float16)((ep.relu && f < 0.f) ? 0.f : f);
            } else {
                if (ep.residual) f += static_cast<const float *>(ep.residual)[o + r];
                static_cast<float *>(ep.y)[o + r] = (ep.relu && f < 0.f) ? 0.f : f;
            }
        }
    }
}

template <int WM, int WN, int WAVES, bool BLK, class Rows, int RING, class Ep>
__global__ __launch_bounds__(64 * WAVES) void mid_kernel(Rows rows, const u32x4 *__restrict__ native, int64_t M, int Kb,
                                                         int npairs, int64_t N, int64_t Nb, int tiles_n, int by_rows,
                                                         Ep ep) {
    constexpr int kFrag = 16 * 128, kSlot = WM * kFrag, kWave = RING * kSlot;   // bytes: 16 rows x 128 B per fragment
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & 63, kg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, g = lane >> 4;
    unsigned char *win = smem + kg * kWave;
    // Tiles are numbered n fastest. Dealt round-robin, every XCD meets every row tile: its L2 reads all of x and an
    // eighth of the weights. When x is the larger operand the XCDs take consecutive runs of tiles instead -- an
    // eighth of the rows each, all weights (M = 4096, K = 8192, N = 512: 56.8 -> 37.8 us).
    const int tile = by_rows ? xcd_contiguous(blockIdx.x, gridDim.x) : (int)blockIdx.x;
    const int tm = tile / tiles_n, tn = tile % tiles_n;
    const int64_t m0 = (int64_t)tm * (16 * WM), n0 = (int64_t)tn * (16 * WN);

    floatx4 acc[WM][WN];
#pragma unroll
    for (int mi = 0; mi < WM; mi++)
#pragma unroll
        for (int nj = 0; nj < WN; nj++) acc[mi][nj] = floatx4{0.f, 0.f, 0.f, 0.f};

    const uint32_t *wb[WN];                                       // dword d of block kb: wb[nj][kb * 256 + d]
#pragma unroll
    for (int nj = 0; nj < WN; nj++) {
        int64_t nb = n0 / 16 + nj;
        if (nb >= Nb) nb = Nb - 1;                                  // finite bits, never stored
        wb[nj] = reinterpret_cast<const uint32_t *>(native + (nb * Kb) * 64 + lane);
    }
    typename Rows::template State<WM> st;
    rows.template prepare<WM>(st, m0, lane);
    BufferResource rsrc;
    if constexpr (Rows::kBuffer) rsrc = make_buffer_resource(rows.x, rows.bytes());
    const ThreadColumns cc = load_column_constants<WN>(n0, N, ep);

    // operand (row j, chunk ch) of a fragment sits at position ch ^ ((j / 2) % 8) of its row
    const int key = (j >> 1) & 7;
    const unsigned char *rd = win + j * 128;

    if constexpr (BLK) {
        // The reduction dealt out in whole weight blocks (4 pairs): wavefront kg takes blocks kg, kg + WAVES, ...
        // A lane's 16 bytes of a block arrive with one load per channel block (instead of four dword loads, one per
        // pair: the CU's vector-memory pipeline is what this kernel keeps busiest), one block ahead; the
        // activations go pair by pair through the two slots as below.
        const u32x4 *wbb[WN];
#pragma unroll
        for (int nj = 0; nj < WN; nj++) wbb[nj] = reinterpret_cast<const u32x4 *>(wb[nj]);
        const int nt = Kb > kg ? (Kb - kg + WAVES - 1) / WAVES : 0;
        auto wloadb = [&](u32x4 (&w)[WN], int t) {
            const int64_t kb = kg + (int64_t)t * WAVES;
#pragma unroll
            for (int nj = 0; nj < WN; nj++) w[nj] = wbb[nj][kb * 64];
        };
        auto fillb = [&](int slot, int t, int q) {
            const typename Rows::Pair pr = rows.pair(((int64_t)(kg + t * WAVES) * 4 + q) * 64);
#pragma unroll
            for (int mi = 0; mi < WM; mi++)
#pragma unroll
                for (int c = 0; c < 2; c++)
                    if constexpr (Rows::kBuffer)
                        buffer_to_lds(rsrc, rows.template offset<WM>(st, pr, mi, c), win + slot * kSlot + mi * kFrag + c * 1024);
                    else
                        load_to_lds(rows.template source<WM>(st, pr, mi, c, lane), win + slot * kSlot + mi * kFrag + c * 1024);
        };
        if (nt > 0) {
            u32x4 wq[2][WN];
            wloadb(wq[0], 0);
            fillb(0, 0, 0);
            constexpr int kWaitW = (WN & 15) | (7 << 4) | (15 << 8) | ((WN >> 4) << 14);   // vmcnt(WN)
            // pair q of block t; `par` = parity of t (weight register set), slot = q % 2
            auto step = [&](int t, auto par_tag, auto q_tag) {
                constexpr int par = decltype(par_tag)::value, q = decltype(q_tag)::value, slot = q & 1;
                const bool more = t + 1 < nt;
                // this pair's activations must have landed; at q == 3 the next block's weights, issued one
                // step ago behind them, may still be on their way
                if (q == 3 && more) __builtin_amdgcn_s_waitcnt(kWaitW);
                else __builtin_amdgcn_s_waitcnt(0x0F70);
                __builtin_amdgcn_sched_barrier(0);
                half8 a[2][WM];
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                    for (int mi = 0; mi < WM; mi++)
                        a[s2][mi] = *reinterpret_cast<const half8 *>(rd + slot * kSlot + mi * kFrag + (((4 * s2 + g) ^ key) * 16));
                __builtin_amdgcn_sched_barrier(0);
                if (q < 3) fillb(slot ^ 1, t, q + 1);
                else if (more) fillb(slot ^ 1, t + 1, 0);
                if (q == 2 && more) wloadb(wq[par ^ 1], t + 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                    for (int nj = 0; nj < WN; nj++) {
                        const half8 w = decode_step(wq[par][nj][q], s2);
#pragma unroll
                        for (int mi = 0; mi < WM; mi++) acc[mi][nj] = mfma16(w, a[s2][mi], acc[mi][nj]);
                    }
                __builtin_amdgcn_sched_barrier(0);
            };
            auto block = [&](int t, auto par_tag) {
                step(t, par_tag, std::integral_constant<int, 0>{});
                step(t, par_tag, std::integral_constant<int, 1>{});
                step(t, par_tag, std::integral_constant<int, 2>{});
                step(t, par_tag, std::integral_constant<int, 3>{});
            };
            int t = 0;
            for (; t + 2 <= nt; t += 2) {
                block(t, std::integral_constant<int, 0>{});
                block(t + 1, std::integral_constant<int, 1>{});
            }
            if (t < nt) block(t, std::integral_constant<int, 0>{});
        }
        reduce_and_store<WM, WN, WAVES>(smem, acc, kg, lane, m0, n0, M, N, ep, cc);
        return;
    }

    // the reduction is dealt out in pairs: wavefront kg takes pairs kg, kg + WAVES, ...
    const int np = npairs > kg ? (npairs - kg + WAVES - 1) / WAVES : 0;
    auto wload = [&](uint32_t (&w)[WN], int p) {
        const int pi = kg + p * WAVES;
#pragma unroll
        for (int nj = 0; nj < WN; nj++) w[nj] = wb[nj][(int64_t)(pi >> 2) * 256 + (pi & 3)];
    };
    // asynchronous fill of one LDS slot with a pair: 2 WM loads of 1 KiB, lane l -> byte 16 l
    auto fill = [&](int slot, int p) {
        const typename Rows::Pair pr = rows.pair((int64_t)(kg + p * WAVES) * 64);
#pragma unroll
        for (int mi = 0; mi < WM; mi++)
#pragma unroll
            for (int c = 0; c < 2; c++)
                if constexpr (Rows::kBuffer)
                    buffer_to_lds(rsrc, rows.template offset<WM>(st, pr, mi, c), win + slot * kSlot + mi * kFrag + c * 1024);
                else
                    load_to_lds(rows.template source<WM>(st, pr, mi, c, lane), win + slot * kSlot + mi * kFrag + c * 1024);
    };
    if constexpr (RING == 3) {
        // Two pairs ahead instead of one: with one wavefront per SIMD (the 64 x 128 tile) a pair's multiplications
        // are shorter than a trip to L2, so a load issued one pair ahead is still waited for. Every step issues
        // its refill unconditionally (past the end: the last pair again, into a slot already read out), so
        // that every wait leaves exactly one refill in flight and the compiler's own counts stay exact.
        if (np > 0) {
            uint32_t wq[3][WN];
            auto refill = [&](int slot, uint32_t (&w)[WN], int p) {
                const int pc = p < np ? p : np - 1;
                fill(slot, pc);
                wload(w, pc);
            };
            refill(0, wq[0], 0);
            refill(1, wq[1], 1);
            constexpr int kN = 2 * WM + WN;
            constexpr int kWait1 = (kN & 15) | (7 << 4) | (15 << 8) | ((kN >> 4) << 14);   // vmcnt(one refill)
            auto step = [&](int p, auto slot_tag) {
                constexpr int slot = decltype(slot_tag)::value, nxt = (slot + 2) % 3;
                __builtin_amdgcn_s_waitcnt(kWait1);
                __builtin_amdgcn_sched_barrier(0);
                half8 a[2][WM];
#pragma unroll
                for (int s = 0; s < 2; s++)
#pragma unroll
                    for (int mi = 0; mi < WM; mi++)
                        a[s][mi] = *reinterpret_cast<const half8 *>(rd + slot * kSlot + mi * kFrag + (((4 * s + g) ^ key) * 16));
                __builtin_amdgcn_sched_barrier(0);
                refill(nxt, wq[nxt], p + 2);      // slot nxt was read out one pair ago
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int s = 0; s < 2; s++)
#pragma unroll
                    for (int nj = 0; nj < WN; nj++) {
                        const half8 w = decode_step(wq[slot][nj], s);
#pragma unroll
                        for (int mi = 0; mi < WM; mi++) acc[mi][nj] = mfma16(w, a[s][mi], acc[mi][nj]);
                    }
                __builtin_amdgcn_sched_barrier(0);
            };
            int p = 0;
            for (; p + 3 <= np; p += 3) {
                step(p, std::integral_constant<int, 0>{});
                step(p + 1, std::integral_constant<int, 1>{});
                step(p + 2, std::integral_constant<int, 2>{});
            }
            if (p < np) step(p, std::integral_constant<int, 0>{});
            if (p + 1 < np) step(p + 1, std::integral_constant<int, 1>{});
            __builtin_amdgcn_s_waitcnt(0x0F70);   // the surplus refills must land before the window is reused
        }
    } else if (np > 0) {
        uint32_t wq[2][WN];
        wload(wq[0], 0);
        fill(0, 0);
        // one pair; `par` (static) = parity of p = LDS slot and weight register set of the pair
        auto step = [&](int p, auto par_tag) {
            constexpr int par = decltype(par_tag)::value;
            // the fill of this slot (and the weight dwords) must have landed
            __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
            __builtin_amdgcn_sched_barrier(0);
            half8 a[2][WM];                        // all operand reads of the pair
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
                for (int mi = 0; mi < WM; mi++)
                    a[s][mi] = *reinterpret_cast<const half8 *>(rd + par * kSlot + mi * kFrag + (((4 * s + g) ^ key) * 16));
            __builtin_amdgcn_sched_barrier(0);
            // the other slot was read out one pair ago: start filling it with the next pair
            if (p + 1 < np) {
                fill(par ^ 1, p + 1);
                wload(wq[par ^ 1], p + 1);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
                for (int nj = 0; nj < WN; nj++) {
                    const half8 w = decode_step(wq[par][nj], s);
#pragma unroll
                    for (int mi = 0; mi < WM; mi++) acc[mi][nj] = mfma16(w, a[s][mi], acc[mi][nj]);
                }
            // keeps the next pair's wait below these multiplications: hoisted above them it would make
            // them wait for the loads just issued
            __builtin_amdgcn_sched_barrier(0);
        };
        int p = 0;
        for (; p + 2 <= np; p += 2) {
            step(p, std::integral_constant<int, 0>{});
            step(p + 1, std::integral_constant<int, 1>{});
        }
        if (p < np) step(p, std::integral_constant<int, 0>{});
    }

    reduce_and_store<WM, WN, WAVES>(smem, acc, kg, lane, m0, n0, M, N, ep, cc);
}

template <int WM, int WN, int WAVES, class Rows, bool BLK = false, int RING = 2, class Ep>
int launch(const Rows &rows, const void *native, int64_t M, int64_t K, int64_t N, const Ep &ep, void *stream) {
    constexpr int BM = 16 * WM, BN = 16 * WN;
    const int64_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN, Kb = native_blocks_k(K);
    if (tm * tn > 0x7FFFFFFF || Kb > (1 << 20)) return TMQ_ERR_TOO_LARGE;
    constexpr size_t win = (size_t)WAVES * RING * WM * 16 * 128;
    constexpr size_t redb = (size_t)WAVES * WM * WN * (1024 + 64);
    constexpr size_t lds = win > redb ? win : redb;
    static_assert(lds <= 152 * 1024, "LDS budget");
    auto kernel = mid_kernel<WM, WN, WAVES, BLK, Rows, RING, Ep>;
    if (int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) return st;
    hipLaunchKernelGGL(kernel, dim3((uint32_t)(tm * tn)), dim3(64 * WAVES), lds, as_stream(stream), rows,
                       static_cast<const u32x4 *>(native), M, (int)Kb, (int)((K + 63) / 64), N, native_blocks_n(N),
                       (int)tn, (2 * M * 4 > N) ? 1 : 0 /* bytes of x (2 M K) against bytes of weights (N K / 4) */, ep);
    return check_launch();
}

// ---- weight stream, at most 16 rows ------------------------------------------------------------------
// Large layers with a handful of rows (batched decoding): the job is to read the weights once at HBM
// speed. A workgroup of WAVES wavefronts owns 16 WN output channels and splits the reduction over its
// wavefronts by whole weight blocks (256 reduction indices): wavefront kg takes blocks kg, kg + WAVES, ...
// Unlike mid_kernel, whose pipeline unit is a 64-index pair loaded one step ahead, a wavefront here keeps
// D of its blocks in flight -- the WN weight blocks as whole 1 KiB loads (one instruction per block
// instead of four dword loads) in D register sets, and the R x 512 bytes of activations that go with
// them in a private LDS window of D slots -- enough outstanding bytes to cover the latency of HBM. An
// operand read from LDS feeds WN multiplications.
//
// R = 16, 8, 4 or 2 >= M rows are staged (fewer rows: smaller slots, deeper pipeline). One staging
// instruction moves 1 KiB, lane l to byte 16 l of its destination: 8 rows x 128 bytes for R >= 8 (the
// layout of mid_kernel), else R rows x 1024 / R bytes. Rows lie a multiple of 256 bytes apart, i.e. on the
// same banks, so the 16-byte chunk c of row r is stored at position c ^ swz(r); the XOR is applied to the
// source address and undone by the reader. Rows past M repeat row M - 1; MFMA columns past M read row
// M - 1 too and are never stored. Requires K % 256 == 0.
template <int R>
struct StreamRows {
    static constexpr int kLoads = R / 2;                             // staging instructions per block: R x 512 B / 1 KiB
    static constexpr int kSlot = R * 512;                            // bytes of a block's activations
    // element offset (without the block's k0) of what lane `lane` fetches in instruction i
    __device__ static uint32_t source(int i, int lane, int64_t M, int64_t K) {
        int row, k;
        if constexpr (R >= 8) {                                        // instruction = (pair, half): 8 rows x 128 B
            const int p = R == 16 ? i >> 1 : i, c = R == 16 ? i & 1 : 0;
            row = 8 * c + (lane >> 3);
            k = p * 64 + (((lane & 7) ^ ((row >> 1) & 7)) * 8);
        } else {                                                       // R rows x (1024 / R) B
            constexpr int kPieces = 64 / R;                            // 16-byte pieces per row and instruction
            row = lane / kPieces;
            k = i * (kPieces * 8) + (((lane % kPieces) ^ (row << 2)) * 8);
        }
        if (row >= M) row = (int)M - 1;
        return (uint32_t)(row * K + k);
    }
    // LDS offset inside a slot of (row r, MFMA step i of the block, lane group g)
    __device__ static int operand(int r, int i, int g) {
        if constexpr (R >= 8) {
            const int p = i >> 1, c = 4 * (i & 1) + g;                 // pair, chunk of the pair
            return p * (R * 128) + r * 128 + ((c ^ ((r >> 1) & 7)) * 16);
        } else {
            constexpr int kPieces = 64 / R;
            const int c = 4 * i + g;                                   // chunk of the block's 32
            return (c / kPieces) * 1024 + r * (kPieces * 16) + (((c % kPieces) ^ (r << 2)) * 16);
        }
    }
};

// Wavefronts per SIMD the LDS windows leave room for: the register budget the compiler has to keep to.
constexpr int stream_waves_per_simd(int WN, int WAVES, int R, int D) {
    const int win = WAVES * D * R * 512, redb = WAVES * WN * (1024 + 64), lds = win > redb ? win : redb;
    int wgs = (160 * 1024) / lds;
    if (wgs > 32 / WAVES) wgs = 32 / WAVES;
    if (wgs < 1) wgs = 1;
    const int w = wgs * WAVES / 4;
    return w < 1 ? 1 : (w > 4 ? 4 : w);
}

template <int WN, int WAVES, int R, int D, bool LONG, class Pairs>
__global__ __launch_bounds__(64 * WAVES, stream_waves_per_simd(WN, WAVES, R, D)) void stream_kernel(const _Float16 *__restrict__ x, const u32x4 *__restrict__ native,
                                                            int64_t M, int64_t K, int Kb, int64_t N, int64_t Nb,
                                                            MidEpilogue ep, Pairs pairs) {
    using Rows = StreamRows<R>;
    constexpr int kLoads = Rows::kLoads, kSlot = Rows::kSlot, kWave = D * kSlot, kPerBlock = WN + kLoads;
    static_assert((D - 1) * kPerBlock < 64, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & 63, kg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, g = lane >> 4;
    unsigned char *win = smem + kg * kWave;
    const int64_t n0 = (int64_t)blockIdx.x * (16 * WN);

    floatx4 acc[1][WN];
#pragma unroll
    for (int nj = 0; nj < WN; nj++) acc[0][nj] = floatx4{0.f, 0.f, 0.f, 0.f};

    const u32x4 *wb[WN];                                          // block kb of channel block nj: wb[nj][kb * 64]
#pragma unroll
    for (int nj = 0; nj < WN; nj++) {
        int64_t nb = n0 / 16 + nj;
        if (nb >= Nb) nb = Nb - 1;                                  // finite bits, never stored
        wb[nj] = native + (nb * Kb) * 64 + lane;
    }
    uint32_t src[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; i++) src[i] = Rows::source(i, lane, M, K);
    int rd[8];                                                      // operand offsets of the 8 MFMA steps
    {
        const int r = j < M ? j : (int)M - 1;
#pragma unroll
        for (int i = 0; i < 8; i++) rd[i] = Rows::operand(r, i, g);
    }

    const int nt = Kb > kg ? (Kb - kg + WAVES - 1) / WAVES : 0;   // weight blocks of this wavefront
    auto wload = [&](u32x4 (&w)[WN], int t) {
        const int64_t kb = kg + (int64_t)t * WAVES;
#pragma unroll
        for (int nj = 0; nj < WN; nj++) w[nj] = __builtin_nontemporal_load(wb[nj] + kb * 64);
    };
    auto fill = [&](int slot, int t) {
        const _Float16 *xb = x + (kg + (int64_t)t * WAVES) * kKB;
#pragma unroll
        for (int i = 0; i < kLoads; i++) load_to_lds(xb + src[i], win + slot * kSlot + i * 1024);
    };
    if constexpr (R == 16) {
        // One block out of slot / register set PAR with at most BEHIND younger blocks still on their way (loads
        // complete in issue order), refilling the slot with block t + D if REFILL. Everything about the pipeline
        // state is a template argument: the wait below is exact, and so are the waits the compiler adds before it
        // lets the weight registers be used -- after a conditional refill it could only wait for everything.
        u32x4 wq[D][WN];
        auto step = [&](int t, auto par_tag, auto behind_tag, auto refill_tag) {
            constexpr int PAR = decltype(par_tag)::value, BEHIND = decltype(behind_tag)::value;
            constexpr bool REFILL = decltype(refill_tag)::value;
            static_assert(BEHIND >= 0 && BEHIND < D && BEHIND * kPerBlock < 64, "vmcnt is a 6-bit counter");
            constexpr int kCount = BEHIND * kPerBlock;
            __builtin_amdgcn_s_waitcnt((kCount & 15) | (7 << 4) | (15 << 8) | ((kCount >> 4) << 14));   // vmcnt(kCount)
            __builtin_amdgcn_sched_barrier(0);
            half8 a[8];                                                // all operand reads of the block
#pragma unroll
            for (int i = 0; i < 8; i++) a[i] = *reinterpret_cast<const half8 *>(win + PAR * kSlot + rd[i]);
            // the slot is free again once the reads have returned
            __builtin_amdgcn_s_waitcnt(0xC07F);                        // lgkmcnt(0)
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (REFILL) fill(PAR, t + D);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 8; i++)
#pragma unroll
                for (int nj = 0; nj < WN; nj++)
                    acc[0][nj] = mfma16(decode_step(wq[PAR][nj][i >> 1], i & 1), a[i], acc[0][nj]);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (REFILL) wload(wq[PAR], t + D);
            __builtin_amdgcn_sched_barrier(0);
        };
        // the first COUNT blocks, in the order the waits count on
        auto prologue = [&](auto count_tag) {
            constexpr int COUNT = decltype(count_tag)::value;
#pragma unroll
            for (int d = 0; d < COUNT; d++) {
                fill(d, d);
                wload(wq[d], d);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // the last D + REM blocks (t a multiple of D, blocks t .. t + D - 1 in flight): D steps of which the first
        // REM still refill, then REM steps
        auto drain = [&](int t, auto rem_tag) {
            constexpr int REM = decltype(rem_tag)::value;
            auto first = [&](auto j_tag) {
                constexpr int J = decltype(j_tag)::value;
                if constexpr (J < D)
                    step(t + J, j_tag, std::integral_constant<int, D - 1 - J + (J < REM ? J : REM)>{}, std::bool_constant<(J < REM)>{});
            };
            first(std::integral_constant<int, 0>{});
            first(std::integral_constant<int, 1>{});
            first(std::integral_constant<int, 2>{});
            first(std::integral_constant<int, 3>{});
            auto second = [&](auto j_tag) {
                constexpr int J = decltype(j_tag)::value;
                if constexpr (J < REM) step(t + D + J, j_tag, std::integral_constant<int, REM - 1 - J>{}, std::false_type{});
            };
            second(std::integral_constant<int, 0>{});
            second(std::integral_constant<int, 1>{});
            second(std::integral_constant<int, 2>{});
        };
        // fewer than D blocks in all: everything in flight at once
        auto few = [&](auto nt_tag) {
            constexpr int NT = decltype(nt_tag)::value;
            if constexpr (NT < D) {
                prologue(nt_tag);
                auto one = [&](auto j_tag) {
                    constexpr int J = decltype(j_tag)::value;
                    if constexpr (J < NT) step(J, j_tag, std::integral_constant<int, NT - 1 - J>{}, std::false_type{});
                };
                one(std::integral_constant<int, 0>{});
                one(std::integral_constant<int, 1>{});
                one(std::integral_constant<int, 2>{});
            }
        };
        static_assert(D >= 1 && D <= 4, "cases below");

        if (nt >= D) {
            prologue(std::integral_constant<int, D>{});
            int t = 0;
            while (t + 2 * D <= nt) {                                  // steady state: D - 1 blocks behind, always refill
                step(t, std::integral_constant<int, 0>{}, std::integral_constant<int, D - 1>{}, std::true_type{});
                if constexpr (D > 1) step(t + 1, std::integral_constant<int, 1>{}, std::integral_constant<int, D - 1>{}, std::true_type{});
                if constexpr (D > 2) step(t + 2, std::integral_constant<int, 2>{}, std::integral_constant<int, D - 1>{}, std::true_type{});
                if constexpr (D > 3) step(t + 3, std::integral_constant<int, 3>{}, std::integral_constant<int, D - 1>{}, std::true_type{});
                t += D;
            }
            switch (nt - t - D) {                                      // 0 .. D - 1 blocks not yet requested
                case 0: drain(t, std::integral_constant<int, 0>{}); break;
                case 1: if constexpr (D > 1) drain(t, std::integral_constant<int, 1>{}); break;
                case 2: if constexpr (D > 2) drain(t, std::integral_constant<int, 2>{}); break;
                default: if constexpr (D > 3) drain(t, std::integral_constant<int, 3>{}); break;
            }
        } else {
            switch (nt) {
                case 1: few(std::integral_constant<int, 1>{}); break;
                case 2: few(std::integral_constant<int, 2>{}); break;
                case 3: few(std::integral_constant<int, 3>{}); break;
                default: break;
            }
        }
    } else {
        // Fewer than 16 rows: several workgroups share a CU, and the fully static pipeline above costs the
        // registers that residency depends on (measured slower). Here only the steady state is static (template
        // argument LONG: every wavefront has at least 2 D blocks) and the drain works with guards.
        // wait until at most n blocks' loads are outstanding (loads complete in issue order)
        auto wait_blocks = [&](int n) {
            static_assert(D <= 4, "cases below");
            constexpr auto enc = [](int c) { return (c & 15) | (7 << 4) | (15 << 8) | ((c >> 4) << 14); };
            if (n >= 3 && D > 3) __builtin_amdgcn_s_waitcnt(enc(3 * kPerBlock));
            else if (n == 2 && D > 2) __builtin_amdgcn_s_waitcnt(enc(2 * kPerBlock));
            else if (n == 1) __builtin_amdgcn_s_waitcnt(enc(kPerBlock));
            else __builtin_amdgcn_s_waitcnt(enc(0));
        };

        if (nt > 0) {
            u32x4 wq[D][WN];
            // one block; `par` (static) = t % D = LDS slot and weight register set of the block. In the steady
            // state every step refills unconditionally, so the number of loads behind the one being waited for
            // is a constant -- for the wait below and for the waits the compiler adds before it lets the
            // weight registers be used (with a conditional refill it can only wait for everything).
            auto step = [&](int t, auto par_tag, auto steady_tag) {
                constexpr int par = decltype(par_tag)::value;
                constexpr bool kSteady = decltype(steady_tag)::value;
                if constexpr (kSteady) {
                    wait_blocks(D - 1);
                } else {
                    const int ahead = nt - 1 - t;                     // blocks issued after this one
                    wait_blocks(ahead < D - 1 ? ahead : D - 1);
                }
                __builtin_amdgcn_sched_barrier(0);
                half8 a[8];                                            // all operand reads of the block
#pragma unroll
                for (int i = 0; i < 8; i++) a[i] = *reinterpret_cast<const half8 *>(win + par * kSlot + rd[i]);
                // the slot is free again once the reads have returned: refill it with the block D ahead
                __builtin_amdgcn_s_waitcnt(0xC07F);                    // lgkmcnt(0)
                __builtin_amdgcn_sched_barrier(0);
                if (kSteady || t + D < nt) fill(par, t + D);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < 8; i++)
#pragma unroll
                    for (int nj = 0; nj < WN; nj++)
                        acc[0][nj] = mfma16(decode_step(wq[par][nj][i >> 1], i & 1), a[i], acc[0][nj]);
                __builtin_amdgcn_sched_barrier(0);
                if (kSteady || t + D < nt) wload(wq[par], t + D);
                __builtin_amdgcn_sched_barrier(0);
            };
            auto round = [&](int t, auto steady_tag) {
                step(t, std::integral_constant<int, 0>{}, steady_tag);
                if constexpr (D > 1) step(t + 1, std::integral_constant<int, 1>{}, steady_tag);
                if constexpr (D > 2) step(t + 2, std::integral_constant<int, 2>{}, steady_tag);
                if constexpr (D > 3) step(t + 3, std::integral_constant<int, 3>{}, steady_tag);
            };
            int t = 0;
            if constexpr (LONG) {
                // every wavefront has at least 2 D blocks (the host checks): an unconditional prologue and at
                // least one steady round, entered from one known sequence of outstanding loads
#pragma unroll
                for (int d = 0; d < D; d++) {
                    fill(d, d);
                    wload(wq[d], d);
                    __builtin_amdgcn_sched_barrier(0);                // the order of issue the waits count on
                }
                do {
                    round(t, std::true_type{});
                    t += D;
                } while (t + 2 * D <= nt);
            } else {
#pragma unroll
                for (int d = 0; d < D; d++)
                    if (d < nt) {
                        fill(d, d);
                        wload(wq[d], d);
                        __builtin_amdgcn_sched_barrier(0);
                    }
            }
            // drain: at most 2 D - 1 blocks with wave-uniform guards
            for (; t + D <= nt; t += D) round(t, std::false_type{});
            if (t < nt) step(t, std::integral_constant<int, 0>{}, std::false_type{});
            if constexpr (D > 2) if (t + 1 < nt) step(t + 1, std::integral_constant<int, 1>{}, std::false_type{});
            if constexpr (D > 3) if (t + 2 < nt) step(t + 2, std::integral_constant<int, 2>{}, std::false_type{});
        }
    }
    int64_t rows_out = M;
    if constexpr (Pairs::kOn) rows_out = pairs.pair;
    reduce_and_store<1, WN, WAVES>(smem, acc, kg, lane, 0, n0, rows_out, N, ep, load_column_constants<WN>(n0, N, ep), pairs);
}

// pairs: null, or the fp16 rows are M / 2 fp32 rows' hi terms followed by their lo terms
template <int WN, int WAVES, int R, int D>
int launch_stream(const void *x, const void *native, int64_t M, int64_t K, int64_t N, const MidEpilogue &ep, void *stream,
                  const RowPairs *pairs = nullptr) {
    const int64_t tn = (N + 16 * WN - 1) / (16 * WN), Kb = native_blocks_k(K);
    if (tn > 0x7FFFFFFF || Kb > (1 << 20)) return TMQ_ERR_TOO_LARGE;
    constexpr size_t win = (size_t)WAVES * D * R * 512, redb = (size_t)WAVES * WN * (1024 + 64);
    constexpr size_t lds = win > redb ? win : redb;
    static_assert(lds <= 152 * 1024, "LDS budget");
    // the variant with a steady-state loop needs 2 D blocks in every wavefront; with fewer, half the depth
    // and a steady state beats the full depth without one
    if constexpr (D == 4) {
        if (Kb / WAVES < 2 * D && Kb / WAVES >= D) return launch_stream<WN, WAVES, R, 2>(x, native, M, K, N, ep, stream, pairs);
    }
    auto go = [&](auto kernel, auto pairs_arg) {
        if (int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) return st;
        hipLaunchKernelGGL(kernel, dim3((uint32_t)tn), dim3(64 * WAVES), lds, as_stream(stream),
                           static_cast<const _Float16 *>(x), static_cast<const u32x4 *>(native), M, K, (int)Kb, N,
                           native_blocks_n(N), ep, pairs_arg);
        return check_launch();
    };
    const bool steady = R != 16 && Kb / WAVES >= 2 * D;
    if constexpr (R >= 4) {
        if (pairs)
            return steady ? go(stream_kernel<WN, WAVES, R, D, true, RowPairs>, *pairs) : go(stream_kernel<WN, WAVES, R, D, false, RowPairs>, *pairs);
    }
    if (pairs) return TMQ_ERR_UNSUPPORTED;
    return steady ? go(stream_kernel<WN, WAVES, R, D, true, NoPairs>, NoPairs{}) : go(stream_kernel<WN, WAVES, R, D, false, NoPairs>, NoPairs{});
}

// ---- weight stream, fp32 activations, at most 16 rows -------------------------------------------------
// The reference's GEMV (ternary_mvm_cuda) takes an fp32 vector. Same plan as stream_kernel with 16 channels
// per workgroup, but the activations of a block (256 fp32 = 1 KiB per row, one 16-byte load per lane) travel
// through registers: each value is split into two fp16 terms (hi = fp16(x), lo = fp16(x - hi), together 22
// significant bits), the terms go through a small wavefront-private LDS area into operand order, and
// every weight fragment is multiplied with both. All loads are register loads, so the compiler counts the
// waits itself -- exactly, as long as the steady state refills unconditionally (template argument LONG:
// every wavefront has at least 2 D blocks; otherwise a guarded pipeline).
template <int WAVES, int MR, int D, bool LONG>
__global__ __launch_bounds__(64 * WAVES) void stream32_kernel(const float *__restrict__ x, const u32x4 *__restrict__ native,
                                                              int64_t M, int64_t K, int Kb, int64_t N, int64_t Nb,
                                                              MidEpilogue ep) {
    constexpr int kRow = 1024 + 32;                                 // bytes per staged row: hi plane, lo plane, pad
    constexpr int kWave = MR * kRow;
    constexpr size_t kRed = (size_t)WAVES * (1024 + 64);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & 63, kg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, g = lane >> 4;
    unsigned char *win = smem + kRed + kg * kWave;                  // behind the reduction area: no reuse, no barrier
    const int64_t n0 = (int64_t)blockIdx.x * 16;

    floatx4 acc[1][1] = {{floatx4{0.f, 0.f, 0.f, 0.f}}};
    int64_t nb = n0 / 16;
    if (nb >= Nb) nb = Nb - 1;
    const u32x4 *wb = native + (nb * Kb) * 64 + lane;
    const float *xr[MR];                                            // this lane's four values of a block, per row
#pragma unroll
    for (int r = 0; r < MR; r++) xr[r] = x + (int64_t)(r < M ? r : M - 1) * K + lane * 4;
    const int rrow = j < M ? j : (int)M - 1;                        // the row whose operand this lane supplies
    const unsigned char *rd = win + rrow * kRow + g * 16;

    const int nt = Kb > kg ? (Kb - kg + WAVES - 1) / WAVES : 0;   // weight blocks of this wavefront
    u32x4 wq[D];
    floatx4 xq[D][MR];
    auto load = [&](int slot, int t) {
        const int64_t kb = kg + (int64_t)t * WAVES;
        wq[slot] = __builtin_nontemporal_load(wb + kb * 64);
#pragma unroll
        for (int r = 0; r < MR; r++) xq[slot][r] = *reinterpret_cast<const floatx4 *>(xr[r] + kb * kKB);
    };
    auto multiply = [&](int slot) {
#pragma unroll
        for (int r = 0; r < MR; r++) {
            half4 hi, lo;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                hi[e] = (_Float16)xq[slot][r][e];
                lo[e] = (_Float16)(xq[slot][r][e] - (float)hi[e]);
            }
            *reinterpret_cast<half4 *>(win + r * kRow + lane * 8) = hi;
            *reinterpret_cast<half4 *>(win + r * kRow + 512 + lane * 8) = lo;
        }
        __builtin_amdgcn_wave_barrier();
        half8 a[8], b[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            a[i] = *reinterpret_cast<const half8 *>(rd + i * 64);
            b[i] = *reinterpret_cast<const half8 *>(rd + 512 + i * 64);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const half8 w = decode_step(wq[slot][i >> 1], i & 1);
            acc[0][0] = mfma16(w, a[i], acc[0][0]);
            acc[0][0] = mfma16(w, b[i], acc[0][0]);
        }
        __builtin_amdgcn_wave_barrier();
    };
    static_assert(D == 2 || D == 4, "unrolled by hand");
    int t = 0;
    if constexpr (LONG) {
#pragma unroll
        for (int d = 0; d < D; d++) load(d, d);
        do {
            multiply(0); load(0, t + D);
            multiply(1); load(1, t + D + 1);
            if constexpr (D > 2) {
                multiply(2); load(2, t + D + 2);
                multiply(3); load(3, t + D + 3);
            }
            t += D;
        } while (t + 2 * D <= nt);
    } else {
#pragma unroll
        for (int d = 0; d < D; d++)
            if (d < nt) load(d, d);
    }
    for (; t < nt; t += D) {
        if (t < nt) { multiply(0); if (t + D < nt) load(0, t + D); }
        if (t + 1 < nt) { multiply(1); if (t + D + 1 < nt) load(1, t + D + 1); }
        if constexpr (D > 2) {
            if (t + 2 < nt) { multiply(2); if (t + D + 2 < nt) load(2, t + D + 2); }
            if (t + 3 < nt) { multiply(3); if (t + D + 3 < nt) load(3, t + D + 3); }
        }
    }
    reduce_and_store<1, 1, WAVES>(smem, acc, kg, lane, 0, n0, M, N, ep, load_column_constants<1>(n0, N, ep));
}

template <int MR>
int launch_stream32(const void *x, const void *native, int64_t M, int64_t K, int64_t N, const MidEpilogue &ep, void *stream) {
    constexpr int WAVES = 8, D = MR <= 4 ? 4 : 2;                  // D x MR x 4 registers hold the activations
    const int64_t tn = (N + 15) / 16, Kb = native_blocks_k(K);
    if (tn > 0x7FFFFFFF || Kb > (1 << 20)) return TMQ_ERR_TOO_LARGE;
    constexpr size_t lds = (size_t)WAVES * (1024 + 64) + (size_t)WAVES * MR * (1024 + 32);
    auto kernel = Kb / WAVES >= 2 * D ? stream32_kernel<WAVES, MR, D, true> : stream32_kernel<WAVES, MR, D, false>;
    hipLaunchKernelGGL(kernel, dim3((uint32_t)tn), dim3(64 * WAVES), lds, as_stream(stream), static_cast<const float *>(x),
                       static_cast<const u32x4 *>(native), M, K, (int)Kb, N, native_blocks_n(N), ep);
    return check_launch();
}

// Geometry: 64 x 128 tiles where they save a pass over the CUs (below); else the largest smaller tile
// that keeps most CUs busy; then as many wavefronts per tile as it takes to put about ten on every CU,
// each with at least two pairs to multiply.
template <class Rows, class Ep>
int dispatch(const Rows &rows, const void *native, int64_t M, int64_t K, int64_t N, const Ep &ep,
             void *stream) {
    const int64_t npairs = (K + 63) / 64, tn = (N + 63) / 64;
    // Whole weight blocks per wavefront (one 16-byte load per lane and block instead of four dword loads) when the
    // blocks deal out evenly (or there are many); else pairs (K = 4608 over 4 wavefronts: 18 blocks would leave two
    // wavefronts with five and two with four, which costs more than the loads save).
    // M = 256 at K = N = 4096: 14.5 -> 13.1 us, M = 128 at K = 8192: 15.2 -> 12.3 us.
    const int64_t Kb = native_blocks_k(K);
    auto by_blocks = [&](int waves) { return K % 256 == 0 && (Kb % waves == 0 || Kb >= 8 * waves); };
    // 64 x 128 tiles with four wavefronts read each activation row half as often (the weights are
    // 2 bits, so a wide tile is the cheap direction) but a pass over them takes ~1.7 times as long as
    // one over 64 x 64 tiles with eight wavefronts; both run one workgroup per CU. They win when they
    // save a whole pass: M = 512 at K = N = 4096 27.5 -> 23.9 us, the 512-channel 7 x 7 convolutions
    // of ResNet-18 33 -> 29.6 us; with a single pass of 64 x 64 tiles (M = 256) they lose.
    // Convolutions with a long reduction over one to two 64 x 64 tiles per CU: four wavefronts per tile, single pairs,
    // so that two workgroups share a CU (eight wavefronts with their double buffers fill its LDS alone) -- all tiles
    // are resident at once and a CU's second workgroup fills the gaps that the im2col address arithmetic leaves in the
    // first: the 512-channel 7 x 7 convolutions of ResNet-18 at batch 64 29.3 -> 26.6 us against the 64 x 128 tiles
    // below, 256 -> 512 channels at stride 2 18.5 -> 16.7, 1024 -> 512 channels 47.8 -> 43.8 (whole weight blocks per
    // wavefront lose here: 61 us). Dense problems of these sizes stay as they are (M = 512 at K = N = 4096: 24.0 us on
    // 64 x 128 tiles, 27.6 this way), and so do convolutions with fewer tiles (98 tiles: 27 us on smaller tiles, 56 so).
    constexpr bool kConv = Rows::kBuffer;
    if (kConv && npairs >= 16 && ((M + 63) / 64) * tn >= 256 && ((M + 63) / 64) * tn <= 512)
        return launch<4, 4, 4, Rows>(rows, native, M, K, N, ep, stream);
    {
        const int64_t tm = (M + 63) / 64, passes64 = (tm * tn + 255) / 256, passes128 = (tm * ((N + 127) / 128) + 255) / 256;
        if (npairs >= 16 && passes64 >= 2 && 17 * passes128 < 10 * passes64)
        {
            if (by_blocks(4)) return launch<4, 8, 4, Rows, true>(rows, native, M, K, N, ep, stream);
            // pairs two ahead (three LDS slots) once a wavefront has six or more: K = 4608 at M = 512, N = 4096
            // 25.9 -> 24.7 us, the 512-channel convolutions of ResNet-18 29.5 -> 29.2 us
            if (npairs >= 24) return launch<4, 8, 4, Rows, false, 3>(rows, native, M, K, N, ep, stream);
            return launch<4, 8, 4, Rows>(rows, native, M, K, N, ep, stream);
        }
    }
    // Otherwise the largest of 64 x 64, 32 x 64, 32 x 32, 16 x 32 that still gives most CUs a tile (measured
    // at K = N = 4096: M = 64 10.0 -> 7.6 us with 32 x 32, M = 17 9.7 -> 6.4 us with 16 x 32, while
    // M = 96 .. 128 stay best on 32 x 64).
    auto tiles = [&](int bm, int bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    int bm = 16, bn = 32;
    if (tiles(64, 64) >= 256) { bm = 64; bn = 64; }
    else if (tiles(32, 64) >= 192) { bm = 32; bn = 64; }
    else if (tiles(32, 32) >= 192) { bm = 32; bn = 32; }
    int waves = 1;
    while (waves < 8 && tiles(bm, bn) * waves < 2560 && npairs >= 4 * waves) waves *= 2;
    auto go = [&](auto wm_tag, auto wn_tag) {
        constexpr int WM = decltype(wm_tag)::value, WN = decltype(wn_tag)::value;
        if (by_blocks(waves)) {
            switch (waves) {
                case 1: return launch<WM, WN, 1, Rows, true>(rows, native, M, K, N, ep, stream);
                case 2: return launch<WM, WN, 2, Rows, true>(rows, native, M, K, N, ep, stream);
                case 4: return launch<WM, WN, 4, Rows, true>(rows, native, M, K, N, ep, stream);
                default: return launch<WM, WN, 8, Rows, true>(rows, native, M, K, N, ep, stream);
            }
        }
        switch (waves) {
            case 1: return launch<WM, WN, 1, Rows>(rows, native, M, K, N, ep, stream);
            case 2: return launch<WM, WN, 2, Rows>(rows, native, M, K, N, ep, stream);
            case 4: return launch<WM, WN, 4, Rows>(rows, native, M, K, N, ep, stream);
            default: return launch<WM, WN, 8, Rows>(rows, native, M, K, N, ep, stream);
        }
    };
    if (bm == 64) return go(std::integral_constant<int, 4>{}, std::integral_constant<int, 4>{});
    if (bn == 64) return go(std::integral_constant<int, 2>{}, std::integral_constant<int, 4>{});
    if (bm == 32) return go(std::integral_constant<int, 2>{}, std::integral_constant<int, 2>{});
    return go(std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{});
}

}  // namespace

// True when the staged split-reduction kernel can take a dense fp16 problem.
bool mid_dense_ok(const void *x, int64_t M, int64_t K) {
    return (K % 64 == 0) && aligned16(x) && M * K < (int64_t)0x7FFFFFFF;
}

int launch_mid_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                     const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream) {
    MidEpilogue ep{scale, bias, residual, y, relu, y_f16};
    return dispatch(DenseRows{static_cast<const _Float16 *>(x), M, K}, native, M, K, N, ep, stream);
}

// The same on M16 fp16 rows that are the hi / lo terms of rows_out fp32 rows in groups of eight (PairMap).
int launch_mid_dense_pairs(const void *x16, int64_t M16, int64_t K, const void *native, int64_t N, const float *scale,
                           const float *bias, const void *residual, int relu, void *y, int y_f16, int64_t rows_out,
                           const float *group_scale, void *stream) {
    MidEpilogueT<PairMap> ep{scale, bias, residual, y, relu, y_f16, PairMap{rows_out, group_scale}};
    return dispatch(DenseRows{static_cast<const _Float16 *>(x16), M16, K}, native, M16, K, N, ep, stream);
}

// True when the weight-stream kernel can take a dense fp16 problem of at most 16 rows.
bool stream_dense_ok(const void *x, int64_t M, int64_t K) {
    return M >= 1 && M <= 16 && (K % kKB == 0) && aligned16(x) && M * K < (int64_t)0x7FFFFFFF;
}

// fp32 rows with whole weight blocks that take the fp32 weight-stream kernel: up to 8, or up to 16 on short reductions.
bool stream32_dense_ok(const void *x, int64_t M, int64_t K) {
    // 9 .. 16 rows: the activations of two blocks (128 registers) only pay on short reductions -- measured faster
    // than the older kernel at K = 2048 .. 5120 (K = N = 4096, M = 16: 11.4 -> 9.2 us), slower at K >= 8192
    return M >= 1 && (M <= 8 || (M <= 16 && K <= 6144)) && (K % kKB == 0) && aligned16(x);
}

int launch_stream32_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                          const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream) {
    MidEpilogue ep{scale, bias, residual, y, relu, y_f16};
    if (M == 1) return launch_stream32<1>(x, native, M, K, N, ep, stream);
    if (M == 2) return launch_stream32<2>(x, native, M, K, N, ep, stream);
    if (M <= 4) return launch_stream32<4>(x, native, M, K, N, ep, stream);
    if (M <= 8) return launch_stream32<8>(x, native, M, K, N, ep, stream);
    return launch_stream32<16>(x, native, M, K, N, ep, stream);
}

// Geometry of the weight-stream kernel (stream_dense_ok must hold). Rows staged: the power of two >= M.
// What decides is that all workgroups are resident at once: a second, partly filled pass over the CUs
// costs more than running with fewer workgroups than CUs (N = 5120 at M = 16: 320 workgroups of one per CU
// 9.0 us, 160 twice as wide 6.1 us). Residency per CU follows from the LDS windows: 4 workgroups at R = 2,
// 2 at R = 4 and at R = 8 with two blocks in flight, 1 at R = 16 (2 with four wavefronts). So: the
// narrowest tile whose workgroups fit in one pass (narrow tiles mean more wavefronts streaming), measured
// on 4096 x {4096, 5120, 11008, 13824}, 8192 x {6144, 8192, 16384, 28672} and 16384^2.
static int stream_by_shape(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const MidEpilogue &ep,
                           void *stream, const RowPairs *pairs) {
    const int64_t Nb = native_blocks_n(N);
    if (M <= 2 && !pairs) return launch_stream<1, 8, 2, 4>(x, native, M, K, N, ep, stream, pairs);   // (a pair is added where four rows meet)
    if (M <= 4) {
        if (Nb >= 512) return launch_stream<2, 8, 4, 4>(x, native, M, K, N, ep, stream, pairs);
        return launch_stream<1, 8, 4, 4>(x, native, M, K, N, ep, stream, pairs);
    }
    if (M <= 8) {
        if (Nb <= 256) return launch_stream<1, 8, 8, 4>(x, native, M, K, N, ep, stream, pairs);
        if (Nb <= 1024) return launch_stream<2, 8, 8, 2>(x, native, M, K, N, ep, stream, pairs);
        return launch_stream<4, 8, 8, 2>(x, native, M, K, N, ep, stream, pairs);
    }
    if (Nb <= 256) return launch_stream<1, 8, 16, 2>(x, native, M, K, N, ep, stream, pairs);
    if (Nb <= 512) return launch_stream<2, 8, 16, 2>(x, native, M, K, N, ep, stream, pairs);
    if (Nb <= 1024) return launch_stream<4, 8, 16, 2>(x, native, M, K, N, ep, stream, pairs);
    return launch_stream<4, 4, 16, 2>(x, native, M, K, N, ep, stream, pairs);
}

int launch_stream_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                        const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream) {
    return stream_by_shape(x, M, K, native, N, MidEpilogue{scale, bias, residual, y, relu, y_f16}, stream, nullptr);
}

// M fp32 rows as 2 M fp16 rows (x16: the M hi terms, then the M lo terms; row_scale[m] undoes row m's power of two):
// one pass of the weight-stream kernel, the two sums of a row added in its epilogue. 2 <= 2 M <= 16.
int launch_stream_pairs(const void *x16, int64_t M, int64_t K, const void *native, int64_t N, const float *row_scale,
                        const float *scale, const float *bias, const void *residual, int relu, void *y, int y_f16,
                        void *stream) {
    const RowPairs pairs{(int)M, row_scale};
    return stream_by_shape(x16, 2 * M, K, native, N, MidEpilogue{scale, bias, residual, y, relu, y_f16}, stream, &pairs);
}

bool mid_conv_ok(const void *x, const tmq_conv_shape *s) {
    return (s->C % 64 == 0) && aligned16(x) && (int64_t)s->B * s->H * s->W * s->C < (int64_t)0x7FFFFFF0;
}

int launch_mid_conv(const void *x, const tmq_conv_shape *s, int ho, int wo, const void *native, const float *scale,
                    const float *bias, const void *residual, int relu, void *y, int y_f16, const RowMap *map, void *stream) {
    const int64_t M = (int64_t)s->B * ho * wo, K = (int64_t)s->C * s->ky * s->kx;
    const ConvRows rows{static_cast<const _Float16 *>(x), M, K, s->B, s->C, s->H, s->W, ho, wo, s->ky, s->kx, s->sy,
                        s->sx, s->py, s->px, s->dy, s->dx, FastDiv((uint32_t)wo), FastDiv((uint32_t)ho),
                        FastDiv((uint32_t)s->C), FastDiv((uint32_t)s->kx)};
    if (map) return dispatch(rows, native, M, K, s->N, MidEpilogueT<RowMap>{scale, bias, residual, y, relu, y_f16, *map}, stream);
    return dispatch(rows, native, M, K, s->N, MidEpilogue{scale, bias, residual, y, relu, y_f16, {}}, stream);
}

}  // namespace tmq
