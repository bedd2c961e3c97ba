// 17 .. 32 activation rows against a very large layer: the weights stream from HBM once, and the reduction is
// cut across workgroups (the caller brings a workspace for the partial sums).
//
// With this few rows a product over tens of MiB of packed weights is a weight stream first and a matrix product
// second. The kernels that split the reduction inside a workgroup give every wavefront an activation window of
// its own, which caps the weight bytes a CU can keep in flight at ~32 KiB; the tile kernels fetch one weight
// block ahead per wavefront, which comes to the same (both stream 16384 x 16384 weights at ~1.5 TB/s). Here:
//   * a workgroup of eight wavefronts owns all rows x 256 channels over a slice of the reduction; the wavefronts
//     split the CHANNELS (two 16-channel blocks each), so one activation window per 256 reduction indices serves
//     all of them: rows x 512 bytes, copied global -> LDS by buffer loads (16-byte chunks XOR-swizzled on the
//     global side, so the operand reads of 16 rows hit 16 different bank groups);
//   * every wavefront keeps four weight blocks per channel block in registers -- loads issued three
//     256-index steps ahead, 8 KiB per wavefront -- and the windows run just as far ahead (a ring of four): a
//     wavefront's loads complete in the order they were issued, so a window requested one step ahead would make
//     every step wait for the weight loads issued just before it;
//   * one barrier per 256 reduction indices; an expanded weight operand feeds two MFMAs;
//   * slice s of the reduction writes raw fp32 sums to partial[s][M][N]; a second launch adds the slices in
//     order and applies the epilogue (deterministic, no atomics).
// Measured (HIP-graph replays over rotating weight buffers): the loop streams at 2.9 TB/s, but the two launches,
// the simultaneous start of every workgroup and the partial sums (written and read once) cost a fixed ~12 us, so
// it only wins where the weights are 64 MiB or more: 16384 x 16384, 17 rows 38.3 -> 31-33 us, 32 rows 38.6 ->
// 34.6-35.5 us; 8192 x 8192, 32 rows 12.4 -> 18.1 us (not taken). A 64-row form (four windows of 64 rows: one
// workgroup per CU) ran at 52 % of the MFMA peak in its loop and still lost to the single-launch kernel at every
// size tried (16384^2 44 -> 49.5 us, 8192^2 15.9 -> 23.5, 8192 x 28672 at 48 rows 41.5 -> 49-51); it is not kept.
// Cutting the reduction of tile_solo_kernel (gemm.hip) across workgroups the same way lost everywhere as well
// (64 rows at 16384^2 44.9 -> 47.8-48.5 us, 256 rows at 4096^2 13.2 -> 20.3, ResNet-18's 3 x 3 convolutions
// over 7 x 7 and 14 x 14 positions 28.0 -> 30.2-41.8 and 24.6 -> 31.2-39.9): that is not kept either.
#include "common.h"
#include "mfma.h"
#include "tile_epilogue.h"

#include <utility>

namespace tmq {

// gemm.hip: adds the slices of a split reduction and applies the epilogue
int launch_splitk_reduce(const float *partial, int slices, int64_t M, int64_t N, const Epilogue &ep, void *stream);

namespace {

constexpr int kRowsWaves = 8, kRowsWN = 2, kRowsRing = 4;          // wavefronts, channel blocks per wavefront, weight stages
constexpr int kRowsBN = kRowsWaves * kRowsWN * 16;                 // channels per workgroup

template <class F, int... I>
__device__ __forceinline__ void unrolled_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N_, class F>
__device__ __forceinline__ void unrolled(F &&f) {
    unrolled_impl(f, std::make_integer_sequence<int, N_>{});
}

// WM: row fragments of 16 (2: up to 32 rows).
template <int WM>
__global__ __launch_bounds__(64 * kRowsWaves, 2) void rows_split_kernel(const _Float16 *__restrict__ x, const u32x4 *__restrict__ native,
                                                                        int M, int64_t K, int Kb, int64_t N, int64_t Nb,
                                                                        int slice_blocks, float *__restrict__ partial) {
    constexpr int RM = 16 * WM, kWindow = RM * 512, kCopies = RM / 2 / kRowsWaves;   // bytes per window; 1 KiB copies per wavefront
    static_assert(RM / 2 % kRowsWaves == 0, "whole copies per wavefront");
    extern __shared__ __attribute__((aligned(16))) unsigned char window[];           // [kRowsRing][RM][512]
    const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    const int slice = blockIdx.y;
    const int kb0 = slice * slice_blocks;
    int nkb = Kb - kb0;                                            // weight blocks of this slice
    if (nkb > slice_blocks) nkb = slice_blocks;

    // this lane's chunk of each of the wavefront's copies: copy q moves rows 2 i, 2 i + 1 (i = wv + 8 q), lane l the
    // chunk that belongs at position l % 32 of row 2 i + l / 32
    const BufferResource rows = make_buffer_resource(x, (uint32_t)((int64_t)M * K * 2));
    uint32_t src[kCopies];
#pragma unroll
    for (int q = 0; q < kCopies; q++) {
        const int row = 2 * (wv + kRowsWaves * q) + (lane >> 5), c = (lane & 31) ^ (row & 15);
        src[q] = row < M ? (uint32_t)((int64_t)row * K * 2) + (uint32_t)c * 16u : kPastTheEnd;   // rows past M: zeros
    }
    auto copy_window = [&](int kb, int buf) {                      // block kb0 + kb of the rows -> window buf
        const uint32_t k2 = (uint32_t)(kb0 + (kb < nkb ? kb : nkb - 1)) * 512u;
#pragma unroll
        for (int q = 0; q < kCopies; q++)
            buffer_to_lds(rows, src[q] == kPastTheEnd ? kPastTheEnd : src[q] + k2,
                          window + buf * kWindow + (wv + kRowsWaves * q) * 1024);
    };

    const u32x4 *wp[kRowsWN];
#pragma unroll
    for (int j = 0; j < kRowsWN; j++) {
        int64_t nb = (int64_t)blockIdx.x * (kRowsWaves * kRowsWN) + wv * kRowsWN + j;
        if (nb >= Nb) nb = Nb - 1;                                 // finite bits, never stored
        wp[j] = native + (nb * Kb + kb0) * 64 + lane;
    }
    u32x4 w[kRowsRing][kRowsWN];
    auto load_weights = [&](int kb, auto stage) {
        constexpr int S = decltype(stage)::value;
        const int at = kb < nkb ? kb : nkb - 1;                    // past the slice: re-read its last block (multiplied by zero)
#pragma unroll
        for (int j = 0; j < kRowsWN; j++) w[S][j] = __builtin_nontemporal_load(wp[j] + (int64_t)at * 64);
    };

    floatx4 acc[WM][kRowsWN];
#pragma unroll
    for (int i = 0; i < WM; i++)
#pragma unroll
        for (int j = 0; j < kRowsWN; j++) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    // prologue: the first kRowsRing - 1 windows, then the first kRowsRing weight blocks
#pragma unroll
    for (int t = 0; t < kRowsRing - 1; t++) copy_window(t, t);
    unrolled<kRowsRing>([&](auto s) { load_weights(decltype(s)::value, s); });
    __builtin_amdgcn_sched_barrier(0);

    const unsigned char *rd = window + r16 * 512;                  // this lane's row of fragment 0
    const int rounds = (nkb + kRowsRing - 1) / kRowsRing;
    for (int rnd = 0; rnd < rounds; rnd++) {
        unrolled<kRowsRing>([&](auto sc) {
            constexpr int S = decltype(sc)::value;
            const int kb = rnd * kRowsRing + S;
            constexpr int buf = S;                                 // window kb lives in slot kb % kRowsRing
            // This wavefront's copies of window kb have landed. Loads complete in issue order, and behind those
            // copies it has issued, step by step: weights, window, weights, window, weights (in the first steps
            // the tail of the prologue, which is no less) -- 3 kRowsWN + 2 kCopies loads may stay outstanding.
            static_assert(3 * kRowsWN + 2 * kCopies < 16, "vmcnt immediate");
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0x0F70 | (3 * kRowsWN + 2 * kCopies));
            __builtin_amdgcn_s_waitcnt(0xC07F);                    // (its operand reads of the step before are done)
            __builtin_amdgcn_s_barrier();                          // ... and everybody's: the window read last is free
            __builtin_amdgcn_sched_barrier(0);
            copy_window(kb + kRowsRing - 1, (S + kRowsRing - 1) % kRowsRing);
            __builtin_amdgcn_sched_barrier(0);
            const uint32_t mask = kb < nkb ? 0xC000C000u : 0u;     // steps past the slice multiply by zero
            const unsigned char *base = rd + buf * kWindow;
#pragma unroll
            for (int d = 0; d < 4; d++)
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    half8 a[kRowsWN];
#pragma unroll
                    for (int j = 0; j < kRowsWN; j++) {
                        const uint32_t word = w[S][j][d];
                        u32x4 r;
                        r[0] = (word << (8 * s + 0)) & mask;
                        r[1] = (word << (8 * s + 2)) & mask;
                        r[2] = (word << (8 * s + 4)) & mask;
                        r[3] = (word << (8 * s + 6)) & mask;
                        a[j] = __builtin_bit_cast(half8, r);
                    }
                    const int pos = ((8 * d + 4 * s + g) ^ r16) * 16;
#pragma unroll
                    for (int i = 0; i < WM; i++) {
                        const half8 b = *reinterpret_cast<const half8 *>(base + i * (16 * 512) + pos);
#pragma unroll
                        for (int j = 0; j < kRowsWN; j++) acc[i][j] = mfma16(a[j], b, acc[i][j]);
                    }
                }
            __builtin_amdgcn_sched_barrier(0);
            load_weights(kb + kRowsRing, sc);                      // this stage's registers are free again
        });
    }
    // the requests past the slice (repeats of its last block) must have landed before the LDS can go to another workgroup
    __builtin_amdgcn_s_waitcnt(0x0F70);
    float *out = partial + (int64_t)slice * M * N;
#pragma unroll
    for (int j = 0; j < kRowsWN; j++) {
        const int64_t n = ((int64_t)blockIdx.x * (kRowsWaves * kRowsWN) + wv * kRowsWN + j) * 16 + 4 * g;
        if (n >= N) continue;                                      // N is a multiple of 16: whole groups of four
#pragma unroll
        for (int i = 0; i < WM; i++) {
            const int m = 16 * i + r16;
            if (m < M) *reinterpret_cast<floatx4 *>(out + (int64_t)m * N + n) = acc[i][j] * (1.0f / kWeightUnit);
        }
    }
}

}  // namespace

// Slices of the reduction for M rows over K x N weights, or 0 when this kernel does not apply / does not pay
// (measured against the split-reduction kernel of mid.hip, which takes these shapes without a workspace).
int rows_split_slices(const void *x, int64_t M, int64_t K, int64_t N) {
    if (M < 17 || M > 32 || K % kKB != 0 || N % 16 != 0 || !aligned16(x)) return 0;
    if (K < 16 * kKB || (double)K * (double)N < 268435456.0 || M * K * 2 >= (int64_t)kPastTheEnd - 16) return 0;
    const int64_t Kb = K / kKB, chunks = (N + kRowsBN - 1) / kRowsBN;
    // about as many workgroups as fit at once (two per CU), slices of whole rounds of kRowsRing blocks, at
    // least two rounds each
    int64_t slices = (512 + chunks - 1) / chunks;
    int64_t blocks = (Kb + slices - 1) / slices;
    blocks = (blocks + kRowsRing - 1) / kRowsRing * kRowsRing;
    if (blocks < 2 * kRowsRing) blocks = 2 * kRowsRing;
    slices = (Kb + blocks - 1) / blocks;
    return slices >= 2 ? (int)slices : 0;
}

int launch_rows_split(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const Epilogue &ep, float *partial,
                      int slices, void *stream) {
    const int64_t Kb = K / kKB, Nb = native_blocks_n(N), chunks = (N + kRowsBN - 1) / kRowsBN;
    int64_t blocks = (Kb + slices - 1) / slices;
    blocks = (blocks + kRowsRing - 1) / kRowsRing * kRowsRing;
    if (blocks < 2 * kRowsRing) blocks = 2 * kRowsRing;
    if (M > 32 || (Kb + blocks - 1) / blocks != slices || chunks > 0x7FFFFFFF || slices > 65535) return TMQ_ERR_INVALID_ARG;
    const dim3 grid((uint32_t)chunks, (uint32_t)slices);
    const size_t lds = kRowsRing * 32 * 512;
    hipLaunchKernelGGL(rows_split_kernel<2>, grid, dim3(64 * kRowsWaves), lds, as_stream(stream), static_cast<const _Float16 *>(x),
                       static_cast<const u32x4 *>(native), (int)M, K, (int)Kb, N, Nb, (int)blocks, partial);
    const int rc = check_launch();
    if (rc != TMQ_OK) return rc;
    return launch_splitk_reduce(partial, slices, M, N, ep, stream);
}

}  // namespace tmq
