// Ternary linear layers on gfx950: y[m][n] = scale[n] * sum_k x[m][k] * T[k][n] + bias[n].
//
//   prepack_kernel    : reference packing words[K][ceil(N/16)] -> kernel-native blocks (mfma.h)
//   skinny_kernel     : M <= 64 rows of any shape and type (fp32 activations, ragged K, unaligned rows).
//                       Bound by streaming the 2-bit weights: every wavefront fetches 1 KiB weight blocks
//                       with one coalesced dwordx4 load, expands them in registers to exact +-2/0 fp16
//                       MFMA operands (two VALU ops per register), and contracts with the activations on
//                       v_mfma_f32_16x16x32_f16 (fp32 accumulate). K is split over the wavefronts of a
//                       workgroup and reduced through LDS in a fixed order (deterministic).
//   gemv_short_kernel, short_rows_kernel : M = 1 / 2..16 fp16 rows with K < 2048: everything in flight at once
//   mid_kernel, mid_lds_kernel : older split-reduction kernels, kept for what mid.hip does not take
//                       (K % 64 != 0, unaligned rows, fp32 activations)
//   split_terms_kernel : fp32 -> two fp16 terms, for the two-pass route of fp32 activations
//   tmq_ternary_linear : the dispatch. fp16 rows with whole blocks go to mid.hip (weight-stream kernel up to
//                       16 rows, split-reduction kernel for few output tiles) or gemm.hip (MFMA-bound tiles).
#include "common.h"
#include "mfma.h"

namespace tmq {

// gemm.hip: the MFMA-bound tile kernels for large M (fp16 activations)
int launch_gemm_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                      const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream);
// mid.hip: staged split-reduction kernel for mid-size fp16 problems
bool mid_dense_ok(const void *x, int64_t M, int64_t K);
bool stream_dense_ok(const void *x, int64_t M, int64_t K);
bool stream32_dense_ok(const void *x, int64_t M, int64_t K);
int launch_stream32_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                          const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream);
int launch_stream_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                        const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream);
int launch_mid_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                     const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream);
// gemv8.hip: one fp16 row on the 8-bit matrix instructions
bool gemv8_dense_ok(const void *x, int64_t M, int64_t K, int64_t N);
int launch_gemv8_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale, const float *bias,
                       const void *residual, int relu, void *y, int y_f16, void *stream);
bool gemv8_planes_ok(int64_t M, int64_t K);
int64_t gemv8_padded_rows(int64_t M);
int launch_gemv8_planes(const void *planes, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                        const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream);
int launch_gemv8_prepare(const void *x, int64_t M, int64_t K, void *planes, void *stream);
bool gemv8_dense32_ok(const void *x, int64_t M, int64_t K, int64_t N);
int launch_gemv8_dense32(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale, const float *bias,
                         const void *residual, int relu, void *y, int y_f16, void *stream);

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

template <bool X32>
__device__ __forceinline__ XFrag<X32> load_x(const void *x, int64_t m, int64_t M, int64_t K, int64_t k, bool vec) {
    XFrag<X32> f;
    f.hi = half8{0, 0, 0, 0, 0, 0, 0, 0};
    f.lo = f.hi;
    if (m >= M || k >= K) return f;
    if constexpr (!X32) {
        const _Float16 *p = static_cast<const _Float16 *>(x) + m * K + k;
        if (vec && k + 8 <= K) {
            f.hi = *reinterpret_cast<const half8 *>(p);
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (k + e < K) f.hi[e] = p[e];
        }
    } else {
        const float *p = static_cast<const float *>(x) + m * K + k;
        float v[8];
        if (vec && k + 8 <= K) {
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
// A workgroup of `waves` wavefronts owns GW consecutive blocks of 16 output channels. Wavefront w
// works on channel block (w % GW) and, of it, on the weight blocks kb = w / GW, w / GW + waves / GW,
// ... MT = number of 16-row activation tiles (M <= 16 MT). D[n][m]: the weights are the A operand of
// the MFMA.
//
// The kernel is a weight stream; besides HBM two things bound it:
//   * bytes in flight: every wavefront keeps kAhead 1 KiB blocks outstanding in a rolling pipeline
//     (a block's registers are reloaded as soon as it has been consumed);
//   * VALU: two operations per operand register to expand the 2-bit codes -- nothing else is left
//     in the inner loop. XLDS: the activations are staged once per workgroup in LDS, fp32
//     activations already split into their two fp16 terms, zero-padded to whole weight blocks, so an
//     operand read is one ds_read_b128 at (lane base + block offset + immediate) with no edge cases.
// Lanes whose activation row does not exist (m >= M) read row M - 1: columns of D are independent,
// and those columns are never stored.
constexpr size_t kSkinnyLdsMax = 152 * 1024;
constexpr int kAhead = 4;

template <int MT, bool X32, bool XLDS>
__global__ __launch_bounds__(1024) void skinny_kernel(const void *__restrict__ x, int64_t M, int64_t K, int vec,
                                                      const u32x4 *__restrict__ native, int Kb, int64_t N, int64_t Nb,
                                                      int GW, const float *__restrict__ scale,
                                                      const float *__restrict__ bias, const void *__restrict__ residual,
                                                      int relu, void *__restrict__ y, int y_f16) {
    constexpr int kPlanes = X32 ? 2 : 1;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // the wavefront index is uniform: telling the compiler keeps the loop control in scalar registers
    const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), waves = blockDim.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int sub = wv % GW, ks = wv / GW, nks = waves / GW;
    const int64_t nb0 = (int64_t)blockIdx.x * GW + sub;
    const bool valid = nb0 < Nb;
    const int pitch = (Kb * kKB + 8) * 2;                              // bytes per staged activation row
    const size_t plane = (size_t)M * pitch;
    floatx4 *slot = reinterpret_cast<floatx4 *>(smem + (XLDS ? kPlanes * plane : 0));

    // The first GW wavefronts run the epilogue of one channel block each; its constants are fetched
    // now so that their latency hides behind the weight stream.
    float sc4[4] = {1.f, 1.f, 1.f, 1.f}, bi4[4] = {0.f, 0.f, 0.f, 0.f};
    if (wv < GW && valid) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t n = nb0 * 16 + g * 4 + r;
            if (n < N) {
                if (scale) sc4[r] = scale[n];
                if (bias) bi4[r] = bias[n];
            }
        }
    }

    floatx4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

    const u32x4 *wb = native + (valid ? nb0 * Kb : 0) * 64 + lane;
    const int nt = valid && Kb > ks ? (Kb - ks + nks - 1) / nks : 0;   // weight blocks of this wavefront

    // Prologue loads. A long stream issues them unconditionally: only then can the compiler count the
    // loads behind the one it waits for in the steady-state loop below.
    u32x4 cur[kAhead];
    auto fetch = [&](int u, int t) { cur[u] = __builtin_nontemporal_load(wb + (ks + t * nks) * 64); };
    const bool steady = nt >= 2 * kAhead;
    if (steady) {
#pragma unroll
        for (int u = 0; u < kAhead; u++) fetch(u, u);
    } else {
#pragma unroll
        for (int u = 0; u < kAhead; u++)
            if (u < nt) fetch(u, u);
    }

    // per-lane operand base (row m, or the last row for lanes past M)
    const unsigned char *xl[MT];
    if constexpr (XLDS) {
        const int cpr = Kb * (kKB / 8), total = (int)M * cpr;          // 8-element chunks per row, in all
        // four chunks per pass: the loads of a pass are all issued before its LDS stores
        constexpr int kBatch = 4;
        for (int id0 = threadIdx.x; id0 < total; id0 += kBatch * blockDim.x) {
            XFrag<X32> f[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; u++) {
                const int id = id0 + u * blockDim.x, row = id / cpr, c = id - row * cpr;
                f[u] = load_x<X32>(x, id < total ? row : M, M, K, (int64_t)c * 8, vec);   // past the end: zeros, not stored
            }
#pragma unroll
            for (int u = 0; u < kBatch; u++) {
                const int id = id0 + u * blockDim.x, row = id / cpr, c = id - row * cpr;
                if (id < total) {
                    *reinterpret_cast<half8 *>(smem + (size_t)row * pitch + c * 16) = f[u].hi;
                    if constexpr (X32) *reinterpret_cast<half8 *>(smem + plane + (size_t)row * pitch + c * 16) = f[u].lo;
                }
            }
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const int m = t * 16 + j;
            xl[t] = smem + (size_t)(m < M ? m : (int)M - 1) * pitch + g * 16;
        }
        __syncthreads();
    }

    // One weight block against the activations: 8 MFMA steps of 32 reduction indices.
    auto contract = [&](const u32x4 &wq, int kb) {
        if constexpr (XLDS && MT == 1) {
            // all operand reads of the block are issued ahead of the decode work
            const unsigned char *xp = xl[0] + kb * (kKB * 2);
            half8 xv[8], xw[X32 ? 8 : 1];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                xv[i] = *reinterpret_cast<const half8 *>(xp + i * 64);
                if constexpr (X32) xw[i] = *reinterpret_cast<const half8 *>(xp + plane + i * 64);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const half8 a = decode_step(wq[i >> 1], i & 1);
                acc[0] = mfma16(a, xv[i], acc[0]);
                if constexpr (X32) acc[0] = mfma16(a, xw[i], acc[0]);
            }
        } else if constexpr (XLDS) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const half8 a = decode_step(wq[i >> 1], i & 1);
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const unsigned char *xp = xl[t] + kb * (kKB * 2) + i * 64;
                    acc[t] = mfma16(a, *reinterpret_cast<const half8 *>(xp), acc[t]);
                    if constexpr (X32) acc[t] = mfma16(a, *reinterpret_cast<const half8 *>(xp + plane), acc[t]);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int64_t k0 = (int64_t)kb * kKB + i * 32;
                if (k0 >= K) continue;   // wave-uniform
                const half8 a = decode_step(wq[i >> 1], i & 1);
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const XFrag<X32> xf = load_x<X32>(x, t * 16 + j, M, K, k0 + g * 8, vec);
                    acc[t] = mfma16(a, xf.hi, acc[t]);
                    if constexpr (X32) acc[t] = mfma16(a, xf.lo, acc[t]);
                }
            }
        }
    };

    // Steady state: every slot is consumed and refilled unconditionally, so the number of loads
    // behind the one being waited for is known at compile time.
    int t0 = 0;
    if (steady) {
        // Start from a known state (nothing outstanding): paths that skipped the staging waits above
        // would otherwise make the compiler wait for every load at the loop header.
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        do {
#pragma unroll
            for (int u = 0; u < kAhead; u++) {
                contract(cur[u], ks + (t0 + u) * nks);
                __builtin_amdgcn_sched_barrier(0);   // keep the refill here, not batched at the loop end
                fetch(u, t0 + kAhead + u);
                __builtin_amdgcn_sched_barrier(0);
            }
            t0 += kAhead;
        } while (t0 + 2 * kAhead <= nt);
    }
    // Drain: at most two rounds with wave-uniform guards.
    for (; t0 < nt; t0 += kAhead) {
#pragma unroll
        for (int u = 0; u < kAhead; u++) {
            if (t0 + u < nt) contract(cur[u], ks + (t0 + u) * nks);
            if (t0 + kAhead + u < nt) fetch(u, t0 + kAhead + u);
        }
    }

    // Cross-wave reduction in wave order, then the epilogue. Lane slot (w, t, lane) holds
    // y[m = 16 t + j][n = 16 nb + 4 g + r], r = 0..3, of wavefront w's channel block.
#pragma unroll
    for (int t = 0; t < MT; t++) slot[(wv * MT + t) * 64 + lane] = acc[t];
    __syncthreads();
    if (wv < GW && valid) {
        const int64_t nb = nb0;
        for (int t = 0; t < MT; t++) {
            floatx4 s = slot[(wv * MT + t) * 64 + lane];
            for (int w = wv + GW; w < waves; w += GW) {
                const floatx4 p = slot[(w * MT + t) * 64 + lane];
                s[0] += p[0]; s[1] += p[1]; s[2] += p[2]; s[3] += p[3];
            }
            const int64_t m = t * 16 + j, n0 = nb * 16 + g * 4;
            if (m >= M) continue;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int64_t n = n0 + r;
                if (n < N) {
                    float v = s[r] * (sc4[r] * (1.0f / kWeightUnit)) + bi4[r];
                    const int64_t o = m * N + n;
                    if (y_f16) {
                        if (residual) v += (float)static_cast<const _Float16 *>(residual)[o];
                        if (relu) v = v < 0.f ? 0.f : v;
                        static_cast<_Float16 *>(y)[o] = (_Float16)v;
                    } else {
                        if (residual) v += static_cast<const float *>(residual)[o];
                        if (relu) v = v < 0.f ? 0.f : v;
                        static_cast<float *>(y)[o] = v;
                    }
                }
            }
        }
    }
}

// ---- short GEMV -------------------------------------------------------------------------------------
// M = 1 with at most two weight blocks per wavefront (K <= 8192 at 16 wavefronts): the whole job of a
// wavefront is in flight at once -- its weight blocks and the 512 bytes of the activation vector that
// go with each of them -- so a launch costs one trip to memory and no barrier before the arithmetic.
// Lane (j, g) supplies column j of the B operand; only column 0 is stored, so every lane uses the
// vector's chunk g of each step. The wavefront fetches its 512 bytes with ONE load (8 bytes per lane)
// and passes them through its own LDS row, from which the eight operand reads are broadcasts: eight
// global loads per lane instead cost the CU's address unit 16 cycles each for 64 bytes of payload,
// ~0.5 us per launch at 16 wavefronts (measured: 4.47 -> 3.95 us).
// Requires fp16 activations, K % 256 == 0, 16-byte aligned x.
__global__ __launch_bounds__(1024) void gemv_short_kernel(const _Float16 *__restrict__ x, const u32x4 *__restrict__ native,
                                                          int Kb, int64_t N, const float *__restrict__ scale,
                                                          const float *__restrict__ bias, const void *__restrict__ residual,
                                                          int relu, void *__restrict__ y, int y_f16) {
    __shared__ floatx4 slot[16 * 64];
    __shared__ __attribute__((aligned(16))) _Float16 xs[16][2][kKB + 8];   // +8: rows of one wavefront on different banks
    const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), waves = blockDim.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int64_t nb = blockIdx.x;
    const bool two = wv + waves < Kb;
    const u32x4 *wp = native + (nb * Kb + wv) * 64 + lane;
    const _Float16 *xp = x + (int64_t)wv * kKB + lane * 4;
    u32x4 w0 = __builtin_nontemporal_load(wp), w1 = {0u, 0u, 0u, 0u};
    u32x2 xa = *reinterpret_cast<const u32x2 *>(xp), xb = {0u, 0u};
    if (two) {
        w1 = __builtin_nontemporal_load(wp + (int64_t)waves * 64);
        xb = *reinterpret_cast<const u32x2 *>(xp + (int64_t)waves * kKB);
    }
    *reinterpret_cast<u32x2 *>(&xs[wv][0][lane * 4]) = xa;
    if (two) *reinterpret_cast<u32x2 *>(&xs[wv][1][lane * 4]) = xb;
    __builtin_amdgcn_wave_barrier();
    half8 x0[8], x1[8];
#pragma unroll
    for (int i = 0; i < 8; i++) x0[i] = *reinterpret_cast<const half8 *>(&xs[wv][0][i * 32 + g * 8]);
    if (two) {
#pragma unroll
        for (int i = 0; i < 8; i++) x1[i] = *reinterpret_cast<const half8 *>(&xs[wv][1][i * 32 + g * 8]);
    }
    float sc4[4] = {1.f, 1.f, 1.f, 1.f}, bi4[4] = {0.f, 0.f, 0.f, 0.f};
    if (wv == 0) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t n = nb * 16 + g * 4 + r;
            if (n < N) {
                if (scale) sc4[r] = scale[n];
                if (bias) bi4[r] = bias[n];
            }
        }
    }
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 8; i++) acc = mfma16(decode_step(w0[i >> 1], i & 1), x0[i], acc);
    if (two) {
#pragma unroll
        for (int i = 0; i < 8; i++) acc = mfma16(decode_step(w1[i >> 1], i & 1), x1[i], acc);
    }
    // only column 0 (lanes j == 0) carries the result: 4 lanes x 4 channels per wavefront
    if (j == 0) slot[wv * 4 + g] = acc;
    __syncthreads();
    if (wv == 0 && j == 0) {
        floatx4 s = slot[g];
        for (int w = 1; w < waves; w++) {
            const floatx4 p = slot[w * 4 + g];
            s[0] += p[0]; s[1] += p[1]; s[2] += p[2]; s[3] += p[3];
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t n = nb * 16 + g * 4 + r;
            if (n < N) {
                float v = s[r] * (sc4[r] * (1.0f / kWeightUnit)) + bi4[r];
                if (y_f16) {
                    if (residual) v += (float)static_cast<const _Float16 *>(residual)[n];
                    if (relu) v = v < 0.f ? 0.f : v;
                    static_cast<_Float16 *>(y)[n] = (_Float16)v;
                } else {
                    if (residual) v += static_cast<const float *>(residual)[n];
                    if (relu) v = v < 0.f ? 0.f : v;
                    static_cast<float *>(y)[n] = v;
                }
            }
        }
    }
}

// ---- short reductions, up to 16 rows -----------------------------------------------------------------
// The same plan as gemv_short_kernel for 2 <= M <= 16 (one row tile): a wavefront owns one or two weight
// blocks and fetches, together with them, its own 512-byte slice of every activation row -- two rows per
// 16-byte-per-lane load -- into a private LDS window. No workgroup-wide staging of all of x and no
// barrier before the arithmetic: a launch is one trip to memory, the MFMAs, one reduction.
// Rows of a window are 528 bytes apart (512 + 16) to spread the operand reads of 16 rows over the banks.
// Requires fp16 activations, K % 256 == 0, 16-byte aligned x, at most two blocks per wavefront.
constexpr int kShortRowPitch = kKB * 2 + 16;

__global__ __launch_bounds__(1024) void short_rows_kernel(const _Float16 *__restrict__ x, int M, int64_t K,
                                                          const u32x4 *__restrict__ native, int Kb, int64_t N,
                                                          const float *__restrict__ scale, const float *__restrict__ bias,
                                                          const void *__restrict__ residual, int relu, void *__restrict__ y,
                                                          int y_f16) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), waves = blockDim.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int64_t nb = blockIdx.x;
    const bool two = wv + waves < Kb;
    const int win_bytes = M * kShortRowPitch;                       // one block's window
    floatx4 *slot = reinterpret_cast<floatx4 *>(smem);               // [waves][64] partial sums, then the windows
    unsigned char *win = smem + waves * 64 * sizeof(floatx4) + (size_t)wv * (Kb > waves ? 2 : 1) * win_bytes;

    const u32x4 *wp = native + (nb * Kb + wv) * 64 + lane;
    u32x4 w0 = __builtin_nontemporal_load(wp), w1 = {0u, 0u, 0u, 0u};
    if (two) w1 = __builtin_nontemporal_load(wp + (int64_t)waves * 64);
    // lane -> (row r0 + lane / 32, 16-byte chunk lane % 32) of the slice; rows past M repeat the last one
    const int lr = lane >> 5, lc = lane & 31;
    for (int r0 = 0; r0 < M; r0 += 2) {
        const int r = r0 + lr < M ? r0 + lr : M - 1;
        const _Float16 *src = x + (int64_t)r * K + (int64_t)wv * kKB + lc * 8;
        const u32x4 a = *reinterpret_cast<const u32x4 *>(src);
        u32x4 b = {0u, 0u, 0u, 0u};
        if (two) b = *reinterpret_cast<const u32x4 *>(src + (int64_t)waves * kKB);
        *reinterpret_cast<u32x4 *>(win + r * kShortRowPitch + lc * 16) = a;
        if (two) *reinterpret_cast<u32x4 *>(win + win_bytes + r * kShortRowPitch + lc * 16) = b;
    }
    float sc4[4] = {1.f, 1.f, 1.f, 1.f}, bi4[4] = {0.f, 0.f, 0.f, 0.f};
    if (wv == 0) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t n = nb * 16 + g * 4 + r;
            if (n < N) {
                if (scale) sc4[r] = scale[n];
                if (bias) bi4[r] = bias[n];
            }
        }
    }
    __builtin_amdgcn_wave_barrier();
    // B operand: lane (j, g) supplies row j (rows past M: the last row, never stored)
    const unsigned char *xr = win + (j < M ? j : M - 1) * kShortRowPitch + g * 16;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    {
        half8 xv[8];
#pragma unroll
        for (int i = 0; i < 8; i++) xv[i] = *reinterpret_cast<const half8 *>(xr + i * 64);
#pragma unroll
        for (int i = 0; i < 8; i++) acc = mfma16(decode_step(w0[i >> 1], i & 1), xv[i], acc);
    }
    if (two) {
        half8 xv[8];
#pragma unroll
        for (int i = 0; i < 8; i++) xv[i] = *reinterpret_cast<const half8 *>(xr + win_bytes + i * 64);
#pragma unroll
        for (int i = 0; i < 8; i++) acc = mfma16(decode_step(w1[i >> 1], i & 1), xv[i], acc);
    }
    // lane (j, g) holds y[m = j][n = 16 nb + 4 g + r], r = 0..3, of this wavefront's share of K
    slot[wv * 64 + lane] = acc;
    __syncthreads();
    if (wv == 0 && j < M) {
        floatx4 s = slot[lane];
        for (int w = 1; w < waves; w++) {
            const floatx4 p = slot[w * 64 + lane];
            s[0] += p[0]; s[1] += p[1]; s[2] += p[2]; s[3] += p[3];
        }
        const int64_t n0 = nb * 16 + g * 4;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t n = n0 + r;
            if (n < N) {
                float v = s[r] * (sc4[r] * (1.0f / kWeightUnit)) + bi4[r];
                const int64_t o = (int64_t)j * N + n;
                if (y_f16) {
                    if (residual) v += (float)static_cast<const _Float16 *>(residual)[o];
                    if (relu) v = v < 0.f ? 0.f : v;
                    static_cast<_Float16 *>(y)[o] = (_Float16)v;
                } else {
                    if (residual) v += static_cast<const float *>(residual)[o];
                    if (relu) v = v < 0.f ? 0.f : v;
                    static_cast<float *>(y)[o] = v;
                }
            }
        }
    }
}

struct SkinnyArgs {
    const void *x;
    int64_t M, K;
    int vec;
    const u32x4 *native;
    int Kb;
    int64_t N, Nb;
    int GW;
    const tmq_epilogue *ep;
    void *y;
};

template <int MT, bool X32, bool XLDS>
int launch_skinny_as(dim3 grid, dim3 block, size_t lds, void *stream, const SkinnyArgs &a) {
    auto kernel = skinny_kernel<MT, X32, XLDS>;
    if (lds > 64 * 1024) {
        if (int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), kSkinnyLdsMax)) return st;
    }
    const tmq_epilogue &ep = *a.ep;
    const float *scale = ep.scale, *bias = ep.bias;
    const void *residual = ep.residual;
    const int relu = ep.relu, y_f16 = ep.y_dtype == TMQ_F16;
    hipLaunchKernelGGL(kernel, grid, block, lds, as_stream(stream), a.x, a.M, a.K, a.vec, a.native, a.Kb, a.N, a.Nb,
                       a.GW, scale, bias, residual, relu, a.y, y_f16);
    return check_launch();
}

template <int MT, bool X32>
int launch_skinny(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const tmq_epilogue &ep,
                  void *y, void *stream) {
    const int64_t Nb = native_blocks_n(N), Kb = native_blocks_k(K);
    if (Kb > (1 << 20)) return TMQ_ERR_TOO_LARGE;
    if constexpr (MT == 1 && !X32) {
        if (M == 1 && K % kKB == 0 && Kb <= 32 && aligned16(x) && Nb <= 0x7FFFFFFF) {
            int waves = Kb > 16 ? 16 : 8;            // two blocks per wavefront already at K = 4096: half the partial sums
            while (waves > Kb) waves >>= 1;
            if (Kb <= 2 * waves) {
                hipLaunchKernelGGL(gemv_short_kernel, dim3((uint32_t)Nb), dim3(64 * waves), 0, as_stream(stream),
                                   static_cast<const _Float16 *>(x), static_cast<const u32x4 *>(native), (int)Kb, N,
                                   ep.scale, ep.bias, ep.residual, ep.relu, y, ep.y_dtype == TMQ_F16);
                return check_launch();
            }
        }
    }
    if constexpr (MT == 1 && !X32) {
        // 2 .. 16 rows with at most two weight blocks per wavefront: private windows instead of staging all of x
        // (M = 16 at K = N = 4096: 7.4 -> 5.6 us; M = 2 .. 8: 5.5-5.9 -> 4.3-4.8 us)
        if (M >= 2 && K % kKB == 0 && Kb <= 32 && aligned16(x) && Nb <= 0x7FFFFFFF) {
            int waves = Kb > 16 ? 16 : 8;
            while (waves > Kb) waves >>= 1;
            const int per_wave = Kb > waves ? 2 : 1;      // windows (weight blocks) per wavefront
            const size_t lds = (size_t)waves * 64 * sizeof(floatx4) + (size_t)waves * per_wave * M * kShortRowPitch;
            if (Kb <= 2 * waves && lds <= kSkinnyLdsMax) {
                if (lds > 64 * 1024) {
                    if (int st = allow_dynamic_lds(reinterpret_cast<const void *>(short_rows_kernel), kSkinnyLdsMax)) return st;
                }
                hipLaunchKernelGGL(short_rows_kernel, dim3((uint32_t)Nb), dim3(64 * waves), lds, as_stream(stream),
                                   static_cast<const _Float16 *>(x), (int)M, K, static_cast<const u32x4 *>(native), (int)Kb, N,
                                   ep.scale, ep.bias, ep.residual, ep.relu, y, ep.y_dtype == TMQ_F16);
                return check_launch();
            }
        }
    }
    // Geometry: 16 wavefronts where the reduction slots allow; short reductions give their spare
    // wavefronts to more channel blocks (GW) as long as >= 256 workgroups remain, else shrink.
    int waves = 16, GW = 1;
    while (waves * MT > 32) waves >>= 1;
    while (waves / GW > Kb && waves / GW > 1) {
        if (Nb >= 512 * (int64_t)GW) GW <<= 1;
        else waves >>= 1;
    }
    const size_t xbytes = (size_t)(X32 ? 2 : 1) * (size_t)M * (size_t)(Kb * kKB + 8) * 2;
    const bool xlds = xbytes + (size_t)waves * MT * 64 * sizeof(floatx4) <= kSkinnyLdsMax;
    // Wide single-tile layers: half-size workgroups that own two channel blocks each. Several of
    // them fit a CU, so one group's staging and reduction overlap another's streaming (measured best
    // among {4, 8, 16} wavefronts x {1, 2, 4} blocks at 8192^2 .. 32768 x 16384), and each group
    // stages the activations for twice the weights.
    if (MT == 1 && xlds && waves == 16 && GW == 1 && Nb >= 512 && Kb >= 32) { waves = 8; GW = 2; }
    const size_t red = (size_t)waves * MT * 64 * sizeof(floatx4);
    const int64_t wgs = (Nb + GW - 1) / GW;
    if (wgs > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    dim3 grid((uint32_t)wgs), block(64 * waves);
    const SkinnyArgs a{x, M, K, (K % 8 == 0) && aligned16(x), static_cast<const u32x4 *>(native), (int)Kb, N, Nb, GW, &ep, y};
    if (!xlds) return launch_skinny_as<MT, X32, false>(grid, block, red, stream, a);
    return launch_skinny_as<MT, X32, true>(grid, block, xbytes + red, stream, a);
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

// ---- mid kernel -----------------------------------------------------------------------------------
// Batches between the skinny case and the big-tile GEMM (64 < M <~ 2048): too few output tiles to
// fill 256 CUs with large tiles, too many rows to stage in LDS. A workgroup of 16 wavefronts owns a
// (16 WM WGM) x (16 WN) output tile and splits the reduction over its wavefronts: wavefront
// (wgm, kg) multiplies rows [16 WM wgm, +16 WM) by the weight blocks kb = kg, kg + KG, ...
// (KG = 16 / WGM). Both operands come straight from global memory -- the weights as whole 1 KiB
// native blocks (one coalesced dwordx4 per block), the activations as 16-byte row pieces two MFMA
// steps ahead of their use -- and the partial tiles are summed through LDS in a fixed order, so the
// result does not depend on scheduling. No activation byte is read twice by a workgroup.
//
// FAST: K is a multiple of 256 and rows are 16-byte aligned (no edge handling in the loop; rows past
// M are clamped to the last row, their columns of D are never stored).
template <int WM, int WN, int WGM, int WAVES, int D, bool X32, bool FAST>
__global__ __launch_bounds__(64 * WAVES) void mid_kernel(const void *__restrict__ x, int64_t M, int64_t K,
                                                   const u32x4 *__restrict__ native, int Kb, int64_t N, int64_t Nb,
                                                   int tiles_n, const float *__restrict__ scale,
                                                   const float *__restrict__ bias, const void *__restrict__ residual,
                                                   int relu, void *__restrict__ y, int y_f16) {
    constexpr int KG = WAVES / WGM, NF = WM * WN;
    static_assert(8 % D == 0, "the window must divide a weight block");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    floatx4 *red = reinterpret_cast<floatx4 *>(smem);
    const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, g = lane >> 4;
    const int wgm = wv % WGM, kg = wv / WGM;
    const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
    const int64_t mw = ((int64_t)tm * WGM + wgm) * (16 * WM);      // first row of this wavefront
    const int64_t n0 = (int64_t)tn * (16 * WN);

    // epilogue constants of the first fragment this wavefront finalises (fragment kg), fetched early
    float sc4[4] = {1.f, 1.f, 1.f, 1.f}, bi4[4] = {0.f, 0.f, 0.f, 0.f};
    auto load_consts = [&](int f) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t n = n0 + (f % WN) * 16 + g * 4 + r;
            sc4[r] = (n < N && scale) ? scale[n] : 1.f;
            bi4[r] = (n < N && bias) ? bias[n] : 0.f;
        }
    };
    if (kg < NF) load_consts(kg);

    floatx4 acc[WM][WN];
#pragma unroll
    for (int mi = 0; mi < WM; mi++)
#pragma unroll
        for (int nj = 0; nj < WN; nj++) acc[mi][nj] = floatx4{0.f, 0.f, 0.f, 0.f};

    const u32x4 *wb[WN];
#pragma unroll
    for (int nj = 0; nj < WN; nj++) {
        int64_t nb = n0 / 16 + nj;
        if (nb >= Nb) nb = Nb - 1;                                  // finite bits, never stored
        wb[nj] = native + (nb * Kb) * 64 + lane;
    }
    int64_t xoff[WM];                                               // element offset of the lane's row piece
#pragma unroll
    for (int mi = 0; mi < WM; mi++) {
        int64_t m = mw + mi * 16 + j;
        if (m >= M) m = M - 1;
        xoff[mi] = m * K + g * 8;
    }
    const int nt = Kb > kg ? (Kb - kg + KG - 1) / KG : 0;           // weight blocks of this wavefront

    // activation window: raw 16 (fp16) or 32 (fp32) bytes per fragment, D steps ahead
    u32x4 xa[D][WM], xb[X32 ? D : 1][X32 ? WM : 1];
    auto issue = [&](int slot, int s) {
        const int64_t k0 = (int64_t)(kg + (s >> 3) * KG) * kKB + (s & 7) * 32;
#pragma unroll
        for (int mi = 0; mi < WM; mi++) {
            if constexpr (FAST) {
                if constexpr (X32) {
                    const float *p = static_cast<const float *>(x) + xoff[mi] + k0;
                    xa[slot][mi] = *reinterpret_cast<const u32x4 *>(p);
                    xb[slot][mi] = *reinterpret_cast<const u32x4 *>(p + 4);
                } else {
                    xa[slot][mi] = *reinterpret_cast<const u32x4 *>(static_cast<const _Float16 *>(x) + xoff[mi] + k0);
                }
            } else {
                int64_t m = mw + mi * 16 + j;
                if (m >= M) m = M - 1;
                const XFrag<X32> f = load_x<X32>(x, m, M, K, k0 + g * 8, false);
                xa[slot][mi] = __builtin_bit_cast(u32x4, f.hi);
                if constexpr (X32) xb[slot][mi] = __builtin_bit_cast(u32x4, f.lo);
            }
        }
    };
    auto consume = [&](int slot, const u32x4 (&wq)[WN], int i) {
        half8 hi[WM], lo[X32 ? WM : 1];
#pragma unroll
        for (int mi = 0; mi < WM; mi++) {
            if constexpr (X32 && FAST) {
                const floatx4 a = __builtin_bit_cast(floatx4, xa[slot][mi]), b = __builtin_bit_cast(floatx4, xb[slot][mi]);
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float v = e < 4 ? a[e] : b[e - 4];
                    const _Float16 h = (_Float16)v;
                    hi[mi][e] = h;
                    lo[mi][e] = (_Float16)(v - (float)h);
                }
            } else {
                hi[mi] = __builtin_bit_cast(half8, xa[slot][mi]);
                if constexpr (X32) lo[mi] = __builtin_bit_cast(half8, xb[slot][mi]);
            }
        }
#pragma unroll
        for (int nj = 0; nj < WN; nj++) {
            const half8 a = decode_step(wq[nj][i >> 1], i & 1);
#pragma unroll
            for (int mi = 0; mi < WM; mi++) {
                acc[mi][nj] = mfma16(a, hi[mi], acc[mi][nj]);
                if constexpr (X32) acc[mi][nj] = mfma16(a, lo[mi], acc[mi][nj]);
            }
        }
    };

    if (nt > 0) {
        u32x4 wq[WN], wn[WN];
#pragma unroll
        for (int nj = 0; nj < WN; nj++) wq[nj] = __builtin_nontemporal_load(wb[nj] + kg * 64);
#pragma unroll
        for (int d = 0; d < D; d++) issue(d, d);
        for (int t = 0; t + 1 < nt; t++) {
#pragma unroll
            for (int nj = 0; nj < WN; nj++) wn[nj] = __builtin_nontemporal_load(wb[nj] + (kg + (t + 1) * KG) * 64);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                consume(i % D, wq, i);
                issue(i % D, t * 8 + i + D);
            }
#pragma unroll
            for (int nj = 0; nj < WN; nj++) wq[nj] = wn[nj];
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            consume(i % D, wq, i);
            if (i + D < 8) issue(i % D, (nt - 1) * 8 + i + D);
        }
    }

    // Sum the KG partial tiles in wavefront order; fragment f = (mi, nj) of row group wgm is finalised
    // by wavefront (wgm, kg = f mod KG). Lane (j, g) of a fragment holds y[16 mi + j][16 nj + 4 g + r].
#pragma unroll
    for (int mi = 0; mi < WM; mi++)
#pragma unroll
        for (int nj = 0; nj < WN; nj++) red[(wv * NF + mi * WN + nj) * 64 + lane] = acc[mi][nj];
    __syncthreads();
    for (int f = kg; f < NF; f += KG) {
        if (f != kg) load_consts(f);
        floatx4 s = red[(wgm * NF + f) * 64 + lane];
        for (int q = 1; q < KG; q++) {
            const floatx4 p = red[((q * WGM + wgm) * NF + f) * 64 + lane];
            s[0] += p[0]; s[1] += p[1]; s[2] += p[2]; s[3] += p[3];
        }
        const int64_t m = mw + (f / WN) * 16 + j, nq = n0 + (f % WN) * 16 + g * 4;
        if (m >= M) continue;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t n = nq + r;
            if (n < N) {
                float v = s[r] * (sc4[r] * (1.0f / kWeightUnit)) + bi4[r];
                const int64_t o = m * N + n;
                if (y_f16) {
                    if (residual) v += (float)static_cast<const _Float16 *>(residual)[o];
                    if (relu) v = v < 0.f ? 0.f : v;
                    static_cast<_Float16 *>(y)[o] = (_Float16)v;
                } else {
                    if (residual) v += static_cast<const float *>(residual)[o];
                    if (relu) v = v < 0.f ? 0.f : v;
                    static_cast<float *>(y)[o] = v;
                }
            }
        }
    }
}

template <int WM, int WN, int WGM, int WAVES, int D, bool X32>
int launch_mid(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const tmq_epilogue &ep, void *y,
               void *stream) {
    constexpr int BM = 16 * WM * WGM, BN = 16 * WN;
    const int64_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN, Kb = native_blocks_k(K);
    if (tm * tn > 0x7FFFFFFF || Kb > (1 << 20)) return TMQ_ERR_TOO_LARGE;
    const size_t lds = (size_t)WAVES * WM * WN * 64 * sizeof(floatx4);
    const bool fast = (K % kKB == 0) && aligned16(x);
    const float *scale = ep.scale, *bias = ep.bias;
    const void *residual = ep.residual;
    const int relu = ep.relu, y_f16 = ep.y_dtype == TMQ_F16;
    auto go = [&](auto kernel) -> int {
        if (int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) return st;
        hipLaunchKernelGGL(kernel, dim3((uint32_t)(tm * tn)), dim3(64 * WAVES), lds, as_stream(stream), x, M, K,
                           static_cast<const u32x4 *>(native), (int)Kb, N, native_blocks_n(N), (int)tn, scale, bias,
                           residual, relu, y, y_f16);
        return check_launch();
    };
    if (fast) return go(mid_kernel<WM, WN, WGM, WAVES, D, X32, true>);
    return go(mid_kernel<WM, WN, WGM, WAVES, D, X32, false>);
}

// ---- mid kernel, staged -----------------------------------------------------------------------------
// Same work split as mid_kernel with WGM = 1 (every wavefront owns the whole (16 WM) x (16 WN) tile
// for its share of the reduction), but the activations take the detour an MFMA operand needs: a
// lane wants 16 bytes of row (lane % 16), and 16 neighbouring lanes reading 16 different rows cost
// the texture path a cache-line access each. Here a wavefront loads whole 128-byte row pieces (8
// lanes per row), writes them to a private LDS window and reads them back in operand order. The
// window belongs to one wavefront, so the loop has no workgroup barrier: LDS operations of a
// wavefront execute in order, a wave barrier keeps the compiler from reordering them.
//
// Unit of the pipeline: a "pair" = 64 reduction indices = one dword of every native weight block =
// two MFMA steps. While pair p is multiplied, pair p + 1 already sits in the other LDS slot and
// pairs p + 2, p + 3 are in flight from global memory into registers.
// Requires K % 256 == 0 and 16-byte aligned rows. fp32 activations are split into their two fp16
// terms when they are written to LDS.
template <int WM, int WN, int WAVES, bool X32>
__global__ __launch_bounds__(64 * WAVES) void mid_lds_kernel(const void *__restrict__ x, int64_t M, int64_t K,
                                                             const u32x4 *__restrict__ native, int Kb, int64_t N,
                                                             int64_t Nb, int tiles_n, const float *__restrict__ scale,
                                                             const float *__restrict__ bias,
                                                             const void *__restrict__ residual, int relu,
                                                             void *__restrict__ y, int y_f16) {
    constexpr int NF = WM * WN, kPlanes = X32 ? 2 : 1;
    constexpr int kRow = 144;                                  // LDS bytes per 64-index row piece (+16: conflict-free reads)
    constexpr int kFrag = 16 * kRow, kSlot = kPlanes * WM * kFrag, kWave = 2 * kSlot;
    constexpr int NL = X32 ? 4 : 2;                            // 1 KiB global loads per fragment and pair
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    floatx4 *red = reinterpret_cast<floatx4 *>(smem);
    const int lane = threadIdx.x & 63, kg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, g = lane >> 4;
    unsigned char *win = smem + kg * kWave;
    const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
    const int64_t m0 = (int64_t)tm * (16 * WM), n0 = (int64_t)tn * (16 * WN);

    float sc4[4] = {1.f, 1.f, 1.f, 1.f}, bi4[4] = {0.f, 0.f, 0.f, 0.f};
    auto load_consts = [&](int f) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t n = n0 + (f % WN) * 16 + g * 4 + r;
            sc4[r] = (n < N && scale) ? scale[n] : 1.f;
            bi4[r] = (n < N && bias) ? bias[n] : 0.f;
        }
    };

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
    // global side: load c of a fragment covers rows [c * 16 / NL, +16 / NL), whole row pieces;
    // 32-bit byte offsets from x (the host checks that the matrix is smaller than 4 GiB)
    constexpr int kLanesPerRow = 64 * NL / 16;                     // 8 (fp16) or 16 (fp32)
    const int lrow = lane / kLanesPerRow, lchunk = lane % kLanesPerRow;
    uint32_t goff[WM][NL];
#pragma unroll
    for (int mi = 0; mi < WM; mi++)
#pragma unroll
        for (int c = 0; c < NL; c++) {
            int64_t m = m0 + mi * 16 + c * (16 / NL) + lrow;
            if (m >= M) m = M - 1;
            goff[mi][c] = (uint32_t)((m * K) * (X32 ? 4 : 2) + lchunk * 16);
        }
    const int nt = Kb > kg ? (Kb - kg + WAVES - 1) / WAVES : 0;      // weight blocks of this wavefront
    auto pair_k = [&](int p) { return (int64_t)(kg + (p >> 2) * WAVES) * kKB + (p & 3) * 64; };

    u32x4 stage[2][WM][NL];
    auto gload = [&](int set, int p) {
        const unsigned char *base = static_cast<const unsigned char *>(x) + pair_k(p) * (X32 ? 4 : 2);   // uniform
#pragma unroll
        for (int mi = 0; mi < WM; mi++)
#pragma unroll
            for (int c = 0; c < NL; c++) stage[set][mi][c] = *reinterpret_cast<const u32x4 *>(base + goff[mi][c]);
    };
    auto lwrite = [&](int set, int slot) {
#pragma unroll
        for (int mi = 0; mi < WM; mi++)
#pragma unroll
            for (int c = 0; c < NL; c++) {
                unsigned char *dst = win + slot * kSlot + mi * kFrag + (c * (16 / NL) + lrow) * kRow;
                if constexpr (X32) {
                    const floatx4 v = __builtin_bit_cast(floatx4, stage[set][mi][c]);
                    half4 hi, lo;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        hi[e] = (_Float16)v[e];
                        lo[e] = (_Float16)(v[e] - (float)hi[e]);
                    }
                    *reinterpret_cast<half4 *>(dst + lchunk * 8) = hi;
                    *reinterpret_cast<half4 *>(dst + WM * kFrag + lchunk * 8) = lo;
                } else {
                    *reinterpret_cast<u32x4 *>(dst + lchunk * 16) = stage[set][mi][c];
                }
            }
    };
    auto compute = [&](int slot, const uint32_t (&wq)[WN][4], int q) {
        const unsigned char *src = win + slot * kSlot + j * kRow + g * 16;
#pragma unroll
        for (int st = 0; st < 2; st++) {
            half8 hi[WM], lo[X32 ? WM : 1];
#pragma unroll
            for (int mi = 0; mi < WM; mi++) {
                hi[mi] = *reinterpret_cast<const half8 *>(src + mi * kFrag + st * 64);
                if constexpr (X32) lo[mi] = *reinterpret_cast<const half8 *>(src + (WM + mi) * kFrag + st * 64);
            }
#pragma unroll
            for (int nj = 0; nj < WN; nj++) {
                const half8 a = decode_step(wq[nj][q], st);
#pragma unroll
                for (int mi = 0; mi < WM; mi++) {
                    acc[mi][nj] = mfma16(a, hi[mi], acc[mi][nj]);
                    if constexpr (X32) acc[mi][nj] = mfma16(a, lo[mi], acc[mi][nj]);
                }
            }
        }
    };

    if (nt > 0) {
        // weight dwords: dword q of a block is only used by pair q and is refilled from the next
        // block right after (the 1 KiB blocks stay in L1 / L2 between the four dword loads)
        uint32_t wq[WN][4];
#pragma unroll
        for (int nj = 0; nj < WN; nj++)
#pragma unroll
            for (int q = 0; q < 4; q++) wq[nj][q] = wb[nj][(int64_t)kg * 256 + q];
        gload(0, 0);
        gload(1, 1);
        lwrite(0, 0);
        gload(0, 2);
        lwrite(1, 1);
        gload(1, 3);
        __builtin_amdgcn_wave_barrier();
        for (int t = 0; t + 1 < nt; t++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                compute(q & 1, wq, q);
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int nj = 0; nj < WN; nj++) wq[nj][q] = wb[nj][(int64_t)(kg + (t + 1) * WAVES) * 256 + q];
                lwrite(q & 1, q & 1);                 // pair p + 2 replaces pair p
                gload(q & 1, t * 4 + q + 4);
                __builtin_amdgcn_wave_barrier();
            }
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            compute(q & 1, wq, q);
            __builtin_amdgcn_wave_barrier();
            if (q < 2) lwrite(q & 1, q & 1);
            __builtin_amdgcn_wave_barrier();
        }
    }

    // Sum the WAVES partial tiles in wavefront order (the windows are dead by now); fragment f is
    // finalised by wavefront f mod WAVES. Lane (j, g) holds y[16 mi + j][16 nj + 4 g + r].
    __syncthreads();
#pragma unroll
    for (int mi = 0; mi < WM; mi++)
#pragma unroll
        for (int nj = 0; nj < WN; nj++) red[(kg * NF + mi * WN + nj) * 64 + lane] = acc[mi][nj];
    __syncthreads();
    for (int f = kg; f < NF; f += WAVES) {
        load_consts(f);
        floatx4 s = red[f * 64 + lane];
        for (int q = 1; q < WAVES; q++) {
            const floatx4 p = red[(q * NF + f) * 64 + lane];
            s[0] += p[0]; s[1] += p[1]; s[2] += p[2]; s[3] += p[3];
        }
        const int64_t m = m0 + (f / WN) * 16 + j, nq = n0 + (f % WN) * 16 + g * 4;
        if (m >= M) continue;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int64_t n = nq + r;
            if (n < N) {
                float v = s[r] * (sc4[r] * (1.0f / kWeightUnit)) + bi4[r];
                const int64_t o = m * N + n;
                if (y_f16) {
                    if (residual) v += (float)static_cast<const _Float16 *>(residual)[o];
                    if (relu) v = v < 0.f ? 0.f : v;
                    static_cast<_Float16 *>(y)[o] = (_Float16)v;
                } else {
                    if (residual) v += static_cast<const float *>(residual)[o];
                    if (relu) v = v < 0.f ? 0.f : v;
                    static_cast<float *>(y)[o] = v;
                }
            }
        }
    }
}

template <int WM, int WN, int WAVES, bool X32>
int launch_mid_lds(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const tmq_epilogue &ep, void *y,
                   void *stream) {
    constexpr int BM = 16 * WM, BN = 16 * WN;
    const int64_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN, Kb = native_blocks_k(K);
    if (tm * tn > 0x7FFFFFFF || Kb > (1 << 20)) return TMQ_ERR_TOO_LARGE;
    constexpr size_t win = (size_t)WAVES * 2 * (X32 ? 2 : 1) * WM * 16 * 144;
    constexpr size_t redb = (size_t)WAVES * WM * WN * 64 * sizeof(floatx4);
    constexpr size_t lds = win > redb ? win : redb;
    static_assert(lds <= kSkinnyLdsMax, "mid kernel LDS");
    auto kernel = mid_lds_kernel<WM, WN, WAVES, X32>;
    if (int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) return st;
    const float *scale = ep.scale, *bias = ep.bias;
    const void *residual = ep.residual;
    const int relu = ep.relu, y_f16 = ep.y_dtype == TMQ_F16;
    hipLaunchKernelGGL(kernel, dim3((uint32_t)(tm * tn)), dim3(64 * WAVES), lds, as_stream(stream), x, M, K,
                       static_cast<const u32x4 *>(native), (int)Kb, N, native_blocks_n(N), (int)tn, scale, bias,
                       residual, relu, y, y_f16);
    return check_launch();
}

// Tile choice of the mid kernel: the largest tile that yields at least one workgroup per CU.
template <bool X32>
int mid_rows(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const tmq_epilogue &ep, void *y,
             void *stream) {
    auto wgs = [&](int bm, int bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    if constexpr (X32) {
        if ((K % kKB == 0) && aligned16(x) && (uint64_t)M * (uint64_t)K * 4 < (1ull << 32)) {
            // the smallest tile that still fills one pass over the CUs, as for fp16 rows (mid.hip)
            // (K = N = 4096, M = 17: 13.7 -> 8.3 us; K = 4096, N = 1024, M = 64: 13.8 -> 8.0 us)
            if (wgs(32, 64) >= 192) return launch_mid_lds<2, 4, 8, true>(x, M, K, native, N, ep, y, stream);
            if (wgs(32, 32) >= 192) return launch_mid_lds<2, 2, 8, true>(x, M, K, native, N, ep, y, stream);
            return launch_mid_lds<1, 2, 8, true>(x, M, K, native, N, ep, y, stream);
        }
    } else {
        if (mid_dense_ok(x, M, K))
            return launch_mid_dense(x, M, K, native, N, ep.scale, ep.bias, ep.residual, ep.relu, y,
                                    ep.y_dtype == TMQ_F16, stream);
    }
    if constexpr (!X32) {
        // more than 64 fp16 rows of a length that is no multiple of 64 (16-byte aligned, a multiple of 8): the tile
        // kernel's register-staged loader fetches such rows in whole 16-byte chunks, the kernel below element by element
        // (K = 784, M = 128, N = 1024: 25.0 -> 9.0 us; K = 4000, M = 1024: 225 -> 27; up to 64 rows the skinny kernels
        // stay: K = 4000, M = 32 10.1 against 25.6)
        if (K % 8 == 0 && aligned16(x))
            return launch_gemm_dense(x, M, K, native, N, ep.scale, ep.bias, ep.residual, ep.relu, y, ep.y_dtype == TMQ_F16, stream);
    }
    if (wgs(64, 32) >= 256) return launch_mid<2, 2, 2, 16, 2, X32>(x, M, K, native, N, ep, y, stream);
    return launch_mid<2, 1, 2, 16, 2, X32>(x, M, K, native, N, ep, y, stream);
}

// ---- read probe -------------------------------------------------------------------------------------
// The weight stream of the skinny kernel and nothing else: wavefront w of a workgroup reads the
// 1 KiB pieces w, w + 16, ... of the workgroup's share.
__global__ __launch_bounds__(1024) void probe_read_kernel(const u32x4 *__restrict__ src, int per_wave, uint32_t *sink) {
    const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const u32x4 *p = src + ((int64_t)blockIdx.x * 16 * per_wave + wv) * 64 + lane;
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (int t = 0; t < per_wave; t++) acc ^= __builtin_nontemporal_load(p + (int64_t)t * 16 * 64);
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9E3779B9u && (acc[0] + acc[1]) == 0x7F4A7C15u) *sink = acc[2];
}

}  // namespace

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

int tmq_fp32_rows_self_scaled(const void *x, int64_t M, int64_t K) {
    return M == 1 && gemv8_dense32_ok(x, M, K, 16) ? 1 : 0;
}

int tmq_fp32_rows_self_scaled_for(const void *x, int64_t M, int64_t K, int64_t N) {
    return gemv8_dense32_ok(x, M, K, N) ? 1 : 0;
}

int tmq_fp32_rows_prefer_split(int64_t M, int64_t K, int64_t N) {
    // Measured: at K = N = 4096 the two fp16 passes win from about 512 rows (M = 4096: 400 -> 238 us), at
    // K = N = 1024 from about 4096; over large layers already from 9 rows (8192^2, M = 16: 34 -> 23 us) or,
    // beyond 2^27 weights, from 3 (16384^2, M = 4: 65 -> 39 us, M = 16: 118 -> 45 us): there the fp16
    // weight-stream kernel run twice beats every kernel that splits on the fly.
    if (M <= 0 || K <= 0 || N <= 0) return 0;
    const bool many_rows = M >= 512 && (double)M * (double)K * (double)N >= 4294967296.0;
    // up to 8 rows have an fp32 stream kernel, which holds its own up to about 2^26 weights
    const double weights = (double)K * (double)N;
    const bool large_layer = (M >= 9 && weights >= 67108864.0) || (M >= 3 && weights >= 134217728.0);
    return many_rows || large_layer;
}

int tmq_probe_stream_read(const void *src, size_t bytes, uint32_t *sink, void *stream) {
    if (!src || !sink || bytes == 0 || bytes % 1024 != 0 || !aligned16(src)) return TMQ_ERR_INVALID_ARG;
    const size_t pieces = bytes / 1024;
    // one piece per wavefront up to 4096 workgroups, then more pieces per wavefront
    size_t per_wave = 1;
    while (pieces / (16 * per_wave) > 4096 && pieces % (32 * per_wave) == 0) per_wave *= 2;
    if (pieces % (16 * per_wave) != 0) return TMQ_ERR_INVALID_ARG;
    const size_t wgs = pieces / (16 * per_wave);
    if (wgs > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    hipLaunchKernelGGL(probe_read_kernel, dim3((uint32_t)wgs), dim3(1024), 0, as_stream(stream),
                       static_cast<const u32x4 *>(src), (int)per_wave, sink);
    return check_launch();
}

size_t tmq_gemv8_planes_bytes(int64_t M, int64_t K) {
    if (!gemv8_planes_ok(M, K)) return 0;
    return (size_t)(gemv8_padded_rows(M) * 4 * (K + 32));
}

int tmq_gemv8_prepare(const void *x, int64_t M, int64_t K, void *planes, void *stream) {
    if (!x || !planes || !aligned16(x) || !aligned16(planes)) return TMQ_ERR_INVALID_ARG;
    if (!gemv8_planes_ok(M, K)) return TMQ_ERR_UNSUPPORTED;
    return launch_gemv8_prepare(x, M, K, planes, stream);
}

int tmq_ternary_linear_planes(const void *planes, int64_t M, int64_t K, const void *native, int64_t N,
                              const tmq_epilogue *epilogue, void *y, void *stream) {
    if (K <= 0 || N <= 0) return TMQ_ERR_INVALID_ARG;
    if (!planes || !native || !y || !aligned16(native) || !aligned16(planes)) return TMQ_ERR_INVALID_ARG;
    if (!gemv8_planes_ok(M, K)) return TMQ_ERR_UNSUPPORTED;
    tmq_epilogue ep = {nullptr, nullptr, nullptr, 0, TMQ_F32};
    if (epilogue) ep = *epilogue;
    if (ep.y_dtype != TMQ_F16 && ep.y_dtype != TMQ_F32) return TMQ_ERR_UNSUPPORTED;
    return launch_gemv8_planes(planes, M, K, native, N, ep.scale, ep.bias, ep.residual, ep.relu, y, ep.y_dtype == TMQ_F16, stream);
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
    // One fp16 row, K a multiple of 256 from 2048 to 16384 (two rows to 4096 and where gemv8_dense_ok measured them
    // faster beyond): weights and
    // activations as 8-bit MFMA operands (gemv8.hip), half the decode work per weight of the kernels below (4096^2:
    // 3.75 -> 3.0 us, 16384^2: 17.7 -> 15.6 us).
    if (!x32 && gemv8_dense_ok(x, M, K, N))
        return launch_gemv8_dense(x, M, K, native, N, ep.scale, ep.bias, ep.residual, ep.relu, y, ep.y_dtype == TMQ_F16, stream);
    // ... and one fp32 row (the reference's GEMV convention) up to K = 16384, two over small layers: the same kernel on the rows' two fp16 halves
    if (x32 && gemv8_dense32_ok(x, M, K, N))
        return launch_gemv8_dense32(x, M, K, native, N, ep.scale, ep.bias, ep.residual, ep.relu, y, ep.y_dtype == TMQ_F16, stream);
    // At most 16 fp16 rows against eight or more weight blocks per channel: the weight-stream kernel (mid.hip).
    // Against the kernels below: M = 16 at 16384^2 67 -> 20 us, M = 8 at 8192 x 28672 34 -> 17 us, M = 1 at
    // 11008 x 4096 7.2 -> 6.2 us, even at 4096^2.
    if (!x32 && stream_dense_ok(x, M, K) && K >= 8 * kKB)
        return launch_stream_dense(x, M, K, native, N, ep.scale, ep.bias, ep.residual, ep.relu, y, ep.y_dtype == TMQ_F16, stream);
    // ... and a few fp32 rows (the reference's GEMV convention; up to 8, up to 16 on short reductions): its fp32 form (M = 1 at 4096^2: 6.0 -> 4.5 us,
    // M = 8 at 8192^2: 24 -> 17 us)
    if (x32 && stream32_dense_ok(x, M, K) && K >= 8 * kKB)
        return launch_stream32_dense(x, M, K, native, N, ep.scale, ep.bias, ep.residual, ep.relu, y, ep.y_dtype == TMQ_F16, stream);
    // Otherwise up to 16 rows take the skinny kernels (activations staged in LDS). They also take 17 .. 64
    // rows when K is ragged or the rows are unaligned; with whole 64-index tiles of aligned rows the split-reduction
    // kernels are as fast at K = 4096 and two to five times faster elsewhere, where staging all of x in every
    // workgroup dominates (M = 64, K = 512: 11.2 -> 4.6 us; K = 576, N = 512: 15.7 -> 3.8; K = 8256, N = 16384:
    // 126 -> 23; fp32 input at K = 4096: 33 -> 14 us). fp32 rows need whole 256-index blocks for their kernel.
    const bool blocks_ok = (K % (x32 ? kKB : 64) == 0) && aligned16(x);
    if (M <= 16 || (M <= 64 && !blocks_ok))
        return x32 ? skinny_rows<true>(x, M, K, native, N, ep, y, stream)
                   : skinny_rows<false>(x, M, K, native, N, ep, y, stream);
    // fp32 activations always take the mid kernel (two fp16 terms per value keep fp32 accuracy; the
    // tile kernel is fp16 only).
    if (x32) return mid_rows<true>(x, M, K, native, N, ep, y, stream);
    if (split_reduction_pays(M, K, N)) return mid_rows<false>(x, M, K, native, N, ep, y, stream);
    return launch_gemm_dense(x, M, K, native, N, ep.scale, ep.bias, ep.residual, ep.relu, y, ep.y_dtype == TMQ_F16,
                             stream);
}

}  // extern "C"
