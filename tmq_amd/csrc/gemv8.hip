// M = 1 on the 8-bit matrix instructions: v_mfma_f32_16x16x32_fp8_bf8.
//
// The fp16 MFMA kernels expand every 2-bit code into an fp16 operand, one VALU lane-operation per weight,
// and for a single activation row that expansion, not memory, is what a launch waits for. The fp8 operand
// format takes four weights per register: the native layout's (sign, nonzero) pairs sit two bits apart, so
// `(word << 2 f) & 0xC0C0C0C0` puts the pairs of four weights into the top two bits of the four bytes, which
// read as e4m3 are +-2.0 or 0 -- half the VALU work per weight. The activation vector has to become 8-bit as
// well, exactly: an fp16 value is a sum of four scaled bf8 (e5m2) terms, because the top byte of an fp16 number
// IS a bf8 number (same sign and exponent, the two leading mantissa bits): take the top byte, subtract it
// (exact), rescale the remainder, repeat -- three significant bits per term (bf8_terms below). The four term
// vectors ride in rows 0..3 of the MFMA's sixteen activation columns, which a single row leaves unused anyway,
// so the instruction count does not grow; the four result columns are added, with their scales, at the end. Products are exact
// and the accumulation is fp32, as in the fp16 kernels. One difference remains: the hardware adds the 32
// products of one instruction in a fixed-point window below the largest of them (measured: ~2^-17 of it), so a
// vector whose neighbouring elements differ by more than five orders of magnitude loses the small ones'
// contribution earlier than an fp32 sum would (1e-4 of the largest output in a constructed case with 65504
// next to values of order one; 1.4e-6 on normally distributed data; exact on small integers).
//
// Structure: a workgroup of WAVES wavefronts owns CB blocks of 16 channels; KS = WAVES / CB wavefronts share a
// channel block, wavefront ks taking the weight blocks ks, ks + KS, ... (NT of them, all in flight at once as
// 16-byte-per-lane loads issued in the order they are used). The workgroup first turns the activation vector
// into the four term planes in LDS, in the byte order the weight registers imply (a thread per 8 values: two
// 8-byte loads, 28 operations for the terms, 8 byte permutes, four 8-byte LDS writes), while its weight loads
// are on their way; then every MFMA takes its activation operand with one 8-byte LDS read. Sums of the KS
// wavefronts meet in LDS in wavefront order (deterministic). Measured (HIP-graph replays over rotating weight
// buffers): K = N = 4096 3.0 us (fp16 weight-stream kernel 3.75), 8192^2 5.5 us, 16384^2 15.6 us (17.7).
//
// Requires M == 1, K a multiple of 256 from 2048 to 16384 (fp32 activations, carried as two fp16 halves, too),
// 16-byte aligned x.
//
// Two to four rows (MR = 2, 4; three rows run as four with one of zeros) take the same kernel: row m's four
// term planes ride in activation columns 4 m .. 4 m + 3, so four rows fill exactly the sixteen columns of the
// instruction the single row already issues -- no extra MFMA, no extra weight expansion; only the planes (and
// the work of preparing them) grow with the rows, which is what limits the rows: two split inside the kernel
// (gemv8_dense_ok), three and four only with the planes prepared beforehand.
//
// The planes can also come ready-made from memory (PRE): tmq_gemv8_prepare writes them once per activation
// vector (or a producing kernel could), and the workgroup then copies its image global -> LDS with buffer loads
// that bypass the registers -- no conversion arithmetic and no LDS writes in the GEMV, which is what every
// workgroup otherwise repeats for the whole row. Up to 16384 / MR reduction indices (64 KiB of planes).
#include "common.h"
#include "mfma.h"

#include <math.h>
#include <type_traits>

namespace tmq {
namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// Four bf8 terms of the two fp16 values packed in one register: t[i] carries term i of both values in the high
// byte of each half-word, and x = t0 + t1 / 4 + t2 / 32 + t3 / 256 exactly, for every finite fp16 x.
//   t0 = the top byte of x (its three leading significant bits, truncated);
//   r1 = 4 (x - t0), below |x| in magnitude;         t1 = r1 rounded to three significant bits;
//   r2 = 8 (r1 - t1), at most |r1| (half an ulp x 8); t2 = r2 rounded;     r3 = 8 (r2 - t2);     t3 = r3, exact.
// Rounding is an integer add on the bit patterns (half of the kept unit, then the mask): it carries into the
// exponent correctly and treats subnormals like normals. The rescaling is what keeps small values exact: without
// it a remainder below 2^-14 would be subnormal in its own right and lose everything under 2^-16 to the mask;
// with it the four terms resolve 2^-16, 2^-18, 2^-21 and 2^-24, the smallest fp16 subnormal. Every difference
// and product is exact in fp16 (each term holds leading bits of its remainder; the factors are powers of two and
// nothing grows past |x|).
__device__ __forceinline__ void bf8_terms(uint32_t x2, uint32_t (&t)[4]) {
    const half2_t four = {(_Float16)4.0f, (_Float16)4.0f}, eight = {(_Float16)8.0f, (_Float16)8.0f};
    t[0] = x2 & 0xFF00FF00u;
    half2_t r = (__builtin_bit_cast(half2_t, x2) - __builtin_bit_cast(half2_t, t[0])) * four;
#pragma unroll
    for (int i = 1; i < 3; i++) {
        t[i] = (__builtin_bit_cast(uint32_t, r) + 0x00800080u) & 0xFF00FF00u;
        r = (r - __builtin_bit_cast(half2_t, t[i])) * eight;
    }
    t[3] = __builtin_bit_cast(uint32_t, r) & 0xFF00FF00u;
}

struct Gemv8Epilogue {
    const float *scale, *bias;
    const void *residual;
    void *y;
    int relu, y_f16;
    int rows;               // rows of x that exist (<= MR; the others are zero planes and are not stored)
};

// weight blocks (1 KiB per wavefront each) a wavefront has asked for ahead of the one it multiplies: 3 and 4 measured
// level at 16384^2 and 12288 x 16384, 2 and 6 about 3 % slower, 8 7 % and all 16 at once 25 %
constexpr int kGemv8Ahead = 4;

// vmcnt(n), nothing else waited for
constexpr int vmcnt_only(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0F70; }

// ORDER: what separates the activation loads from the weight loads. 0: nothing. 1: a workgroup barrier, so that
// no wavefront's activation loads queue behind another's weight loads (8192^2: 5.65 -> 5.3 us). 2: the
// wavefront waits for its activation values before it asks for weights, so they do not queue behind the weight
// requests of the whole chip either (16384^2, where 64 MiB are requested at once: 16.7 -> 15.8 us).
//
// X32: the row is fp32, of any magnitude (the kernel scales it by a power of two itself). Each value becomes
// hi = fp16(x) and lo = fp16(x - hi) -- 22 significant bits -- and both halves their four bf8 terms: eight
// planes, eight of the sixteen activation columns, still one MFMA per weight operand.
template <int WAVES, int CB, int NT, int ORDER, bool X32, int MR, bool PRE>
__global__ __launch_bounds__(64 * WAVES) void gemv8_kernel(const void *__restrict__ xv, const u32x4 *__restrict__ native,
                                                           int Kb, int64_t N, int64_t Nb, Gemv8Epilogue ep) {
    static_assert(!X32 || (MR <= 2 && !PRE), "fp32 rows: one or two, split in the kernel");
    constexpr int KS = WAVES / CB, kUnits = (KS * NT + 2 * WAVES - 1) / (2 * WAVES);   // units of 8 values per thread and row: ceil(32 Kb / threads)
    constexpr int NP = (X32 ? 8 : 4) * MR;                       // term planes
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int K = Kb * kKB;
    const int plane = K + 32;                                    // bytes per term plane; +32 puts the planes on different banks
    unsigned char *planes = smem;
    const int image = PRE ? ((NP * plane + 1023) & ~1023) : NP * plane;   // the copy from memory moves whole KiB
    float *red = reinterpret_cast<float *>(smem + image);       // [WAVES][MR][16]
    const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, g = lane >> 4;
    const int cb = wv / KS, ks = wv % KS;
    int64_t nb = (int64_t)blockIdx.x * CB + cb;
    if (nb >= Nb) nb = Nb - 1;                                   // finite bits, never stored

    // The activation quads of this thread's units first, then the first weight blocks; loads return in issue
    // order, so waiting for the quads leaves the weights on their way. Unit u = (kb, d, h, g')
    // covers x[256 kb + 64 d + 8 g' + 4 h + {0..3}] (quad A) and the same 32 further on (quad B): the eight
    // values whose weights lane group g' finds in one operand register pair of dword d.
    using Quad = std::conditional_t<X32, u32x4, u32x2>;           // four activation values
    Quad qa[MR][kUnits], qb[MR][kUnits];
    if constexpr (PRE) {
        // the planes as tmq_gemv8_prepare left them: NP x (K + 32) bytes, copied 1 KiB per instruction
        const BufferResource img = make_buffer_resource(xv, (uint32_t)(NP * plane));
        for (int c = wv * 1024; c < image; c += WAVES * 1024) buffer_to_lds(img, (uint32_t)(c + lane * 16), planes + c);
    } else {
#pragma unroll
        for (int m = 0; m < MR; m++)
#pragma unroll
            for (int i = 0; i < kUnits; i++) {
                const int u = threadIdx.x + i * 64 * WAVES;
                const int gq = u & 3, h = (u >> 2) & 1, d = (u >> 3) & 3, kb = u >> 5;
                const int k0 = kKB * kb + 64 * d + 8 * gq + 4 * h;
                qa[m][i] = qb[m][i] = Quad{};
                if (u < K / 8 && m < ep.rows) {
                    if constexpr (X32) {
                        const float *row = static_cast<const float *>(xv) + (size_t)m * K;
                        qa[m][i] = *reinterpret_cast<const u32x4 *>(row + k0);
                        qb[m][i] = *reinterpret_cast<const u32x4 *>(row + k0 + 32);
                    } else {
                        const _Float16 *row = static_cast<const _Float16 *>(xv) + (size_t)m * K;
                        qa[m][i] = *reinterpret_cast<const u32x2 *>(row + k0);
                        qb[m][i] = *reinterpret_cast<const u32x2 *>(row + k0 + 32);
                    }
                }
            }
    }
    if (ORDER == 1) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
    if (ORDER == 2) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0)
        __builtin_amdgcn_sched_barrier(0);
    }
    // wavefront ks takes blocks ks, ks + KS, ...; when Kb is no multiple of KS the last round is short: a
    // wavefront without a block there re-reads block Kb - 1 (weights and activations) and multiplies it by zero
    //
    // Only the first D weight blocks are asked for here, the others one at a time as the blocks in front of them
    // are multiplied. A wavefront cannot issue a load while the CU's memory pipeline is full, and with every
    // wavefront of the chip asking for all of its 16 KiB at once it is full for microseconds: the wavefront then
    // sits at a load instruction instead of preparing its share of the planes, its workgroup's barrier waits for
    // it, and the arithmetic of wavefronts whose weights have long arrived starts when most of the matrix has
    // been read (16384^2: the barrier passed 3.3 .. 10.3 us after the first wavefront started, the kernel ended
    // at 14.2; with four blocks ahead 2.2 .. 6.6 and 12.2 -- by wall-clock stamps of every wavefront).
    constexpr int D = NT < kGemv8Ahead ? NT : kGemv8Ahead;
    const u32x4 *wp = native + nb * Kb * 64 + lane;
    u32x4 wq[NT];
    auto ask = [&](int t) {
        const int kblk = ks + t * KS < Kb ? ks + t * KS : Kb - 1;
        wq[t] = __builtin_nontemporal_load(wp + (int64_t)kblk * 64);
        __builtin_amdgcn_sched_barrier(0);                       // issue order = use order
    };
#pragma unroll
    for (int t = 0; t < D; t++) ask(t);
    if constexpr (PRE) {
        // the copies were issued before the D weight loads and retire first: wait for them alone
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(vmcnt_only(D));
        __builtin_amdgcn_sched_barrier(0);
    }
    // per-channel constants of the threads that will store, asked for now
    float sc = 1.f, bi = 0.f;
    uint32_t res_bits = 0;                                       // converted where it is used: no wait for it here
    const int st_m = (threadIdx.x >> 4) / CB, st_c = (threadIdx.x >> 4) % CB;     // row and channel block this thread stores
    const int64_t n_out = ((int64_t)blockIdx.x * CB + st_c) * 16 + (threadIdx.x & 15);
    const bool stores = threadIdx.x < 16 * CB * MR && st_m < ep.rows && n_out < N;
    const int64_t y_at = (int64_t)st_m * N + n_out;
    if (stores) {
        if (ep.scale) sc = ep.scale[n_out];
        if (ep.bias) bi = ep.bias[n_out];
        if (ep.residual) res_bits = ep.y_f16 ? (uint32_t)static_cast<const uint16_t *>(ep.residual)[y_at]
                                             : static_cast<const uint32_t *>(ep.residual)[y_at];
    }
    // fp32 rows of any magnitude: the row times the power of two that brings its largest finite |x| into
    // [1024, 2048) (exact), undone in the epilogue -- the hi / lo halves then sit well inside fp16's range. Every
    // workgroup holds the whole row, so the maximum is one reduction through LDS.
    float ps[MR], ps_inv[MR];
#pragma unroll
    for (int m = 0; m < MR; m++) ps[m] = ps_inv[m] = 1.f;
    if constexpr (X32) {
        float amax[MR];
#pragma unroll
        for (int m = 0; m < MR; m++) {
            amax[m] = 0.f;
#pragma unroll
            for (int i = 0; i < kUnits; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float a = __builtin_fabsf(__builtin_bit_cast(float, qa[m][i][e])), b = __builtin_fabsf(__builtin_bit_cast(float, qb[m][i][e]));
                    amax[m] = fmaxf(amax[m], a < INFINITY ? a : 0.f);   // NaN and Inf take no part (they propagate anyway)
                    amax[m] = fmaxf(amax[m], b < INFINITY ? b : 0.f);
                }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) amax[m] = fmaxf(amax[m], __shfl_xor(amax[m], off, 64));
            if (lane == 0) red[wv * MR + m] = amax[m];
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);                      // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int m = 0; m < MR; m++) {
#pragma unroll
            for (int q = 0; q < WAVES; q++) amax[m] = fmaxf(amax[m], red[q * MR + m]);
            if (amax[m] > 0.f) {                                 // every row its own power of two
                int e;
                (void)frexpf(amax[m], &e);                       // amax in [2^(e-1), 2^e)
                int p = 11 - e;
                p = p > 126 ? 126 : (p < -126 ? -126 : p);
                ps[m] = ldexpf(1.f, p);
                ps_inv[m] = ldexpf(1.f, -p);
            }
        }
        // (the partial sums below reuse red[] only after the next barrier)
    }
    // the planes of one unit from its two quads as packed fp16 pairs (plane offset P0: 0, or 4 for the lo halves)
    auto write_planes = [&](int u, int p0, uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1) {
        uint32_t ta0[4], ta1[4], tb0[4], tb1[4];
        bf8_terms(a0, ta0);
        bf8_terms(a1, ta1);
        bf8_terms(b0, tb0);
        bf8_terms(b1, tb1);
#pragma unroll
        for (int m = 0; m < 4; m++) {
            // An operand register pair of dword d holds, byte by byte, the weights of (step 1, e), (step 0, e),
            // (step 1, e + 1), (step 0, e + 1), ...: quad B and quad A interleaved, B first.
            const uint32_t lo = __builtin_amdgcn_perm(ta0[m], tb0[m], 0x07030501u);
            const uint32_t hi = __builtin_amdgcn_perm(ta1[m], tb1[m], 0x07030501u);
            *reinterpret_cast<u32x2 *>(planes + (p0 + m) * plane + u * 8) = u32x2{lo, hi};
        }
    };
    if constexpr (!PRE) {
#pragma unroll
        for (int m = 0; m < MR; m++)
#pragma unroll
            for (int i = 0; i < kUnits; i++) {
                const int u = threadIdx.x + i * 64 * WAVES;
                if (u < K / 8) {
                    if constexpr (X32) {
                        uint32_t hi[4], lo[4];                   // pairs (0, 1), (2, 3) of quad A, then of quad B
#pragma unroll
                        for (int p = 0; p < 4; p++) {
                            const float v0 = ps[m] * __builtin_bit_cast(float, p < 2 ? qa[m][i][2 * p] : qb[m][i][2 * p - 4]);
                            const float v1 = ps[m] * __builtin_bit_cast(float, p < 2 ? qa[m][i][2 * p + 1] : qb[m][i][2 * p - 3]);
                            const _Float16 h0 = (_Float16)v0, h1 = (_Float16)v1;
                            const _Float16 l0 = (_Float16)(v0 - (float)h0), l1 = (_Float16)(v1 - (float)h1);
                            hi[p] = __builtin_bit_cast(uint32_t, half2_t{h0, h1});
                            lo[p] = __builtin_bit_cast(uint32_t, half2_t{l0, l1});
                        }
                        write_planes(u, 8 * m, hi[0], hi[1], hi[2], hi[3]);
                        write_planes(u, 8 * m + 4, lo[0], lo[1], lo[2], lo[3]);
                    } else {
                        write_planes(u, 4 * m, qa[m][i][0], qa[m][i][1], qb[m][i][0], qb[m][i][1]);
                    }
                }
            }
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);                          // lgkmcnt(0): this thread's LDS writes are done
    __builtin_amdgcn_s_barrier();                                // (not __syncthreads: that would wait for the weights too)
    __builtin_amdgcn_sched_barrier(0);

    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    const unsigned char *xb = planes + (j & (NP - 1)) * plane + g * 8;   // column j carries plane j % NP; the other columns are never read back
#pragma unroll
    for (int t = 0; t < NT; t++) {
        __builtin_amdgcn_sched_barrier(0);
        if (t + D < NT) ask(t + D);
        const bool live = ks + t * KS < Kb;                      // uniform
        const unsigned char *xp = xb + (live ? ks + t * KS : Kb - 1) * 256;
        const uint32_t mask = live ? 0xC0C0C0C0u : 0u;
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t w = wq[t][d];
            const uint32_t r0 = w & mask, r1 = (w << 2) & mask, r2 = (w << 4) & mask, r3 = (w << 6) & mask;
            const long a0 = (long)(((unsigned long)r1 << 32) | r0), a1 = (long)(((unsigned long)r3 << 32) | r2);
            const long b0 = *reinterpret_cast<const long *>(xp + (d * 2 + 0) * 32);
            const long b1 = *reinterpret_cast<const long *>(xp + (d * 2 + 1) * 32);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_fp8_bf8(a0, b0, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_fp8_bf8(a1, b1, acc, 0, 0, 0);
        }
    }
    // D[n = 4 g + r][column j]: add the four term columns 0..3 (lanes j = 0..3 of each row of 16 lanes), each with
    // the power of two its term was scaled by
    const float term_weight = (j & 3) == 0 ? 1.0f : (j & 3) == 1 ? 0.25f : (j & 3) == 2 ? 0.03125f : 0.00390625f;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        float v = acc[r] * term_weight;
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
        if constexpr (X32)                                       // + the lo half's columns 4..7
            v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x104, 0xF, 0xF, false));   // row_shl:4
        acc[r] = v;
    }
    // lanes j = 4 m now hold row m's sums (X32: lanes j = 8 m)
    constexpr int kCols = X32 ? 8 : 4;
    if ((j & (kCols - 1)) == 0 && j / kCols < MR) {
#pragma unroll
        for (int r = 0; r < 4; r++) red[(wv * MR + j / kCols) * 16 + 4 * g + r] = acc[r];
    }
    __syncthreads();
    if (stores) {
        const int i16 = threadIdx.x & 15;
        float v = red[((st_c * KS) * MR + st_m) * 16 + i16];
#pragma unroll
        for (int q = 1; q < KS; q++) v += red[((st_c * KS + q) * MR + st_m) * 16 + i16];
        if constexpr (X32) v *= MR > 1 && st_m ? ps_inv[MR - 1] : ps_inv[0];
        v = v * (sc * (1.0f / kWeightUnit)) + bi;
        if (ep.residual) v += ep.y_f16 ? (float)__builtin_bit_cast(_Float16, (uint16_t)res_bits) : __builtin_bit_cast(float, res_bits);
        if (ep.relu) v = v < 0.f ? 0.f : v;
        if (ep.y_f16) static_cast<_Float16 *>(ep.y)[y_at] = (_Float16)v;
        else static_cast<float *>(ep.y)[y_at] = v;
    }
}

// The four bf8 term planes of M fp16 rows in the order gemv8_kernel reads them, written to memory once:
// planes[(4 m + t) (K + 32) + 8 u .. + 7] for unit u of row m (rows beyond M: zeros).
__global__ __launch_bounds__(256) void gemv8_prepare_kernel(const _Float16 *__restrict__ x, int M, int K,
                                                            unsigned char *__restrict__ planes) {
    const int plane = K + 32;
    const int u = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
    if (u >= K / 8) return;
    const int gq = u & 3, h = (u >> 2) & 1, d = (u >> 3) & 3, kb = u >> 5;
    const int k0 = kKB * kb + 64 * d + 8 * gq + 4 * h;
    u32x2 a = {0u, 0u}, b = {0u, 0u};
    if (m < M) {
        a = *reinterpret_cast<const u32x2 *>(x + (size_t)m * K + k0);
        b = *reinterpret_cast<const u32x2 *>(x + (size_t)m * K + k0 + 32);
    }
    uint32_t ta0[4], ta1[4], tb0[4], tb1[4];
    bf8_terms(a[0], ta0);
    bf8_terms(a[1], ta1);
    bf8_terms(b[0], tb0);
    bf8_terms(b[1], tb1);
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const uint32_t lo = __builtin_amdgcn_perm(ta0[t], tb0[t], 0x07030501u);
        const uint32_t hi = __builtin_amdgcn_perm(ta1[t], tb1[t], 0x07030501u);
        *reinterpret_cast<u32x2 *>(planes + (size_t)(4 * m + t) * plane + u * 8) = u32x2{lo, hi};
    }
}

constexpr size_t kGemv8LdsMax = 152 * 1024;

template <int WAVES, int CB, int NT, int ORDER, bool X32 = false, int MR = 1, bool PRE = false>
int launch_gemv8(const void *x, const void *native, int64_t Kb, int64_t N, const Gemv8Epilogue &ep, void *stream) {
    const int64_t Nb = native_blocks_n(N), grid = (Nb + CB - 1) / CB;
    if (grid > 0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    size_t image = (X32 ? 8 : 4) * MR * (size_t)(Kb * kKB + 32);
    if (PRE) image = (image + 1023) & ~(size_t)1023;
    const size_t lds = image + (size_t)WAVES * MR * 16 * sizeof(float);
    if (lds > kGemv8LdsMax) return TMQ_ERR_UNSUPPORTED;
    auto kernel = gemv8_kernel<WAVES, CB, NT, ORDER, X32, MR, PRE>;
    if (int st = allow_dynamic_lds(reinterpret_cast<const void *>(kernel), lds)) return st;
    hipLaunchKernelGGL(kernel, dim3((uint32_t)grid), dim3(64 * WAVES), lds, as_stream(stream), x,
                       static_cast<const u32x4 *>(native), (int)Kb, N, Nb, ep);
    return check_launch();
}

// Geometry by the number of weight blocks per channel block: eight wavefronts per workgroup (sixteen for the eight
// planes of an fp32 row beyond 8192 indices or over wide layers); one channel block per workgroup up to 32 weight
// blocks unless the layer is wide, two beyond when that still leaves two workgroups per CU (half as many workgroups
// prepare or copy the activation planes).
template <bool X32, int MR, bool PRE>
int launch_gemv8_by_blocks(const void *x, int64_t Kb, const void *native, int64_t N, const Gemv8Epilogue &ep, void *stream) {
    if constexpr (X32 && MR == 2) {
        // Two fp32 rows: sixteen planes, the LDS of one fp32 row of twice the length (gemv8_dense32_ok: K <= 6144)
        if (Kb > 24) return TMQ_ERR_UNSUPPORTED;
        switch ((Kb + 7) / 8) {
            case 1: return launch_gemv8<8, 1, 1, 0, true, 2, false>(x, native, Kb, N, ep, stream);
            case 2: return launch_gemv8<8, 1, 2, 0, true, 2, false>(x, native, Kb, N, ep, stream);
            default: return launch_gemv8<16, 2, 3, 1, true, 2, false>(x, native, Kb, N, ep, stream);
        }
    } else if constexpr (X32) {
        // wide layers: four channel blocks per workgroup of sixteen wavefronts keep all workgroups resident at once
        // (8192 x 28672: 1792 workgroups in 3.5 rounds -> 448 in one)
        if (Kb > 16 && Kb <= 32 && native_blocks_n(N) >= 1024) {
            switch ((Kb + 3) / 4) {
                case 5: return launch_gemv8<16, 4, 5, 2, true, 1, false>(x, native, Kb, N, ep, stream);
                case 6: return launch_gemv8<16, 4, 6, 2, true, 1, false>(x, native, Kb, N, ep, stream);
                case 7: return launch_gemv8<16, 4, 7, 2, true, 1, false>(x, native, Kb, N, ep, stream);
                default: return launch_gemv8<16, 4, 8, 2, true, 1, false>(x, native, Kb, N, ep, stream);
            }
        }
    }
    if constexpr (!X32 && MR == 1) {
        // 1024 channel blocks or more: two per workgroup, so that all workgroups are resident at once (four fit a CU)
        // and half as many prepare the planes -- 4096 x 28672 8.0 -> 7.3 us, 3072 x 24576 6.7 -> 5.5, 8192 x 28672
        // 13.0 -> 12.0, 8192 x 16384 8.7 -> 8.15
        if (Kb >= 8 && Kb <= 32 && native_blocks_n(N) >= 1024) {
            switch ((Kb + 3) / 4) {
                case 2: return launch_gemv8<8, 2, 2, 0, false, 1, PRE>(x, native, Kb, N, ep, stream);
                case 3: return launch_gemv8<8, 2, 3, 1, false, 1, PRE>(x, native, Kb, N, ep, stream);
                case 4: return launch_gemv8<8, 2, 4, 1, false, 1, PRE>(x, native, Kb, N, ep, stream);
                case 5: return launch_gemv8<8, 2, 5, 2, false, 1, PRE>(x, native, Kb, N, ep, stream);
                case 6: return launch_gemv8<8, 2, 6, 2, false, 1, PRE>(x, native, Kb, N, ep, stream);
                case 7: return launch_gemv8<8, 2, 7, 2, false, 1, PRE>(x, native, Kb, N, ep, stream);
                default: return launch_gemv8<8, 2, 8, 2, false, 1, PRE>(x, native, Kb, N, ep, stream);
            }
        }
    }
    if (Kb <= 32) {
        switch ((Kb + 7) / 8) {                                  // blocks per wavefront, 8 wavefronts per channel block
            case 1: return launch_gemv8<8, 1, 1, 0, X32, MR, PRE>(x, native, Kb, N, ep, stream);
            case 2: return launch_gemv8<8, 1, 2, 0, X32, MR, PRE>(x, native, Kb, N, ep, stream);
            case 3: return launch_gemv8<8, 1, 3, 1, X32, MR, PRE>(x, native, Kb, N, ep, stream);
            default: return launch_gemv8<8, 1, 4, 1, X32, MR, PRE>(x, native, Kb, N, ep, stream);
        }
    }
    if constexpr (X32) {
        // Eight planes of up to 16 KiB each: one workgroup per CU, so sixteen wavefronts in it, four per channel
        // block where the layer is wide enough for that to cover the CUs, else eight
        if (Kb > 64) return TMQ_ERR_UNSUPPORTED;
        if (native_blocks_n(N) >= 1024) {
            switch ((Kb + 3) / 4) {
                case 9: return launch_gemv8<16, 4, 9, 2, true, 1, false>(x, native, Kb, N, ep, stream);
                case 10: return launch_gemv8<16, 4, 10, 2, true, 1, false>(x, native, Kb, N, ep, stream);
                case 11: return launch_gemv8<16, 4, 11, 2, true, 1, false>(x, native, Kb, N, ep, stream);
                case 12: return launch_gemv8<16, 4, 12, 2, true, 1, false>(x, native, Kb, N, ep, stream);
                case 13: return launch_gemv8<16, 4, 13, 2, true, 1, false>(x, native, Kb, N, ep, stream);
                case 14: return launch_gemv8<16, 4, 14, 2, true, 1, false>(x, native, Kb, N, ep, stream);
                case 15: return launch_gemv8<16, 4, 15, 2, true, 1, false>(x, native, Kb, N, ep, stream);
                default: return launch_gemv8<16, 4, 16, 2, true, 1, false>(x, native, Kb, N, ep, stream);
            }
        }
        switch ((Kb + 7) / 8) {
            case 5: return launch_gemv8<16, 2, 5, 2, true, 1, false>(x, native, Kb, N, ep, stream);
            case 6: return launch_gemv8<16, 2, 6, 2, true, 1, false>(x, native, Kb, N, ep, stream);
            case 7: return launch_gemv8<16, 2, 7, 2, true, 1, false>(x, native, Kb, N, ep, stream);
            default: return launch_gemv8<16, 2, 8, 2, true, 1, false>(x, native, Kb, N, ep, stream);
        }
    } else if constexpr (MR == 2 && !PRE) {
        // Two fp16 rows of 8193 .. 16384 indices: eight planes, the shape of an fp32 row's
        if (Kb > 64 || native_blocks_n(N) < 1024) return TMQ_ERR_UNSUPPORTED;
        switch ((Kb + 3) / 4) {
            case 9: return launch_gemv8<16, 4, 9, 2, false, 2, false>(x, native, Kb, N, ep, stream);
            case 10: return launch_gemv8<16, 4, 10, 2, false, 2, false>(x, native, Kb, N, ep, stream);
            case 11: return launch_gemv8<16, 4, 11, 2, false, 2, false>(x, native, Kb, N, ep, stream);
            case 12: return launch_gemv8<16, 4, 12, 2, false, 2, false>(x, native, Kb, N, ep, stream);
            case 13: return launch_gemv8<16, 4, 13, 2, false, 2, false>(x, native, Kb, N, ep, stream);
            case 14: return launch_gemv8<16, 4, 14, 2, false, 2, false>(x, native, Kb, N, ep, stream);
            case 15: return launch_gemv8<16, 4, 15, 2, false, 2, false>(x, native, Kb, N, ep, stream);
            default: return launch_gemv8<16, 4, 16, 2, false, 2, false>(x, native, Kb, N, ep, stream);
        }
    } else if constexpr (MR > 1 && !PRE) {
        return TMQ_ERR_UNSUPPORTED;                              // the planes of such rows stop at 8192 indices
    } else {
        // two channel blocks per workgroup would leave CUs idle on narrow layers, and need two workgroups' LDS per CU
        if (native_blocks_n(N) < 512) {
            switch ((Kb + 7) / 8) {
                case 5: return launch_gemv8<8, 1, 5, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
                case 6: return launch_gemv8<8, 1, 6, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
                case 7: return launch_gemv8<8, 1, 7, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
                default: return launch_gemv8<8, 1, 8, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
            }
        }
        switch ((Kb + 3) / 4) {                                  // 4 wavefronts per channel block
            case 9: return launch_gemv8<8, 2, 9, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
            case 10: return launch_gemv8<8, 2, 10, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
            case 11: return launch_gemv8<8, 2, 11, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
            case 12: return launch_gemv8<8, 2, 12, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
            case 13: return launch_gemv8<8, 2, 13, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
            case 14: return launch_gemv8<8, 2, 14, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
            case 15: return launch_gemv8<8, 2, 15, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
            case 16: return launch_gemv8<8, 2, 16, 2, false, MR, PRE>(x, native, Kb, N, ep, stream);
            default: return TMQ_ERR_UNSUPPORTED;
        }
    }
}

}  // namespace

// True when the 8-bit GEMV can take a dense fp16 problem: one row up to K = 16384, two rows up to 4096 -- every
// workgroup prepares the planes of all rows, and that preparation soon costs more than the weight-stream kernel's
// fp16 expansion (measured: two rows at 4096^2 4.2 -> 3.6 us, at 2048^2 3.1 -> 3.0, at 8192 x 28672 15.5 -> 17.7;
// three or four rows lose at every length -- 2048^2 3.2 -> 3.6 us, 2048 x 11008 4.7 -> 5.9, 4096^2 4.3 -> 5.2 -- and
// reach this kernel only with planes prepared beforehand). Two longer rows where it measured faster (medians,
// weight stream -> this kernel): up to 8192 indices against at most 4096 channels (8192 x 4096 5.1 -> 4.75 us,
// 7168 x 4096 5.2 -> 4.6), up to 6144 indices against at most 6144 channels or when the weight blocks deal out
// evenly over the eight wavefronts (6144 x 11008 7.7 -> 6.85, 6144 x 16384 9.65 -> 8.9; 5120 x 16384 8.3 -> 8.4 and
// 7168 x 11008 8.2 -> 8.8 stay on the weight stream). More than 8192 indices against 16384 or more channels: the
// eight planes fill the LDS like one fp32 row's, the sixteen-wavefront workgroups of that row take them
// (16384^2: 17.9 -> 15.5 us, 12288 x 16384: 13.8 -> 11.9 us; 11008 x 4096, on eight wavefronts: 6.2 -> 7.6 us, refused).
bool gemv8_dense_ok(const void *x, int64_t M, int64_t K, int64_t N) {
    if (M < 1 || M > 2 || K % kKB != 0 || K < 8 * kKB || !aligned16(x)) return false;
    if (M == 2 && K > 32 * kKB) return K <= 64 * kKB && native_blocks_n(N) >= 1024;
    if (M == 2 && K > 16 * kKB) return N <= 4096 || (K <= 24 * kKB && (N <= 6144 || (K / kKB) % 8 == 0));
    return K <= (M == 1 ? 64 : 16) * kKB;
}

// gemv8_dense_ok must hold.
int launch_gemv8_dense(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                       const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream) {
    const Gemv8Epilogue ep{scale, bias, residual, y, relu, y_f16, (int)M};
    const int64_t Kb = K / kKB;
    if (M == 1) return launch_gemv8_by_blocks<false, 1, false>(x, Kb, native, N, ep, stream);
    return launch_gemv8_by_blocks<false, 2, false>(x, Kb, native, N, ep, stream);
}

// One fp32 row: K a multiple of 256 up to 16384 (eight term planes; beyond 8192 they leave room for one workgroup per
// CU only, which then has sixteen wavefronts). Short rows too -- wavefronts without a weight block multiply by zero --
// because the alternative for fp32 is a prescale launch in front of another kernel (K = 1024, N = 4096: 7.1 -> 3.5 us). Two fp32 rows (sixteen planes, all sixteen activation
// columns) while the layer is small: every workgroup splits both rows, which beats a split launch in front of the
// fp16 weight stream up to about 6144^2 (2048^2 5.96 -> 4.3 us, 4096^2 7.45 -> 6.1, 6144^2 9.9 -> 8.7) and loses on
// wider or longer layers (4096 x 11008 9.7 -> 11.5, 8192^2 10.3 -> 11.4, 8192 x 1024 8.1 -> 9.8).
bool gemv8_dense32_ok(const void *x, int64_t M, int64_t K, int64_t N) {
    if (K % kKB != 0 || !aligned16(x)) return false;
    return M == 1 ? K <= 64 * kKB : M == 2 && K <= 24 * kKB && N <= 6144;
}

int launch_gemv8_dense32(const void *x, int64_t M, int64_t K, const void *native, int64_t N, const float *scale, const float *bias,
                         const void *residual, int relu, void *y, int y_f16, void *stream) {
    const Gemv8Epilogue ep{scale, bias, residual, y, relu, y_f16, (int)M};
    if (M == 2) return launch_gemv8_by_blocks<true, 2, false>(x, K / kKB, native, N, ep, stream);
    return launch_gemv8_by_blocks<true, 1, false>(x, K / kKB, native, N, ep, stream);
}

// Ready-made term planes (tmq_gemv8_prepare): rows padded to 1, 2 or 4; up to 64 KiB of planes per workgroup, so
// that two workgroups share a CU (with 128 KiB and one workgroup per CU: two rows at 16384^2 23 us against 18 for
// the weight-stream kernel, four rows at 8192^2 9.4 against 6.4).
int64_t gemv8_padded_rows(int64_t M) { return M <= 1 ? 1 : (M == 2 ? 2 : 4); }

bool gemv8_planes_ok(int64_t M, int64_t K) {
    return M >= 1 && M <= 4 && K % kKB == 0 && K >= 8 * kKB && gemv8_padded_rows(M) * K <= 64 * kKB;
}

int launch_gemv8_planes(const void *planes, int64_t M, int64_t K, const void *native, int64_t N, const float *scale,
                        const float *bias, const void *residual, int relu, void *y, int y_f16, void *stream) {
    const Gemv8Epilogue ep{scale, bias, residual, y, relu, y_f16, (int)M};
    const int64_t Kb = K / kKB;
    switch (gemv8_padded_rows(M)) {
        case 1: return launch_gemv8_by_blocks<false, 1, true>(planes, Kb, native, N, ep, stream);
        case 2: return launch_gemv8_by_blocks<false, 2, true>(planes, Kb, native, N, ep, stream);
        default: return launch_gemv8_by_blocks<false, 4, true>(planes, Kb, native, N, ep, stream);
    }
}

int launch_gemv8_prepare(const void *x, int64_t M, int64_t K, void *planes, void *stream) {
    const int64_t mr = gemv8_padded_rows(M);
    const dim3 grid((uint32_t)((K / 8 + 255) / 256), (uint32_t)mr);
    hipLaunchKernelGGL(gemv8_prepare_kernel, grid, dim3(256), 0, as_stream(stream), static_cast<const _Float16 *>(x), (int)M,
                       (int)K, static_cast<unsigned char *>(planes));
    return check_launch();
}

}  // namespace tmq
