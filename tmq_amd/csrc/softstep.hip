// Soft-staircase transfer function family for gfx950: forward, backward, quantization-loss
// integrand and its gradient, clamp, ternarisation, the fused single pass and the multi-tensor
// forms. All of them are streaming fp32 kernels bounded by HBM bandwidth: every thread moves
// dwordx4 packets (kUnroll of them per tensor, issued before the arithmetic starts) and the
// piecewise-rational evaluation stays in VALU registers.
//
// Arithmetic contract: the reference's CPU path is a chain of separate torch ops, each rounding
// to fp32 (tmq/tmq.py:353-381, 404-438, 456-493). This file is compiled with -ffp-contract=off
// and spells every operation in that association, with IEEE-correct division, so results are
// bit-identical to that chain. Scalars arrive as doubles and are rounded to fp32 once on the
// host (StepK), as torch does with Python scalars.
#include "common.h"
#include "softstep_math.h"

#include <math.h>
#include <mutex>
#include <type_traits>

namespace tmq {
namespace {

#ifndef TMQ_SS_THREADS
#define TMQ_SS_THREADS 512
#endif
#ifndef TMQ_SS_UNROLL
#define TMQ_SS_UNROLL 1
#endif
constexpr int kThreads = TMQ_SS_THREADS;
constexpr int kUnroll = TMQ_SS_UNROLL;                // dwordx4 packets per thread per tensor
constexpr uint32_t kChunk = kThreads * 4 * kUnroll;   // elements per block
typedef float f32x4 __attribute__((ext_vector_type(4)));

// ---- element operators ----------------------------------------------------------------------
// Each Op declares which streams it touches; `apply<CAREFUL>` sees one element.
//   in0  : weight            (always loaded)
//   in1  : second input      (kIn1)
//   out0..out2 : outputs     (kOut0..2); out0 may alias in0 for the in-place ops
//   acc  : per-thread loss accumulator (kLoss). It sums dsig(arg) to ~1 ulp; the constant factor
//          strength*sharpness/c is applied once, in fp64, by the finalisation kernel.
#define TMQ_OP_FLAGS(in1, o0, o1, o2, loss, rd1)                                                   \
    static constexpr bool kIn1 = in1, kOut0 = o0, kOut1 = o1, kOut2 = o2, kLoss = loss, kReadOut1 = rd1

struct FwdOp {  // tmq/tmq.py:417-419
    TMQ_OP_FLAGS(false, true, false, false, false, false);
    StepK s;
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float w, float, float, float &o0, float &, float &, float &) const {
        Frac f = split(w);
        Rational r(clamped_arg<CAREFUL>(f, s.d, s.h));
        float v = cdiv(r.sig(), s.c, s.rc);
        o0 = (v + 0.5f) + f.fw;
        // fw is +-Inf for an infinite weight where the reference has NaN (Inf - Inf in frac)
        if constexpr (CAREFUL) o0 = (f.frac != f.frac) ? f.frac : o0;
    }
};

struct BwdOp {  // tmq/tmq.py:434-438
    TMQ_OP_FLAGS(true, true, false, false, false, false);
    StepK s;
    float scale;
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float w, float g, float, float &o0, float &, float &, float &) const {
        Frac f = split(w);
        Rational r(clamped_arg<CAREFUL>(f, s.d, s.h));
        float grad = cdiv(s.d * r.dsig(), s.c, s.rc);
        o0 = (scale * g) * grad;
    }
};

struct DerivFwdOp {  // tmq/tmq.py:469-473
    TMQ_OP_FLAGS(false, true, false, false, false, false);
    StepK s;
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float w, float, float, float &o0, float &, float &, float &) const {
        Frac f = split(w);
        Rational r(clamped_arg<CAREFUL>(f, s.d, s.h));
        o0 = cdiv(s.k1 * r.dsig(), s.c, s.rc);
    }
};

struct DerivBwdOp {  // tmq/tmq.py:488-493
    TMQ_OP_FLAGS(true, true, false, false, false, false);
    StepK s;
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float w, float g, float, float &o0, float &, float &, float &) const {
        Frac f = split(w);
        Rational r(clamped_arg<CAREFUL>(f, s.d, s.h));
        float grad = cdiv(s.k2 * r.d2sig(), s.c, s.rc);
        o0 = g * grad;
    }
};

struct ClampOp {  // tmq/tmq.py:696, 879 (in place: out0 aliases in0)
    TMQ_OP_FLAGS(false, true, false, false, false, false);
    float lo, hi;
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float w, float, float, float &o0, float &, float &, float &) const {
        o0 = clamp_to<CAREFUL>(w, lo, hi);
    }
};

struct TernarizeOp {  // tmq/tmq.py:293-295 with SoftStep.map 335-338 (in place)
    TMQ_OP_FLAGS(false, true, false, false, false, false);
    StepK s;
    bool use_map;
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float w, float, float, float &o0, float &, float &, float &) const {
        float v = w;
        if (use_map) {
            float fw = floorf(w);
            float arg = (s.d * w - s.d * fw) - s.h;  // association of SoftStep.map
            float x = __builtin_amdgcn_fmed3f(arg, -3.0f, 3.0f);
            if constexpr (CAREFUL) x = (arg != arg) ? arg : x;
            Rational r(x);
            float t = cdiv(r.sig(), s.c, s.rc);
            v = (t + 0.5f) + fw;
            if constexpr (CAREFUL) v = (arg != arg) ? arg : v;
        }
        o0 = rintf(v);  // torch.round: half to even
    }
};

// SoftStep.map / SoftStep.dmap (tmq/tmq.py:328-350): the same staircase and slope with the
// argument association d*w - d*floor(w) - d/2 (map) and w*d - d*floor(w) - d/2 (dmap).
template <bool DERIV>
struct MapOp {
    TMQ_OP_FLAGS(false, true, false, false, false, false);
    StepK s;
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float w, float, float, float &o0, float &, float &, float &) const {
        float fw = floorf(w);
        float arg = (DERIV ? (w * s.d - s.d * fw) : (s.d * w - s.d * fw)) - s.h;
        float x = __builtin_amdgcn_fmed3f(arg, -3.0f, 3.0f);
        if constexpr (CAREFUL) x = (arg != arg) ? arg : x;
        Rational r(x);
        if constexpr (DERIV) {
            o0 = cdiv(s.d * r.dsig(), s.c, s.rc);
        } else {
            float t = cdiv(r.sig(), s.c, s.rc);
            o0 = (t + 0.5f) + fw;
            if constexpr (CAREFUL) o0 = (arg != arg) ? arg : o0;
        }
    }
};

// SoftStep.sigmoid / dsigmoid / d2sigmoid on an arbitrary tensor (tmq/tmq.py:353-381).
template <int WHICH>
struct RationalOp {
    TMQ_OP_FLAGS(false, true, false, false, false, false);
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float v, float, float, float &o0, float &, float &, float &) const {
        float x = __builtin_amdgcn_fmed3f(v, -3.0f, 3.0f);
        x = (v != v) ? v : x;
        Rational r(x);
        o0 = WHICH == 0 ? r.sig() : (WHICH == 1 ? r.dsig() : r.d2sig());
    }
};

// Loss only: acc += dsig(arg). Used by the multi-tensor quantization loss.
struct QLossOp {
    TMQ_OP_FLAGS(false, false, false, false, true, false);
    StepK q;  // sharpness constants
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float w, float, float, float &, float &, float &, float &acc) const {
        Frac f = split(w);
        Rational r(clamped_arg<CAREFUL>(f, q.d, q.h));
        acc += r.dsig_approx();
    }
};

// aux (=|+=) scalar * Q'(w): gradient of the mean quantization loss (out1 is the aux tensor).
template <bool ACC>
struct QLossBwdOp {
    TMQ_OP_FLAGS(false, false, true, false, false, ACC);
    StepK q;
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float w, float, float sc, float &, float &o1, float &, float &) const {
        Frac f = split(w);
        Rational r(clamped_arg<CAREFUL>(f, q.d, q.h));
        float grad = cdiv(q.k2 * r.d2sig(), q.c, q.rc);
        float t = sc * grad;
        o1 = ACC ? (o1 + t) : t;
    }
};

// The fused pass. MASK bits: 1 = y, 2 = dw, 4 = clamp(w), 8 = loss sum.
template <int MASK>
struct FusedOp {
    TMQ_OP_FLAGS((MASK & 2) != 0, (MASK & 1) != 0, (MASK & 2) != 0, (MASK & 4) != 0, (MASK & 8) != 0, false);
    StepK s;  // hardness constants (forward / backward)
    StepK q;  // sharpness constants (quantization loss)
    float gl, lo, hi;
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float w, float g, float, float &o0, float &o1, float &o2, float &acc) const {
        Frac f = split(w);
        if constexpr ((MASK & 3) != 0) {
            Rational r(clamped_arg<CAREFUL>(f, s.d, s.h));
            if constexpr ((MASK & 1) != 0) {
                float v = cdiv(r.sig(), s.c, s.rc);
                o0 = (v + 0.5f) + f.fw;
                if constexpr (CAREFUL) o0 = (f.frac != f.frac) ? f.frac : o0;
            }
            if constexpr ((MASK & 2) != 0) {
                float grad = cdiv(s.d * r.dsig(), s.c, s.rc);
                float t1 = g * grad;  // scale is 1.0 at every reference call site (tmq/tmq.py:650, 812)
                Rational r5(clamped_arg<CAREFUL>(f, q.d, q.h));
                float gq = cdiv(q.k2 * r5.d2sig(), q.c, q.rc);
                float t2 = gl * gq;
                o1 = t1 + t2;
                if constexpr ((MASK & 8) != 0) acc += r5.dsig_approx();
            }
        }
        if constexpr ((MASK & 8) != 0 && (MASK & 2) == 0) {
            Rational r5(clamped_arg<CAREFUL>(f, q.d, q.h));
            acc += r5.dsig_approx();
        }
        if constexpr ((MASK & 4) != 0) o2 = clamp_to<CAREFUL>(w, lo, hi);
    }
};

// Backward of a whole QAT step for one tensor: out1 = g*S'(w) (HAS_G) + sc*Q'(w) (HAS_Q), each term
// rounded as the reference's two backward functions round it (tmq/tmq.py:434-438 with scale 1.0,
// 488-493) and summed once, as autograd's gradient accumulation would. sc is the per-tensor scalar.
template <bool HAS_G, bool HAS_Q>
struct StepBwdOp {
    TMQ_OP_FLAGS(HAS_G, false, true, false, false, false);
    StepK s, q;
    template <bool CAREFUL>
    __device__ __forceinline__ void apply(float w, float g, float sc, float &, float &o1, float &, float &) const {
        Frac f = split(w);
        float t1 = 0.f, t2 = 0.f;
        if constexpr (HAS_G) {
            Rational r(clamped_arg<CAREFUL>(f, s.d, s.h));
            t1 = g * cdiv(s.d * r.dsig(), s.c, s.rc);
        }
        if constexpr (HAS_Q) {
            Rational r5(clamped_arg<CAREFUL>(f, q.d, q.h));
            t2 = sc * cdiv(q.k2 * r5.d2sig(), q.c, q.rc);
        }
        o1 = (HAS_G && HAS_Q) ? (t1 + t2) : (HAS_G ? t1 : t2);
    }
};

// ---- tensor locators ------------------------------------------------------------------------
struct View {
    const float *in0;
    const float *in1;
    float *out0, *out1, *out2;
    uint64_t n;
    uint32_t block;  // block index inside this tensor
    float scalar;
    bool vec;        // all pointers 16-byte aligned
    int seg;         // which tensor of the launch
};

struct Single {
    const float *in0;
    const float *in1;
    float *out0, *out1, *out2;
    uint64_t n;
    bool vec;
    __device__ __forceinline__ View locate(uint32_t b) const {
        return View{in0, in1, out0, out1, out2, n, b, 0.f, vec, 0};
    }
    __device__ __forceinline__ int groups() const { return 1; }
    __device__ __forceinline__ uint32_t group_blocks(int) const { return gridDim.x; }
    __device__ __forceinline__ uint64_t group_elems(int) const { return n; }
};

// Multi-tensor: binary search of the block range table (wave-uniform, scalar loads).
struct Multi {
    const tmq_segment *segs;
    int nseg;
    int inplace;  // out0 = ptr (in-place ops); out1 = aux
    const float *upstream;  // device scalar g: per-tensor scalar becomes g / float(n) (mean backward), or null
    __device__ __forceinline__ View locate(uint32_t b) const {
        int lo = 0, hi = nseg - 1;
        while (lo < hi) {
            int mid = (lo + hi + 1) >> 1;
            if (segs[mid].block_begin <= b) lo = mid;
            else hi = mid - 1;
        }
        const tmq_segment s = segs[lo];
        float *p = static_cast<float *>(s.ptr);
        float *a = static_cast<float *>(s.aux);
        bool vec = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(a)) & 15u) == 0;
        const float sc = upstream ? upstream[0] / (float)s.n : s.scalar;
        return View{p, nullptr, inplace ? p : nullptr, a, nullptr, s.n, b - s.block_begin, sc, vec, lo};
    }
    __device__ __forceinline__ int groups() const { return nseg; }
    __device__ __forceinline__ uint32_t group_blocks(int l) const {
        return (l + 1 < nseg ? segs[l + 1].block_begin : gridDim.x) - segs[l].block_begin;
    }
    __device__ __forceinline__ uint64_t group_elems(int l) const { return segs[l].n; }
};

// Multi-tensor with the table inside the kernel's arguments (nothing to upload: the pointers of a
// training step's gradients change with every step). Up to kArgTensors tensors per launch.
constexpr int kArgTensors = 64;
struct ArgTable {
    const float *w[kArgTensors];
    const float *g[kArgTensors];
    float *out[kArgTensors];
    uint64_t n[kArgTensors];
    uint32_t begin[kArgTensors + 1];   // first block of tensor l; begin[ntensors] = blocks of the launch
    int ntensors;
};
struct MultiArg {
    ArgTable t;
    const float *upstream;   // device scalar u: the per-tensor scalar is u / float(n) (mean backward), or null
    __device__ __forceinline__ View locate(uint32_t b) const {
        int lo = 0, hi = t.ntensors - 1;
        while (lo < hi) {
            int mid = (lo + hi + 1) >> 1;
            if (t.begin[mid] <= b) lo = mid;
            else hi = mid - 1;
        }
        const float *w = t.w[lo];
        const float *g = t.g[lo];
        float *o = t.out[lo];
        const uint64_t n = t.n[lo];
        bool vec = ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(o)) & 15u) == 0;
        const float sc = upstream ? upstream[0] / (float)n : 0.f;
        return View{w, g, o, o, nullptr, n, b - t.begin[lo], sc, vec, lo};
    }
    __device__ __forceinline__ int groups() const { return t.ntensors; }
    __device__ __forceinline__ uint32_t group_blocks(int l) const { return t.begin[l + 1] - t.begin[l]; }
    __device__ __forceinline__ uint64_t group_elems(int l) const { return t.n[l]; }
};

// ---- where a block's loss partial sum goes -----------------------------------------------------
// Partials: one float per block into the workspace; an ordered fp64 finalisation kernel follows.
struct Partials {
    static constexpr int kLanes = 1;
    float *partials;
    template <class Loc>
    __device__ __forceinline__ void commit(float s, const View &, const Loc &) const { partials[blockIdx.x] = s; }
};

// InLaunch: the sum is finished by the launch itself, without a second kernel and without a single
// floating-point addition whose order depends on timing. Thread 0 of a block adds its partial sum as a
// FIXED-POINT INTEGER (integer addition is associative, so a total is the same bits whatever the order of
// arrival) to a 64-bit cell with one returning device-scope atomic, which counts the block in the cell's top
// bits at the same time. The block whose add completes a cell knows the cell's total from the returned value,
// clears the cell and passes the total on to the next level the same way:
//   blocks of a tensor of B > 64 blocks -> its 64 sub cells (block b uses cell b mod 64, so that blocks
//   which run at the same time hit different addresses: atomics on ONE address complete at ~22 per
//   microsecond on this GPU, and a 1152-block layer on a single cell cost 50 us) -> the tensor's top cell;
//   blocks of a smaller tensor -> its top cell directly;
//   the block that completes a top cell turns the total into the tensor's mean (written to per_tensor) and
//   adds the mean / factor, again as an integer, to the launch cell; the block that completes the launch cell
//   writes the total. A launch over one tensor ends at the top cell (sum_out).
// All communication between blocks goes through atomic read-modify-writes, which are coherent whatever cache
// a block's CU sits behind, and a block issues its next atomic only after the previous one has returned, so
// every contribution is in place before the completion that follows it. No fences, no cache write-backs, no
// spinning (nobody waits for anybody); a block that completes nothing pays one atomic, the last block of a
// launch a chain of two or three (~1.5 us each under a streaming load).
//   state (device, 8-byte aligned, tmq_loss_state_bytes()): zero before the first launch that uses it; every
//   launch leaves it zero. Launches that share a state must not overlap.
//   A partial sum that is not a finite number in [0, 2049] (NaN / Inf weights) is counted in the cell's
//   poison field instead, and the result is NaN, as a float sum would be.
// Cell layouts (count | poisoned | sum): sub 15 | 15 | 34 bits, top and launch 7 | 7 | 50 bits. Block sums
// are in units of 2^-F with F = 28 - ceil(log2 B) per tensor (a block contributes less than 2^12: a sub
// cell's B / 64 blocks stay below 2^34, a tensor below 2^40). A float block sum s >= 2^(24 - F) is a
// multiple of the unit, i.e. its conversion is exact (ResNet-18's largest layer, 1152 blocks: F = 17, exact
// from s = 128 on); otherwise the error is at most 2^-(F + 1) per block (B = 2^20: 2^-9 on block sums of
// ~600, 3e-6 -- the 1e-6 bar holds up to 2^18 blocks = 2^29 elements per tensor, which is the limit).
// Means travel as mean / factor in [0, 1] in units of 2^-43. Limits: 64 tensors per launch.
constexpr int kSubs = 64;
constexpr uint32_t kMaxGroupBlocks = 1u << 18;
struct LossState {
    unsigned long long sub[kArgTensors][kSubs];
    unsigned long long top[kArgTensors];
    unsigned long long launch;
    unsigned long long pad;
};

// (count | poisoned | sum) fields of a cell with CB count bits and as many poison bits
template <int CB>
struct Cell {
    static constexpr int kSumBits = 64 - 2 * CB;
    static constexpr unsigned long long kOne = 1ull << (64 - CB), kPoison = 1ull << kSumBits, kSumMask = kPoison - 1;
    static __device__ __forceinline__ unsigned long long pack(bool ok, unsigned long long units) {
        return kOne | (ok ? units : kPoison);
    }
    static __device__ __forceinline__ uint32_t count(unsigned long long c) { return (uint32_t)(c >> (64 - CB)); }
    static __device__ __forceinline__ bool poisoned(unsigned long long c) { return ((c >> kSumBits) & ((1ull << CB) - 1)) != 0; }
    static __device__ __forceinline__ unsigned long long sum(unsigned long long c) { return c & kSumMask; }
};

struct InLaunch {
    static constexpr int kLanes = 1;
    LossState *st;
    double factor;          // strength * sharpness / c
    float *per_tensor;      // optional, [tensors] (multi-tensor launches)
    float *total;           // optional: the sum of the per-tensor means
    double *sum_out;        // single-tensor launches: fp64 sum * factor instead of a mean

    // Called by thread 0 of a block with the block's partial sum.
    template <class Loc>
    __device__ __forceinline__ void commit(float s, const View &v, const Loc &loc) const {
        typedef Cell<15> Sub;
        typedef Cell<7> Top;
        const int grp = v.seg;
        const uint32_t B = loc.group_blocks(grp);
        const int f = 28 - (B <= 1u ? 0 : 32 - __builtin_clz(B - 1u));
        const double unit = __builtin_bit_cast(double, (unsigned long long)(1023 + f) << 52);
        const double inv_unit = __builtin_bit_cast(double, (unsigned long long)(1023 - f) << 52);
        bool ok = s >= 0.f && s <= 2049.f;                             // false for NaN
        unsigned long long units = ok ? (unsigned long long)((double)s * unit + 0.5) : 0ull;
        uint32_t expect = B;                                           // arrivals at the tensor's top cell
        if (B > (uint32_t)kSubs) {
            const uint32_t sub = v.block % (uint32_t)kSubs;
            const unsigned long long add = Sub::pack(ok, units);
            const unsigned long long now = atomicAdd(&st->sub[grp][sub], add) + add;
            if (Sub::count(now) != (B - sub + (uint32_t)kSubs - 1) / (uint32_t)kSubs) return;
            (void)atomicExch(&st->sub[grp][sub], 0ull);
            ok = !Sub::poisoned(now);
            units = Sub::sum(now);
            expect = (uint32_t)kSubs;
        }
        const unsigned long long add = Top::pack(ok, units);
        const unsigned long long now = atomicAdd(&st->top[grp], add) + add;
        if (Top::count(now) != expect) return;
        (void)atomicExch(&st->top[grp], 0ull);
        // this block completed its tensor
        const double avg_unscaled = (double)Top::sum(now) * inv_unit;  // sum of dsig over the tensor
        const bool bad = Top::poisoned(now);
        if (sum_out) {
            sum_out[0] = bad ? __builtin_nan("") : avg_unscaled * factor;
            return;
        }
        const double avg = avg_unscaled / (double)loc.group_elems(grp);   // in [0, 1]
        if (per_tensor) per_tensor[grp] = bad ? __builtin_nanf("") : (float)(avg * factor);
        const int ngrp = loc.groups();
        int live = 0;                                                  // tensors that have blocks at all
        for (int g = 0; g < ngrp; g++) live += loc.group_blocks(g) != 0u;
        const unsigned long long addl = Top::pack(!bad, (unsigned long long)(avg * 8796093022208.0 + 0.5));   // 2^43
        const unsigned long long all = atomicAdd(&st->launch, addl) + addl;
        if (Top::count(all) != (uint32_t)live) return;
        (void)atomicExch(&st->launch, 0ull);
        // this block completed the launch; an empty tensor's mean is NaN (torch.mean of nothing), and so is the total then
        if (live != ngrp && per_tensor)
            for (int g = 0; g < ngrp; g++)
                if (loc.group_blocks(g) == 0u) per_tensor[g] = __builtin_nanf("");
        if (total)
            *total = (Top::poisoned(all) || live != ngrp) ? __builtin_nanf("")
                                                          : (float)((double)Top::sum(all) * (1.0 / 8796093022208.0) * factor);
    }
};

// ---- the streaming kernel ---------------------------------------------------------------------
template <class Op, class Loc, class Fin = Partials>
__global__ __launch_bounds__(kThreads) void stream_kernel(Loc loc, Op op, Fin fin) {
    __shared__ float lds[16];
    const View v = loc.locate(blockIdx.x);
    const uint64_t base = (uint64_t)v.block * kChunk;
    const int tid = threadIdx.x;
    float acc = 0.f;

    if (base + kChunk <= v.n && v.vec) {
        // Full chunk: issue every load first, then compute, then store. Each tensor is touched
        // exactly once per pass, so accesses are marked non-temporal (streaming).
        f32x4 a[kUnroll], b[kUnroll], r1[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint64_t i = base + (uint64_t)(u * kThreads + tid) * 4;
            a[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(v.in0 + i));
            if constexpr (Op::kIn1) b[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(v.in1 + i));
            else b[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            if constexpr (Op::kReadOut1) r1[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(v.out1 + i));
        }
        auto run = [&](auto careful) {
            constexpr bool CAREFUL = decltype(careful)::value;
#pragma unroll
            for (int u = 0; u < kUnroll; u++) {
                const uint64_t i = base + (uint64_t)(u * kThreads + tid) * 4;
                f32x4 o0, o1, o2;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float t0, t1 = 0.f, t2;
                    if constexpr (Op::kReadOut1) t1 = r1[u][e];
                    op.template apply<CAREFUL>(a[u][e], b[u][e], v.scalar, t0, t1, t2, acc);
                    o0[e] = t0; o1[e] = t1; o2[e] = t2;
                }
                if constexpr (Op::kOut0) __builtin_nontemporal_store(o0, reinterpret_cast<f32x4 *>(v.out0 + i));
                if constexpr (Op::kOut1) __builtin_nontemporal_store(o1, reinterpret_cast<f32x4 *>(v.out1 + i));
                if constexpr (Op::kOut2) __builtin_nontemporal_store(o2, reinterpret_cast<f32x4 *>(v.out2 + i));
            }
        };
        // Vote once per wavefront: NaN / Inf weights take the variant with NaN-preserving clamps.
        bool odd = false;
#pragma unroll
        for (int u = 0; u < kUnroll; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) odd |= not_finite(a[u][e]);
        if (__builtin_amdgcn_ballot_w64(odd) == 0) run(std::false_type{});
        else run(std::true_type{});
    } else {
        // Ragged tail or unaligned tensor: element-wise, coalesced dword accesses.
        for (int u = 0; u < kUnroll * 4; u++) {
            const uint64_t i = base + (uint64_t)(u * kThreads + tid);
            if (i < v.n) {
                float o0, o1 = 0.f, o2;
                float g = 0.f;
                if constexpr (Op::kIn1) g = v.in1[i];
                if constexpr (Op::kReadOut1) o1 = v.out1[i];
                op.template apply<true>(v.in0[i], g, v.scalar, o0, o1, o2, acc);
                if constexpr (Op::kOut0) v.out0[i] = o0;
                if constexpr (Op::kOut1) v.out1[i] = o1;
                if constexpr (Op::kOut2) v.out2[i] = o2;
            }
        }
    }
    if constexpr (Op::kLoss) {
        float s = block_sum(acc, lds);
        if (tid < Fin::kLanes) fin.commit(s, v, loc);
    }
}

// Ordered fp64 finalisation of block partial sums: one workgroup of 16 wavefronts. Segment l owns
// the partials [begin_l, begin_{l+1}); its range is cut into tasks of kTaskLen partials, tasks are
// dealt round-robin to the wavefronts (every load of a task is in flight at once, DPP reduction in
// fp64), and one thread then adds the task sums in order. mean_l = float(sum_l / n_l); total = fp32
// running sum in table order (the reference adds per-layer means one by one, tmq/tmq.py:309).
// Deterministic: no atomics, fixed association.
constexpr int kFinThreads = 1024, kFinWaves = kFinThreads / 64, kTaskLen = 2048, kMaxTasks = 2048;

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Block ranges of the tensors whose partial sums are finalised: from a device table, or by value.
struct DevRanges {
    const tmq_segment *segs;   // null: one range [0, total) without a mean
    int nseg;
    uint32_t total;
    __device__ __forceinline__ int count() const { return nseg; }
    __device__ __forceinline__ uint32_t begin(int l) const { return segs ? segs[l].block_begin : 0u; }
    __device__ __forceinline__ uint32_t end(int l) const { return segs ? (l + 1 < nseg ? segs[l + 1].block_begin : total) : total; }
    __device__ __forceinline__ bool has_mean() const { return segs != nullptr; }
    __device__ __forceinline__ uint64_t elems(int l) const { return segs[l].n; }
};
struct ArgRanges {
    uint64_t n[kArgTensors];
    uint32_t first[kArgTensors + 1];
    int ntensors;
    __device__ __forceinline__ int count() const { return ntensors; }
    __device__ __forceinline__ uint32_t begin(int l) const { return first[l]; }
    __device__ __forceinline__ uint32_t end(int l) const { return first[l + 1]; }
    __device__ __forceinline__ bool has_mean() const { return true; }
    __device__ __forceinline__ uint64_t elems(int l) const { return n[l]; }
};

// carry (device, optional): the running total of the tensors finalised by an earlier launch.
template <class R>
__global__ __launch_bounds__(kFinThreads) void finalize_kernel(R rg, const float *partials, double factor,
                                                              float *per_tensor, float *total, double *sum_out,
                                                              const float *carry) {
    __shared__ double task_sum[kMaxTasks];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int nseg = rg.count();
    uint32_t task = 0;
    for (int l = 0; l < nseg; l++) {
        const uint32_t b0 = rg.begin(l), b1 = rg.end(l);
        const uint32_t ntask = (b1 - b0 + kTaskLen - 1) / kTaskLen;
        for (uint32_t t = 0; t < ntask; t++, task++) {
            if ((int)(task % kFinWaves) != wv) continue;
            const uint32_t t0 = b0 + t * kTaskLen, t1 = min(t0 + (uint32_t)kTaskLen, b1);
            double s = 0.0;
#pragma unroll 8
            for (uint32_t i = t0 + lane; i < t1; i += 64) s += (double)partials[i];
            s = wave_sum_f64(s);
            if (lane == 0) task_sum[task] = s;
        }
    }
    __syncthreads();
    // One thread per tensor: its task sums in order, the factor, the mean. Then thread 0 adds the means
    // in table order (the reference adds per-layer means one by one in fp32, tmq/tmq.py:309).
    __shared__ float means[kFinThreads];
    __shared__ float run_s;
    __shared__ int first_s;
    if (threadIdx.x == 0) {
        run_s = carry ? *carry : 0.f;
        first_s = carry == nullptr;
    }
    for (int l0 = 0; l0 < nseg; l0 += kFinThreads) {
        const int l = l0 + threadIdx.x;
        if (l < nseg) {
            uint32_t tk = 0;
            for (int j = 0; j < l; j++) tk += (rg.end(j) - rg.begin(j) + kTaskLen - 1) / kTaskLen;
            const uint32_t ntask = (rg.end(l) - rg.begin(l) + kTaskLen - 1) / kTaskLen;
            double sum = 0.0;
            for (uint32_t t = 0; t < ntask; t++) sum += task_sum[tk + t];
            sum *= factor;   // partials hold sum dsig; factor = strength*sharpness/c
            if (sum_out) sum_out[l] = sum;
            if (rg.has_mean()) {
                const float mean = (float)(sum / (double)rg.elems(l));   // n == 0 gives NaN like torch.mean of an empty tensor
                if (per_tensor) per_tensor[l] = mean;
                means[threadIdx.x] = mean;
            }
        }
        __syncthreads();
        if (threadIdx.x == 0 && rg.has_mean()) {
            float running = run_s;
            bool first = first_s != 0;
            const int cnt = nseg - l0 < kFinThreads ? nseg - l0 : kFinThreads;
            for (int j = 0; j < cnt; j++) {
                running = first ? means[j] : running + means[j];
                first = false;
            }
            run_s = running;
            first_s = 0;
        }
        __syncthreads();
    }
    if (threadIdx.x == 0 && total && rg.has_mean()) *total = run_s;
}

inline bool finalize_fits(int nseg, uint32_t total_blocks) {
    return (uint64_t)nseg + total_blocks / kTaskLen <= (uint64_t)kMaxTasks;
}

// Exhaustive comparison of the FAST division forms with IEEE division.
//   counts[0..2]: sig / dsig / d2sig mismatches over every fp32 x with |x| <= 3 (and NaN)
//   counts[3]   : x / c mismatches over every mantissa, both signs, three binades
//   counts[4]   : arguments visited by the first sweep
__device__ __forceinline__ bool same_bits(float a, float b) {
    return (__builtin_bit_cast(uint32_t, a) == __builtin_bit_cast(uint32_t, b)) || (a != a && b != b);
}
__global__ __launch_bounds__(kThreads) void selfcheck_kernel(float c, float rc, unsigned long long *counts) {
    unsigned long long bad0 = 0, bad1 = 0, bad2 = 0, bad3 = 0, seen = 0;
    const uint64_t stride = (uint64_t)gridDim.x * kThreads;
    for (uint64_t i = (uint64_t)blockIdx.x * kThreads + threadIdx.x; i < (1ull << 32); i += stride) {
        const float x = __builtin_bit_cast(float, (uint32_t)i);
        if (!(fabsf(x) <= 3.0f) && x == x) continue;
        seen++;
        RationalT<true> f(x);
        RationalT<false> r(x);
        bad0 += !same_bits(f.sig(), r.sig());
        bad1 += !same_bits(f.dsig(), r.dsig());
        bad2 += !same_bits(f.d2sig(), r.d2sig());
    }
    for (uint64_t i = (uint64_t)blockIdx.x * kThreads + threadIdx.x; i < (6ull << 23); i += stride) {
        const uint32_t m = (uint32_t)(i & 0x7FFFFFu), sel = (uint32_t)(i >> 23);
        const uint32_t expo = (sel % 3 == 0) ? 107u : ((sel % 3 == 1) ? 127u : 137u);
        const float x = __builtin_bit_cast(float, ((sel >= 3) ? 0x80000000u : 0u) | (expo << 23) | m);
        bad3 += !same_bits(cdiv_t<true>(x, c, rc), cdiv_t<false>(x, c, rc));
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {   // signed zeros and NaN through the constant division
        const float z[3] = {0.0f, -0.0f, __builtin_nanf("")};
        for (float x : z) bad3 += !same_bits(cdiv_t<true>(x, c, rc), cdiv_t<false>(x, c, rc));
    }
    if (bad0) atomicAdd(&counts[0], bad0);
    if (bad1) atomicAdd(&counts[1], bad1);
    if (bad2) atomicAdd(&counts[2], bad2);
    if (bad3) atomicAdd(&counts[3], bad3);
    atomicAdd(&counts[4], seen);
}

inline uint32_t blocks_for(uint64_t n) { return (uint32_t)((n + kChunk - 1) / kChunk); }
constexpr uint64_t kMaxElems = (uint64_t)0x7FFFFFFFu * kChunk / 2;  // keeps block counts in 31 bits

// Scratch of tmq_softstep_fused_noalloc: the block partial sums of the loss reduction live in a
// file-scope device array instead of a caller-provided workspace, so that entry point never needs a
// device allocation. Every GPU holds its own copy of the array at its own address; the name below is
// only a host-side stand-in, the address comes from hipGetSymbolAddress once per device.
constexpr uint64_t kNoAllocMaxElems = (uint64_t)1 << 29;
constexpr size_t kScratchBytes = (size_t)(kNoAllocMaxElems / kChunk) * sizeof(float);   // 1 MiB
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (looked up on the first call per device).
int scratch_address(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return note_hip_error(e);
    if (dev < 0 || dev >= kMaxDevices) return TMQ_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return note_hip_error(e);
        if (!p) return TMQ_ERR_LAUNCH;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return TMQ_OK;
}

template <class Op, class Fin>
int launch_single_fin(const Op &op, const float *in0, const float *in1, float *o0, float *o1, float *o2, size_t n,
                      const Fin &fin, void *stream) {
    if (n == 0) return TMQ_OK;
    if (n > kMaxElems) return TMQ_ERR_TOO_LARGE;
    Single loc{in0, in1, o0, o1, o2, (uint64_t)n,
               aligned16(in0) && aligned16(in1) && aligned16(o0) && aligned16(o1) && aligned16(o2)};
    hipLaunchKernelGGL((stream_kernel<Op, Single, Fin>), dim3(blocks_for(n)), dim3(kThreads), 0, as_stream(stream), loc, op,
                       fin);
    return check_launch();
}

template <class Op>
int launch_single(const Op &op, const float *in0, const float *in1, float *o0, float *o1, float *o2, size_t n,
                  float *partials, void *stream) {
    return launch_single_fin(op, in0, in1, o0, o1, o2, n, Partials{partials}, stream);
}

template <class Op, class Fin>
int launch_multi_fin(const Op &op, const tmq_segment *segs, int nseg, uint32_t total_blocks, int inplace, const Fin &fin,
                     void *stream, const float *upstream = nullptr) {
    if (nseg < 0 || (nseg > 0 && !segs)) return TMQ_ERR_INVALID_ARG;
    if (nseg == 0 || total_blocks == 0) return TMQ_OK;
    Multi loc{segs, nseg, inplace, upstream};
    hipLaunchKernelGGL((stream_kernel<Op, Multi, Fin>), dim3(total_blocks), dim3(kThreads), 0, as_stream(stream), loc, op,
                       fin);
    return check_launch();
}

template <class Op>
int launch_multi(const Op &op, const tmq_segment *segs, int nseg, uint32_t total_blocks, int inplace, float *partials,
                 void *stream, const float *upstream = nullptr) {
    return launch_multi_fin(op, segs, nseg, total_blocks, inplace, Partials{partials}, stream, upstream);
}

bool bad_hardness(double d) { return !(d > 0.0) || !(d <= 1.0e6); }

// Fills an argument table with tensors [first, first + count) of `ts` that pass `keep`; returns the
// launch's block count (0 = nothing to do) or a negative status.
template <class Keep>
int64_t fill_table(ArgTable &t, const tmq_step_tensor *ts, int first, int count, Keep keep) {
    uint64_t b = 0;
    int k = 0;
    for (int i = first; i < first + count; i++) {
        if (!keep(ts[i])) continue;
        if (ts[i].n > kMaxElems) return TMQ_ERR_TOO_LARGE;
        t.w[k] = ts[i].w;
        t.g[k] = ts[i].g;
        t.out[k] = ts[i].out;
        t.n[k] = ts[i].n;
        t.begin[k] = (uint32_t)b;
        b += blocks_for(ts[i].n);
        if (b > 0x7FFFFFFFull) return TMQ_ERR_TOO_LARGE;
        k++;
    }
    t.begin[k] = (uint32_t)b;
    t.ntensors = k;
    return (int64_t)b;
}

template <class Op, class Fin>
int launch_args_fin(const Op &op, const ArgTable &t, uint32_t blocks, const float *upstream, const Fin &fin, void *stream) {
    MultiArg loc{t, upstream};
    hipLaunchKernelGGL((stream_kernel<Op, MultiArg, Fin>), dim3(blocks), dim3(kThreads), 0, as_stream(stream), loc, op, fin);
    return check_launch();
}

template <class Op>
int launch_args(const Op &op, const ArgTable &t, uint32_t blocks, const float *upstream, float *partials, void *stream) {
    return launch_args_fin(op, t, blocks, upstream, Partials{partials}, stream);
}

}  // namespace
}  // namespace tmq

using namespace tmq;

extern "C" {

int tmq_softstep_fwd(const float *w, float *y, size_t n, double digamma, void *stream) {
    if (n && (!w || !y)) return TMQ_ERR_INVALID_ARG;
    if (bad_hardness(digamma)) return TMQ_ERR_INVALID_ARG;
    FwdOp op{make_step(digamma, 0.0)};
    return launch_single(op, w, nullptr, y, nullptr, nullptr, n, nullptr, stream);
}

int tmq_softstep_bwd(const float *w, const float *g, float *dw, size_t n, double digamma, double scale,
                     void *stream) {
    if (n && (!w || !g || !dw)) return TMQ_ERR_INVALID_ARG;
    if (bad_hardness(digamma)) return TMQ_ERR_INVALID_ARG;
    BwdOp op{make_step(digamma, 0.0), (float)scale};
    return launch_single(op, w, g, dw, nullptr, nullptr, n, nullptr, stream);
}

int tmq_softstep_deriv_fwd(const float *w, float *q, size_t n, double digamma, double strength, void *stream) {
    if (n && (!w || !q)) return TMQ_ERR_INVALID_ARG;
    if (bad_hardness(digamma)) return TMQ_ERR_INVALID_ARG;
    DerivFwdOp op{make_step(digamma, strength)};
    return launch_single(op, w, nullptr, q, nullptr, nullptr, n, nullptr, stream);
}

int tmq_softstep_deriv_bwd(const float *w, const float *g, float *dw, size_t n, double digamma, double strength,
                           void *stream) {
    if (n && (!w || !g || !dw)) return TMQ_ERR_INVALID_ARG;
    if (bad_hardness(digamma)) return TMQ_ERR_INVALID_ARG;
    DerivBwdOp op{make_step(digamma, strength)};
    return launch_single(op, w, g, dw, nullptr, nullptr, n, nullptr, stream);
}

int tmq_softstep_map(const float *w, float *y, size_t n, double digamma, int derivative, void *stream) {
    if (n && (!w || !y)) return TMQ_ERR_INVALID_ARG;
    if (bad_hardness(digamma)) return TMQ_ERR_INVALID_ARG;
    const StepK s = make_step(digamma, 0.0);
    if (derivative) return launch_single(MapOp<true>{s}, w, nullptr, y, nullptr, nullptr, n, nullptr, stream);
    return launch_single(MapOp<false>{s}, w, nullptr, y, nullptr, nullptr, n, nullptr, stream);
}

int tmq_sigmoid_piece(const float *x, float *y, size_t n, int order, void *stream) {
    if (n && (!x || !y)) return TMQ_ERR_INVALID_ARG;
    switch (order) {
        case 0: return launch_single(RationalOp<0>{}, x, nullptr, y, nullptr, nullptr, n, nullptr, stream);
        case 1: return launch_single(RationalOp<1>{}, x, nullptr, y, nullptr, nullptr, n, nullptr, stream);
        case 2: return launch_single(RationalOp<2>{}, x, nullptr, y, nullptr, nullptr, n, nullptr, stream);
        default: return TMQ_ERR_INVALID_ARG;
    }
}

int tmq_clamp_inplace(float *w, size_t n, double lo, double hi, void *stream) {
    if (n && !w) return TMQ_ERR_INVALID_ARG;
    if (!(lo <= hi)) return TMQ_ERR_INVALID_ARG;
    ClampOp op{(float)lo, (float)hi};
    return launch_single(op, w, nullptr, w, nullptr, nullptr, n, nullptr, stream);
}

int tmq_ternarize_inplace(float *w, size_t n, double digamma, void *stream) {
    if (n && !w) return TMQ_ERR_INVALID_ARG;
    const bool use_map = digamma > 0.0;
    if (use_map && bad_hardness(digamma)) return TMQ_ERR_INVALID_ARG;
    TernarizeOp op{make_step(use_map ? digamma : 1.0, 0.0), use_map};
    return launch_single(op, w, nullptr, w, nullptr, nullptr, n, nullptr, stream);
}

size_t tmq_softstep_fused_workspace_bytes(size_t n) { return (size_t)blocks_for(n) * sizeof(float) + 16; }

int tmq_softstep_fused(const float *w, const float *g, float *y, float *dw, float *wc, double *loss_sum,
                       void *workspace, size_t n, double digamma, double sharpness, double strength, float gl,
                       double lo, double hi, void *stream) {
    if (n && !w) return TMQ_ERR_INVALID_ARG;
    if (dw && !g) return TMQ_ERR_INVALID_ARG;
    if (loss_sum && !workspace) return TMQ_ERR_INVALID_ARG;
    if (bad_hardness(digamma) || bad_hardness(sharpness) || !(lo <= hi)) return TMQ_ERR_INVALID_ARG;
    if (n > kMaxElems || (loss_sum && !finalize_fits(1, blocks_for(n)))) return TMQ_ERR_TOO_LARGE;
    const int mask = (y ? 1 : 0) | (dw ? 2 : 0) | (wc ? 4 : 0) | (loss_sum ? 8 : 0);
    if (mask == 0) return TMQ_OK;
    float *partials = static_cast<float *>(workspace);
    const StepK s = make_step(digamma, 0.0), q = make_step(sharpness, strength);
    int rc = TMQ_OK;
    if (n) {
        switch (mask) {
#define TMQ_CASE(M)                                                                               \
    case M: {                                                                                     \
        FusedOp<M> op{s, q, gl, (float)lo, (float)hi};                                            \
        rc = launch_single(op, w, g, y, dw, wc, n, partials, stream);                             \
    } break;
            TMQ_CASE(1) TMQ_CASE(2) TMQ_CASE(3) TMQ_CASE(4) TMQ_CASE(5) TMQ_CASE(6) TMQ_CASE(7) TMQ_CASE(8)
            TMQ_CASE(9) TMQ_CASE(10) TMQ_CASE(11) TMQ_CASE(12) TMQ_CASE(13) TMQ_CASE(14) TMQ_CASE(15)
#undef TMQ_CASE
        }
        if (rc != TMQ_OK) return rc;
    }
    if (loss_sum) {
        hipLaunchKernelGGL(finalize_kernel<DevRanges>, dim3(1), dim3(kFinThreads), 0, as_stream(stream),
                           DevRanges{nullptr, 1, blocks_for(n)}, partials, (double)q.k1 / (double)q.c, nullptr, nullptr,
                           loss_sum, nullptr);
        rc = check_launch();
    }
    return rc;
}

size_t tmq_loss_state_bytes(void) { return sizeof(LossState); }

int tmq_softstep_fused_inlaunch(const float *w, const float *g, float *y, float *dw, float *wc, double *loss_sum,
                                void *state, size_t n, double digamma, double sharpness, double strength, float gl,
                                double lo, double hi, void *stream) {
    if (!loss_sum || !state || (reinterpret_cast<uintptr_t>(state) & 7u)) return TMQ_ERR_INVALID_ARG;
    if (n == 0 || !w || (dw && !g)) return TMQ_ERR_INVALID_ARG;   // a sum over nothing: no block would write it
    if (bad_hardness(digamma) || bad_hardness(sharpness) || !(lo <= hi)) return TMQ_ERR_INVALID_ARG;
    if (n > kMaxElems) return TMQ_ERR_TOO_LARGE;
    if (blocks_for(n) > kMaxGroupBlocks) return TMQ_ERR_UNSUPPORTED;
    const int mask = (y ? 1 : 0) | (dw ? 2 : 0) | (wc ? 4 : 0) | 8;
    const StepK s = make_step(digamma, 0.0), q = make_step(sharpness, strength);
    const InLaunch fin{static_cast<LossState *>(state), (double)q.k1 / (double)q.c, nullptr, nullptr, loss_sum};
    switch (mask) {
#define TMQ_CASE(M)                                                                               \
    case M: {                                                                                     \
        FusedOp<M> op{s, q, gl, (float)lo, (float)hi};                                            \
        return launch_single_fin(op, w, g, y, dw, wc, n, fin, stream);                            \
    }
        TMQ_CASE(8) TMQ_CASE(9) TMQ_CASE(10) TMQ_CASE(11) TMQ_CASE(12) TMQ_CASE(13) TMQ_CASE(14) TMQ_CASE(15)
#undef TMQ_CASE
    }
    return TMQ_ERR_INVALID_ARG;
}

int tmq_softstep_fused_noalloc(const float *w, const float *g, float *y, float *dw, float *wc, double *loss_sum,
                               size_t n, double digamma, double sharpness, double strength, float gl, double lo,
                               double hi, void *stream) {
    if (n > kNoAllocMaxElems) return TMQ_ERR_TOO_LARGE;
    void *ws = nullptr;
    if (loss_sum) {
        // Every block of this call writes its own partial sum before the finalisation reads exactly
        // those, so nothing in the array has to start at zero; what earlier calls left behind it is
        // never read.
        const int rc = scratch_address(&ws);
        if (rc != TMQ_OK) return rc;
    }
    return tmq_softstep_fused(w, g, y, dw, wc, loss_sum, ws, n, digamma, sharpness, strength, gl, lo, hi, stream);
}

size_t tmq_softstep_fused_noalloc_max_elements(void) { return (size_t)kNoAllocMaxElems; }

int tmq_selfcheck_division(double digamma, uint64_t *counts, void *stream) {
    if (!counts || bad_hardness(digamma)) return TMQ_ERR_INVALID_ARG;
    const StepK s = make_step(digamma, 0.0);
    hipError_t e = hipMemsetAsync(counts, 0, 5 * sizeof(uint64_t), as_stream(stream));
    if (e != hipSuccess) return note_hip_error(e);
    hipLaunchKernelGGL(selfcheck_kernel, dim3(8192), dim3(kThreads), 0, as_stream(stream), s.c, s.rc,
                       reinterpret_cast<unsigned long long *>(counts));
    return check_launch();
}

int tmq_multi_plan(tmq_segment *segs, int nseg, uint32_t *total_blocks) {
    if (nseg < 0 || (nseg > 0 && !segs) || !total_blocks) return TMQ_ERR_INVALID_ARG;
    uint64_t b = 0;
    for (int i = 0; i < nseg; i++) {
        if (segs[i].n > kMaxElems) return TMQ_ERR_TOO_LARGE;
        segs[i].block_begin = (uint32_t)b;
        b += blocks_for(segs[i].n);
        if (b > 0x7FFFFFFFull) return TMQ_ERR_TOO_LARGE;
    }
    *total_blocks = (uint32_t)b;
    return TMQ_OK;
}

size_t tmq_qloss_multi_workspace_bytes(uint32_t total_blocks) { return (size_t)total_blocks * sizeof(float) + 16; }

int tmq_qloss_multi(const tmq_segment *segs, int nseg, uint32_t total_blocks, double sharpness, double strength,
                    float *per_tensor, float *total, void *workspace, void *stream) {
    if (nseg <= 0 || !segs || !workspace) return TMQ_ERR_INVALID_ARG;
    if (bad_hardness(sharpness)) return TMQ_ERR_INVALID_ARG;
    if (!finalize_fits(nseg, total_blocks)) return TMQ_ERR_TOO_LARGE;
    float *partials = static_cast<float *>(workspace);
    QLossOp op{make_step(sharpness, strength)};
    int rc = launch_multi(op, segs, nseg, total_blocks, 0, partials, stream);
    if (rc != TMQ_OK) return rc;
    hipLaunchKernelGGL(finalize_kernel<DevRanges>, dim3(1), dim3(kFinThreads), 0, as_stream(stream),
                       DevRanges{segs, nseg, total_blocks}, partials, (double)op.q.k1 / (double)op.q.c, per_tensor, total,
                       nullptr, nullptr);
    return check_launch();
}

int tmq_qloss_multi_inlaunch(const tmq_segment *segs, int nseg, uint32_t total_blocks, double sharpness, double strength,
                             float *per_tensor, float *total, void *state, void *stream) {
    if (nseg <= 0 || !segs || !state || (reinterpret_cast<uintptr_t>(state) & 7u) || total_blocks == 0) return TMQ_ERR_INVALID_ARG;
    if (bad_hardness(sharpness)) return TMQ_ERR_INVALID_ARG;
    // the table lives on the device: bound every tensor's block count by the launch's
    if (nseg > kArgTensors || total_blocks > kMaxGroupBlocks) return TMQ_ERR_UNSUPPORTED;
    QLossOp op{make_step(sharpness, strength)};
    const InLaunch fin{static_cast<LossState *>(state), (double)op.q.k1 / (double)op.q.c, per_tensor, total, nullptr};
    return launch_multi_fin(op, segs, nseg, total_blocks, 0, fin, stream);
}

int tmq_qloss_bwd_multi(const tmq_segment *segs, int nseg, uint32_t total_blocks, double sharpness, double strength,
                        const float *upstream, int accumulate, void *stream) {
    if (bad_hardness(sharpness)) return TMQ_ERR_INVALID_ARG;
    const StepK q = make_step(sharpness, strength);
    if (accumulate) return launch_multi(QLossBwdOp<true>{q}, segs, nseg, total_blocks, 0, nullptr, stream, upstream);
    return launch_multi(QLossBwdOp<false>{q}, segs, nseg, total_blocks, 0, nullptr, stream, upstream);
}

size_t tmq_softstep_multi_workspace_bytes(const tmq_step_tensor *ts, int ntensors) {
    uint64_t b = 0;
    for (int i = 0; ts && i < ntensors; i++) b += blocks_for(ts[i].n);
    return (size_t)b * sizeof(float) + 16;
}

int tmq_softstep_fwd_multi(const tmq_step_tensor *ts, int ntensors, double digamma, double sharpness, double strength,
                           float *loss_per_tensor, float *loss_total, void *workspace, void *stream) {
    if (ntensors < 0 || (ntensors > 0 && !ts)) return TMQ_ERR_INVALID_ARG;
    const bool want_loss = loss_per_tensor || loss_total;
    if (bad_hardness(digamma) || (want_loss && (bad_hardness(sharpness) || !workspace))) return TMQ_ERR_INVALID_ARG;
    for (int i = 0; i < ntensors; i++)
        if (ts[i].n && (!ts[i].w || !ts[i].out)) return TMQ_ERR_INVALID_ARG;
    const StepK s = make_step(digamma, 0.0), q = make_step(want_loss ? sharpness : 1.0, want_loss ? strength : 0.0);
    float *partials = static_cast<float *>(workspace);
    bool carried = false;
    if (ntensors == 0 && want_loss) return TMQ_ERR_INVALID_ARG;   // a sum over no tensors: nothing would write it
    for (int first = 0; first < ntensors; first += kArgTensors) {
        const int count = ntensors - first < kArgTensors ? ntensors - first : kArgTensors;
        ArgTable t;
        const int64_t blocks = fill_table(t, ts, first, count, [](const tmq_step_tensor &) { return true; });
        if (blocks < 0) return (int)blocks;
        if (want_loss && !finalize_fits(t.ntensors, (uint32_t)blocks)) return TMQ_ERR_TOO_LARGE;
        int rc = TMQ_OK;
        if (blocks > 0) {
            if (want_loss) rc = launch_args(FusedOp<9>{s, q, 0.f, 0.f, 0.f}, t, (uint32_t)blocks, nullptr, partials, stream);
            else rc = launch_args(FusedOp<1>{s, q, 0.f, 0.f, 0.f}, t, (uint32_t)blocks, nullptr, nullptr, stream);
            if (rc != TMQ_OK) return rc;
        }
        if (want_loss) {
            ArgRanges rg;
            for (int k = 0; k < t.ntensors; k++) { rg.n[k] = t.n[k]; rg.first[k] = t.begin[k]; }
            rg.first[t.ntensors] = t.begin[t.ntensors];
            rg.ntensors = t.ntensors;
            hipLaunchKernelGGL(finalize_kernel<ArgRanges>, dim3(1), dim3(kFinThreads), 0, as_stream(stream), rg, partials,
                               (double)q.k1 / (double)q.c, loss_per_tensor ? loss_per_tensor + first : nullptr, loss_total,
                               nullptr, carried ? loss_total : nullptr);
            rc = check_launch();
            if (rc != TMQ_OK) return rc;
            carried = true;
            partials += blocks;
        }
    }
    return TMQ_OK;
}

int tmq_softstep_fwd_multi_inlaunch(const tmq_step_tensor *ts, int ntensors, double digamma, double sharpness,
                                    double strength, float *loss_per_tensor, float *loss_total, void *state, void *stream) {
    if (ntensors <= 0 || !ts || !state || (reinterpret_cast<uintptr_t>(state) & 7u)) return TMQ_ERR_INVALID_ARG;
    if (!loss_per_tensor && !loss_total) return TMQ_ERR_INVALID_ARG;
    if (bad_hardness(digamma) || bad_hardness(sharpness)) return TMQ_ERR_INVALID_ARG;
    if (ntensors > kArgTensors) return TMQ_ERR_UNSUPPORTED;
    uint64_t elems = 0;
    for (int i = 0; i < ntensors; i++) {
        if (ts[i].n && (!ts[i].w || !ts[i].out)) return TMQ_ERR_INVALID_ARG;
        if ((ts[i].n + kChunk - 1) / kChunk > kMaxGroupBlocks) return TMQ_ERR_UNSUPPORTED;
        elems += ts[i].n;
    }
    if (elems == 0) return TMQ_ERR_UNSUPPORTED;                   // no block would finish the sum
    const StepK s = make_step(digamma, 0.0), q = make_step(sharpness, strength);
    ArgTable t;
    const int64_t blocks = fill_table(t, ts, 0, ntensors, [](const tmq_step_tensor &) { return true; });
    if (blocks < 0) return (int)blocks;
    const InLaunch fin{static_cast<LossState *>(state), (double)q.k1 / (double)q.c, loss_per_tensor, loss_total, nullptr};
    return launch_args_fin(FusedOp<9>{s, q, 0.f, 0.f, 0.f}, t, (uint32_t)blocks, nullptr, fin, stream);
}

int tmq_softstep_bwd_multi(const tmq_step_tensor *ts, int ntensors, double digamma, double sharpness, double strength,
                           const float *loss_upstream, void *stream) {
    if (ntensors < 0 || (ntensors > 0 && !ts)) return TMQ_ERR_INVALID_ARG;
    if (bad_hardness(digamma) || (loss_upstream && bad_hardness(sharpness))) return TMQ_ERR_INVALID_ARG;
    for (int i = 0; i < ntensors; i++) {
        if (ts[i].n && (!ts[i].w || !ts[i].out)) return TMQ_ERR_INVALID_ARG;
        if (!ts[i].g && !loss_upstream) return TMQ_ERR_INVALID_ARG;   // no gradient reaches this tensor: leave it out
    }
    const StepK s = make_step(digamma, 0.0), q = make_step(loss_upstream ? sharpness : 1.0, loss_upstream ? strength : 0.0);
    for (int first = 0; first < ntensors; first += kArgTensors) {
        const int count = ntensors - first < kArgTensors ? ntensors - first : kArgTensors;
        ArgTable t;
        int64_t blocks = fill_table(t, ts, first, count, [](const tmq_step_tensor &x) { return x.g != nullptr; });
        if (blocks < 0) return (int)blocks;
        int rc = TMQ_OK;
        if (blocks > 0) {
            if (loss_upstream) rc = launch_args(StepBwdOp<true, true>{s, q}, t, (uint32_t)blocks, loss_upstream, nullptr, stream);
            else rc = launch_args(StepBwdOp<true, false>{s, q}, t, (uint32_t)blocks, nullptr, nullptr, stream);
            if (rc != TMQ_OK) return rc;
        }
        if (loss_upstream) {   // tensors the forward pass did not use: the loss term alone
            blocks = fill_table(t, ts, first, count, [](const tmq_step_tensor &x) { return x.g == nullptr; });
            if (blocks < 0) return (int)blocks;
            if (blocks > 0) {
                rc = launch_args(StepBwdOp<false, true>{s, q}, t, (uint32_t)blocks, loss_upstream, nullptr, stream);
                if (rc != TMQ_OK) return rc;
            }
        }
    }
    return TMQ_OK;
}

int tmq_clamp_multi(const tmq_segment *segs, int nseg, uint32_t total_blocks, double lo, double hi, void *stream) {
    if (!(lo <= hi)) return TMQ_ERR_INVALID_ARG;
    return launch_multi(ClampOp{(float)lo, (float)hi}, segs, nseg, total_blocks, 1, nullptr, stream);
}

}  // extern "C"
