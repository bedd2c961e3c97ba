// Per-element arithmetic of the soft-staircase family (device) and its host-rounded scalars.
//
// Contract: bit-identical to the reference's CPU chain of separately rounded fp32 torch ops
// (tmq/tmq.py:353-381, 404-438, 456-493). Every multiply/add below is written in that
// association and the file must be compiled with -ffp-contract=off.
//
// Divisions are the expensive part of that chain (eight per element in the fused pass). Two
// forms are provided and selected at compile time:
//   * IEEE: the compiler's correctly rounded `/` (v_div_scale, v_rcp, Newton, v_div_fmas,
//     v_div_fixup: ~15 issue slots each);
//   * FAST (default): the same Newton/residual refinement written out with explicit FMAs but
//     without the scale/fix-up steps, which only matter for exponents this chain never sees,
//     and with one v_rcp_f32 shared by the divisions of a chain. Division by a launch constant
//     uses a host-computed correctly rounded reciprocal and two residual corrections (five FMAs),
//     which is correctly rounded by Markstein's theorem. The variable divisions are proven
//     equal to IEEE division by exhaustion: tmq_selfcheck_division() compares both forms over
//     every fp32 argument in [-3, 3] on the device.
#pragma once

#include <math.h>
#include <stdint.h>

#ifndef TMQ_FAST_DIV
#define TMQ_FAST_DIV 1
#endif

namespace tmq {

// Host-rounded scalars of one staircase evaluation.
struct StepK {
    float d;    // float(digamma)
    float h;    // float(digamma / 2)
    float c;    // float(2 * sig(digamma / 2))
    float rc;   // correctly rounded 1 / c
    float k1;   // float(strength * digamma)
    float k2;   // float(strength * digamma * digamma)
};

inline double scalar_sigmoid(double in) {  // tmq/tmq.py:384-391, evaluated in double like Python
    double x = fmin(3.0, fmax(-3.0, in));
    double x2 = x * x;
    return x * (x2 + 27.0) / (27.0 + x2 * 9.0);
}

// RN(1/c) for a positive normal fp32 c: start from the double quotient and pick the neighbour
// with the smallest exact residual |1 - c*r| (the products are exact in double).
inline float exact_reciprocal(float c) {
    float r = (float)(1.0 / (double)c);
    float cand[3] = {nextafterf(r, 0.0f), r, nextafterf(r, INFINITY)};
    float best = r;
    double berr = fabs(1.0 - (double)c * (double)r);
    for (float v : cand) {
        double err = fabs(1.0 - (double)c * (double)v);
        if (err < berr) { berr = err; best = v; }
    }
    return best;
}

inline StepK make_step(double digamma, double strength) {
    StepK k;
    k.d = (float)digamma;
    k.h = (float)(digamma / 2.0);
    k.c = (float)(2.0 * scalar_sigmoid(digamma / 2.0));
    k.rc = exact_reciprocal(k.c);
    k.k1 = (float)(strength * digamma);
    k.k2 = (float)(strength * digamma * digamma);
    return k;
}

#if defined(__HIPCC__)

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

// x / c for a launch constant c > 0 with rc = RN(1/c). q1 is faithful (error < 1 ulp), the
// second correction rounds correctly (Markstein). Residuals are formed as fma(q, c, -x) and
// negated at use so that a -0 numerator keeps its sign.
template <bool FAST>
__device__ __forceinline__ float cdiv_t(float x, float c, float rc) {
    if constexpr (FAST) {
        float q0 = x * rc;
        float r0 = fma_(q0, c, -x);
        float q1 = fma_(-r0, rc, q0);
        float r1 = fma_(q1, c, -x);
        return fma_(-r1, rc, q1);
    } else {
        return x / c;
    }
}
__device__ __forceinline__ float cdiv(float x, float c, float rc) { return cdiv_t<TMQ_FAST_DIV != 0>(x, c, rc); }

// a / b given y0 ~ 1/b (relative error below 2^-18): one Newton step on the reciprocal, then
// quotient, residual correction, second residual correction -- the refinement the compiler's
// IEEE division performs after v_rcp_f32, minus scaling and fix-up.
__device__ __forceinline__ float vdiv(float a, float b, float y0) {
    float e = fma_(-b, y0, 1.0f);
    float y1 = fma_(e, y0, y0);
    float q0 = a * y1;
    float r0 = fma_(q0, b, -a);
    float q1 = fma_(-r0, y1, q0);
    float r1 = fma_(q1, b, -a);
    return fma_(-r1, y1, q1);
}

__device__ __forceinline__ float rcp_(float x) { return __builtin_amdgcn_rcpf(x); }

// The three rational pieces at one clamped argument x (|x| <= 3 or NaN). They share x^2 and,
// in the FAST form, one reciprocal of b = 3 + x^2: 27 + 9x^2 ~ 9b, (9b)b, ((3b)b)b.
template <bool FAST>
struct RationalT {
    float x, x2, b, rb;
    __device__ __forceinline__ explicit RationalT(float xc) : x(xc) {
        x2 = x * x;
        b = 3.0f + x2;   // == x2 + 3.0f bit for bit (addition commutes)
        rb = FAST ? rcp_(b) : 0.f;
    }
    // tmq/tmq.py:359-360: (x*(x2+27)) / (27 + x2*9)
    __device__ __forceinline__ float sig() const {
        float num = x * (x2 + 27.0f);
        float den = 27.0f + x2 * 9.0f;
        if constexpr (FAST) return vdiv(num, den, rb * 0.11111111f);
        else return num / den;
    }
    // tmq/tmq.py:369-370: ((x2-9)*(x2-9)) / ((9*(3+x2))*(3+x2))
    __device__ __forceinline__ float dsig() const {
        float a = x2 - 9.0f;
        float num = a * a;
        float den = (9.0f * b) * b;
        if constexpr (FAST) return vdiv(num, den, (rb * 0.11111111f) * rb);
        else return num / den;
    }
    // dsig to ~1 ulp (no residual corrections): used only inside the loss reduction, whose
    // result is a sum compared with a relative tolerance, never element by element.
    __device__ __forceinline__ float dsig_approx() const {
        float a = x2 - 9.0f;
        float num = a * a;
        float den = (9.0f * b) * b;
        float y0 = ((FAST ? rb : rcp_(b)) * 0.11111111f) * (FAST ? rb : rcp_(b));
        float e = fma_(-den, y0, 1.0f);
        float y1 = fma_(e, y0, y0);
        return num * y1;
    }
    // tmq/tmq.py:379-381: ((16*x)*(x2-9)) / (((3*a)*a)*a), a = x2+3
    __device__ __forceinline__ float d2sig() const {
        float num = (16.0f * x) * (x2 - 9.0f);
        float den = ((3.0f * b) * b) * b;
        if constexpr (FAST) return vdiv(num, den, ((rb * 0.33333334f) * rb) * rb);
        else return num / den;
    }
};
using Rational = RationalT<TMQ_FAST_DIV != 0>;

// NaN / Inf weights: torch.clamp propagates NaN where v_med3_f32 returns a bound, so such
// elements need two extra selects per chain. The streaming kernel evaluates a chunk with
// CAREFUL = false (v_med3 only), votes across the wavefront whether any weight was not finite,
// and only then re-evaluates the chunk with CAREFUL = true. Finite weights give identical bits
// in both modes.
__device__ __forceinline__ bool not_finite(float w) { return !(__builtin_fabsf(w) < INFINITY); }

// frac = w - floor(w)
struct Frac {
    float fw, frac;
};
__device__ __forceinline__ Frac split(float w) {
    Frac f;
    f.fw = floorf(w);
    f.frac = w - f.fw;
    return f;
}

// x = clamp(d*frac - h, -3, 3) (tmq/tmq.py:358, 418); CAREFUL keeps a NaN argument NaN.
template <bool CAREFUL>
__device__ __forceinline__ float clamped_arg(const Frac &f, float d, float h) {
    float t = d * f.frac;
    float arg = t - h;
    float x = __builtin_amdgcn_fmed3f(arg, -3.0f, 3.0f);
    if constexpr (CAREFUL) return (arg != arg) ? arg : x;
    else return x;
}

template <bool CAREFUL>
__device__ __forceinline__ float clamp_to(float w, float lo, float hi) {
    float x = __builtin_amdgcn_fmed3f(w, lo, hi);
    if constexpr (CAREFUL) return (w != w) ? w : x;
    else return x;
}

#endif  // __HIPCC__

}  // namespace tmq
