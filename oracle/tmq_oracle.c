/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement ("oracle") of the TMQ hot path.
 *
 * Nothing in the shipped package may import, link or call this file. It is used by tests/,
 * by __graft_entry__.smoke() and by bench.py's cpu_baseline leg as the checker / the timed CPU
 * baseline. Plain C, one thread, compiled with -ffp-contract=off so that every fp32 operation
 * is rounded separately, exactly like the chain of separate torch CPU ops in the reference.
 *
 * Every function names the reference lines it restates (paths relative to the reference root).
 *
 * Pinning status (what proves each function right is in tests/test_oracle_*.py):
 *   soft-step family  : exact rationals of the closed forms, fp64 finite differences, symmetry
 *                       and fixed-point invariants, and bit-equality with an independent
 *                       op-for-op torch restatement (oracle/torch_path.py).
 *   pack / unpack     : hand-computed words, brute force over all byte patterns, round trip,
 *                       and the compiled reference (oracle/_ref) where it builds.
 *   gemm / conv       : reduces to a textbook fp64 matrix product on expanded weights.
 *   range coder       : the compiled reference (oracle/_ref) byte-for-byte, round trip.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------
 * Host scalars. The reference evaluates them as Python doubles and hands them to torch, which
 * rounds a Python scalar to fp32 once when it meets an fp32 tensor.
 *   scalar_sigmoid            tmq/tmq.py:384-391
 *   d32 = float(digamma)      tmq/tmq.py:418 ("ctrl.digamma * (weight - fw)")
 *   h32 = float(digamma/2.0)  tmq/tmq.py:418 ("- ctrl.digamma / 2.0")
 *   c32 = float(2.0*sig(d/2)) tmq/tmq.py:419
 * ---------------------------------------------------------------------------------------- */
static double scalar_sigmoid(double in) {
    double x = fmin(3.0, fmax(-3.0, in));
    double x2 = x * x;
    return x * (x2 + 27.0) / (27.0 + x2 * 9.0);
}

void tmq_oracle_consts(double digamma, float *d32, float *h32, float *c32) {
    *d32 = (float)digamma;
    *h32 = (float)(digamma / 2.0);
    *c32 = (float)(2.0 * scalar_sigmoid(digamma / 2.0));
}

/* torch.clamp(x, lo, hi) on fp32: NaN stays NaN (tmq/tmq.py:358, 368, 378). */
static inline float clampf(float x, float lo, float hi) {
    if (x != x) return x;
    float t = x < lo ? lo : x;
    return t > hi ? hi : t;
}

/* SoftStep.sigmoid, tmq/tmq.py:353-360: x*(x2+27) / (27 + x2*9) */
static inline float sig32(float arg) {
    float x = clampf(arg, -3.0f, 3.0f);
    float x2 = x * x;
    float num = x * (x2 + 27.0f);
    float den = 27.0f + x2 * 9.0f;
    return num / den;
}

/* SoftStep.dsigmoid, tmq/tmq.py:363-370: ((x2-9)*(x2-9)) / ((9*(3+x2))*(3+x2)) */
static inline float dsig32(float arg) {
    float x = clampf(arg, -3.0f, 3.0f);
    float x2 = x * x;
    float a = x2 - 9.0f;
    float b = 3.0f + x2;
    float num = a * a;
    float den = (9.0f * b) * b;
    return num / den;
}

/* SoftStep.d2sigmoid, tmq/tmq.py:373-381: ((16*x)*(x2-9)) / (((3*a)*a)*a), a = x2+3 */
static inline float d2sig32(float arg) {
    float x = clampf(arg, -3.0f, 3.0f);
    float x2 = x * x;
    float a = x2 + 3.0f;
    float num = (16.0f * x) * (x2 - 9.0f);
    float den = ((3.0f * a) * a) * a;
    return num / den;
}

/* SoftStep.forward CPU branch, tmq/tmq.py:417-419:
 *   fw = floor(w); arg = d*(w-fw) - d/2; y = sigmoid(arg)/(2*sig(d/2)) + 0.5 + fw          */
void tmq_oracle_softstep_fwd(const float *w, float *y, size_t n, double digamma) {
    float d32, h32, c32;
    tmq_oracle_consts(digamma, &d32, &h32, &c32);
    for (size_t i = 0; i < n; i++) {
        float fw = floorf(w[i]);
        float frac = w[i] - fw;
        float arg = d32 * frac - h32;
        float s = sig32(arg) / c32;
        y[i] = (s + 0.5f) + fw;
    }
}

/* SoftStep.backward CPU branch, tmq/tmq.py:434-438:
 *   grad = (d*dsigmoid(arg))/(2*sig(d/2)); out = (scale*g)*grad                            */
void tmq_oracle_softstep_bwd(const float *w, const float *g, float *dw, size_t n, double digamma,
                             double scale) {
    float d32, h32, c32;
    tmq_oracle_consts(digamma, &d32, &h32, &c32);
    float s32 = (float)scale;
    for (size_t i = 0; i < n; i++) {
        float fw = floorf(w[i]);
        float frac = w[i] - fw;
        float arg = d32 * frac - h32;
        float grad = (d32 * dsig32(arg)) / c32;
        dw[i] = (s32 * g[i]) * grad;
    }
}

/* SoftStepDerivative.forward CPU branch, tmq/tmq.py:469-473:
 *   out = ((strength*digamma) * dsigmoid(arg)) / (2*sig(d/2)); the product strength*digamma
 *   is a Python double rounded to fp32 once.                                                */
void tmq_oracle_deriv_fwd(const float *w, float *q, size_t n, double digamma, double strength) {
    float d32, h32, c32;
    tmq_oracle_consts(digamma, &d32, &h32, &c32);
    float k1 = (float)(strength * digamma);
    for (size_t i = 0; i < n; i++) {
        float fw = floorf(w[i]);
        float frac = w[i] - fw;
        float arg = d32 * frac - h32;
        q[i] = (k1 * dsig32(arg)) / c32;
    }
}

/* SoftStepDerivative.backward CPU branch, tmq/tmq.py:488-493:
 *   grad = ((strength*digamma*digamma) * d2sigmoid(arg)) / (2*sig(d/2)); out = g*grad       */
void tmq_oracle_deriv_bwd(const float *w, const float *g, float *dw, size_t n, double digamma,
                          double strength) {
    float d32, h32, c32;
    tmq_oracle_consts(digamma, &d32, &h32, &c32);
    float k2 = (float)(strength * digamma * digamma);
    for (size_t i = 0; i < n; i++) {
        float fw = floorf(w[i]);
        float frac = w[i] - fw;
        float arg = d32 * frac - h32;
        float grad = (k2 * d2sig32(arg)) / c32;
        dw[i] = g[i] * grad;
    }
}

/* SoftStep.map, tmq/tmq.py:335-337 -- note the different association of the argument:
 *   arg = d*w - d*fw - d/2                                                                  */
void tmq_oracle_map(const float *w, float *y, size_t n, double digamma) {
    float d32, h32, c32;
    tmq_oracle_consts(digamma, &d32, &h32, &c32);
    for (size_t i = 0; i < n; i++) {
        float fw = floorf(w[i]);
        float arg = (d32 * w[i] - d32 * fw) - h32;
        float s = sig32(arg) / c32;
        y[i] = (s + 0.5f) + fw;
    }
}

/* SoftStep.dmap, tmq/tmq.py:348-350: arg = w*d - d*fw - d/2; (d*dsigmoid(arg))/c            */
void tmq_oracle_dmap(const float *w, float *y, size_t n, double digamma) {
    float d32, h32, c32;
    tmq_oracle_consts(digamma, &d32, &h32, &c32);
    for (size_t i = 0; i < n; i++) {
        float fw = floorf(w[i]);
        float arg = (w[i] * d32 - d32 * fw) - h32;
        y[i] = (d32 * dsig32(arg)) / c32;
    }
}

/* QuantizationControl.quantize, tmq/tmq.py:293-295: round_half_even(SoftStep.map(w)).
 * torch.round is round-half-to-even == rintf in the default rounding mode.                  */
void tmq_oracle_ternarize(const float *w, float *out, size_t n, double digamma) {
    tmq_oracle_map(w, out, n, digamma);
    for (size_t i = 0; i < n; i++) out[i] = rintf(out[i]);
}

/* Linear.quantize / Conv2d.quantize / quantize_weights: plain torch.round,
 * tmq/tmq.py:603, 886, 1109.                                                                */
void tmq_oracle_round(const float *w, float *out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = rintf(w[i]);
}

/* Linear.clamp / Conv2d.clamp, tmq/tmq.py:696, 879 with limits from
 * QuantizationControl.clamp, tmq/tmq.py:270 (Python doubles rounded to fp32 by torch).      */
void tmq_oracle_clamp(const float *w, float *out, size_t n, double lo, double hi) {
    float lo32 = (float)lo, hi32 = (float)hi;
    for (size_t i = 0; i < n; i++) out[i] = clampf(w[i], lo32, hi32);
}

/* One fused training pass over a flat tensor: everything the reference does to a weight
 * tensor in one QAT step, in the reference's own per-element op order:
 *   y      = SoftStep.forward(w; digamma)                          tmq/tmq.py:417-419
 *   q      = SoftStepDerivative.forward(w; sharpness, strength)    tmq/tmq.py:469-473
 *   dw     = (scale*g)*S'(w) + gl*Q'(w)    (autograd sums the two) tmq/tmq.py:434-438, 488-493
 *   wc     = clamp(w, lo, hi)                                      tmq/tmq.py:696
 * qsum receives sum(q) in fp64 (the caller divides by n for the mean of tmq/tmq.py:699).    */
void tmq_oracle_fused(const float *w, const float *g, float *y, float *dw, float *wc, double *qsum,
                      size_t n, double digamma, double sharpness, double strength, float gl,
                      double lo, double hi) {
    float d32, h32, c32, e32, f32, c5;
    tmq_oracle_consts(digamma, &d32, &h32, &c32);
    tmq_oracle_consts(sharpness, &e32, &f32, &c5);
    float k1 = (float)(strength * sharpness);
    float k2 = (float)(strength * sharpness * sharpness);
    float lo32 = (float)lo, hi32 = (float)hi;
    double acc = 0.0;
    for (size_t i = 0; i < n; i++) {
        float fw = floorf(w[i]);
        float frac = w[i] - fw;
        float arg = d32 * frac - h32;
        float s = sig32(arg) / c32;
        y[i] = (s + 0.5f) + fw;
        float grad = (d32 * dsig32(arg)) / c32;
        float t1 = (1.0f * g[i]) * grad;
        float arg5 = e32 * frac - f32;
        float q = (k1 * dsig32(arg5)) / c5;
        acc += (double)q;
        float gq = (k2 * d2sig32(arg5)) / c5;
        float t2 = gl * gq;
        dw[i] = t1 + t2;
        wc[i] = clampf(w[i], lo32, hi32);
    }
    *qsum = acc;
}

/* fp64 sum of an fp32 vector (used to check the loss reduction). */
double tmq_oracle_sum64(const float *x, size_t n) {
    double acc = 0.0;
    for (size_t i = 0; i < n; i++) acc += (double)x[i];
    return acc;
}

/* ------------------------------------------------------------------------------------------
 * 2-bit ternary packing.
 *   value -> code      tmq/tmq_native.cpp:161-165 / 198-202: roundf (half away from zero) for
 *                      fp32, plain cast for integer input, clamp to [-1,1], 0->00 +1->01 -1->10
 *   word               16 codes, first element in bits 31:30 (tmq/tmq_native.cpp:166, 203)
 *   matrix [N][K]      -> words [K][ceil(N/16)]; word (k,q) holds W[16q+j][k], j = 0..15
 *                      (transpose at tmq/tmq_native.cpp:311-314, loop 152-171)
 *   conv [N][C][ky][kx]-> words [C*ky*kx][ceil(N/16)] (tmq/tmq_native.cpp:185-208); the row is
 *                      the flat index inside one output channel, so it is the matrix case with
 *                      K = C*ky*kx.
 * The float->int cast of the reference is the x86 cvttss2si: NaN and |v| >= 2^31 give INT_MIN,
 * which the clamp turns into -1. This restatement spells that out instead of relying on UB.
 * ---------------------------------------------------------------------------------------- */
static inline int code_from_int(long long nv) {
    int n = nv > 1 ? 1 : (nv < -1 ? -1 : (int)nv);
    return n == 0 ? 0 : (n == 1 ? 1 : 2);
}

static inline int code_from_f32(float v) {
    float r = roundf(v);
    long long nv;
    if (!(r > -2147483904.0f && r < 2147483648.0f)) nv = -2147483648LL; /* cvttss2si "indefinite" */
    else nv = (long long)r;
    return code_from_int(nv);
}

/* dtype: 0 = fp32, 1 = int32, 2 = int8 */
void tmq_oracle_pack(const void *w, int dtype, int64_t N, int64_t K, uint32_t *out) {
    int64_t Q = (N + 15) / 16;
    for (int64_t k = 0; k < K; k++) {
        for (int64_t q = 0; q < Q; q++) {
            uint32_t word = 0;
            for (int j = 0; j < 16; j++) {
                int64_t n = q * 16 + j;
                int code = 0;
                if (n < N) {
                    if (dtype == 0) code = code_from_f32(((const float *)w)[n * K + k]);
                    else if (dtype == 1) code = code_from_int(((const int32_t *)w)[n * K + k]);
                    else code = code_from_int(((const int8_t *)w)[n * K + k]);
                }
                word = (word << 2) | (uint32_t)code;
            }
            out[k * Q + q] = word;
        }
    }
}

/* code -> value, 11 decodes to 0 (tmq/tmq_cuda.cu:453-467). The host expander maps 11 to -1
 * (tmq/tmq_native.cpp:228, 260) but 11 is never produced by the packer; `strict` selects the
 * host behaviour so both can be tested.                                                      */
static inline float value_from_code(int c, int host_rule) {
    if (c == 0) return 0.0f;
    if (c == 1) return 1.0f;
    if (c == 2) return -1.0f;
    return host_rule ? -1.0f : 0.0f;
}

/* True inverse of tmq_oracle_pack: words [K][ceil(N/16)] -> fp32 [N][K]
 * (the conv expander tmq/tmq_native.cpp:249-266 is this with K = C*ky*kx).                   */
void tmq_oracle_unpack(const uint32_t *in, int64_t N, int64_t K, float *out, int host_rule) {
    int64_t Q = (N + 15) / 16;
    for (int64_t k = 0; k < K; k++)
        for (int64_t q = 0; q < Q; q++) {
            uint32_t word = in[k * Q + q];
            for (int j = 0; j < 16; j++) {
                int64_t n = q * 16 + j;
                if (n < N) out[n * K + k] = value_from_code((int)((word >> (2 * (15 - j))) & 3u), host_rule);
            }
        }
}

/* The reference's 2-D expander as written (tmq/tmq_native.cpp:220-234, called at 520-523 with
 * rows = origShape[0], columns = origShape[1]): it reads the words as [rows][ceil(columns/16)],
 * which is NOT the layout the packer wrote unless rows == columns, and it reads past the end of
 * the packed buffer whenever rows*ceil(columns/16) exceeds the number of words. Kept only to
 * document the defect; `nwords` bounds the reads (returns -1 if the reference would read out of
 * bounds). The product implements tmq_oracle_unpack.                                          */
int tmq_oracle_unpack_ref2d_as_written(const uint32_t *in, int64_t nwords, int64_t rows, int64_t cols, float *out) {
    int64_t Q = (cols + 15) / 16;
    if (rows * Q > nwords) return -1;
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < Q; c++) {
            uint32_t word = in[r * Q + c];
            for (int j = 0; j < 16; j++)
                if (c * 16 + j < cols)
                    out[r * cols + c * 16 + j] = value_from_code((int)((word >> (2 * (15 - j))) & 3u), 1);
        }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Ternary linear / convolution: textbook contraction on expanded weights, fp64 accumulation.
 *   y[m][n] = scale[n] * sum_k x[m][k] * T[k][n] + bias[n]
 * GEMV tmq/tmq_cuda.cu:242-286, GEMM tmq/tmq_cuda.cu:289-427 (both: out = sum_k lhs*T),
 * post-scale and bias tmq/tmq.py:684-687, 865-871. x is given as fp32 (callers convert fp16
 * inputs exactly). scale / bias may be NULL.
 * ---------------------------------------------------------------------------------------- */
void tmq_oracle_gemm(const float *x, int64_t M, int64_t K, const uint32_t *wp, int64_t N,
                     const float *scale, const float *bias, double *y) {
    int64_t Q = (N + 15) / 16;
    float *t = (float *)malloc((size_t)K * (size_t)N * sizeof(float)); /* T[k][n] */
    for (int64_t k = 0; k < K; k++)
        for (int64_t n = 0; n < N; n++) {
            uint32_t word = wp[k * Q + n / 16];
            t[k * N + n] = value_from_code((int)((word >> (2 * (15 - (n % 16)))) & 3u), 0);
        }
    for (int64_t m = 0; m < M; m++) {
        double *row = y + m * N;
        for (int64_t n = 0; n < N; n++) row[n] = 0.0;
        for (int64_t k = 0; k < K; k++) {
            double xv = (double)x[m * K + k];
            if (xv == 0.0) continue;
            const float *tk = t + k * N;
            for (int64_t n = 0; n < N; n++) row[n] += xv * (double)tk[n];
        }
        for (int64_t n = 0; n < N; n++) {
            double v = row[n];
            if (scale) v *= (double)scale[n];
            if (bias) v += (double)bias[n];
            row[n] = v;
        }
    }
    free(t);
}

/* Depthwise convolution on unfolded patches, the arithmetic of ternaryDWConvFP32
 * (tmq/tmq_cuda.cu:166-238): x [P][T][C], weights packed as words[t][ceil(C/16)] (the layout
 * compactTernaryConvKernel, tmq/tmq_native.cpp:279-294, gives a [C][1][ky][kx] tensor), y [P][C]:
 * y[p][c] = sum_t x[p][t][c] * T[c][t]. fp64 accumulation.                                      */
void tmq_oracle_dwconv_patches(const float *x, int64_t P, int64_t T, int64_t C, const uint32_t *wp, double *y) {
    int64_t Q = (C + 15) / 16;
    for (int64_t p = 0; p < P; p++)
        for (int64_t c = 0; c < C; c++) {
            double acc = 0.0;
            for (int64_t t = 0; t < T; t++) {
                uint32_t word = wp[t * Q + c / 16];
                float w = value_from_code((int)((word >> (2 * (15 - (c % 16)))) & 3u), 0);
                acc += (double)x[(p * T + t) * C + c] * (double)w;
            }
            y[p * C + c] = acc;
        }
}

/* Transposed depthwise convolution in column form, the arithmetic of ternaryDWConvTransFP32
 * (tmq/tmq_cuda.cu:118-162): x [B][P][C], words[t][ceil(C/16)], y [B][C*T][P] with
 * y[b][c*T + t][p] = x[b][p][c] * T[c][t] as an fp32 product (a zero weight gives a zero that keeps
 * the sign of x, like the reference's multiply by 0.f). The reference's launch has no batch index
 * (host, 645-686) and so fills batch entry 0 only; here every entry follows the same formula.   */
void tmq_oracle_dwconvtrans_cols(const float *x, int64_t B, int64_t P, int64_t T, int64_t C, const uint32_t *wp, float *y) {
    int64_t Q = (C + 15) / 16;
    for (int64_t b = 0; b < B; b++)
        for (int64_t c = 0; c < C; c++)
            for (int64_t t = 0; t < T; t++) {
                uint32_t word = wp[t * Q + c / 16];
                float w = value_from_code((int)((word >> (2 * (15 - (c % 16)))) & 3u), 0);
                for (int64_t p = 0; p < P; p++) y[(b * C * T + c * T + t) * P + p] = x[(b * P + p) * C + c] * w;
            }
}

/* Direct convolution, NCHW input, weights packed as [C*ky*kx][ceil(N/16)] with row
 * (c*ky + y)*kx + x -- the ordering of F.unfold used at tmq/tmq.py:857-859. Output NCHW fp64.
 * Output size is PyTorch's floor((h + 2p - d(k-1) - 1)/s) + 1.                               */
void tmq_oracle_conv2d(const float *x, int64_t B, int64_t C, int64_t H, int64_t W, const uint32_t *wp,
                       int64_t N, int64_t ky, int64_t kx, int64_t sy, int64_t sx, int64_t py,
                       int64_t px, int64_t dy, int64_t dx, const float *scale, const float *bias,
                       double *y) {
    int64_t Q = (N + 15) / 16;
    int64_t Ho = (H + 2 * py - dy * (ky - 1) - 1) / sy + 1;
    int64_t Wo = (W + 2 * px - dx * (kx - 1) - 1) / sx + 1;
    for (int64_t b = 0; b < B; b++)
        for (int64_t n = 0; n < N; n++)
            for (int64_t oh = 0; oh < Ho; oh++)
                for (int64_t ow = 0; ow < Wo; ow++) {
                    double acc = 0.0;
                    for (int64_t c = 0; c < C; c++)
                        for (int64_t i = 0; i < ky; i++)
                            for (int64_t j = 0; j < kx; j++) {
                                int64_t ih = oh * sy - py + i * dy, iw = ow * sx - px + j * dx;
                                if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                                int64_t row = (c * ky + i) * kx + j;
                                uint32_t word = wp[row * Q + n / 16];
                                float t = value_from_code((int)((word >> (2 * (15 - (n % 16)))) & 3u), 0);
                                acc += (double)x[((b * C + c) * H + ih) * W + iw] * (double)t;
                            }
                    if (scale) acc *= (double)scale[n];
                    if (bias) acc += (double)bias[n];
                    y[((b * N + n) * Ho + oh) * Wo + ow] = acc;
                }
}
