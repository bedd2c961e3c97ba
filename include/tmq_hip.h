/*
 * libtmq_hip -- C ABI of the MI355X (gfx950) implementation of TMQ's GPU hot path.
 *
 * Conventions
 *   - Every entry point returns TMQ_OK (0) or a negative tmq_status; nothing throws.
 *   - Pointers are raw device pointers unless a parameter is documented as host memory.
 *     Tensors are dense and contiguous; `n` counts elements.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream). Work is enqueued
 *     asynchronously; no entry point synchronises, allocates or frees device memory. Workspaces
 *     are passed in by the caller and sized with the *_workspace_bytes helpers.
 *   - Hardness / strength scalars cross the boundary as C doubles, exactly as the Python
 *     caller holds them; the library rounds them to fp32 once, the way torch does when a Python
 *     scalar meets an fp32 tensor, so results are bit-identical to the reference's CPU chain
 *     of separately rounded fp32 operations.
 *   - Thread safe; no hidden mutable global state, with one documented exception: the static
 *     scratch array of tmq_softstep_fused_noalloc.
 *
 * Each declaration cites the reference interface it replaces (paths relative to the reference
 * repository root).
 */
#ifndef TMQ_HIP_H
#define TMQ_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum tmq_status {
    TMQ_OK = 0,
    TMQ_ERR_INVALID_ARG = -1, /* null pointer, negative size, misaligned or inconsistent shape */
    TMQ_ERR_UNSUPPORTED = -2, /* dtype / shape combination this build does not implement */
    TMQ_ERR_LAUNCH = -3,      /* HIP reported an error; see tmq_last_hip_error() */
    TMQ_ERR_TOO_LARGE = -4,   /* size exceeds what the launch geometry can index */
    TMQ_ERR_BAD_DATA = -5     /* host codec: malformed stream or illegal symbol */
} tmq_status;

/* Library version (major*10000 + minor*100 + patch) and a static description of a status. */
int tmq_version(void);
const char *tmq_status_string(int status);
/* hipError_t of the last failing HIP call made by this library on the calling thread. */
int tmq_last_hip_error(void);

/* Element dtypes understood by the packer. */
enum { TMQ_F32 = 0, TMQ_I32 = 1, TMQ_I8 = 2, TMQ_F16 = 3 };

/* ------------------------------------------------------------------------------------------
 * Soft-staircase transfer function (fp32).
 * ---------------------------------------------------------------------------------------- */

/* y = S(w; digamma).
 * Replaces fwd_softstep / forwardSoftStepCUDA (tmq/tmq_cuda.cu:740-764, kernel 80-92) with the
 * arithmetic of SoftStep.forward's CPU branch (tmq/tmq.py:417-419).                          */
int tmq_softstep_fwd(const float *w, float *y, size_t n, double digamma, void *stream);

/* dw = (scale*g) * S'(w; digamma).
 * Replaces bwd_softstep / backwardSoftStepCUDA (tmq/tmq_cuda.cu:768-794, kernel 95-110);
 * arithmetic of tmq/tmq.py:434-438.                                                          */
int tmq_softstep_bwd(const float *w, const float *g, float *dw, size_t n, double digamma,
                     double scale, void *stream);

/* q = strength*digamma*dsig(arg)/(2 sig(digamma/2)) -- the quantization-loss integrand.
 * Replaces fwd_softstep_derivative (tmq/tmq_cuda.cu:690-709, kernel 45-59); arithmetic of
 * tmq/tmq.py:469-473.                                                                        */
int tmq_softstep_deriv_fwd(const float *w, float *q, size_t n, double digamma, double strength,
                           void *stream);

/* dw = g * strength*digamma^2*d2sig(arg)/(2 sig(digamma/2)).
 * Replaces bwd_softstep_derivative (tmq/tmq_cuda.cu:713-735, kernel 62-77); arithmetic of
 * tmq/tmq.py:488-493.                                                                        */
int tmq_softstep_deriv_bwd(const float *w, const float *g, float *dw, size_t n, double digamma,
                           double strength, void *stream);

/* y = SoftStep.map(w) (derivative == 0) or SoftStep.dmap(w) (derivative != 0): the staircase /
 * its slope with the argument association of tmq/tmq.py:335-338 / 348-350 (used for logging and
 * for the final ternarisation).                                                              */
int tmq_softstep_map(const float *w, float *y, size_t n, double digamma, int derivative, void *stream);

/* y = sigmoid / dsigmoid / d2sigmoid (order 0 / 1 / 2) of an arbitrary fp32 tensor: the rational
 * pieces SoftStep.sigmoid, dsigmoid, d2sigmoid (tmq/tmq.py:353-381).                          */
int tmq_sigmoid_piece(const float *x, float *y, size_t n, int order, void *stream);

/* w <- clamp(w, lo, hi) in place (NaN stays NaN).
 * Replaces the torch.clamp pass of Linear.clamp / Conv2d.clamp (tmq/tmq.py:691-696, 874-879)
 * driven by QuantizationControl.clamp (tmq/tmq.py:263-272).                                  */
int tmq_clamp_inplace(float *w, size_t n, double lo, double hi, void *stream);

/* w <- round_half_even(map(w; digamma)) in place, map with the association of
 * SoftStep.map (tmq/tmq.py:335-338). Replaces the body of QuantizationControl.quantize
 * (tmq/tmq.py:284-295). With digamma <= 0 it is plain round_half_even(w), i.e.
 * Linear.quantize / Conv2d.quantize / quantize_weights (tmq/tmq.py:603, 886, 1109).          */
int tmq_ternarize_inplace(float *w, size_t n, double digamma, void *stream);

/* One fused pass over a flat tensor: everything the reference does to a weight tensor in a
 * QAT step -- y = S(w; digamma); loss integrand q(w; sharpness, strength) reduced to a sum;
 * dw = g*S'(w; digamma) + gl*Q'(w; sharpness, strength); wc = clamp(w, lo, hi).
 * Fuses tmq/tmq.py:417-419, 434-438, 469-473 (+ the mean of 699), 488-493 and 696 -- seven
 * separate passes in the reference (tmq/tmq_cuda.cu:45-110 + torch mean/add/clamp).
 * Any of y, dw, wc may be NULL (that output is skipped; g may be NULL iff dw is NULL); wc may
 * alias w. loss_sum (device, 1 double) receives sum_i q_i; it may be NULL. workspace must hold
 * tmq_softstep_fused_workspace_bytes(n) bytes when loss_sum is non-NULL.                      */
size_t tmq_softstep_fused_workspace_bytes(size_t n);
int tmq_softstep_fused(const float *w, const float *g, float *y, float *dw, float *wc,
                       double *loss_sum, void *workspace, size_t n, double digamma,
                       double sharpness, double strength, float gl, double lo, double hi,
                       void *stream);

/* tmq_softstep_fused without a workspace argument and without any device allocation. It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving / training loops, harnesses that forbid hipMalloc. The block partial
 * sums of the loss reduction go to a 1 MiB array that is part of the library's device image (each
 * GPU the library runs on holds its own copy until the process ends); its address is looked up once
 * per device on the first call there. n may be at most tmq_softstep_fused_noalloc_max_elements()
 * (2^29), larger tensors return TMQ_ERR_TOO_LARGE. Results are bit-identical to tmq_softstep_fused.
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different
 * streams or threads) race on it and must be serialised by the caller; calls on one stream are
 * ordered. Nothing in the array needs clearing between calls.                                   */
size_t tmq_softstep_fused_noalloc_max_elements(void);
int tmq_softstep_fused_noalloc(const float *w, const float *g, float *y, float *dw, float *wc,
                               double *loss_sum, size_t n, double digamma, double sharpness,
                               double strength, float gl, double lo, double hi, void *stream);

/* ------------------------------------------------------------------------------------------
 * Multi-tensor (one launch for every registered layer) forms of the per-layer Python loops of
 * QuantizationControl.quantization_loss / clamp (tmq/tmq.py:298-310, 263-272).
 *
 * A segment table describes the tensors. The caller fills ptr/aux/n (+ scalar where stated),
 * calls tmq_multi_plan() on the host copy to assign block ranges, and uploads the table.
 * ---------------------------------------------------------------------------------------- */
typedef struct tmq_segment {
    void *ptr;            /* weight tensor (fp32) */
    void *aux;            /* second tensor of the same size where the op needs one, else NULL */
    uint64_t n;           /* elements */
    uint32_t block_begin; /* filled by tmq_multi_plan */
    float scalar;         /* per-tensor scalar where the op needs one */
} tmq_segment;

/* Host helper: fills block_begin for nseg segments, returns the launch's block count in
 * *total_blocks. Empty tensors are legal.                                                    */
int tmq_multi_plan(tmq_segment *segs_host, int nseg, uint32_t *total_blocks);

/* Workspace (bytes) for tmq_qloss_multi with that plan. */
size_t tmq_qloss_multi_workspace_bytes(uint32_t total_blocks);

/* per_tensor[l] = mean_i q(w_l[i]; sharpness, strength); *total = fp32 sum over l in table
 * order (the reference's Python loop of scalar adds, tmq/tmq.py:305-310). Either output may be
 * NULL. Two launches: block partial sums, then an ordered fp64 finalisation (deterministic). */
int tmq_qloss_multi(const tmq_segment *segs_dev, int nseg, uint32_t total_blocks, double sharpness,
                    double strength, float *per_tensor, float *total, void *workspace,
                    void *stream);

/* aux_l[i] (= or +=) s_l * Q'(w_l[i]; sharpness, strength): the gradient of the loss above w.r.t.
 * every weight. With upstream (device, 1 float: the gradient arriving at the total loss)
 * s_l = upstream / float(n_l), the value autograd's mean backward produces; with upstream NULL
 * s_l is the table's scalar_l. accumulate != 0 adds into aux (fused grad accumulation), else
 * overwrites. Arithmetic of tmq/tmq.py:488-493.                                              */
int tmq_qloss_bwd_multi(const tmq_segment *segs_dev, int nseg, uint32_t total_blocks,
                        double sharpness, double strength, const float *upstream, int accumulate,
                        void *stream);

/* The same for the tensors of a training step, whose outputs and gradients sit at new addresses in
 * every step: the table is a HOST array that the library copies into the kernels' arguments, so
 * nothing is uploaded or cached (up to 64 tensors per launch, more are split over several).
 * Replaces the per-layer launches of SoftStep.forward / backward (tmq/tmq.py:404-438, called from
 * Linear.forward_wrap 650 and Conv2d.forward 812 for every layer) together with the quantization loss
 * (298-310, 456-493) and autograd's accumulation of the two gradient terms.                       */
typedef struct tmq_step_tensor {
    const float *w; /* weights (device, fp32) */
    const float *g; /* backward only: dL/dy of this tensor (device), NULL if none arrived */
    float *out;     /* forward: y = S(w); backward: dw */
    uint64_t n;     /* elements */
} tmq_step_tensor;

/* Workspace (bytes) of tmq_softstep_fwd_multi when a loss output is requested. */
size_t tmq_softstep_multi_workspace_bytes(const tmq_step_tensor *tensors_host, int ntensors);

/* out_l = S(w_l; digamma) for every tensor; with loss_per_tensor / loss_total non-NULL also
 * loss_per_tensor[l] = mean_i q(w_l[i]; sharpness, strength) and *loss_total = their fp32 sum in
 * table order (as tmq_qloss_multi), from the same pass over the weights.                         */
int tmq_softstep_fwd_multi(const tmq_step_tensor *tensors_host, int ntensors, double digamma,
                           double sharpness, double strength, float *loss_per_tensor,
                           float *loss_total, void *workspace, void *stream);

/* out_l = g_l * S'(w_l; digamma) + (u / float(n_l)) * Q'(w_l; sharpness, strength): the weight
 * gradient of a whole step, u = *loss_upstream (device, 1 float: the gradient arriving at the total
 * quantization loss; NULL = the loss took no part, the second term is dropped). A tensor with g NULL
 * gets the second term alone. Each term is rounded as the reference's backward functions round it
 * (tmq/tmq.py:434-438, 488-493) and the two are added once, as autograd's accumulation would.    */
int tmq_softstep_bwd_multi(const tmq_step_tensor *tensors_host, int ntensors, double digamma,
                           double sharpness, double strength, const float *loss_upstream,
                           void *stream);

/* The loss reductions above finished inside the launch that computes them: no finalisation launch, no
 * workspace. Every block adds its partial sum to a 64-bit cell as a fixed-point integer (integer addition is
 * associative, so the result does not depend on the order in which blocks arrive; the unit, 2^-28 .. 2^-10, is
 * chosen per tensor from its size) with one returning device-scope atomic that also counts the block; a large
 * tensor's blocks are spread over 64 cells; the block that completes a cell passes its total on (cell ->
 * tensor -> launch), and the block that completes the launch writes the total; every cell is zero again by
 * then. Deterministic and within 1e-6 relative of the fp64 finalisation of the two-launch forms; NaN / Inf
 * weights give NaN as there. *total is the sum of the per-tensor means accumulated as integers (the two-launch
 * form adds them in fp32 in table order; the two agree to fp32 rounding).
 *   state: tmq_loss_state_bytes() bytes of device memory, 8-byte aligned, ZERO before the first call that uses
 *   it; every call leaves it zero, so one memset at allocation serves all later calls (and HIP-graph replays).
 *   Calls that share a state must not overlap in time (one state per stream).
 * TMQ_ERR_UNSUPPORTED (use the two-launch form): more than 64 tensors, a tensor beyond 2^18 blocks of 2048
 * elements (tmq_qloss_multi_inlaunch: a launch beyond 2^18 blocks), nothing to sum.
 * tmq_softstep_fused_inlaunch: tmq_softstep_fused with loss_sum required (tmq/tmq.py:417-419, 434-438,
 * 469-473 + 699, 488-493, 696). tmq_qloss_multi_inlaunch: tmq_qloss_multi (tmq/tmq.py:298-310).
 * tmq_softstep_fwd_multi_inlaunch: tmq_softstep_fwd_multi with a loss output (tmq/tmq.py:404-419 for every
 * layer + 298-310).                                                                                      */
size_t tmq_loss_state_bytes(void);
int tmq_softstep_fused_inlaunch(const float *w, const float *g, float *y, float *dw, float *wc,
                                double *loss_sum, void *state, size_t n, double digamma,
                                double sharpness, double strength, float gl, double lo, double hi,
                                void *stream);
int tmq_qloss_multi_inlaunch(const tmq_segment *segs_dev, int nseg, uint32_t total_blocks,
                             double sharpness, double strength, float *per_tensor, float *total,
                             void *state, void *stream);
int tmq_softstep_fwd_multi_inlaunch(const tmq_step_tensor *tensors_host, int ntensors,
                                    double digamma, double sharpness, double strength,
                                    float *loss_per_tensor, float *loss_total, void *state,
                                    void *stream);


/* w_l <- clamp(w_l, lo, hi) for every segment, one launch. */
int tmq_clamp_multi(const tmq_segment *segs_dev, int nseg, uint32_t total_blocks, double lo,
                    double hi, void *stream);

/* ------------------------------------------------------------------------------------------
 * 2-bit ternary packing (16 codes per 32-bit word, first element in bits 31:30; 0->00, +1->01,
 * -1->10; ragged tails zero-filled).
 * ---------------------------------------------------------------------------------------- */

/* W[N][K] (row-major, dtype TMQ_F32 / TMQ_I32 / TMQ_I8) -> words[K][ceil(N/16)]; word (k,q)
 * holds W[16q+j][k], j = 0..15. fp32 values are rounded half away from zero, integers cast,
 * then clamped to [-1,1].
 * Replaces compactify_ternary (tmq/tmq_native.cpp:418-425): a Linear weight [out][in] is the
 * case N=out, K=in (matrixTo2BitTernary 152-171 after the transpose at 311-314); a Conv2d
 * weight [out][in][ky][kx] is N=out, K=in*ky*kx (kernelTo2BitTernary 185-208).                */
int tmq_pack_ternary(const void *w, int dtype, int64_t N, int64_t K, uint32_t *words, void *stream);

/* words[K][ceil(N/16)] -> fp32 W[N][K] in {-1,0,+1} (code 11 -> 0, as tmq/tmq_cuda.cu:464-466).
 * Replaces expand_ternary (tmq/tmq_native.cpp:516-544; compactKernelTo32BitFloat 249-266).
 * This is the true inverse of tmq_pack_ternary also for 2-D tensors.                         */
int tmq_unpack_ternary(const uint32_t *words, int64_t N, int64_t K, float *w, void *stream);

/* ------------------------------------------------------------------------------------------
 * Ternary inference: y[m][n] = scale[n] * sum_k x[m][k] * T[k][n] + bias[n], fp32 accumulation.
 *
 * The kernels read a kernel-native re-tiling of the packed weights (still 2 bits per weight:
 * blocks of 16 channels x 256 reduction indices laid out in MFMA operand order). It is produced
 * once per layer from the reference-format words by tmq_prepack_weights and cached by the
 * caller; the reference-format tensor itself is never modified.
 * ---------------------------------------------------------------------------------------- */

/* Bytes of the native buffer for N output channels and reduction length K. */
size_t tmq_native_weight_bytes(int64_t N, int64_t K);

/* words[K][ceil(N/16)], K = C*ky*kx with row (c*ky + i)*kx + j (the format written by
 * tmq_pack_ternary / compactify_ternary, tmq/tmq_native.cpp:152-208) -> native (16-byte aligned).
 * Linear layers pass C = K, ky = kx = 1. For ky*kx > 1 the reduction index is reordered to
 * (i, j, c) so that im2col rows are contiguous in NHWC activations. Code 11 becomes 0, as in the
 * reference's device LUT (tmq/tmq_cuda.cu:464-466).                                           */
int tmq_prepack_weights(const uint32_t *words, int64_t N, int64_t C, int64_t ky, int64_t kx,
                        void *native, void *stream);

/* Fused epilogue of the inference kernels: y = relu?( scale[n]*acc + bias[n] + residual ).
 * scale / bias: optional fp32 [N] (NULL = 1 / 0) -- the per-channel generalisation of the
 * reference's scalar post_scale and bias (tmq/tmq.py:684-687, 865-871), which is also where an
 * eval-mode BatchNorm folds. residual: optional tensor of y's shape and dtype. y_dtype: TMQ_F32 or
 * TMQ_F16. A NULL epilogue pointer means plain fp32 output.                                   */
typedef struct tmq_epilogue {
    const float *scale;
    const float *bias;
    const void *residual;
    int32_t relu;
    int32_t y_dtype;
} tmq_epilogue;

/* x [M][K] row-major, x_dtype TMQ_F16 or TMQ_F32; y [M][N].
 * fp32 activations are carried as two fp16 terms (22 significant bits), so they must lie inside fp16's
 * exponent range: max|x| at most 65504, and values below ~6e-5 lose precision. Tensors of any other
 * magnitude go through tmq_f32_prescale first (exact power-of-two scaling, undone in the per-channel scale of
 * the epilogue); the Python / PyTorch bindings of this library always do, because the reference multiplies
 * fp32 activations in fp32 and has no such limit. One case needs no prescale: fp32 rows for which
 * tmq_fp32_rows_self_scaled_for returns 1 (one row, or two over a small layer) are scaled inside the kernel, each by
 * its own power of two, and may have any magnitude.
 * Arithmetic: exact products, fp32 accumulation. One fp16 row (M == 1) with K a multiple of 256 from 2048 to 16384
 * runs on the 8-bit matrix instructions (weights as fp8, the row as four exact bf8 terms); there the hardware adds
 * 32 products at a time aligned to the largest of them, so the result can differ from an fp32 running sum by a few
 * 1e-6 of the largest output (about 1e-4 when values near 65504 sit next to values of order one) -- inside the
 * 1e-3 tolerance of this path, and exact whenever all partial sums are integers below 2^24.
 * Replaces ternary_mvm_cuda (tmq/tmq_cuda.cu:563-603, kernel 242-286) for M == 1 and
 * ternary_mmm_cuda (tmq/tmq_cuda.cu:478-549, kernel 289-427) for M > 1, plus the post-scale /
 * bias passes of Linear.compact_forward (tmq/tmq.py:684-687). Any M, K, N (ragged tails masked). */
int tmq_ternary_linear(const void *x, int x_dtype, int64_t M, int64_t K, const void *native,
                       int64_t N, const tmq_epilogue *epilogue, void *y, void *stream);

/* tmq_ternary_linear for callers that bring a workspace (the reference's hosts allocate what they need
 * themselves, tmq/tmq_cuda.cu:478-549; this ABI never allocates): a product whose reduction pays to be cut across
 * workgroups -- today 17 .. 32 fp16 rows over 2^28 weights or more -- runs as slices of whole 256-index weight
 * blocks with fp32 partial sums in the workspace, added in slice order by a second launch (deterministic, no
 * atomics). fp32 rows (the reference's kernels take fp32 activations, tmq/tmq_cuda.cu:242-427) use the workspace
 * differently, unless tmq_ternary_linear scales them itself in one launch (tmq_fp32_rows_self_scaled_for). Up to
 * sixteen rows: a first launch splits every row into two fp16 rows (hi = fp16(s x), lo = fp16(s x - hi), s the row's
 * own power of two: any magnitude, 22 significant bits), the fp16 weight-stream kernel then runs once over twice the
 * rows (from nine rows: twice, over about half of them each) and adds each pair in its epilogue (256 + 4 M K" bytes,
 * K" = K rounded up to a multiple of 256: the pairs of a ragged length are written with zeros behind). Seventeen
 * rows or more are split in groups of eight rows, each group under a power of two of its own, laid out so that a
 * row's two terms share a 16-row MFMA fragment; the fp16 GEMM kernels then run once over 16 ceil(M / 8) rows and add
 * the pairs where they write the tile (ceil(M / 8) floats rounded up to 256 bytes + 32 ceil(M / 8) K' bytes, K' = K
 * rounded up to a multiple of 64, zeros behind the K-th value again).
 * Seventeen fp16 rows or more whose K is no multiple of 64 are copied once to rows of the next multiple of 64, zeros
 * behind (2 M ceil(K / 64) 64 bytes), and take the kernels that want whole 64-index tiles of 16-byte aligned rows
 * instead of the one that guards every load (K = 4000, M = 1024, N = 4096: 261 -> 39 us).
 * tmq_ternary_linear_workspace_bytes returns what a shape can use (0: the single-launch kernels are at
 * least as fast); with a NULL or smaller workspace tmq_ternary_linear_ws is tmq_ternary_linear. Same results to
 * fp32 rounding (the summation order differs). The workspace must be 16-byte aligned.                     */
size_t tmq_ternary_linear_workspace_bytes(int x_dtype, int64_t M, int64_t K, int64_t N);
int tmq_ternary_linear_ws(const void *x, int x_dtype, int64_t M, int64_t K, const void *native, int64_t N,
                          const tmq_epilogue *epilogue, void *y, void *workspace, size_t workspace_bytes,
                          void *stream);

/* One to four fp16 rows with the activations already in the operand form of the 8-bit matrix instructions.
 * The GEMV for a few rows (the reference's ternaryMVFP32, tmq/tmq_cuda.cu:242-286, 563-603; its row-batched
 * caller tmq/tmq.py:680-683) multiplies fp8 weight operands with the rows carried exactly as four bf8 terms per
 * value ("planes"); tmq_ternary_linear derives the planes inside every workgroup, these two calls do it once:
 *   tmq_gemv8_prepare          x: fp16 [M][K], 16-byte aligned -> planes (tmq_gemv8_planes_bytes(M, K) bytes,
 *                              16-byte aligned; an opaque image, valid for this M and K)
 *   tmq_ternary_linear_planes  y = epilogue(x W^T) from the planes; same results as tmq_ternary_linear on x
 * so that a vector multiplied with several layers (q / k / v, gate / up) or produced once and consumed later is
 * converted once. M <= 4, K a multiple of 256 from 2048 to 16384 and M' K <= 16384 with M' = M padded to 1, 2 or
 * 4 (else TMQ_ERR_UNSUPPORTED, and tmq_gemv8_planes_bytes returns 0).                                      */
size_t tmq_gemv8_planes_bytes(int64_t M, int64_t K);
int tmq_gemv8_prepare(const void *x, int64_t M, int64_t K, void *planes, void *stream);
int tmq_ternary_linear_planes(const void *planes, int64_t M, int64_t K, const void *native, int64_t N,
                              const tmq_epilogue *epilogue, void *y, void *stream);

/* 1 when tmq_ternary_linear(x, TMQ_F32, M, K, ...) takes fp32 activations of any magnitude as they are (one
 * 16-byte aligned row, K a multiple of 256 up to 16384: the kernel finds the row's largest finite |x| and scales
 * by a power of two itself), 0 when the caller has to keep them inside fp16's range (tmq_f32_prescale). */
int tmq_fp32_rows_self_scaled(const void *x, int64_t M, int64_t K);
/* The same question for a layer of N channels: also 1 for two 16-byte aligned rows with K a multiple of 256 up to
 * 6144 and N <= 6144 (each row scaled by its own power of two inside the one launch). */
int tmq_fp32_rows_self_scaled_for(const void *x, int64_t M, int64_t K, int64_t N);

/* Range handling for fp32 activations (no counterpart in the reference, whose kernels multiply fp32
 * activations in fp32, tmq/tmq_cuda.cu:242-427). Scans n fp32 values and writes prescale[0] = s,
 * prescale[1] = 1 / s (device, 2 floats): s is the power of two that brings the largest finite |x| into
 * [1024, 2048) (s = 1 for an all-zero tensor). Optionally, in the same call:
 *   xs (n floats)             xs[i] = s * x[i] (exact), the tensor to hand to tmq_ternary_linear;
 *   scale_out (channels)      scale_out[c] = (scale_in ? scale_in[c] : 1) / s, the epilogue scale that
 *                             undoes the prescale (bias and residual are added after it, unscaled).
 * Up to 65536 values are handled by one launch; beyond that by two (three with xs) and `workspace` must
 * hold tmq_f32_prescale_workspace_bytes(n) bytes.                                                  */
size_t tmq_f32_prescale_workspace_bytes(int64_t n);
int tmq_f32_prescale(const float *x, int64_t n, float *prescale, float *xs, const float *scale_in,
                     float *scale_out, int64_t channels, void *workspace, void *stream);

/* hi[i] = fp16(s x[i]), lo[i] = fp16(s x[i] - hi[i]) for n fp32 values (device pointers; hi, lo fp16), s =
 * prescale[0] (device; NULL = 1). lo may be NULL when one term is enough (the convolutions take fp16).
 * No counterpart in the reference, whose ternary_mmm_cuda (tmq/tmq_cuda.cu:478-549) multiplies fp32
 * activations in fp32: for many rows a caller that may allocate runs the fp16 kernels on the two terms,
 *   t = tmq_ternary_linear(hi, ..., scale, bias, residual)  (fp32 out, no ReLU)
 *   y = tmq_ternary_linear(lo, ..., scale, residual = t, ReLU)
 * which keeps ~fp32 accuracy at MFMA speed (M = 4096, K = N = 4096: 400 -> 238 us); the bindings in
 * tmq_amd/ops.py and tmq_amd/csrc/torch_ext.cpp do so where tmq_fp32_rows_prefer_split says it pays.
 * tmq_split_f32 is the form without a prescale.                                                     */
int tmq_split_f32_scaled(const float *x, const float *prescale, void *hi, void *lo, int64_t n, void *stream);
int tmq_split_f32(const float *x, void *hi, void *lo, int64_t n, void *stream);

/* tmq_f32_prescale followed by tmq_split_f32_scaled(..., lo = NULL) in two launches whatever the size: the largest
 * finite |x| (partial maxima in `workspace`, tmq_f32_to_f16_prescaled_workspace_bytes(n) bytes), then hi[i] = fp16(s x[i])
 * with prescale[0] = s, prescale[1] = 1 / s and, when scale_out is given, scale_out[c] = (scale_in ? scale_in[c] : 1) / s.
 * What a convolution on fp32 activations needs in front of it (the reference's convolutions take fp32,
 * tmq/tmq.py:822-871); same values as the two separate calls.                                            */
size_t tmq_f32_to_f16_prescaled_workspace_bytes(int64_t n);
int tmq_f32_to_f16_prescaled(const float *x, int64_t n, float *prescale, void *hi, const float *scale_in, float *scale_out,
                             int64_t channels, void *workspace, void *stream);

/* 1 if M fp32 rows against a K x N layer are faster as two fp16 passes over tmq_split_f32's terms than
 * as one tmq_ternary_linear call with x_dtype TMQ_F32 (many rows, or a few rows over a large
 * layer), else 0. Host-only arithmetic on the shape; no counterpart in the reference.               */
int tmq_fp32_rows_prefer_split(int64_t M, int64_t K, int64_t N);

/* Geometry of a 2-D convolution. */
typedef struct tmq_conv_shape {
    int32_t B, C, H, W;   /* input extents (batch, channels, height, width) */
    int32_t N;            /* output channels */
    int32_t ky, kx, sy, sx, py, px, dy, dx;
    int32_t py_end, px_end; /* zero rows / columns after the last input row / column; py, px
                             * count those before the first. Equal to py, px for the usual
                             * symmetric padding.                                           */
} tmq_conv_shape;

/* Output extents, floor((h + p + p_end - d(k-1) - 1)/s) + 1 (PyTorch's formula for symmetric
 * padding; the reference's own expression at tmq/tmq.py:842-845 agrees with it on every ResNet
 * shape).                                                                                     */
int tmq_conv2d_out_hw(const tmq_conv_shape *s, int32_t *ho, int32_t *wo);

/* Ternary implicit-GEMM convolution, no materialised im2col. x: fp16 NHWC [B][H][W][C]
 * (channels_last memory); native: tmq_prepack_weights(words, N, C, ky, kx); y: NHWC
 * [B][Ho][Wo][N] in epilogue->y_dtype. Replaces the unfold + ternary_mmm_cuda + fold path of
 * Conv2d.compact_forward (tmq/tmq.py:856-871) and its per-batch kernel launches
 * (tmq/tmq_cuda.cu:531-536).                                                                 */
int tmq_ternary_conv2d(const void *x, const tmq_conv_shape *shape, const void *native,
                       const tmq_epilogue *epilogue, void *y, void *stream);

/* tmq_ternary_conv2d whose output positions go into a strided NHWC destination instead of a dense
 * [B][Ho][Wo][N] tensor. Of the computed grid (Ho x Wo per image, tmq_conv2d_out_hw) the positions
 * h0 <= oh < h0 + h_cnt, w0 <= ow < w0 + w_cnt are kept, the others are computed and dropped; position
 * (b, oh, ow) is written to the N contiguous channels at
 *   y + (b * stride_b + (oh - h0) * stride_h + (ow - w0) * stride_w) * N      (strides in pixels),
 * and epilogue->residual, when given, is read at the same offsets. view == NULL is tmq_ternary_conv2d.
 * This is how a transposed convolution with groups == 1 is written in one pass: each phase of its output
 * grid is a stride-1 convolution with the taps that reach it, and its view is the phase's share of the
 * interleaved output (stride_w = sx, stride_h = sy * Wout, stride_b = Hout * Wout, y at the phase's first
 * position) -- no dense temporary and no strided copy, where ConvTranspose2d.compact_forward
 * (tmq/tmq.py:1007-1042) plans a GEMM into columns followed by F.fold.                               */
typedef struct tmq_output_view {
    int32_t h0, w0;          /* first kept row / column of the computed grid */
    int32_t h_cnt, w_cnt;    /* kept rows / columns */
    int64_t stride_b, stride_h, stride_w;   /* destination strides in pixels of N elements */
} tmq_output_view;
int tmq_ternary_conv2d_view(const void *x, const tmq_conv_shape *shape, const void *native,
                            const tmq_epilogue *epilogue, void *y, const tmq_output_view *view, void *stream);

/* Depthwise ternary convolution (groups == channels; shape->N must equal shape->C). x: fp16 NHWC;
 * words: the reference packing of a [C][1][ky][kx] weight tensor, words[ky*kx][ceil(C/16)]
 * (tmq_pack_ternary with N = C, K = ky*kx) -- read directly, no re-tiling; y: NHWC in
 * epilogue->y_dtype. Replaces the unfold + ternary_dwconv_cuda + fold branch of
 * Conv2d.compact_forward (tmq/tmq.py:849-853; kernel tmq/tmq_cuda.cu:166-238, host 607-642) without
 * materialising the patches.                                                                    */
int tmq_ternary_dwconv2d(const void *x, const tmq_conv_shape *shape, const uint32_t *words,
                         const tmq_epilogue *epilogue, void *y, void *stream);

/* The same arithmetic on unfolded patches, the calling convention of ternary_dwconv_cuda
 * (tmq/tmq_cuda.cu:607-642): x [P][taps][C] (TMQ_F32 or TMQ_F16), y fp32 [P][C],
 * y[p][c] = sum_t x[p][t][c] * T[c][t].                                                         */
int tmq_ternary_dwconv_patches(const void *x, int x_dtype, int64_t P, int32_t taps, int64_t C,
                               const uint32_t *words, float *y, void *stream);

/* Depthwise transposed convolution (groups == channels, one filter per channel), fused:
 *   y[b][oh][ow][c] = sum_{i,j} x[b][ih][iw][c] * T[c][i][j],  oh = ih*sy - py + i*dy, ow likewise.
 * x: fp16 NHWC [B][H][W][C]; shape describes the transposed convolution (N == C; py_end / px_end are
 * ignored); out_pad_*: PyTorch's output_padding; words: the reference packing of the
 * [C][1][ky][kx] weight, words[ky*kx][ceil(C/16)]; y: NHWC [B][Ho][Wo][C] in epilogue->y_dtype with
 * Ho = (H-1)*sy - 2*py + dy*(ky-1) + 1 + out_pad_y. Replaces ternary_dwconvtrans_cuda + F.fold in
 * ConvTranspose2d.compact_forward (tmq/tmq.py:1025-1029) without materialising the columns.      */
int tmq_convtranspose2d_out_hw(const tmq_conv_shape *shape, int32_t out_pad_y, int32_t out_pad_x,
                               int32_t *ho, int32_t *wo);
int tmq_ternary_dwconvtrans2d(const void *x, const tmq_conv_shape *shape, int32_t out_pad_y, int32_t out_pad_x,
                              const uint32_t *words, const tmq_epilogue *epilogue, void *y, void *stream);

/* The column form, the calling convention of ternary_dwconvtrans_cuda (tmq/tmq_cuda.cu:645-686,
 * kernel 118-162): x fp32 [B][P][C], y fp32 [B][C*taps][P], y[b][c*taps + t][p] = x[b][p][c] * T[c][t]
 * (the caller scatters y with F.fold). Every batch entry is processed (the reference's launch covers
 * the first only).                                                                                */
int tmq_ternary_dwconvtrans_cols(const float *x, int64_t B, int64_t P, int32_t taps, int64_t C,
                                 const uint32_t *words, float *y, void *stream);

/* ------------------------------------------------------------------------------------------
 * Memory-bound companions of the convolutions on fp16 NHWC feature maps. No counterpart in the
 * reference, whose ResNet sample (samples/resnet_test.py:91-118) leaves pooling to PyTorch on NCHW
 * fp32 tensors; a network that keeps fp16 NHWC between the ternary convolutions needs them.
 * ---------------------------------------------------------------------------------------- */

/* Max-pool, PyTorch's nn.MaxPool2d(kernel, stride, padding) with dilation 1 and floor mode:
 * x [B][H][W][C] fp16 -> y [B][Ho][Wo][C] fp16, Ho = floor((H + 2 py - ky) / sy) + 1. Padding takes
 * no part in the maximum (needs 2 p <= k).                                                       */
int tmq_maxpool2d_nhwc(const void *x, int32_t B, int32_t C, int32_t H, int32_t W, int32_t ky, int32_t kx,
                       int32_t sy, int32_t sx, int32_t py, int32_t px, void *y, void *stream);

/* The opening of a ResNet in one launch: tmq_ternary_conv2d with a ReLU epilogue and fp16 output,
 * followed by tmq_maxpool2d_nhwc(3, 3, 2, 2, 1, 1), without the convolution's output ever reaching
 * memory. x, shape, native, scale and bias as for tmq_ternary_conv2d (no residual); y fp16
 * [B][Po][Pwo][N] with Po = (Ho - 1) / 2 + 1 for the convolution's Ho, likewise Pwo. The result equals the
 * two separate calls bit for bit (finite inputs; a NaN loses against any number in the maximum, as in
 * tmq_maxpool2d_nhwc). For few-channel inputs with a short reduction only: C of 8, 16 or 32,
 * C * ky * kx <= 256, N <= 64 in whole groups of 8, and an input window per 15 x 17 outputs of under 64 KiB;
 * anything else returns TMQ_ERR_UNSUPPORTED and the caller makes the two calls.                   */
int tmq_ternary_conv2d_relu_maxpool(const void *x, const tmq_conv_shape *shape, const void *native,
                                    const float *scale, const float *bias, void *y, void *stream);

/* The same opening straight from the network's own input: x is NCHW fp16 [B][planes][H][2 W] with 1 .. 4 planes,
 * read as shape->C == 8 channel "super-pixels" of two neighbouring pixels x 4 channels (missing planes zero), i.e.
 * exactly the tensor tmq_nchw_to_nhwc4 would have written and shape describes ([B][H][W][8]) -- without that tensor ever
 * existing in memory. Same result bit for bit as tmq_nchw_to_nhwc4 followed by tmq_ternary_conv2d_relu_maxpool.
 * planes == 0 is tmq_ternary_conv2d_relu_maxpool (x NHWC). x 4-byte aligned. No counterpart in the reference.        */
int tmq_ternary_conv2d_relu_maxpool_planar(const void *x, int32_t planes, const tmq_conv_shape *shape, const void *native,
                                           const float *scale, const float *bias, void *y, void *stream);

/* Global average pool: x [B][HW][C] fp16 -> y [B][C] (TMQ_F16 or TMQ_F32), fp32 accumulation.    */
int tmq_avgpool_global_nhwc(const void *x, int64_t B, int64_t HW, int64_t C, void *y, int y_dtype,
                            void *stream);

/* A classifier head in one launch: tmq_avgpool_global_nhwc into fp16 means followed by tmq_ternary_linear of those
 * means (native: tmq_prepack_weights(words, N, C, 1, 1); epilogue: scale, bias, ReLU, output type; no residual),
 * y [B][N]. The means are computed and rounded as tmq_avgpool_global_nhwc does; the product's fp32 sums may differ from
 * the two-call form in the last bits (another order of accumulation). C <= 512 in whole groups of 8 and 16-byte
 * aligned x; anything else returns TMQ_ERR_UNSUPPORTED and the caller makes the two calls. No counterpart in the
 * reference (its sample leaves the head to PyTorch: samples/resnet_test.py:91-118).                             */
int tmq_avgpool_linear(const void *x, int64_t B, int64_t HW, int64_t C, const void *native, int64_t N,
                       const tmq_epilogue *epilogue, void *y, void *stream);

/* Network input repack: x [B][C][H][W] (TMQ_F16 or TMQ_F32, C <= 4, W % 4 == 0) -> y [B][H][W][4]
 * fp16, channels C..3 zero (the layout the few-channel convolution loader wants).               */
int tmq_nchw_to_nhwc4(const void *x, int x_dtype, int64_t B, int32_t C, int64_t H, int64_t W, void *y,
                      void *stream);

/* ------------------------------------------------------------------------------------------
 * DIAGNOSTICS AND MEASUREMENT AIDS. Not part of the product surface: nothing in the library's own
 * call paths uses them and a caller never needs them. They exist for the test suite (device-side
 * proofs about the kernels' arithmetic) and for the benchmark (a read-only stream as the floor a
 * GEMV is compared with). None has a counterpart in the reference.
 * ---------------------------------------------------------------------------------------- */

/* Diagnostic with no counterpart in the reference: the kernels above replace IEEE division by
 * cheaper FMA sequences; this proves on the device that they are bit-identical to IEEE
 * division. counts (device, 5 x uint64) receives: [0..2] mismatches of the three rational
 * pieces over every fp32 argument in [-3,3] (and NaN), [3] mismatches of x / c(digamma) over
 * every mantissa, both signs, three binades, [4] the number of arguments swept (a sanity
 * figure, 2*0x40400000 + 1 + NaNs). All mismatch counts must be 0.                           */
int tmq_selfcheck_division(double digamma, uint64_t *counts, void *stream);

/* Measurement aid with no counterpart in the reference: streams `bytes` (a multiple of 1024)
 * from src with the launch geometry of the M = 1 path of tmq_ternary_linear (1 KiB per
 * wavefront and load, 16 wavefronts per workgroup) and does nothing else; *sink (device, 4
 * bytes) is only written if the data has an impossible checksum. Its duration is the floor for
 * a kernel that has to read that many bytes once: launch + one trip to memory.               */
int tmq_probe_stream_read(const void *src, size_t bytes, uint32_t *sink, void *stream);

/* Diagnostic with no counterpart in the reference, host only: the convolution and pooling kernels
 * turn an output pixel's index into (batch, row, column) with a multiply-high by constants computed on
 * the host instead of integer divisions. Returns how many of n[0 .. count) (host memory, each below
 * 2^31) the same constants divide wrongly by `divisor` (1 <= divisor < 2^31): must be 0.            */
int64_t tmq_selfcheck_fastdiv(uint32_t divisor, const uint32_t *n, int64_t count);

/* ------------------------------------------------------------------------------------------
 * Host entropy codec for packed tensors (host memory in, host memory out; no GPU involved).
 * ---------------------------------------------------------------------------------------- */

/* Upper bound of the container size for rows*columns symbols. */
size_t tmq_compress_bound(int64_t rows, int64_t columns);

/* Range-code words[rows][ceil(columns/16)] into out (capacity out_cap); *out_size receives the
 * container size. Byte-compatible with compress_ternary (tmq/tmq_native.cpp:439-477 ->
 * entropyEncodeTernary 50-97 -> RangeEncoder tmq/rangecoder.h:41-112).                       */
int tmq_compress_ternary(const uint32_t *words_host, int64_t rows, int64_t columns, uint8_t *out,
                         size_t out_cap, size_t *out_size);

/* Inverse. Replaces decompress_ternary (tmq/tmq_native.cpp:489-503 -> entropyDecodeTernary
 * 111-140 -> RangeDecoder tmq/rangecoder.h:124-193).                                         */
int tmq_decompress_ternary(const uint8_t *in, size_t in_size, uint32_t *words_host, int64_t rows,
                           int64_t columns);

#ifdef __cplusplus
}
#endif
#endif /* TMQ_HIP_H */
