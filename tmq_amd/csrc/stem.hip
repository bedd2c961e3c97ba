// The opening of a ResNet in one kernel, gfx950: ternary convolution over few input channels -> per-channel
// scale and bias (a folded BatchNorm) -> ReLU -> 3 x 3 / stride 2 / pad 1 max-pool, fp16 NHWC in and out. The
// convolution's output, four times the size of the pooled result, never reaches memory.
//
// The general implicit-GEMM kernel copies every input pixel once per kernel tap into its im2col tile (28 times
// for a 7 x 4 window) and spends ~15 vector-ALU instructions per MFMA on the addresses of those copies; with a
// reduction of only 224 that, not the matrix work, is what it waits for. Here a workgroup loads the input
// window of its patch of outputs into LDS once (35 x 20 pixels of 16 bytes for a 15 x 17 patch of the
// 7 x 4 / stride (2, 1) stem) and the MFMA operands are read straight out of it: with 8 channels per pixel
// the 8 consecutive reduction indices a lane feeds into v_mfma_f32_16x16x32_f16 are exactly one pixel of one
// tap, so an operand is one ds_read_b128 at (row's window origin) + (tap's displacement), one addition.
//
// Work split: a workgroup (4 wavefronts) owns the 15 x 17 patch of convolution outputs that 7 x 8 pooled
// positions need (rows 14 th - 1 .. 14 th + 13, columns 16 tw - 1 .. 16 tw + 15 of image b); neighbouring
// patches share their border row and column, 255 positions computed for 224 new ones. The patch is a
// 256-row GEMM tile by up to 64 output channels; a wavefront takes 128 rows x 32 channels. Rows 16 f .. 16 f + 15
// (one MFMA row fragment) are columns 0 .. 15 of patch row f < 15 -- neighbouring pixels of the window, so the
// 16 lanes of an operand read touch 16 consecutive pieces, every LDS bank once -- and rows 240 .. 254 are column
// 16 of the 15 patch rows (row 255 repeats row 254 and is never pooled). The results go, as fp16, into a
// [256][64] tile in LDS (over the input window, which is no longer needed), and the workgroup pools that.
#include "common.h"
#include "mfma.h"

namespace tmq {
namespace {

constexpr int kPoolH = 7, kPoolW = 8;                                  // pooled positions per patch
constexpr int kPatchH = 2 * kPoolH + 1, kPatchW = 2 * kPoolW + 1;       // convolution outputs per patch
constexpr int kTilePitch = 144;                                         // bytes per row of the fp16 [256][64] tile (16 of padding)
constexpr int kTileBytes = 256 * kTilePitch;
constexpr int kThreads = 256;
constexpr int kMaxLds = 64 * 1024;

struct StemShape {
    const _Float16 *x;
    uint32_t x_bytes;
    int cshift;                  // log2 of the input channels (3 .. 5)
    int H, W, Ho, Wo, kx, sy, sx, py, px, dy, dx;
    int Po, Pwo;                 // pooled extents
    int PC;                      // pixels per row of a patch's input window
    int chunks;                  // 16-byte pieces in the window
    int zero_off;                // LDS byte offset of a zeroed copy of the window's extent (behind the window), or 0 if not needed
    int tab_off;                 // LDS byte offset of the table of piece displacements (behind both)
    int const_off;               // LDS byte offset of scale[64], bias[64] (behind the tile as well)
    int kchunks;                 // 16-byte pieces (8 reduction indices) per output: K / 8
    FastDiv by_tw, by_th, by_kx, by_row;   // patches per image row / column, kernel width, 16-byte pieces per window row
    int planes;                  // 0: x is NHWC; 1 .. 4: x is the network's own NCHW fp16 input with that many channels, read as
                                 // 8-channel "super-pixels" of two neighbouring pixels x 4 channels (cshift == 3, W = width / 2)
};

template <int WM, int WN>
__global__ __launch_bounds__(kThreads, 3) void stem_pool_kernel(StemShape p, const uint32_t *__restrict__ native, int N,
                                                                const float *__restrict__ scale, const float *__restrict__ bias,
                                                                _Float16 *__restrict__ y, int tiles) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63, wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int WGN = 4 / WN, D = WM / 2;          // wavefronts side by side; how many row fragments ahead the operand reads run
    static_assert(WM * WN == 16 && (WN == 2 || WN == 4), "a wavefront takes 16 WM rows x 16 WN channels of the 256 x 64 tile");
    const int wm = wv / WGN, wn = wv % WGN;
    const int r16 = lane & 15, g = lane >> 4;

    // patch of this workgroup; the workgroups of one XCD (one L2) take neighbouring patches, which share input rows
    int tw, th;
    const uint32_t t = p.by_tw.divmod((uint32_t)xcd_contiguous(blockIdx.x, tiles), tw);
    const int b = (int)p.by_th.divmod(t, th);
    const int oh0 = 2 * kPoolH * th - 1, ow0 = 2 * kPoolW * tw - 1;
    const int ih_base = oh0 * p.sy - p.py, iw_base = ow0 * p.sx - p.px;

    // ---- the input window -> LDS, 16 bytes per lane; pixels outside the image (padding) arrive as zeros ----
    const BufferResource rsrc = make_buffer_resource(p.x, p.x_bytes);
    const int sub_mask = (1 << (p.cshift - 3)) - 1;
    if (p.planes) {
        // Planar input: a piece of the window is two neighbouring pixels of up to four planes. One 4-byte load per plane
        // (the pixel pair), interleaved in registers to (c0 c1 c2 c3 | c0 c1 c2 c3) and written to the place the
        // 16-byte copy of the NHWC path would have filled: no repacked copy of the input ever exists in memory.
        const int64_t plane = (int64_t)p.H * p.W;                       // pixel pairs per plane
        const uint32_t *img = reinterpret_cast<const uint32_t *>(p.x) + (int64_t)b * p.planes * plane;
        for (int c0 = 0; c0 < p.chunks; c0 += kThreads) {
            const int c = c0 + tid;
            int rc;
            const int prow = (int)p.by_row.divmod((uint32_t)c, rc);
            const int ih = ih_base + prow, iw = iw_base + rc;
            const bool in = (c < p.chunks) & ((unsigned)ih < (unsigned)p.H) & ((unsigned)iw < (unsigned)p.W);
            uint32_t v[4] = {0u, 0u, 0u, 0u};
            if (in) {
                const uint32_t *src = img + (int64_t)ih * p.W + iw;
#pragma unroll
                for (int q = 0; q < 4; q++)
                    if (q < p.planes) v[q] = src[q * plane];
            }
            if (c < p.chunks)
                *reinterpret_cast<u32x4 *>(lds + c * 16) = u32x4{(v[0] & 0xFFFFu) | (v[1] << 16), (v[2] & 0xFFFFu) | (v[3] << 16),
                                                                (v[0] >> 16) | (v[1] & 0xFFFF0000u), (v[2] >> 16) | (v[3] & 0xFFFF0000u)};
        }
    } else
    for (int c0 = 0; c0 < p.chunks; c0 += kThreads) {
        const int c = c0 + tid;
        int rc;
        const int prow = (int)p.by_row.divmod((uint32_t)c, rc);
        const int ih = ih_base + prow, iw = iw_base + (rc >> (p.cshift - 3));
        const bool in = (c < p.chunks) & ((unsigned)ih < (unsigned)p.H) & ((unsigned)iw < (unsigned)p.W);
        const uint32_t off = ((uint32_t)(((b * p.H + ih) * p.W + iw) << p.cshift) + (uint32_t)((rc & sub_mask) * 8)) * 2u;
        buffer_to_lds(rsrc, in ? off : kPastTheEnd, lds + (c0 + wv * 64) * 16);
    }
    // a reduction that ends inside an MFMA step: the step's lanes past K read zeros -- a zeroed region as large as the
    // window behind it, so that (row's origin) + zero_off is a zero piece for every row and no read needs a select
    if (p.zero_off)
        for (int c = tid; c < p.chunks; c += kThreads) *reinterpret_cast<u32x4 *>(lds + p.zero_off + c * 16) = u32x4{0u, 0u, 0u, 0u};

    // ---- while that is on its way: weights (the whole reduction is one native block), constants, addresses ----
    const int Nb = (N + 15) >> 4;
    u32x4 wblk[WN];
#pragma unroll
    for (int j = 0; j < WN; j++) {
        int nb = wn * WN + j;
        nb = nb < Nb ? nb : Nb - 1;                 // columns past N: finite bits, never pooled
        wblk[j] = *reinterpret_cast<const u32x4 *>(native + nb * 256 + lane * 4);
    }
    // LDS byte offset of the window origin of the lane's row in each of its row fragments
    int rowbase[WM];
    const int pixel_shift = p.cshift + 1, lane_col = (r16 * p.sx) << pixel_shift;
#pragma unroll
    for (int i = 0; i < WM; i++) rowbase[i] = ((((wm * WM + i) * p.sy) * p.PC) << pixel_shift) + lane_col;
    if (wm == 16 / WM - 1)                          // the last fragment: column 16 of the 15 patch rows
        rowbase[WM - 1] = (((r16 < kPatchH ? r16 : kPatchH - 1) * p.sy) * p.PC + (kPatchW - 1) * p.sx) << pixel_shift;
    // Displacement of piece u of the reduction (indices 8 u .. 8 u + 7 = one tap, 8 channels): a table, since a lane needs
    // piece 4 s + g in MFMA step s. Pieces past K point into the zeroed region.
    if (tid < 32) {
        int j;
        const int i = (int)p.by_kx.divmod((uint32_t)(tid >> (p.cshift - 3)), j);
        const int d = ((((i * p.dy) * p.PC + j * p.dx) << (p.cshift - 3)) + (tid & sub_mask)) * 16;
        *reinterpret_cast<int *>(lds + p.tab_off + tid * 4) = tid < p.kchunks ? d : p.zero_off;
    }
    // Per-channel scale (the weight unit folded in) and bias go through a table behind everything else in LDS: the
    // trip to memory ends while the window is on its way, where a load in the epilogue would make every wavefront wait.
    float *const constants = reinterpret_cast<float *>(lds + p.const_off);
    if (tid < 64) {
        constants[tid] = (tid < N && scale ? scale[tid] : 1.f) * (1.0f / kWeightUnit);
        constants[64 + tid] = tid < N && bias ? bias[tid] : 0.f;
    }
    const int S = (p.kchunks + 3) >> 2;

    floatx4 acc[WM][WN];
    __syncthreads();                                // waits for this thread's loads, then for everybody's

    // ---- WM row fragments x WN column fragments per 32-wide step; operand reads run D fragments ahead ----
    auto operand = [&](int i, int disp) { return *reinterpret_cast<const half8 *>(lds + rowbase[i] + disp); };
    const floatx4 none = {0.f, 0.f, 0.f, 0.f};
    half8 a[WM];
    int disps[8];
#pragma unroll
    for (int st = 0; st < 8; st++) disps[st] = *reinterpret_cast<const int *>(lds + p.tab_off + st * 16 + g * 4);
    int disp = disps[0], disp_next = 0;
#pragma unroll
    for (int q = 0; q < D; q++) a[q] = operand(q, disp);
#pragma unroll
    for (int kt = 0; kt < 4; kt++) {
        if (2 * kt >= S) break;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int s = 2 * kt + h;
            if (s >= S) break;
            half8 b[WN];
#pragma unroll
            for (int j = 0; j < WN; j++) b[j] = decode_step(wblk[j][kt], h);
            const bool more = s + 1 < S;
            if (more) disp_next = disps[s + 1 < 8 ? s + 1 : 7];
#pragma unroll
            for (int q = 0; q < WM; q++) {
#pragma unroll
                for (int j = 0; j < WN; j++) acc[q][j] = mfma16(b[j], a[q], s == 0 ? none : acc[q][j]);
                if (q < WM - D) a[q + D] = operand(q + D, disp);
                else if (more) a[q - (WM - D)] = operand(q - (WM - D), disp_next);
            }
            disp = disp_next;
        }
    }
    // Scale and bias of the lane's channels, out of the table: with the weights as the first MFMA operand an accumulator
    // holds channels 4 g .. 4 g + 3 of its 16-channel block at position r16 of its row fragment, four neighbours of a
    // tile row.
    floatx4 sc[WN], bi[WN];
#pragma unroll
    for (int j = 0; j < WN; j++) {
        sc[j] = *reinterpret_cast<const floatx4 *>(constants + (wn * WN + j) * 16 + g * 4);
        bi[j] = *reinterpret_cast<const floatx4 *>(constants + 64 + (wn * WN + j) * 16 + g * 4);
    }
    __syncthreads();                                // everybody is done with the window: the tile goes over it

    // ---- results -> fp16 tile: the value the convolution alone would store before its ReLU ----
    unsigned char *dst = lds + (wm * WM * 16 + r16) * kTilePitch + (wn * WN * 16 + g * 4) * 2;
#pragma unroll
    for (int i = 0; i < WM; i++)
#pragma unroll
        for (int j = 0; j < WN; j++) {
            const floatx4 v = acc[i][j] * sc[j] + bi[j];
            *reinterpret_cast<half4 *>(dst + i * 16 * kTilePitch + j * 32) = half4{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
        }
    __syncthreads();

    // ---- 3 x 3 maxima, 8 channels per thread and item. Patch positions outside the convolution's output (the pooling's
    //      padding; only in patches on the border) take no part. The ReLU commutes with the maximum and with the rounding
    //      to fp16, so it comes last. ----
    const bool whole = oh0 >= 0 && oh0 + kPatchH <= p.Ho && ow0 >= 0 && ow0 + kPatchW <= p.Wo;   // uniform
    const _Float16 ninf = (_Float16)(-__builtin_inff());
    const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0}, lowest = {ninf, ninf, ninf, ninf, ninf, ninf, ninf, ninf};
    for (int item = tid; item < kPoolH * kPoolW * 8; item += kThreads) {
        // lanes: channel octet fastest, then pooled columns 4 apart -- 16 lanes read 256 bytes on distinct banks
        const int c8 = item & 7, q = item >> 3, pw_ = ((q & 1) << 2) | ((q >> 1) & 3), ph_ = q >> 3;
        const int ph = th * kPoolH + ph_, pw = tw * kPoolW + pw_;
        if (ph >= p.Po || pw >= p.Pwo || c8 * 8 >= N) continue;
        // tile row of patch position (r, c): 16 r + c, or 240 + r for c = 16 (the third column of the last pooled column)
        const unsigned char *src = lds + ((2 * ph_) * 16 + 2 * pw_) * kTilePitch + c8 * 16;
        const bool edge = pw_ == kPoolW - 1;
        const unsigned char *third = edge ? lds + (240 + 2 * ph_) * kTilePitch + c8 * 16 : src + 2 * kTilePitch;
        const int third_step = edge ? kTilePitch : 16 * kTilePitch;
        auto tap = [&](int e) {
            return *reinterpret_cast<const half8 *>(e % 3 == 2 ? third + (e / 3) * third_step : src + ((e / 3) * 16 + e % 3) * kTilePitch);
        };
        half8 m = tap(4);                                   // the centre always exists
        if (whole) {
#pragma unroll
            for (int e = 0; e < 9; e++)
                if (e != 4) m = __builtin_elementwise_max(m, tap(e));
        } else {
            const int oh = 2 * ph - 1, ow = 2 * pw - 1;
#pragma unroll
            for (int e = 0; e < 9; e++) {
                if (e == 4) continue;
                const bool out = ((unsigned)(oh + e / 3) < (unsigned)p.Ho) & ((unsigned)(ow + e % 3) < (unsigned)p.Wo);
                m = __builtin_elementwise_max(m, out ? tap(e) : lowest);
            }
        }
        m = __builtin_elementwise_max(m, zero);
        *reinterpret_cast<half8 *>(y + (((int64_t)b * p.Po + ph) * p.Pwo + pw) * N + c8 * 8) = m;
    }
}

}  // namespace

extern "C" {

int tmq_ternary_conv2d_relu_maxpool(const void *x, const tmq_conv_shape *s, const void *native, const float *scale,
                                    const float *bias, void *y, void *stream) {
    return tmq_ternary_conv2d_relu_maxpool_planar(x, 0, s, native, scale, bias, y, stream);
}

int tmq_ternary_conv2d_relu_maxpool_planar(const void *x, int32_t planes, const tmq_conv_shape *s, const void *native,
                                           const float *scale, const float *bias, void *y, void *stream) {
    if (!s || !x || !native || !y || !aligned16(native) || planes < 0 || planes > 4) return TMQ_ERR_INVALID_ARG;
    if (planes && (s->C != 8 || (reinterpret_cast<uintptr_t>(x) & 3u))) return TMQ_ERR_UNSUPPORTED;
    int32_t ho, wo;
    const int rc = tmq_conv2d_out_hw(s, &ho, &wo);
    if (rc != TMQ_OK) return rc;
    if (s->B < 0 || s->C <= 0 || s->H <= 0 || s->W <= 0 || s->N <= 0 || s->py < 0 || s->px < 0) return TMQ_ERR_INVALID_ARG;
    if (ho <= 0 || wo <= 0) return TMQ_ERR_INVALID_ARG;
    const int64_t K = (int64_t)s->C * s->ky * s->kx, x_bytes = (int64_t)s->B * s->H * s->W * s->C * 2;
    if (!(s->C == 8 || s->C == 16 || s->C == 32) || K > kKB || s->N > 64 || s->N % 8 != 0 || (!planes && !aligned16(x)) || !aligned16(y) ||
        x_bytes >= (int64_t)kPastTheEnd - 16)
        return TMQ_ERR_UNSUPPORTED;
    StemShape p{};
    p.planes = planes;
    p.x = static_cast<const _Float16 *>(x);
    p.x_bytes = (uint32_t)x_bytes;
    p.cshift = s->C == 8 ? 3 : (s->C == 16 ? 4 : 5);
    p.H = s->H; p.W = s->W; p.Ho = ho; p.Wo = wo; p.kx = s->kx;
    p.sy = s->sy; p.sx = s->sx; p.py = s->py; p.px = s->px; p.dy = s->dy; p.dx = s->dx;
    p.Po = (ho - 1) / 2 + 1;
    p.Pwo = (wo - 1) / 2 + 1;
    // the input window of a patch: its first and last output rows / columns and the kernel's extent
    const int64_t PR = (int64_t)(kPatchH - 1) * s->sy + (int64_t)(s->ky - 1) * s->dy + 1;
    const int64_t PC = (int64_t)(kPatchW - 1) * s->sx + (int64_t)(s->kx - 1) * s->dx + 1;
    const int64_t chunks = PR * PC * (s->C / 8), padded = (chunks + kThreads - 1) / kThreads * kThreads;
    const bool ragged = (K / 8) % 4 != 0;                 // the last MFMA step reaches past K
    const int64_t lds_window = padded * 16 + (ragged ? chunks * 16 : 0) + 32 * 4;   // window, zeros, displacement table
    if (lds_window + 128 * 4 > kMaxLds) return TMQ_ERR_UNSUPPORTED;
    p.PC = (int)PC;
    p.chunks = (int)chunks;
    p.zero_off = ragged ? (int)(padded * 16) : 0;
    p.tab_off = (int)(lds_window - 32 * 4);
    p.kchunks = (int)(K / 8);
    const int th = (p.Po + kPoolH - 1) / kPoolH, tw = (p.Pwo + kPoolW - 1) / kPoolW;
    p.by_tw = FastDiv((uint32_t)tw);
    p.by_th = FastDiv((uint32_t)th);
    p.by_kx = FastDiv((uint32_t)s->kx);
    p.by_row = FastDiv((uint32_t)(PC * (s->C / 8)));
    const int64_t tiles = (int64_t)s->B * th * tw;
    if (tiles > (int64_t)0x7FFFFFFF) return TMQ_ERR_TOO_LARGE;
    if (tiles == 0) return TMQ_OK;
    p.const_off = (int)(lds_window > kTileBytes ? lds_window : kTileBytes);
    const size_t lds = (size_t)p.const_off + 128 * 4;
    hipLaunchKernelGGL((stem_pool_kernel<4, 4>), dim3((uint32_t)tiles), dim3(kThreads), lds, as_stream(stream), p,
                       static_cast<const uint32_t *>(native), (int)s->N, scale, bias, static_cast<_Float16 *>(y), (int)tiles);
    return check_launch();
}

}  // extern "C"
}  // namespace tmq
