// Epilogue shared by the tile kernels (dense / implicit-GEMM convolution): per-column scale and bias,
// optional residual and ReLU, fp32 or fp16 output, written row-wise through an LDS transpose.
#pragma once

#include "common.h"
#include "mfma.h"

namespace tmq {

template <class Map>
struct EpilogueT {
    const float *scale;      // [N] or null
    const float *bias;       // [N] or null
    const void *residual;    // same shape/dtype as y, or null
    void *y;
    int relu;
    int y_f16;
    [[no_unique_address]] Map map;   // where row m goes: pixel m (NoMap, no bytes) or a strided destination (RowMap)
};
using Epilogue = EpilogueT<NoMap>;
using ViewEpilogue = EpilogueT<RowMap>;
using PairEpilogue = EpilogueT<PairMap>;
static_assert(sizeof(Epilogue) == 40, "the dense epilogue carries no map");

#if defined(__HIPCC__)

// fp16 results whose rows are whole 16-byte pieces are written 8 columns (16 bytes) per lane, everything
// else 4 columns per lane: a store instruction costs the CU's address unit the same 16 cycles either way.
template <class Ep>
__device__ __forceinline__ bool wide_rows(const Ep &ep, int64_t N) {
    return ep.y_f16 && (N % 8 == 0) &&
           ((reinterpret_cast<uintptr_t>(ep.y) | reinterpret_cast<uintptr_t>(ep.residual)) & 15u) == 0;
}

// Per-column scale (the weight unit folded in) and bias of the columns a lane writes in write_tile:
// columns nw0 + 4 (lane % (4 WN)) .. + 3 in sc[0] / bi[0], or, for wide rows, nw0 + 8 (lane % (2 WN)) .. + 7
// in sc[0..1] / bi[0..1]. 16-byte loads where the vectors allow it.
struct ColumnConstants {
    floatx4 sc[2], bi[2];
};

template <int WN, class Ep>
__device__ __forceinline__ void load_scale_bias(const Ep &ep, int lane, int64_t nw0, int64_t N, ColumnConstants &cc) {
    const bool wide = wide_rows(ep, N);
    const int64_t n = wide ? nw0 + (lane % (2 * WN)) * 8 : nw0 + (lane % (4 * WN)) * 4;
    const bool vec = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(ep.scale) | reinterpret_cast<uintptr_t>(ep.bias)) & 15u) == 0;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        cc.sc[h] = floatx4{1.f, 1.f, 1.f, 1.f};
        cc.bi[h] = floatx4{0.f, 0.f, 0.f, 0.f};
        if (h == 1 && !wide) break;
        const int64_t nh = n + 4 * h;
        if (vec) {
            if (nh < N) {
                if (ep.scale) cc.sc[h] = *reinterpret_cast<const floatx4 *>(ep.scale + nh);
                if (ep.bias) cc.bi[h] = *reinterpret_cast<const floatx4 *>(ep.bias + nh);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (nh + e < N) {
                    if (ep.scale) cc.sc[h][e] = ep.scale[nh + e];
                    if (ep.bias) cc.bi[h][e] = ep.bias[nh + e];
                }
        }
        cc.sc[h] *= 1.0f / kWeightUnit;
    }
}

// v + (float)h for the low / high half of a packed pair: one v_fma_mix_f32 (conversion and addition in one
// instruction, rounded once -- the same value as a conversion followed by an addition).
__device__ __forceinline__ float add_half_lo(uint32_t pair, float v) {
    float r;
    asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(pair), "v"(v));
    return r;
}
__device__ __forceinline__ float add_half_hi(uint32_t pair, float v) {
    float r;
    asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(pair), "v"(v));
    return r;
}

// write_tile for fp16 results in whole 16-byte row pieces (wide_rows): 8 columns per lane. The residual pieces of
// up to kAhead slabs are requested before the slabs are transposed, so that their trip to memory overlaps with
// the LDS traffic instead of standing between a slab's arithmetic and its stores; a piece's offset is computed
// once, for the request, and kept for the store. Conversions are packed (v_cvt_pk_f16_f32), the residual is
// added with v_fma_mix_f32.
template <int WM, int WN, class Ep>
__device__ __forceinline__ void write_tile_wide(float *slab, const floatx4 (&acc)[WM][WN], const ColumnConstants &cc, int lane,
                                                int64_t mw0, int64_t nw0, int64_t M, int64_t N, const Ep &ep) {
    typedef float float2v __attribute__((ext_vector_type(2)));
    constexpr int kEP = 16 * WN + 4, kPieces = (WN + 1) / 2;       // pieces of 8 columns per lane and slab
    constexpr int kAhead = WM * kPieces <= 8 ? WM : (8 / kPieces > 0 ? 8 / kPieces : 1);
    const int r16 = lane & 15, g = lane >> 4;
    const _Float16 *res = static_cast<const _Float16 *>(ep.residual);
    int64_t off[kAhead][kPieces];                                  // element offset of the lane's piece, -1: none
    u32x4 rs[kAhead][kPieces];
    float gs[WM];                                                  // row pairs: 1 / s of each fragment's group
    if constexpr (decltype(ep.map)::kPairs) {
#pragma unroll
        for (int i = 0; i < WM; i++) gs[i] = ep.map.fragment_scale(mw0 + (int64_t)i * 16);
    }
    auto request = [&](int i, int slot) {
#pragma unroll
        for (int t = 0; t < kPieces; t++) {
            const int idx = t * 64 + lane, row = idx / (2 * WN), c8 = idx % (2 * WN);
            const int64_t m = mw0 + (int64_t)i * 16 + row, n = nw0 + c8 * 8;
            int64_t o = -1;
            if (idx < 32 * WN && m < M && n < N) {
                const int64_t px = ep.map.pixel(m);
                if (!decltype(ep.map)::kDrops || px >= 0) o = px * N + n;
            }
            off[slot][t] = o;
            if (res && o >= 0) rs[slot][t] = *reinterpret_cast<const u32x4 *>(res + o);
        }
    };
#pragma unroll
    for (int i = 0; i < kAhead; i++) request(i, i);
#pragma unroll
    for (int i = 0; i < WM; i++) {
#pragma unroll
        for (int j = 0; j < WN; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) slab[(g * 4 + r) * kEP + j * 16 + r16] = acc[i][j][r];
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int t = 0; t < kPieces; t++) {
            const int idx = t * 64 + lane, row = idx / (2 * WN), c8 = idx % (2 * WN);
            if (idx >= 32 * WN) continue;
            floatx4 v0 = *reinterpret_cast<const floatx4 *>(&slab[row * kEP + c8 * 8]);
            floatx4 v1 = *reinterpret_cast<const floatx4 *>(&slab[row * kEP + c8 * 8 + 4]);
            if constexpr (decltype(ep.map)::kPairs) {              // (hi row + its lo row) / s
                v0 = (v0 + *reinterpret_cast<const floatx4 *>(&slab[(row ^ 8) * kEP + c8 * 8])) * gs[i];
                v1 = (v1 + *reinterpret_cast<const floatx4 *>(&slab[(row ^ 8) * kEP + c8 * 8 + 4])) * gs[i];
            }
            v0 = v0 * cc.sc[0] + cc.bi[0];
            v1 = v1 * cc.sc[1] + cc.bi[1];
            const int64_t o = off[i % kAhead][t];
            if (o < 0) continue;
            if (res) {
                const u32x4 q = rs[i % kAhead][t];
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    v0[2 * e] = add_half_lo(q[e], v0[2 * e]);
                    v0[2 * e + 1] = add_half_hi(q[e], v0[2 * e + 1]);
                    v1[2 * e] = add_half_lo(q[2 + e], v1[2 * e]);
                    v1[2 * e + 1] = add_half_hi(q[2 + e], v1[2 * e + 1]);
                }
            }
            if (ep.relu) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    v0[e] = v0[e] < 0.f ? 0.f : v0[e];
                    v1[e] = v1[e] < 0.f ? 0.f : v1[e];
                }
            }
            half8 h;
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const half2v lo = __builtin_convertvector(float2v{v0[2 * e], v0[2 * e + 1]}, half2v);
                const half2v hi = __builtin_convertvector(float2v{v1[2 * e], v1[2 * e + 1]}, half2v);
                h[2 * e] = lo[0]; h[2 * e + 1] = lo[1];
                h[4 + 2 * e] = hi[0]; h[4 + 2 * e + 1] = hi[1];
            }
            *reinterpret_cast<half8 *>(static_cast<_Float16 *>(ep.y) + o) = h;
        }
        __builtin_amdgcn_wave_barrier();
        if (i + kAhead < WM) request(i + kAhead, i % kAhead);
    }
}

// Epilogue of one wavefront's (16 WM) x (16 WN) accumulator block. A lane holds rows 4g + r, column
// r16 of each 16 x 16 accumulator -- 64-byte row pieces if stored directly. Instead the wavefront
// transposes one 16-row slab (16 x 16 WN values) at a time through its own slice of LDS (`slab`, the
// idle activation buffer) and writes whole rows, 16 bytes per lane: 4 fp32 or, for wide rows, 8 fp16
// values. cc: scale and bias of the lane's columns (load_scale_bias).
template <int WM, int WN, class Ep>
__device__ __forceinline__ void write_tile(float *slab, const floatx4 (&acc)[WM][WN], const ColumnConstants &cc, int lane,
                                           int64_t mw0, int64_t nw0, int64_t M, int64_t N, const Ep &ep) {
    constexpr int kEP = 16 * WN + 4;                       // slab row pitch in floats (+4: conflict-free)
    const int r16 = lane & 15, g = lane >> 4;
    const bool vec = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(ep.y) | reinterpret_cast<uintptr_t>(ep.residual)) & 15u) == 0;
    if (wide_rows(ep, N)) return write_tile_wide<WM, WN>(slab, acc, cc, lane, mw0, nw0, M, N, ep);
    float gs[WM];                                          // row pairs: 1 / s of each fragment's group
    if constexpr (decltype(ep.map)::kPairs) {
#pragma unroll
        for (int i = 0; i < WM; i++) gs[i] = ep.map.fragment_scale(mw0 + (int64_t)i * 16);
    }
#pragma unroll
    for (int i = 0; i < WM; i++) {
#pragma unroll
        for (int j = 0; j < WN; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) slab[(g * 4 + r) * kEP + j * 16 + r16] = acc[i][j][r];
        __builtin_amdgcn_wave_barrier();
        const int64_t mrow0 = mw0 + (int64_t)i * 16;
#pragma unroll
        for (int t = 0; t < WN; t++) {                     // 16 rows x (16 WN / 4) float4 = 64 WN float4 per slab
            const int idx = t * 64 + lane, row = idx / (4 * WN), c4 = idx % (4 * WN);
            const int64_t m = mrow0 + row, n = nw0 + c4 * 4;
            floatx4 v = *reinterpret_cast<const floatx4 *>(&slab[row * kEP + c4 * 4]);
            if constexpr (decltype(ep.map)::kPairs) v = (v + *reinterpret_cast<const floatx4 *>(&slab[(row ^ 8) * kEP + c4 * 4])) * gs[i];
            v = v * cc.sc[0] + cc.bi[0];
            if (m >= M || n >= N) continue;
            const int64_t px = ep.map.pixel(m);
            if (decltype(ep.map)::kDrops && px < 0) continue;
            const int64_t o = px * N + n;
            if (vec) {
                if (ep.y_f16) {
                    if (ep.residual) {
                        const half4 rs = *reinterpret_cast<const half4 *>(static_cast<const _Float16 *>(ep.residual) + o);
#pragma unroll
                        for (int e = 0; e < 4; e++) v[e] += (float)rs[e];
                    }
                    half4 h;
#pragma unroll
                    for (int e = 0; e < 4; e++) h[e] = (_Float16)((ep.relu && v[e] < 0.f) ? 0.f : v[e]);
                    *reinterpret_cast<half4 *>(static_cast<_Float16 *>(ep.y) + o) = h;
                } else {
                    if (ep.residual) {
                        const floatx4 rs = *reinterpret_cast<const floatx4 *>(static_cast<const float *>(ep.residual) + o);
                        v += rs;
                    }
                    if (ep.relu) {
#pragma unroll
                        for (int e = 0; e < 4; e++) v[e] = v[e] < 0.f ? 0.f : v[e];
                    }
                    __builtin_nontemporal_store(v, reinterpret_cast<floatx4 *>(static_cast<float *>(ep.y) + o));
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    if (n + e >= N) break;
                    float f = v[e];
                    if (ep.y_f16) {
                        if (ep.residual) f += (float)static_cast<const _Float16 *>(ep.residual)[o + e];
                        if (ep.relu) f = f < 0.f ? 0.f : f;
                        static_cast<_Float16 *>(ep.y)[o + e] = (_Float16)f;
                    } else {
                        if (ep.residual) f += static_cast<const float *>(ep.residual)[o + e];
                        if (ep.relu) f = f < 0.f ? 0.f : f;
                        static_cast<float *>(ep.y)[o + e] = f;
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

#endif

}  // namespace tmq
