// MFMA helpers and the kernel-native weight layout shared by the ternary linear / conv kernels.
//
// Native layout ("n16k256"): the weight matrix T[k][n] is cut into blocks of 16 output channels
// x 256 reduction indices. A block is 1 KiB: 64 lanes x one dwordx4, stored in lane order, so a
// wavefront fetches a block with a single fully coalesced load and every lane receives exactly
// the bits its own MFMA operand needs -- no LDS, no shuffles, no lane-dependent selects.
//
//   block index   = nb * Kb + kb            (nb = n / 16, kb = k / 256, Kb = ceil(K / 256))
//   lane l        : n = 16 nb + (l % 16), g = l / 16
//   dword d (0..3): k in [256 kb + 64 d, 256 kb + 64 d + 64)
//   inside a dword: two MFMA steps s (32 k each); step s, element e (0..7) is
//                   k = 256 kb + 64 d + 32 s + 8 g + e, the operand layout of
//                   v_mfma_f32_16x16x32_f16 (lane (i, g) holds k = 8g .. 8g+7 of row/col i).
//   bit position  : field f = 4 s + e / 2; even e in the low half-word, odd e in the high one,
//                   fields MSB first: bits [15 - 2f : 14 - 2f] (+16 for odd e).
//   field         : (sign, nonzero): 0 -> 00, +1 -> 01, -1 -> 11.
//
// Decoding an operand register pair is then `(word << 2f) & 0xC000C000`: both half-words become
// the fp16 numbers +-2.0 (0x4000 / 0xC000) or 0. The factor 2 is exact and is folded into the
// epilogue scale. Products x * (+-2) and the fp32 accumulation inside the MFMA are exact /
// fp32-rounded, so results equal an fp32-accumulated product with the +-1/0 weights.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tmq {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kNB = 16;     // output channels per native block
constexpr int kKB = 256;    // reduction indices per native block
constexpr float kWeightUnit = 2.0f;   // decoded magnitude

inline int64_t native_blocks_n(int64_t N) { return (N + kNB - 1) / kNB; }
inline int64_t native_blocks_k(int64_t K) { return (K + kKB - 1) / kKB; }

#if defined(__HIPCC__)

// Operand registers (8 fp16 = 4 dwords) of step s from one native dword.
__device__ __forceinline__ half8 decode_step(uint32_t word, int s) {
    u32x4 r;
    r[0] = (word << (8 * s + 0)) & 0xC000C000u;
    r[1] = (word << (8 * s + 2)) & 0xC000C000u;
    r[2] = (word << (8 * s + 4)) & 0xC000C000u;
    r[3] = (word << (8 * s + 6)) & 0xC000C000u;
    return __builtin_bit_cast(half8, r);
}

// D += A * B, A: 16 x 32 (lane (i, g) holds A[i][8g..8g+7]), B: 32 x 16 (lane (j, g) holds
// B[8g..8g+7][j]), D: 16 x 16 fp32 (lane (j, g) holds D[4g..4g+3][j]).
__device__ __forceinline__ floatx4 mfma16(half8 a, half8 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

#endif

}  // namespace tmq
