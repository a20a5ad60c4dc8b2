// Operand helpers shared by the MFMA attention kernels (gfx950, v_mfma_f32_16x16x32_{f16,bf16}).
//
// Register layouts relied upon (lane l of a 64-lane wavefront, li = l % 16, lq = l / 16):
//   A operand (16 x 32): row li, eight consecutive k-slots of group lq
//   B operand (32 x 16): column li, the same eight k-slots of group lq
//   C/D       (16 x 16): column li, rows 4*lq + r in register r (r = 0..3)
// Which logical index a k-slot stands for is free as long as A and B agree, and the C layout of
// a product whose rows are tokens is already the B layout of a product that contracts over
// tokens (lane (li, lq) holds tokens 4*lq + r): that is what lets P stay in its lanes.
#pragma once
#include "common.hpp"

namespace hs {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ half8 pack_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    u32x4 t = {a, b, c, d};
    return __builtin_bit_cast(half8, t);
}
__device__ __forceinline__ bf16x8 pack_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    u32x4 t = {a, b, c, d};
    return __builtin_bit_cast(bf16x8, t);
}

// Eight int8 codes (two dwords, byte order = k-slot order) -> eight fp16 holding code + 1152 exactly.
__device__ __forceinline__ half8 int8x8_to_f16_biased(uint32_t w0, uint32_t w1) {
    const uint32_t x0 = w0 ^ 0x80808080u, x1 = w1 ^ 0x80808080u;
    return pack_half8(__builtin_amdgcn_perm(0x64646464u, x0, 0x04010400u),
                      __builtin_amdgcn_perm(0x64646464u, x0, 0x04030402u),
                      __builtin_amdgcn_perm(0x64646464u, x1, 0x04010400u),
                      __builtin_amdgcn_perm(0x64646464u, x1, 0x04030402u));
}

// Byte `bsel` (0..3) of `lo` and of `hi` -> two fp16 holding the int8 codes exactly (offset removed).
__device__ __forceinline__ uint32_t int8_pair_to_f16(uint32_t lo, uint32_t hi, int bsel) {
    const uint32_t sel = 0x0c040c00u + (uint32_t)bsel + ((uint32_t)bsel << 16);
    const uint32_t w = __builtin_amdgcn_perm(hi, lo, sel) ^ 0x64806480u;
    const half2v hv = __builtin_bit_cast(half2v, w) - (half2v){(_Float16)1152.0f, (_Float16)1152.0f};
    return __builtin_bit_cast(uint32_t, hv);
}

// e4m3fn codes -> fp16.  A code shifted into bits 14..7 of a half (sign kept in bit 15) is the fp16 number
// value/256, subnormal codes included (fp16 subnormals have the same shape eight binades lower); the producer
// multiplies by 256 * scale afterwards.  `t` holds one code in the high byte of each half.
__device__ __forceinline__ uint32_t e4m3_high_bytes_to_f16(uint32_t t) {
    return (t & 0x80008000u) | ((t & 0x7f007f00u) >> 1);
}
// Eight e4m3fn codes (two dwords, byte order = k-slot order) -> eight fp16 holding value/256.
__device__ __forceinline__ half8 e4m3x8_to_f16_div256(uint32_t w0, uint32_t w1) {
    return pack_half8(e4m3_high_bytes_to_f16(__builtin_amdgcn_perm(0u, w0, 0x010c000cu)),
                      e4m3_high_bytes_to_f16(__builtin_amdgcn_perm(0u, w0, 0x030c020cu)),
                      e4m3_high_bytes_to_f16(__builtin_amdgcn_perm(0u, w1, 0x010c000cu)),
                      e4m3_high_bytes_to_f16(__builtin_amdgcn_perm(0u, w1, 0x030c020cu)));
}
// Byte `bsel` (0..3) of `lo` and of `hi` (e4m3fn codes) -> two fp16 holding value/256.
__device__ __forceinline__ uint32_t e4m3_pair_to_f16_div256(uint32_t lo, uint32_t hi, int bsel) {
    const uint32_t sel = ((4u + (uint32_t)bsel) << 24) | 0x000c000cu | ((uint32_t)bsel << 8);
    return e4m3_high_bytes_to_f16(__builtin_amdgcn_perm(hi, lo, sel));
}

// 16-bit half `hsel` (0 = low, 1 = high) of `lo` and of `hi` packed into one dword (lo first).
__device__ __forceinline__ uint32_t pick_halves(uint32_t lo, uint32_t hi, int hsel) {
    return __builtin_amdgcn_perm(hi, lo, hsel ? 0x07060302u : 0x05040100u);
}

// Reductions over the four lanes that share a column (li, li+16, li+32, li+48): two gfx950 lane-swap
// VALU instructions instead of LDS-crossbar shuffles.  v_permlane32_swap exchanges the upper half of
// its first operand with the lower half of the second; v_permlane16_swap does the same on 16-lane rows.
__device__ __forceinline__ float quad_max(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const float m = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const uint32_t v = __float_as_uint(m);
    const auto c = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    return fmaxf(__uint_as_float(c[0]), __uint_as_float(c[1]));
}
__device__ __forceinline__ float quad_sum(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const float m = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const uint32_t v = __float_as_uint(m);
    const auto c = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    return __uint_as_float(c[0]) + __uint_as_float(c[1]);
}

__device__ __forceinline__ uint32_t pack_f16x2(float a, float b) {
    half2v h = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, h);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    bf16x2 h = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(uint32_t, h);
}

}  // namespace hs
