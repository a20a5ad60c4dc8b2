// QK-norm + rotary embedding of bf16 rows with a lane working on a long piece of a row: shared by the pre-pass kernel
// over whole tensors and by the prefill launch that runs the q side itself.
#pragma once
#include "mfma_common.hpp"
#include "quant_device.hpp"

namespace hs {

// One side (q or k) of an hs_qk_prologue as the kernels take it.
struct RowPrologue {
    NormSpec norm;                                  // kind 0: no QK-norm
    const void *sin_t = nullptr, *cos_t = nullptr;  // bf16 [rope_len, rd / 2]; nullptr: no rotation
    int32_t rope_len = 0, rd = 0;
    int32_t on = 0;
};

// The rotary_dim values prologue_row_part serves for pieces of E elements: whole pieces on either side of the rotation's
// halves (the partner is another lane's piece), or the rotated part is exactly one piece (both halves in the lane).
__host__ __device__ inline bool prologue_parts_serve(int rd, int E) { return rd == E || (rd / 2) % E == 0; }

// N consecutive bf16 values (N a multiple of 8) from a 16-byte aligned address, as fp32.
template <int N>
__device__ __forceinline__ void load_bf16_row(const uint16_t *p, float (&x)[N]) {
#pragma unroll
    for (int i = 0; i < N / 8; ++i) {
        const u32x4 w = *(const u32x4 *)(p + 8 * i);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            x[8 * i + 2 * e] = __uint_as_float(w[e] << 16);
            x[8 * i + 2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
        }
    }
}

// Two fp32 values rounded to bf16 and widened again: one conversion instruction for the pair, then a shift and a mask.
__device__ __forceinline__ void round2_bf16(float &a, float &b) {
    const uint32_t r = pack_bf16x2(a, b);
    a = __uint_as_float(r << 16);
    b = __uint_as_float(r & 0xffff0000u);
}

// QK-norm and rotary embedding of piece `part` (E consecutive elements from d0 = E part) of the bf16 row at `src`; the
// D/E lanes lane0 + LS part of the wavefront hold the row's pieces and all of them make this call together.  The
// operations and roundings are those of the one-row-per-wavefront kernel (norm_square / norm_rrms / norm_apply, then
// rope_rotate's three rounded operations): the same bits.  With 32 elements to a lane the per-row work (position, the
// reciprocal root's chain of roundings, the reduction of the sum over the row's lanes) is paid once per 32 elements, the
// inputs arrive through 16-byte loads, the rotation's partner elements come normalised from the lane that holds them,
// and values are rounded two at a time.  The lower half's "own cos - other sin" is computed as own cos + other (-sin)
// with the sign flipped on the packed table words: rounding is symmetric, so the bits are the same.
// p.rd must pass prologue_parts_serve(rd, E).  Result: the piece as packed bf16 pairs.
template <int D, int E>
__device__ __forceinline__ void prologue_row_part(const RowPrologue &p, const uint16_t *src, int head, int pos, int part,
                                                  int LS, int lane, u32x4 (&res)[E / 8]) {
#pragma clang fp contract(off)
    constexpr int P = D / E;
    const int d0 = E * part;
    const int kind = p.norm.kind;
    float x[E];
    load_bf16_row<E>(src + d0, x);
    if (kind != 0) {
        double ss = 0.0;
        if (kind == 1) {
#pragma unroll
            for (int e = 0; e < E; e += 2) {
                float s0 = x[e] * x[e], s1 = x[e + 1] * x[e + 1];
                round2_bf16(s0, s1);
                ss += (double)s0;
                ss += (double)s1;
            }
        } else {
#pragma unroll
            for (int e = 0; e < E; ++e) ss += (double)(x[e] * x[e]);
        }
#pragma unroll
        for (int o = 1; o < P; o <<= 1) ss += __shfl_xor(ss, o * LS, 64);
        const float rrms = norm_rrms(ss, D, HS_BF16, kind, p.norm.eps);
        float w[E];
        const int64_t w0 = (int64_t)head * p.norm.head_stride + d0;
        if (kind == 1) {
            load_bf16_row<E>((const uint16_t *)p.norm.weight + w0, w);
#pragma unroll
            for (int e = 0; e < E; e += 2) {
                float a0 = x[e] * rrms, a1 = x[e + 1] * rrms;
                round2_bf16(a0, a1);
                a0 = a0 * w[e];
                a1 = a1 * w[e + 1];
                round2_bf16(a0, a1);
                x[e] = a0;
                x[e + 1] = a1;
            }
        } else {
#pragma unroll
            for (int i = 0; i < E / 4; ++i) {
                const float4v t = *(const float4v *)((const float *)p.norm.weight + w0 + 4 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) w[4 * i + e] = t[e];
            }
#pragma unroll
            for (int e = 0; e < E; e += 2) {
                float a0 = (x[e] * rrms) * (w[e] + 1.0f), a1 = (x[e + 1] * rrms) * (w[e + 1] + 1.0f);
                round2_bf16(a0, a1);
                x[e] = a0;
                x[e + 1] = a1;
            }
        }
    }
    bool packed = false;
    if (p.sin_t != nullptr && d0 < p.rd) {
        const int half = p.rd / 2;
        const int pp = pos < 0 ? 0 : (pos >= p.rope_len ? p.rope_len - 1 : pos);
        const uint16_t *sin_row = (const uint16_t *)p.sin_t + (int64_t)pp * half;
        const uint16_t *cos_row = (const uint16_t *)p.cos_t + (int64_t)pp * half;
        if (half >= E) {  // the partner elements d +- rd/2 are another lane's piece, half/E pieces away
            const bool upper = d0 >= half;
            const int j0 = upper ? d0 - half : d0;
            const int partner = upper ? lane - half / E * LS : lane + half / E * LS;
            const uint32_t flip = upper ? 0u : 0x80008000u;  // the lower half subtracts the sine term
#pragma unroll
            for (int i = 0; i < E / 8; ++i) {
                const u32x4 sw = *(const u32x4 *)(sin_row + j0 + 8 * i), cw = *(const u32x4 *)(cos_row + j0 + 8 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int k = 8 * i + 2 * e;
                    const uint32_t sv = sw[e] ^ flip;
                    float own0 = x[k] * __uint_as_float(cw[e] << 16), own1 = x[k + 1] * __uint_as_float(cw[e] & 0xffff0000u);
                    float oth0 = __shfl(x[k], partner, 64) * __uint_as_float(sv << 16);
                    float oth1 = __shfl(x[k + 1], partner, 64) * __uint_as_float(sv & 0xffff0000u);
                    round2_bf16(own0, own1);
                    round2_bf16(oth0, oth1);
                    res[i][e] = pack_bf16x2(own0 + oth0, own1 + oth1);
                }
            }
            packed = true;
        } else {  // rd = E: both halves of the rotated part are this lane's
#pragma unroll
            for (int i = 0; i < E / 16; ++i) {
                const u32x4 sw = *(const u32x4 *)(sin_row + 8 * i), cw = *(const u32x4 *)(cos_row + 8 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int k = 8 * i + 2 * e;
                    const float s0 = __uint_as_float(sw[e] << 16), s1 = __uint_as_float(sw[e] & 0xffff0000u);
                    const float c0 = __uint_as_float(cw[e] << 16), c1 = __uint_as_float(cw[e] & 0xffff0000u);
                    const float lo0 = x[k], lo1 = x[k + 1], hi0 = x[E / 2 + k], hi1 = x[E / 2 + k + 1];
                    float lc0 = lo0 * c0, lc1 = lo1 * c1, hs0 = hi0 * s0, hs1 = hi1 * s1;
                    float ls0 = lo0 * s0, ls1 = lo1 * s1, hc0 = hi0 * c0, hc1 = hi1 * c1;
                    round2_bf16(lc0, lc1);
                    round2_bf16(hs0, hs1);
                    round2_bf16(ls0, ls1);
                    round2_bf16(hc0, hc1);
                    x[k] = lc0 - hs0;        // rounded by the packing below
                    x[k + 1] = lc1 - hs1;
                    x[E / 2 + k] = ls0 + hc0;
                    x[E / 2 + k + 1] = ls1 + hc1;
                }
            }
        }
    }
    if (!packed) {
#pragma unroll
        for (int i = 0; i < E / 8; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) res[i][e] = pack_bf16x2(x[8 * i + 2 * e], x[8 * i + 2 * e + 1]);
    }
}

}  // namespace hs
