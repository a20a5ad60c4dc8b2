// Device-side row quantizer shared by the quantize-on-write kernel and the decode-step prologue.
#pragma once
#include "common.hpp"

namespace hs {

// Per-head RMS normalisation of q / k ahead of the rotary embedding (kind 0 = none).
//   kind 1  LlamaAttention::apply_qk_norm (architectures/llama.rs:929-991, Gemma3): square, mean, + eps, reciprocal,
//           sqrt, x * rrms, * weight as separate ops in the tensor dtype (each result rounded to it; the scalar eps is
//           cast to the dtype first); weight in the tensor dtype.
//   kind 2  Qwen3_5Model::apply_qknorm (architectures/qwen3_5.rs:1077-1091): fp32, rrms = 1/sqrt(mean(x^2) + eps),
//           (x * rrms) * (1 + weight), one cast to the tensor dtype; weight fp32.
// weight is [H, D] (head_stride = D) or one [D] vector for all heads (head_stride = 0).
struct NormSpec {
    const void *weight = nullptr;
    int32_t kind = 0, head_stride = 0;
    float eps = 0.0f;
};

struct QuantArgs {
    const void *src[2];   // K, V  [B, S, Hkv, D]
    void *codes[2];
    float *scales[2];     // int8: written; fp8: read ([B, Hkv])
    KvAddr addr[2];
    const int32_t *positions;
    int32_t start_pos, B, S, Hkv, D, dtype;
    // optional rotary embedding of K before it is quantized: sin/cos tables [rope_len, D/2] in the source
    // dtype, row = the token's position; nullptr = K arrives rotated
    const void *rope_sin = nullptr, *rope_cos = nullptr;
    int32_t rope_len = 0;
    int32_t rotary_dim = 0;  // rotated leading part of each K row (pairs d, d + rotary_dim/2); 0 = the whole row
    NormSpec norm;           // optional QK-norm of K ahead of the rotation
};

// Round an fp32 value to the tensor dtype and back: libtorch's elementwise ops on bf16/fp16 tensors compute in
// fp32 and round the result of EVERY op to the tensor dtype.
__device__ __forceinline__ float round_to_dtype(float v, int dtype) {
    if (dtype == HS_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
    if (dtype == HS_F16) return (float)(_Float16)v;
    return v;
}

__device__ __forceinline__ float norm_square(float v, int dtype, int kind) {
#pragma clang fp contract(off)
    return kind == 1 ? round_to_dtype(v * v, dtype) : v * v;
}

// rrms of a row from the sum of its squares.  The sum is taken in double and rounded to fp32 once: squares of 16-bit
// values are exact in fp32 and their double sum is exact, so this is the correctly rounded fp32 sum whatever the order.
__device__ __forceinline__ float norm_rrms(double sumsq, int D, int dtype, int kind, float eps) {
#pragma clang fp contract(off)
    const float sum = (float)sumsq;
    if (kind == 1) {
        const float mean = round_to_dtype(sum / (float)D, dtype);
        const float t = round_to_dtype(mean + round_to_dtype(eps, dtype), dtype);
        const float rc = round_to_dtype(1.0f / t, dtype);
        return round_to_dtype(sqrtf(rc), dtype);
    }
    const float mean = sum / (float)D;
    return 1.0f / sqrtf(mean + eps);
}

__device__ __forceinline__ float norm_apply(float v, float w, float rrms, int dtype, int kind) {
#pragma clang fp contract(off)
    if (kind == 1) return round_to_dtype(round_to_dtype(v * rrms, dtype) * w, dtype);
    return round_to_dtype((v * rrms) * (w + 1.0f), dtype);
}

// E consecutive weights of head h starting at element d0, as fp32.
template <int E>
__device__ __forceinline__ void norm_weights(const NormSpec &n, int dtype, int h, int d0, float (&w)[E]) {
    load_src<E>(n.weight, n.kind == 1 ? dtype : HS_F32, (int64_t)h * n.head_stride + d0, w);
}

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Half-split rotary embedding of this lane's E consecutive elements (first element d0) of one head row:
//   d <  D/2 : x[d]*cos[d]       - x[d + D/2]*sin[d]
//   d >= D/2 : x[d - D/2]*sin[j] + x[d]*cos[j],  j = d - D/2
// as four products and two sums, each rounded to the tensor dtype (RoPE::apply_rotary_pos_emb,
// crates/hyprstream/src/runtime/rope.rs:206-248, with tables cast to the dtype, rope.rs:118-119).
// `src_row` = element index of the row's first element in `src`.
// With a QK-norm (norm != nullptr, x already normalised by the caller) the partner elements read from `src` are
// normalised here with the row's rrms and the weights of head `h`.
template <int E>
__device__ __forceinline__ void rope_rotate(const void *src, int dtype, int64_t src_row, int D, const void *sin_t,
                                            const void *cos_t, int rope_len, int pos, int d0, float (&x)[E],
                                            const NormSpec *norm = nullptr, float rrms = 0.0f, int h = 0) {
#pragma clang fp contract(off)
    const int half = D / 2;
    const bool upper = d0 >= half;
    const int j0 = upper ? d0 - half : d0;
    const int p = pos < 0 ? 0 : (pos >= rope_len ? rope_len - 1 : pos);
    float other[E], sn[E], cs[E];
    const int dother = upper ? d0 - half : d0 + half;
    load_src<E>(src, dtype, src_row + dother, other);
    if (norm != nullptr && norm->kind != 0) {
        float w[E];
        norm_weights<E>(*norm, dtype, h, dother, w);
#pragma unroll
        for (int e = 0; e < E; ++e) other[e] = norm_apply(other[e], w[e], rrms, dtype, norm->kind);
    }
    load_src<E>(sin_t, dtype, (int64_t)p * half + j0, sn);
    load_src<E>(cos_t, dtype, (int64_t)p * half + j0, cs);
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const float own_cos = round_to_dtype(x[e] * cs[e], dtype);
        const float other_sin = round_to_dtype(other[e] * sn[e], dtype);
        x[e] = round_to_dtype(upper ? other_sin + own_cos : own_cos - other_sin, dtype);
    }
}

__device__ __forceinline__ uint32_t f32_to_e4m3fn_bits(float y) {
#pragma clang fp contract(off)
    uint32_t u = __float_as_uint(y);
    uint32_t sign = (u >> 24) & 0x80u;
    u &= 0x7fffffffu;
    if (u >= 0x43f00000u) return sign | 0x7fu;  // >= 480, inf, NaN
    float a = __uint_as_float(u);
    uint32_t r;
    if (a < 0.015625f) {
        r = (uint32_t)rintf(a * 512.0f);  // subnormal grid 2^-9; 8 == smallest normal
    } else {
        r = (u + 0x7ffffu + ((u >> 20) & 1u)) >> 20;  // RNE on the 3 kept mantissa bits
        r -= (120u << 3);                              // rebias 127 -> 7
        if (r > 0x7fu) r = 0x7fu;
    }
    return sign | r;
}

// One wavefront quantizes row `row` (= (b*S + s)*Hkv + h) of tensor `which` (0 = K, 1 = V).
template <int E, bool FP8>
__device__ __forceinline__ void quantize_row(const QuantArgs &a, int which, int64_t row, int lane) {
#pragma clang fp contract(off)  // exactly the fp32 operations written: bit-exact with the CPU oracle
    const int h = (int)(row % a.Hkv);
    const int64_t bs = row / a.Hkv;
    const int s = (int)(bs % a.S);
    const int b = (int)(bs / a.S);
    const int pos = (a.positions ? a.positions[b] : 0) + a.start_pos + s;
    const KvAddr &ad = a.addr[which];
    int64_t unit;
    int slot;
    if (!resolve(ad, b, pos, unit, slot)) return;

    float x[E];
    load_src<E>(a.src[which], a.dtype, row * a.D + lane * E, x);
    if (which == 0) {
        float rrms = 0.0f;
        if (a.norm.kind != 0) {  // QK-norm of the K row, then the rotation of the normalised row
            double ss = 0.0;
#pragma unroll
            for (int e = 0; e < E; ++e) ss += (double)norm_square(x[e], a.dtype, a.norm.kind);
            rrms = norm_rrms(wave_sum_f64(ss), a.D, a.dtype, a.norm.kind, a.norm.eps);
            float w[E];
            norm_weights<E>(a.norm, a.dtype, h, lane * E, w);
#pragma unroll
            for (int e = 0; e < E; ++e) x[e] = norm_apply(x[e], w[e], rrms, a.dtype, a.norm.kind);
        }
        const int rd = a.rotary_dim > 0 ? a.rotary_dim : a.D;
        if (a.rope_sin != nullptr && lane * E < rd)
            rope_rotate<E>(a.src[0], a.dtype, row * a.D, rd, a.rope_sin, a.rope_cos, a.rope_len, pos, lane * E, x, &a.norm, rrms, h);
    }

    uint8_t *dst = (uint8_t *)a.codes[which] + unit * ad.code_stride_seq + (int64_t)h * ad.code_stride_head +
                   (int64_t)slot * a.D + lane * E;
    uint32_t packed = 0;
    if (!FP8) {
        float m = 0.0f;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float v = fabsf(x[e]);
            m = v > m ? v : m;
        }
        m = wave_max(m);
        float sc = 0.0f;
        if (m > 0.0f) {
            sc = m / 127.0f;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                float q = rintf(x[e] / sc);
                q = q > 127.0f ? 127.0f : q;
                q = q < -127.0f ? -127.0f : q;
                if (q != q) q = 0.0f;
                packed |= ((uint32_t)(int)q & 0xffu) << (8 * e);
            }
        }
        if (lane == 0) a.scales[which][unit * ad.scale_stride_seq + (int64_t)h * ad.scale_stride_head + slot] = sc;
    } else {
        const float sc = a.scales[which][(int64_t)b * a.Hkv + h];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float y = 0.0f;
            if (sc > 0.0f) {
                y = x[e] / sc;
                if (y > 448.0f) y = 448.0f;
                if (y < -448.0f) y = -448.0f;
            }
            packed |= f32_to_e4m3fn_bits(y) << (8 * e);
        }
    }
    if (E == 4) *(uint32_t *)dst = packed;
    else if (E == 2) *(uint16_t *)dst = (uint16_t)packed;
    else *dst = (uint8_t)packed;
}

}  // namespace hs
