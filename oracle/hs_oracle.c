/*
 * hs_oracle.c -- CPU restatement of hyprstream's quantized-KV attention path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this file: it is the checker that the parity tests, the smoke test
 * and the CPU-baseline leg of the benchmark compare the HIP kernels against.
 * It is written for clarity (plain loops, double accumulation), not speed.
 *
 * What each function restates (paths relative to the reference checkout):
 *
 *  - orc_quant_int8_*        symmetric absmax int8 on one (token, kv-head) row.
 *                            The reference's int8 grid is the linear codebook
 *                            code[i] = (i-127)/127 with an fp32 absmax per block
 *                            (crates/bitsandbytes-sys/src/lib.rs:104-121, call
 *                            sites crates/hyprstream/src/runtime/kv_cache.rs:
 *                            797-840); here the block is the head_dim row, the
 *                            stored index is i-127 as int8 and the stored scale
 *                            is absmax/127.  Arithmetic order (all fp32, IEEE):
 *                              a = max_d |x_d| ; s = a / 127 ;
 *                              q_d = clamp(rint(x_d / s), -127, 127)   (RNE)
 *                            all-zero row: s = 0, q = 0.
 *                            Pinned by: golden vectors made with libtorch CPU
 *                            ops (amax, div, round), brute-force nearest-code
 *                            search on tiny inputs, and invariants (tests/).
 *  - orc_fp8_e4m3fn_*        OCP e4m3fn conversion (round-to-nearest-even,
 *                            subnormals below 2^-6, |x| >= 464-rounding-up and
 *                            NaN -> 0x7f), the algorithm libtorch applies for
 *                            Tensor.to(float8_e4m3fn).  Pinned exhaustively
 *                            against libtorch over all 2^16 bf16 inputs and
 *                            every one of the 256 codes (tests/).
 *  - orc_quant_fp8_*         x -> e4m3fn(clamp(x / s, +-448)) with one fp32 scale
 *                            per (sequence, kv-head); s = amax/448 from
 *                            orc_fp8_calibrate.  New format (the reference has
 *                            no FP8 KV cache), pinned as above.
 *  - orc_decode_attn         softmax(q K^T * scale) V for one query token per
 *                            sequence over the dequantized cache, GQA mapping
 *                            q-head h -> kv-head h / (Hq/Hkv)
 *                            (architectures/llama.rs:847-872, 1023-1119;
 *                            qwen3_5.rs:1001-1053), ragged lengths as in the
 *                            batched mask rule (llama.rs:2544-2572).  Double
 *                            accumulation.
 *  - orc_prefill_attn        the same with S query rows and the causal rule
 *                            "query row i sits at absolute position
 *                            (k_len - q_len) + i" (llama.rs:1074-1084).
 *  - orc_prefill_attn_window the same with the sliding window of local layers
 *                            (apply_sliding_window_mask, llama.rs:1086-1091,
 *                            1123-1155): valid = causal AND i - j < window.  The
 *                            reference builds that mask as [q_len, q_len] and adds it
 *                            to the [q_len, k_len] scores, which has a meaning only
 *                            for a prompt on an empty cache (k_len == q_len; at
 *                            q_len == 1 the mask is a single zero, i.e. decode is
 *                            NOT windowed there).  With history the restatement
 *                            uses absolute positions: query p attends keys in
 *                            (p - window, p].  Pinned by golden vectors of the
 *                            libtorch op sequence for the empty-cache case, by
 *                            window >= length == no window, window 1 == own V row,
 *                            and by a brute-force restriction of the keys
 *                            (tests/test_oracle_attention.py).
 *  - orc_deltanet_recurrent  the gated delta rule, one token at a time
 *                            (qwen3_5.rs:725-751), with the L2 normalisation
 *                            x / max(||x||, 1e-3) (qwen3_5.rs:331-335) and the
 *                            k/q-head -> v-head expansion (qwen3_5.rs:704-720).
 *  - orc_rope_apply_*        rotary embedding in the half-split convention,
 *                            x1' = x1*cos - x2*sin, x2' = x1*sin + x2*cos with
 *                            x1 = x[..., :D/2], x2 = x[..., D/2:]
 *                            (crates/hyprstream/src/runtime/rope.rs:206-248).
 *                            The tables are fp32 values cast to the tensor dtype
 *                            (rope.rs:100-122) and the four products and two
 *                            sums are separate libtorch ops in that dtype, so a
 *                            bf16 tensor is rounded to bf16 after EVERY op; the
 *                            restatement does exactly that.  Pinned by golden
 *                            vectors and a live comparison with libtorch CPU ops
 *                            on bf16/fp32 tensors, identity at position 0, norm
 *                            preservation and the relative-position property
 *                            (tests/test_oracle_rope.py).
 *  - orc_deltanet_prepare    what GatedDeltaNetLayer::forward does between the input
 *                            projection and the delta rule (qwen3_5.rs:617-720):
 *                            depthwise causal conv1d (kernel 4, the 3 frames before
 *                            the call carried as state) + SiLU on the mixed q|k|v
 *                            channels in the model dtype, g = -exp(A_log) *
 *                            softplus(a + dt_bias) and beta = sigmoid(b) in fp32.
 *                            The conv accumulates in fp32 in tap order and rounds
 *                            once to bf16; libtorch's bf16 conv1d does not promise an
 *                            accumulation order, so parity with it is to one bf16 ulp,
 *                            not to the bit (tests/test_oracle_deltanet_glue.py).
 *  - orc_gated_rmsnorm       RMSNormGated::forward (qwen3_5.rs:292-313):
 *                            x * rsqrt(mean(x^2) + eps) * w * silu(z) in fp32.
 *
 * parity unpinned: the reference's own int8 format (bitsandbytes 0.45.0
 * blockwise-64 codes, tie-breaking of its binary search) is not restated here
 * because bitsandbytes is neither vendored in the reference nor installed.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* ---------------------------------------------------------------- helpers */

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* fp32 -> bf16, round-to-nearest-even, NaN kept quiet (what libtorch does). */
ORC_API uint16_t orc_f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

ORC_API void orc_f32_to_bf16_array(const float *x, int64_t n, uint16_t *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(x[i]);
}

ORC_API void orc_bf16_to_f32_array(const uint16_t *x, int64_t n, float *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = bf16_to_f32(x[i]);
}

/* ------------------------------------------------------ int8 quantization */

static void quant_row_int8(const float *x, int D, int8_t *codes, float *scale) {
    float a = 0.0f;
    for (int d = 0; d < D; ++d) {
        float v = fabsf(x[d]);
        if (v > a) a = v; /* NaN never wins: matches a max that ignores NaN lanes */
    }
    if (!(a > 0.0f)) {
        *scale = 0.0f;
        memset(codes, 0, (size_t)D);
        return;
    }
    volatile float s = a / 127.0f; /* volatile: forbid x87/fma contraction games */
    *scale = s;
    for (int d = 0; d < D; ++d) {
        volatile float r = x[d] / s;
        float q = rintf(r); /* FE_TONEAREST: ties to even, same as torch.round */
        if (q > 127.0f) q = 127.0f;
        if (q < -127.0f) q = -127.0f;
        if (q != q) q = 0.0f;
        codes[d] = (int8_t)q;
    }
}

/* x: [rows, D] fp32, codes: [rows, D], scales: [rows]. */
ORC_API void orc_quant_int8_f32(const float *x, int64_t rows, int D, int8_t *codes, float *scales) {
    for (int64_t r = 0; r < rows; ++r) quant_row_int8(x + r * D, D, codes + r * D, scales + r);
}

/* bf16 source: widened exactly to fp32 first. */
ORC_API void orc_quant_int8_bf16(const uint16_t *x, int64_t rows, int D, int8_t *codes, float *scales) {
    float *tmp = (float *)malloc(sizeof(float) * (size_t)D);
    for (int64_t r = 0; r < rows; ++r) {
        for (int d = 0; d < D; ++d) tmp[d] = bf16_to_f32(x[r * D + d]);
        quant_row_int8(tmp, D, codes + r * D, scales + r);
    }
    free(tmp);
}

ORC_API void orc_dequant_int8(const int8_t *codes, const float *scales, int64_t rows, int D, float *out) {
    for (int64_t r = 0; r < rows; ++r)
        for (int d = 0; d < D; ++d) out[r * D + d] = scales[r] * (float)codes[r * D + d];
}

/* ------------------------------------------------------- fp8 e4m3fn codec */

/* Decode: sign | 4-bit exponent (bias 7) | 3-bit mantissa; no infinities,
 * 0x7f / 0xff are NaN, exponent 0 is subnormal (2^-6 * m/8). */
ORC_API float orc_fp8_e4m3fn_to_f32(uint8_t b) {
    int sign = b >> 7, e = (b >> 3) & 0xf, m = b & 7;
    float v;
    if (e == 0xf && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return sign ? -v : v;
}

/* Encode with round-to-nearest-even on the 3-bit mantissa.  Magnitudes that
 * round to or beyond 480 (the bit pattern of NaN) and NaN inputs give 0x7f. */
ORC_API uint8_t orc_fp8_e4m3fn_from_f32(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    u &= 0x7fffffffu;
    if (u >= 0x43f00000u) return (uint8_t)(sign | 0x7f); /* |x| >= 480, inf, NaN */
    float a;
    memcpy(&a, &u, 4);
    uint8_t r;
    if (a < 0.015625f) {
        /* subnormal target: spacing 2^-9; rint is RNE in the default mode and
         * a * 512 is exact (power-of-two scaling of a value far above fp32's
         * own subnormal range, or exactly representable below it). */
        float k = rintf(a * 512.0f);
        r = (uint8_t)k; /* 0..8 ; 8 == 0x08 == smallest normal 2^-6 */
    } else {
        int e;
        float f = frexpf(a, &e);          /* a = f * 2^e, f in [0.5, 1) */
        float m = rintf(f * 16.0f);       /* 8..16 : 1.mmm scaled by 8 */
        int ee = e - 1;                   /* exponent of the leading one */
        if (m == 16.0f) { m = 8.0f; ee += 1; }
        int be = ee + 7;
        int v = (be << 3) | ((int)m - 8);
        if (v >= 0x7f) v = 0x7f;          /* rounded up into the NaN pattern */
        r = (uint8_t)v;
    }
    return (uint8_t)(sign | r);
}

ORC_API void orc_fp8_encode_array(const float *x, int64_t n, uint8_t *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_fp8_e4m3fn_from_f32(x[i]);
}

ORC_API void orc_fp8_decode_array(const uint8_t *x, int64_t n, float *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_fp8_e4m3fn_to_f32(x[i]);
}

/* x: [B, S, H, D] fp32.  scales[b, h] = max over (s, d) |x| / 448. */
ORC_API void orc_fp8_calibrate(const float *x, int B, int S, int H, int D, float *scales) {
    for (int b = 0; b < B; ++b)
        for (int h = 0; h < H; ++h) {
            float a = 0.0f;
            for (int s = 0; s < S; ++s) {
                const float *row = x + (((int64_t)b * S + s) * H + h) * D;
                for (int d = 0; d < D; ++d) {
                    float v = fabsf(row[d]);
                    if (v > a) a = v;
                }
            }
            volatile float sc = a / 448.0f;
            scales[b * H + h] = sc;
        }
}

/* x: [B, S, H, D] fp32, scales: [B, H], codes: [B, S, H, D]. */
ORC_API void orc_quant_fp8_f32(const float *x, const float *scales, int B, int S, int H, int D, uint8_t *codes) {
    for (int b = 0; b < B; ++b)
        for (int s = 0; s < S; ++s)
            for (int h = 0; h < H; ++h) {
                int64_t off = (((int64_t)b * S + s) * H + h) * D;
                float sc = scales[b * H + h];
                for (int d = 0; d < D; ++d) {
                    float y;
                    if (!(sc > 0.0f)) y = 0.0f;
                    else {
                        volatile float t = x[off + d] / sc;
                        y = t;
                        if (y > 448.0f) y = 448.0f;
                        if (y < -448.0f) y = -448.0f;
                    }
                    codes[off + d] = orc_fp8_e4m3fn_from_f32(y);
                }
            }
}

/* ------------------------------------------------------------- attention */

/* Dequantized element of the canonical cache layout [B, T, Hkv, D].
 * fmt 0: int8 codes, scales [B, T, Hkv].  fmt 1: e4m3fn codes, scales [B, Hkv].
 * fmt 2: dense fp32 values (codes points at float), scales unused. */
static inline double kv_at(const void *codes, const float *scales, int fmt, int T, int Hkv, int D,
                           int b, int t, int h, int d) {
    int64_t row = ((int64_t)b * T + t) * Hkv + h;
    if (fmt == 0) return (double)scales[row] * (double)((const int8_t *)codes)[row * D + d];
    if (fmt == 1)
        return (double)scales[b * Hkv + h] *
               (double)orc_fp8_e4m3fn_to_f32(((const uint8_t *)codes)[row * D + d]);
    return (double)((const float *)codes)[row * D + d];
}

/*
 * q:   [B, S, Hq, D] fp32 (bf16 values widened by the caller)
 * k/v: canonical layout [B, Tcap, Hkv, D] (see kv_at)
 * kv_lens[b]: number of valid cached tokens of row b (including the S new ones)
 * Query row i of sequence b sits at absolute position kv_lens[b] - S + i and
 * attends keys 0..=that position.  out: [B, S, Hq, D] fp32.
 * A row whose kv_len is 0 (or < S) yields zeros.
 */
ORC_API void orc_prefill_attn_window(const float *q, const void *kc, const void *vc, const float *ks, const float *vs,
                                     int fmt, const int32_t *kv_lens, int B, int S, int Hq, int Hkv, int D, int Tcap,
                                     float softmax_scale, int window, float *out) {
    int G = Hq / Hkv;
    double *p = (double *)malloc(sizeof(double) * (size_t)(Tcap > 0 ? Tcap : 1));
    double *acc = (double *)malloc(sizeof(double) * (size_t)D);
    for (int b = 0; b < B; ++b) {
        int L = kv_lens[b];
        for (int i = 0; i < S; ++i)
            for (int hq = 0; hq < Hq; ++hq) {
                float *o = out + (((int64_t)b * S + i) * Hq + hq) * D;
                int last = L - S + i; /* inclusive */
                if (L <= 0 || last < 0) {
                    memset(o, 0, sizeof(float) * (size_t)D);
                    continue;
                }
                int h = hq / G;
                const float *qr = q + (((int64_t)b * S + i) * Hq + hq) * D;
                double mx = -INFINITY;
                /* window > 0: keys at distance >= window from the query's position are masked out */
                int first = (window > 0 && last - window + 1 > 0) ? last - window + 1 : 0;
                for (int t = first; t <= last; ++t) {
                    double s = 0.0;
                    for (int d = 0; d < D; ++d) s += (double)qr[d] * kv_at(kc, ks, fmt, Tcap, Hkv, D, b, t, h, d);
                    s *= (double)softmax_scale;
                    p[t] = s;
                    if (s > mx) mx = s;
                }
                double l = 0.0;
                for (int t = first; t <= last; ++t) {
                    p[t] = exp(p[t] - mx);
                    l += p[t];
                }
                for (int d = 0; d < D; ++d) acc[d] = 0.0;
                for (int t = first; t <= last; ++t) {
                    double w = p[t];
                    for (int d = 0; d < D; ++d) acc[d] += w * kv_at(vc, vs, fmt, Tcap, Hkv, D, b, t, h, d);
                }
                for (int d = 0; d < D; ++d) o[d] = (float)(acc[d] / l);
            }
    }
    free(p);
    free(acc);
}

ORC_API void orc_prefill_attn(const float *q, const void *kc, const void *vc, const float *ks, const float *vs,
                              int fmt, const int32_t *kv_lens, int B, int S, int Hq, int Hkv, int D, int Tcap,
                              float softmax_scale, float *out) {
    orc_prefill_attn_window(q, kc, vc, ks, vs, fmt, kv_lens, B, S, Hq, Hkv, D, Tcap, softmax_scale, 0, out);
}

/* Decode = prefill with one query row per sequence. q, out: [B, Hq, D]. */
ORC_API void orc_decode_attn(const float *q, const void *kc, const void *vc, const float *ks, const float *vs,
                             int fmt, const int32_t *seq_lens, int B, int Hq, int Hkv, int D, int Tcap,
                             float softmax_scale, float *out) {
    orc_prefill_attn(q, kc, vc, ks, vs, fmt, seq_lens, B, 1, Hq, Hkv, D, Tcap, softmax_scale, out);
}

/* --------------------------------------------------------------- DeltaNet */

/*
 * q, k: [B, T, nk, dk] fp32;  v: [B, T, nv, dv];  g, beta: [B, T, nv];
 * state: [B, nv, dk, dv] fp32, read as the initial state and overwritten with
 * the final one;  out: [B, T, nv, dv] fp32.
 * v-head j uses q/k-head j / (nv/nk).  With l2norm != 0, q and k are replaced
 * by x / max(||x||_2, 1e-3) first; q is then multiplied by q_scale.
 * Per token:  S *= exp(g);  m = k^T S;  delta = (v - m) * beta;
 *             S += k (x) delta;  o = q^T S.
 */
ORC_API void orc_deltanet_recurrent(const float *q, const float *k, const float *v, const float *g,
                                    const float *beta, float *state, int B, int T, int nk, int nv, int dk,
                                    int dv, float q_scale, int l2norm, float *out) {
    int rep = nv / nk;
    double *S = (double *)malloc(sizeof(double) * (size_t)dk * dv);
    double *qq = (double *)malloc(sizeof(double) * (size_t)dk);
    double *kk = (double *)malloc(sizeof(double) * (size_t)dk);
    double *m = (double *)malloc(sizeof(double) * (size_t)dv);
    for (int b = 0; b < B; ++b)
        for (int j = 0; j < nv; ++j) {
            float *st = state + ((int64_t)b * nv + j) * dk * dv;
            for (int i = 0; i < dk * dv; ++i) S[i] = st[i];
            int hk = j / rep;
            for (int t = 0; t < T; ++t) {
                const float *qr = q + (((int64_t)b * T + t) * nk + hk) * dk;
                const float *kr = k + (((int64_t)b * T + t) * nk + hk) * dk;
                const float *vr = v + (((int64_t)b * T + t) * nv + j) * dv;
                double gt = g[((int64_t)b * T + t) * nv + j];
                double bt = beta[((int64_t)b * T + t) * nv + j];
                double qn = 1.0, kn = 1.0;
                if (l2norm) {
                    double sq = 0, sk = 0;
                    for (int i = 0; i < dk; ++i) { sq += (double)qr[i] * qr[i]; sk += (double)kr[i] * kr[i]; }
                    qn = sqrt(sq); kn = sqrt(sk);
                    if (qn < 1e-3) qn = 1e-3;
                    if (kn < 1e-3) kn = 1e-3;
                }
                for (int i = 0; i < dk; ++i) { qq[i] = (double)qr[i] / qn * (double)q_scale; kk[i] = (double)kr[i] / kn; }
                double decay = exp(gt);
                for (int c = 0; c < dv; ++c) m[c] = 0.0;
                for (int i = 0; i < dk; ++i)
                    for (int c = 0; c < dv; ++c) {
                        S[i * dv + c] *= decay;
                        m[c] += kk[i] * S[i * dv + c];
                    }
                for (int c = 0; c < dv; ++c) m[c] = ((double)vr[c] - m[c]) * bt; /* delta */
                float *o = out + (((int64_t)b * T + t) * nv + j) * dv;
                for (int c = 0; c < dv; ++c) {
                    double acc = 0.0;
                    for (int i = 0; i < dk; ++i) {
                        S[i * dv + c] += kk[i] * m[c];
                        acc += qq[i] * S[i * dv + c];
                    }
                    o[c] = (float)acc;
                }
            }
            for (int i = 0; i < dk * dv; ++i) st[i] = (float)S[i];
        }
    free(S); free(qq); free(kk); free(m);
}

/* --------------------------------------------------------------------- RoPE */

static inline float rbf(float f) { return bf16_to_f32(orc_f32_to_bf16(f)); }

/* x, out: bf16 bit patterns [rows, H, D] with rows = B*S; sin/cos: bf16 bit patterns [table_len, D/2];
 * pos[rows]: table row of each token.  Every product and every sum is rounded to bf16 (see the header). */
ORC_API void orc_rope_apply_bf16(const uint16_t *x, const uint16_t *sin_t, const uint16_t *cos_t, const int32_t *pos,
                                 int64_t rows, int H, int D, uint16_t *out) {
    const int half = D / 2;
    for (int64_t r = 0; r < rows; ++r) {
        const uint16_t *st = sin_t + (int64_t)pos[r] * half, *ct = cos_t + (int64_t)pos[r] * half;
        for (int h = 0; h < H; ++h) {
            const uint16_t *xi = x + (r * H + h) * D;
            uint16_t *oi = out + (r * H + h) * D;
            for (int d = 0; d < half; ++d) {
                const float x1 = bf16_to_f32(xi[d]), x2 = bf16_to_f32(xi[d + half]);
                const float c = bf16_to_f32(ct[d]), s = bf16_to_f32(st[d]);
                const volatile float a = rbf(x1 * c), b = rbf(x2 * s), e = rbf(x1 * s), f = rbf(x2 * c);
                oi[d] = orc_f32_to_bf16(a - b);
                oi[d + half] = orc_f32_to_bf16(e + f);
            }
        }
    }
}

/* The same in fp32 (tables fp32, no rounding below fp32, products and sums not fused). */
ORC_API void orc_rope_apply_f32(const float *x, const float *sin_t, const float *cos_t, const int32_t *pos, int64_t rows,
                                int H, int D, float *out) {
    const int half = D / 2;
    for (int64_t r = 0; r < rows; ++r) {
        const float *st = sin_t + (int64_t)pos[r] * half, *ct = cos_t + (int64_t)pos[r] * half;
        for (int h = 0; h < H; ++h) {
            const float *xi = x + (r * H + h) * D;
            float *oi = out + (r * H + h) * D;
            for (int d = 0; d < half; ++d) {
                const volatile float a = xi[d] * ct[d], b = xi[d + half] * st[d];
                const volatile float e = xi[d] * st[d], f = xi[d + half] * ct[d];
                oi[d] = a - b;
                oi[d + half] = e + f;
            }
        }
    }
}

/* ------------------------------------------------------------------ QK-norm */

/* Per-head RMS normalisation of q / k right before the rotary embedding, bf16 tensors [rows, H, D].
 *
 * kind 1 -- LlamaAttention::apply_qk_norm (architectures/llama.rs:929-991, Gemma3): every op in the tensor dtype,
 *   i.e. computed in fp32 and rounded to bf16 after EACH libtorch op:
 *     x2 = square(x); mean = mean_dim(x2, -1, dtype = bf16)  [fp32 sum, divided by D, rounded once];
 *     rrms = sqrt(reciprocal(mean + eps))  [eps is a scalar operand of a bf16 tensor op: it is cast to bf16 first];
 *     out = (x * rrms) * weight, weight bf16 [H, D] (head_stride = D) or [D] (head_stride = 0).
 * kind 2 -- Qwen3_5Model::apply_qknorm (architectures/qwen3_5.rs:1077-1091): fp32 throughout, one rounding to bf16 at
 *   the end:  xf = float(x); mean_sq = mean(xf * xf); rrms = rsqrt(mean_sq + eps) = 1 / sqrt(.);
 *     out = bf16((xf * rrms) * (weight + 1)), weight fp32 [D] (head_stride 0) or [H, D].
 * The sum of the squares is accumulated in double and rounded to fp32 once (the squares of bf16 values are exact in
 * fp32, so this is the correctly rounded fp32 sum); libtorch's own fp32 summation order depends on the host's vector
 * width and can differ from it in the last fp32 bit, which moves a bf16 result in a few rows per million. */
ORC_API void orc_qk_norm_bf16(const uint16_t *x, int64_t rows, int H, int D, int kind, const void *weight, int head_stride,
                              float eps, uint16_t *out) {
    for (int64_t r = 0; r < rows; ++r)
        for (int h = 0; h < H; ++h) {
            const uint16_t *xi = x + (r * H + h) * D;
            uint16_t *oi = out + (r * H + h) * D;
            double acc = 0.0;
            if (kind == 1) {
                const uint16_t *w = (const uint16_t *)weight + (int64_t)h * head_stride;
                for (int d = 0; d < D; ++d) {
                    const float v = bf16_to_f32(xi[d]);
                    const volatile float sq = rbf(v * v);
                    acc += (double)sq;
                }
                const volatile float sum = (float)acc;
                const volatile float mean = rbf(sum / (float)D);
                const volatile float t = rbf(mean + rbf(eps));
                const volatile float rc = rbf(1.0f / t);
                const volatile float rrms = rbf(sqrtf(rc));
                for (int d = 0; d < D; ++d) {
                    const volatile float y = rbf(bf16_to_f32(xi[d]) * rrms);
                    oi[d] = orc_f32_to_bf16(y * bf16_to_f32(w[d]));
                }
            } else {
                const float *w = (const float *)weight + (int64_t)h * head_stride;
                for (int d = 0; d < D; ++d) {
                    const float v = bf16_to_f32(xi[d]);
                    const volatile float sq = v * v;
                    acc += (double)sq;
                }
                const volatile float sum = (float)acc;
                const volatile float mean = sum / (float)D;
                const volatile float t = mean + eps;
                const volatile float sr = sqrtf(t);
                const volatile float rrms = 1.0f / sr;
                for (int d = 0; d < D; ++d) {
                    const volatile float y = bf16_to_f32(xi[d]) * rrms;
                    const volatile float w1 = w[d] + 1.0f;
                    oi[d] = orc_f32_to_bf16(y * w1);
                }
            }
        }
}

/* ------------------------------------------------------- DeltaNet surroundings */

static inline float silu_f(float x) { return x / (1.0f + expf(-x)); }

/* x: bf16 [B, S, C] (C = conv channels), w: bf16 [C, K] (tap K-1 multiplies the current frame),
 * state: bf16 [B, C, K-1] in/out (the K-1 frames before this call, oldest first; zeros before the first call),
 * y: bf16 [B, S, C] = silu(conv) rounded to bf16 after the conv and after the SiLU. */
ORC_API void orc_deltanet_conv_silu_bf16(const uint16_t *x, const uint16_t *w, uint16_t *state, int B, int S, int C, int K,
                                         uint16_t *y) {
    for (int b = 0; b < B; ++b)
        for (int c = 0; c < C; ++c) {
            float hist[16];
            for (int i = 0; i < K - 1; ++i) hist[i] = bf16_to_f32(state[((int64_t)b * C + c) * (K - 1) + i]);
            for (int t = 0; t < S; ++t) {
                hist[K - 1] = bf16_to_f32(x[((int64_t)b * S + t) * C + c]);
                float acc = 0.0f;
                for (int i = 0; i < K; ++i) {
                    const volatile float p = bf16_to_f32(w[(int64_t)c * K + i]) * hist[i];
                    acc += p;
                }
                const float r = rbf(acc);
                y[((int64_t)b * S + t) * C + c] = orc_f32_to_bf16(silu_f(r));
                for (int i = 0; i < K - 1; ++i) hist[i] = hist[i + 1];
            }
            for (int i = 0; i < K - 1; ++i) state[((int64_t)b * C + c) * (K - 1) + i] = orc_f32_to_bf16(hist[i]);
        }
}

/* a, bb: bf16 [rows, nv]; neg_a_exp, dt_bias: fp32 [nv];  g = neg_a_exp * softplus(a + dt_bias), beta = sigmoid(bb). */
ORC_API void orc_deltanet_gates(const uint16_t *a, const uint16_t *bb, const float *neg_a_exp, const float *dt_bias,
                                int64_t rows, int nv, float *g, float *beta) {
    for (int64_t r = 0; r < rows; ++r)
        for (int j = 0; j < nv; ++j) {
            const float x = bf16_to_f32(a[r * nv + j]) + dt_bias[j];
            const float sp = x > 20.0f ? x : log1pf(expf(x)); /* libtorch softplus, beta 1, threshold 20 */
            g[r * nv + j] = neg_a_exp[j] * sp;
            beta[r * nv + j] = 1.0f / (1.0f + expf(-bf16_to_f32(bb[r * nv + j])));
        }
}

/* x: fp32 [rows, D]; z: bf16 [rows, D]; w: fp32 [D]; out: bf16 [rows, D]. */
ORC_API void orc_gated_rmsnorm(const float *x, const uint16_t *z, const float *w, float eps, int64_t rows, int D,
                               uint16_t *out) {
    for (int64_t r = 0; r < rows; ++r) {
        double ss = 0.0;
        for (int d = 0; d < D; ++d) ss += (double)x[r * D + d] * x[r * D + d];
        const float rrms = 1.0f / sqrtf((float)(ss / D) + eps);
        for (int d = 0; d < D; ++d) {
            const float n = x[r * D + d] * rrms;
            out[r * D + d] = orc_f32_to_bf16(n * w[d] * silu_f(bf16_to_f32(z[r * D + d])));
        }
    }
}
