// Causal prefill attention on the MFMA pipe with online softmax (gfx950, wave64).
//
// One call serves S new tokens per sequence (a prompt, or one chunk of a chunked prefill).  Query
// row i sits at absolute position hist_len + i and attends
//   (1) the hist_len tokens already in the int8 cache, dequantized on the fly, and
//   (2) new tokens 0..=i in exact bf16,
// which is softmax(Q K^T * scale + causal mask) V over [history | this call's K/V].
//
// Work split.  A wavefront owns 64 (query, head) columns = 4 MFMA column blocks of 16: with
// G = Hq/Hkv >= 4 that is 16 queries x 4 query heads of one kv-head, so every K/V tile it loads
// and converts is used four times; smaller G trade heads for more queries.  A workgroup is four
// such wavefronts on consecutive queries; grid = (query tiles, kv-heads x head groups, sequences).
// Wavefronts never synchronise: each keeps its own online-softmax state per column and walks the
// keys in 32-key steps with the next step's tile already in flight (register double buffer).
//
// Products (both on v_mfma_f32_16x16x32, keys on the M axis, columns on N):
//   S^T[key, col]  = sum_d K[key, d] Q[col, d]
//   O^T[d, col]   += sum_key V^T[d, key] P^T[key, col]
// History part: f16 MFMA, int8 codes enter as exact fp16 integers (see decode_attn.hip); Q is scaled
// per column by a power of two into fp16 range; per-token K scale on the fp32 score, per-token V
// scale folded into P (fp16).  New-token part: bf16 MFMA straight from the caller's bf16 K/V, V^T
// built with byte permutes in registers, P rounded to bf16.  Accumulation, softmax: fp32.
#include "mfma_common.hpp"
#include "quant_device.hpp"

namespace hs {

constexpr int kPD = 128;
constexpr int kPStep = 32;
#ifndef HS_PREFILL_NB
#define HS_PREFILL_NB 2
#endif
constexpr float kPLog2e = 1.4426950408889634f;
constexpr float kPPScale = 64.0f;

struct PrefillArgs {
    const uint16_t *q, *kn, *vn;  // [B,S,Hq,D], [B,S,Hkv,D], [B,S,Hkv,D] bf16
    const uint8_t *kc, *vc;
    const float *ks, *vs;
    KvAddr ka, va;
    uint16_t *out;  // [B,S,Hq,D] bf16
    int32_t B, S, Hq, Hkv, G, HW, QT, hist_len;
    float scale_log2e;
};

struct HistStage {
    u32x4 k[2][2];
    u32x2 v[8];
    float4v sk[2], sv[2];
};
struct NewStage {
    u32x4 k[2][4];  // tile u, MFMA j: eight bf16 (d = 32*lq + 8*j ..)
    u32x4 v[8];     // key slot e: eight bf16 (d = 8*li ..)
};

template <int kNB>  // column blocks (16 columns each) per wavefront
__global__ __launch_bounds__(256, 1) void prefill_attn_kernel(PrefillArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int li = lane & 15, lq = lane >> 4;
    const int b = blockIdx.z;
    const int groups = a.G / a.HW;
    const int kvh = blockIdx.y / groups, hg = blockIdx.y % groups;
    const int S = a.S, H = a.hist_len;
    const int qw0 = (blockIdx.x * 4 + wave) * 16 * a.QT;  // first query of this wavefront
    if (qw0 >= S) return;
    const int qw_last = min(S - 1, qw0 + 16 * a.QT - 1);

    int head[kNB], qi[kNB];
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
        head[nb] = kvh * a.G + hg * a.HW + nb % a.HW;
        qi[nb] = qw0 + 16 * (nb / a.HW) + li;
    }

    float4v acc[kNB][8];
    float m_run[kNB], l_run[kNB];
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
        m_run[nb] = -INFINITY;
        l_run[nb] = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[nb][i] = (float4v){0.f, 0.f, 0.f, 0.f};
    }

    // Online softmax in two halves so that the code between them is straight-line for all column blocks
    // (MFMA issue of one block overlaps the VALU work of another): raise_max() takes the blocks' step
    // maxima and rescales under ONE wave-uniform branch that is rarely taken once the maxima settle;
    // weights() turns scores into exp2 weights times pv[].
    auto raise_max = [&](const float (&mx)[kNB]) {
        bool changed = false;
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb) changed |= mx[nb] > m_run[nb];
        if (__builtin_amdgcn_ballot_w64(changed) != 0) {
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
                const float m_new = fmaxf(m_run[nb], mx[nb]);
                const float alpha = (m_new == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m_run[nb] - m_new);
                l_run[nb] *= alpha;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[nb][i] *= alpha;
                m_run[nb] = m_new;
            }
        }
    };
    auto weights = [&](int nb, const float (&sc)[8], const float (&pv)[8], float (&p)[8]) {
        const float mref = (m_run[nb] == -INFINITY) ? 0.0f : m_run[nb];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float e = __builtin_amdgcn_exp2f(sc[i] - mref);
            l_run[nb] += e;
            p[i] = e * pv[i];
        }
    };

    // =============================== history: int8 cache, f16 MFMA ===============================
    if (H > 0) {
        half8 qop[kNB][4];
        float cq[kNB], cinit[kNB];
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb) {
            const uint16_t *qp = a.q + (((int64_t)b * S + min(qi[nb], S - 1)) * a.Hq + head[nb]) * kPD + 32 * lq;
            float qf[32], amax = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const u32x4 w = *(const u32x4 *)(qp + 8 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    qf[8 * i + 2 * e] = __uint_as_float(w[e] << 16);
                    qf[8 * i + 2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
                }
            }
#pragma unroll
            for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(qf[i]));
            amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
            amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
            int ex = 0;
            if (amax > 0.0f && amax < 3.0e38f) (void)frexpf(amax, &ex);
            float qsum = 0.0f;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const _Float16 hq = (_Float16)ldexpf(qf[8 * j + e], -ex);
                    qop[nb][j][e] = hq;
                    qsum += (float)hq;
                }
            qsum += __shfl_xor(qsum, 16, 64);
            qsum += __shfl_xor(qsum, 32, 64);
            cq[nb] = ldexpf(a.scale_log2e, ex);
            cinit[nb] = -1152.0f * qsum;
        }

        const int nsteps = (H + kPStep - 1) / kPStep;
        auto load_hist = [&](HistStage &st, int step) {
            const int t0 = step * kPStep;
            int64_t ku, vu;
            int kslot, vslot;
            resolve(a.ka, b, t0, ku, kslot);
            resolve(a.va, b, t0, vu, vslot);
            const int last = H - 1 - t0;
            const uint8_t *kb = a.kc + ku * a.ka.code_stride_seq + (int64_t)kvh * a.ka.code_stride_head + (int64_t)kslot * kPD;
            const uint8_t *vb = a.vc + vu * a.va.code_stride_seq + (int64_t)kvh * a.va.code_stride_head + (int64_t)vslot * kPD;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const uint8_t *p = kb + min(16 * u + li, last) * kPD + 32 * lq;
                st.k[u][0] = *(const u32x4 *)p;
                st.k[u][1] = *(const u32x4 *)(p + 16);
            }
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    st.v[4 * u + r] = *(const u32x2 *)(vb + min(16 * u + 4 * lq + r, last) * kPD + 8 * li);
            const float *ksb = a.ks + ku * a.ka.scale_stride_seq + (int64_t)kvh * a.ka.scale_stride_head + kslot;
            const float *vsb = a.vs + vu * a.va.scale_stride_seq + (int64_t)kvh * a.va.scale_stride_head + vslot;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int tok = min(16 * u + 4 * lq, last & ~3);
                st.sk[u] = *(const float4v *)(ksb + tok);
                st.sv[u] = *(const float4v *)(vsb + tok);
            }
        };
        HistStage st;
        load_hist(st, 0);
        for (int step = 0; step < nsteps; ++step) {
            const int t0 = step * kPStep;
            // raw tile -> MFMA operands; the raw registers are then free for the next tile's loads
            half8 ak[2][4], av[8];
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    ak[u][j] = int8x8_to_f16_biased(st.k[u][j >> 1][2 * (j & 1)], st.k[u][j >> 1][2 * (j & 1) + 1]);
#pragma unroll
            for (int bb = 0; bb < 8; ++bb)
                av[bb] = pack_half8(int8_pair_to_f16(st.v[0][bb >> 2], st.v[1][bb >> 2], bb & 3),
                                    int8_pair_to_f16(st.v[2][bb >> 2], st.v[3][bb >> 2], bb & 3),
                                    int8_pair_to_f16(st.v[4][bb >> 2], st.v[5][bb >> 2], bb & 3),
                                    int8_pair_to_f16(st.v[6][bb >> 2], st.v[7][bb >> 2], bb & 3));
            float ksc[8], pv[8];
            const bool tail = t0 + kPStep > H;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const bool dead = tail && (t0 + 16 * u + 4 * lq + r >= H);
                    ksc[4 * u + r] = dead ? 0.0f : st.sk[u][r];
                    pv[4 * u + r] = dead ? 0.0f : st.sv[u][r] * kPPScale;
                }
            if (step + 1 < nsteps) load_hist(st, step + 1);
            float sc[kNB][8], mx[kNB];
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
                float4v s[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    s[u] = (float4v){cinit[nb], cinit[nb], cinit[nb], cinit[nb]};
#pragma unroll
                    for (int j = 0; j < 4; ++j) s[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ak[u][j], qop[nb][j], s[u], 0, 0, 0);
                }
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        sc[nb][4 * u + r] = s[u][r] * ksc[4 * u + r] * cq[nb];
                        if (tail && (t0 + 16 * u + 4 * lq + r >= H)) sc[nb][4 * u + r] = -INFINITY;
                    }
                float m = sc[nb][0];
#pragma unroll
                for (int i = 1; i < 8; ++i) m = fmaxf(m, sc[nb][i]);
                mx[nb] = quad_max(m);
            }
            raise_max(mx);
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
                float p[8];
                weights(nb, sc[nb], pv, p);
                const half8 pop = pack_half8(pack_f16x2(p[0], p[1]), pack_f16x2(p[2], p[3]), pack_f16x2(p[4], p[5]),
                                             pack_f16x2(p[6], p[7]));
#pragma unroll
                for (int bb = 0; bb < 8; ++bb)
                    acc[nb][bb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[bb], pop, acc[nb][bb], 0, 0, 0);
            }
        }
    }

    // =============================== new tokens: bf16, causal ===============================
    {
        bf16x8 qop[kNB][4];
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb) {
            const uint16_t *qp = a.q + (((int64_t)b * S + min(qi[nb], S - 1)) * a.Hq + head[nb]) * kPD + 32 * lq;
#pragma unroll
            for (int j = 0; j < 4; ++j) qop[nb][j] = __builtin_bit_cast(bf16x8, *(const u32x4 *)(qp + 8 * j));
        }
        const float cq = a.scale_log2e;
        const int nsteps = qw_last / kPStep + 1;
        const uint16_t *knb = a.kn + ((int64_t)b * S * a.Hkv + kvh) * kPD;
        const uint16_t *vnb = a.vn + ((int64_t)b * S * a.Hkv + kvh) * kPD;
        const int64_t rstride = (int64_t)a.Hkv * kPD;  // elements between consecutive tokens
        auto load_new = [&](NewStage &st, int step) {
            const int t0 = step * kPStep;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const uint16_t *p = knb + (int64_t)min(t0 + 16 * u + li, S - 1) * rstride + 32 * lq;
#pragma unroll
                for (int j = 0; j < 4; ++j) st.k[u][j] = *(const u32x4 *)(p + 8 * j);
            }
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    st.v[4 * u + r] = *(const u32x4 *)(vnb + (int64_t)min(t0 + 16 * u + 4 * lq + r, S - 1) * rstride + 8 * li);
        };
        NewStage st;
        load_new(st, 0);
        for (int step = 0; step < nsteps; ++step) {
            const int t0 = step * kPStep;
            bf16x8 av[8], ak[2][4];
#pragma unroll
            for (int bb = 0; bb < 8; ++bb)
                av[bb] = pack_bf16x8(pick_halves(st.v[0][bb >> 1], st.v[1][bb >> 1], bb & 1),
                                     pick_halves(st.v[2][bb >> 1], st.v[3][bb >> 1], bb & 1),
                                     pick_halves(st.v[4][bb >> 1], st.v[5][bb >> 1], bb & 1),
                                     pick_halves(st.v[6][bb >> 1], st.v[7][bb >> 1], bb & 1));
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int j = 0; j < 4; ++j) ak[u][j] = __builtin_bit_cast(bf16x8, st.k[u][j]);
            if (step + 1 < nsteps) load_new(st, step + 1);
            const float pv[8] = {kPPScale, kPPScale, kPPScale, kPPScale, kPPScale, kPPScale, kPPScale, kPPScale};
            float sc[kNB][8], mx[kNB];
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
                float4v s[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    s[u] = (float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = 0; j < 4; ++j) s[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ak[u][j], qop[nb][j], s[u], 0, 0, 0);
                }
                const int qlim = min(qi[nb], S - 1);
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        sc[nb][4 * u + r] = (t0 + 16 * u + 4 * lq + r <= qlim) ? s[u][r] * cq : -INFINITY;
                float m = sc[nb][0];
#pragma unroll
                for (int i = 1; i < 8; ++i) m = fmaxf(m, sc[nb][i]);
                mx[nb] = quad_max(m);
            }
            raise_max(mx);
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
                float p[8];
                weights(nb, sc[nb], pv, p);
                const bf16x8 pop = pack_bf16x8(pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]),
                                               pack_bf16x2(p[6], p[7]));
#pragma unroll
                for (int bb = 0; bb < 8; ++bb)
                    acc[nb][bb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[bb], pop, acc[nb][bb], 0, 0, 0);
            }
        }
    }

    // =============================== normalise and store ===============================
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
        const float l = quad_sum(l_run[nb]);
        if (qi[nb] >= S) continue;
        const float inv = 1.0f / (l * kPPScale);
        uint16_t *op = a.out + (((int64_t)b * S + qi[nb]) * a.Hq + head[nb]) * kPD + 32 * lq;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            u32x4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                w[e] = pack_bf16x2(acc[nb][2 * e][r] * inv, acc[nb][2 * e + 1][r] * inv);
            *(u32x4 *)(op + 8 * r) = w;
        }
    }
}

int validate_layout(const hs_kv_layout *l, int B, int S, int Hkv, int D, bool need_scales);

}  // namespace hs

extern "C" int hs_prefill_attn_int8(const void *q, const void *k_new, const void *v_new, int8_t *k_codes,
                                    int8_t *v_codes, float *k_scales, float *v_scales, const hs_kv_layout *layout,
                                    int32_t hist_len, void *out, int32_t B, int32_t S, int32_t Hq, int32_t Hkv,
                                    int32_t D, float softmax_scale, int quantize_on_write, hs_stream_t stream) {
    using namespace hs;
    if (int rc = validate_layout(layout, B, S, Hkv, D, true)) return rc;
    if (D != kPD) return fail(HS_ERR_INVALID_ARGUMENT, "prefill attention is built for head_dim 128, got %d", D);
    if (!q || !k_new || !v_new || !out) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if ((hist_len > 0 || quantize_on_write) && (!k_codes || !v_codes || !k_scales || !v_scales))
        return fail(HS_ERR_INVALID_ARGUMENT, "null cache buffer");
    if (hist_len < 0) return fail(HS_ERR_INVALID_ARGUMENT, "negative hist_len");
    const int G = Hq > 0 && Hkv > 0 ? Hq / Hkv : 0;
    if (Hq <= 0 || Hq % Hkv != 0 || (G != 1 && G != 2 && G % 4 != 0))
        return fail(HS_ERR_INVALID_ARGUMENT, "need Hq/Hkv in {1, 2, 4k} (Hq=%d Hkv=%d)", Hq, Hkv);
    const int64_t cap = layout->k_block_table ? (int64_t)layout->capacity_tokens * layout->block_table_stride
                                              : layout->capacity_tokens;
    if ((int64_t)hist_len + (quantize_on_write ? S : 0) > cap)
        return fail(HS_ERR_OVERFLOW, "Cache overflow: trying to cache %d tokens starting at position %d, but capacity is %lld",
                    S, hist_len, (long long)cap);
    if (layout->k_block_table && (layout->capacity_tokens % kPStep) != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "paged blocks must hold a multiple of %d tokens", kPStep);
    if (B == 0 || S == 0) return HS_OK;
    hipStream_t st = (hipStream_t)stream;
    PrefillArgs a;
    a.q = (const uint16_t *)q; a.kn = (const uint16_t *)k_new; a.vn = (const uint16_t *)v_new;
    a.kc = (const uint8_t *)k_codes; a.vc = (const uint8_t *)v_codes;
    a.ks = k_scales; a.vs = v_scales;
    a.ka = make_addr(*layout, 0); a.va = make_addr(*layout, 1);
    a.out = (uint16_t *)out;
    a.B = B; a.S = S; a.Hq = Hq; a.Hkv = Hkv; a.G = G; a.hist_len = hist_len;
    constexpr int NB = HS_PREFILL_NB;
    a.HW = G >= NB ? NB : G;
    a.QT = NB / a.HW;
    a.scale_log2e = softmax_scale * kPLog2e;
    const int q_per_wg = 64 * a.QT;
    dim3 grid((S + q_per_wg - 1) / q_per_wg, Hkv * (G / a.HW), B);
    prefill_attn_kernel<NB><<<grid, 256, 0, st>>>(a);
    if (int rc = check_launch("prefill_attn")) return rc;
    if (quantize_on_write)
        return hs_kv_quantize_int8(k_new, v_new, HS_BF16, k_codes, v_codes, k_scales, v_scales, layout, nullptr,
                                   hist_len, B, S, Hkv, D, stream);
    return HS_OK;
}
