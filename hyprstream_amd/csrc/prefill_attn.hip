// Causal prefill attention on the MFMA pipe with online softmax (gfx950, wave64).
//
// One call serves S new tokens per sequence (a prompt, or one chunk of a chunked prefill).  Query
// row i sits at absolute position hist_len + i and attends
//   (1) the hist_len tokens already in the int8 cache, dequantized on the fly, and
//   (2) new tokens 0..=i in exact bf16,
// which is softmax(Q K^T * scale + causal mask) V over [history | this call's K/V].
//
// Work split.  A 512-thread workgroup (8 wavefronts, 2 per SIMD) owns 256 (query, head) columns of
// one kv-head -- with G = Hq/Hkv >= 4: 64 consecutive queries x 4 query heads -- and walks the keys
// in 32-key steps.  Every step's K and V tile is converted ONCE per workgroup into ready-to-issue
// MFMA A operands in LDS (16 blocks of 64 lanes x 16 B: K as 2 tiles x 4 k-groups, V^T as 8 row
// groups) by the eight wavefronts together, double-buffered, one barrier per step; each wavefront
// then reads the operands with conflict-free ds_read_b128 and uses each one for its two 16-column
// blocks.  Grid = (query tiles, kv-heads x head groups, sequences).
//
// Products (both on v_mfma_f32_16x16x32, keys on the M axis, columns on N):
//   S^T[key, col]  = sum_d K[key, d] Q[col, d]
//   O^T[d, col]   += sum_key V^T[d, key] P^T[key, col]
// History part: f16 MFMA, int8 codes enter as exact fp16 integers (see decode_attn.hip); Q is scaled
// per column by a power of two into fp16 range; the per-token K scale multiplies the fp32 score, the
// per-token V scale is folded into P (fp16).  New-token part: bf16 MFMA straight from the caller's
// bf16 K/V, V^T built with permutes, P rounded to bf16.  Softmax and accumulation are fp32; the
// score layout of the first product is the B-operand layout of the second, so P stays in its lanes.
#include "mfma_common.hpp"
#include "quant_device.hpp"

namespace hs {

constexpr int kPD = 128;
constexpr int kPStep = 32;
constexpr int kPWaves = 8;
constexpr int kNB = 2;  // 16-column blocks per wavefront
constexpr float kPLog2e = 1.4426950408889634f;
constexpr float kPPScale = 64.0f;
constexpr float kSlack = 4.0f;  // log2 units by which the softmax reference value overshoots a new maximum

struct PrefillArgs {
    const uint16_t *q, *kn, *vn;  // [B,S,Hq,D], [B,S,Hkv,D], [B,S,Hkv,D] bf16
    const uint8_t *kc, *vc;
    const float *ks, *vs;
    KvAddr ka, va;
    uint16_t *out;  // [B,S,Hq,D] bf16
    int32_t B, S, Hq, Hkv, G, HG, hist_len;
    float scale_log2e;
};

struct alignas(16) StepTile {
    uint8_t k[8][1024];  // block 4*u + j: K tile u (16 keys), k-group j; 64 lanes x 16 B in MFMA lane order
    uint8_t v[8][1024];  // block bb: V^T rows d = 8*li + bb, 32 keys
    float ksc[32];       // K scale of the step's tokens (0 for tokens past the end)
    float pv[32];        // V scale x 64 (0 past the end)
};

__global__ __launch_bounds__(512, 2) void prefill_attn_kernel(PrefillArgs a) {
    __shared__ StepTile tiles[2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int li = lane & 15, lq = lane >> 4;
    // XCD-aware placement.  Workgroups are handed to the 8 XCDs round-robin by linear id, and each XCD has
    // its own L2.  All query tiles that read the same (sequence, kv-head) K/V stream are therefore given
    // linear ids that are congruent mod 8, so the stream is fetched into ONE L2 and shared there instead of
    // being pulled into all eight.
    int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
    {
        const int X = gridDim.x, YZ = gridDim.y * gridDim.z;
        if ((YZ & 7) == 0) {
            const int p = bx + X * (by + gridDim.y * bz);  // dispatch order
            const int grp = (p & 7) + 8 * (p / (8 * X));   // (kv-head group, sequence) unit
            bx = (p >> 3) % X;
            by = grp % gridDim.y;
            bz = grp / gridDim.y;
        }
    }
    const int b = bz;
    const int groups = a.G / a.HG;
    const int kvh = by / groups, hg = by % groups;
    const int S = a.S, H = a.hist_len;
    const int q_per_wg = 16 * (kNB * kPWaves / a.HG);
    const int q0 = bx * q_per_wg;
    if (q0 >= S) return;
    const int wg_qlast = min(S - 1, q0 + q_per_wg - 1);

    int head[kNB], qi[kNB];
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
        const int bi = kNB * wave + nb;
        head[nb] = kvh * a.G + hg * a.HG + bi % a.HG;
        qi[nb] = q0 + 16 * (bi / a.HG) + li;
    }
    const int wv_q0 = q0 + 16 * ((kNB * wave) / a.HG);  // first query of this wavefront
    const int wv_qlast = min(S - 1, q0 + 16 * ((kNB * wave + kNB - 1) / a.HG) + 15);
    const bool wv_active = wv_q0 < S;

    float4v acc[kNB][8];
    float m_run[kNB], l_run[kNB];
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
        m_run[nb] = -INFINITY;
        l_run[nb] = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[nb][i] = (float4v){0.f, 0.f, 0.f, 0.f};
    }

    // Online softmax: raise_max() takes the blocks' step maxima (already reduced over the column).  The
    // reference value m_run is not the running maximum itself but an upper bound of it: when a column's
    // maximum passes m_run, m_run is set kSlack above the new maximum, so that later small increases need no
    // rescaling of the 64 accumulator registers.  Every weight is then exp2(s - m_run) <= 1, the largest at
    // least 2^-kSlack; numerator and denominator carry the same factor, which cancels in the final division.
    auto raise_max = [&](const float (&mx)[kNB]) {
        bool changed = false;
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb) changed |= mx[nb] > m_run[nb];
        if (__builtin_amdgcn_ballot_w64(changed) != 0) {
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
                const float m_new = mx[nb] > m_run[nb] ? mx[nb] + kSlack : m_run[nb];
                const float alpha = (m_new == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m_run[nb] - m_new);
                l_run[nb] *= alpha;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[nb][i] *= alpha;
                m_run[nb] = m_new;
            }
        }
    };

    const int obase = lane * 16;  // this lane's 16 bytes inside an operand block

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
            amax = quad_max(amax);
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
            qsum = quad_sum(qsum);
            cq[nb] = ldexpf(a.scale_log2e, ex);
            cinit[nb] = -1152.0f * qsum;
        }

        const int nsteps = (H + kPStep - 1) / kPStep;
        // ---- producer roles: wavefronts 0-3 convert K (tile u = wave/2, k-groups 2*(wave&1) and +1);
        //      wavefronts 4-7 convert V (token group wave-4, byte columns 2x and 2x+1 with x = lane/16);
        //      wavefront 0 also stages the scales.
        u32x4 rawk = {0u, 0u, 0u, 0u};
        uint32_t rawv[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
        float raws = 0.0f;
        auto issue = [&](int step) {
            const int t0 = step * kPStep;
            const int last = H - 1 - t0;
            int64_t unit;
            int slot;
            if (wave < 4) {
                resolve(a.ka, b, t0, unit, slot);
                const uint8_t *kb = a.kc + unit * a.ka.code_stride_seq + (int64_t)kvh * a.ka.code_stride_head + (int64_t)slot * kPD;
                rawk = *(const u32x4 *)(kb + min(16 * (wave >> 1) + li, last) * kPD + 32 * lq + 16 * (wave & 1));
                if (wave == 0) {
                    const int tok = lane & 31;
                    if (lane < 32) {
                        raws = a.ks[unit * a.ka.scale_stride_seq + (int64_t)kvh * a.ka.scale_stride_head + slot + min(tok, last)];
                    } else {
                        resolve(a.va, b, t0, unit, slot);
                        raws = a.vs[unit * a.va.scale_stride_seq + (int64_t)kvh * a.va.scale_stride_head + slot + min(tok, last)] * kPPScale;
                    }
                    if (tok > last) raws = 0.0f;
                }
            } else {
                resolve(a.va, b, t0, unit, slot);
                const uint8_t *vb = a.vc + unit * a.va.code_stride_seq + (int64_t)kvh * a.va.code_stride_head + (int64_t)slot * kPD;
                const int g4 = wave - 4;
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    rawv[e] = *(const uint32_t *)(vb + min(16 * (e >> 2) + 4 * g4 + (e & 3), last) * kPD + 8 * li + 4 * (lq >> 1));
            }
        };
        auto commit = [&](StepTile &t) {
            if (wave < 4) {
                const int blk = 4 * (wave >> 1) + 2 * (wave & 1);
                *(half8 *)(t.k[blk] + obase) = int8x8_to_f16_biased(rawk[0], rawk[1]);
                *(half8 *)(t.k[blk + 1] + obase) = int8x8_to_f16_biased(rawk[2], rawk[3]);
                if (wave == 0) (lane < 32 ? t.ksc : t.pv)[lane & 31] = raws;
            } else {
                const int dst = (li + 16 * (wave - 4)) * 16;  // operand lane = (li, token group wave-4)
                const int bsel = 2 * (lq & 1);
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    *(half8 *)(t.v[2 * lq + i] + dst) =
                        pack_half8(int8_pair_to_f16(rawv[0], rawv[1], bsel + i), int8_pair_to_f16(rawv[2], rawv[3], bsel + i),
                                   int8_pair_to_f16(rawv[4], rawv[5], bsel + i), int8_pair_to_f16(rawv[6], rawv[7], bsel + i));
            }
        };
        auto consume = [&](const StepTile &t, int step) {
            const int t0 = step * kPStep;
            const bool tail = t0 + kPStep > H;
            float ksc[8], pv[8];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const float4v k4 = *(const float4v *)(t.ksc + 16 * u + 4 * lq);
                const float4v p4 = *(const float4v *)(t.pv + 16 * u + 4 * lq);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    ksc[4 * u + r] = k4[r];
                    pv[4 * u + r] = p4[r];
                }
            }
            float4v s[kNB][2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb) s[nb][u] = (float4v){cinit[nb], cinit[nb], cinit[nb], cinit[nb]};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const half8 ak = *(const half8 *)(t.k[4 * u + j] + obase);
#pragma unroll
                    for (int nb = 0; nb < kNB; ++nb)
                        s[nb][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ak, qop[nb][j], s[nb][u], 0, 0, 0);
                }
            }
            float sc[kNB][8], mx[kNB];
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int r = 0; r < 4; ++r) sc[nb][4 * u + r] = s[nb][u][r] * ksc[4 * u + r];
                if (tail) {
#pragma unroll
                    for (int u = 0; u < 2; ++u)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (t0 + 16 * u + 4 * lq + r >= H) sc[nb][4 * u + r] = -INFINITY;
                }
                float m = sc[nb][0];
#pragma unroll
                for (int i = 1; i < 8; ++i) m = fmaxf(m, sc[nb][i]);
                mx[nb] = quad_max(m) * cq[nb];  // cq > 0: max(t) * cq == max(t * cq); -inf stays -inf
            }
            raise_max(mx);
            half8 pop[kNB];
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
                const float mref = (m_run[nb] == -INFINITY) ? 0.0f : m_run[nb];
                float p[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float e = __builtin_amdgcn_exp2f(sc[nb][i] * cq[nb] - mref);
                    l_run[nb] += e;
                    p[i] = e * pv[i];
                }
                pop[nb] = pack_half8(pack_f16x2(p[0], p[1]), pack_f16x2(p[2], p[3]), pack_f16x2(p[4], p[5]), pack_f16x2(p[6], p[7]));
            }
#pragma unroll
            for (int bb = 0; bb < 8; ++bb) {
                const half8 av = *(const half8 *)(t.v[bb] + obase);
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb)
                    acc[nb][bb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, pop[nb], acc[nb][bb], 0, 0, 0);
            }
        };
        issue(0);
        commit(tiles[0]);
        if (nsteps > 1) issue(1);
        __syncthreads();
        for (int step = 0; step < nsteps; ++step) {
            if (step + 1 < nsteps) commit(tiles[(step + 1) & 1]);
            if (step + 2 < nsteps) issue(step + 2);
            if (wv_active) consume(tiles[step & 1], step);
            __syncthreads();
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
        const int nsteps = wg_qlast / kPStep + 1;
        const uint16_t *knb = a.kn + ((int64_t)b * S * a.Hkv + kvh) * kPD;
        const uint16_t *vnb = a.vn + ((int64_t)b * S * a.Hkv + kvh) * kPD;
        const int64_t rstride = (int64_t)a.Hkv * kPD;  // elements between consecutive tokens
        // producer roles: wavefronts 0-3: K tile u = wave/2, k-groups 2*(wave&1), +1 (bf16 rows are operands as
        // they are); wavefronts 4-7: V^T, token group wave-4, columns 2x, 2x+1 (x = lane/16) of this lane's 8.
        u32x4 rawk[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
        uint32_t rawv[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
        auto issue = [&](int step) {
            const int t0 = step * kPStep;
            if (wave < 4) {
                const uint16_t *p = knb + (int64_t)min(t0 + 16 * (wave >> 1) + li, S - 1) * rstride + 32 * lq + 16 * (wave & 1);
                rawk[0] = *(const u32x4 *)p;
                rawk[1] = *(const u32x4 *)(p + 8);
            } else {
                const int g4 = wave - 4;
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    rawv[e] = *(const uint32_t *)(vnb + (int64_t)min(t0 + 16 * (e >> 2) + 4 * g4 + (e & 3), S - 1) * rstride + 8 * li + 2 * lq);
            }
        };
        auto commit = [&](StepTile &t) {
            if (wave < 4) {
                const int blk = 4 * (wave >> 1) + 2 * (wave & 1);
                *(u32x4 *)(t.k[blk] + obase) = rawk[0];
                *(u32x4 *)(t.k[blk + 1] + obase) = rawk[1];
            } else {
                const int dst = (li + 16 * (wave - 4)) * 16;
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const u32x4 w = {pick_halves(rawv[0], rawv[1], i), pick_halves(rawv[2], rawv[3], i),
                                     pick_halves(rawv[4], rawv[5], i), pick_halves(rawv[6], rawv[7], i)};
                    *(u32x4 *)(t.v[2 * lq + i] + dst) = w;
                }
            }
        };
        auto consume = [&](const StepTile &t, int step) {
            const int t0 = step * kPStep;
            float4v s[kNB][2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb) s[nb][u] = (float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const bf16x8 ak = *(const bf16x8 *)(t.k[4 * u + j] + obase);
#pragma unroll
                    for (int nb = 0; nb < kNB; ++nb)
                        s[nb][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ak, qop[nb][j], s[nb][u], 0, 0, 0);
                }
            }
            const bool diag = t0 + kPStep - 1 > wv_q0;  // some (key, query) pair of this step is in the future
            float sc[kNB][8], mx[kNB];
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int r = 0; r < 4; ++r) sc[nb][4 * u + r] = s[nb][u][r] * cq;
                if (diag) {
                    const int qlim = min(qi[nb], S - 1);
#pragma unroll
                    for (int u = 0; u < 2; ++u)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (t0 + 16 * u + 4 * lq + r > qlim) sc[nb][4 * u + r] = -INFINITY;
                }
                float m = sc[nb][0];
#pragma unroll
                for (int i = 1; i < 8; ++i) m = fmaxf(m, sc[nb][i]);
                mx[nb] = quad_max(m);
            }
            raise_max(mx);
            bf16x8 pop[kNB];
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
                const float mref = (m_run[nb] == -INFINITY) ? 0.0f : m_run[nb];
                float p[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float e = __builtin_amdgcn_exp2f(sc[nb][i] - mref);
                    l_run[nb] += e;
                    p[i] = e * kPPScale;
                }
                pop[nb] = pack_bf16x8(pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]), pack_bf16x2(p[6], p[7]));
            }
#pragma unroll
            for (int bb = 0; bb < 8; ++bb) {
                const bf16x8 av = *(const bf16x8 *)(t.v[bb] + obase);
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb)
                    acc[nb][bb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, pop[nb], acc[nb][bb], 0, 0, 0);
            }
        };
        issue(0);
        commit(tiles[0]);
        if (nsteps > 1) issue(1);
        __syncthreads();
        for (int step = 0; step < nsteps; ++step) {
            if (step + 1 < nsteps) commit(tiles[(step + 1) & 1]);
            if (step + 2 < nsteps) issue(step + 2);
            if (wv_active && step * kPStep <= wv_qlast) consume(tiles[step & 1], step);
            __syncthreads();
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
            for (int e = 0; e < 4; ++e) w[e] = pack_bf16x2(acc[nb][2 * e][r] * inv, acc[nb][2 * e + 1][r] * inv);
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
    a.HG = G >= 4 ? 4 : G;
    a.scale_log2e = softmax_scale * kPLog2e;
    const int q_per_wg = 16 * (kNB * kPWaves / a.HG);
    dim3 grid((S + q_per_wg - 1) / q_per_wg, Hkv * (G / a.HG), B);
    prefill_attn_kernel<<<grid, 512, 0, st>>>(a);
    if (int rc = check_launch("prefill_attn")) return rc;
    if (quantize_on_write)
        return hs_kv_quantize_int8(k_new, v_new, HS_BF16, k_codes, v_codes, k_scales, v_scales, layout, nullptr,
                                   hist_len, B, S, Hkv, D, stream);
    return HS_OK;
}
