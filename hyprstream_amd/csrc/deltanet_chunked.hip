// Gated delta rule over a prompt in chunks of 64 tokens on the MFMA pipe (gfx950, wave64).
//
// The reference's own prefill formulation (chunked_delta_rule, qwen3_5.rs:342-498; chunk size 64): with
// G_t the running sum of the log-decays g inside a chunk, k and q L2-normalised (q also scaled), and
//   L[i][j] = -beta_i (k_i . k_j) exp(G_i - G_j)  for j < i (0 otherwise),      N = (I - L)^-1,
//   U = N (v * beta),     W = N (k * beta * exp(G)),
// a chunk that starts from the state S (dk x dv) gives
//   V' = U - W S
//   O  = (q * exp(G)) S + tril(q k^T * exp(G_i - G_j)) V'
//   S <- exp(G_63) S + (k * exp(G_63 - G))^T V'.
// It is the token recurrence S <- S e^g; S += k (v - k^T S) beta; o = q^T S regrouped, so the results differ
// from the recurrent kernel only by rounding.
//
// Two kernels.  deltanet_chunk_prepare_kernel does everything that does not involve S, for all chunks of all
// (sequence, v-head) pairs in parallel (one 512-thread workgroup per chunk): normalisation, the two 64x64
// products on MFMA, the inverses of the four diagonal 16x16 blocks of I - L (repeated squaring, one wavefront per block), then
// [U | W] = N [v beta | k beta e^G] by block forward substitution on MFMA (the rest of N is never formed), and
// writes every matrix the second kernel needs into the workspace ALREADY in MFMA operand order (fp16).
// deltanet_chunk_scan_kernel walks the chunks of one (sequence, v-head, half of the state columns) in order with
// the state in accumulator registers: 28 MFMAs per computing wavefront and chunk, S and V' exchanged between the wavefronts through LDS
// in operand order, the chunk's operands brought in by two wavefronts that do nothing else.
//
// Operands are fp16 (11-bit significands; every decay factor is <= 1, so nothing overflows and what underflows
// is negligible in absolute terms), accumulation and the state are fp32.  Against the fp32 recurrence the
// outputs differ by about 1e-3 relative.
//
// MFMA layouts (v_mfma_f32_16x16x32_f16, lane l: li = l % 16, lq = l / 16): A row li / B column li hold eight
// k-slots of group lq; C/D column li holds rows 4*lq + r.  Where one operand of a product is the accumulator
// of an earlier one (S, V', the masked q k^T), the k-slots stand for the rows that accumulator layout
// holds -- slots 0-3: row 4*lq + r of the even 16-row tile of a 32-row slab, slots 4-7: the same rows of the
// odd tile -- and the other operand is read in the same order.
#include <algorithm>
#include <climits>
#include <type_traits>

#include "mfma_common.hpp"

namespace hs {

constexpr int kC = 64;               // tokens per chunk
constexpr int kWD = 128;             // dk = dv = 128
constexpr float kLog2eC = 1.4426950408889634f;
typedef _Float16 half4v __attribute__((ext_vector_type(4)));

// Workspace, chunk-major; every matrix is a list of 64-lane blocks in MFMA operand order.
// Per (sequence, k-head, chunk) -- the normalised q and k do not depend on the v-head, so the v-heads of a k-head
// share them and the decays that make them "q e^G" and "(k e^(G63-G))^T" travel as two vectors per v-head:
constexpr int kOffQh = 0;        // q (normalised, scaled)  A operand [token tile 4][dk slab 4][lane] 16 B
constexpr int kOffKt = 16384;    // k^T (normalised)        A operand [dk tile 8][token slab 2][lane] 16 B
constexpr int kHeadBytes = 32768;
// Per (sequence, v-head, chunk):
constexpr int kOffWn = 0;        // -W      A operand [token tile 4][dk slab 4][lane] 16 B
constexpr int kOffQK = 16384;    // masked q k^T     A operand [token tile 4][token slab 2][lane] 16 B
constexpr int kOffU = 24576;     // U       accumulator tiles [token tile 4][dv tile 8][lane] 8 B
constexpr int kOffEG = 40960;    // exp(G_t), 64 floats
constexpr int kOffEGl = 41216;   // exp(G_63 - G_t), 64 floats
constexpr int kOffDecay = 41472; // exp(G63), one float
constexpr int kUnitBytes = 41728;
// Behind all chunks' operands, per (chunk, sequence, v-head): 2 x 64 floats -- per column half, the sums of squares of the
// chunk's output rows over that half's 64 columns (the fused gated norm's exchange between the two halves; -1 = not
// there yet).  A region of its own: inside the units it changed their stride, and the plain scan ran 7 % slower.
constexpr int kSsqBytes = 512;
// The same matrices inside the scan kernel's LDS operand buffer:
constexpr int kOpsWn = 0, kOpsQh = 16384, kOpsKt = 32768, kOpsQK = 49152, kOpsFac = 57344, kOpsBytes = 57856;

struct ChunkArgs {
    const uint16_t *q, *k, *v;  // bf16 [B,T,nk,128], [B,T,nk,128], [B,T,nv,128]
    const float *g, *beta;      // [B,T,nv]
    float *state;               // [B,nv,128,128]
    float *out;                 // [B,T,nv,128]
    uint8_t *ws;
    int32_t B, T, nk, nv, nc;
    float q_scale;
    int32_t l2norm;
    // scan with the gated RMSNorm in its epilogue (out is then unused): z [B,T,nv,128] bf16, weight [128], bf16 result
    const uint16_t *z;
    const float *norm_w;
    uint16_t *out_norm;
    float norm_eps;
    int32_t b_base, b_count;  // the sequences this scan launch covers (all of them unless the launch is cooperative)
};

__device__ __forceinline__ half8 f32x8_to_half8(const float4v &a, const float4v &b) {
    half8 h;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        h[e] = (_Float16)a[e];
        h[4 + e] = (_Float16)b[e];
    }
    return h;
}

// ------------------------------------------------------------------------------------------------ prepare
constexpr int kPitchH = 136;  // halves per row of the row-major k / q tiles
constexpr int kPitchT = 72;   // halves per row of the transposed k / v tiles
constexpr int kPitchL = 68;   // halves per row of the 64x64 matrix L (fp16: it is only ever an MFMA operand)
constexpr int kPitchD = 20;   // floats per row of a 16x16 fp32 block (diagonal blocks of L / of the inverse, and their scratch)
constexpr int kBlockD = 16 * kPitchD;
// 51 KB, three workgroups per CU.  Region A holds the row-major k / q tiles, then the scratch blocks of the four
// inverses, then the transposed tiles; L (below its diagonal blocks) and the diagonal blocks live beside it.
constexpr int kLdsKh = 0, kLdsQh = 17408, kLdsKT = 0, kLdsVT = 18432;                   // region A: 36,864 B
constexpr int kLdsS = 0;                                                                // scratch blocks, 3 per wavefront 0-3
constexpr int kLdsL = 36864, kLdsD = kLdsL + 64 * kPitchL * 2, kLdsF = kLdsD + 4 * kBlockD * 4, kLdsBytes = kLdsF + 1536;
static_assert(kLdsBytes <= 54528, "three workgroups of the prepare kernel per CU");

// Transposed tiles [feature d][token]: the eight-token (16-byte) pieces of a row are permuted by d / 16, so that the
// threads of a wavefront, which write one token each for features 16 apart, hit different banks.
__device__ __forceinline__ int tpos(int d, int tok) { return d * kPitchT + ((((tok >> 3) ^ (d >> 4)) & 7) << 3) + (tok & 7); }

__global__ __launch_bounds__(512, 6) void deltanet_chunk_prepare_kernel(ChunkArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[kLdsBytes];
    _Float16 *kh = (_Float16 *)(lds + kLdsKh), *qh = (_Float16 *)(lds + kLdsQh);
    _Float16 *KT = (_Float16 *)(lds + kLdsKT), *VT = (_Float16 *)(lds + kLdsVT);
    _Float16 *Lh = (_Float16 *)(lds + kLdsL);  // L, strictly below its diagonal blocks
    float *Dm = (float *)(lds + kLdsD);        // the four diagonal blocks of L, later of N = (I - L)^-1
    float *Sm = (float *)(lds + kLdsS);        // scratch blocks of the inverses, once the k / q row tiles are dead
    float *gs = (float *)(lds + kLdsF), *bs = gs + 64, *Gs = gs + 128, *eG = gs + 192, *eGl = gs + 256, *be = gs + 320;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lq = lane >> 4;
    const int64_t unit = blockIdx.x;
    const int c = (int)(unit % a.nc);
    const int j = (int)((unit / a.nc) % a.nv);
    const int b = (int)(unit / ((int64_t)a.nc * a.nv));
    const int hk = j / (a.nv / a.nk);
    // chunk-major workspace: the workgroups of the scan kernel walk the chunks in step, so what they read at one
    // moment is one contiguous region spread over all memory channels (sequence-major, they would all sit at the
    // same offset of regions a fixed stride apart and queue up on a few channels)
    const int rep = a.nv / a.nk;
    uint8_t *wsc = a.ws + (int64_t)c * ((int64_t)a.B * a.nk * kHeadBytes + (int64_t)a.B * a.nv * kUnitBytes);
    uint8_t *wsh = wsc + ((int64_t)b * a.nk + hk) * kHeadBytes;  // written by the first v-head of the k-head
    uint8_t *wsu = wsc + (int64_t)a.B * a.nk * kHeadBytes + ((int64_t)b * a.nv + j) * kUnitBytes;
    const bool first_of_head = j % rep == 0;

    // ---- 1. load 64 tokens, normalise, stage: thread = (token tt, 16 consecutive elements)
    half8 kreg[2], vreg[2];  // this thread's k-hat and v, written transposed once the inverse is done
    const int tt = tid >> 3, part = tid & 7;
    {
        const int t = c * kC + tt;
        const bool valid = t < a.T;
        float kf[16], qf[16], vf[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) kf[e] = qf[e] = vf[e] = 0.0f;
        if (valid) {
            const int64_t bt = (int64_t)b * a.T + t;
            const uint16_t *kp = a.k + (bt * a.nk + hk) * kWD + 16 * part;
            const uint16_t *qp = a.q + (bt * a.nk + hk) * kWD + 16 * part;
            const uint16_t *vp = a.v + (bt * a.nv + j) * kWD + 16 * part;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const u32x4 kw = *(const u32x4 *)(kp + 8 * i), qw = *(const u32x4 *)(qp + 8 * i), vw = *(const u32x4 *)(vp + 8 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    kf[8 * i + 2 * e] = __uint_as_float(kw[e] << 16);
                    kf[8 * i + 2 * e + 1] = __uint_as_float(kw[e] & 0xffff0000u);
                    qf[8 * i + 2 * e] = __uint_as_float(qw[e] << 16);
                    qf[8 * i + 2 * e + 1] = __uint_as_float(qw[e] & 0xffff0000u);
                    vf[8 * i + 2 * e] = __uint_as_float(vw[e] << 16);
                    vf[8 * i + 2 * e + 1] = __uint_as_float(vw[e] & 0xffff0000u);
                }
            }
        }
        float kmul = 1.0f, qmul = a.q_scale;
        if (a.l2norm) {
            float sk = 0.0f, sq = 0.0f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                sk += kf[e] * kf[e];
                sq += qf[e] * qf[e];
            }
#pragma unroll
            for (int o = 1; o < 8; o <<= 1) {  // the eight threads of a token are eight consecutive lanes
                sk += __shfl_xor(sk, o, 64);
                sq += __shfl_xor(sq, o, 64);
            }
            kmul = 1.0f / fmaxf(sqrtf(sk), 1e-3f);
            qmul = a.q_scale / fmaxf(sqrtf(sq), 1e-3f);
        }
        half8 k8[2], q8[2];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const _Float16 kk = (_Float16)(kf[e] * kmul);
            k8[e >> 3][e & 7] = kk;
            q8[e >> 3][e & 7] = (_Float16)(qf[e] * qmul);
            vreg[e >> 3][e & 7] = (_Float16)vf[e];
        }
        kreg[0] = k8[0];
        kreg[1] = k8[1];
        *(half8 *)&kh[tt * kPitchH + 16 * part] = k8[0];
        *(half8 *)&kh[tt * kPitchH + 16 * part + 8] = k8[1];
        *(half8 *)&qh[tt * kPitchH + 16 * part] = q8[0];
        *(half8 *)&qh[tt * kPitchH + 16 * part + 8] = q8[1];
        if (part == 0) {
            gs[tt] = valid ? a.g[((int64_t)b * a.T + t) * a.nv + j] : 0.0f;
            bs[tt] = valid ? a.beta[((int64_t)b * a.T + t) * a.nv + j] : 0.0f;
        }
    }
    __syncthreads();

    // ---- 2. running sum of g and the decay factors (wavefront 0)
    if (wave == 0) {
        float x = gs[lane];
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float y = __shfl_up(x, o, 64);
            if (lane >= o) x += y;
        }
        const float g63 = __shfl(x, 63, 64);
        const float e = expf(x);
        Gs[lane] = x;
        eG[lane] = e;
        eGl[lane] = expf(g63 - x);
        be[lane] = bs[lane] * e;
        if (lane == 63) *(float *)(wsu + kOffDecay) = e;
#ifndef EXP_NOSENT
        float *ssq = (float *)(a.ws + a.nc * ((int64_t)a.B * a.nk * kHeadBytes + (int64_t)a.B * a.nv * kUnitBytes) +
                               ((int64_t)c * a.B * a.nv + (int64_t)b * a.nv + j) * kSsqBytes);
        ssq[lane] = -1.0f;  // both halves' exchange slots: nothing there yet
        ssq[64 + lane] = -1.0f;
#endif
    }

    // ---- 3. k k^T (rows i, columns j) and k q^T (rows j, columns i): wavefront w owns row tile w/2, column tiles 2(w%2), +1
    float4v kk[2], qk[2];
    const int mt = wave >> 1;
    {
#pragma unroll
        for (int x = 0; x < 2; ++x) {
            kk[x] = (float4v){0.f, 0.f, 0.f, 0.f};
            qk[x] = (float4v){0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const half8 ar = *(const half8 *)&kh[(16 * mt + li) * kPitchH + 32 * s + 8 * lq];
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                const int nt = 2 * (wave & 1) + x;
                const half8 bk = *(const half8 *)&kh[(16 * nt + li) * kPitchH + 32 * s + 8 * lq];
                const half8 bq = *(const half8 *)&qh[(16 * nt + li) * kPitchH + 32 * s + 8 * lq];
                kk[x] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ar, bk, kk[x], 0, 0, 0);
                qk[x] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ar, bq, qk[x], 0, 0, 0);
            }
        }
    }
    __syncthreads();  // G and the factors are visible
#pragma unroll
    for (int x = 0; x < 2; ++x) {
        const int nt = 2 * (wave & 1) + x;
        const int col = 16 * nt + li;
        const float gcol = Gs[col];
        half4v m;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = 16 * mt + 4 * lq + r;
            // L[i = row][j = col]: the diagonal blocks in fp32 for the inverse, the rest as the fp16 operand it will be
            const float lv = col < row ? -bs[row] * kk[x][r] * __builtin_amdgcn_exp2f((Gs[row] - gcol) * kLog2eC) : 0.0f;
            if (nt == mt) Dm[mt * kBlockD + (4 * lq + r) * kPitchD + li] = lv;
            else Lh[row * kPitchL + col] = (_Float16)lv;
            // masked q k^T: row = key j, col = query i, kept for j <= i
            m[r] = (_Float16)(row <= col ? qk[x][r] * __builtin_amdgcn_exp2f((gcol - Gs[row]) * kLog2eC) : 0.0f);
        }
        *(half4v *)(wsu + kOffQK + ((nt * 2 + (mt >> 1)) * 64 + lane) * 16 + 8 * (mt & 1)) = m;
    }
    // q as the A operand of q S: block (token tile, dk slab), lane (token li, group lq); the scan applies e^G
    if (first_of_head) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int item = tid + 512 * it, blk = item >> 6, ln = item & 63;
            const int tok = 16 * (blk >> 2) + (ln & 15), d0 = 32 * (blk & 3) + 4 * (ln >> 4);
            const half4v lo = *(const half4v *)&qh[tok * kPitchH + d0], hi = *(const half4v *)&qh[tok * kPitchH + d0 + 16];
            half8 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                o[e] = lo[e];
                o[4 + e] = hi[e];
            }
            *(half8 *)(wsh + kOffQh + (blk * 64 + ln) * 16) = o;
        }
    }
    if (tid < 64) {
        *(float *)(wsu + kOffEG + 4 * tid) = eG[tid];
        *(float *)(wsu + kOffEGl + 4 * tid) = eGl[tid];
    }
    __syncthreads();  // L complete; the row-major k / q tiles are dead from here on

    // ---- 4. the diagonal 16x16 blocks of N = (I - L)^-1: N_aa = (I + L)(I + L^2)(I + L^4)(I + L^8) with L = L_aa.
    //         Wavefront a < 4 does block a by itself -- six 16x16x16 products on MFMA (fp16 operands, fp32
    //         accumulation), the matrices passing through its own LDS blocks between products (the operations of
    //         one wavefront on LDS complete in order, so no workgroup barrier is needed until all four are done).
    if (wave < 4) {
        auto f4h = [](const float4v &x) { return (half4v){(_Float16)x[0], (_Float16)x[1], (_Float16)x[2], (_Float16)x[3]}; };
        // dst = (add ? add : 0) + X Y; lane (li, lq) holds rows 4 lq + r of column li of the result
        auto mm = [&](float *dst, const float *X, const float *Y, const float *add) {
            const half4v xa = f4h(*(const float4v *)&X[li * kPitchD + 4 * lq]);
            float4v yb, c;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                yb[r] = Y[(4 * lq + r) * kPitchD + li];
                c[r] = add ? add[(4 * lq + r) * kPitchD + li] : 0.0f;
            }
            c = __builtin_amdgcn_mfma_f32_16x16x16f16(xa, f4h(yb), c, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; ++r) dst[(4 * lq + r) * kPitchD + li] = c[r];
            __builtin_amdgcn_wave_barrier();
        };
        float *Lb = Dm + wave * kBlockD, *Nb = Sm + (3 * wave) * kBlockD, *Pb = Nb + kBlockD, *Qb = Pb + kBlockD;
#pragma unroll
        for (int r = 0; r < 4; ++r) Nb[(4 * lq + r) * kPitchD + li] = Lb[(4 * lq + r) * kPitchD + li] + (4 * lq + r == li ? 1.0f : 0.0f);
        __builtin_amdgcn_wave_barrier();
        mm(Qb, Lb, Lb, nullptr);  // L^2
        mm(Lb, Nb, Qb, Nb);       // (I + L)(I + L^2), into L's block (L itself is not needed any more)
        mm(Pb, Qb, Qb, nullptr);  // L^4
        mm(Nb, Lb, Pb, Lb);       // ... (I + L^4)
        mm(Qb, Pb, Pb, nullptr);  // L^8
        mm(Lb, Nb, Qb, Nb);       // ... (I + L^8): the inverse, where the diagonal block of L was
    }
    __syncthreads();

    // ---- 5. X = N [v beta | k beta e^G] by block forward substitution, X_a = N_aa (R_a + sum_{m<a} L_am X_m), on
    //         v_mfma_f32_16x16x16_f16.  A wavefront owns 32 columns (wavefronts 0-3: U, two dv tiles each; 4-7: W, the
    //         two dk tiles of one slab) and walks the four row blocks with X_m in registers: the accumulator layout
    //         of X_m (column li, rows 4 lq + r) is the B operand layout of the next level, so nothing is exchanged.
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        KT[tpos(16 * part + e, tt)] = kreg[e >> 3][e & 7];
        VT[tpos(16 * part + e, tt)] = vreg[e >> 3][e & 7];
    }
    __syncthreads();
    // k^T as the A operand of the state update: block (dk tile, token slab), lane (dk li, group lq); the scan
    // applies e^(G63 - G)
    if (first_of_head) {
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int item = tid + 512 * it, blk = item >> 6, ln = item & 63;
            const int dk = 16 * (blk >> 1) + (ln & 15), t0 = 32 * (blk & 1) + 4 * (ln >> 4);
            const half4v lo = *(const half4v *)&KT[tpos(dk, t0)], hi = *(const half4v *)&KT[tpos(dk, t0 + 16)];
            half8 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                o[e] = lo[e];
                o[4 + e] = hi[e];
            }
            *(half8 *)(wsh + kOffKt + (blk * 64 + ln) * 16) = o;
        }
    }
    __syncthreads();  // the transposed k tile has been read for the output above: its rows may be reused below
    {
        const bool is_w = wave >= 4;
        const _Float16 *T = is_w ? KT : VT;
        const float *fac = is_w ? be : bs;
        const int tile0 = 2 * (wave & 3);
        auto f4h = [](const float4v &x) { return (half4v){(_Float16)x[0], (_Float16)x[1], (_Float16)x[2], (_Float16)x[3]}; };
        half4v xh[2][4];
#pragma unroll
        for (int ra = 0; ra < 4; ++ra) {
#pragma unroll
            for (int x = 0; x < 2; ++x) {
                const int col = 16 * (tile0 + x) + li;
                const half4v rr = *(const half4v *)&T[tpos(col, 16 * ra + 4 * lq)];
                float4v acc;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[r] = (float)rr[r] * fac[16 * ra + 4 * lq + r];
#pragma unroll
                for (int m = 0; m < ra; ++m) {
                    const half4v la = *(const half4v *)&Lh[(16 * ra + li) * kPitchL + 16 * m + 4 * lq];
                    acc = __builtin_amdgcn_mfma_f32_16x16x16f16(la, xh[x][m], acc, 0, 0, 0);
                }
                const half4v na = f4h(*(const float4v *)&Dm[ra * kBlockD + li * kPitchD + 4 * lq]);
                const float4v xa = __builtin_amdgcn_mfma_f32_16x16x16f16(na, f4h(acc), (float4v){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                xh[x][ra] = f4h(xa);
                if (!is_w) *(half4v *)(wsu + kOffU + ((ra * 8 + tile0 + x) * 64 + lane) * 8) = xh[x][ra];
            }
        }
        if (is_w) {
            // -W as the A operand of the scan (row = token, k-slots = the slab's dk in accumulator order): element
            // (token 4 lq + r, dk li of tile x) belongs to lane (4 lq + r) + 16 (li / 4), slot li % 4 + 4 x.  Shuffled
            // through this wavefront's own 32 rows of the transposed k tile, which nobody reads any more.
            uint8_t *stg = (uint8_t *)(KT + (32 * (wave & 3)) * kPitchT);
#pragma unroll
            for (int ra = 0; ra < 4; ++ra)
#pragma unroll
                for (int x = 0; x < 2; ++x)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        *(_Float16 *)(stg + (ra * 64 + 4 * lq + r + 16 * (li >> 2)) * 16 + 2 * ((li & 3) + 4 * x)) = -xh[x][ra][r];
            __builtin_amdgcn_wave_barrier();  // LDS operations of one wavefront complete in order
#pragma unroll
            for (int ra = 0; ra < 4; ++ra)
                *(u32x4 *)(wsu + kOffWn + ((ra * 4 + (wave & 3)) * 64 + lane) * 16) = *(const u32x4 *)(stg + (ra * 64 + lane) * 16);
        }
    }
}

// --------------------------------------------------------------------------------------------------- scan
// Workgroup barrier that orders LDS traffic only: __syncthreads() would also wait for the operand prefetch of the
// next chunk, which is issued at the top of the loop and not needed before the next iteration.
__device__ __forceinline__ void lds_sync() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

constexpr int kYT = 2;  // 16-column tiles of the state per wavefront (a workgroup owns 64 of the 128 columns)
constexpr int kScanThreads = 640;      // eight computing wavefronts and two that only move operands
constexpr int kScanNormThreads = 768;  // ... and two that finish the output rows (NORM)
static_assert(kOpsFac == 28 * 128 * 16, "28 16-byte pieces per loader thread");

// Two workgroups per (sequence, v-head), 64 of the 128 state columns each (with one, half the CUs stay idle at
// B x nv = 128; the second reader of the common operands finds them in the L2 it shares with the first).
// Wavefront w < 8: token tile w % 4 (also the 32-row dk slab of the state it owns) x column tiles 2*(w / 4), +1.
// The A operands are common to the
// wavefronts of a token tile, so they are fetched once per workgroup, one chunk ahead, and handed round through
// LDS -- by wavefronts 8 and 9, which do nothing else: a wavefront that issues 1-KB loads waits behind the CU's
// address unit (measured: ~2500 cycles per chunk for the 72 KB), and a computing wavefront that waits there holds
// up every barrier of the chunk.  Only U is read by the wavefront that uses it.
// NORM: the gated RMSNorm of the layer (RMSNormGated, qwen3_5.rs:305-313) in the epilogue -- the output rows leave as
// bf16(o * rsqrt(mean(o^2) + eps) * w * silu(z)) instead of fp32 o.  A row's 128 columns belong to two workgroups, so
// each publishes the sums of squares of its 64 columns per chunk (the exchange slots; reset by the prepare kernel) at the start of
// the next chunk and reads the other's a chunk and a half later, long after it was written, so nothing waits.  Until
// then the rows of a chunk stay in LDS (four chunks deep), and two more wavefronts, which do nothing else, finish
// them: eight adjacent columns per lane with 16-byte loads of z and 16-byte stores (twelve wavefronts are still three
// per SIMD, so they cost the others no registers).  The two workgroups must be resident together: the host launches this instance cooperatively (all
// workgroups of a launch resident) and the wait for the other half is bounded all the same.
constexpr int kRing = 4;     // chunks of output rows waiting in LDS for the other half's sums
constexpr int kOPitch = 68;  // floats per staged output row: 64 columns + 4, so the four row groups of a store hit different banks
constexpr int kNormSpin = 1 << 16;  // about 0.1 s: the other half is resident and at most a chunk apart
// The scan kernel exists twice: deltanet_chunk_scan_kernel, and deltanet_chunk_scan_norm_kernel with the gated norm in
// its epilogue.  One text, deltanet_chunk_scan.inc, included once with HS_SCAN_NORM 0 and once with 1 -- not one
// template: with the norm's shared arrays, arguments or branches merely present (empty, unused or constant-false) the
// compiler laid out LDS and ordered the chunk loop of the plain kernel differently, and it ran 5 % slower.
#define HS_SCAN_NORM 0
#include "deltanet_chunk_scan.inc"
#undef HS_SCAN_NORM
#define HS_SCAN_NORM 1
#include "deltanet_chunk_scan.inc"
#undef HS_SCAN_NORM

}  // namespace hs

extern "C" {

size_t hs_deltanet_chunked_workspace_bytes(int32_t B, int32_t T, int32_t nk, int32_t nv) {
    if (B <= 0 || T <= 0 || nk <= 0 || nv <= 0) return 0;
    return (size_t)((T + hs::kC - 1) / hs::kC) * ((size_t)B * nk * hs::kHeadBytes + (size_t)B * nv * (hs::kUnitBytes + hs::kSsqBytes));
}

static int chunked_common(const void *q, const void *k, const void *v, const float *g, const float *beta, float *state,
                          int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk, int32_t dv, float q_scale, int l2norm,
                          void *workspace, size_t workspace_bytes, hs::ChunkArgs &a) {
    using namespace hs;
    if (B > 0 && T > 0 && (!q || !k || !v || !g || !beta || !state)) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (dk != kWD || dv != kWD) return fail(HS_ERR_INVALID_ARGUMENT, "deltanet is built for dk = dv = 128, got %d x %d", dk, dv);
    if (B < 0 || T < 0 || nk <= 0 || nv <= 0 || nv % nk != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "bad shape B=%d T=%d nk=%d nv=%d (need nv %% nk == 0)", B, T, nk, nv);
    if (B == 0 || T == 0) return HS_OK;
    const int64_t units = (int64_t)B * nv * ((T + kC - 1) / kC);
    if (units > INT32_MAX || (int64_t)B * nv > (1 << 29)) return fail(HS_ERR_INVALID_ARGUMENT, "too many chunks (%lld)", (long long)units);
    const size_t need = hs_deltanet_chunked_workspace_bytes(B, T, nk, nv);
    if (!workspace || workspace_bytes < need) return fail(HS_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    if ((((uintptr_t)workspace | (uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "q, k, v and the workspace must be 16-byte aligned");
    a = ChunkArgs{};
    a.q = (const uint16_t *)q; a.k = (const uint16_t *)k; a.v = (const uint16_t *)v;
    a.g = g; a.beta = beta; a.state = state; a.ws = (uint8_t *)workspace;
    a.B = B; a.T = T; a.nk = nk; a.nv = nv; a.nc = (T + kC - 1) / kC; a.q_scale = q_scale; a.l2norm = l2norm ? 1 : 0;
    a.b_base = 0; a.b_count = B;
    return -1;  // go on
}

int hs_deltanet_forward_chunked(const void *q, const void *k, const void *v, const float *g, const float *beta, float *state,
                                float *out, int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk, int32_t dv,
                                float q_scale, int l2norm, void *workspace, size_t workspace_bytes, hs_stream_t stream) {
    using namespace hs;
    if (B > 0 && T > 0 && !out) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    ChunkArgs a;
    if (int rc = chunked_common(q, k, v, g, beta, state, B, T, nk, nv, dk, dv, q_scale, l2norm, workspace, workspace_bytes, a); rc >= 0)
        return rc;
    a.out = out;
    hipStream_t st = (hipStream_t)stream;
    deltanet_chunk_prepare_kernel<<<(unsigned)((int64_t)B * nv * a.nc), 512, 0, st>>>(a);
    if (int rc = check_launch("deltanet_chunk_prepare")) return rc;
    deltanet_chunk_scan_kernel<<<(unsigned)(2 * B * nv), kScanThreads, 0, st>>>(a);
    return check_launch("deltanet_chunk_scan");
}

int hs_deltanet_forward_chunked_gated_norm(const void *q, const void *k, const void *v, const float *g, const float *beta,
                                           float *state, const void *z, const float *norm_weight, float norm_eps, void *out,
                                           int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk, int32_t dv,
                                           float q_scale, int l2norm, void *workspace, size_t workspace_bytes,
                                           hs_stream_t stream) {
    using namespace hs;
    if (B > 0 && T > 0 && (!out || !z || !norm_weight)) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    ChunkArgs a;
    if (int rc = chunked_common(q, k, v, g, beta, state, B, T, nk, nv, dk, dv, q_scale, l2norm, workspace, workspace_bytes, a); rc >= 0)
        return rc;
    if ((((uintptr_t)z | (uintptr_t)norm_weight | (uintptr_t)out) & 15) != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "z, norm_weight and out must be 16-byte aligned");
    a.z = (const uint16_t *)z; a.norm_w = norm_weight; a.norm_eps = norm_eps; a.out_norm = (uint16_t *)out;
    // The two workgroups of a (sequence, v-head) wait for each other once per chunk, so every workgroup of a scan
    // launch has to be resident: a cooperative launch, over as many whole sequences as the device holds at a time.
    // (what the device holds is looked up once per device; a second thread doing the same stores the same values)
    constexpr int kMaxDevices = 64;
    static int resident_of[kMaxDevices];  // 0: not asked yet, -1: no cooperative launches, else workgroups resident at once
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return fail(HS_ERR_LAUNCH, "cannot query the device for a cooperative launch");
    }
    if (resident_of[dev] == 0) {
        int cus = 0, per_cu = 0, coop = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            hipDeviceGetAttribute(&coop, hipDeviceAttributeCooperativeLaunch, dev) != hipSuccess ||
            hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, deltanet_chunk_scan_norm_kernel, kScanNormThreads, 0) != hipSuccess) {
            (void)hipGetLastError();
            return fail(HS_ERR_LAUNCH, "cannot query the device for a cooperative launch");
        }
        resident_of[dev] = coop ? std::max(1, cus * per_cu) : -1;
    }
    if (resident_of[dev] < 0)
        return fail(HS_ERR_LAUNCH, "the device does not support cooperative launches: run hs_deltanet_forward_chunked and hs_deltanet_gated_norm");
    const int64_t resident = resident_of[dev];
    if (resident < 2 * (int64_t)nv)
        return fail(HS_ERR_INVALID_ARGUMENT,
                    "%d v-heads need %d workgroups resident at once, the device holds %lld: run hs_deltanet_forward_chunked "
                    "and hs_deltanet_gated_norm", nv, 2 * nv, (long long)resident);
    hipStream_t st = (hipStream_t)stream;
    deltanet_chunk_prepare_kernel<<<(unsigned)((int64_t)B * nv * a.nc), 512, 0, st>>>(a);
    if (int rc = check_launch("deltanet_chunk_prepare")) return rc;
    const int per_launch = (int)std::min<int64_t>(B, resident / (2 * nv));
    for (int b0 = 0; b0 < B; b0 += per_launch) {
        a.b_base = b0;
        a.b_count = std::min(per_launch, B - b0);
        void *args[] = {&a};
        const hipError_t e = hipLaunchCooperativeKernel((const void *)deltanet_chunk_scan_norm_kernel, dim3((unsigned)(2 * a.b_count * nv)),
                                                        dim3(kScanNormThreads), args, 0, st);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return fail(HS_ERR_LAUNCH, "deltanet_chunk_scan (cooperative): %s", hipGetErrorString(e));
        }
    }
    return HS_OK;
}

}  // extern "C"
