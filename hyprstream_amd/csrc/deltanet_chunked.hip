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
constexpr int kOffSsq = 41728;   // 2 x 64 floats: per column half, the sums of squares of the chunk's output rows over that
                                 // half's 64 columns (the fused gated norm's exchange between the two halves; -1 = not there yet)
constexpr int kUnitBytes = 42240;
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
        *(float *)(wsu + kOffSsq + 4 * lane) = -1.0f;  // both halves' exchange slots: nothing there yet
        *(float *)(wsu + kOffSsq + 256 + 4 * lane) = -1.0f;
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
// each publishes the sums of squares of its 64 columns per chunk (kOffSsq; reset by the prepare kernel) at the start of
// the next chunk and reads the other's a chunk and a half later, long after it was written, so nothing waits.  Until
// then the rows of a chunk stay in LDS (four chunks deep), and two more wavefronts, which do nothing else, finish
// them: eight adjacent columns per lane with 16-byte loads of z and 16-byte stores (twelve wavefronts are still three
// per SIMD, so they cost the others no registers).  The two workgroups must be resident together: the host launches this instance cooperatively (all
// workgroups of a launch resident) and the wait for the other half is bounded all the same.
constexpr int kNormSpin = 1 << 16;  // about 0.1 s: the other half is resident and at most a chunk apart
template <bool NORM>
__global__ __launch_bounds__(NORM ? kScanNormThreads : kScanThreads) void deltanet_chunk_scan_kernel(ChunkArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t ops[kOpsBytes];          // this chunk's A operands and decay vectors
    __shared__ __attribute__((aligned(16))) uint8_t s_lds[4 * 4 * 64 * 16];  // S:  [dk slab][column tile][lane] 16 B
    __shared__ __attribute__((aligned(16))) uint8_t v_lds[2 * 4 * 64 * 16];  // V': [token slab][column tile][lane] 16 B
    constexpr int kOPitch = 68;  // floats per staged output row: 64 columns + 4, so the four row groups of a store hit different banks
    constexpr int kRing = 4;     // chunks of output rows waiting in LDS for the other half's sums
    __shared__ float ssq_lds[NORM ? kRing : 1][2][NORM ? 64 : 1];           // [chunk % kRing][column pair][token]
    __shared__ __attribute__((aligned(16))) float o_lds[NORM ? kRing : 1][NORM ? 64 : 1][NORM ? kOPitch : 4];  // [chunk % kRing][token][column]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lq = lane >> 4;
    // Workgroups go to the 8 XCDs round-robin by linear id, and each XCD has its own L2.  The two column halves of a
    // (sequence, v-head) read the same -W / masked q k^T, and all v-heads of a k-head (both halves of each) the same q and
    // k^T: the 2 * rep workgroups of a (sequence, k-head) get linear ids congruent mod 8, consecutive in that XCD's
    // order, so that each of those operands comes from HBM once and the other readers find it in L2.
    const int p = blockIdx.x, pairs = a.b_count * a.nv, rep = a.nv / a.nk;
    int pair, half;
    if (((a.b_count * a.nk) & 7) == 0) {
        const int i = p >> 3, per = 2 * rep;                   // position in the XCD's order; workgroups per k-head
        const int ku = (p & 7) + 8 * (i / per), sub = i % per;  // (sequence, k-head) unit; member of its group
        pair = ku * rep + (sub >> 1);
        half = sub & 1;
    } else if ((pairs & 7) == 0) {
        pair = (p & 7) + 8 * (p >> 4);
        half = (p >> 3) & 1;
    } else {
        pair = p >> 1;
        half = p & 1;
    }
    pair += a.b_base * a.nv;
    const int b = pair / a.nv, j = pair % a.nv;
    const int tw = wave & 3, cp = wave >> 2;
    const int64_t chunk_stride = (int64_t)a.B * a.nk * kHeadBytes + (int64_t)a.B * a.nv * kUnitBytes;
    const uint8_t *wsh = a.ws + ((int64_t)b * a.nk + j / (a.nv / a.nk)) * kHeadBytes;        // + ci * chunk_stride
    const uint8_t *wsp = a.ws + (int64_t)a.B * a.nk * kHeadBytes + (int64_t)pair * kUnitBytes;  // + ci * chunk_stride

    if (NORM && wave >= 10) {  // ---- the two wavefronts that finish the output rows
        const int lt = tid - 640;
        // Wavefront fw finishes token rows 32 fw .. 32 fw + 31 of a chunk, eight rows per instruction: lane = (row
        // 8 i + lane / 8, the eight columns 8 (lane % 8) .. + 7), so eight lanes cover a row's 128 bytes and every load
        // of z and store of the result moves whole lines.  Lane l also owns the sums of row 32 fw + l % 32.
        const int fw = lt >> 6, ecol = 8 * (lane & 7), rsub = lane >> 3, srow = 32 * fw + (lane & 31);
        float other = 0.0f;
        u32x4 zr[4];
        const float4v wa = *(const float4v *)(a.norm_w + 64 * half + ecol), wb = *(const float4v *)(a.norm_w + 64 * half + ecol + 4);
        const float wv[8] = {wa[0], wa[1], wa[2], wa[3], wb[0], wb[1], wb[2], wb[3]};
        // sums of squares of chunk c over this workgroup's 64 columns -> the exchange slots of this half.  Device-scope
        // stores and loads of single floats: nothing else has to be ordered.
        auto publish = [&](int c) {
            if (lane < 32) {
                float *slot = (float *)(a.ws + (wsp - a.ws) + c * chunk_stride + kOffSsq + 256 * half) + srow;
                __hip_atomic_store(slot, ssq_lds[c % kRing][0][srow] + ssq_lds[c % kRing][1][srow], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        };
        auto their_slot = [&](int c) { return (const float *)(wsp + c * chunk_stride + kOffSsq + 256 * (half ^ 1)) + srow; };
        auto elem = [&](int c, int i) {  // first of this lane's eight elements of row 8 i + rsub of its wavefront's rows
            const int t = min(c * kC + 32 * fw + 8 * i + rsub, a.T - 1);
            return (((int64_t)b * a.T + t) * a.nv + j) * kWD + 64 * half + ecol;
        };
        // what finishing chunk c needs from memory
        auto load_other = [&](int c) { other = __hip_atomic_load(their_slot(c), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
        auto load_z = [&](int c) {
#pragma unroll
            for (int i = 0; i < 4; ++i) zr[i] = __builtin_nontemporal_load((const u32x4 *)(a.z + elem(c, i)));
        };
        auto finish = [&](int c) {
            if (__builtin_amdgcn_ballot_w64(other < 0.0f) != 0) {  // not the normal case: the other half is chunks behind
                for (int spin = kNormSpin; spin > 0; --spin) {
                    __builtin_amdgcn_s_sleep(8);
                    other = __hip_atomic_load(their_slot(c), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (__builtin_amdgcn_ballot_w64(other < 0.0f) == 0) break;
                }
            }
            // a half that never arrived (its workgroup is not running: the launch was not cooperative) poisons the row
            const float ss = other >= 0.0f ? ssq_lds[c % kRing][0][srow] + ssq_lds[c % kRing][1][srow] + other : __builtin_nanf("");
            const float rrms_mine = 1.0f / sqrtf(ss / (float)kWD + a.norm_eps);  // of row srow
            typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 32 * fw + 8 * i + rsub;
                const float rrms = __shfl(rrms_mine, 8 * i + rsub, 64);
                const float4v xa = *(const float4v *)&o_lds[c % kRing][row][ecol], xb = *(const float4v *)&o_lds[c % kRing][row][ecol + 4];
                const float xv[8] = {xa[0], xa[1], xa[2], xa[3], xb[0], xb[1], xb[2], xb[3]};
                uint32_t o4[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const float z0 = __uint_as_float(zr[i][u] << 16), z1 = __uint_as_float(zr[i][u] & 0xffff0000u);
                    const float s0 = z0 * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z0 * -1.4426950408889634f));
                    const float s1 = z1 * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z1 * -1.4426950408889634f));
                    const bf16x2 pr = {(__bf16)(xv[2 * u] * rrms * wv[2 * u] * s0), (__bf16)(xv[2 * u + 1] * rrms * wv[2 * u + 1] * s1)};
                    o4[u] = __builtin_bit_cast(uint32_t, pr);
                }
                if (c * kC + row < a.T) __builtin_nontemporal_store((u32x4){o4[0], o4[1], o4[2], o4[3]}, (u32x4 *)(a.out_norm + elem(c, i)));
            }
        };
        // Chunk c: rows in LDS at the end of step c, sums published in round c + 1, the other half's sums and z
        // requested in round c + 2 (a chunk and a half after they were published), the rows finished in round c + 3 (a
        // chunk after the request): these wavefronts never wait for memory, so they never hold up a barrier.
        for (int ci = 0; ci < a.nc; ++ci) {
            lds_sync();  // the rows and sums of chunk ci - 1 are in LDS now
            if (ci > 0) publish(ci - 1);
            lds_sync();
            if (ci > 2) finish(ci - 3);
            if (ci > 1) {
                load_z(ci - 2);
                load_other(ci - 2);
            }
        }
        lds_sync();  // the last chunk's rows and sums are in LDS
        publish(a.nc - 1);
        if (a.nc > 2) finish(a.nc - 3);
        for (int c = max(a.nc - 2, 0); c < a.nc; ++c) {
            load_z(c);
            load_other(c);
            finish(c);
        }
        return;
    }
    if (wave >= 8) {  // ---- the two loader wavefronts
        // (Plain loads: these operands are shared with the other column half through L2, and the non-temporal hint
        // that helps the U loads and the output stores (scan 165 -> 152 us) cost 3 % here.  The prepare kernel's
        // workspace stores are plain too: with the hint it took the same time and wrote 5 % more.)
        // Region A of `ops` (-W, q and the decay vectors: 32.5 KB) is read between the two barriers of a chunk, region
        // B (k^T and the masked q k^T: 24 KB) after the second one.  So A of the next chunk is written after the second barrier, B of a chunk
        // after its first barrier -- neither write holds anybody up -- and each is fetched a whole chunk earlier.
        const int lt = tid - 512;
        u32x4 sa[16], sb[12];
        float fac = 0.0f;  // one of the 128 decay factors per loader thread
        auto fetch_a = [&](int ci) {
            const int64_t o = min(ci, a.nc - 1) * chunk_stride;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                sa[i] = *(const u32x4 *)(wsp + o + kOffWn + (lt + 128 * i) * 16);
                sa[8 + i] = *(const u32x4 *)(wsh + o + kOffQh + (lt + 128 * i) * 16);
            }
            fac = *(const float *)(wsp + o + kOffEG + 4 * lt);  // e^G (64 floats) then e^(G63-G) (64 floats)
        };
        auto fetch_b = [&](int ci) {
            const int64_t o = min(ci, a.nc - 1) * chunk_stride;
#pragma unroll
            for (int i = 0; i < 8; ++i) sb[i] = *(const u32x4 *)(wsh + o + kOffKt + (lt + 128 * i) * 16);
#pragma unroll
            for (int i = 0; i < 4; ++i) sb[8 + i] = *(const u32x4 *)(wsp + o + kOffQK + (lt + 128 * i) * 16);
        };
        auto park_a = [&]() {
#pragma unroll
            for (int i = 0; i < 16; ++i) *(u32x4 *)(ops + (lt + 128 * i) * 16) = sa[i];
            *(float *)(ops + kOpsFac + 4 * lt) = fac;
        };
        auto park_b = [&]() {
#pragma unroll
            for (int i = 0; i < 12; ++i) *(u32x4 *)(ops + kOpsKt + (lt + 128 * i) * 16) = sb[i];
        };
        fetch_a(0);
        fetch_b(0);
        park_a();
        fetch_a(1);
        for (int ci = 0; ci < a.nc; ++ci) {
            lds_sync();  // A of chunk ci is visible; nobody reads B of chunk ci - 1 any more
            park_b();
            fetch_b(ci + 1);
            lds_sync();  // B of chunk ci is visible; nobody reads A of chunk ci any more
            park_a();
            fetch_a(ci + 2);
        }
        if constexpr (NORM) lds_sync();  // the hand-over of the last chunk's rows (every wavefront takes part)
        return;
    }

    float4v S[2][kYT];  // [dk tile 2*tw + x][column tile kYT*cp + y]
    float *sp = a.state + ((int64_t)pair * kWD) * kWD + 64 * half + 16 * kYT * cp + li;
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
        for (int y = 0; y < kYT; ++y)
#pragma unroll
            for (int r = 0; r < 4; ++r) S[x][y][r] = sp[(int64_t)(16 * (2 * tw + x) + 4 * lq + r) * kWD + 16 * y];

    u32x2 uu[kYT], un[kYT];
    float decay, decay_n;
    auto fetch = [&](int ci) {
        const uint8_t *u = wsp + ci * chunk_stride;
#pragma unroll
        for (int y = 0; y < kYT; ++y) un[y] = __builtin_nontemporal_load((const u32x2 *)(u + kOffU + ((tw * 8 + 4 * half + kYT * cp + y) * 64 + lane) * 8));
        decay_n = *(const float *)(u + kOffDecay);
    };
    auto park = [&]() {
#pragma unroll
        for (int y = 0; y < kYT; ++y) uu[y] = un[y];
        decay = decay_n;
    };
    auto opA = [&](int off, int blk) { return *(const half8 *)(ops + off + (blk * 64 + lane) * 16); };

    fetch(0);
    park();
    // One chunk.  `guard`: the chunk may reach past T (only the last one can); full chunks store without a predicate.
    auto step = [&](int ci, auto guard_tag) {
        constexpr bool guard = decltype(guard_tag)::value;
        fetch(min(ci + 1, a.nc - 1));  // the last iteration re-reads its own chunk: one path through the loop
        // S as the B operand of W S and q S
#pragma unroll
        for (int y = 0; y < kYT; ++y)
            *(half8 *)(s_lds + ((tw * 4 + kYT * cp + y) * 64 + lane) * 16) = f32x8_to_half8(S[0][y], S[1][y]);
        lds_sync();  // also: the loaders have parked this chunk's -W and q e^G
        // decay vectors (region A of the buffer: read them before the second barrier).  e^G of this lane's token row;
        // e^(G63-G) of the tokens that are the k-slots of the state update: 32 s + 4 lq + e and 32 s + 16 + 4 lq + e
        const _Float16 eg_row = (_Float16)*(const float *)(ops + kOpsFac + 4 * (16 * tw + li));
        half8 egl[2];
#pragma unroll
        for (int s = 0; s < 2; ++s)
            egl[s] = f32x8_to_half8(*(const float4v *)(ops + kOpsFac + 256 + 4 * (32 * s + 4 * lq)),
                                    *(const float4v *)(ops + kOpsFac + 256 + 4 * (32 * s + 16 + 4 * lq)));
        float4v vp[kYT], o[kYT];
#pragma unroll
        for (int y = 0; y < kYT; ++y) {
            const half4v u4 = __builtin_bit_cast(half4v, uu[y]);
            vp[y] = (float4v){(float)u4[0], (float)u4[1], (float)u4[2], (float)u4[3]};
            o[y] = (float4v){0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const half8 wn = opA(kOpsWn, tw * 4 + s), qp = opA(kOpsQh, tw * 4 + s) * eg_row;
#pragma unroll
            for (int y = 0; y < kYT; ++y) {
                const half8 sb = *(const half8 *)(s_lds + ((s * 4 + kYT * cp + y) * 64 + lane) * 16);
                vp[y] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wn, sb, vp[y], 0, 0, 0);
                o[y] = __builtin_amdgcn_mfma_f32_16x16x32_f16(qp, sb, o[y], 0, 0, 0);
            }
        }
        // V' (this wavefront's 16 tokens) as half of a B operand block
#pragma unroll
        for (int y = 0; y < kYT; ++y) {
            half4v h;
#pragma unroll
            for (int r = 0; r < 4; ++r) h[r] = (_Float16)vp[y][r];
            *(half4v *)(v_lds + (((tw >> 1) * 4 + kYT * cp + y) * 64 + lane) * 16 + 8 * (tw & 1)) = h;
        }
        lds_sync();
        const float dec = decay;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const half8 qk = opA(kOpsQK, tw * 2 + s), kd0 = opA(kOpsKt, (2 * tw) * 2 + s) * egl[s], kd1 = opA(kOpsKt, (2 * tw + 1) * 2 + s) * egl[s];
#pragma unroll
            for (int y = 0; y < kYT; ++y) {
                if (s == 0) {
                    S[0][y] *= dec;
                    S[1][y] *= dec;
                }
                const half8 vb = *(const half8 *)(v_lds + ((s * 4 + kYT * cp + y) * 64 + lane) * 16);
                o[y] = __builtin_amdgcn_mfma_f32_16x16x32_f16(qk, vb, o[y], 0, 0, 0);
                S[0][y] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kd0, vb, S[0][y], 0, 0, 0);
                S[1][y] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kd1, vb, S[1][y], 0, 0, 0);
            }
        }
        if constexpr (!NORM) {
#pragma unroll
            for (int y = 0; y < kYT; ++y)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int t = ci * kC + 16 * tw + 4 * lq + r;
                    if (!guard || t < a.T) __builtin_nontemporal_store(o[y][r], &a.out[(((int64_t)b * a.T + t) * a.nv + j) * kWD + 64 * half + 16 * (kYT * cp + y) + li]);
                }
        } else {
            // the rows wait in LDS for the other half's sums; their sums of squares over this wavefront's 32 columns too
            float4v sq = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int y = 0; y < kYT; ++y) {
                sq += o[y] * o[y];
#pragma unroll
                for (int r = 0; r < 4; ++r) o_lds[ci % kRing][16 * tw + 4 * lq + r][16 * (kYT * cp + y) + li] = o[y][r];
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
#pragma unroll
                for (int sh = 1; sh < 16; sh <<= 1) sq[r] += __shfl_xor(sq[r], sh, 64);
            }
            if (li == 0) *(float4v *)&ssq_lds[ci % kRing][cp][16 * tw + 4 * lq] = sq;
        }
        park();
    };
    const int nfull = a.T / kC;
    for (int ci = 0; ci < nfull; ++ci) step(ci, std::false_type());
    if (nfull < a.nc) step(nfull, std::true_type());
    if constexpr (NORM) lds_sync();  // hands the last chunk's rows to the finishing wavefronts
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
        for (int y = 0; y < kYT; ++y)
#pragma unroll
            for (int r = 0; r < 4; ++r) sp[(int64_t)(16 * (2 * tw + x) + 4 * lq + r) * kWD + 16 * y] = S[x][y][r];
}

}  // namespace hs

extern "C" {

size_t hs_deltanet_chunked_workspace_bytes(int32_t B, int32_t T, int32_t nk, int32_t nv) {
    if (B <= 0 || T <= 0 || nk <= 0 || nv <= 0) return 0;
    return (size_t)((T + hs::kC - 1) / hs::kC) * ((size_t)B * nk * hs::kHeadBytes + (size_t)B * nv * hs::kUnitBytes);
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
    deltanet_chunk_scan_kernel<false><<<(unsigned)(2 * B * nv), kScanThreads, 0, st>>>(a);
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
    a.z = (const uint16_t *)z; a.norm_w = norm_weight; a.norm_eps = norm_eps; a.out_norm = (uint16_t *)out;
    // The two workgroups of a (sequence, v-head) wait for each other once per chunk, so every workgroup of a scan
    // launch has to be resident: a cooperative launch, over as many whole sequences as the device holds at a time.
    int dev = 0, cus = 0, per_cu = 0, coop = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipDeviceGetAttribute(&coop, hipDeviceAttributeCooperativeLaunch, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, deltanet_chunk_scan_kernel<true>, kScanNormThreads, 0) != hipSuccess) {
        (void)hipGetLastError();
        return fail(HS_ERR_LAUNCH, "cannot query the device for a cooperative launch");
    }
    if (!coop) return fail(HS_ERR_LAUNCH, "the device does not support cooperative launches: run hs_deltanet_forward_chunked and hs_deltanet_gated_norm");
    const int64_t resident = (int64_t)cus * per_cu;
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
        const hipError_t e = hipLaunchCooperativeKernel((const void *)deltanet_chunk_scan_kernel<true>, dim3((unsigned)(2 * a.b_count * nv)),
                                                        dim3(kScanNormThreads), args, 0, st);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return fail(HS_ERR_LAUNCH, "deltanet_chunk_scan (cooperative): %s", hipGetErrorString(e));
        }
    }
    return HS_OK;
}

}  // extern "C"
