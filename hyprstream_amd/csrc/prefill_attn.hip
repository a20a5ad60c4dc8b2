// Causal prefill attention on the MFMA pipe with online softmax (gfx950, wave64).
//
// One call serves S new tokens per sequence (a prompt, or one chunk of a chunked prefill).  Query
// row i sits at absolute position hist_len + i and attends
//   (1) the hist_len tokens already in the cache (int8 with token scales, or e4m3fn with head scales),
//       dequantized on the fly, and
//   (2) new tokens 0..=i in exact bf16,
// which is softmax(Q K^T * scale + causal mask) V over [history | this call's K/V].
//
// Work split (numbers for head_dim 128; head_dim 256 is the same template with half the columns per wavefront
// and twice the operand blocks per key step, head_dim 64 with the same columns and half the operand blocks, see
// PShape).  A 512-thread workgroup (8 wavefronts, 2 per SIMD)
// owns 256 (query, head) columns of
// one kv-head -- with G = Hq/Hkv >= 4: 64 consecutive queries x 4 query heads -- and walks the keys,
// 64 per step.  Every step's K and V tiles are
// converted ONCE per workgroup into ready-to-issue MFMA A operands in LDS (blocks of 64 lanes x 16 B:
// per 32 keys K as 2 tiles x 4 k-groups, V^T as 8 row groups) by the eight wavefronts together,
// double-buffered, one barrier per step; each wavefront then reads the operands with conflict-free
// ds_read_b128 and uses each one for its two 16-column blocks.
// Grid = (query tiles, kv-heads x head groups, sequences).
//
// Products (both on v_mfma_f32_16x16x32, keys on the M axis, columns on N):
//   S^T[key, col]  = sum_d K[key, d] Q[col, d]
//   O^T[d, col]   += sum_key V^T[d, key] P^T[key, col]
// History part: f16 MFMA.  The eight wavefronts that convert a tile apply the scales while they are at it, so
// the LDS operands are fp16(code * scale) and the consumers see plain K and V.  New-token part: bf16 MFMA
// straight from the caller's bf16 K/V, V^T built with permutes, P rounded to bf16.  In both parts Q carries
// the softmax scale and log2(e), the score accumulators start from minus the softmax reference, and the row
// sums are one more MFMA with a ones operand.  Softmax and accumulation are fp32; the score layout of the first
// product is the B-operand layout of the second, so P stays in its lanes.  The fp16 operands are taken
// relative to a power-of-two reference per (sequence, kv-head) (see the history phase), so the absolute magnitude of
// the cache does not matter; a row whose scale is more than 2^11 times that head's reference saturates.
#include <climits>
#include <type_traits>

#include "prefill_common.hpp"

namespace hs {

// head_dim 128 or 256.  What a wavefront holds is the same for both: its output tile is (16 kNB columns) x D, so
// D = 256 halves the columns of a wavefront (and of a workgroup: 128 instead of 256) and doubles the operand
// blocks of a key step.
template <int D> struct PShape {
    static constexpr int kNB = D == 256 ? 1 : 2;  // 16-column blocks per wavefront
    static constexpr int KG = D / 32;             // K operand blocks per 16-key tile (32 d each)
    static constexpr int VB = D / 16;             // V^T operand blocks per 32 keys (16 rows of d each)
    static constexpr int DW = D < 128 ? D : 128;  // width of a group of d: what one pass of the producers and of the output loop covers
    static constexpr int NC = D / DW;             // groups of d
    static constexpr int VBG = DW / 16;           // V^T operand blocks of a group: block bb holds rows d = VBG * li + bb
};
template <int D> struct alignas(16) StepTile {
    uint8_t k[2 * PShape<D>::KG][1024];  // block KG*u + j: K tile u (16 keys), k-group j; 64 lanes x 16 B in MFMA lane order
    uint8_t v[PShape<D>::VB][1024];      // block 8*c + bb: V^T rows d = 128*c + 8*li + bb, 32 keys
};

template <int D> struct alignas(16) HistTile {
    StepTile<D> h[2];  // keys 0..31 and 32..63 of a 64-key step (history or new tokens)
};

// A step of one wavefront (64 keys, as two 32-key tiles) is
//   scores  : S^T = K Q^T                     -- MFMA, operands from LDS
//   softmax : P from S, running max and sum   -- VALU only
//   output  : O^T += V^T P^T                  -- MFMA, operands from LDS
// with one workgroup barrier per step: while tile s is consumed every wavefront converts its share of tile s+1
// into the other buffer and starts the global loads of tile s+2.
// What was measured on this loop (gfx950, two wavefronts per SIMD): an MFMA 16x16x32 occupies the SIMD's
// vector issue port for about half of its 16 cycles, plain vector instructions run in its shadow (two per MFMA
// are free), v_exp_f32 one per MFMA, while v_dot2_f32_f16 stalls the matrix pipe (row sums are therefore an
// MFMA with a ones operand, not dot products or additions).  Variants that paired the matrix work of one
// wavefront with the vector work of the other behind a second barrier per step, or that software-pipelined
// scores(s+1) against softmax(s) inside one wavefront, were correct but not faster than this order; steps of
// 64 keys instead of 32 were (the per-step bookkeeping is shared by twice the MFMAs).
// kPD: head_dim (64, 128 or 256; PShape); FP8: the history holds e4m3fn codes with head scales instead of int8 codes
// with token scales.
// kCols: 16-column blocks per wavefront if not PShape's (1 at head_dim 128: half the columns per workgroup, for grids
// that would leave most CUs without a workgroup).
// kWin: the instance with a sliding window (the checks it adds to every step cost the plain instance 2 % at 4 x 4096
// tokens, so they are compiled in only where a window is asked for).
// kWaves: 8, or 16 wavefronts of one 16-column block each (kCols = 1, head_dim 128): the same 256 columns per workgroup
// on four wavefronts per SIMD with at most 128 registers; wavefronts 0-7 then convert K, wavefronts 8-15 V.
// kSplit: the 64-key steps of a query tile (history, then the call's own tokens) are cut into a.nsplit equal runs, one
// workgroup each (blockIdx.x = tile * nsplit + part).  Every part writes its unnormalised accumulators, softmax
// reference and row sums to the workspace and counts itself in at the tile's counter; the part that finds all others
// already there adds their partials to its registers, normalises and stores.  Nobody waits for anybody.  For calls
// whose tiles are too few to occupy the CUs (a chunk of one sequence).
// kShadow: the history comes from the bf16 operand-order copy of the prompt's dequantized K/V (PrefillArgs::shadow)
// instead of the codes: whole 32 KB step images go global -> LDS (no registers, no conversion) into a ring of four
// buffers, three steps ahead, and are consumed by the bf16 products of the new-token phase.  head_dim 128, full width.
template <int kPD, bool FP8, int kCols = 0, bool kWin = false, int kWaves = 8, bool kSplit = false, bool kShadow = false>
__global__ __launch_bounds__(64 * kWaves, kWaves == 16 ? 4 : 2) void prefill_attn_kernel(PrefillArgs a) {
    static_assert(!kShadow || (kPD == 128 && !kWin && kWaves == 8), "shadow history: head_dim 128, eight wavefronts, no window");
    static_assert(kWaves == 8 || (kWaves == 16 && kCols == 1 && kPD == 128), "sixteen wavefronts: one column block each, head_dim 128");
    static_assert(!kSplit || (!kWin && kWaves == 8), "key split: eight wavefronts, no window");
    constexpr int kNB = kCols ? kCols : PShape<kPD>::kNB, KG = PShape<kPD>::KG, VB = PShape<kPD>::VB, NC = PShape<kPD>::NC;
    constexpr int DW = PShape<kPD>::DW, VBG = PShape<kPD>::VBG;
    constexpr int kRow = kPD;  // elements per row of q, k, v, out and of the cache
    // head_dim 64: a 16-key K tile is 1 KB, one load instruction of a wavefront, and a step's V rows are half as many
    // 8-byte pieces -- wavefronts 0-3 convert K (a tile each), wavefronts 4-7 convert V.  Otherwise every wavefront
    // converts an eighth of both.
    constexpr bool kSplitRoles = kPD == 64;
    typedef HistTile<kPD> HistTile;
    __shared__ __attribute__((aligned(16))) uint8_t lds[(kShadow ? 4 : 2) * sizeof(HistTile)];  // two step buffers (shadow history: a ring of four)
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: wavefront-dependent branches stay uniform
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
            if (a.heavy_first) bx = X - 1 - bx;  // late query tiles have the most keys: start them first
            by = grp % gridDim.y;
            bz = grp / gridDim.y;
        }
    }
    int part = 0;
    if constexpr (kSplit) {
        part = bx % a.nsplit;
        bx /= a.nsplit;
    }
    const int b = bz;
    const int groups = (a.G + a.HG - 1) / a.HG;  // the last group of a kv-head may be partly padding (G = 3, 5, 6, 7 ...)
    const int kvh = by / groups, hg = by % groups;
    const int S = a.S, H = a.hist_lens ? min(max(a.hist_lens[b], 0), a.hist_len) : a.hist_len;
    const int q_per_wg = 16 * (kNB * kWaves / a.HG);
    const int q0 = bx * q_per_wg;
    if (q0 >= S) return;
    const int wg_qlast = min(S - 1, q0 + q_per_wg - 1);
    // key split: this part's run of the tile's history steps [h_lo, h_hi) and new-token steps [n_lo, n_hi)
    int h_lo = 0, h_hi = 0, n_lo = 0, n_hi = 0;
    if constexpr (kSplit) {
        const int hn = (H + 63) / 64, total = hn + wg_qlast / 64 + 1;
        const int g0 = total * part / a.nsplit, g1 = total * (part + 1) / a.nsplit;
        h_lo = min(g0, hn);
        h_hi = min(g1, hn);
        n_lo = max(g0 - hn, 0);
        n_hi = max(g1 - hn, 0);
    }

    int head[kNB], qi[kNB];
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
        const int bi = kNB * wave + nb;
        head[nb] = kvh * a.G + min(hg * a.HG + bi % a.HG, a.G - 1);  // a padding column repeats the group's last head
        qi[nb] = q0 + 16 * (bi / a.HG) + li;
    }
    const int wv_q0 = q0 + 16 * ((kNB * wave) / a.HG);  // first query of this wavefront
    const int wv_qlast = min(S - 1, q0 + 16 * ((kNB * wave + kNB - 1) / a.HG) + 15);
    const bool wv_active = wv_q0 < S;
    // Sliding window: the query in-call index i sees the keys whose distance to it is below W.  The first visible key
    // of the workgroup's (wavefront's) first query bounds where the walks start; steps below a wavefront's bound are
    // skipped by that wavefront, steps that a bound cuts through take the masking path of the softmax.
    const int W = kWin && a.window > 0 ? a.window : (1 << 30);
    // in-call index of the first key column nb sees (negative: that many history tokens back)
    auto qlo = [&](int nb) { return min(qi[nb], S - 1) - W + 1; };
    const int wg_lo = q0 - W + 1, wv_lo = wv_q0 - W + 1, wv_lo_last = wv_qlast - W + 1;

    // q arrives as projected: its QK-norm and rotation run here, once per workgroup.  A lane's piece of the row is the
    // piece its Q operands are made of, so the history phase takes it from registers; the row also goes to the
    // workgroup's own rows of `out` (which nobody else touches before the final store), where the new-token phase reads
    // it back -- each lane exactly what it wrote.  (Measured at 4 x 512 tokens per launch, Llama-flavour norm and
    // whole-head rotation: 10 us per launch, half of it arithmetic; the same code as loops over 8-element groups, which
    // is a fifth of the instructions, took 15 us: every iteration waits for its own loads.)
    // (Key split: several workgroups, possibly on different XCDs, share the tile's rows of `out`, and a staged row left
    // dirty in one XCD's L2 could be written back over the final output stored from another.  The runs therefore stage
    // their q pieces in their own record of the workspace and `out` is touched by the merging workgroup alone.)
    constexpr int kSplitThreads = 64 * kWaves, kSplitSlots = kNB * VB + 1 + kNB * KG;  // 16-byte slots per thread and run
    int tile_id = 0;
    u32x4 *qstage = nullptr;
    if constexpr (kSplit) {
        tile_id = (bz * gridDim.y + by) * (gridDim.x / a.nsplit) + bx;
        qstage = (u32x4 *)a.split_ws + (((int64_t)tile_id * a.nsplit + part) * kSplitSlots + kNB * VB + 1) * kSplitThreads + threadIdx.x;
    }
    const uint16_t *qsrc = a.q;
    u32x4 qpre[kNB][KG];
    if (a.qpro.on) {
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb) {
            const int qrow = min(qi[nb], S - 1);
            const int64_t row = (((int64_t)b * S + qrow) * a.Hq + head[nb]) * kRow;
            prologue_row_part<kPD, 8 * KG>(a.qpro, a.q + row, head[nb], H + qrow, lq, 16, lane, qpre[nb]);
#pragma unroll
            for (int j = 0; j < KG; ++j) {
                if constexpr (kSplit) qstage[(nb * KG + j) * kSplitThreads] = qpre[nb][j];
                else *(u32x4 *)(a.out + row + 8 * KG * lq + 8 * j) = qpre[nb][j];
            }
        }
        qsrc = a.out;
    }

    float4v acc[kNB][VB];
    float m_run[kNB];
    float4v l_run[kNB];  // row sums, kept on the matrix pipe: ones(16x32) x P^T, every register holds the column's sum
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
        m_run[nb] = -INFINITY;
        l_run[nb] = (float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < VB; ++i) acc[nb][i] = (float4v){0.f, 0.f, 0.f, 0.f};
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
                for (int i = 0; i < VB; ++i) acc[nb][i] *= alpha;
                m_run[nb] = m_new;
            }
        }
    };

    // A column that has seen no key yet (everything so far masked) has no reference: its lanes keep sending the
    // wavefront through the branch that sets one, because the common path would accumulate weights that the first
    // real reference then scales by exp2(-inf).
    auto pending = [&]() {
        int f = INT_MIN;
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb)
            if (m_run[nb] == -INFINITY) f = INT_MAX;
        return f;
    };
    const int obase = lane * 16;  // this lane's 16 bytes inside an operand block
    const float qscale = a.scale_log2e;
    const bool late = __builtin_amdgcn_readfirstlane((wave >> 2) & 1) != 0;  // wavefronts w and w+4 share a SIMD
    const int pw = kWaves == 16 ? wave & 7 : wave;  // index among the wavefronts of this one's producer role
    float vup = 1.0f;  // 2^E of the history's V operands, folded back into the accumulators when the history ends

    // =============================== history: int8 cache, f16 MFMA ===============================
    if (!kShadow && H > 0 && (!kSplit || h_lo < h_hi)) {
        // The history operands are fp16(code * scale), and fp16 spans 2^-14 .. 65504 only.  Each (sequence, kv-head)
        // therefore gets a power-of-two reference for K and one for V, taken from the largest scale among its first
        // cached tokens (int8; up to 64 of them, inside one block) or from its head scale (fp8): operands are
        // fp16(code * scale * 2^-E), with that reference scale landing in [1/8, 1/4).  K's 2^E goes into the Q
        // operands, V's into the accumulators when the history ends -- both exact.  What matters is then a scale's
        // size RELATIVE to the head's own: rows up to 2^11 above the reference and down to 2^-11 below it keep full
        // precision, whatever the absolute magnitude of the cache.
        float kdown = 1.0f, kup = 1.0f, vdown = 1.0f;
        {
            float rk, rv;
            if (FP8) {
                rk = a.ks[(int64_t)b * a.Hkv + kvh];
                rv = a.vs[(int64_t)b * a.Hkv + kvh];
            } else {
                int64_t unit;
                int slot;
                resolve(a.ka, b, 0, unit, slot);
                int n = min(min(H, 64), a.ka.capacity_tokens - slot);
                rk = a.ks[unit * a.ka.scale_stride_seq + (int64_t)kvh * a.ka.scale_stride_head + slot + min(lane, n - 1)];
                resolve(a.va, b, 0, unit, slot);
                n = min(min(H, 64), a.va.capacity_tokens - slot);
                rv = a.vs[unit * a.va.scale_stride_seq + (int64_t)kvh * a.va.scale_stride_head + slot + min(lane, n - 1)];
                rk = wave_max(rk);
                rv = wave_max(rv);
            }
            auto ref_exp = [](float r) {  // E with r * 2^-E in [1/8, 1/4); 0 for a zero or non-finite reference
                int e = 0;
                if (r > 0.0f && r < 3.0e38f) {
                    (void)frexpf(r, &e);
                    e = min(max(e + 2, -100), 100);
                }
                return __builtin_amdgcn_readfirstlane(e);
            };
            const int ek = ref_exp(rk), ev = ref_exp(rv);
            kdown = ldexpf(1.0f, -ek);
            kup = ldexpf(1.0f, ek);
            vdown = ldexpf(1.0f, -ev);
            vup = ldexpf(1.0f, ev);
        }
        // Q operands carry the softmax scale and log2(e) and K's reference: qop = fp16(q * scale * log2e * 2^E * 2^-ex),
        // so the MFMA result is the score in log2 units times 2^-ex.  ex is zero unless a column's scaled |q| would
        // leave the range fp16 holds well (then the wavefront takes the path that multiplies the scores by cq = 2^ex).
        half8 qop[kNB][KG];
        float cq[kNB];
        bool scaled = false;
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb) {
            const uint16_t *qp = qsrc + (((int64_t)b * S + min(qi[nb], S - 1)) * a.Hq + head[nb]) * kRow + 8 * KG * lq;
            float qf[8 * KG], amax = 0.0f;
#pragma unroll
            for (int i = 0; i < KG; ++i) {
                const u32x4 w = a.qpro.on ? qpre[nb][i] : *(const u32x4 *)(qp + 8 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    qf[8 * i + 2 * e] = __uint_as_float(w[e] << 16) * qscale * kup;
                    qf[8 * i + 2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u) * qscale * kup;
                }
            }
#pragma unroll
            for (int i = 0; i < 8 * KG; ++i) amax = fmaxf(amax, fabsf(qf[i]));
            amax = quad_max(amax);
            int ex = 0;
            if ((amax > 32768.0f || amax < 0.0009765625f) && amax > 0.0f && amax < 3.0e38f) (void)frexpf(amax, &ex);
            scaled |= ex != 0;
#pragma unroll
            for (int j = 0; j < KG; ++j)
#pragma unroll
                for (int e = 0; e < 8; ++e) qop[nb][j][e] = (_Float16)ldexpf(qf[8 * j + e], -ex);
            cq[nb] = ldexpf(1.0f, ex);
        }
        scaled = __builtin_amdgcn_ballot_w64(scaled) != 0;

        // A history step covers 64 keys: two 32-key tiles (halves) in the layout of StepTile.  The work that comes
        // once per step whatever its size -- barrier, loop and address bookkeeping, the overflow check, waits --
        // is shared by twice as many MFMAs as in a 32-key step.
        constexpr int kHStep = 64;
        const int nsteps = kSplit ? h_hi : (H + kHStep - 1) / kHStep;
        const int st0 = kSplit ? h_lo : kWin ? min(max(H + wg_lo, 0) / kHStep, nsteps) : 0;  // first step that holds a key some query of the workgroup sees
        HistTile *htiles = (HistTile *)lds;
        // ---- producers: every wavefront converts one eighth of the step's K tiles and of its V tiles.
        //      K: wavefront w takes 16-key block u4 = w/2 and the d-halves jp = w%2 of every 32-d group: lane
        //         (li, lq) loads the 16 codes K[16u4 + li][32lq + 16jp ..] and writes operand blocks j = 2jp and
        //         2jp+1 of tile u4/2 (eight codes = the d's of Q operand j each).
        //      V: lane = (d-octet x = lane%16, key pair pp = 4w + lane/16).  Pair pp = 16hh + 4g + pe of tile hh:
        //         slots 2pe, 2pe+1 of key group g are the adjacent keys 16*(pe/2) + 4g + 2*(pe%2), +1; eight
        //         bytes of each give the fp16 pairs for d = 8x + bb, stored in block bb at operand lane (x, g).
        //      The per-token scales are applied here, once per workgroup, rather than to every score and weight:
        //      the operands are fp16(code * scale) (relative rounding 2^-11, finer than a bf16 cache would keep).
        // (head_dim 64: eight d-octets per row, so a wavefront covers eight key pairs and wavefronts 4-7 the 32 of a
        //  step; d = 8x + bb lives in block bb % 4 at operand lane 2x + bb / 4.  K: wavefront w < 4 takes tile w whole.)
        const int vx = kSplitRoles ? lane & 7 : lane & 15;
        const int vpp = kSplitRoles ? 8 * (wave & 3) + (lane >> 3) : 4 * pw + (lane >> 4);
        const int vhh = vpp >> 4, vg = (vpp >> 2) & 3, vpe = vpp & 3;
        const int vkey = 32 * vhh + 16 * (vpe >> 1) + 4 * vg + 2 * (vpe & 1);
        const int vdst = ((kSplitRoles ? 2 * vx : vx) + 16 * vg) * 16 + 4 * vpe;
        const int ku4 = kSplitRoles ? wave & 3 : pw >> 1, kjp = kSplitRoles ? 0 : pw & 1;
        const bool does_k = kWaves == 16 ? wave < 8 : (!kSplitRoles || wave < 4), does_v = kWaves == 16 ? wave >= 8 : (!kSplitRoles || wave >= 4);
        const int krow = 16 * ku4 + li, kcol = 8 * KG * lq + 16 * kjp, vcol = 8 * vx;
        const uint32_t koff = krow * kRow + kcol, voff = vkey * kRow + vcol;
        // head_dim 256: the same lane also takes the d-halves jp + 2 (32 codes further) and the d-octet x + 16
        u32x4 rawk[NC];
        u32x2 rawv[NC][2];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            rawk[c] = (u32x4){0u, 0u, 0u, 0u};
            rawv[c][0] = rawv[c][1] = (u32x2){0u, 0u};
        }
        float rawsk = 0.0f, rawsv[2] = {0.0f, 0.0f};
        if (FP8) {  // one scale per (sequence, kv-head); the codes convert to value/256 (see e4m3_high_bytes_to_f16)
            rawsk = 256.0f * a.ks[(int64_t)b * a.Hkv + kvh];
            rawsv[0] = rawsv[1] = 256.0f * a.vs[(int64_t)b * a.Hkv + kvh];
        }
        const float kdn = kdown, vdn = vdown;
        // issue() is called for steps 0, 1, 2, ... in order, so the (scalar) addresses of a step's codes and
        // scales advance by a constant; a block table is consulted only when a cursor leaves its block.
        const uint8_t *kb = a.kc, *vb = a.vc;
        const float *ksp = a.ks, *vsp = a.vs;
        int kleft = 0, vleft = 0;  // tokens between the cursor and the end of its storage unit
        auto issue = [&](int step) {
            const int t0 = step * kHStep;
            const int last = H - 1 - t0;
            if (kleft <= 0) {
                int64_t unit;
                int slot;
                resolve(a.ka, b, t0, unit, slot);
                kb = a.kc + unit * a.ka.code_stride_seq + (int64_t)kvh * a.ka.code_stride_head + (int64_t)slot * kRow;
                if (!FP8) ksp = a.ks + unit * a.ka.scale_stride_seq + (int64_t)kvh * a.ka.scale_stride_head + slot;
                kleft = a.ka.capacity_tokens - slot;
            }
            if (vleft <= 0) {
                int64_t unit;
                int slot;
                resolve(a.va, b, t0, unit, slot);
                vb = a.vc + unit * a.va.code_stride_seq + (int64_t)kvh * a.va.code_stride_head + (int64_t)slot * kRow;
                if (!FP8) vsp = a.vs + unit * a.va.scale_stride_seq + (int64_t)kvh * a.va.scale_stride_head + slot;
                vleft = a.va.capacity_tokens - slot;
            }
            // The loaded values are only touched in commit(): nothing waits for a load here.  Addresses are the
            // step's (scalar) base plus a 32-bit lane offset; only the last, partial step clamps rows.
            uint32_t ko = koff, vo0 = voff, vo1 = voff + kRow, sk = 4u * krow, sv = 4u * vkey;
            uint32_t sv1 = sv + 4u;
            if (last < kHStep - 1) {
                ko = min(krow, last) * kRow + kcol;
                vo0 = min(vkey, last) * kRow + vcol;
                vo1 = min(vkey + 1, last) * kRow + vcol;
                sk = 4u * min(krow, last);
                sv = 4u * min(vkey, last);
                sv1 = 4u * min(vkey + 1, last);
            }
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (does_k) rawk[c] = *(const u32x4 *)(kb + ko + 32 * c);
                if (does_v) {
                    rawv[c][0] = *(const u32x2 *)(vb + vo0 + 128 * c);
                    rawv[c][1] = *(const u32x2 *)(vb + vo1 + 128 * c);
                }
            }
            if (!FP8) {
                if (does_k) rawsk = *(const float *)((const uint8_t *)ksp + sk);
                if (does_v) {
                    rawsv[0] = *(const float *)((const uint8_t *)vsp + sv);
                    rawsv[1] = *(const float *)((const uint8_t *)vsp + sv1);
                }
            }
            kb += kHStep * kRow; vb += kHStep * kRow;
            ksp += kHStep; vsp += kHStep;
            kleft -= kHStep; vleft -= kHStep;
        };
        auto commit = [&](HistTile &t, int step) {
            const int last = H - 1 - step * kHStep;  // keys past the end become zero rows
            float fk = rawsk * kdn, fv0 = rawsv[0] * vdn, fv1 = rawsv[1] * vdn;
            if (last < kHStep - 1) {  // the last, partial step only
                if (krow > last) fk = 0.0f;
                if (vkey > last) fv0 = 0.0f;
                if (vkey + 1 > last) fv1 = 0.0f;
            }
            // largest operand: 127 * scale (int8), 1.75 * 256 * scale (fp8), scale relative to the head's reference:
            // rows more than 2^11 above it saturate here instead of overflowing
            const float smax = FP8 ? 64.0f * kMaxScale : kMaxScale;
            const _Float16 sk = (_Float16)fminf(fk, smax);
            const _Float16 bias = (_Float16)1152.0f;
            const half2v sv = {(_Float16)fminf(fv0, smax), (_Float16)fminf(fv1, smax)};
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (does_k) {
                    uint8_t *kd = t.h[ku4 >> 1].k[KG * (ku4 & 1) + 2 * kjp + 4 * c] + obase;
                    if (FP8) {
                        *(half8 *)kd = e4m3x8_to_f16_div256(rawk[c][0], rawk[c][1]) * sk;
                        *(half8 *)(kd + 1024) = e4m3x8_to_f16_div256(rawk[c][2], rawk[c][3]) * sk;
                    } else {
                        *(half8 *)kd = (int8x8_to_f16_biased(rawk[c][0], rawk[c][1]) - bias) * sk;
                        *(half8 *)(kd + 1024) = (int8x8_to_f16_biased(rawk[c][2], rawk[c][3]) - bias) * sk;
                    }
                }
                if (does_v) {
#pragma unroll
                    for (int bb = 0; bb < 8; ++bb) {
                        const uint32_t pair = FP8 ? e4m3_pair_to_f16_div256(rawv[c][0][bb >> 2], rawv[c][1][bb >> 2], bb & 3)
                                                  : int8_pair_to_f16(rawv[c][0][bb >> 2], rawv[c][1][bb >> 2], bb & 3);
                        const half2v hv = __builtin_bit_cast(half2v, pair) * sv;
                        *(uint32_t *)(t.h[vhh].v[VBG * c + bb % VBG] + vdst + 16 * (bb / VBG)) = __builtin_bit_cast(uint32_t, hv);
                    }
                }
            }
        };
        float4v s[kNB][4];    // scores of the step: key block u4 = 2*half + u
        half8 pop[kNB][2];    // P^T operands per half
        constexpr int KU = kPD == 128 && kWaves == 8 ? 2 : 1;  // 16-key tiles whose K operands are read at once
        half8 kop[KU * KG], vop[VBG];
        half8 ones;
#pragma unroll
        for (int e = 0; e < 8; ++e) ones[e] = (_Float16)1.0f;
        float sref[kNB];
        float4v sinit[kNB];
        int force = INT_MAX;  // takes the first step through the branch that sets the reference
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb) {
            sref[nb] = 0.0f;
            sinit[nb] = (float4v){0.f, 0.f, 0.f, 0.f};
        }
        auto scores = [&](const HistTile &t) {
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
#pragma unroll
                for (int u0 = 0; u0 < 2; u0 += KU) {
#pragma unroll
                    for (int i = 0; i < KU * KG; ++i) kop[i] = *(const half8 *)(t.h[hh].k[KG * u0 + i] + obase);
#pragma unroll
                    for (int u = u0; u < u0 + KU; ++u) {
#pragma unroll
                        for (int nb = 0; nb < kNB; ++nb) s[nb][2 * hh + u] = sinit[nb];
#pragma unroll
                        for (int j = 0; j < KG; ++j)
#pragma unroll
                            for (int nb = 0; nb < kNB; ++nb)
                                s[nb][2 * hh + u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kop[KG * (u - u0) + j], qop[nb][j], s[nb][2 * hh + u], 0, 0, 0);
                    }
                }
            }
        };
        // V^T operands of half hh, 128-wide group c of d; output() consumes them and, for head_dim 256, goes on to
        // the second group by itself
        // (sixteen wavefronts: the operands are read four at a time where they are used, to stay within 128 registers)
        auto load_v = [&](const HistTile &t, int hh, int c = 0) {
            if constexpr (kWaves == 16) return;
#pragma unroll
            for (int i = 0; i < VBG; ++i) vop[i] = *(const half8 *)(t.h[hh].v[VBG * c + i] + obase);
        };
        auto output = [&](const HistTile &t, int hh) {
            if constexpr (kWaves == 16) {
#pragma unroll
                for (int q4 = 0; q4 < VBG; q4 += 4) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) vop[i] = *(const half8 *)(t.h[hh].v[q4 + i] + obase);
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[0][q4 + i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vop[i], pop[0][hh], acc[0][q4 + i], 0, 0, 0);
                }
                return;
            }
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (c > 0) load_v(t, hh, c);
#pragma unroll
                for (int bb = 0; bb < VBG; ++bb)
#pragma unroll
                    for (int nb = 0; nb < kNB; ++nb)
                        acc[nb][VBG * c + bb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vop[bb], pop[nb][hh], acc[nb][VBG * c + bb], 0, 0, 0);
            }
        };
        // softmax(): e = exponent of each weight (score in log2 units minus sref).  The common step only checks,
        // per lane and on the bit patterns (a positive float orders like its bits; a NaN reads as large), whether
        // any exponent exceeds kPShift, i.e. whether a score passed m_run; only then, at the first step and at a
        // partial last step does the wavefront reduce the column maxima and move the reference.
        auto softmax_for = [&](auto scaled_tag) {
            constexpr bool kScaled = decltype(scaled_tag)::value;
            return [&](int step) {
                const int lim = H - step * kHStep;  // keys of this step that exist
                const bool edge = kWin && step * kHStep < H + wv_lo_last;  // the window of some query starts inside or after this step
                float e[kNB][16];
                int over = force;
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb) {
#pragma unroll
                    for (int u4 = 0; u4 < 4; ++u4)
#pragma unroll
                        for (int r = 0; r < 4; ++r) e[nb][4 * u4 + r] = kScaled ? s[nb][u4][r] * cq[nb] : s[nb][u4][r];
#pragma unroll
                    for (int i = 0; i < 16; ++i) over = max(over, __float_as_int(e[nb][i]));
                }
                const bool slow = __builtin_amdgcn_ballot_w64(over > __float_as_int(kPShift)) != 0;
                if (slow || lim < kHStep || edge) {
                    float mx[kNB];
#pragma unroll
                    for (int nb = 0; nb < kNB; ++nb) {
                        if (lim < kHStep) {
#pragma unroll
                            for (int u4 = 0; u4 < 4; ++u4)
#pragma unroll
                                for (int r = 0; r < 4; ++r)
                                    if (4 * lq >= lim - (16 * u4 + r)) e[nb][4 * u4 + r] = -INFINITY;
                        }
                        if (edge) {
                            const int first = H + qlo(nb) - step * kHStep - 4 * lq;  // key offsets 16u4 + r below this are out of the window
#pragma unroll
                            for (int u4 = 0; u4 < 4; ++u4)
#pragma unroll
                                for (int r = 0; r < 4; ++r)
                                    if (16 * u4 + r < first) e[nb][4 * u4 + r] = -INFINITY;
                        }
                        float m = e[nb][0];
#pragma unroll
                        for (int i = 1; i < 16; ++i) m = fmaxf(m, e[nb][i]);
                        mx[nb] = quad_max(m) + sref[nb];  // the column's largest score of this step, log2 units
                    }
                    raise_max(mx);
                    force = pending();
#pragma unroll
                    for (int nb = 0; nb < kNB; ++nb) {
                        const float nref = (m_run[nb] == -INFINITY) ? 0.0f : m_run[nb] - kPShift;
                        const float d = nref - sref[nb];
#pragma unroll
                        for (int i = 0; i < 16; ++i) e[nb][i] -= d;
                        sref[nb] = nref;
                        const float c0 = kScaled ? -nref / cq[nb] : -nref;
                        sinit[nb] = (float4v){c0, c0, c0, c0};
                    }
                }
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
                    for (int hh = 0; hh < 2; ++hh) {
                        uint32_t pk[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const half2v h = {(_Float16)__builtin_amdgcn_exp2f(e[nb][8 * hh + 2 * i]),
                                              (_Float16)__builtin_amdgcn_exp2f(e[nb][8 * hh + 2 * i + 1])};
                            pk[i] = __builtin_bit_cast(uint32_t, h);
                        }
                        pop[nb][hh] = pack_half8(pk[0], pk[1], pk[2], pk[3]);
                        l_run[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pop[nb][hh], l_run[nb], 0, 0, 0);
                    }
            };
        };
        // One barrier per step: while tile s is consumed every wavefront converts its share of tile s+1 into
        // the other buffer and starts the global loads of tile s+2.  The second wavefront of each SIMD does its
        // conversion at the end of the step instead of the beginning, so that its matrix phases tend to meet
        // the other one's vector phases.
        // Eight wavefronts: operand reads run kAhead blocks ahead of the products that use them, through a ring of eight
        // registers, in a pinned order (see the copy-fed walk of the new-token phase for what that is worth).  A half of a
        // step holds NKB = 2 KG blocks of K (tile-major) and NVB = VB blocks of V^T.
        constexpr bool kRing = kWaves == 8;
        constexpr int kAhead = 6, NKB = 2 * KG, NVB = VB;
        half8 ring[8];
        auto kblk = [&](const HistTile &t, int k) { return *(const half8 *)(t.h[k / NKB].k[k % NKB] + obase); };
        auto vblk = [&](const HistTile &t, int k) { return *(const half8 *)(t.h[k / NVB].v[k % NVB] + obase); };
        auto scores_ahead = [&](const HistTile &t) {  // leaves the first V blocks in the ring
#pragma unroll
            for (int k = 0; k < kAhead; ++k) ring[k] = kblk(t, k);
#pragma unroll
            for (int k = 0; k < 2 * NKB; ++k) {
                if (k + kAhead < 2 * NKB) ring[(k + kAhead) & 7] = kblk(t, k + kAhead);
                else if (k + kAhead - 2 * NKB < 2 * NVB) ring[(k + kAhead) & 7] = vblk(t, k + kAhead - 2 * NKB);
                __builtin_amdgcn_sched_barrier(0);
                const int tile = 2 * (k / NKB) + (k % NKB) / KG, j = k % KG;
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb)
                    s[nb][tile] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ring[k & 7], qop[nb][j], j == 0 ? sinit[nb] : s[nb][tile], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        auto output_ahead = [&](const HistTile &t) {  // V^T block k of the step sits in ring slot (2 NKB + k) % 8
#pragma unroll
            for (int k = 0; k < 2 * NVB; ++k) {
                if (k + kAhead < 2 * NVB) ring[(2 * NKB + k + kAhead) & 7] = vblk(t, k + kAhead);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb)
                    acc[nb][k % NVB] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ring[(2 * NKB + k) & 7], pop[nb][k / NVB], acc[nb][k % NVB], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        auto walk = [&](auto softmax) {
            if (st0 >= nsteps) return;  // the window of every query of the workgroup starts after the history
            issue(st0);
            commit(htiles[st0 & 1], st0);
            if (st0 + 1 < nsteps) issue(st0 + 1);
            lds_barrier();
            for (int st = st0; st < nsteps; ++st) {
                if (!late) {
                    if (st + 1 < nsteps) commit(htiles[(st + 1) & 1], st + 1);
                    if (st + 2 < nsteps) issue(st + 2);
                }
                const HistTile &t = htiles[st & 1];
                if (!kWin || st * kHStep + kHStep > H + wv_lo) {  // else: no query of this wavefront sees a key of the step
                    if constexpr (kRing) {
                        scores_ahead(t);
                        softmax(st);
                        output_ahead(t);
                    } else {
                        scores(t);
                        load_v(t, 0);
                        softmax(st);
                        output(t, 0);
                        load_v(t, 1);
                        output(t, 1);
                    }
                }
                if (late) {
                    if (st + 1 < nsteps) commit(htiles[(st + 1) & 1], st + 1);
                    if (st + 2 < nsteps) issue(st + 2);
                }
                lds_barrier();
            }
        };
        if (scaled)
            walk(softmax_for(std::true_type{}));
        else
            walk(softmax_for(std::false_type{}));
        if (vup != 1.0f) {
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
                for (int i = 0; i < VB; ++i) acc[nb][i] *= vup;
        }
    }

    // =============================== new tokens: bf16, causal ===============================
    // (with the bf16 copy, the history steps of this workgroup run in here too, ahead of the call's own tokens)
    const bool hist_here = kShadow && H > 0 && (!kSplit || h_lo < h_hi), new_here = !kSplit || n_lo < n_hi;
    if (hist_here || new_here) {
        // Q operands carry the softmax scale and log2(e), rounded back to bf16 (2^-9 relative, the precision the
        // weights are rounded to anyway), so that the MFMA result needs no multiplication; as in the history
        // phase the score accumulators start from -sref and the common step only checks for an overflow.
        bf16x8 qop[kNB][KG];
        float sref[kNB];
        float4v sinit[kNB];
        int force = pending();  // columns that have seen nothing yet: their first step sets the reference
        if (a.qpro.on) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the finished q rows this lane stored to `out`
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb) {
            const uint16_t *qp = qsrc + (((int64_t)b * S + min(qi[nb], S - 1)) * a.Hq + head[nb]) * kRow + 8 * KG * lq;
#pragma unroll
            for (int j = 0; j < KG; ++j) {
                const u32x4 w = kSplit && a.qpro.on ? qstage[(nb * KG + j) * kSplitThreads] : *(const u32x4 *)(qp + 8 * j);
                uint32_t o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    o[e] = pack_bf16x2(__uint_as_float(w[e] << 16) * qscale, __uint_as_float(w[e] & 0xffff0000u) * qscale);
                qop[nb][j] = pack_bf16x8(o[0], o[1], o[2], o[3]);
            }
            sref[nb] = (m_run[nb] == -INFINITY) ? 0.0f : m_run[nb] - kPShift;
            sinit[nb] = (float4v){-sref[nb], -sref[nb], -sref[nb], -sref[nb]};
        }
        // 64 keys per step, as two 32-key tiles in the layout of the history phase.
        constexpr int kNStep = 64;
        const int nsteps = kSplit ? n_hi : wg_qlast / kNStep + 1;
        const int st0 = kSplit ? n_lo : kWin ? max(wg_lo, 0) / kNStep : 0;  // first step with a key inside the window of the workgroup's first query
        HistTile *ntiles = (HistTile *)lds;
        const uint16_t *knb = a.kn + ((int64_t)b * S * a.Hkv + kvh) * kRow;
        const uint16_t *vnb = a.vn + ((int64_t)b * S * a.Hkv + kvh) * kRow;
        const int64_t rstride = (int64_t)a.Hkv * kRow;  // elements between consecutive tokens
        // producers, split as in the history phase (bf16 rows are operands as they are): wavefront w copies the
        // 16-key block u4 = w/2, d-halves jp = w%2 (32 bytes per lane = operand blocks 2jp and 2jp+1); for V a lane
        // takes the d-octet x = lane%16 of two adjacent keys (16 bytes of each) and stores the eight (key, key+1)
        // bf16 pairs of d = 8x + bb into block bb.
        // (head_dim 64: eight d-octets per row, so a wavefront covers eight key pairs and wavefronts 4-7 the 32 of a
        //  step; d = 8x + bb lives in block bb % 4 at operand lane 2x + bb / 4.  K: wavefront w < 4 takes tile w whole.)
        const int vx = kSplitRoles ? lane & 7 : lane & 15;
        const int vpp = kSplitRoles ? 8 * (wave & 3) + (lane >> 3) : 4 * pw + (lane >> 4);
        const int vhh = vpp >> 4, vg = (vpp >> 2) & 3, vpe = vpp & 3;
        const int vkey = 32 * vhh + 16 * (vpe >> 1) + 4 * vg + 2 * (vpe & 1);
        const int vdst = ((kSplitRoles ? 2 * vx : vx) + 16 * vg) * 16 + 4 * vpe;
        const int ku4 = kSplitRoles ? wave & 3 : pw >> 1, kjp = kSplitRoles ? 0 : pw & 1;
        const bool does_k = kWaves == 16 ? wave < 8 : (!kSplitRoles || wave < 4), does_v = kWaves == 16 ? wave >= 8 : (!kSplitRoles || wave >= 4);
        const int krow = 16 * ku4 + li, kcol = 8 * KG * lq + 16 * kjp, vcol = 8 * vx;
        const uint32_t koff = krow * (uint32_t)rstride + kcol, voff = vkey * (uint32_t)rstride + vcol;  // elements
        u32x4 rawk[NC][2], rawv[NC][2];  // head_dim 256: also the d-halves jp + 2 (32 elements on) and the d-octet x + 16
#pragma unroll
        for (int c = 0; c < NC; ++c) rawk[c][0] = rawk[c][1] = rawv[c][0] = rawv[c][1] = (u32x4){0u, 0u, 0u, 0u};
        auto issue = [&](int step) {
            const int t0 = step * kNStep;
            const uint16_t *kp, *vp0, *vp1;
            if (t0 + kNStep <= S) {  // full step: scalar base + this lane's fixed offsets
                const uint16_t *kb = knb + (int64_t)t0 * rstride, *vb = vnb + (int64_t)t0 * rstride;
                kp = kb + koff;
                vp0 = vb + voff;
                vp1 = vb + voff + (uint32_t)rstride;
            } else {  // rows past the last token repeat it; the causal mask removes them
                kp = knb + (int64_t)min(t0 + krow, S - 1) * rstride + kcol;
                vp0 = vnb + (int64_t)min(t0 + vkey, S - 1) * rstride + vcol;
                vp1 = vnb + (int64_t)min(t0 + vkey + 1, S - 1) * rstride + vcol;
            }
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (does_k) {
                    rawk[c][0] = *(const u32x4 *)(kp + 32 * c);
                    rawk[c][1] = *(const u32x4 *)(kp + 32 * c + 8);
                }
                if (does_v) {
                    rawv[c][0] = *(const u32x4 *)(vp0 + 128 * c);
                    rawv[c][1] = *(const u32x4 *)(vp1 + 128 * c);
                }
            }
        };
        auto commit = [&](HistTile &t) {
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (does_k) {
                    uint8_t *kd = t.h[ku4 >> 1].k[KG * (ku4 & 1) + 2 * kjp + 4 * c] + obase;
                    *(u32x4 *)kd = rawk[c][0];
                    *(u32x4 *)(kd + 1024) = rawk[c][1];
                }
                if (does_v) {
#pragma unroll
                    for (int bb = 0; bb < 8; ++bb)
                        *(uint32_t *)(t.h[vhh].v[VBG * c + bb % VBG] + vdst + 16 * (bb / VBG)) = pick_halves(rawv[c][0][bb >> 1], rawv[c][1][bb >> 1], bb & 1);
                }
            }
        };
        float4v s[kNB][4];
        bf16x8 pop[kNB][2];
        // Halves of step `step` that hold a key some query of this wavefront may see (0: the step is skipped).
        auto halves = [&](int step) {
            if (!wv_active || step * kNStep > wv_qlast || (kWin && step * kNStep + kNStep <= wv_lo)) return 0;
            return step * kNStep + 32 > wv_qlast ? 1 : 2;
        };
        constexpr int KU = kPD == 128 && kWaves == 8 ? 2 : 1;  // 16-key tiles whose K operands are read at once
        bf16x8 kop[KU * KG], vop[VBG], ones;
#pragma unroll
        for (int e = 0; e < 8; ++e) ones[e] = (__bf16)1.0f;
        auto scores = [&](const HistTile &t, int nh) {
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                if (hh >= nh) break;
#pragma unroll
                for (int u0 = 0; u0 < 2; u0 += KU) {
#pragma unroll
                    for (int i = 0; i < KU * KG; ++i) kop[i] = *(const bf16x8 *)(t.h[hh].k[KG * u0 + i] + obase);
#pragma unroll
                    for (int u = u0; u < u0 + KU; ++u) {
#pragma unroll
                        for (int nb = 0; nb < kNB; ++nb) s[nb][2 * hh + u] = sinit[nb];
#pragma unroll
                        for (int j = 0; j < KG; ++j)
#pragma unroll
                            for (int nb = 0; nb < kNB; ++nb)
                                s[nb][2 * hh + u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[KG * (u - u0) + j], qop[nb][j], s[nb][2 * hh + u], 0, 0, 0);
                    }
                }
            }
        };
        // (sixteen wavefronts: the operands are read four at a time where they are used, to stay within 128 registers)
        auto load_v = [&](const HistTile &t, int hh, int c = 0) {
            if constexpr (kWaves == 16) return;
#pragma unroll
            for (int i = 0; i < VBG; ++i) vop[i] = *(const bf16x8 *)(t.h[hh].v[VBG * c + i] + obase);
        };
        auto output = [&](const HistTile &t, int hh) {
            if constexpr (kWaves == 16) {
#pragma unroll
                for (int q4 = 0; q4 < VBG; q4 += 4) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) vop[i] = *(const bf16x8 *)(t.h[hh].v[q4 + i] + obase);
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[0][q4 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop[i], pop[0][hh], acc[0][q4 + i], 0, 0, 0);
                }
                return;
            }
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (c > 0) load_v(t, hh, c);
#pragma unroll
                for (int bb = 0; bb < VBG; ++bb)
#pragma unroll
                    for (int nb = 0; nb < kNB; ++nb)
                        acc[nb][VBG * c + bb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vop[bb], pop[nb][hh], acc[nb][VBG * c + bb], 0, 0, 0);
            }
        };
        // hist_lim: -1 for a step of the call's own tokens; for a step of the shadow history, the number of its keys that
        // exist (all 64 but in the last step): every query sees those and nothing else of the step.
        // kind 0: a step of the call's own tokens.  Shadow history: 1 = a whole step (every query sees every key: no
        // mask code at all -- as a run-time flag the compiler turned the masks into 64 selects per step), 2 = the last,
        // partial step, of which hist_lim keys exist.
        auto softmax = [&](int step, int nh, auto kind_tag, int hist_lim = -1) {
            constexpr int kKind = decltype(kind_tag)::value;
            const int t0 = step * kNStep;
            // some (key, query) pair of this step is in the future, or out of the query's window
            const bool diag = kKind == 1 ? false : kKind == 2 ? true : (t0 + kNStep - 1 > wv_q0 || (kWin && t0 < wv_lo_last));
            float e[kNB][16];
            int over = force;
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
#pragma unroll
                for (int u4 = 0; u4 < 4; ++u4)
#pragma unroll
                    for (int r = 0; r < 4; ++r) e[nb][4 * u4 + r] = (u4 < 2 * nh) ? s[nb][u4][r] : -INFINITY;
                if (kKind != 1 && diag) {
                    const int qrel = (kKind == 2 ? hist_lim - 1 : min(qi[nb], S - 1) - t0) - 4 * lq;  // key offsets 16u4 + r beyond this are in the future
#pragma unroll
                    for (int u4 = 0; u4 < 4; ++u4)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (16 * u4 + r > qrel || (kWin && 16 * u4 + r < qrel - W + 1)) e[nb][4 * u4 + r] = -INFINITY;
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) over = max(over, __float_as_int(e[nb][i]));
            }
            if (__builtin_amdgcn_ballot_w64(over > __float_as_int(kPShift)) != 0) {
                float mx[kNB];
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb) {
                    float m = e[nb][0];
#pragma unroll
                    for (int i = 1; i < 16; ++i) m = fmaxf(m, e[nb][i]);
                    mx[nb] = quad_max(m) + sref[nb];
                }
                raise_max(mx);
                force = pending();
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb) {
                    const float nref = (m_run[nb] == -INFINITY) ? 0.0f : m_run[nb] - kPShift;
                    const float d = nref - sref[nb];
#pragma unroll
                    for (int i = 0; i < 16; ++i) e[nb][i] -= d;
                    sref[nb] = nref;
                    sinit[nb] = (float4v){-nref, -nref, -nref, -nref};
                }
            }
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    if (hh >= nh) break;
                    float p[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) p[i] = __builtin_amdgcn_exp2f(e[nb][8 * hh + i]);
                    pop[nb][hh] = pack_bf16x8(pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]), pack_bf16x2(p[6], p[7]));
                    l_run[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pop[nb][hh], l_run[nb], 0, 0, 0);
                }
        };
        if constexpr (kShadow) {
            if (hist_here) {
                // wavefront w moves bytes [4096 w, 4096 w + 4096) of a step image: four 1 KB pieces, lane i its 16 bytes
                const int hs0 = kSplit ? h_lo : 0, hsteps = kSplit ? h_hi : (H + 63) / 64;  // this workgroup's run of history steps
                const uint8_t *img = (const uint8_t *)a.shadow + ((int64_t)b * a.Hkv + kvh) * a.shadow_steps * (int64_t)kShadowStepBytes + 4096 * wave + 16 * lane;
                typedef __attribute__((address_space(3))) void *lds_ptr;
                auto fetch = [&](int hs) {
                    const uint8_t *src = img + (int64_t)hs * kShadowStepBytes;
                    uint8_t *dst = lds + (hs & 3) * kShadowStepBytes + 4096 * wave;
#pragma unroll
                    for (int i = 0; i < 4; ++i) __builtin_amdgcn_global_load_lds(src + 1024 * i, (lds_ptr)(dst + 1024 * i), 16, 0, 0);
                };
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the Q rows above: the counts below are of step pieces only)
#pragma unroll
                for (int i = 0; i < 3; ++i)
                    if (hs0 + i < hsteps) fetch(hs0 + i);
                // Operand reads run kAhead blocks ahead of the products that use them, through a ring of eight registers,
                // in a pinned order: a wavefront that first issues its sixteen products of a tile and only then asks for
                // the next operands leaves the matrix pipe idle for an LDS round trip per tile, and its SIMD partner is
                // at the same point (measured on this loop: 1.70 us per step, 1.12 with the operand reads taken out).
                constexpr int kAhead = 6;
                bf16x8 ring[8];
                auto kblk = [&](const HistTile &t, int k) { return *(const bf16x8 *)(t.h[k >> 3].k[k & 7] + obase); };
                auto vblk = [&](const HistTile &t, int k) { return *(const bf16x8 *)(t.h[k >> 3].v[k & 7] + obase); };
                auto scores_ahead = [&](const HistTile &t) {  // K block k = 8 half + 4 tile-of-half + d-group; leaves the first V blocks in the ring
#pragma unroll
                    for (int k = 0; k < kAhead; ++k) ring[k] = kblk(t, k);
#pragma unroll
                    for (int k = 0; k < 16; ++k) {
                        ring[(k + kAhead) & 7] = k + kAhead < 16 ? kblk(t, k + kAhead) : vblk(t, k + kAhead - 16);
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int nb = 0; nb < kNB; ++nb)
                            s[nb][k >> 2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[k & 7], qop[nb][k & 3], (k & 3) == 0 ? sinit[nb] : s[nb][k >> 2], 0, 0, 0);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                };
                auto output_ahead = [&](const HistTile &t) {  // V^T block k = 8 half + row block
#pragma unroll
                    for (int k = 0; k < 16; ++k) {
                        if (k + kAhead < 16) ring[(k + kAhead) & 7] = vblk(t, k + kAhead);
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int nb = 0; nb < kNB; ++nb)
                            acc[nb][k & 7] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ring[k & 7], pop[nb][k >> 3], acc[nb][k & 7], 0, 0, 0);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                };
                auto hist_step = [&](int hs, auto kind_tag) {
                    // this wavefront's pieces of step hs have landed once at most the pieces of the later steps are pending
                    if (hs + 2 < hsteps) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
                    else if (hs + 1 < hsteps) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
                    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    lds_barrier();  // everybody's pieces of step hs are in; everybody is done with step hs - 1
                    if (hs + 3 < hsteps) fetch(hs + 3);  // into the buffer of step hs - 1
                    if (wv_active) {
                        const HistTile &t = ntiles[hs & 3];
                        scores_ahead(t);
                        softmax(0, 2, kind_tag, H - hs * 64);
                        output_ahead(t);
                    }
                };
                const int whole = H / 64;  // the steps every key of which exists; a last, partial one has its own code
                for (int hs = hs0; hs < min(whole, hsteps); ++hs) hist_step(hs, std::integral_constant<int, 1>{});
                if (whole < hsteps) hist_step(whole, std::integral_constant<int, 2>{});
                lds_barrier();  // the ring is free for the tiles of the call's own tokens
            }
        }
        if (new_here) {
        issue(st0);
        commit(ntiles[st0 & 1]);
        if (st0 + 1 < nsteps) issue(st0 + 1);
        lds_barrier();
        for (int st = st0; st < nsteps; ++st) {
            if (st + 1 < nsteps) commit(ntiles[(st + 1) & 1]);
            if (st + 2 < nsteps) issue(st + 2);
            const int nh = halves(st);
            if (nh > 0) {
                const HistTile &t = ntiles[st & 1];
                scores(t, nh);
                load_v(t, 0);
                softmax(st, nh, std::integral_constant<int, 0>{});
                output(t, 0);
                if (nh > 1) {
                    load_v(t, 1);
                    output(t, 1);
                }
            }
            lds_barrier();
        }
        }
    }

    // =============================== key split: hand over or merge ===============================
    if constexpr (kSplit) {
        static_assert(kNB <= 2, "softmax reference and row sum of a thread's columns in one 16-byte slot");
        constexpr int kThreads = kSplitThreads, kSlots = kSplitSlots;  // accumulators, softmax state, staged q pieces
        const auto word = [&](int prt, int i) {  // word i of this thread's record in run prt: a wavefront's 256 bytes are contiguous
            return a.split_ws + (((int64_t)tile_id * a.nsplit + prt) * (4 * kSlots) + i) * kThreads + threadIdx.x;
        };
        // The partials travel between workgroups that may sit on different XCDs, whose L2s do not see each other's
        // lines.  They are written and read with device-scope accesses (relaxed atomics: written through to, and read
        // from, the memory side), a few hundred per thread; the alternative -- ordinary accesses between a device-scope
        // release and acquire fence -- writes back and invalidates whole L2s once per workgroup and measured 24 us per
        // launch at four runs per tile (15 us per run with a fence in every thread).
        const auto put = [](float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
        const auto get = [](const float *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
            for (int i = 0; i < VB; ++i)
#pragma unroll
                for (int c = 0; c < 4; ++c) put(word(part, 4 * (nb * VB + i) + c), acc[nb][i][c]);
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb) {
            put(word(part, 4 * kNB * VB + 2 * nb), m_run[nb]);
            put(word(part, 4 * kNB * VB + 2 * nb + 1), l_run[nb][0]);
        }
        if (a.write_new && hg == 0 && part == 0) write_new_rows<kRow, FP8, kWaves>(a, b, kvh, H, q0, q_per_wg, wave, lane);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's partial has reached the memory side
        __syncthreads();
        if (threadIdx.x == 0) {
            const uint32_t before = atomicAdd(a.split_cnt + tile_id, 1u);  // device scope
            const bool last_in = before == (uint32_t)a.nsplit - 1;
            if (last_in) __hip_atomic_store(a.split_cnt + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
            *(volatile int *)lds = last_in;
        }
        __syncthreads();
        if (*(volatile int *)lds == 0) return;
        // The runs are added in their order, this one's own read back like the others, so that the result does not
        // depend on which workgroup happened to finish last.
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb) {
            m_run[nb] = -INFINITY;
            l_run[nb] = (float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < VB; ++i) acc[nb][i] = (float4v){0.f, 0.f, 0.f, 0.f};
        }
        for (int prt = 0; prt < a.nsplit; ++prt) {
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb) {
                const float mo = get(word(prt, 4 * kNB * VB + 2 * nb)), lo = get(word(prt, 4 * kNB * VB + 2 * nb + 1));
                float4v other[VB];
#pragma unroll
                for (int i = 0; i < VB; ++i)
#pragma unroll
                    for (int c = 0; c < 4; ++c) other[i][c] = get(word(prt, 4 * (nb * VB + i) + c));
                const float m_new = fmaxf(m_run[nb], mo);
                const float mine = m_run[nb] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m_run[nb] - m_new);
                const float theirs = mo == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mo - m_new);
                l_run[nb] = l_run[nb] * mine + lo * theirs;
#pragma unroll
                for (int i = 0; i < VB; ++i) acc[nb][i] = acc[nb][i] * mine + other[i] * theirs;
                m_run[nb] = m_new;
            }
        }
    }

    // =============================== normalise and store ===============================
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
        const float l = l_run[nb][0];
        if (qi[nb] >= S || hg * a.HG + (kNB * wave + nb) % a.HG >= a.G) continue;  // padding columns write nothing
        const float inv = 1.0f / l;
        uint16_t *op = a.out + (((int64_t)b * S + qi[nb]) * a.Hq + head[nb]) * kRow + 4 * VBG * lq;
        const uint16_t *gp = a.out_gate ? a.out_gate + (op - a.out) : nullptr;  // the output gate's elements of this lane
        auto gate2 = [](uint32_t o2, uint32_t g2) {  // two bf16 outputs times the bf16-rounded sigmoid of two bf16 gates
            auto one = [](uint32_t o, uint32_t g) {
                const float sg = bf16_bits_to_f32(f32_to_bf16_bits(1.0f / (1.0f + expf(-bf16_bits_to_f32(g)))));
                return f32_to_bf16_bits(bf16_bits_to_f32(o) * sg);
            };
            return one(o2 & 0xffffu, g2 & 0xffffu) | (one(o2 >> 16, g2 >> 16) << 16);
        };
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r) {  // acc[VBG c + bb][r] is d = DW c + 4 VBG lq + VBG r + bb
                uint32_t w[VBG / 2];
#pragma unroll
                for (int e = 0; e < VBG / 2; ++e) w[e] = pack_bf16x2(acc[nb][VBG * c + 2 * e][r] * inv, acc[nb][VBG * c + 2 * e + 1][r] * inv);
                if (gp != nullptr) {
#pragma unroll
                    for (int e = 0; e < VBG / 2; ++e) w[e] = gate2(w[e], *(const uint32_t *)(gp + DW * c + VBG * r + 2 * e));
                }
                if constexpr (VBG == 8) *(u32x4 *)(op + DW * c + VBG * r) = (u32x4){w[0], w[1], w[2], w[3]};
                else *(u32x2 *)(op + DW * c + VBG * r) = (u32x2){w[0], w[1]};
            }
    }

    if (!kSplit && a.write_new && hg == 0) write_new_rows<kRow, FP8, kWaves>(a, b, kvh, H, q0, q_per_wg, wave, lane);
}

int validate_layout(const hs_kv_layout *l, int B, int S, int Hkv, int D, bool need_scales);
int check_prologue(const hs_qk_prologue *p, int dtype, int D, bool need_q, bool need_k);
NormSpec norm_spec(const hs_qk_prologue *p, int which);
void launch_prefill_wide(bool fp8, const PrefillArgs &a, dim3 grid, hipStream_t st);  // prefill_attn_wide.hip

// Key split of small calls: at most this many runs per query tile; per (tile, run) a workgroup's 512 threads store
// their accumulators (64 registers at every head_dim), one slot of softmax state and, when the launch runs q's
// prologue, their pieces of the finished q rows, 16 bytes each.
constexpr int kMaxKeySplits = 8;
static size_t split_tile_bytes(int D, bool narrow) {  // accumulator slots + one of softmax state + the staged q pieces
    return (size_t)512 * 16 * ((D == 64 ? 8 : 16) / (narrow ? 2 : 1) + 1 + (D == 64 ? 4 : 8) / (narrow ? 2 : 1));
}
// The arrival counters sit in front of the partials in a region of fixed size: every call finds them in the same place
// whatever its tile count and width, so the partials of one call can never land where another call keeps a counter
// (counters are zero between launches -- the last arriver of a tile clears its own -- and nothing else may write there).
constexpr int64_t kMaxSplitTiles = 4096;
constexpr size_t kSplitCounterBytes = (size_t)kMaxSplitTiles * 4;

__global__ void zero_words_kernel(uint32_t *p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// CUs of the current device (looked up once per device; 256 if the query fails).
static int compute_units() {
    static int cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
    }
    return n;
}

static int launch_prefill(bool fp8, const void *q, const void *k_new, const void *v_new, void *k_codes, void *v_codes,
                          float *k_scales, float *v_scales, const hs_kv_layout *layout, int32_t hist_len, void *out,
                          int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D, float softmax_scale,
                          int quantize_on_write, hs_stream_t stream, const int32_t *hist_lens = nullptr) {
    if (int rc = validate_layout(layout, B, S, Hkv, D, !fp8)) return rc;
    if (D != 64 && D != 128 && D != 256)
        return fail(HS_ERR_INVALID_ARGUMENT, "prefill attention is built for head_dim 64, 128 and 256, got %d", D);
    const bool empty = B == 0 || S == 0;  // an empty problem may come with null pointers (an empty tensor has none)
    if (!empty && (!q || !k_new || !v_new || !out)) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if ((hist_len > 0 || quantize_on_write) && (!k_codes || !v_codes || !k_scales || !v_scales))
        return fail(HS_ERR_INVALID_ARGUMENT, "null cache buffer");
    if (hist_len < 0) return fail(HS_ERR_INVALID_ARGUMENT, "negative hist_len");
    if (layout->prefill_window < 0) return fail(HS_ERR_INVALID_ARGUMENT, "negative prefill_window");
    const int G = Hq > 0 && Hkv > 0 ? Hq / Hkv : 0;
    if (Hq <= 0 || Hq % Hkv != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "need Hq %% Hkv == 0 (Hq=%d Hkv=%d)", Hq, Hkv);
    const int64_t cap = layout->k_block_table ? (int64_t)layout->capacity_tokens * layout->block_table_stride
                                              : layout->capacity_tokens;
    if ((int64_t)hist_len + (quantize_on_write ? S : 0) > cap)
        return fail(HS_ERR_OVERFLOW, "Cache overflow: trying to cache %d tokens starting at position %d, but capacity is %lld",
                    S, hist_len, (long long)cap);
    if (layout->k_block_table && (layout->capacity_tokens % 64) != 0)  // a history step reads 64 tokens of one block
        return fail(HS_ERR_INVALID_ARGUMENT, "paged blocks must hold a multiple of 64 tokens");
    if (B == 0 || S == 0) return HS_OK;
    hipStream_t st = (hipStream_t)stream;
    PrefillArgs a;
    a.q = (const uint16_t *)q; a.kn = (const uint16_t *)k_new; a.vn = (const uint16_t *)v_new;
    a.kc = (const uint8_t *)k_codes; a.vc = (const uint8_t *)v_codes;
    a.ks = k_scales; a.vs = v_scales;
    a.ka = make_addr(*layout, 0); a.va = make_addr(*layout, 1);
    a.out = (uint16_t *)out;
    a.out_gate = (const uint16_t *)layout->out_gate;
    a.B = B; a.S = S; a.Hq = Hq; a.Hkv = Hkv; a.G = G; a.hist_len = hist_len;
    a.hist_lens = hist_lens;
    a.write_new = quantize_on_write ? 1 : 0;
    a.window = layout->prefill_window;
    if (const hs_qk_prologue *qp = layout->prefill_q_prologue) {
        if (int rc = check_prologue(qp, HS_BF16, D, true, false)) return rc;
        const int rd = qp->rotary_dim > 0 ? qp->rotary_dim : D;
        if (qp->rope_sin && !prologue_parts_serve(rd, D / 4))
            return fail(HS_ERR_INVALID_ARGUMENT,
                        "the prefill launch rotates head_dim, head_dim/2 or head_dim/4 leading elements of q, not %d: run "
                        "hs_qk_prologue_apply on q as well", rd);
        if (qp->rope_sin && (int64_t)hist_len + S > qp->rope_len)
            return fail(HS_ERR_INVALID_ARGUMENT, "positions %d..%d exceed the rotary tables (%d rows)", hist_len,
                        hist_len + S - 1, qp->rope_len);
        for (const void *p : {qp->rope_sin, qp->rope_cos, qp->norm_kind != HS_QKNORM_NONE ? qp->q_norm_weight : nullptr})
            if (((uintptr_t)p & 15) != 0)
                return fail(HS_ERR_INVALID_ARGUMENT, "prefill_q_prologue needs 16-byte aligned norm weights and rotary tables");
        if (q == out) return fail(HS_ERR_INVALID_ARGUMENT, "prefill_q_prologue: q and out must be different buffers");
        a.qpro.norm = norm_spec(qp, 0);
        a.qpro.sin_t = qp->rope_sin; a.qpro.cos_t = qp->rope_cos;
        a.qpro.rope_len = qp->rope_len; a.qpro.rd = rd;
        a.qpro.on = 1;
    }
    a.HG = G >= 3 ? 4 : G;  // query heads per workgroup; a group size that is not 1, 2 or 4k pads its last group
    a.scale_log2e = softmax_scale * kPLog2e;
    int q_per_wg = 16 * ((D == 256 ? 1 : 2) * kPWaves / a.HG);  // PShape<D>::kNB column blocks per wavefront
    dim3 grid((S + q_per_wg - 1) / q_per_wg, Hkv * ((G + a.HG - 1) / a.HG), B);
    // A small problem (one short sequence, a chunk of a single prompt) would occupy a fraction of the CUs with 256
    // columns per workgroup: with half the columns there are twice the workgroups, each with half the matrix work
    // per step and the same conversion work.
    bool narrow = D <= 128 && q_per_wg >= 32 && 2 * (int64_t)grid.x * grid.y * grid.z <= compute_units();
    const int hint = layout->prefill_columns_hint;
    if (hint == 256 || hint == 128 || hint == 32 || hint == 16)  // the caller fixes the width
        narrow = D <= 128 && q_per_wg >= 32 && hint == 128;
    // 32: head_dim 128 at full width without a window on 32x32x16 MFMA tiles (prefill_attn_wide.hip).  Measured slower
    // than the 16x16x32 instance at 4 x 4096 tokens in 512-token chunks (0.77 against 0.65 ms), so the library never
    // picks it by itself; elsewhere 32 is the same as 256.
    const bool wide32 = D == 128 && !narrow && a.window == 0 && hint == 32 && !a.qpro.on;  // (its Q layout has no prologue)
    // 16: the same 256 columns per workgroup on sixteen wavefronts of one 16-column block each (four per SIMD, at most
    // 128 registers), head_dim 128 without a window; elsewhere the same as 256.
    const bool waves16 = D == 128 && !narrow && a.window == 0 && hint == 16;
    // Key split: every query tile cut into runs of 64-key steps for several workgroups, when the tiles alone would leave
    // most CUs idle and every run still has a few steps to amortise the merge (the caller gives scratch).  Half-width
    // tiles in two runs move half the partial bytes of full-width tiles in four and merge them on twice the CUs.
    if (layout->prefill_split_workspace != nullptr && layout->prefill_key_splits != 1 && a.window == 0 &&
        (hint == 0 || hint == 256 || hint == 128)) {
        int64_t tiles = (int64_t)grid.x * grid.y * grid.z;  // full width
        const int max_steps = (hist_len + 63) / 64 + (S + 63) / 64;
        const bool can_narrow = D <= 128 && q_per_wg >= 32;
        int P = layout->prefill_key_splits;
        bool split_narrow = can_narrow && hint == 128;
        if (P == 0) {
            P = (int)std::min<int64_t>(kMaxKeySplits, compute_units() / tiles);
            P = std::min(P, max_steps / 4);  // at least four steps to a run
            if (P < 3) P = 1;                // two runs of full-width tiles: the half-width workgroups do as well without a merge
            if (P >= 4 && can_narrow && hint != 256) {  // half-width tiles (the library's choice, or asked for): half the runs
                split_narrow = true;
                P /= 2;
            } else if (split_narrow) {
                P = 1;  // half-width asked for, too few steps to split those: the plain half-width launch
            }
        }
        if (P < 1 || P > kMaxKeySplits)
            return fail(HS_ERR_INVALID_ARGUMENT, "prefill_key_splits %d not in [0, %d]", P, kMaxKeySplits);
        if (P > 1) {
            if (split_narrow) tiles = (int64_t)((S + q_per_wg / 2 - 1) / (q_per_wg / 2)) * grid.y * grid.z;
            if (tiles > kMaxSplitTiles)
                return fail(HS_ERR_INVALID_ARGUMENT, "prefill_key_splits: %lld query tiles, at most %lld can be split (a call of this size fills the chip without)",
                            (long long)tiles, (long long)kMaxSplitTiles);
            const size_t cnt_bytes = kSplitCounterBytes;
            const size_t need = cnt_bytes + (size_t)tiles * P * split_tile_bytes(D, split_narrow);
            if (layout->prefill_split_workspace_bytes < 0 || (size_t)layout->prefill_split_workspace_bytes < need)
                return fail(HS_ERR_WORKSPACE, "prefill split workspace of %lld bytes, %zu needed",
                            (long long)layout->prefill_split_workspace_bytes, need);
            if (((uintptr_t)layout->prefill_split_workspace & 255) != 0)
                return fail(HS_ERR_INVALID_ARGUMENT, "prefill split workspace must be 256-byte aligned");
            a.nsplit = P;
            a.split_cnt = (uint32_t *)layout->prefill_split_workspace;
            a.split_ws = (float *)((uint8_t *)layout->prefill_split_workspace + cnt_bytes);
            narrow = split_narrow;
        }
    }
    if (narrow) {
        q_per_wg /= 2;
        grid.x = (S + q_per_wg - 1) / q_per_wg;
    }
    grid.x *= a.nsplit;
    // The bf16 copy of the prompt's K/V: every instance that writes the cache appends to it; the full-width instance
    // reads the history from it.
    bool shadow_read = false;
    if (layout->prefill_shadow != nullptr) {
        const int tokens = layout->prefill_shadow_tokens;
        const bool can_append = D == 128;
        if (!can_append) {
            if (hist_len > 0)
                return fail(HS_ERR_INVALID_ARGUMENT, "prefill_shadow serves head_dim 128; this call could not append to it");
        } else {
            if (tokens <= 0 || (tokens & 63) != 0 || (int64_t)hist_len + S > tokens)
                return fail(HS_ERR_INVALID_ARGUMENT, "prefill_shadow_tokens %d must be a multiple of 64 and hold hist_len + S = %lld tokens",
                            tokens, (long long)hist_len + S);
            const size_t need = (size_t)B * Hkv * (tokens / 64) * kShadowStepBytes;
            if (layout->prefill_shadow_bytes < 0 || (size_t)layout->prefill_shadow_bytes < need)
                return fail(HS_ERR_WORKSPACE, "prefill shadow of %lld bytes, %zu needed", (long long)layout->prefill_shadow_bytes, need);
            if (((uintptr_t)layout->prefill_shadow & 255) != 0)
                return fail(HS_ERR_INVALID_ARGUMENT, "prefill_shadow must be 256-byte aligned");
            if (!quantize_on_write && hist_len == 0) {
                // nothing to read and nothing appended: the copy plays no part in this call
            } else {
                if (!quantize_on_write)
                    return fail(HS_ERR_INVALID_ARGUMENT, "prefill_shadow needs quantize_on_write: a call that caches nothing leaves a hole in the copy");
                a.shadow = (uint16_t *)layout->prefill_shadow;
                a.shadow_steps = tokens / 64;
                shadow_read = hist_len > 0 && a.window == 0 && !wide32 && !waves16 && hist_lens == nullptr;  // (rows at different positions append, and read the codes)
            }
        }
    }
    // One workgroup fills a CU.  When the grid takes several rounds, the query tiles with the most keys go first so
    // that the launch does not end on them; a single round keeps the plain order.
    a.heavy_first = (int64_t)grid.x * grid.y * grid.z > compute_units();
#define HS_PREFILL_LAUNCH(WIN)                                                                              \
    do {                                                                                                    \
        if (D == 64 && narrow) {                                                                            \
            if (fp8) prefill_attn_kernel<64, true, 1, WIN><<<grid, 512, 0, st>>>(a);                    \
            else prefill_attn_kernel<64, false, 1, WIN><<<grid, 512, 0, st>>>(a);                       \
        } else if (D == 64) {                                                                               \
            if (fp8) prefill_attn_kernel<64, true, 0, WIN><<<grid, 512, 0, st>>>(a);                    \
            else prefill_attn_kernel<64, false, 0, WIN><<<grid, 512, 0, st>>>(a);                       \
        } else if (D == 128 && narrow) {                                                                    \
            if (fp8) prefill_attn_kernel<128, true, 1, WIN><<<grid, 512, 0, st>>>(a);                  \
            else prefill_attn_kernel<128, false, 1, WIN><<<grid, 512, 0, st>>>(a);                     \
        } else if (D == 128) {                                                                              \
            if (fp8) prefill_attn_kernel<128, true, 0, WIN><<<grid, 512, 0, st>>>(a);                  \
            else prefill_attn_kernel<128, false, 0, WIN><<<grid, 512, 0, st>>>(a);                     \
        } else {                                                                                            \
            if (fp8) prefill_attn_kernel<256, true, 0, WIN><<<grid, 512, 0, st>>>(a);                  \
            else prefill_attn_kernel<256, false, 0, WIN><<<grid, 512, 0, st>>>(a);                     \
        }                                                                                                   \
    } while (0)
    if (shadow_read) {
#define HS_PREFILL_COPY(F8)                                                                                  \
    do {                                                                                                     \
        if (a.nsplit > 1) {                                                                                  \
            if (narrow) prefill_attn_kernel<128, F8, 1, false, 8, true, true><<<grid, 512, 0, st>>>(a);       \
            else prefill_attn_kernel<128, F8, 0, false, 8, true, true><<<grid, 512, 0, st>>>(a);              \
        } else {                                                                                             \
            if (narrow) prefill_attn_kernel<128, F8, 1, false, 8, false, true><<<grid, 512, 0, st>>>(a);      \
            else prefill_attn_kernel<128, F8, 0, false, 8, false, true><<<grid, 512, 0, st>>>(a);             \
        }                                                                                                    \
    } while (0)
        if (fp8) HS_PREFILL_COPY(true);
        else HS_PREFILL_COPY(false);
#undef HS_PREFILL_COPY
    } else if (a.nsplit > 1) {
#define HS_PREFILL_SPLIT(DD, CC)                                                                     \
    do {                                                                                             \
        if (fp8) prefill_attn_kernel<DD, true, CC, false, 8, true><<<grid, 512, 0, st>>>(a);         \
        else prefill_attn_kernel<DD, false, CC, false, 8, true><<<grid, 512, 0, st>>>(a);            \
    } while (0)
        if (D == 64 && narrow) HS_PREFILL_SPLIT(64, 1);
        else if (D == 64) HS_PREFILL_SPLIT(64, 0);
        else if (D == 128 && narrow) HS_PREFILL_SPLIT(128, 1);
        else if (D == 128) HS_PREFILL_SPLIT(128, 0);
        else HS_PREFILL_SPLIT(256, 0);
#undef HS_PREFILL_SPLIT
    } else if (waves16) {
        if (fp8) prefill_attn_kernel<128, true, 1, false, 16><<<grid, 1024, 0, st>>>(a);
        else prefill_attn_kernel<128, false, 1, false, 16><<<grid, 1024, 0, st>>>(a);
    } else if (wide32) launch_prefill_wide(fp8, a, grid, st);
    else if (a.window > 0) HS_PREFILL_LAUNCH(true);
    else HS_PREFILL_LAUNCH(false);
#undef HS_PREFILL_LAUNCH
    if (int rc = check_launch("prefill_attn")) return rc;
    return HS_OK;
}

}  // namespace hs

extern "C" {

size_t hs_prefill_attn_split_workspace_bytes(int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D) {
    if (B <= 0 || S <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || (D != 64 && D != 128 && D != 256)) return 0;
    const int G = Hq / Hkv, HG = G >= 3 ? 4 : G;
    const int q_per_wg = 16 * ((D == 256 ? 1 : 2) * hs::kPWaves / HG);
    const int64_t tiles = (int64_t)((S + q_per_wg - 1) / q_per_wg) * Hkv * ((G + HG - 1) / HG) * B;
    // full-width tiles, or (head_dim <= 128) twice as many half-width ones: whichever record layout is larger
    const size_t wide = hs::kSplitCounterBytes + (size_t)tiles * hs::kMaxKeySplits * hs::split_tile_bytes(D, false);
    const size_t half = D <= 128 && q_per_wg >= 32
                            ? hs::kSplitCounterBytes + (size_t)2 * tiles * hs::kMaxKeySplits * hs::split_tile_bytes(D, true)
                            : 0;
    return wide > half ? wide : half;
}

size_t hs_prefill_shadow_bytes(int32_t B, int32_t Hkv, int32_t D, int32_t max_tokens) {
    if (B <= 0 || Hkv <= 0 || max_tokens <= 0 || D != 128) return 0;
    return (size_t)B * Hkv * (((size_t)max_tokens + 63) / 64) * hs::kShadowStepBytes;
}

int hs_prefill_shadow_init(void *shadow, size_t bytes, hs_stream_t stream) {
    return hs_prefill_attn_split_workspace_init(shadow, bytes, stream);  // the same clearing launch
}

int hs_prefill_attn_split_workspace_init(void *workspace, size_t bytes, hs_stream_t stream) {
    if (!workspace || ((uintptr_t)workspace & 255) != 0)
        return hs::fail(HS_ERR_INVALID_ARGUMENT, "prefill split workspace must be a 256-byte aligned device buffer");
    // the arrival counters sit in front of the partials; the whole buffer is cleared
    const size_t words = bytes / 4;
    if (words == 0) return HS_OK;
    hs::zero_words_kernel<<<dim3((unsigned)((words + 255) / 256)), 256, 0, (hipStream_t)stream>>>((uint32_t *)workspace, words);
    return hs::check_launch("prefill_split_workspace_init");
}

int hs_prefill_attn_int8(const void *q, const void *k_new, const void *v_new, int8_t *k_codes, int8_t *v_codes,
                         float *k_scales, float *v_scales, const hs_kv_layout *layout, int32_t hist_len, void *out,
                         int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D, float softmax_scale,
                         int quantize_on_write, hs_stream_t stream) {
    return hs::launch_prefill(false, q, k_new, v_new, k_codes, v_codes, k_scales, v_scales, layout, hist_len, out, B, S,
                              Hq, Hkv, D, softmax_scale, quantize_on_write, stream);
}

int hs_prefill_attn_fp8(const void *q, const void *k_new, const void *v_new, uint8_t *k_codes, uint8_t *v_codes,
                        const float *k_scales, const float *v_scales, const hs_kv_layout *layout, int32_t hist_len,
                        void *out, int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D, float softmax_scale,
                        int quantize_on_write, hs_stream_t stream) {
    return hs::launch_prefill(true, q, k_new, v_new, k_codes, v_codes, (float *)k_scales, (float *)v_scales, layout,
                              hist_len, out, B, S, Hq, Hkv, D, softmax_scale, quantize_on_write, stream);
}

int hs_prefill_attn_int8_ragged(const void *q, const void *k_new, const void *v_new, int8_t *k_codes, int8_t *v_codes,
                                float *k_scales, float *v_scales, const hs_kv_layout *layout, const int32_t *hist_lens,
                                int32_t max_hist_len, void *out, int32_t B, int32_t S, int32_t Hq, int32_t Hkv,
                                int32_t D, float softmax_scale, int quantize_on_write, hs_stream_t stream) {
    if (B > 0 && !hist_lens) return hs::fail(HS_ERR_INVALID_ARGUMENT, "hist_lens is NULL");
    return hs::launch_prefill(false, q, k_new, v_new, k_codes, v_codes, k_scales, v_scales, layout, max_hist_len, out, B,
                              S, Hq, Hkv, D, softmax_scale, quantize_on_write, stream, hist_lens);
}

int hs_prefill_attn_fp8_ragged(const void *q, const void *k_new, const void *v_new, uint8_t *k_codes, uint8_t *v_codes,
                               const float *k_scales, const float *v_scales, const hs_kv_layout *layout,
                               const int32_t *hist_lens, int32_t max_hist_len, void *out, int32_t B, int32_t S,
                               int32_t Hq, int32_t Hkv, int32_t D, float softmax_scale, int quantize_on_write,
                               hs_stream_t stream) {
    if (B > 0 && !hist_lens) return hs::fail(HS_ERR_INVALID_ARGUMENT, "hist_lens is NULL");
    return hs::launch_prefill(true, q, k_new, v_new, k_codes, v_codes, (float *)k_scales, (float *)v_scales, layout,
                              max_hist_len, out, B, S, Hq, Hkv, D, softmax_scale, quantize_on_write, stream, hist_lens);
}

}  // extern "C"
