// Causal prefill attention for head_dim 128 on v_mfma_f32_32x32x16 (gfx950, wave64): the instance of
// prefill_attn.hip's algorithm that serves full-width grids without a sliding window.  Same arguments, same
// arithmetic (fp16 operands for the quantized history around a power-of-two reference per (sequence, kv-head),
// bf16 operands for the call's own tokens, fp32 softmax and accumulation, overflow-check online softmax), another
// schedule.
//
// What the schedule is built on, measured on this machine with issue probes: a wavefront issues its instructions
// in order and alone gets one plain vector instruction per ~6 cycles, so vector work that is not issued in the
// shadow of a matrix instruction adds its full length to the wavefront's step; a 32x32x16 MFMA (32 cycles) hides six
// plain vector instructions or three v_exp_f32 behind it, a 16x16x32 MFMA (16 cycles) two, and one wavefront issuing
// 32x32x16 MFMAs back to back keeps the matrix pipe busy (32.5 cycles each) where 16x16x32 leaves an eighth of it
// idle; an LDS operand read takes ~64 cycles to come back, which a wavefront pays in full whenever it issues a
// batch of reads and waits for them before the MFMAs that use them.  Hence:
//   * every operand read is issued four MFMAs ahead of its use into a ring of eight operand registers;
//   * the conversion of the NEXT step's K/V tile (the producer work every wavefront shares) is cut into pieces that
//     are issued between the score MFMAs of the current step;
//   * the exponentials of a 16-key group are issued between the output MFMAs of the group before it.
//
// Work split: a 512-thread workgroup owns 256 (query, head) columns of one kv-head, a wavefront 32 of them as ONE
// 32-column MFMA tile (lane = column n = lane % 32, half hf = lane / 32).  Keys are on the M axis:
//   S^T[key, col]  = sum_d K[key, d] Q[col, d]        A = K block (32 keys x 16 d), B = Q, C: key 8(r/4) + 4hf + r%4
//   O^T[d, col]   += sum_key V^T[d, key] P^T[key, col] A = V^T block (32 rows of d x 16 keys), B = P
// The k-slots of the second product are taken in the order the score accumulators hold the keys (slot (hf, e) of
// the MFMA over keys 16m .. 16m+15 is key 16m + 8(e/4) + 4hf + e%4), so P never leaves its lanes.  A V^T block holds
// the rows d = 8(rho % 16) + 2 blk + rho / 16 (rho = row, blk = block 0..3): the sixteen lanes that convert the
// sixteen d-octets of a key pair then write sixteen different 16-byte slots of ONE block (no bank conflicts), and a
// lane ends up with whole octets of d for its 16-byte output stores.
#include "prefill_common.hpp"

namespace hs {

typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kWKBytes = 16384;     // K operand blocks of a 64-key step: [tile 2][d-group 8] x 1 KB
constexpr int kWStepBytes = 32768;  // ... followed by the V^T blocks: [tile 2][key half 2][row block 4] x 1 KB

// Operands travel as four dwords; the element type only matters to the MFMA and to the rounding of P.
template <bool BF> struct WideOp;
template <> struct WideOp<false> {
    static __device__ __forceinline__ float16v mfma(u32x4 x, u32x4 y, float16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, x), __builtin_bit_cast(half8, y), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float p0, float p1) { return pack_f16x2(p0, p1); }
    static constexpr uint32_t kOnes = 0x3c003c00u;
};
template <> struct WideOp<true> {
    static __device__ __forceinline__ float16v mfma(u32x4 x, u32x4 y, float16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, x), __builtin_bit_cast(bf16x8, y), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float p0, float p1) { return pack_bf16x2(p0, p1); }
    static constexpr uint32_t kOnes = 0x3f803f80u;
};

// max over the two lanes that share a column (lane, lane ^ 32)
__device__ __forceinline__ float half_max(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
}

__device__ __forceinline__ float half_sum(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(a[0]) + __uint_as_float(a[1]);
}

__device__ __forceinline__ float16v splat16(float x) {
    float16v v;
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = x;
    return v;
}

template <bool FP8>
__global__ __launch_bounds__(512, 2) void prefill_attn_wide_kernel(PrefillArgs a) {
    constexpr int kRow = 128;
    constexpr int kStep = 64;  // keys per step, history and new tokens alike
    __shared__ __attribute__((aligned(16))) uint8_t lds[4 * kWStepBytes];  // a ring of four step buffers
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 31, hf = lane >> 5;
    // XCD-aware placement (as in prefill_attn.hip): the query tiles that read one (sequence, kv-head) stream get
    // linear ids congruent mod 8, so the stream is pulled into one XCD's L2.
    int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
    {
        const int X = gridDim.x, YZ = gridDim.y * gridDim.z;
        if ((YZ & 7) == 0) {
            const int p = bx + X * (by + gridDim.y * bz);
            const int grp = (p & 7) + 8 * (p / (8 * X));
            bx = (p >> 3) % X;
            if (a.heavy_first) bx = X - 1 - bx;
            by = grp % gridDim.y;
            bz = grp / gridDim.y;
        }
    }
    const int b = bz;
    const int groups = (a.G + a.HG - 1) / a.HG;
    const int kvh = by / groups, hg = by % groups;
    const int S = a.S, H = a.hist_lens ? min(max(a.hist_lens[b], 0), a.hist_len) : a.hist_len;
    const int q_per_wg = 16 * (2 * kPWaves / a.HG);
    const int q0 = bx * q_per_wg;
    if (q0 >= S) return;
    const int wg_qlast = min(S - 1, q0 + q_per_wg - 1);
    // column n of wavefront w is 16-column block bi = 2w + n/16 of the workgroup: head bi % HG of the group, query
    // 16 (bi / HG) + n % 16 of the tile (the assignment of prefill_attn.hip)
    const int bi = 2 * wave + (n >> 4);
    const int head = kvh * a.G + min(hg * a.HG + bi % a.HG, a.G - 1);  // a padding column repeats the group's last head
    const int qi = q0 + 16 * (bi / a.HG) + (n & 15);
    const bool col_live = qi < S && hg * a.HG + bi % a.HG < a.G;
    const int wv_q0 = q0 + 16 * ((2 * wave) / a.HG);
    const int wv_qlast = min(S - 1, q0 + 16 * ((2 * wave + 1) / a.HG) + 15);
    const bool wv_active = wv_q0 < S;

    float16v acc[4];  // O^T: acc[blk][r] is row rho = 8(r/4) + 4hf + r%4 of block blk, i.e. d = 8(rho%16) + 2blk + rho/16
    // Row sums.  History: on the matrix pipe, ones(32x16) x P^T, every register of lsum holds the column's sum (its walk has
    // no vector issue slots to spare).  New tokens: lrow, this lane's half of the column summed with plain additions (that
    // walk has the slots and needs the sixteen registers); the history's sum is folded into it when the history ends.
    float16v lsum = splat16(0.0f);
    float lrow = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = splat16(0.0f);
    float m_run = -INFINITY;

    // Online softmax with a reference that overshoots (prefill_attn.hip): m_run is an upper bound of the running
    // maximum, moved kSlack above a new maximum when one passes it.
    auto raise_max = [&](float mx) {
        if (__builtin_amdgcn_ballot_w64(mx > m_run) != 0) {
            const float m_new = mx > m_run ? mx + kSlack : m_run;
            const float alpha = (m_new == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
            lsum *= alpha;
            lrow *= alpha;
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] *= alpha;
            m_run = m_new;
        }
    };
    const float qscale = a.scale_log2e;
    const uint32_t lane16 = lane * 16;
    float vup = 1.0f;

    // Producer roles, the same in both phases.  K: wavefront w takes the 16-key block u4 = w/2 and the 16-d halves
    // jp = w%2 of every 32 d: lane (li, lq) holds K[16 u4 + li][32 lq + 16 jp .. + 15], which is the whole 16-d group
    // j = 2 lq + jp of that key: slot (key % 32, half 0) and (key % 32, half 1) of block (tile u4/2, j).
    // V: wavefront w takes (tile t, key half m, lane half hh) = (w/4, (w/2)%2, w%2); lane = (d-octet x = lane % 16,
    // (a, c) = lane / 16): the adjacent keys 32t + 16m + 8a + 4hh + 2c, + 1 are k-slots e = 4a + 2c, + 1 of lane half hh
    // in the MFMA over key half m.  Their eight (key, key + 1) pairs, d = 8x + bb, go to block (t, m, bb/2), slot
    // (x + 16 (bb%2), hh), bytes 4 (2a + c) ..: the 64 lanes of a wavefront write 64 different banks.
    const int pli = lane & 15, plq = lane >> 4;
    const int ku4 = wave >> 1, kjp = wave & 1;
    const int krow = 16 * ku4 + pli;
    const uint32_t kdst = ((ku4 >> 1) * 8 + 2 * plq + kjp) * 1024 + (16 * (ku4 & 1) + pli) * 16;
    const int vt = wave >> 2, vm = (wave >> 1) & 1, vhh = wave & 1, vx = lane & 15, vac = lane >> 4;
    const int vkey = 32 * vt + 16 * vm + 8 * (vac >> 1) + 4 * vhh + 2 * (vac & 1);
    const uint32_t vdst = kWKBytes + (vt * 2 + vm) * 4096 + (vx + 32 * vhh) * 16 + 4 * vac;

    // A step of a wavefront (64 keys) is four phases, each closed by a workgroup barrier:
    //   M1  scores: 16 MFMAs (tile t = i/8, d-group j = i%8), operands read from LDS four MFMAs ahead
    //   V1  softmax: the largest score against the reference (rarely: new reference, rescale), then the step's 32
    //       weights exp2(score - sref), rounded and packed as the B operands of M2
    //   M2  output: 4 groups (tile g/2, key half g%2) of 4 MFMAs (+ the row-sum MFMA in the history walk)
    //   V2  producer work: this wavefront's share of the tile two steps ahead goes into LDS, the rows of the tile three
    //       steps ahead are requested
    // Wavefronts 4-7 run ONE PHASE BEHIND wavefronts 0-3 (w and w + 4 share a SIMD): while one wavefront of a SIMD is
    // in a matrix phase the other is in a vector phase, so the vector work of a step runs in the shadow of the other
    // wavefront's MFMAs without any instruction-level interleaving, and a matrix phase has the pipe to itself (one
    // wavefront issuing 32x32x16 MFMAs back to back keeps it busy).  The tiles are therefore converted two steps ahead
    // and live in a ring of four LDS buffers.
    // A weight is exp2(score - sref), sref = m_run - kPShift.  Seeded (the history walk unless Q was rescaled): the score
    // accumulators start from -sref, a 16-register tuple of copies, and the MFMA result is the exponent itself.
    // Unseeded: accumulators start from zero and an fma (with the factor cq of a rescaled Q) precedes every exponential.
    float16v s[2];
    float sref = 0.0f;
    float16v sinit = splat16(0.0f);
    uint32_t pk[16];  // the step's weights: four B operands of M2
    const bool late = __builtin_amdgcn_readfirstlane(wave >> 2) != 0;

    auto scores_phase = [&](auto tag, const uint8_t *buf, const u32x4 (&qop)[8], const float16v &init) {
        typedef WideOp<decltype(tag)::value> Op;
        u32x4 ring[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) ring[i] = *(const u32x4 *)(buf + i * 1024);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if (i + 4 < 16) ring[(i + 4) & 7] = *(const u32x4 *)(buf + (i + 4) * 1024);
            s[i >> 3] = Op::mfma(ring[i & 7], qop[i & 7], (i & 7) == 0 ? init : s[i >> 3]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // largest accumulator of the step in this lane's column half (masked scores are -inf)
    auto step_max = [&]() {
        float m = fmaxf(s[0][0], s[1][0]);
#pragma unroll
        for (int r = 1; r < 16; ++r) m = fmaxf(m, fmaxf(s[0][r], s[1][r]));
        return m;
    };
    // In (almost) every step no score passes the reference and nothing happens in the branch.
    auto softmax_phase = [&](auto tag, auto seed_tag, float cq) {
        typedef WideOp<decltype(tag)::value> Op;
        constexpr bool kSeed = decltype(seed_tag)::value;
        constexpr bool kOnesMfma = !decltype(tag)::value;  // history (f16 operands): row sums by MFMA
        const float m = kSeed ? step_max() + sref : step_max() * cq;  // the largest score, log2 units
        const float thr = (m_run == -INFINITY) ? -INFINITY : sref + kPShift;
        if (__builtin_amdgcn_ballot_w64(m > thr) != 0) {
            raise_max(half_max(m));
            const float nref = (m_run == -INFINITY) ? 0.0f : m_run - kPShift;
            if (kSeed) {  // this step's accumulators started from the old reference
                const float d = nref - sref;
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int r = 0; r < 16; ++r) s[t][r] -= d;
                sinit = splat16(-nref);
            }
            sref = nref;
        }
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int k = 0; k < 4; ++k) {  // k-slots 2k, 2k + 1 of group g
                const int t = g >> 1, r = 8 * (g & 1) + 2 * k;
                const float p0 = __builtin_amdgcn_exp2f(kSeed ? s[t][r] : fmaf(s[t][r], cq, -sref));
                const float p1 = __builtin_amdgcn_exp2f(kSeed ? s[t][r + 1] : fmaf(s[t][r + 1], cq, -sref));
                if (!kOnesMfma) lrow += p0 + p1;
                pk[4 * g + k] = Op::pack2(p0, p1);
            }
    };
    auto output_phase = [&](auto tag, const uint8_t *vbuf, int ngroups) {
        typedef WideOp<decltype(tag)::value> Op;
        constexpr bool kOnesMfma = !decltype(tag)::value;
        const u32x4 ones = {Op::kOnes, Op::kOnes, Op::kOnes, Op::kOnes};
        u32x4 ring[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) ring[i] = *(const u32x4 *)(vbuf + i * 1024);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            if (g >= ngroups) break;
            const u32x4 pop = {pk[4 * g], pk[4 * g + 1], pk[4 * g + 2], pk[4 * g + 3]};
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                const int i = 4 * g + blk;
                if (i + 4 < 16) ring[(i + 4) & 7] = *(const u32x4 *)(vbuf + (i + 4) * 1024);
                acc[blk] = Op::mfma(ring[i & 7], pop, acc[blk]);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (kOnesMfma) lsum = Op::mfma(ones, pop, lsum);
        }
    };
    auto tile_buf = [&](int tile) { return lds + (tile & 3) * kWStepBytes; };

    // ------------------------------------------------------------------------------------------ history
    if (H > 0) {
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
                int cnt = min(min(H, 64), a.ka.capacity_tokens - slot);
                rk = a.ks[unit * a.ka.scale_stride_seq + (int64_t)kvh * a.ka.scale_stride_head + slot + min(lane, cnt - 1)];
                resolve(a.va, b, 0, unit, slot);
                cnt = min(min(H, 64), a.va.capacity_tokens - slot);
                rv = a.vs[unit * a.va.scale_stride_seq + (int64_t)kvh * a.va.scale_stride_head + slot + min(lane, cnt - 1)];
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
        // Q operands: fp16(q * scale * log2e * 2^E * 2^-ex); ex = 0 (cq = 1) unless a column's scaled |q| leaves the
        // range fp16 holds well, then the scores are multiplied back by cq = 2^ex where the weights are formed
        u32x4 qop[8];
        float cq = 1.0f;
        {
            const uint16_t *qp = a.q + (((int64_t)b * S + min(qi, S - 1)) * a.Hq + head) * kRow + 8 * hf;
            u32x4 w[8];
            float amax = 0.0f;
            const float qs = qscale * kup;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                w[j] = *(const u32x4 *)(qp + 16 * j);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    amax = fmaxf(amax, fmaxf(fabsf(__uint_as_float(w[j][e] << 16)), fabsf(__uint_as_float(w[j][e] & 0xffff0000u))));
            }
            amax = half_max(amax) * fabsf(qs);
            int ex = 0;
            if ((amax > 32768.0f || amax < 0.0009765625f) && amax > 0.0f && amax < 3.0e38f) (void)frexpf(amax, &ex);
            cq = ldexpf(1.0f, ex);
            const float qdown = ldexpf(qs, -ex);  // one factor: both are powers of two times the softmax scale
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    qop[j][e] = pack_f16x2(__uint_as_float(w[j][e] << 16) * qdown, __uint_as_float(w[j][e] & 0xffff0000u) * qdown);
        }

        const int nsteps = (H + kStep - 1) / kStep;
        // ---- producer state: raw codes and scales of the tile that is converted next
        u32x4 rawk = {0u, 0u, 0u, 0u};
        u32x2 rawv[2] = {{0u, 0u}, {0u, 0u}};
        float rawsk = 0.0f, rawsv[2] = {0.0f, 0.0f};
        if (FP8) {
            rawsk = 256.0f * a.ks[(int64_t)b * a.Hkv + kvh];
            rawsv[0] = rawsv[1] = 256.0f * a.vs[(int64_t)b * a.Hkv + kvh];
        }
        const uint32_t koff = krow * kRow + 32 * plq + 16 * kjp, voff = vkey * kRow + 8 * vx;
        const uint8_t *kb = a.kc, *vb = a.vc;
        const float *ksp = a.ks, *vsp = a.vs;
        int kleft = 0, vleft = 0;
        // issue() is called for tiles 0, 1, 2, ... in order, so the (scalar) addresses advance by a constant; a block
        // table is consulted only when a cursor leaves its block.
        auto issue = [&](int step) {
            const int t0 = step * kStep;
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
            uint32_t ko = koff, vo0 = voff, vo1 = voff + kRow, sk = 4u * krow, sv = 4u * vkey;
            uint32_t sv1 = sv + 4u;
            if (last < kStep - 1) {  // the last, partial tile: rows past the end repeat the last one (and convert to zero)
                ko = min(krow, last) * kRow + 32 * plq + 16 * kjp;
                vo0 = min(vkey, last) * kRow + 8 * vx;
                vo1 = min(vkey + 1, last) * kRow + 8 * vx;
                sk = 4u * min(krow, last);
                sv = 4u * min(vkey, last);
                sv1 = 4u * min(vkey + 1, last);
            }
            rawk = *(const u32x4 *)(kb + ko);
            rawv[0] = *(const u32x2 *)(vb + vo0);
            rawv[1] = *(const u32x2 *)(vb + vo1);
            if (!FP8) {
                rawsk = *(const float *)((const uint8_t *)ksp + sk);
                rawsv[0] = *(const float *)((const uint8_t *)vsp + sv);
                rawsv[1] = *(const float *)((const uint8_t *)vsp + sv1);
            }
            kb += kStep * kRow; vb += kStep * kRow;
            ksp += kStep; vsp += kStep;
            kleft -= kStep; vleft -= kStep;
        };
        // The conversion of tile `step` into `dst`.  The token scales are applied here, once per workgroup: operands are
        // fp16(code * scale * 2^-E), zero rows past the end, rows far above the head's reference saturated
        // (prefill_attn.hip).
        auto commit = [&](uint8_t *dst, int step) {
            const int last = H - 1 - step * kStep;
            float fk = rawsk * kdown, fv0 = rawsv[0] * vdown, fv1 = rawsv[1] * vdown;
            if (last < kStep - 1) {
                if (krow > last) fk = 0.0f;
                if (vkey > last) fv0 = 0.0f;
                if (vkey + 1 > last) fv1 = 0.0f;
            }
            const float smax = FP8 ? 64.0f * kMaxScale : kMaxScale;
            const _Float16 csk = (_Float16)fminf(fk, smax);
            const half2v csv = {(_Float16)fminf(fv0, smax), (_Float16)fminf(fv1, smax)};
            const _Float16 bias = (_Float16)1152.0f;
#pragma unroll
            for (int i = 0; i < 2; ++i) {  // K codes 0-7 / 8-15 of the lane's sixteen
                const uint32_t w0 = rawk[2 * i], w1 = rawk[2 * i + 1];
                const half8 kconv = FP8 ? e4m3x8_to_f16_div256(w0, w1) : int8x8_to_f16_biased(w0, w1) - bias;
                *(half8 *)(dst + kdst + 512 * i) = kconv * csk;
            }
#pragma unroll
            for (int bb = 0; bb < 8; ++bb) {  // V: the lane's eight (key, key + 1) pairs
                const uint32_t pair = FP8 ? e4m3_pair_to_f16_div256(rawv[0][bb >> 2], rawv[1][bb >> 2], bb & 3)
                                          : int8_pair_to_f16(rawv[0][bb >> 2], rawv[1][bb >> 2], bb & 3);
                const half2v hv = __builtin_bit_cast(half2v, pair) * csv;
                *(uint32_t *)(dst + vdst + (bb >> 1) * 1024 + (bb & 1) * 256) = __builtin_bit_cast(uint32_t, hv);
            }
        };

        // prologue: tiles 0 and 1 converted, tile 2 requested
        issue(0);
        commit(tile_buf(0), 0);
        if (1 < nsteps) issue(1);
        commit(tile_buf(1), 1);
        if (2 < nsteps) issue(2);
        lds_barrier();
        auto walk = [&](auto seed_tag) {
            constexpr bool kSeed = decltype(seed_tag)::value;
            if (late) lds_barrier();  // one phase behind
            for (int st = 0; st < nsteps; ++st) {
                const uint8_t *buf = tile_buf(st) + lane16;
                __builtin_amdgcn_s_setprio(1);
                scores_phase(std::false_type{}, buf, qop, kSeed ? sinit : splat16(0.0f));
                __builtin_amdgcn_s_setprio(0);
                lds_barrier();
                const int lim = H - st * kStep;
                if (lim < kStep) {  // the last, partial step
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            if (32 * t + 8 * (r >> 2) + 4 * hf + (r & 3) >= lim) s[t][r] = -INFINITY;
                }
                softmax_phase(std::false_type{}, seed_tag, cq);
                lds_barrier();
                __builtin_amdgcn_s_setprio(1);
                output_phase(std::false_type{}, buf + kWKBytes, 4);
                __builtin_amdgcn_s_setprio(0);
                lds_barrier();
                commit(tile_buf(st + 2), st + 2);  // past the last tile: zero rows into a buffer nobody reads
                if (st + 3 < nsteps) issue(st + 3);
                lds_barrier();
            }
            if (!late) lds_barrier();
        };
        if (__builtin_amdgcn_ballot_w64(cq != 1.0f) != 0)
            walk(std::false_type{});
        else
            walk(std::true_type{});
        if (vup != 1.0f) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] *= vup;
        }
        if (hf == 0) lrow = lsum[0];  // both lanes of a column hold the whole sum: one of them carries it on
    }

    // ------------------------------------------------------------------------------------------ new tokens: bf16, causal
    {
        // Q operands carry the softmax scale and log2(e), rounded back to bf16 (2^-9 relative, the precision the
        // weights are rounded to anyway)
        u32x4 qop[8];
        {
            const uint16_t *qp = a.q + (((int64_t)b * S + min(qi, S - 1)) * a.Hq + head) * kRow + 8 * hf;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const u32x4 w = *(const u32x4 *)(qp + 16 * j);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    qop[j][e] = pack_bf16x2(__uint_as_float(w[e] << 16) * qscale, __uint_as_float(w[e] & 0xffff0000u) * qscale);
            }
        }
        const int nsteps = wg_qlast / kStep + 1;
        const uint16_t *knb = a.kn + ((int64_t)b * S * a.Hkv + kvh) * kRow;
        const uint16_t *vnb = a.vn + ((int64_t)b * S * a.Hkv + kvh) * kRow;
        const int64_t rstride = (int64_t)a.Hkv * kRow;  // elements between consecutive tokens
        // bf16 rows are operands as they are.  K blocks are filled by loads that go from global memory straight into
        // LDS (lane l's 16 bytes land at base + 16 l, which IS the block layout: lane = (key % 32, half)): wavefront w
        // fills blocks (tile w/4, d-groups 2(w%4), + 1); no registers, no LDS write instructions.  V^T needs the
        // (key, key + 1) pairs picked out of two rows, so V still goes through registers.
        const int kt = wave >> 2, kj = 2 * (wave & 3);
        const uint32_t voff = vkey * (uint32_t)rstride + 8 * vx;
        u32x4 rawv[2];
        rawv[0] = rawv[1] = (u32x4){0u, 0u, 0u, 0u};
        auto issue_k = [&](int step) {
            uint8_t *dst = tile_buf(step);
            const int row = min(step * kStep + 32 * kt + n, S - 1);  // rows past the last token repeat it (masked)
            const uint16_t *kp = knb + (int64_t)row * rstride + 16 * kj + 8 * hf;
            typedef __attribute__((address_space(3))) void *lds_ptr;
            __builtin_amdgcn_global_load_lds(kp, (lds_ptr)(dst + (kt * 8 + kj) * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds(kp + 16, (lds_ptr)(dst + (kt * 8 + kj + 1) * 1024), 16, 0, 0);
        };
        auto issue_v = [&](int step) {
            const int t0 = step * kStep;
            const uint16_t *vp0, *vp1;
            if (t0 + kStep <= S) {
                vp0 = vnb + (int64_t)t0 * rstride + voff;
                vp1 = vp0 + (uint32_t)rstride;
            } else {
                vp0 = vnb + (int64_t)min(t0 + vkey, S - 1) * rstride + 8 * vx;
                vp1 = vnb + (int64_t)min(t0 + vkey + 1, S - 1) * rstride + 8 * vx;
            }
            rawv[0] = *(const u32x4 *)vp0;
            rawv[1] = *(const u32x4 *)vp1;
        };
        auto commit_v = [&](int step) {
            uint8_t *dst = tile_buf(step);
#pragma unroll
            for (int bb = 0; bb < 8; ++bb)
                *(uint32_t *)(dst + vdst + (bb >> 1) * 1024 + (bb & 1) * 256) = pick_halves(rawv[0][bb >> 1], rawv[1][bb >> 1], bb & 1);
        };
        // The direct loads write LDS behind the compiler's back.  Every V2 phase starts by waiting for all of this
        // wavefront's loads (the V rows it is about to commit were requested after the K loads of the V2 phase before),
        // and its closing barrier publishes them: the K blocks of tile st + 3, requested in V2 of step st, are published
        // by the barrier that closes V2 of step st + 1, two steps before their first reader.
        // prologue: K tiles 0, 1, 2 requested; V tiles 0 and 1 committed, V tile 2 requested
        issue_k(0);
        if (1 < nsteps) issue_k(1);
        if (2 < nsteps) issue_k(2);
        issue_v(0);
        commit_v(0);
        if (1 < nsteps) issue_v(1);
        commit_v(1);
        if (2 < nsteps) issue_v(2);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        lds_barrier();
        if (late) lds_barrier();  // one phase behind
        for (int st = 0; st < nsteps; ++st) {
            const uint8_t *buf = tile_buf(st) + lane16;
            const int t0 = st * kStep;
            // a step none of whose keys a query of this wavefront may see leaves only the producer work
            const bool active = wv_active && t0 <= wv_qlast;
            if (active) {
                __builtin_amdgcn_s_setprio(1);
                scores_phase(std::true_type{}, buf, qop, splat16(0.0f));
                __builtin_amdgcn_s_setprio(0);
            }
            lds_barrier();
            if (active) {
                if (t0 + kStep - 1 > wv_q0) {  // some (key, query) pair of this step is in the future
                    const int qrel = min(qi, S - 1) - t0 - 4 * hf;  // key offsets 32t + 8(r/4) + r%4 beyond this are masked
#pragma unroll
                    for (int t = 0; t < 2; ++t)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            if (32 * t + 8 * (r >> 2) + (r & 3) > qrel) s[t][r] = -INFINITY;
                }
                softmax_phase(std::true_type{}, std::false_type{}, 1.0f);
            }
            lds_barrier();
            if (active) {
                __builtin_amdgcn_s_setprio(1);
                output_phase(std::true_type{}, buf + kWKBytes, t0 + 32 > wv_qlast ? 2 : 4);
                __builtin_amdgcn_s_setprio(0);
            }
            lds_barrier();
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            commit_v(st + 2);  // past the last tile: the last rows again, into a buffer nobody reads
            if (st + 3 < nsteps) {
                issue_k(st + 3);
                issue_v(st + 3);
            }
            lds_barrier();
        }
        if (!late) lds_barrier();
    }

    // ------------------------------------------------------------------------------------------ normalise and store
    if (col_live) {
        const float inv = 1.0f / half_sum(lrow);
        uint16_t *op = a.out + (((int64_t)b * S + qi) * a.Hq + head) * kRow;
        const uint16_t *gp = a.out_gate ? a.out_gate + (op - a.out) : nullptr;
        auto gate2 = [](uint32_t o2, uint32_t g2) {  // two bf16 outputs times the bf16-rounded sigmoid of two bf16 gates
            auto one = [](uint32_t o, uint32_t g) {
                const float sg = bf16_bits_to_f32(f32_to_bf16_bits(1.0f / (1.0f + expf(-bf16_bits_to_f32(g)))));
                return f32_to_bf16_bits(bf16_bits_to_f32(o) * sg);
            };
            return one(o2 & 0xffffu, g2 & 0xffffu) | (one(o2 >> 16, g2 >> 16) << 16);
        };
        // d-octet 8 jj + 4 hf + i holds, at position e, acc[e / 2][8 (e % 2) + 4 jj + i]
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int oct = 8 * jj + 4 * hf + i;
                uint32_t w[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) w[k] = pack_bf16x2(acc[k][4 * jj + i] * inv, acc[k][8 + 4 * jj + i] * inv);
                if (gp != nullptr) {
                    const u32x4 gw = *(const u32x4 *)(gp + 8 * oct);
#pragma unroll
                    for (int k = 0; k < 4; ++k) w[k] = gate2(w[k], gw[k]);
                }
                *(u32x4 *)(op + 8 * oct) = (u32x4){w[0], w[1], w[2], w[3]};
            }
    }

    if (a.write_new && hg == 0) write_new_rows<kRow, FP8>(a, b, kvh, H, q0, q_per_wg, wave, lane);
}

void launch_prefill_wide(bool fp8, const PrefillArgs &a, dim3 grid, hipStream_t st) {
    if (fp8) prefill_attn_wide_kernel<true><<<grid, 512, 0, st>>>(a);
    else prefill_attn_wide_kernel<false><<<grid, 512, 0, st>>>(a);
}

}  // namespace hs
