// Gated delta rule (Qwen3.5 linear-attention layers) with the recurrent state held in registers (gfx950).
//
//   S <- S * exp(g);  m = k^T S;  delta = (v - m) * beta;  S <- S + k (x) delta;  o = q^T S
//
// The [dk, dv] = [128, 128] fp32 state of one (sequence, v-head) is independent per column, so it is cut into
// column slices and ONE wavefront owns one slice for the whole call.  The two contractions over dk are per-lane
// partial sums plus a reduction over the lanes that share a column.
//   T == 1 (decode):  deltanet_decode_kernel, a 32-column x 64-row piece per wavefront read and written with 16-byte
//          non-temporal accesses; a single read and a single write of the state: HBM bound, 2*dk*dv*4 bytes per
//          (sequence, head).
//   T  > 1 (prefill): deltanet_prefill_kernel, 8-column slices (16 state registers per lane), eight wavefronts
//          per workgroup sharing the token inputs through LDS; tokens are processed in order.  Bound by VALU
//          issue: about 85 instructions per token and wavefront, 2 x 4096 wavefront-tokens per SIMD at B=4 x 4096.
// q and k arrive in bf16; with l2norm they are normalised as x / max(||x||, 1e-3) in fp32.
#include "mfma_common.hpp"

namespace hs {

constexpr int kDK = 128, kDV = 128;

struct DeltaArgs {
    const uint16_t *q, *k, *v;  // bf16 [B,T,nk,dk], [B,T,nk,dk], [B,T,nv,dv]
    const float *g, *beta;      // [B,T,nv]
    float *state;               // [B,nv,dk,dv]
    float *out;                 // [B,T,nv,dv]
    int32_t B, T, nk, nv;
    float q_scale;
    int32_t l2norm;
};

// Prefill (T > 1) with the token inputs staged through LDS.  A 512-thread workgroup owns 64 state columns of one
// (sequence, v-head): wavefront w the columns 8w .. 8w+7, lane l column l%8 of rows [16*(l/8), +16) -- 16 state
// registers per lane.  The eight wavefronts together convert a chunk of kChunk tokens once (bf16 -> fp32, L2
// normalisation folded into k and q, exp(g)) into LDS while the previous chunk is consumed, instead of every
// wavefront unpacking and normalising the same k and q for itself.  The per-token work of a wavefront is then
// the three passes over its state slice (k^T S, the rank-1 update, q^T S) plus two column reductions done with
// lane-swap VALU instructions.
constexpr int kChunk = 32;

struct alignas(16) TokenChunk {
    float k[kChunk][kDK];   // k * kmul
    float q[kChunk][kDK];   // q * qmul (includes q_scale)
    float v[kChunk][64];    // this workgroup's 64 columns
    float4v scal[kChunk];   // {exp(g), exp(-g), beta, unused}
};

// sum over the 8 lanes l, l+8, ..., l+56 that hold the row groups of one column
__device__ __forceinline__ float rowgroup_sum(float x) {
    x += __uint_as_float(__builtin_amdgcn_update_dpp(0, __float_as_uint(x), 0x128, 0xf, 0xf, false));  // row_ror:8
    const uint32_t u = __float_as_uint(x);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const float m = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const uint32_t v = __float_as_uint(m);
    const auto c = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    return __uint_as_float(c[0]) + __uint_as_float(c[1]);
}

__global__ __launch_bounds__(512) void deltanet_prefill_kernel(DeltaArgs a) {
    __shared__ TokenChunk chunks[2];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = blockIdx.x & 1;
    const int j = (int)((blockIdx.x >> 1) % a.nv);
    const int b = (int)((blockIdx.x >> 1) / a.nv);
    const int hk = j / (a.nv / a.nk);
    const int c = lane & 7, rg = lane >> 3;
    const int lcol = 8 * wave + c;          // column inside the workgroup's 64
    const int col = 64 * half + lcol;
    float S[16];
    float *sp = a.state + (((int64_t)b * a.nv + j) * kDK + rg * 16) * kDV + col;
#pragma unroll
    for (int r = 0; r < 16; ++r) S[r] = sp[(int64_t)r * kDV];

    // ---- staging roles: thread -> (token tt, 8 consecutive k/q elements starting at 8*part), 4 v columns
    const int tt = tid >> 4, part = tid & 15;
    u32x4 rk = {0u, 0u, 0u, 0u}, rq = {0u, 0u, 0u, 0u};
    u32x2 rv = {0u, 0u};
    float rg_ = 0.0f, rb_ = 0.0f;
    auto issue = [&](int t0) {
        const int t = min(t0 + tt, a.T - 1);
        const int64_t bt = (int64_t)b * a.T + t;
        rk = *(const u32x4 *)(a.k + (bt * a.nk + hk) * kDK + 8 * part);
        rq = *(const u32x4 *)(a.q + (bt * a.nk + hk) * kDK + 8 * part);
        rv = *(const u32x2 *)(a.v + (bt * a.nv + j) * kDV + 64 * half + 4 * part);
        if (part == 0) {
            rg_ = a.g[bt * a.nv + j];
            rb_ = a.beta[bt * a.nv + j];
        }
    };
    auto commit = [&](TokenChunk &ch) {
        float kf[8], qf[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            kf[2 * i] = __uint_as_float(rk[i] << 16);
            kf[2 * i + 1] = __uint_as_float(rk[i] & 0xffff0000u);
            qf[2 * i] = __uint_as_float(rq[i] << 16);
            qf[2 * i + 1] = __uint_as_float(rq[i] & 0xffff0000u);
        }
        float kmul = 1.0f, qmul = a.q_scale;
        if (a.l2norm) {
            float sk = 0.0f, sq = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                sk += kf[i] * kf[i];
                sq += qf[i] * qf[i];
            }
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) {  // the 16 threads of a token are 16 consecutive lanes
                sk += __shfl_xor(sk, o, 64);
                sq += __shfl_xor(sq, o, 64);
            }
            kmul = 1.0f / fmaxf(sqrtf(sk), 1e-3f);
            qmul = a.q_scale / fmaxf(sqrtf(sq), 1e-3f);
        }
        float4v k0 = {kf[0] * kmul, kf[1] * kmul, kf[2] * kmul, kf[3] * kmul};
        float4v k1 = {kf[4] * kmul, kf[5] * kmul, kf[6] * kmul, kf[7] * kmul};
        float4v q0 = {qf[0] * qmul, qf[1] * qmul, qf[2] * qmul, qf[3] * qmul};
        float4v q1 = {qf[4] * qmul, qf[5] * qmul, qf[6] * qmul, qf[7] * qmul};
        *(float4v *)&ch.k[tt][8 * part] = k0;
        *(float4v *)&ch.k[tt][8 * part + 4] = k1;
        *(float4v *)&ch.q[tt][8 * part] = q0;
        *(float4v *)&ch.q[tt][8 * part + 4] = q1;
        float4v vv = {__uint_as_float(rv[0] << 16), __uint_as_float(rv[0] & 0xffff0000u), __uint_as_float(rv[1] << 16),
                      __uint_as_float(rv[1] & 0xffff0000u)};
        *(float4v *)&ch.v[tt][4 * part] = vv;
        if (part == 0) ch.scal[tt] = (float4v){expf(rg_), expf(-rg_), rb_, 0.0f};
    };

    const int nchunks = (a.T + kChunk - 1) / kChunk;
    issue(0);
    commit(chunks[0]);
    if (nchunks > 1) issue(kChunk);
    __syncthreads();
    float D = 1.0f, invD = 1.0f;
    float *op = a.out + (((int64_t)b * a.T) * a.nv + j) * kDV + col;
    const int64_t ostride = (int64_t)a.nv * kDV;
    for (int ci = 0; ci < nchunks; ++ci) {
        if (ci + 1 < nchunks) commit(chunks[(ci + 1) & 1]);
        if (ci + 2 < nchunks) issue((ci + 2) * kChunk);
        const TokenChunk &ch = chunks[ci & 1];
        const int nt = min(kChunk, a.T - ci * kChunk);
        for (int t = 0; t < nt; ++t) {
            float kf[16], qf[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4v kk = *(const float4v *)&ch.k[t][16 * rg + 4 * i];
                const float4v qq = *(const float4v *)&ch.q[t][16 * rg + 4 * i];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    kf[4 * i + e] = kk[e];
                    qf[4 * i + e] = qq[e];
                }
            }
            const float vv = ch.v[t][lcol];
            const float4v sc = ch.scal[t];
            const float decay = sc[0], beta = sc[2];
            // The registers hold S / D with D the product of the decays since the last fold, so a token costs one
            // FMA per state element instead of a multiply and an FMA.  D is folded back in before it can underflow.
            if (D * decay < 1e-20f) {
                const float f = D * decay;
#pragma unroll
                for (int r = 0; r < 16; ++r) S[r] *= f;
                D = 1.0f;
                invD = 1.0f;
            } else {
                D *= decay;
                invD *= sc[1];
            }
            float m0 = 0.0f, m1 = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                m0 += kf[r] * S[r];
                m1 += kf[r + 1] * S[r + 1];
            }
            const float m = rowgroup_sum(m0 + m1) * D;  // k^T (S_prev * decay)
            const float kd = (vv - m) * beta * invD;    // delta / D
            float o0 = 0.0f, o1 = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                S[r] += kf[r] * kd;
                S[r + 1] += kf[r + 1] * kd;
                o0 += qf[r] * S[r];
                o1 += qf[r + 1] * S[r + 1];
            }
            const float o = rowgroup_sum(o0 + o1) * D;
            if (rg == 0) op[(int64_t)(ci * kChunk + t) * ostride] = o;
        }
        // fold at every chunk end: a prefill split into calls of a multiple of kChunk tokens (state carried through
        // memory) then rounds exactly like one call
#pragma unroll
        for (int r = 0; r < 16; ++r) S[r] *= D;
        D = 1.0f;
        invD = 1.0f;
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) sp[(int64_t)r * kDV] = S[r];
}

// Decode step (T == 1), tuned for HBM streaming.  A 256-thread workgroup owns 64 columns of one (sequence, v-head);
// wavefront w the 32-column slice w % 2 of the row half w / 2: 8 KB of state per wavefront, lane l columns
// 4*(l%8) .. +3 (one 16-byte access per row) of rows [64*(w/2) + 8*(l/8), +8), so every load and store instruction of
// the wavefront moves eight full 128-byte row segments.  The two contractions over dk meet between the two row halves
// through LDS (32 floats each way).  With 16 KB per wavefront (all 128 rows, no exchange) the step took 47.9 us at
// B = 64 x 32 heads; a plain read-scale-write kernel of the same shape takes 46.2 us with 16 KB per wavefront and
// 43.1 us with 8 KB (more wavefronts in flight, shorter ones).
//
// LAYER: the whole decode branch of GatedDeltaNetLayer::forward between the two projections in one launch
// (qwen3_5.rs:629-686 conv1d + SiLU + gates, :725-751 the step, :305-313 RMSNormGated).  A 512-thread workgroup owns
// all 128 columns of its (sequence, v-head) -- the norm runs over them -- as two such 64-column halves.  While the
// state loads travel, 384 threads compute the head's q, k and v channels from the mixed projection (depthwise causal
// conv over [3 carried frames | the new one], SiLU, each rounded to bf16 as the separate kernels store them) into
// LDS and thread 384 the two gates; the step then reads them from there, and its output row goes through the gated
// norm instead of to memory.  Every value is computed with the expressions of deltanet_conv8_kernel,
// deltanet_gates_kernel, the plain instance of this kernel and gated_rmsnorm_rows_kernel, in their order.
struct LayerArgs {
    const uint16_t *x;         // [B, 1, C] bf16 mixed q|k|v projection, C = 2*key_dim + val_dim
    const uint16_t *w;         // [C, 4] bf16 conv taps, tap 3 multiplies the new frame
    const uint16_t *state_in;  // [B, C, 3] bf16 or nullptr (= zeros)
    uint16_t *state_out;       // [B, C, 3]
    const uint16_t *a_in, *b_in;          // [B, 1, nv] bf16
    const float *neg_a_exp, *dt_bias;     // [nv]
    const uint16_t *z;         // [B, 1, nv, dv] bf16 gate of the norm
    const float *norm_w;       // [dv]
    uint16_t *out;             // [B, 1, nv, dv] bf16
    float eps;
    int32_t C, key_dim;
};

// SiLU through v_exp_f32 and v_rcp_f32, as deltanet_glue.hip computes it
__device__ __forceinline__ float silu_fast_layer(float x) {
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

template <bool LAYER>
__global__ __launch_bounds__(LAYER ? 512 : 256) void deltanet_decode_kernel(DeltaArgs a, LayerArgs la) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    constexpr int NH = LAYER ? 2 : 1;             // column halves in this workgroup
    __shared__ f4 sm_m[NH][4][8], sm_o[NH][4][8];  // [half][wavefront of the half][column quad]
    __shared__ __attribute__((aligned(16))) float sm_in[LAYER ? 3 * 128 + 4 : 4];  // q | k | v of the head, then g and beta
    __shared__ __attribute__((aligned(16))) float sm_row[LAYER ? 128 : 4];        // the step's output row
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int w4 = wave & 3, sl = wave & 1, rh = (wave >> 1) & 1;
    const int unit = LAYER ? (int)blockIdx.x : (int)(blockIdx.x >> 1);
    const int chalf = LAYER ? wave >> 2 : (int)(blockIdx.x & 1), hx = LAYER ? chalf : 0;
    const int j = unit % a.nv;
    const int b = unit / a.nv;
    const int hk = j / (a.nv / a.nk);
    const int c4 = lane & 7, rg = lane >> 3;
    const int col = chalf * 64 + sl * 32 + 4 * c4;
    const int row0 = rh * 64 + rg * 8;
    float *sp = a.state + (((int64_t)b * a.nv + j) * kDK + row0) * kDV + col;
    const int64_t bt = b;  // T == 1
    // LAYER: the small loads of the prologue are issued ahead of the state's (loads return in order: behind the 8 KB
    // of state they would arrive last, and the arithmetic that hides under the state loads would wait).  The norm's
    // own inputs are loaded where they are used: held from here they cost 14 registers and a resident workgroup
    // (51.5 against 50.6 us per step at B = 64).
    const int pt = threadIdx.x, ppart = pt >> 7;  // 0: q, 1: k (channels of k-head hk), 2: v (of v-head j)
    const int pc = ppart == 2 ? 2 * la.key_dim + j * kDV + (pt & 127) : ppart * la.key_dim + hk * kDK + (pt & 127);
    uint32_t ps0 = 0u, ps1 = 0u, ps2 = 0u, pxn = 0u, pw01 = 0u, pw23 = 0u, pab = 0u;
    if constexpr (LAYER) {
        if (pt < 3 * 128) {
            if (la.state_in) {
                const uint16_t *sin = la.state_in + ((int64_t)b * la.C + pc) * 3;
                ps0 = sin[0]; ps1 = sin[1]; ps2 = sin[2];
            }
            pxn = la.x[(int64_t)b * la.C + pc];
            pw01 = *(const uint32_t *)(la.w + (int64_t)pc * 4);
            pw23 = *(const uint32_t *)(la.w + (int64_t)pc * 4 + 2);
        } else if (pt == 3 * 128) {
            pab = (uint32_t)la.a_in[bt * a.nv + j] | ((uint32_t)la.b_in[bt * a.nv + j] << 16);
        }
    }
    f4 S[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) S[r] = __builtin_nontemporal_load((const f4 *)(sp + (int64_t)r * kDV));  // read once

    float kf[8], qf[8];
    f4 v;
    float g, beta;
    if constexpr (LAYER) {
        {
#pragma clang fp contract(off)
            const int t = pt;
            if (t < 3 * 128) {
                const int part = ppart, c = pc;
                const uint32_t s0 = ps0, s1 = ps1, s2 = ps2, xn = pxn;
                float acc = bf16_bits_to_f32(pw01 & 0xffffu) * bf16_bits_to_f32(s0);
                acc += bf16_bits_to_f32(pw01 >> 16) * bf16_bits_to_f32(s1);
                acc += bf16_bits_to_f32(pw23 & 0xffffu) * bf16_bits_to_f32(s2);
                acc += bf16_bits_to_f32(pw23 >> 16) * bf16_bits_to_f32(xn);
                const float y = silu_fast_layer((float)(__bf16)acc);  // the conv output is a bf16 tensor before the SiLU
                sm_in[t] = (float)(__bf16)y;
                // the carried frames move up by one; the k-head's channels are written by its first v-head only
                if (part == 2 || j % (a.nv / a.nk) == 0) {
                    uint16_t *so = la.state_out + ((int64_t)b * la.C + c) * 3;
                    so[0] = (uint16_t)s1;
                    so[1] = (uint16_t)s2;
                    so[2] = (uint16_t)xn;
                }
            } else if (t == 3 * 128) {
                const float xa = bf16_bits_to_f32(pab & 0xffffu) + la.dt_bias[j];
                const float spl = xa > 20.0f ? xa : log1pf(expf(xa));  // softplus with libtorch's linear threshold
                sm_in[3 * 128] = la.neg_a_exp[j] * spl;
                sm_in[3 * 128 + 1] = 1.0f / (1.0f + expf(-bf16_bits_to_f32(pab >> 16)));
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            qf[r] = sm_in[row0 + r];
            kf[r] = sm_in[128 + row0 + r];
        }
        v = *(const f4 *)&sm_in[256 + col];
        g = sm_in[3 * 128];
        beta = sm_in[3 * 128 + 1];
    } else {
        const uint16_t *kfull = a.k + (bt * a.nk + hk) * kDK, *qfull = a.q + (bt * a.nk + hk) * kDK;
        const u32x4 kw = *(const u32x4 *)(kfull + row0), qw = *(const u32x4 *)(qfull + row0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            kf[2 * i] = __uint_as_float(kw[i] << 16);
            kf[2 * i + 1] = __uint_as_float(kw[i] & 0xffff0000u);
            qf[2 * i] = __uint_as_float(qw[i] << 16);
            qf[2 * i + 1] = __uint_as_float(qw[i] & 0xffff0000u);
        }
        const uint32_t v01 = *(const uint32_t *)(a.v + (bt * a.nv + j) * kDV + col);
        const uint32_t v23 = *(const uint32_t *)(a.v + (bt * a.nv + j) * kDV + col + 2);
        v = (f4){__uint_as_float(v01 << 16), __uint_as_float(v01 & 0xffff0000u), __uint_as_float(v23 << 16),
                 __uint_as_float(v23 & 0xffff0000u)};
        g = a.g[bt * a.nv + j];
        beta = a.beta[bt * a.nv + j];
    }
    auto rows_sum = [](float x) {  // over the 8 row groups: lanes with equal l % 8
        x += __shfl_xor(x, 8, 64);
        x += __shfl_xor(x, 16, 64);
        x += __shfl_xor(x, 32, 64);
        return x;
    };
    float kmul = 1.0f, qmul = a.q_scale;
    if (a.l2norm) {  // the norms run over all 128 elements: lane l takes elements 2l and 2l + 1 of each vector
        float k0, k1, q0, q1;
        if constexpr (LAYER) {
            k0 = sm_in[128 + 2 * lane]; k1 = sm_in[128 + 2 * lane + 1];
            q0 = sm_in[2 * lane]; q1 = sm_in[2 * lane + 1];
        } else {
            const uint16_t *kfull = a.k + (bt * a.nk + hk) * kDK, *qfull = a.q + (bt * a.nk + hk) * kDK;
            const uint32_t k2 = ((const uint32_t *)kfull)[lane], q2 = ((const uint32_t *)qfull)[lane];
            k0 = __uint_as_float(k2 << 16); k1 = __uint_as_float(k2 & 0xffff0000u);
            q0 = __uint_as_float(q2 << 16); q1 = __uint_as_float(q2 & 0xffff0000u);
        }
        float sk = k0 * k0 + k1 * k1, sq = q0 * q0 + q1 * q1;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            sk += __shfl_xor(sk, o, 64);
            sq += __shfl_xor(sq, o, 64);
        }
        kmul = 1.0f / fmaxf(sqrtf(sk), 1e-3f);
        qmul = a.q_scale / fmaxf(sqrtf(sq), 1e-3f);
    }
    const float decay = expf(g);
    f4 m = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        kf[r] *= kmul;
        m += kf[r] * S[r];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) m[e] = rows_sum(m[e]);
    if (rg == 0) sm_m[hx][w4][c4] = m;
    __syncthreads();
    m = (sm_m[hx][sl][c4] + sm_m[hx][sl + 2][c4]) * decay;  // both row halves form the same sum in the same order
    const f4 delta = (v - m) * beta;
    f4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        S[r] = S[r] * decay + kf[r] * delta;
        o += qf[r] * S[r];
        __builtin_nontemporal_store(S[r], (f4 *)(sp + (int64_t)r * kDV));
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = rows_sum(o[e]);
    if (rg == 0) sm_o[hx][w4][c4] = o;
    __syncthreads();
    if constexpr (!LAYER) {
        if (rh == 0 && rg == 0) *(f4 *)(a.out + (bt * a.nv + j) * kDV + col) = (sm_o[0][sl][c4] + sm_o[0][sl + 2][c4]) * qmul;
    } else {
        if (rh == 0 && rg == 0) *(f4 *)&sm_row[col] = (sm_o[hx][sl][c4] + sm_o[hx][sl + 2][c4]) * qmul;
        __syncthreads();
        if (wave == 0 && lane < 16) {  // RMSNormGated over the 128 columns: 16 lanes x 8 elements, as gated_rmsnorm_rows_kernel<16>
            const int sub = lane;
            const f4 xa = *(const f4 *)&sm_row[8 * sub], xb = *(const f4 *)&sm_row[8 * sub + 4];
            const int64_t e0 = (bt * a.nv + j) * kDV + 8 * sub;
            const u32x4 zz = *(const u32x4 *)(la.z + e0);
            const f4 wa = *(const f4 *)(la.norm_w + 8 * sub), wb = *(const f4 *)(la.norm_w + 8 * sub + 4);
            const float xv[8] = {xa[0], xa[1], xa[2], xa[3], xb[0], xb[1], xb[2], xb[3]};
            const float wv[8] = {wa[0], wa[1], wa[2], wa[3], wb[0], wb[1], wb[2], wb[3]};
            float ss = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) ss += xv[e] * xv[e];
#pragma unroll
            for (int o2 = 1; o2 < 16; o2 <<= 1) ss += __shfl_xor(ss, o2, 64);
            const float rrms = 1.0f / sqrtf(ss / (float)kDV + la.eps);
            typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
            uint32_t o4[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float z0 = __uint_as_float(zz[i] << 16), z1 = __uint_as_float(zz[i] & 0xffff0000u);
                const bf16x2 pr = {(__bf16)(xv[2 * i] * rrms * wv[2 * i] * silu_fast_layer(z0)),
                                   (__bf16)(xv[2 * i + 1] * rrms * wv[2 * i + 1] * silu_fast_layer(z1))};
                o4[i] = __builtin_bit_cast(uint32_t, pr);
            }
            *(u32x4 *)(la.out + e0) = (u32x4){o4[0], o4[1], o4[2], o4[3]};
        }
    }
}

}  // namespace hs

extern "C" int hs_deltanet_forward(const void *q, const void *k, const void *v, const float *g, const float *beta,
                                   float *state, float *out, int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk,
                                   int32_t dv, float q_scale, int l2norm, hs_stream_t stream) {
    using namespace hs;
    if (B > 0 && T > 0 && (!q || !k || !v || !g || !beta || !state || !out)) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (dk != kDK || dv != kDV) return fail(HS_ERR_INVALID_ARGUMENT, "deltanet is built for dk = dv = 128, got %d x %d", dk, dv);
    if (B < 0 || T < 0 || nk <= 0 || nv <= 0 || nv % nk != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "bad shape B=%d T=%d nk=%d nv=%d (need nv %% nk == 0)", B, T, nk, nv);
    if (B == 0 || T == 0) return HS_OK;
    DeltaArgs a;
    a.q = (const uint16_t *)q; a.k = (const uint16_t *)k; a.v = (const uint16_t *)v;
    a.g = g; a.beta = beta; a.state = state; a.out = out;
    a.B = B; a.T = T; a.nk = nk; a.nv = nv; a.q_scale = q_scale; a.l2norm = l2norm ? 1 : 0;
    hipStream_t st = (hipStream_t)stream;
    if (T == 1) {
        deltanet_decode_kernel<false><<<(unsigned)((int64_t)B * nv * 2), 256, 0, st>>>(a, LayerArgs{});
    } else {
        deltanet_prefill_kernel<<<(unsigned)((int64_t)B * nv * 2), 512, 0, st>>>(a);
    }
    return check_launch("deltanet");
}

extern "C" int hs_deltanet_decode_layer(const void *mixed_qkv, const void *conv_weight, const void *conv_state_in,
                                        void *conv_state_out, const void *a_in, const void *b_in, const float *neg_a_exp,
                                        const float *dt_bias, const void *z, const float *norm_weight, float norm_eps,
                                        float *state, void *out, int32_t B, int32_t nk, int32_t nv, int32_t dk, int32_t dv,
                                        float q_scale, int l2norm, hs_stream_t stream) {
    using namespace hs;
    if (B > 0 && (!mixed_qkv || !conv_weight || !conv_state_out || !a_in || !b_in || !neg_a_exp || !dt_bias || !z ||
                  !norm_weight || !state || !out))
        return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (conv_state_out && conv_state_in == conv_state_out)
        return fail(HS_ERR_INVALID_ARGUMENT, "conv_state_out must not alias conv_state_in");
    if (dk != kDK || dv != kDV) return fail(HS_ERR_INVALID_ARGUMENT, "deltanet is built for dk = dv = 128, got %d x %d", dk, dv);
    if (B < 0 || nk <= 0 || nv <= 0 || nv % nk != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "bad shape B=%d nk=%d nv=%d (need nv %% nk == 0)", B, nk, nv);
    if ((((uintptr_t)z | (uintptr_t)norm_weight | (uintptr_t)out) & 15) != 0 || ((uintptr_t)conv_weight & 7) != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "z, norm_weight and out must be 16-byte aligned, conv_weight 8-byte");
    if (B == 0) return HS_OK;
    DeltaArgs a{};
    a.state = state;
    a.B = B; a.T = 1; a.nk = nk; a.nv = nv; a.q_scale = q_scale; a.l2norm = l2norm ? 1 : 0;
    LayerArgs la;
    la.x = (const uint16_t *)mixed_qkv; la.w = (const uint16_t *)conv_weight;
    la.state_in = (const uint16_t *)conv_state_in; la.state_out = (uint16_t *)conv_state_out;
    la.a_in = (const uint16_t *)a_in; la.b_in = (const uint16_t *)b_in;
    la.neg_a_exp = neg_a_exp; la.dt_bias = dt_bias;
    la.z = (const uint16_t *)z; la.norm_w = norm_weight; la.out = (uint16_t *)out; la.eps = norm_eps;
    la.key_dim = nk * dk; la.C = 2 * nk * dk + nv * dv;
    deltanet_decode_kernel<true><<<(unsigned)((int64_t)B * nv), 512, 0, (hipStream_t)stream>>>(a, la);
    return check_launch("deltanet_decode_layer");
}
