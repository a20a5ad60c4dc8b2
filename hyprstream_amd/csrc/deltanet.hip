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
__global__ __launch_bounds__(256) void deltanet_decode_kernel(DeltaArgs a) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ f4 sm_m[4][8], sm_o[4][8];  // [wavefront][column quad]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int sl = wave & 1, rh = wave >> 1;
    const int chalf = (int)(blockIdx.x & 1);
    const int j = (int)((blockIdx.x >> 1) % a.nv);
    const int b = (int)((blockIdx.x >> 1) / a.nv);
    const int hk = j / (a.nv / a.nk);
    const int c4 = lane & 7, rg = lane >> 3;
    const int col = chalf * 64 + sl * 32 + 4 * c4;
    const int row0 = rh * 64 + rg * 8;
    float *sp = a.state + (((int64_t)b * a.nv + j) * kDK + row0) * kDV + col;
    f4 S[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) S[r] = __builtin_nontemporal_load((const f4 *)(sp + (int64_t)r * kDV));  // read once

    const int64_t bt = b;  // T == 1
    const uint16_t *kfull = a.k + (bt * a.nk + hk) * kDK, *qfull = a.q + (bt * a.nk + hk) * kDK;
    const u32x4 kw = *(const u32x4 *)(kfull + row0), qw = *(const u32x4 *)(qfull + row0);
    float kf[8], qf[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        kf[2 * i] = __uint_as_float(kw[i] << 16);
        kf[2 * i + 1] = __uint_as_float(kw[i] & 0xffff0000u);
        qf[2 * i] = __uint_as_float(qw[i] << 16);
        qf[2 * i + 1] = __uint_as_float(qw[i] & 0xffff0000u);
    }
    const uint32_t v01 = *(const uint32_t *)(a.v + (bt * a.nv + j) * kDV + col);
    const uint32_t v23 = *(const uint32_t *)(a.v + (bt * a.nv + j) * kDV + col + 2);
    const f4 v = {__uint_as_float(v01 << 16), __uint_as_float(v01 & 0xffff0000u), __uint_as_float(v23 << 16),
                  __uint_as_float(v23 & 0xffff0000u)};
    const float g = a.g[bt * a.nv + j], beta = a.beta[bt * a.nv + j];
    auto rows_sum = [](float x) {  // over the 8 row groups: lanes with equal l % 8
        x += __shfl_xor(x, 8, 64);
        x += __shfl_xor(x, 16, 64);
        x += __shfl_xor(x, 32, 64);
        return x;
    };
    float kmul = 1.0f, qmul = a.q_scale;
    if (a.l2norm) {  // the norms run over all 128 elements: lane l takes elements 2l and 2l + 1 of each vector
        const uint32_t k2 = ((const uint32_t *)kfull)[lane], q2 = ((const uint32_t *)qfull)[lane];
        const float k0 = __uint_as_float(k2 << 16), k1 = __uint_as_float(k2 & 0xffff0000u);
        const float q0 = __uint_as_float(q2 << 16), q1 = __uint_as_float(q2 & 0xffff0000u);
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
    if (rg == 0) sm_m[wave][c4] = m;
    __syncthreads();
    m = (sm_m[sl][c4] + sm_m[sl + 2][c4]) * decay;  // both row halves form the same sum in the same order
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
    if (rg == 0) sm_o[wave][c4] = o;
    __syncthreads();
    if (rh == 0 && rg == 0) *(f4 *)(a.out + (bt * a.nv + j) * kDV + col) = (sm_o[sl][c4] + sm_o[sl + 2][c4]) * qmul;
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
        deltanet_decode_kernel<<<(unsigned)((int64_t)B * nv * 2), 256, 0, st>>>(a);
    } else {
        deltanet_prefill_kernel<<<(unsigned)((int64_t)B * nv * 2), 512, 0, st>>>(a);
    }
    return check_launch("deltanet");
}
