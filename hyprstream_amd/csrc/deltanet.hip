// Gated delta rule (Qwen3.5 linear-attention layers) with the recurrent state held in registers (gfx950).
//
//   S <- S * exp(g);  m = k^T S;  delta = (v - m) * beta;  S <- S + k (x) delta;  o = q^T S
//
// The [dk, dv] = [128, 128] fp32 state of one (sequence, v-head) is independent per column, so it is
// cut into slices of NC columns and ONE wavefront owns one slice for the whole call: lane l holds
// column c = l % NC of rows [rg*RPL, (rg+1)*RPL) with rg = l / NC, RPL = 128*NC/64 rows in registers.
// The two contractions over dk are per-lane partial sums plus a butterfly over the 64/NC lanes that
// share a column; nothing goes through LDS and wavefronts never synchronise with each other.
//   T == 1 (decode): deltanet_decode_kernel, a 32-column slice per wavefront read and written with
//          16-byte accesses; a single read and a single write of the state: HBM bound,
//          2*dk*dv*4 bytes per (sequence, head).
//   T  > 1 (prefill): NC = 8 -> 16 state registers per lane and 16x more wavefronts; tokens are
//          processed in order with the next token's q/k/v/g/beta already in flight.
// q and k arrive in bf16; with l2norm they are normalised as x / max(||x||, 1e-3) in fp32.
#include "common.hpp"

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

template <int NC>
__device__ __forceinline__ float column_sum(float x) {  // sum over the lanes l with equal l % NC
#pragma unroll
    for (int o = NC; o < 64; o <<= 1) x += __shfl_xor(x, o, 64);
    return x;
}

template <int NC>
struct TokenIn {  // one token's inputs as this lane needs them
    static constexpr int RPL = 2 * NC;
    uint32_t kq[2][RPL / 2];  // packed bf16 pairs: k rows, q rows of this lane's row group
    float v, g, beta;
};

template <int NC>
__global__ __launch_bounds__(256) void deltanet_kernel(DeltaArgs a) {
    constexpr int RPL = 2 * NC;          // rows per lane
    constexpr int SLICES = kDV / NC;     // column slices per head
    const int lane = threadIdx.x & 63;
    const int64_t wid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t nw = (int64_t)a.B * a.nv * SLICES;
    if (wid >= nw) return;
    const int slice = (int)(wid % SLICES);
    const int j = (int)((wid / SLICES) % a.nv);
    const int b = (int)(wid / SLICES / a.nv);
    const int hk = j / (a.nv / a.nk);
    const int c = lane % NC, rg = lane / NC;
    const int col = slice * NC + c;

    float S[RPL];
    float *sp = a.state + (((int64_t)b * a.nv + j) * kDK + rg * RPL) * kDV + col;
#pragma unroll
    for (int r = 0; r < RPL; ++r) S[r] = sp[(int64_t)r * kDV];

    auto load_token = [&](TokenIn<NC> &x, int t) {
        const int64_t bt = (int64_t)b * a.T + t;
        const uint16_t *kp = a.k + (bt * a.nk + hk) * kDK + rg * RPL;
        const uint16_t *qp = a.q + (bt * a.nk + hk) * kDK + rg * RPL;
#pragma unroll
        for (int i = 0; i < RPL / 2; ++i) {
            x.kq[0][i] = ((const uint32_t *)kp)[i];
            x.kq[1][i] = ((const uint32_t *)qp)[i];
        }
        x.v = bf16_bits_to_f32(a.v[(bt * a.nv + j) * kDV + col]);
        x.g = a.g[bt * a.nv + j];
        x.beta = a.beta[bt * a.nv + j];
    };

    TokenIn<NC> cur, nxt;
    load_token(cur, 0);
    for (int t = 0; t < a.T; ++t) {
        if (t + 1 < a.T) load_token(nxt, t + 1);
        float kf[RPL], qf[RPL];
#pragma unroll
        for (int i = 0; i < RPL / 2; ++i) {
            kf[2 * i] = __uint_as_float(cur.kq[0][i] << 16);
            kf[2 * i + 1] = __uint_as_float(cur.kq[0][i] & 0xffff0000u);
            qf[2 * i] = __uint_as_float(cur.kq[1][i] << 16);
            qf[2 * i + 1] = __uint_as_float(cur.kq[1][i] & 0xffff0000u);
        }
        float kmul = 1.0f, qmul = a.q_scale;
        if (a.l2norm) {
            float sk = 0.0f, sq = 0.0f;
#pragma unroll
            for (int r = 0; r < RPL; ++r) {
                sk += kf[r] * kf[r];
                sq += qf[r] * qf[r];
            }
            sk = column_sum<NC>(sk);
            sq = column_sum<NC>(sq);
            kmul = 1.0f / fmaxf(sqrtf(sk), 1e-3f);
            qmul = a.q_scale / fmaxf(sqrtf(sq), 1e-3f);
        }
        const float decay = expf(cur.g);
        float m = 0.0f;
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
            kf[r] *= kmul;
            m += kf[r] * S[r];
        }
        m = column_sum<NC>(m) * decay;  // k^T (S * decay)
        const float delta = (cur.v - m) * cur.beta;
        float o = 0.0f;
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
            S[r] = S[r] * decay + kf[r] * delta;
            o += qf[r] * S[r];
        }
        o = column_sum<NC>(o) * qmul;
        if (rg == 0) a.out[(((int64_t)b * a.T + t) * a.nv + j) * kDV + col] = o;
        cur = nxt;
    }
#pragma unroll
    for (int r = 0; r < RPL; ++r) sp[(int64_t)r * kDV] = S[r];
}

// Decode step (T == 1), tuned for HBM streaming: one wavefront owns 32 columns x 128 rows; lane l holds
// columns 4*(l%8) .. +3 (one 16-byte access per row) of rows [16*(l/8), +16): every load and store
// instruction of the wavefront moves eight full 128-byte row segments.
__global__ __launch_bounds__(256) void deltanet_decode_kernel(DeltaArgs a) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const int lane = threadIdx.x & 63;
    const int64_t wid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t nw = (int64_t)a.B * a.nv * 4;
    if (wid >= nw) return;
    const int slice = (int)(wid & 3);
    const int j = (int)((wid >> 2) % a.nv);
    const int b = (int)((wid >> 2) / a.nv);
    const int hk = j / (a.nv / a.nk);
    const int c4 = lane & 7, rg = lane >> 3;
    const int col = slice * 32 + 4 * c4;
    float *sp = a.state + (((int64_t)b * a.nv + j) * kDK + rg * 16) * kDV + col;
    f4 S[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) S[r] = __builtin_nontemporal_load((const f4 *)(sp + (int64_t)r * kDV));  // read once

    const int64_t bt = b;  // T == 1
    const uint16_t *kp = a.k + (bt * a.nk + hk) * kDK + rg * 16;
    const uint16_t *qp = a.q + (bt * a.nk + hk) * kDK + rg * 16;
    float kf[16], qf[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t kw = ((const uint32_t *)kp)[i], qw = ((const uint32_t *)qp)[i];
        kf[2 * i] = __uint_as_float(kw << 16);
        kf[2 * i + 1] = __uint_as_float(kw & 0xffff0000u);
        qf[2 * i] = __uint_as_float(qw << 16);
        qf[2 * i + 1] = __uint_as_float(qw & 0xffff0000u);
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
    if (a.l2norm) {
        float sk = 0.0f, sq = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            sk += kf[r] * kf[r];
            sq += qf[r] * qf[r];
        }
        kmul = 1.0f / fmaxf(sqrtf(rows_sum(sk)), 1e-3f);
        qmul = a.q_scale / fmaxf(sqrtf(rows_sum(sq)), 1e-3f);
    }
    const float decay = expf(g);
    f4 m = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        kf[r] *= kmul;
        m += kf[r] * S[r];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) m[e] = rows_sum(m[e]) * decay;
    const f4 delta = (v - m) * beta;
    f4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        S[r] = S[r] * decay + kf[r] * delta;
        o += qf[r] * S[r];
        __builtin_nontemporal_store(S[r], (f4 *)(sp + (int64_t)r * kDV));
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = rows_sum(o[e]) * qmul;
    if (rg == 0) *(f4 *)(a.out + (bt * a.nv + j) * kDV + col) = o;
}

}  // namespace hs

extern "C" int hs_deltanet_forward(const void *q, const void *k, const void *v, const float *g, const float *beta,
                                   float *state, float *out, int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk,
                                   int32_t dv, float q_scale, int l2norm, hs_stream_t stream) {
    using namespace hs;
    if (!q || !k || !v || !g || !beta || !state || !out) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
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
        const int64_t waves = (int64_t)B * nv * (kDV / 32);
        deltanet_decode_kernel<<<(unsigned)((waves + 3) / 4), 256, 0, st>>>(a);
    } else {
        const int64_t waves = (int64_t)B * nv * (kDV / 8);
        deltanet_kernel<8><<<(unsigned)((waves + 3) / 4), 256, 0, st>>>(a);
    }
    return check_launch("deltanet");
}
