// The elementwise steps of a gated-DeltaNet layer on either side of the delta rule (gfx950):
//   hs_deltanet_prepare     depthwise causal conv1d (kernel 4, carried 3-frame state) + SiLU on the mixed q|k|v
//                           channels, split into the q, k, v tensors the recurrence reads, plus the gates
//                           g = -exp(A_log) * softplus(a + dt_bias) and beta = sigmoid(b)
//                           (GatedDeltaNetLayer::forward, crates/hyprstream/src/runtime/architectures/qwen3_5.rs:629-686)
//   hs_deltanet_gated_norm  norm(o) * w * silu(z) (RMSNormGated::forward, qwen3_5.rs:305-313)
// All of it is HBM-trivial streaming work: one read of the inputs, one write of the outputs.
#include "common.hpp"

namespace hs {

constexpr int kConvK = 4;        // linear_conv_kernel_dim
constexpr int kConvTimeBlock = 64;

struct PrepArgs {
    const uint16_t *x;        // [B, S, C] bf16, C = 2*key_dim + val_dim
    const uint16_t *w;        // [C, 4] bf16, tap 3 multiplies the current frame
    const uint16_t *state_in; // [B, C, 3] bf16 or nullptr (= zeros)
    uint16_t *state_out;      // [B, C, 3]
    uint16_t *q, *k, *v;      // [B, S, key_dim], [B, S, key_dim], [B, S, val_dim]
    int32_t B, S, C, key_dim, val_dim;
};

__device__ __forceinline__ float rbf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }
__device__ __forceinline__ float silu(float x) { return x / (1.0f + expf(-x)); }

// thread = (sequence, block of 64 frames, channel); channels are the fastest index, so loads and stores coalesce
__global__ __launch_bounds__(256) void deltanet_conv_kernel(PrepArgs a) {
#pragma clang fp contract(off)
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= a.C) return;
    const int t0 = blockIdx.y * kConvTimeBlock, b = blockIdx.z;
    const int t1 = min(a.S, t0 + kConvTimeBlock);
    auto frame = [&](int t) -> float {  // input frame t of this channel; t < 0 reaches into the carried state
        if (t >= 0) return bf16_bits_to_f32(a.x[((int64_t)b * a.S + t) * a.C + c]);
        return a.state_in ? bf16_bits_to_f32(a.state_in[((int64_t)b * a.C + c) * (kConvK - 1) + (kConvK - 1 + t)]) : 0.0f;
    };
    float wt[kConvK];
#pragma unroll
    for (int i = 0; i < kConvK; ++i) wt[i] = bf16_bits_to_f32(a.w[(int64_t)c * kConvK + i]);
    float h0 = frame(t0 - 3), h1 = frame(t0 - 2), h2 = frame(t0 - 1);
    uint16_t *dst;
    int64_t stride, off;
    if (c < a.key_dim) { dst = a.q; stride = a.key_dim; off = c; }
    else if (c < 2 * a.key_dim) { dst = a.k; stride = a.key_dim; off = c - a.key_dim; }
    else { dst = a.v; stride = a.val_dim; off = c - 2 * a.key_dim; }
    for (int t = t0; t < t1; ++t) {
        const float h3 = frame(t);
        float acc = wt[0] * h0;
        acc += wt[1] * h1;
        acc += wt[2] * h2;
        acc += wt[3] * h3;
        dst[((int64_t)b * a.S + t) * stride + off] = (uint16_t)f32_to_bf16_bits(silu(rbf16(acc)));
        h0 = h1; h1 = h2; h2 = h3;
    }
    if (t1 == a.S) {  // this thread saw the end of the sequence: the last three frames are the new state
        uint16_t *so = a.state_out + ((int64_t)b * a.C + c) * (kConvK - 1);
        so[0] = (uint16_t)f32_to_bf16_bits(h0);
        so[1] = (uint16_t)f32_to_bf16_bits(h1);
        so[2] = (uint16_t)f32_to_bf16_bits(h2);
    }
}

__global__ __launch_bounds__(256) void deltanet_gates_kernel(const uint16_t *a_in, const uint16_t *b_in, const float *neg_a_exp,
                                                            const float *dt_bias, float *g, float *beta, int64_t n, int nv) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int j = (int)(i % nv);
    const float x = bf16_bits_to_f32(a_in[i]) + dt_bias[j];
    const float sp = x > 20.0f ? x : log1pf(expf(x));  // softplus with libtorch's linear threshold
    g[i] = neg_a_exp[j] * sp;
    beta[i] = 1.0f / (1.0f + expf(-bf16_bits_to_f32(b_in[i])));
}

// one wavefront per (token, head) row of D = 64 * E elements
template <int E>
__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(const float *x, const uint16_t *z, const float *w, float eps,
                                                           uint16_t *out, int64_t rows) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    constexpr int D = 64 * E;
    float xv[E], ss = 0.0f;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        xv[e] = x[row * D + lane * E + e];
        ss += xv[e] * xv[e];
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) ss += __shfl_xor(ss, o, 64);
    const float rrms = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int d = lane * E + e;
        out[row * D + d] = (uint16_t)f32_to_bf16_bits(xv[e] * rrms * w[d] * silu(bf16_bits_to_f32(z[row * D + d])));
    }
}

}  // namespace hs

extern "C" {

int hs_deltanet_prepare(const void *mixed_qkv, const void *conv_weight, const void *conv_state_in, void *conv_state_out,
                        const void *a_in, const void *b_in, const float *neg_a_exp, const float *dt_bias, void *q, void *k,
                        void *v, float *g, float *beta, int32_t B, int32_t S, int32_t nk, int32_t nv, int32_t dk, int32_t dv,
                        hs_stream_t stream) {
    using namespace hs;
    if (B > 0 && S > 0 &&
        (!mixed_qkv || !conv_weight || !conv_state_out || !a_in || !b_in || !neg_a_exp || !dt_bias || !q || !k || !v || !g || !beta))
        return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (conv_state_out && conv_state_in == conv_state_out) return fail(HS_ERR_INVALID_ARGUMENT, "conv_state_out must not alias conv_state_in");
    if (B < 0 || S < 0 || nk <= 0 || nv <= 0 || dk <= 0 || dv <= 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "bad shape B=%d S=%d nk=%d nv=%d dk=%d dv=%d", B, S, nk, nv, dk, dv);
    if (B == 0 || S == 0) return HS_OK;
    PrepArgs a;
    a.x = (const uint16_t *)mixed_qkv; a.w = (const uint16_t *)conv_weight;
    a.state_in = (const uint16_t *)conv_state_in; a.state_out = (uint16_t *)conv_state_out;
    a.q = (uint16_t *)q; a.k = (uint16_t *)k; a.v = (uint16_t *)v;
    a.B = B; a.S = S; a.key_dim = nk * dk; a.val_dim = nv * dv; a.C = 2 * a.key_dim + a.val_dim;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((unsigned)((a.C + 255) / 256), (unsigned)((S + kConvTimeBlock - 1) / kConvTimeBlock), (unsigned)B);
    deltanet_conv_kernel<<<grid, 256, 0, st>>>(a);
    if (int rc = check_launch("deltanet_conv")) return rc;
    const int64_t n = (int64_t)B * S * nv;
    deltanet_gates_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>((const uint16_t *)a_in, (const uint16_t *)b_in, neg_a_exp,
                                                                       dt_bias, g, beta, n, nv);
    return check_launch("deltanet_gates");
}

int hs_deltanet_gated_norm(const float *x, const void *z, const float *weight, float eps, void *out, int64_t rows, int32_t D,
                           hs_stream_t stream) {
    using namespace hs;
    if (rows > 0 && (!x || !z || !weight || !out)) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (rows < 0 || (D != 64 && D != 128 && D != 256)) return fail(HS_ERR_INVALID_ARGUMENT, "bad shape rows=%lld D=%d", (long long)rows, D);
    if (rows == 0) return HS_OK;
    const unsigned blocks = (unsigned)((rows + 3) / 4);
    hipStream_t st = (hipStream_t)stream;
    if (D == 64) gated_rmsnorm_kernel<1><<<blocks, 256, 0, st>>>(x, (const uint16_t *)z, weight, eps, (uint16_t *)out, rows);
    else if (D == 128) gated_rmsnorm_kernel<2><<<blocks, 256, 0, st>>>(x, (const uint16_t *)z, weight, eps, (uint16_t *)out, rows);
    else gated_rmsnorm_kernel<4><<<blocks, 256, 0, st>>>(x, (const uint16_t *)z, weight, eps, (uint16_t *)out, rows);
    return check_launch("gated_rmsnorm");
}

}  // extern "C"
