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

// SiLU through v_exp_f32 and v_rcp_f32 (a few fp32 ulp; the result is rounded to bf16 right after).
__device__ __forceinline__ float silu_fast(float x) {
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

// The same for channel counts that are multiples of 8: a thread owns 8 adjacent channels (16-byte accesses) and
// kConvFrames frames, and issues all its loads before it computes, so the kernel runs at memory speed instead of
// at the latency of one 2-byte load per frame.  thread = (sequence, frame block, channel octet).
constexpr int kConvFrames = 16;
__global__ __launch_bounds__(256) void deltanet_conv8_kernel(PrepArgs a) {
#pragma clang fp contract(off)
    const int c = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (c >= a.C) return;
    const int t0 = blockIdx.y * kConvFrames, b = blockIdx.z;
    const int nt = min(a.S - t0, kConvFrames);
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 fr[kConvFrames + 3];  // frames t0-3 .. t0+kConvFrames-1, 8 channels each
#pragma unroll
    for (int i = 0; i < kConvFrames + 3; ++i) {
        const int t = t0 - 3 + i;
        fr[i] = (u32x4){0u, 0u, 0u, 0u};
        if (t >= 0) {
            if (i < nt + 3) fr[i] = __builtin_nontemporal_load((const u32x4 *)(a.x + ((int64_t)b * a.S + t) * a.C + c));
        } else if (a.state_in) {  // carried state [B, C, 3]: frame -3 + j of channel c + e is element 3*e + j
            const uint16_t *sp = a.state_in + ((int64_t)b * a.C + c) * 3 + (3 + t);
            uint32_t h[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) h[e] = sp[3 * e];
            fr[i] = (u32x4){h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
        }
    }
    u32x4 wq[4];  // w[c + e][tap] = element 4*e + tap of these 64 bytes
#pragma unroll
    for (int i = 0; i < 4; ++i) wq[i] = *(const u32x4 *)(a.w + (int64_t)c * kConvK + 8 * i);
    auto lo = [](uint32_t w) { return __uint_as_float(w << 16); };
    auto hi = [](uint32_t w) { return __uint_as_float(w & 0xffff0000u); };
    float wt[8][kConvK];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t w01 = wq[e >> 1][2 * (e & 1)], w23 = wq[e >> 1][2 * (e & 1) + 1];
        wt[e][0] = lo(w01); wt[e][1] = hi(w01); wt[e][2] = lo(w23); wt[e][3] = hi(w23);
    }
    uint16_t *dst;
    int64_t stride, off;
    if (c < a.key_dim) { dst = a.q; stride = a.key_dim; off = c; }
    else if (c < 2 * a.key_dim) { dst = a.k; stride = a.key_dim; off = c - a.key_dim; }
    else { dst = a.v; stride = a.val_dim; off = c - 2 * a.key_dim; }
    auto chan = [&](const u32x4 &f, int e) { return (e & 1) ? hi(f[e >> 1]) : lo(f[e >> 1]); };
#pragma unroll
    for (int i = 0; i < kConvFrames; ++i) {
        if (i >= nt) continue;
        float y[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float acc = wt[e][0] * chan(fr[i], e);
            acc += wt[e][1] * chan(fr[i + 1], e);
            acc += wt[e][2] * chan(fr[i + 2], e);
            acc += wt[e][3] * chan(fr[i + 3], e);
            y[e] = silu_fast((float)(__bf16)acc);  // the conv output is a bf16 tensor before the SiLU
        }
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        uint32_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {  // hardware round-to-nearest-even conversion, two values per instruction
            const bf16x2 p = {(__bf16)y[2 * e], (__bf16)y[2 * e + 1]};
            o[e] = __builtin_bit_cast(uint32_t, p);
        }
        __builtin_nontemporal_store((u32x4){o[0], o[1], o[2], o[3]}, (u32x4 *)(dst + ((int64_t)b * a.S + t0 + i) * stride + off));
    }
    if (t0 + nt == a.S) {  // this thread saw the end of the sequence: the last three frames are the new state
        uint16_t *so = a.state_out + ((int64_t)b * a.C + c) * 3;
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            u32x4 f = fr[0];
#pragma unroll
            for (int i = 0; i < kConvFrames + 3; ++i)
                if (i == nt + j) f = fr[i];
#pragma unroll
            for (int e = 0; e < 8; ++e) so[3 * e + j] = (uint16_t)((e & 1) ? f[e >> 1] >> 16 : f[e >> 1] & 0xffffu);
        }
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

// The same with D/8 lanes per row (eight elements each: 16-byte accesses, 64/(D/8) rows per wavefront).
template <int LPR>
__global__ __launch_bounds__(256) void gated_rmsnorm_rows_kernel(const float *x, const uint16_t *z, const float *w, float eps,
                                                                uint16_t *out, int64_t rows) {
    constexpr int D = 8 * LPR;
    const int lane = threadIdx.x & 63, sub = lane % LPR;
    int64_t row = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * (64 / LPR) + lane / LPR;
    const bool live = row < rows;  // lanes past the end still take part in the shuffles
    if (!live) row = rows - 1;
    const int64_t e0 = row * D + sub * 8;
    typedef float f4v __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const f4v xa = __builtin_nontemporal_load((const f4v *)(x + e0)), xb = __builtin_nontemporal_load((const f4v *)(x + e0 + 4));
    const u32x4 zz = __builtin_nontemporal_load((const u32x4 *)(z + e0));
    const float4 wa = *(const float4 *)(w + sub * 8), wb = *(const float4 *)(w + sub * 8 + 4);
    const float xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
    const float wv[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
    const uint32_t zw[4] = {zz[0], zz[1], zz[2], zz[3]};
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += xv[e] * xv[e];
#pragma unroll
    for (int o = 1; o < LPR; o <<= 1) ss += __shfl_xor(ss, o, 64);
    const float rrms = 1.0f / sqrtf(ss / (float)D + eps);
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    uint32_t o4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float z0 = __uint_as_float(zw[i] << 16), z1 = __uint_as_float(zw[i] & 0xffff0000u);
        const bf16x2 p = {(__bf16)(xv[2 * i] * rrms * wv[2 * i] * silu_fast(z0)),
                          (__bf16)(xv[2 * i + 1] * rrms * wv[2 * i + 1] * silu_fast(z1))};
        o4[i] = __builtin_bit_cast(uint32_t, p);
    }
    if (live) __builtin_nontemporal_store((u32x4){o4[0], o4[1], o4[2], o4[3]}, (u32x4 *)(out + e0));
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
    const bool wide = (a.key_dim % 8) == 0 && (a.val_dim % 8) == 0 &&
                      (((uintptr_t)mixed_qkv | (uintptr_t)conv_weight | (uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) == 0;
    if (wide) {
        dim3 grid((unsigned)((a.C / 8 + 255) / 256), (unsigned)((S + kConvFrames - 1) / kConvFrames), (unsigned)B);
        deltanet_conv8_kernel<<<grid, 256, 0, st>>>(a);
    } else {
        dim3 grid((unsigned)((a.C + 255) / 256), (unsigned)((S + kConvTimeBlock - 1) / kConvTimeBlock), (unsigned)B);
        deltanet_conv_kernel<<<grid, 256, 0, st>>>(a);
    }
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
    hipStream_t st = (hipStream_t)stream;
    if ((((uintptr_t)x | (uintptr_t)z | (uintptr_t)weight | (uintptr_t)out) & 15) == 0) {  // several rows per wavefront
        const int rows_per_wg = 4 * (64 / (D / 8));
        const unsigned g = (unsigned)((rows + rows_per_wg - 1) / rows_per_wg);
        if (D == 64) gated_rmsnorm_rows_kernel<8><<<g, 256, 0, st>>>(x, (const uint16_t *)z, weight, eps, (uint16_t *)out, rows);
        else if (D == 128) gated_rmsnorm_rows_kernel<16><<<g, 256, 0, st>>>(x, (const uint16_t *)z, weight, eps, (uint16_t *)out, rows);
        else gated_rmsnorm_rows_kernel<32><<<g, 256, 0, st>>>(x, (const uint16_t *)z, weight, eps, (uint16_t *)out, rows);
        return check_launch("gated_rmsnorm");
    }
    const unsigned blocks = (unsigned)((rows + 3) / 4);
    if (D == 64) gated_rmsnorm_kernel<1><<<blocks, 256, 0, st>>>(x, (const uint16_t *)z, weight, eps, (uint16_t *)out, rows);
    else if (D == 128) gated_rmsnorm_kernel<2><<<blocks, 256, 0, st>>>(x, (const uint16_t *)z, weight, eps, (uint16_t *)out, rows);
    else gated_rmsnorm_kernel<4><<<blocks, 256, 0, st>>>(x, (const uint16_t *)z, weight, eps, (uint16_t *)out, rows);
    return check_launch("gated_rmsnorm");
}

// The prompt branch of the layer as one call: the launches of the three steps in a row, the intermediate tensors in the
// workspace.
static size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

size_t hs_deltanet_prefill_layer_workspace_bytes(int32_t B, int32_t S, int32_t nk, int32_t nv, int32_t dk, int32_t dv) {
    if (B <= 0 || S <= 0 || nk <= 0 || nv <= 0 || dk <= 0 || dv <= 0) return 0;
    const size_t bs = (size_t)B * S;
    return align256(hs_deltanet_chunked_gated_norm_workspace_bytes(B, S, nk, nv)) + 2 * align256(bs * nk * dk * 2) + align256(bs * nv * dv * 2) +
           2 * align256(bs * nv * 4);
}

int hs_deltanet_prefill_layer(const void *mixed_qkv, const void *conv_weight, const void *conv_state_in, void *conv_state_out,
                              const void *a_in, const void *b_in, const float *neg_a_exp, const float *dt_bias, const void *z,
                              const float *norm_weight, float norm_eps, float *state, void *out, int32_t B, int32_t S,
                              int32_t nk, int32_t nv, int32_t dk, int32_t dv, float q_scale, int l2norm, void *workspace,
                              size_t workspace_bytes, hs_stream_t stream) {
    using namespace hs;
    if (B < 0 || S < 0 || nk <= 0 || nv <= 0 || dk <= 0 || dv <= 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "bad shape B=%d S=%d nk=%d nv=%d dk=%d dv=%d", B, S, nk, nv, dk, dv);
    if (B == 0 || S == 0) return HS_OK;
    const size_t need = hs_deltanet_prefill_layer_workspace_bytes(B, S, nk, nv, dk, dv);
    if (!workspace || workspace_bytes < need) return fail(HS_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    if (((uintptr_t)workspace & 255) != 0) return fail(HS_ERR_INVALID_ARGUMENT, "workspace must be 256-byte aligned");
    const size_t bs = (size_t)B * S;
    uint8_t *p = (uint8_t *)workspace;
    void *chunk_ws = p;
    const size_t chunk_bytes = hs_deltanet_chunked_gated_norm_workspace_bytes(B, S, nk, nv);
    p += align256(chunk_bytes);
    void *q = p; p += align256(bs * nk * dk * 2);
    void *k = p; p += align256(bs * nk * dk * 2);
    void *v = p; p += align256(bs * nv * dv * 2);
    float *g = (float *)p; p += align256(bs * nv * 4);
    float *beta = (float *)p;
    if (int rc = hs_deltanet_prepare(mixed_qkv, conv_weight, conv_state_in, conv_state_out, a_in, b_in, neg_a_exp, dt_bias, q, k, v,
                                     g, beta, B, S, nk, nv, dk, dv, stream))
        return rc;
    return hs_deltanet_forward_chunked_gated_norm(q, k, v, g, beta, state, z, norm_weight, norm_eps, out, B, S, nk, nv, dk, dv,
                                                  q_scale, l2norm, chunk_ws, chunk_bytes, stream);
}

}  // extern "C"
