// Quantize-on-write and dense-view kernels for the int8 / FP8-e4m3fn KV cache (gfx950).
//
// One 64-lane wavefront owns one (sequence, token, kv-head) row of head_dim elements,
// E = D/64 consecutive elements per lane: the absmax is a wavefront max-reduction, the
// row's codes leave as one coalesced store, the scale as a single dword.  HBM traffic is
// read 2 or 4 B + write 1 B per element (+4 B per row); only the S new tokens are touched.
//
// Arithmetic is written to be bit-identical to the CPU oracle: IEEE fp32 division
// (-fhip-fp32-correctly-rounded-divide-sqrt), round-half-even (v_rndne_f32), no fast-math.
#include "prologue_rows.hpp"
#include "quant_device.hpp"

namespace hs {

template <int E, bool FP8>
__global__ __launch_bounds__(256) void kv_quantize_kernel(QuantArgs a) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (int64_t)a.B * a.S * a.Hkv) return;
    quantize_row<E, FP8>(a, blockIdx.y, row, threadIdx.x & 63);
}

// Quantize-on-write for many rows: LPR = D/8 lanes own one row (eight consecutive elements each, one 16-byte
// load for 16-bit sources and one 8-byte store of codes), so a wavefront carries 64/LPR rows and the per-row
// bookkeeping -- index arithmetic, address resolution, the absmax reduction, the scale store -- is paid once
// per wavefront instead of once per row.  The arithmetic per element is that of quantize_row (same IEEE
// divisions, same rounding): the codes and scales are the same bits.  Grid: (row groups of one sequence, K/V, B).
template <int LPR, bool FP8>
__global__ __launch_bounds__(256) void kv_quantize_rows_kernel(QuantArgs a) {
#pragma clang fp contract(off)
    constexpr int kRowsPerWave = 64 / LPR;
    const int which = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, sub = lane % LPR;
    const int r = (blockIdx.x * 4 + (threadIdx.x >> 6)) * kRowsPerWave + lane / LPR;  // row inside the sequence
    const int nr = a.S * a.Hkv;
    const bool live = r < nr;  // lanes of rows past the end still take part in the shuffles
    const int rr = live ? r : nr - 1;
    const int s = rr / a.Hkv, h = rr - s * a.Hkv;
    const int pos = (a.positions ? a.positions[b] : 0) + a.start_pos + s;
    const KvAddr &ad = a.addr[which];
    int64_t unit;
    int slot;
    const bool ok = resolve(ad, b, pos, unit, slot) && live;
    const int64_t e0 = ((int64_t)b * nr + rr) * a.D + sub * 8;  // first of this lane's eight elements
    float x[8];
    if (a.dtype == HS_F32) {
        const float4 lo = *(const float4 *)((const float *)a.src[which] + e0), hi = *(const float4 *)((const float *)a.src[which] + e0 + 4);
        x[0] = lo.x; x[1] = lo.y; x[2] = lo.z; x[3] = lo.w; x[4] = hi.x; x[5] = hi.y; x[6] = hi.z; x[7] = hi.w;
    } else {
        const uint4 w = *(const uint4 *)((const uint16_t *)a.src[which] + e0);
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (a.dtype == HS_BF16) {
                x[2 * i] = __uint_as_float(ww[i] << 16);
                x[2 * i + 1] = __uint_as_float(ww[i] & 0xffff0000u);
            } else {
                _Float16 f[2];
                __builtin_memcpy(f, &ww[i], 4);
                x[2 * i] = (float)f[0];
                x[2 * i + 1] = (float)f[1];
            }
        }
    }
    float sc = 0.0f;
    uint32_t packed[2] = {0u, 0u};
    if (FP8) {  // one scale per (sequence, kv-head), read; the element arithmetic of quantize_row
        sc = a.scales[which][(int64_t)b * a.Hkv + h];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float y = 0.0f;
            if (sc > 0.0f) {
                y = x[e] / sc;
                if (y > 448.0f) y = 448.0f;
                if (y < -448.0f) y = -448.0f;
            }
            packed[e >> 2] |= f32_to_e4m3fn_bits(y) << (8 * (e & 3));
        }
    } else {
        float m = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float v = fabsf(x[e]);
            m = v > m ? v : m;
        }
#pragma unroll
        for (int o = LPR / 2; o > 0; o >>= 1) {
            const float w = __shfl_xor(m, o, 64);
            m = m > w ? m : w;
        }
        if (m > 0.0f) {
            sc = m / 127.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float q = rintf(x[e] / sc);
                q = q > 127.0f ? 127.0f : q;
                q = q < -127.0f ? -127.0f : q;
                if (q != q) q = 0.0f;
                packed[e >> 2] |= ((uint32_t)(int)q & 0xffu) << (8 * (e & 3));
            }
        }
    }
    if (!ok) return;
    uint8_t *dst = (uint8_t *)a.codes[which] + unit * ad.code_stride_seq + (int64_t)h * ad.code_stride_head +
                   (int64_t)slot * a.D + sub * 8;
    *(uint2 *)dst = make_uint2(packed[0], packed[1]);
    if (!FP8 && sub == 0) a.scales[which][unit * ad.scale_stride_seq + (int64_t)h * ad.scale_stride_head + slot] = sc;
}

struct RopeArgs {
    const void *x, *sin_t, *cos_t;
    void *out;
    const int32_t *positions;
    int32_t start_pos, rope_len, B, S, H, D, dtype;
    int32_t rd;  // rotated leading part of each row (pairs d, d + rd/2); elements [rd, D) pass through
};

// Rotary embedding of a [B, S, H, D] tensor (the query side of a step; K is rotated inside the cache write).
template <int E>
__global__ __launch_bounds__(256) void rope_apply_kernel(RopeArgs a) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (int64_t)a.B * a.S * a.H) return;
    const int64_t bs = row / a.H;
    const int s = (int)(bs % a.S), b = (int)(bs / a.S);
    const int pos = (a.positions ? a.positions[b] : 0) + a.start_pos + s;
    float x[E];
    load_src<E>(a.x, a.dtype, row * a.D + lane * E, x);
    if (lane * E < a.rd) rope_rotate<E>(a.x, a.dtype, row * a.D, a.rd, a.sin_t, a.cos_t, a.rope_len, pos, lane * E, x);
    const int64_t o = row * a.D + lane * E;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        if (a.dtype == HS_F32) ((float *)a.out)[o + e] = x[e];
        else if (a.dtype == HS_BF16) ((uint16_t *)a.out)[o + e] = (uint16_t)f32_to_bf16_bits(x[e]);
        else {
            _Float16 f = (_Float16)x[e];
            __builtin_memcpy((uint16_t *)a.out + o + e, &f, 2);
        }
    }
}

struct PrologueArgs {
    const void *x[2];   // q [B, S, Hq, D], k [B, S, Hkv, D] (either may be null)
    void *out[2];
    NormSpec norm[2];
    const void *sin_t, *cos_t;  // null: no rotation
    const int32_t *positions;
    int32_t start_pos, rope_len, B, S, H[2], D, dtype, rd;
};

// What runs on q and k between the projections and cache.update / attention, in one launch over both tensors:
// per-head QK-norm (NormSpec) and the (partial) rotary embedding of the normalised rows.  One wavefront per
// (token, head) row, E = D/64 consecutive elements per lane; row r of the launch is head r % (Hq + Hkv) of token
// r / (Hq + Hkv), the q heads first.
template <int E>
__global__ __launch_bounds__(256) void qk_prologue_kernel(PrologueArgs a) {
#pragma clang fp contract(off)
    const int lane = threadIdx.x & 63;
    const int HH = a.H[0] + a.H[1];
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= (int64_t)a.B * a.S * HH) return;
    const int64_t bs = r / HH;
    const int hh = (int)(r - bs * HH);
    const int which = hh >= a.H[0] ? 1 : 0, h = which ? hh - a.H[0] : hh;
    const int s = (int)(bs % a.S), b = (int)(bs / a.S);
    const int pos = (a.positions ? a.positions[b] : 0) + a.start_pos + s;
    const int64_t row = bs * a.H[which] + h;
    const NormSpec &n = a.norm[which];
    float x[E];
    load_src<E>(a.x[which], a.dtype, row * a.D + lane * E, x);
    float rrms = 0.0f;
    if (n.kind != 0) {
        double ss = 0.0;
#pragma unroll
        for (int e = 0; e < E; ++e) ss += (double)norm_square(x[e], a.dtype, n.kind);
        rrms = norm_rrms(wave_sum_f64(ss), a.D, a.dtype, n.kind, n.eps);
        float w[E];
        norm_weights<E>(n, a.dtype, h, lane * E, w);
#pragma unroll
        for (int e = 0; e < E; ++e) x[e] = norm_apply(x[e], w[e], rrms, a.dtype, n.kind);
    }
    if (a.sin_t != nullptr && lane * E < a.rd)
        rope_rotate<E>(a.x[which], a.dtype, row * a.D, a.rd, a.sin_t, a.cos_t, a.rope_len, pos, lane * E, x, &n, rrms, h);
    const int64_t o = row * a.D + lane * E;
    void *out = a.out[which];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        if (a.dtype == HS_F32) ((float *)out)[o + e] = x[e];
        else if (a.dtype == HS_BF16) ((uint16_t *)out)[o + e] = (uint16_t)f32_to_bf16_bits(x[e]);
        else {
            _Float16 f = (_Float16)x[e];
            __builtin_memcpy((uint16_t *)out + o + e, &f, 2);
        }
    }
}

// qk_prologue_kernel for 16-bit tensors with 16-byte-aligned buffers: D/8 lanes own a row, eight consecutive
// elements each (one 16-byte load, one 16-byte store; 16-byte loads of the weights and of the sin/cos entries), so a
// wavefront carries 64/(D/8) rows.  The sum of squares is reduced over the lanes of the row; the rotation takes a
// partner's NORMALISED value from the lane that holds it instead of reading and normalising the partner again.  Per
// element the operations and their roundings are those of the one-row-per-wavefront kernel: the same bits.
// DT: the tensor dtype (HS_BF16 or HS_F16) as a compile-time constant, so that the per-operation rounding is one
// instruction and not a three-way choice.
template <int LPR, int DT>
__global__ __launch_bounds__(256) void qk_prologue_rows_kernel(PrologueArgs a) {
#pragma clang fp contract(off)
    constexpr int kRowsPerWave = 64 / LPR;
    const int lane = threadIdx.x & 63, sub = lane % LPR;
    const int HH = a.H[0] + a.H[1];
    const int total = a.B * a.S * HH;  // the host sends larger problems to the one-row-per-wavefront kernel
    // Row -> (token, head) and token -> (sequence, position) with the divisions done once per wavefront on scalars:
    // a lane's row is at most kRowsPerWave - 1 past the wavefront's first one, so it only steps forward from there.
    const int wave_row = (blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6)) * kRowsPerWave;
    const int r_raw = wave_row + lane / LPR;
    const bool live = r_raw < total;  // lanes of rows past the end still take part in the shuffles
    const int first = min(wave_row, total - 1);
    int bs = first / HH, hh = first - bs * HH + (min(r_raw, total - 1) - first);
    while (hh >= HH) {
        hh -= HH;
        ++bs;
    }
    const int bs0 = first / HH;
    int b = bs0 / a.S, s = bs0 - b * a.S + (bs - bs0);
    while (s >= a.S) {
        s -= a.S;
        ++b;
    }
    const int which = hh >= a.H[0] ? 1 : 0, h = which ? hh - a.H[0] : hh;
    const int pos = (a.positions ? a.positions[b] : 0) + a.start_pos + s;
    const int64_t row = (int64_t)bs * a.H[which] + h;
    const NormSpec &n = a.norm[which];
    const int d0 = sub * 8;
    const auto unpack = [&](const uint4 v, float (&f)[8]) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint16_t h16 = (uint16_t)((i & 1) ? w[i >> 1] >> 16 : w[i >> 1] & 0xffffu);
            if (DT == HS_BF16) f[i] = bf16_bits_to_f32(h16);
            else {
                _Float16 t;
                __builtin_memcpy(&t, &h16, 2);
                f[i] = (float)t;
            }
        }
    };
    float x[8];
    unpack(*(const uint4 *)((const uint16_t *)a.x[which] + row * a.D + d0), x);
    if (n.kind != 0) {
        double ss = 0.0;
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += (double)norm_square(x[e], DT, n.kind);
#pragma unroll
        for (int o = LPR / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
        const float rrms = norm_rrms(ss, a.D, DT, n.kind, n.eps);
        float w[8];
        if (n.kind == 1) {
            unpack(*(const uint4 *)((const uint16_t *)n.weight + (int64_t)h * n.head_stride + d0), w);
        } else {
            const float4 w0 = *(const float4 *)((const float *)n.weight + (int64_t)h * n.head_stride + d0);
            const float4 w1 = *(const float4 *)((const float *)n.weight + (int64_t)h * n.head_stride + d0 + 4);
            w[0] = w0.x; w[1] = w0.y; w[2] = w0.z; w[3] = w0.w;
            w[4] = w1.x; w[5] = w1.y; w[6] = w1.z; w[7] = w1.w;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = norm_apply(x[e], w[e], rrms, DT, n.kind);
    }
    if (a.sin_t != nullptr) {
        const int half = a.rd / 2;
        const bool rotated = d0 < a.rd, upper = d0 >= half;
        // the partner's eight elements sit half/8 lanes away in the same row
        const int src_lane = rotated ? (upper ? lane - half / 8 : lane + half / 8) : lane;
        float other[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) other[e] = __shfl(x[e], src_lane, 64);
        if (rotated) {
            const int p = pos < 0 ? 0 : (pos >= a.rope_len ? a.rope_len - 1 : pos);
            const int j0 = upper ? d0 - half : d0;
            float sn[8], cs[8];
            unpack(*(const uint4 *)((const uint16_t *)a.sin_t + (int64_t)p * half + j0), sn);
            unpack(*(const uint4 *)((const uint16_t *)a.cos_t + (int64_t)p * half + j0), cs);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float own_cos = round_to_dtype(x[e] * cs[e], DT);
                const float other_sin = round_to_dtype(other[e] * sn[e], DT);
                x[e] = round_to_dtype(upper ? other_sin + own_cos : own_cos - other_sin, DT);
            }
        }
    }
    if (!live) return;
    uint32_t res[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t r2[2];
#pragma unroll
        for (int hsel = 0; hsel < 2; ++hsel) {
            const float y = x[2 * i + hsel];
            if (DT == HS_BF16) r2[hsel] = f32_to_bf16_bits(y);
            else {
                const _Float16 t = (_Float16)y;
                uint16_t h16;
                __builtin_memcpy(&h16, &t, 2);
                r2[hsel] = h16;
            }
        }
        res[i] = r2[0] | (r2[1] << 16);
    }
    *(uint4 *)((uint16_t *)a.out[which] + row * a.D + d0) = make_uint4(res[0], res[1], res[2], res[3]);
}

// qk_prologue_rows_kernel for bf16 with longer pieces: a lane owns E = 32 consecutive elements of a row (16 at head_dim
// 64), D/E adjacent lanes a row (prologue_row_part).  What comes once per lane whatever its share -- row and position
// arithmetic, the reciprocal root's chain of roundings, the reduction steps, the exchange's addressing -- is spread over
// four times as many elements, which is what bounds this launch (its arithmetic, not its bytes).
// Serves the rotary_dim values of prologue_parts_serve(rd, E).
template <int D>
__global__ __launch_bounds__(256) void qk_prologue_parts_kernel(PrologueArgs a) {
    constexpr int E = D == 64 ? 16 : 32, P = D / E, kRowsPerWave = 64 / P;
    const int lane = threadIdx.x & 63, part = lane % P;
    const int HH = a.H[0] + a.H[1];
    const int total = a.B * a.S * HH;
    const int wave_row = (blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6)) * kRowsPerWave;
    const int r_raw = wave_row + lane / P;
    const bool live = r_raw < total;  // lanes of rows past the end still take part in the shuffles
    const int first = min(wave_row, total - 1);
    int bs = first / HH, hh = first - bs * HH + (min(r_raw, total - 1) - first);
    while (hh >= HH) {
        hh -= HH;
        ++bs;
    }
    const int bs0 = first / HH;
    int b = bs0 / a.S, s = bs0 - b * a.S + (bs - bs0);
    while (s >= a.S) {
        s -= a.S;
        ++b;
    }
    const int which = hh >= a.H[0] ? 1 : 0, h = which ? hh - a.H[0] : hh;
    const int pos = (a.positions ? a.positions[b] : 0) + a.start_pos + s;
    const int64_t row = (int64_t)bs * a.H[which] + h;
    RowPrologue p;
    p.norm = a.norm[which];
    p.sin_t = a.sin_t;
    p.cos_t = a.cos_t;
    p.rope_len = a.rope_len;
    p.rd = a.rd;
    u32x4 res[E / 8];
    prologue_row_part<D, E>(p, (const uint16_t *)a.x[which] + row * D, h, pos, part, 1, lane, res);
    if (!live) return;
    uint16_t *dst = (uint16_t *)a.out[which] + row * D + E * part;
#pragma unroll
    for (int i = 0; i < E / 8; ++i) *(u32x4 *)(dst + 8 * i) = res[i];
}

// The same for many rows of a 16-bit tensor: D/8 lanes own a row, eight consecutive elements each (16-byte loads
// of the lane's elements, of their partners half a row away and of the sin/cos entries; one 16-byte store), so a
// wavefront carries 64/(D/8) rows.  Per element the operations and their roundings are those of rope_rotate().
template <int LPR>
__global__ __launch_bounds__(256) void rope_apply_rows_kernel(RopeArgs a) {
#pragma clang fp contract(off)
    constexpr int kRowsPerWave = 64 / LPR;
    const int lane = threadIdx.x & 63, sub = lane % LPR;
    const int64_t row = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * kRowsPerWave + lane / LPR;
    if (row >= (int64_t)a.B * a.S * a.H) return;
    const int64_t bs = row / a.H;
    const int s = (int)(bs % a.S), b = (int)(bs / a.S);
    const int pos = (a.positions ? a.positions[b] : 0) + a.start_pos + s;
    const int p = pos < 0 ? 0 : (pos >= a.rope_len ? a.rope_len - 1 : pos);
    const int half = a.rd / 2, d0 = sub * 8;
    const uint16_t *xr = (const uint16_t *)a.x + row * a.D;
    const uint4 own = *(const uint4 *)(xr + d0);
    if (d0 >= a.rd) {  // beyond the rotated part
        *(uint4 *)((uint16_t *)a.out + row * a.D + d0) = own;
        return;
    }
    const bool upper = d0 >= half;
    const int j0 = upper ? d0 - half : d0;
    const uint4 oth = *(const uint4 *)(xr + (upper ? d0 - half : d0 + half));
    const uint4 sn = *(const uint4 *)((const uint16_t *)a.sin_t + (int64_t)p * half + j0);
    const uint4 cs = *(const uint4 *)((const uint16_t *)a.cos_t + (int64_t)p * half + j0);
    const uint32_t wo[4] = {own.x, own.y, own.z, own.w}, wp[4] = {oth.x, oth.y, oth.z, oth.w};
    const uint32_t ws[4] = {sn.x, sn.y, sn.z, sn.w}, wc[4] = {cs.x, cs.y, cs.z, cs.w};
    uint32_t res[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t r2[2];
#pragma unroll
        for (int hsel = 0; hsel < 2; ++hsel) {
            const auto f = [&](uint32_t w) {
                const uint16_t h16 = (uint16_t)(hsel ? w >> 16 : w & 0xffffu);
                if (a.dtype == HS_BF16) return bf16_bits_to_f32(h16);
                _Float16 t;
                __builtin_memcpy(&t, &h16, 2);
                return (float)t;
            };
            const float own_cos = round_to_dtype(f(wo[i]) * f(wc[i]), a.dtype);
            const float other_sin = round_to_dtype(f(wp[i]) * f(ws[i]), a.dtype);
            const float y = upper ? other_sin + own_cos : own_cos - other_sin;
            if (a.dtype == HS_BF16) r2[hsel] = f32_to_bf16_bits(y);
            else {
                const _Float16 t = (_Float16)y;
                uint16_t h16;
                __builtin_memcpy(&h16, &t, 2);
                r2[hsel] = h16;
            }
        }
        res[i] = r2[0] | (r2[1] << 16);
    }
    *(uint4 *)((uint16_t *)a.out + row * a.D + d0) = make_uint4(res[0], res[1], res[2], res[3]);
}

// scale[b, h] = max_{s, d} |x| / 448.  One workgroup per (b, h, tensor).
__global__ __launch_bounds__(256) void fp8_calibrate_kernel(const void *k_src, const void *v_src, int dtype,
                                                           float *k_scales, float *v_scales, int B, int S, int Hkv,
                                                           int D) {
    const int which = blockIdx.y;
    const int b = blockIdx.x / Hkv, h = blockIdx.x % Hkv;
    const void *src = which ? v_src : k_src;
    float m = 0.0f;
    const int per_row = D;
    for (int64_t i = threadIdx.x; i < (int64_t)S * per_row; i += 256) {
        int s = (int)(i / per_row), d = (int)(i % per_row);
        float x[1];
        load_src<1>(src, dtype, (((int64_t)b * S + s) * Hkv + h) * D + d, x);
        float v = fabsf(x[0]);
        m = v > m ? v : m;
    }
    m = wave_max(m);
    __shared__ float red[4];
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        (which ? v_scales : k_scales)[b * Hkv + h] = m / 448.0f;
    }
}

// The same for 16-bit sources: 1024 threads per (b, h, tensor), 16-byte loads (eight elements), many rows in flight.
__global__ __launch_bounds__(1024) void fp8_calibrate16_kernel(const uint16_t *k_src, const uint16_t *v_src, int dtype,
                                                              float *k_scales, float *v_scales, int B, int S, int Hkv, int D) {
    const int which = blockIdx.y;
    const int b = blockIdx.x / Hkv, h = blockIdx.x % Hkv;
    const uint16_t *src = which ? v_src : k_src;
    const int lpr = D / 8, sub = threadIdx.x % lpr, rows_per_pass = 1024 / lpr;
    float m = 0.0f;
    for (int s0 = threadIdx.x / lpr; s0 < S; s0 += rows_per_pass) {
        const uint4 w = *(const uint4 *)(src + (((int64_t)b * S + s0) * Hkv + h) * D + sub * 8);
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float x0, x1;
            if (dtype == HS_BF16) {
                x0 = __uint_as_float(ww[i] << 16);
                x1 = __uint_as_float(ww[i] & 0xffff0000u);
            } else {
                _Float16 f[2];
                __builtin_memcpy(f, &ww[i], 4);
                x0 = (float)f[0];
                x1 = (float)f[1];
            }
            const float a0 = fabsf(x0), a1 = fabsf(x1);
            m = a0 > m ? a0 : m;
            m = a1 > m ? a1 : m;
        }
    }
    m = wave_max(m);
    __shared__ float red[16];
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int i = 1; i < 16; ++i) m = fmaxf(m, red[i]);
        (which ? v_scales : k_scales)[b * Hkv + h] = m / 448.0f;
    }
}

__device__ __forceinline__ float e4m3fn_bits_to_f32(uint32_t c) {
    uint32_t e = (c >> 3) & 0xfu, m = c & 7u;
    float v;
    if (e == 0) v = (float)m * 0.001953125f;  // m * 2^-9
    else if (e == 15 && m == 7) v = __uint_as_float(0x7fc00000u);
    else v = __uint_as_float(((e + 120u) << 23) | (m << 20));
    return (c & 0x80u) ? -v : v;
}

struct DequantArgs {
    const void *codes;
    const float *scales;
    KvAddr addr;
    void *out;
    int32_t B, T, Hkv, D, out_dtype, fp8;
};

template <int E>
__global__ __launch_bounds__(256) void kv_dequantize_kernel(DequantArgs a) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (int64_t)a.B * a.T * a.Hkv) return;
    const int h = (int)(row % a.Hkv);
    const int64_t bt = row / a.Hkv;
    const int t = (int)(bt % a.T);
    const int b = (int)(bt / a.T);
    int64_t unit;
    int slot;
    float v[E];
    if (resolve(a.addr, b, t, unit, slot)) {
        const uint8_t *src = (const uint8_t *)a.codes + unit * a.addr.code_stride_seq +
                             (int64_t)h * a.addr.code_stride_head + (int64_t)slot * a.D + lane * E;
        float sc = a.fp8 ? a.scales[(int64_t)b * a.Hkv + h]
                         : a.scales[unit * a.addr.scale_stride_seq + (int64_t)h * a.addr.scale_stride_head + slot];
#pragma unroll
        for (int e = 0; e < E; ++e)
            v[e] = sc * (a.fp8 ? e4m3fn_bits_to_f32(src[e]) : (float)(int8_t)src[e]);
    } else {
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] = 0.0f;
    }
    const int64_t o = row * a.D + lane * E;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        if (a.out_dtype == HS_F32) ((float *)a.out)[o + e] = v[e];
        else if (a.out_dtype == HS_BF16) ((uint16_t *)a.out)[o + e] = (uint16_t)f32_to_bf16_bits(v[e]);
        else {
            _Float16 f = (_Float16)v[e];
            __builtin_memcpy((uint16_t *)a.out + o + e, &f, 2);
        }
    }
}

// The same with D/8 lanes per row: 8-byte code loads, 16- or 32-byte stores, 64/(D/8) rows per wavefront.
template <int LPR>
__global__ __launch_bounds__(256) void kv_dequantize_rows_kernel(DequantArgs a) {
    const int lane = threadIdx.x & 63, sub = lane % LPR;
    const int64_t row = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * (64 / LPR) + lane / LPR;
    if (row >= (int64_t)a.B * a.T * a.Hkv) return;
    const int h = (int)(row % a.Hkv);
    const int64_t bt = row / a.Hkv;
    const int t = (int)(bt % a.T);
    const int b = (int)(bt / a.T);
    int64_t unit;
    int slot;
    float v[8];
    if (resolve(a.addr, b, t, unit, slot)) {
        const uint8_t *src = (const uint8_t *)a.codes + unit * a.addr.code_stride_seq +
                             (int64_t)h * a.addr.code_stride_head + (int64_t)slot * a.D + sub * 8;
        const float sc = a.fp8 ? a.scales[(int64_t)b * a.Hkv + h]
                               : a.scales[unit * a.addr.scale_stride_seq + (int64_t)h * a.addr.scale_stride_head + slot];
        const uint2 c8 = *(const uint2 *)src;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t byte = ((e < 4 ? c8.x : c8.y) >> (8 * (e & 3))) & 0xffu;
            v[e] = sc * (a.fp8 ? e4m3fn_bits_to_f32(byte) : (float)(int8_t)byte);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.0f;
    }
    const int64_t o = row * a.D + sub * 8;
    if (a.out_dtype == HS_F32) {
        *(float4 *)((float *)a.out + o) = make_float4(v[0], v[1], v[2], v[3]);
        *(float4 *)((float *)a.out + o + 4) = make_float4(v[4], v[5], v[6], v[7]);
    } else {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t h2[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (a.out_dtype == HS_BF16) h2[j] = f32_to_bf16_bits(v[2 * i + j]);
                else {
                    const _Float16 f = (_Float16)v[2 * i + j];
                    uint16_t u;
                    __builtin_memcpy(&u, &f, 2);
                    h2[j] = u;
                }
            }
            w[i] = h2[0] | (h2[1] << 16);
        }
        *(uint4 *)((uint16_t *)a.out + o) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

// ------------------------------------------------------------------ host launchers

static int check_common(const hs_kv_layout *l, int B, int S, int Hkv, int D, bool need_scales) {
    if (!l) return fail(HS_ERR_INVALID_ARGUMENT, "layout is NULL");
    if (B < 0 || S < 0 || Hkv <= 0) return fail(HS_ERR_INVALID_ARGUMENT, "bad shape B=%d S=%d Hkv=%d", B, S, Hkv);
    if (D != 64 && D != 128 && D != 256) return fail(HS_ERR_INVALID_ARGUMENT, "head_dim %d not in {64,128,256}", D);
    if (l->capacity_tokens <= 0) return fail(HS_ERR_INVALID_ARGUMENT, "capacity_tokens must be positive");
    if (l->code_stride_head < (int64_t)l->capacity_tokens * D || (l->code_stride_head & 15))
        return fail(HS_ERR_INVALID_ARGUMENT, "code_stride_head %lld too small or not a multiple of 16",
                    (long long)l->code_stride_head);
    if (need_scales && (l->scale_stride_head < l->capacity_tokens || (l->scale_stride_head & 3) ||
                        (l->scale_stride_seq & 3) || (l->code_stride_seq & 15)))
        return fail(HS_ERR_INVALID_ARGUMENT, "scale_stride_head %lld too small or not a multiple of 4",
                    (long long)l->scale_stride_head);
    if ((l->k_block_table == nullptr) != (l->v_block_table == nullptr))
        return fail(HS_ERR_INVALID_ARGUMENT, "give both block tables or neither");
    if (l->k_block_table && l->block_table_stride <= 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "block_table_stride must be positive when paged");
    return HS_OK;
}

int validate_layout(const hs_kv_layout *l, int B, int S, int Hkv, int D, bool need_scales) {
    return check_common(l, B, S, Hkv, D, need_scales);
}

template <bool FP8>
static int launch_quantize(const void *k_src, const void *v_src, int dtype, void *kc, void *vc, float *ks, float *vs,
                           const hs_kv_layout *l, const int32_t *positions, int start_pos, int B, int S, int Hkv,
                           int D, hipStream_t stream, const void *rope_sin = nullptr, const void *rope_cos = nullptr,
                           int rope_len = 0, int rotary_dim = 0, const NormSpec *norm = nullptr) {
    if (int rc = check_common(l, B, S, Hkv, D, !FP8)) return rc;
    if ((rope_sin == nullptr) != (rope_cos == nullptr)) return fail(HS_ERR_INVALID_ARGUMENT, "give sin and cos or neither");
    if (rope_sin && rope_len <= 0) return fail(HS_ERR_INVALID_ARGUMENT, "rope_len must be positive");
    if (rope_sin && !positions && (int64_t)start_pos + S > rope_len)
        return fail(HS_ERR_INVALID_ARGUMENT, "positions %d..%d exceed the rotary tables (%d rows)", start_pos,
                    start_pos + S - 1, rope_len);
    const bool empty = (int64_t)B * S == 0;  // an empty problem may come with null pointers (an empty tensor has none)
    if (!empty && (!k_src || !v_src || !kc || !vc || !ks || !vs)) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (dtype != HS_BF16 && dtype != HS_F32 && dtype != HS_F16)
        return fail(HS_ERR_INVALID_ARGUMENT, "unknown src_dtype %d", dtype);
    if (!positions) {
        if (start_pos < 0) return fail(HS_ERR_INVALID_ARGUMENT, "negative start_pos");
        int64_t cap = l->k_block_table ? (int64_t)l->capacity_tokens * l->block_table_stride : l->capacity_tokens;
        if ((int64_t)start_pos + S > cap)
            return fail(HS_ERR_OVERFLOW,
                        "Cache overflow: trying to cache %d tokens starting at position %d, but capacity is %lld", S,
                        start_pos, (long long)cap);
    }
    const int64_t rows = (int64_t)B * S * Hkv;
    if (rows == 0) return HS_OK;
    QuantArgs a;
    a.src[0] = k_src; a.src[1] = v_src;
    a.codes[0] = kc; a.codes[1] = vc;
    a.scales[0] = ks; a.scales[1] = vs;
    a.addr[0] = make_addr(*l, 0); a.addr[1] = make_addr(*l, 1);
    a.positions = positions; a.start_pos = start_pos;
    a.B = B; a.S = S; a.Hkv = Hkv; a.D = D; a.dtype = dtype;
    a.rope_sin = rope_sin; a.rope_cos = rope_cos; a.rope_len = rope_len; a.rotary_dim = rotary_dim;
    if (norm) a.norm = *norm;
    // Bulk writes without rotation take the kernel that packs several rows into a wavefront; it wants
    // 16-byte aligned sources and 8-byte aligned code rows and at most 65535 sequences (grid.z).
    const bool aligned = (((uintptr_t)k_src | (uintptr_t)v_src) & 15) == 0 && (((uintptr_t)kc | (uintptr_t)vc) & 7) == 0 &&
                         (l->code_stride_seq & 7) == 0;
    if (!rope_sin && a.norm.kind == 0 && aligned && B <= 65535 && (int64_t)S * Hkv < (1 << 30)) {
        const int lpr = D / 8, rows_per_wg = 4 * (64 / lpr);
        dim3 g((unsigned)(((int64_t)S * Hkv + rows_per_wg - 1) / rows_per_wg), 2, B);
        if (D == 64) kv_quantize_rows_kernel<8, FP8><<<g, 256, 0, stream>>>(a);
        else if (D == 128) kv_quantize_rows_kernel<16, FP8><<<g, 256, 0, stream>>>(a);
        else kv_quantize_rows_kernel<32, FP8><<<g, 256, 0, stream>>>(a);
        return check_launch(FP8 ? "kv_quantize_fp8" : "kv_quantize_int8");
    }
    dim3 grid((unsigned)((rows + 3) / 4), 2);
    if (D == 64) kv_quantize_kernel<1, FP8><<<grid, 256, 0, stream>>>(a);
    else if (D == 128) kv_quantize_kernel<2, FP8><<<grid, 256, 0, stream>>>(a);
    else kv_quantize_kernel<4, FP8><<<grid, 256, 0, stream>>>(a);
    return check_launch(FP8 ? "kv_quantize_fp8" : "kv_quantize_int8");
}

}  // namespace hs

extern "C" {

int hs_kv_quantize_int8(const void *k_src, const void *v_src, int src_dtype, int8_t *k_codes, int8_t *v_codes,
                        float *k_scales, float *v_scales, const hs_kv_layout *layout, const int32_t *positions,
                        int32_t start_pos, int32_t B, int32_t S, int32_t Hkv, int32_t D, hs_stream_t stream) {
    return hs::launch_quantize<false>(k_src, v_src, src_dtype, k_codes, v_codes, k_scales, v_scales, layout, positions,
                                      start_pos, B, S, Hkv, D, (hipStream_t)stream);
}

int hs_kv_quantize_int8_rope(const void *k_src, const void *v_src, int src_dtype, const void *rope_sin,
                             const void *rope_cos, int32_t rope_len, int8_t *k_codes, int8_t *v_codes, float *k_scales,
                             float *v_scales, const hs_kv_layout *layout, const int32_t *positions, int32_t start_pos,
                             int32_t B, int32_t S, int32_t Hkv, int32_t D, hs_stream_t stream) {
    if (!rope_sin || !rope_cos) return hs::fail(HS_ERR_INVALID_ARGUMENT, "null rotary table");
    return hs::launch_quantize<false>(k_src, v_src, src_dtype, k_codes, v_codes, k_scales, v_scales, layout, positions,
                                      start_pos, B, S, Hkv, D, (hipStream_t)stream, rope_sin, rope_cos, rope_len);
}

}  // extern "C"

namespace hs {

// Checks of an hs_qk_prologue shared by the entry points that take one; fills the K-side NormSpec / rotary_dim.
int check_prologue(const hs_qk_prologue *p, int dtype, int D, bool need_q, bool need_k) {
    if (!p) return fail(HS_ERR_INVALID_ARGUMENT, "null hs_qk_prologue");
    if (p->norm_kind < HS_QKNORM_NONE || p->norm_kind > HS_QKNORM_QWEN35)
        return fail(HS_ERR_INVALID_ARGUMENT, "unknown norm_kind %d", p->norm_kind);
    if (p->norm_kind != HS_QKNORM_NONE) {
        if ((need_q && !p->q_norm_weight) || (need_k && !p->k_norm_weight))
            return fail(HS_ERR_INVALID_ARGUMENT, "QK-norm without a weight vector");
        if ((p->q_norm_head_stride != 0 && p->q_norm_head_stride != D) || (p->k_norm_head_stride != 0 && p->k_norm_head_stride != D))
            return fail(HS_ERR_INVALID_ARGUMENT, "norm weight head stride must be 0 (one [D] vector) or D (per-head rows)");
        if (!(p->norm_eps >= 0.0f)) return fail(HS_ERR_INVALID_ARGUMENT, "negative norm_eps");
    }
    if ((p->rope_sin == nullptr) != (p->rope_cos == nullptr)) return fail(HS_ERR_INVALID_ARGUMENT, "give sin and cos or neither");
    if (p->rope_sin) {
        if (p->rope_len <= 0) return fail(HS_ERR_INVALID_ARGUMENT, "rope_len must be positive");
        const int rd = p->rotary_dim > 0 ? p->rotary_dim : D;
        if (rd > D || (rd % 16) != 0)
            return fail(HS_ERR_INVALID_ARGUMENT, "rotary_dim %d must be a multiple of 16 in (0, head_dim %d]", rd, D);
    }
    (void)dtype;
    return HS_OK;
}

NormSpec norm_spec(const hs_qk_prologue *p, int which) {
    NormSpec n;
    n.kind = p->norm_kind;
    n.eps = p->norm_eps;
    n.weight = which ? p->k_norm_weight : p->q_norm_weight;
    n.head_stride = which ? p->k_norm_head_stride : p->q_norm_head_stride;
    return n;
}

}  // namespace hs

extern "C" {

int hs_qk_prologue_apply(const void *q, const void *k, int dtype, const hs_qk_prologue *prologue,
                         const int32_t *positions, int32_t start_pos, void *q_out, void *k_out, int32_t B, int32_t S,
                         int32_t Hq, int32_t Hkv, int32_t D, hs_stream_t stream) {
    using namespace hs;
    if (dtype != HS_BF16 && dtype != HS_F32 && dtype != HS_F16) return fail(HS_ERR_INVALID_ARGUMENT, "unknown dtype %d", dtype);
    if (D != 64 && D != 128 && D != 256) return fail(HS_ERR_INVALID_ARGUMENT, "head_dim %d not in {64,128,256}", D);
    if (B < 0 || S < 0 || Hq < 0 || Hkv < 0) return fail(HS_ERR_INVALID_ARGUMENT, "bad shape B=%d S=%d Hq=%d Hkv=%d", B, S, Hq, Hkv);
    const int hq = q ? Hq : 0, hk = k ? Hkv : 0;
    if (int rc = check_prologue(prologue, dtype, D, hq > 0, hk > 0)) return rc;
    if ((q && !q_out) || (k && !k_out)) return fail(HS_ERR_INVALID_ARGUMENT, "null output buffer");
    if (q && q == q_out && prologue->rope_sin) return fail(HS_ERR_INVALID_ARGUMENT, "the rotation cannot run in place: give q_out its own buffer");
    if (k && k == k_out && prologue->rope_sin) return fail(HS_ERR_INVALID_ARGUMENT, "the rotation cannot run in place: give k_out its own buffer");
    if (prologue->rope_sin && !positions && (start_pos < 0 || (int64_t)start_pos + S > prologue->rope_len))
        return fail(HS_ERR_INVALID_ARGUMENT, "positions %d..%d exceed the rotary tables (%d rows)", start_pos,
                    start_pos + S - 1, prologue->rope_len);
    const int64_t rows = (int64_t)B * S * (hq + hk);
    if (rows == 0) return HS_OK;
    PrologueArgs a;
    a.x[0] = q; a.x[1] = k; a.out[0] = q_out; a.out[1] = k_out;
    a.norm[0] = norm_spec(prologue, 0); a.norm[1] = norm_spec(prologue, 1);
    a.sin_t = prologue->rope_sin; a.cos_t = prologue->rope_cos; a.positions = positions; a.start_pos = start_pos;
    a.rope_len = prologue->rope_len; a.B = B; a.S = S; a.H[0] = hq; a.H[1] = hk; a.D = D; a.dtype = dtype;
    a.rd = prologue->rotary_dim > 0 ? prologue->rotary_dim : D;
    uintptr_t bits = (uintptr_t)q | (uintptr_t)k | (uintptr_t)q_out | (uintptr_t)k_out | (uintptr_t)a.sin_t | (uintptr_t)a.cos_t;
    if (prologue->norm_kind != HS_QKNORM_NONE) bits |= (uintptr_t)a.norm[0].weight | (uintptr_t)a.norm[1].weight;
    if (dtype == HS_BF16 && (bits & 15) == 0 && rows < (1ll << 30) && (!a.sin_t || prologue_parts_serve(a.rd, D == 64 ? 16 : 32))) {
        const int rows_per_wg = 4 * (64 / (D / (D == 64 ? 16 : 32)));  // bf16, 16-byte accesses, 32 elements per lane
        dim3 g((unsigned)((rows + rows_per_wg - 1) / rows_per_wg));
        if (D == 64) qk_prologue_parts_kernel<64><<<g, 256, 0, (hipStream_t)stream>>>(a);
        else if (D == 128) qk_prologue_parts_kernel<128><<<g, 256, 0, (hipStream_t)stream>>>(a);
        else qk_prologue_parts_kernel<256><<<g, 256, 0, (hipStream_t)stream>>>(a);
        return check_launch("qk_prologue");
    }
    if (dtype != HS_F32 && (bits & 15) == 0 && rows < (1ll << 30)) {  // 16-bit tensors, 16-byte accesses: several rows per wavefront
        const int rows_per_wg = 4 * (64 / (D / 8));
        dim3 g((unsigned)((rows + rows_per_wg - 1) / rows_per_wg));
        const bool bf = dtype == HS_BF16;
        if (D == 64) bf ? qk_prologue_rows_kernel<8, HS_BF16><<<g, 256, 0, (hipStream_t)stream>>>(a) : qk_prologue_rows_kernel<8, HS_F16><<<g, 256, 0, (hipStream_t)stream>>>(a);
        else if (D == 128) bf ? qk_prologue_rows_kernel<16, HS_BF16><<<g, 256, 0, (hipStream_t)stream>>>(a) : qk_prologue_rows_kernel<16, HS_F16><<<g, 256, 0, (hipStream_t)stream>>>(a);
        else bf ? qk_prologue_rows_kernel<32, HS_BF16><<<g, 256, 0, (hipStream_t)stream>>>(a) : qk_prologue_rows_kernel<32, HS_F16><<<g, 256, 0, (hipStream_t)stream>>>(a);
        return check_launch("qk_prologue");
    }
    dim3 grid((unsigned)((rows + 3) / 4));
    if (D == 64) qk_prologue_kernel<1><<<grid, 256, 0, (hipStream_t)stream>>>(a);
    else if (D == 128) qk_prologue_kernel<2><<<grid, 256, 0, (hipStream_t)stream>>>(a);
    else qk_prologue_kernel<4><<<grid, 256, 0, (hipStream_t)stream>>>(a);
    return check_launch("qk_prologue");
}

int hs_kv_quantize_int8_prologue(const void *k_src, const void *v_src, int src_dtype, const hs_qk_prologue *prologue,
                                 int8_t *k_codes, int8_t *v_codes, float *k_scales, float *v_scales,
                                 const hs_kv_layout *layout, const int32_t *positions, int32_t start_pos, int32_t B,
                                 int32_t S, int32_t Hkv, int32_t D, hs_stream_t stream) {
    if (int rc = hs::check_prologue(prologue, src_dtype, D, false, true)) return rc;
    const hs::NormSpec n = hs::norm_spec(prologue, 1);
    return hs::launch_quantize<false>(k_src, v_src, src_dtype, k_codes, v_codes, k_scales, v_scales, layout, positions,
                                      start_pos, B, S, Hkv, D, (hipStream_t)stream, prologue->rope_sin,
                                      prologue->rope_cos, prologue->rope_len, prologue->rotary_dim, &n);
}

int hs_rope_apply(const void *x, int dtype, const void *rope_sin, const void *rope_cos, int32_t rope_len,
                  const int32_t *positions, int32_t start_pos, void *out, int32_t B, int32_t S, int32_t H, int32_t D,
                  hs_stream_t stream) {
    return hs_rope_apply_partial(x, dtype, rope_sin, rope_cos, rope_len, positions, start_pos, out, B, S, H, D, D, stream);
}

int hs_rope_apply_partial(const void *x, int dtype, const void *rope_sin, const void *rope_cos, int32_t rope_len,
                          const int32_t *positions, int32_t start_pos, void *out, int32_t B, int32_t S, int32_t H,
                          int32_t D, int32_t rotary_dim, hs_stream_t stream) {
    using namespace hs;
    if (rotary_dim <= 0 || rotary_dim > D || (rotary_dim % 16) != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "rotary_dim %d must be a multiple of 16 in (0, head_dim %d]", rotary_dim, D);
    if ((int64_t)B * S > 0 && (!x || !out || !rope_sin || !rope_cos)) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (dtype != HS_BF16 && dtype != HS_F32 && dtype != HS_F16) return fail(HS_ERR_INVALID_ARGUMENT, "unknown dtype %d", dtype);
    if (B < 0 || S < 0 || H <= 0) return fail(HS_ERR_INVALID_ARGUMENT, "bad shape B=%d S=%d H=%d", B, S, H);
    if (D != 64 && D != 128 && D != 256) return fail(HS_ERR_INVALID_ARGUMENT, "head_dim %d not in {64,128,256}", D);
    if (rope_len <= 0) return fail(HS_ERR_INVALID_ARGUMENT, "rope_len must be positive");
    if (!positions && (start_pos < 0 || (int64_t)start_pos + S > rope_len))
        return fail(HS_ERR_INVALID_ARGUMENT, "positions %d..%d exceed the rotary tables (%d rows)", start_pos,
                    start_pos + S - 1, rope_len);
    const int64_t rows = (int64_t)B * S * H;
    if (rows == 0) return HS_OK;
    RopeArgs a;
    a.x = x; a.sin_t = rope_sin; a.cos_t = rope_cos; a.out = out; a.positions = positions; a.start_pos = start_pos;
    a.rope_len = rope_len; a.B = B; a.S = S; a.H = H; a.D = D; a.dtype = dtype; a.rd = rotary_dim;
    const bool aligned = (((uintptr_t)x | (uintptr_t)out | (uintptr_t)rope_sin | (uintptr_t)rope_cos) & 15) == 0;
    if (dtype != HS_F32 && aligned) {  // 16-bit tensors: several rows per wavefront
        const int rows_per_wg = 4 * (64 / (D / 8));
        dim3 g((unsigned)((rows + rows_per_wg - 1) / rows_per_wg));
        if (D == 64) rope_apply_rows_kernel<8><<<g, 256, 0, (hipStream_t)stream>>>(a);
        else if (D == 128) rope_apply_rows_kernel<16><<<g, 256, 0, (hipStream_t)stream>>>(a);
        else rope_apply_rows_kernel<32><<<g, 256, 0, (hipStream_t)stream>>>(a);
        return check_launch("rope_apply");
    }
    dim3 grid((unsigned)((rows + 3) / 4));
    if (D == 64) rope_apply_kernel<1><<<grid, 256, 0, (hipStream_t)stream>>>(a);
    else if (D == 128) rope_apply_kernel<2><<<grid, 256, 0, (hipStream_t)stream>>>(a);
    else rope_apply_kernel<4><<<grid, 256, 0, (hipStream_t)stream>>>(a);
    return check_launch("rope_apply");
}

int hs_kv_quantize_fp8(const void *k_src, const void *v_src, int src_dtype, uint8_t *k_codes, uint8_t *v_codes,
                       const float *k_scales, const float *v_scales, const hs_kv_layout *layout,
                       const int32_t *positions, int32_t start_pos, int32_t B, int32_t S, int32_t Hkv, int32_t D,
                       hs_stream_t stream) {
    return hs::launch_quantize<true>(k_src, v_src, src_dtype, k_codes, v_codes, (float *)k_scales, (float *)v_scales,
                                     layout, positions, start_pos, B, S, Hkv, D, (hipStream_t)stream);
}

int hs_kv_fp8_calibrate(const void *k_src, const void *v_src, int src_dtype, float *k_scales, float *v_scales,
                        int32_t B, int32_t S, int32_t Hkv, int32_t D, hs_stream_t stream) {
    if (!k_src || !v_src || !k_scales || !v_scales) return hs::fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (B <= 0 || S <= 0 || Hkv <= 0 || D <= 0)
        return hs::fail(HS_ERR_INVALID_ARGUMENT, "bad shape B=%d S=%d Hkv=%d D=%d", B, S, Hkv, D);
    if (src_dtype != HS_BF16 && src_dtype != HS_F32 && src_dtype != HS_F16)
        return hs::fail(HS_ERR_INVALID_ARGUMENT, "unknown src_dtype %d", src_dtype);
    if (src_dtype != HS_F32 && (D == 64 || D == 128 || D == 256) && (((uintptr_t)k_src | (uintptr_t)v_src) & 15) == 0)
        hs::fp8_calibrate16_kernel<<<dim3(B * Hkv, 2), 1024, 0, (hipStream_t)stream>>>(
            (const uint16_t *)k_src, (const uint16_t *)v_src, src_dtype, k_scales, v_scales, B, S, Hkv, D);
    else
        hs::fp8_calibrate_kernel<<<dim3(B * Hkv, 2), 256, 0, (hipStream_t)stream>>>(k_src, v_src, src_dtype, k_scales,
                                                                                   v_scales, B, S, Hkv, D);
    return hs::check_launch("fp8_calibrate");
}

int hs_kv_dequantize(const void *codes, const float *scales, int fmt_fp8, const hs_kv_layout *layout, int which_table,
                     void *out, int out_dtype, int32_t B, int32_t T, int32_t Hkv, int32_t D, hs_stream_t stream) {
    if (int rc = hs::validate_layout(layout, B, T, Hkv, D, !fmt_fp8)) return rc;
    if ((int64_t)B * T > 0 && (!codes || !scales || !out)) return hs::fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (out_dtype != HS_BF16 && out_dtype != HS_F32 && out_dtype != HS_F16)
        return hs::fail(HS_ERR_INVALID_ARGUMENT, "unknown out_dtype %d", out_dtype);
    const int64_t rows = (int64_t)B * T * Hkv;
    if (rows == 0) return HS_OK;
    hs::DequantArgs a;
    a.codes = codes; a.scales = scales; a.addr = hs::make_addr(*layout, which_table ? 1 : 0);
    a.out = out; a.B = B; a.T = T; a.Hkv = Hkv; a.D = D; a.out_dtype = out_dtype; a.fp8 = fmt_fp8 ? 1 : 0;
    if ((((uintptr_t)codes) & 7) == 0 && (((uintptr_t)out) & 15) == 0 && (layout->code_stride_seq & 7) == 0) {
        const int rows_per_wg = 4 * (64 / (D / 8));
        dim3 g((unsigned)((rows + rows_per_wg - 1) / rows_per_wg));
        if (D == 64) hs::kv_dequantize_rows_kernel<8><<<g, 256, 0, (hipStream_t)stream>>>(a);
        else if (D == 128) hs::kv_dequantize_rows_kernel<16><<<g, 256, 0, (hipStream_t)stream>>>(a);
        else hs::kv_dequantize_rows_kernel<32><<<g, 256, 0, (hipStream_t)stream>>>(a);
        return hs::check_launch("kv_dequantize");
    }
    dim3 grid((unsigned)((rows + 3) / 4));
    if (D == 64) hs::kv_dequantize_kernel<1><<<grid, 256, 0, (hipStream_t)stream>>>(a);
    else if (D == 128) hs::kv_dequantize_kernel<2><<<grid, 256, 0, (hipStream_t)stream>>>(a);
    else hs::kv_dequantize_kernel<4><<<grid, 256, 0, (hipStream_t)stream>>>(a);
    return hs::check_launch("kv_dequantize");
}

}  // extern "C"
