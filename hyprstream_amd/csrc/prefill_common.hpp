// Declarations shared by the prefill attention kernels (prefill_attn.hip: every head_dim, sliding windows, narrow
// grids; prefill_attn_wide.hip: head_dim 128 on 32x32x16 MFMAs).
#pragma once
#include <climits>
#include <type_traits>

#include "mfma_common.hpp"
#include "prologue_rows.hpp"
#include "quant_device.hpp"

namespace hs {

constexpr int kPWaves = 8;
constexpr float kPLog2e = 1.4426950408889634f;
constexpr float kPShift = 6.0f;  // weights are carried as 2^6 * exp2(s - m_run): keeps small ones out of the fp16 subnormals
constexpr float kMaxScale = 512.0f;  // 127 * scale stays finite in fp16; larger magnitudes saturate instead of overflowing
constexpr float kSlack = 4.0f;  // log2 units by which the softmax reference value overshoots a new maximum

struct PrefillArgs {
    const uint16_t *q, *kn, *vn;  // [B,S,Hq,D], [B,S,Hkv,D], [B,S,Hkv,D] bf16
    const uint8_t *kc, *vc;
    const float *ks, *vs;
    KvAddr ka, va;
    uint16_t *out;  // [B,S,Hq,D] bf16
    const uint16_t *out_gate;  // optional [B,S,Hq,D] bf16: out = bf16(bf16(attention) * bf16(sigmoid(gate)))
    int32_t B, S, Hq, Hkv, G, HG, hist_len;
    const int32_t *hist_lens;  // optional, device [B]: cached tokens per sequence (then hist_len is their upper bound)
    int32_t heavy_first;  // the grid outnumbers the CUs: order the query tiles by decreasing work
    int32_t write_new;    // quantize-on-write of the call's K/V rows by the workgroups that finish early
    int32_t window;       // sliding window of local layers: a query at position p attends keys in (p - window, p]; 0 = none
    float scale_log2e;
    // keys of a query tile split over nsplit workgroups (prefill_attn_kernel<..., kSplit>): partial accumulators and an
    // arrival counter per tile in the caller's workspace; the workgroup that arrives last merges and stores
    int32_t nsplit = 1;
    float *split_ws = nullptr;
    uint32_t *split_cnt = nullptr;
    // bf16 copy of the prompt's dequantized K/V in MFMA operand order (hs_kv_layout.prefill_shadow): one 64-key step is a
    // HistTile<128> image, shadow_steps of them per (sequence, kv-head).  Every launch appends its tokens; the instance
    // that can read it copies whole steps into LDS instead of converting codes.
    uint16_t *shadow = nullptr;
    int32_t shadow_steps = 0;
    RowPrologue qpro;     // the q side of the layer's prologue run inside the launch (hs_kv_layout.prefill_q_prologue)
};


// Bytes of one 64-key step of the shadow at head_dim 128 (= sizeof(HistTile<128>): two halves of 8 K + 8 V^T blocks).
constexpr int kShadowStepBytes = 32768;

// Workgroup barrier that orders LDS traffic only.  __syncthreads() would also wait for every outstanding global
// load, i.e. for the tile prefetch that was issued a moment earlier and is not needed before the next step.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Quantize-on-write of the call's own K/V rows by a workgroup that has finished its attention.
// The query tiles at the front of the prompt walk the fewest keys and finish first: the first half of them
// (head group 0 of each kv-head) write the rows of two tiles each into the cache while the late tiles still
// compute.  Nothing in this launch reads those rows (the history ends below them).  D/8 lanes own a row, as in
// the stand-alone bulk writer, and the arithmetic per element is the same: the same codes and scales.
template <int kRow, bool FP8, int kWaves = kPWaves>
__device__ __forceinline__ void write_new_rows(const PrefillArgs &a, int b, int kvh, int H, int q0, int q_per_wg, int wave, int lane) {
#pragma clang fp contract(off)
    const int S = a.S;
    constexpr int LPR = kRow / 8, RPW = 64 / LPR;
    const int tile = q0 / q_per_wg, tiles = (S + q_per_wg - 1) / q_per_wg;
    if (tile < (tiles + 1) / 2) {
        const int t_lo = 2 * tile * q_per_wg, t_hi = min(S, t_lo + 2 * q_per_wg);
        const int sub = lane % LPR;
#pragma unroll 2
        for (int tb = t_lo + wave * RPW; tb < t_hi; tb += kWaves * RPW) {
            const int t = tb + lane / LPR;
            const bool live = t < t_hi;  // lanes of rows past the end still take part in the shuffles
            const int tt = live ? t : t_hi - 1;
            const int64_t e0 = (((int64_t)b * S + tt) * a.Hkv + kvh) * kRow + sub * 8;
            const u32x4 wk = *(const u32x4 *)(a.kn + e0), wv = *(const u32x4 *)(a.vn + e0);
#pragma unroll
            for (int which = 0; which < 2; ++which) {
                const KvAddr &ad = which ? a.va : a.ka;
                const u32x4 w = which ? wv : wk;
                float *scales = const_cast<float *>(which ? a.vs : a.ks);
                int64_t unit;
                int slot;
                const bool ok = resolve(ad, b, H + tt, unit, slot) && live;
                float x[8];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    x[2 * i] = __uint_as_float(w[i] << 16);
                    x[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
                }
                float sc = 0.0f;
                uint32_t packed[2] = {0u, 0u};
                if (FP8) {
                    sc = scales[(int64_t)b * a.Hkv + kvh];
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
                        const float w2 = __shfl_xor(m, o, 64);
                        m = m > w2 ? m : w2;
                    }
                    if (m > 0.0f) {
                        sc = m / 127.0f;
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            float qv = rintf(x[e] / sc);
                            qv = qv > 127.0f ? 127.0f : qv;
                            qv = qv < -127.0f ? -127.0f : qv;
                            if (qv != qv) qv = 0.0f;
                            packed[e >> 2] |= ((uint32_t)(int)qv & 0xffu) << (8 * (e & 3));
                        }
                    }
                }
                if constexpr (kRow == 128) {
                    if (a.shadow != nullptr && live) {
                        // the dequantized row (code * scale, rounded to bf16: what the reference's get() hands to its
                        // attention) into the step image of its position; `packed` holds the codes
                        const int pos = H + tt, kk = pos & 31;
                        uint16_t *img = a.shadow + (((int64_t)b * a.Hkv + kvh) * a.shadow_steps + (pos >> 6)) * (kShadowStepBytes / 2) +
                                        ((pos >> 5) & 1) * (kShadowStepBytes / 4);  // this half: K blocks [2 KG][512 el], then V^T blocks [VB][512 el]
                        float dq[8];
                        if constexpr (FP8) {
                            const half8 hv = e4m3x8_to_f16_div256(packed[0], packed[1]);  // exact: the codes' values / 256
#pragma unroll
                            for (int e = 0; e < 8; ++e) dq[e] = (float)hv[e] * 256.0f * sc;
                        } else {
#pragma unroll
                            for (int e = 0; e < 8; ++e) dq[e] = (float)(int8_t)(packed[e >> 2] >> (8 * (e & 3))) * sc;
                        }
                        if (which == 0) {
                            // K block (tile u = kk / 16, d-group j): lane (li = key, lq) holds d = 32 lq + 8 j ..; this lane has d = 8 sub ..
                            const int blk = 4 * (kk >> 4) + (sub & 3), ln = (sub >> 2) * 16 + (kk & 15);
                            *(u32x4 *)(img + blk * 512 + ln * 8) = (u32x4){pack_bf16x2(dq[0], dq[1]), pack_bf16x2(dq[2], dq[3]),
                                                                           pack_bf16x2(dq[4], dq[5]), pack_bf16x2(dq[6], dq[7])};
                        } else {
                            // V^T block bb: lane (li = d / 8, lq = (kk % 16) / 4), slot 4 (kk / 16) + kk % 4, row d = 8 li + bb
                            uint16_t *vp = img + 8 * 512 + (((kk & 15) >> 2) * 16 + sub) * 8 + 4 * (kk >> 4) + (kk & 3);
#pragma unroll
                            for (int e = 0; e < 8; ++e) vp[e * 512] = (uint16_t)f32_to_bf16_bits(dq[e]);
                        }
                    }
                }
                if (ok) {
                    uint8_t *dst = const_cast<uint8_t *>(which ? a.vc : a.kc) + unit * ad.code_stride_seq +
                                   (int64_t)kvh * ad.code_stride_head + (int64_t)slot * kRow + sub * 8;
                    *(u32x2 *)dst = (u32x2){packed[0], packed[1]};
                    if (!FP8 && sub == 0)
                        scales[unit * ad.scale_stride_seq + (int64_t)kvh * ad.scale_stride_head + slot] = sc;
                }
            }
        }
    }
}

}  // namespace hs
