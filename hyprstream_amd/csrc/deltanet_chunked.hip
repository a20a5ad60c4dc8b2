// Gated delta rule over a prompt in chunks of 64 tokens on the MFMA pipe (gfx950, wave64): the reference's own prefill
// formulation (chunked_delta_rule, qwen3_5.rs:342-498; chunk size 64), regrouped so that little has to pass through
// memory between the part that is parallel over chunks and the part that walks them in order.
//
// With G_t the running sum of the log-decays inside a chunk, k and q L2-normalised (q also scaled) and
//   L[i][j] = -beta_i (k_i . k_j) exp(G_i - G_j)  (j < i),      N = (I - L)^-1,      N' = N diag(beta),
//   M[i][j] = (q_i . k_j) exp(G_i - G_j)          (j <= i),
// a chunk that starts from the state S (dk x dv) gives
//   X  = v - (k e^G) S
//   V' = N' X                                  (= N (v beta) - N (k beta e^G) S, the U - W S of the reference)
//   O  = (q e^G) S + M V'
//   S <- e^(G_63) S + (k e^(G_63 - G))^T V'.
// Only N' and M (two 64 x 64 triangles per chunk and v-head) do not follow from one row of the inputs at a time, so
// only they go through memory: deltanet_chunk_factor_kernel makes them for all chunks in parallel, and
// deltanet_chunk_walk_kernel walks the chunks of one (sequence, v-head, half or quarter of the state columns) in
// order, reading q, k and v as they were given.  A workspace that also carried W, U and the normalised q and k in operand order
// would move 58 KB instead of 13 KB per chunk and v-head through HBM twice.
//
// The walk: two wavefronts, each alone on its SIMD, own 32 state columns each (16 in the instance for batches that
// leave the device part empty otherwise: half the products of a chunk step) -- all 128 rows, in accumulator
// registers -- for the whole prompt.  Nothing passes between them: the accumulator layout of S, X and V' (lane
// (li, lq): column li, rows 4 lq + r) is the B operand layout of the next product once the k-slots of the A operand
// are taken in that order (slots 0-3: rows 4 lq + r of the even 16-row tile of a 32-row slab, slots 4-7: of the odd
// tile), so a chunk is 128 MFMAs and three conversions in registers per wavefront, and one workgroup barrier (the
// hand-over of the operand buffer).  Six more wavefronts do the moving: they read k, q, v rows and the two triangles
// two chunks ahead, fold normalisation and decay factors in, write everything as A operands into the other half of a
// two-chunk LDS buffer, and carry the finished output rows from LDS to memory.
//
// Operands are fp16 (v: bf16 as given), accumulation and the state fp32 (every decay factor is <= 1: nothing overflows).
#include <algorithm>
#include <climits>
#include <type_traits>

#include "mfma_common.hpp"

namespace hs {

constexpr int kC = 64;    // tokens per chunk
constexpr int kWD = 128;  // dk = dv = 128
constexpr float kLog2e = 1.4426950408889634f;
typedef _Float16 half4v __attribute__((ext_vector_type(4)));

// Workspace, chunk-major: per (chunk, sequence, v-head)
// The triangles as A operands, 64-lane blocks of 16 B: block (token tile tt, token slab s) for the six pairs with
// 32 s <= 16 tt + 15 (the other two are zero and are neither stored nor multiplied), at index tri_block(tt, s).
constexpr int kOffNt = 0;         // N' (A operand of N' X), 6 KB
constexpr int kOffQK = 6144;      // M  (A operand of M V'), 6 KB
constexpr int kOffFn = 12288;     // -exp(G_t) / |k_t|            (what turns a row of k into a row of -k-hat e^G), 64 floats
constexpr int kOffFq = 12544;     // exp(G_t) q_scale / |q_t|
constexpr int kOffFt = 12800;     // exp(G_63 - G_t) / |k_t|
constexpr int kOffDecay = 13056;  // exp(G_63)
constexpr int kUnitBytes = 13312;
__host__ __device__ constexpr int tri_block(int tt, int s) { return tt < 2 ? tt : 2 * tt - 2 + s; }

struct WalkArgs {
    const uint16_t *q, *k, *v;  // bf16 [B,T,nk,128], [B,T,nk,128], [B,T,nv,128]
    const float *g, *beta;      // [B,T,nv]
    float *state;               // [B,nv,128,128]
    float *out;                 // [B,T,nv,128]
    uint8_t *ws;
    int32_t B, T, nk, nv, nc;
    float q_scale;
    int32_t l2norm;
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
__device__ __forceinline__ half4v f32x4_to_half4(const float4v &x) {
    return (half4v){(_Float16)x[0], (_Float16)x[1], (_Float16)x[2], (_Float16)x[3]};
}

// Sixteen bf16 (two 16-byte pieces) -> fp32
__device__ __forceinline__ void unpack16(const u32x4 &a, const u32x4 &b, float *f) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        f[2 * e] = __uint_as_float(a[e] << 16);
        f[2 * e + 1] = __uint_as_float(a[e] & 0xffff0000u);
        f[8 + 2 * e] = __uint_as_float(b[e] << 16);
        f[8 + 2 * e + 1] = __uint_as_float(b[e] & 0xffff0000u);
    }
}

// Workgroup barrier that orders LDS traffic only: __syncthreads() would also wait for global accesses in flight (the
// walk's prefetch, the factor kernel's stores into the workspace, which nothing in the same launch reads).
__device__ __forceinline__ void lds_sync() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// v of the lane a DPP control selects (0x110 + n: n lanes down inside a row of 16; 0x142 / 0x143: lane 15 / 31 of the
// preceding rows), 0 for a lane without a source or in a row that kRows masks out.
template <int kCtrl, int kRows>
__device__ __forceinline__ float dpp_or_zero(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, kRows, 0xf, false));
}

// ------------------------------------------------------------------------------------------------- factors
constexpr int kPitchH = 136;  // halves per row of the row-major k / q tiles
constexpr int kPitchL = 68;   // halves per row of the 64 x 64 matrix P = L^T
constexpr int kPitchD = 20;   // floats per row of a 16 x 16 fp32 block
constexpr int kBlockD = 16 * kPitchD;
// Region A: the row-major k / q tiles; once the two products are done, P and its diagonal blocks.
constexpr int kLdsKh = 0, kLdsQh = 17408;
constexpr int kLdsP = 0, kLdsD = kLdsP + 64 * kPitchL * 2;
static_assert(kLdsD + 4 * kBlockD * 4 <= 34816, "P and the diagonal blocks inside the dead k / q tiles");
constexpr int kLdsF = 34816, kLdsBytes = kLdsF + 1536;
static_assert(4 * kLdsBytes <= 163840, "four workgroups of the factor kernel per CU");

// One 512-thread workgroup per (sequence, v-head, chunk), four to a CU.  Everything is built transposed -- P = L^T, the diagonal
// blocks of (I - P)^-1 = N^T, then N^T by block back substitution -- because the accumulator layout of a tile of
// N^T (lane: column i, rows j = 4 lq + r) is the A operand layout the walk needs for N (row i, k-slots j).
__global__ __launch_bounds__(512, 8) void deltanet_chunk_factor_kernel(WalkArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[kLdsBytes];
    _Float16 *kh = (_Float16 *)(lds + kLdsKh), *qh = (_Float16 *)(lds + kLdsQh);
    _Float16 *Ph = (_Float16 *)(lds + kLdsP);  // P[j][i] = L[i][j], outside the diagonal blocks
    float *Dm = (float *)(lds + kLdsD);        // the four diagonal blocks of P, later of (I - P)^-1
    float *gs = (float *)(lds + kLdsF), *bs = gs + 64, *Gs = gs + 128, *km = gs + 192;  // km: 64 x (kmul, qmul)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lq = lane >> 4;
    const uint32_t unit = blockIdx.x, uv = unit / (uint32_t)a.nc;  // 32-bit: the grid is one
    const int c = (int)(unit - uv * (uint32_t)a.nc);
    const int b = (int)(uv / (uint32_t)a.nv), j = (int)(uv - (uint32_t)b * (uint32_t)a.nv);
    const int hk = j / (a.nv / a.nk);
    uint8_t *wsu = a.ws + ((int64_t)c * a.B * a.nv + (int64_t)b * a.nv + j) * kUnitBytes;

    // ---- 1. 64 tokens of k and q, normalised, row-major in LDS: thread = (token tt, 16 consecutive elements)
    const int tt = tid >> 3, part = tid & 7;
    {
        const int t = c * kC + tt;
        const bool valid = t < a.T;  // a row past T reads the last row and gets the factor zero
        float kf[16], qf[16], gt = 0.0f, bt_ = 0.0f;
        {
            const int64_t bt = (int64_t)b * a.T + min(t, a.T - 1);
            if (part == 0) {  // requested with the rows, not where they are used
                gt = a.g[bt * a.nv + j];
                bt_ = a.beta[bt * a.nv + j];
            }
            const uint16_t *kp = a.k + (bt * a.nk + hk) * kWD + 16 * part;
            const uint16_t *qp = a.q + (bt * a.nk + hk) * kWD + 16 * part;
            unpack16(*(const u32x4 *)kp, *(const u32x4 *)(kp + 8), kf);
            unpack16(*(const u32x4 *)qp, *(const u32x4 *)(qp + 8), qf);
        }
        float kmul = 1.0f, qmul = a.q_scale;
        if (a.l2norm) {
            float sk = 0.0f, sq = 0.0f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                sk += kf[e] * kf[e];
                sq += qf[e] * qf[e];
            }
            // the eight threads of a token are eight consecutive lanes: neighbours in a quad, the other pair of the quad
            // (quad_perm [1,0,3,2], [2,3,0,1]), then the mirrored lane of the other quad (row_half_mirror); every
            // lane adds the same two numbers at each step, so all eight hold the same sum
            sk += dpp_or_zero<0xb1, 0xf>(sk);
            sq += dpp_or_zero<0xb1, 0xf>(sq);
            sk += dpp_or_zero<0x4e, 0xf>(sk);
            sq += dpp_or_zero<0x4e, 0xf>(sq);
            sk += dpp_or_zero<0x141, 0xf>(sk);
            sq += dpp_or_zero<0x141, 0xf>(sq);
            // 1 / max(|x|, 1e-3) as min(rsq(|x|^2), 1e3): one instruction (1 ulp) instead of a rounded sqrt and divide
            kmul = fminf(__builtin_amdgcn_rsqf(sk), 1e3f);
            qmul = a.q_scale * fminf(__builtin_amdgcn_rsqf(sq), 1e3f);
        }
        if (!valid) kmul = qmul = 0.0f;
        half8 k8[2], q8[2];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            k8[e >> 3][e & 7] = (_Float16)(kf[e] * kmul);
            q8[e >> 3][e & 7] = (_Float16)(qf[e] * qmul);
        }
        *(half8 *)&kh[tt * kPitchH + 16 * part] = k8[0];
        *(half8 *)&kh[tt * kPitchH + 16 * part + 8] = k8[1];
        *(half8 *)&qh[tt * kPitchH + 16 * part] = q8[0];
        *(half8 *)&qh[tt * kPitchH + 16 * part + 8] = q8[1];
        if (part == 0) {
            gs[tt] = valid ? gt : 0.0f;
            bs[tt] = valid ? bt_ : 0.0f;
            km[2 * tt] = kmul;
            km[2 * tt + 1] = qmul;
        }
    }
    lds_sync();

    // ---- 2. running sum of g and the decay factors (wavefront 0)
    if (wave == 0) {
        // inclusive scan over the 64 lanes with DPP moves (no trip through the LDS pipe per step): inside each row of
        // 16 lanes by shifts of 1, 2, 4, 8 (a lane with no source gets 0), then lane 15 of a row into the next row
        // (rows 1 and 3) and lane 31 into rows 2 and 3
        float x = gs[lane];
        x += dpp_or_zero<0x111, 0xf>(x);
        x += dpp_or_zero<0x112, 0xf>(x);
        x += dpp_or_zero<0x114, 0xf>(x);
        x += dpp_or_zero<0x118, 0xf>(x);
        x += dpp_or_zero<0x142, 0xa>(x);
        x += dpp_or_zero<0x143, 0xc>(x);
        const float g63 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 63));
        const float e = expf(x);
        Gs[lane] = x;
        *(float *)(wsu + kOffFn + 4 * lane) = -e * km[2 * lane];
        *(float *)(wsu + kOffFq + 4 * lane) = e * km[2 * lane + 1];
        *(float *)(wsu + kOffFt + 4 * lane) = expf(g63 - x) * km[2 * lane];
        if (lane == 63) *(float *)(wsu + kOffDecay) = e;
    }

    // ---- 3. k k^T (rows i, columns j) and k q^T (rows j, columns i): wavefront w owns row tile w/2, column tiles 2(w%2), +1
    float4v kk[2], qk[2];
    const int mt = wave >> 1;
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
            if (nt <= mt) {  // L is kept below the diagonal only, M on and above it: 20 of the 32 tile products
                const half8 bk = *(const half8 *)&kh[(16 * nt + li) * kPitchH + 32 * s + 8 * lq];
                kk[x] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ar, bk, kk[x], 0, 0, 0);
            }
            if (nt >= mt) {
                const half8 bq = *(const half8 *)&qh[(16 * nt + li) * kPitchH + 32 * s + 8 * lq];
                qk[x] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ar, bq, qk[x], 0, 0, 0);
            }
        }
    }
    lds_sync();  // G and beta are visible
#pragma unroll
    for (int x = 0; x < 2; ++x) {
        const int nt = 2 * (wave & 1) + x;
        const int col = 16 * nt + li;
        const float gcol = Gs[col];
        float4v lv;
        half4v m;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = 16 * mt + 4 * lq + r;
            lv[r] = col < row ? -bs[row] * kk[x][r] * __builtin_amdgcn_exp2f((Gs[row] - gcol) * kLog2e) : 0.0f;  // L[row][col]
            // masked q k^T: row = key j, col = query i, kept for j <= i
            m[r] = (_Float16)(row <= col ? qk[x][r] * __builtin_amdgcn_exp2f((gcol - Gs[row]) * kLog2e) : 0.0f);
        }
        // P[col][row]: the diagonal blocks in fp32 for the inverse, the rest as the fp16 operand it will be
        if (nt == mt) *(float4v *)&Dm[mt * kBlockD + li * kPitchD + 4 * lq] = lv;
        else *(half4v *)&Ph[col * kPitchL + 16 * mt + 4 * lq] = f32x4_to_half4(lv);
        if (nt >= 2 || mt < 2) *(half4v *)(wsu + kOffQK + (tri_block(nt, mt >> 1) * 64 + lane) * 16 + 8 * (mt & 1)) = m;
    }
    lds_sync();  // P complete; the row-major k / q tiles are dead from here on

    // ---- 4. the diagonal 16 x 16 blocks of (I - P)^-1: (I + D)(I + D^2)(I + D^4)(I + D^8) with D the (nilpotent) block.
    //         Wavefront a < 4 does block a by itself, in registers, on v_mfma_f32_16x16x16_f16.  With c(W) the
    //         accumulator layout of a matrix W (lane (li, lq): W[4 lq + r][li]), the B operand of W is c(W) and its A
    //         operand c(W^T) (both rounded to fp16), so a matrix kept as the pair c(W), c(W^T) multiplies without
    //         leaving the registers: eight products in a chain of four, where a trip through LDS per product was 2,200
    //         cycles.  The result is wanted as an A operand (step 5), i.e. as c of its transpose.
    if (wave < 4) {
        auto mm = [](const half4v &xa, const half4v &yb, const float4v &add) { return __builtin_amdgcn_mfma_f32_16x16x16f16(xa, yb, add, 0, 0, 0); };
        const float4v zero = {0.f, 0.f, 0.f, 0.f};
        float *Lb = Dm + wave * kBlockD;
        float4v d, it = *(const float4v *)&Lb[li * kPitchD + 4 * lq];  // c(D), c(D^T)
#pragma unroll
        for (int r = 0; r < 4; ++r) d[r] = Lb[(4 * lq + r) * kPitchD + li];
        const half4v hd = f32x4_to_half4(d), hdt = f32x4_to_half4(it);
#pragma unroll
        for (int r = 0; r < 4; ++r) it[r] += 4 * lq + r == li ? 1.0f : 0.0f;            // c((I + D)^T)
        const half4v hq = f32x4_to_half4(mm(hdt, hd, zero)), hqt = f32x4_to_half4(mm(hd, hdt, zero));  // D^2 and its transpose
        const float4v a1t = mm(hq, f32x4_to_half4(it), it);                             // ((I + D)(I + D^2))^T
        const half4v hp = f32x4_to_half4(mm(hqt, hq, zero)), hpt = f32x4_to_half4(mm(hq, hqt, zero));  // D^4
        const float4v a2t = mm(hp, f32x4_to_half4(a1t), a1t);                           // (... (I + D^4))^T
        const half4v hr = f32x4_to_half4(mm(hpt, hp, zero));                            // D^8
        const float4v a3t = mm(hr, f32x4_to_half4(a2t), a2t);                           // the inverse, transposed
        *(float4v *)&Lb[li * kPitchD + 4 * lq] = a3t;  // row li, columns 4 lq + r: where the diagonal block was
    }
    lds_sync();

    // ---- 5. Y = (I - P)^-1 = N^T by block back substitution, Y_b = Y_bb (I_b + sum_{m>b} P_bm Y_m), on
    //         v_mfma_f32_16x16x16_f16: wavefront w < 4 owns the 16 columns i of block w and walks the row blocks
    //         upwards with Y_m in registers (the accumulator layout of Y_m is the B operand layout of the next level).
    //         Rows are then scaled by beta_j (N' = N diag(beta)) and stored as the A operand of N' X.
    if (wave < 4) {
        half4v yh[4];
#pragma unroll
        for (int m = 0; m < 4; ++m) yh[m] = (half4v){(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
            const int bl = 3 - bb;
            float4v ya = {0.f, 0.f, 0.f, 0.f};
            if (bl <= wave) {
                float4v acc;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[r] = (bl == wave && 4 * lq + r == li) ? 1.0f : 0.0f;
#pragma unroll
                for (int m = bl + 1; m < 4; ++m) {
                    if (m <= wave) {
                        const half4v pa = *(const half4v *)&Ph[(16 * bl + li) * kPitchL + 16 * m + 4 * lq];
                        acc = __builtin_amdgcn_mfma_f32_16x16x16f16(pa, yh[m], acc, 0, 0, 0);
                    }
                }
                const half4v da = f32x4_to_half4(*(const float4v *)&Dm[bl * kBlockD + li * kPitchD + 4 * lq]);
                ya = __builtin_amdgcn_mfma_f32_16x16x16f16(da, f32x4_to_half4(acc), (float4v){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                yh[bl] = f32x4_to_half4(ya);
            }
            half4v o;
#pragma unroll
            for (int r = 0; r < 4; ++r) o[r] = (_Float16)(ya[r] * bs[16 * bl + 4 * lq + r]);
            if (wave >= 2 || bl < 2) *(half4v *)(wsu + kOffNt + (tri_block(wave, bl >> 1) * 64 + lane) * 16 + 8 * (bl & 1)) = o;
        }
    }
}

// ---------------------------------------------------------------------------------------------------- walk

// One chunk's operands in LDS; A operand blocks are 64 lanes x 16 B.
constexpr int kPitchT = 68;  // halves per row of the transposed k tile [dk][token]: 34 words, so the 16 rows an 8-byte read of a
                             // wavefront's quarter touches, and the rows 8 apart that its 2-byte writes touch, fall on different banks
                             // (72 gave two-way conflicts on both)
constexpr int oKn = 0;                        // -k e^G        [token tile 4][dk slab 4]
constexpr int oQg = oKn + 16384;              // q e^G         [token tile 4][dk slab 4]
constexpr int oKt = oQg + 16384;              // k e^(G63-G), transposed [dk 128][token 64], eight-token pieces permuted
constexpr int oNt = oKt + kWD * kPitchT * 2;  // N'            six blocks, tri_block order
constexpr int oQK = oNt + 6144;               // M             six blocks
constexpr int oV = oQK + 6144;                // v, the workgroup's columns: [token tile 4][32-column slab], natural k order
constexpr int oDec = oV + 8192;               // e^(G63)
constexpr int kBufBytes = oDec + 16;
// Behind the two operand buffers: the finished output rows of a chunk on their way out, and who has fetched them.
constexpr int kOutPitch = 68;  // floats per staged row: 64 columns + 4, so the four rows of a 16-byte read hit different banks
constexpr int oOut = 2 * kBufBytes, kLdsWalk = oOut + kC * kOutPitch * 4;
static_assert(kLdsWalk + 16 <= 163840, "two chunks of operands and one of output rows in the CU's LDS");

// Permutation of the 16-byte pieces inside a (-k e^G) / (q e^G) operand block: bits 1 and 2 of the piece index are
// flipped by the piece's row group (lq / 2) and by the parity of the block.  Readers (a lane per piece, 16 bytes) stay
// conflict-free: eight consecutive lanes still cover an aligned 128 bytes.
__device__ __forceinline__ int kq_swizzle(int lq, int blk) { return 2 * (lq >> 1) + 4 * (blk & 1); }

// Transposed tile [feature d][token]: the eight-token (16-byte) pieces of a row are permuted by d / 16, so that the
// threads of a wavefront, which write one token each for features 16 apart, hit different banks.
__device__ __forceinline__ int tpos(int d, int tok) { return d * kPitchT + ((((tok >> 3) ^ (d >> 4)) & 7) << 3) + (tok & 7); }

constexpr int kWalkThreads = 512;

// kCT: 16-column tiles per computing wavefront.  2: a workgroup owns 64 state columns, two workgroups per (sequence,
// v-head).  1: 32 columns, four workgroups -- half the products per chunk step for the same loading work, for batches
// whose walk would otherwise leave most of the chip idle (the chunk steps of a sequence are a chain).
template <int kCT>
__global__ __launch_bounds__(kWalkThreads) void deltanet_chunk_walk_kernel(WalkArgs a) {
    constexpr int kW = 32 * kCT;           // state columns of a workgroup
    constexpr int NP = kWD / kW;           // workgroups per (sequence, v-head)
    constexpr int kPitchO = kW + 4;        // floats per staged output row: the rows of a 16-byte read hit different banks
    static_assert(kPitchO <= kOutPitch, "the staging area is sized for 64 columns");
    __shared__ __attribute__((aligned(16))) uint8_t lds[kLdsWalk];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lq = lane >> 4;
    // Workgroups go to the 8 XCDs round-robin by linear id, and each XCD has its own L2.  The two column halves of a
    // (sequence, v-head) read the same triangles, and all v-heads of a k-head (both halves of each) the same q and k
    // rows: the 2 * rep workgroups of a (sequence, k-head) get linear ids congruent mod 8, consecutive in that XCD's
    // order, so that each of those comes from HBM once and the other readers find it in L2.
    const int p = blockIdx.x, pairs = a.B * a.nv, rep = a.nv / a.nk;
    int pair, part;  // part: which kW columns of the v-head
    if (((a.B * a.nk) & 7) == 0) {
        const int i = p >> 3, per = NP * rep;
        const int ku = (p & 7) + 8 * (i / per), sub = i % per;
        pair = ku * rep + sub / NP;
        part = sub % NP;
    } else if ((pairs & 7) == 0) {
        pair = (p & 7) + 8 * (p / (8 * NP));
        part = (p >> 3) % NP;
    } else {
        pair = p / NP;
        part = p % NP;
    }
    const int b = pair / a.nv, j = pair % a.nv, hk = j / rep;
    const int64_t chunk_stride = (int64_t)a.B * a.nv * kUnitBytes;
    const uint8_t *wsp = a.ws + (int64_t)pair * kUnitBytes;  // + ci * chunk_stride
    __shared__ int flag[2];  // the last chunk + 1 whose staged rows wavefront 2 / 3 has fetched

    // Roles by wavefront (wavefront w runs on SIMD w % 4): 0 and 1 compute, one per SIMD; 2, 3, 6 and 7 bring in the k
    // and q rows (the vector work of the loaders, on the two SIMDs without a computing wavefront) and 2 and 3 also carry
    // the finished output rows from LDS to memory; 4 and 5 copy the triangles and v.  A computing wavefront issues no
    // global access inside the walk: 32 four-byte stores per chunk cost it 2200 cycles of issue (a third of the chunk).
    if (wave == 4 || wave == 5) {  // ---- N', M, v, e^(G63): thread ct of 128; plain copies, no arithmetic
        const int ct = tid - 256;
        struct Stage {
            u32x4 nm[6], vr[2 * kCT];
            float dec;
        };
        auto fetch = [&](Stage &st, int ci) {
            ci = min(ci, a.nc - 1);
            const uint8_t *u = wsp + ci * chunk_stride;
#pragma unroll
            for (int i = 0; i < 6; ++i) st.nm[i] = *(const u32x4 *)(u + (ct + 128 * i) * 16);
#pragma unroll
            for (int i = 0; i < 2 * kCT; ++i) {  // item = (token, eight of this workgroup's columns)
                const int item = ct + 128 * i, tok = item / (kW / 8), pc = item % (kW / 8);
                const int64_t bt = (int64_t)b * a.T + min(ci * kC + tok, a.T - 1);
                st.vr[i] = __builtin_nontemporal_load((const u32x4 *)(a.v + (bt * a.nv + j) * kWD + kW * part + 8 * pc));
            }
            st.dec = *(const float *)(u + kOffDecay);
        };
        auto put = [&](const Stage &st, int ci, uint8_t *buf) {
#pragma unroll
            for (int i = 0; i < 6; ++i) *(u32x4 *)(buf + oNt + (ct + 128 * i) * 16) = st.nm[i];
#pragma unroll
            for (int i = 0; i < 2 * kCT; ++i) {
                const int item = ct + 128 * i, tok = item / (kW / 8), pc = item % (kW / 8);
                const bool valid = ci * kC + tok < a.T;  // rows past T are zero
                // eight bf16 as they are: one 16-byte piece of an A operand block of the bf16 MFMA (row = token, k-slots =
                // columns, natural order); the piece of lane (li, lq) sits at 4 li + lq, so that the eight tokens x four
                // pieces a wavefront writes are contiguous
                *(u32x4 *)(buf + oV + (((tok >> 4) * kCT + (pc >> 2)) * 64 + (tok & 15) * 4 + (pc & 3)) * 16) =
                    valid ? st.vr[i] : (u32x4){0u, 0u, 0u, 0u};
            }
            if (ct == 0) *(float *)(buf + oDec) = st.dec;
        };
        // Round c (after the barrier that publishes chunk c): chunk c + 1 goes into the other operand buffer, chunk c + 3
        // is requested.
        auto round = [&](Stage &st, int c) {
            lds_sync();
            if (c + 1 < a.nc) {
                put(st, c + 1, lds + ((c + 1) & 1) * kBufBytes);
                fetch(st, c + 3);
            }
        };
        Stage sa, sb;
        fetch(sa, 0);
        fetch(sb, 1);
        put(sa, 0, lds);
        fetch(sa, 2);
        for (int c = 0; c <= a.nc; c += 2) {  // chunk c + 1 comes from sb in even rounds, from sa in odd ones
            round(sb, c);
            if (c + 1 <= a.nc) round(sa, c + 1);
        }
        return;
    }
    if (wave >= 2) {
        // ---- k and q rows: thread = (token tl and tl + 32, dk 8 dp .. + 7 and 64 + 8 dp .. + 7: the eight threads
        //      of a token read whole 128-byte lines)
        const int lt = ((wave & 1) | ((wave >> 2) << 1)) * 64 + lane, tl = lt >> 3, dp = lt & 7;
        if (lt == 0) {  // visible to the computing wavefronts after the first barrier
            flag[0] = 0;
            flag[1] = 0;
        }
        struct Stage {
            u32x4 kr[2][2], qr[2][2];
            float fn[2], fq[2], ft[2];
        };
        auto fetch = [&](Stage &st, int ci) {
            ci = min(ci, a.nc - 1);
            const uint8_t *u = wsp + ci * chunk_stride;
#pragma unroll
            for (int ps = 0; ps < 2; ++ps) {
                const int tok = tl + 32 * ps;
                const int64_t bt = (int64_t)b * a.T + min(ci * kC + tok, a.T - 1);
                const uint16_t *kp = a.k + (bt * a.nk + hk) * kWD + 8 * dp;
                const uint16_t *qp = a.q + (bt * a.nk + hk) * kWD + 8 * dp;
                st.kr[ps][0] = *(const u32x4 *)kp;
                st.kr[ps][1] = *(const u32x4 *)(kp + 64);
                st.qr[ps][0] = *(const u32x4 *)qp;
                st.qr[ps][1] = *(const u32x4 *)(qp + 64);
                st.fn[ps] = *(const float *)(u + kOffFn + 4 * tok);  // zero for rows past T
                st.fq[ps] = *(const float *)(u + kOffFq + 4 * tok);
                st.ft[ps] = *(const float *)(u + kOffFt + 4 * tok);
            }
        };
        auto put = [&](const Stage &st, uint8_t *buf) {
            _Float16 *KT = (_Float16 *)(buf + oKt);
#pragma unroll
            for (int ps = 0; ps < 2; ++ps) {
                const int tok = tl + 32 * ps;
                float kf[16], qf[16];  // elements 0-7: dk 8 dp + e, 8-15: dk 64 + 8 dp + e
                unpack16(st.kr[ps][0], st.kr[ps][1], kf);
                unpack16(st.qr[ps][0], st.qr[ps][1], qf);
                const float fn = st.fn[ps], fq = st.fq[ps], ft = st.ft[ps];
#pragma unroll
                for (int h8 = 0; h8 < 2; ++h8) {
                    // dk 64 h8 + 8 dp + e: slab 2 h8 + dp / 4; inside the slab at 8 (dp % 4) + e, i.e. the tile of
                    // the slab (slots 0-3 or 4-7) is (dp / 2) % 2 and the row groups are lq = 2 (dp % 2), + 1
                    // The 16-byte pieces of a block are permuted: piece index (= reader lane) ^ kq_swizzle.  Unpermuted, the
                    // 16 lanes an 8-byte write handles per cycle (two tokens x eight dp) met in four bank pairs, four deep.
                    const int blk = (tok >> 4) * 4 + 2 * h8 + (dp >> 2);
                    const int o = blk * 1024 + (((2 * (dp & 1) * 16 + (tok & 15)) ^ kq_swizzle(2 * (dp & 1), blk)) * 16) + 8 * ((dp >> 1) & 1);
#pragma unroll
                    for (int g4 = 0; g4 < 2; ++g4) {
                        half4v hn, hq;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int i = 8 * h8 + 4 * g4 + e;
                            hn[e] = (_Float16)(kf[i] * fn);
                            hq[e] = (_Float16)(qf[i] * fq);
                            KT[tpos(64 * h8 + 8 * dp + 4 * g4 + e, tok)] = (_Float16)(kf[i] * ft);
                        }
                        *(half4v *)(buf + oKn + o + g4 * 256) = hn;
                        *(half4v *)(buf + oQg + o + g4 * 256) = hq;
                    }
                }
            }
        };
        // Two chunks of rows are in flight in registers: what is written into LDS for chunk c + 1 was requested while
        // chunk c - 1 was being computed.
        // Round c (after the barrier that publishes chunk c).  Wavefronts 2 and 3 (thread lt of 128) first take the
        // staged rows of chunk c - 1 into registers and release the staging area.  Then chunk c + 1 goes into the other
        // operand buffer; the rows leave for memory, 16 B per lane (kW / 4 lanes cover the bytes this workgroup owns of a
        // token's row); chunk c + 3 is requested.
        auto round = [&](Stage &st, int c) {
            lds_sync();
            u32x4 orow[4 * kCT];
            const bool carry = wave < 4 && c >= 1;
            if (carry) {
#pragma unroll
                for (int i = 0; i < 4 * kCT; ++i) {  // piece = (row, four columns)
                    const int pc = lt + 128 * i;
                    orow[i] = *(const u32x4 *)(lds + oOut + ((pc / (kW / 4)) * kPitchO + 4 * (pc % (kW / 4))) * 4);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (lane == 0) __hip_atomic_store(&flag[wave - 2], c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
            if (c + 1 < a.nc) put(st, lds + ((c + 1) & 1) * kBufBytes);
            if (carry) {
#pragma unroll
                for (int i = 0; i < 4 * kCT; ++i) {
                    const int pc = lt + 128 * i, t = (c - 1) * kC + pc / (kW / 4);
                    if (t < a.T) __builtin_nontemporal_store(orow[i], (u32x4 *)(a.out + (((int64_t)b * a.T + t) * a.nv + j) * kWD + kW * part + 4 * (pc % (kW / 4))));
                }
            }
            if (c + 1 < a.nc) fetch(st, c + 3);
        };
        Stage sa, sb;
        fetch(sa, 0);
        fetch(sb, 1);
        put(sa, lds);
        fetch(sa, 2);
        for (int c = 0; c <= a.nc; c += 2) {
            round(sb, c);
            if (c + 1 <= a.nc) round(sa, c + 1);
        }
        return;
    }

    // ---- the two computing wavefronts: wavefront w owns state columns kW part + 16 kCT w .. (kCT 16-column tiles c)
    const int col = kW * part + 16 * kCT * wave + li;
    float4v S[8][kCT];  // dk tile x: rows 16 x + 4 lq + r
    float *sp = a.state + ((int64_t)pair * kWD) * kWD + col;
#pragma unroll
    for (int x = 0; x < 8; ++x)
#pragma unroll
        for (int c = 0; c < kCT; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r) S[x][c][r] = sp[(int64_t)(16 * x + 4 * lq + r) * kWD + 16 * c];
    // the B operands (bf16, like v itself) that pick column tile c of this wavefront out of a 32-column slab of v
    bf16x8 pick[kCT];
#pragma unroll
    for (int c = 0; c < kCT; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e) pick[c][e] = (__bf16)(8 * lq + e == (16 * (kCT * wave + c)) % 32 + li ? 1.0f : 0.0f);
    const float4v zero = {0.f, 0.f, 0.f, 0.f};
    float *stage = (float *)(lds + oOut) + (4 * lq) * kPitchO + 16 * kCT * wave + li;  // + (16 tt + r) * kPitchO + 16 c

#define HS_MFMA(A, B, C) __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B, C, 0, 0, 0)
    // One chunk.  Every A operand read from LDS feeds two products (the two column tiles), and the reads of a group of
    // eight products are issued one group ahead (the scheduling barriers keep the compiler from sinking each read to
    // its use, which would serialise read latency and MFMA).
    for (int ci = 0; ci < a.nc; ++ci) {
        lds_sync();
        const uint8_t *buf = lds + (ci & 1) * kBufBytes;
        auto opA = [&](int off, int blk) { return *(const half8 *)(buf + off + blk * 1024 + lane * 16); };
        auto opKQ = [&](int off, int blk) { return *(const half8 *)(buf + off + blk * 1024 + (lane ^ kq_swizzle(lq, blk)) * 16); };
        const _Float16 *KT = (const _Float16 *)(buf + oKt);
        auto opKt = [&](int x, int s) {  // (k e^(G63-G))^T: row dk 16 x + li, k-slots = tokens of slab s in accumulator order
            const half4v lo = *(const half4v *)&KT[tpos(16 * x + li, 32 * s + 4 * lq)];
            const half4v hi = *(const half4v *)&KT[tpos(16 * x + li, 32 * s + 16 + 4 * lq)];
            return (half8){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        };
        float4v X[4][kCT], V[4][kCT];
        half8 an[2][4], nt[6], sh[kCT];
        bf16x8 va[4];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            va[tt] = *(const bf16x8 *)(buf + oV + (tt * kCT + (kCT * wave) / 2) * 1024 + (li * 4 + lq) * 16);
            an[0][tt] = opKQ(oKn, tt * 4);
        }
        const float dec = *(const float *)(buf + oDec);
        __builtin_amdgcn_sched_barrier(0);
        // X = v - (k e^G) S
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int c = 0; c < kCT; ++c) X[tt][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[tt], pick[c], zero, 0, 0, 0);
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {  // dk slab sl
            if (sl < 3) {
#pragma unroll
                for (int tt = 0; tt < 4; ++tt) an[(sl + 1) & 1][tt] = opKQ(oKn, tt * 4 + sl + 1);
            } else {
#pragma unroll
                for (int i = 0; i < 6; ++i) nt[i] = opA(oNt, i);
            }
#pragma unroll
            for (int c = 0; c < kCT; ++c) sh[c] = f32x8_to_half8(S[2 * sl][c], S[2 * sl + 1][c]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int c = 0; c < kCT; ++c) X[tt][c] = HS_MFMA(an[sl & 1][tt], sh[c], X[tt][c]);
            __builtin_amdgcn_sched_barrier(0);
        }
        half8 aq[2][4];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) aq[0][tt] = opKQ(oQg, tt * 4);
        half8 Xh[2][kCT];
#pragma unroll
        for (int c = 0; c < kCT; ++c) {
            Xh[0][c] = f32x8_to_half8(X[0][c], X[1][c]);
            Xh[1][c] = f32x8_to_half8(X[2][c], X[3][c]);
        }
        __builtin_amdgcn_sched_barrier(0);
        // V' = N' X (N' is lower triangular: token tiles 0 and 1 see only the first slab)
#pragma unroll
        for (int c = 0; c < kCT; ++c) {
            V[0][c] = HS_MFMA(nt[tri_block(0, 0)], Xh[0][c], zero);
            V[1][c] = HS_MFMA(nt[tri_block(1, 0)], Xh[0][c], zero);
            V[2][c] = HS_MFMA(nt[tri_block(2, 0)], Xh[0][c], zero);
            V[3][c] = HS_MFMA(nt[tri_block(3, 0)], Xh[0][c], zero);
        }
#pragma unroll
        for (int c = 0; c < kCT; ++c) {
            V[2][c] = HS_MFMA(nt[tri_block(2, 1)], Xh[1][c], V[2][c]);
            V[3][c] = HS_MFMA(nt[tri_block(3, 1)], Xh[1][c], V[3][c]);
        }
        __builtin_amdgcn_sched_barrier(0);
        // O = (q e^G) S + M V'
        float4v O[4][kCT];
        half8 qm[6], kt[2][4];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int c = 0; c < kCT; ++c) O[tt][c] = zero;
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            if (sl < 3) {
#pragma unroll
                for (int tt = 0; tt < 4; ++tt) aq[(sl + 1) & 1][tt] = opKQ(oQg, tt * 4 + sl + 1);
            } else {
#pragma unroll
                for (int i = 0; i < 6; ++i) qm[i] = opA(oQK, i);
            }
#pragma unroll
            for (int c = 0; c < kCT; ++c) sh[c] = f32x8_to_half8(S[2 * sl][c], S[2 * sl + 1][c]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int c = 0; c < kCT; ++c) O[tt][c] = HS_MFMA(aq[sl & 1][tt], sh[c], O[tt][c]);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) kt[0][i] = opKt(i >> 1, i & 1);
        half8 Vh[2][kCT];
#pragma unroll
        for (int c = 0; c < kCT; ++c) {
            Vh[0][c] = f32x8_to_half8(V[0][c], V[1][c]);
            Vh[1][c] = f32x8_to_half8(V[2][c], V[3][c]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < kCT; ++c) {
            O[0][c] = HS_MFMA(qm[tri_block(0, 0)], Vh[0][c], O[0][c]);
            O[1][c] = HS_MFMA(qm[tri_block(1, 0)], Vh[0][c], O[1][c]);
            O[2][c] = HS_MFMA(qm[tri_block(2, 0)], Vh[0][c], O[2][c]);
            O[3][c] = HS_MFMA(qm[tri_block(3, 0)], Vh[0][c], O[3][c]);
        }
#pragma unroll
        for (int c = 0; c < kCT; ++c) {
            O[2][c] = HS_MFMA(qm[tri_block(2, 1)], Vh[1][c], O[2][c]);
            O[3][c] = HS_MFMA(qm[tri_block(3, 1)], Vh[1][c], O[3][c]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 4; ++i) kt[1][i] = opKt(2 + (i >> 1), i & 1);
#pragma unroll
        for (int x = 0; x < 8; ++x)
#pragma unroll
            for (int c = 0; c < kCT; ++c) S[x][c] *= dec;
        __builtin_amdgcn_sched_barrier(0);
        // S <- e^(G63) S + (k e^(G63-G))^T V', two dk tiles at a time
#pragma unroll
        for (int xp = 0; xp < 4; ++xp) {
#pragma unroll
            for (int sl = 0; sl < 2; ++sl)
#pragma unroll
                for (int xo = 0; xo < 2; ++xo)
#pragma unroll
                    for (int c = 0; c < kCT; ++c)
                        S[2 * xp + xo][c] = HS_MFMA(kt[xp & 1][2 * xo + sl], Vh[sl][c], S[2 * xp + xo][c]);
            __builtin_amdgcn_sched_barrier(0);
            if (xp < 2) {
#pragma unroll
                for (int i = 0; i < 4; ++i) kt[xp & 1][i] = opKt(2 * (xp + 2) + (i >> 1), i & 1);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // The finished rows go to the staging area once the rows of the chunk before have been taken out of it (they
        // were, right after this chunk's barrier: the wait is there for the guarantee, not for the time).
        if (ci > 0)
            while (__hip_atomic_load(&flag[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < ci ||
                   __hip_atomic_load(&flag[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < ci)
                __builtin_amdgcn_s_sleep(1);
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int c = 0; c < kCT; ++c)
#pragma unroll
                for (int r = 0; r < 4; ++r) stage[(16 * tt + r) * kPitchO + 16 * c] = O[tt][c][r];
    }
#undef HS_MFMA
    lds_sync();  // the last chunk's rows are staged: wavefronts 2 and 3 take them from here
    float *sq = sp;  // opaque to the compiler: it would otherwise keep the 64 addresses of the first loads alive (spilled) across the walk
    asm volatile("" : "+v"(sq));
#pragma unroll
    for (int x = 0; x < 8; ++x)
#pragma unroll
        for (int c = 0; c < kCT; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r) sq[(int64_t)(16 * x + 4 * lq + r) * kWD + 16 * c] = S[x][c][r];
}

}  // namespace hs

extern "C" {

size_t hs_deltanet_chunked_workspace_bytes(int32_t B, int32_t T, int32_t nk, int32_t nv) {
    if (B <= 0 || T <= 0 || nk <= 0 || nv <= 0) return 0;
    return (size_t)((T + hs::kC - 1) / hs::kC) * (size_t)B * nv * hs::kUnitBytes;
}

// ... plus the fp32 output rows between the walk and the norm
size_t hs_deltanet_chunked_gated_norm_workspace_bytes(int32_t B, int32_t T, int32_t nk, int32_t nv) {
    if (B <= 0 || T <= 0 || nk <= 0 || nv <= 0) return 0;
    return ((hs_deltanet_chunked_workspace_bytes(B, T, nk, nv) + 255) & ~(size_t)255) + (size_t)B * T * nv * hs::kWD * sizeof(float);
}

// Workgroups of the walk the current device runs at once: one per CU (its LDS), looked up once per device.
static int walk_slots() {
    constexpr int kMaxDevices = 64;
    static int slots[kMaxDevices];  // 0: not asked yet (a second thread asking at the same time stores the same value)
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return 0;
    }
    if (slots[dev] == 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
            (void)hipGetLastError();
            return 0;
        }
        slots[dev] = cus > 0 ? cus : -1;
    }
    return slots[dev] > 0 ? slots[dev] : 0;
}

static int chunked_launch(const void *q, const void *k, const void *v, const float *g, const float *beta, float *state,
                          float *out, int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk, int32_t dv, float q_scale,
                          int l2norm, void *workspace, hipStream_t st) {
    using namespace hs;
    WalkArgs a{};
    a.q = (const uint16_t *)q; a.k = (const uint16_t *)k; a.v = (const uint16_t *)v;
    a.g = g; a.beta = beta; a.state = state; a.out = out; a.ws = (uint8_t *)workspace;
    a.B = B; a.T = T; a.nk = nk; a.nv = nv; a.nc = (T + kC - 1) / kC; a.q_scale = q_scale; a.l2norm = l2norm ? 1 : 0;
    deltanet_chunk_factor_kernel<<<(unsigned)((int64_t)B * nv * a.nc), 512, 0, st>>>(a);
    if (int rc = check_launch("deltanet_chunk_factor")) return rc;
    // 32-column workgroups while four of them per (sequence, v-head) still fit the device in one round
    if (4 * (int64_t)B * nv <= walk_slots()) deltanet_chunk_walk_kernel<1><<<(unsigned)(4 * B * nv), kWalkThreads, 0, st>>>(a);
    else deltanet_chunk_walk_kernel<2><<<(unsigned)(2 * B * nv), kWalkThreads, 0, st>>>(a);
    return check_launch("deltanet_chunk_walk");
}

// Argument checks common to both entry points; -1 = go on.
static int chunked_check(const void *q, const void *k, const void *v, const float *g, const float *beta, const float *state,
                         const void *out, int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk, int32_t dv,
                         const void *workspace, size_t workspace_bytes, size_t need) {
    using namespace hs;
    if (B > 0 && T > 0 && (!q || !k || !v || !g || !beta || !state || !out)) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (dk != kWD || dv != kWD) return fail(HS_ERR_INVALID_ARGUMENT, "deltanet is built for dk = dv = 128, got %d x %d", dk, dv);
    if (B < 0 || T < 0 || nk <= 0 || nv <= 0 || nv % nk != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "bad shape B=%d T=%d nk=%d nv=%d (need nv %% nk == 0)", B, T, nk, nv);
    if (B == 0 || T == 0) return HS_OK;
    const int64_t units = (int64_t)B * nv * ((T + kC - 1) / kC);
    if (units > INT32_MAX || (int64_t)B * nv > (1 << 29)) return fail(HS_ERR_INVALID_ARGUMENT, "too many chunks (%lld)", (long long)units);
    if (!workspace || workspace_bytes < need) return fail(HS_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    if ((((uintptr_t)workspace | (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "q, k, v, out and the workspace must be 16-byte aligned");
    return -1;
}

int hs_deltanet_forward_chunked(const void *q, const void *k, const void *v, const float *g, const float *beta, float *state,
                                float *out, int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk, int32_t dv,
                                float q_scale, int l2norm, void *workspace, size_t workspace_bytes, hs_stream_t stream) {
    if (int rc = chunked_check(q, k, v, g, beta, state, out, B, T, nk, nv, dk, dv, workspace, workspace_bytes,
                               hs_deltanet_chunked_workspace_bytes(B, T, nk, nv)); rc >= 0)
        return rc;
    return chunked_launch(q, k, v, g, beta, state, out, B, T, nk, nv, dk, dv, q_scale, l2norm, workspace, (hipStream_t)stream);
}

int hs_deltanet_forward_chunked_gated_norm(const void *q, const void *k, const void *v, const float *g, const float *beta,
                                           float *state, const void *z, const float *norm_weight, float norm_eps, void *out,
                                           int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk, int32_t dv,
                                           float q_scale, int l2norm, void *workspace, size_t workspace_bytes,
                                           hs_stream_t stream) {
    using namespace hs;
    if (B > 0 && T > 0 && (!z || !norm_weight)) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (int rc = chunked_check(q, k, v, g, beta, state, out, B, T, nk, nv, dk, dv, workspace, workspace_bytes,
                               hs_deltanet_chunked_gated_norm_workspace_bytes(B, T, nk, nv)); rc >= 0)
        return rc;
    if ((((uintptr_t)z | (uintptr_t)norm_weight) & 15) != 0)
        return fail(HS_ERR_INVALID_ARGUMENT, "z and norm_weight must be 16-byte aligned");
    float *rows = (float *)((uint8_t *)workspace + ((hs_deltanet_chunked_workspace_bytes(B, T, nk, nv) + 255) & ~(size_t)255));
    if (int rc = chunked_launch(q, k, v, g, beta, state, rows, B, T, nk, nv, dk, dv, q_scale, l2norm, workspace, (hipStream_t)stream))
        return rc;
    return hs_deltanet_gated_norm(rows, z, norm_weight, norm_eps, out, (int64_t)B * T * nv, dv, stream);
}

}  // extern "C"
