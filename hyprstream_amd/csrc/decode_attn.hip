// Dequant-fused GQA decode attention over the int8 / FP8-e4m3fn KV cache (gfx950, wave64).
//
// Split-K flash decoding.  Grid = (chunks, kv-heads, sequences); one 256-thread workgroup owns
// one chunk of `chunk_tokens` cached tokens of one (sequence, kv-head) and all G = Hq/Hkv query
// heads that read it, so every K/V byte is fetched from HBM exactly once.  Each of the four
// wavefronts walks its own 32-token steps of the chunk with a private online-softmax state;
// the next step's K/V/scales are already in flight (register double buffer) while the current
// one is consumed.  The wavefronts' (m, l, o) are merged through LDS.  With one chunk per sequence
// the workgroup normalises and writes the bf16 output itself (one launch per decode step);
// otherwise the chunk partial goes to the workspace and a second small kernel merges the chunks.
// Quantize-on-write of the step's new token rides in the same launch: the workgroup whose chunk
// ends at the sequence end quantizes that token's K and V rows (one wavefront each), stores codes
// and scales, and passes a barrier before any load that can cover that token, so the token it reads
// back is the one it wrote.
//
// Cache codes and scales are read exactly once per launch, so they are loaded with the non-temporal
// hint (streamed past the caches instead of displacing lines): measured 192 -> 181 us at B=64 x 8192.
// The 32 + 32 token scales of a step arrive with one 4-byte load per lane and reach the lanes that
// need them through a per-wavefront LDS hand-off (another 10 us less than per-lane 16-byte loads).
//
// Arithmetic.  Both products run on the MFMA pipe (v_mfma_f32_16x16x32_f16) with the G query
// heads on the N axis (padded to 16):
//   S[t, g]  = sum_d K[t, d] Q[g, d]          A = K codes, 16 tokens x 32 d per issue
//   O[d, g] += sum_t V^T[d, t] P[t, g]        A = V codes transposed in registers, B = P
// int8 codes enter the MFMA as EXACT fp16 integers: byte b -> fp16 bits 0x6400 | (b ^ 0x80)
// = 1152 + code.  For K the 1152 offset is cancelled by seeding the accumulator with
// -1152 * sum_d Q[g, d]; for V it is subtracted with one packed fp16 add (exact).  Q (bf16) is
// scaled per head by a power of two into fp16 range (exact) and the power is folded back into
// the softmax scale.  Scores, softmax and all accumulation are fp32; the per-token K scale is
// applied to the fp32 score, the per-token V scale is folded into P before P is rounded to fp16.
// The score accumulator layout (lane = head + 16*q, register r -> token 4q + r) is exactly the
// B-operand layout of the second product, so P never crosses lanes; the only cross-lane traffic
// is the running max (two butterfly steps over the lanes that share a head).
//
// HBM bytes per cached token and kv-head: 2*D codes + 8 B of scales (int8) -- 264 B at D = 128.
#include <atomic>
#include <mutex>

#include "quant_device.hpp"

namespace hs {

// Split-K scratch of the one entry point that takes no workspace (hs_decode_attn_int8_static): callers that cannot
// allocate (code under graph capture, serving loops or harnesses that forbid hipMalloc) get the chunk partials'
// memory from this array instead of a workspace argument.  Every device the library runs on holds its own copy at its
// own address for the life of the process.  In host code the NAME below is only a handle for hipGetSymbolAddress, never
// a device address: host code uses the per-device pointer kept in g_scratch_ptr.
constexpr size_t kScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
static std::atomic<void *> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the caller's current device; looked up once per device (first call there).
static int scratch_of_current_device(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(HS_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(HS_ERR_INVALID_ARGUMENT, "device ordinal %d out of range", dev);
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(HS_ERR_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing first calls store the same address
    }
    *out = p;
    return HS_OK;
}

// Calls that use the array must not overlap on a GPU.  Calls on one stream follow each other; a call on another
// stream is refused while the stream of the previous call still has work pending.  No event is created or recorded
// (the entry point allocates nothing and may run under graph capture): the test is hipStreamQuery on the previous
// stream, which is conservative (any pending work there counts).
struct ScratchUse {
    std::mutex mu;
    hipStream_t last = nullptr;
    bool valid = false;
};
static ScratchUse g_scratch_use[kMaxDevices];

static bool stream_blocks_with_default(hipStream_t s) {
    if (!s) return true;
    unsigned flags = 0;
    if (hipStreamGetFlags(s, &flags) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return (flags & hipStreamNonBlocking) == 0;
}

static int claim_scratch(hipStream_t stream) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(HS_ERR_LAUNCH, "hipGetDevice failed");
    ScratchUse &u = g_scratch_use[dev];
    std::lock_guard<std::mutex> lock(u.mu);
    if (u.valid && u.last != stream) {
        // the legacy default stream and a blocking stream wait for each other's work: ordered like one stream
        const bool ordered = (!stream && stream_blocks_with_default(u.last)) || (!u.last && stream_blocks_with_default(stream));
        if (!ordered) {
            hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
            if (u.last && hipStreamIsCapturing(u.last, &cs) != hipSuccess) {
                (void)hipGetLastError();  // the stream no longer exists: nothing of it is pending
                cs = hipStreamCaptureStatusNone;
                u.valid = false;
            }
            if (cs != hipStreamCaptureStatusNone)
                return fail(HS_ERR_BUSY, "the built-in split-K scratch of this GPU is being captured on another stream");
            if (u.valid) {
                const hipError_t q = hipStreamQuery(u.last);
                if (q == hipErrorNotReady)
                    return fail(HS_ERR_BUSY,
                                "the built-in split-K scratch of this GPU is in use on another stream: call on that "
                                "stream, wait for it, or use hs_decode_attn_int8 with a workspace per stream");
                if (q != hipSuccess) (void)hipGetLastError();
            }
        }
    }
    u.last = stream;
    u.valid = true;
    return HS_OK;
}

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// head_dim 64, 128 or 256.  A wavefront step always covers 8 KB of codes: 64 tokens at D = 64, 32 at D = 128, 16 at
// D = 256 (the second product then runs on v_mfma_f32_16x16x16_f16, whose operand layout matches one 16-token tile).
template <int D> struct Shape {
    static constexpr int kStep = 4096 / D;            // tokens per wavefront step
    static constexpr int NT = kStep / 16;             // 16-token score tiles per step
    static constexpr int NJ = D / 32;                 // MFMAs per score tile (32 d each)
    static constexpr int VW = D >= 128 ? 2 : 1;       // dwords of V codes a lane takes per token (d = 4*VW*li ..)
    static constexpr int NBB = 4 * VW;                // V^T row blocks (MFMAs) per column group
    static constexpr int CW = 16 * NBB;               // columns of a group: 128, or the whole head at D = 64
    static constexpr int NC = D / CW;                 // column groups of V / O
    static constexpr int NS = kStep > 32 ? 2 : 1;     // scale loads per lane and step
};
template <int VW> struct VCodes { typedef u32x2 type; };
template <> struct VCodes<1> { typedef uint32_t type; };
__device__ __forceinline__ uint32_t vword(const u32x2 &x, int i) { return x[i]; }
__device__ __forceinline__ uint32_t vword(uint32_t x, int) { return x; }
constexpr int kWavesPerWg = 4;
constexpr int kMaxBalancedB = 1024;  // most sequences a batch may have for the balanced (token-range) split
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kPScale = 64.0f;  // P is carried as 64*p*s_v in fp16 (keeps small weights normal)

struct DecodeArgs {
    const uint16_t *q;   // [B, Hq, D] bf16
    const uint8_t *kc, *vc;
    const float *ks, *vs;
    KvAddr ka, va;
    const int32_t *seq_lens;
    float *part_o;   // [B, Hq, nchunks, D]
    float *part_ml;  // [B, Hq, nchunks, 2]   (m in log2 units, l)
    uint16_t *out;       // [B, Hq, D] bf16
    const uint16_t *out_gate;  // optional [B, Hq, D] bf16: out = bf16(bf16(attention) * bf16(sigmoid(gate)))
    QuantArgs nt;        // the step's new token (nt.src[0] == nullptr: none); position = seq_len - 1
    int32_t direct;      // 1: single chunk, write `out` directly; 0: leave partials in the workspace
    int32_t B, Hq, Hkv, G, chunk_tokens, nchunks, max_seq_len;
    // balanced mode (ragged batches): the cached tokens of a kv-head over the whole batch, counted in 64-token
    // granules, are cut into `pieces` equal ranges, one per workgroup; min_granules bounds how small a range may get
    // (and with it the partial slots a sequence can need: nchunks)
    int32_t balanced, pieces, min_granules;
    float scale_log2e;
    // optional rotary embedding of q (bf16 tables [rope_len, D/2]); the new token's K is rotated by nt.rope_*
    const uint16_t *rope_sin, *rope_cos;
    int32_t rope_len, rotary_dim;
    NormSpec qnorm;  // optional QK-norm of q ahead of the rotation (the new token's K: nt.norm)
};

// Half-split rotary embedding of the query elements a lane holds, in bf16 arithmetic (every product and sum rounded
// to bf16, as the separate libtorch ops of RoPE::apply_rotary_pos_emb do, rope.rs:206-248).  Element qf[8*i + e] is
// d = 64*(i/2) + 16*lq + 8*(i%2) + e (i < NJ = D/32; at D = 64: d = 16*lq + 8*i + e).  The first `rd` elements of the
// head are rotated in pairs (d, d + rd/2), tables [.., rd/2]:
//   rd >= 128  a lane holds both halves of each pair (register blocks i and i + rd/64);
//   rd = 64    the halves sit 32 lanes apart (blocks 0 and 1 of lanes lq and lq ^ 2);
//   rd = 32    16 lanes apart (blocks 0 and 1 of lanes lq = 0 and 1).
// Cross-lane pairs exchange their elements and each lane computes its own half.
template <int NJ, int NJR>
__device__ __forceinline__ void rope_q_inlane(float (&qf)[8 * NJ], const uint16_t *sin_row, const uint16_t *cos_row, int lq) {
#pragma clang fp contract(off)
    auto rb = [](float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); };
#pragma unroll
    for (int i = 0; i < NJR / 2; ++i) {
        const int j0 = 64 * (i >> 1) + 16 * lq + 8 * (i & 1);
        const u32x4 sw = *(const u32x4 *)(sin_row + j0), cw = *(const u32x4 *)(cos_row + j0);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float sn = (e & 1) ? __uint_as_float(sw[e >> 1] & 0xffff0000u) : __uint_as_float(sw[e >> 1] << 16);
            const float cs = (e & 1) ? __uint_as_float(cw[e >> 1] & 0xffff0000u) : __uint_as_float(cw[e >> 1] << 16);
            const float x1 = qf[8 * i + e], x2 = qf[8 * (i + NJR / 2) + e];
            qf[8 * i + e] = rb(rb(x1 * cs) - rb(x2 * sn));
            qf[8 * (i + NJR / 2) + e] = rb(rb(x1 * sn) + rb(x2 * cs));
        }
    }
}
template <int NJ, int XOR>  // rd = 2 * XOR: 64 or 32
__device__ __forceinline__ void rope_q_crosslane(float (&qf)[8 * NJ], const uint16_t *sin_row, const uint16_t *cos_row, int lq) {
#pragma clang fp contract(off)
    auto rb = [](float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); };
    if (16 * lq >= 2 * XOR) return;  // this lane's elements of blocks 0 and 1 lie beyond the rotated part
    const bool upper = 16 * lq >= XOR;  // this lane holds x2 of its pairs
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int j0 = ((16 * lq) & (XOR - 1)) + 8 * i;
        const u32x4 sw = *(const u32x4 *)(sin_row + j0), cw = *(const u32x4 *)(cos_row + j0);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float sn = (e & 1) ? __uint_as_float(sw[e >> 1] & 0xffff0000u) : __uint_as_float(sw[e >> 1] << 16);
            const float cs = (e & 1) ? __uint_as_float(cw[e >> 1] & 0xffff0000u) : __uint_as_float(cw[e >> 1] << 16);
            const float mine = qf[8 * i + e], other = __shfl_xor(mine, XOR, 64);
            qf[8 * i + e] = upper ? rb(rb(other * sn) + rb(mine * cs)) : rb(rb(mine * cs) - rb(other * sn));
        }
    }
}
// Normalises the 8 elements d0 .. d0 + 7 of a head's row in place, given the row's reciprocal root.
__device__ __forceinline__ void norm_q_group(float (&x)[8], const NormSpec &n, int head, int d0, float rrms) {
#pragma clang fp contract(off)
    float w[8];
    if (n.kind == 1) {
        const u32x4 ww = *(const u32x4 *)((const uint16_t *)n.weight + (int64_t)head * n.head_stride + d0);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            w[2 * e] = __uint_as_float(ww[e] << 16);
            w[2 * e + 1] = __uint_as_float(ww[e] & 0xffff0000u);
        }
    } else {
        const float *wp = (const float *)n.weight + (int64_t)head * n.head_stride + d0;
        const float4v w0 = *(const float4v *)wp, w1 = *(const float4v *)(wp + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            w[e] = w0[e];
            w[4 + e] = w1[e];
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = norm_apply(x[e], w[e], rrms, HS_BF16, n.kind);
}

// Per-head QK-norm of the query elements a lane holds (bf16 tensor; NormSpec in quant_device.hpp).  The four lanes
// lq = 0..3 of a head share its sum of squares.  Returns the row's reciprocal root.
template <int NJ>
__device__ __forceinline__ float norm_q(float (&qf)[8 * NJ], const NormSpec &n, int head, int lq, int D) {
#pragma clang fp contract(off)
    double ss = 0.0;
#pragma unroll
    for (int i = 0; i < 8 * NJ; ++i) ss += (double)norm_square(qf[i], HS_BF16, n.kind);
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    const float rrms = norm_rrms(ss, D, HS_BF16, n.kind, n.eps);
#pragma unroll
    for (int i = 0; i < NJ; ++i) {
        const int d0 = NJ == 2 ? 16 * lq + 8 * i : 64 * (i >> 1) + 16 * lq + 8 * (i & 1);
        float x[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = qf[8 * i + e];
        norm_q_group(x, n, head, d0, rrms);
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[8 * i + e] = x[e];
    }
    return rrms;
}

// Any other rotated length (a multiple of 16): the 8 partners of a lane's 8 elements are 8 consecutive elements of the
// row, which the lane reads from the q tensor and normalises itself (the norm is elementwise once the row's reciprocal
// root is known) instead of finding the lane and register that hold them.
template <int NJ>
__device__ __forceinline__ void rope_q_general(float (&qf)[8 * NJ], const uint16_t *sin_row, const uint16_t *cos_row, int lq, int rd,
                                               const uint16_t *q_row, const NormSpec &n, int head, float rrms) {
#pragma clang fp contract(off)
    auto rb = [](float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); };
    const int half = rd / 2;
#pragma unroll
    for (int i = 0; i < NJ; ++i) {
        const int d0 = NJ == 2 ? 16 * lq + 8 * i : 64 * (i >> 1) + 16 * lq + 8 * (i & 1);
        if (d0 >= rd) continue;
        const bool upper = d0 >= half;  // this lane holds x2 of its pairs
        const int pd0 = upper ? d0 - half : d0 + half, j0 = upper ? pd0 : d0;
        const u32x4 pw = *(const u32x4 *)(q_row + pd0);
        float other[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            other[2 * e] = __uint_as_float(pw[e] << 16);
            other[2 * e + 1] = __uint_as_float(pw[e] & 0xffff0000u);
        }
        if (n.kind != 0) norm_q_group(other, n, head, pd0, rrms);
        const u32x4 sw = *(const u32x4 *)(sin_row + j0), cw = *(const u32x4 *)(cos_row + j0);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float sn = (e & 1) ? __uint_as_float(sw[e >> 1] & 0xffff0000u) : __uint_as_float(sw[e >> 1] << 16);
            const float cs = (e & 1) ? __uint_as_float(cw[e >> 1] & 0xffff0000u) : __uint_as_float(cw[e >> 1] << 16);
            const float mine = qf[8 * i + e];
            qf[8 * i + e] = upper ? rb(rb(other[e] * sn) + rb(mine * cs)) : rb(rb(mine * cs) - rb(other[e] * sn));
        }
    }
}

template <int NJ>
__device__ __forceinline__ void rope_rotate_q(float (&qf)[8 * NJ], const uint16_t *sin_row, const uint16_t *cos_row, int lq, int rd,
                                              const uint16_t *q_row, const NormSpec &n, int head, float rrms) {
    if constexpr (NJ >= 4) {
        if (rd == 32 * NJ) return rope_q_inlane<NJ, NJ>(qf, sin_row, cos_row, lq);
    }
    if constexpr (NJ == 8) {
        if (rd == 128) return rope_q_inlane<NJ, 4>(qf, sin_row, cos_row, lq);
    }
    if (rd == 64) return rope_q_crosslane<NJ, 32>(qf, sin_row, cos_row, lq);
    if (rd == 32) return rope_q_crosslane<NJ, 16>(qf, sin_row, cos_row, lq);
    rope_q_general<NJ>(qf, sin_row, cos_row, lq, rd, q_row, n, head, rrms);
}

template <int D>
struct Stage {
    u32x4 k[Shape<D>::NT][Shape<D>::NJ / 2];  // [16-token tile][64-byte piece of the row]: 16 B at byte 64*piece + 16*lq of row li
    typename VCodes<Shape<D>::VW>::type v[Shape<D>::NC][4 * Shape<D>::NT];  // [column group c][token slot e = 4u + r]: d = CW*c + 4*VW*(lane%16) ..
    // int8 only.  Steps of up to 32 tokens: lanes [0, kStep) hold the K scale of token `lane`, lanes [kStep, 2*kStep)
    // the V scales; 64-token steps: [0] the K scale and [1] the V scale of token `lane`
    float sraw[Shape<D>::NS];
};

__device__ __forceinline__ half8 as_half8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    u32x4 t = {a, b, c, d};
    return __builtin_bit_cast(half8, t);
}

// Two bytes (in the high byte of each 16-bit half of t) holding e4m3fn codes -> two fp16 whose
// value is code_value * 2^-8 (exponent bias 15 instead of 7; the factor is folded into the scale).
__device__ __forceinline__ uint32_t fp8x2_to_f16x2(uint32_t t) {
    return (t & 0x80008000u) | ((t >> 1) & 0x3f803f80u);
}

template <int kD, bool FP8, bool ROPE, bool BAL>
__global__ __launch_bounds__(256, 2) void decode_attn_kernel(DecodeArgs a_in) {
    const DecodeArgs &a = a_in;
    constexpr int kStep = Shape<kD>::kStep, NT = Shape<kD>::NT, NJ = Shape<kD>::NJ, NC = Shape<kD>::NC;
    constexpr int VW = Shape<kD>::VW, NBB = Shape<kD>::NBB, CW = Shape<kD>::CW, NS = Shape<kD>::NS;
    constexpr bool kPreloadNext = BAL;
    const int h = blockIdx.y;
    const int G = a.G;
    // the wavefront index as a scalar: everything derived from it (the steps this wavefront walks, block-table lookups,
    // base addresses) then stays in scalar registers and scalar loads
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15, lq = lane >> 4;
    __shared__ __attribute__((aligned(16))) float sm_sc[kWavesPerWg][64 * NS];
    __shared__ float sm_m[kWavesPerWg][16], sm_l[kWavesPerWg][16];
    __shared__ float sm_o[kWavesPerWg][16][CW + 4];  // one column group of O at a time
    // One work item: tokens [t_begin, t_end) of sequence b (L cached tokens), partial slot `chunk`.
    struct Item {
        int b, L, t_begin, t_end, chunk;
    };
    // The two stages of the load pipeline and the location of the step this wavefront loads next live outside an
    // item: a workgroup that walks several items (balanced mode) issues the first loads of the next item before it
    // merges and writes out the current one, so that the pipeline does not run empty at every sequence end.
    Stage<kD> sa, sb;
    int64_t nku = 0, nvu = 0;
    int nks = 0, nvs = 0;
    // `preloaded`: the first stage of this item is already in flight (issued at the end of the previous item);
    // `next`: the item whose first loads this one issues before it merges (has_next), else ignored.
    auto run_item = [&](const Item it, const bool preloaded, const Item next, const bool has_next) {
    const int b = it.b, L = it.L, chunk = it.chunk;
    // Balanced mode runs this body in a loop over items.  Read through the kernel's own parameter, every argument an
    // item needs anywhere (new-token sources, Q, outputs, tables: far more than the scalar register file holds) is
    // loaded once ahead of that loop and stays live across it, and the loop over the steps runs on spilled scalars.
    // Each item therefore reads its arguments anew from the kernel-argument segment, through a pointer the compiler
    // cannot see through: they are loaded where they are used and die there, as in the one-item instances.
    uintptr_t seg = (uintptr_t)__builtin_amdgcn_kernarg_segment_ptr();  // DecodeArgs is the kernel's only parameter
    if constexpr (BAL) asm volatile("" : "+s"(seg));
    const DecodeArgs &a = BAL ? *(const DecodeArgs *)(const __attribute__((address_space(4))) DecodeArgs *)seg : a_in;
    // This workgroup reads the newest token if it owns the end of the sequence: it then writes it first (K by
    // wavefront 0, V by wavefront 1).  With five or more steps the token sits beyond every wavefront's first tile,
    // so those first loads are issued ahead of the write and its barrier instead of behind them.
    const int t_begin = it.t_begin, t_end = it.t_end;
    const bool writes_new = a.nt.src[0] != nullptr && t_end == L;
    auto write_new_token = [&]() {
        if (wave < 2) quantize_row<kD / 64, FP8>(a.nt, wave, (int64_t)b * a.Hkv + h, lane);
        __syncthreads();  // codes and scales are visible to the whole workgroup before any load that covers them
    };

    half8 qop[NJ];
    float cq = 0.0f, cinit = 0.0f;
    // fp8: the V scale is one constant per (sequence, head); it multiplies the finished partial.
    const float out_scale = (1.0f / kPScale) * (FP8 ? 256.0f * a.vs[(int64_t)b * a.Hkv + h] : 1.0f);

    float4v acc[NBB * NC];  // O[d = CW*c + 4*NBB*lq + NBB*r + bb][head li] in acc[NBB*c + bb][r]
#pragma unroll
    for (int i = 0; i < NBB * NC; ++i) acc[i] = (float4v){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.0f;

    const int nsteps = (t_end - t_begin + kStep - 1) / kStep;

    // Where the step this wavefront loads next lives (sequence or block, slot).  With block tables the lookup is a
    // dependent (scalar) load in front of every address, so it is issued one stage ahead: load_stage() uses the
    // location found while the previous stage was loaded and starts the lookup for the one after.
    auto locate = [&](const Item &w, int step) {
        const int t0 = w.t_begin + step * kStep;
        if (t0 < w.t_end) {
            resolve(a.ka, w.b, t0, nku, nks);
            resolve(a.va, w.b, t0, nvu, nvs);
        }
    };
    auto load_stage = [&](Stage<kD> &st, const Item &w, int step) {
        const int t0 = w.t_begin + step * kStep;
        const int64_t ku = nku, vu = nvu;
        const int kslot = nks, vslot = nvs;
        locate(w, step + kWavesPerWg);
        const int last = w.L - 1 - t0;  // last valid row offset inside this step (>= 0)
        const uint8_t *kb = a.kc + ku * a.ka.code_stride_seq + (int64_t)h * a.ka.code_stride_head + (int64_t)kslot * kD;
        const uint8_t *vb = a.vc + vu * a.va.code_stride_seq + (int64_t)h * a.va.code_stride_head + (int64_t)vslot * kD;
#pragma unroll
        for (int u = 0; u < NT; ++u) {
            const int row = min(16 * u + li, last);
            const uint8_t *p = kb + row * kD + 16 * lq;  // each load covers one 64-byte piece of 16 rows
#pragma unroll
            for (int hf = 0; hf < NJ / 2; ++hf) st.k[u][hf] = __builtin_nontemporal_load((const u32x4 *)(p + 64 * hf));
        }
        if (!FP8) {
            // one 4-byte load per lane brings the step's K scales and V scales (two full 128-byte lines at 32 tokens);
            // compute_stage hands them to the lanes that need them through LDS
            const float *ksb = a.ks + ku * a.ka.scale_stride_seq + (int64_t)h * a.ka.scale_stride_head + kslot;
            const float *vsb = a.vs + vu * a.va.scale_stride_seq + (int64_t)h * a.va.scale_stride_head + vslot;
            if constexpr (NS == 1) {
                const int sl = lane & (2 * kStep - 1);  // 16-token steps: the upper 32 lanes repeat the lower ones
                st.sraw[0] = __builtin_nontemporal_load((sl < kStep ? ksb : vsb) + min(sl & (kStep - 1), last));
            } else {
                st.sraw[0] = __builtin_nontemporal_load(ksb + min(lane, last));
                st.sraw[1] = __builtin_nontemporal_load(vsb + min(lane, last));
            }
        }
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int u = 0; u < NT; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = min(16 * u + 4 * lq + r, last);
                    st.v[c][4 * u + r] = __builtin_nontemporal_load((const typename VCodes<VW>::type *)(vb + row * kD + CW * c + 4 * VW * li));
                }
    };

    auto compute_stage = [&](const Stage<kD> &st, int step) {
        const int t0 = t_begin + step * kStep;
        // ---- token scales: lane (li, lq) needs those of tokens 16u + 4*lq + r, the rows of its score registers.
        //      LDS operations of one wavefront complete in order, so the reads see the write without a barrier.
        float4v sk[NT], sv[NT];
        if (!FP8) {
            sm_sc[wave][lane] = st.sraw[0];
            if constexpr (NS == 2) sm_sc[wave][64 + lane] = st.sraw[1];
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int u = 0; u < NT; ++u) {
                sk[u] = *(const float4v *)&sm_sc[wave][16 * u + 4 * lq];
                sv[u] = *(const float4v *)&sm_sc[wave][kStep + 16 * u + 4 * lq];
            }
        }
        // ---- scores: NT tiles x NJ MFMAs (the head dimension in pieces of 32)
        float4v s[NT];
#pragma unroll
        for (int u = 0; u < NT; ++u) {
            s[u] = (float4v){cinit, cinit, cinit, cinit};
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const uint32_t w0 = st.k[u][j >> 1][2 * (j & 1)], w1 = st.k[u][j >> 1][2 * (j & 1) + 1];
                half8 ak;
                if (FP8) {
                    ak = as_half8(fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, w0, 0x010c000cu)),
                                  fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, w0, 0x030c020cu)),
                                  fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, w1, 0x010c000cu)),
                                  fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, w1, 0x030c020cu)));
                } else {
                    const uint32_t x0 = w0 ^ 0x80808080u, x1 = w1 ^ 0x80808080u;
                    ak = as_half8(__builtin_amdgcn_perm(0x64646464u, x0, 0x04010400u),
                                  __builtin_amdgcn_perm(0x64646464u, x0, 0x04030402u),
                                  __builtin_amdgcn_perm(0x64646464u, x1, 0x04010400u),
                                  __builtin_amdgcn_perm(0x64646464u, x1, 0x04030402u));
                }
                s[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ak, qop[j], s[u], 0, 0, 0);
            }
        }
        // ---- scale to log2 units, mask the tail
        float sc[4 * NT], pv[4 * NT];
#pragma unroll
        for (int u = 0; u < NT; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                sc[4 * u + r] = FP8 ? s[u][r] * cq : s[u][r] * sk[u][r] * cq;
                pv[4 * u + r] = FP8 ? kPScale : sv[u][r] * kPScale;
            }
        const bool tail = t0 + kStep > L;
        if (tail) {
#pragma unroll
            for (int u = 0; u < NT; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (t0 + 16 * u + 4 * lq + r >= L) {
                        sc[4 * u + r] = -INFINITY;
                        pv[4 * u + r] = 0.0f;
                    }
        }
        // ---- online softmax (max shared by the 4 lanes of a head)
        float mx = sc[0];
#pragma unroll
        for (int i = 1; i < 4 * NT; ++i) mx = fmaxf(mx, sc[i]);
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= alpha;
#pragma unroll
            for (int i = 0; i < NBB * NC; ++i) acc[i] *= alpha;
            m_run = m_new;
        }
        uint32_t pb[2 * NT];
#pragma unroll
        for (int i = 0; i < 2 * NT; ++i) {
            const float p0 = __builtin_amdgcn_exp2f(sc[2 * i] - m_run);
            const float p1 = __builtin_amdgcn_exp2f(sc[2 * i + 1] - m_run);
            l_run += p0 + p1;
            half2v hp = {(_Float16)(p0 * pv[2 * i]), (_Float16)(p1 * pv[2 * i + 1])};
            pb[i] = __builtin_bit_cast(uint32_t, hp);
        }
        // ---- O += V^T P : one MFMA per 32 tokens and byte column bb of this lane's d's
#pragma unroll
        for (int cb = 0; cb < NBB * NC; ++cb) {
            const int c = cb / NBB, bb = cb % NBB;
            uint32_t av[2 * NT];
#pragma unroll
            for (int p = 0; p < 2 * NT; ++p) {
                const uint32_t lo = vword(st.v[c][2 * p], bb >> 2), hi = vword(st.v[c][2 * p + 1], bb >> 2);
                if (FP8) {
                    const uint32_t sel = 0x040c000cu + ((uint32_t)(bb & 3) << 8) + ((uint32_t)(bb & 3) << 24);
                    av[p] = fp8x2_to_f16x2(__builtin_amdgcn_perm(hi, lo, sel));
                } else {
                    const uint32_t sel = 0x0c040c00u + (uint32_t)(bb & 3) + ((uint32_t)(bb & 3) << 16);
                    const uint32_t w = __builtin_amdgcn_perm(hi, lo, sel) ^ 0x64806480u;
                    half2v hv = __builtin_bit_cast(half2v, w) - (half2v){(_Float16)1152.0f, (_Float16)1152.0f};
                    av[p] = __builtin_bit_cast(uint32_t, hv);
                }
            }
            if constexpr (NT >= 2) {
#pragma unroll
                for (int tg = 0; tg < NT / 2; ++tg)  // 32 tokens (two score tiles) per MFMA
                    acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(av[4 * tg], av[4 * tg + 1], av[4 * tg + 2], av[4 * tg + 3]),
                                                                     as_half8(pb[4 * tg], pb[4 * tg + 1], pb[4 * tg + 2], pb[4 * tg + 3]),
                                                                     acc[cb], 0, 0, 0);
            } else {
                const u32x2 aw = {av[0], av[1]}, pw = {pb[0], pb[1]};
                acc[cb] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4, aw), __builtin_bit_cast(half4, pw),
                                                                acc[cb], 0, 0, 0);
            }
        }
    };

    // ---- software pipeline over this wavefront's steps (wave, wave+4, ...)
    int step = wave;
    const bool early_loads = nsteps >= kWavesPerWg + 1;  // a preloaded item always has them
    if (writes_new && !early_loads) write_new_token();
    if (!preloaded) {
        locate(it, step);
        if (step < nsteps) load_stage(sa, it, step);
    }
    if (writes_new && early_loads) write_new_token();
    // ---- Q operand (prepared while the first K/V tiles are in flight): lane (head li, quarter lq) holds
    //      Q[head][64*(j/2) + 16*lq + 8*(j%2) + e] for MFMA j.
    {
        float qf[8 * NJ];
        float amax = 0.0f;
        if (li < G) {
            const uint16_t *qp = a.q + ((int64_t)b * a.Hq + h * G + li) * kD + 16 * lq;
#pragma unroll
            for (int i = 0; i < NJ; ++i) {  // MFMA i contracts d = 64*(i/2) + 16*lq + 8*(i%2) + e, as the K loads do
                u32x4 w = *(const u32x4 *)(qp + 64 * (i >> 1) + 8 * (i & 1));
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    qf[8 * i + 2 * e] = __uint_as_float(w[e] << 16);
                    qf[8 * i + 2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
                }
            }
            if (ROPE) {  // the step's prologue on q: QK-norm, then the rotation
                float rrms = 0.0f;
                if (a.qnorm.kind != 0) rrms = norm_q<NJ>(qf, a.qnorm, h * G + li, lq, kD);
                if (a.rope_sin != nullptr) {
                    const int p = min(max(a.seq_lens[b] - 1, 0), a.rope_len - 1);  // the query is the newest token
                    const int half = a.rotary_dim / 2;
                    rope_rotate_q<NJ>(qf, a.rope_sin + (int64_t)p * half, a.rope_cos + (int64_t)p * half, lq, a.rotary_dim,
                                      qp - 16 * lq, a.qnorm, h * G + li, rrms);
                }
            }
#pragma unroll
            for (int i = 0; i < 8 * NJ; ++i) amax = fmaxf(amax, fabsf(qf[i]));
        } else {
#pragma unroll
            for (int i = 0; i < 8 * NJ; ++i) qf[i] = 0.0f;
        }
        amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        // amax = f * 2^ex with f in [0.5, 1); scaling by 2^-ex is exact (a multiplication by a power of two)
        int ex = 0;
        if (amax > 0.0f && amax < 3.0e38f) ex = min(126, max(-125, (int)((__float_as_uint(amax) >> 23) & 0xff) - 126));
        const float down = __uint_as_float((uint32_t)(127 - ex) << 23), up = __uint_as_float((uint32_t)(127 + ex) << 23);
        float qsum = 0.0f;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                _Float16 hq = (_Float16)(qf[8 * j + e] * down);
                qop[j][e] = hq;
                qsum += (float)hq;
            }
        }
        qsum += __shfl_xor(qsum, 16, 64);
        qsum += __shfl_xor(qsum, 32, 64);
        if (li < G) {
            cq = a.scale_log2e * up;
            if (FP8) {
                cq *= 256.0f * a.ks[(int64_t)b * a.Hkv + h];  // 2^8 rebias of the fp16 view of e4m3
            } else {
                cinit = -1152.0f * qsum;
            }
        }
    }
    while (step < nsteps) {
        const int n1 = step + kWavesPerWg;
        if (n1 < nsteps) load_stage(sb, it, n1);
        compute_stage(sa, step);
        if (n1 >= nsteps) break;
        const int n2 = n1 + kWavesPerWg;
        if (n2 < nsteps) load_stage(sa, it, n2);
        compute_stage(sb, n1);
        step = n2;
    }

    // ---- the next item's first tiles travel while this one is merged and written out
    if (kPreloadNext && has_next) {
        locate(next, wave);
        if (wave * kStep < next.t_end - next.t_begin) load_stage(sa, next, wave);
    }
    // ---- merge the four wavefronts through LDS
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (lq == 0) {
        sm_m[wave][li] = m_run;
        sm_l[wave][li] = l_run;
    }
    __syncthreads();
    float M = sm_m[0][li];
#pragma unroll
    for (int w = 1; w < kWavesPerWg; ++w) M = fmaxf(M, sm_m[w][li]);
    const float f = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_run - M);
    const int64_t prow = ((int64_t)b * a.Hq + h * G) * a.nchunks + chunk;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        if (c > 0) __syncthreads();  // the previous group has been read
        if (li < G) {
#pragma unroll
            for (int bb = 0; bb < NBB; ++bb)
#pragma unroll
                for (int r = 0; r < 4; ++r) sm_o[wave][li][4 * NBB * lq + NBB * r + bb] = acc[NBB * c + bb][r] * f;
        }
        __syncthreads();
        if (a.direct) {
            // single chunk: normalise and write the output, no workspace traffic
            for (int idx = threadIdx.x; idx < G * CW; idx += 256) {
                const int g = idx / CW, d = idx % CW;
                float o = 0.0f, l = 0.0f, Mg = sm_m[0][g];
#pragma unroll
                for (int w = 1; w < kWavesPerWg; ++w) Mg = fmaxf(Mg, sm_m[w][g]);
#pragma unroll
                for (int w = 0; w < kWavesPerWg; ++w) {
                    o += sm_o[w][g][d];
                    l += sm_m[w][g] == -INFINITY ? 0.0f : sm_l[w][g] * __builtin_amdgcn_exp2f(sm_m[w][g] - Mg);
                }
                const int64_t oi = ((int64_t)b * a.Hq + h * G + g) * kD + CW * c + d;
                a.out[oi] = (uint16_t)gated_bf16_bits(o * out_scale / l, a.out_gate, oi);
            }
        } else {
            for (int idx = threadIdx.x; idx < G * CW; idx += 256) {
                const int g = idx / CW, d = idx % CW;
                float o = 0.0f;
#pragma unroll
                for (int w = 0; w < kWavesPerWg; ++w) o += sm_o[w][g][d];
                a.part_o[(prow + (int64_t)g * a.nchunks) * kD + CW * c + d] = o * out_scale;
            }
        }
    }
    if (!a.direct && threadIdx.x < G) {
        const int g = threadIdx.x;
        float Mg = sm_m[0][g];
        for (int w = 1; w < kWavesPerWg; ++w) Mg = fmaxf(Mg, sm_m[w][g]);
        float l = 0.0f;
        for (int w = 0; w < kWavesPerWg; ++w)
            l += sm_m[w][g] == -INFINITY ? 0.0f : sm_l[w][g] * __builtin_amdgcn_exp2f(sm_m[w][g] - Mg);
        float *ml = a.part_ml + (prow + (int64_t)g * a.nchunks) * 2;
        ml[0] = Mg;
        ml[1] = l;
    }
    };  // run_item

    // Fixed chunks, grid (chunks, kv-heads, sequences): one item.  Workgroups go to the 8 XCDs round-robin by linear
    // id.  Low chunk indices always hold work, high ones only for long sequences, so the chunk index is rotated by
    // (head + sequence): every XCD then sees every index equally often instead of two XCDs getting all the first chunks.
    // Balanced, grid (pieces, kv-heads): the sequences of the batch are laid end to end in units of 64-token
    // granules; workgroup p owns granules [p W, (p+1) W) of that line, W = ceil(total / pieces), so every workgroup
    // streams the same number of bytes whatever the lengths are.  A range that crosses sequence ends holds several
    // items; a sequence cut by range ends leaves one partial per range, in slots counted from its first range.
    if constexpr (!BAL) {
        const int b = blockIdx.z;
        const int slot = (int)((blockIdx.x + blockIdx.y + blockIdx.z) % gridDim.x);
        const int L = min(a.seq_lens[b], a.max_seq_len);
        const int t_begin = slot * a.chunk_tokens;
        if (t_begin >= L) {
            if (slot == 0 && a.direct)  // a sequence without cached tokens: its output rows are zero
                for (int i = threadIdx.x; i < G * kD; i += 256) a.out[((int64_t)b * a.Hq + h * G) * kD + i] = 0;
            return;
        }
        const Item it = {b, L, t_begin, min(L, t_begin + a.chunk_tokens), slot};
        run_item(it, false, it, false);
    } else {
        __shared__ int sm_pref[kMaxBalancedB + 1];  // granules before sequence b
        if (wave == 0) {
            int running = 0;
            for (int b0 = 0; b0 < a.B; b0 += 64) {
                const int bb = b0 + lane;
                int g = bb < a.B ? (min(max(a.seq_lens[bb], 0), a.max_seq_len) + 63) >> 6 : 0;
#pragma unroll
                for (int o = 1; o < 64; o <<= 1) {  // inclusive scan over the lanes
                    const int up = __shfl_up(g, o, 64);
                    if (lane >= o) g += up;
                }
                if (bb < a.B) sm_pref[bb + 1] = running + g;
                running += __shfl(g, 63, 64);
            }
            if (lane == 0) sm_pref[0] = 0;
        }
        __syncthreads();
        // values read from LDS are the same in every lane; saying so keeps all that follows from them (addresses,
        // trip counts, block-table lookups) in scalar registers, as in the fixed-chunk instance
        auto uni = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
        const int total = uni(sm_pref[a.B]);
        const int W = max((total + a.pieces - 1) / a.pieces, a.min_granules);
        const int g_lo = blockIdx.x * W, g_hi = min(total, g_lo + W);
        if (g_lo >= g_hi) return;
        int lo = 0, hi = a.B - 1;  // first sequence that reaches into the range: smallest b with pref[b + 1] > g_lo
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (uni(sm_pref[mid + 1]) > g_lo) hi = mid; else lo = mid + 1;
        }
        // the item of the first non-empty sequence at or after b that reaches into the range (returns B: none); an
        // empty sequence is skipped, the merge kernel writes its zeros
        auto item_from = [&](int b, Item &it) {
            for (; b < a.B; ++b) {
                const int pb = uni(sm_pref[b]);
                if (pb >= g_hi) return a.B;
                if (uni(sm_pref[b + 1]) == pb) continue;
                const int L = min(a.seq_lens[b], a.max_seq_len);
                it = {b, L, max(g_lo - pb, 0) * 64, min(L, (g_hi - pb) * 64), (int)blockIdx.x - pb / W};
                return b;
            }
            return a.B;
        };
        Item cur = {0, 0, 0, 0, 0}, nxt = cur;
        int b = item_from(lo, cur);
        bool preloaded = false;
        while (b < a.B) {
            const int nb = item_from(b + 1, nxt);
            // the next item's first loads may go out early unless they could cover a token it has yet to write
            const bool ahead = kPreloadNext && nb < a.B &&
                               (a.nt.src[0] == nullptr || nxt.t_end != nxt.L || nxt.t_end - nxt.t_begin > kWavesPerWg * kStep);
            run_item(cur, preloaded, nxt, ahead);
            if (nb < a.B) __syncthreads();  // this item's merge buffers have been read
            preloaded = ahead;
            cur = nxt;
            b = nb;
        }
    }
}



// Merge the chunk partials of one (sequence, query head): out = sum_c 2^(m_c - M) o_c / sum_c 2^(m_c - M) l_c.
// 256 threads: D/4 column lanes (four output elements each) x 1024/D chunk lanes, so the partials of a long
// sequence (up to 128 chunks) are read by many lanes at once instead of one after the other; the chunk lanes meet
// in LDS.  D is 64, 128 or 256.
__global__ __launch_bounds__(256) void decode_merge_kernel(const float *part_o, const float *part_ml,
                                                          const int32_t *seq_lens, uint16_t *out, const uint16_t *out_gate, int Hq, int nchunks,
                                                          int chunk_tokens, int max_seq_len, int kD, int B, int pieces,
                                                          int min_granules) {
    const int hq = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int L = min(seq_lens[b], max_seq_len);
    __shared__ float sm_max[4], sm_l[16];
    __shared__ __attribute__((aligned(16))) float sm_o[1024];
    __shared__ int sm_cnt[2][4];
    int n;
    if (pieces > 0) {
        // balanced split: recompute where this sequence starts on the granule line and how wide a range is; its
        // partials sit in slots 0 .. (last range - first range)
        int before = 0, total = 0;
        for (int i = tid; i < B; i += 256) {
            const int g = (min(max(seq_lens[i], 0), max_seq_len) + 63) >> 6;
            total += g;
            if (i < b) before += g;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            total += __shfl_xor(total, o, 64);
            before += __shfl_xor(before, o, 64);
        }
        if ((tid & 63) == 0) {
            sm_cnt[0][tid >> 6] = total;
            sm_cnt[1][tid >> 6] = before;
        }
        __syncthreads();
        total = sm_cnt[0][0] + sm_cnt[0][1] + sm_cnt[0][2] + sm_cnt[0][3];
        before = sm_cnt[1][0] + sm_cnt[1][1] + sm_cnt[1][2] + sm_cnt[1][3];
        const int W = max((total + pieces - 1) / pieces, min_granules);
        const int g = (max(L, 0) + 63) >> 6;
        n = g == 0 ? 0 : min(nchunks, (before + g - 1) / W - before / W + 1);
    } else {
        n = L <= 0 ? 0 : min(nchunks, (L + chunk_tokens - 1) / chunk_tokens);
    }
    const int64_t row = ((int64_t)b * Hq + hq) * nchunks;
    float M = -INFINITY;
    for (int c = tid; c < n; c += 256) M = fmaxf(M, part_ml[(row + c) * 2]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o, 64));
    if ((tid & 63) == 0) sm_max[tid >> 6] = M;
    __syncthreads();
    M = fmaxf(fmaxf(sm_max[0], sm_max[1]), fmaxf(sm_max[2], sm_max[3]));
    const int cx = kD >> 2, tx = tid % cx, ty = tid / cx, ny = 256 / cx;
    float4v o = {0.f, 0.f, 0.f, 0.f};
    float l = 0.0f;
#pragma unroll 4
    for (int c = ty; c < n; c += ny) {
        const float m = part_ml[(row + c) * 2], lc = part_ml[(row + c) * 2 + 1];
        const float4v v = *(const float4v *)(part_o + (row + c) * kD + 4 * tx);
        const float w = __builtin_amdgcn_exp2f(m - M);
        l += w * lc;
        o += w * v;
    }
    *(float4v *)&sm_o[ty * kD + 4 * tx] = o;
    if (tx == 0) sm_l[ty] = l;
    __syncthreads();
    if (tid < kD) {
        float os = 0.0f, ls = 0.0f;
        for (int y = 0; y < ny; ++y) {
            os += sm_o[y * kD + tid];
            ls += sm_l[y];
        }
        const int64_t oi = ((int64_t)b * Hq + hq) * kD + tid;
        out[oi] = (uint16_t)gated_bf16_bits(n > 0 ? os / ls : 0.0f, out_gate, oi);
    }
}

// The balanced instances read their arguments anew from the kernel-argument segment, reinterpreted as DecodeArgs:
// that is only right while DecodeArgs is the kernel's sole parameter (it then starts at offset 0 of the segment) and
// is passed by value as plain bytes.
static_assert(std::is_trivially_copyable<DecodeArgs>::value, "DecodeArgs is read back as raw kernel-argument bytes");
static_assert(std::is_same<decltype(&decode_attn_kernel<128, false, false, true>), void (*)(DecodeArgs)>::value,
              "decode_attn_kernel must take DecodeArgs and nothing else");

int validate_layout(const hs_kv_layout *l, int B, int S, int Hkv, int D, bool need_scales);
int check_prologue(const hs_qk_prologue *p, int dtype, int D, bool need_q, bool need_k);
NormSpec norm_spec(const hs_qk_prologue *p, int which);

// Workgroups of a balanced launch: two resident on each of 256 CUs, one round.  Measured at B=64, lengths U[512, 8192]
// (us per step): 116 with 512, 139 with 640 and 768, 125 with 1024, 129 with 1536, 136 with 2048 -- a second, partial
// round costs more than the finer balance gains.
constexpr int kBalancedWorkgroups = 512;

struct Split {
    int chunk_tokens, nchunks;            // fixed-length chunks: grid (nchunks, Hkv, B)
    int balanced, pieces, min_granules;   // balanced token ranges: grid (pieces, Hkv), nchunks = partial slots per sequence
};

static Split pick_split(int B, int Hkv, int max_seq_len, int64_t total_tokens_hint) {
    Split s{};
    // A workgroup costs about 1.5 us of prologue/epilogue, so chunks are as long as the grid allows:
    // with >= 512 (sequence, kv-head) units (two resident workgroups on each of 256 CUs) nothing is
    // split and the step is a single launch; below that, split until about 512 workgroups exist -- one round of
    // resident workgroups.  Chunks are a multiple of 128 tokens (a whole number of wavefront steps at every
    // head_dim).  Measured on MI355X, whole step in us by chunks per sequence: 1 x 8 heads x 32768 tokens: 25.1 at
    // 128, 20.5 at 64, 20.8 at 32, 29.8 at 16; 4 x 8 x 16384: 39.7 at 64, 33.7 at 32, 30.7 at 16, 31.2 at 8;
    // 8 x 8 x 16384: 54.5 at 16, 52.9 at 8; 16 x 8 x 8192: 54.3 at 8, 53.8 at 4; 32 x 8 x 32768: the same at 2, 3 and 4;
    // 64 x 8 x 8192 (unsplit by the rule above): 193 unsplit, 196 in 2, 205 in 8.
    const int64_t units = (int64_t)B * Hkv;
    const int64_t want_chunks = units >= 512 ? 1 : (512 + units - 1) / units;
    int64_t ct = ((int64_t)max_seq_len + want_chunks - 1) / want_chunks;
    ct = (ct + 127) / 128 * 128;
    if (ct < 256) ct = 256;
    s.chunk_tokens = (int)ct;
    s.nchunks = (max_seq_len + s.chunk_tokens - 1) / s.chunk_tokens;
    // Ragged batch (the caller says how many tokens the batch holds in total, and the mean length is under 4/5 of
    // the longest): with fixed chunks the longest sequence sets the time of the launch while the workgroups of short
    // ones idle, and cutting finer pays a workgroup's start-up more often.  Instead every workgroup gets the same
    // number of 64-token granules of the batch laid end to end, whatever sequences they belong to.  A range is at
    // least 512 tokens and at least 1/16 of the longest sequence, which bounds the partials of one sequence at 17.
    if (total_tokens_hint > 0 && B > 0 && B <= kMaxBalancedB) {
        const int64_t mean = std::max<int64_t>(1, (total_tokens_hint + B - 1) / B);
        if (mean * 5 < (int64_t)max_seq_len * 4) {
            const int gmax = (max_seq_len + 63) / 64;
            s.balanced = 1;
            s.pieces = std::max(1, kBalancedWorkgroups / Hkv);
            s.min_granules = std::max(8, (gmax + 15) / 16);
            s.nchunks = (gmax + s.min_granules - 1) / s.min_granules + 1;
        }
    }
    return s;
}

// Most partial slots per sequence that a call with THIS max_seq_len or any smaller one can use, whatever its hint:
// a caller sizes its workspace once, for the capacity of its cache, and then calls with the length it has reached.
// pick_split's own slot count is not monotone in max_seq_len (chunks are rounded up to 128 tokens, so
// ceil(L / chunk_tokens) drops when L passes certain multiples), hence a bound and not pick_split's value:
// fixed chunks never exceed want_chunks nor ceil(L / 256) (a chunk is at least 256 tokens); balanced ranges never
// exceed ceil(g / 8) + 1 while a range is 8 granules (g <= 128 granules of 64 tokens) and 17 beyond.
static int max_slots(int B, int Hkv, int max_seq_len) {
    const int64_t units = (int64_t)B * Hkv;
    const int64_t want_chunks = units >= 512 ? 1 : (512 + units - 1) / units;
    const int64_t fixed = std::min<int64_t>(want_chunks, ((int64_t)max_seq_len + 255) / 256);
    const int gmax = (max_seq_len + 63) / 64;
    const int64_t balanced = B <= kMaxBalancedB ? (gmax <= 128 ? (gmax + 7) / 8 + 1 : 17) : 1;
    return (int)std::max<int64_t>(1, std::max(fixed, balanced));
}

struct NewToken {  // optional quantize-on-write of one token per sequence inside the same call
    const void *k_src = nullptr, *v_src = nullptr;  // [B, 1, Hkv, D]
    int dtype = HS_BF16;
    const void *rope_sin = nullptr, *rope_cos = nullptr;  // rotate q and k_new (bf16 tables [rope_len, rotary_dim/2])
    int rope_len = 0, rotary_dim = 0;                     // 0 = head_dim
    NormSpec qnorm, knorm;                                // QK-norm of q and k_new ahead of the rotation
    bool prologue = false;                                // the kernel instance with the q-side prologue
};

// static_scratch: the partials go to this device's copy of `scratch` (ws / ws_bytes ignored) and the size check is
// against what THIS call's split needs, not the worst case a caller-sized workspace has to cover.
static int launch_decode(bool fp8, int phases, const NewToken &nt, const void *q, void *kc, void *vc, float *ks,
                         float *vs, const hs_kv_layout *l, const int32_t *seq_lens, void *out, void *ws,
                         size_t ws_bytes, int B, int Hq, int Hkv, int D, int max_seq_len, float softmax_scale,
                         hipStream_t stream, bool static_scratch = false) {
    if (int rc = validate_layout(l, B, 0, Hkv, D, !fp8)) return rc;
    if (D != 64 && D != 128 && D != 256)
        return fail(HS_ERR_INVALID_ARGUMENT, "decode attention is built for head_dim 64, 128 and 256, got %d", D);
    if (B > 0 && (!q || !kc || !vc || !ks || !vs || !seq_lens || !out)) return fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if ((nt.k_src == nullptr) != (nt.v_src == nullptr)) return fail(HS_ERR_INVALID_ARGUMENT, "give k_new and v_new or neither");
    if (nt.k_src && nt.dtype != HS_BF16 && nt.dtype != HS_F32 && nt.dtype != HS_F16)
        return fail(HS_ERR_INVALID_ARGUMENT, "unknown src_dtype %d", nt.dtype);
    if (Hq <= 0 || Hq % Hkv != 0 || Hq / Hkv > 16)
        return fail(HS_ERR_INVALID_ARGUMENT, "need Hq %% Hkv == 0 and Hq/Hkv <= 16 (Hq=%d Hkv=%d)", Hq, Hkv);
    if (max_seq_len <= 0) return fail(HS_ERR_INVALID_ARGUMENT, "max_seq_len must be positive");
    if (l->k_block_table && (l->capacity_tokens % (D == 64 ? 64 : 32)) != 0)  // a wavefront step stays inside one block
        return fail(HS_ERR_INVALID_ARGUMENT, "paged blocks must hold a multiple of %d tokens", D == 64 ? 64 : 32);
    if (B == 0) return HS_OK;
    {
        const int64_t cap = l->k_block_table ? (int64_t)l->capacity_tokens * l->block_table_stride : l->capacity_tokens;
        if (max_seq_len > cap)
            return fail(HS_ERR_OVERFLOW, "max_seq_len %d exceeds what the cache can hold (%lld tokens)", max_seq_len,
                        (long long)cap);
    }
    DecodeArgs a;
    const Split sp = pick_split(B, Hkv, max_seq_len, l->total_tokens_hint);
    a.chunk_tokens = sp.chunk_tokens; a.nchunks = sp.nchunks;
    a.balanced = sp.balanced; a.pieces = sp.pieces; a.min_granules = sp.min_granules;
    if (static_scratch) {
        const size_t need = a.nchunks == 1 ? 0 : (size_t)B * Hq * a.nchunks * ((size_t)D + 2) * sizeof(float);
        if (need > kScratchBytes)
            return fail(HS_ERR_WORKSPACE,
                        "this shape needs %zu bytes of split-K scratch (%d chunks per sequence), the built-in scratch "
                        "holds %zu: use hs_decode_attn_int8 with a caller workspace", need, a.nchunks, kScratchBytes);
        if (int rc = scratch_of_current_device(&ws)) return rc;
        if (need > 0)
            if (int rc = claim_scratch(stream)) return rc;
    } else {
        const size_t need = hs_decode_attn_workspace_bytes(B, Hq, Hkv, D, max_seq_len);
        if (!ws || ws_bytes < need)
            return fail(HS_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed", ws_bytes, need);
        if (((uintptr_t)ws & 255) != 0) return fail(HS_ERR_INVALID_ARGUMENT, "workspace must be 256-byte aligned");
    }
    a.q = (const uint16_t *)q;
    a.kc = (const uint8_t *)kc; a.vc = (const uint8_t *)vc;
    a.ks = ks; a.vs = vs;
    a.ka = make_addr(*l, 0); a.va = make_addr(*l, 1);
    a.seq_lens = seq_lens;
    a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.G = Hq / Hkv; a.max_seq_len = max_seq_len;
    a.part_o = (float *)ws;
    a.part_ml = a.part_o + (size_t)B * Hq * a.nchunks * D;
    a.out = (uint16_t *)out;
    a.out_gate = (const uint16_t *)l->out_gate;
    a.scale_log2e = softmax_scale * kLog2e;
    a.direct = (phases == 3 && a.nchunks == 1) ? 1 : 0;
    a.nt.src[0] = nt.k_src; a.nt.src[1] = nt.v_src;
    a.nt.codes[0] = kc; a.nt.codes[1] = vc;
    a.nt.scales[0] = ks; a.nt.scales[1] = vs;
    a.nt.addr[0] = a.ka; a.nt.addr[1] = a.va;
    a.nt.positions = seq_lens; a.nt.start_pos = -1;  // the new token is the last cached one
    a.nt.B = B; a.nt.S = 1; a.nt.Hkv = Hkv; a.nt.D = D; a.nt.dtype = nt.dtype;
    if (nt.rope_sin) {
        if (!nt.rope_cos || nt.rope_len <= 0) return fail(HS_ERR_INVALID_ARGUMENT, "bad rotary tables");
        if (!nt.k_src || nt.dtype != HS_BF16)
            return fail(HS_ERR_INVALID_ARGUMENT, "the rotary decode step takes a bf16 new token");
    }
    const int rd = nt.rotary_dim > 0 ? nt.rotary_dim : D;
    if (nt.rope_sin && (rd <= 0 || rd > D || (rd % 16) != 0))
        return fail(HS_ERR_INVALID_ARGUMENT, "rotary_dim %d must be a multiple of 16 in (0, head_dim %d]", rd, D);
    if ((nt.qnorm.kind != 0 || nt.knorm.kind != 0) && (!nt.k_src || nt.dtype != HS_BF16))
        return fail(HS_ERR_INVALID_ARGUMENT, "the decode step with a QK-norm takes a bf16 new token");
    a.nt.rope_sin = nt.rope_sin; a.nt.rope_cos = nt.rope_cos; a.nt.rope_len = nt.rope_len; a.nt.rotary_dim = rd;
    a.nt.norm = nt.knorm;
    a.rope_sin = (const uint16_t *)nt.rope_sin; a.rope_cos = (const uint16_t *)nt.rope_cos; a.rope_len = nt.rope_len;
    a.rotary_dim = rd;
    a.qnorm = nt.qnorm;
    const bool pro = nt.prologue || a.rope_sin != nullptr;
    // the fused prologue reads the norm weights and the rotary tables with 16-byte loads
    for (const void *p : {(const void *)a.rope_sin, (const void *)a.rope_cos, (const void *)nt.qnorm.weight,
                          (const void *)nt.knorm.weight})
        if (((uintptr_t)p & 15) != 0)
            return fail(HS_ERR_INVALID_ARGUMENT,
                        "the fused decode step needs 16-byte aligned norm weights and rotary tables: run "
                        "hs_qk_prologue_apply (which takes any alignment) and hs_decode_step_* instead");
    if (phases & 1) {
        const dim3 grid = a.balanced ? dim3(a.pieces, Hkv, 1) : dim3(a.nchunks, Hkv, B);
#define HS_DECODE_LAUNCH(DD, BAL)                                                                      \
    do {                                                                                               \
        if (fp8 && pro) decode_attn_kernel<DD, true, true, BAL><<<grid, 256, 0, stream>>>(a);          \
        else if (fp8) decode_attn_kernel<DD, true, false, BAL><<<grid, 256, 0, stream>>>(a);           \
        else if (pro) decode_attn_kernel<DD, false, true, BAL><<<grid, 256, 0, stream>>>(a);           \
        else decode_attn_kernel<DD, false, false, BAL><<<grid, 256, 0, stream>>>(a);                   \
    } while (0)
        if (a.balanced) {
            if (D == 64) HS_DECODE_LAUNCH(64, true);
            else if (D == 128) HS_DECODE_LAUNCH(128, true);
            else HS_DECODE_LAUNCH(256, true);
        } else {
            if (D == 64) HS_DECODE_LAUNCH(64, false);
            else if (D == 128) HS_DECODE_LAUNCH(128, false);
            else HS_DECODE_LAUNCH(256, false);
        }
#undef HS_DECODE_LAUNCH
        if (int rc = check_launch("decode_attn")) return rc;
    }
    if ((phases & 2) && !a.direct) {
        decode_merge_kernel<<<dim3(Hq, B), 256, 0, stream>>>(a.part_o, a.part_ml, seq_lens, (uint16_t *)out, a.out_gate, Hq,
                                                               a.nchunks, a.chunk_tokens, max_seq_len, D, B,
                                                               a.balanced ? a.pieces : 0, a.min_granules);
        return check_launch("decode_merge");
    }
    return HS_OK;
}

}  // namespace hs

extern "C" {

size_t hs_decode_attn_workspace_bytes(int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len) {
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || max_seq_len <= 0) return 0;
    // room for the most partial slots per sequence any hint can lead to
    const size_t nchunks = (size_t)hs::max_slots(B, Hkv, max_seq_len);
    const size_t n = (size_t)B * Hq * nchunks * ((size_t)D + 2) * sizeof(float);
    return (n + 255) / 256 * 256;
}

int32_t hs_decode_attn_num_chunks(int32_t B, int32_t Hkv, int32_t max_seq_len, int64_t total_tokens_hint) {
    if (B <= 0 || Hkv <= 0 || max_seq_len <= 0) return 0;
    return hs::pick_split(B, Hkv, max_seq_len, total_tokens_hint).nchunks;
}

int hs_decode_attn_int8(const void *q, const int8_t *k_codes, const int8_t *v_codes, const float *k_scales,
                        const float *v_scales, const hs_kv_layout *layout, const int32_t *seq_lens, void *out,
                        void *workspace, size_t workspace_bytes, int32_t B, int32_t Hq, int32_t Hkv, int32_t D,
                        int32_t max_seq_len, float softmax_scale, hs_stream_t stream) {
    return hs::launch_decode(false, 3, hs::NewToken(), q, (void *)k_codes, (void *)v_codes, (float *)k_scales,
                             (float *)v_scales, layout, seq_lens, out, workspace, workspace_bytes, B, Hq, Hkv, D,
                             max_seq_len, softmax_scale, (hipStream_t)stream);
}

int hs_decode_attn_int8_static(const void *q, const int8_t *k_codes, const int8_t *v_codes, const float *k_scales,
                               const float *v_scales, const hs_kv_layout *layout, const int32_t *seq_lens, void *out,
                               int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len, float softmax_scale,
                               hs_stream_t stream) {
    return hs::launch_decode(false, 3, hs::NewToken(), q, (void *)k_codes, (void *)v_codes, (float *)k_scales,
                             (float *)v_scales, layout, seq_lens, out, nullptr, 0, B, Hq, Hkv, D, max_seq_len,
                             softmax_scale, (hipStream_t)stream, /*static_scratch=*/true);
}

int hs_decode_attn_fp8(const void *q, const uint8_t *k_codes, const uint8_t *v_codes, const float *k_scales,
                       const float *v_scales, const hs_kv_layout *layout, const int32_t *seq_lens, void *out,
                       void *workspace, size_t workspace_bytes, int32_t B, int32_t Hq, int32_t Hkv, int32_t D,
                       int32_t max_seq_len, float softmax_scale, hs_stream_t stream) {
    return hs::launch_decode(true, 3, hs::NewToken(), q, (void *)k_codes, (void *)v_codes, (float *)k_scales,
                             (float *)v_scales, layout, seq_lens, out, workspace, workspace_bytes, B, Hq, Hkv, D,
                             max_seq_len, softmax_scale, (hipStream_t)stream);
}

int hs_decode_step_int8(const void *q, const void *k_new, const void *v_new, int src_dtype, int8_t *k_codes,
                        int8_t *v_codes, float *k_scales, float *v_scales, const hs_kv_layout *layout,
                        const int32_t *seq_lens, void *out, void *workspace, size_t workspace_bytes, int32_t B,
                        int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len, float softmax_scale,
                        hs_stream_t stream) {
    if (!k_new || !v_new) return hs::fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    hs::NewToken nt;
    nt.k_src = k_new; nt.v_src = v_new; nt.dtype = src_dtype;
    return hs::launch_decode(false, 3, nt, q, k_codes, v_codes, k_scales, v_scales, layout, seq_lens, out, workspace,
                             workspace_bytes, B, Hq, Hkv, D, max_seq_len, softmax_scale, (hipStream_t)stream);
}

int hs_decode_step_int8_rope(const void *q, const void *k_new, const void *v_new, const void *rope_sin,
                             const void *rope_cos, int32_t rope_len, int8_t *k_codes, int8_t *v_codes, float *k_scales,
                             float *v_scales, const hs_kv_layout *layout, const int32_t *seq_lens, void *out,
                             void *workspace, size_t workspace_bytes, int32_t B, int32_t Hq, int32_t Hkv, int32_t D,
                             int32_t max_seq_len, float softmax_scale, hs_stream_t stream) {
    if (!k_new || !v_new || !rope_sin || !rope_cos) return hs::fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    hs::NewToken nt;
    nt.k_src = k_new; nt.v_src = v_new; nt.dtype = HS_BF16;
    nt.rope_sin = rope_sin; nt.rope_cos = rope_cos; nt.rope_len = rope_len;
    return hs::launch_decode(false, 3, nt, q, k_codes, v_codes, k_scales, v_scales, layout, seq_lens, out, workspace,
                             workspace_bytes, B, Hq, Hkv, D, max_seq_len, softmax_scale, (hipStream_t)stream);
}

int hs_decode_step_int8_prologue(const void *q, const void *k_new, const void *v_new, const hs_qk_prologue *prologue,
                                 int8_t *k_codes, int8_t *v_codes, float *k_scales, float *v_scales,
                                 const hs_kv_layout *layout, const int32_t *seq_lens, void *out, void *workspace,
                                 size_t workspace_bytes, int32_t B, int32_t Hq, int32_t Hkv, int32_t D,
                                 int32_t max_seq_len, float softmax_scale, hs_stream_t stream) {
    if (!k_new || !v_new) return hs::fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (int rc = hs::check_prologue(prologue, HS_BF16, D, true, true)) return rc;
    hs::NewToken nt;
    nt.k_src = k_new; nt.v_src = v_new; nt.dtype = HS_BF16;
    nt.rope_sin = prologue->rope_sin; nt.rope_cos = prologue->rope_cos; nt.rope_len = prologue->rope_len;
    nt.rotary_dim = prologue->rotary_dim;
    nt.qnorm = hs::norm_spec(prologue, 0); nt.knorm = hs::norm_spec(prologue, 1);
    nt.prologue = true;
    return hs::launch_decode(false, 3, nt, q, k_codes, v_codes, k_scales, v_scales, layout, seq_lens, out, workspace,
                             workspace_bytes, B, Hq, Hkv, D, max_seq_len, softmax_scale, (hipStream_t)stream);
}

int hs_decode_step_fp8_prologue(const void *q, const void *k_new, const void *v_new, const hs_qk_prologue *prologue,
                                uint8_t *k_codes, uint8_t *v_codes, const float *k_scales, const float *v_scales,
                                const hs_kv_layout *layout, const int32_t *seq_lens, void *out, void *workspace,
                                size_t workspace_bytes, int32_t B, int32_t Hq, int32_t Hkv, int32_t D,
                                int32_t max_seq_len, float softmax_scale, hs_stream_t stream) {
    if (!k_new || !v_new) return hs::fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    if (int rc = hs::check_prologue(prologue, HS_BF16, D, true, true)) return rc;
    hs::NewToken nt;
    nt.k_src = k_new; nt.v_src = v_new; nt.dtype = HS_BF16;
    nt.rope_sin = prologue->rope_sin; nt.rope_cos = prologue->rope_cos; nt.rope_len = prologue->rope_len;
    nt.rotary_dim = prologue->rotary_dim;
    nt.qnorm = hs::norm_spec(prologue, 0); nt.knorm = hs::norm_spec(prologue, 1);
    nt.prologue = true;
    return hs::launch_decode(true, 3, nt, q, k_codes, v_codes, (float *)k_scales, (float *)v_scales, layout, seq_lens, out,
                             workspace, workspace_bytes, B, Hq, Hkv, D, max_seq_len, softmax_scale, (hipStream_t)stream);
}

int hs_decode_step_fp8(const void *q, const void *k_new, const void *v_new, int src_dtype, uint8_t *k_codes,
                       uint8_t *v_codes, const float *k_scales, const float *v_scales, const hs_kv_layout *layout,
                       const int32_t *seq_lens, void *out, void *workspace, size_t workspace_bytes, int32_t B,
                       int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len, float softmax_scale,
                       hs_stream_t stream) {
    if (!k_new || !v_new) return hs::fail(HS_ERR_INVALID_ARGUMENT, "null buffer");
    hs::NewToken nt;
    nt.k_src = k_new; nt.v_src = v_new; nt.dtype = src_dtype;
    return hs::launch_decode(true, 3, nt, q, k_codes, v_codes, (float *)k_scales, (float *)v_scales, layout, seq_lens,
                             out, workspace, workspace_bytes, B, Hq, Hkv, D, max_seq_len, softmax_scale,
                             (hipStream_t)stream);
}

int hs_decode_attn_phases(int fmt_fp8, int phases, const void *q, const void *k_codes, const void *v_codes,
                          const float *k_scales, const float *v_scales, const hs_kv_layout *layout,
                          const int32_t *seq_lens, void *out, void *workspace, size_t workspace_bytes, int32_t B,
                          int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len, float softmax_scale,
                          hs_stream_t stream) {
    if (phases < 1 || phases > 3) return hs::fail(HS_ERR_INVALID_ARGUMENT, "phases must be 1, 2 or 3");
    return hs::launch_decode(fmt_fp8 != 0, phases, hs::NewToken(), q, (void *)k_codes, (void *)v_codes,
                             (float *)k_scales, (float *)v_scales, layout, seq_lens, out, workspace, workspace_bytes,
                             B, Hq, Hkv, D, max_seq_len, softmax_scale, (hipStream_t)stream);
}

}  // extern "C"
