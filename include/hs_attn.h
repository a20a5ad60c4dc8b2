/*
 * hs_attn.h -- C ABI of libhs_attn.so: hyprstream's attention hot path over a
 * quantized KV cache, hand-written for AMD MI355X (gfx950).
 *
 * Shape of the interface.  It follows the reference's only native boundary,
 * crates/bitsandbytes-sys (crates/bitsandbytes-sys/src/bindings.rs:15-334):
 * extern "C", raw device pointers, integer sizes, a trailing stream handle
 * (bindings.rs:13 `bnb_stream_t`), the CALLER allocates every buffer and the
 * library keeps no pointer and no state between calls
 * (crates/hyprstream/src/runtime/kv_cache.rs:797-865, 915-957); the one exception
 * is hs_decode_attn_int8_static, whose split-K scratch is an array inside the library.  Two deliberate
 * differences from that precedent: every entry point returns an int status
 * (0 = HS_OK) with the message available from hs_attn_last_error(), because
 * the bitsandbytes symbols return void and cannot report a bad launch; and
 * element counts that can exceed 2^31 are int64_t (bindings.rs uses c_int).
 *
 * Notation: B sequences, S new tokens in this call, T cached tokens,
 * Hq query heads, Hkv key/value heads (Hq % Hkv == 0, q-head h reads kv-head
 * h / (Hq/Hkv): architectures/llama.rs:847-872), D head_dim.
 *
 * Cache layout in device memory (buffers allocated by the caller):
 *   codes   one byte per element, head-major inside a sequence:
 *           code(b, h, t, d) at  codes + b*code_stride_seq + h*code_stride_head + t*D + d
 *   int8 scales  fp32, one per (token, kv-head):
 *           scale(b, h, t)   at  scales + b*scale_stride_seq + h*scale_stride_head + t
 *   fp8 scales   fp32 [B, Hkv], one per (sequence, kv-head)
 * With block tables (paged mode, the reference's BlockPool of fixed-size token
 * blocks, kv_cache.rs:477-693) "b" above is replaced by the block id found at
 * table[b*block_table_stride + t / capacity_tokens] and t by t % capacity_tokens.
 * Decode attention reads a block in whole wavefront steps: capacity_tokens of a paged layout is a
 * multiple of 32 there (of 64 at D = 64); the reference's 256-token blocks satisfy both.
 * A dense [B, T, Hkv, D] tensor, as LayerKVCache::get returns it
 * (kv_cache.rs:1499-1643), is produced on request by hs_kv_dequantize.
 *
 * Threading: every function is re-entrant; work is enqueued on `stream`
 * (NULL = the default stream, which is what tch/libtorch uses) of the caller's
 * current device and nothing synchronises with the host.
 */
#ifndef HS_ATTN_H
#define HS_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HS_ATTN_ABI_VERSION 8

typedef void *hs_stream_t; /* hipStream_t */

#if defined(__GNUC__)
#define HS_API __attribute__((visibility("default")))
#else
#define HS_API
#endif

enum hs_status {
    HS_OK = 0,
    HS_ERR_INVALID_ARGUMENT = 1, /* null pointer, bad shape, unsupported head_dim, misaligned stride */
    HS_ERR_OVERFLOW = 2,         /* write past capacity_tokens (kv_cache.rs:1288-1294 "Cache overflow") */
    HS_ERR_WORKSPACE = 3,        /* workspace too small */
    HS_ERR_LAUNCH = 4,           /* hipGetLastError() after the launch */
    HS_ERR_POOL_EXHAUSTED = 5,   /* host-side block pool has no free block (fail-soft, hs_kv_cache.h) */
    HS_ERR_BUSY = 6              /* hs_decode_attn_int8_static: the GPU's built-in scratch is in use on another stream */
};

enum hs_dtype { HS_BF16 = 0, HS_F32 = 1, HS_F16 = 2 };

struct hs_qk_prologue;

typedef struct hs_kv_layout {
    int64_t code_stride_seq;    /* bytes between sequences (or blocks when paged) */
    int64_t code_stride_head;   /* bytes between kv-heads inside a sequence/block; >= capacity_tokens*D, multiple of 16 */
    int64_t scale_stride_seq;   /* fp32 elements between sequences (or blocks); int8 format only */
    int64_t scale_stride_head;  /* fp32 elements between kv-heads; >= capacity_tokens, multiple of 4 */
    int32_t capacity_tokens;    /* tokens one sequence (or one block) can hold */
    int32_t block_table_stride; /* entries per sequence in the block tables; 0 = not paged */
    const int32_t *k_block_table; /* device, [B, block_table_stride]; NULL = not paged */
    const int32_t *v_block_table; /* device, may equal k_block_table when K and V pools are separate buffers */
    int64_t total_tokens_hint;  /* decode only, optional: sum of seq_lens over the batch as the host knows it
                                   (0 = unknown).  A ragged batch is then cut into equal token ranges over all
                                   sequences (the lengths themselves are read on the device), so that long
                                   sequences do not set the time of the launch. */
    int32_t prefill_columns_hint; /* prefill only, optional: 0 = the library picks the (query, head) columns a
                                   workgroup owns from the size of the grid; 256 or 128 fixes them, 32 asks for 256
                                   columns on 32x32 MFMA tiles, 16 for 256 columns on sixteen wavefronts of at most
                                   128 registers (both: head_dim 128 without a window; elsewhere the same as 256;
                                   measured variants the library never picks by itself).  Results are the same
                                   within rounding every way; head_dim 256 always uses its one width. */
    int32_t prefill_window;     /* prefill only, optional: sliding window of local-attention layers (Gemma3 / Mistral;
                                   apply_sliding_window_mask, llama.rs:1086-1091, 1123-1155): a query at absolute
                                   position p attends the keys in (p - window, p].  0 = no window.  For a prompt on an
                                   empty cache this is the reference's mask; with history it is the same rule on
                                   absolute positions (the reference's [q_len, q_len] mask has no meaning there).
                                   Decode entry points ignore it, as the reference applies no window at q_len == 1. */
    const void *out_gate;       /* attention calls, optional: bf16, device, the shape of `out`.  The output gate of the
                                   Qwen3.5 full-attention layers (qwen3_5.rs:1056-1059: ctx * sigmoid(gate) in the model
                                   dtype): out = bf16(bf16(attention) * bf16(sigmoid(gate))) written by the same launch.
                                   NULL = none. */
    const struct hs_qk_prologue *prefill_q_prologue;
                                /* prefill only, optional: q arrives AS PROJECTED and the launch runs the q side of the
                                   prologue below on it (QK-norm with q_norm_weight, then the rotary embedding at
                                   position hist_len + s), the bits hs_qk_prologue_apply writes; only q: k_new must
                                   arrive normalised and rotated (hs_qk_prologue_apply with q = NULL over the prompt's
                                   K).  Rotated parts served: rotary_dim = head_dim, head_dim / 2 or head_dim / 4,
                                   anything else is HS_ERR_INVALID_ARGUMENT (run the pre-pass on q as well); weights and
                                   tables 16-byte aligned.  NULL = q arrives ready. */
    void *prefill_split_workspace;
    int64_t prefill_split_workspace_bytes;
    int32_t prefill_key_splits;
    int32_t reserved0;          /* prefill only, optional: device scratch that lets a call whose query tiles are too few
                                   to occupy the GPU (a chunk of ONE sequence: 64 tiles on 256 compute units) cut the
                                   keys of every tile into runs for several workgroups, the last of which to finish
                                   merges the partial results.  At least hs_prefill_attn_split_workspace_bytes(...)
                                   bytes, 256-byte aligned, prepared once by hs_prefill_attn_split_workspace_init and
                                   left ready by every call; calls that overlap in time need workspaces of their own.
                                   NULL = never split.  prefill_key_splits: 0 = the library decides whether and how
                                   far to split, 1 = never, 2..8 = this many runs (tests, measurements; a call of
                                   more than 4096 query tiles has no counters to be split with and is
                                   HS_ERR_INVALID_ARGUMENT).  A workspace that is too small for the call is
                                   HS_ERR_WORKSPACE.  The first 16 KB of the workspace hold the tiles' arrival
                                   counters, zero between calls; calls of any shape and width may share a workspace
                                   one after the other.  Outputs agree with the unsplit launch within the rounding of
                                   a different summation order; the cache rows written are the same bits.  Not
                                   combined with a window or a width hint of 32 or 16 (those calls run unsplit). */
    void *prefill_shadow;
    int64_t prefill_shadow_bytes;
    int32_t prefill_shadow_tokens;
    int32_t reserved1;          /* prefill only, optional, head_dim 128 (int8 or fp8 cache): a bf16 copy of the prompt's
                                   DEQUANTIZED K/V (code * scale, the values the reference's get() hands to its
                                   attention, kv_cache.rs:1493-1560) in the order the matrix instructions take them,
                                   kept by the caller for as long as one prompt is being prefilled into one layer's
                                   cache.  Every prefill call with quantize_on_write = 1 appends its tokens to it; a
                                   call with history reads the history from it instead of converting the cached codes
                                   in every workgroup that needs them (-15 % per history step at 4 x 512 queries).  The
                                   int8 cache is written as always and stays the cache; the copy may be dropped after
                                   the prompt.  Contract: hs_prefill_shadow_bytes(B, Hkv, D, prefill_shadow_tokens)
                                   bytes, 256-byte aligned, cleared once by hs_prefill_shadow_init; prefill_shadow_tokens
                                   a multiple of 64 and >= hist_len + S; every token below hist_len must have been
                                   appended by earlier prefill calls with the same copy and the same B, Hkv (tokens
                                   written by decode steps or by hs_kv_quantize_* are not in it: leave the field NULL
                                   for such calls).  NULL = none.  Calls that cannot read it (a window, rows at different
                                   positions, the 32 and 16 width hints) still append; a call WITH history at another
                                   head_dim is refused rather than leaving a hole. */
} hs_kv_layout;

/* Message of the last failing call on this thread ("" if none). */
HS_API const char *hs_attn_last_error(void);
HS_API int hs_attn_abi_version(void);

/* ---- quantize-on-write (replaces the buffer + flush + requantize-everything scheme of
 * LayerKVCache::update / flush_buffer, kv_cache.rs:1275-1432, 1204-1272, and the
 * cquantize_blockwise_* calls at kv_cache.rs:823-840) ------------------------------------
 * k_src, v_src: [B, S, Hkv, D] contiguous, dtype src_dtype (K already rotated: the cache
 * holds post-RoPE keys, llama.rs:598-611).  Token s of sequence b goes to position
 * (positions ? positions[b] : 0) + start_pos + s.  `positions` is a device array of B ints.
 * int8: per (token, kv-head) row  s = max|x| / 127 (fp32), code = clamp(rint(x / s), +-127),
 * all-zero row -> s = 0, codes 0.  Only the S new tokens are touched.
 * Errors: HS_ERR_OVERFLOW when positions == NULL and start_pos + S > capacity (not paged);
 * rows whose device-side position falls outside the capacity/table are skipped. */
HS_API int hs_kv_quantize_int8(const void *k_src, const void *v_src, int src_dtype,
                        int8_t *k_codes, int8_t *v_codes, float *k_scales, float *v_scales,
                        const hs_kv_layout *layout, const int32_t *positions, int32_t start_pos,
                        int32_t B, int32_t S, int32_t Hkv, int32_t D, hs_stream_t stream);

/* ---- rotary embedding fused into the write (RoPE::forward / apply_rotary_pos_emb, rope.rs:150-248, which
 * the reference runs on q and k right before cache.update, llama.rs:598-611, qwen3_5.rs:977-990) ----------
 * rope_sin, rope_cos: device tables [rope_len, D/2] in the tensor's dtype, row p = sin/cos(p * base^(-2i/D))
 * computed in fp32 and cast (rope.rs:100-122); built and kept by the caller, as the reference caches them.
 * Half-split convention: x1 = x[..., :D/2], x2 = x[..., D/2:];  x1' = x1*cos - x2*sin, x2' = x1*sin + x2*cos,
 * each product and sum rounded to the dtype like the separate libtorch ops they replace, so codes and scales
 * equal those of quantizing the reference's rotated K.  The table row of token (b, s) is its cache position
 * (positions ? positions[b] : 0) + start_pos + s, clamped to the table.
 * hs_kv_quantize_int8_rope: k_src arrives UNROTATED; V is written as it is.
 * hs_rope_apply: x, out [B, S, H, D] in `dtype` (the query side; out may equal x only if no other row reads it,
 * i.e. never: use a separate buffer). */
HS_API int hs_kv_quantize_int8_rope(const void *k_src, const void *v_src, int src_dtype,
                        const void *rope_sin, const void *rope_cos, int32_t rope_len,
                        int8_t *k_codes, int8_t *v_codes, float *k_scales, float *v_scales,
                        const hs_kv_layout *layout, const int32_t *positions, int32_t start_pos,
                        int32_t B, int32_t S, int32_t Hkv, int32_t D, hs_stream_t stream);
HS_API int hs_rope_apply(const void *x, int dtype, const void *rope_sin, const void *rope_cos, int32_t rope_len,
                        const int32_t *positions, int32_t start_pos, void *out,
                        int32_t B, int32_t S, int32_t H, int32_t D, hs_stream_t stream);
/* Partial rotary embedding (Qwen3.5: the first rotary_dim = head_dim/4 elements of each head are rotated, the
 * rest pass through; qwen3_5.rs:977-990 does narrow + rope + cat).  Tables are [rope_len, rotary_dim/2]; the
 * rotated pairs are (d, d + rotary_dim/2).  rotary_dim is a multiple of 16, at most D; == D is hs_rope_apply. */
HS_API int hs_rope_apply_partial(const void *x, int dtype, const void *rope_sin, const void *rope_cos, int32_t rope_len,
                        const int32_t *positions, int32_t start_pos, void *out,
                        int32_t B, int32_t S, int32_t H, int32_t D, int32_t rotary_dim, hs_stream_t stream);

/* ---- everything the reference runs on q and k between the projections and cache.update: per-head QK-norm, then the
 * rotary embedding (llama.rs:589-611: apply_qk_norm llama.rs:929-991, then apply_rope; qwen3_5.rs:973-990: apply_qknorm
 * qwen3_5.rs:1077-1091, then the partial rotary embedding) ----------------------------------------------------------
 * HS_QKNORM_LLAMA (Gemma3 and other Llama-architecture models with q_norm / k_norm): square, mean, + eps, reciprocal,
 *   sqrt, x * rrms, * weight as separate ops in the tensor dtype, each result rounded to it (the reference hard-codes
 *   eps = 1e-6 there); weights in the tensor dtype, [H, D] (head stride D) or one [D] vector (head stride 0).
 * HS_QKNORM_QWEN35: in fp32, rrms = 1 / sqrt(mean(x^2) + eps), out = (x * rrms) * (1 + weight), one cast back; fp32 weights.
 * The sum of squares is the correctly rounded fp32 sum of the row (libtorch's own summation order depends on the host).
 * rope_sin / rope_cos: tables [rope_len, rotary_dim / 2] in the tensor dtype as for hs_rope_apply_partial, NULL = no
 * rotation; rotary_dim 0 means head_dim.  Results equal those of the separate ops: the rotated rows are bit-exact
 * functions of the normalised rows, and codes written from them are those of hs_kv_quantize_int8. */
enum hs_qk_norm_kind { HS_QKNORM_NONE = 0, HS_QKNORM_LLAMA = 1, HS_QKNORM_QWEN35 = 2 };
typedef struct hs_qk_prologue {
    int32_t norm_kind;            /* enum hs_qk_norm_kind */
    float norm_eps;
    const void *q_norm_weight;    /* device; HS_QKNORM_LLAMA: tensor dtype, HS_QKNORM_QWEN35: fp32 */
    const void *k_norm_weight;
    int32_t q_norm_head_stride;   /* elements between the weight rows of consecutive heads: D, or 0 for one shared [D] */
    int32_t k_norm_head_stride;
    const void *rope_sin;         /* device, [rope_len, rotary_dim / 2]; NULL: no rotation */
    const void *rope_cos;
    int32_t rope_len;
    int32_t rotary_dim;           /* leading elements of each head that are rotated; 0 = head_dim */
} hs_qk_prologue;
/* q [B, S, Hq, D] -> q_out, k [B, S, Hkv, D] -> k_out in one launch (either pair may be NULL); token (b, s) takes table
 * row (positions ? positions[b] : 0) + start_pos + s.  The pre-pass of a prefill call: q_out and k_out are what
 * hs_prefill_attn_* expects (rotated q, rotated K for its own bf16 part and for quantize_on_write). */
HS_API int hs_qk_prologue_apply(const void *q, const void *k, int dtype, const hs_qk_prologue *prologue,
                        const int32_t *positions, int32_t start_pos, void *q_out, void *k_out,
                        int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D, hs_stream_t stream);
/* hs_kv_quantize_int8 with K normalised and rotated on the way in (k_src arrives as projected); V as it is. */
HS_API int hs_kv_quantize_int8_prologue(const void *k_src, const void *v_src, int src_dtype, const hs_qk_prologue *prologue,
                        int8_t *k_codes, int8_t *v_codes, float *k_scales, float *v_scales,
                        const hs_kv_layout *layout, const int32_t *positions, int32_t start_pos,
                        int32_t B, int32_t S, int32_t Hkv, int32_t D, hs_stream_t stream);

/* FP8 e4m3fn cache with one fp32 scale per (sequence, kv-head).  Calibration computes
 * scale[b, h] = max over (s, d) |x| / 448 from the tokens given (typically the prompt);
 * quantization stores e4m3fn(clamp(x / scale, +-448)), round-to-nearest-even. */
HS_API int hs_kv_fp8_calibrate(const void *k_src, const void *v_src, int src_dtype,
                        float *k_scales, float *v_scales,
                        int32_t B, int32_t S, int32_t Hkv, int32_t D, hs_stream_t stream);
HS_API int hs_kv_quantize_fp8(const void *k_src, const void *v_src, int src_dtype,
                       uint8_t *k_codes, uint8_t *v_codes, const float *k_scales, const float *v_scales,
                       const hs_kv_layout *layout, const int32_t *positions, int32_t start_pos,
                       int32_t B, int32_t S, int32_t Hkv, int32_t D, hs_stream_t stream);

/* ---- dense view (what LayerKVCache::get materialises, kv_cache.rs:1517-1580; replaces
 * cdequantize_blockwise_*, bindings.rs:47-75).  Not on the attention path: the attention
 * kernels read codes directly.  out: [B, T, Hkv, D] in out_dtype; which_table 0 = K table,
 * 1 = V table (paged only).  fmt_fp8 0: int8 codes + per-token scales; 1: e4m3fn + per-head. */
HS_API int hs_kv_dequantize(const void *codes, const float *scales, int fmt_fp8, const hs_kv_layout *layout,
                     int which_table, void *out, int out_dtype,
                     int32_t B, int32_t T, int32_t Hkv, int32_t D, hs_stream_t stream);

/* ---- decode attention (replaces get() + GQA expand + compute_attention_masked for q_len == 1:
 * llama.rs:605-636, 1023-1119; qwen3_5.rs:993-1053; ragged rows as in forward_batched,
 * llama.rs:710-844, 2544-2572) ---------------------------------------------------------------
 * q, out: [B, Hq, D] bf16.  seq_lens: device [B], cached tokens per sequence INCLUDING the
 * one just written; rows with seq_len <= 0 produce zeros.  max_seq_len >= every seq_lens[b]
 * (host-side bound used to size the grid).  out = softmax(q K^T * softmax_scale) V with
 * fp32 accumulation, K/V dequantized on the fly.  D is 64, 128 or 256 (Hq/Hkv <= 16); anything
 * else is HS_ERR_INVALID_ARGUMENT.  workspace: device scratch of at least
 * hs_decode_attn_workspace_bytes(...) bytes, 256-byte aligned, owned by the caller. */
HS_API size_t hs_decode_attn_workspace_bytes(int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len);
/* Partials per sequence the decode entry points will keep for this shape and hint (1 = a step is a single launch
 * and no workspace is touched).  Without a hint: fixed-length chunks.  With a hint that marks the batch ragged
 * (mean length under 4/5 of max_seq_len, B <= 1024): the batch is cut into equal token ranges over all sequences and
 * the value is the most ranges one sequence can span (at most 17). */
HS_API int32_t hs_decode_attn_num_chunks(int32_t B, int32_t Hkv, int32_t max_seq_len, int64_t total_tokens_hint);
HS_API int hs_decode_attn_int8(const void *q, const int8_t *k_codes, const int8_t *v_codes,
                        const float *k_scales, const float *v_scales, const hs_kv_layout *layout,
                        const int32_t *seq_lens, void *out, void *workspace, size_t workspace_bytes,
                        int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len,
                        float softmax_scale, hs_stream_t stream);
/* hs_decode_attn_int8 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): no workspace argument.  It has no counterpart in the reference.  The
 * split-K partials live in a 32 MiB array inside the library's device image (one copy per GPU the library runs on,
 * held until the process ends); the call allocates and frees nothing.  Same kernels and same results as
 * hs_decode_attn_int8.  A shape whose split needs more than 32 MiB of partials
 * (B * Hq * chunks * (D + 2) * 4 bytes, chunks = hs_decode_attn_num_chunks(...); nothing when chunks == 1) is refused
 * with HS_ERR_WORKSPACE.  The array keeps the previous call's partials; nothing in it has to start at zero, because the
 * merge reads only what the same call wrote.  All calls on one GPU share that GPU's array, so calls that could overlap
 * on one GPU are refused: a call whose split uses the array, on a stream other than the one the previous such call on
 * this GPU was given, returns HS_ERR_BUSY (nothing launched) while that previous stream still has work pending
 * (hipStreamQuery; the legacy default stream and a blocking stream order each other and count as one).  Calls on one
 * stream follow each other and are always accepted.  What the guard cannot see: launches recorded under graph capture
 * run when the graph is replayed, so keep replays of graphs that hold this call and other users of the array on one
 * stream.  The array's address is looked up on the first call on each device (hipGetSymbolAddress, no allocation);
 * make that first call outside graph capture. */
HS_API int hs_decode_attn_int8_static(const void *q, const int8_t *k_codes, const int8_t *v_codes,
                        const float *k_scales, const float *v_scales, const hs_kv_layout *layout,
                        const int32_t *seq_lens, void *out,
                        int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len,
                        float softmax_scale, hs_stream_t stream);
HS_API int hs_decode_attn_fp8(const void *q, const uint8_t *k_codes, const uint8_t *v_codes,
                       const float *k_scales, const float *v_scales, const hs_kv_layout *layout,
                       const int32_t *seq_lens, void *out, void *workspace, size_t workspace_bytes,
                       int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len,
                       float softmax_scale, hs_stream_t stream);

/* One decode step in a single call: quantize-on-write of ONE new token per sequence (k_new, v_new:
 * [B, 1, Hkv, D] in src_dtype, written at position seq_lens[b] - 1, i.e. seq_lens already counts it)
 * followed by decode attention over the seq_lens[b] cached tokens.  Same results as
 * hs_kv_quantize_* + hs_decode_attn_*; the write rides in the attention call's prologue kernel
 * (what LlamaAttention::forward does per layer: cache.update then cache.get then attention,
 * llama.rs:605-636). */
HS_API int hs_decode_step_int8(const void *q, const void *k_new, const void *v_new, int src_dtype,
                               int8_t *k_codes, int8_t *v_codes, float *k_scales, float *v_scales,
                               const hs_kv_layout *layout, const int32_t *seq_lens, void *out,
                               void *workspace, size_t workspace_bytes,
                               int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len,
                               float softmax_scale, hs_stream_t stream);
/* The same step with the rotary embedding of q and k_new done inside the kernel (the reference rotates both
 * right before cache.update, llama.rs:598-611): q [B, Hq, D] and k_new [B, 1, Hkv, D] arrive UNROTATED in
 * bf16, rope_sin / rope_cos are bf16 tables [rope_len, D/2] (see hs_rope_apply), the table row is the new
 * token's position seq_lens[b] - 1.  Results equal hs_rope_apply(q) + hs_kv_quantize_int8_rope + decode. */
HS_API int hs_decode_step_int8_rope(const void *q, const void *k_new, const void *v_new,
                               const void *rope_sin, const void *rope_cos, int32_t rope_len,
                               int8_t *k_codes, int8_t *v_codes, float *k_scales, float *v_scales,
                               const hs_kv_layout *layout, const int32_t *seq_lens, void *out,
                               void *workspace, size_t workspace_bytes,
                               int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len,
                               float softmax_scale, hs_stream_t stream);
/* The step with the whole prologue inside the launch: QK-norm of q and k_new, then their rotation (hs_qk_prologue above;
 * q [B, Hq, D], k_new [B, 1, Hkv, D], v_new in bf16 as projected; table row = seq_lens[b] - 1).  rotary_dim is any
 * multiple of 16 up to head_dim, as for hs_qk_prologue_apply (head_dim, 128, 64 and 32 pair their elements between the
 * lanes that hold them; other lengths read the partners from q again).  The norm weights and the rotary tables
 * must be 16-byte aligned here (the launch reads them 16 bytes at a time; hs_qk_prologue_apply takes any alignment),
 * else HS_ERR_INVALID_ARGUMENT.  Results equal those calls' bit for bit. */
HS_API int hs_decode_step_int8_prologue(const void *q, const void *k_new, const void *v_new, const hs_qk_prologue *prologue,
                               int8_t *k_codes, int8_t *v_codes, float *k_scales, float *v_scales,
                               const hs_kv_layout *layout, const int32_t *seq_lens, void *out,
                               void *workspace, size_t workspace_bytes,
                               int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len,
                               float softmax_scale, hs_stream_t stream);
HS_API int hs_decode_step_fp8(const void *q, const void *k_new, const void *v_new, int src_dtype,
                              uint8_t *k_codes, uint8_t *v_codes, const float *k_scales, const float *v_scales,
                              const hs_kv_layout *layout, const int32_t *seq_lens, void *out,
                              void *workspace, size_t workspace_bytes,
                              int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len,
                              float softmax_scale, hs_stream_t stream);
/* hs_decode_step_int8_prologue for the FP8 cache (qwen3_5.rs:1077-1091 + rope.rs:206-248 in front of
 * kv_cache.rs:459-497 with an FP8 cache): k_new is normalised and rotated, then encoded with the sequence's calibrated
 * scale; q is normalised and rotated on its way into the attention.  Same argument rules and served rotary_dim values as
 * the int8 call; results equal hs_qk_prologue_apply + hs_decode_step_fp8 bit for bit. */
HS_API int hs_decode_step_fp8_prologue(const void *q, const void *k_new, const void *v_new, const hs_qk_prologue *prologue,
                              uint8_t *k_codes, uint8_t *v_codes, const float *k_scales, const float *v_scales,
                              const hs_kv_layout *layout, const int32_t *seq_lens, void *out,
                              void *workspace, size_t workspace_bytes,
                              int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len,
                              float softmax_scale, hs_stream_t stream);

/* The two phases of split-K decode attention on their own: phases = 1 runs only the attention kernel
 * and leaves per-chunk partials (m, l, o) in the workspace, 2 only the merge of those partials into
 * `out`, 3 is identical to the calls above (which skip the workspace altogether when a sequence is a
 * single chunk).  No counterpart in the reference; it exists so that the phases can be timed
 * separately and so that partials produced for different token ranges (for instance on different
 * devices) can share one merge. */
HS_API int hs_decode_attn_phases(int fmt_fp8, int phases, const void *q, const void *k_codes, const void *v_codes,
                                 const float *k_scales, const float *v_scales, const hs_kv_layout *layout,
                                 const int32_t *seq_lens, void *out, void *workspace, size_t workspace_bytes,
                                 int32_t B, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_seq_len,
                                 float softmax_scale, hs_stream_t stream);

/* ---- causal prefill over [int8 history] + [this call's bf16 K/V] (replaces update + get +
 * compute_attention_masked for q_len > 1: llama.rs:1066-1112, mask rule "query row i sits at
 * absolute position (k_len - q_len) + i", llama.rs:1074-1084) --------------------------------
 * q: [B, S, Hq, D] bf16; k_new, v_new: [B, S, Hkv, D] bf16; out: [B, S, Hq, D] bf16.
 * hist_len tokens per sequence are already in the int8 cache; query row i attends the whole
 * history (dequantized) and new tokens 0..=i (exact bf16).  With quantize_on_write != 0 the S
 * new tokens are also written to the cache at positions hist_len .. hist_len+S-1.
 * D is 64, 128 or 256; Hq a multiple of Hkv (groups of 1, 2 or 4k query heads fill the workgroups, any
 * other group size pads its last group of four).  A paged layout needs capacity_tokens (tokens per block)
 * to be a multiple of 64 here.
 * Magnitudes: the cached history enters the matrix products as fp16(code * scale * 2^-E), E a power-of-two reference
 * per (sequence, kv-head) taken from the largest token scale among the first min(hist_len, 64) cached tokens (their
 * first block when paged; fp8: from the head scale), 2^E re-applied exactly.  Any overall magnitude of K and V is
 * therefore served with the same relative precision (2^-11 per operand).  Inside one (sequence, kv-head), a token
 * whose scale exceeds 2^11 times that reference saturates at 65024 * 2^E, and one below 2^-11 times it loses bits in
 * proportion (its contribution is then below 2^-22 of the head's typical row anyway).  Decode has no such window. */
HS_API int hs_prefill_attn_int8(const void *q, const void *k_new, const void *v_new,
                         int8_t *k_codes, int8_t *v_codes, float *k_scales, float *v_scales,
                         const hs_kv_layout *layout, int32_t hist_len, void *out,
                         int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D,
                         float softmax_scale, int quantize_on_write, hs_stream_t stream);
/* The same over an FP8 e4m3fn history with per-(sequence, kv-head) scales [B, Hkv] (read, never written: they
 * come from hs_kv_fp8_calibrate or from the model); quantize_on_write writes the codes hs_kv_quantize_fp8 would. */
HS_API int hs_prefill_attn_fp8(const void *q, const void *k_new, const void *v_new,
                        uint8_t *k_codes, uint8_t *v_codes, const float *k_scales, const float *v_scales,
                        const hs_kv_layout *layout, int32_t hist_len, void *out,
                        int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D,
                        float softmax_scale, int quantize_on_write, hs_stream_t stream);

/* The same for a batch whose rows sit at different positions (forward_batched with q_len > 1: every row brings
 * S new tokens at its own start position, llama.rs:710-844, mask rule llama.rs:2544-2572).  hist_lens: device [B],
 * cached tokens per sequence, each clamped to [0, max_hist_len]; max_hist_len is the host-side bound the capacity
 * check uses (max_hist_len + S must fit the cache when quantize_on_write != 0).  Row b attends its hist_lens[b]
 * cached tokens and its own new tokens causally, and writes them at hist_lens[b] .. hist_lens[b] + S - 1. */
HS_API int hs_prefill_attn_int8_ragged(const void *q, const void *k_new, const void *v_new,
                                int8_t *k_codes, int8_t *v_codes, float *k_scales, float *v_scales,
                                const hs_kv_layout *layout, const int32_t *hist_lens, int32_t max_hist_len,
                                void *out, int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D,
                                float softmax_scale, int quantize_on_write, hs_stream_t stream);
HS_API int hs_prefill_attn_fp8_ragged(const void *q, const void *k_new, const void *v_new,
                               uint8_t *k_codes, uint8_t *v_codes, const float *k_scales, const float *v_scales,
                               const hs_kv_layout *layout, const int32_t *hist_lens, int32_t max_hist_len,
                               void *out, int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D,
                               float softmax_scale, int quantize_on_write, hs_stream_t stream);

/* Scratch for the key split of small prefill calls (hs_kv_layout.prefill_split_workspace): bytes needed for calls of
 * at most B x S new tokens, whatever their history; _init zeroes the arrival counters (a small fill launch on
 * `stream`) and is needed once per allocation.  No counterpart in the reference, whose attention is one libtorch
 * matmul per call (llama.rs:1066-1112). */
HS_API size_t hs_prefill_attn_split_workspace_bytes(int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D);
HS_API int hs_prefill_attn_split_workspace_init(void *workspace, size_t bytes, hs_stream_t stream);

/* The bf16 operand-order copy of a prompt's K/V (hs_kv_layout.prefill_shadow): bytes for B sequences of max_tokens
 * tokens (rounded up to 64); _init clears it (a fill launch on `stream`), once per allocation and again whenever the
 * copy is reused for another prompt.  0 for a head_dim it does not serve.  No counterpart in the reference, which
 * materialises the whole dequantized cache on every get(). */
HS_API size_t hs_prefill_shadow_bytes(int32_t B, int32_t Hkv, int32_t D, int32_t max_tokens);
HS_API int hs_prefill_shadow_init(void *shadow, size_t bytes, hs_stream_t stream);

/* ---- gated delta rule (replaces the decode branch qwen3_5.rs:725-751 and
 * chunked_delta_rule qwen3_5.rs:342-498) -------------------------------------------------------
 * q, k: [B, T, nk, dk] bf16; v: [B, T, nv, dv] bf16; g, beta: [B, T, nv] fp32 (g = log decay <= 0);
 * state: [B, nv, dk, dv] fp32, updated in place; out: [B, T, nv, dv] fp32.
 * v-head j reads q/k-head j / (nv/nk) (qwen3_5.rs:704-720).  With l2norm != 0, q and k are first
 * replaced by x / max(||x||, 1e-3) (qwen3_5.rs:331-335); q is then multiplied by q_scale.
 * T == 1 is the decode step; T > 1 runs the same recurrence token by token with the state held
 * on chip.  Both entry points are built for dk = dv = 128 (the Qwen3.5 head size); any other size is
 * HS_ERR_INVALID_ARGUMENT, nothing is padded. */
HS_API int hs_deltanet_forward(const void *q, const void *k, const void *v, const float *g, const float *beta,
                        float *state, float *out,
                        int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk, int32_t dv,
                        float q_scale, int l2norm, hs_stream_t stream);

/* The same function over a prompt in the reference's chunked form (chunked_delta_rule, qwen3_5.rs:342-498, chunk
 * size 64) on the matrix pipe: per chunk the triangular system (I + tril(beta k k^T decay))^-1 is inverted (diagonal
 * blocks with fp32 accumulation, the rest by block substitution), everything else is fp16-operand / fp32-accumulate
 * MFMA.  Mathematically identical to hs_deltanet_forward; outputs and the final state differ from it by rounding
 * (about 1e-3 relative).  Arguments as hs_deltanet_forward, plus a device workspace of
 * hs_deltanet_chunked_workspace_bytes(B, T, nk, nv) bytes (13,312 per 64-token chunk and (sequence, v-head): the two
 * triangular factors of the chunk and three vectors), 16-byte aligned, owned by the caller; q, k, v and out must be
 * 16-byte aligned.  A prompt split into calls of a multiple of 64 tokens (state carried through `state`) gives the
 * bits of one call.  Operands are fp16: with l2norm = 0 the caller's q and k (times q_scale) and their dot products
 * inside a chunk must stay inside the fp16 range (65,504); with l2norm != 0, the reference's setting, they are <= 1. */
HS_API size_t hs_deltanet_chunked_workspace_bytes(int32_t B, int32_t T, int32_t nk, int32_t nv);
HS_API int hs_deltanet_forward_chunked(const void *q, const void *k, const void *v, const float *g, const float *beta,
                        float *state, float *out,
                        int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk, int32_t dv,
                        float q_scale, int l2norm, void *workspace, size_t workspace_bytes, hs_stream_t stream);
/* hs_deltanet_forward_chunked followed by the layer's gated RMSNorm (RMSNormGated::forward, qwen3_5.rs:305-313; what
 * hs_deltanet_gated_norm computes) as one call: out [B, T, nv, dv] bf16 = bf16(o * rsqrt(mean(o^2) + eps) * weight *
 * silu(z)) with z [B, T, nv, dv] bf16 and weight [dv] fp32 (both, and out, 16-byte aligned).  The fp32 rows o pass
 * through the workspace, which is therefore larger: hs_deltanet_chunked_gated_norm_workspace_bytes.  Results are those
 * of the two calls bit for bit; three ordinary launches (capturable in a HIP graph). */
HS_API size_t hs_deltanet_chunked_gated_norm_workspace_bytes(int32_t B, int32_t T, int32_t nk, int32_t nv);
HS_API int hs_deltanet_forward_chunked_gated_norm(const void *q, const void *k, const void *v, const float *g,
                        const float *beta, float *state, const void *z, const float *norm_weight, float norm_eps,
                        void *out, int32_t B, int32_t T, int32_t nk, int32_t nv, int32_t dk, int32_t dv,
                        float q_scale, int l2norm, void *workspace, size_t workspace_bytes, hs_stream_t stream);

/* ---- the elementwise steps of a gated-DeltaNet layer around the delta rule ("next" of hs_deltanet_forward) ----
 * hs_deltanet_prepare (GatedDeltaNetLayer::forward between the input projection and the recurrence,
 * qwen3_5.rs:629-686): depthwise causal conv1d with kernel 4 over [3 carried frames | the S new frames] of the
 * mixed q|k|v channels, then SiLU, in bf16 (fp32 accumulation in tap order, one rounding after the conv, one
 * after the SiLU); the result is split into q, k [B, S, nk, dk] and v [B, S, nv, dv], the inputs of
 * hs_deltanet_forward (which L2-normalises q and k itself).  Gates in fp32: g = neg_a_exp * softplus(a + dt_bias)
 * with neg_a_exp = -exp(A_log) precomputed by the caller as the reference does (qwen3_5.rs:563-568),
 * beta = sigmoid(b).
 *   mixed_qkv [B, S, 2*nk*dk + nv*dv] bf16;  conv_weight [C, 4] bf16 (the [C, 1, 4] conv1d weight);
 *   conv_state_in [B, C, 3] bf16 or NULL (first call: zeros);  conv_state_out [B, C, 3] bf16, a different buffer;
 *   a_in, b_in [B, S, nv] bf16;  neg_a_exp, dt_bias [nv] fp32;  g, beta [B, S, nv] fp32.
 * hs_deltanet_gated_norm (RMSNormGated::forward, qwen3_5.rs:305-313): out = x * rsqrt(mean(x^2) + eps) * w *
 * silu(z) per row of D elements; x fp32 [rows, D] (the recurrence output viewed as [B*S*nv, dv]), z bf16, w fp32 [D],
 * out bf16. */
HS_API int hs_deltanet_prepare(const void *mixed_qkv, const void *conv_weight, const void *conv_state_in,
                               void *conv_state_out, const void *a_in, const void *b_in, const float *neg_a_exp,
                               const float *dt_bias, void *q, void *k, void *v, float *g, float *beta,
                               int32_t B, int32_t S, int32_t nk, int32_t nv, int32_t dk, int32_t dv, hs_stream_t stream);
HS_API int hs_deltanet_gated_norm(const float *x, const void *z, const float *weight, float eps, void *out,
                                  int64_t rows, int32_t D, hs_stream_t stream);
/* The decode branch of GatedDeltaNetLayer::forward between the two projections as ONE launch (qwen3_5.rs:629-686 conv1d
 * + SiLU + gates for the new token, :725-751 the recurrent step with L2-normalised q and k, :305-313 RMSNormGated):
 * hs_deltanet_prepare (S = 1) + hs_deltanet_forward (T = 1) + hs_deltanet_gated_norm, with the arguments of those
 * calls and their results bit for bit (conv_state_out, state, out; for 16-byte aligned buffers, the case those calls
 * serve with their wide kernels), but q, k, v, g, beta and the fp32 output row never leave the chip.
 *   mixed_qkv [B, 1, 2*nk*dk + nv*dv] bf16;  conv_state_in [B, C, 3] bf16 or NULL;  conv_state_out a different buffer;
 *   a_in, b_in [B, 1, nv] bf16;  z [B, 1, nv, dv] bf16;  norm_weight [dv] fp32;  state [B, nv, dk, dv] fp32 in place;
 *   out [B, 1, nv, dv] bf16.  dk = dv = 128; z, norm_weight and out 16-byte aligned, conv_weight 8-byte. */
HS_API int hs_deltanet_decode_layer(const void *mixed_qkv, const void *conv_weight, const void *conv_state_in,
                                    void *conv_state_out, const void *a_in, const void *b_in, const float *neg_a_exp,
                                    const float *dt_bias, const void *z, const float *norm_weight, float norm_eps,
                                    float *state, void *out, int32_t B, int32_t nk, int32_t nv, int32_t dk, int32_t dv,
                                    float q_scale, int l2norm, hs_stream_t stream);

/* The prompt branch of GatedDeltaNetLayer::forward between the two projections as ONE call (qwen3_5.rs:629-686, :753-769,
 * :771-786): hs_deltanet_prepare + hs_deltanet_forward_chunked_gated_norm, five launches in a row with q, k, v, g, beta,
 * the chunk factors and the fp32 output rows in the workspace (hs_deltanet_prefill_layer_workspace_bytes, 256-byte
 * aligned); arguments and results as those calls (mixed_qkv [B, S, C], z and out [B, S, nv, dv] bf16).  The
 * counterpart of hs_deltanet_decode_layer for seq > 1. */
HS_API size_t hs_deltanet_prefill_layer_workspace_bytes(int32_t B, int32_t S, int32_t nk, int32_t nv, int32_t dk, int32_t dv);
HS_API int hs_deltanet_prefill_layer(const void *mixed_qkv, const void *conv_weight, const void *conv_state_in,
                                     void *conv_state_out, const void *a_in, const void *b_in, const float *neg_a_exp,
                                     const float *dt_bias, const void *z, const float *norm_weight, float norm_eps,
                                     float *state, void *out, int32_t B, int32_t S, int32_t nk, int32_t nv, int32_t dk,
                                     int32_t dv, float q_scale, int l2norm, void *workspace, size_t workspace_bytes,
                                     hs_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* HS_ATTN_H */
