/*
 * hs_kv_cache.h -- C view of the host-side LayerKVCache mirror (libhs_kv_cache.so).
 *
 * The C++ class hs::LayerKVCache (hyprstream_amd/host/kv_cache.hpp) keeps the call surface of the
 * reference's LayerKVCache (crates/hyprstream/src/runtime/kv_cache.rs:1027-1891) over device-resident
 * int8 / fp8 storage.  These functions expose it to C, Rust (extern "C") and ctypes; unlike the kernel
 * library (hs_attn.h) this layer OWNS device memory: it allocates the cache at the first update and
 * frees it in clear()/destroy().  Every call returns an hs_status code (hs_attn.h); the message of the
 * last failing call on a cache is read with hs_cache_last_error().
 */
#ifndef HS_KV_CACHE_H
#define HS_KV_CACHE_H

#include "hs_attn.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct hs_cache hs_cache; /* opaque: one LayerKVCache */

enum hs_kv_quant { HS_KV_NONE = 0, HS_KV_INT8 = 1, HS_KV_FP8 = 2 };

/* LayerKVCache::new(max_seq_len, quant_type), kv_cache.rs:1043-1072 */
HS_API hs_cache *hs_cache_create(int64_t max_seq_len, int quant_type);
HS_API void hs_cache_destroy(hs_cache *c);
HS_API const char *hs_cache_last_error(const hs_cache *c);

/* LayerKVCache::update(new_keys, new_values, start_pos), kv_cache.rs:1275-1496.
 * new_keys/new_values: device [batch, seq_len, num_kv_heads, head_dim] in `dtype` (hs_dtype). */
HS_API int hs_cache_update(hs_cache *c, const void *new_keys, const void *new_values, int dtype,
                           int32_t batch, int32_t seq_len, int32_t num_kv_heads, int32_t head_dim,
                           int64_t start_pos, hs_stream_t stream);

/* LayerKVCache::get(), kv_cache.rs:1499-1643, as dense [batch, seq_pos, num_kv_heads, head_dim]
 * tensors written to caller memory in `dtype`.  Fails with "Cache is empty" when seq_pos == 0. */
HS_API int hs_cache_get_dense(hs_cache *c, void *keys_out, void *values_out, int dtype, hs_stream_t stream);

/* get() as a view: pointers to the codes/scales and their layout (no copy). */
HS_API int hs_cache_get_view(hs_cache *c, void **k_codes, void **v_codes, float **k_scales, float **v_scales,
                             hs_kv_layout *layout, int32_t *batch, int32_t *num_kv_heads, int32_t *head_dim);

HS_API int64_t hs_cache_seq_pos(const hs_cache *c);      /* pub seq_pos, kv_cache.rs:1031 */
HS_API int64_t hs_cache_max_seq_len(const hs_cache *c);  /* pub max_seq_len, kv_cache.rs:1033 */
HS_API void hs_cache_clear(hs_cache *c);                 /* kv_cache.rs:1646-1698 */
HS_API void hs_cache_truncate_to(hs_cache *c, int64_t pos); /* kv_cache.rs:1707-1750 */
HS_API int hs_cache_is_initialized(const hs_cache *c);   /* kv_cache.rs:1753-1764 */
HS_API int64_t hs_cache_memory_usage(const hs_cache *c); /* kv_cache.rs:1767-1831 */
HS_API int hs_cache_quant_type(const hs_cache *c);       /* kv_cache.rs:1861 */
/* Canonical lowercase name of a storage format, the string KvQuantMode::as_canonical_str feeds into the
 * compatibility fingerprint (kv_compat.rs:215-237): "none", and for the two device formats served here
 * "int8-token" (int8 codes, one fp32 absmax scale per token and kv-head) and "fp8-e4m3fn-head" (e4m3fn codes,
 * one fp32 scale per sequence and kv-head).  They differ from the reference's "int8" (blockwise-64 codes) on
 * purpose: a cache written in one format must never be reused as another.  NULL for an unknown value. */
HS_API const char *hs_kv_quant_canonical_str(int quant_type);

/* ---- cache identity: which cached K/V may be reused (kv_compat.rs:84-560, 836-1130) ---------------------------------
 * hs_compat is a KvCompatDescriptor (kv_compat.rs:285-378): an ordered set of named fields whose SHA-256 over the
 * reference's canonical byte framing (kv_compat.rs:458-520) is the fingerprint stamped on a cache; a fingerprint
 * computed here equals the Rust side's for the same values (the reference's own pinned digest is a test vector).
 * Fields are set by the names of the Rust struct ("head_dim", "rope_theta_bits", "weights.base_revision",
 * "moe.num_experts", "tokenizer_hash", ...): hs_compat_set_uint for integers, bools and f32 bit patterns,
 * hs_compat_set_opt_uint for Option<u32> / Option<usize>, hs_compat_set_str for strings ("dtype" takes a dtype name,
 * NULL clears "tokenizer_hash").  An unknown field or a value of the wrong kind is HS_ERR_INVALID_ARGUMENT.
 * KvQuantMode (kv_compat.rs:215-237) has two variants more than the reference, one per device format of this library,
 * so that a cache written in one format is never reused as another or as the reference's blockwise "int8". */
typedef struct hs_compat hs_compat;
enum hs_kv_quant_mode { HS_KVQ_NONE = 0, HS_KVQ_INT8 = 1, HS_KVQ_NF4 = 2, HS_KVQ_FP4 = 3,
                        HS_KVQ_INT8_TOKEN = 4,        /* "int8-token": int8 codes + fp32 scale per (token, kv-head) */
                        HS_KVQ_FP8_E4M3FN_HEAD = 5 }; /* "fp8-e4m3fn-head": e4m3fn codes + fp32 scale per (sequence, kv-head) */
enum hs_cache_reuse { HS_REUSE = 0, HS_STAMP_FRESH = 1, HS_DISCARD_AND_RECOMPUTE = 2 }; /* CacheReuseDecision, kv_compat.rs:1087-1101 */
HS_API hs_compat *hs_compat_create(void);  /* format_version = 3, dtype bfloat16, everything else zero / empty / None */
HS_API void hs_compat_destroy(hs_compat *c);
HS_API int hs_compat_set_uint(hs_compat *c, const char *field, uint64_t value);
HS_API int hs_compat_set_opt_uint(hs_compat *c, const char *field, int has_value, uint64_t value);
HS_API int hs_compat_set_str(hs_compat *c, const char *field, const char *value);
HS_API int hs_compat_add_layer_type(hs_compat *c, const char *value);
HS_API int hs_compat_set_rope_scaling(hs_compat *c, const char *rope_type, float factor); /* NULL type = None */
HS_API int hs_compat_set_kv_quant(hs_compat *c, int mode);                                 /* enum hs_kv_quant_mode */
HS_API int hs_compat_is_authoritatively_complete(const hs_compat *c);                      /* kv_compat.rs:426-428 */
HS_API int hs_compat_fingerprint(const hs_compat *c, uint8_t out32[32]);                   /* kv_compat.rs:440-442 */
/* check_compatibility (kv_compat.rs:836-1080): 0 = compatible; 1 = not, and `field` receives the first differing
 * field in the reference's fixed order ("weights" and "moe_routing" for the nested structs); -1 = null argument. */
HS_API int hs_compat_check(const hs_compat *expected, const hs_compat *observed, char *field, size_t field_cap);
/* decide_cache_reuse (kv_compat.rs:1118-1128), fail-closed; fingerprints are 32 bytes or NULL (= None). */
HS_API int hs_compat_decide_reuse(const uint8_t *expected32, const uint8_t *stored32, int cache_is_empty);
HS_API const char *hs_kv_quant_mode_str(int mode); /* KvQuantMode::as_canonical_str; NULL for an unknown value */
HS_API int hs_kv_quant_mode_of(int quant_type);    /* the mode of a cache's storage format (enum hs_kv_quant); -1 unknown */

/* cache.get() + GQA expand + compute_attention for one query token per sequence
 * (llama.rs:605-636, 847-872, 1023-1119).  q, out: bf16 [batch, num_q_heads, head_dim]. */
HS_API int hs_cache_decode_attention(hs_cache *c, const void *q, void *out, int32_t num_q_heads,
                                     float softmax_scale, hs_stream_t stream);
/* cache.update(one token) + the above, one kernel launch. k_new, v_new: [batch, 1, num_kv_heads, head_dim]. */
HS_API int hs_cache_decode_step(hs_cache *c, const void *q, const void *k_new, const void *v_new, int dtype,
                                void *out, int32_t num_q_heads, float softmax_scale, hs_stream_t stream);
/* cache.update(seq_len tokens at start_pos) + causal attention of those tokens (bf16 q / keys / values; an FP8
 * cache calibrates its scales on the tokens written at start_pos 0, as update does). */
HS_API int hs_cache_prefill(hs_cache *c, const void *q, const void *new_keys, const void *new_values, void *out,
                            int32_t batch, int32_t seq_len, int32_t num_q_heads, int32_t num_kv_heads,
                            int32_t head_dim, int64_t start_pos, float softmax_scale, hs_stream_t stream);

/* Opt in to faster prompts through hs_cache_prefill (no counterpart in the reference, whose get() dequantizes the whole
 * cache on every call, kv_cache.rs:1493-1560).  After this call prefill offers the library a key-split workspace (a
 * chunk of ONE sequence is too few query tiles for the GPU: the keys of a tile are then split over workgroups) and,
 * at head_dim 128, keeps a bf16 copy of the prompt's dequantized K/V in the order the matrix
 * instructions take it, which later chunks of the same prompt read instead of converting the codes in every
 * workgroup.  The copy holds 2 x the int8 bytes of max_prompt_tokens tokens, is allocated by the first prefill after
 * this call and freed by hs_cache_drop_prompt_scratch, hs_cache_clear and hs_cache_destroy.  It follows the prompt by
 * itself: a chunk at start_pos 0 begins it, a chunk that starts where the last one ended extends it, anything else
 * written into or cut from the cache (update, decode_step, truncate_to) retires it until the next prompt
 * (hs_cache_prompt_copy_active reports which).  max_prompt_tokens = 0 turns it off again. */
HS_API void hs_cache_enable_prompt_scratch(hs_cache *c, int64_t max_prompt_tokens);
HS_API void hs_cache_drop_prompt_scratch(hs_cache *c);
HS_API int hs_cache_prompt_copy_active(const hs_cache *c);

/* ---- paged mode: shared block pool, per-sequence paged caches, ragged-batch decode step -----------------
 * BlockPool (kv_cache.rs:508-676): 256-token blocks, LIFO free list, every block tagged with its owner.
 * An owner is (kind, id, name) as CacheOwner (kv_cache.rs:49-82): kind 0 = Stateless(id), 1 = Session(name),
 * 2 = Training(name, id).  Allocation on an empty pool returns HS_ERR_POOL_EXHAUSTED with the message
 * "block pool exhausted (all N blocks in use)" (BlockPoolExhausted, kv_cache.rs:489-506): fail-soft, the
 * caller may retry later.  Freeing someone else's block, a free block or an invalid id is refused and
 * changes nothing (kv_cache.rs:606-637).  The bookkeeping needs no GPU; device memory (int8 codes +
 * per-token scales for every block) is allocated at the first update. */
typedef struct hs_pool hs_pool;
typedef struct hs_paged_cache hs_paged_cache;

HS_API hs_pool *hs_pool_create(int64_t num_blocks, int32_t num_kv_heads, int32_t head_dim); /* int8 blocks */
/* The same with the block format chosen: HS_KV_INT8 (codes + per-token scales in every block) or HS_KV_FP8 (e4m3fn
 * codes only: the per-(sequence, kv-head) scales belong to each paged cache, which calibrates them on the tokens
 * written at start_pos 0 exactly as the contiguous FP8 cache does).  NULL for any other format. */
HS_API hs_pool *hs_pool_create_format(int64_t num_blocks, int32_t num_kv_heads, int32_t head_dim, int quant_type);
HS_API int hs_pool_quant_type(const hs_pool *p);
HS_API void hs_pool_destroy(hs_pool *p); /* the blocks live until the last cache of the pool is destroyed */
HS_API const char *hs_pool_last_error(const hs_pool *p);
HS_API int hs_pool_allocate(hs_pool *p, int owner_kind, uint64_t owner_id, const char *owner_name, int32_t *block_id);
HS_API int hs_pool_free(hs_pool *p, int owner_kind, uint64_t owner_id, const char *owner_name, int32_t block_id);
/* 1 and the owner's fields when the block is in use, 0 when it is free or invalid */
HS_API int hs_pool_owner_of(const hs_pool *p, int32_t block_id, int *owner_kind, uint64_t *owner_id,
                            char *owner_name, size_t owner_name_cap);
HS_API int64_t hs_pool_used_blocks(const hs_pool *p);
HS_API int64_t hs_pool_free_block_count(const hs_pool *p);
HS_API int64_t hs_pool_total_blocks(const hs_pool *p);
HS_API int64_t hs_pool_used_memory(const hs_pool *p);

/* LayerKVCache::new_paged(max_seq_len, pool, owner), kv_cache.rs:1100-1120: one sequence, in the pool's format.
 * update takes [1, seq_len, num_kv_heads, head_dim]; blocks are taken in (K, V) pairs and a failed pair is
 * rolled back (kv_cache.rs:1456-1471); clear, truncate_to and destroy return blocks (kv_cache.rs:1679-1750,
 * 1873-1891). */
HS_API hs_paged_cache *hs_paged_cache_create(int64_t max_seq_len, hs_pool *pool, int owner_kind, uint64_t owner_id,
                                             const char *owner_name);
HS_API void hs_paged_cache_destroy(hs_paged_cache *c);
HS_API const char *hs_paged_cache_last_error(const hs_paged_cache *c);
HS_API int hs_paged_cache_update(hs_paged_cache *c, const void *new_keys, const void *new_values, int dtype,
                                 int32_t seq_len, int64_t start_pos, hs_stream_t stream);
HS_API int hs_paged_cache_get_dense(hs_paged_cache *c, void *keys_out, void *values_out, int dtype, hs_stream_t stream);
HS_API int hs_paged_cache_decode_attention(hs_paged_cache *c, const void *q, void *out, int32_t num_q_heads,
                                           float softmax_scale, hs_stream_t stream);
/* update(seq_len bf16 tokens at start_pos) + causal attention of those tokens over [cached history | themselves];
 * q, out: bf16 [1, seq_len, num_q_heads, head_dim]; new_keys, new_values: bf16 [1, seq_len, num_kv_heads, head_dim]. */
HS_API int hs_paged_cache_prefill(hs_paged_cache *c, const void *q, const void *new_keys, const void *new_values, void *out,
                                  int32_t seq_len, int32_t num_q_heads, int64_t start_pos, float softmax_scale,
                                  hs_stream_t stream);
HS_API void hs_paged_cache_clear(hs_paged_cache *c);
HS_API void hs_paged_cache_truncate_to(hs_paged_cache *c, int64_t pos);
HS_API int64_t hs_paged_cache_seq_pos(const hs_paged_cache *c);
HS_API int64_t hs_paged_cache_num_blocks(const hs_paged_cache *c); /* K blocks held (= V blocks held) */

/* One decode step over n paged caches of one pool, one kernel launch: each row caches one new token and attends
 * all its tokens (what forward_batched does with pad + cat + additive mask, llama.rs:710-844, 2544-2572).
 * q, out: bf16 [n, num_q_heads, head_dim]; k_new, v_new: [n, 1, num_kv_heads, head_dim] in dtype.
 * If a row needs a block pair the pool cannot give, the call fails with HS_ERR_POOL_EXHAUSTED before any launch
 * and no row's seq_pos moves; the message is read with hs_pool_last_error. */
HS_API int hs_paged_batch_decode_step(hs_pool *pool, hs_paged_cache *const *rows, int32_t n, const void *q,
                                      const void *k_new, const void *v_new, int dtype, void *out,
                                      int32_t num_q_heads, float softmax_scale, hs_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* HS_KV_CACHE_H */
