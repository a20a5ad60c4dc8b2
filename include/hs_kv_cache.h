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

/* cache.get() + GQA expand + compute_attention for one query token per sequence
 * (llama.rs:605-636, 847-872, 1023-1119).  q, out: bf16 [batch, num_q_heads, head_dim]. */
HS_API int hs_cache_decode_attention(hs_cache *c, const void *q, void *out, int32_t num_q_heads,
                                     float softmax_scale, hs_stream_t stream);
/* cache.update(one token) + the above, one kernel launch. k_new, v_new: [batch, 1, num_kv_heads, head_dim]. */
HS_API int hs_cache_decode_step(hs_cache *c, const void *q, const void *k_new, const void *v_new, int dtype,
                                void *out, int32_t num_q_heads, float softmax_scale, hs_stream_t stream);
/* cache.update(seq_len tokens at start_pos) + causal attention of those tokens (int8 format). */
HS_API int hs_cache_prefill(hs_cache *c, const void *q, const void *new_keys, const void *new_values, void *out,
                            int32_t batch, int32_t seq_len, int32_t num_q_heads, int32_t num_kv_heads,
                            int32_t head_dim, int64_t start_pos, float softmax_scale, hs_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* HS_KV_CACHE_H */
