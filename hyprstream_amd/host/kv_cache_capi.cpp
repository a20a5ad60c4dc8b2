// extern "C" wrappers over hs::LayerKVCache (see include/hs_kv_cache.h).
#include <new>
#include <string>

#include "../../include/hs_kv_cache.h"
#include "kv_cache.hpp"

struct hs_cache {
    hs::LayerKVCache cache;
    std::string last_error;
    hs_cache(size_t n, hs::KVQuantType q) : cache(n, q) {}
    int done(const hs::Status &s) {
        if (!s.ok()) last_error = s.message;
        return s.code;
    }
};

extern "C" {

hs_cache *hs_cache_create(int64_t max_seq_len, int quant_type) {
    if (max_seq_len <= 0 || quant_type < 0 || quant_type > 2) return nullptr;
    return new (std::nothrow) hs_cache((size_t)max_seq_len, (hs::KVQuantType)quant_type);
}
void hs_cache_destroy(hs_cache *c) { delete c; }
const char *hs_cache_last_error(const hs_cache *c) { return c ? c->last_error.c_str() : "null cache"; }

int hs_cache_update(hs_cache *c, const void *k, const void *v, int dtype, int32_t batch, int32_t seq_len, int32_t heads,
                    int32_t dim, int64_t start_pos, hs_stream_t stream) {
    if (!c || start_pos < 0) return HS_ERR_INVALID_ARGUMENT;
    return c->done(c->cache.update(k, v, dtype, batch, seq_len, heads, dim, (size_t)start_pos, stream));
}
int hs_cache_get_dense(hs_cache *c, void *k, void *v, int dtype, hs_stream_t stream) {
    if (!c) return HS_ERR_INVALID_ARGUMENT;
    return c->done(c->cache.get_dense(k, v, dtype, stream));
}
int hs_cache_get_view(hs_cache *c, void **kc, void **vc, float **ks, float **vs, hs_kv_layout *layout, int32_t *batch,
                      int32_t *heads, int32_t *dim) {
    if (!c) return HS_ERR_INVALID_ARGUMENT;
    hs::KVView v;
    int rc = c->done(c->cache.get(&v));
    if (rc != HS_OK) return rc;
    if (kc) *kc = v.k_codes;
    if (vc) *vc = v.v_codes;
    if (ks) *ks = v.k_scales;
    if (vs) *vs = v.v_scales;
    if (layout) *layout = v.layout;
    if (batch) *batch = v.batch;
    if (heads) *heads = v.num_kv_heads;
    if (dim) *dim = v.head_dim;
    return HS_OK;
}
int64_t hs_cache_seq_pos(const hs_cache *c) { return c ? (int64_t)c->cache.seq_pos : 0; }
int64_t hs_cache_max_seq_len(const hs_cache *c) { return c ? (int64_t)c->cache.max_seq_len : 0; }
void hs_cache_clear(hs_cache *c) { if (c) c->cache.clear(); }
void hs_cache_truncate_to(hs_cache *c, int64_t pos) { if (c && pos >= 0) c->cache.truncate_to((size_t)pos); }
int hs_cache_is_initialized(const hs_cache *c) { return c && c->cache.is_initialized(); }
int64_t hs_cache_memory_usage(const hs_cache *c) { return c ? (int64_t)c->cache.memory_usage() : 0; }
int hs_cache_quant_type(const hs_cache *c) { return c ? (int)c->cache.quant_type() : 0; }
const char *hs_kv_quant_canonical_str(int quant_type) {
    switch (quant_type) {
        case HS_KV_NONE: return "none";
        case HS_KV_INT8: return "int8-token";
        case HS_KV_FP8: return "fp8-e4m3fn-head";
        default: return nullptr;
    }
}

int hs_cache_decode_attention(hs_cache *c, const void *q, void *out, int32_t hq, float scale, hs_stream_t stream) {
    if (!c) return HS_ERR_INVALID_ARGUMENT;
    return c->done(c->cache.decode_attention(q, out, hq, scale, stream));
}
int hs_cache_decode_step(hs_cache *c, const void *q, const void *k_new, const void *v_new, int dtype, void *out, int32_t hq,
                         float scale, hs_stream_t stream) {
    if (!c) return HS_ERR_INVALID_ARGUMENT;
    return c->done(c->cache.decode_step(q, k_new, v_new, dtype, out, hq, scale, stream));
}
int hs_cache_prefill(hs_cache *c, const void *q, const void *k, const void *v, void *out, int32_t batch, int32_t seq_len,
                     int32_t hq, int32_t heads, int32_t dim, int64_t start_pos, float scale, hs_stream_t stream) {
    if (!c || start_pos < 0) return HS_ERR_INVALID_ARGUMENT;
    return c->done(c->cache.prefill(q, k, v, out, batch, seq_len, hq, heads, dim, (size_t)start_pos, scale, stream));
}

void hs_cache_enable_prompt_scratch(hs_cache *c, int64_t max_prompt_tokens) {
    if (c && max_prompt_tokens >= 0) c->cache.enable_prompt_scratch((size_t)max_prompt_tokens);
}
void hs_cache_drop_prompt_scratch(hs_cache *c) {
    if (c) c->cache.drop_prompt_scratch();
}
int hs_cache_prompt_copy_active(const hs_cache *c) { return c && c->cache.prompt_copy_active() ? 1 : 0; }

}  // extern "C"
