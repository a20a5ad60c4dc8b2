// extern "C" wrappers over hs::BlockPool, hs::PagedLayerKVCache and hs::PagedBatch (see include/hs_kv_cache.h).
#include <cstring>
#include <memory>
#include <new>
#include <string>
#include <vector>

#include "../../include/hs_kv_cache.h"
#include "block_pool.hpp"

struct hs_pool {
    std::shared_ptr<hs::BlockPool> pool;
    hs::PagedBatch batch;
    std::string last_error;
    hs_pool(size_t n, int32_t h, int32_t d, hs::KVQuantType f) : pool(std::make_shared<hs::BlockPool>(n, h, d, f)), batch(pool) {}
    int done(const hs::Status &s) {
        if (!s.ok()) last_error = s.message;
        return s.code;
    }
};

struct hs_paged_cache {
    hs::PagedLayerKVCache cache;
    std::string last_error;
    hs_paged_cache(size_t n, std::shared_ptr<hs::BlockPool> p, hs::CacheOwner o) : cache(n, std::move(p), std::move(o)) {}
    int done(const hs::Status &s) {
        if (!s.ok()) last_error = s.message;
        return s.code;
    }
};

namespace {
hs::CacheOwner owner(int kind, uint64_t id, const char *name) {
    hs::CacheOwner o;
    o.kind = kind == 1 ? hs::CacheOwner::Session : kind == 2 ? hs::CacheOwner::Training : hs::CacheOwner::Stateless;
    o.id = id;
    if (name) o.name = name;
    return o;
}
}  // namespace

extern "C" {

hs_pool *hs_pool_create_format(int64_t num_blocks, int32_t heads, int32_t dim, int quant_type) {
    if (num_blocks < 0 || heads <= 0 || (dim != 64 && dim != 128 && dim != 256)) return nullptr;
    if (quant_type != HS_KV_INT8 && quant_type != HS_KV_FP8) return nullptr;
    return new (std::nothrow) hs_pool((size_t)num_blocks, heads, dim, quant_type == HS_KV_FP8 ? hs::KVQuantType::Fp8 : hs::KVQuantType::Int8);
}
hs_pool *hs_pool_create(int64_t num_blocks, int32_t heads, int32_t dim) { return hs_pool_create_format(num_blocks, heads, dim, HS_KV_INT8); }
int hs_pool_quant_type(const hs_pool *p) { return p ? (int)p->pool->format() : 0; }
void hs_pool_destroy(hs_pool *p) { delete p; }
const char *hs_pool_last_error(const hs_pool *p) { return p ? p->last_error.c_str() : "null pool"; }

int hs_pool_allocate(hs_pool *p, int kind, uint64_t id, const char *name, int32_t *block_id) {
    if (!p || !block_id) return HS_ERR_INVALID_ARGUMENT;
    return p->done(p->pool->allocate(owner(kind, id, name), block_id));
}
int hs_pool_free(hs_pool *p, int kind, uint64_t id, const char *name, int32_t block_id) {
    if (!p) return HS_ERR_INVALID_ARGUMENT;
    return p->done(p->pool->free(owner(kind, id, name), block_id));
}
int hs_pool_owner_of(const hs_pool *p, int32_t block_id, int *kind, uint64_t *id, char *name, size_t cap) {
    if (!p) return 0;
    const hs::CacheOwner *o = p->pool->owner_of(block_id);
    if (!o) return 0;
    if (kind) *kind = (int)o->kind;
    if (id) *id = o->id;
    if (name && cap) {
        std::strncpy(name, o->name.c_str(), cap - 1);
        name[cap - 1] = 0;
    }
    return 1;
}
int64_t hs_pool_used_blocks(const hs_pool *p) { return p ? (int64_t)p->pool->used_blocks() : 0; }
int64_t hs_pool_free_block_count(const hs_pool *p) { return p ? (int64_t)p->pool->free_block_count() : 0; }
int64_t hs_pool_total_blocks(const hs_pool *p) { return p ? (int64_t)p->pool->total_blocks() : 0; }
int64_t hs_pool_used_memory(const hs_pool *p) { return p ? (int64_t)p->pool->used_memory() : 0; }

hs_paged_cache *hs_paged_cache_create(int64_t max_seq_len, hs_pool *pool, int kind, uint64_t id, const char *name) {
    if (!pool || max_seq_len <= 0) return nullptr;
    return new (std::nothrow) hs_paged_cache((size_t)max_seq_len, pool->pool, owner(kind, id, name));
}
void hs_paged_cache_destroy(hs_paged_cache *c) { delete c; }
const char *hs_paged_cache_last_error(const hs_paged_cache *c) { return c ? c->last_error.c_str() : "null cache"; }
int hs_paged_cache_update(hs_paged_cache *c, const void *k, const void *v, int dtype, int32_t seq_len, int64_t start_pos,
                          hs_stream_t stream) {
    if (!c || start_pos < 0) return HS_ERR_INVALID_ARGUMENT;
    return c->done(c->cache.update(k, v, dtype, seq_len, (size_t)start_pos, stream));
}
int hs_paged_cache_get_dense(hs_paged_cache *c, void *k, void *v, int dtype, hs_stream_t stream) {
    if (!c) return HS_ERR_INVALID_ARGUMENT;
    return c->done(c->cache.get_dense(k, v, dtype, stream));
}
int hs_paged_cache_decode_attention(hs_paged_cache *c, const void *q, void *out, int32_t hq, float scale, hs_stream_t stream) {
    if (!c) return HS_ERR_INVALID_ARGUMENT;
    return c->done(c->cache.decode_attention(q, out, hq, scale, stream));
}
int hs_paged_cache_prefill(hs_paged_cache *c, const void *q, const void *new_keys, const void *new_values, void *out,
                           int32_t seq_len, int32_t hq, int64_t start_pos, float scale, hs_stream_t stream) {
    if (!c || start_pos < 0) return HS_ERR_INVALID_ARGUMENT;
    return c->done(c->cache.prefill(q, new_keys, new_values, out, seq_len, hq, (size_t)start_pos, scale, stream));
}
void hs_paged_cache_clear(hs_paged_cache *c) { if (c) c->cache.clear(); }
void hs_paged_cache_truncate_to(hs_paged_cache *c, int64_t pos) { if (c && pos >= 0) c->cache.truncate_to((size_t)pos); }
int64_t hs_paged_cache_seq_pos(const hs_paged_cache *c) { return c ? (int64_t)c->cache.seq_pos : 0; }
int64_t hs_paged_cache_num_blocks(const hs_paged_cache *c) { return c ? (int64_t)c->cache.num_blocks() : 0; }

int hs_paged_batch_decode_step(hs_pool *pool, hs_paged_cache *const *rows, int32_t n, const void *q, const void *k_new,
                               const void *v_new, int dtype, void *out, int32_t hq, float scale, hs_stream_t stream) {
    if (!pool || !rows || n <= 0) return HS_ERR_INVALID_ARGUMENT;
    std::vector<hs::PagedLayerKVCache *> r((size_t)n);
    for (int32_t i = 0; i < n; ++i) {
        if (!rows[i]) return HS_ERR_INVALID_ARGUMENT;
        r[(size_t)i] = &rows[i]->cache;
    }
    return pool->done(pool->batch.decode_step(r.data(), n, q, k_new, v_new, dtype, out, hq, scale, stream));
}

}  // extern "C"
