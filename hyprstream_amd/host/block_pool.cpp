// Block pool, paged per-sequence cache and ragged-batch decode step (see block_pool.hpp).  Host code only.
#include "block_pool.hpp"

#include <hip/hip_runtime_api.h>

#include "device_fill.hpp"

#include <algorithm>
#include <cstdio>
#include <cstring>

namespace hs {

namespace {
Status err(int code, const std::string &m) { return Status{code, m}; }
Status from_abi(int rc) { return rc == HS_OK ? Status{} : Status{rc, hs_attn_last_error()}; }
Status hip_err(hipError_t e, const char *what) {
    return e == hipSuccess ? Status{} : Status{HS_ERR_LAUNCH, std::string(what) + ": " + hipGetErrorString(e)};
}
Status overflow(int32_t n, size_t start, size_t cap) {
    char buf[200];
    snprintf(buf, sizeof(buf), "Cache overflow: trying to cache %d tokens starting at position %zu, but max_seq_len is %zu", n,
             start, cap);
    return err(HS_ERR_OVERFLOW, buf);
}
}  // namespace

std::string CacheOwner::str() const {
    switch (kind) {
        case Stateless: return "Stateless(" + std::to_string(id) + ")";
        case Session: return "Session(\"" + name + "\")";
        default: return "Training(\"" + name + "\", " + std::to_string(id) + ")";
    }
}

// ------------------------------------------------------------------------------------------------ BlockPool

BlockPool::BlockPool(size_t num_blocks, int32_t heads, int32_t dim, KVQuantType format)
    : total_(num_blocks), heads_(heads), dim_(dim), format_(format) {
    free_list_.reserve(num_blocks);
    for (size_t id = 0; id < num_blocks; ++id) free_list_.push_back((BlockId)id);  // pop() hands out the highest id first
    owner_.resize(num_blocks);
}

BlockPool::~BlockPool() {
    if (codes_) (void)hipFree(codes_);
    if (scales_) (void)hipFree(scales_);
}

Status BlockPool::allocate(const CacheOwner &owner, BlockId *id) {
    std::lock_guard<std::mutex> g(mu_);
    if (free_list_.empty())
        return err(HS_ERR_POOL_EXHAUSTED, "block pool exhausted (all " + std::to_string(total_) + " blocks in use)");
    *id = free_list_.back();
    free_list_.pop_back();
    owner_[(size_t)*id] = std::make_unique<CacheOwner>(owner);
    return {};
}

Status BlockPool::free(const CacheOwner &owner, BlockId id) {
    std::lock_guard<std::mutex> g(mu_);
    if (id < 0 || (size_t)id >= total_) return err(HS_ERR_INVALID_ARGUMENT, "Invalid block ID: " + std::to_string(id));
    const auto &cur = owner_[(size_t)id];
    if (!cur) return err(HS_ERR_INVALID_ARGUMENT, "double-free of block " + std::to_string(id) + " (already in free list)");
    if (!(*cur == owner))
        return err(HS_ERR_INVALID_ARGUMENT, "cross-owner block free rejected: block " + std::to_string(id) + " owned by " +
                                                cur->str() + ", freed by " + owner.str());
    owner_[(size_t)id].reset();
    free_list_.push_back(id);
    return {};
}

const CacheOwner *BlockPool::owner_of(BlockId id) const {
    std::lock_guard<std::mutex> g(mu_);
    if (id < 0 || (size_t)id >= total_) return nullptr;
    return owner_[(size_t)id].get();
}

size_t BlockPool::used_blocks() const {
    std::lock_guard<std::mutex> g(mu_);
    return total_ - free_list_.size();
}

size_t BlockPool::free_block_count() const {
    std::lock_guard<std::mutex> g(mu_);
    return free_list_.size();
}

size_t BlockPool::used_memory() const { return used_blocks() * block_bytes(); }

Status BlockPool::ensure_device() {
    std::lock_guard<std::mutex> g(mu_);
    if (codes_) return {};
    if (total_ == 0) return err(HS_ERR_INVALID_ARGUMENT, "the pool has no blocks");
    const size_t cb = total_ * (size_t)heads_ * kBlockSize * (size_t)dim_;
    // fp8 blocks carry no scales; a token array of the smallest size keeps the pointer non-null for the kernel ABI
    const size_t sb = fp8() ? 256 : total_ * (size_t)heads_ * kBlockSize * sizeof(float);
    hipError_t e;
    if ((e = hipMalloc((void **)&codes_, cb)) != hipSuccess) return hip_err(e, "allocating the block pool");
    if ((e = hipMalloc((void **)&scales_, sb)) != hipSuccess) {
        (void)hipFree(codes_);
        codes_ = nullptr;
        return hip_err(e, "allocating the block pool");
    }
    // all-zero blocks, as the reference's pre-zeroed pool (kv_cache.rs:551-556)
    if ((e = hipMemset(codes_, 0, cb)) != hipSuccess || (e = hipMemset(scales_, 0, sb)) != hipSuccess)
        return hip_err(e, "clearing the block pool");
    return {};
}

hs_kv_layout BlockPool::layout(const int32_t *k_table, const int32_t *v_table, int32_t stride) const {
    hs_kv_layout l{};
    l.code_stride_head = (int64_t)kBlockSize * dim_;
    l.code_stride_seq = l.code_stride_head * heads_;
    l.scale_stride_head = (int64_t)kBlockSize;
    l.scale_stride_seq = (int64_t)kBlockSize * heads_;
    l.capacity_tokens = (int32_t)kBlockSize;
    l.block_table_stride = stride;
    l.k_block_table = k_table;
    l.v_block_table = v_table;
    return l;
}

// ---------------------------------------------------------------------------------------- PagedLayerKVCache

PagedLayerKVCache::PagedLayerKVCache(size_t max_len, std::shared_ptr<BlockPool> pool, CacheOwner owner)
    : max_seq_len(max_len), pool_(std::move(pool)), owner_(std::move(owner)) {}

PagedLayerKVCache::~PagedLayerKVCache() {
    clear();
    for (void *p : {(void *)table_dev_, (void *)len_dev_, (void *)head_scales_dev_, workspace_})
        if (p) (void)hipFree(p);
    if (table_host_) (void)hipHostFree(table_host_);
    if (table_copied_) (void)hipEventDestroy(table_copied_);
}

Status PagedLayerKVCache::reserve(size_t end_pos) {
    if (end_pos > max_seq_len) return overflow((int32_t)(end_pos - seq_pos), seq_pos, max_seq_len);
    const size_t need = (end_pos + kBlockSize - 1) / kBlockSize;
    while (key_blocks_.size() < need) {
        BlockId kid, vid;
        if (Status s = pool_->allocate(owner_, &kid); !s.ok()) return s;
        if (Status s = pool_->allocate(owner_, &vid); !s.ok()) {
            (void)pool_->free(owner_, kid);  // keep the pair balanced: the key block is not leaked
            return s;
        }
        key_blocks_.push_back(kid);
        value_blocks_.push_back(vid);
    }
    return {};
}

// New table entries (a block pair every 256 tokens) go to the device with a copy ordered on the caller's stream, so
// a kernel of an earlier step on that stream never sees a table that changes under it.  The copy's source is a
// pinned mirror of the table (a copy from pageable std::vector storage is staged by the runtime, blocks the host and
// cannot be recorded under stream capture).  Appending never touches mirror entries an earlier copy may still be
// reading; only after blocks were returned (clear / truncate_to) are entries rewritten, and then the last copy's
// event is waited for first.
Status PagedLayerKVCache::sync_table(hs_stream_t stream) {
    const size_t max_blocks = std::max<size_t>((max_seq_len + kBlockSize - 1) / kBlockSize, 1);
    hipError_t e;
    if (!table_dev_) {
        if ((e = hipMalloc((void **)&table_dev_, 2 * max_blocks * sizeof(int32_t))) != hipSuccess)
            return hip_err(e, "allocating the block table");
        if ((e = hipHostMalloc((void **)&table_host_, 2 * max_blocks * sizeof(int32_t), hipHostMallocDefault)) != hipSuccess)
            return hip_err(e, "allocating the pinned block table");
        if ((e = hipEventCreateWithFlags(&table_copied_, hipEventDisableTiming)) != hipSuccess) return hip_err(e, "creating an event");
        if ((e = hipMalloc((void **)&len_dev_, sizeof(int32_t))) != hipSuccess) return hip_err(e, "allocating the length");
        if (pool_->fp8() && (e = hipMalloc((void **)&head_scales_dev_, 2 * sizeof(float) * pool_->num_kv_heads())) != hipSuccess)
            return hip_err(e, "allocating the head scales");
        table_synced_ = 0;
        mirror_high_ = 0;
    }
    if (table_synced_ > key_blocks_.size()) table_synced_ = 0;  // blocks were returned: rewrite what is left
    const size_t n = key_blocks_.size() - table_synced_;
    if (n) {
        if (table_synced_ < mirror_high_) {  // entries an earlier copy read are about to change
            if ((e = hipEventSynchronize(table_copied_)) != hipSuccess) return hip_err(e, "waiting for the last table upload");
            mirror_high_ = table_synced_;
        }
        int32_t *hk = table_host_ + table_synced_, *hv = table_host_ + max_blocks + table_synced_;
        std::copy(key_blocks_.begin() + table_synced_, key_blocks_.end(), hk);
        std::copy(value_blocks_.begin() + table_synced_, value_blocks_.end(), hv);
        if ((e = hipMemcpyAsync(table_dev_ + table_synced_, hk, n * sizeof(int32_t), hipMemcpyHostToDevice,
                                (hipStream_t)stream)) != hipSuccess ||
            (e = hipMemcpyAsync(table_dev_ + max_blocks + table_synced_, hv, n * sizeof(int32_t), hipMemcpyHostToDevice,
                                (hipStream_t)stream)) != hipSuccess)
            return hip_err(e, "uploading the block table");
        if ((e = hipEventRecord(table_copied_, (hipStream_t)stream)) != hipSuccess) return hip_err(e, "recording the table upload");
        table_synced_ = key_blocks_.size();
        mirror_high_ = std::max(mirror_high_, table_synced_);
    }
    return {};
}

Status PagedLayerKVCache::update(const void *new_keys, const void *new_values, int dtype, int32_t seq_len, size_t start_pos,
                                 hs_stream_t stream) {
    if (seq_len < 0) return err(HS_ERR_INVALID_ARGUMENT, "negative seq_len");
    const size_t end_pos = start_pos + (size_t)seq_len;
    if (end_pos > max_seq_len) return overflow(seq_len, start_pos, max_seq_len);
    if (Status s = reserve(end_pos); !s.ok()) return s;
    if (seq_len > 0) {
        if (Status s = pool_->ensure_device(); !s.ok()) return s;
        if (Status s = sync_table(stream); !s.ok()) return s;
        const int32_t stride = (int32_t)((max_seq_len + kBlockSize - 1) / kBlockSize);
        const hs_kv_layout l = pool_->layout(table_dev_, table_dev_ + stride, stride);
        int rc;
        if (pool_->fp8()) {
            float *ks = head_scales_dev_, *vs = head_scales_dev_ + pool_->num_kv_heads();
            if (start_pos == 0) {  // fresh prompt: calibrate the per-head scales on it, as the contiguous cache does
                rc = hs_kv_fp8_calibrate(new_keys, new_values, dtype, ks, vs, 1, seq_len, pool_->num_kv_heads(), pool_->head_dim(), stream);
                if (rc != HS_OK) return from_abi(rc);
            }
            rc = hs_kv_quantize_fp8(new_keys, new_values, dtype, (uint8_t *)pool_->codes(), (uint8_t *)pool_->codes(), ks, vs, &l,
                                    nullptr, (int32_t)start_pos, 1, seq_len, pool_->num_kv_heads(), pool_->head_dim(), stream);
        } else {
            rc = hs_kv_quantize_int8(new_keys, new_values, dtype, pool_->codes(), pool_->codes(), pool_->scales(), pool_->scales(),
                                     &l, nullptr, (int32_t)start_pos, 1, seq_len, pool_->num_kv_heads(), pool_->head_dim(), stream);
        }
        if (rc != HS_OK) return from_abi(rc);
    }
    seq_pos = end_pos;
    return {};
}

Status PagedLayerKVCache::prefill(const void *q, const void *new_keys, const void *new_values, void *out, int32_t seq_len,
                                  int32_t hq, size_t start_pos, float scale, hs_stream_t stream) {
    if (seq_len < 0) return err(HS_ERR_INVALID_ARGUMENT, "negative seq_len");
    const size_t end_pos = start_pos + (size_t)seq_len;
    if (end_pos > max_seq_len) return overflow(seq_len, start_pos, max_seq_len);
    if (start_pos > seq_pos) return err(HS_ERR_INVALID_ARGUMENT, "start_pos is past the cached tokens");
    if (Status s = reserve(end_pos); !s.ok()) return s;
    if (seq_len > 0) {
        if (Status s = pool_->ensure_device(); !s.ok()) return s;
        if (Status s = sync_table(stream); !s.ok()) return s;
        const int32_t stride = (int32_t)((max_seq_len + kBlockSize - 1) / kBlockSize);
        const hs_kv_layout l = pool_->layout(table_dev_, table_dev_ + stride, stride);
        int rc;
        if (pool_->fp8()) {
            float *ks = head_scales_dev_, *vs = head_scales_dev_ + pool_->num_kv_heads();
            if (start_pos == 0) {
                rc = hs_kv_fp8_calibrate(new_keys, new_values, HS_BF16, ks, vs, 1, seq_len, pool_->num_kv_heads(), pool_->head_dim(), stream);
                if (rc != HS_OK) return from_abi(rc);
            }
            rc = hs_prefill_attn_fp8(q, new_keys, new_values, (uint8_t *)pool_->codes(), (uint8_t *)pool_->codes(), ks, vs, &l,
                                     (int32_t)start_pos, out, 1, seq_len, hq, pool_->num_kv_heads(), pool_->head_dim(), scale, 1, stream);
        } else {
            rc = hs_prefill_attn_int8(q, new_keys, new_values, pool_->codes(), pool_->codes(), pool_->scales(), pool_->scales(), &l,
                                      (int32_t)start_pos, out, 1, seq_len, hq, pool_->num_kv_heads(), pool_->head_dim(), scale, 1,
                                      stream);
        }
        if (rc != HS_OK) return from_abi(rc);
    }
    seq_pos = end_pos;
    return {};
}

Status PagedLayerKVCache::get_dense(void *keys_out, void *values_out, int dtype, hs_stream_t stream) {
    if (seq_pos == 0) return err(HS_ERR_INVALID_ARGUMENT, "Cache is empty");
    if (Status s = sync_table(stream); !s.ok()) return s;
    const int32_t stride = (int32_t)((max_seq_len + kBlockSize - 1) / kBlockSize);
    const hs_kv_layout l = pool_->layout(table_dev_, table_dev_ + stride, stride);
    const int fp8 = pool_->fp8();
    const float *ks = fp8 ? head_scales_dev_ : pool_->scales(), *vs = fp8 ? head_scales_dev_ + pool_->num_kv_heads() : pool_->scales();
    int rc = hs_kv_dequantize(pool_->codes(), ks, fp8, &l, 0, keys_out, dtype, 1, (int32_t)seq_pos,
                              pool_->num_kv_heads(), pool_->head_dim(), stream);
    if (rc == HS_OK)
        rc = hs_kv_dequantize(pool_->codes(), vs, fp8, &l, 1, values_out, dtype, 1, (int32_t)seq_pos,
                              pool_->num_kv_heads(), pool_->head_dim(), stream);
    return from_abi(rc);
}

Status PagedLayerKVCache::decode_attention(const void *q, void *out, int32_t hq, float scale, hs_stream_t stream) {
    if (seq_pos == 0) return err(HS_ERR_INVALID_ARGUMENT, "Cache is empty");
    if (Status s = sync_table(stream); !s.ok()) return s;
    const int32_t heads = pool_->num_kv_heads(), dim = pool_->head_dim();
    const size_t need = hs_decode_attn_workspace_bytes(1, hq, heads, dim, (int32_t)max_seq_len);  // sized once
    hipError_t e;
    if (need > workspace_bytes_) {
        if (workspace_) {
            if ((e = hipDeviceSynchronize()) != hipSuccess) return hip_err(e, "waiting before the workspace grows");
            (void)hipFree(workspace_);
        }
        workspace_ = nullptr;
        workspace_bytes_ = 0;
        if ((e = hipMalloc(&workspace_, need)) != hipSuccess) return hip_err(e, "allocating the workspace");
        workspace_bytes_ = need;
    }
    const int32_t len = (int32_t)seq_pos;
    if ((e = fill_i32(len_dev_, 1, len, (hipStream_t)stream)) != hipSuccess) return hip_err(e, "setting the length");
    const int32_t stride = (int32_t)((max_seq_len + kBlockSize - 1) / kBlockSize);
    const hs_kv_layout l = pool_->layout(table_dev_, table_dev_ + stride, stride);
    if (pool_->fp8())
        return from_abi(hs_decode_attn_fp8(q, (const uint8_t *)pool_->codes(), (const uint8_t *)pool_->codes(), head_scales_dev_,
                                           head_scales_dev_ + heads, &l, len_dev_, out, workspace_, workspace_bytes_, 1, hq, heads,
                                           dim, len, scale, stream));
    return from_abi(hs_decode_attn_int8(q, pool_->codes(), pool_->codes(), pool_->scales(), pool_->scales(), &l, len_dev_, out,
                                        workspace_, workspace_bytes_, 1, hq, heads, dim, len, scale, stream));
}

void PagedLayerKVCache::clear() {
    for (BlockId id : key_blocks_) (void)pool_->free(owner_, id);
    for (BlockId id : value_blocks_) (void)pool_->free(owner_, id);
    key_blocks_.clear();
    value_blocks_.clear();
    table_synced_ = 0;
    seq_pos = 0;
}

void PagedLayerKVCache::truncate_to(size_t pos) {
    if (pos >= seq_pos) return;
    const size_t needed = pos == 0 ? 0 : (pos - 1) / kBlockSize + 1;
    if (key_blocks_.size() > needed) {
        for (size_t i = needed; i < key_blocks_.size(); ++i) (void)pool_->free(owner_, key_blocks_[i]);
        for (size_t i = needed; i < value_blocks_.size(); ++i) (void)pool_->free(owner_, value_blocks_[i]);
        key_blocks_.resize(needed);
        value_blocks_.resize(needed);
        table_synced_ = std::min(table_synced_, needed);
    }
    seq_pos = pos;
}

// ----------------------------------------------------------------------------------------------- PagedBatch

PagedBatch::PagedBatch(std::shared_ptr<BlockPool> pool) : pool_(std::move(pool)) {}

PagedBatch::~PagedBatch() {
    for (Slot &sl : slots_) {
        if (sl.dev) (void)hipFree(sl.dev);
        if (sl.host) (void)hipHostFree(sl.host);
        if (sl.done) (void)hipEventDestroy(sl.done);
    }
    if (workspace_) (void)hipFree(workspace_);
}

// A step's tables and lengths travel through one of kSlots (pinned host buffer, device buffer) pairs with a copy
// ordered on the caller's stream; a pair is reused only after the step that last used it has finished on the GPU
// (an event per pair; in steady state it has long fired, so nothing blocks).
Status PagedBatch::slot_for(size_t ints, Slot **out) {
    Slot &sl = slots_[next_slot_++ % kSlots];
    hipError_t e;
    if (sl.done && sl.in_use) {
        if ((e = hipEventSynchronize(sl.done)) != hipSuccess) return hip_err(e, "waiting for a table slot");
        sl.in_use = false;
    }
    if (!sl.done && (e = hipEventCreateWithFlags(&sl.done, hipEventDisableTiming)) != hipSuccess) return hip_err(e, "creating an event");
    if (ints > sl.cap) {
        if (sl.dev) (void)hipFree(sl.dev);
        if (sl.host) (void)hipHostFree(sl.host);
        sl.dev = nullptr; sl.host = nullptr; sl.cap = 0;
        const size_t cap = ints * 2;
        if ((e = hipMalloc((void **)&sl.dev, cap * sizeof(int32_t))) != hipSuccess) return hip_err(e, "allocating the block tables");
        if ((e = hipHostMalloc((void **)&sl.host, cap * sizeof(int32_t), hipHostMallocDefault)) != hipSuccess)
            return hip_err(e, "allocating the pinned block tables");
        sl.cap = cap;
    }
    *out = &sl;
    return {};
}

Status PagedBatch::decode_step(PagedLayerKVCache *const *rows, int32_t n, const void *q, const void *k_new, const void *v_new,
                               int dtype, void *out, int32_t hq, float scale, hs_stream_t stream) {
    if (n <= 0) return err(HS_ERR_INVALID_ARGUMENT, "empty batch");
    size_t max_len = 0, stride = 1;
    for (int32_t i = 0; i < n; ++i) {
        PagedLayerKVCache *r = rows[i];
        if (!r || r->pool().get() != pool_.get()) return err(HS_ERR_INVALID_ARGUMENT, "row " + std::to_string(i) + " is not a cache of this pool");
        if (r->seq_pos + 1 > r->max_seq_len) return overflow(1, r->seq_pos, r->max_seq_len);
    }
    for (int32_t i = 0; i < n; ++i) {  // all block pairs first: a refusal leaves every seq_pos where it was
        if (Status s = rows[i]->reserve(rows[i]->seq_pos + 1); !s.ok()) return s;
        max_len = std::max(max_len, rows[i]->seq_pos + 1);
        stride = std::max(stride, rows[i]->num_blocks());
    }
    if (Status s = pool_->ensure_device(); !s.ok()) return s;
    // int32 units of the slot: K tables, V tables, lengths; an fp8 step adds (8-byte aligned) the rows' scale pointers
    // and the gathered [2][n][Hkv] scales
    const bool fp8 = pool_->fp8();
    const int32_t hk = pool_->num_kv_heads();
    const size_t base_ints = (size_t)n * stride * 2 + (size_t)n;
    const size_t ptr_off = (base_ints + 1) / 2 * 2;
    const size_t gath_off = ptr_off + 2 * (size_t)n;
    const size_t ints = fp8 ? gath_off + 2 * (size_t)n * hk : base_ints;
    if (fp8)
        for (int32_t i = 0; i < n; ++i)
            if (!rows[i]->head_scales()) return err(HS_ERR_INVALID_ARGUMENT, "row " + std::to_string(i) + " has no calibrated scales yet (cache is empty)");
    Slot *sl = nullptr;
    if (Status s = slot_for(ints, &sl); !s.ok()) return s;
    std::fill(sl->host, sl->host + ints, 0);
    int32_t *kt = sl->host, *vt = kt + (size_t)n * stride, *lens = vt + (size_t)n * stride;
    size_t max_cap = 0;
    for (int32_t i = 0; i < n; ++i) max_cap = std::max(max_cap, rows[i]->max_seq_len);
    for (int32_t i = 0; i < n; ++i) {
        std::copy(rows[i]->key_blocks().begin(), rows[i]->key_blocks().end(), kt + (size_t)i * stride);
        std::copy(rows[i]->value_blocks().begin(), rows[i]->value_blocks().end(), vt + (size_t)i * stride);
        lens[i] = (int32_t)(rows[i]->seq_pos + 1);
        if (fp8) {
            const float *src = rows[i]->head_scales();
            std::memcpy(sl->host + ptr_off + 2 * (size_t)i, &src, sizeof(src));
        }
    }
    hipError_t e;
    if ((e = hipMemcpyAsync(sl->dev, sl->host, (fp8 ? gath_off : base_ints) * sizeof(int32_t), hipMemcpyHostToDevice,
                            (hipStream_t)stream)) != hipSuccess)
        return hip_err(e, "uploading the block tables");
    float *gk = (float *)(sl->dev + gath_off), *gv = gk + (size_t)n * hk;
    if (fp8 && (e = gather_head_scales((const float *const *)(sl->dev + ptr_off), gk, gv, n, hk, (hipStream_t)stream)) != hipSuccess)
        return hip_err(e, "gathering the head scales");
    int32_t *tables_dev_ = sl->dev;
    const int32_t heads = pool_->num_kv_heads(), dim = pool_->head_dim();
    const size_t need = hs_decode_attn_workspace_bytes(n, hq, heads, dim, (int32_t)max_cap);  // for the rows' capacity: grows rarely
    if (need > workspace_bytes_) {
        if (workspace_) {
            if ((e = hipDeviceSynchronize()) != hipSuccess) return hip_err(e, "waiting before the workspace grows");
            (void)hipFree(workspace_);
        }
        workspace_ = nullptr;
        workspace_bytes_ = 0;
        if ((e = hipMalloc(&workspace_, need)) != hipSuccess) return hip_err(e, "allocating the workspace");
        workspace_bytes_ = need;
    }
    hs_kv_layout l = pool_->layout(tables_dev_, tables_dev_ + (size_t)n * stride, (int32_t)stride);
    for (int32_t i = 0; i < n; ++i) l.total_tokens_hint += lens[i];  // lets the kernel library balance a ragged batch
    int rc = fp8 ? hs_decode_step_fp8(q, k_new, v_new, dtype, (uint8_t *)pool_->codes(), (uint8_t *)pool_->codes(), gk, gv, &l,
                                      tables_dev_ + 2 * (size_t)n * stride, out, workspace_, workspace_bytes_, n, hq, heads, dim,
                                      (int32_t)max_len, scale, stream)
                 : hs_decode_step_int8(q, k_new, v_new, dtype, pool_->codes(), pool_->codes(), pool_->scales(), pool_->scales(), &l,
                                       tables_dev_ + 2 * (size_t)n * stride, out, workspace_, workspace_bytes_, n, hq, heads, dim,
                                       (int32_t)max_len, scale, stream);
    if (rc != HS_OK) return from_abi(rc);
    if ((e = hipEventRecord(sl->done, (hipStream_t)stream)) != hipSuccess) return hip_err(e, "recording the slot event");
    sl->in_use = true;
    for (int32_t i = 0; i < n; ++i) rows[i]->seq_pos += 1;
    return {};
}

}  // namespace hs
