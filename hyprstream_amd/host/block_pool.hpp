// Paged KV storage for the device-resident int8 format: a shared pool of fixed-size blocks, a per-sequence
// paged cache on top of it, and the glue that runs one decode step over a ragged batch of such caches.
//
// Mirrors, name for name, the reference's paged mode (crates/hyprstream/src/runtime/kv_cache.rs):
//   BLOCK_SIZE = 256                         :477      BlockPoolExhausted (fail-soft)        :489-506
//   BlockPool::{new, allocate, free,         :508-676  LayerKVCache::new_paged               :1100-1120
//     owner_of, used_blocks, free_block_count,          paged update (K/V pairs, rollback)   :1433-1489
//     total_blocks, used_memory}                        paged clear / truncate_to / drop      :1679-1750
// with two differences that follow from the storage format: a block holds int8 codes plus per-token scales
// ([Hkv][256][D] bytes + [Hkv][256] fp32) instead of a dense tensor, and reads never concatenate blocks
// (kv_cache.rs:1581-1641): the attention kernels walk the block table.
// Bookkeeping is plain host code and needs no GPU; device memory is allocated at the first call that needs it.
#pragma once
#include <cstddef>
#include <cstdint>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "kv_cache.hpp"

namespace hs {

constexpr size_t kBlockSize = 256;  // tokens per block (BLOCK_SIZE, kv_cache.rs:477)
using BlockId = int32_t;

// Who holds a cache or a block (CacheOwner, kv_cache.rs:49-82): a stateless request id, a named session, or a
// training run.  Two owners are the same tenant only if kind, id and name all match.
struct CacheOwner {
    enum Kind : int { Stateless = 0, Session = 1, Training = 2 } kind = Stateless;
    uint64_t id = 0;
    std::string name;
    static CacheOwner stateless(uint64_t id) { return CacheOwner{Stateless, id, {}}; }
    static CacheOwner session(std::string n) { return CacheOwner{Session, 0, std::move(n)}; }
    bool operator==(const CacheOwner &o) const { return kind == o.kind && id == o.id && name == o.name; }
    std::string str() const;
};

class BlockPool {
  public:
    // format: Int8 (codes + per-token scales in every block) or Fp8 (e4m3fn codes only; the per-(sequence, kv-head)
    // scales belong to the caches, not to the blocks)
    BlockPool(size_t num_blocks, int32_t num_kv_heads, int32_t head_dim, KVQuantType format = KVQuantType::Int8);
    ~BlockPool();
    BlockPool(const BlockPool &) = delete;
    BlockPool &operator=(const BlockPool &) = delete;

    // Pops the most recently freed block (LIFO) and tags it with `owner`.  With no free block left the status is
    // HS_ERR_POOL_EXHAUSTED, "block pool exhausted (all N blocks in use)": a fail-soft signal a scheduler can turn
    // into admission-defer.
    Status allocate(const CacheOwner &owner, BlockId *id);
    // Returns a block.  A block of another owner, a free block or an invalid id is refused and nothing changes.
    Status free(const CacheOwner &owner, BlockId id);
    const CacheOwner *owner_of(BlockId id) const;  // nullptr when free or invalid
    size_t used_blocks() const;
    size_t free_block_count() const;
    size_t total_blocks() const { return total_; }
    size_t used_memory() const;  // bytes of the blocks in use
    size_t block_bytes() const { return (size_t)heads_ * kBlockSize * ((size_t)dim_ + (fp8() ? 0 : 4)); }
    KVQuantType format() const { return format_; }
    bool fp8() const { return format_ == KVQuantType::Fp8; }
    int32_t num_kv_heads() const { return heads_; }
    int32_t head_dim() const { return dim_; }

    // Device side (allocated once, on first use): codes [blocks][Hkv][256][D] and scales [blocks][Hkv][256].
    Status ensure_device();
    int8_t *codes() const { return codes_; }
    float *scales() const { return scales_; }
    // Layout for the kernel library; K and V blocks come from the same pool, so both code pointers are codes().
    hs_kv_layout layout(const int32_t *k_table, const int32_t *v_table, int32_t table_stride) const;

  private:
    mutable std::mutex mu_;
    size_t total_;
    int32_t heads_, dim_;
    KVQuantType format_;
    std::vector<BlockId> free_list_;
    std::vector<std::unique_ptr<CacheOwner>> owner_;
    int8_t *codes_ = nullptr;
    float *scales_ = nullptr;
};

// LayerKVCache::new_paged(max_seq_len, pool, owner): one sequence (batch 1), int8 format.
class PagedLayerKVCache {
  public:
    PagedLayerKVCache(size_t max_seq_len, std::shared_ptr<BlockPool> pool, CacheOwner owner);
    ~PagedLayerKVCache();  // returns every block (kv_cache.rs:1873-1891)
    PagedLayerKVCache(const PagedLayerKVCache &) = delete;
    PagedLayerKVCache &operator=(const PagedLayerKVCache &) = delete;

    // new_keys/new_values: device [1, seq_len, num_kv_heads, head_dim] in `dtype`.  Blocks are taken in (K, V) pairs
    // as the write crosses block boundaries; if the V block of a pair cannot be had the K block goes back and the
    // error is the pool's fail-soft status (kv_cache.rs:1456-1471).  Blocks taken by earlier pairs of the same call stay.
    Status update(const void *new_keys, const void *new_values, int dtype, int32_t seq_len, size_t start_pos,
                  hs_stream_t stream = nullptr);
    Status get_dense(void *keys_out, void *values_out, int dtype, hs_stream_t stream = nullptr);
    Status decode_attention(const void *q, void *out, int32_t num_q_heads, float softmax_scale, hs_stream_t stream = nullptr);
    // update(seq_len bf16 tokens at start_pos) + causal attention of those tokens over [cached history | themselves];
    // q, out: bf16 [1, seq_len, num_q_heads, head_dim].  Blocks are taken as in update().
    Status prefill(const void *q, const void *new_keys, const void *new_values, void *out, int32_t seq_len, int32_t num_q_heads,
                   size_t start_pos, float softmax_scale, hs_stream_t stream = nullptr);
    void clear();
    void truncate_to(size_t pos);  // frees the blocks beyond the last needed one (kv_cache.rs:1725-1748)
    size_t num_blocks() const { return key_blocks_.size(); }
    const std::vector<BlockId> &key_blocks() const { return key_blocks_; }
    const std::vector<BlockId> &value_blocks() const { return value_blocks_; }
    // Makes sure blocks exist for positions < end_pos (host bookkeeping only; used by the batch step).
    Status reserve(size_t end_pos);
    const CacheOwner &owner() const { return owner_; }
    const float *head_scales() const { return head_scales_dev_; }
    const std::shared_ptr<BlockPool> &pool() const { return pool_; }

    size_t seq_pos = 0;
    size_t max_seq_len = 0;

  private:
    Status sync_table(hs_stream_t stream);
    std::shared_ptr<BlockPool> pool_;
    CacheOwner owner_;
    std::vector<BlockId> key_blocks_, value_blocks_;
    int32_t *table_dev_ = nullptr;  // [2][max_blocks]: row 0 = K blocks, row 1 = V blocks
    int32_t *len_dev_ = nullptr;
    float *head_scales_dev_ = nullptr;  // fp8 pools: [2][Hkv], K then V, calibrated by the update at start_pos 0
    int32_t *table_host_ = nullptr; // pinned mirror of the table, the source of the uploads
    hipEvent_t table_copied_ = nullptr;  // recorded behind the last upload
    size_t table_synced_ = 0;       // number of blocks the device table already holds
    size_t mirror_high_ = 0;        // mirror entries below this index may still be read by an upload in flight
    void *workspace_ = nullptr;
    size_t workspace_bytes_ = 0;
};

// One decode step over several paged caches of one pool (the batched path of the reference pads and concatenates
// the rows' K/V and builds an additive mask, llama.rs:710-844, 2544-2572; here the rows' block tables and lengths
// go to one kernel launch).  Each row caches one new token and attends all its tokens.
class PagedBatch {
  public:
    explicit PagedBatch(std::shared_ptr<BlockPool> pool);
    ~PagedBatch();
    // q, out: bf16 [n, num_q_heads, head_dim]; k_new, v_new: [n, 1, num_kv_heads, head_dim] in `dtype`.
    // Fails with the pool's fail-soft status, before anything is launched or any seq_pos moves, if a row needs a
    // new block pair that the pool cannot give.
    Status decode_step(PagedLayerKVCache *const *rows, int32_t n, const void *q, const void *k_new, const void *v_new,
                       int dtype, void *out, int32_t num_q_heads, float softmax_scale, hs_stream_t stream = nullptr);

  private:
    static constexpr int kSlots = 4;
    struct Slot {  // K tables, V tables and lengths of one step: pinned host copy, device copy, "step finished" event
        int32_t *host = nullptr, *dev = nullptr;
        size_t cap = 0;  // in int32 units; an fp8 step also carries the rows' scale pointers and the gathered scales
        hipEvent_t done = nullptr;
        bool in_use = false;
    };
    Status slot_for(size_t ints, Slot **out);
    std::shared_ptr<BlockPool> pool_;
    Slot slots_[kSlots];
    unsigned next_slot_ = 0;
    void *workspace_ = nullptr;
    size_t workspace_bytes_ = 0;
};

}  // namespace hs
