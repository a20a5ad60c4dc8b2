// Host-side mirror of hyprstream's LayerKVCache for the device-resident quantized formats.
//
// Same call surface as the reference type (crates/hyprstream/src/runtime/kv_cache.rs:1027-1891):
//   new(max_seq_len, quant_type)   :1043      update(keys, values, start_pos) :1275
//   get()                          :1499      clear()                         :1646
//   truncate_to(pos)               :1707      is_initialized()                :1753
//   memory_usage()                 :1767      quant_type()                    :1861
// with the storage replaced: codes and scales live on the GPU in the library's head-major layout,
// update() quantizes ONLY the new tokens (no 64-token buffer, no flush that re-quantizes the whole
// history, no host copy of the codes: kv_cache.rs:1204-1272, 842-856), and attention reads the codes
// directly, so get() hands out a view (pointers + layout + length) instead of materialising dense
// tensors; get_dense() is the literal get() for callers that still want [B, T, Hkv, D] tensors.
// Tensors are raw device pointers plus explicit shapes (the reference passes tch::Tensor).
// Errors are returned, never thrown across the boundary: hs::Status carries the reference's messages
// ("Cache overflow: ...", "Cache is empty", "Expected 4D tensor ..." becomes a shape check).
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>

#include "../../include/hs_attn.h"

namespace hs {

// KVQuantType of the reference is {None, Int8, Nf4, Fp4} (hyprstream-rpc-std/schema/model.capnp:251-257).
// This library serves two device formats: Int8 = symmetric absmax per (token, kv-head);
// Fp8 = e4m3fn with one scale per (sequence, kv-head), calibrated on the first (prompt) update.
enum class KVQuantType : int { None = 0, Int8 = 1, Fp8 = 2 };

struct Status {
    int code = HS_OK;
    std::string message;
    bool ok() const { return code == HS_OK; }
};

// What get() returns: everything the attention entry points need.
struct KVView {
    void *k_codes = nullptr, *v_codes = nullptr;
    float *k_scales = nullptr, *v_scales = nullptr;
    hs_kv_layout layout{};
    int32_t batch = 0, seq_pos = 0, num_kv_heads = 0, head_dim = 0;
    KVQuantType quant_type = KVQuantType::None;
};

class LayerKVCache {
  public:
    LayerKVCache(size_t max_seq_len, KVQuantType quant_type);
    ~LayerKVCache();
    LayerKVCache(const LayerKVCache &) = delete;
    LayerKVCache &operator=(const LayerKVCache &) = delete;

    // new_keys/new_values: device pointers to [batch, seq_len, num_kv_heads, head_dim] in `dtype`
    // (HS_BF16 / HS_F32 / HS_F16).  Tokens land at start_pos .. start_pos+seq_len-1; seq_pos becomes
    // start_pos + seq_len.  start_pos == 0 starts a fresh prompt (kv_cache.rs:1341-1349).
    Status update(const void *new_keys, const void *new_values, int dtype, int32_t batch, int32_t seq_len,
                  int32_t num_kv_heads, int32_t head_dim, size_t start_pos, hs_stream_t stream = nullptr);

    Status get(KVView *view) const;  // "Cache is empty" when seq_pos == 0
    // Dense [batch, seq_pos, num_kv_heads, head_dim] K and V in `dtype`, as the reference's get() returns.
    Status get_dense(void *keys_out, void *values_out, int dtype, hs_stream_t stream = nullptr) const;

    // Attention over the cached tokens: q, out are bf16 [batch, num_q_heads, head_dim] (one query token
    // per sequence, every sequence at seq_pos tokens).  decode_step() first caches one new token.
    Status decode_attention(const void *q, void *out, int32_t num_q_heads, float softmax_scale,
                            hs_stream_t stream = nullptr);
    Status decode_step(const void *q, const void *k_new, const void *v_new, int dtype, void *out, int32_t num_q_heads,
                       float softmax_scale, hs_stream_t stream = nullptr);
    // Causal attention of seq_len new tokens at start_pos over [cached 0..start_pos) | new tokens], then
    // caches them (update + get + attention of LlamaAttention::forward in one call; int8 format only).
    Status prefill(const void *q, const void *new_keys, const void *new_values, void *out, int32_t batch,
                   int32_t seq_len, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, size_t start_pos,
                   float softmax_scale, hs_stream_t stream = nullptr);

    // Opt in to faster prompts: prefill() then offers the library a key-split workspace (calls with few query tiles,
    // i.e. one sequence) and, at head_dim 128, keeps a bf16 operand-order copy of the prompt's K/V
    // that later chunks read instead of converting the codes (2 x the int8 bytes of the prompt, allocated at the
    // first prefill after this call for max_prompt_tokens tokens, dropped by drop_prompt_scratch(), clear() and the
    // destructor).  The copy follows the prompt: a chunk at start_pos 0 begins it, a chunk that starts where the
    // last one ended extends it, and anything else written into the cache (update, decode_step) or taken out of it
    // (truncate_to) retires it until the next prompt.  Results are those of prefill() without it within rounding.
    void enable_prompt_scratch(size_t max_prompt_tokens) { prompt_tokens_ = max_prompt_tokens; }
    void drop_prompt_scratch();
    bool prompt_copy_active() const { return copy_upto_ >= 0; }  // for tests: the next chunk would read the copy

    void clear();
    void truncate_to(size_t pos);
    bool is_initialized() const { return k_codes_ != nullptr && seq_pos > 0; }
    size_t memory_usage() const;
    KVQuantType quant_type() const { return quant_type_; }

    size_t seq_pos = 0;      // number of cached tokens (public in the reference too)
    size_t max_seq_len = 0;  // hard limit

  private:
    Status ensure_storage(int32_t batch, int32_t num_kv_heads, int32_t head_dim);
    Status ensure_scratch(int32_t num_q_heads, int32_t batch, hs_stream_t stream);
    void release();

    KVQuantType quant_type_;
    void *k_codes_ = nullptr, *v_codes_ = nullptr;
    float *k_scales_ = nullptr, *v_scales_ = nullptr;
    int32_t *seq_lens_dev_ = nullptr;  // [batch]; set to seq_pos by a fill launch on the step's stream
    void *workspace_ = nullptr;
    size_t workspace_bytes_ = 0;
    hs_kv_layout layout_{};
    int32_t batch_ = 0, heads_ = 0, dim_ = 0;
    size_t bytes_ = 0;
    // prompt scratch (enable_prompt_scratch)
    size_t prompt_tokens_ = 0;       // 0 = not enabled
    void *split_ws_ = nullptr, *copy_ = nullptr;
    size_t split_ws_bytes_ = 0, copy_bytes_ = 0;
    int32_t split_tokens_ = 0, copy_tokens_ = 0;
    int64_t copy_upto_ = -1;         // tokens 0 .. copy_upto_ - 1 of the cache are in the copy; -1: it is not in step with the cache
};

}  // namespace hs
