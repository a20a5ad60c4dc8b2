// Implementation of the LayerKVCache mirror (see kv_cache.hpp).  Host code only: it allocates device
// memory with hipMalloc and calls the C ABI of libhs_attn for every kernel.
#include "kv_cache.hpp"

#include <algorithm>

#include <hip/hip_runtime_api.h>

#include "device_fill.hpp"

#include <cstdio>
#include <vector>

namespace hs {

namespace {
Status err(int code, const std::string &m) { return Status{code, m}; }
Status from_abi(int rc) { return rc == HS_OK ? Status{} : Status{rc, hs_attn_last_error()}; }
Status hip_err(hipError_t e, const char *what) {
    return e == hipSuccess ? Status{} : Status{HS_ERR_LAUNCH, std::string(what) + ": " + hipGetErrorString(e)};
}
}  // namespace

LayerKVCache::LayerKVCache(size_t max_len, KVQuantType qt) : max_seq_len(max_len), quant_type_(qt) {}

LayerKVCache::~LayerKVCache() { release(); }

void LayerKVCache::drop_prompt_scratch() {
    for (void *p : {split_ws_, copy_})
        if (p) (void)hipFree(p);
    split_ws_ = copy_ = nullptr;
    split_ws_bytes_ = copy_bytes_ = 0;
    split_tokens_ = copy_tokens_ = 0;
    copy_upto_ = -1;
}

void LayerKVCache::release() {
    drop_prompt_scratch();
    for (void *p : {k_codes_, v_codes_, (void *)k_scales_, (void *)v_scales_, (void *)seq_lens_dev_, workspace_})
        if (p) (void)hipFree(p);
    k_codes_ = v_codes_ = workspace_ = nullptr;
    k_scales_ = v_scales_ = nullptr;
    seq_lens_dev_ = nullptr;
    workspace_bytes_ = 0;
    batch_ = heads_ = dim_ = 0;
    bytes_ = 0;
}

// Storage is allocated once, at the first update, for max_seq_len tokens (the reference grows in
// 1024-token chunks, kv_cache.rs:700, 1146-1200; a head-major layout would have to be re-strided on
// every growth step and 288 GB of HBM make the up-front allocation the cheaper choice).
Status LayerKVCache::ensure_storage(int32_t batch, int32_t heads, int32_t dim) {
    if (k_codes_) {
        if (batch != batch_ || heads != heads_ || dim != dim_)
            return err(HS_ERR_INVALID_ARGUMENT, "update shape [" + std::to_string(batch) + ", _, " + std::to_string(heads) +
                                                    ", " + std::to_string(dim) + "] does not match the cached tensors");
        return {};
    }
    const size_t cap = max_seq_len;
    const size_t cap_s = (cap + 3) / 4 * 4;
    layout_ = hs_kv_layout{};
    layout_.code_stride_head = (int64_t)cap * dim;
    layout_.code_stride_seq = layout_.code_stride_head * heads;
    layout_.scale_stride_head = (int64_t)cap_s;
    layout_.scale_stride_seq = (int64_t)cap_s * heads;
    layout_.capacity_tokens = (int32_t)cap;
    const size_t code_bytes = (size_t)batch * heads * cap * dim;
    const size_t scale_bytes = quant_type_ == KVQuantType::Fp8 ? (size_t)batch * heads * 4 : (size_t)batch * heads * cap_s * 4;
    hipError_t e;
    if ((e = hipMalloc(&k_codes_, code_bytes)) != hipSuccess || (e = hipMalloc(&v_codes_, code_bytes)) != hipSuccess ||
        (e = hipMalloc((void **)&k_scales_, scale_bytes)) != hipSuccess ||
        (e = hipMalloc((void **)&v_scales_, scale_bytes)) != hipSuccess ||
        (e = hipMalloc((void **)&seq_lens_dev_, sizeof(int32_t) * batch)) != hipSuccess) {
        release();
        return hip_err(e, "allocating the KV cache");
    }
    batch_ = batch; heads_ = heads; dim_ = dim;
    bytes_ = 2 * code_bytes + 2 * scale_bytes;
    return {};
}

// The split-K workspace is sized ONCE for max_seq_len (it only ever grows if a later call brings more query heads),
// so steady-state steps neither allocate nor free.  The sequence lengths reach the device through a fill launch on
// the caller's stream, ordered with the attention launch that reads them.
Status LayerKVCache::ensure_scratch(int32_t hq, int32_t batch, hs_stream_t stream) {
    const size_t bytes = hs_decode_attn_workspace_bytes(batch, hq, heads_, dim_, (int32_t)max_seq_len);
    if (bytes > workspace_bytes_) {
        if (workspace_) {
            // an earlier step on some stream may still use the old buffer
            if (hipError_t e = hipDeviceSynchronize(); e != hipSuccess) return hip_err(e, "waiting before the workspace grows");
            (void)hipFree(workspace_);
        }
        workspace_ = nullptr;
        workspace_bytes_ = 0;
        if (hipError_t e = hipMalloc(&workspace_, bytes); e != hipSuccess) return hip_err(e, "allocating the workspace");
        workspace_bytes_ = bytes;
    }
    return hip_err(fill_i32(seq_lens_dev_, batch, (int32_t)seq_pos, (hipStream_t)stream), "setting the sequence lengths");
}

Status LayerKVCache::update(const void *new_keys, const void *new_values, int dtype, int32_t batch, int32_t seq_len,
                            int32_t heads, int32_t dim, size_t start_pos, hs_stream_t stream) {
    if (quant_type_ == KVQuantType::None)
        return err(HS_ERR_INVALID_ARGUMENT, "full-precision storage is not served by this library; use Int8 or Fp8");
    if (batch <= 0 || seq_len < 0 || heads <= 0 || dim <= 0)
        return err(HS_ERR_INVALID_ARGUMENT, "Expected 4D tensor for keys, got [" + std::to_string(batch) + ", " +
                                                std::to_string(seq_len) + ", " + std::to_string(heads) + ", " + std::to_string(dim) + "]");
    const size_t end_pos = start_pos + (size_t)seq_len;
    if (end_pos > max_seq_len) {
        char buf[200];
        snprintf(buf, sizeof(buf), "Cache overflow: trying to cache %d tokens starting at position %zu, but max_seq_len is %zu",
                 seq_len, start_pos, max_seq_len);
        return err(HS_ERR_OVERFLOW, buf);
    }
    if (Status s = ensure_storage(batch, heads, dim); !s.ok()) return s;
    copy_upto_ = -1;  // tokens written here are not in the prompt copy
    int rc;
    if (quant_type_ == KVQuantType::Fp8) {
        if (start_pos == 0) {  // fresh prompt: calibrate the per-(sequence, head) scales on it
            rc = hs_kv_fp8_calibrate(new_keys, new_values, dtype, k_scales_, v_scales_, batch, seq_len, heads, dim, stream);
            if (rc != HS_OK) return from_abi(rc);
        }
        rc = hs_kv_quantize_fp8(new_keys, new_values, dtype, (uint8_t *)k_codes_, (uint8_t *)v_codes_, k_scales_, v_scales_,
                                &layout_, nullptr, (int32_t)start_pos, batch, seq_len, heads, dim, stream);
    } else {
        rc = hs_kv_quantize_int8(new_keys, new_values, dtype, (int8_t *)k_codes_, (int8_t *)v_codes_, k_scales_, v_scales_,
                                 &layout_, nullptr, (int32_t)start_pos, batch, seq_len, heads, dim, stream);
    }
    if (rc != HS_OK) return from_abi(rc);
    seq_pos = end_pos;
    return {};
}

Status LayerKVCache::get(KVView *v) const {
    if (seq_pos == 0) return err(HS_ERR_INVALID_ARGUMENT, "Cache is empty");
    if (!k_codes_) return err(HS_ERR_INVALID_ARGUMENT, "Keys/values cache not initialized");
    v->k_codes = k_codes_; v->v_codes = v_codes_;
    v->k_scales = k_scales_; v->v_scales = v_scales_;
    v->layout = layout_;
    v->batch = batch_; v->seq_pos = (int32_t)seq_pos; v->num_kv_heads = heads_; v->head_dim = dim_;
    v->quant_type = quant_type_;
    return {};
}

Status LayerKVCache::get_dense(void *keys_out, void *values_out, int dtype, hs_stream_t stream) const {
    KVView v;
    if (Status s = get(&v); !s.ok()) return s;
    const int fp8 = quant_type_ == KVQuantType::Fp8;
    int rc = hs_kv_dequantize(k_codes_, k_scales_, fp8, &layout_, 0, keys_out, dtype, batch_, (int32_t)seq_pos, heads_, dim_, stream);
    if (rc == HS_OK)
        rc = hs_kv_dequantize(v_codes_, v_scales_, fp8, &layout_, 1, values_out, dtype, batch_, (int32_t)seq_pos, heads_, dim_, stream);
    return from_abi(rc);
}

Status LayerKVCache::decode_attention(const void *q, void *out, int32_t hq, float scale, hs_stream_t stream) {
    KVView v;
    if (Status s = get(&v); !s.ok()) return s;
    if (Status s = ensure_scratch(hq, batch_, stream); !s.ok()) return s;
    int rc = quant_type_ == KVQuantType::Fp8
                 ? hs_decode_attn_fp8(q, (const uint8_t *)k_codes_, (const uint8_t *)v_codes_, k_scales_, v_scales_, &layout_,
                                      seq_lens_dev_, out, workspace_, workspace_bytes_, batch_, hq, heads_, dim_, (int32_t)seq_pos, scale, stream)
                 : hs_decode_attn_int8(q, (const int8_t *)k_codes_, (const int8_t *)v_codes_, k_scales_, v_scales_, &layout_,
                                       seq_lens_dev_, out, workspace_, workspace_bytes_, batch_, hq, heads_, dim_, (int32_t)seq_pos, scale, stream);
    return from_abi(rc);
}

Status LayerKVCache::decode_step(const void *q, const void *k_new, const void *v_new, int dtype, void *out, int32_t hq,
                                 float scale, hs_stream_t stream) {
    if (!k_codes_ || seq_pos == 0) return err(HS_ERR_INVALID_ARGUMENT, "Cache is empty");
    if (seq_pos + 1 > max_seq_len) {
        char buf[200];
        snprintf(buf, sizeof(buf), "Cache overflow: trying to cache 1 tokens starting at position %zu, but max_seq_len is %zu", seq_pos, max_seq_len);
        return err(HS_ERR_OVERFLOW, buf);
    }
    copy_upto_ = -1;  // the new token is not in the prompt copy
    seq_pos += 1;  // the entry point writes the new token at seq_pos - 1 and attends seq_pos tokens
    Status s = ensure_scratch(hq, batch_, stream);
    int rc = HS_OK;
    if (s.ok()) {
        rc = quant_type_ == KVQuantType::Fp8
                 ? hs_decode_step_fp8(q, k_new, v_new, dtype, (uint8_t *)k_codes_, (uint8_t *)v_codes_, k_scales_, v_scales_, &layout_,
                                      seq_lens_dev_, out, workspace_, workspace_bytes_, batch_, hq, heads_, dim_, (int32_t)seq_pos, scale, stream)
                 : hs_decode_step_int8(q, k_new, v_new, dtype, (int8_t *)k_codes_, (int8_t *)v_codes_, k_scales_, v_scales_, &layout_,
                                       seq_lens_dev_, out, workspace_, workspace_bytes_, batch_, hq, heads_, dim_, (int32_t)seq_pos, scale, stream);
        s = from_abi(rc);
    }
    if (!s.ok()) seq_pos -= 1;
    return s;
}

Status LayerKVCache::prefill(const void *q, const void *new_keys, const void *new_values, void *out, int32_t batch,
                             int32_t seq_len, int32_t hq, int32_t heads, int32_t dim, size_t start_pos, float scale,
                             hs_stream_t stream) {
    if (quant_type_ == KVQuantType::None)
        return err(HS_ERR_INVALID_ARGUMENT, "full-precision storage is not served by this library; use Int8 or Fp8");
    const size_t end_pos = start_pos + (size_t)seq_len;
    if (end_pos > max_seq_len) {
        char buf[200];
        snprintf(buf, sizeof(buf), "Cache overflow: trying to cache %d tokens starting at position %zu, but max_seq_len is %zu",
                 seq_len, start_pos, max_seq_len);
        return err(HS_ERR_OVERFLOW, buf);
    }
    if (start_pos > seq_pos) return err(HS_ERR_INVALID_ARGUMENT, "start_pos is past the cached tokens");
    if (Status s = ensure_storage(batch, heads, dim); !s.ok()) return s;
    int rc;
    hs_kv_layout lay = layout_;
    bool with_copy = false;
    if (prompt_tokens_ > 0) {
        // key-split workspace: sized for the longest chunk seen (grows like the decode workspace)
        if (seq_len > split_tokens_) {
            if (split_ws_) {
                if (hipError_t e = hipDeviceSynchronize(); e != hipSuccess) return hip_err(e, "waiting before the split workspace grows");
                (void)hipFree(split_ws_);
                split_ws_ = nullptr;
            }
            split_ws_bytes_ = hs_prefill_attn_split_workspace_bytes(batch, seq_len, hq, heads, dim);
            split_tokens_ = 0;
            if (split_ws_bytes_ > 0) {
                if (hipError_t e = hipMalloc(&split_ws_, split_ws_bytes_); e != hipSuccess) return hip_err(e, "allocating the split workspace");
                if (int rc2 = hs_prefill_attn_split_workspace_init(split_ws_, split_ws_bytes_, stream); rc2 != HS_OK) return from_abi(rc2);
                split_tokens_ = seq_len;
            }
        }
        if (split_ws_) {
            lay.prefill_split_workspace = split_ws_;
            lay.prefill_split_workspace_bytes = (int64_t)split_ws_bytes_;
        }
        // the bf16 copy: begun by a chunk at position 0, extended by a chunk that starts where the copy ends
        const size_t want = std::min(prompt_tokens_, max_seq_len);
        if (dim == 128 && end_pos <= want && (start_pos == 0 || (copy_upto_ >= 0 && (size_t)copy_upto_ == start_pos))) {
            if (!copy_) {
                copy_tokens_ = (int32_t)((want + 63) / 64 * 64);
                copy_bytes_ = hs_prefill_shadow_bytes(batch, heads, dim, copy_tokens_);
                if (hipError_t e = hipMalloc(&copy_, copy_bytes_); e != hipSuccess) return hip_err(e, "allocating the prompt copy");
                if (int rc2 = hs_prefill_shadow_init(copy_, copy_bytes_, stream); rc2 != HS_OK) return from_abi(rc2);
            }
            lay.prefill_shadow = copy_;
            lay.prefill_shadow_bytes = (int64_t)copy_bytes_;
            lay.prefill_shadow_tokens = copy_tokens_;
            with_copy = true;
        }
    }
    if (quant_type_ == KVQuantType::Fp8) {
        if (start_pos == 0) {  // fresh prompt: calibrate the per-(sequence, head) scales on it, as update() does
            rc = hs_kv_fp8_calibrate(new_keys, new_values, HS_BF16, k_scales_, v_scales_, batch, seq_len, heads, dim, stream);
            if (rc != HS_OK) return from_abi(rc);
        }
        rc = hs_prefill_attn_fp8(q, new_keys, new_values, (uint8_t *)k_codes_, (uint8_t *)v_codes_, k_scales_, v_scales_, &lay,
                                 (int32_t)start_pos, out, batch, seq_len, hq, heads, dim, scale, 1, stream);
    } else {
        rc = hs_prefill_attn_int8(q, new_keys, new_values, (int8_t *)k_codes_, (int8_t *)v_codes_, k_scales_, v_scales_, &lay,
                                  (int32_t)start_pos, out, batch, seq_len, hq, heads, dim, scale, 1, stream);
    }
    copy_upto_ = rc == HS_OK && with_copy ? (int64_t)end_pos : -1;
    if (rc != HS_OK) return from_abi(rc);
    seq_pos = end_pos;
    return {};
}

void LayerKVCache::clear() {
    release();
    seq_pos = 0;
}

// Per-token scales make truncation a position move for both formats (the reference clears its
// quantized storage instead because its blockwise codes straddle tokens, kv_cache.rs:1716-1720).
void LayerKVCache::truncate_to(size_t pos) {
    if (pos >= seq_pos) return;
    seq_pos = pos;
    copy_upto_ = -1;  // (a prompt that continues from here starts its copy again at position 0 only)
}

size_t LayerKVCache::memory_usage() const { return k_codes_ ? bytes_ : 0; }

}  // namespace hs
