// KV-cache compatibility identity: host-side mirror of the part of the reference's kv_compat module that decides
// whether cached K/V may be reused (crates/hyprstream/src/runtime/kv_compat.rs:84-560, 836-1130).
//
// A descriptor is an ordered list of named fields; its fingerprint is the SHA-256 of the reference's canonical byte
// framing (little-endian fixed widths, length-prefixed strings, tag-prefixed options, kv_compat.rs:458-520), so a
// fingerprint computed here equals the one the Rust side computes for the same values.  The storage formats of this
// library are KvQuantMode variants of their own ("int8-token", "fp8-e4m3fn-head"): a cache written in one format
// has a different fingerprint from one written in another, or in the reference's blockwise "int8", and is refused.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace hs {

constexpr uint32_t kKvCompatFormatVersion = 3;  // KV_COMPAT_FORMAT_VERSION, kv_compat.rs:84
constexpr uint64_t kKvBlockSizeDefault = 256;   // KV_BLOCK_SIZE_DEFAULT, kv_compat.rs:91

// KvQuantMode (kv_compat.rs:215-237) plus the two device formats of this library.
enum class KvQuantMode : int { None = 0, Int8 = 1, Nf4 = 2, Fp4 = 3, Int8Token = 4, Fp8E4m3fnHead = 5 };
const char *kv_quant_canonical_str(KvQuantMode m);  // nullptr for an unknown value

// CacheReuseDecision (kv_compat.rs:1087-1101)
enum class CacheReuseDecision : int { Reuse = 0, StampFresh = 1, DiscardAndRecompute = 2 };

void sha256(const uint8_t *data, size_t n, uint8_t out[32]);

class KvCompatDescriptor {
public:
    KvCompatDescriptor();
    // Setters by field name (the names of the Rust struct's fields; weights.base_revision and
    // weights.adapter_generation, moe.* for the nested ones).  Return false for an unknown name or a kind mismatch.
    bool set_uint(const std::string &field, uint64_t v);                 // integers, bools, f32 bit patterns
    bool set_opt_uint(const std::string &field, bool has, uint64_t v);   // Option<u32> / Option<usize>
    bool set_str(const std::string &field, const char *v);               // nullptr clears an Option<String>
    void add_layer_type(const std::string &v) { layer_types_.push_back(v); }
    void set_rope_scaling(const char *rope_type, float factor);          // nullptr = None
    bool set_kv_quant(int mode);
    bool set_dtype(const std::string &name);                             // KvDtype::from_name, kv_compat.rs:179-189

    bool is_authoritatively_complete() const;                            // kv_compat.rs:426-428
    void fingerprint(uint8_t out[32]) const;                             // kv_compat.rs:440-442, 533-543
    // First differing field in the reference's fixed order, "" if compatible (check_compatibility, kv_compat.rs:836-1080).
    std::string check_against(const KvCompatDescriptor &observed) const;

private:
    struct Slot {
        const char *name;
        int kind;
        uint64_t u = 0;
        bool has = false;
        std::string s;
    };
    std::vector<Slot> slots_;  // canonical order
    std::vector<std::string> layer_types_;
    bool has_rope_scaling_ = false;
    std::string rope_type_;
    uint32_t rope_factor_bits_ = 0;
    KvQuantMode kv_quant_ = KvQuantMode::None;
    Slot *find(const std::string &name);
    const Slot *find(const std::string &name) const;
    void canonical_bytes(std::vector<uint8_t> &out) const;
};

// decide_cache_reuse, kv_compat.rs:1118-1128: fail-closed.
CacheReuseDecision decide_cache_reuse(const uint8_t *expected32, const uint8_t *stored32, bool cache_is_empty);

}  // namespace hs
