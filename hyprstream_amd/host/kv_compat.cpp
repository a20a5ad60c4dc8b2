// See kv_compat.hpp.  Plain C++17, no GPU.
#include "kv_compat.hpp"

#include <algorithm>
#include <cstring>

namespace hs {

const char *kv_quant_canonical_str(KvQuantMode m) {
    switch (m) {
        case KvQuantMode::None: return "none";
        case KvQuantMode::Int8: return "int8";
        case KvQuantMode::Nf4: return "nf4";
        case KvQuantMode::Fp4: return "fp4";
        case KvQuantMode::Int8Token: return "int8-token";
        case KvQuantMode::Fp8E4m3fnHead: return "fp8-e4m3fn-head";
    }
    return nullptr;
}

// ---------------------------------------------------------------- SHA-256 (FIPS 180-4)
namespace {
inline uint32_t rotr(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }
const uint32_t kK[64] = {
    0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01,
    0x243185be, 0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174, 0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc,
    0x2de92c6f, 0x4a7484aa, 0x5cb0a9dc, 0x76f988da, 0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147,
    0x06ca6351, 0x14292967, 0x27b70a85, 0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85,
    0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3, 0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070, 0x19a4c116, 0x1e376c08,
    0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f, 0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208,
    0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};

void compress(uint32_t h[8], const uint8_t *blk) {
    uint32_t w[64];
    for (int i = 0; i < 16; ++i)
        w[i] = (uint32_t)blk[4 * i] << 24 | (uint32_t)blk[4 * i + 1] << 16 | (uint32_t)blk[4 * i + 2] << 8 | blk[4 * i + 3];
    for (int i = 16; i < 64; ++i) {
        const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3);
        const uint32_t s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
        w[i] = w[i - 16] + s0 + w[i - 7] + s1;
    }
    uint32_t a = h[0], b = h[1], c = h[2], d = h[3], e = h[4], f = h[5], g = h[6], hh = h[7];
    for (int i = 0; i < 64; ++i) {
        const uint32_t S1 = rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25), ch = (e & f) ^ (~e & g);
        const uint32_t t1 = hh + S1 + ch + kK[i] + w[i];
        const uint32_t S0 = rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22), mj = (a & b) ^ (a & c) ^ (b & c);
        const uint32_t t2 = S0 + mj;
        hh = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + t2;
    }
    h[0] += a; h[1] += b; h[2] += c; h[3] += d; h[4] += e; h[5] += f; h[6] += g; h[7] += hh;
}
}  // namespace

void sha256(const uint8_t *data, size_t n, uint8_t out[32]) {
    uint32_t h[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
    size_t i = 0;
    for (; i + 64 <= n; i += 64) compress(h, data + i);
    uint8_t tail[128] = {0};
    const size_t rem = n - i;
    if (rem) std::memcpy(tail, data + i, rem);
    tail[rem] = 0x80;
    const size_t total = rem + 1 + 8 <= 64 ? 64 : 128;
    const uint64_t bits = (uint64_t)n * 8;
    for (int k = 0; k < 8; ++k) tail[total - 1 - k] = (uint8_t)(bits >> (8 * k));
    compress(h, tail);
    if (total == 128) compress(h, tail + 64);
    for (int k = 0; k < 8; ++k) {
        out[4 * k] = (uint8_t)(h[k] >> 24); out[4 * k + 1] = (uint8_t)(h[k] >> 16);
        out[4 * k + 2] = (uint8_t)(h[k] >> 8); out[4 * k + 3] = (uint8_t)h[k];
    }
}

// ---------------------------------------------------------------- descriptor
namespace {
enum Kind { U32, U64, USIZE, BOOL, STR, CANON_STR, OPT_U32, OPT_USIZE, OPT_STR, LAYER_TYPES, ROPE_SCALING, DTYPE, KV_QUANT };

// The fields in the order the reference hashes them (write_canonical, kv_compat.rs:458-520), which is also the order
// in which check_compatibility compares them (kv_compat.rs:836-1080).
const struct { const char *name; Kind kind; } kOrder[] = {
    {"format_version", U32},
    {"weights.base_revision", STR}, {"weights.adapter_generation", U64},
    {"model_name", STR}, {"architecture", STR}, {"model_version", U32},
    {"num_hidden_layers", USIZE}, {"num_attention_heads", USIZE}, {"num_key_value_heads", USIZE}, {"head_dim", USIZE},
    {"hidden_size", USIZE},
    {"use_qk_norm", BOOL}, {"partial_rotary_factor_bits", OPT_U32}, {"layer_types", LAYER_TYPES},
    {"linear_key_head_dim", USIZE}, {"linear_value_head_dim", USIZE}, {"linear_num_key_heads", USIZE},
    {"linear_num_value_heads", USIZE}, {"linear_conv_kernel_dim", USIZE},
    {"rms_norm_eps_bits", U32}, {"layer_norm_eps_bits", OPT_U32}, {"hidden_activation", CANON_STR},
    {"scale_embeddings", BOOL}, {"query_pre_attn_scalar_bits", OPT_U32},
    {"moe.is_moe", BOOL}, {"moe.num_experts", USIZE}, {"moe.num_experts_per_tok", USIZE},
    {"moe.moe_intermediate_size", USIZE}, {"moe.shared_expert_intermediate_size", USIZE},
    {"sliding_window", OPT_USIZE}, {"rope_local_base_freq_bits", OPT_U32},
    {"rope_theta_bits", U32}, {"rope_scaling", ROPE_SCALING}, {"max_position_embeddings", USIZE},
    {"dtype", DTYPE}, {"kv_quant", KV_QUANT}, {"block_size", USIZE}, {"max_context", USIZE},
    {"vocab_size", USIZE}, {"tokenizer_hash", OPT_STR},
};

std::string canon(const std::string &s) {  // trim + ASCII lowercase (canon_str, kv_compat.rs:1192-1195)
    size_t a = 0, b = s.size();
    while (a < b && (unsigned char)s[a] <= ' ') ++a;
    while (b > a && (unsigned char)s[b - 1] <= ' ') --b;
    std::string r = s.substr(a, b - a);
    for (char &c : r)
        if (c >= 'A' && c <= 'Z') c = (char)(c - 'A' + 'a');
    return r;
}
void put_le(std::vector<uint8_t> &o, uint64_t v, int bytes) {
    for (int i = 0; i < bytes; ++i) o.push_back((uint8_t)(v >> (8 * i)));
}
void put_str(std::vector<uint8_t> &o, const std::string &s) {
    put_le(o, s.size(), 8);
    o.insert(o.end(), s.begin(), s.end());
}
}  // namespace

KvCompatDescriptor::KvCompatDescriptor() {
    for (const auto &f : kOrder) {
        Slot s;
        s.name = f.name;
        s.kind = f.kind;
        slots_.push_back(s);
    }
    set_uint("format_version", kKvCompatFormatVersion);
    find("dtype")->s = "bfloat16";  // KvDtype's #[default] (kv_compat.rs:165-174); every other field defaults to zero / empty / None
}

KvCompatDescriptor::Slot *KvCompatDescriptor::find(const std::string &name) {
    for (auto &s : slots_)
        if (name == s.name) return &s;
    return nullptr;
}
const KvCompatDescriptor::Slot *KvCompatDescriptor::find(const std::string &name) const {
    for (const auto &s : slots_)
        if (name == s.name) return &s;
    return nullptr;
}

bool KvCompatDescriptor::set_uint(const std::string &field, uint64_t v) {
    Slot *s = find(field);
    if (!s || !(s->kind == U32 || s->kind == U64 || s->kind == USIZE || s->kind == BOOL)) return false;
    if (s->kind == U32 && v > 0xffffffffull) return false;
    s->u = s->kind == BOOL ? (v != 0) : v;
    return true;
}
bool KvCompatDescriptor::set_opt_uint(const std::string &field, bool has, uint64_t v) {
    Slot *s = find(field);
    if (!s || !(s->kind == OPT_U32 || s->kind == OPT_USIZE)) return false;
    if (s->kind == OPT_U32 && v > 0xffffffffull) return false;
    s->has = has;
    s->u = has ? v : 0;
    return true;
}
bool KvCompatDescriptor::set_str(const std::string &field, const char *v) {
    Slot *s = find(field);
    if (!s) return false;
    if (s->kind == DTYPE) return v && set_dtype(v);
    if (s->kind == OPT_STR) {
        s->has = v != nullptr;
        s->s = v ? v : "";
        return true;
    }
    if (s->kind != STR && s->kind != CANON_STR) return false;
    if (!v) return false;
    s->s = s->kind == CANON_STR ? canon(v) : std::string(v);
    return true;
}
void KvCompatDescriptor::set_rope_scaling(const char *rope_type, float factor) {
    has_rope_scaling_ = rope_type != nullptr;
    rope_type_ = rope_type ? canon(rope_type) : "";  // RopeScalingFp::new, kv_compat.rs:257-262
    std::memcpy(&rope_factor_bits_, &factor, 4);
    if (!rope_type) rope_factor_bits_ = 0;
}
bool KvCompatDescriptor::set_kv_quant(int mode) {
    if (!kv_quant_canonical_str((KvQuantMode)mode) || mode < 0) return false;
    kv_quant_ = (KvQuantMode)mode;
    return true;
}
bool KvCompatDescriptor::set_dtype(const std::string &name) {
    const std::string n = canon(name);
    std::string c = n;  // KvDtype::Other(name) hashes the canonicalised name itself
    if (n == "float64" || n == "double" || n == "f64") c = "float64";
    else if (n == "float32" || n == "float" || n == "f32") c = "float32";
    else if (n == "float16" || n == "half" || n == "fp16" || n == "f16") c = "float16";
    else if (n == "bfloat16" || n == "bf16") c = "bfloat16";
    find("dtype")->s = c;
    return true;
}

bool KvCompatDescriptor::is_authoritatively_complete() const {
    return !find("weights.base_revision")->s.empty() && find("tokenizer_hash")->has;
}

void KvCompatDescriptor::canonical_bytes(std::vector<uint8_t> &o) const {
    for (const Slot &s : slots_) {
        switch (s.kind) {
            case U32: put_le(o, s.u, 4); break;
            case U64: case USIZE: put_le(o, s.u, 8); break;
            case BOOL: o.push_back(s.u ? 1 : 0); break;
            case STR: put_str(o, s.s); break;
            case CANON_STR: put_str(o, canon(s.s)); break;
            case OPT_U32: o.push_back(s.has ? 1 : 0); if (s.has) put_le(o, s.u, 4); break;
            case OPT_USIZE: o.push_back(s.has ? 1 : 0); if (s.has) put_le(o, s.u, 8); break;
            case OPT_STR: o.push_back(s.has ? 1 : 0); if (s.has) put_str(o, s.s); break;
            case LAYER_TYPES:
                put_le(o, layer_types_.size(), 8);
                for (const auto &t : layer_types_) put_str(o, canon(t));
                break;
            case ROPE_SCALING:
                o.push_back(has_rope_scaling_ ? 1 : 0);
                if (has_rope_scaling_) {
                    put_str(o, rope_type_);
                    put_le(o, rope_factor_bits_, 4);
                }
                break;
            case DTYPE: put_str(o, s.s); break;
            case KV_QUANT: put_str(o, kv_quant_canonical_str(kv_quant_)); break;
        }
    }
}

void KvCompatDescriptor::fingerprint(uint8_t out[32]) const {
    std::vector<uint8_t> bytes;
    canonical_bytes(bytes);
    sha256(bytes.data(), bytes.size(), out);
}

std::string KvCompatDescriptor::check_against(const KvCompatDescriptor &obs) const {
    // nested structs are compared, and reported, as a whole (Weights, MoeRouting; kv_compat.rs:846-851, 962-967)
    auto report = [](const char *name) {
        std::string n = name;
        const size_t dot = n.find('.');
        if (dot == std::string::npos) return n;
        return n.substr(0, dot) == "moe" ? std::string("moe_routing") : n.substr(0, dot);
    };
    for (size_t i = 0; i < slots_.size(); ++i) {
        const Slot &a = slots_[i], &b = obs.slots_[i];
        bool same = true;
        switch (a.kind) {
            case LAYER_TYPES: {
                same = layer_types_.size() == obs.layer_types_.size();
                for (size_t k = 0; same && k < layer_types_.size(); ++k) same = canon(layer_types_[k]) == canon(obs.layer_types_[k]);
                break;
            }
            case ROPE_SCALING:
                same = has_rope_scaling_ == obs.has_rope_scaling_ &&
                       (!has_rope_scaling_ || (rope_type_ == obs.rope_type_ && rope_factor_bits_ == obs.rope_factor_bits_));
                break;
            case KV_QUANT: same = kv_quant_ == obs.kv_quant_; break;
            case CANON_STR: same = canon(a.s) == canon(b.s); break;
            default: same = a.u == b.u && a.has == b.has && a.s == b.s;
        }
        if (!same) return report(a.name);
    }
    return "";
}

CacheReuseDecision decide_cache_reuse(const uint8_t *expected32, const uint8_t *stored32, bool cache_is_empty) {
    if (expected32 && stored32 && std::memcmp(expected32, stored32, 32) == 0) return CacheReuseDecision::Reuse;
    if (expected32 && !stored32 && cache_is_empty) return CacheReuseDecision::StampFresh;
    return CacheReuseDecision::DiscardAndRecompute;
}

}  // namespace hs
