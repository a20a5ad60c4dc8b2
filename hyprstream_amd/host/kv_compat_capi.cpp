// extern "C" view of hs::KvCompatDescriptor (include/hs_kv_cache.h).
#include <cstring>
#include <new>

#include "../../include/hs_kv_cache.h"
#include "kv_compat.hpp"

struct hs_compat {
    hs::KvCompatDescriptor d;
};

extern "C" {

hs_compat *hs_compat_create(void) { return new (std::nothrow) hs_compat(); }
void hs_compat_destroy(hs_compat *c) { delete c; }

int hs_compat_set_uint(hs_compat *c, const char *field, uint64_t value) {
    return c && field && c->d.set_uint(field, value) ? HS_OK : HS_ERR_INVALID_ARGUMENT;
}
int hs_compat_set_opt_uint(hs_compat *c, const char *field, int has_value, uint64_t value) {
    return c && field && c->d.set_opt_uint(field, has_value != 0, value) ? HS_OK : HS_ERR_INVALID_ARGUMENT;
}
int hs_compat_set_str(hs_compat *c, const char *field, const char *value) {
    return c && field && c->d.set_str(field, value) ? HS_OK : HS_ERR_INVALID_ARGUMENT;
}
int hs_compat_add_layer_type(hs_compat *c, const char *value) {
    if (!c || !value) return HS_ERR_INVALID_ARGUMENT;
    c->d.add_layer_type(value);
    return HS_OK;
}
int hs_compat_set_rope_scaling(hs_compat *c, const char *rope_type, float factor) {
    if (!c) return HS_ERR_INVALID_ARGUMENT;
    c->d.set_rope_scaling(rope_type, factor);
    return HS_OK;
}
int hs_compat_set_kv_quant(hs_compat *c, int mode) {
    return c && c->d.set_kv_quant(mode) ? HS_OK : HS_ERR_INVALID_ARGUMENT;
}
int hs_compat_is_authoritatively_complete(const hs_compat *c) { return c && c->d.is_authoritatively_complete(); }
int hs_compat_fingerprint(const hs_compat *c, uint8_t out32[32]) {
    if (!c || !out32) return HS_ERR_INVALID_ARGUMENT;
    c->d.fingerprint(out32);
    return HS_OK;
}
int hs_compat_check(const hs_compat *expected, const hs_compat *observed, char *field, size_t field_cap) {
    if (!expected || !observed) return -1;
    const std::string f = expected->d.check_against(observed->d);
    if (field && field_cap) {
        std::strncpy(field, f.c_str(), field_cap - 1);
        field[field_cap - 1] = 0;
    }
    return f.empty() ? 0 : 1;
}
int hs_compat_decide_reuse(const uint8_t *expected32, const uint8_t *stored32, int cache_is_empty) {
    return (int)hs::decide_cache_reuse(expected32, stored32, cache_is_empty != 0);
}
const char *hs_kv_quant_mode_str(int mode) { return hs::kv_quant_canonical_str((hs::KvQuantMode)mode); }
int hs_kv_quant_mode_of(int quant_type) {
    switch (quant_type) {
        case HS_KV_NONE: return HS_KVQ_NONE;
        case HS_KV_INT8: return HS_KVQ_INT8_TOKEN;
        case HS_KV_FP8: return HS_KVQ_FP8_E4M3FN_HEAD;
        default: return -1;
    }
}

}  // extern "C"
