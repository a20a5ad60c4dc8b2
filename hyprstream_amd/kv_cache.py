"""ctypes view of libhs_kv_cache.so, the C++ LayerKVCache mirror (hyprstream_amd/host/).

Plumbing for tests and examples: method names and error behaviour follow the reference's
LayerKVCache (crates/hyprstream/src/runtime/kv_cache.rs:1027-1891); tensors are torch tensors
on the GPU, whose pointers go straight through to the C API in include/hs_kv_cache.h.
"""
import ctypes
import os

from . import bindings as hb

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libhs_kv_cache.so")
NONE, INT8, FP8 = 0, 1, 2

EXPORTS = [
    "hs_cache_create", "hs_cache_destroy", "hs_cache_last_error", "hs_cache_update", "hs_cache_get_dense",
    "hs_cache_get_view", "hs_cache_seq_pos", "hs_cache_max_seq_len", "hs_cache_clear", "hs_cache_truncate_to",
    "hs_cache_is_initialized", "hs_cache_memory_usage", "hs_cache_quant_type", "hs_cache_decode_attention",
    "hs_cache_decode_step", "hs_cache_prefill", "hs_cache_enable_prompt_scratch", "hs_cache_drop_prompt_scratch",
    "hs_cache_prompt_copy_active", "hs_paged_cache_prefill", "hs_kv_quant_canonical_str",
    "hs_pool_create", "hs_pool_create_format", "hs_pool_quant_type", "hs_pool_destroy", "hs_pool_last_error", "hs_pool_allocate", "hs_pool_free", "hs_pool_owner_of",
    "hs_pool_used_blocks", "hs_pool_free_block_count", "hs_pool_total_blocks", "hs_pool_used_memory",
    "hs_paged_cache_create", "hs_paged_cache_destroy", "hs_paged_cache_last_error", "hs_paged_cache_update",
    "hs_paged_cache_get_dense", "hs_paged_cache_decode_attention", "hs_paged_cache_clear", "hs_paged_cache_truncate_to",
    "hs_paged_cache_seq_pos", "hs_paged_cache_num_blocks", "hs_paged_batch_decode_step",
    "hs_compat_create", "hs_compat_destroy", "hs_compat_set_uint", "hs_compat_set_opt_uint", "hs_compat_set_str",
    "hs_compat_add_layer_type", "hs_compat_set_rope_scaling", "hs_compat_set_kv_quant",
    "hs_compat_is_authoritatively_complete", "hs_compat_fingerprint", "hs_compat_check", "hs_compat_decide_reuse",
    "hs_kv_quant_mode_str", "hs_kv_quant_mode_of",
]
BLOCK_SIZE = 256  # tokens per pool block
STATELESS, SESSION, TRAINING = 0, 1, 2  # owner kinds

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("libhs_kv_cache.so not built: run `python -m hyprstream_amd.build`")
        hb.lib()  # dependency, loaded first so the loader finds it whatever the search path
        L = ctypes.CDLL(LIB_PATH)
        L.hs_cache_create.restype = ctypes.c_void_p
        L.hs_cache_create.argtypes = [ctypes.c_int64, ctypes.c_int]
        L.hs_cache_last_error.restype = ctypes.c_char_p
        for f in ("hs_cache_seq_pos", "hs_cache_max_seq_len", "hs_cache_memory_usage", "hs_pool_used_blocks",
                  "hs_pool_free_block_count", "hs_pool_total_blocks", "hs_pool_used_memory", "hs_paged_cache_seq_pos",
                  "hs_paged_cache_num_blocks"):
            getattr(L, f).restype = ctypes.c_int64
        L.hs_kv_quant_canonical_str.restype = ctypes.c_char_p
        L.hs_pool_create.restype = ctypes.c_void_p
        L.hs_pool_create.argtypes = [ctypes.c_int64, ctypes.c_int32, ctypes.c_int32]
        L.hs_pool_create_format.restype = ctypes.c_void_p
        L.hs_pool_create_format.argtypes = [ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_int]
        L.hs_pool_last_error.restype = ctypes.c_char_p
        L.hs_paged_cache_create.restype = ctypes.c_void_p
        L.hs_paged_cache_create.argtypes = [ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_uint64, ctypes.c_char_p]
        L.hs_paged_cache_last_error.restype = ctypes.c_char_p
        L.hs_pool_allocate.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_uint64, ctypes.c_char_p,
                                       ctypes.POINTER(ctypes.c_int32)]
        L.hs_pool_free.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_uint64, ctypes.c_char_p, ctypes.c_int32]
        L.hs_compat_create.restype = ctypes.c_void_p
        L.hs_compat_destroy.argtypes = [ctypes.c_void_p]
        L.hs_compat_set_uint.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_uint64]
        L.hs_compat_set_opt_uint.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_uint64]
        L.hs_compat_set_str.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p]
        L.hs_compat_add_layer_type.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
        L.hs_compat_set_rope_scaling.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_float]
        L.hs_compat_set_kv_quant.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.hs_compat_is_authoritatively_complete.argtypes = [ctypes.c_void_p]
        L.hs_compat_fingerprint.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
        L.hs_compat_check.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t]
        L.hs_compat_decide_reuse.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int]
        L.hs_kv_quant_mode_str.restype = ctypes.c_char_p
        for f in EXPORTS:
            if f != "hs_cache_create":
                fn = getattr(L, f)
                if fn.argtypes is None:
                    fn.argtypes = None
        _lib = L
    return _lib


class CacheError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(msg)
        self.code = code


class _Handle:
    """Owner of a C handle.  The destroy function is taken at construction and kept on the object: at interpreter exit
    this module's globals, lib() among them, may already be gone when the last objects are collected."""
    _h = None
    _destroy = None

    def close(self):
        h, destroy = self._h, self._destroy
        if h and destroy:
            destroy(h)
            self._h = None

    __del__ = close


class LayerKVCache(_Handle):
    def __init__(self, max_seq_len, quant_type=INT8):
        self._destroy = lib().hs_cache_destroy
        self._h = ctypes.c_void_p(lib().hs_cache_create(max_seq_len, quant_type))
        if not self._h:
            raise ValueError("bad max_seq_len / quant_type")

    def _check(self, rc):
        if rc != hb.HS_OK:
            raise CacheError(rc, lib().hs_cache_last_error(self._h).decode())

    @property
    def seq_pos(self):
        return lib().hs_cache_seq_pos(self._h)

    @property
    def max_seq_len(self):
        return lib().hs_cache_max_seq_len(self._h)

    def update(self, new_keys, new_values, start_pos):
        if new_keys.dim() != 4:
            raise CacheError(hb.HS_ERR_INVALID_ARGUMENT, "Expected 4D tensor for keys, got %s" % list(new_keys.shape))
        B, S, H, D = new_keys.shape
        k, v = new_keys.contiguous(), new_values.contiguous()
        self._check(lib().hs_cache_update(self._h, hb._ptr(k), hb._ptr(v), hb._dtype_code(k), B, S, H, D,
                                          ctypes.c_int64(start_pos), hb._stream()))

    def get(self, dtype=None):
        """Dense (K, V) [B, seq_pos, Hkv, D], as the reference's get() returns them."""
        import torch
        B, H, D = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int32()
        self._check(lib().hs_cache_get_view(self._h, None, None, None, None, None, ctypes.byref(B), ctypes.byref(H),
                                            ctypes.byref(D)))
        dtype = dtype or torch.bfloat16
        k = torch.empty(B.value, self.seq_pos, H.value, D.value, dtype=dtype, device="cuda")
        v = torch.empty_like(k)
        self._check(lib().hs_cache_get_dense(self._h, hb._ptr(k), hb._ptr(v), hb._dtype_code(k), hb._stream()))
        return k, v

    def clear(self):
        lib().hs_cache_clear(self._h)

    def truncate_to(self, pos):
        lib().hs_cache_truncate_to(self._h, ctypes.c_int64(pos))

    def is_initialized(self):
        return bool(lib().hs_cache_is_initialized(self._h))

    def memory_usage(self):
        return lib().hs_cache_memory_usage(self._h)

    def quant_type(self):
        return lib().hs_cache_quant_type(self._h)

    def decode_attention(self, q, softmax_scale):
        import torch
        out = torch.empty_like(q)
        self._check(lib().hs_cache_decode_attention(self._h, hb._ptr(q), hb._ptr(out), q.shape[1],
                                                    ctypes.c_float(softmax_scale), hb._stream()))
        return out

    def decode_step(self, q, k_new, v_new, softmax_scale):
        import torch
        out = torch.empty_like(q)
        k, v = k_new.contiguous(), v_new.contiguous()
        self._check(lib().hs_cache_decode_step(self._h, hb._ptr(q), hb._ptr(k), hb._ptr(v), hb._dtype_code(k),
                                               hb._ptr(out), q.shape[1], ctypes.c_float(softmax_scale), hb._stream()))
        return out

    def prefill(self, q, new_keys, new_values, start_pos, softmax_scale):
        import torch
        B, S, Hq, D = q.shape
        out = torch.empty_like(q)
        k, v = new_keys.contiguous(), new_values.contiguous()
        self._check(lib().hs_cache_prefill(self._h, hb._ptr(q.contiguous()), hb._ptr(k), hb._ptr(v), hb._ptr(out), B, S, Hq,
                                           k.shape[2], D, ctypes.c_int64(start_pos), ctypes.c_float(softmax_scale),
                                           hb._stream()))
        return out

    def enable_prompt_scratch(self, max_prompt_tokens):
        """Opt in to the key split of small prefill calls and to the bf16 copy of the prompt (hs_cache_enable_prompt_scratch)."""
        lib().hs_cache_enable_prompt_scratch(self._h, ctypes.c_int64(max_prompt_tokens))

    def drop_prompt_scratch(self):
        lib().hs_cache_drop_prompt_scratch(self._h)

    @property
    def prompt_copy_active(self):
        return bool(lib().hs_cache_prompt_copy_active(self._h))


# ------------------------------------------------------------------------------------------- paged mode
def _owner(owner):
    """owner: int -> Stateless(id); str -> Session(name); (name, id) -> Training."""
    if isinstance(owner, int):
        return STATELESS, owner, None
    if isinstance(owner, str):
        return SESSION, 0, owner.encode()
    name, ident = owner
    return TRAINING, ident, name.encode()


class BlockPoolExhausted(CacheError):
    """Fail-soft: the pool has no free block; retry once other sequences have released theirs."""


class BlockPool(_Handle):
    """BlockPool of the reference (kv_cache.rs:508-676) over int8 blocks; bookkeeping works without a GPU."""

    def __init__(self, num_blocks, num_kv_heads, head_dim, quant_type=INT8):
        self._destroy = lib().hs_pool_destroy
        self._h = ctypes.c_void_p(lib().hs_pool_create_format(num_blocks, num_kv_heads, head_dim, quant_type))
        if not self._h:
            raise ValueError("bad pool shape")
        self.num_kv_heads, self.head_dim = num_kv_heads, head_dim

    def _check(self, rc):
        if rc != hb.HS_OK:
            cls = BlockPoolExhausted if rc == hb.HS_ERR_POOL_EXHAUSTED else CacheError
            raise cls(rc, lib().hs_pool_last_error(self._h).decode())

    def allocate(self, owner):
        kind, ident, name = _owner(owner)
        out = ctypes.c_int32(-1)
        self._check(lib().hs_pool_allocate(self._h, kind, ident, name, ctypes.byref(out)))
        return out.value

    def free(self, owner, block_id):
        kind, ident, name = _owner(owner)
        self._check(lib().hs_pool_free(self._h, kind, ident, name, block_id))

    def owner_of(self, block_id):
        kind, ident = ctypes.c_int(), ctypes.c_uint64()
        name = ctypes.create_string_buffer(256)
        if not lib().hs_pool_owner_of(self._h, ctypes.c_int32(block_id), ctypes.byref(kind), ctypes.byref(ident), name,
                                      ctypes.c_size_t(256)):
            return None
        if kind.value == STATELESS:
            return ident.value
        if kind.value == SESSION:
            return name.value.decode()
        return (name.value.decode(), ident.value)

    def used_blocks(self):
        return lib().hs_pool_used_blocks(self._h)

    def free_block_count(self):
        return lib().hs_pool_free_block_count(self._h)

    def total_blocks(self):
        return lib().hs_pool_total_blocks(self._h)

    def used_memory(self):
        return lib().hs_pool_used_memory(self._h)


class PagedLayerKVCache(_Handle):
    """LayerKVCache::new_paged (kv_cache.rs:1100-1120): one sequence, int8 blocks from a shared pool."""

    def __init__(self, max_seq_len, pool, owner):
        kind, ident, name = _owner(owner)
        self.pool = pool  # keeps the Python pool object alive as long as the cache
        self._destroy = lib().hs_paged_cache_destroy
        self._h = ctypes.c_void_p(lib().hs_paged_cache_create(max_seq_len, pool._h, kind, ident, name))
        if not self._h:
            raise ValueError("bad max_seq_len / pool")

    def _check(self, rc):
        if rc != hb.HS_OK:
            cls = BlockPoolExhausted if rc == hb.HS_ERR_POOL_EXHAUSTED else CacheError
            raise cls(rc, lib().hs_paged_cache_last_error(self._h).decode())

    @property
    def seq_pos(self):
        return lib().hs_paged_cache_seq_pos(self._h)

    @property
    def num_blocks(self):
        return lib().hs_paged_cache_num_blocks(self._h)

    def update(self, new_keys, new_values, start_pos):
        if new_keys.dim() != 4 or new_keys.shape[0] != 1:
            raise CacheError(hb.HS_ERR_INVALID_ARGUMENT, "Expected [1, S, H, D] keys, got %s" % list(new_keys.shape))
        k, v = new_keys.contiguous(), new_values.contiguous()
        self._check(lib().hs_paged_cache_update(self._h, hb._ptr(k), hb._ptr(v), hb._dtype_code(k), k.shape[1],
                                                ctypes.c_int64(start_pos), hb._stream()))

    def get(self, dtype=None):
        import torch
        dtype = dtype or torch.bfloat16
        k = torch.empty(1, max(self.seq_pos, 0), self.pool.num_kv_heads, self.pool.head_dim, dtype=dtype, device="cuda")
        v = torch.empty_like(k)
        self._check(lib().hs_paged_cache_get_dense(self._h, hb._ptr(k), hb._ptr(v), hb._dtype_code(k), hb._stream()))
        return k, v

    def decode_attention(self, q, softmax_scale):
        import torch
        out = torch.empty_like(q)
        self._check(lib().hs_paged_cache_decode_attention(self._h, hb._ptr(q), hb._ptr(out), q.shape[1],
                                                          ctypes.c_float(softmax_scale), hb._stream()))
        return out

    def prefill(self, q, new_keys, new_values, start_pos, softmax_scale):
        import torch
        _, S, Hq, _ = q.shape
        k, v = new_keys.contiguous(), new_values.contiguous()
        out = torch.empty_like(q)
        self._check(lib().hs_paged_cache_prefill(self._h, hb._ptr(q.contiguous()), hb._ptr(k), hb._ptr(v), hb._ptr(out), S, Hq,
                                                 ctypes.c_int64(start_pos), ctypes.c_float(softmax_scale), hb._stream()))
        return out

    def clear(self):
        lib().hs_paged_cache_clear(self._h)

    def truncate_to(self, pos):
        lib().hs_paged_cache_truncate_to(self._h, ctypes.c_int64(pos))


def paged_batch_decode_step(pool, rows, q, k_new, v_new, softmax_scale):
    """One launch for all rows: each caches its new token and attends its own history.  q [n, Hq, D] bf16."""
    import torch
    n = len(rows)
    arr = (ctypes.c_void_p * n)(*[r._h for r in rows])
    out = torch.empty_like(q)
    k, v = k_new.contiguous(), v_new.contiguous()
    rc = lib().hs_paged_batch_decode_step(pool._h, arr, n, hb._ptr(q), hb._ptr(k), hb._ptr(v), hb._dtype_code(k),
                                          hb._ptr(out), q.shape[1], ctypes.c_float(softmax_scale), hb._stream())
    pool._check(rc)
    return out



# ---------------------------------------------------------------- cache identity (kv_compat.rs)
KVQ_NONE, KVQ_INT8, KVQ_NF4, KVQ_FP4, KVQ_INT8_TOKEN, KVQ_FP8_E4M3FN_HEAD = range(6)
REUSE, STAMP_FRESH, DISCARD_AND_RECOMPUTE = 0, 1, 2


def f32_bits(x):
    import struct
    return struct.unpack("<I", struct.pack("<f", x))[0]


class KvCompatDescriptor(_Handle):
    """ctypes handle on hs_compat; fields are set by the names of the reference's struct."""

    def __init__(self, **fields):
        self._destroy = lib().hs_compat_destroy
        self._h = ctypes.c_void_p(lib().hs_compat_create())
        self.set(**fields)

    def set(self, **fields):
        L = lib()
        for name, v in fields.items():
            key = name.replace("__", ".").encode()
            if name == "kv_quant":
                rc = L.hs_compat_set_kv_quant(self._h, v)
            elif name == "layer_types":
                rc = 0
                for t in v:
                    rc |= L.hs_compat_add_layer_type(self._h, t.encode())
            elif name == "rope_scaling":
                rc = L.hs_compat_set_rope_scaling(self._h, None if v is None else v[0].encode(), 0.0 if v is None else v[1])
            elif isinstance(v, str) or (v is None and name == "tokenizer_hash"):
                rc = L.hs_compat_set_str(self._h, key, None if v is None else v.encode())
            elif isinstance(v, tuple):  # ("opt", value-or-None)
                rc = L.hs_compat_set_opt_uint(self._h, key, int(v[1] is not None), 0 if v[1] is None else v[1])
            else:
                rc = L.hs_compat_set_uint(self._h, key, int(v))
            if rc != 0:
                raise ValueError("bad field %s=%r" % (name, v))
        return self

    def fingerprint(self):
        buf = ctypes.create_string_buffer(32)
        assert lib().hs_compat_fingerprint(self._h, buf) == 0
        return buf.raw

    def is_authoritatively_complete(self):
        return bool(lib().hs_compat_is_authoritatively_complete(self._h))

    def check_against(self, observed):
        """None if compatible, else the first differing field."""
        buf = ctypes.create_string_buffer(64)
        rc = lib().hs_compat_check(self._h, observed._h, buf, 64)
        assert rc in (0, 1)
        return None if rc == 0 else buf.value.decode()


def decide_cache_reuse(expected, stored, cache_is_empty):
    return lib().hs_compat_decide_reuse(expected, stored, int(cache_is_empty))
