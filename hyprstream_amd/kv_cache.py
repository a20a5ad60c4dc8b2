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
    "hs_cache_decode_step", "hs_cache_prefill",
]

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
        for f in ("hs_cache_seq_pos", "hs_cache_max_seq_len", "hs_cache_memory_usage"):
            getattr(L, f).restype = ctypes.c_int64
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


class LayerKVCache:
    def __init__(self, max_seq_len, quant_type=INT8):
        self._h = ctypes.c_void_p(lib().hs_cache_create(max_seq_len, quant_type))
        if not self._h:
            raise ValueError("bad max_seq_len / quant_type")

    def __del__(self):
        if getattr(self, "_h", None):
            lib().hs_cache_destroy(self._h)
            self._h = None

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
