"""CPU-only checks of the C-ABI library: it loads, exports every symbol the header declares, and its
host-side validation rejects bad arguments before anything touches a GPU."""
import ctypes
import os
import re

import pytest

from hyprstream_amd import bindings as hb

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header="hs_attn.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    return sorted(set(re.findall(r"HS_API\s+[\w\s\*]+?\b(hs_\w+)\s*\(", text)))


def test_header_declares_what_bindings_expect():
    decl = declared_symbols()
    assert decl, "no HS_API declarations found"
    for name in hb.EXPORTS:
        assert name in decl


def _c_arity(header):
    """name -> number of parameters, from the header text."""
    text = re.sub(r"/\*.*?\*/", " ", open(os.path.join(ROOT, "include", header)).read(), flags=re.S)
    out = {}
    for m in re.finditer(r"HS_API\s+[^;{]*?\b(hs_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        args = " ".join(m.group(2).split())
        out[m.group(1)] = 0 if args in ("void", "") else args.count(",") + 1
    return out


def _rust_arity():
    text = open(os.path.join(ROOT, "hs-attn-sys", "src", "bindings.rs")).read()
    out = {}
    for m in re.finditer(r"pub fn (hs_\w+)\(([^)]*)\)", text):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if not args else args.count(":")
    return out


def test_rust_bindings_match_the_headers_name_for_name_and_in_arity():
    """hs-attn-sys/src/bindings.rs is what a maintainer compiles in hyprstream's tree (no rustc here): every entry point
    of both headers must be declared there with the same number of parameters, and nothing else."""
    want = dict(_c_arity("hs_attn.h"))
    want.update(_c_arity("hs_kv_cache.h"))
    got = _rust_arity()
    assert len(want) > 70
    assert sorted(got) == sorted(want), (sorted(set(want) - set(got)), sorted(set(got) - set(want)))
    assert {n: a for n, a in got.items() if want[n] != a} == {}
    text = open(os.path.join(ROOT, "hs-attn-sys", "src", "bindings.rs")).read()
    assert "pub const HS_ATTN_ABI_VERSION: c_int = %d;" % hb.lib().hs_attn_abi_version() in text
    # the structs carry every field of the C structs, in order
    for struct, cls in (("hs_kv_layout", hb.KvLayout), ("hs_qk_prologue", hb.QkPrologue)):
        body = re.search(r"pub struct %s \{(.*?)\}" % struct, text, flags=re.S).group(1)
        assert re.findall(r"pub (\w+):", body) == [f[0] for f in cls._fields_]


def test_rust_wrappers_call_only_declared_bindings():
    lib_rs = open(os.path.join(ROOT, "hs-attn-sys", "src", "lib.rs")).read()
    used = set(re.findall(r"bindings::(hs_\w+)\(", lib_rs))
    assert used and used <= set(_rust_arity())


def test_library_exports_every_declared_symbol():
    L = hb.lib()
    missing = [s for s in declared_symbols() if not hasattr(L, s)]
    assert not missing, "declared in include/hs_attn.h but not exported: %s" % missing


def test_abi_version_and_empty_error():
    assert hb.lib().hs_attn_abi_version() == 8


def test_layout_struct_matches_header_size():
    # 4 x int64 + 2 x int32 + 2 pointers + int64 + 2 x int32 + 3 pointers + int64 + 2 x int32 + pointer + int64 + 2 x int32
    assert ctypes.sizeof(hb.KvLayout) == 4 * 8 + 2 * 4 + 2 * 8 + 8 + 2 * 4 + 3 * 8 + 8 + 2 * 4 + 8 + 8 + 2 * 4


def _call_quant(layout, B=1, S=1, Hkv=2, D=128, start_pos=0, fake=0x1000):
    p = ctypes.c_void_p(fake)
    return hb.lib().hs_kv_quantize_int8(p, p, hb.HS_BF16, p, p, p, p, ctypes.byref(layout), None,
                                        ctypes.c_int32(start_pos), B, S, Hkv, D, None)


def test_quantize_rejects_overflow_like_the_reference_cache():
    """LayerKVCache::update fails with "Cache overflow" when start_pos + S > max_seq_len
    (kv_cache.rs:1288-1294); the ABI reports the same condition before launching anything."""
    lay = hb.contiguous_layout(2, 16, 128)
    rc = _call_quant(lay, S=4, start_pos=13)
    assert rc == hb.HS_ERR_OVERFLOW
    assert b"Cache overflow" in hb.lib().hs_attn_last_error()


def test_quantize_rejects_bad_head_dim_and_null():
    lay = hb.contiguous_layout(2, 16, 96)
    assert _call_quant(lay, D=96) == hb.HS_ERR_INVALID_ARGUMENT
    lay = hb.contiguous_layout(2, 16, 128)
    assert _call_quant(lay, fake=0) == hb.HS_ERR_INVALID_ARGUMENT
    lay.code_stride_head = 16 * 128 - 16  # heads would overlap
    assert _call_quant(lay) == hb.HS_ERR_INVALID_ARGUMENT


def test_decode_rejects_small_workspace_and_bad_gqa():
    L = hb.lib()
    lay = hb.contiguous_layout(2, 512, 128)
    p = ctypes.c_void_p(0x1000)
    need = L.hs_decode_attn_workspace_bytes(3, 8, 2, 128, 512)
    assert need > 0 and need % 256 == 0
    rc = L.hs_decode_attn_int8(p, p, p, p, p, ctypes.byref(lay), p, p, p, ctypes.c_size_t(need - 256), 3, 8, 2, 128,
                               512, ctypes.c_float(0.088), None)
    assert rc == hb.HS_ERR_WORKSPACE
    rc = L.hs_decode_attn_int8(p, p, p, p, p, ctypes.byref(lay), p, p, p, ctypes.c_size_t(need), 3, 7, 2, 128, 512,
                               ctypes.c_float(0.088), None)
    assert rc == hb.HS_ERR_INVALID_ARGUMENT
    rc = L.hs_decode_attn_int8(p, p, p, p, p, ctypes.byref(lay), p, p, p, ctypes.c_size_t(need), 3, 8, 2, 128, 513,
                               ctypes.c_float(0.088), None)
    assert rc == hb.HS_ERR_OVERFLOW


# ------------------------------------------------------------------ host mirror (libhs_kv_cache.so)
def test_cache_library_exports_every_declared_symbol():
    from hyprstream_amd import kv_cache as kc
    L = kc.lib()
    decl = declared_symbols("hs_kv_cache.h")
    assert sorted(decl) == sorted(kc.EXPORTS)
    missing = [s for s in decl if not hasattr(L, s)]
    assert not missing, missing


def test_cache_host_logic_without_a_gpu():
    """Bookkeeping and error paths of LayerKVCache that return before any device work."""
    from hyprstream_amd import kv_cache as kc
    L = kc.lib()
    assert not L.hs_cache_create(0, kc.INT8) and not L.hs_cache_create(16, 7)
    c = ctypes.c_void_p(L.hs_cache_create(100, kc.INT8))
    assert L.hs_cache_seq_pos(c) == 0 and L.hs_cache_max_seq_len(c) == 100
    assert not L.hs_cache_is_initialized(c) and L.hs_cache_memory_usage(c) == 0
    assert L.hs_cache_quant_type(c) == kc.INT8
    p = ctypes.c_void_p(0x1000)
    # get() on an empty cache: "Cache is empty" (kv_cache.rs:1500-1502)
    assert L.hs_cache_get_dense(c, p, p, hb.HS_BF16, None) != hb.HS_OK
    assert L.hs_cache_last_error(c) == b"Cache is empty"
    # update past max_seq_len: "Cache overflow: ..." (kv_cache.rs:1288-1294)
    rc = L.hs_cache_update(c, p, p, hb.HS_BF16, 1, 10, 8, 128, ctypes.c_int64(95), None)
    assert rc == hb.HS_ERR_OVERFLOW
    assert L.hs_cache_last_error(c) == (b"Cache overflow: trying to cache 10 tokens starting at position 95, "
                                        b"but max_seq_len is 100")
    assert L.hs_cache_seq_pos(c) == 0
    L.hs_cache_truncate_to(c, ctypes.c_int64(5))  # nothing to truncate
    L.hs_cache_clear(c)
    assert L.hs_cache_seq_pos(c) == 0
    L.hs_cache_destroy(c)
    n = ctypes.c_void_p(L.hs_cache_create(10, kc.NONE))
    assert L.hs_cache_update(n, p, p, hb.HS_BF16, 1, 1, 8, 128, ctypes.c_int64(0), None) == hb.HS_ERR_INVALID_ARGUMENT
    L.hs_cache_destroy(n)


def test_chunk_policy_unsplit_for_uniform_and_split_for_ragged_hint():
    """The headline shape stays one launch; a batch whose mean length is well below its maximum is cut into
    balanced token ranges (at most 17 partials per sequence), and the workspace the library asks for covers that."""
    B, Hq, Hkv, D, T = 64, 32, 8, 128, 8192
    assert hb.decode_num_chunks(B, Hkv, T) == 1
    assert hb.decode_num_chunks(B, Hkv, T, B * T) == 1            # hint says uniform
    n = hb.decode_num_chunks(B, Hkv, T, B * 4352)                 # U[512, 8192] has mean 4352
    assert 2 <= n <= 17
    assert hb.decode_num_chunks(2, Hkv, T) > 1                    # few sequences: split for occupancy as before
    per_chunk = B * Hq * (D + 2) * 4
    assert hb.decode_workspace_bytes(B, Hq, Hkv, D, T) >= 17 * per_chunk >= n * per_chunk


@pytest.mark.parametrize("cap", [2508, 10000, 20000, 40960, 100000, 128000])
def test_workspace_sized_for_the_capacity_covers_every_shorter_call(cap):
    """A cache object sizes its workspace once, for its capacity, and then calls with the length it has reached
    (LayerKVCache::decode_step passes seq_pos).  The split's slot count is not monotone in the length (chunks are
    rounded up to 128 tokens), so the size the library asks for must bound every shorter call, with any hint."""
    L = hb.lib()
    Hq, D = 32, 128
    for B, Hkv in ((1, 8), (1, 4), (2, 2), (4, 8), (64, 8)):
        have = L.hs_decode_attn_workspace_bytes(B, Hq, Hkv, D, cap)
        per_slot = B * Hq * (D + 2) * 4
        step = 1 if cap <= 20000 else 7
        worst = 0
        for n in list(range(1, cap + 1, step)) + [cap]:
            worst = max(worst, L.hs_decode_attn_num_chunks(B, Hkv, n, 0),
                        L.hs_decode_attn_num_chunks(B, Hkv, n, ctypes.c_int64(max(1, B * n // 2))))
            # the check launch_decode itself makes is against the size for THIS call's length: it must not ask for
            # more than the capacity's size
            if n % 97 == 0 or n == cap:
                assert L.hs_decode_attn_workspace_bytes(B, Hq, Hkv, D, n) <= have, (B, Hkv, n)
        assert worst * per_slot <= have, (B, Hkv, worst, have // per_slot)


def test_format_names_are_distinct_and_stable():
    """The names feed the reference's compatibility fingerprint (kv_compat.rs:215-237): the device formats must
    not collide with each other or with the reference's own "int8" / "nf4" / "fp4"."""
    from hyprstream_amd import kv_cache as kc
    L = kc.lib()
    names = [L.hs_kv_quant_canonical_str(i) for i in (kc.NONE, kc.INT8, kc.FP8)]
    assert names == [b"none", b"int8-token", b"fp8-e4m3fn-head"]
    assert not set(names) & {b"int8", b"nf4", b"fp4"}
    assert L.hs_kv_quant_canonical_str(9) is None



def test_workspace_sizes_are_host_arithmetic():
    """The workspace functions need no GPU: sizes a caller can plan with."""
    # chunked delta rule: per 64-token chunk 32,768 B per (sequence, k-head) and 42,240 B per (sequence, v-head)
    assert hb.deltanet_chunked_workspace_bytes(4, 4096, 16, 32) == 64 * 4 * 32 * 13312  # per chunk and (sequence, v-head)
    assert hb.deltanet_chunked_workspace_bytes(1, 1, 1, 1) == 13312
    assert hb.deltanet_chunked_workspace_bytes(1, 65, 2, 4) == 2 * 4 * 13312
    assert hb.deltanet_chunked_workspace_bytes(0, 64, 1, 1) == 0
    # with the norm: the fp32 output rows behind the factors (256-byte aligned)
    assert hb.deltanet_chunked_gated_norm_workspace_bytes(1, 65, 2, 4) == 2 * 4 * 13312 + 65 * 4 * 128 * 4
    assert hb.deltanet_chunked_gated_norm_workspace_bytes(0, 64, 1, 1) == 0
    # decode: room for (D + 2) floats per (sequence, query head, chunk), a multiple of 256 bytes, growing with head_dim
    small, big = hb.decode_workspace_bytes(64, 32, 8, 128, 8192), hb.decode_workspace_bytes(64, 32, 8, 256, 8192)
    assert small % 256 == 0 and big % 256 == 0 and big > small >= 64 * 32 * 130 * 4


def test_chunked_delta_rule_rejects_bad_arguments_before_launching():
    p = ctypes.c_void_p(0x1000)
    L = hb.lib()
    call = lambda nk, nv, dk, ws, nbytes: L.hs_deltanet_forward_chunked(p, p, p, p, p, p, p, 1, 64, nk, nv, dk, 128, ctypes.c_float(1.0), 1,
                                                                      ws, ctypes.c_size_t(nbytes), None)
    assert call(3, 4, 128, p, 1 << 30) == hb.HS_ERR_INVALID_ARGUMENT      # nv not a multiple of nk
    assert call(2, 4, 64, p, 1 << 30) == hb.HS_ERR_INVALID_ARGUMENT       # dk must be 128
    assert call(2, 4, 128, p, 100) == hb.HS_ERR_WORKSPACE                 # too small
    assert b"workspace" in L.hs_attn_last_error()
    assert call(2, 4, 128, None, 0) == hb.HS_ERR_WORKSPACE                # none at all
    assert call(2, 4, 128, ctypes.c_void_p(0x1004), 1 << 30) == hb.HS_ERR_INVALID_ARGUMENT  # misaligned


def test_prefill_rejects_bad_arguments_before_launching():
    """Argument checks of the prefill entry points are host code: head_dim, head grouping, capacity (with the
    reference's overflow message), and the per-sequence history array of the ragged form."""
    L = hb.lib()
    p = ctypes.c_void_p(0x1000)
    f = ctypes.c_float(0.088)

    def call(lay, hist, B=2, S=8, Hq=8, Hkv=2, D=128, q=p):
        return L.hs_prefill_attn_int8(q, p, p, p, p, p, p, ctypes.byref(lay), hist, p, B, S, Hq, Hkv, D, f, 1, None)

    assert call(hb.contiguous_layout(2, 64, 96), 0, D=96) == hb.HS_ERR_INVALID_ARGUMENT
    lay = hb.contiguous_layout(2, 64, 128)
    assert call(lay, 0, Hq=7) == hb.HS_ERR_INVALID_ARGUMENT          # Hq is not a multiple of Hkv
    assert call(lay, -1) == hb.HS_ERR_INVALID_ARGUMENT
    assert call(lay, 0, q=None) == hb.HS_ERR_INVALID_ARGUMENT
    assert call(lay, 60) == hb.HS_ERR_OVERFLOW and b"Cache overflow" in L.hs_attn_last_error()
    rc = L.hs_prefill_attn_int8_ragged(p, p, p, p, p, p, p, ctypes.byref(lay), None, 16, p, 2, 8, 8, 2, 128, f, 1, None)
    assert rc == hb.HS_ERR_INVALID_ARGUMENT and b"hist_lens" in L.hs_attn_last_error()
    rc = L.hs_prefill_attn_int8_ragged(p, p, p, p, p, p, p, ctypes.byref(lay), p, 60, p, 2, 8, 8, 2, 128, f, 1, None)
    assert rc == hb.HS_ERR_OVERFLOW                                   # the bound, not the array, is what the host checks
    assert call(lay, 0, B=0) == hb.HS_OK and call(lay, 0, S=0) == hb.HS_OK  # empty problems are not an error


def _call_prefill(layout, hist_len=0, B=1, S=64, Hq=4, Hkv=1, D=128, write=1, fake=0x1000):
    p = ctypes.c_void_p(fake)
    out = ctypes.c_void_p(fake + 0x100000)
    return hb.lib().hs_prefill_attn_int8(p, p, p, p, p, p, p, ctypes.byref(layout), ctypes.c_int32(hist_len), out, B, S, Hq,
                                         Hkv, D, ctypes.c_float(0.1), write, None)


def test_prefill_scratch_sizes_and_contracts_without_a_gpu():
    """The two optional prefill buffers: their size functions, and the checks that refuse a bad one before any launch."""
    L = hb.lib()
    # key-split workspace: grows with the tokens of a call, zero for shapes the kernels do not serve
    small = L.hs_prefill_attn_split_workspace_bytes(1, 512, 32, 8, 128)
    assert small > 0 and small % 256 == 0
    assert L.hs_prefill_attn_split_workspace_bytes(1, 1024, 32, 8, 128) > small
    assert L.hs_prefill_attn_split_workspace_bytes(1, 512, 32, 8, 96) == 0
    assert L.hs_prefill_attn_split_workspace_bytes(1, 512, 30, 8, 128) == 0
    # bf16 copy: 512 bytes per token and kv-head at head_dim 128, whole 64-token steps
    assert L.hs_prefill_shadow_bytes(4, 8, 128, 4096) == 4 * 8 * 4096 * 512
    assert L.hs_prefill_shadow_bytes(1, 1, 128, 65) == 128 * 512
    assert L.hs_prefill_shadow_bytes(1, 1, 64, 64) == 0
    lay = hb.contiguous_layout(1, 256, 128)
    lay.prefill_shadow, lay.prefill_shadow_bytes, lay.prefill_shadow_tokens = 0x200000, 128 * 512, 100
    assert _call_prefill(lay) == hb.HS_ERR_INVALID_ARGUMENT            # tokens not a multiple of 64
    assert b"prefill_shadow_tokens" in L.hs_attn_last_error()
    lay.prefill_shadow_tokens = 128
    assert _call_prefill(lay, hist_len=128) == hb.HS_ERR_INVALID_ARGUMENT  # 128 + 64 tokens do not fit
    lay.prefill_shadow_bytes = 64 * 512
    assert _call_prefill(lay, hist_len=64) == hb.HS_ERR_WORKSPACE
    lay.prefill_shadow_bytes = 128 * 512
    assert _call_prefill(lay, hist_len=64, write=0) == hb.HS_ERR_INVALID_ARGUMENT  # history, nothing cached
    lay.prefill_shadow = 0x200010
    assert _call_prefill(lay, hist_len=64) == hb.HS_ERR_INVALID_ARGUMENT   # alignment
    # key split: too small a workspace, a count out of range
    lay = hb.contiguous_layout(1, 256, 128)
    lay.prefill_split_workspace, lay.prefill_split_workspace_bytes, lay.prefill_key_splits = 0x300000, 4096, 4
    assert _call_prefill(lay, hist_len=128) == hb.HS_ERR_WORKSPACE
    lay.prefill_key_splits = 9
    assert _call_prefill(lay, hist_len=128) == hb.HS_ERR_INVALID_ARGUMENT
