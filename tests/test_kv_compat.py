"""Cache identity: the host mirror of the reference's kv_compat module (no GPU).

Pins: SHA-256 against hashlib; the canonical framing against the reference's own pinned golden digest of its baseline
descriptor (kv_compat.rs:1262-1304, 1829-1841 `golden_digest_is_pinned`); the rejection order and the fail-closed reuse
matrix as the reference's tests state them (kv_compat.rs:1118-1128, 1640-1730, 1960-2013); and that the two device
formats of this library are storage modes of their own, so a cache of one is refused as another."""
import ctypes
import hashlib

import pytest

from hyprstream_amd import kv_cache as kc

GOLDEN_BASELINE = "2c1658e12b2935e6444e0503c35b9e36b3f2e941614d9078b445776eae5cc55c"  # kv_compat.rs:1833


def baseline(**over):
    """The reference tests' `baseline()` descriptor (kv_compat.rs:1262-1304)."""
    f = dict(weights__base_revision="sha256:my-model-weights", model_name="my-model", architecture="llama",
             model_version=1, num_hidden_layers=32, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
             hidden_size=4096, use_qk_norm=0, rms_norm_eps_bits=kc.f32_bits(1e-5), hidden_activation="silu",
             rope_theta_bits=kc.f32_bits(10000.0), max_position_embeddings=4096, dtype="bfloat16",
             kv_quant=kc.KVQ_NONE, block_size=256, max_context=4096, vocab_size=32000, tokenizer_hash="deadbeef")
    f.update(over)
    return kc.KvCompatDescriptor(**f)


def test_fingerprint_of_the_reference_baseline_is_its_pinned_golden_digest():
    assert baseline().fingerprint().hex() == GOLDEN_BASELINE


def test_fingerprint_is_sha256_of_the_canonical_framing():
    """An independent statement of the framing for the baseline: little-endian fixed widths, u64 length prefixes,
    one tag byte per Option (kv_compat.rs:458-520)."""
    u32 = lambda v: v.to_bytes(4, "little")
    u64 = lambda v: v.to_bytes(8, "little")
    st = lambda s: u64(len(s)) + s.encode()
    b = u32(3) + st("sha256:my-model-weights") + u64(0) + st("my-model") + st("llama") + u32(1)
    b += u64(32) + u64(32) + u64(8) + u64(128) + u64(4096)
    b += b"\x00" + b"\x00" + u64(0) + u64(0) * 5
    b += u32(kc.f32_bits(1e-5)) + b"\x00" + st("silu") + b"\x00" + b"\x00" + b"\x00" + u64(0) * 4 + b"\x00" + b"\x00"
    b += u32(kc.f32_bits(10000.0)) + b"\x00" + u64(4096)
    b += st("bfloat16") + st("none") + u64(256) + u64(4096) + u64(32000) + b"\x01" + st("deadbeef")
    assert hashlib.sha256(b).hexdigest() == GOLDEN_BASELINE
    assert baseline().fingerprint() == hashlib.sha256(b).digest()


@pytest.mark.parametrize("n", [0, 1, 55, 56, 63, 64, 65, 119, 120, 1000])
def test_sha256_padding_boundaries_through_a_string_field(n):
    # model_name of n bytes moves the message length across every padding case of SHA-256
    name = "x" * n
    d = kc.KvCompatDescriptor(model_name=name, tokenizer_hash=None)
    u32 = lambda v: v.to_bytes(4, "little")
    u64 = lambda v: v.to_bytes(8, "little")
    st = lambda s: u64(len(s)) + s.encode()
    b = u32(3) + st("") + u64(0) + st(name) + st("") + u32(0) + u64(0) * 5 + b"\x00\x00" + u64(0) + u64(0) * 5
    b += u32(0) + b"\x00" + st("") + b"\x00\x00\x00" + u64(0) * 4 + b"\x00\x00" + u32(0) + b"\x00" + u64(0)
    b += st("bfloat16") + st("none") + u64(0) + u64(0) + u64(0) + b"\x00"
    assert d.fingerprint() == hashlib.sha256(b).digest()


def test_device_formats_are_storage_modes_of_their_own():
    L = kc.lib()
    names = [L.hs_kv_quant_mode_str(m) for m in range(6)]
    assert names == [b"none", b"int8", b"nf4", b"fp4", b"int8-token", b"fp8-e4m3fn-head"]
    assert L.hs_kv_quant_mode_str(6) is None and L.hs_kv_quant_mode_str(-1) is None
    assert L.hs_kv_quant_mode_of(kc.INT8) == kc.KVQ_INT8_TOKEN and L.hs_kv_quant_mode_of(kc.FP8) == kc.KVQ_FP8_E4M3FN_HEAD
    assert L.hs_kv_quant_mode_of(kc.NONE) == kc.KVQ_NONE and L.hs_kv_quant_mode_of(9) == -1
    # the strings the cache objects report are the ones that are hashed
    assert L.hs_kv_quant_canonical_str(kc.INT8) == b"int8-token" and L.hs_kv_quant_canonical_str(kc.FP8) == b"fp8-e4m3fn-head"
    fps = {m: baseline(kv_quant=m).fingerprint() for m in range(6)}
    assert len(set(fps.values())) == 6
    assert fps[kc.KVQ_NONE].hex() == GOLDEN_BASELINE
    # cross-format reuse is refused, naming the field (kv_compat.rs:1038-1043)
    exp = baseline(kv_quant=kc.KVQ_INT8_TOKEN)
    for other in (kc.KVQ_INT8, kc.KVQ_FP8_E4M3FN_HEAD, kc.KVQ_NONE):
        assert exp.check_against(baseline(kv_quant=other)) == "kv_quant"
        assert kc.decide_cache_reuse(exp.fingerprint(), fps[other], False) == kc.DISCARD_AND_RECOMPUTE
    assert exp.check_against(baseline(kv_quant=kc.KVQ_INT8_TOKEN)) is None
    assert kc.decide_cache_reuse(exp.fingerprint(), fps[kc.KVQ_INT8_TOKEN], False) == kc.REUSE


CHANGES = [  # (field that is changed, kwargs, name reported) in the reference's comparison order
    ("format", dict(format_version=2), "format_version"),
    ("weights", dict(weights__adapter_generation=1), "weights"),
    ("model_name", dict(model_name="other"), "model_name"),
    ("architecture", dict(architecture="qwen2"), "architecture"),
    ("model_version", dict(model_version=2), "model_version"),
    ("layers", dict(num_hidden_layers=16), "num_hidden_layers"),
    ("heads", dict(num_attention_heads=16), "num_attention_heads"),
    ("kv_heads", dict(num_key_value_heads=4), "num_key_value_heads"),
    ("head_dim", dict(head_dim=64), "head_dim"),
    ("hidden", dict(hidden_size=2048), "hidden_size"),
    ("qk_norm", dict(use_qk_norm=1), "use_qk_norm"),
    ("partial_rotary", dict(partial_rotary_factor_bits=("opt", kc.f32_bits(0.25))), "partial_rotary_factor_bits"),
    ("layer_types", dict(layer_types=["full_attention", "linear_attention"]), "layer_types"),
    ("linear", dict(linear_num_value_heads=32), "linear_num_value_heads"),
    ("rms_eps", dict(rms_norm_eps_bits=kc.f32_bits(1e-6)), "rms_norm_eps_bits"),
    ("ln_eps", dict(layer_norm_eps_bits=("opt", kc.f32_bits(1e-5))), "layer_norm_eps_bits"),
    ("activation", dict(hidden_activation="gelu_pytorch_tanh"), "hidden_activation"),
    ("scale_emb", dict(scale_embeddings=1), "scale_embeddings"),
    ("qpas", dict(query_pre_attn_scalar_bits=("opt", kc.f32_bits(256.0))), "query_pre_attn_scalar_bits"),
    ("moe", dict(moe__is_moe=1, moe__num_experts=8), "moe_routing"),
    ("window", dict(sliding_window=("opt", 1024)), "sliding_window"),
    ("local_freq", dict(rope_local_base_freq_bits=("opt", kc.f32_bits(10000.0))), "rope_local_base_freq_bits"),
    ("theta", dict(rope_theta_bits=kc.f32_bits(500000.0)), "rope_theta_bits"),
    ("scaling", dict(rope_scaling=("linear", 2.0)), "rope_scaling"),
    ("max_pos", dict(max_position_embeddings=8192), "max_position_embeddings"),
    ("dtype", dict(dtype="float16"), "dtype"),
    ("kv_quant", dict(kv_quant=kc.KVQ_FP8_E4M3FN_HEAD), "kv_quant"),
    ("block", dict(block_size=128), "block_size"),
    ("ctx", dict(max_context=2048), "max_context"),
    ("vocab", dict(vocab_size=128256), "vocab_size"),
    ("tok", dict(tokenizer_hash="cafebabe"), "tokenizer_hash"),
]


@pytest.mark.parametrize("label,kw,reported", CHANGES, ids=[c[0] for c in CHANGES])
def test_every_authoritative_field_participates(label, kw, reported):
    """kv_compat.rs `every_authoritative_field_participates`: each field changes the fingerprint and is the reported mismatch."""
    base, changed = baseline(), baseline(**kw)
    assert base.fingerprint() != changed.fingerprint()
    assert base.check_against(changed) == reported
    assert changed.check_against(changed) is None


def test_first_difference_in_fixed_order_is_reported():
    a = baseline()
    b = baseline(head_dim=64, kv_quant=kc.KVQ_INT8_TOKEN, vocab_size=1)
    assert a.check_against(b) == "head_dim"
    c = baseline(kv_quant=kc.KVQ_INT8_TOKEN, vocab_size=1)
    assert a.check_against(c) == "kv_quant"


def test_canonicalisation_of_strings():
    # aliases must not disagree between hash and comparison (kv_compat.rs:1192-1215)
    a = baseline(hidden_activation="  SiLU ", dtype="BF16", layer_types=["GLOBAL", " local"])
    b = baseline(hidden_activation="silu", dtype="bfloat16", layer_types=["global", "local"])
    assert a.fingerprint() == b.fingerprint() and a.check_against(b) is None
    assert baseline(rope_scaling=(" Linear", 2.0)).fingerprint() == baseline(rope_scaling=("linear", 2.0)).fingerprint()
    # model_name is NOT canonicalised
    assert baseline(model_name="My-Model").check_against(baseline()) == "model_name"
    # an unknown dtype is keyed by its canonicalised name
    assert baseline(dtype="Float8_E4M3").fingerprint() == baseline(dtype="float8_e4m3").fingerprint()
    assert baseline(dtype="float8_e4m3").check_against(baseline()) == "dtype"


def test_reuse_decision_matrix_is_fail_closed():
    e, s = baseline().fingerprint(), baseline(max_context=1).fingerprint()
    assert kc.decide_cache_reuse(e, e, False) == kc.REUSE and kc.decide_cache_reuse(e, e, True) == kc.REUSE
    assert kc.decide_cache_reuse(e, s, False) == kc.DISCARD_AND_RECOMPUTE
    assert kc.decide_cache_reuse(e, s, True) == kc.DISCARD_AND_RECOMPUTE
    assert kc.decide_cache_reuse(e, None, True) == kc.STAMP_FRESH
    assert kc.decide_cache_reuse(e, None, False) == kc.DISCARD_AND_RECOMPUTE  # unstamped but populated
    for stored in (None, e):
        for empty in (True, False):
            assert kc.decide_cache_reuse(None, stored, empty) == kc.DISCARD_AND_RECOMPUTE  # no authoritative identity


def test_authoritative_completeness():
    assert baseline().is_authoritatively_complete()
    assert not baseline(tokenizer_hash=None).is_authoritatively_complete()
    assert not baseline(weights__base_revision="").is_authoritatively_complete()


def test_setters_reject_unknown_fields_and_wrong_kinds():
    L = kc.lib()
    d = baseline()
    assert L.hs_compat_set_uint(d._h, b"no_such_field", 1) != 0
    assert L.hs_compat_set_uint(d._h, b"model_name", 1) != 0
    assert L.hs_compat_set_str(d._h, b"head_dim", b"x") != 0
    assert L.hs_compat_set_uint(d._h, b"model_version", 1 << 40) != 0  # a u32
    assert L.hs_compat_set_kv_quant(d._h, 17) != 0
    assert L.hs_compat_check(None, d._h, None, 0) == -1
    assert d.fingerprint().hex() == GOLDEN_BASELINE  # rejected calls changed nothing
