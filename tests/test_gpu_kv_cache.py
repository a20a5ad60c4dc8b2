"""GPU tests of the LayerKVCache mirror, written after the reference's own cache tests
(crates/hyprstream/src/runtime/kv_cache.rs:2240-2330): update/get shapes and positions, incremental
updates, overflow, clear and truncate -- plus what the reference cannot check: the values."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import kv_cache as kc
from hyprstream_amd import workloads as wl
from gpu_util import DEV

pytestmark = pytest.mark.gpu


def randn(stream, *shape, dtype=torch.bfloat16):
    x = wl.philox(stream).standard_normal(shape).astype(np.float32)
    return torch.from_numpy(x).to(DEV).to(dtype)


@pytest.mark.parametrize("quant", [kc.INT8, kc.FP8])
def test_layer_kv_cache_quantized(quant):
    """test_layer_kv_cache_quantized_int8 (kv_cache.rs:2277-2330): prompt of 100 tokens, get, one more token."""
    cache = kc.LayerKVCache(1000, quant)
    B, S, H, D = 1, 100, 2, 64
    keys, values = randn(1, B, S, H, D, dtype=torch.float32), randn(2, B, S, H, D, dtype=torch.float32)
    cache.update(keys, values, 0)
    assert cache.seq_pos == S
    ck, cv = cache.get()
    assert list(ck.shape) == [B, S, H, D] and list(cv.shape) == [B, S, H, D]
    ck2, _ = cache.get()
    assert torch.equal(ck, ck2)
    nk, nv = randn(3, B, 1, H, D, dtype=torch.float32), randn(4, B, 1, H, D, dtype=torch.float32)
    cache.update(nk, nv, S)
    fk, fv = cache.get()
    assert list(fk.shape) == [B, S + 1, H, D] and cache.seq_pos == S + 1
    # values: what get() returns is the oracle's dequantized view rounded to bf16
    full_k = torch.cat([keys, nk], 1).cpu().numpy()
    if quant == kc.INT8:
        want = oracle.dequant_int8(*oracle.quant_int8(full_k))
    else:
        s = oracle.fp8_calibrate(keys.cpu().numpy())  # scales come from the prompt
        want = oracle.dequant_fp8(oracle.quant_fp8(full_k, s), s)
    assert torch.equal(fk.cpu(), torch.from_numpy(want).bfloat16())
    assert torch.equal(fk[:, :S], ck)  # the history is untouched by the incremental update


def test_update_positions_overflow_and_empty_get():
    cache = kc.LayerKVCache(16, kc.INT8)
    with pytest.raises(kc.CacheError, match="Cache is empty"):
        cache.get()
    k = randn(5, 2, 10, 2, 128)
    cache.update(k, k, 0)
    with pytest.raises(kc.CacheError, match="Cache overflow: trying to cache 10 tokens starting at position 10"):
        cache.update(k, k, 10)
    assert cache.seq_pos == 10  # a failed update leaves the cache as it was
    with pytest.raises(kc.CacheError, match="Expected 4D tensor"):
        cache.update(k[0], k[0], 0)
    with pytest.raises(kc.CacheError, match="does not match"):
        cache.update(randn(6, 2, 1, 4, 128), randn(6, 2, 1, 4, 128), 10)
    assert cache.is_initialized() and cache.memory_usage() == 2 * 2 * 2 * 16 * 128 + 2 * 2 * 2 * 16 * 4


def test_fresh_prompt_restarts_and_truncate_keeps_prefix():
    cache = kc.LayerKVCache(64, kc.INT8)
    a, b = randn(7, 1, 20, 2, 128), randn(8, 1, 5, 2, 128)
    cache.update(a, a, 0)
    k20, _ = cache.get()
    cache.truncate_to(12)  # per-token scales: truncation is a position move, the prefix survives bit for bit
    assert cache.seq_pos == 12
    k12, _ = cache.get()
    assert torch.equal(k12, k20[:, :12])
    cache.truncate_to(30)  # pos >= seq_pos: nothing to do
    assert cache.seq_pos == 12
    cache.update(b, b, 0)  # start_pos == 0: a fresh prompt replaces the cache
    assert cache.seq_pos == 5
    cache.clear()
    assert cache.seq_pos == 0 and not cache.is_initialized() and cache.memory_usage() == 0
    cache.update(b, b, 0)  # usable again after clear()
    assert cache.seq_pos == 5


@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("quant", [kc.INT8, kc.FP8])
def test_attention_through_the_cache_object(quant, D):
    """update + get + attention as LlamaAttention::forward strings them together (llama.rs:605-636)."""
    B, T, Hq, Hkv = 2, 150, 8, 2
    sig = 1.0 if quant == kc.INT8 else 0.5
    k, v = randn(9, B, T, Hkv, D) * sig, randn(10, B, T, Hkv, D) * sig
    q = randn(11, B, Hq, D)
    cache = kc.LayerKVCache(256, quant)
    cache.update(k[:, :T - 1], v[:, :T - 1], 0)
    out = cache.decode_step(q, k[:, T - 1:], v[:, T - 1:], 1 / np.sqrt(D))
    torch.cuda.synchronize()
    assert cache.seq_pos == T
    again = cache.decode_attention(q, 1 / np.sqrt(D))
    torch.cuda.synchronize()
    assert torch.equal(out, again)
    kf, vf = k.float().cpu().numpy(), v.float().cpu().numpy()
    if quant == kc.INT8:
        kc_, ks_ = oracle.quant_int8(kf)
        vc_, vs_ = oracle.quant_int8(vf)
        fmt = oracle.FMT_INT8
    else:
        ks_, vs_ = oracle.fp8_calibrate(kf[:, :T - 1]), oracle.fp8_calibrate(vf[:, :T - 1])
        kc_, vc_ = oracle.quant_fp8(kf, ks_), oracle.quant_fp8(vf, vs_)
        fmt = oracle.FMT_FP8
    want = oracle.decode_attn(q.float().cpu().numpy(), kc_, vc_, ks_, vs_, fmt, np.full(B, T, np.int32), 1 / np.sqrt(D))
    d = np.abs(out.float().cpu().numpy() - want)
    assert d.max() < 2e-2 and d.mean() < 2e-3


@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("fmt", ["int8", "fp8"])
def test_chunked_prefill_then_decode_through_the_cache_object(fmt, D):
    B, Hq, Hkv, C = 1, 8, 2, 96
    cache = kc.LayerKVCache(512, kc.INT8 if fmt == "int8" else kc.FP8)
    q, k, v = randn(12, B, 2 * C, Hq, D), randn(13, B, 2 * C, Hkv, D), randn(14, B, 2 * C, Hkv, D)
    o0 = cache.prefill(q[:, :C], k[:, :C], v[:, :C], 0, 1 / np.sqrt(D))
    o1 = cache.prefill(q[:, C:], k[:, C:], v[:, C:], C, 1 / np.sqrt(D))
    torch.cuda.synchronize()
    assert cache.seq_pos == 2 * C
    kd, vd = cache.get(torch.float32)
    kn, vn = k.float().cpu().numpy(), v.float().cpu().numpy()
    want0 = oracle.prefill_attn(q[:, :C].float().cpu().numpy(), kn[:, :C], vn[:, :C], None, None, oracle.FMT_DENSE,
                                np.array([C], np.int32), 1 / np.sqrt(D))
    k1 = np.concatenate([kd[:, :C].cpu().numpy(), kn[:, C:]], 1)
    v1 = np.concatenate([vd[:, :C].cpu().numpy(), vn[:, C:]], 1)
    want1 = oracle.prefill_attn(q[:, C:].float().cpu().numpy(), k1, v1, None, None, oracle.FMT_DENSE,
                                np.array([2 * C], np.int32), 1 / np.sqrt(D))
    for got, want in ((o0, want0), (o1, want1)):
        d = np.abs(got.float().cpu().numpy() - want)
        assert d.max() < 2e-2 and d.mean() < 2e-3
    with pytest.raises(kc.CacheError, match="past the cached tokens"):
        cache.prefill(q[:, :C], k[:, :C], v[:, :C], 300, 1 / np.sqrt(D))


def test_decode_step_where_the_split_has_more_chunks_than_at_capacity():
    """The workspace of a cache object is sized once for its capacity, the step is launched with the length reached.
    Capacity 20000 with one sequence of 8 KV heads: chunks of 384 tokens = 53 slots at the capacity, but a sequence
    of 13569..16384 tokens is cut into 256-token chunks, up to 64 of them.  The step must run there (it returned a
    workspace error when the size was taken from the split at the capacity) and match the oracle."""
    from hyprstream_amd import bindings as hb
    B, T, Hq, Hkv, D = 1, 14000, 32, 8, 128
    assert hb.decode_num_chunks(B, Hkv, T) > hb.decode_num_chunks(B, Hkv, 20000)
    k, v = randn(21, B, T, Hkv, D), randn(22, B, T, Hkv, D)
    q = randn(23, B, Hq, D)
    cache = kc.LayerKVCache(20000, kc.INT8)
    cache.update(k[:, :T - 1], v[:, :T - 1], 0)
    out = cache.decode_step(q, k[:, T - 1:], v[:, T - 1:], 1 / np.sqrt(D))
    torch.cuda.synchronize()
    assert cache.seq_pos == T
    kf, vf = k.float().cpu().numpy(), v.float().cpu().numpy()
    kc_, ks_ = oracle.quant_int8(kf)
    vc_, vs_ = oracle.quant_int8(vf)
    want = oracle.decode_attn(q.float().cpu().numpy(), kc_, vc_, ks_, vs_, oracle.FMT_INT8, np.full(B, T, np.int32),
                              1 / np.sqrt(D))
    d = np.abs(out.float().cpu().numpy() - want)
    assert d.max() < 2e-2 and d.mean() < 2e-3
    # the same through a paged cache of that capacity
    pool = kc.BlockPool(128, Hkv, D)   # 55 K blocks + 55 V blocks of 256 tokens
    paged = kc.PagedLayerKVCache(20000, pool, 1)
    paged.update(k, v, 0)
    got = paged.decode_attention(q, 1 / np.sqrt(D))
    torch.cuda.synchronize()
    assert torch.equal(got, out)
    paged.close()


@pytest.mark.parametrize("fmt", ["int8", "fp8"])
def test_prompt_scratch_of_the_cache_object(fmt):
    """hs_cache_enable_prompt_scratch: one sequence prefilled in 512-token chunks through the cache object with the
    key-split workspace and the bf16 copy of the prompt.  Outputs agree with a cache object that has neither (within
    the rounding of another summation order and operand format) and with the oracle; the codes and scales are the same
    bits; the copy follows the prompt (active after each chunk in sequence), retires at a decode step, and a new
    prompt at position 0 begins it again; the decode step after the prompt is the same either way."""
    B, Hq, Hkv, D, C, T = 1, 32, 8, 128, 512, 2048
    q, k, v = randn(31, B, T, Hq, D), randn(32, B, T, Hkv, D), randn(33, B, T, Hkv, D)
    qt = kc.INT8 if fmt == "int8" else kc.FP8
    plain, fast = kc.LayerKVCache(T + 64, qt), kc.LayerKVCache(T + 64, qt)
    fast.enable_prompt_scratch(T)
    assert not fast.prompt_copy_active
    outs = []
    for lo in range(0, T, C):
        o_plain = plain.prefill(q[:, lo:lo + C], k[:, lo:lo + C], v[:, lo:lo + C], lo, 1 / np.sqrt(D))
        o_fast = fast.prefill(q[:, lo:lo + C], k[:, lo:lo + C], v[:, lo:lo + C], lo, 1 / np.sqrt(D))
        torch.cuda.synchronize()
        assert fast.prompt_copy_active and not plain.prompt_copy_active
        d = (o_fast.float() - o_plain.float()).abs().max().item()
        assert d <= 2.0 ** -6 * max(1.0, o_plain.float().abs().max().item()), (lo, d)
        outs.append(o_fast)
    kp, vp = plain.get(torch.float32)
    kf, vf = fast.get(torch.float32)
    assert torch.equal(kp, kf) and torch.equal(vp, vf)  # dequantized views of identical codes and scales
    # last chunk against the oracle over the dequantized history
    lo = T - C
    kn, vn = k.float().cpu().numpy(), v.float().cpu().numpy()
    k1 = np.concatenate([kp[:, :lo].cpu().numpy(), kn[:, lo:]], 1)
    v1 = np.concatenate([vp[:, :lo].cpu().numpy(), vn[:, lo:]], 1)
    want = oracle.prefill_attn(q[:, lo:].float().cpu().numpy(), k1, v1, None, None, oracle.FMT_DENSE, np.array([T], np.int32),
                               1 / np.sqrt(D))
    d = np.abs(outs[-1].float().cpu().numpy() - want)
    assert d.max() < 2e-2 and d.mean() < 2e-3
    # a decode step retires the copy; the step itself does not depend on it
    qd, kd, vd = randn(34, B, Hq, D), randn(35, B, 1, Hkv, D), randn(36, B, 1, Hkv, D)
    s_plain = plain.decode_step(qd, kd, vd, 1 / np.sqrt(D))
    s_fast = fast.decode_step(qd, kd, vd, 1 / np.sqrt(D))
    torch.cuda.synchronize()
    assert torch.equal(s_plain, s_fast) and not fast.prompt_copy_active
    # a chunk that does not start at 0 now reads the codes (and is then the plain call, bit for bit, split aside)
    fast.truncate_to(C)
    plain.truncate_to(C)
    o_plain = plain.prefill(q[:, C:2 * C], k[:, C:2 * C], v[:, C:2 * C], C, 1 / np.sqrt(D))
    o_fast = fast.prefill(q[:, C:2 * C], k[:, C:2 * C], v[:, C:2 * C], C, 1 / np.sqrt(D))
    torch.cuda.synchronize()
    assert not fast.prompt_copy_active
    assert (o_fast.float() - o_plain.float()).abs().max().item() <= 2.0 ** -7 * max(1.0, o_plain.float().abs().max().item())
    # a new prompt begins the copy again
    fast.prefill(q[:, :C], k[:, :C], v[:, :C], 0, 1 / np.sqrt(D))
    torch.cuda.synchronize()
    assert fast.prompt_copy_active
    fast.drop_prompt_scratch()
    assert not fast.prompt_copy_active
