"""hs_decode_attn_int8_static: the decode entry point that takes no workspace and allocates nothing (its split-K
partials live in a device array inside the library).  It must give the bits of hs_decode_attn_int8 -- same kernels,
same split -- on two calls in a row, the second smaller than the first (the array then still holds the first call's
partials), and stay within the attention tolerance of the oracle."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl

import gpu_util as gu

pytestmark = pytest.mark.gpu

TOL_MAX, TOL_MEAN = 2e-2, 2e-3


def _case(seed, B, Hq, Hkv, D, T, ragged):
    case = wl.decode_case(seed, B, Hq, Hkv, D, T, ragged=ragged, outliers=True, min_len=T // 3)
    cache = gu.DeviceCache(B, Hkv, T, D)
    cache.write(torch.from_numpy(case["k"]).to(gu.DEV).bfloat16(), torch.from_numpy(case["v"]).to(gu.DEV).bfloat16())
    return case, cache


def _both(case, cache, Hq, T, hint=0):
    B, Hkv, D = cache.B, cache.Hkv, cache.D
    q = gu.bf16_from_bits(case["q_bits"]).to(gu.DEV)
    lens = torch.from_numpy(case["seq_lens"]).to(gu.DEV)
    lay = hb.contiguous_layout(Hkv, T, D)
    lay.total_tokens_hint = hint
    scale = 1.0 / float(np.sqrt(D))
    want = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=gu.DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=gu.DEV)
    hb.decode_attn(q, cache.k_codes, cache.v_codes, cache.k_scales, cache.v_scales, lay, lens, want, ws, Hkv, T, scale)
    got = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=gu.DEV)
    hb.decode_attn_static(q, cache.k_codes, cache.v_codes, cache.k_scales, cache.v_scales, lay, lens, got, Hkv, T, scale)
    torch.cuda.synchronize()
    return got, want


def _check_oracle(case, cache, got, T):
    kc, vc, ks, vs = cache.canonical(T)
    ref = oracle.decode_attn(oracle.bf16_to_f32(case["q_bits"]), kc, vc, ks, vs, oracle.FMT_INT8, case["seq_lens"],
                             1.0 / np.sqrt(cache.D))
    d = np.abs(got.float().cpu().numpy() - ref)
    assert d.max() < TOL_MAX and d.mean() < TOL_MEAN, (d.max(), d.mean())


def test_two_calls_in_a_row_second_smaller():
    # first call: 3 sequences x 8 kv-heads, 4096 tokens -> split into many chunks per sequence (partials in the scratch)
    Hq, Hkv, D = 32, 8, 128
    case1, cache1 = _case(11, 3, Hq, Hkv, D, 4096, ragged=True)
    assert hb.decode_num_chunks(3, Hkv, 4096) > 1
    got1, want1 = _both(case1, cache1, Hq, 4096)
    assert torch.equal(got1.view(torch.int16), want1.view(torch.int16))
    _check_oracle(case1, cache1, got1, 4096)
    # second call, smaller in every respect (fewer sequences, fewer tokens, fewer chunks): stale partials must not leak
    case2, cache2 = _case(12, 2, Hq, Hkv, D, 1024, ragged=True)
    assert 1 < hb.decode_num_chunks(2, Hkv, 1024) < hb.decode_num_chunks(3, Hkv, 4096)
    got2, want2 = _both(case2, cache2, Hq, 1024)
    assert torch.equal(got2.view(torch.int16), want2.view(torch.int16))
    _check_oracle(case2, cache2, got2, 1024)
    # and the first shape again, after the smaller one
    got3, want3 = _both(case1, cache1, Hq, 4096)
    assert torch.equal(got3.view(torch.int16), want1.view(torch.int16))


def test_balanced_split_through_the_scratch_then_a_smaller_unhinted_call():
    """The ragged-batch split (token ranges over the whole batch, up to 17 partial slots per sequence, counted from a
    sequence's first range) through the built-in scratch: bits of hs_decode_attn_int8 under the same hint, and no stale
    balanced partial leaks into a smaller fixed-chunk call that follows."""
    Hq, Hkv, D, T = 32, 8, 128, 4096
    B = 24
    case = wl.decode_case(15, B, Hq, Hkv, D, T, ragged=True, outliers=True, min_len=64)
    case["seq_lens"][0] = T          # the longest sequence fixes max_seq_len; most are far shorter
    case["seq_lens"][1:] = np.minimum(case["seq_lens"][1:], T // 3)
    cache = gu.DeviceCache(B, Hkv, T, D)
    cache.write(torch.from_numpy(case["k"]).to(gu.DEV).bfloat16(), torch.from_numpy(case["v"]).to(gu.DEV).bfloat16())
    hint = int(case["seq_lens"].sum())
    assert hb.decode_num_chunks(B, Hkv, T, hint) > 1 and hb.decode_num_chunks(B, Hkv, T, hint) != hb.decode_num_chunks(B, Hkv, T)
    got, want = _both(case, cache, Hq, T, hint=hint)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    _check_oracle(case, cache, got, T)
    case2, cache2 = _case(16, 2, Hq, Hkv, D, 1024, ragged=True)
    got2, want2 = _both(case2, cache2, Hq, 1024)
    assert torch.equal(got2.view(torch.int16), want2.view(torch.int16))
    _check_oracle(case2, cache2, got2, 1024)


def test_a_call_on_another_stream_is_refused_while_the_first_stream_is_busy():
    """All calls on a GPU share one scratch array.  A call on a second (non-blocking) stream while the first stream
    still has work pending returns HS_ERR_BUSY and launches nothing; once the first stream has drained it is accepted
    and gives the same bits."""
    Hq, Hkv, D, T = 32, 8, 128, 2048
    case, cache = _case(17, 2, Hq, Hkv, D, T, ragged=True)
    assert hb.decode_num_chunks(2, Hkv, T) > 1
    want, _ = _both(case, cache, Hq, T)
    q = gu.bf16_from_bits(case["q_bits"]).to(gu.DEV)
    lens = torch.from_numpy(case["seq_lens"]).to(gu.DEV)
    lay = hb.contiguous_layout(Hkv, T, D)
    scale = 1.0 / float(np.sqrt(D))
    args = (q, cache.k_codes, cache.v_codes, cache.k_scales, cache.v_scales, lay, lens)
    out1 = torch.zeros(2, Hq, D, dtype=torch.bfloat16, device=gu.DEV)
    out2 = torch.full((2, Hq, D), 7.0, dtype=torch.bfloat16, device=gu.DEV)
    big = torch.randn(8192, 8192, device=gu.DEV)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()   # non-blocking streams, default priority
    with torch.cuda.stream(s1):
        for _ in range(20):
            big = big @ big * 1e-4                       # a few hundred ms of work ahead of the call
        hb.decode_attn_static(*args, out1, Hkv, T, scale)
    with torch.cuda.stream(s2):
        with pytest.raises(hb.HsError) as e:
            hb.decode_attn_static(*args, out2, Hkv, T, scale)
        assert e.value.code == hb.HS_ERR_BUSY and "another stream" in str(e.value)
    s1.synchronize()
    assert torch.all(out2 == 7.0)                        # the refused call launched nothing
    with torch.cuda.stream(s2):
        hb.decode_attn_static(*args, out2, Hkv, T, scale)  # the first stream has drained: accepted
    s2.synchronize()
    assert torch.equal(out1.view(torch.int16), want.view(torch.int16))
    assert torch.equal(out2.view(torch.int16), want.view(torch.int16))
    # back on the stream the rest of the suite uses
    torch.cuda.synchronize()
    got, _ = _both(case, cache, Hq, T)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_no_allocation_during_the_call():
    Hq, Hkv, D, T = 16, 4, 256, 2048
    case, cache = _case(13, 2, Hq, Hkv, D, T, ragged=False)
    _both(case, cache, Hq, T)  # the first call on the device looks the array's address up
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    q = gu.bf16_from_bits(case["q_bits"]).to(gu.DEV)
    lens = torch.from_numpy(case["seq_lens"]).to(gu.DEV)
    out = torch.empty(2, Hq, D, dtype=torch.bfloat16, device=gu.DEV)
    lay = hb.contiguous_layout(Hkv, T, D)
    free1, _ = torch.cuda.mem_get_info()
    for _ in range(5):
        hb.decode_attn_static(q, cache.k_codes, cache.v_codes, cache.k_scales, cache.v_scales, lay, lens, out, Hkv, T,
                              1.0 / float(np.sqrt(D)))
    torch.cuda.synchronize()
    free2, _ = torch.cuda.mem_get_info()
    assert free2 == free1  # device memory in use did not move while the entry point ran
    assert free1 <= free0


def test_single_chunk_shape_needs_no_scratch_and_matches():
    # 64 x 8 units: unsplit, the workgroup writes the output itself
    Hq, Hkv, D, T = 32, 8, 128, 512
    case, cache = _case(14, 64, Hq, Hkv, D, T, ragged=True)
    assert hb.decode_num_chunks(64, Hkv, T) == 1
    got, want = _both(case, cache, Hq, T)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_refuses_what_the_scratch_cannot_hold():
    # B * Hq * slots * (D + 2) * 4 bytes > 32 MiB: 48 sequences x 64 heads x 17 partial slots x 258 x 4 = 53.9 MB
    B, Hq, Hkv, D, T = 48, 64, 8, 256, 8192
    lay = hb.contiguous_layout(Hkv, T, D)
    lay.total_tokens_hint = B * 1024  # ragged hint -> balanced token ranges, up to 17 partials per sequence
    assert hb.decode_num_chunks(B, Hkv, T, lay.total_tokens_hint) == 17
    p = ctypes.c_void_p(0x1000)
    rc = hb.lib().hs_decode_attn_int8_static(p, p, p, p, p, ctypes.byref(lay), p, p, B, Hq, Hkv, D, ctypes.c_int32(T),
                                             ctypes.c_float(0.0625), None)
    assert rc == hb.HS_ERR_WORKSPACE
    assert b"32" in hb.lib().hs_attn_last_error() or b"33554432" in hb.lib().hs_attn_last_error()
