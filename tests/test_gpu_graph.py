"""The entry points enqueue kernels and nothing else (no allocation, no synchronisation, no memset), so a caller
can record them into a HIP graph.  Each graph is replayed several times with eager work and synchronisations in
between, and every replay is compared with the eager result."""
import numpy as np
import pytest
import torch

from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV, DeviceCache

pytestmark = pytest.mark.gpu


def _capture(fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g


@pytest.mark.parametrize("B,T", [(64, 700), (2, 3000)])  # one launch per step / split-K + merge kernel
def test_decode_step_in_a_graph(B, T):
    Hq, Hkv, D = 32, 8, 128
    r = wl.philox(1500 + B)
    c = DeviceCache(B, Hkv, T, D)
    rnd = lambda *s: torch.from_numpy(r.standard_normal(s).astype(np.float32)).to(torch.bfloat16).to(DEV)
    c.write(rnd(B, T, Hkv, D), rnd(B, T, Hkv, D))
    q, kn, vn = rnd(B, Hq, D), rnd(B, 1, Hkv, D), rnd(B, 1, Hkv, D)
    lens = torch.full((B,), T, dtype=torch.int32, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    out = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    step = lambda: hb.decode_step(q, kn, vn, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, lens, out, ws, Hkv, T, 0.0884)
    step()
    torch.cuda.synchronize()
    want = out.clone()
    g = _capture(step)
    for i in range(4):
        out.fill_(float("nan"))
        ws.fill_(0xFF)  # stale partials must not matter
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert bool(torch.equal(out, want)), "replay %d differs from the eager result" % i
        (q.float().reshape(B, -1) @ q.float().reshape(B, -1).T).sum().item()  # unrelated eager work between replays


def test_chunked_prefill_in_a_graph():
    B, S, Hq, Hkv, D, H = 2, 128, 8, 2, 128, 256
    r = wl.philox(1510)
    rnd = lambda *s: torch.from_numpy(r.standard_normal(s).astype(np.float32)).to(torch.bfloat16).to(DEV)
    c = DeviceCache(B, Hkv, H + S, D)
    c.write(rnd(B, H, Hkv, D), rnd(B, H, Hkv, D))
    q, k, v = rnd(B, S, Hq, D), rnd(B, S, Hkv, D), rnd(B, S, Hkv, D)
    out = torch.empty(B, S, Hq, D, dtype=torch.bfloat16, device=DEV)
    call = lambda: hb.prefill_attn(q, k, v, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, H, out, 0.0884, True)
    call()
    torch.cuda.synchronize()
    want, want_codes = out.clone(), c.k_codes.clone()
    g = _capture(call)
    for i in range(3):
        out.zero_()
        c.k_codes[:, :, H:].zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert bool(torch.equal(out, want)) and bool(torch.equal(c.k_codes, want_codes)), "replay %d" % i


@pytest.mark.parametrize("cols,runs,copy", [(0, 3, False), (128, 2, True), (0, 0, True)])
def test_split_and_copy_fed_prefill_in_a_graph(cols, runs, copy):
    """The key split keeps state between launches (arrival counters that every launch leaves at zero) and the prompt
    copy is appended to by every call: a captured chunk call replays to the same bits, three times, with eager work
    and synchronisations in between."""
    B, S, Hq, Hkv, D, H = 1, 192, 8, 2, 128, 320
    r = wl.philox(1520 + cols + runs)
    rnd = lambda *s: torch.from_numpy(r.standard_normal(s).astype(np.float32)).to(torch.bfloat16).to(DEV)
    c = DeviceCache(B, Hkv, H + S, D)
    ws = hb.prefill_split_workspace(B, S, Hq, Hkv, D)
    sh = hb.prefill_shadow(B, Hkv, D, H + S) if copy else None
    o0 = torch.empty(B, H, Hq, D, dtype=torch.bfloat16, device=DEV)
    hb.prefill_attn(rnd(B, H, Hq, D), rnd(B, H, Hkv, D), rnd(B, H, Hkv, D), c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, 0,
                    o0, 0.0884, True, columns=256, key_splits=1, shadow=sh)  # the history (and its part of the copy)
    q, k, v = rnd(B, S, Hq, D), rnd(B, S, Hkv, D), rnd(B, S, Hkv, D)
    out = torch.empty(B, S, Hq, D, dtype=torch.bfloat16, device=DEV)
    call = lambda: hb.prefill_attn(q, k, v, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, H, out, 0.0884, True,
                                   columns=cols, split_workspace=ws, key_splits=runs, shadow=sh)
    call()
    torch.cuda.synchronize()
    want, want_codes = out.clone(), c.k_codes.clone()
    g = _capture(call)
    for i in range(3):
        out.zero_()
        c.k_codes[:, :, H:].zero_()
        (q.float().reshape(S, -1) @ q.float().reshape(S, -1).T).sum().item()  # unrelated eager work between replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert bool(torch.equal(out, want)) and bool(torch.equal(c.k_codes, want_codes)), "replay %d" % i


def test_chunked_deltanet_with_its_norm_in_a_graph():
    """hs_deltanet_forward_chunked_gated_norm is three ordinary launches (factor, walk, norm): recorded once, replayed
    with the state put back before every replay, it gives the eager bits each time."""
    B, T, nk, nv = 2, 200, 2, 4
    case = wl.deltanet_case(1530, B, T, nk, nv, 128, 128)
    from gpu_util import bf16_from_bits
    q, k, v = (bf16_from_bits(case[n]).to(DEV) for n in ("q_bits", "k_bits", "v_bits"))
    g, beta = torch.from_numpy(case["g"]).to(DEV), torch.from_numpy(case["beta"]).to(DEV)
    r = wl.philox(1531)
    z = torch.from_numpy(r.standard_normal((B, T, nv, 128)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    w = torch.from_numpy((1.0 + 0.2 * r.standard_normal(128)).astype(np.float32)).to(DEV)
    s0 = torch.from_numpy((r.standard_normal((B, nv, 128, 128)) * 0.2).astype(np.float32)).to(DEV)
    st = s0.clone()
    out = torch.empty(B, T, nv, 128, dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.deltanet_chunked_gated_norm_workspace_bytes(B, T, nk, nv), dtype=torch.uint8, device=DEV)
    call = lambda: hb.deltanet_forward_chunked_gated_norm(q, k, v, g, beta, st, z, w, 1e-6, out, 0.0884, True, workspace=ws)
    call()
    torch.cuda.synchronize()
    want, want_state = out.clone(), st.clone()
    st.copy_(s0)
    gr = _capture(call)
    for i in range(3):
        out.zero_()
        st.copy_(s0)
        ws.zero_()
        torch.cuda.synchronize()
        gr.replay()
        torch.cuda.synchronize()
        assert bool(torch.equal(out, want)) and bool(torch.equal(st, want_state)), "replay %d" % i


def _cache_with_history(B, T0, cap, Hkv, D, seed, quant):
    from hyprstream_amd import kv_cache as kc
    r = wl.philox(seed)
    rnd = lambda *s: torch.from_numpy(r.standard_normal(s).astype(np.float32)).to(torch.bfloat16).to(DEV)
    c = kc.LayerKVCache(cap, quant)
    c.update(rnd(B, T0, Hkv, D), rnd(B, T0, Hkv, D), 0)
    return c, rnd


@pytest.mark.parametrize("B,T0", [(64, 300), (2, 2500)])
def test_cache_object_decode_step_in_a_graph(B, T0):
    """A decode step through the LayerKVCache mirror (hs_cache_decode_step) is launches only -- the sequence lengths
    reach the device through a fill launch on the step's stream, the workspace is sized once for max_seq_len -- so it
    can be captured.  A captured step replays at the position it was captured at: the host rewinds with truncate_to."""
    from hyprstream_amd import kv_cache as kc
    Hq, Hkv, D = 32, 8, 128
    c, rnd = _cache_with_history(B, T0, T0 + 8, Hkv, D, 1520 + B, kc.INT8)
    q, kn, vn = rnd(B, Hq, D), rnd(B, 1, Hkv, D), rnd(B, 1, Hkv, D)
    want = c.decode_step(q, kn, vn, 0.0884)  # eager: also sizes the workspace, outside any capture
    torch.cuda.synchronize()
    assert c.seq_pos == T0 + 1
    kw, vw = c.get()
    out = torch.empty_like(q)
    L = kc.lib()
    import ctypes

    def step():
        rc = L.hs_cache_decode_step(c._h, hb._ptr(q), hb._ptr(kn), hb._ptr(vn), hb.HS_BF16, hb._ptr(out), Hq,
                                    ctypes.c_float(0.0884), hb._stream())
        assert rc == 0, L.hs_cache_last_error(c._h)

    c.truncate_to(T0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    c.truncate_to(T0)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    assert c.seq_pos == T0 + 1
    for i in range(4):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert bool(torch.equal(out, want)), "replay %d differs from the eager step" % i
        (q.float().reshape(B, -1) @ q.float().reshape(B, -1).T).sum().item()
    k2, v2 = c.get()
    assert bool(torch.equal(k2, kw)) and bool(torch.equal(v2, vw))


def test_cache_object_steps_on_a_side_stream_match_the_default_stream():
    """Steps enqueued back to back on a non-blocking side stream, with no host synchronisation in between: each step's
    lengths are ordered behind the previous step's kernel on that stream, so no step reads another step's length."""
    from hyprstream_amd import kv_cache as kc
    B, Hq, Hkv, D, T0, n = 3, 16, 4, 128, 500, 12
    outs = []
    for use_side in (False, True):
        c, rnd = _cache_with_history(B, T0, T0 + n, Hkv, D, 1530, kc.INT8)
        toks = [(rnd(B, Hq, D), rnd(B, 1, Hkv, D), rnd(B, 1, Hkv, D)) for _ in range(n)]
        torch.cuda.synchronize()
        stream = torch.cuda.Stream() if use_side else torch.cuda.current_stream()
        with torch.cuda.stream(stream):
            res = [c.decode_step(q, k, v, 0.0884) for q, k, v in toks]
        stream.synchronize()
        torch.cuda.synchronize()
        assert c.seq_pos == T0 + n
        outs.append((torch.stack(res), c.get()))
    assert bool(torch.equal(outs[0][0], outs[1][0]))
    assert bool(torch.equal(outs[0][1][0], outs[1][1][0])) and bool(torch.equal(outs[0][1][1], outs[1][1][1]))
