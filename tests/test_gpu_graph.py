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
