"""A seeded sweep over decode attention: random head shapes, batch sizes, context lengths and ragged length patterns
(full, uniform, long, some sequences empty), int8 and FP8 caches, each through the fixed-chunk launch, the balanced
split that a batch-total hint selects, the two-phase form and (int8) the entry point with the built-in scratch --
every output against the oracle on the cache's codes."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from gpu_util import DEV, DeviceCache

pytestmark = pytest.mark.gpu
TOL_MAX, TOL_MEAN = 2e-2, 2e-3


@pytest.mark.parametrize("seed", [21, 22])
def test_every_launch_form_against_the_oracle(seed):
    rng = np.random.default_rng(seed)
    for t in range(60):
        D = int(rng.choice([64, 128, 128, 256]))
        Hkv = int(rng.choice([1, 2, 4, 8]))
        G = int(rng.choice([1, 2, 3, 4, 4, 5, 8, 16]))
        Hq = G * Hkv
        B = int(rng.choice([1, 2, 3, 7, 16, 33]))
        T = int(rng.choice([1, 17, 64, 129, 500, 1024, 2047]))
        while B * Hq * T * D > 3e7:  # keeps the oracle's share of a trial to a fraction of a second
            T = max(1, T // 2)
        fp8 = bool(rng.integers(0, 2))
        kind = int(rng.integers(0, 4))
        if kind == 0:
            lens = np.full(B, T)
        elif kind == 1:
            lens = rng.integers(0, T + 1, B)
        elif kind == 2:
            lens = rng.integers(max(1, T // 2), T + 1, B)
        else:
            lens = np.where(rng.integers(0, 3, B) == 0, 0, rng.integers(1, T + 1, B))
        lens = lens.astype(np.int32)
        cfg = dict(seed=seed, t=t, D=D, Hq=Hq, Hkv=Hkv, B=B, T=T, fp8=fp8, lens=lens.tolist()[:8])
        g = torch.Generator(device=DEV)
        g.manual_seed(7000 * seed + t)
        sg = 0.5 if fp8 else 1.0
        k = (sg * torch.randn(B, T, Hkv, D, generator=g, device=DEV)).bfloat16()
        v = (sg * torch.randn(B, T, Hkv, D, generator=g, device=DEV)).bfloat16()
        q = torch.randn(B, Hq, D, generator=g, device=DEV).bfloat16()
        c = DeviceCache(B, Hkv, T, D, fp8=fp8)
        if fp8:
            hb.kv_fp8_calibrate(k, v, c.k_scales, c.v_scales)
        c.write(k, v)
        lens_d = torch.from_numpy(lens).to(DEV)
        scale = 1 / np.sqrt(D)
        ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
        new = lambda: torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        outs = {"fixed": new(), "balanced": new(), "phases": new()}
        hb.decode_attn(q, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, lens_d, outs["fixed"], ws, Hkv, T, scale, fp8=fp8)
        lay = hb.contiguous_layout(Hkv, T, D)
        lay.total_tokens_hint = int(max(1, lens.sum()))
        hb.decode_attn(q, c.k_codes, c.v_codes, c.k_scales, c.v_scales, lay, lens_d, outs["balanced"], ws, Hkv, T, scale, fp8=fp8)
        for ph in (1, 2):
            hb.decode_attn(q, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, lens_d, outs["phases"], ws, Hkv, T, scale,
                           fp8=fp8, phases=ph)
        if not fp8:
            outs["static"] = new()
            hb.decode_attn_static(q, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, lens_d, outs["static"], Hkv, T, scale)
        torch.cuda.synchronize()
        kc, vc, ks, vs = c.canonical(T)
        want = oracle.decode_attn(q.float().cpu().numpy(), kc, vc, ks, vs, oracle.FMT_FP8 if fp8 else oracle.FMT_INT8, lens, scale)
        for name, o in outs.items():
            x = o.float().cpu().numpy()
            assert np.isfinite(x).all(), (name, cfg)
            d = np.abs(x - want)
            assert d.max() < TOL_MAX and d.mean() < TOL_MEAN, (name, cfg, d.max(), d.mean())
