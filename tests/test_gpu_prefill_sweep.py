"""A seeded sweep over the prefill entry point's options: random head shapes, chunkings of a prompt, cache formats,
windows, workgroup widths, key-run counts and the bf16 prompt copy, every call checked against the plain launch
(full width, no split, no copy -- the form test_gpu_prefill.py pins to the oracle) and the finished caches bit for bit.
All trials of a sweep share ONE split workspace in one process, one after the other, so that whatever a call leaves
behind in it meets calls of other shapes, widths and run counts (that is how partial results of a full-width call were
once found where a half-width call kept its arrival counters).  The first chunk of some trials is also checked against
the oracle directly."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from gpu_util import DEV, DeviceCache

pytestmark = pytest.mark.gpu
TOL_MAX, TOL_MEAN = 2e-2, 2e-3


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_options_agree_with_the_plain_launch(seed):
    rng = np.random.default_rng(seed)
    ws = hb.prefill_split_workspace(3, 700, 64, 8, 128)
    refused = 0
    for t in range(120):
        D = int(rng.choice([64, 128, 128, 128, 256]))
        Hkv = int(rng.choice([1, 2, 4, 8]))
        G = int(rng.choice([1, 2, 3, 4, 4, 6, 8]))
        Hq, B = G * Hkv, int(rng.integers(1, 4))
        chunks = [int(rng.choice([1, 7, 16, 33, 64, 65, 100, 128, 200, 256, 300])) for _ in range(int(rng.integers(1, 5)))]
        while sum(chunks) > 700:
            chunks.pop()
        chunks = chunks or [64]
        T = sum(chunks)
        fp8 = bool(rng.integers(0, 2))
        window = int(rng.choice([0, 0, 0, 50, 130]))
        cols = int(rng.choice([0, 0, 256, 128, 32, 16]))
        runs = int(rng.choice([0, 0, 1, 2, 3, 5, 8]))
        copy = bool(D == 128 and rng.integers(0, 2))
        ragged = bool(rng.integers(0, 4) == 0)
        cfg = dict(seed=seed, t=t, D=D, Hq=Hq, Hkv=Hkv, B=B, chunks=chunks, fp8=fp8, window=window, cols=cols, runs=runs,
                   copy=copy, ragged=ragged)
        g = torch.Generator(device=DEV)
        g.manual_seed(1000 * seed + t)
        sg = 0.5 if fp8 else 1.0
        q = torch.randn(B, T, Hq, D, generator=g, device=DEV).bfloat16()
        k = (sg * torch.randn(B, T, Hkv, D, generator=g, device=DEV)).bfloat16()
        v = (sg * torch.randn(B, T, Hkv, D, generator=g, device=DEV)).bfloat16()
        a, r = DeviceCache(B, Hkv, T + 64, D, fp8=fp8), DeviceCache(B, Hkv, T + 64, D, fp8=fp8)
        if fp8:
            for c in (a, r):
                hb.kv_fp8_calibrate(k[:, :chunks[0]].contiguous(), v[:, :chunks[0]].contiguous(), c.k_scales, c.v_scales)
        sh = hb.prefill_shadow(B, Hkv, D, T + 64) if copy else None
        lo = 0
        try:
            for n in chunks:
                qs, ks_, vs_ = (x[:, lo:lo + n].contiguous() for x in (q, k, v))
                got = torch.full((B, n, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
                want = torch.full_like(got, float("nan"))
                hl = torch.full((B,), lo, dtype=torch.int32, device=DEV) if ragged else None
                hb.prefill_attn(qs, ks_, vs_, r.k_codes, r.v_codes, r.k_scales, r.v_scales, r.layout, lo, want, 1 / np.sqrt(D),
                                True, fp8=fp8, hist_lens=hl, columns=256, window=window, key_splits=1)
                hb.prefill_attn(qs, ks_, vs_, a.k_codes, a.v_codes, a.k_scales, a.v_scales, a.layout, lo, got, 1 / np.sqrt(D),
                                True, fp8=fp8, hist_lens=hl, columns=cols, window=window, split_workspace=ws, key_splits=runs,
                                shadow=sh)
                torch.cuda.synchronize()
                x, y = got.float(), want.float()
                assert bool(torch.isfinite(x).all()) and bool(torch.isfinite(y).all()), (cfg, lo)
                d = (x - y).abs()
                assert float(d.max()) < TOL_MAX and float(d.mean()) < TOL_MEAN, (cfg, lo, float(d.max()), float(d.mean()))
                if lo == 0 and window == 0 and t % 8 == 0 and B * n * Hq <= 6000:  # the reference form itself, against the oracle
                    o = oracle.prefill_attn(qs.float().cpu().numpy(), ks_.float().cpu().numpy(), vs_.float().cpu().numpy(), None,
                                            None, oracle.FMT_DENSE, np.full(B, n, np.int32), 1.0 / np.sqrt(D))
                    e = np.abs(y.cpu().numpy() - o)
                    assert e.max() < TOL_MAX and e.mean() < TOL_MEAN, (cfg, e.max(), e.mean())
                lo += n
        except hb.HsError:
            refused += 1  # (a combination the entry point does not serve says so; none is expected among these)
            continue
        assert torch.equal(a.k_codes, r.k_codes) and torch.equal(a.v_codes, r.v_codes), cfg
        assert torch.equal(a.k_scales, r.k_scales) and torch.equal(a.v_scales, r.v_scales), cfg
    assert refused == 0
