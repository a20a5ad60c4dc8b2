"""A seeded sweep over the gated delta rule: random batch, length, head grouping, decay strength, L2-norm setting and
initial state; the chunked form against the recurrent kernel (which test_gpu_deltanet.py pins to the fp64 oracle),
a prompt cut into calls at random multiples of 64 tokens against one call bit for bit (state carried through `state`,
one workspace for all trials), and the chunked form followed by the gated norm as one call against the two calls."""
import numpy as np
import pytest
import torch

from hyprstream_amd import bindings as hb
from gpu_util import DEV

pytestmark = pytest.mark.gpu
REL = 3e-3


@pytest.mark.parametrize("seed", [51, 52])
def test_chunked_recurrent_and_cut_calls_agree(seed):
    rng = np.random.default_rng(seed)
    ws = torch.empty(hb.deltanet_chunked_gated_norm_workspace_bytes(3, 448, 8, 8), dtype=torch.uint8, device=DEV)
    for t in range(40):
        B, T = int(rng.integers(1, 4)), int(rng.choice([1, 5, 64, 65, 128, 200, 320, 448]))
        nk = int(rng.choice([1, 2, 4]))
        nv = nk * int(rng.choice([1, 2]))
        l2norm = bool(rng.integers(0, 2))
        gscale = float(rng.choice([0.0, 0.02, 1.0, 3.0]))
        cfg = dict(seed=seed, t=t, B=B, T=T, nk=nk, nv=nv, l2norm=l2norm, gscale=gscale)
        g_ = torch.Generator(device=DEV)
        g_.manual_seed(500 * seed + t)
        rn = lambda *s: torch.randn(*s, generator=g_, device=DEV)
        amp = 1.0 if l2norm else 0.08  # un-normalised rows stay small enough for the fp16 operands
        q, k = (amp * rn(B, T, nk, 128)).bfloat16(), (amp * rn(B, T, nk, 128)).bfloat16()
        v = rn(B, T, nv, 128).bfloat16()
        g = (-gscale * torch.rand(B, T, nv, generator=g_, device=DEV)).float()
        beta = torch.sigmoid(rn(B, T, nv)).float()
        s0 = (0.2 * rn(B, nv, 128, 128)).float() if rng.integers(0, 2) else torch.zeros(B, nv, 128, 128, device=DEV)
        qs = 1 / np.sqrt(128.0)

        def chunked(cuts):
            st = s0.clone()
            out = torch.full((B, T, nv, 128), float("nan"), device=DEV)
            lo = 0
            for hi in list(cuts) + [T]:
                o = torch.full((B, hi - lo, nv, 128), float("nan"), device=DEV)
                hb.deltanet_forward_chunked(*(x[:, lo:hi].contiguous() for x in (q, k, v, g, beta)), st, o, qs, l2norm, workspace=ws)
                out[:, lo:hi] = o
                lo = hi
            return out, st

        whole, st_whole = chunked(())
        rec_st = s0.clone()
        rec = torch.empty(B, T, nv, 128, device=DEV)
        hb.deltanet_forward(q, k, v, g, beta, rec_st, rec, qs, l2norm)
        torch.cuda.synchronize()
        assert bool(torch.isfinite(whole).all()) and bool(torch.isfinite(st_whole).all()), cfg
        eo, es = float((whole - rec).abs().max()), float((st_whole - rec_st).abs().max())
        assert eo <= REL * max(float(rec.abs().max()), 1e-6) and es <= REL * max(float(rec_st.abs().max()), 1e-6), (cfg, eo, es)
        if T > 64:
            marks = sorted(set(int(c) for c in rng.choice(np.arange(64, T, 64), size=min(2, (T - 1) // 64), replace=False)))
            parts, st_parts = chunked(marks)
            torch.cuda.synchronize()
            assert torch.equal(whole, parts) and torch.equal(st_whole, st_parts), (cfg, marks)
        # the chunked form + gated norm as one call: the bits of the two calls
        z = rn(B, T, nv, 128).bfloat16()
        w = (1 + 0.1 * rn(128)).float()
        two = hb.deltanet_gated_norm(whole, z, w, 1e-6)
        st1 = s0.clone()
        one = torch.empty(B, T, nv, 128, dtype=torch.bfloat16, device=DEV)
        hb.deltanet_forward_chunked_gated_norm(q, k, v, g, beta, st1, z, w, 1e-6, one, qs, l2norm, workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(one.view(torch.int16), two.view(torch.int16)) and torch.equal(st1, st_whole), cfg
