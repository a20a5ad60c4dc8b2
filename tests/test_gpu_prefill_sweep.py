"""A seeded sweep over the prefill entry point's options: random head shapes, chunkings of a prompt, cache formats,
windows, workgroup widths, key-run counts and the bf16 prompt copy, every call checked against the plain launch
(full width, no split, no copy -- the form test_gpu_prefill.py pins to the oracle) and the finished caches bit for bit.
All trials of a sweep share ONE split workspace in one process, one after the other, so that whatever a call leaves
behind in it meets calls of other shapes, widths and run counts (that is how partial results of a full-width call were
once found where a half-width call kept its arrival counters).  The first chunk of some trials is also checked against
the oracle directly.  A second sweep adds paged caches, the output gate and q's prologue inside the launch."""
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


@pytest.mark.parametrize("seed", [14, 15])
def test_paged_caches_the_output_gate_and_the_q_prologue(seed):
    """The remaining options, drawn together with the ones above: the cache behind a shuffled block table (blocks of 64,
    128 or 256 tokens), the output gate, q's QK-norm and rotation inside the launch (against hs_qk_prologue_apply on q
    followed by the call without it).  Reference: the plain launch on a contiguous cache; the finished codes agree block
    by block."""
    from oracle import reference_path as ref
    rng = np.random.default_rng(seed)
    ws = hb.prefill_split_workspace(3, 600, 64, 8, 128)
    tables = {}
    for t in range(100):
        D, Hkv, G = int(rng.choice([64, 128, 128, 256])), int(rng.choice([1, 2, 4, 8])), int(rng.choice([1, 2, 3, 4, 6, 8]))
        Hq, B = G * Hkv, int(rng.integers(1, 4))
        chunks = [int(rng.choice([1, 7, 33, 64, 100, 128, 256, 300])) for _ in range(int(rng.integers(1, 4)))]
        while sum(chunks) > 600:
            chunks.pop()
        chunks = chunks or [64]
        T = sum(chunks)
        cap = T + 64
        fp8 = bool(rng.integers(0, 2))
        cols, runs = int(rng.choice([0, 0, 256, 128, 16])), int(rng.choice([0, 0, 1, 2, 3, 8]))
        copy = bool(D == 128 and rng.integers(0, 2))
        BT = int(rng.choice([64, 128, 256]))
        paged, gate, qpro = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        rd = int(rng.choice([D, D // 2, D // 4])) if qpro else 0
        kind = int(rng.integers(0, 3)) if qpro else 0
        cfg = dict(seed=seed, t=t, D=D, Hq=Hq, Hkv=Hkv, B=B, chunks=chunks, fp8=fp8, cols=cols, runs=runs, copy=copy, paged=paged,
                   BT=BT, gate=gate, qpro=qpro, rd=rd, kind=kind)
        g = torch.Generator(device=DEV)
        g.manual_seed(3000 * seed + t)
        sg = 0.5 if fp8 else 1.0
        q = torch.randn(B, T, Hq, D, generator=g, device=DEV).bfloat16()
        k = (sg * torch.randn(B, T, Hkv, D, generator=g, device=DEV)).bfloat16()
        v = (sg * torch.randn(B, T, Hkv, D, generator=g, device=DEV)).bfloat16()
        gt = torch.randn(B, T, Hq, D, generator=g, device=DEV).bfloat16() if gate else None
        cdt = torch.uint8 if fp8 else torch.int8

        def cache(pg):
            if pg:
                nblk = (cap + BT - 1) // BT
                tab = torch.from_numpy(rng.permutation(B * nblk + 2).astype(np.int32)[:B * nblk].reshape(B, nblk)).to(DEV)
                kc = torch.zeros(B * nblk + 2, Hkv, BT, D, dtype=cdt, device=DEV)
                ks = torch.zeros(B, Hkv, device=DEV) if fp8 else torch.zeros(B * nblk + 2, Hkv, BT, device=DEV)
                return kc, torch.zeros_like(kc), ks, ks.clone(), hb.paged_layout(Hkv, BT, D, tab, tab), tab
            lay = hb.contiguous_layout(Hkv, cap, D)
            kc = torch.zeros(B, Hkv, cap, D, dtype=cdt, device=DEV)
            ks = torch.zeros(B, Hkv, device=DEV) if fp8 else torch.zeros(B, Hkv, lay.scale_stride_head, device=DEV)
            return kc, torch.zeros_like(kc), ks, ks.clone(), lay, None

        A, R = cache(paged), cache(False)
        if fp8:
            for c in (A, R):
                hb.kv_fp8_calibrate(k[:, :chunks[0]].contiguous(), v[:, :chunks[0]].contiguous(), c[2], c[3])
        sh = hb.prefill_shadow(B, Hkv, D, cap) if copy else None
        pro = None
        if qpro:
            if rd not in tables:
                tables[rd] = tuple(x.contiguous().to(DEV) for x in ref.rope_tables(rd, 10000.0, 1024, torch.bfloat16))
            wq = None
            if kind == hb.QKNORM_LLAMA:
                wq = (1 + 0.2 * torch.randn(Hq, D, generator=g, device=DEV)).bfloat16()
            elif kind == hb.QKNORM_QWEN35:
                wq = (0.05 * torch.randn(Hq, D, generator=g, device=DEV)).float()
            pro = hb.qk_prologue(kind, 1e-6, wq, None, tables[rd][0], tables[rd][1], rd)
        lo = 0
        for n in chunks:
            qs, ks_, vs_ = (x[:, lo:lo + n].contiguous() for x in (q, k, v))
            gs = gt[:, lo:lo + n].contiguous() if gate else None
            got = torch.full((B, n, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
            want = torch.full_like(got, float("nan"))
            q_ref = qs
            if qpro:
                q_ref = torch.empty_like(qs)
                hb.qk_prologue_apply(qs, None, pro, q_ref, None, None, lo)
            for (kc, vc, ks2, vs2, lay, _), o, qq, kw in (
                    (R, want, q_ref, dict(columns=256, key_splits=1)),
                    (A, got, qs, dict(columns=cols, split_workspace=ws, key_splits=runs, shadow=sh, q_prologue=pro))):
                lay.out_gate = gs.data_ptr() if gate else None
                hb.prefill_attn(qq, ks_, vs_, kc, vc, ks2, vs2, lay, lo, o, 1 / np.sqrt(D), True, fp8=fp8, **kw)
            torch.cuda.synchronize()
            x, y = got.float(), want.float()
            assert bool(torch.isfinite(x).all()) and bool(torch.isfinite(y).all()), (cfg, lo)
            d = (x - y).abs()
            assert float(d.max()) < TOL_MAX and float(d.mean()) < TOL_MEAN, (cfg, lo, float(d.max()), float(d.mean()))
            lo += n
        kcA, vcA = A[0], A[1]
        if paged:
            idx = A[5].long()
            kcA = kcA[idx].permute(0, 2, 1, 3, 4).reshape(B, Hkv, idx.shape[1] * BT, D)
            vcA = vcA[idx].permute(0, 2, 1, 3, 4).reshape(B, Hkv, idx.shape[1] * BT, D)
        assert torch.equal(kcA[:, :, :T], R[0][:, :, :T]) and torch.equal(vcA[:, :, :T], R[1][:, :, :T]), cfg


@pytest.mark.parametrize("seed", [16])
def test_rows_at_different_positions_against_one_sequence_at_a_time(seed):
    """hs_prefill_attn_*_ragged (the reference's forward_batched with q_len > 1): sequences with DIFFERENT numbers of
    cached tokens take S new tokens in one call.  Against the same sequences one at a time (B = 1 calls at their own
    history length, the form the other tests pin to the oracle): outputs within rounding, caches bit for bit."""
    rng = np.random.default_rng(seed)
    ws = hb.prefill_split_workspace(4, 300, 64, 8, 128)
    for t in range(60):
        D, Hkv, G = int(rng.choice([64, 128, 128, 256])), int(rng.choice([1, 2, 8])), int(rng.choice([1, 2, 4, 6]))
        Hq, B = G * Hkv, int(rng.integers(2, 5))
        S = int(rng.choice([1, 5, 64, 100, 257, 300]))
        hist = [int(rng.choice([0, 0, 1, 63, 64, 200, 513])) for _ in range(B)]
        fp8 = bool(rng.integers(0, 2))
        cols, runs = int(rng.choice([0, 0, 256, 128])), int(rng.choice([0, 0, 1, 3]))
        cap = max(hist) + S
        cfg = dict(seed=seed, t=t, D=D, Hq=Hq, Hkv=Hkv, B=B, S=S, hist=hist, fp8=fp8, cols=cols, runs=runs)
        g = torch.Generator(device=DEV)
        g.manual_seed(5000 * seed + t)
        sg = 0.5 if fp8 else 1.0
        mk = lambda *s: (sg * torch.randn(*s, generator=g, device=DEV)).bfloat16()
        a, r = DeviceCache(B, Hkv, cap, D, fp8=fp8), DeviceCache(B, Hkv, cap, D, fp8=fp8)
        one = lambda c, b: (c.k_codes[b:b + 1], c.v_codes[b:b + 1], c.k_scales[b:b + 1], c.v_scales[b:b + 1])
        if fp8:
            kcal, vcal = mk(B, 64, Hkv, D), mk(B, 64, Hkv, D)
            for c in (a, r):
                hb.kv_fp8_calibrate(kcal, vcal, c.k_scales, c.v_scales)
        for b in range(B):  # each sequence's own history, the same in both caches
            if hist[b]:
                kh, vh = mk(1, hist[b], Hkv, D), mk(1, hist[b], Hkv, D)
                for c in (a, r):
                    (hb.kv_quantize_fp8 if fp8 else hb.kv_quantize_int8)(kh, vh, *one(c, b), c.layout, None, 0)
        q, k, v = torch.randn(B, S, Hq, D, generator=g, device=DEV).bfloat16(), mk(B, S, Hkv, D), mk(B, S, Hkv, D)
        got = torch.full((B, S, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        want = torch.full_like(got, float("nan"))
        hl = torch.tensor(hist, dtype=torch.int32, device=DEV)
        hb.prefill_attn(q, k, v, a.k_codes, a.v_codes, a.k_scales, a.v_scales, a.layout, max(hist), got, 1 / np.sqrt(D), True, fp8=fp8,
                        hist_lens=hl, columns=cols, split_workspace=ws, key_splits=runs)
        for b in range(B):
            hb.prefill_attn(q[b:b + 1], k[b:b + 1], v[b:b + 1], *one(r, b), r.layout, hist[b], want[b:b + 1], 1 / np.sqrt(D), True, fp8=fp8,
                            columns=256, key_splits=1)
        torch.cuda.synchronize()
        x, y = got.float(), want.float()
        assert bool(torch.isfinite(x).all()) and bool(torch.isfinite(y).all()), cfg
        d = (x - y).abs()
        assert float(d.max()) < TOL_MAX and float(d.mean()) < TOL_MEAN, (cfg, float(d.max()))
        for b in range(B):
            n = hist[b] + S
            assert torch.equal(a.k_codes[b, :, :n], r.k_codes[b, :, :n]) and torch.equal(a.v_codes[b, :, :n], r.v_codes[b, :, :n]), (cfg, b)
            if not fp8:
                assert torch.equal(a.k_scales[b, :, :n], r.k_scales[b, :, :n]), (cfg, b)
