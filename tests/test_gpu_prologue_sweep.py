"""A seeded sweep over the QK-norm + rotary prologue: every rotated length that is a multiple of 16, the three norm
settings, shared or per-head weights, random row counts, head counts and positions.  hs_qk_prologue_apply against the
oracle's op-by-op rounded norm and rotation bit for bit (its kernels differ by shape: pieces of a row per lane, several
rows per wavefront, one row per wavefront), then the decode step that runs the prologue inside its launch -- for either
cache format -- against the pre-pass followed by the plain step, bit for bit in outputs and cache."""
import numpy as np
import pytest
import torch

from hyprstream_amd import bindings as hb
from gpu_util import DEV, DeviceCache
from test_gpu_qk_prologue import _bf, _bits, _tables, _weights, oracle_prologue

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [61, 62])
def test_prepass_against_the_oracle_and_fused_step_against_the_prepass(seed):
    rng = np.random.default_rng(seed)
    tables = {}
    for t in range(60):
        D = int(rng.choice([64, 128, 256]))
        rd = int(rng.choice(np.arange(0, D + 1, 16)))  # 0: no rotation
        kind = int(rng.choice([hb.QKNORM_NONE, hb.QKNORM_LLAMA, hb.QKNORM_QWEN35]))
        if rd == 0 and kind == hb.QKNORM_NONE:
            kind = hb.QKNORM_LLAMA
        Hkv, G = int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 3, 4, 8]))
        Hq, B, S, L = G * Hkv, int(rng.integers(1, 5)), int(rng.choice([1, 2, 13, 64, 100])), 1024
        cfg = dict(seed=seed, t=t, D=D, rd=rd, kind=kind, Hq=Hq, Hkv=Hkv, B=B, S=S)
        if rd and rd not in tables:
            tables[rd] = _tables(rd, 10000.0, L)
        sin, cos = tables[rd] if rd else (None, None)
        q = _bf(rng.standard_normal((B, S, Hq, D)) * 2)
        k = _bf(rng.standard_normal((B, S, Hkv, D)) * rng.random((B, S, Hkv, 1)) * 3)
        per_head = bool(rng.integers(0, 2))
        wq = _weights(rng, kind, Hq, D, per_head) if kind else None
        wk = _weights(rng, kind, Hkv, D, not per_head) if kind else None
        pro = hb.qk_prologue(kind, 1e-6, wq.to(DEV) if kind else None, wk.to(DEV) if kind else None,
                             sin.to(DEV) if rd else None, cos.to(DEV) if rd else None, rd)
        pos0 = rng.integers(0, L - S - 3, B).astype(np.int32)
        q_out = torch.full_like(q, float("nan"), device=DEV)
        k_out = torch.full_like(k, float("nan"), device=DEV)
        hb.qk_prologue_apply(q.to(DEV), k.to(DEV), pro, q_out, k_out, torch.from_numpy(pos0).to(DEV), start_pos=3)
        torch.cuda.synchronize()
        pos = (pos0[:, None] + 3 + np.arange(S, dtype=np.int32)[None]).reshape(-1)
        wantq = oracle_prologue(_bits(q).reshape(B * S, Hq, D), kind, wq, 1e-6, sin, cos, pos, rd)
        wantk = oracle_prologue(_bits(k).reshape(B * S, Hkv, D), kind, wk, 1e-6, sin, cos, pos, rd)
        assert np.array_equal(_bits(q_out).reshape(B * S, Hq, D), wantq), cfg
        assert np.array_equal(_bits(k_out).reshape(B * S, Hkv, D), wantk), cfg
        # the decode step with the prologue inside the launch (the new token at seq_len - 1)
        fp8 = bool(rng.integers(0, 2))
        T = int(rng.choice([1, 40, 300, 700]))
        lens = rng.integers(1, T + 1, B).astype(np.int32)
        sg = 0.5 if fp8 else 1.0
        hk, hv = _bf(sg * rng.standard_normal((B, T, Hkv, D))).to(DEV), _bf(sg * rng.standard_normal((B, T, Hkv, D))).to(DEV)
        qd, kn, vn = q[:, 0].contiguous().to(DEV), (sg * k[:, :1]).bfloat16().contiguous().to(DEV), _bf(sg * rng.standard_normal((B, 1, Hkv, D))).to(DEV)
        lens_d = torch.from_numpy(lens).to(DEV)
        ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)

        def fresh():
            c = DeviceCache(B, Hkv, T, D, fp8=fp8)
            if fp8:
                hb.kv_fp8_calibrate(hk, hv, c.k_scales, c.v_scales)
            c.write(hk, hv)
            return c

        c1, c2 = fresh(), fresh()
        out1 = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        hb.decode_step_prologue(qd, kn, vn, pro, c1.k_codes, c1.v_codes, c1.k_scales, c1.v_scales, c1.layout, lens_d, out1, ws,
                                Hkv, T, 1 / np.sqrt(D), fp8=fp8)
        q2, k2 = torch.empty(B, 1, Hq, D, dtype=torch.bfloat16, device=DEV), torch.empty_like(kn)
        hb.qk_prologue_apply(qd.view(B, 1, Hq, D), kn, pro, q2, k2, lens_d - 1, 0)
        out2 = torch.full_like(out1, float("nan"))
        hb.decode_step(q2.view(B, Hq, D), k2, vn, c2.k_codes, c2.v_codes, c2.k_scales, c2.v_scales, c2.layout, lens_d, out2, ws,
                       Hkv, T, 1 / np.sqrt(D), fp8=fp8)
        torch.cuda.synchronize()
        assert bool(torch.isfinite(out1.float()).all()), cfg
        assert torch.equal(out1.view(torch.int16), out2.view(torch.int16)), (cfg, fp8, T)
        assert torch.equal(c1.k_codes, c2.k_codes) and torch.equal(c1.v_codes, c2.v_codes), (cfg, fp8, T)
        assert torch.equal(c1.k_scales, c2.k_scales) and torch.equal(c1.v_scales, c2.v_scales), (cfg, fp8, T)


@pytest.mark.parametrize("seed", [63])
def test_cache_write_with_the_prologue_and_the_stand_alone_rotation(seed):
    """hs_kv_quantize_int8_prologue (K normalised and rotated inside the cache write, any rotated length that is a
    multiple of 16, rows placed by a scalar start or per-sequence positions): codes and scales of the oracle's
    quantizer applied to the oracle's normalised, rotated K; V as plain.  hs_rope_apply_partial on its own: the
    oracle's rotation bit for bit, the unrotated tail copied."""
    import oracle
    from oracle import hs_oracle as orc
    rng = np.random.default_rng(seed)
    tables = {}
    for t in range(60):
        D = int(rng.choice([64, 128, 256]))
        rd = int(rng.choice(np.arange(16, D + 1, 16)))
        kind = int(rng.choice([hb.QKNORM_NONE, hb.QKNORM_LLAMA, hb.QKNORM_QWEN35]))
        Hkv, B, S, L = int(rng.choice([1, 2, 3, 8])), int(rng.integers(1, 4)), int(rng.choice([1, 2, 21, 64, 130])), 1024
        by_position = bool(rng.integers(0, 2))
        cfg = dict(seed=seed, t=t, D=D, rd=rd, kind=kind, Hkv=Hkv, B=B, S=S, by_position=by_position)
        if rd not in tables:
            tables[rd] = _tables(rd, 10000.0, L)
        sin, cos = tables[rd]
        k = _bf(rng.standard_normal((B, S, Hkv, D)) * 2)
        v = _bf(rng.standard_normal((B, S, Hkv, D)))
        wk = _weights(rng, kind, Hkv, D, bool(rng.integers(0, 2))) if kind else None
        pro = hb.qk_prologue(kind, 1e-6, None, wk.to(DEV) if kind else None, sin.to(DEV), cos.to(DEV), rd)
        cap = int(rng.integers(S, S + 200))
        starts = rng.integers(0, cap - S + 1, B).astype(np.int32) if by_position else np.full(B, int(rng.integers(0, cap - S + 1)), np.int32)
        c = DeviceCache(B, Hkv, cap, D)
        hb.kv_quantize_int8_prologue(k.to(DEV), v.to(DEV), pro, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout,
                                     torch.from_numpy(starts).to(DEV) if by_position else None, 0 if by_position else int(starts[0]))
        torch.cuda.synchronize()
        kc, vc, ks, vs = c.canonical(cap)
        pos = (starts[:, None] + np.arange(S, dtype=np.int32)[None]).reshape(-1)
        k_fin = oracle_prologue(_bits(k).reshape(B * S, Hkv, D), kind, wk, 1e-6, sin, cos, pos, rd).reshape(B, S, Hkv, D)
        wkc, wks = oracle.quant_int8(oracle.bf16_to_f32(k_fin))
        wvc, wvs = oracle.quant_int8(v.float().numpy())
        for b in range(B):
            lo = int(starts[b])
            assert np.array_equal(kc[b, lo:lo + S], wkc[b]) and np.array_equal(ks[b, lo:lo + S].view(np.uint32), wks[b].view(np.uint32)), (cfg, b)
            assert np.array_equal(vc[b, lo:lo + S], wvc[b]) and np.array_equal(vs[b, lo:lo + S].view(np.uint32), wvs[b].view(np.uint32)), (cfg, b)
            rest = np.ones(cap, bool)
            rest[lo:lo + S] = False
            assert not kc[b, rest].any() and not vc[b, rest].any(), (cfg, b)
        # the rotation alone
        x = k.to(DEV)
        out = torch.full_like(x, float("nan"))
        hb.rope_apply(x, sin.to(DEV), cos.to(DEV), out, torch.from_numpy(starts).to(DEV) if by_position else None,
                      0 if by_position else int(starts[0]), rotary_dim=rd)
        torch.cuda.synchronize()
        want = _bits(k).reshape(B * S, Hkv, D).copy()
        want[..., :rd] = orc.rope_apply_bf16(np.ascontiguousarray(want[..., :rd]), _bits(sin), _bits(cos), pos)
        assert np.array_equal(_bits(out).reshape(B * S, Hkv, D), want), cfg
