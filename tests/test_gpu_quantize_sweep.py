"""A seeded sweep over quantize-on-write: source dtype (bf16 / fp16 / fp32), head_dim, row counts that do and do not fill
a wavefront, magnitudes from 1e-30 to 1e30 with outliers, zeros and whole zero rows, int8 and FP8, a contiguous cache
or a pool of 256-token blocks behind a shuffled table, rows placed by a scalar start or by per-sequence device
positions -- codes and scales bit for bit against the oracle, everything else in the cache untouched."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from gpu_util import DEV

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [71, 72])
def test_codes_and_scales_bit_exact(seed):
    rng = np.random.default_rng(seed)
    for t in range(60):
        D, Hkv = int(rng.choice([64, 128, 256])), int(rng.choice([1, 2, 3, 8]))
        B, S = int(rng.integers(1, 5)), int(rng.choice([1, 2, 7, 31, 64, 100, 257]))
        dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 3))]
        fp8, paged, by_position = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        cap = int(rng.choice([S, S + 5, 2 * S + 300]))
        cfg = dict(seed=seed, t=t, D=D, Hkv=Hkv, B=B, S=S, dtype=str(dtype), fp8=fp8, paged=paged, by_position=by_position, cap=cap)
        mag = 10.0 ** rng.uniform(-4 if dtype == torch.float16 else -30, 4 if dtype == torch.float16 else 30, (B, S, Hkv, 1))
        x = rng.standard_normal((B, S, Hkv, D)) * (mag if rng.integers(0, 2) else 1.0)
        x[rng.random(x.shape) < 0.01] *= 8
        x[rng.random(x.shape) < 0.02] = 0.0
        x[rng.random((B, S, Hkv)) < 0.03] = 0.0
        src = torch.from_numpy(x.astype(np.float32)).to(dtype)
        xs = src.float().numpy()  # what the source dtype holds
        src = src.to(DEV).contiguous()
        src_v = (src.float() * 0.5).to(dtype).contiguous()
        xv = src_v.float().cpu().numpy()
        starts = rng.integers(0, cap - S + 1, B).astype(np.int32) if by_position else np.full(B, int(rng.integers(0, cap - S + 1)), np.int32)
        BT = 256
        nblk = (cap + BT - 1) // BT
        cdt = torch.uint8 if fp8 else torch.int8
        if paged:
            perm = torch.from_numpy(rng.permutation(B * nblk + 3).astype(np.int32)[:B * nblk].reshape(B, nblk)).to(DEV)
            kc = torch.full((B * nblk + 3, Hkv, BT, D), 7, dtype=cdt, device=DEV)
            vc = torch.full_like(kc, 7)
            lay = hb.paged_layout(Hkv, BT, D, perm, perm)
            ks = torch.full((B, Hkv), 0.0, device=DEV) if fp8 else torch.full((B * nblk + 3, Hkv, BT), -1.0, device=DEV)
        else:
            kc = torch.full((B, Hkv, cap, D), 7, dtype=cdt, device=DEV)
            vc = torch.full_like(kc, 7)
            lay = hb.contiguous_layout(Hkv, cap, D)
            ks = torch.full((B, Hkv), 0.0, device=DEV) if fp8 else torch.full((B, Hkv, lay.scale_stride_head), -1.0, device=DEV)
        vs = ks.clone()
        if fp8:
            hb.kv_fp8_calibrate(src, src_v, ks, vs)
            wks, wvs = oracle.fp8_calibrate(xs), oracle.fp8_calibrate(xv)
            assert np.array_equal(ks.cpu().numpy().view(np.uint32), wks.view(np.uint32)), cfg
        pos_d = torch.from_numpy(starts).to(DEV) if by_position else None
        fn = hb.kv_quantize_fp8 if fp8 else hb.kv_quantize_int8
        fn(src, src_v, kc, vc, ks, vs, lay, pos_d, 0 if by_position else int(starts[0]))
        torch.cuda.synchronize()
        # gather the cache as [B, cap, Hkv, D] / [B, cap, Hkv]
        if paged:
            idx = perm.long()
            gk = kc[idx].permute(0, 1, 3, 2, 4).reshape(B, nblk * BT, Hkv, D)[:, :cap]
            gv = vc[idx].permute(0, 1, 3, 2, 4).reshape(B, nblk * BT, Hkv, D)[:, :cap]
            if not fp8:
                gks = ks[idx].permute(0, 1, 3, 2).reshape(B, nblk * BT, Hkv)[:, :cap]
                gvs = vs[idx].permute(0, 1, 3, 2).reshape(B, nblk * BT, Hkv)[:, :cap]
        else:
            gk, gv = kc.permute(0, 2, 1, 3), vc.permute(0, 2, 1, 3)
            if not fp8:
                gks, gvs = ks[:, :, :cap].permute(0, 2, 1), vs[:, :, :cap].permute(0, 2, 1)
        gk, gv = gk.cpu().numpy(), gv.cpu().numpy()
        if fp8:
            wk, wv = oracle.quant_fp8(xs, wks), oracle.quant_fp8(xv, wvs)
        else:
            (wk, wsk), (wv, wsv) = oracle.quant_int8(xs), oracle.quant_int8(xv)
            gks, gvs = gks.cpu().numpy(), gvs.cpu().numpy()
        for b in range(B):
            lo = int(starts[b])
            assert np.array_equal(gk[b, lo:lo + S], wk[b]) and np.array_equal(gv[b, lo:lo + S], wv[b]), (cfg, b)
            untouched = np.ones(cap, bool)
            untouched[lo:lo + S] = False
            assert (gk[b, untouched] == 7).all() and (gv[b, untouched] == 7).all(), (cfg, b)
            if not fp8:
                assert np.array_equal(gks[b, lo:lo + S].view(np.uint32), wsk[b].view(np.uint32)), (cfg, b)
                assert np.array_equal(gvs[b, lo:lo + S].view(np.uint32), wsv[b].view(np.uint32)), (cfg, b)
                assert (gks[b, untouched] == -1.0).all(), (cfg, b)
