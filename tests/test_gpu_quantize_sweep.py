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


@pytest.mark.parametrize("seed", [73])
def test_dense_view_of_random_caches(seed):
    """hs_kv_dequantize (LayerKVCache::get): random codes and scales -- every code value, scales over many decades, zero
    scales -- in a contiguous cache or behind a shuffled block table, read back in bf16, fp16 or fp32 for a prefix of
    the capacity: the oracle's dequantisation, rounded once to the view's dtype."""
    rng = np.random.default_rng(seed)
    for t in range(60):
        D, Hkv, B = int(rng.choice([64, 128, 256])), int(rng.choice([1, 2, 3, 8])), int(rng.integers(1, 4))
        cap = int(rng.choice([1, 7, 64, 100, 300, 700]))
        T = int(rng.integers(1, cap + 1))
        fp8, paged = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 3))]
        cfg = dict(seed=seed, t=t, D=D, Hkv=Hkv, B=B, cap=cap, T=T, fp8=fp8, paged=paged, dtype=str(dtype))
        span = 4 if dtype == torch.float16 else 20  # (fp16 views of huge values would just be infinities)
        if fp8:
            codes = rng.integers(0, 256, (B, cap, Hkv, D)).astype(np.uint8)
            codes[(codes & 0x7f) == 0x7f] = 0x7e  # e4m3fn's NaN patterns never come out of the quantizer
            scales = (10.0 ** rng.uniform(-span, span - 3, (B, Hkv))).astype(np.float32)
            want = oracle.dequant_fp8(codes, scales)
        else:
            codes = rng.integers(-127, 128, (B, cap, Hkv, D)).astype(np.int8)
            scales = (10.0 ** rng.uniform(-span, span - 3, (B, cap, Hkv))).astype(np.float32)
            scales[rng.random(scales.shape) < 0.05] = 0.0
            want = oracle.dequant_int8(codes, scales)
        BT = 256
        nblk = (cap + BT - 1) // BT
        ct = torch.from_numpy(codes).to(DEV)
        if paged:
            tab = torch.from_numpy(rng.permutation(B * nblk + 2).astype(np.int32)[:B * nblk].reshape(B, nblk)).to(DEV)
            pool = torch.zeros(B * nblk + 2, Hkv, BT, D, dtype=ct.dtype, device=DEV)
            padded = torch.zeros(B, nblk * BT, Hkv, D, dtype=ct.dtype, device=DEV)
            padded[:, :cap] = ct
            pool[tab.long()] = padded.view(B, nblk, BT, Hkv, D).permute(0, 1, 3, 2, 4)
            lay = hb.paged_layout(Hkv, BT, D, tab, tab)
            if fp8:
                sc = torch.from_numpy(scales).to(DEV)
            else:
                sp = torch.zeros(B, nblk * BT, Hkv, device=DEV)
                sp[:, :cap] = torch.from_numpy(scales).to(DEV)
                sc = torch.zeros(B * nblk + 2, Hkv, BT, device=DEV)
                sc[tab.long()] = sp.view(B, nblk, BT, Hkv).permute(0, 1, 3, 2)
            store = pool
        else:
            lay = hb.contiguous_layout(Hkv, cap, D)
            store = ct.permute(0, 2, 1, 3).contiguous()
            if fp8:
                sc = torch.from_numpy(scales).to(DEV)
            else:
                sc = torch.zeros(B, Hkv, lay.scale_stride_head, device=DEV)
                sc[:, :, :cap] = torch.from_numpy(scales).to(DEV).permute(0, 2, 1)
        out = torch.full((B, T, Hkv, D), float("nan"), dtype=dtype, device=DEV)
        hb.kv_dequantize(store, sc, fp8, lay, 0, out)
        torch.cuda.synchronize()
        w = torch.from_numpy(want[:, :T]).to(dtype)
        got = out.cpu()
        same = (got == w) | (torch.isnan(got) & torch.isnan(w))
        assert bool(same.all()), (cfg, int((~same).sum()))
