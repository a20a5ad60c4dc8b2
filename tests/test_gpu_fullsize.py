"""GPU parity at the benchmark configurations' FULL sizes.

The oracle cannot redo these sizes in seconds, so each test checks (a) a sample of (sequence, head) units or
query rows against the oracle, bit-exact for codes and within the path's tolerance for attention, and
(b) size-independent properties: constant V gives constant output, split-K equals unsplit, chunked equals
carried state.  Inputs are generated on the device from the seed."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV

pytestmark = pytest.mark.gpu
TOL_MAX, TOL_MEAN = 2e-2, 2e-3


def gen(seed):
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    return g


def source(g, shape, sigma=1.0, outliers=False):
    x = torch.randn(shape, generator=g, device=DEV) * sigma
    if outliers:
        m = torch.rand(shape, generator=g, device=DEV) < 0.01
        x = torch.where(m, torch.sign(x) * 8.0 * sigma, x)
    return x.to(torch.bfloat16)


def fill_cache(g, B, Hkv, T, D, fp8, sigma, outliers, keep=()):
    """Quantize-on-write of T tokens per sequence, one sequence at a time; returns buffers and the bf16
    sources of the sequences listed in `keep`."""
    lay = hb.contiguous_layout(Hkv, T, D)
    cdt = torch.uint8 if fp8 else torch.int8
    kc = torch.empty(B, Hkv, T, D, dtype=cdt, device=DEV)
    vc = torch.empty_like(kc)
    if fp8:
        ks = torch.empty(B, Hkv, dtype=torch.float32, device=DEV)
    else:
        ks = torch.empty(B, Hkv, lay.scale_stride_head, dtype=torch.float32, device=DEV)
    vs = torch.empty_like(ks)
    kept = {}
    for b in range(B):
        k, v = source(g, (1, T, Hkv, D), sigma, outliers), source(g, (1, T, Hkv, D), sigma, outliers)
        if fp8:
            hb.kv_fp8_calibrate(k, v, ks[b:b + 1], vs[b:b + 1])
            hb.kv_quantize_fp8(k, v, kc[b:b + 1], vc[b:b + 1], ks[b:b + 1], vs[b:b + 1], lay, None, 0)
        else:
            hb.kv_quantize_int8(k, v, kc[b:b + 1], vc[b:b + 1], ks[b:b + 1], vs[b:b + 1], lay, None, 0)
        if b in keep:
            kept[b] = (k.float().cpu().numpy(), v.float().cpu().numpy())
    torch.cuda.synchronize()
    return lay, kc, vc, ks, vs, kept


def decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, fp8, phases=3):
    B, Hq, D = q.shape
    out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    for ph in ([1, 2] if phases == 12 else [3]):
        hb.decode_attn(q, kc, vc, ks, vs, lay, lens, out, ws, Hkv, T, 1.0 / np.sqrt(D), fp8=fp8, phases=ph)
    torch.cuda.synchronize()
    return out


def sample_check(out, q, kc, vc, ks, vs, lens, units, G, fp8):
    for b, h in units:
        n = int(lens[b])
        kcb = kc[b, h, :n].cpu().numpy()[None, :, None, :]
        vcb = vc[b, h, :n].cpu().numpy()[None, :, None, :]
        if fp8:
            ksb, vsb = ks[b, h].cpu().numpy().reshape(1, 1), vs[b, h].cpu().numpy().reshape(1, 1)
        else:
            ksb, vsb = ks[b, h, :n].cpu().numpy()[None, :, None], vs[b, h, :n].cpu().numpy()[None, :, None]
        qb = q[b, h * G:(h + 1) * G].float().cpu().numpy()[None]
        want = oracle.decode_attn(qb, kcb, vcb, ksb, vsb, oracle.FMT_FP8 if fp8 else oracle.FMT_INT8,
                                  np.array([n], np.int32), 1.0 / np.sqrt(q.shape[-1]))[0]
        d = np.abs(out[b, h * G:(h + 1) * G].float().cpu().numpy() - want)
        assert d.max() < TOL_MAX and d.mean() < TOL_MEAN, (b, h, d.max(), d.mean())
        # at these lengths the outputs themselves are about the size of the absolute tolerance (an average of thousands
        # of N(0,1) values), so the check that bites is relative: 2^-7 of the unit's largest output
        assert d.max() <= 2.0 ** -7 * np.abs(want).max(), (b, h, d.max(), np.abs(want).max())


def decode_step_check(g, q, kc, vc, ks, vs, lay, lens, Hkv, T, fp8, sigma, outliers, units):
    """The fused step (new-token write in the attention launch) at full size against (a) the oracle's quantizer for
    the written rows, bit for bit, (b) the unfused flow -- the stand-alone writer then attention -- bit for bit,
    (c) the oracle's attention for sampled units.  Restores nothing: the caches hold the new token afterwards."""
    B, Hq, D = q.shape
    G = Hq // Hkv
    k_new, v_new = source(g, (B, 1, Hkv, D), sigma, outliers), source(g, (B, 1, Hkv, D), sigma, outliers)
    kc2, vc2, ks2, vs2 = kc.clone(), vc.clone(), ks.clone(), vs.clone()
    pos = (lens - 1).contiguous()
    # unfused: writer, then attention
    (hb.kv_quantize_fp8 if fp8 else hb.kv_quantize_int8)(k_new, v_new, kc2, vc2, ks2, vs2, lay, pos, 0)
    want = decode(q, kc2, vc2, ks2, vs2, lay, lens, Hkv, T, fp8)
    # fused
    out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    hb.decode_step(q, k_new, v_new, kc, vc, ks, vs, lay, lens, out, ws, Hkv, T, 1.0 / np.sqrt(D), fp8=fp8)
    torch.cuda.synchronize()
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2), "fused write differs from the stand-alone writer"
    assert torch.equal(ks, ks2) and torch.equal(vs, vs2)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16)), "fused step differs from write-then-attend"
    lens_h = lens.cpu().numpy()
    kn, vn = k_new.float().cpu().numpy(), v_new.float().cpu().numpy()
    for b in sorted({0, B - 1} | {u[0] for u in units}):
        p = int(lens_h[b]) - 1
        if fp8:
            sk, sv = ks[b].cpu().numpy()[None], vs[b].cpu().numpy()[None]
            assert np.array_equal(oracle.quant_fp8(kn[b:b + 1], sk)[0, 0], kc[b, :, p].cpu().numpy()), b
            assert np.array_equal(oracle.quant_fp8(vn[b:b + 1], sv)[0, 0], vc[b, :, p].cpu().numpy()), b
        else:
            wk, wks = oracle.quant_int8(kn[b:b + 1])
            wv, wvs = oracle.quant_int8(vn[b:b + 1])
            assert np.array_equal(wk[0, 0], kc[b, :, p].cpu().numpy()) and np.array_equal(wks[0, 0], ks[b, :, p].cpu().numpy()), b
            assert np.array_equal(wv[0, 0], vc[b, :, p].cpu().numpy()) and np.array_equal(wvs[0, 0], vs[b, :, p].cpu().numpy()), b
    sample_check(out, q, kc, vc, ks, vs, lens_h, units, G, fp8)


def test_config2_full_size_int8_decode():
    """B=64, Hq 32 / Hkv 8, D 128, T 8192 (headline) and ragged lengths U[512, 8192]."""
    B, Hq, Hkv, D, T = 64, 32, 8, 128, 8192
    g = gen(wl.SEED)
    lay, kc, vc, ks, vs, kept = fill_cache(g, B, Hkv, T, D, False, 1.0, True, keep=(0, 63))
    for b, (k, v) in kept.items():  # codes written at full size are the oracle's, bit for bit
        wk, wks = oracle.quant_int8(k[:, :, 3])
        assert np.array_equal(kc[b, 3].cpu().numpy(), wk[0]) and np.array_equal(ks[b, 3, :T].cpu().numpy(), wks[0])
    q = torch.randn(B, Hq, D, generator=g, device=DEV).to(torch.bfloat16)
    full = torch.full((B,), T, dtype=torch.int32, device=DEV)
    out = decode(q, kc, vc, ks, vs, lay, full, Hkv, T, False)
    assert torch.isfinite(out.float()).all()
    sample_check(out, q, kc, vc, ks, vs, full.cpu().numpy(), [(0, 0), (17, 5), (63, 7)], 4, False)
    two = decode(q, kc, vc, ks, vs, lay, full, Hkv, T, False, phases=12)  # partials + stand-alone merge
    assert (two.float() - out.float()).abs().max() <= 2 ** -8 * max(1.0, float(out.float().abs().max()))
    # the launch the benchmark times: one fused step (new token per sequence quantized on write, single launch)
    assert hb.decode_num_chunks(B, Hkv, T) == 1
    decode_step_check(g, q, kc, vc, ks, vs, lay, full, Hkv, T, False, 1.0, True, [(0, 3), (29, 0), (63, 7)])
    lens = torch.randint(512, T + 1, (B,), generator=g, device=DEV, dtype=torch.int32)
    rag = decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, False)
    sample_check(rag, q, kc, vc, ks, vs, lens.cpu().numpy(), [(1, 2), (40, 6)], 4, False)
    vc.fill_(64)
    vs.fill_(0.125)
    const = decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, False)
    assert (const.float() - 8.0).abs().max() <= 2 ** -5  # weights sum to one at every length


def test_config4_full_size_fp8_decode():
    """B=32, Hq 64 / Hkv 8, D 128, T 32768, e4m3 cache with per-(sequence, head) scales."""
    B, Hq, Hkv, D, T = 32, 64, 8, 128, 32768
    g = gen(wl.SEED + 4)
    lay, kc, vc, ks, vs, kept = fill_cache(g, B, Hkv, T, D, True, 0.5, False, keep=(5,))
    k, v = kept[5]
    sk = oracle.fp8_calibrate(k)
    assert np.array_equal(sk[0], ks[5].cpu().numpy())
    assert np.array_equal(oracle.quant_fp8(k[:, :4096], sk)[0, :, 2], kc[5, 2, :4096].cpu().numpy())
    q = torch.randn(B, Hq, D, generator=g, device=DEV).to(torch.bfloat16)
    full = torch.full((B,), T, dtype=torch.int32, device=DEV)
    out = decode(q, kc, vc, ks, vs, lay, full, Hkv, T, True)
    assert torch.isfinite(out.float()).all()
    sample_check(out, q, kc, vc, ks, vs, full.cpu().numpy(), [(0, 0), (31, 7)], 8, True)
    # the fused step at this size: two chunks per sequence, the chunk that owns the sequence end writes the token
    decode_step_check(g, q, kc, vc, ks, vs, lay, full, Hkv, T, True, 0.5, False, [(3, 1), (31, 6)])


@pytest.mark.parametrize("Hq,Hkv,D", [(32, 8, 128), (16, 4, 256), (32, 8, 64)])
def test_config3_full_size_chunked_prefill(Hq, Hkv, D):
    """B=4 x 4096 tokens in 512-token chunks: sampled query rows of every chunk against the oracle over
    [dequantized int8 cache of earlier chunks | own bf16 K/V]; the cache ends up equal to one-shot quantization.
    Also at the head shape of Qwen3.5's full-attention layers (head_dim 256, the same flops and bytes)."""
    B, T, C = 4, 4096, 512
    g = gen(wl.SEED + 3 + D)
    q, k, v = source(g, (B, T, Hq, D)), source(g, (B, T, Hkv, D)), source(g, (B, T, Hkv, D))
    lay = hb.contiguous_layout(Hkv, T, D)
    kc = torch.zeros(B, Hkv, T, D, dtype=torch.int8, device=DEV)
    vc = torch.zeros_like(kc)
    ks = torch.zeros(B, Hkv, lay.scale_stride_head, dtype=torch.float32, device=DEV)
    vs = torch.zeros_like(ks)
    outs = []
    for i in range(0, T, C):
        o = torch.empty(B, C, Hq, D, dtype=torch.bfloat16, device=DEV)
        hb.prefill_attn(q[:, i:i + C].contiguous(), k[:, i:i + C].contiguous(), v[:, i:i + C].contiguous(), kc, vc, ks, vs,
                        lay, i, o, 1.0 / np.sqrt(D), True)
        outs.append(o)
    torch.cuda.synchronize()
    out = torch.cat(outs, 1)
    assert torch.isfinite(out.float()).all()
    r = wl.philox(33)
    for _ in range(6):
        b, h, pos = int(r.integers(B)), int(r.integers(Hkv)), int(r.integers(T))
        c0 = pos // C * C  # start of the chunk this row belongs to
        kd = torch.cat([kc[b, h, :c0].float() * ks[b, h, :c0, None], k[b, c0:pos + 1, h].float()]).cpu().numpy()
        vd = torch.cat([vc[b, h, :c0].float() * vs[b, h, :c0, None], v[b, c0:pos + 1, h].float()]).cpu().numpy()
        qb = q[b, pos, 4 * h:4 * h + 4].float().cpu().numpy()[None]
        want = oracle.decode_attn(qb, kd[None, :, None], vd[None, :, None], None, None, oracle.FMT_DENSE,
                                  np.array([pos + 1], np.int32), 1.0 / np.sqrt(D))[0]
        d = np.abs(out[b, pos, 4 * h:4 * h + 4].float().cpu().numpy() - want)
        assert d.max() < TOL_MAX and d.mean() < TOL_MEAN, (b, h, pos, d.max(), d.mean())
    wk, wks = oracle.quant_int8(k[1, :, Hkv - 3].float().cpu().numpy())
    assert np.array_equal(kc[1, Hkv - 3].cpu().numpy(), wk) and np.array_equal(ks[1, Hkv - 3, :T].cpu().numpy(), wks)


def test_config3_shape_with_fp8_history():
    """The same shape over an FP8 e4m3fn cache (per-head scales calibrated on the first chunk, N(0, 0.5^2) sources as
    in the FP8 decode configuration): sampled query rows against the oracle over [dequantized fp8 cache of earlier
    chunks | own bf16 K/V]; the finished cache holds the oracle's codes."""
    B, T, C, Hq, Hkv, D = 4, 4096, 512, 32, 8, 128
    g = gen(wl.SEED + 7)
    q = source(g, (B, T, Hq, D))
    k, v = source(g, (B, T, Hkv, D), 0.5), source(g, (B, T, Hkv, D), 0.5)
    lay = hb.contiguous_layout(Hkv, T, D)
    kc = torch.zeros(B, Hkv, T, D, dtype=torch.uint8, device=DEV)
    vc = torch.zeros_like(kc)
    ks = torch.zeros(B, Hkv, dtype=torch.float32, device=DEV)
    vs = torch.zeros_like(ks)
    hb.kv_fp8_calibrate(k[:, :C].contiguous(), v[:, :C].contiguous(), ks, vs)
    outs = []
    for i in range(0, T, C):
        o = torch.empty(B, C, Hq, D, dtype=torch.bfloat16, device=DEV)
        hb.prefill_attn(q[:, i:i + C].contiguous(), k[:, i:i + C].contiguous(), v[:, i:i + C].contiguous(), kc, vc, ks, vs,
                        lay, i, o, 1.0 / np.sqrt(D), True, fp8=True)
        outs.append(o)
    torch.cuda.synchronize()
    out = torch.cat(outs, 1)
    assert torch.isfinite(out.float()).all()
    ksn, vsn = ks.cpu().numpy(), vs.cpu().numpy()
    r = wl.philox(37)
    for _ in range(6):
        b, h, pos = int(r.integers(B)), int(r.integers(Hkv)), int(r.integers(T))
        c0 = pos // C * C
        kh = oracle.dequant_fp8(kc[b, h, :c0].cpu().numpy()[None, :, None], ksn[b:b + 1, h:h + 1])[0, :, 0]
        vh = oracle.dequant_fp8(vc[b, h, :c0].cpu().numpy()[None, :, None], vsn[b:b + 1, h:h + 1])[0, :, 0]
        kd = np.concatenate([kh, k[b, c0:pos + 1, h].float().cpu().numpy()])
        vd = np.concatenate([vh, v[b, c0:pos + 1, h].float().cpu().numpy()])
        qb = q[b, pos, 4 * h:4 * h + 4].float().cpu().numpy()[None]
        want = oracle.decode_attn(qb, kd[None, :, None], vd[None, :, None], None, None, oracle.FMT_DENSE,
                                  np.array([pos + 1], np.int32), 1.0 / np.sqrt(D))[0]
        d = np.abs(out[b, pos, 4 * h:4 * h + 4].float().cpu().numpy() - want)
        assert d.max() < TOL_MAX and d.mean() < TOL_MEAN, (b, h, pos, d.max(), d.mean())
    # the finished cache holds the oracle's codes for a sampled (sequence, head)
    wk = oracle.quant_fp8(k[2, :, 3].float().cpu().numpy()[None, :, None], ksn[2:3, 3:4])[0, :, 0]
    assert np.array_equal(kc[2, 3].cpu().numpy(), wk)


@pytest.mark.parametrize("B,copy,fp8", [(4, True, False), (4, True, True), (1, False, False), (1, True, False)])
def test_config3_full_size_prompt_copy_and_single_sequence(B, copy, fp8):
    """The launches the other prefill workloads time, at their size: 4096-token prompts in 512-token chunks with the
    history read from the bf16 copy of the prompt (int8 and FP8 caches), and one sequence alone, where the library
    splits the keys of a query tile over several workgroups (with the codes and with the copy).  Sampled query rows of
    every part of the prompt against the oracle over [dequantized cache of earlier chunks | own bf16 K/V]; the cache
    ends up as the oracle's codes; a second run gives the same bits (the merge order of the key runs is fixed)."""
    T, C, Hq, Hkv, D = 4096, 512, 32, 8, 128
    g = gen(wl.SEED + 11 + B + 2 * copy + 4 * fp8)
    sg = 0.5 if fp8 else 1.0
    q, k, v = source(g, (B, T, Hq, D)), source(g, (B, T, Hkv, D), sg), source(g, (B, T, Hkv, D), sg)
    lay = hb.contiguous_layout(Hkv, T, D)
    split_ws = hb.prefill_split_workspace(B, C, Hq, Hkv, D)

    def run():
        kc = torch.zeros(B, Hkv, T, D, dtype=torch.uint8 if fp8 else torch.int8, device=DEV)
        vc = torch.zeros_like(kc)
        ks = torch.zeros((B, Hkv) if fp8 else (B, Hkv, lay.scale_stride_head), dtype=torch.float32, device=DEV)
        vs = torch.zeros_like(ks)
        if fp8:
            hb.kv_fp8_calibrate(k[:, :C].contiguous(), v[:, :C].contiguous(), ks, vs)
        shadow = hb.prefill_shadow(B, Hkv, D, T) if copy else None
        outs = []
        for i in range(0, T, C):
            o = torch.full((B, C, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
            hb.prefill_attn(q[:, i:i + C].contiguous(), k[:, i:i + C].contiguous(), v[:, i:i + C].contiguous(), kc, vc, ks, vs,
                            lay, i, o, 1.0 / np.sqrt(D), True, fp8=fp8, columns=0, split_workspace=split_ws, shadow=shadow)
            outs.append(o)
        torch.cuda.synchronize()
        return torch.cat(outs, 1), kc, vc, ks, vs

    out, kc, vc, ks, vs = run()
    assert torch.isfinite(out.float()).all()
    again = run()[0]
    assert torch.equal(out.view(torch.int16), again.view(torch.int16))
    ksn, vsn = ks.cpu().numpy(), vs.cpu().numpy()
    r = wl.philox(41 + B + copy)
    for i in range(8):
        b, h = int(r.integers(B)), int(r.integers(Hkv))
        pos = C * i + int(r.integers(C))  # one row of every chunk: every history length and key-run count
        c0 = pos // C * C
        if fp8:
            kh = oracle.dequant_fp8(kc[b, h, :c0].cpu().numpy()[None, :, None], ksn[b:b + 1, h:h + 1])[0, :, 0]
            vh = oracle.dequant_fp8(vc[b, h, :c0].cpu().numpy()[None, :, None], vsn[b:b + 1, h:h + 1])[0, :, 0]
        else:
            kh = (kc[b, h, :c0].float() * ks[b, h, :c0, None]).cpu().numpy()
            vh = (vc[b, h, :c0].float() * vs[b, h, :c0, None]).cpu().numpy()
        kd = np.concatenate([kh, k[b, c0:pos + 1, h].float().cpu().numpy()])
        vd = np.concatenate([vh, v[b, c0:pos + 1, h].float().cpu().numpy()])
        qb = q[b, pos, 4 * h:4 * h + 4].float().cpu().numpy()[None]
        want = oracle.decode_attn(qb, kd[None, :, None], vd[None, :, None], None, None, oracle.FMT_DENSE,
                                  np.array([pos + 1], np.int32), 1.0 / np.sqrt(D))[0]
        d = np.abs(out[b, pos, 4 * h:4 * h + 4].float().cpu().numpy() - want)
        assert d.max() < TOL_MAX and d.mean() < TOL_MEAN, (b, h, pos, d.max(), d.mean())
    b, h = B - 1, Hkv - 3
    if fp8:
        wk = oracle.quant_fp8(k[b, :, h].float().cpu().numpy()[None, :, None], ksn[b:b + 1, h:h + 1])[0, :, 0]
        assert np.array_equal(kc[b, h].cpu().numpy(), wk)
    else:
        wk, wks = oracle.quant_int8(k[b, :, h].float().cpu().numpy())
        assert np.array_equal(kc[b, h].cpu().numpy(), wk) and np.array_equal(ks[b, h, :T].cpu().numpy(), wks)


def test_cache_tensors_beyond_2_gib():
    """Maximum sizes: K and V code tensors of 2.5 GiB each (80 sequences x 32768 tokens x 8 heads x 128), where a 32-bit
    element or byte offset wraps (the reference's `n as i32` counts do at this scale, kv_cache.rs:832).  The bulk
    writer, decode attention, the fused decode step and a prefill chunk over the longest history, each checked against
    the oracle on sequences whose offsets lie beyond 2^31; then the same codes read through a block table whose entries
    point beyond 2^31 bytes into the pool."""
    B, Hq, Hkv, D, T = 80, 32, 8, 128, 32768
    assert B * Hkv * T * D > 2 ** 31
    g = gen(wl.SEED + 21)
    lay, kc, vc, ks, vs, kept = fill_cache(g, B, Hkv, T, D, False, 1.0, True, keep=(79,))
    k79, _ = kept[79]
    wk, wks = oracle.quant_int8(k79[:, :, 6])
    assert np.array_equal(kc[79, 6].cpu().numpy(), wk[0]) and np.array_equal(ks[79, 6, :T].cpu().numpy(), wks[0])
    q = torch.randn(B, Hq, D, generator=g, device=DEV).to(torch.bfloat16)
    lens = torch.full((B,), T - 64, dtype=torch.int32, device=DEV)
    lens[70] = 20001
    out = decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, False)
    assert torch.isfinite(out.float()).all()
    sample_check(out, q, kc, vc, ks, vs, lens.cpu().numpy(), [(0, 0), (70, 3), (79, 7)], 4, False)
    decode_step_check(g, q, kc, vc, ks, vs, lay, lens, Hkv, T, False, 1.0, True, [(66, 1), (79, 6)])
    # a 64-token chunk on top of T - 64 cached tokens, rows of the last sequences against the oracle
    S, H = 64, T - 64
    qn, kn, vn = source(g, (B, S, Hq, D)), source(g, (B, S, Hkv, D)), source(g, (B, S, Hkv, D))
    lens.fill_(H)  # (the decode step above moved nothing: it rewrote position len - 1)
    o = torch.full((B, S, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    hb.prefill_attn(qn, kn, vn, kc, vc, ks, vs, lay, H, o, 1.0 / np.sqrt(D), True)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all()
    for b, h, pos in ((79, 7, 63), (72, 0, 5)):
        kd = torch.cat([kc[b, h, :H].float() * ks[b, h, :H, None], kn[b, :pos + 1, h].float()]).cpu().numpy()
        vd = torch.cat([vc[b, h, :H].float() * vs[b, h, :H, None], vn[b, :pos + 1, h].float()]).cpu().numpy()
        qb = qn[b, pos, 4 * h:4 * h + 4].float().cpu().numpy()[None]
        want = oracle.decode_attn(qb, kd[None, :, None], vd[None, :, None], None, None, oracle.FMT_DENSE,
                                  np.array([H + pos + 1], np.int32), 1.0 / np.sqrt(D))[0]
        d = np.abs(o[b, pos, 4 * h:4 * h + 4].float().cpu().numpy() - want)
        assert d.max() < TOL_MAX and d.mean() < TOL_MEAN, (b, h, pos, d.max(), d.mean())
    wkn, wksn = oracle.quant_int8(kn[79].float().cpu().numpy()[None])
    assert np.array_equal(kc[79, :, H:].cpu().numpy(), wkn[0].transpose(1, 0, 2))
    assert np.array_equal(ks[79, :, H:T].cpu().numpy(), wksn[0].transpose(1, 0))
    # the same memory as a pool of 256-token blocks [B * T / 256 blocks, Hkv, 256, D]: sequence b's blocks are
    # b * 128 .. b * 128 + 127 of a layout in which a block is one (sequence, 256-token) slab -- which the contiguous
    # [B, Hkv, T, D] tensor is not, so the pool is filled from it for three sequences at the far end
    BT, nblk = 256, T // 256
    pool_k = torch.zeros(B * nblk, Hkv, BT, D, dtype=torch.int8, device=DEV)
    pool_v = torch.zeros_like(pool_k)
    pool_ks = torch.zeros(B * nblk, Hkv, BT, dtype=torch.float32, device=DEV)
    pool_vs = torch.zeros_like(pool_ks)
    tab = torch.zeros(B, nblk, dtype=torch.int32, device=DEV)
    perm = torch.randperm(B * nblk, generator=g, device=DEV).to(torch.int32).view(B, nblk)
    tab.copy_(perm)
    far = [b for b in range(B) if int(perm[b].max()) * Hkv * BT * D > 2 ** 31][:3]
    assert len(far) == 3
    for b in far:
        idx = perm[b].long()
        pool_k[idx] = kc[b].view(Hkv, nblk, BT, D).permute(1, 0, 2, 3)
        pool_v[idx] = vc[b].view(Hkv, nblk, BT, D).permute(1, 0, 2, 3)
        pool_ks[idx] = ks[b, :, :T].reshape(Hkv, nblk, BT).permute(1, 0, 2)
        pool_vs[idx] = vs[b, :, :T].reshape(Hkv, nblk, BT).permute(1, 0, 2)
    play = hb.paged_layout(Hkv, BT, D, tab, tab)
    plens = torch.zeros(B, dtype=torch.int32, device=DEV)
    for b in far:
        plens[b] = T
    pout = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    hb.decode_attn(q, pool_k, pool_v, pool_ks, pool_vs, play, plens, pout, ws, Hkv, T, 1.0 / np.sqrt(D))
    full = torch.full((B,), T, dtype=torch.int32, device=DEV)
    cout = decode(q, kc, vc, ks, vs, lay, full, Hkv, T, False)
    torch.cuda.synchronize()
    for b in far:  # the same codes, the same chunking: the same bits
        assert torch.equal(pout[b].view(torch.int16), cout[b].view(torch.int16)), b


def test_config5_full_size_deltanet():
    """Decode at B = 64 (whole batch against the oracle) and prefill at B = 4 x 4096 (two sampled heads against
    the oracle, and chunked calls with carried state against the single call)."""
    nk, nv, d = 16, 32, 128
    g = gen(wl.SEED + 5)
    nrm = lambda x: (x / x.norm(dim=-1, keepdim=True).clamp_min(1e-3)).to(torch.bfloat16)
    B = 64
    q, k = nrm(torch.randn(B, 1, nk, d, generator=g, device=DEV)), nrm(torch.randn(B, 1, nk, d, generator=g, device=DEV))
    v = torch.randn(B, 1, nv, d, generator=g, device=DEV).to(torch.bfloat16)
    gg = -torch.nn.functional.softplus(torch.randn(B, 1, nv, generator=g, device=DEV))
    beta = torch.sigmoid(torch.randn(B, 1, nv, generator=g, device=DEV))
    s0 = torch.randn(B, nv, d, d, generator=g, device=DEV) * 0.1
    st, out = s0.clone(), torch.empty(B, 1, nv, d, device=DEV)
    hb.deltanet_forward(q, k, v, gg, beta, st, out, 1 / np.sqrt(d), False)
    torch.cuda.synchronize()
    wo, ws = oracle.deltanet_recurrent(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(),
                                       gg.cpu().numpy(), beta.cpu().numpy(), s0.cpu().numpy(), 1 / np.sqrt(d), False)
    assert np.abs(out.cpu().numpy() - wo).max() < 1e-5 and np.abs(st.cpu().numpy() - ws).max() < 1e-5
    B, T = 4, 4096
    q, k = nrm(torch.randn(B, T, nk, d, generator=g, device=DEV)), nrm(torch.randn(B, T, nk, d, generator=g, device=DEV))
    v = torch.randn(B, T, nv, d, generator=g, device=DEV).to(torch.bfloat16)
    gg = -torch.nn.functional.softplus(torch.randn(B, T, nv, generator=g, device=DEV))
    beta = torch.sigmoid(torch.randn(B, T, nv, generator=g, device=DEV))
    st, out = torch.zeros(B, nv, d, d, device=DEV), torch.empty(B, T, nv, d, device=DEV)
    hb.deltanet_forward(q, k, v, gg, beta, st, out, 1 / np.sqrt(d), False)
    st2, out2 = torch.zeros(B, nv, d, d, device=DEV), torch.empty(B, T, nv, d, device=DEV)
    for i in range(0, T, 1024):  # four calls carrying the state
        o = torch.empty(B, 1024, nv, d, device=DEV)
        hb.deltanet_forward(q[:, i:i + 1024].contiguous(), k[:, i:i + 1024].contiguous(), v[:, i:i + 1024].contiguous(),
                            gg[:, i:i + 1024].contiguous(), beta[:, i:i + 1024].contiguous(), st2, o, 1 / np.sqrt(d), False)
        out2[:, i:i + 1024] = o
    torch.cuda.synchronize()
    assert torch.equal(out, out2) and torch.equal(st, st2)
    for b, j in ((0, 0), (3, 31)):  # v-head j reads k-head j // 2
        hk = j // 2
        wo, ws = oracle.deltanet_recurrent(q[b:b + 1, :, hk:hk + 1].float().cpu().numpy(), k[b:b + 1, :, hk:hk + 1].float().cpu().numpy(),
                                           v[b:b + 1, :, j:j + 1].float().cpu().numpy(), gg[b:b + 1, :, j:j + 1].cpu().numpy(),
                                           beta[b:b + 1, :, j:j + 1].cpu().numpy(), None, 1 / np.sqrt(d), False)
        assert np.abs(out[b, :, j].cpu().numpy() - wo[0, :, 0]).max() < 1e-4
        assert np.abs(st[b, j].cpu().numpy() - ws[0, 0]).max() < 1e-4


def test_config5_full_size_chunked_deltanet():
    """B = 4 x 4096 tokens, chunk size 64, on the matrix pipe: sampled (sequence, head) pairs against the oracle of
    the recurrence, the whole output against the fp32 recurrent kernel, and four calls carrying the state
    (cut at multiples of 64) against the single call, bit for bit."""
    nk, nv, d = 16, 32, 128
    g = gen(wl.SEED + 55)
    nrm = lambda x: (x / x.norm(dim=-1, keepdim=True).clamp_min(1e-3)).to(torch.bfloat16)
    B, T = 4, 4096
    q, k = nrm(torch.randn(B, T, nk, d, generator=g, device=DEV)), nrm(torch.randn(B, T, nk, d, generator=g, device=DEV))
    v = torch.randn(B, T, nv, d, generator=g, device=DEV).to(torch.bfloat16)
    gg = -torch.nn.functional.softplus(torch.randn(B, T, nv, generator=g, device=DEV))
    beta = torch.sigmoid(torch.randn(B, T, nv, generator=g, device=DEV))
    qs = 1 / np.sqrt(d)
    st, out = torch.zeros(B, nv, d, d, device=DEV), torch.full((B, T, nv, d), float("nan"), device=DEV)
    ws = hb.deltanet_forward_chunked(q, k, v, gg, beta, st, out, qs, False)
    st2, out2 = torch.zeros(B, nv, d, d, device=DEV), torch.empty(B, T, nv, d, device=DEV)
    for i in range(0, T, 1024):
        o = torch.empty(B, 1024, nv, d, device=DEV)
        hb.deltanet_forward_chunked(q[:, i:i + 1024].contiguous(), k[:, i:i + 1024].contiguous(), v[:, i:i + 1024].contiguous(),
                                    gg[:, i:i + 1024].contiguous(), beta[:, i:i + 1024].contiguous(), st2, o, qs, False, workspace=ws)
        out2[:, i:i + 1024] = o
    st3, out3 = torch.zeros(B, nv, d, d, device=DEV), torch.empty(B, T, nv, d, device=DEV)
    hb.deltanet_forward(q, k, v, gg, beta, st3, out3, qs, False)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all() and torch.equal(out, out2) and torch.equal(st, st2)
    rel = 3e-3
    assert float((out - out3).abs().max()) <= rel * float(out3.abs().max())
    assert float((st - st3).abs().max()) <= rel * float(st3.abs().max())
    for b, j in ((0, 1), (3, 30)):
        hk = j // 2
        wo, wst = oracle.deltanet_recurrent(q[b:b + 1, :, hk:hk + 1].float().cpu().numpy(), k[b:b + 1, :, hk:hk + 1].float().cpu().numpy(),
                                            v[b:b + 1, :, j:j + 1].float().cpu().numpy(), gg[b:b + 1, :, j:j + 1].cpu().numpy(),
                                            beta[b:b + 1, :, j:j + 1].cpu().numpy(), None, qs, False)
        eo = np.abs(out[b, :, j].cpu().numpy() - wo[0, :, 0]).max()
        es = np.abs(st[b, j].cpu().numpy() - wst[0, 0]).max()
        assert eo <= rel * np.abs(wo).max() and es <= rel * np.abs(wst).max(), (b, j, eo, es)
        assert eo < TOL_MAX


def test_head_dim_256_full_size_decode():
    """The Qwen3.5 full-attention head shape at the size of config 2: B=64, Hq 16 / Hkv 4, D 256, T 8192, int8."""
    B, Hq, Hkv, D, T = 64, 16, 4, 256, 8192
    g = gen(wl.SEED + 256)
    lay, kc, vc, ks, vs, kept = fill_cache(g, B, Hkv, T, D, False, 1.0, True, keep=(7,))
    kk, _ = kept[7]
    wk, wks = oracle.quant_int8(kk[:, :, 1])
    assert np.array_equal(kc[7, 1].cpu().numpy(), wk[0]) and np.array_equal(ks[7, 1, :T].cpu().numpy(), wks[0])
    q = torch.randn(B, Hq, D, generator=g, device=DEV).to(torch.bfloat16)
    lens = torch.randint(512, T + 1, (B,), generator=g, device=DEV, dtype=torch.int32)
    lens[0] = T
    out = decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, False)
    assert torch.isfinite(out.float()).all()
    sample_check(out, q, kc, vc, ks, vs, lens.cpu().numpy(), [(0, 0), (33, 3)], 4, False)
    two = decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, False, phases=12)
    assert (two.float() - out.float()).abs().max() <= 2 ** -8 * max(1.0, float(out.float().abs().max()))
    vc.fill_(64)
    vs.fill_(0.125)
    const = decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, False)
    assert (const.float() - 8.0).abs().max() <= 2 ** -5


def test_head_dim_64_full_size_decode():
    """64-wide heads at the cache size of config 2: B=64, Hq 32 / Hkv 16, D 64, T 8192, int8 (64-token wavefront steps)."""
    B, Hq, Hkv, D, T = 64, 32, 16, 64, 8192
    g = gen(wl.SEED + 64)
    lay, kc, vc, ks, vs, kept = fill_cache(g, B, Hkv, T, D, False, 1.0, True, keep=(7,))
    kk, _ = kept[7]
    wk, wks = oracle.quant_int8(kk[:, :, 1])
    assert np.array_equal(kc[7, 1].cpu().numpy(), wk[0]) and np.array_equal(ks[7, 1, :T].cpu().numpy(), wks[0])
    q = torch.randn(B, Hq, D, generator=g, device=DEV).to(torch.bfloat16)
    lens = torch.randint(512, T + 1, (B,), generator=g, device=DEV, dtype=torch.int32)
    lens[0] = T
    out = decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, False)
    assert torch.isfinite(out.float()).all()
    sample_check(out, q, kc, vc, ks, vs, lens.cpu().numpy(), [(0, 0), (33, 11)], 2, False)
    two = decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, False, phases=12)
    assert (two.float() - out.float()).abs().max() <= 2 ** -8 * max(1.0, float(out.float().abs().max()))
    vc.fill_(64)
    vs.fill_(0.125)
    const = decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, False)
    assert (const.float() - 8.0).abs().max() <= 2 ** -5
