"""GPU parity: causal prefill attention over [int8 history | bf16 new tokens] against the CPU oracle."""
import os

import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV, DeviceCache, bf16_from_bits, run_decode

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["auto", "256", "128", "32", "16", "split8", "split2x128"])
def columns_per_workgroup(request, monkeypatch):
    """Every test runs with the library's own choice of workgroup width (half-width workgroups for small grids) and
    with each instance forced -- 256 columns on 16x16x32 MFMA tiles, 128 columns, 256 columns on 32x32x16 tiles, 256
    columns on sixteen wavefronts (the last two: head_dim 128 without a window; elsewhere the same as 256) -- so that
    small shapes exercise every kernel; and with the keys of every query tile split into runs whose partial results the
    last workgroup to finish merges: 8 runs of full-width tiles, 2 of half-width ones (runs may be empty: most of these
    shapes have fewer steps than 8)."""
    name = request.param
    split = int(name[5]) if name.startswith("split") else 0
    cols = int(name.split("x")[1]) if "x" in name else 0 if split or name == "auto" else int(name)
    monkeypatch.setattr(hb, "PREFILL_COLUMNS", cols)
    monkeypatch.setattr(hb, "PREFILL_KEY_SPLITS", split)

TOL_MAX, TOL_MEAN = 2e-2, 2e-3


def _fixes_its_own_instance():
    """For tests that pass the width and the split themselves: run them once, not once per value of the fixture."""
    if hb.PREFILL_COLUMNS != 0 or hb.PREFILL_KEY_SPLITS != 0:
        pytest.skip("chooses its own instance: run under the fixture's first value only")


def bf16r(x):
    return wl.bf16_bits_to_f32(wl.to_bf16_bits(x))


def make(stream, B, S, Hq, Hkv, D=128, sigma=1.0):
    r = wl.philox(stream)
    q = bf16r(r.standard_normal((B, S, Hq, D)).astype(np.float32))
    k = bf16r((r.standard_normal((B, S, Hkv, D)) * sigma).astype(np.float32))
    v = bf16r((r.standard_normal((B, S, Hkv, D)) * sigma).astype(np.float32))
    return q, k, v


def gpu_prefill(cache, q, k, v, hist, write=True):
    B, S, Hq, D = q.shape
    qt, kt, vt = (torch.from_numpy(x).to(DEV).bfloat16().contiguous() for x in (q, k, v))
    out = torch.full((B, S, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    hb.prefill_attn(qt, kt, vt, cache.k_codes, cache.v_codes, cache.k_scales, cache.v_scales, cache.layout, hist, out,
                    1.0 / np.sqrt(D), write, fp8=cache.fp8)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


def oracle_prefill(q, k_hist_deq, v_hist_deq, k, v):
    """Dense fp32 K/V = [dequantized history | exact new tokens]; causal with the k_len - q_len offset."""
    B, S = q.shape[:2]
    kd = np.concatenate([k_hist_deq, k], 1) if k_hist_deq is not None else k
    vd = np.concatenate([v_hist_deq, v], 1) if v_hist_deq is not None else v
    T = kd.shape[1]
    return oracle.prefill_attn(q, kd, vd, None, None, oracle.FMT_DENSE, np.full(B, T, np.int32),
                               1.0 / np.sqrt(q.shape[-1]))


def compare(got, want, label):
    assert np.isfinite(got).all(), label
    d = np.abs(got - want)
    print("%s max-abs %.3e mean-abs %.3e" % (label, d.max(), d.mean()), flush=True)
    assert d.max() < TOL_MAX and d.mean() < TOL_MEAN, label


@pytest.mark.parametrize("S", [1, 5, 16, 33, 100, 257])
def test_prompt_without_history(S):
    q, k, v = make(20 + S, 2, S, 32, 8)
    c = DeviceCache(2, 8, S, 128)
    got = gpu_prefill(c, q, k, v, 0)
    compare(got, oracle_prefill(q, None, None, k, v), "prompt S=%d" % S)
    # quantize-on-write left the whole prompt in the cache, bit-exact with the oracle
    kc, vc, ks, vs = c.canonical(S)
    wk, wks = oracle.quant_int8(k)
    wv, wvs = oracle.quant_int8(v)
    assert np.array_equal(kc, wk) and np.array_equal(vc, wv) and np.array_equal(ks, wks) and np.array_equal(vs, wvs)


def test_long_prompt_more_workgroups_than_cus():
    """18 query tiles x 8 kv-heads x 2 sequences = 288 workgroups: more than the chip's CUs, which is when the
    kernel starts the query tiles with the most keys first."""
    q, k, v = make(33, 2, 1100, 32, 8)
    c = DeviceCache(2, 8, 1100, 128)
    got = gpu_prefill(c, q, k, v, 0)
    compare(got, oracle_prefill(q, None, None, k, v), "prompt S=1100")


def test_paged_blocks_must_hold_multiples_of_64_tokens():
    B, Hq, Hkv, D, BT = 1, 8, 2, 128, 96
    q, k, v = make(34, B, 8, Hq, Hkv)
    tab = torch.zeros(B, 2, dtype=torch.int32, device=DEV)
    pool_c = torch.zeros(4, Hkv, BT, D, dtype=torch.int8, device=DEV)
    pool_s = torch.zeros(4, Hkv, BT, dtype=torch.float32, device=DEV)
    lay = hb.paged_layout(Hkv, BT, D, tab, tab)
    qt, kt, vt = (torch.from_numpy(x).to(DEV).bfloat16().contiguous() for x in (q, k, v))
    out = torch.empty(B, 8, Hq, D, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(hb.HsError, match="multiple of 64"):
        hb.prefill_attn(qt, kt, vt, pool_c, pool_c, pool_s, pool_s, lay, 0, out, 1.0 / np.sqrt(D), False)


@pytest.mark.parametrize("hist,S", [(19, 5), (1, 1), (32, 64), (100, 37), (256, 256)])
def test_cached_prefill_with_int8_history(hist, S):
    """New rows on top of an int8 history: the reference's partial-prefill case (tril(k_len - q_len))."""
    B, Hq, Hkv = 2, 8, 2
    qh, kh, vh = make(40 + hist, B, hist, Hq, Hkv)
    q, k, v = make(41 + S, B, S, Hq, Hkv)
    c = DeviceCache(B, Hkv, hist + S, 128)
    hk, hv = torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16()
    c.write(hk, hv, None, 0)
    got = gpu_prefill(c, q, k, v, hist)
    kc, vc, ks, vs = c.canonical(hist)
    want = oracle_prefill(q, oracle.dequant_int8(kc, ks), oracle.dequant_int8(vc, vs), k, v)
    compare(got, want, "hist=%d S=%d" % (hist, S))
    assert c.k_codes[:, :, hist:hist + S].any()  # the new rows were cached behind the history


@pytest.mark.parametrize("kmag,vmag", [(1e-5, 1e5), (1e5, 1e-5), (3e-7, 3e-7), (1.0, 1e9)])
@pytest.mark.parametrize("fp8", [False, True])
def test_history_magnitude_ranges(kmag, vmag, fp8):
    """The prefill twin of the decode test of large and tiny magnitudes.  The history enters the products as fp16, which
    holds 2^-14 .. 65504 only; operands are taken relative to a power-of-two reference per (sequence, kv-head), so a
    cache that is tiny or huge as a whole (a model with small or large K/V projections) keeps the relative accuracy of
    an N(0,1) one.  Sequence 1 carries the opposite magnitudes of sequence 0.  The comparison is relative to the
    largest output, because the outputs themselves scale with vmag."""
    B, Hq, Hkv, hist, S = 2, 8, 2, 150, 70
    qh, kh, vh = make(90, B, hist, Hq, Hkv)
    q, k, v = make(91, B, S, Hq, Hkv)
    mags = np.array([[kmag, vmag], [vmag, kmag]], np.float32)
    kh, vh = bf16r(kh * mags[:, 0, None, None, None]), bf16r(vh * mags[:, 1, None, None, None])
    k, v = bf16r(k * mags[:, 0, None, None, None]), bf16r(v * mags[:, 1, None, None, None])
    q = bf16r(q / np.maximum(mags[:, 0, None, None, None], 1e-3))  # keeps the scores of a size where several keys matter
    c = DeviceCache(B, Hkv, hist + S, 128, fp8=fp8)
    hk, hv = torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16()
    if fp8:
        hb.kv_fp8_calibrate(hk, hv, c.k_scales, c.v_scales)
    c.write(hk, hv, None, 0)
    got = gpu_prefill(c, q, k, v, hist, write=False)
    kc, vc, ks, vs = c.canonical(hist)
    deq = oracle.dequant_fp8 if fp8 else oracle.dequant_int8
    want = oracle_prefill(q, deq(kc, ks), deq(vc, vs), k, v)
    assert np.isfinite(got).all()
    for b in range(B):
        top = np.abs(want[b]).max()
        d = np.abs(got[b] - want[b])
        assert d.max() < 2e-2 * top and d.mean() < 2e-3 * top, (b, d.max() / top, d.mean() / top)


def test_history_row_far_above_its_heads_reference_saturates():
    """Inside one (sequence, kv-head) the fp16 window is relative: a cached token whose scale is more than 2^11 times
    the largest scale among the head's first 64 tokens saturates (pinned here: finite output, and equal to attention
    over the history with that row's scale clamped to 512 * 2^E), while one 2^10 times the reference is still exact."""
    B, Hq, Hkv, hist, S = 1, 4, 1, 128, 16
    qh, kh, vh = make(92, B, hist, Hq, Hkv)
    q, k, v = make(93, B, S, Hq, Hkv)
    vh[0, 100] *= 2.0 ** 10   # inside the window
    c = DeviceCache(B, Hkv, hist + S, 128)
    c.write(torch.from_numpy(bf16r(vh * 0 + kh)).to(DEV).bfloat16(), torch.from_numpy(bf16r(vh)).to(DEV).bfloat16(), None, 0)
    got = gpu_prefill(c, q, k, v, hist, write=False)
    kc, vc, ks, vs = c.canonical(hist)
    want = oracle_prefill(q, oracle.dequant_int8(kc, ks), oracle.dequant_int8(vc, vs), k, v)
    top = np.abs(want).max()
    assert np.abs(got - want).max() < 2e-2 * top
    # far outside: V row 100 at 2^14 times the typical scale
    vh[0, 100] *= 2.0 ** 4
    c.write(torch.from_numpy(bf16r(kh)).to(DEV).bfloat16(), torch.from_numpy(bf16r(vh)).to(DEV).bfloat16(), None, 0)
    got = gpu_prefill(c, q, k, v, hist, write=False)
    assert np.isfinite(got).all()
    kc, vc, ks, vs = c.canonical(hist)
    ref_scale = vs[0, :64, 0].max()
    E = np.frexp(ref_scale)[1] + 2                       # reference * 2^-E in [1/8, 1/4)
    vd = oracle.dequant_int8(vc, vs)
    assert vs[0, 100, 0] * 2.0 ** -E > 512.0
    vd[0, 100] = vc[0, 100].astype(np.float32) * np.float32(512.0 * 2.0 ** E)  # the relative scale clamps at 512
    sat = oracle_prefill(q, oracle.dequant_int8(kc, ks), vd, k, v)
    assert np.abs(got - sat).max() < 2e-2 * np.abs(sat).max()


@pytest.mark.parametrize("hist,S,sigma", [(19, 5, 1.0), (64, 64, 0.5), (150, 70, 0.5), (333, 200, 1.0)])
def test_cached_prefill_with_fp8_history(hist, S, sigma):
    """The same over an e4m3fn history with per-head scales: the new rows are encoded with the scales calibrated
    on the history (values beyond 448 * scale clamp, as in the oracle), then join the attended history."""
    B, Hq, Hkv = 2, 8, 2
    qh, kh, vh = make(70 + hist, B, hist, Hq, Hkv, sigma=sigma)
    q, k, v = make(71 + S, B, S, Hq, Hkv, sigma=sigma)
    c = DeviceCache(B, Hkv, hist + S, 128, fp8=True)
    hk, hv = torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16()
    hb.kv_fp8_calibrate(hk, hv, c.k_scales, c.v_scales)
    c.write(hk, hv, None, 0)
    got = gpu_prefill(c, q, k, v, hist)
    kc, vc, ks, vs = c.canonical(hist + S)
    want = oracle_prefill(q, oracle.dequant_fp8(kc[:, :hist], ks), oracle.dequant_fp8(vc[:, :hist], vs), k, v)
    compare(got, want, "fp8 hist=%d S=%d" % (hist, S))
    # the new rows were cached behind the history with the oracle's codes
    ek, ev = oracle.quant_fp8(k, ks), oracle.quant_fp8(v, vs)
    assert np.array_equal(kc[:, hist:], ek) and np.array_equal(vc[:, hist:], ev)


def test_fp8_history_with_subnormal_codes_and_every_code_value():
    """All 254 finite e4m3fn codes (subnormals included) in the history convert exactly: one key per code value
    in V (K codes cycle too), compared with the oracle's dequantized view."""
    B, Hq, Hkv, D, hist, S = 1, 4, 1, 128, 256, 16
    r = wl.philox(77)
    codes = np.arange(256, dtype=np.uint8)
    codes[codes == 0x7f] = 0x7e
    codes[codes == 0xff] = 0xfe
    kc = np.stack([np.roll(codes, 3 * d) for d in range(D)], -1).reshape(1, hist, 1, D)
    vc = np.stack([np.roll(codes, 7 * d + 1) for d in range(D)], -1).reshape(1, hist, 1, D)
    ks = np.array([[0.004]], np.float32)
    vs = np.array([[0.02]], np.float32)
    c = DeviceCache(B, Hkv, hist + S, D, fp8=True)
    c.load_canonical(kc, vc, ks, vs)
    q, k, v = make(78, B, S, Hq, Hkv)
    got = gpu_prefill(c, q, k, v, hist, write=False)
    want = oracle_prefill(q, oracle.dequant_fp8(kc, ks), oracle.dequant_fp8(vc, vs), k, v)
    compare(got, want, "fp8 all codes")


def test_paged_fp8_history_matches_contiguous():
    """FP8 history in 64-token blocks scattered through one pool: the same bits as over the contiguous cache."""
    B, Hq, Hkv, D, hist, S, BT = 2, 8, 2, 128, 150, 70, 64
    qh, kh, vh = make(110, B, hist, Hq, Hkv, sigma=0.5)
    q, k, v = make(111, B, S, Hq, Hkv, sigma=0.5)
    c = DeviceCache(B, Hkv, hist + S, D, fp8=True)
    hk, hv = torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16()
    hb.kv_fp8_calibrate(hk, hv, c.k_scales, c.v_scales)
    c.write(hk, hv, None, 0)
    want = gpu_prefill(c, q, k, v, hist)
    nblk = (hist + S + BT - 1) // BT
    ids = wl.philox(112).permutation(2 * B * nblk + 3).astype(np.int32)
    kt, vt = ids[:B * nblk].reshape(B, nblk), ids[B * nblk:2 * B * nblk].reshape(B, nblk)
    pool_c = torch.zeros(len(ids), Hkv, BT, D, dtype=torch.uint8, device=DEV)
    k_tab, v_tab = torch.from_numpy(kt).to(DEV), torch.from_numpy(vt).to(DEV)
    lay = hb.paged_layout(Hkv, BT, D, k_tab, v_tab)
    hb.kv_quantize_fp8(hk, hv, pool_c, pool_c, c.k_scales, c.v_scales, lay, None, 0)
    qt, knew, vnew = (torch.from_numpy(x).to(DEV).bfloat16().contiguous() for x in (q, k, v))
    out = torch.empty(B, S, Hq, D, dtype=torch.bfloat16, device=DEV)
    hb.prefill_attn(qt, knew, vnew, pool_c, pool_c, c.k_scales, c.v_scales, lay, hist, out, 1.0 / np.sqrt(D), True, fp8=True)
    torch.cuda.synchronize()
    assert np.array_equal(out.float().cpu().numpy(), want)
    dense = torch.empty(B, hist + S, Hkv, D, dtype=torch.float32, device=DEV)
    ref = torch.empty_like(dense)
    hb.kv_dequantize(pool_c, c.k_scales, True, lay, 0, dense)
    hb.kv_dequantize(c.k_codes, c.k_scales, True, c.layout, 0, ref)
    torch.cuda.synchronize()
    assert torch.equal(dense, ref)


@pytest.mark.parametrize("qscale", [4.0e5, 1.0e-3])
def test_query_magnitudes_outside_the_fp16_range(qscale):
    """|q| * scale * log2(e) above 2^15 takes the kernel's rescaled-operand path (attention is one-hot there);
    tiny queries give near-uniform weights.  One-hot columns whose two best scores lie within 1% of each other
    are skipped: which of the two keys wins is decided by rounding."""
    B, Hq, Hkv, hist, S = 1, 8, 2, 100, 37
    qh, kh, vh = make(60, B, hist, Hq, Hkv)
    q, k, v = make(61, B, S, Hq, Hkv)
    q = bf16r(q * np.float32(qscale))
    c = DeviceCache(B, Hkv, hist + S, 128)
    c.write(torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16(), None, 0)
    got = gpu_prefill(c, q, k, v, hist)
    kc, vc, ks, vs = c.canonical(hist)
    kd = np.concatenate([oracle.dequant_int8(kc, ks), k], 1)
    want = oracle_prefill(q, oracle.dequant_int8(kc, ks), oracle.dequant_int8(vc, vs), k, v)
    assert np.isfinite(got).all()
    d = np.abs(got - want).max(-1)  # [B, S, Hq]
    checked = 0
    for si in range(S):
        for h in range(Hq):
            sc = kd[0, :hist + si + 1, h // (Hq // Hkv)].astype(np.float64) @ q[0, si, h].astype(np.float64)
            top = np.sort(sc)[-2:]
            if qscale > 1 and len(sc) > 1 and top[1] - top[0] < 1e-2 * abs(top[1]):
                continue
            checked += 1
            assert d[0, si, h] < TOL_MAX, (si, h, d[0, si, h])
    assert checked > 0.9 * S * Hq


@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (4, 2), (8, 2), (16, 2), (32, 8), (3, 1), (10, 2), (12, 2), (28, 4), (14, 2), (9, 1)])
def test_gqa_group_sizes(Hq, Hkv):
    hist, S = 40, 50
    qh, kh, vh = make(60, 1, hist, Hq, Hkv)
    q, k, v = make(61, 1, S, Hq, Hkv)
    c = DeviceCache(1, Hkv, hist + S, 128)
    c.write(torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16(), None, 0)
    got = gpu_prefill(c, q, k, v, hist, write=False)
    kc, vc, ks, vs = c.canonical(hist)
    compare(got, oracle_prefill(q, oracle.dequant_int8(kc, ks), oracle.dequant_int8(vc, vs), k, v),
            "gqa %d/%d" % (Hq, Hkv))
    assert not c.k_codes[:, :, hist:].any()  # quantize_on_write = 0 leaves the cache alone


def test_chunked_prefill_config3_reduced():
    """Config 3 at reduced size: 4 chunks of 128 tokens; chunk c attends the dequantized int8 cache of the
    earlier chunks plus its own bf16 K/V, and is itself quantized on write."""
    B, Hq, Hkv, C, n = 1, 8, 2, 128, 4
    q, k, v = make(70, B, C * n, Hq, Hkv)
    c = DeviceCache(B, Hkv, C * n, 128)
    for i in range(n):
        sl = slice(i * C, (i + 1) * C)
        got = gpu_prefill(c, q[:, sl], k[:, sl], v[:, sl], i * C)
        if i:
            kc, vc, ks, vs = c.canonical(i * C)
            want = oracle_prefill(q[:, sl], oracle.dequant_int8(kc, ks), oracle.dequant_int8(vc, vs), k[:, sl], v[:, sl])
        else:
            want = oracle_prefill(q[:, sl], None, None, k[:, sl], v[:, sl])
        compare(got, want, "chunk %d" % i)
    kc, vc, ks, vs = c.canonical(C * n)
    wk, wks = oracle.quant_int8(k)
    assert np.array_equal(kc, wk) and np.array_equal(ks, wks)


def test_two_token_cached_forward_equals_two_decode_steps():
    """The reference's equivalence test (llama.rs:3746-3785) across the two kernels: a 2-token cached forward
    vs two single-token decode steps.  The second token's view of the first differs (bf16 in the prefill call,
    int8 in the decode steps), so agreement is to the path's tolerance."""
    B, Hq, Hkv, hist = 2, 8, 2, 77
    qh, kh, vh = make(80, B, hist, Hq, Hkv)
    q, k, v = make(81, B, 2, Hq, Hkv)
    c1 = DeviceCache(B, Hkv, hist + 2, 128)
    c1.write(torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16(), None, 0)
    two = gpu_prefill(c1, q, k, v, hist)
    c2 = DeviceCache(B, Hkv, hist + 2, 128)
    c2.write(torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16(), None, 0)
    for t in range(2):
        kt = torch.from_numpy(k[:, t:t + 1]).to(DEV).bfloat16().contiguous()
        vt = torch.from_numpy(v[:, t:t + 1]).to(DEV).bfloat16().contiguous()
        c2.write(kt, vt, None, hist + t)
        step = run_decode(c2, wl.to_bf16_bits(q[:, t]), np.full(B, hist + t + 1, np.int32), Hq)
        d = np.abs(step - two[:, t])
        assert d.max() < TOL_MAX and d.mean() < TOL_MEAN
    assert torch.equal(c1.k_codes, c2.k_codes) and torch.equal(c1.v_scales, c2.v_scales)


def test_overflow_is_an_error():
    q, k, v = make(90, 1, 8, 8, 2)
    c = DeviceCache(1, 2, 10, 128)
    with pytest.raises(hb.HsError) as e:
        gpu_prefill(c, q, k, v, 4)
    assert e.value.code == hb.HS_ERR_OVERFLOW


def test_paged_history_matches_contiguous():
    """History in 64-token blocks scattered through one pool (K and V blocks interleaved): prefill over it,
    its quantize-on-write into the pool, and the dense view must equal the contiguous-cache results."""
    B, Hq, Hkv, D, hist, S, BT = 2, 8, 2, 128, 150, 70, 64
    qh, kh, vh = make(100, B, hist, Hq, Hkv)
    q, k, v = make(101, B, S, Hq, Hkv)
    c = DeviceCache(B, Hkv, hist + S, D)
    hk, hv = torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16()
    c.write(hk, hv, None, 0)
    want = gpu_prefill(c, q, k, v, hist)
    nblk = (hist + S + BT - 1) // BT
    ids = wl.philox(102).permutation(2 * B * nblk + 3).astype(np.int32)
    kt, vt = ids[:B * nblk].reshape(B, nblk), ids[B * nblk:2 * B * nblk].reshape(B, nblk)
    pool_c = torch.zeros(len(ids), Hkv, BT, D, dtype=torch.int8, device=DEV)
    pool_s = torch.zeros(len(ids), Hkv, BT, dtype=torch.float32, device=DEV)
    k_tab, v_tab = torch.from_numpy(kt).to(DEV), torch.from_numpy(vt).to(DEV)
    lay = hb.paged_layout(Hkv, BT, D, k_tab, v_tab)
    hb.kv_quantize_int8(hk, hv, pool_c, pool_c, pool_s, pool_s, lay, None, 0)
    qt, knew, vnew = (torch.from_numpy(x).to(DEV).bfloat16().contiguous() for x in (q, k, v))
    out = torch.empty(B, S, Hq, D, dtype=torch.bfloat16, device=DEV)
    hb.prefill_attn(qt, knew, vnew, pool_c, pool_c, pool_s, pool_s, lay, hist, out, 1.0 / np.sqrt(D), True)
    dense_k = torch.empty(B, hist + S, Hkv, D, dtype=torch.float32, device=DEV)
    dense_v = torch.empty_like(dense_k)
    hb.kv_dequantize(pool_c, pool_s, False, lay, 0, dense_k)
    hb.kv_dequantize(pool_c, pool_s, False, lay, 1, dense_v)
    torch.cuda.synchronize()
    assert np.array_equal(out.float().cpu().numpy(), want)
    ck, cv = torch.empty_like(dense_k), torch.empty_like(dense_v)
    hb.kv_dequantize(c.k_codes, c.k_scales, False, c.layout, 0, ck)
    hb.kv_dequantize(c.v_codes, c.v_scales, False, c.layout, 1, cv)
    torch.cuda.synchronize()
    assert torch.equal(dense_k, ck) and torch.equal(dense_v, cv)


@pytest.mark.parametrize("seed", range(8))
def test_random_shapes(seed):
    """Seeded random batch sizes, head groupings, history and prompt lengths and history formats against the oracle."""
    r = np.random.default_rng(2000 + seed)
    B = int(r.integers(1, 4))
    Hkv = int(r.choice([1, 2, 4]))
    G = int(r.choice([1, 2, 3, 4, 6, 7, 8]))
    hist = int(r.choice([0, 1, 63, 64, 65, 200, 333]))
    S = int(r.integers(1, 300))
    fp8 = bool(r.integers(0, 2)) and hist > 0
    sigma = 0.5 if fp8 else 1.0
    Hq = Hkv * G
    pad = int(r.integers(0, 50))
    D = int(r.choice([64, 128]))
    q, k, v = make(300 + seed, B, S, Hq, Hkv, D=D, sigma=sigma)
    c = DeviceCache(B, Hkv, hist + S + pad, D, fp8=fp8)
    kd = vd = None
    if hist > 0:
        _, kh, vh = make(400 + seed, B, hist, Hq, Hkv, D=D, sigma=sigma)
        hk, hv = torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16()
        if fp8:
            hb.kv_fp8_calibrate(hk, hv, c.k_scales, c.v_scales)
        c.write(hk, hv, None, 0)
        kc, vc, ks, vs = c.canonical(hist)
        deq = oracle.dequant_fp8 if fp8 else oracle.dequant_int8
        kd, vd = deq(kc, ks), deq(vc, vs)
    got = gpu_prefill(c, q, k, v, hist)
    compare(got, oracle_prefill(q, kd, vd, k, v), "random B=%d Hkv=%d G=%d D=%d hist=%d S=%d fp8=%s" % (B, Hkv, G, D, hist, S, fp8))


# ------------------------------------------------------------------ head_dim 256 (128 query columns per workgroup)
@pytest.mark.parametrize("hist,S,fp8", [(0, 1, False), (0, 33, False), (0, 257, False), (19, 5, False), (64, 64, False),
                                        (200, 130, False), (333, 200, True), (65, 31, True)])
@pytest.mark.parametrize("D", [256, 64])
def test_head_dim_256_and_64(hist, S, fp8, D):
    """head_dim 256 is an instance of its own; head_dim 64 runs in the 128 layout with zero padding of Q."""
    B, Hq, Hkv = 2, 8, 2
    sigma = 0.5 if fp8 else 1.0
    q, k, v = make(500 + hist + S, B, S, Hq, Hkv, D=D, sigma=sigma)
    c = DeviceCache(B, Hkv, hist + S, D, fp8=fp8)
    kd = vd = None
    if hist > 0:
        _, kh, vh = make(600 + hist, B, hist, Hq, Hkv, D=D, sigma=sigma)
        hk, hv = torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16()
        if fp8:
            hb.kv_fp8_calibrate(hk, hv, c.k_scales, c.v_scales)
        c.write(hk, hv, None, 0)
        kc, vc, ks, vs = c.canonical(hist)
        deq = oracle.dequant_fp8 if fp8 else oracle.dequant_int8
        kd, vd = deq(kc, ks), deq(vc, vs)
    got = gpu_prefill(c, q, k, v, hist)
    compare(got, oracle_prefill(q, kd, vd, k, v), "d%d hist=%d S=%d fp8=%s" % (D, hist, S, fp8))
    if not fp8:  # the new rows were cached behind the history with the oracle's codes
        kc, vc, ks, vs = c.canonical(hist + S)
        wk, wks = oracle.quant_int8(k)
        assert np.array_equal(kc[:, hist:], wk) and np.array_equal(ks[:, hist:], wks)


@pytest.mark.parametrize("D", [256, 64])
@pytest.mark.parametrize("Hq,Hkv", [(2, 2), (4, 2), (16, 4), (16, 2), (6, 2), (7, 1)])
def test_head_dim_256_and_64_group_sizes(Hq, Hkv, D):
    B, S, hist = 1, 70, 100
    q, k, v = make(700 + Hq, B, S, Hq, Hkv, D=D)
    _, kh, vh = make(701 + Hq, B, hist, Hq, Hkv, D=D)
    c = DeviceCache(B, Hkv, hist + S, D)
    c.write(torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16(), None, 0)
    kc, vc, ks, vs = c.canonical(hist)
    got = gpu_prefill(c, q, k, v, hist)
    compare(got, oracle_prefill(q, oracle.dequant_int8(kc, ks), oracle.dequant_int8(vc, vs), k, v), "d%d gqa %d/%d" % (D, Hq, Hkv))


@pytest.mark.parametrize("D,fp8", [(128, False), (128, True), (64, False), (256, False)])
def test_ragged_history_lengths(D, fp8):
    """Rows at different positions (the reference's forward_batched with q_len > 1): every row attends its own
    history length and its new tokens, and caches them behind its own history."""
    hists, S, Hq, Hkv = [0, 70, 333, 64], 90, 8, 2
    B, Hmax = len(hists), max(hists)
    sigma = 0.5 if fp8 else 1.0
    q, k, v = make(900 + D, B, S, Hq, Hkv, D=D, sigma=sigma)
    _, kh, vh = make(901 + D, B, Hmax, Hq, Hkv, D=D, sigma=sigma)
    c = DeviceCache(B, Hkv, Hmax + S + 5, D, fp8=fp8)
    hk, hv = torch.from_numpy(kh).to(DEV).bfloat16(), torch.from_numpy(vh).to(DEV).bfloat16()
    if fp8:
        hb.kv_fp8_calibrate(hk, hv, c.k_scales, c.v_scales)
    c.write(hk, hv, None, 0)  # every row gets Hmax tokens; a row's own history is the first hists[b] of them
    kc, vc, ks, vs = c.canonical(Hmax)
    deq = oracle.dequant_fp8 if fp8 else oracle.dequant_int8
    kd, vd = deq(kc, ks), deq(vc, vs)
    qt, kt, vt = (torch.from_numpy(x).to(DEV).bfloat16().contiguous() for x in (q, k, v))
    out = torch.full((B, S, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    hb.prefill_attn(qt, kt, vt, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, Hmax, out, 1.0 / np.sqrt(D),
                    True, fp8=fp8, hist_lens=torch.tensor(hists, dtype=torch.int32, device=DEV))
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    kc2, vc2, ks2, vs2 = c.canonical(Hmax + S)
    for b, h in enumerate(hists):
        want = oracle_prefill(q[b:b + 1], kd[b:b + 1, :h] if h else None, vd[b:b + 1, :h] if h else None, k[b:b + 1], v[b:b + 1])
        compare(got[b:b + 1], want, "ragged D=%d fp8=%s row %d hist=%d" % (D, fp8, b, h))
        if not fp8:  # the row's new tokens sit behind its own history with the oracle's codes
            wk, wks = oracle.quant_int8(k[b:b + 1])
            wv, wvs = oracle.quant_int8(v[b:b + 1])
            assert np.array_equal(kc2[b, h:h + S], wk[0]) and np.array_equal(ks2[b, h:h + S], wks[0])
            assert np.array_equal(vc2[b, h:h + S], wv[0]) and np.array_equal(vs2[b, h:h + S], wvs[0])
            assert np.array_equal(kc2[b, :h], kc[b, :h])  # and the history below is untouched


# ---------------------------------------------------------------- sliding window (local layers)
def gpu_prefill_window(cache, q, k, v, hist, window, hist_lens=None, write=True):
    B, S, Hq, D = q.shape
    qt, kt, vt = (torch.from_numpy(x).to(DEV).bfloat16().contiguous() for x in (q, k, v))
    out = torch.full((B, S, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    hl = None if hist_lens is None else torch.from_numpy(np.asarray(hist_lens, np.int32)).to(DEV)
    hb.prefill_attn(qt, kt, vt, cache.k_codes, cache.v_codes, cache.k_scales, cache.v_scales, cache.layout, hist, out,
                    1.0 / np.sqrt(D), write, fp8=cache.fp8, hist_lens=hl, window=window)
    cache.layout.prefill_window = 0
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


def test_windowed_prompt_matches_the_reference_golden():
    """The libtorch op sequence of apply_sliding_window_mask on prompts over an empty cache (llama.rs:1086-1091,
    1123-1155), fp32 inputs rounded to bf16 for the kernel: same tolerance as every prefill test."""
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "attention_window.npz"))
    for tag in "abde":  # head_dim 64 and 128
        q, k, v, W = bf16r(g[tag + "_q"]), bf16r(g[tag + "_k"]), bf16r(g[tag + "_v"]), int(g[tag + "_window"])
        B, S, Hq, D = q.shape
        c = DeviceCache(B, k.shape[2], S, D)
        got = gpu_prefill_window(c, q, k, v, 0, W)
        want = oracle.prefill_attn(q, k, v, None, None, oracle.FMT_DENSE, np.full(B, S, np.int32), 1.0 / np.sqrt(D), window=W)
        compare(got, want, "window golden " + tag)
        assert np.abs(got - g[tag + "_out"]).max() < 3e-2  # the golden output comes from unrounded fp32 inputs


@pytest.mark.parametrize("D,Hq,Hkv", [(128, 32, 8), (64, 8, 4), (256, 8, 2), (128, 7, 1)])
@pytest.mark.parametrize("W", [1, 17, 64, 100, 300, 4096])
def test_windowed_prompt_without_history(D, Hq, Hkv, W):
    B, S = 2, 333
    q, k, v = make(900 + D + W, B, S, Hq, Hkv, D)
    c = DeviceCache(B, Hkv, S, D)
    got = gpu_prefill_window(c, q, k, v, 0, W)
    want = oracle.prefill_attn(q, k, v, None, None, oracle.FMT_DENSE, np.full(B, S, np.int32), 1.0 / np.sqrt(D), window=W)
    compare(got, want, "window %d D=%d" % (W, D))
    if W >= S:  # a window that covers the prompt changes nothing
        plain = gpu_prefill(DeviceCache(B, Hkv, S, D), q, k, v, 0)
        if (D == 128 and hb.PREFILL_COLUMNS == 32) or hb.PREFILL_KEY_SPLITS > 1:  # the unwindowed launch is another kernel
            # the unwindowed call runs on the 32x32 MFMA instance here, the windowed one never does: the same values
            # summed in another order, then rounded to bf16
            assert np.abs(got - plain).max() <= 2.0 ** -7 * max(1.0, np.abs(plain).max())
        else:
            assert np.array_equal(got, plain)
    kc, vc, ks, vs = c.canonical(S)  # the cache write does not depend on the window
    wk, wks = oracle.quant_int8(k)
    assert np.array_equal(kc, wk) and np.array_equal(ks, wks)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("H,S,W", [(700, 130, 64), (700, 130, 200), (700, 130, 701), (1000, 64, 1), (129, 200, 150),
                                   (2000, 512, 1024), (640, 512, 100)])
def test_windowed_chunk_over_a_history(fp8, H, S, W):
    """With cached tokens the window runs over absolute positions: query p attends keys in (p - W, p], of which some,
    all or none are history.  Steps wholly before a workgroup's window are never loaded."""
    B, Hq, Hkv, D = 2, 16, 4, 128
    r = wl.philox(7000 + H + S + W)
    kh = bf16r(r.standard_normal((B, H, Hkv, D)).astype(np.float32))
    vh = bf16r(r.standard_normal((B, H, Hkv, D)).astype(np.float32))
    q, k, v = make(7100 + H + W, B, S, Hq, Hkv, D)
    c = DeviceCache(B, Hkv, H + S, D, fp8=fp8)
    kt, vt = torch.from_numpy(kh).to(DEV), torch.from_numpy(vh).to(DEV)
    if fp8:
        hb.kv_fp8_calibrate(kt, vt, c.k_scales, c.v_scales)
    c.write(kt, vt, None, 0)
    kc, vc, ks, vs = c.canonical(H)
    deq = oracle.dequant_fp8 if fp8 else oracle.dequant_int8
    kd, vd = deq(kc, ks), deq(vc, vs)
    got = gpu_prefill_window(c, q, k, v, H, W)
    want = oracle.prefill_attn(q, np.concatenate([kd, k], 1), np.concatenate([vd, v], 1), None, None, oracle.FMT_DENSE,
                               np.full(B, H + S, np.int32), 1.0 / np.sqrt(D), window=W)
    compare(got, want, "window %d over H=%d S=%d fp8=%s" % (W, H, S, fp8))


def test_windowed_ragged_rows():
    """Rows at different positions (hist_lens): each row's window is cut at its own history length."""
    B, S, Hq, Hkv, D, W = 3, 96, 8, 2, 128, 80
    hist = [300, 0, 77]
    Hmax = max(hist)
    r = wl.philox(7300)
    kh = bf16r(r.standard_normal((B, Hmax, Hkv, D)).astype(np.float32))
    vh = bf16r(r.standard_normal((B, Hmax, Hkv, D)).astype(np.float32))
    q, k, v = make(7301, B, S, Hq, Hkv, D)
    c = DeviceCache(B, Hkv, Hmax + S, D)
    c.write(torch.from_numpy(kh).to(DEV), torch.from_numpy(vh).to(DEV), None, 0)
    kc, vc, ks, vs = c.canonical(Hmax)
    kd, vd = oracle.dequant_int8(kc, ks), oracle.dequant_int8(vc, vs)
    got = gpu_prefill_window(c, q, k, v, Hmax, W, hist_lens=hist, write=False)
    for b in range(B):
        h = hist[b]
        want = oracle.prefill_attn(q[b:b + 1], np.concatenate([kd[b:b + 1, :h], k[b:b + 1]], 1),
                                   np.concatenate([vd[b:b + 1, :h], v[b:b + 1]], 1), None, None, oracle.FMT_DENSE,
                                   np.array([h + S], np.int32), 1.0 / np.sqrt(D), window=W)
        compare(got[b:b + 1], want, "ragged window row %d" % b)


def test_negative_window_is_refused():
    c = DeviceCache(1, 2, 16, 128)
    q, k, v = make(7400, 1, 4, 4, 2)
    with pytest.raises(hb.HsError):
        gpu_prefill_window(c, q, k, v, 0, -1)
    c.layout.prefill_window = 0


@pytest.mark.parametrize("D,fp8", [(128, False), (128, True), (64, False), (256, False)])
def test_key_split_the_library_picks_for_a_chunk_of_one_sequence(D, fp8):
    """One sequence, a 512-token chunk over 1536 cached tokens (llama.rs:492-668 runs prompts one sequence at a time): 64
    full-width query tiles on 256 compute units, so with a workspace the library cuts every tile's 24 + up to 8 steps
    into runs.  Outputs agree with the unsplit launch within the rounding of another summation order and with the
    oracle; the cache rows are the same bits; the workspace is left ready for the next call (second call, same
    answer)."""
    _fixes_its_own_instance()
    B, S, H, Hq, Hkv = 1, 512, 1536, (32 if D != 256 else 16), (8 if D != 256 else 4)
    r = wl.philox(7300 + D + fp8)
    sigma = 0.5 if fp8 else 1.0
    q, k, v = make(7400 + D, B, S, Hq, Hkv, D, sigma)
    hk = bf16r((sigma * r.standard_normal((B, H, Hkv, D))).astype(np.float32))
    hv = bf16r((sigma * r.standard_normal((B, H, Hkv, D))).astype(np.float32))
    dev = lambda x: torch.from_numpy(x).to(DEV).bfloat16().contiguous()
    ws = hb.prefill_split_workspace(B, S, Hq, Hkv, D)
    caches, outs = [], []
    for use_ws in (None, ws, ws):
        c = DeviceCache(B, Hkv, H + S, D, fp8=fp8)
        if fp8:
            hb.kv_fp8_calibrate(dev(hk), dev(hv), c.k_scales, c.v_scales)
        c.write(dev(hk), dev(hv))
        out = torch.full((B, S, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        hb.prefill_attn(dev(q), dev(k), dev(v), c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, H, out,
                        1.0 / np.sqrt(D), True, fp8=fp8, columns=0, split_workspace=use_ws, key_splits=0 if use_ws is not None else 1)
        torch.cuda.synchronize()
        caches.append(c)
        outs.append(out.float().cpu().numpy())
    assert np.isfinite(outs[1]).all()
    assert np.abs(outs[1] - outs[0]).max() <= 2.0 ** -7 * max(1.0, np.abs(outs[0]).max())
    assert np.array_equal(outs[1], outs[2])
    for c in caches[1:]:
        assert torch.equal(c.k_codes, caches[0].k_codes) and torch.equal(c.v_codes, caches[0].v_codes)
        assert torch.equal(c.k_scales, caches[0].k_scales) and torch.equal(c.v_scales, caches[0].v_scales)
    if not fp8:
        kc, vc, ks, vs = caches[0].canonical(H)
        want = oracle_prefill(q, oracle.dequant_int8(kc, ks), oracle.dequant_int8(vc, vs), k, v)
        compare(outs[1], want, "key split D=%d" % D)


def test_key_split_workspace_errors():
    _fixes_its_own_instance()
    B, S, Hq, Hkv, D = 1, 128, 8, 2, 128
    q, k, v = (torch.zeros(B, S, H, D, dtype=torch.bfloat16, device=DEV) for H in (Hq, Hkv, Hkv))
    c = DeviceCache(B, Hkv, S, D)
    out = torch.empty_like(q)
    small = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    with pytest.raises(hb.HsError) as e:
        hb.prefill_attn(q, k, v, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, 0, out, 0.1, False,
                        columns=0, split_workspace=small, key_splits=4)
    assert e.value.code == hb.HS_ERR_WORKSPACE
    ws = hb.prefill_split_workspace(B, S, Hq, Hkv, D)
    with pytest.raises(hb.HsError) as e:
        hb.prefill_attn(q, k, v, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, 0, out, 0.1, False,
                        columns=0, split_workspace=ws, key_splits=9)
    assert e.value.code == 1


def test_one_split_workspace_for_calls_of_every_width_and_size():
    """Calls that split at full width, at half width (twice the tiles), with other run counts and for other lengths take
    turns on ONE workspace: the arrival counters have a fixed place in it, so the partial results of one call never
    land where a later call, with more tiles, looks for a counter (they did once, when the counter region was sized by
    the call: all rows of the later call's second sequence stayed unwritten).  Over a history, so that every run of
    every tile, the first included, holds numbers."""
    _fixes_its_own_instance()
    B, H, S, Hq, Hkv, D = 2, 256, 844, 32, 8, 128
    q, k, v = make(77, B, H + S, Hq, Hkv)
    ws = hb.prefill_split_workspace(B, S, Hq, Hkv, D)
    dev = lambda x: torch.from_numpy(x).to(DEV).bfloat16().contiguous()
    qd, kd, vd = dev(q), dev(k), dev(v)

    def run(n, cols, runs):
        c = DeviceCache(B, Hkv, H + S, D)
        o0 = torch.empty(B, H, Hq, D, dtype=torch.bfloat16, device=DEV)
        hb.prefill_attn(qd[:, :H].contiguous(), kd[:, :H].contiguous(), vd[:, :H].contiguous(), c.k_codes, c.v_codes, c.k_scales,
                        c.v_scales, c.layout, 0, o0, 1.0 / np.sqrt(D), True, columns=256, key_splits=1)
        out = torch.full((B, n, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        hb.prefill_attn(qd[:, H:H + n].contiguous(), kd[:, H:H + n].contiguous(), vd[:, H:H + n].contiguous(), c.k_codes, c.v_codes,
                        c.k_scales, c.v_scales, c.layout, H, out, 1.0 / np.sqrt(D), True, columns=cols, split_workspace=ws,
                        key_splits=runs)
        torch.cuda.synchronize()
        return out.float().cpu().numpy()

    want = run(S, 256, 1)
    assert np.isfinite(want).all()
    for n, cols, runs in ((S, 256, 2), (S, 128, 3), (300, 256, 8), (S, 128, 4), (S, 256, 3), (700, 128, 2), (S, 128, 2)):
        got = run(n, cols, runs)
        assert np.isfinite(got).all(), (n, cols, runs)
        d = np.abs(got - want[:, :n])
        assert d.max() < 2e-2 and d.mean() < 2e-3, (n, cols, runs, d.max())


def test_key_split_refuses_more_tiles_than_it_has_counters_for():
    _fixes_its_own_instance()
    B, S, Hq, Hkv, D = 8, 2048, 32, 8, 128  # 64 x 8 x 8 = 4096 tiles of half width... and twice that below
    q, k, v = (torch.zeros(B, 2 * S, H, D, dtype=torch.bfloat16, device=DEV) for H in (Hq, Hkv, Hkv))
    c = DeviceCache(B, Hkv, 2 * S, D)
    out = torch.empty_like(q)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)
    with pytest.raises(hb.HsError) as e:
        hb.prefill_attn(q, k, v, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, 0, out, 0.1, False,
                        columns=128, split_workspace=ws, key_splits=2)
    assert e.value.code == 1 and "4096" in str(e.value)


@pytest.mark.parametrize("variant", ["full", "half", "split3", "split2-half"])
@pytest.mark.parametrize("chunks", [(64, 64, 64), (100, 37, 200, 91), (512, 512), (1, 63, 64, 300)])
@pytest.mark.parametrize("Hq,Hkv", [(8, 2), (6, 2), (4, 4)])
def test_history_from_the_bf16_shadow(chunks, Hq, Hkv, variant):
    """hs_kv_layout.prefill_shadow: every call appends its dequantized rows to a bf16 operand-order copy and calls with
    history read that copy instead of the codes.  A prompt in uneven chunks (history lengths that are not multiples of
    the 64-key step, a partial last step whose remaining rows the same launch is writing) against the same calls
    without the copy and against the oracle; the int8 cache is the same bits either way.  At full and at half width,
    and with every tile's steps split into runs (a run may hold history steps only, new-token steps only, or both)."""
    _fixes_its_own_instance()
    B, D = 2, 128
    cols = 128 if variant.endswith("half") else 256
    runs = int(variant[5]) if variant.startswith("split") else 1
    T = sum(chunks)
    q, k, v = make(8100 + T + Hq, B, T, Hq, Hkv, D)
    dev = lambda x: torch.from_numpy(x).to(DEV).bfloat16().contiguous()
    shadow = hb.prefill_shadow(B, Hkv, D, T)
    with_copy, without = DeviceCache(B, Hkv, T, D), DeviceCache(B, Hkv, T, D)
    lo = 0
    for n in chunks:
        hi = lo + n
        outs = []
        for c, sh in ((without, None), (with_copy, shadow)):
            out = torch.full((B, n, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
            ws = hb.prefill_split_workspace(B, n, Hq, Hkv, D) if runs > 1 else None
            hb.prefill_attn(dev(q[:, lo:hi]), dev(k[:, lo:hi]), dev(v[:, lo:hi]), c.k_codes, c.v_codes, c.k_scales, c.v_scales,
                            c.layout, lo, out, 1.0 / np.sqrt(D), True, columns=cols, key_splits=runs, split_workspace=ws, shadow=sh)
            torch.cuda.synchronize()
            outs.append(out.float().cpu().numpy())
        assert np.isfinite(outs[1]).all(), (lo, hi)
        # the copy holds bf16(code * scale) where the other path uses fp16(code * scale): both within the oracle's bar
        assert np.abs(outs[1] - outs[0]).max() <= 2.0 ** -6 * max(1.0, np.abs(outs[0]).max()), (lo, hi)
        if lo > 0:
            kc, vc, ks, vs = without.canonical(lo)
            want = oracle_prefill(q[:, lo:hi], oracle.dequant_int8(kc, ks), oracle.dequant_int8(vc, vs), k[:, lo:hi], v[:, lo:hi])
            compare(outs[1], want, "shadow history %d..%d" % (lo, hi))
        lo = hi
    assert torch.equal(with_copy.k_codes, without.k_codes) and torch.equal(with_copy.v_codes, without.v_codes)
    assert torch.equal(with_copy.k_scales, without.k_scales) and torch.equal(with_copy.v_scales, without.v_scales)


def test_shadow_contract_errors():
    _fixes_its_own_instance()
    B, S, Hq, Hkv, D = 1, 64, 4, 1, 128
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
    c = DeviceCache(B, Hkv, 256, D)
    q, k, o = z(B, S, Hq, D), z(B, S, Hkv, D), z(B, S, Hq, D)
    run = lambda sh, hist=0, write=True: hb.prefill_attn(q, k, k, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, hist, o,
                                                          0.1, write, columns=0, key_splits=1, shadow=sh)
    buf, tokens = hb.prefill_shadow(B, Hkv, D, 128)
    run((buf, tokens))                                   # fits
    with pytest.raises(hb.HsError) as e:                 # 128 + 64 tokens do not
        run((buf, tokens), hist=128)
    assert e.value.code == 1 and "prefill_shadow_tokens" in str(e.value)
    with pytest.raises(hb.HsError) as e:                 # a buffer shorter than its token count says
        run((buf[: buf.numel() // 2], tokens), hist=64)
    assert e.value.code == hb.HS_ERR_WORKSPACE
    with pytest.raises(hb.HsError) as e:                 # history but no cache write: would leave a hole
        run((buf, tokens), hist=64, write=False)
    assert e.value.code == 1 and "quantize_on_write" in str(e.value)
    assert hb.lib().hs_prefill_shadow_bytes(1, 1, 256, 128) == 0


def test_shadow_over_a_paged_pool_and_random_chunkings():
    """The copy is indexed by the call's sequences, not by the cache's storage: the same prompt prefilled into a paged pool
    (64-token blocks scattered, K and V interleaved) with the copy gives the outputs of the contiguous cache with the
    copy, bit for bit, and the same pool contents as without it; chunk boundaries drawn at random."""
    _fixes_its_own_instance()
    B, Hq, Hkv, D, BT = 2, 8, 2, 128, 64
    r = wl.philox(8300)
    for trial in range(3):
        cuts = sorted(set(int(x) for x in r.integers(1, 700, size=4)))
        T = cuts[-1]
        q, k, v = make(8310 + trial, B, T, Hq, Hkv, D)
        dev = lambda x: torch.from_numpy(x).to(DEV).bfloat16().contiguous()
        nblk = (T + BT - 1) // BT
        ids = r.permutation(2 * B * nblk + 3).astype(np.int32)
        k_tab = torch.from_numpy(ids[:B * nblk].reshape(B, nblk)).to(DEV)
        v_tab = torch.from_numpy(ids[B * nblk:2 * B * nblk].reshape(B, nblk)).to(DEV)
        pools = []
        outs = {}
        for name in ("contiguous+copy", "paged+copy", "paged"):
            if name.startswith("paged"):
                codes = torch.zeros(len(ids), Hkv, BT, D, dtype=torch.int8, device=DEV)
                scales = torch.zeros(len(ids), Hkv, BT, dtype=torch.float32, device=DEV)
                bufs, lay = (codes, codes, scales, scales), hb.paged_layout(Hkv, BT, D, k_tab, v_tab)
                pools.append((codes, scales))
            else:
                c = DeviceCache(B, Hkv, T, D)
                bufs, lay = (c.k_codes, c.v_codes, c.k_scales, c.v_scales), c.layout
            sh = hb.prefill_shadow(B, Hkv, D, T) if name.endswith("copy") else None
            got, lo = [], 0
            for hi in cuts:
                out = torch.full((B, hi - lo, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
                hb.prefill_attn(dev(q[:, lo:hi]), dev(k[:, lo:hi]), dev(v[:, lo:hi]), *bufs, lay, lo, out, 1.0 / np.sqrt(D), True,
                                columns=256, key_splits=1, shadow=sh)
                got.append(out)
                lo = hi
            torch.cuda.synchronize()
            outs[name] = torch.cat(got, 1)
        assert not torch.isnan(outs["paged+copy"].float()).any()
        assert torch.equal(outs["paged+copy"].view(torch.int16), outs["contiguous+copy"].view(torch.int16)), cuts
        assert torch.equal(pools[0][0], pools[1][0]) and torch.equal(pools[0][1], pools[1][1])
        d = (outs["paged+copy"].float() - outs["paged"].float()).abs().max().item()
        assert d <= 2.0 ** -6 * max(1.0, outs["paged"].float().abs().max().item()), (cuts, d)


@pytest.mark.parametrize("variant", ["full", "split2-half"])
def test_bf16_shadow_over_an_fp8_cache(variant):
    """The copy holds the dequantized e4m3fn codes (code value x head scale, rounded to bf16): a prompt in uneven chunks
    over an FP8 cache with and without the copy -- outputs within the operand rounding of each other and inside the
    oracle's bar, the cache the same bits."""
    _fixes_its_own_instance()
    B, Hq, Hkv, D = 2, 8, 2, 128
    chunks = (150, 70, 200, 64)
    T = sum(chunks)
    q, k, v = make(8500, B, T, Hq, Hkv, D, 0.5)
    dev = lambda x: torch.from_numpy(x).to(DEV).bfloat16().contiguous()
    cols = 128 if variant.endswith("half") else 256
    runs = int(variant[5]) if variant.startswith("split") else 1
    shadow = hb.prefill_shadow(B, Hkv, D, T)
    with_copy, without = DeviceCache(B, Hkv, T, D, fp8=True), DeviceCache(B, Hkv, T, D, fp8=True)
    for c in (with_copy, without):
        hb.kv_fp8_calibrate(dev(k[:, :chunks[0]]), dev(v[:, :chunks[0]]), c.k_scales, c.v_scales)
    lo = 0
    for n in chunks:
        hi = lo + n
        outs = []
        for c, sh in ((without, None), (with_copy, shadow)):
            out = torch.full((B, n, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
            ws = hb.prefill_split_workspace(B, n, Hq, Hkv, D) if runs > 1 else None
            hb.prefill_attn(dev(q[:, lo:hi]), dev(k[:, lo:hi]), dev(v[:, lo:hi]), c.k_codes, c.v_codes, c.k_scales, c.v_scales,
                            c.layout, lo, out, 1.0 / np.sqrt(D), True, fp8=True, columns=cols, key_splits=runs,
                            split_workspace=ws, shadow=sh)
            torch.cuda.synchronize()
            outs.append(out.float().cpu().numpy())
        assert np.isfinite(outs[1]).all(), (lo, hi)
        assert np.abs(outs[1] - outs[0]).max() <= 2.0 ** -6 * max(1.0, np.abs(outs[0]).max()), (lo, hi)
        if lo > 0:
            kc, vc, ks, vs = without.canonical(lo)
            want = oracle_prefill(q[:, lo:hi], oracle.dequant_fp8(kc, ks), oracle.dequant_fp8(vc, vs), k[:, lo:hi], v[:, lo:hi])
            compare(outs[1], want, "fp8 shadow history %d..%d" % (lo, hi))
        lo = hi
    assert torch.equal(with_copy.k_codes, without.k_codes) and torch.equal(with_copy.v_codes, without.v_codes)


@pytest.mark.parametrize("kmag,vmag", [(1e-5, 1e5), (1e5, 1e-5), (3e-7, 3e-7), (1.0, 1e9)])
def test_shadow_history_magnitude_ranges(kmag, vmag):
    """test_history_magnitude_ranges with the history read from the bf16 copy: bf16 has fp32's exponent range, so caches
    that are tiny or huge as a whole need no reference scale there -- and a row far above its head's other rows, which
    saturates the fp16 operands of the code path, does not saturate here."""
    _fixes_its_own_instance()
    B, Hq, Hkv, hist, S, D = 2, 8, 2, 150, 70, 128
    qh, kh, vh = make(90, B, hist, Hq, Hkv)
    q, k, v = make(91, B, S, Hq, Hkv)
    mags = np.array([[kmag, vmag], [vmag, kmag]], np.float32)
    kh, vh = bf16r(kh * mags[:, 0, None, None, None]), bf16r(vh * mags[:, 1, None, None, None])
    vh[0, 100] *= 2.0 ** 13  # one cached row 2^13 above its head's first tokens: beyond the fp16 window of the code path
    vh = bf16r(vh)
    k, v = bf16r(k * mags[:, 0, None, None, None]), bf16r(v * mags[:, 1, None, None, None])
    q = bf16r(q / np.maximum(mags[:, 0, None, None, None], 1e-3))
    dev = lambda x: torch.from_numpy(x).to(DEV).bfloat16().contiguous()
    c = DeviceCache(B, Hkv, hist + S, D)
    shadow = hb.prefill_shadow(B, Hkv, D, hist + S)
    o0 = torch.empty(B, hist, Hq, D, dtype=torch.bfloat16, device=DEV)
    hb.prefill_attn(dev(qh), dev(kh), dev(vh), c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, 0, o0, 1.0 / np.sqrt(D), True,
                    columns=256, key_splits=1, shadow=shadow)
    out = torch.full((B, S, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    hb.prefill_attn(dev(q), dev(k), dev(v), c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, hist, out, 1.0 / np.sqrt(D), True,
                    columns=256, key_splits=1, shadow=shadow)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    kc, vc, ks, vs = c.canonical(hist)
    want = oracle_prefill(q, bf16r(oracle.dequant_int8(kc, ks)), bf16r(oracle.dequant_int8(vc, vs)), k, v)  # the copy's values
    assert np.isfinite(got).all()
    for b in range(B):
        top = np.abs(want[b]).max()
        d = np.abs(got[b] - want[b])
        assert d.max() < 2e-2 * top and d.mean() < 2e-3 * top, (b, d.max() / top, d.mean() / top)
