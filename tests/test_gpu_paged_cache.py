"""GPU tests of the paged mode through libhs_kv_cache.so: the reference's paged-cache tests
(kv_cache.rs:2466-2508 update/get/clear, :2623-2645 blocks returned on drop) on the int8 block format, plus the
ragged-batch decode step against the oracle."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import kv_cache as kc
from hyprstream_amd import workloads as wl
from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _rand(r, *shape):
    return torch.from_numpy(r.standard_normal(shape).astype(np.float32)).to(torch.bfloat16).to(DEV)


def _dense_reference(k_src):
    """what get() must return: dequant(quant(k)) rounded to bf16, via the oracle"""
    x = k_src.float().cpu().numpy()
    codes, scales = oracle.quant_int8(x)
    return oracle.dequant_int8(codes, scales)


def test_paged_kv_cache_update_and_get():
    r = wl.philox(900)
    Hkv, D = 2, 64
    pool = kc.BlockPool(8, Hkv, D)
    cache = kc.PagedLayerKVCache(1024, pool, 1)
    k, v = _rand(r, 1, 10, Hkv, D), _rand(r, 1, 10, Hkv, D)
    cache.update(k, v, 0)
    assert cache.seq_pos == 10 and pool.used_blocks() == 2
    gk, gv = cache.get(torch.float32)
    assert gk.shape == (1, 10, Hkv, D)
    assert np.array_equal(gk.cpu().numpy(), _dense_reference(k)) and np.array_equal(gv.cpu().numpy(), _dense_reference(v))
    k2, v2 = _rand(r, 1, 5, Hkv, D), _rand(r, 1, 5, Hkv, D)
    cache.update(k2, v2, 10)
    assert cache.seq_pos == 15
    gk, _ = cache.get(torch.float32)
    assert gk.shape[1] == 15 and np.array_equal(gk[:, 10:].cpu().numpy(), _dense_reference(k2))
    used = pool.used_blocks()
    cache.clear()
    assert pool.used_blocks() == used - 2 and cache.seq_pos == 0


def test_update_across_block_boundaries_and_truncate():
    r = wl.philox(901)
    Hkv, D = 2, 64
    pool = kc.BlockPool(16, Hkv, D)
    cache = kc.PagedLayerKVCache(2048, pool, "sess")
    k, v = _rand(r, 1, 600, Hkv, D), _rand(r, 1, 600, Hkv, D)
    cache.update(k[:, :250], v[:, :250], 0)
    assert cache.num_blocks == 1
    cache.update(k[:, 250:], v[:, 250:], 250)   # crosses into blocks 1 and 2
    assert cache.num_blocks == 3 and pool.used_blocks() == 6
    gk, gv = cache.get(torch.float32)
    assert np.array_equal(gk.cpu().numpy(), _dense_reference(k)) and np.array_equal(gv.cpu().numpy(), _dense_reference(v))
    cache.truncate_to(300)                      # keeps blocks 0 and 1, returns block 2 (kv_cache.rs:1725-1748)
    assert cache.seq_pos == 300 and cache.num_blocks == 2 and pool.used_blocks() == 4
    gk, _ = cache.get(torch.float32)
    assert np.array_equal(gk.cpu().numpy(), _dense_reference(k[:, :300]))
    cache.update(k[:, 300:600], v[:, 300:600], 300)  # grows again into a (possibly different) block
    gk, _ = cache.get(torch.float32)
    assert np.array_equal(gk.cpu().numpy(), _dense_reference(k))


@pytest.mark.parametrize("D", [64, 128, 256])
def test_chunked_prefill_through_a_paged_cache(D):
    """Two prompt chunks that cross block boundaries: attention of each chunk over [cached blocks | itself] against
    the oracle, and the blocks end up holding what update() would have written."""
    r = wl.philox(905 + D)
    Hq, Hkv, C = 8, 2, 300
    pool = kc.BlockPool(16, Hkv, D)
    cache = kc.PagedLayerKVCache(2048, pool, 7)
    q, k, v = _rand(r, 1, 2 * C, Hq, D), _rand(r, 1, 2 * C, Hkv, D), _rand(r, 1, 2 * C, Hkv, D)
    o0 = cache.prefill(q[:, :C], k[:, :C], v[:, :C], 0, 1 / np.sqrt(D))
    assert cache.seq_pos == C and cache.num_blocks == 2
    o1 = cache.prefill(q[:, C:], k[:, C:], v[:, C:], C, 1 / np.sqrt(D))
    torch.cuda.synchronize()
    assert cache.seq_pos == 2 * C and cache.num_blocks == 3
    kd, vd = cache.get(torch.float32)
    assert np.array_equal(kd.cpu().numpy(), _dense_reference(k)) and np.array_equal(vd.cpu().numpy(), _dense_reference(v))
    kn, vn = k.float().cpu().numpy(), v.float().cpu().numpy()
    want0 = oracle.prefill_attn(q[:, :C].float().cpu().numpy(), kn[:, :C], vn[:, :C], None, None, oracle.FMT_DENSE,
                                np.array([C], np.int32), 1 / np.sqrt(D))
    k1 = np.concatenate([kd[:, :C].cpu().numpy(), kn[:, C:]], 1)
    v1 = np.concatenate([vd[:, :C].cpu().numpy(), vn[:, C:]], 1)
    want1 = oracle.prefill_attn(q[:, C:].float().cpu().numpy(), k1, v1, None, None, oracle.FMT_DENSE,
                                np.array([2 * C], np.int32), 1 / np.sqrt(D))
    for got, want in ((o0, want0), (o1, want1)):
        d = np.abs(got.float().cpu().numpy() - want)
        assert d.max() < 2e-2 and d.mean() < 2e-3
    with pytest.raises(kc.CacheError, match="past the cached tokens"):
        cache.prefill(q[:, :C], k[:, :C], v[:, :C], 1000, 1 / np.sqrt(D))


def test_paged_cache_frees_blocks_on_drop():
    r = wl.philox(902)
    pool = kc.BlockPool(8, 2, 64)
    cache = kc.PagedLayerKVCache(1024, pool, 7)
    cache.update(_rand(r, 1, 10, 2, 64), _rand(r, 1, 10, 2, 64), 0)
    assert pool.used_blocks() == 2
    cache.close()  # dropped WITHOUT an explicit clear()
    assert pool.used_blocks() == 0 and pool.free_block_count() == 8


def test_exhaustion_midway_keeps_earlier_pairs_and_is_retryable():
    r = wl.philox(903)
    pool = kc.BlockPool(3, 2, 64)  # one pair fits, the second pair does not
    cache = kc.PagedLayerKVCache(1024, pool, 1)
    k, v = _rand(r, 1, 300, 2, 64), _rand(r, 1, 300, 2, 64)
    with pytest.raises(kc.BlockPoolExhausted):
        cache.update(k, v, 0)
    assert cache.seq_pos == 0 and pool.used_blocks() == 2  # first pair held, the lone K block of the second returned
    other = pool.allocate(9)
    pool.free(9, other)
    cache.update(k[:, :256], v[:, :256], 0)  # what fits still works
    assert cache.seq_pos == 256


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("lens", [[5, 255, 256, 700], [1, 1, 1]])
def test_ragged_batch_decode_step_matches_oracle(lens, D):
    r = wl.philox(910 + len(lens) + D)
    Hq, Hkv = 8, 2
    n = len(lens)
    pool = kc.BlockPool(64, Hkv, D)
    rows, hist = [], []
    for i, L in enumerate(lens):
        c = kc.PagedLayerKVCache(2048, pool, i)
        if L > 1:
            k, v = _rand(r, 1, L - 1, Hkv, D), _rand(r, 1, L - 1, Hkv, D)
            c.update(k, v, 0)
        else:
            k = v = torch.empty(1, 0, Hkv, D, dtype=torch.bfloat16, device=DEV)
        rows.append(c)
        hist.append((k, v))
    q = _rand(r, n, Hq, D)
    k_new, v_new = _rand(r, n, 1, Hkv, D), _rand(r, n, 1, Hkv, D)
    scale = 1.0 / np.sqrt(D)
    out = kc.paged_batch_decode_step(pool, rows, q, k_new, v_new, scale)
    torch.cuda.synchronize()
    assert [c.seq_pos for c in rows] == lens
    T = max(lens)
    kc_all = np.zeros((n, T, Hkv, D), np.int8); vc_all = np.zeros_like(kc_all)
    ks_all = np.zeros((n, T, Hkv), np.float32); vs_all = np.zeros_like(ks_all)
    for i, L in enumerate(lens):
        kf = torch.cat([hist[i][0], k_new[i:i + 1]], 1).float().cpu().numpy()
        vf = torch.cat([hist[i][1], v_new[i:i + 1]], 1).float().cpu().numpy()
        kc_all[i, :L], ks_all[i, :L] = (a[0] for a in oracle.quant_int8(kf))
        vc_all[i, :L], vs_all[i, :L] = (a[0] for a in oracle.quant_int8(vf))
        # the cache itself holds exactly these codes (dense view == oracle dequant)
        gk, gv = rows[i].get(torch.float32)
        assert np.array_equal(gk.cpu().numpy()[0], oracle.dequant_int8(kc_all[i, :L], ks_all[i, :L]))
        assert np.array_equal(gv.cpu().numpy()[0], oracle.dequant_int8(vc_all[i, :L], vs_all[i, :L]))
    want = oracle.decode_attn(q.float().cpu().numpy(), kc_all, vc_all, ks_all, vs_all, oracle.FMT_INT8,
                              np.array(lens, np.int32), scale)
    err = np.abs(out.float().cpu().numpy() - want)
    assert err.max() < 2e-2 and err.mean() < 2e-3
    # the single-sequence path of one row agrees with the batch path
    single = rows[0].decode_attention(q[:1], scale)
    assert np.abs(single.float().cpu().numpy() - want[:1]).max() < 2e-2


def test_batch_step_refuses_before_launch_when_the_pool_is_empty():
    r = wl.philox(920)
    Hq, Hkv, D = 8, 2, 128
    pool = kc.BlockPool(4, Hkv, D)
    a = kc.PagedLayerKVCache(1024, pool, 1)
    b = kc.PagedLayerKVCache(1024, pool, 2)
    a.update(_rand(r, 1, 256, Hkv, D), _rand(r, 1, 256, Hkv, D), 0)   # a's next token needs a new pair
    b.update(_rand(r, 1, 10, Hkv, D), _rand(r, 1, 10, Hkv, D), 0)
    assert pool.free_block_count() == 0
    with pytest.raises(kc.BlockPoolExhausted):
        kc.paged_batch_decode_step(pool, [a, b], _rand(r, 2, Hq, D), _rand(r, 2, 1, Hkv, D), _rand(r, 2, 1, Hkv, D), 0.1)
    assert a.seq_pos == 256 and b.seq_pos == 10 and pool.used_blocks() == 4
    b.clear()                                                          # another sequence releases its blocks
    out = kc.paged_batch_decode_step(pool, [a], _rand(r, 1, Hq, D), _rand(r, 1, 1, Hkv, D), _rand(r, 1, 1, Hkv, D), 0.1)
    torch.cuda.synchronize()
    assert a.seq_pos == 257 and a.num_blocks == 2 and bool(torch.isfinite(out.float()).all())


# ---------------------------------------------------------------------------------------------- FP8 blocks
def _fp8_reference(k_all, calib_tokens):
    """Dense view of an FP8 cache: scales calibrated on the first `calib_tokens` tokens, codes of every token."""
    x = k_all.float().cpu().numpy()
    sc = oracle.fp8_calibrate(x[:, :calib_tokens])
    return oracle.dequant_fp8(oracle.quant_fp8(x, sc), sc), sc


@pytest.mark.parametrize("D", [64, 128])
def test_fp8_paged_cache_equals_the_contiguous_fp8_cache(D):
    """The FP8 block format: update (calibration at start_pos 0), get, truncate, chunked prefill and decode through a
    paged cache give what the contiguous FP8 LayerKVCache gives, and the oracle's codes."""
    r = wl.philox(930 + D)
    Hq, Hkv, T = 8, 2, 600
    pool = kc.BlockPool(16, Hkv, D, kc.FP8)
    assert kc.lib().hs_pool_quant_type(pool._h) == kc.FP8
    paged = kc.PagedLayerKVCache(2048, pool, "fp8")
    flat = kc.LayerKVCache(2048, kc.FP8)
    k, v = _rand(r, 1, T, Hkv, D) * 0.5, _rand(r, 1, T, Hkv, D) * 0.5
    for c in (paged, flat):
        c.update(k[:, :250], v[:, :250], 0)
        c.update(k[:, 250:], v[:, 250:], 250)
    assert paged.num_blocks == 3 and pool.used_blocks() == 6
    gk, gv = paged.get(torch.float32)
    fk, fv = flat.get(torch.float32)
    assert bool(torch.equal(gk, fk)) and bool(torch.equal(gv, fv))
    wk, _ = _fp8_reference(k, 250)
    wv, _ = _fp8_reference(v, 250)
    assert np.array_equal(gk.cpu().numpy(), wk) and np.array_equal(gv.cpu().numpy(), wv)
    q = _rand(r, 1, Hq, D)
    scale = 1.0 / np.sqrt(D)
    op, of = paged.decode_attention(q, scale), flat.decode_attention(q, scale)
    torch.cuda.synchronize()
    assert np.abs(op.float().cpu().numpy() - of.float().cpu().numpy()).max() < 2e-3
    want = oracle.decode_attn(q.float().cpu().numpy(), wk, wv, None, None, oracle.FMT_DENSE, np.array([T], np.int32), scale)
    assert np.abs(op.float().cpu().numpy() - want).max() < 2e-2
    paged.truncate_to(300)
    assert paged.num_blocks == 2 and pool.used_blocks() == 4
    gk, _ = paged.get(torch.float32)
    assert np.array_equal(gk.cpu().numpy(), wk[:, :300])
    # chunked prefill on top of what is left: the scales stay those of the first update
    S = 100
    qn, kn, vn = _rand(r, 1, S, Hq, D), _rand(r, 1, S, Hkv, D) * 0.5, _rand(r, 1, S, Hkv, D) * 0.5
    flat.truncate_to(300)
    o1, o2 = paged.prefill(qn, kn, vn, 300, scale), flat.prefill(qn, kn, vn, 300, scale)
    torch.cuda.synchronize()
    assert paged.seq_pos == 400 and np.abs(o1.float().cpu().numpy() - o2.float().cpu().numpy()).max() < 4e-3
    gk, gv = paged.get(torch.float32)
    fk, fv = flat.get(torch.float32)
    assert bool(torch.equal(gk, fk)) and bool(torch.equal(gv, fv))


@pytest.mark.parametrize("lens", [[5, 255, 256, 700], [2, 2]])
def test_fp8_ragged_batch_decode_step_matches_oracle(lens):
    """One launch over paged FP8 caches with their own per-head scales (gathered on the device for the step)."""
    r = wl.philox(940 + len(lens))
    Hq, Hkv, D = 8, 2, 128
    n = len(lens)
    pool = kc.BlockPool(64, Hkv, D, kc.FP8)
    rows, hist = [], []
    for i, L in enumerate(lens):
        c = kc.PagedLayerKVCache(2048, pool, i)
        k, v = _rand(r, 1, L - 1, Hkv, D) * (0.3 + 0.2 * i), _rand(r, 1, L - 1, Hkv, D) * (0.3 + 0.2 * i)
        c.update(k, v, 0)
        rows.append(c)
        hist.append((k, v))
    q = _rand(r, n, Hq, D)
    k_new, v_new = _rand(r, n, 1, Hkv, D) * 0.4, _rand(r, n, 1, Hkv, D) * 0.4
    scale = 1.0 / np.sqrt(D)
    out = kc.paged_batch_decode_step(pool, rows, q, k_new, v_new, scale)
    torch.cuda.synchronize()
    assert [c.seq_pos for c in rows] == lens
    T = max(lens)
    kd, vd = np.zeros((n, T, Hkv, D), np.float32), np.zeros((n, T, Hkv, D), np.float32)
    for i, L in enumerate(lens):
        kd[i, :L], _ = _fp8_reference(torch.cat([hist[i][0], k_new[i:i + 1]], 1), L - 1)
        vd[i, :L], _ = _fp8_reference(torch.cat([hist[i][1], v_new[i:i + 1]], 1), L - 1)
        gk, gv = rows[i].get(torch.float32)
        assert np.array_equal(gk.cpu().numpy()[0], kd[i, :L]) and np.array_equal(gv.cpu().numpy()[0], vd[i, :L])
    want = oracle.decode_attn(q.float().cpu().numpy(), kd, vd, None, None, oracle.FMT_DENSE, np.array(lens, np.int32), scale)
    err = np.abs(out.float().cpu().numpy() - want)
    assert err.max() < 2e-2 and err.mean() < 2e-3


def test_fp8_batch_step_refuses_a_row_without_scales():
    pool = kc.BlockPool(8, 2, 128, kc.FP8)
    empty = kc.PagedLayerKVCache(512, pool, 1)
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(kc.CacheError, match="no calibrated scales"):
        kc.paged_batch_decode_step(pool, [empty], z(1, 8, 128), z(1, 1, 2, 128), z(1, 1, 2, 128), 0.1)
    assert empty.seq_pos == 0
