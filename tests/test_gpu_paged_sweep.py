"""The random life of a block pool: up to five paged caches over one pool (int8 or FP8 blocks) grow by updates, prefill
chunks and batched decode steps, shrink by truncation and clearing, close and are replaced, run the pool dry and carry
on (a refused call leaves its cache where it was).  Every paged cache is shadowed by a contiguous cache object that is
fed the same tokens: dense views the same bits, attention outputs within tolerance, and after every operation the
pool's accounting equals two blocks (K and V) per 256 tokens held."""
import numpy as np
import pytest
import torch

from hyprstream_amd import kv_cache as kvc
from gpu_util import DEV

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [41, 42])
def test_paged_caches_shadowed_by_contiguous_ones(seed):
    rng = np.random.default_rng(seed)
    names = ["new", "update", "prefill", "batch", "trunc", "clear", "close", "attend"]
    exhausted = 0
    for t in range(50):
        D, Hkv, G = int(rng.choice([64, 128, 128, 256])), int(rng.choice([1, 2, 8])), int(rng.choice([1, 2, 4]))
        Hq = G * Hkv
        qt = kvc.FP8 if rng.integers(0, 2) else kvc.INT8
        pool = kvc.BlockPool(int(rng.choice([6, 12, 24])) * 2, Hkv, D, qt)
        cap = 1500
        g = torch.Generator(device=DEV)
        g.manual_seed(97 * seed + t)
        sg = 0.5 if qt == kvc.FP8 else 1.0
        mk = lambda *s: (sg * torch.randn(*s, generator=g, device=DEV)).bfloat16()
        scale = 1 / np.sqrt(D)
        rows, next_id = {}, 0  # id -> (paged, contiguous)
        log = [dict(seed=seed, t=t, D=D, Hq=Hq, Hkv=Hkv, fp8=qt == kvc.FP8, blocks=pool.total_blocks())]

        def check(i):
            p, c = rows[i]
            assert p.seq_pos == c.seq_pos, log
            if p.seq_pos > 0:
                (kp, vp), (kc_, vc_) = p.get(), c.get()
                assert torch.equal(kp, kc_) and torch.equal(vp, vc_), log

        for _ in range(int(rng.integers(10, 40))):
            op = rng.choice(names, p=[.12, .2, .2, .2, .08, .04, .08, .08])
            if op == "new" and len(rows) < 5:
                rows[next_id] = (kvc.PagedLayerKVCache(cap, pool, ("session", next_id)), kvc.LayerKVCache(cap, qt))
                log.append(("new", next_id))
                next_id += 1
            elif op in ("update", "prefill") and rows:
                i = int(rng.choice(list(rows)))
                p, c = rows[i]
                pos = p.seq_pos
                n = int(min(cap - pos, rng.choice([1, 7, 64, 255, 256, 257, 600])))
                if n < 1:
                    continue
                k, v = mk(1, n, Hkv, D), mk(1, n, Hkv, D)
                try:
                    if op == "update":
                        p.update(k, v, pos)
                        c.update(k, v, pos)
                    else:
                        q = mk(1, n, Hq, D)
                        got = p.prefill(q, k, v, pos, scale)
                        want = c.prefill(q, k, v, pos, scale)
                        torch.cuda.synchronize()
                        assert bool(torch.isfinite(got.float()).all()), log
                        assert float((got.float() - want.float()).abs().max()) < 2e-2, log
                    log.append((str(op), i, pos, n))
                except kvc.BlockPoolExhausted:
                    exhausted += 1
                    log.append((str(op) + " refused", i, pos, n))
                    assert p.seq_pos == pos, log
                check(i)
            elif op == "batch" and rows:
                ids = [i for i in rows if 1 <= rows[i][0].seq_pos < cap]
                if not ids:
                    continue
                ids = [int(i) for i in rng.choice(ids, size=int(rng.integers(1, len(ids) + 1)), replace=False)]
                n = len(ids)
                q, k, v = mk(n, Hq, D), mk(n, 1, Hkv, D), mk(n, 1, Hkv, D)
                before = [rows[i][0].seq_pos for i in ids]
                try:
                    got = kvc.paged_batch_decode_step(pool, [rows[i][0] for i in ids], q, k, v, scale)
                except kvc.BlockPoolExhausted:
                    exhausted += 1
                    log.append(("batch refused", ids))
                    assert [rows[i][0].seq_pos for i in ids] == before, log
                    continue
                log.append(("batch", ids))
                assert bool(torch.isfinite(got.float()).all()), log
                for j, i in enumerate(ids):
                    want = rows[i][1].decode_step(q[j:j + 1], k[j:j + 1], v[j:j + 1], scale)
                    torch.cuda.synchronize()
                    assert float((got[j:j + 1].float() - want.float()).abs().max()) < 2e-2, log
                    check(i)
            elif op == "trunc" and rows:
                i = int(rng.choice(list(rows)))
                p, c = rows[i]
                if p.seq_pos < 2:
                    continue
                m = int(rng.integers(1, p.seq_pos))
                p.truncate_to(m)
                c.truncate_to(m)
                log.append(("trunc", i, m))
                check(i)
            elif op == "clear" and rows:
                i = int(rng.choice(list(rows)))
                rows[i][0].clear()
                rows[i][1].clear()
                log.append(("clear", i))
                check(i)
            elif op == "close" and rows:
                i = int(rng.choice(list(rows)))
                rows[i][0].close()
                del rows[i]
                log.append(("close", i))
            elif op == "attend" and rows:
                i = int(rng.choice(list(rows)))
                p, c = rows[i]
                if p.seq_pos < 1:
                    continue
                q = mk(1, Hq, D)
                d = (p.decode_attention(q, scale).float() - c.decode_attention(q, scale).float()).abs()
                torch.cuda.synchronize()
                assert float(d.max()) < 2e-2, log
            used = 2 * sum(rows[i][0].num_blocks for i in rows)
            assert pool.used_blocks() == used and pool.free_block_count() == pool.total_blocks() - used, log
        for i in list(rows):
            rows[i][0].close()
        assert pool.used_blocks() == 0, log
    assert exhausted > 0  # the sweep does reach the fail-soft path
