"""Random sequences of operations on the cache object (prefill in chunks of many sizes, decode steps, plain updates,
truncations, attention without a write, clear, dropping the scratch) applied to two instances at once: one that
switches its prompt scratch on at some point (key split of small calls + the bf16 copy of the prompt, with the
bookkeeping of how far the copy is valid), one plain.  After every operation the outputs agree within the attention
tolerance and the dense views returned by get() are the same bits."""
import numpy as np
import pytest
import torch

from hyprstream_amd import kv_cache as kvc
from gpu_util import DEV

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [31, 32])
def test_scratch_and_plain_instances_stay_together(seed):
    rng = np.random.default_rng(seed)
    ops = ["prefill", "step", "update", "trunc", "attend", "clear", "drop"]
    for t in range(80):
        D, Hkv, G = int(rng.choice([64, 128, 128, 128, 256])), int(rng.choice([1, 2, 8])), int(rng.choice([1, 2, 4, 6]))
        Hq, B, cap = G * Hkv, int(rng.integers(1, 4)), int(rng.choice([300, 700, 1500]))
        qt = kvc.FP8 if rng.integers(0, 2) else kvc.INT8
        a, r = kvc.LayerKVCache(cap, qt), kvc.LayerKVCache(cap, qt)
        scratch_at = int(rng.integers(0, 4))
        g = torch.Generator(device=DEV)
        g.manual_seed(31 * seed + t)
        sg = 0.5 if qt == kvc.FP8 else 1.0
        mk = lambda *s: (sg * torch.randn(*s, generator=g, device=DEV)).bfloat16()
        scale = 1 / np.sqrt(D)
        log = [dict(D=D, Hq=Hq, Hkv=Hkv, B=B, cap=cap, fp8=qt == kvc.FP8, scratch_at=scratch_at)]
        for op_i in range(int(rng.integers(3, 12))):
            if op_i == scratch_at:
                a.enable_prompt_scratch(cap)
            pos = a.seq_pos
            assert pos == r.seq_pos, log
            room = cap - pos
            op = rng.choice(ops, p=[.52, .22, .08, .08, .05, .02, .03])
            oa = orf = None
            if op == "prefill" and room >= 1:
                n = int(min(room, rng.choice([1, 5, 64, 100, 128, 257, 512])))
                q, k, v = mk(B, n, Hq, D), mk(B, n, Hkv, D), mk(B, n, Hkv, D)
                oa, orf = a.prefill(q, k, v, pos, scale), r.prefill(q, k, v, pos, scale)
                log.append(("prefill", pos, n))
            elif op == "step" and room >= 1 and pos >= 1:
                q, k, v = mk(B, Hq, D), mk(B, 1, Hkv, D), mk(B, 1, Hkv, D)
                oa, orf = a.decode_step(q, k, v, scale), r.decode_step(q, k, v, scale)
                log.append(("step", pos))
            elif op == "update" and room >= 1:
                n = int(min(room, rng.choice([1, 3, 64, 200])))
                k, v = mk(B, n, Hkv, D), mk(B, n, Hkv, D)
                a.update(k, v, pos)
                r.update(k, v, pos)
                log.append(("update", pos, n))
            elif op == "trunc" and pos > 1:
                m = int(rng.integers(1, pos))
                a.truncate_to(m)
                r.truncate_to(m)
                log.append(("trunc", m))
            elif op == "attend" and pos >= 1:
                q = mk(B, Hq, D)
                oa, orf = a.decode_attention(q, scale), r.decode_attention(q, scale)
                log.append(("attend", pos))
            elif op == "clear":
                a.clear()
                r.clear()
                log.append(("clear",))
            elif op == "drop":
                a.drop_prompt_scratch()
                log.append(("drop",))
            else:
                continue
            torch.cuda.synchronize()
            if oa is not None:
                x, y = oa.float(), orf.float()
                assert bool(torch.isfinite(x).all()), log
                assert float((x - y).abs().max()) < 2e-2 and float((x - y).abs().mean()) < 2e-3, log
            if a.seq_pos > 0 and a.is_initialized():
                (ka, va), (kr, vr) = a.get(), r.get()
                assert torch.equal(ka, kr) and torch.equal(va, vr), log
