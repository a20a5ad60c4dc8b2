"""GPU parity of the launches the benchmark times, at the size they are timed at.

test_gpu_fullsize.py checks the configurations themselves; this file checks the other launches `bench.py` quotes a
roofline figure for, each with the arguments the benchmark passes:

  c2-ragged      B=64, lengths U[512, 8192], `total_tokens_hint = sum(lens)`  -> the balanced token-range split
  c2-paged       B=64 x 8192 through a shuffled table of 256-token blocks (kv_cache.rs:477-693)
  c2-prologue    hs_decode_step_int8_prologue at 64 x 8192 (Llama-flavour QK-norm + whole-head rotation, llama.rs:589-611)
  c4-prologue    hs_decode_step_fp8_prologue at 32 x 32768
  c5-prefill     hs_deltanet_forward_chunked at 4 x 4096 with l2norm = 1 on un-normalised q, k (qwen3_5.rs:678-682)

The oracle cannot redo these sizes whole, so sampled (sequence, kv-head) units are compared with it, rows the launch
writes are compared bit for bit with the oracle's quantizer, and each launch is compared with the unfused / unhinted /
contiguous launch of the same work."""
import numpy as np
import pytest
import torch

import oracle
from oracle import hs_oracle as orc
from oracle import reference_path as ref
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV
from test_gpu_fullsize import TOL_MAX, TOL_MEAN, decode, decode_step_check, fill_cache, gen, sample_check, source

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def test_config2_ragged_with_the_batch_total_hint():
    """What `--workload c2-ragged` launches: the hint selects decode_attn_kernel's balanced instance (equal token
    ranges of the whole batch, one per workgroup, up to 17 partials per sequence) and the merge that recounts them."""
    B, Hq, Hkv, D, T = 64, 32, 8, 128, 8192
    g = gen(wl.SEED + 21)
    lay, kc, vc, ks, vs, _ = fill_cache(g, B, Hkv, T, D, False, 1.0, True)
    q = torch.randn(B, Hq, D, generator=g, device=DEV).to(torch.bfloat16)
    lens = torch.randint(512, T + 1, (B,), generator=g, device=DEV, dtype=torch.int32)
    lens[5], lens[6] = T, 512                                  # both ends of the range are present
    plain = decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, False)  # unhinted: one workgroup per (sequence, head)
    lay.total_tokens_hint = int(lens.sum().item())
    assert hb.decode_num_chunks(B, Hkv, T) == 1 and hb.decode_num_chunks(B, Hkv, T, lay.total_tokens_hint) > 1
    bal = decode(q, kc, vc, ks, vs, lay, lens, Hkv, T, False)
    assert torch.isfinite(bal.float()).all()
    # a different summation order, the same attention: within a bf16 rounding of the unsplit launch everywhere
    assert (bal.float() - plain.float()).abs().max() <= 2 ** -7 * max(1.0, float(plain.float().abs().max()))
    lens_h = lens.cpu().numpy()
    order = np.argsort(lens_h)
    units = [(int(order[0]), 0), (int(order[-1]), 7), (int(order[B // 2]), 3), (5, 2), (6, 5), (63, 1)]
    sample_check(bal, q, kc, vc, ks, vs, lens_h, units, Hq // Hkv, False)
    # the fused step under the same hint (new token written by the workgroup whose range holds the sequence end)
    decode_step_check(g, q, kc, vc, ks, vs, lay, lens, Hkv, T, False, 1.0, True, [(int(order[0]), 4), (int(order[-1]), 0), (31, 6)])


def test_config2_through_a_shuffled_block_table():
    """What `--workload c2-paged` launches: K and V blocks of 256 tokens from one pool in a random order."""
    B, Hq, Hkv, D, T, BT = 64, 32, 8, 128, 8192, 256
    g = gen(wl.SEED + 22)
    lay, kc, vc, ks, vs, _ = fill_cache(g, B, Hkv, T, D, False, 1.0, True)
    q = torch.randn(B, Hq, D, generator=g, device=DEV).to(torch.bfloat16)
    full = torch.full((B,), T, dtype=torch.int32, device=DEV)
    want = decode(q, kc, vc, ks, vs, lay, full, Hkv, T, False)
    nb = T // BT
    perm = torch.randperm(2 * B * nb, generator=torch.Generator().manual_seed(wl.SEED)).to(torch.int32)
    k_tab = perm[: B * nb].reshape(B, nb).contiguous().to(DEV)
    v_tab = perm[B * nb:].reshape(B, nb).contiguous().to(DEV)
    pc = torch.empty(2 * B * nb, Hkv, BT, D, dtype=torch.int8, device=DEV)
    ps = torch.empty(2 * B * nb, Hkv, BT, dtype=torch.float32, device=DEV)
    blocks = lambda c: c.reshape(B, Hkv, nb, BT, D).permute(0, 2, 1, 3, 4).reshape(B * nb, Hkv, BT, D)
    sblocks = lambda s: s[:, :, :T].reshape(B, Hkv, nb, BT).permute(0, 2, 1, 3).reshape(B * nb, Hkv, BT)
    pc[k_tab.long().reshape(-1)] = blocks(kc)
    pc[v_tab.long().reshape(-1)] = blocks(vc)
    ps[k_tab.long().reshape(-1)] = sblocks(ks)
    ps[v_tab.long().reshape(-1)] = sblocks(vs)
    play = hb.paged_layout(Hkv, BT, D, k_tab, v_tab)
    got = decode(q, pc, pc, ps, ps, play, full, Hkv, T, False)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))  # the same walk over the same bytes
    sample_check(got, q, kc, vc, ks, vs, full.cpu().numpy(), [(0, 0), (22, 4), (63, 7)], Hq // Hkv, False)
    # the fused step, as timed: the new token lands in the last block of each sequence's table
    k_new, v_new = source(g, (B, 1, Hkv, D), 1.0, True), source(g, (B, 1, Hkv, D), 1.0, True)
    kc2, vc2, ks2, vs2 = kc.clone(), vc.clone(), ks.clone(), vs.clone()
    hb.kv_quantize_int8(k_new, v_new, kc2, vc2, ks2, vs2, lay, (full - 1).contiguous(), 0)
    want2 = decode(q, kc2, vc2, ks2, vs2, lay, full, Hkv, T, False)
    out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    hb.decode_step(q, k_new, v_new, pc, pc, ps, ps, play, full, out, ws, Hkv, T, 1.0 / np.sqrt(D))
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), want2.view(torch.int16))
    last_k, last_v = k_tab[:, -1].long(), v_tab[:, -1].long()
    assert torch.equal(pc[last_k, :, BT - 1], kc2[:, :, T - 1]) and torch.equal(pc[last_v, :, BT - 1], vc2[:, :, T - 1])
    assert torch.equal(ps[last_k, :, BT - 1], ks2[:, :, T - 1]) and torch.equal(ps[last_v, :, BT - 1], vs2[:, :, T - 1])
    wk, wks = oracle.quant_int8(k_new.float().cpu().numpy())
    assert np.array_equal(wk[:, 0], kc2[:, :, T - 1].cpu().numpy()) and np.array_equal(wks[:, 0], ks2[:, :, T - 1].cpu().numpy())


def _llama_prologue(g, D, T):
    """The prologue `bench.py --workload c2-prologue / c4-prologue` passes: Llama-flavour norm, whole-head rotation."""
    sin, cos = ref.rope_tables(D, 10000.0, T, torch.bfloat16)  # libtorch CPU ops in the reference's order: test data
    qw = (1.0 + 0.1 * torch.randn(D, generator=g, device=DEV)).to(torch.bfloat16)
    kw = (1.0 + 0.1 * torch.randn(D, generator=g, device=DEV)).to(torch.bfloat16)
    pro = hb.qk_prologue(hb.QKNORM_LLAMA, 1e-6, qw, kw, sin.contiguous().to(DEV), cos.contiguous().to(DEV))
    return pro, qw, kw, sin.contiguous(), cos.contiguous()


def _oracle_prologue(x_bits, w, sin, cos, pos):
    y = orc.qk_norm_bf16(x_bits, hb.QKNORM_LLAMA, _bits(w), 1e-6)
    return orc.rope_apply_bf16(np.ascontiguousarray(y), _bits(sin), _bits(cos), pos)


@pytest.mark.parametrize("fp8", [False, True])
def test_decode_step_with_prologue_at_the_timed_size(fp8):
    """64 x 8192 int8 (c2-prologue) and 32 x 32768 fp8 (c4-prologue): the row the launch writes is the oracle's
    quantizer applied to the oracle's normalised and rotated k_new, bit for bit; the launch equals the pre-pass
    followed by the plain step bit for bit; sampled units agree with the oracle's attention over the oracle's q."""
    if fp8:
        B, Hq, Hkv, D, T, sigma, outl = 32, 64, 8, 128, 32768, 0.5, False
    else:
        B, Hq, Hkv, D, T, sigma, outl = 64, 32, 8, 128, 8192, 1.0, True
    g = gen(wl.SEED + 23 + int(fp8))
    lay, kc, vc, ks, vs, _ = fill_cache(g, B, Hkv, T, D, fp8, sigma, outl)
    pro, qw, kw, sin, cos = _llama_prologue(g, D, T)
    q = (torch.randn(B, Hq, D, generator=g, device=DEV) * 1.5).to(torch.bfloat16)
    k_new, v_new = source(g, (B, 1, Hkv, D), sigma, outl), source(g, (B, 1, Hkv, D), sigma, outl)
    lens = torch.full((B,), T, dtype=torch.int32, device=DEV)
    lens[1] = T - 1000                                         # one row at another position of the table
    scale = 1.0 / np.sqrt(D)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    # unfused on copies: pre-pass, then the plain fused step
    kc2, vc2 = kc.clone(), vc.clone()
    ks2, vs2 = ks.clone(), vs.clone()
    q2 = torch.empty(B, 1, Hq, D, dtype=torch.bfloat16, device=DEV)
    k2 = torch.empty(B, 1, Hkv, D, dtype=torch.bfloat16, device=DEV)
    hb.qk_prologue_apply(q.view(B, 1, Hq, D), k_new, pro, q2, k2, (lens - 1).contiguous(), 0)
    want = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    hb.decode_step(q2.view(B, Hq, D), k2, v_new, kc2, vc2, ks2, vs2, lay, lens, want, ws, Hkv, T, scale, fp8=fp8)
    out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    hb.decode_step_prologue(q, k_new, v_new, pro, kc, vc, ks, vs, lay, lens, out, ws, Hkv, T, scale, fp8=fp8)
    torch.cuda.synchronize()
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2) and torch.equal(ks, ks2) and torch.equal(vs, vs2)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    # the oracle's prologue and quantizer for every sequence's written row
    pos = (lens - 1).cpu().numpy().astype(np.int32)
    q_fin = _oracle_prologue(_bits(q).reshape(B, Hq, D), qw, sin, cos, pos)
    k_fin = _oracle_prologue(_bits(k_new).reshape(B, Hkv, D), kw, sin, cos, pos)
    assert np.array_equal(_bits(q2).reshape(B, Hq, D), q_fin)
    rows = torch.arange(B, device=DEV)
    got_kc = kc[rows, :, (lens - 1).long()].cpu().numpy()      # [B, Hkv, D]
    got_vc = vc[rows, :, (lens - 1).long()].cpu().numpy()
    if fp8:
        ksn, vsn = ks.cpu().numpy(), vs.cpu().numpy()
        assert np.array_equal(oracle.quant_fp8(oracle.bf16_to_f32(k_fin).reshape(B, 1, Hkv, D), ksn)[:, 0], got_kc)
        assert np.array_equal(oracle.quant_fp8(v_new.float().cpu().numpy(), vsn)[:, 0], got_vc)
    else:
        wkc, wks = oracle.quant_int8(oracle.bf16_to_f32(k_fin).reshape(B, 1, Hkv, D))
        wvc, wvs = oracle.quant_int8(v_new.float().cpu().numpy())
        got_ks = ks[rows, :, (lens - 1).long()].cpu().numpy()
        got_vs = vs[rows, :, (lens - 1).long()].cpu().numpy()
        assert np.array_equal(wkc[:, 0], got_kc) and np.array_equal(wks[:, 0].view(np.uint32), got_ks.view(np.uint32))
        assert np.array_equal(wvc[:, 0], got_vc) and np.array_equal(wvs[:, 0].view(np.uint32), got_vs.view(np.uint32))
    # attention of the oracle's q over the cache, sampled units
    q_or = torch.from_numpy(oracle.bf16_to_f32(q_fin)).to(DEV).to(torch.bfloat16)
    sample_check(out, q_or, kc, vc, ks, vs, lens.cpu().numpy(), [(0, 0), (1, 3), (B - 1, 7)], Hq // Hkv, fp8)


def test_config5_chunked_deltanet_normalising_in_the_kernel():
    """B = 4 x 4096, chunk 64, q and k as the projections give them (NOT normalised) and l2norm = 1, the reference's
    setting (the layer normalises inside, qwen3_5.rs:678-682): sampled (sequence, head) pairs against the oracle of
    the recurrence with its own normalisation, the whole output against the fp32 recurrent kernel."""
    nk, nv, d = 16, 32, 128
    g = gen(wl.SEED + 56)
    B, T = 4, 4096
    mag = 0.5 + 3.0 * torch.rand(B, T, nk, 1, generator=g, device=DEV)     # row norms far from one
    q = (torch.randn(B, T, nk, d, generator=g, device=DEV) * mag).to(torch.bfloat16)
    k = (torch.randn(B, T, nk, d, generator=g, device=DEV) * mag.flip(1)).to(torch.bfloat16)
    v = torch.randn(B, T, nv, d, generator=g, device=DEV).to(torch.bfloat16)
    gg = -torch.nn.functional.softplus(torch.randn(B, T, nv, generator=g, device=DEV))
    beta = torch.sigmoid(torch.randn(B, T, nv, generator=g, device=DEV))
    qs = 1 / np.sqrt(d)
    st, out = torch.zeros(B, nv, d, d, device=DEV), torch.full((B, T, nv, d), float("nan"), device=DEV)
    hb.deltanet_forward_chunked(q, k, v, gg, beta, st, out, qs, True)
    st3, out3 = torch.zeros(B, nv, d, d, device=DEV), torch.empty(B, T, nv, d, device=DEV)
    hb.deltanet_forward(q, k, v, gg, beta, st3, out3, qs, True)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all() and torch.isfinite(st).all()
    rel = 3e-3
    assert float((out - out3).abs().max()) <= rel * float(out3.abs().max())
    assert float((st - st3).abs().max()) <= rel * float(st3.abs().max())
    for b, j in ((0, 2), (2, 17), (3, 31)):
        hk = j // 2
        wo, wst = oracle.deltanet_recurrent(q[b:b + 1, :, hk:hk + 1].float().cpu().numpy(), k[b:b + 1, :, hk:hk + 1].float().cpu().numpy(),
                                            v[b:b + 1, :, j:j + 1].float().cpu().numpy(), gg[b:b + 1, :, j:j + 1].cpu().numpy(),
                                            beta[b:b + 1, :, j:j + 1].cpu().numpy(), None, qs, True)
        eo = np.abs(out[b, :, j].cpu().numpy() - wo[0, :, 0]).max()
        es = np.abs(st[b, j].cpu().numpy() - wst[0, 0]).max()
        assert eo <= rel * np.abs(wo).max() and es <= rel * np.abs(wst).max(), (b, j, eo, es)
        assert eo < TOL_MAX
