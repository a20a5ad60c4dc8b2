"""GPU parity of the decode path's balanced split: a ragged batch (the layout's total_tokens_hint says so) is cut
into equal token ranges over all sequences instead of fixed chunks per sequence.  Each case runs the hinted call,
the call without a hint (fixed chunks) and the CPU oracle on the same cache.

Tolerance of the path (fp32 comparison of the bf16 output): max-abs 2e-2, mean-abs 2e-3; hinted against
unhinted (same arithmetic, another summation order): max-abs 1e-2."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV, bf16_from_bits, run_decode
from test_gpu_decode import build_cache, TOL_MAX, TOL_MEAN

pytestmark = pytest.mark.gpu


def hinted_layout(c, D, hint):
    lay = hb.contiguous_layout(c.Hkv, c.cap, D)
    lay.total_tokens_hint = int(hint)
    return lay


def three_way(case, Hq, Hkv, D, T, fp8=False, hint=None, label=""):
    c = build_cache(case, Hkv, D, fp8=fp8)
    lens = case["seq_lens"]
    hint = max(1, int(np.clip(lens, 0, T).sum())) if hint is None else hint
    B = len(lens)
    assert hb.decode_num_chunks(B, Hkv, T, hint) > 1, "the case must select the balanced split"
    plain = run_decode(c, case["q_bits"], lens, Hq, max_seq_len=T)
    hinted = run_decode(c, case["q_bits"], lens, Hq, max_seq_len=T, layout=hinted_layout(c, D, hint))
    kc, vc, ks, vs = c.canonical(T)
    want = oracle.decode_attn(oracle.bf16_to_f32(case["q_bits"]), kc, vc, ks, vs,
                              oracle.FMT_FP8 if fp8 else oracle.FMT_INT8, np.clip(lens, 0, T), 1.0 / np.sqrt(D))
    assert np.isfinite(hinted).all(), label
    for got in (plain, hinted):
        d = np.abs(got - want)
        assert d.max() < TOL_MAX and d.mean() < TOL_MEAN, label
    assert np.abs(plain - hinted).max() < 1e-2, label
    return hinted


@pytest.mark.parametrize("D,fp8", [(64, False), (128, False), (256, False), (128, True), (64, True), (256, True)])
def test_ragged_batch_every_head_dim_and_format(D, fp8):
    B, Hq, Hkv, T = 24, 16, 4, 2500
    case = wl.decode_case(70 + D + int(fp8), B, Hq, Hkv, D, T, ragged=True, outliers=not fp8, min_len=1)
    case["seq_lens"][0] = T  # the longest sequence spans several ranges
    three_way(case, Hq, Hkv, D, T, fp8=fp8, label="D%d fp8=%s" % (D, fp8))


@pytest.mark.parametrize("lens", [
    [4000, 1, 1, 1, 1, 1, 1, 1],                 # one long sequence and many of one token
    [0, 3000, 0, 0, 17, 0, 64, 0],               # empty sequences between the others, also first and last
    [63, 64, 65, 127, 128, 129, 2047, 2048],     # granule edges
    [1, 2, 3],                                   # fewer granules in the batch than one range holds
    [5000] + [700] * 40,                         # many sequences per range
    [-5, 9999, 300],                             # negative = empty, above max_seq_len = clipped to it
])
def test_length_patterns(lens):
    B, Hq, Hkv, D, T = len(lens), 8, 2, 128, 5000
    case = wl.decode_case(77, B, Hq, Hkv, D, T, outliers=True)
    case["seq_lens"] = np.array(lens, np.int32)
    got = three_way(case, Hq, Hkv, D, T, label=str(lens[:8]))
    for b, n in enumerate(lens):
        if n <= 0:
            assert not got[b].any()


def test_wrong_hints_change_nothing():
    """The hint only selects the split; the ranges come from the lengths read on the device."""
    B, Hq, Hkv, D, T = 16, 8, 2, 128, 3000
    case = wl.decode_case(78, B, Hq, Hkv, D, T, ragged=True, min_len=10)
    c = build_cache(case, Hkv, D)
    lens = case["seq_lens"]
    outs = [run_decode(c, case["q_bits"], lens, Hq, max_seq_len=T, layout=hinted_layout(c, D, h))
            for h in (int(lens.sum()), 1, B * 64, B * T // 2)]
    for o in outs[1:]:
        assert np.array_equal(o, outs[0])


def test_more_sequences_than_the_prefix_table_falls_back_to_fixed_chunks():
    B, Hq, Hkv, D, T = 1100, 2, 1, 64, 300
    assert hb.decode_num_chunks(B, Hkv, T, B * 100) == hb.decode_num_chunks(B, Hkv, T)
    assert hb.decode_num_chunks(1024, Hkv, T, 1024 * 100) > 1
    case = wl.decode_case(79, B, Hq, Hkv, D, T, ragged=True)
    c = build_cache(case, Hkv, D)
    a = run_decode(c, case["q_bits"], case["seq_lens"], Hq, max_seq_len=T)
    b = run_decode(c, case["q_bits"], case["seq_lens"], Hq, max_seq_len=T,
                   layout=hinted_layout(c, D, int(case["seq_lens"].sum())))
    assert np.array_equal(a, b)


def test_a_thousand_short_sequences():
    B, Hq, Hkv, D, T = 1024, 4, 2, 64, 400
    case = wl.decode_case(80, B, Hq, Hkv, D, T, ragged=True)
    case["seq_lens"][::7] = 0
    three_way(case, Hq, Hkv, D, T, label="B1024")


@pytest.mark.parametrize("fp8", [False, True])
def test_decode_step_writes_the_new_token_in_the_range_that_owns_the_end(fp8):
    """hs_decode_step with the hint: codes and scales written equal those of the unhinted step, outputs agree."""
    B, Hq, Hkv, D, T = 12, 16, 4, 128, 2100
    case = wl.decode_case(81, B, Hq, Hkv, D, T, ragged=True, outliers=not fp8, min_len=2)
    case["seq_lens"][3] = T
    lens_np = case["seq_lens"]
    lens = torch.from_numpy(lens_np).to(DEV)
    q = bf16_from_bits(case["q_bits"]).to(DEV)
    idx = torch.from_numpy(lens_np.astype(np.int64) - 1)
    nk = torch.from_numpy(case["k"])[torch.arange(B), idx].unsqueeze(1).to(torch.bfloat16).to(DEV).contiguous()
    nv = torch.from_numpy(case["v"])[torch.arange(B), idx].unsqueeze(1).to(torch.bfloat16).to(DEV).contiguous()
    res = []
    for hint in (0, int(lens_np.sum())):
        c = build_cache(case, Hkv, D, fp8=fp8)
        for b in range(B):  # forget the last token: the step has to write it
            c.k_codes[b, :, lens_np[b] - 1] = 0
            c.v_codes[b, :, lens_np[b] - 1] = 0
            if not fp8:
                c.k_scales[b, :, lens_np[b] - 1] = 0
                c.v_scales[b, :, lens_np[b] - 1] = 0
        out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
        hb.decode_step(q, nk, nv, c.k_codes, c.v_codes, c.k_scales, c.v_scales, hinted_layout(c, D, hint), lens, out, ws,
                       Hkv, T, 1.0 / np.sqrt(D), fp8=fp8)
        torch.cuda.synchronize()
        res.append((out.float().cpu().numpy(), c))
    (o0, c0), (o1, c1) = res
    assert torch.equal(c0.k_codes, c1.k_codes) and torch.equal(c0.v_codes, c1.v_codes)
    assert torch.equal(c0.k_scales, c1.k_scales) and torch.equal(c0.v_scales, c1.v_scales)
    assert np.isfinite(o1).all() and np.abs(o0 - o1).max() < 1e-2
    ref = build_cache(case, Hkv, D, fp8=fp8)  # the same cache written by the quantize entry point
    assert torch.equal(ref.k_codes, c1.k_codes) and torch.equal(ref.v_codes, c1.v_codes)


def test_paged_cache_with_the_hint():
    """Block tables in shuffled order, 64-token blocks: the balanced ranges walk them like the fixed chunks do."""
    B, Hq, Hkv, D, T, bt = 10, 8, 2, 128, 1536, 64
    case = wl.decode_case(82, B, Hq, Hkv, D, T, ragged=True, min_len=1)
    case["seq_lens"][0] = T
    kc, ksc = oracle.quant_int8(case["k"])
    vc, vsc = oracle.quant_int8(case["v"])
    nb = T // bt
    r = np.random.default_rng(5)
    perm = r.permutation(B * nb).astype(np.int32)
    table = torch.from_numpy(perm.reshape(B, nb)).to(DEV)
    lay = hb.paged_layout(Hkv, bt, D, table, table)
    pad = lay.scale_stride_head
    kp = torch.zeros(B * nb, Hkv, bt, D, dtype=torch.int8, device=DEV)
    vp = torch.zeros_like(kp)
    ksp = torch.zeros(B * nb, Hkv, pad, dtype=torch.float32, device=DEV)
    vsp = torch.zeros_like(ksp)
    for b in range(B):
        for j in range(nb):
            blk = int(perm[b * nb + j])
            sl = slice(j * bt, (j + 1) * bt)
            kp[blk] = torch.from_numpy(kc[b, sl]).permute(1, 0, 2).to(DEV)
            vp[blk] = torch.from_numpy(vc[b, sl]).permute(1, 0, 2).to(DEV)
            ksp[blk, :, :bt] = torch.from_numpy(ksc[b, sl]).permute(1, 0).to(DEV)
            vsp[blk, :, :bt] = torch.from_numpy(vsc[b, sl]).permute(1, 0).to(DEV)
    q = bf16_from_bits(case["q_bits"]).to(DEV)
    lens = torch.from_numpy(case["seq_lens"]).to(DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    outs = []
    for hint in (0, int(case["seq_lens"].sum())):
        lay.total_tokens_hint = hint
        out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        hb.decode_attn(q, kp, vp, ksp, vsp, lay, lens, out, ws, Hkv, T, 1.0 / np.sqrt(D))
        torch.cuda.synchronize()
        outs.append(out.float().cpu().numpy())
    want = oracle.decode_attn(oracle.bf16_to_f32(case["q_bits"]), kc, vc, ksc, vsc, oracle.FMT_INT8, case["seq_lens"],
                              1.0 / np.sqrt(D))
    for got in outs:
        d = np.abs(got - want)
        assert d.max() < TOL_MAX and d.mean() < TOL_MEAN
    assert np.abs(outs[0] - outs[1]).max() < 1e-2


@pytest.mark.parametrize("D,rd", [(128, 128), (64, 64), (256, 64)])
def test_decode_step_with_the_prologue_inside_a_hinted_launch(D, rd):
    """QK-norm + rotation of q and k_new inside the launch (hs_decode_step_int8_prologue) on a ragged batch with the
    hint: the cache rows written equal those of the unhinted launch bit for bit (the prologue's arithmetic does not
    depend on the split), the outputs agree like any two splits, and both equal the separate pre-pass
    (hs_qk_prologue_apply) followed by the plain step."""
    B, Hq, Hkv, T = 9, 8, 2, 1700
    case = wl.decode_case(83 + D, B, Hq, Hkv, D, T, ragged=True, min_len=2)
    case["seq_lens"][1] = T
    lens_np = case["seq_lens"]
    lens = torch.from_numpy(lens_np).to(DEV)
    r = wl.philox(900 + D)
    q = torch.from_numpy(r.standard_normal((B, Hq, D)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    nk = torch.from_numpy(r.standard_normal((B, 1, Hkv, D)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    nv = torch.from_numpy(r.standard_normal((B, 1, Hkv, D)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    qw = torch.from_numpy(1.0 + 0.1 * r.standard_normal(D).astype(np.float32)).to(torch.bfloat16).to(DEV)
    kw = torch.from_numpy(1.0 + 0.1 * r.standard_normal(D).astype(np.float32)).to(torch.bfloat16).to(DEV)
    ang = torch.arange(T, dtype=torch.float32)[:, None] / (10000.0 ** (torch.arange(0, rd, 2, dtype=torch.float32) / rd))[None, :]
    sin, cos = ang.sin().to(torch.bfloat16).to(DEV).contiguous(), ang.cos().to(torch.bfloat16).to(DEV).contiguous()
    pro = hb.qk_prologue(hb.QKNORM_LLAMA, 1e-6, qw, kw, sin, cos, rotary_dim=rd)
    scale = 1.0 / np.sqrt(D)

    def fresh():
        c = build_cache(case, Hkv, D)
        for b in range(B):  # the step has to write the last token
            c.k_codes[b, :, lens_np[b] - 1] = 0
            c.v_codes[b, :, lens_np[b] - 1] = 0
            c.k_scales[b, :, lens_np[b] - 1] = 0
            c.v_scales[b, :, lens_np[b] - 1] = 0
        return c

    res = []
    for hint in (0, int(lens_np.sum())):
        c = fresh()
        out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
        hb.decode_step_prologue(q, nk, nv, pro, c.k_codes, c.v_codes, c.k_scales, c.v_scales, hinted_layout(c, D, hint), lens,
                                out, ws, Hkv, T, scale)
        torch.cuda.synchronize()
        res.append((out.float().cpu().numpy(), c))
    (o0, c0), (o1, c1) = res
    assert torch.equal(c0.k_codes, c1.k_codes) and torch.equal(c0.v_codes, c1.v_codes)
    assert torch.equal(c0.k_scales, c1.k_scales) and torch.equal(c0.v_scales, c1.v_scales)
    assert np.isfinite(o1).all() and np.abs(o0 - o1).max() < 1e-2
    # the pre-pass + the plain hinted step: the same rows in the cache, outputs bit for bit (same split, same q)
    c2 = fresh()
    q_rot, k_rot = torch.empty(B, 1, Hq, D, dtype=torch.bfloat16, device=DEV), torch.empty_like(nk)
    hb.qk_prologue_apply(q.view(B, 1, Hq, D), nk, pro, q_rot, k_rot, (lens - 1).to(torch.int32).contiguous(), 0)
    out2 = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    hb.decode_step(q_rot.view(B, Hq, D).contiguous(), k_rot, nv, c2.k_codes, c2.v_codes, c2.k_scales, c2.v_scales,
                   hinted_layout(c2, D, int(lens_np.sum())), lens, out2, ws, Hkv, T, scale)
    torch.cuda.synchronize()
    assert torch.equal(c2.k_codes, c1.k_codes) and torch.equal(c2.k_scales, c1.k_scales)
    assert np.array_equal(out2.float().cpu().numpy(), o1)
