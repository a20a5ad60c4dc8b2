"""GPU parity: dequant-fused GQA decode attention against the CPU oracle.

Tolerance of the path (fp32 comparison of the bf16 output): max-abs 2e-2, mean-abs 2e-3."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV, DeviceCache, bf16_from_bits, run_decode

pytestmark = pytest.mark.gpu

TOL_MAX, TOL_MEAN = 2e-2, 2e-3


def build_cache(case, Hkv, D, cap=None, via_gpu_quantizer=True, fp8=False):
    k, v = case["k"], case["v"]
    B, T = k.shape[:2]
    c = DeviceCache(B, Hkv, cap or T, D, fp8=fp8)
    if via_gpu_quantizer:
        ks, vs = torch.from_numpy(k).to(DEV), torch.from_numpy(v).to(DEV)
        if fp8:
            hb.kv_fp8_calibrate(ks, vs, c.k_scales, c.v_scales)
        c.write(ks, vs, None, 0)
    else:
        if fp8:
            sk, sv = oracle.fp8_calibrate(k), oracle.fp8_calibrate(v)
            c.load_canonical(oracle.quant_fp8(k, sk), oracle.quant_fp8(v, sv), sk, sv)
        else:
            kc, ksc = oracle.quant_int8(k)
            vc, vsc = oracle.quant_int8(v)
            c.load_canonical(kc, vc, ksc, vsc)
    torch.cuda.synchronize()
    return c


def check(case, Hq, Hkv, D, fp8=False, cap=None, label=""):
    c = build_cache(case, Hkv, D, cap=cap, fp8=fp8)
    T = case["k"].shape[1]
    got = run_decode(c, case["q_bits"], case["seq_lens"], Hq)
    kc, vc, ks, vs = c.canonical(T)
    want = oracle.decode_attn(oracle.bf16_to_f32(case["q_bits"]), kc, vc, ks, vs,
                              oracle.FMT_FP8 if fp8 else oracle.FMT_INT8, case["seq_lens"], 1.0 / np.sqrt(D))
    assert np.isfinite(got).all(), label
    d = np.abs(got - want)
    print("%s max-abs %.3e mean-abs %.3e" % (label, d.max(), d.mean()), flush=True)
    assert d.max() < TOL_MAX and d.mean() < TOL_MEAN, label
    return got, want


def test_config1_single_sequence_fp32_source():
    """B=1, Hq 32 / Hkv 8, D 128, T 2048, K/V fp32 N(0,1): the single-sequence benchmark configuration."""
    case = wl.decode_case(1, 1, 32, 8, 128, 2048, bf16_source=False)
    got, want = check(case, 32, 8, 128, label="config1")
    assert np.abs(got - want).max() < 4e-3  # far inside the stated tolerance


def test_codes_written_by_gpu_equal_oracle_codes():
    case = wl.decode_case(2, 2, 8, 2, 128, 300, outliers=True)
    c = build_cache(case, 2, 128)
    kc, vc, ks, vs = c.canonical(300)
    wk, wks = oracle.quant_int8(case["k"])
    wv, wvs = oracle.quant_int8(case["v"])
    assert np.array_equal(kc, wk) and np.array_equal(vc, wv)
    assert np.array_equal(ks, wks) and np.array_equal(vs, wvs)


@pytest.mark.parametrize("lens", [[1], [31], [32], [33], [127, 128, 129], [1, 700, 64, 257, 5]])
def test_ragged_lengths_and_step_boundaries(lens):
    B = len(lens)
    case = wl.decode_case(3, B, 32, 8, 128, max(lens), outliers=True)
    case["seq_lens"] = np.array(lens, np.int32)
    check(case, 32, 8, 128, cap=max(lens) + 3, label="ragged%s" % lens)


def test_ragged_uniform_lengths_config2_shape_reduced():
    case = wl.decode_case(4, 6, 32, 8, 128, 1500, ragged=True, outliers=True, min_len=100)
    check(case, 32, 8, 128, label="ragged-uniform")


def test_ragged_batch_hint_changes_the_split_not_the_result():
    """B*Hkv = 512 units (unsplit without a hint) with lengths U[100, 3000]: the hinted call cuts the long
    sequences into several chunks, merges them, and must agree with the unsplit call and the oracle."""
    B, Hq, Hkv, D, T = 64, 32, 8, 128, 3000
    case = wl.decode_case(41, B, Hq, Hkv, D, T, ragged=True, outliers=True, min_len=100)
    c = build_cache(case, Hkv, D)
    lens = case["seq_lens"]
    plain = run_decode(c, case["q_bits"], lens, Hq, max_seq_len=T)
    lay = hb.contiguous_layout(Hkv, c.cap, D)
    lay.total_tokens_hint = int(lens.sum())
    assert hb.decode_num_chunks(B, Hkv, T) == 1 and hb.decode_num_chunks(B, Hkv, T, lay.total_tokens_hint) > 1
    hinted = run_decode(c, case["q_bits"], lens, Hq, max_seq_len=T, layout=lay)
    kc, vc, ks, vs = c.canonical(T)
    want = oracle.decode_attn(oracle.bf16_to_f32(case["q_bits"]), kc, vc, ks, vs, oracle.FMT_INT8, lens, 1.0 / np.sqrt(D))
    for got in (plain, hinted):
        d = np.abs(got - want)
        assert d.max() < TOL_MAX and d.mean() < TOL_MEAN
    assert np.abs(plain - hinted).max() < 1e-2  # same math, different summation order and one more bf16 rounding path


@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (8, 4), (16, 2), (16, 1), (64, 8)])
def test_gqa_group_sizes(Hq, Hkv):
    case = wl.decode_case(5, 2, Hq, Hkv, 128, 200)
    check(case, Hq, Hkv, 128, label="gqa%d/%d" % (Hq, Hkv))


def test_many_chunks_single_head():
    """One sequence, one kv-head: the split-K path uses many chunks and the merge kernel does the work."""
    case = wl.decode_case(6, 1, 4, 1, 128, 9000)
    check(case, 4, 1, 128, label="many-chunks")


def test_zero_and_invalid_lengths_give_zero_rows():
    case = wl.decode_case(7, 3, 8, 2, 128, 64)
    case["seq_lens"] = np.array([0, 64, -3], np.int32)
    c = build_cache(case, 2, 128)
    got = run_decode(c, case["q_bits"], case["seq_lens"], 8, max_seq_len=64)
    assert not got[0].any() and not got[2].any() and np.isfinite(got).all() and got[1].any()


def test_tail_garbage_is_never_read_as_data():
    """Codes/scales past seq_len are poison (NaN scales, extreme codes): results must not change."""
    case = wl.decode_case(8, 2, 8, 2, 128, 100)
    case["seq_lens"] = np.array([70, 33], np.int32)
    c = build_cache(case, 2, 128, cap=128)
    clean = run_decode(c, case["q_bits"], case["seq_lens"], 8)
    for b, n in enumerate(case["seq_lens"]):
        c.k_codes[b, :, n:] = 127
        c.v_codes[b, :, n:] = -127
        c.k_scales[b, :, n:] = float("nan")
        c.v_scales[b, :, n:] = float("inf")
    dirty = run_decode(c, case["q_bits"], case["seq_lens"], 8)
    assert np.array_equal(clean, dirty)


def test_large_q_and_scale_ranges():
    """Q far outside fp16 range and K/V with huge / tiny magnitudes: the power-of-two rescaling keeps it exact."""
    case = wl.decode_case(9, 2, 8, 2, 128, 96)
    q = oracle.bf16_to_f32(case["q_bits"])
    q[0] *= 3.0e5
    q[1] *= 2.0e-6
    case["q_bits"] = wl.to_bf16_bits(q)
    case["k"][0] *= 1e-5
    case["k"][1] *= 1e5
    c = build_cache(case, 2, 128)
    got = run_decode(c, case["q_bits"], case["seq_lens"], 8)
    kc, vc, ks, vs = c.canonical(96)
    want = oracle.decode_attn(oracle.bf16_to_f32(case["q_bits"]), kc, vc, ks, vs, oracle.FMT_INT8, case["seq_lens"],
                              1.0 / np.sqrt(128))
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < TOL_MAX


def test_batched_equals_serial():
    """The reference's own test idea (llama.rs:3658-3711): a ragged batch must equal row-by-row runs."""
    case = wl.decode_case(10, 4, 8, 2, 128, 300, ragged=True)
    c = build_cache(case, 2, 128)
    full = run_decode(c, case["q_bits"], case["seq_lens"], 8)
    for b in range(4):
        one = DeviceCache(1, 2, 300, 128)
        one.k_codes.copy_(c.k_codes[b:b + 1]); one.v_codes.copy_(c.v_codes[b:b + 1])
        one.k_scales.copy_(c.k_scales[b:b + 1]); one.v_scales.copy_(c.v_scales[b:b + 1])
        row = run_decode(one, case["q_bits"][b:b + 1], case["seq_lens"][b:b + 1], 8)
        assert np.abs(row[0] - full[b]).max() < 2e-3


def test_paged_block_table_matches_contiguous():
    """Blocks of 64 tokens scattered through a pool (the reference pool uses 256-token blocks,
    kv_cache.rs:477; 64 keeps the test small) must give the same result as the contiguous cache."""
    B, Hq, Hkv, D, T, BT = 3, 8, 2, 128, 200, 64
    case = wl.decode_case(11, B, Hq, Hkv, D, T, ragged=True)
    c = build_cache(case, Hkv, D)
    want = run_decode(c, case["q_bits"], case["seq_lens"], Hq)
    nblk = (T + BT - 1) // BT
    r = wl.philox(12)
    ids = r.permutation(2 * B * nblk + 5).astype(np.int32)
    kt, vt = ids[: B * nblk].reshape(B, nblk), ids[B * nblk: 2 * B * nblk].reshape(B, nblk)
    pool = len(ids)
    pk = torch.zeros(pool, Hkv, BT, D, dtype=torch.int8, device=DEV)
    ps = torch.zeros(pool, Hkv, BT, dtype=torch.float32, device=DEV)
    k_tab, v_tab = torch.from_numpy(kt).to(DEV), torch.from_numpy(vt).to(DEV)
    lay = hb.paged_layout(Hkv, BT, D, k_tab, v_tab)
    # write through the paged quantizer (one pool for K and V, as the reference's BlockPool)
    ksrc, vsrc = torch.from_numpy(case["k"]).to(DEV), torch.from_numpy(case["v"]).to(DEV)
    hb.kv_quantize_int8(ksrc, vsrc, pk, pk, ps, ps, lay, None, 0)
    torch.cuda.synchronize()
    # block contents equal the contiguous cache's
    for b in range(B):
        for j in range(nblk):
            n = min(BT, T - j * BT)
            assert torch.equal(pk[kt[b, j], :, :n], c.k_codes[b, :, j * BT: j * BT + n])
            assert torch.equal(pk[vt[b, j], :, :n], c.v_codes[b, :, j * BT: j * BT + n])
    q = bf16_from_bits(case["q_bits"]).to(DEV)
    out = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    hb.decode_attn(q, pk, pk, ps, ps, lay, torch.from_numpy(case["seq_lens"]).to(DEV), out, ws, Hkv, T,
                   1.0 / np.sqrt(D))
    torch.cuda.synchronize()
    assert np.array_equal(out.float().cpu().numpy(), want)


def test_constant_values_give_constant_output():
    """Softmax weights sum to one: with every V element equal, the output is that value."""
    case = wl.decode_case(13, 2, 8, 2, 128, 500)
    c = build_cache(case, 2, 128)
    c.v_codes.fill_(64)
    c.v_scales.fill_(0.125)
    got = run_decode(c, case["q_bits"], case["seq_lens"], 8)
    assert np.abs(got - 8.0).max() <= 2 ** -5  # one bf16 ulp at 8.0 is 2^-4... round-to-nearest gives half


# ------------------------------------------------------------------ fp8 cache
def test_fp8_decode_parity():
    case = wl.decode_case(14, 2, 64, 8, 128, 700, sigma=0.5)
    check(case, 64, 8, 128, fp8=True, label="fp8")


def test_fp8_subnormal_codes_survive():
    """Values far below the head's amax land in e4m3 subnormals; they must not be flushed."""
    case = wl.decode_case(15, 1, 8, 1, 128, 128, sigma=0.5)
    case["v"] *= 2.0 ** -15     # most of V quantizes to subnormal codes ...
    case["v"][0, 0, 0, 0] = 1.0  # ... because one element pins the scale
    case["k"] *= 2.0 ** -15
    case["k"][0, 0, 0, 0] = 1.0
    c = build_cache(case, 1, 128, fp8=True)
    kc, vc, ks, vs = c.canonical(128)
    assert ((vc & 0x78) == 0).mean() > 0.5  # exponent field zero = subnormal
    got = run_decode(c, case["q_bits"], case["seq_lens"], 8)
    want = oracle.decode_attn(oracle.bf16_to_f32(case["q_bits"]), kc, vc, ks, vs, oracle.FMT_FP8, case["seq_lens"],
                              1.0 / np.sqrt(128))
    scale = np.abs(want).max()
    print("fp8 subnormal: |want| max %.3e err %.3e" % (scale, np.abs(got - want).max()), flush=True)
    assert np.abs(got - want).max() < 0.02 * scale  # flushing subnormals to zero would lose most of the output


# ------------------------------------------------------------------ fused step and phases
def test_decode_step_equals_write_then_attend_and_oracle():
    """hs_decode_step = quantize-on-write of one new token per row at seq_len-1, then attention."""
    B, Hq, Hkv, D, T = 5, 32, 8, 128, 700
    case = wl.decode_case(16, B, Hq, Hkv, D, T, ragged=True, outliers=True)
    case["seq_lens"][0] = 0  # an empty row: nothing written, zero output
    r = wl.philox(17)
    new_k = wl.bf16_bits_to_f32(wl.to_bf16_bits(r.standard_normal((B, 1, Hkv, D)).astype(np.float32)))
    new_v = wl.bf16_bits_to_f32(wl.to_bf16_bits(r.standard_normal((B, 1, Hkv, D)).astype(np.float32)))
    lens = case["seq_lens"]
    # reference flow: two calls
    c1 = build_cache(case, Hkv, D)
    pos = torch.from_numpy((lens - 1).astype(np.int32)).to(DEV)
    nk, nv = torch.from_numpy(new_k).to(DEV).bfloat16(), torch.from_numpy(new_v).to(DEV).bfloat16()
    c1.write(nk, nv, pos, 0)
    want_gpu = run_decode(c1, case["q_bits"], lens, Hq, max_seq_len=T)
    # fused flow
    c2 = build_cache(case, Hkv, D)
    q = bf16_from_bits(case["q_bits"]).to(DEV)
    out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    hb.decode_step(q, nk, nv, c2.k_codes, c2.v_codes, c2.k_scales, c2.v_scales, c2.layout,
                   torch.from_numpy(lens).to(DEV), out, ws, Hkv, T, 1.0 / np.sqrt(D))
    torch.cuda.synchronize()
    same = [bool(torch.equal(x, y)) for x, y in ((c1.k_codes, c2.k_codes), (c1.v_codes, c2.v_codes),
                                                 (c1.k_scales, c2.k_scales), (c1.v_scales, c2.v_scales))]
    assert all(same), same
    got = out.float().cpu().numpy()
    assert np.array_equal(got, want_gpu)
    assert not got[0].any()
    # and against the oracle, with the new token's codes made by the oracle
    k, v = case["k"].copy(), case["v"].copy()
    for b in range(1, B):
        k[b, lens[b] - 1], v[b, lens[b] - 1] = new_k[b, 0], new_v[b, 0]
    wk, wks = oracle.quant_int8(k)
    wv, wvs = oracle.quant_int8(v)
    kc, vc, ks, vs = c2.canonical(T)
    for b in range(1, B):
        n = lens[b]
        assert np.array_equal(kc[b, :n], wk[b, :n]) and np.array_equal(ks[b, :n], wks[b, :n])
        assert np.array_equal(vc[b, :n], wv[b, :n]) and np.array_equal(vs[b, :n], wvs[b, :n])
    want = oracle.decode_attn(oracle.bf16_to_f32(case["q_bits"]), wk, wv, wks, wvs, oracle.FMT_INT8, lens,
                              1.0 / np.sqrt(D))
    d = np.abs(got - want)
    assert d.max() < TOL_MAX and d.mean() < TOL_MEAN


@pytest.mark.parametrize("shape", [(1, 4, 1, 9000), (3, 32, 8, 3000), (64, 32, 8, 300)])
def test_partials_plus_standalone_merge_equal_fused_call(shape):
    """phases 1 then 2 (split-K kernel, then the stand-alone merge) == phases 3 (last workgroup merges)."""
    B, Hq, Hkv, T = shape
    case = wl.decode_case(18, B, Hq, Hkv, 128, T, ragged=True)
    c = build_cache(case, Hkv, 128)
    fused = run_decode(c, case["q_bits"], case["seq_lens"], Hq, max_seq_len=T)
    again = run_decode(c, case["q_bits"], case["seq_lens"], Hq, max_seq_len=T)
    assert np.array_equal(fused, again)  # arrival counters are left clean: a second call gives the same bits
    q = bf16_from_bits(case["q_bits"]).to(DEV)
    lens = torch.from_numpy(case["seq_lens"]).to(DEV)
    out = torch.full((B, Hq, 128), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, 128, T), dtype=torch.uint8, device=DEV)
    for ph in (1, 2):
        hb.decode_attn(q, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, lens, out, ws, Hkv, T,
                       1.0 / np.sqrt(128), phases=ph)
    torch.cuda.synchronize()
    two = out.float().cpu().numpy()
    assert np.abs(two - fused).max() <= 2.0 ** -8 * max(1.0, np.abs(fused).max())  # same math, other summation order


# ------------------------------------------------------------------ head_dim 256 (16-token wavefront steps)
@pytest.mark.parametrize("lens", [[1], [15], [16], [17], [63, 64, 65], [1, 700, 64, 257, 5]])
def test_head_dim_256_ragged_lengths_and_step_boundaries(lens):
    B = len(lens)
    case = wl.decode_case(30, B, 16, 4, 256, max(lens), outliers=True)
    case["seq_lens"] = np.array(lens, np.int32)
    check(case, 16, 4, 256, cap=max(lens) + 3, label="d256-ragged%s" % lens)


@pytest.mark.parametrize("Hq,Hkv,T", [(16, 4, 3000), (4, 1, 9000), (32, 2, 500)])
def test_head_dim_256_split_and_group_sizes(Hq, Hkv, T):
    case = wl.decode_case(31, 2, Hq, Hkv, 256, T, ragged=True, outliers=True, min_len=T // 2)
    check(case, Hq, Hkv, 256, label="d256-%d/%d-%d" % (Hq, Hkv, T))


def test_head_dim_256_fp8():
    case = wl.decode_case(32, 2, 16, 4, 256, 700, sigma=0.5)
    check(case, 16, 4, 256, fp8=True, label="d256-fp8")


def test_head_dim_256_fused_step_equals_write_then_attend():
    B, Hq, Hkv, D, T = 4, 16, 4, 256, 600
    case = wl.decode_case(33, B, Hq, Hkv, D, T, ragged=True, outliers=True)
    r = wl.philox(34)
    nk = torch.from_numpy(r.standard_normal((B, 1, Hkv, D)).astype(np.float32)).to(DEV).bfloat16()
    nv = torch.from_numpy(r.standard_normal((B, 1, Hkv, D)).astype(np.float32)).to(DEV).bfloat16()
    lens = case["seq_lens"]
    c1 = build_cache(case, Hkv, D)
    c1.write(nk, nv, torch.from_numpy((lens - 1).astype(np.int32)).to(DEV), 0)
    want = run_decode(c1, case["q_bits"], lens, Hq, max_seq_len=T)
    c2 = build_cache(case, Hkv, D)
    out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    hb.decode_step(bf16_from_bits(case["q_bits"]).to(DEV), nk, nv, c2.k_codes, c2.v_codes, c2.k_scales, c2.v_scales,
                   c2.layout, torch.from_numpy(lens).to(DEV), out, ws, Hkv, T, 1.0 / np.sqrt(D))
    torch.cuda.synchronize()
    for name in ("k_codes", "v_codes", "k_scales", "v_scales"):
        assert torch.equal(getattr(c1, name), getattr(c2, name)), name
    assert np.array_equal(out.float().cpu().numpy(), want)
    kc, vc, ks, vs = c2.canonical(T)
    ref = oracle.decode_attn(oracle.bf16_to_f32(case["q_bits"]), kc, vc, ks, vs, oracle.FMT_INT8, lens, 1.0 / np.sqrt(D))
    d = np.abs(want - ref)
    assert d.max() < TOL_MAX and d.mean() < TOL_MEAN


def test_head_dim_256_paged_block_table():
    B, Hq, Hkv, D, T, BT = 2, 8, 2, 256, 200, 64
    case = wl.decode_case(35, B, Hq, Hkv, D, T, ragged=True)
    c = build_cache(case, Hkv, D)
    want = run_decode(c, case["q_bits"], case["seq_lens"], Hq)
    nblk = (T + BT - 1) // BT
    ids = wl.philox(36).permutation(2 * B * nblk + 3).astype(np.int32)
    kt, vt = ids[: B * nblk].reshape(B, nblk), ids[B * nblk: 2 * B * nblk].reshape(B, nblk)
    pk = torch.zeros(len(ids), Hkv, BT, D, dtype=torch.int8, device=DEV)
    ps = torch.zeros(len(ids), Hkv, BT, dtype=torch.float32, device=DEV)
    k_tab, v_tab = torch.from_numpy(kt).to(DEV), torch.from_numpy(vt).to(DEV)  # the layout holds their addresses: keep them alive
    lay = hb.paged_layout(Hkv, BT, D, k_tab, v_tab)
    hb.kv_quantize_int8(torch.from_numpy(case["k"]).to(DEV), torch.from_numpy(case["v"]).to(DEV), pk, pk, ps, ps, lay, None, 0)
    out = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    hb.decode_attn(bf16_from_bits(case["q_bits"]).to(DEV), pk, pk, ps, ps, lay, torch.from_numpy(case["seq_lens"]).to(DEV),
                   out, ws, Hkv, T, 1.0 / np.sqrt(D))
    torch.cuda.synchronize()
    assert np.array_equal(out.float().cpu().numpy(), want)


# ------------------------------------------------------------------ head_dim 64 (64-token wavefront steps)
@pytest.mark.parametrize("lens", [[1], [63], [64], [65], [255, 256, 257], [1, 700, 64, 513, 5]])
def test_head_dim_64_ragged_lengths_and_step_boundaries(lens):
    B = len(lens)
    case = wl.decode_case(40, B, 16, 4, 64, max(lens), outliers=True)
    case["seq_lens"] = np.array(lens, np.int32)
    check(case, 16, 4, 64, cap=max(lens) + 3, label="d64-ragged%s" % lens)


@pytest.mark.parametrize("Hq,Hkv,T", [(16, 4, 3000), (4, 1, 9000), (32, 2, 500), (5, 5, 300)])
def test_head_dim_64_split_and_group_sizes(Hq, Hkv, T):
    case = wl.decode_case(41, 2, Hq, Hkv, 64, T, ragged=True, outliers=True, min_len=T // 2)
    check(case, Hq, Hkv, 64, label="d64-%d/%d-%d" % (Hq, Hkv, T))


def test_head_dim_64_fp8():
    case = wl.decode_case(42, 2, 16, 4, 64, 700, sigma=0.5)
    check(case, 16, 4, 64, fp8=True, label="d64-fp8")


def test_head_dim_64_fused_step_equals_write_then_attend():
    B, Hq, Hkv, D, T = 4, 16, 4, 64, 600
    case = wl.decode_case(43, B, Hq, Hkv, D, T, ragged=True, outliers=True)
    r = wl.philox(44)
    nk = torch.from_numpy(r.standard_normal((B, 1, Hkv, D)).astype(np.float32)).to(DEV).bfloat16()
    nv = torch.from_numpy(r.standard_normal((B, 1, Hkv, D)).astype(np.float32)).to(DEV).bfloat16()
    lens = case["seq_lens"]
    c1 = build_cache(case, Hkv, D)
    c1.write(nk, nv, torch.from_numpy((lens - 1).astype(np.int32)).to(DEV), 0)
    want = run_decode(c1, case["q_bits"], lens, Hq, max_seq_len=T)
    c2 = build_cache(case, Hkv, D)
    out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    hb.decode_step(bf16_from_bits(case["q_bits"]).to(DEV), nk, nv, c2.k_codes, c2.v_codes, c2.k_scales, c2.v_scales,
                   c2.layout, torch.from_numpy(lens).to(DEV), out, ws, Hkv, T, 1.0 / np.sqrt(D))
    torch.cuda.synchronize()
    for name in ("k_codes", "v_codes", "k_scales", "v_scales"):
        assert torch.equal(getattr(c1, name), getattr(c2, name)), name
    assert np.array_equal(out.float().cpu().numpy(), want)
    kc, vc, ks, vs = c2.canonical(T)
    ref = oracle.decode_attn(oracle.bf16_to_f32(case["q_bits"]), kc, vc, ks, vs, oracle.FMT_INT8, lens, 1.0 / np.sqrt(D))
    d = np.abs(want - ref)
    assert d.max() < TOL_MAX and d.mean() < TOL_MEAN


def test_head_dim_64_paged_block_table():
    B, Hq, Hkv, D, T, BT = 2, 8, 2, 64, 300, 64
    case = wl.decode_case(45, B, Hq, Hkv, D, T, ragged=True)
    c = build_cache(case, Hkv, D)
    want = run_decode(c, case["q_bits"], case["seq_lens"], Hq)
    nblk = (T + BT - 1) // BT
    ids = wl.philox(46).permutation(2 * B * nblk + 3).astype(np.int32)
    kt, vt = ids[: B * nblk].reshape(B, nblk), ids[B * nblk: 2 * B * nblk].reshape(B, nblk)
    pk = torch.zeros(len(ids), Hkv, BT, D, dtype=torch.int8, device=DEV)
    ps = torch.zeros(len(ids), Hkv, BT, dtype=torch.float32, device=DEV)
    k_tab, v_tab = torch.from_numpy(kt).to(DEV), torch.from_numpy(vt).to(DEV)  # the layout holds their addresses: keep them alive
    lay = hb.paged_layout(Hkv, BT, D, k_tab, v_tab)
    hb.kv_quantize_int8(torch.from_numpy(case["k"]).to(DEV), torch.from_numpy(case["v"]).to(DEV), pk, pk, ps, ps, lay, None, 0)
    out = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    hb.decode_attn(bf16_from_bits(case["q_bits"]).to(DEV), pk, pk, ps, ps, lay, torch.from_numpy(case["seq_lens"]).to(DEV),
                   out, ws, Hkv, T, 1.0 / np.sqrt(D))
    torch.cuda.synchronize()
    assert np.array_equal(out.float().cpu().numpy(), want)
    lay32 = hb.paged_layout(Hkv, 32, D, k_tab, v_tab)  # a 64-token wavefront step would straddle two 32-token blocks
    with pytest.raises(hb.HsError, match="multiple of 64"):
        hb.decode_attn(bf16_from_bits(case["q_bits"]).to(DEV), pk, pk, ps, ps, lay32, torch.from_numpy(case["seq_lens"]).to(DEV),
                       out, ws, Hkv, 32, 1.0 / np.sqrt(D))


def test_unsupported_head_dim_is_rejected():
    c = DeviceCache(1, 2, 64, 192)
    q = torch.zeros(1, 4, 192, dtype=torch.bfloat16, device=DEV)
    out = torch.empty_like(q)
    ws = torch.empty(1 << 16, dtype=torch.uint8, device=DEV)
    with pytest.raises(hb.HsError) as e:
        hb.decode_attn(q, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, torch.tensor([64], dtype=torch.int32, device=DEV),
                       out, ws, 2, 64, 0.125)
    assert e.value.code == hb.HS_ERR_INVALID_ARGUMENT and "head_dim" in str(e.value)


@pytest.mark.parametrize("seed", range(10))
def test_random_shapes(seed):
    """Seeded random batch sizes, head groupings, head_dim, lengths and cache formats against the oracle."""
    r = np.random.default_rng(1000 + seed)
    B = int(r.integers(1, 6))
    Hkv = int(r.choice([1, 2, 3, 4, 8]))
    G = int(r.choice([1, 2, 4, 5, 8, 16]))
    D = int(r.choice([64, 128, 256]))
    T = int(r.integers(1, 1400))
    fp8 = bool(r.integers(0, 2))
    case = wl.decode_case(200 + seed, B, Hkv * G, Hkv, D, T, ragged=True, outliers=not fp8, sigma=0.5 if fp8 else 1.0)
    if seed % 3 == 0:
        case["seq_lens"][0] = 0  # an empty row
    got, _ = check(case, Hkv * G, Hkv, D, fp8=fp8, cap=T + int(r.integers(0, 70)),
                   label="random B=%d Hkv=%d G=%d D=%d T=%d fp8=%s" % (B, Hkv, G, D, T, fp8))
    if seed % 3 == 0:
        assert not got[0].any()
