"""GPU parity of the chunk-64 gated delta rule on the matrix pipe (hs_deltanet_forward_chunked) against the fp64
oracle of the token recurrence, which the chunked form regroups (chunked_delta_rule, qwen3_5.rs:342-498).

Operands are fp16 with fp32 accumulation, so the bar is relative: 3e-3 of the largest output / state magnitude
(measured: below 1e-3), far inside max-abs 2e-2 / mean-abs 2e-3 on outputs of order 0.1."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV, bf16_from_bits

pytestmark = pytest.mark.gpu
REL = 3e-3


def _dev(case):
    q, k, v = (bf16_from_bits(case[n]).to(DEV) for n in ("q_bits", "k_bits", "v_bits"))
    return q, k, v, torch.from_numpy(case["g"]).to(DEV), torch.from_numpy(case["beta"]).to(DEV)


def run(case, state0, q_scale, l2norm, cuts=()):
    q, k, v, g, beta = _dev(case)
    B, T, nv = case["g"].shape
    st = torch.from_numpy(state0).to(DEV).clone()
    out = torch.full((B, T, nv, 128), float("nan"), dtype=torch.float32, device=DEV)
    lo = 0
    for hi in list(cuts) + [T]:
        o = torch.full((B, hi - lo, nv, 128), float("nan"), dtype=torch.float32, device=DEV)
        hb.deltanet_forward_chunked(q[:, lo:hi].contiguous(), k[:, lo:hi].contiguous(), v[:, lo:hi].contiguous(),
                                    g[:, lo:hi].contiguous(), beta[:, lo:hi].contiguous(), st, o, q_scale, l2norm)
        out[:, lo:hi] = o
        lo = hi
    torch.cuda.synchronize()
    return out.cpu().numpy(), st.cpu().numpy()


def want(case, state0, q_scale, l2norm):
    f = wl.bf16_bits_to_f32
    return oracle.deltanet_recurrent(f(case["q_bits"]), f(case["k_bits"]), f(case["v_bits"]), case["g"], case["beta"],
                                     state0, q_scale, l2norm)


def check(o, s, wo, ws, label):
    eo, es = np.abs(o - wo).max(), np.abs(s - ws).max()
    print("%s: out err %.2e of %.2e, state err %.2e of %.2e" % (label, eo, np.abs(wo).max(), es, np.abs(ws).max()), flush=True)
    assert np.isfinite(o).all() and np.isfinite(s).all(), label
    assert eo <= REL * np.abs(wo).max() and es <= REL * np.abs(ws).max(), label
    assert eo < 2e-2 and np.abs(o - wo).mean() < 2e-3, label


@pytest.mark.parametrize("T", [1, 2, 63, 64, 65, 128, 300])
@pytest.mark.parametrize("l2norm", [True, False])
def test_chunked_matches_the_recurrence(T, l2norm):
    B, nk, nv = 2, 2, 4
    case = wl.deltanet_case(60 + T, B, T, nk, nv, 128, 128)
    s0 = (wl.philox(61 + T).standard_normal((B, nv, 128, 128)) * 0.2).astype(np.float32)
    o, s = run(case, s0, 1 / np.sqrt(128.0), l2norm)
    wo, ws = want(case, s0, 1 / np.sqrt(128.0), l2norm)
    check(o, s, wo, ws, "T=%d l2norm=%s" % (T, l2norm))


@pytest.mark.parametrize("gscale", [0.0, 0.02, 3.0])
def test_slow_and_fast_decay(gscale):
    """g = 0 keeps everything (the state grows over the whole prompt); a large |g| forgets within a few tokens
    and drives the in-chunk decay factors to the fp16 underflow range."""
    B, T, nk, nv = 1, 1024, 1, 2
    case = wl.deltanet_case(70, B, T, nk, nv, 128, 128)
    case["g"] = (case["g"] * gscale).astype(np.float32)
    s0 = np.zeros((B, nv, 128, 128), np.float32)
    o, s = run(case, s0, 1 / np.sqrt(128.0), True)
    wo, ws = want(case, s0, 1 / np.sqrt(128.0), True)
    check(o, s, wo, ws, "gscale=%g" % gscale)


def test_config5_head_shape_reduced():
    """nk 16 / nv 32 (two v-heads per k-head) at B = 1, T = 200."""
    case = wl.deltanet_case(71, 1, 200, 16, 32, 128, 128)
    s0 = np.zeros((1, 32, 128, 128), np.float32)
    o, s = run(case, s0, 1 / np.sqrt(128.0), True)
    wo, ws = want(case, s0, 1 / np.sqrt(128.0), True)
    check(o, s, wo, ws, "config5 heads")


def test_calls_cut_at_chunk_multiples_give_the_bits_of_one_call():
    B, T, nk, nv = 1, 300, 1, 2
    case = wl.deltanet_case(72, B, T, nk, nv, 128, 128)
    s0 = (wl.philox(73).standard_normal((B, nv, 128, 128)) * 0.2).astype(np.float32)
    whole = run(case, s0, 0.5, True)
    parts = run(case, s0, 0.5, True, cuts=(64, 256))
    assert np.array_equal(whole[0], parts[0]) and np.array_equal(whole[1], parts[1])
    # any other cut is the same function up to rounding
    odd = run(case, s0, 0.5, True, cuts=(10, 111))
    wo, ws = want(case, s0, 0.5, True)
    check(odd[0], odd[1], wo, ws, "odd cuts")


def test_chunked_agrees_with_the_recurrent_kernel():
    B, T, nk, nv = 2, 130, 2, 4
    case = wl.deltanet_case(74, B, T, nk, nv, 128, 128)
    s0 = (wl.philox(75).standard_normal((B, nv, 128, 128)) * 0.2).astype(np.float32)
    o, s = run(case, s0, 1 / np.sqrt(128.0), True)
    q, k, v, g, beta = _dev(case)
    st = torch.from_numpy(s0).to(DEV)
    out = torch.empty(B, T, nv, 128, dtype=torch.float32, device=DEV)
    hb.deltanet_forward(q, k, v, g, beta, st, out, 1 / np.sqrt(128.0), True)
    torch.cuda.synchronize()
    check(o, s, out.cpu().numpy(), st.cpu().numpy(), "against the recurrent kernel")


def test_workspace_and_shape_errors():
    case = wl.deltanet_case(76, 1, 70, 1, 2, 128, 128)
    q, k, v, g, beta = _dev(case)
    st = torch.zeros(1, 2, 128, 128, device=DEV)
    out = torch.empty(1, 70, 2, 128, device=DEV)
    need = hb.deltanet_chunked_workspace_bytes(1, 70, 1, 2)
    assert need == 2 * 2 * 13312  # per chunk and v-head: the two triangular factors and three vectors
    small = torch.empty(need - 1, dtype=torch.uint8, device=DEV)
    with pytest.raises(hb.HsError) as e:
        hb.deltanet_forward_chunked(q, k, v, g, beta, st, out, 1.0, True, workspace=small)
    assert e.value.code == hb.HS_ERR_WORKSPACE
    with pytest.raises(hb.HsError) as e:  # nv must be a multiple of nk
        hb.deltanet_forward_chunked(q.repeat(1, 1, 3, 1), k.repeat(1, 1, 3, 1), v, g, beta, st, out, 1.0, True)
    assert e.value.code == hb.HS_ERR_INVALID_ARGUMENT
    flat = torch.empty(out.numel() + 4, device=DEV)  # the rows leave in 16-byte stores: out must be aligned like q, k, v
    with pytest.raises(hb.HsError) as e:
        hb.deltanet_forward_chunked(q, k, v, g, beta, st, flat[1:1 + out.numel()].view(out.shape), 1.0, True)
    assert e.value.code == hb.HS_ERR_INVALID_ARGUMENT and "aligned" in str(e.value)
    torch.cuda.synchronize()


def test_against_the_numpy_restatement_of_the_reference_chunked_form():
    """oracle/deltanet_chunked.py follows chunked_delta_rule (qwen3_5.rs:342-498) statement by statement."""
    from oracle import deltanet_chunked as dc
    B, T, nk, nv = 1, 200, 2, 4
    case = wl.deltanet_case(77, B, T, nk, nv, 128, 128)
    s0 = (wl.philox(78).standard_normal((B, nv, 128, 128)) * 0.2).astype(np.float32)
    o, s = run(case, s0, 1 / np.sqrt(128.0), True)
    f = wl.bf16_bits_to_f32
    rep = nv // nk
    qn = dc.l2_normalize(f(case["q_bits"])) / np.sqrt(128.0)
    kn = dc.l2_normalize(f(case["k_bits"]))
    hm = lambda x: np.repeat(x, rep, axis=2).transpose(0, 2, 1, 3)  # [B,T,nk,d] -> [B,nv,T,d]
    wo, ws = dc.chunked_delta_rule(hm(qn), hm(kn), f(case["v_bits"]).transpose(0, 2, 1, 3), case["g"].transpose(0, 2, 1),
                                   case["beta"].transpose(0, 2, 1), s0, dtype=np.float64)
    check(o, s, np.asarray(wo, np.float32).transpose(0, 2, 1, 3), np.asarray(ws, np.float32), "numpy chunked form")


@pytest.mark.parametrize("B,nk,nv", [(3, 2, 2), (3, 1, 4), (3, 3, 3), (8, 1, 4), (2, 1, 4), (4, 2, 8),
                                     (40, 2, 4), (17, 1, 4), (24, 4, 4)])
def test_head_groupings(B, nk, nv):
    """One, several or all v-heads per k-head; the three ways the walk places its workgroups on the XCDs (B * nk a
    multiple of 8: the workgroups of a k-head together; B * nv a multiple of 8: the parts of a v-head together; otherwise
    in grid order); and both widths of its workgroups (32 state columns while 4 B nv workgroups fit the device in one
    round -- the first six cases --, 64 columns beyond)."""
    T = 130 if B < 10 else 70
    case = wl.deltanet_case(80 + nk + nv, B, T, nk, nv, 128, 128)
    s0 = (wl.philox(81).standard_normal((B, nv, 128, 128)) * 0.2).astype(np.float32)
    o, s = run(case, s0, 1 / np.sqrt(128.0), True)
    wo, ws = want(case, s0, 1 / np.sqrt(128.0), True)
    check(o, s, wo, ws, "B=%d nk=%d nv=%d" % (B, nk, nv))


def test_both_workgroup_widths_give_the_same_bits():
    """The first two sequences of a batch of 40 (64-column workgroups) against the same two alone (32-column
    workgroups): a state column's sums do not depend on which wavefront owns it."""
    B, T, nk, nv = 40, 130, 2, 4
    case = wl.deltanet_case(90, B, T, nk, nv, 128, 128)
    s0 = (wl.philox(91).standard_normal((B, nv, 128, 128)) * 0.2).astype(np.float32)
    o, s = run(case, s0, 1 / np.sqrt(128.0), True)
    two = {n: np.ascontiguousarray(a[:2]) for n, a in case.items() if isinstance(a, np.ndarray) and a.shape[:1] == (B,)}
    o2, s2 = run(two, np.ascontiguousarray(s0[:2]), 1 / np.sqrt(128.0), True)
    assert np.array_equal(o[:2], o2) and np.array_equal(s[:2], s2)


def test_rows_below_the_norm_floor():
    """l2_normalize divides by max(|x|, 1e-3) (qwen3_5.rs:331-335): rows of k and q with a norm of about 1e-4 are scaled
    by 1e3 and stay small, all-zero rows stay zero (no 0 * inf)."""
    B, T, nk, nv = 1, 150, 2, 4
    case = wl.deltanet_case(92, B, T, nk, nv, 128, 128)
    f, tb = wl.bf16_bits_to_f32, wl.to_bf16_bits
    for name in ("k_bits", "q_bits"):
        x = f(case[name]).copy()
        x[:, 3::7] *= 2.0 ** -17  # exact in bf16
        x[:, 5::11] = 0.0
        case[name] = tb(x)
    s0 = (wl.philox(93).standard_normal((B, nv, 128, 128)) * 0.2).astype(np.float32)
    o, s = run(case, s0, 1 / np.sqrt(128.0), True)
    wo, ws = want(case, s0, 1 / np.sqrt(128.0), True)
    check(o, s, wo, ws, "rows below the norm floor")
