"""hs_deltanet_forward_chunked_gated_norm: the chunk-64 delta rule followed by the layer's gated RMSNorm, one call
(chunked_delta_rule qwen3_5.rs:342-498 + RMSNormGated :305-313), against the two calls it stands for
(hs_deltanet_forward_chunked + hs_deltanet_gated_norm: state and rows bit for bit) and against the CPU oracle (fp64
recurrence, then the norm)."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from oracle import hs_oracle as orc
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV, bf16_from_bits

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _ulps(a_bits, b_bits):
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7fff), u & 0x7fff)
    return np.abs(key(a_bits) - key(b_bits))


def _case(seed, B, T, nk, nv):
    case = wl.deltanet_case(seed, B, T, nk, nv, 128, 128)
    r = wl.philox(seed + 1)
    z = torch.from_numpy(r.standard_normal((B, T, nv, 128)).astype(np.float32)).to(torch.bfloat16)
    w = torch.from_numpy((1.0 + 0.2 * r.standard_normal(128)).astype(np.float32))
    s0 = (r.standard_normal((B, nv, 128, 128)) * 0.2).astype(np.float32)
    return case, z, w, s0


def _both(case, z, w, s0, l2norm=True):
    q, k, v = (bf16_from_bits(case[n]).to(DEV) for n in ("q_bits", "k_bits", "v_bits"))
    g, beta = torch.from_numpy(case["g"]).to(DEV), torch.from_numpy(case["beta"]).to(DEV)
    B, T, nv = case["g"].shape
    qs = 1.0 / np.sqrt(128.0)
    st_a, st_b = torch.from_numpy(s0).to(DEV).clone(), torch.from_numpy(s0).to(DEV).clone()
    o32 = torch.empty(B, T, nv, 128, dtype=torch.float32, device=DEV)
    hb.deltanet_forward_chunked(q, k, v, g, beta, st_a, o32, qs, l2norm)
    want = hb.deltanet_gated_norm(o32, z.to(DEV), w.to(DEV), 1e-6)
    got = torch.full((B, T, nv, 128), float("nan"), dtype=torch.bfloat16, device=DEV)
    hb.deltanet_forward_chunked_gated_norm(q, k, v, g, beta, st_b, z.to(DEV), w.to(DEV), 1e-6, got, qs, l2norm)
    torch.cuda.synchronize()
    return got, want, st_b, st_a, o32


@pytest.mark.parametrize("B,T,nk,nv", [(2, 64, 2, 4), (1, 1, 1, 1), (2, 150, 2, 4), (4, 300, 2, 4), (3, 200, 1, 2), (1, 520, 4, 8)])
def test_equals_the_two_calls(B, T, nk, nv):
    case, z, w, s0 = _case(9100 + T, B, T, nk, nv)
    got, want, st_b, st_a, _ = _both(case, z, w, s0)
    assert torch.isfinite(got.float()).all()
    assert torch.equal(st_b, st_a)
    assert _ulps(_bits(got), _bits(want)).max() == 0


def test_more_workgroups_than_the_device_holds_at_once():
    B, T, nk, nv = 70, 70, 2, 2  # 280 workgroups of the walk; the device holds 256 at a time
    case, z, w, s0 = _case(9200, B, T, nk, nv)
    got, want, st_b, st_a, _ = _both(case, z, w, s0)
    assert torch.equal(st_b, st_a)
    assert _ulps(_bits(got), _bits(want)).max() == 0


def test_workspace_of_the_norm_variant_is_checked():
    case, z, w, s0 = _case(9250, 1, 70, 1, 2)
    q, k, v = (bf16_from_bits(case[n]).to(DEV) for n in ("q_bits", "k_bits", "v_bits"))
    g, beta = torch.from_numpy(case["g"]).to(DEV), torch.from_numpy(case["beta"]).to(DEV)
    need = hb.deltanet_chunked_gated_norm_workspace_bytes(1, 70, 1, 2)
    assert need == 2 * 2 * 13312 + 70 * 2 * 128 * 4
    out = torch.empty(1, 70, 2, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(hb.HsError) as e:  # the plain call's workspace is too small for this one
        hb.deltanet_forward_chunked_gated_norm(q, k, v, g, beta, torch.from_numpy(s0).to(DEV), z.to(DEV), w.to(DEV), 1e-6, out,
                                               1.0, True, workspace=torch.empty(need - 1, dtype=torch.uint8, device=DEV))
    assert e.value.code == hb.HS_ERR_WORKSPACE
    torch.cuda.synchronize()


def test_against_the_oracle():
    B, T, nk, nv = 2, 130, 2, 4
    case, z, w, s0 = _case(9300, B, T, nk, nv)
    got, _, st_b, _, _ = _both(case, z, w, s0)
    f = wl.bf16_bits_to_f32
    wo, ws = oracle.deltanet_recurrent(f(case["q_bits"]), f(case["k_bits"]), f(case["v_bits"]), case["g"], case["beta"], s0,
                                       1 / np.sqrt(128.0), True)
    want_bits = orc.gated_rmsnorm(wo.astype(np.float32).reshape(-1, 128), _bits(z).reshape(-1, 128), w.numpy(), 1e-6)
    want = wl.bf16_bits_to_f32(want_bits).reshape(B, T, nv, 128)
    err = np.abs(got.float().cpu().numpy() - want)
    # the rows are O(1) after the norm; the chunked form's 1e-3 relative error in o carries over, plus bf16 rounding
    assert (err - 2.0 ** -7 * np.abs(want)).max() < 2e-2 and err.mean() < 2e-3
    assert np.abs(st_b.cpu().numpy() - ws).max() <= 3e-3 * np.abs(ws).max()


def test_prefill_layer_is_prepare_plus_the_chunked_call_and_carries_state_across_calls():
    """hs_deltanet_prefill_layer (one call for the prompt branch of the layer) against hs_deltanet_prepare +
    hs_deltanet_forward_chunked_gated_norm, bit for bit, for a prompt given in two calls of 128 and 70 tokens with the
    conv state and the recurrent state carried; and against the reference's op sequence for the whole run."""
    from oracle import reference_path as ref
    B, nk, nv, dk, dv, S = 2, 2, 4, 128, 128, 198
    r = wl.philox(9400)
    C = 2 * nk * dk + nv * dv
    t = lambda *s, scale=1.0: torch.from_numpy((r.standard_normal(s) * scale).astype(np.float32))
    p = dict(x=t(B, S, C).to(torch.bfloat16), w=t(C, 4, scale=0.5).to(torch.bfloat16), st=t(B, C, 3).to(torch.bfloat16),
             a=t(B, S, nv, scale=2).to(torch.bfloat16), b=t(B, S, nv, scale=2).to(torch.bfloat16), nae=-t(nv).exp(), dtb=t(nv),
             z=t(B, S, nv, dv).to(torch.bfloat16), nw=t(dv))
    d = {k_: v_.to(DEV) for k_, v_ in p.items()}
    qs = 1.0 / np.sqrt(dk)
    state_a, state_b = torch.zeros(B, nv, dk, dv, device=DEV), torch.zeros(B, nv, dk, dv, device=DEV)
    cs_a = cs_b = d["st"]
    outs_a, outs_b = [], []
    for lo, hi in ((0, 128), (128, S)):
        sl = slice(lo, hi)
        x, a_in, b_in, z = (d[n][:, sl].contiguous() for n in ("x", "a", "b", "z"))
        y, cs_a, _ = hb.deltanet_prefill_layer(x, d["w"], cs_a, a_in, b_in, d["nae"], d["dtb"], z, d["nw"], 1e-6, state_a,
                                               nk, nv, dk, dv, qs, True)
        outs_a.append(y)
        q, k, v, g, beta, cs_b = hb.deltanet_prepare(x, d["w"], cs_b, a_in, b_in, d["nae"], d["dtb"], nk, nv, dk, dv)
        y2 = torch.empty(B, hi - lo, nv, dv, dtype=torch.bfloat16, device=DEV)
        hb.deltanet_forward_chunked_gated_norm(q, k, v, g, beta, state_b, z, d["nw"], 1e-6, y2, qs, True)
        outs_b.append(y2)
    torch.cuda.synchronize()
    ya, yb = torch.cat(outs_a, 1), torch.cat(outs_b, 1)
    assert torch.equal(ya.view(torch.int16), yb.view(torch.int16)) and torch.equal(state_a, state_b)
    assert torch.equal(cs_a.view(torch.int16), cs_b.view(torch.int16))
    # the reference's ops over the whole run (GatedDeltaNetLayer::forward, qwen3_5.rs:629-786, recurrence iterated)
    conv, ref_cs, rg, rb = ref.deltanet_prepare(p["x"], p["w"].unsqueeze(1), p["st"], p["a"], p["b"], p["nae"], p["dtb"])
    kd = nk * dk
    l2 = lambda t_: t_ / t_.norm(dim=-1, keepdim=True).clamp_min(1e-3)
    rq = l2(conv[..., :kd].reshape(B, S, nk, dk).float()) * qs
    rk = l2(conv[..., kd:2 * kd].reshape(B, S, nk, dk).float())
    rv = conv[..., 2 * kd:].reshape(B, S, nv, dv).float()
    rq, rk = rq.repeat_interleave(nv // nk, 2), rk.repeat_interleave(nv // nk, 2)
    st = torch.zeros(B, nv, dk, dv)
    rows = []
    for i in range(S):
        ot, st = ref.deltanet_decode_step(rq[:, i], rk[:, i], rv[:, i], rg[:, i], rb[:, i], st)
        rows.append(ot)
    want = ref.gated_rmsnorm(torch.stack(rows, 1), p["z"], p["nw"], 1e-6)
    err = (ya.float().cpu() - want.float()).abs()
    assert (err - 2.0 ** -7 * want.float().abs()).max() < 3e-2 and err.mean() < 2e-3
    assert (state_a.cpu() - st).abs().max() < 3e-3 * float(st.abs().max())
    assert torch.equal(cs_a.cpu().view(torch.int16), ref_cs.contiguous().view(torch.int16))


def test_prefill_layer_workspace_is_checked():
    L = hb.lib()
    L.hs_deltanet_prefill_layer_workspace_bytes.restype = ctypes.c_size_t
    need = L.hs_deltanet_prefill_layer_workspace_bytes(1, 64, 1, 1, 128, 128)
    assert need >= hb.deltanet_chunked_gated_norm_workspace_bytes(1, 64, 1, 1) + 64 * (3 * 128 * 2 + 2 * 4) and need % 256 == 0
    x = torch.zeros(1, 64, 384, dtype=torch.bfloat16, device=DEV)
    f = torch.zeros(128 * 128, device=DEV)
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    p = hb._ptr
    st = torch.zeros(1, 384, 3, dtype=torch.bfloat16, device=DEV)
    rc = L.hs_deltanet_prefill_layer(p(x), p(x), None, p(st), p(x), p(x), p(f), p(f), p(x), p(f), ctypes.c_float(1e-6), p(f), p(x),
                                     1, 64, 1, 1, 128, 128, ctypes.c_float(1.0), 1, p(ws), ctypes.c_size_t(need - 1), None)
    assert rc == hb.HS_ERR_WORKSPACE
