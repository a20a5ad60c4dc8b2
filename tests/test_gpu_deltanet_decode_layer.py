"""hs_deltanet_decode_layer: the decode branch of a gated-DeltaNet layer between its projections in one launch, against
(a) the three calls it replaces -- hs_deltanet_prepare, hs_deltanet_forward (T = 1), hs_deltanet_gated_norm -- bit for
bit, over several steps with the conv state and the recurrent state carried, and (b) the reference's libtorch op
sequence (GatedDeltaNetLayer::forward, qwen3_5.rs:617-786: conv1d + SiLU + gates, the decode-step recurrence
:725-751, RMSNormGated :292-313)."""
import numpy as np
import pytest
import torch

from oracle import reference_path as ref
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _inputs(seed, B, steps, nk, nv, dk, dv):
    r = wl.philox(seed)
    C = 2 * nk * dk + nv * dv
    t = lambda *s, scale=1.0: torch.from_numpy((r.standard_normal(s) * scale).astype(np.float32))
    return dict(x=t(B, steps, C).to(torch.bfloat16), w=t(C, 4, scale=0.5).to(torch.bfloat16), st=t(B, C, 3).to(torch.bfloat16),
                a=t(B, steps, nv, scale=2).to(torch.bfloat16), b=t(B, steps, nv, scale=2).to(torch.bfloat16),
                nae=-t(nv).exp(), dtb=t(nv), z=t(B, steps, nv, dv).to(torch.bfloat16), nw=t(dv),
                s0=t(B, nv, dk, dv, scale=0.3))


def _three_calls(d, t, conv_state, state, nk, nv, dk, dv, l2norm):
    """The unfused decode step of the layer; `state` is updated in place.  Returns (out bf16, new conv state)."""
    sl = slice(t, t + 1)
    q, k, v, g, beta, cs = hb.deltanet_prepare(d["x"][:, sl].contiguous(), d["w"], conv_state, d["a"][:, sl].contiguous(),
                                               d["b"][:, sl].contiguous(), d["nae"], d["dtb"], nk, nv, dk, dv)
    o = torch.empty(q.shape[0], 1, nv, dv, device=DEV)
    hb.deltanet_forward(q, k, v, g, beta, state, o, 1.0 / np.sqrt(dk), l2norm)
    return hb.deltanet_gated_norm(o, d["z"][:, sl].contiguous(), d["nw"], 1e-6), cs


@pytest.mark.parametrize("B,nk,nv,l2norm,first_state", [(3, 2, 4, True, True), (2, 1, 1, True, False), (1, 2, 6, False, True),
                                                         (5, 4, 4, True, True)])
def test_equals_the_three_calls_bit_for_bit(B, nk, nv, l2norm, first_state):
    dk = dv = 128
    steps = 4
    p = _inputs(7100 + B, B, steps, nk, nv, dk, dv)
    d = {k_: v_.to(DEV) for k_, v_ in p.items()}
    cs_a = d["st"] if first_state else None
    cs_b = cs_a
    state_a, state_b = d["s0"].clone(), d["s0"].clone()
    for t in range(steps):
        sl = slice(t, t + 1)
        want, cs_a = _three_calls(d, t, cs_a, state_a, nk, nv, dk, dv, l2norm)
        got, cs_b = hb.deltanet_decode_layer(d["x"][:, sl].contiguous(), d["w"], cs_b, d["a"][:, sl].contiguous(),
                                             d["b"][:, sl].contiguous(), d["nae"], d["dtb"], d["z"][:, sl].contiguous(),
                                             d["nw"], 1e-6, state_b, nk, nv, dk, dv, 1.0 / np.sqrt(dk), l2norm)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), "output row, step %d" % t
        assert torch.equal(cs_b.view(torch.int16), cs_a.view(torch.int16)), "conv state, step %d" % t
        assert torch.equal(state_b, state_a), "recurrent state, step %d" % t


def test_matches_the_reference_op_sequence():
    B, nk, nv, dk, dv, steps = 2, 2, 4, 128, 128, 6
    p = _inputs(7200, B, steps, nk, nv, dk, dv)
    d = {k_: v_.to(DEV) for k_, v_ in p.items()}
    state = torch.zeros(B, nv, dk, dv, device=DEV)
    cs = d["st"]
    ys = []
    for t in range(steps):
        sl = slice(t, t + 1)
        y, cs = hb.deltanet_decode_layer(d["x"][:, sl].contiguous(), d["w"], cs, d["a"][:, sl].contiguous(),
                                         d["b"][:, sl].contiguous(), d["nae"], d["dtb"], d["z"][:, sl].contiguous(), d["nw"],
                                         1e-6, state, nk, nv, dk, dv, 1.0 / np.sqrt(dk), True)
        ys.append(y)
    torch.cuda.synchronize()
    y = torch.cat(ys, 1)
    # the reference's ops over the same six tokens (the conv over the whole run equals its step-by-step form)
    conv, ref_cs, rg, rb = ref.deltanet_prepare(p["x"], p["w"].unsqueeze(1), p["st"], p["a"], p["b"], p["nae"], p["dtb"])
    kd = nk * dk
    l2 = lambda t_: t_ / t_.norm(dim=-1, keepdim=True).clamp_min(1e-3)
    rq = l2(conv[..., :kd].reshape(B, steps, nk, dk).float()) * (1.0 / np.sqrt(dk))
    rk = l2(conv[..., kd:2 * kd].reshape(B, steps, nk, dk).float())
    rv = conv[..., 2 * kd:].reshape(B, steps, nv, dv).float()
    rq, rk = rq.repeat_interleave(nv // nk, 2), rk.repeat_interleave(nv // nk, 2)
    st = torch.zeros(B, nv, dk, dv)
    outs = []
    for t in range(steps):
        ot, st = ref.deltanet_decode_step(rq[:, t], rk[:, t], rv[:, t], rg[:, t], rb[:, t], st)
        outs.append(ot)
    want = ref.gated_rmsnorm(torch.stack(outs, 1), p["z"], p["nw"], 1e-6)
    err = (y.float().cpu() - want.float()).abs()
    # as in the unfused layer test: a couple of bf16 ulps where the SiLU ulp differs, one ulp of the value itself
    assert (err - 2.0 ** -7 * want.float().abs()).max() < 3e-2 and err.mean() < 2e-3
    assert (state.cpu() - st).abs().max() < 1e-3
    assert torch.equal(cs.cpu().view(torch.int16), ref_cs.contiguous().view(torch.int16))


def test_rejects_bad_arguments():
    L = hb.lib()
    p = hb._ptr
    x = torch.zeros(1, 1, 384, dtype=torch.bfloat16, device=DEV)
    st = torch.zeros(1, 384, 3, dtype=torch.bfloat16, device=DEV)
    f = torch.zeros(128 * 128, device=DEV)
    import ctypes
    args = lambda cs_in, cs_out, dk: (p(x), p(x), cs_in, cs_out, p(x), p(x), p(f), p(f), p(x), p(f), ctypes.c_float(1e-6),
                                     p(f), p(x), 1, 1, 1, dk, 128, ctypes.c_float(1.0), 1, None)
    assert L.hs_deltanet_decode_layer(*args(p(st), p(st), 128)) == hb.HS_ERR_INVALID_ARGUMENT and b"alias" in L.hs_attn_last_error()
    assert L.hs_deltanet_decode_layer(*args(None, p(st), 64)) == hb.HS_ERR_INVALID_ARGUMENT and b"128" in L.hs_attn_last_error()
    assert L.hs_deltanet_decode_layer(*args(None, None, 128)) == hb.HS_ERR_INVALID_ARGUMENT
