"""GPU parity of the steps around the delta rule (through the C ABI) against the oracle, and a whole
gated-DeltaNet layer core (prepare -> recurrence -> gated norm) against the reference's libtorch op sequence.

Reference: GatedDeltaNetLayer::forward, qwen3_5.rs:617-786; RMSNormGated :292-313."""
import numpy as np
import pytest
import torch

from oracle import hs_oracle as orc
from oracle import reference_path as ref
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _ulps(a_bits, b_bits):
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7fff), u & 0x7fff)
    return np.abs(key(a_bits) - key(b_bits))


def _layer_inputs(seed, B, S, nk, nv, dk, dv):
    r = wl.philox(seed)
    C = 2 * nk * dk + nv * dv
    t = lambda *s, scale=1.0: torch.from_numpy((r.standard_normal(s) * scale).astype(np.float32))
    return dict(x=t(B, S, C).to(torch.bfloat16), w=t(C, 4, scale=0.5).to(torch.bfloat16), st=t(B, C, 3).to(torch.bfloat16),
                a=t(B, S, nv, scale=2).to(torch.bfloat16), b=t(B, S, nv, scale=2).to(torch.bfloat16),
                nae=-t(nv).exp(), dtb=t(nv), z=t(B, S, nv, dv).to(torch.bfloat16), nw=t(dv))


@pytest.mark.parametrize("S", [1, 2, 5, 64, 65, 200])
def test_prepare_matches_oracle(S):
    B, nk, nv, dk, dv = 2, 2, 4, 128, 128
    p = _layer_inputs(1000 + S, B, S, nk, nv, dk, dv)
    q, k, v, g, beta, st = hb.deltanet_prepare(p["x"].to(DEV), p["w"].to(DEV), p["st"].to(DEV), p["a"].to(DEV), p["b"].to(DEV),
                                               p["nae"].to(DEV), p["dtb"].to(DEV), nk, nv, dk, dv)
    torch.cuda.synchronize()
    y, want_st = orc.deltanet_conv_silu_bf16(_bits(p["x"]), _bits(p["w"]), _bits(p["st"]))
    kd = nk * dk
    # expf on the device and in libm may differ in the last bit of the SiLU: one bf16 ulp
    assert _ulps(_bits(q).reshape(B, S, kd), y[..., :kd]).max() <= 1
    assert _ulps(_bits(k).reshape(B, S, kd), y[..., kd:2 * kd]).max() <= 1
    assert _ulps(_bits(v).reshape(B, S, nv * dv), y[..., 2 * kd:]).max() <= 1
    assert np.array_equal(_bits(st), want_st)
    wg, wb = orc.deltanet_gates(_bits(p["a"]), _bits(p["b"]), p["nae"].numpy(), p["dtb"].numpy())
    assert np.allclose(g.cpu().numpy(), wg, rtol=3e-6, atol=1e-30) and np.allclose(beta.cpu().numpy(), wb, rtol=3e-6)


def test_first_call_without_state_and_split_calls():
    B, S, nk, nv, dk, dv = 1, 70, 2, 2, 128, 128
    p = _layer_inputs(1100, B, S, nk, nv, dk, dv)
    d = {k_: v_.to(DEV) for k_, v_ in p.items()}
    whole = hb.deltanet_prepare(d["x"], d["w"], None, d["a"], d["b"], d["nae"], d["dtb"], nk, nv, dk, dv)
    zero = hb.deltanet_prepare(d["x"], d["w"], torch.zeros_like(d["st"]), d["a"], d["b"], d["nae"], d["dtb"], nk, nv, dk, dv)
    assert all(bool(torch.equal(a, b)) for a, b in zip(whole, zero))  # NULL state == zero state
    st, parts = None, []
    for lo, hi in ((0, 3), (3, 4), (4, 70)):  # a short prompt chunk, one decode token, the rest
        out = hb.deltanet_prepare(d["x"][:, lo:hi].contiguous(), d["w"], st, d["a"][:, lo:hi], d["b"][:, lo:hi], d["nae"], d["dtb"],
                                  nk, nv, dk, dv)
        st = out[5]
        parts.append(out)
    torch.cuda.synchronize()
    for i in range(5):
        assert bool(torch.equal(torch.cat([o[i] for o in parts], 1), whole[i]))
    assert bool(torch.equal(st, whole[5]))


@pytest.mark.parametrize("D", [64, 128, 256])
def test_gated_norm_matches_oracle(D):
    r = wl.philox(1200 + D)
    x = torch.from_numpy((r.standard_normal((3, 7, 4, D)) * 2).astype(np.float32))
    z = torch.from_numpy(r.standard_normal((3, 7, 4, D)).astype(np.float32)).to(torch.bfloat16)
    w = torch.from_numpy(r.standard_normal(D).astype(np.float32))
    got = hb.deltanet_gated_norm(x.to(DEV), z.to(DEV), w.to(DEV), 1e-6)
    torch.cuda.synchronize()
    want = orc.gated_rmsnorm(x.numpy(), _bits(z), w.numpy(), 1e-6)
    assert _ulps(_bits(got), want).max() <= 1


@pytest.mark.parametrize("chunked,S", [(False, 48), (True, 48), (True, 150)])
def test_layer_core_matches_the_reference_op_sequence(chunked, S):
    """prepare -> delta rule (L2-normalised q, k; q scaled) -> gated norm, against libtorch: conv/SiLU/gates as the
    layer does them, the decode-step recurrence iterated (qwen3_5.rs:725-751), RMSNormGated.  `chunked`: the delta
    rule in its chunk-64 form on the matrix pipe, as the layer runs a prompt (qwen3_5.rs:753-769)."""
    B, nk, nv, dk, dv = 2, 2, 4, 128, 128
    p = _layer_inputs(1300, B, S, nk, nv, dk, dv)
    d = {k_: v_.to(DEV) for k_, v_ in p.items()}
    q, k, v, g, beta, _ = hb.deltanet_prepare(d["x"], d["w"], d["st"], d["a"], d["b"], d["nae"], d["dtb"], nk, nv, dk, dv)
    state = torch.zeros(B, nv, dk, dv, device=DEV)
    o = torch.empty(B, S, nv, dv, device=DEV)
    (hb.deltanet_forward_chunked if chunked else hb.deltanet_forward)(q, k, v, g, beta, state, o, 1.0 / np.sqrt(dk), True)
    y = hb.deltanet_gated_norm(o, d["z"], d["nw"], 1e-6)
    torch.cuda.synchronize()
    # reference op sequence on the CPU
    conv, _, rg, rb = ref.deltanet_prepare(p["x"], p["w"].unsqueeze(1), p["st"], p["a"], p["b"], p["nae"], p["dtb"])
    kd = nk * dk
    l2 = lambda t: t / t.norm(dim=-1, keepdim=True).clamp_min(1e-3)
    rq = l2(conv[..., :kd].reshape(B, S, nk, dk).float()) * (1.0 / np.sqrt(dk))
    rk = l2(conv[..., kd:2 * kd].reshape(B, S, nk, dk).float())
    rv = conv[..., 2 * kd:].reshape(B, S, nv, dv).float()
    rq, rk = rq.repeat_interleave(nv // nk, 2), rk.repeat_interleave(nv // nk, 2)
    st = torch.zeros(B, nv, dk, dv)
    outs = []
    for t in range(S):
        ot, st = ref.deltanet_decode_step(rq[:, t], rk[:, t], rv[:, t], rg[:, t], rb[:, t], st)
        outs.append(ot)
    ro = torch.stack(outs, 1)
    want = ref.gated_rmsnorm(ro, p["z"], p["nw"], 1e-6)
    err = (y.float().cpu() - want.float()).abs()
    # bf16 outputs of O(1..16): a couple of ulps where the SiLU ulp differs, and one ulp of the value itself (2^-7
    # relative) where a difference far below it flips the final rounding
    assert (err - 2.0 ** -7 * want.float().abs()).max() < 3e-2 and err.mean() < 2e-3
    assert (state.cpu() - st).abs().max() < (3e-3 * float(st.abs().max()) if chunked else 1e-3)


def test_prepare_rejects_aliased_state_and_nulls():
    x = torch.zeros(1, 4, 2 * 128 + 128, dtype=torch.bfloat16, device=DEV)
    st = torch.zeros(1, 384, 3, dtype=torch.bfloat16, device=DEV)
    L = hb.lib()
    p = hb._ptr
    f = torch.zeros(8, device=DEV)
    rc = L.hs_deltanet_prepare(p(x), p(x), p(st), p(st), p(x), p(x), p(f), p(f), p(x), p(x), p(x), p(f), p(f), 1, 4, 1, 1, 128, 128, None)
    assert rc == hb.HS_ERR_INVALID_ARGUMENT and b"alias" in L.hs_attn_last_error()


def test_inputs_without_16_byte_alignment_take_the_narrow_kernels():
    """An input whose address is only element-aligned is served by the one-channel / one-row kernels, to the same bar."""
    def misaligned(t):
        buf = torch.empty(t.numel() + 1, dtype=t.dtype, device=DEV)
        out = buf[1:].view(t.shape)
        out.copy_(t)
        assert out.data_ptr() % 16 != 0
        return out

    B, S, nk, nv, dk, dv = 2, 37, 2, 4, 128, 128
    p = _layer_inputs(1300, B, S, nk, nv, dk, dv)
    q, k, v, g, beta, st = hb.deltanet_prepare(misaligned(p["x"]), p["w"].to(DEV), p["st"].to(DEV), p["a"].to(DEV), p["b"].to(DEV),
                                               p["nae"].to(DEV), p["dtb"].to(DEV), nk, nv, dk, dv)
    torch.cuda.synchronize()
    y, want_st = orc.deltanet_conv_silu_bf16(_bits(p["x"]), _bits(p["w"]), _bits(p["st"]))
    kd = nk * dk
    assert _ulps(_bits(q).reshape(B, S, kd), y[..., :kd]).max() <= 1
    assert _ulps(_bits(k).reshape(B, S, kd), y[..., kd:2 * kd]).max() <= 1
    assert _ulps(_bits(v).reshape(B, S, nv * dv), y[..., 2 * kd:]).max() <= 1
    assert np.array_equal(_bits(st), want_st)

    r = wl.philox(1301)
    x = torch.from_numpy((r.standard_normal((5, 3, 128)) * 2).astype(np.float32))
    z = torch.from_numpy(r.standard_normal((5, 3, 128)).astype(np.float32)).to(torch.bfloat16)
    w = torch.from_numpy(r.standard_normal(128).astype(np.float32))
    got = hb.deltanet_gated_norm(misaligned(x), z.to(DEV), w.to(DEV), 1e-6)
    torch.cuda.synchronize()
    assert _ulps(_bits(got), orc.gated_rmsnorm(x.numpy(), _bits(z), w.numpy(), 1e-6)).max() <= 1
