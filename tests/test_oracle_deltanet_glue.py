"""Oracle restatement of the steps around the delta rule (GatedDeltaNetLayer::forward, qwen3_5.rs:617-720, and
RMSNormGated, :292-313) against libtorch CPU ops and the mathematics.

libtorch's bf16 conv1d does not promise an accumulation order, so the conv is compared to one bf16 ulp; what the
mathematics fixes (identity taps, causality, carried state, closed forms of the gates) is checked exactly."""
import numpy as np
import torch

from oracle import hs_oracle as orc
from oracle import reference_path as ref


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _ulp_diff_bf16(a_bits, b_bits):
    """distance in bf16 ulps between two bit patterns of finite values of (almost always) equal sign"""
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7fff), u & 0x7fff)
    return np.abs(key(a_bits) - key(b_bits))


def _case(seed, B=2, S=37, C=48, K=4):
    r = np.random.default_rng(seed)
    x = torch.from_numpy(r.standard_normal((B, S, C)).astype(np.float32)).to(torch.bfloat16)
    w = torch.from_numpy((r.standard_normal((C, 1, K)) * 0.5).astype(np.float32)).to(torch.bfloat16)
    st = torch.from_numpy(r.standard_normal((B, C, K - 1)).astype(np.float32)).to(torch.bfloat16)
    return x, w, st


def test_conv_silu_matches_libtorch_to_one_ulp():
    x, w, st = _case(1)
    want, want_state, _, _ = ref.deltanet_prepare(x, w, st, torch.zeros(2, 37, 4), torch.zeros(2, 37, 4), torch.zeros(4), torch.zeros(4))
    got, got_state = orc.deltanet_conv_silu_bf16(_bits(x), _bits(w[:, 0]), _bits(st))
    assert _ulp_diff_bf16(got, _bits(want)).max() <= 1
    assert np.array_equal(got_state, _bits(want_state))


def test_identity_tap_gives_silu_of_the_input_and_taps_are_causal():
    x, w, st = _case(2, B=1, S=9, C=5)
    w = torch.zeros_like(w)
    w[:, 0, 3] = 1.0  # only the current frame
    got, _ = orc.deltanet_conv_silu_bf16(_bits(x), _bits(w[:, 0]), _bits(st))
    want = torch.nn.functional.silu(x.float()).to(torch.bfloat16)
    assert np.array_equal(got, _bits(want))
    w = torch.zeros_like(w)
    w[:, 0, 0] = 1.0  # only the frame three steps back: the first three outputs are the carried state
    got, _ = orc.deltanet_conv_silu_bf16(_bits(x), _bits(w[:, 0]), _bits(st))
    seq = torch.cat([st.permute(0, 2, 1), x], 1)[:, :9]
    assert np.array_equal(got, _bits(torch.nn.functional.silu(seq.float()).to(torch.bfloat16)))


def test_carried_state_makes_split_calls_equal_one_call():
    x, w, st = _case(3, B=2, S=20, C=16)
    whole, whole_state = orc.deltanet_conv_silu_bf16(_bits(x), _bits(w[:, 0]), _bits(st))
    y1, s1 = orc.deltanet_conv_silu_bf16(_bits(x[:, :7]), _bits(w[:, 0]), _bits(st))
    y2, s2 = orc.deltanet_conv_silu_bf16(_bits(x[:, 7:8]), _bits(w[:, 0]), s1)       # a single decode token
    y3, s3 = orc.deltanet_conv_silu_bf16(_bits(x[:, 8:]), _bits(w[:, 0]), s2)
    assert np.array_equal(np.concatenate([y1, y2, y3], 1), whole) and np.array_equal(s3, whole_state)
    # the state is the last three input frames
    assert np.array_equal(whole_state, _bits(x[:, -3:].permute(0, 2, 1)))


def test_gates_match_libtorch_and_closed_forms():
    r = np.random.default_rng(4)
    nv = 8
    a = torch.from_numpy((r.standard_normal((3, 11, nv)) * 4).astype(np.float32)).to(torch.bfloat16)
    b = torch.from_numpy((r.standard_normal((3, 11, nv)) * 4).astype(np.float32)).to(torch.bfloat16)
    a[0, 0, 0], a[0, 0, 1] = 30.0, -30.0  # beyond softplus' linear threshold; deep in the exponential tail
    a_log = torch.from_numpy(r.standard_normal(nv).astype(np.float32))
    dt_bias = torch.from_numpy(r.standard_normal(nv).astype(np.float32))
    neg_a_exp = -a_log.exp()
    _, _, wg, wb = ref.deltanet_prepare(torch.zeros(3, 11, 4, dtype=torch.bfloat16), torch.zeros(4, 1, 4, dtype=torch.bfloat16), None,
                                        a, b, neg_a_exp, dt_bias)
    g, beta = orc.deltanet_gates(_bits(a), _bits(b), neg_a_exp.numpy(), dt_bias.numpy())
    assert np.allclose(g, wg.numpy(), rtol=2e-6, atol=1e-30) and np.allclose(beta, wb.numpy(), rtol=2e-6)
    assert (g <= 0).all() and ((beta > 0) & (beta < 1)).all()
    assert g[0, 0, 0] == neg_a_exp[0].item() * (30.0 + dt_bias[0].item())       # softplus(x) = x above 20
    assert abs(g[0, 0, 1] / (neg_a_exp[1].item() * np.exp(-30.0 + dt_bias[1].item())) - 1) < 1e-5  # ~ exp(x) far below


def test_gated_rmsnorm_matches_libtorch_and_normalises():
    r = np.random.default_rng(5)
    x = torch.from_numpy((r.standard_normal((2, 5, 4, 128)) * 3).astype(np.float32))
    z = torch.from_numpy(r.standard_normal((2, 5, 4, 128)).astype(np.float32)).to(torch.bfloat16)
    w = torch.from_numpy(r.standard_normal(128).astype(np.float32))
    want = ref.gated_rmsnorm(x, z, w, 1e-6)
    got = orc.gated_rmsnorm(x.numpy(), _bits(z), w.numpy(), 1e-6)
    assert _ulp_diff_bf16(got, _bits(want)).max() <= 1
    # w = 1 and a large gate (silu(z) ~ z): rows have unit mean square times z
    ones = np.ones(128, np.float32)
    zz = torch.full((1, 128), 16.0, dtype=torch.bfloat16)
    y = orc.bf16_to_f32(orc.gated_rmsnorm(x.numpy()[0, 0, :1], _bits(zz), ones, 0.0)) / 16.0
    assert abs((y.astype(np.float64) ** 2).mean() - 1.0) < 2e-2
    # scale invariance of the normalisation
    y2 = orc.gated_rmsnorm(x.numpy() * 8.0, _bits(z), w.numpy(), 0.0)
    y1 = orc.gated_rmsnorm(x.numpy(), _bits(z), w.numpy(), 0.0)
    assert _ulp_diff_bf16(y1, y2).max() <= 1
