"""Pin the DeltaNet oracle: golden vectors from the reference's decode-step op sequence, the chunked
restatement against the recurrence, and delta-rule invariants."""
import os

import numpy as np

import oracle
from oracle import deltanet_chunked as dc
from conftest import GOLDEN


def philox(stream):
    return np.random.Generator(np.random.Philox(key=55, counter=stream))


def case(stream, B=2, T=70, nk=2, nv=4, dk=32, dv=24):
    r = philox(stream)
    q = r.standard_normal((B, T, nk, dk)).astype(np.float32)
    k = r.standard_normal((B, T, nk, dk)).astype(np.float32)
    v = r.standard_normal((B, T, nv, dv)).astype(np.float32)
    x = r.standard_normal((B, T, nv)).astype(np.float32)
    g = -np.log1p(np.exp(x)).astype(np.float32)
    beta = (1 / (1 + np.exp(-r.standard_normal((B, T, nv))))).astype(np.float32)
    return q, k, v, g, beta


def test_recurrent_matches_reference_decode_step_golden():
    g = np.load(os.path.join(GOLDEN, "deltanet.npz"))
    dk = g["q"].shape[-1]
    out, st = oracle.deltanet_recurrent(g["q"], g["k"], g["v"], g["g"], g["beta"], g["state0"], 1 / np.sqrt(dk), True)
    assert np.abs(out - g["out"]).max() < 5e-6
    assert np.abs(st - g["state"]).max() < 5e-6


def test_chunked_restatement_equals_recurrence():
    q, k, v, g, beta = case(1)  # T = 70: exercises the pad-to-64 branch
    B, T, nk, dk = q.shape
    nv = v.shape[2]
    s0 = (philox(10).standard_normal((B, nv, dk, v.shape[-1])) * 0.1).astype(np.float32)
    want, want_state = oracle.deltanet_recurrent(q, k, v, g, beta, s0, 1 / np.sqrt(dk), True)
    rep = nv // nk
    qh = np.repeat(dc.l2_normalize(q) / np.sqrt(dk), rep, 2).transpose(0, 2, 1, 3)
    kh = np.repeat(dc.l2_normalize(k), rep, 2).transpose(0, 2, 1, 3)
    out, st = dc.chunked_delta_rule(qh, kh, v.transpose(0, 2, 1, 3), g.transpose(0, 2, 1), beta.transpose(0, 2, 1),
                                    s0, np.float64)
    assert np.abs(out.transpose(0, 2, 1, 3) - want).max() < 1e-5
    assert np.abs(st - want_state).max() < 1e-5
    # fp32 as the reference runs it: the "~1e-3 chunked-vs-recurrent noise" it documents
    out32, st32 = dc.chunked_delta_rule(qh, kh, v.transpose(0, 2, 1, 3), g.transpose(0, 2, 1),
                                        beta.transpose(0, 2, 1), s0, np.float32)
    assert np.abs(out32.transpose(0, 2, 1, 3) - want).max() < 2e-3


def test_beta_zero_only_decays_state():
    q, k, v, g, beta = case(2, T=5)
    beta[:] = 0
    s0 = philox(11).standard_normal((2, 4, 32, 24)).astype(np.float32)
    _, st = oracle.deltanet_recurrent(q, k, v, g, beta, s0, 1.0, True)
    want = s0 * np.exp(g.astype(np.float64).sum(1))[:, :, None, None]
    assert np.abs(st - want).max() < 1e-6


def test_delta_rule_writes_v_exactly_when_g0_beta1_unit_k():
    q, k, v, g, beta = case(3, T=1)
    g[:] = 0
    beta[:] = 1
    s0 = philox(12).standard_normal((2, 4, 32, 24)).astype(np.float32)
    _, st = oracle.deltanet_recurrent(q, k, v, g, beta, s0, 1.0, True)
    kn = np.repeat(dc.l2_normalize(k)[:, 0], 2, 1)  # [B, nv, dk]
    read = np.einsum("bhk,bhkv->bhv", kn.astype(np.float64), st.astype(np.float64))
    assert np.abs(read - v[:, 0]).max() < 1e-5


def test_head_expansion_is_repeat_interleave():
    q, k, v, g, beta = case(4, T=3)
    out, _ = oracle.deltanet_recurrent(q, k, v, g, beta, None, 0.25, False)
    for j in range(4):
        one, _ = oracle.deltanet_recurrent(q[:, :, j // 2:j // 2 + 1], k[:, :, j // 2:j // 2 + 1], v[:, :, j:j + 1],
                                           g[:, :, j:j + 1], beta[:, :, j:j + 1], None, 0.25, False)
        assert np.array_equal(one[:, :, 0], out[:, :, j])


def test_l2norm_floor():
    x = np.zeros((1, 1, 1, 8), np.float32)
    x[..., 0] = 1e-4
    assert np.allclose(dc.l2_normalize(x)[..., 0], 0.1)
