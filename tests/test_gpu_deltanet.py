"""GPU parity: gated delta rule (decode step and token-by-token prefill) against the fp64 oracle."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV, bf16_from_bits

pytestmark = pytest.mark.gpu


def run(case, state0, q_scale, l2norm):
    q, k, v = (bf16_from_bits(case[n]).to(DEV) for n in ("q_bits", "k_bits", "v_bits"))
    g, beta = torch.from_numpy(case["g"]).to(DEV), torch.from_numpy(case["beta"]).to(DEV)
    B, T, nv = case["g"].shape
    st = torch.from_numpy(state0).to(DEV).clone()
    out = torch.full((B, T, nv, 128), float("nan"), dtype=torch.float32, device=DEV)
    hb.deltanet_forward(q, k, v, g, beta, st, out, q_scale, l2norm)
    torch.cuda.synchronize()
    return out.cpu().numpy(), st.cpu().numpy()


def want(case, state0, q_scale, l2norm):
    f = wl.bf16_bits_to_f32
    return oracle.deltanet_recurrent(f(case["q_bits"]), f(case["k_bits"]), f(case["v_bits"]), case["g"], case["beta"],
                                     state0, q_scale, l2norm)


@pytest.mark.parametrize("l2norm", [False, True])
def test_decode_step_config5_reduced(l2norm):
    """One token, nk 16 / nv 32, dk = dv = 128, carried state (config 5 decode at B = 3)."""
    B, nk, nv = 3, 16, 32
    case = wl.deltanet_case(30, B, 1, nk, nv, 128, 128)
    s0 = (wl.philox(31).standard_normal((B, nv, 128, 128)) * 0.1).astype(np.float32)
    o, s = run(case, s0, 1 / np.sqrt(128.0), l2norm)
    wo, ws = want(case, s0, 1 / np.sqrt(128.0), l2norm)
    print("decode l2norm=%s out err %.2e state err %.2e" % (l2norm, np.abs(o - wo).max(), np.abs(s - ws).max()))
    assert np.abs(o - wo).max() < 1e-5 and np.abs(s - ws).max() < 1e-5


@pytest.mark.parametrize("T", [2, 17, 64, 70, 300])
def test_prefill_recurrence(T):
    B, nk, nv = 2, 2, 4
    case = wl.deltanet_case(40 + T, B, T, nk, nv, 128, 128)
    s0 = np.zeros((B, nv, 128, 128), np.float32)
    o, s = run(case, s0, 1 / np.sqrt(128.0), True)
    wo, ws = want(case, s0, 1 / np.sqrt(128.0), True)
    print("prefill T=%d out err %.2e state err %.2e" % (T, np.abs(o - wo).max(), np.abs(s - ws).max()))
    assert np.abs(o - wo).max() < 2e-5 and np.abs(s - ws).max() < 2e-5


def test_prefill_equals_decode_steps_and_carries_state():
    """A T-token call must equal T single-token calls (the kernel switches column slicing between them)."""
    B, T, nk, nv = 1, 9, 2, 2
    case = wl.deltanet_case(50, B, T, nk, nv, 128, 128)
    s0 = (wl.philox(51).standard_normal((B, nv, 128, 128)) * 0.1).astype(np.float32)
    o, s = run(case, s0, 0.5, False)
    st = s0.copy()
    for t in range(T):
        one = {n: case[n][:, t:t + 1] for n in case}
        ot, st = run(one, st, 0.5, False)
        assert np.abs(ot[:, 0] - o[:, t]).max() < 1e-6
    assert np.abs(st - s).max() < 1e-6


def test_delta_rule_invariants_on_gpu():
    """beta = 0 only decays the state; g = 0, beta = 1 writes v exactly (k^T S_new = v)."""
    B, nk, nv = 1, 2, 2
    case = wl.deltanet_case(60, B, 1, nk, nv, 128, 128)
    s0 = wl.philox(61).standard_normal((B, nv, 128, 128)).astype(np.float32)
    case["beta"][:] = 0
    _, s = run(case, s0, 1.0, True)
    assert np.abs(s - s0 * np.exp(case["g"][:, 0])[:, :, None, None]).max() < 1e-6
    case["beta"][:] = 1
    case["g"][:] = 0
    _, s = run(case, s0, 1.0, True)
    k = wl.bf16_bits_to_f32(case["k_bits"])[:, 0]
    kn = np.repeat(k / np.linalg.norm(k, axis=-1, keepdims=True), nv // nk, 1)
    read = np.einsum("bhk,bhkv->bhv", kn.astype(np.float64), s.astype(np.float64))
    assert np.abs(read - wl.bf16_bits_to_f32(case["v_bits"])[:, 0]).max() < 1e-4


def test_bad_shapes_are_rejected():
    t = torch.zeros(1, 1, 2, 64, dtype=torch.bfloat16, device=DEV)
    f = torch.zeros(1, 1, 2, dtype=torch.float32, device=DEV)
    with pytest.raises(hb.HsError):
        hb.deltanet_forward(t, t, t, f, f, torch.zeros(1, 2, 64, 64, device=DEV), torch.zeros(1, 1, 2, 64, device=DEV), 1.0)
