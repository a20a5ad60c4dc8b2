"""hs_deltanet_forward_chunked_gated_norm: the chunk-64 delta rule with the layer's gated RMSNorm in the scan's epilogue
(chunked_delta_rule qwen3_5.rs:342-498 + RMSNormGated :305-313), against the two calls it replaces
(hs_deltanet_forward_chunked + hs_deltanet_gated_norm: same state bit for bit, rows within one bf16 ulp -- only the
order in which a row's squares are added differs) and against the CPU oracle (fp64 recurrence, then the norm)."""
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
    u = _ulps(_bits(got), _bits(want))
    assert u.max() <= 1 and (u != 0).mean() < 0.02, (int(u.max()), float((u != 0).mean()))


def test_more_sequences_than_one_launch_holds():
    """2 * nv * B workgroups beyond what the device keeps resident: the scan runs as several cooperative launches."""
    B, T, nk, nv = 70, 70, 2, 2  # 280 workgroups; the device holds 256 at a time
    case, z, w, s0 = _case(9200, B, T, nk, nv)
    got, want, st_b, st_a, _ = _both(case, z, w, s0)
    assert torch.equal(st_b, st_a)
    assert _ulps(_bits(got), _bits(want)).max() <= 1


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
