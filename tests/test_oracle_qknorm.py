"""Pins the oracle's QK-norm (oracle/hs_oracle.c::orc_qk_norm_bf16), the per-head RMS normalisation the reference runs
on q and k right before the rotary embedding:

  kind 1  LlamaAttention::apply_qk_norm, llama.rs:929-991 (Gemma3): bf16 op by op
  kind 2  Qwen3_5Model::apply_qknorm, qwen3_5.rs:1077-1091: fp32, (1 + w), one cast back

against golden vectors written by libtorch CPU ops in the reference's order (tests/golden/make_golden.py), a live
comparison with the same ops on larger inputs, and what the mathematics fixes.  libtorch's CPU result is itself not a
single bit pattern: the fp32 sum of the squares is added up in an order that depends on the host's vector width and its
vectorised rsqrt is not correctly rounded, so one machine's output can differ from another's (and from the oracle,
which takes the correctly rounded fp32 sum and 1/sqrt) by one bf16 ulp in a few elements per million.  The live test
states that bound; the golden vectors agree exactly."""
import os

import numpy as np
import pytest
import torch

from oracle import hs_oracle as orc
from oracle import reference_path as ref
from hyprstream_amd import workloads as wl


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(b):
    return torch.from_numpy(np.ascontiguousarray(b).view(np.int16)).view(torch.bfloat16)


@pytest.mark.parametrize("D", [64, 128, 256])
def test_golden_vectors(golden_dir, D):
    g = np.load(os.path.join(golden_dir, "qknorm.npz"))
    x, w1, w2 = g["x_%d" % D], g["w1_%d" % D], g["w2_%d" % D]
    assert np.array_equal(orc.qk_norm_bf16(x, 1, w1, 1e-6), g["llama_%d" % D])
    assert np.array_equal(orc.qk_norm_bf16(x, 1, w1[0], 1e-6), g["llama_shared_%d" % D])
    assert np.array_equal(orc.qk_norm_bf16(x, 2, w2, 1e-6), g["qwen_%d" % D])


def _ulp_apart(a_bits, b_bits):
    """bf16 patterns of the same sign that differ: distance in units of the last place."""
    return np.abs(a_bits.astype(np.int32) - b_bits.astype(np.int32))


@pytest.mark.parametrize("D", [64, 128, 256])
def test_live_against_libtorch_ops(D):
    r = wl.philox(900 + D)
    rows, H = 3000, 4
    x = torch.from_numpy((r.standard_normal((1, rows, H, D)) * r.random((1, rows, H, 1)) * 4).astype(np.float32)).to(torch.bfloat16)
    w1 = torch.from_numpy((1.0 + 0.2 * r.standard_normal((H, D))).astype(np.float32)).to(torch.bfloat16)
    w2 = torch.from_numpy((0.05 * r.standard_normal(D)).astype(np.float32))
    for kind, want in ((1, ref.qk_norm_llama(x, w1.reshape(-1))), (2, ref.qk_norm_qwen35(x, w2, 1e-6))):
        got = orc.qk_norm_bf16(bits(x[0]), kind, bits(w1) if kind == 1 else w2.numpy(), 1e-6)
        wb = bits(want[0])
        diff = got != wb
        assert diff.mean() <= 5e-5, (kind, diff.mean())          # a few per million on this machine
        if diff.any():
            assert _ulp_apart(got[diff], wb[diff]).max() == 1   # and then by one bf16 ulp
            # kind 1: a differing mean moves the whole head row; kind 2: single elements


def test_closed_forms():
    D, H = 128, 2
    # a head of +-c: mean square c^2, normalised values +-1 (times the weight) -- kind 2 with w = 0 gives +-1 up to eps
    x = np.full((1, H, D), 3.0, np.float32)
    x[0, :, ::2] = -3.0
    xb = wl.to_bf16_bits(x)
    out = wl.bf16_bits_to_f32(orc.qk_norm_bf16(xb, 2, np.zeros(D, np.float32), 0.0))
    assert np.array_equal(out, np.sign(x))
    # (1 + w) flavour: w = 1 doubles the output
    out2 = wl.bf16_bits_to_f32(orc.qk_norm_bf16(xb, 2, np.ones(D, np.float32), 0.0))
    assert np.array_equal(out2, 2 * np.sign(x))
    # kind 1 multiplies by the weight itself (w = 1 is the identity on a +-1-normalised row; eps = 1e-6 rounds away)
    out3 = wl.bf16_bits_to_f32(orc.qk_norm_bf16(xb, 1, wl.to_bf16_bits(np.ones((H, D), np.float32)), 1e-6))
    assert np.array_equal(out3, np.sign(x))
    # per-head weights are per head
    w = np.ones((H, D), np.float32)
    w[1] = 0.5
    out4 = wl.bf16_bits_to_f32(orc.qk_norm_bf16(xb, 1, wl.to_bf16_bits(w), 1e-6))
    assert np.array_equal(out4[0, 0], np.sign(x[0, 0])) and np.array_equal(out4[0, 1], 0.5 * np.sign(x[0, 1]))
    # an all-zero head stays zero (rrms = 1/sqrt(eps) is finite)
    z = np.zeros((1, H, D), np.uint16)
    assert not orc.qk_norm_bf16(z, 1, wl.to_bf16_bits(w), 1e-6).any()
    assert not orc.qk_norm_bf16(z, 2, np.zeros(D, np.float32), 1e-6).any()


def test_scale_invariance_of_kind2():
    # fp32 flavour: scaling a head by a power of two scales mean_sq exactly by its square; with eps = 0 the output is unchanged
    r = wl.philox(931)
    x = wl.bf16_bits_to_f32(wl.to_bf16_bits(r.standard_normal((5, 3, 128)).astype(np.float32)))
    w = (0.1 * r.standard_normal(128)).astype(np.float32)
    a = orc.qk_norm_bf16(wl.to_bf16_bits(x), 2, w, 0.0)
    b = orc.qk_norm_bf16(wl.to_bf16_bits(x * 64.0), 2, w, 0.0)
    assert np.array_equal(a, b)
