"""The oracle's RoPE restatement against libtorch golden vectors, live libtorch ops and the mathematics.

Reference: crates/hyprstream/src/runtime/rope.rs:100-122 (tables, fp32 then cast) and :206-248 (half-split
rotation as separate tensor ops in the tensor dtype)."""
import os

import numpy as np
import pytest
import torch

from oracle import hs_oracle as orc
from oracle import reference_path as ref

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "rope.npz"))


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("tag", ["a", "b", "c"])
def test_bf16_golden_bit_exact(tag):
    x, y = G[f"{tag}_bf16_x"], G[f"{tag}_bf16_y"]
    sin, cos = G[f"{tag}_bf16_sin"], G[f"{tag}_bf16_cos"]  # rows already selected per token
    B, S, H, D = x.shape
    pos = np.tile(np.arange(S, dtype=np.int32), B)
    got = orc.rope_apply_bf16(x.reshape(B * S, H, D), sin, cos, pos).reshape(x.shape)
    assert np.array_equal(got, y)


@pytest.mark.parametrize("tag", ["a", "b", "c"])
def test_f32_golden_bit_exact(tag):
    x, y = G[f"{tag}_f32_x"], G[f"{tag}_f32_y"]
    sin, cos = G[f"{tag}_f32_sin"], G[f"{tag}_f32_cos"]
    B, S, H, D = x.shape
    pos = np.tile(np.arange(S, dtype=np.int32), B)
    got = orc.rope_apply_f32(x.reshape(B * S, H, D), sin, cos, pos).reshape(x.shape)
    assert np.array_equal(got.view(np.uint32), y.view(np.uint32))


def test_live_libtorch_bf16_random_positions():
    rng = np.random.default_rng(7)
    D, L, S, H = 128, 4096, 40, 5
    sin, cos = ref.rope_tables(D, 500000.0, L, torch.bfloat16)
    pos = rng.integers(0, L, S)
    x = torch.from_numpy(rng.standard_normal((1, S, H, D)).astype(np.float32) * 3).to(torch.bfloat16)
    want = _bits(ref.rope_apply(x, sin, cos, torch.from_numpy(pos)))
    got = orc.rope_apply_bf16(_bits(x).reshape(S, H, D), _bits(sin), _bits(cos), pos.astype(np.int32))
    assert np.array_equal(got.reshape(want.shape), want)


def test_position_zero_is_identity_and_tables_start_at_one_zero():
    sin, cos = ref.rope_tables(128, 10000.0, 4, torch.float32)
    assert torch.all(sin[0] == 0) and torch.all(cos[0] == 1)
    x = np.random.default_rng(1).standard_normal((3, 2, 128)).astype(np.float32)
    got = orc.rope_apply_f32(x, sin.numpy(), cos.numpy(), np.zeros(3, np.int32))
    assert np.array_equal(got, x)


def test_rotation_preserves_pair_norms_and_relative_position():
    rng = np.random.default_rng(2)
    D, L = 64, 512
    sin, cos = ref.rope_tables(D, 10000.0, L, torch.float32)
    q = rng.standard_normal((1, 1, D)).astype(np.float32)
    k = rng.standard_normal((1, 1, D)).astype(np.float32)
    half = D // 2

    def rot(x, p):
        return orc.rope_apply_f32(x, sin.numpy(), cos.numpy(), np.array([p], np.int32))[0, 0].astype(np.float64)

    r = rot(q, 137)
    # a rotation of each (d, d + D/2) pair: pair norms are unchanged
    assert np.allclose(r[:half] ** 2 + r[half:] ** 2, q[0, 0, :half].astype(np.float64) ** 2 + q[0, 0, half:].astype(np.float64) ** 2, rtol=1e-5)
    # <rope(q, m), rope(k, n)> depends on m - n only
    d1 = rot(q, 200) @ rot(k, 180)
    d2 = rot(q, 50) @ rot(k, 30)
    assert abs(d1 - d2) < 1e-3 * (np.linalg.norm(q) * np.linalg.norm(k))
    # and equals the closed form  sum_j Re[(q1 + i q2)(k1 - i k2) e^{i (m-n) w_j}]
    w = 10000.0 ** (-np.arange(half) * 2.0 / D)
    qc = q[0, 0, :half].astype(np.float64) + 1j * q[0, 0, half:].astype(np.float64)
    kc = k[0, 0, :half].astype(np.float64) + 1j * k[0, 0, half:].astype(np.float64)
    closed = np.real(qc * np.conj(kc) * np.exp(1j * 20 * w)).sum()
    assert abs(d1 - closed) < 1e-3 * (np.linalg.norm(q) * np.linalg.norm(k))


def test_sign_of_the_rotation():
    # one pair, angle pi/2 at table row 1: (1, 0) -> (cos, sin) = (0, 1); a swapped sign would give (0, -1)
    sin = np.array([[0.0], [1.0]], np.float32)
    cos = np.array([[1.0], [0.0]], np.float32)
    x = np.array([[[1.0, 0.0]]], np.float32)
    got = orc.rope_apply_f32(x, sin, cos, np.array([1], np.int32))
    assert np.array_equal(got, np.array([[[0.0, 1.0]]], np.float32))
