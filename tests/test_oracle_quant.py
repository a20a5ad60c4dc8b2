"""Pin the oracle's quantizers: golden vectors (libtorch CPU ops), brute force, invariants."""
import os

import numpy as np
import pytest
import torch

import oracle
from conftest import GOLDEN


def load(name):
    return np.load(os.path.join(GOLDEN, name))


def philox(stream):
    return np.random.Generator(np.random.Philox(key=77, counter=stream))


# ------------------------------------------------------------------ int8
def test_int8_matches_libtorch_golden():
    g = load("int8_quant.npz")
    codes, scales = oracle.quant_int8(g["x"])
    assert np.array_equal(scales.view(np.uint32), g["scales"].view(np.uint32))
    assert np.array_equal(codes, g["codes"])


def test_int8_bf16_source_matches_golden():
    g = load("int8_quant.npz")
    codes, scales = oracle.quant_int8_bf16(g["x_bf16_bits"])
    assert np.array_equal(scales.view(np.uint32), g["scales_bf16"].view(np.uint32))
    assert np.array_equal(codes, g["codes_bf16"])


def test_int8_live_libtorch_random():
    x = philox(1).standard_normal((512, 128)).astype(np.float32) * np.float32(3.7)
    xt = torch.from_numpy(x)
    s = xt.abs().amax(-1) / 127.0
    q = torch.round(xt / s[:, None]).clamp(-127, 127).to(torch.int8)
    codes, scales = oracle.quant_int8(x)
    assert np.array_equal(scales, s.numpy())
    assert np.array_equal(codes, q.numpy())


def test_int8_brute_force_nearest_code():
    """q must be a nearest point of the grid {s*i}: brute force over all 255 codes in float64."""
    x = philox(2).standard_normal((16, 32)).astype(np.float32)
    codes, scales = oracle.quant_int8(x)
    grid = np.arange(-127, 128, dtype=np.float64)
    for r in range(x.shape[0]):
        err = np.abs(x[r].astype(np.float64)[:, None] - scales[r].astype(np.float64) * grid[None, :])
        best = err.min(1)
        mine = err[np.arange(x.shape[1]), codes[r].astype(np.int64) + 127]
        # equal to the optimum up to the fp32 rounding of x/s (a half-ulp tie can go either way)
        assert np.all(mine <= best + 1e-6 * np.abs(x[r]).max())


def test_int8_invariants():
    x = philox(3).standard_normal((64, 128)).astype(np.float32)
    idx = philox(4).random((64, 128)) < 0.01
    x[idx] = np.sign(x[idx]) * 8
    codes, scales = oracle.quant_int8(x)
    assert codes.min() >= -127 and codes.max() <= 127
    am = np.abs(x).argmax(1)
    assert np.all(np.abs(codes[np.arange(64), am]) == 127)          # the max element maps to +-127
    deq = oracle.dequant_int8(codes, scales)
    assert np.all(np.abs(deq - x) <= scales[:, None] * 0.5000001)     # half a step at most
    c2, s2 = oracle.quant_int8(-x)                                    # sign symmetry
    assert np.array_equal(c2, -codes) and np.array_equal(s2, scales)
    c3, s3 = oracle.quant_int8(deq)                                   # idempotent on its own output
    assert np.array_equal(c3, codes)
    assert np.allclose(s3, scales, rtol=1e-6)


def test_int8_zero_row_and_single_element():
    x = np.zeros((2, 128), np.float32)
    x[1, 7] = -2.5
    codes, scales = oracle.quant_int8(x)
    assert scales[0] == 0 and not codes[0].any()
    assert codes[1, 7] == -127 and np.count_nonzero(codes[1]) == 1
    assert scales[1] == np.float32(2.5) / np.float32(127)


def test_int8_ties_round_to_even():
    x = np.zeros((1, 128), np.float32)
    x[0, 0] = 127.0
    x[0, 1:6] = [0.5, 1.5, 2.5, -0.5, -3.5]
    codes, _ = oracle.quant_int8(x)
    assert codes[0, 1:6].tolist() == [0, 2, 2, 0, -4]


# ------------------------------------------------------------------- fp8
def test_fp8_encode_all_bf16_inputs_match_libtorch_golden():
    g = load("fp8_codec.npz")
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = oracle.bf16_to_f32(bits)
    mine = oracle.fp8_encode(x)
    want = g["bf16_to_fp8"]
    nan = np.isnan(x)
    assert np.array_equal(mine[~nan], want[~nan])
    assert np.all((mine[nan] & 0x7F) == 0x7F) and np.all((want[nan] & 0x7F) == 0x7F)


def test_fp8_midpoints_and_random_fp32_match_golden():
    g = load("fp8_codec.npz")
    assert np.array_equal(oracle.fp8_encode(g["probe"]), g["probe_codes"])


def test_fp8_decode_all_codes():
    g = load("fp8_codec.npz")
    mine = oracle.fp8_decode(np.arange(256, dtype=np.uint32).astype(np.uint8))
    want = g["code_values"]
    assert np.array_equal(np.isnan(mine), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(mine[ok], want[ok])
    assert mine[0x7E] == 448.0 and mine[0x08] == 2.0 ** -6 and mine[0x01] == 2.0 ** -9


def test_fp8_live_libtorch_random():
    x = (philox(5).standard_normal(200000) * 30).astype(np.float32)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(oracle.fp8_encode(x), want)


def test_fp8_round_trip_is_identity_on_codes():
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], np.uint8)
    assert np.array_equal(oracle.fp8_encode(oracle.fp8_decode(codes)), codes)


def test_fp8_quant_matches_golden():
    g = load("fp8_quant.npz")
    s = oracle.fp8_calibrate(g["x"])
    assert np.array_equal(s, g["scales"])
    assert np.array_equal(oracle.quant_fp8(g["x"], s), g["codes"])
    late = oracle.quant_fp8(g["x_late"], s)
    assert np.array_equal(late, g["codes_late"])
    assert not np.any((late & 0x7F) == 0x7F)          # clamped to +-448, never the NaN pattern
    assert np.any((late & 0x7F) == 0x7E)              # and the clamp was actually exercised


def test_fp8_quant_error_bound():
    x = (philox(6).standard_normal((2, 16, 4, 128)) * 0.5).astype(np.float32)
    s = oracle.fp8_calibrate(x)
    deq = oracle.dequant_fp8(oracle.quant_fp8(x, s), s)
    # e4m3 keeps 4 significant bits: relative error <= 2^-4 for normals, absolute 2^-10*s below 2^-6*s
    bound = np.maximum(np.abs(x) * 2.0 ** -4, s[:, None, :, None] * 2.0 ** -10) * 1.0001
    assert np.all(np.abs(deq - x) <= bound)


def test_bf16_rounding_matches_libtorch():
    x = (philox(7).standard_normal(100000) * 5).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16(x), want)
