"""Pin the oracle's attention: golden vectors from the reference's libtorch op sequence, invariants."""
import os

import numpy as np
import torch

import oracle
from oracle import reference_path as ref
from conftest import GOLDEN

TOL_MAX, TOL_MEAN = 2e-2, 2e-3  # the path's stated tolerance (fp32 comparison)


def philox(stream):
    return np.random.Generator(np.random.Philox(key=99, counter=stream))


def small_case(stream, B=2, T=33, Hq=8, Hkv=2, D=128):
    r = philox(stream)
    q = oracle.round_bf16(r.standard_normal((B, Hq, D)).astype(np.float32))
    k = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    v = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    kc, ks = oracle.quant_int8(k)
    vc, vs = oracle.quant_int8(v)
    return q, kc, ks, vc, vs


def test_decode_matches_reference_op_sequence_golden():
    g = np.load(os.path.join(GOLDEN, "attention.npz"))
    out = oracle.decode_attn(g["a_q"][:, 0], g["a_kq"], g["a_vq"], g["a_ks"], g["a_vs"], oracle.FMT_INT8,
                             g["a_lens"], 1.0 / np.sqrt(128.0))
    assert np.abs(out - g["a_out"][:, 0]).max() < 2e-6


def test_cached_prefill_matches_reference_op_sequence_golden():
    g = np.load(os.path.join(GOLDEN, "attention.npz"))
    B, S = g["b_q"].shape[:2]
    T = g["b_k"].shape[1]
    out = oracle.prefill_attn(g["b_q"], g["b_k"], g["b_v"], None, None, oracle.FMT_DENSE,
                              np.full(B, T, np.int32), 1.0 / np.sqrt(64.0))
    assert np.abs(out - g["b_out"]).max() < 2e-6


def test_decode_vs_live_reference_path_with_bf16_dequant_view():
    """The reference rounds the dequantized view to bf16 (get() returns the model dtype) and the
    output to bf16; the oracle keeps exact s*c.  The two must agree within the path's tolerance."""
    q, kc, ks, vc, vs = small_case(1, B=2, T=257, Hq=8, Hkv=2)
    mine = oracle.decode_attn(q, kc, vc, ks, vs, oracle.FMT_INT8, np.array([257, 257], np.int32), 1 / np.sqrt(128.0))
    qt = torch.from_numpy(q).to(torch.bfloat16)[:, None]
    theirs = ref.decode_attention_int8(qt, torch.from_numpy(kc), torch.from_numpy(vc), torch.from_numpy(ks),
                                       torch.from_numpy(vs)).float().numpy()[:, 0]
    d = np.abs(mine - theirs)
    assert d.max() < TOL_MAX and d.mean() < TOL_MEAN


def test_softmax_weights_sum_to_one_constant_v():
    q, kc, ks, vc, vs = small_case(2)
    vc[:] = 64
    vs[:] = 0.125  # every dequantized V element is 8.0
    out = oracle.decode_attn(q, kc, vc, ks, vs, oracle.FMT_INT8, np.array([33, 20], np.int32), 0.0883883)
    assert np.allclose(out, 8.0, atol=1e-5)


def test_invariant_to_kv_permutation():
    q, kc, ks, vc, vs = small_case(3)
    lens = np.array([33, 33], np.int32)
    a = oracle.decode_attn(q, kc, vc, ks, vs, oracle.FMT_INT8, lens, 0.0883883)
    p = philox(30).permutation(33)
    b = oracle.decode_attn(q, kc[:, p], vc[:, p], ks[:, p], vs[:, p], oracle.FMT_INT8, lens, 0.0883883)
    assert np.abs(a - b).max() < 1e-6


def test_gqa_maps_query_head_to_floor_h_over_g():
    q, kc, ks, vc, vs = small_case(4, Hq=8, Hkv=2)
    lens = np.array([33, 33], np.int32)
    full = oracle.decode_attn(q, kc, vc, ks, vs, oracle.FMT_INT8, lens, 0.0883883)
    for hq in range(8):
        h = hq // 4
        one = oracle.decode_attn(q[:, hq:hq + 1], kc[:, :, h:h + 1], vc[:, :, h:h + 1], ks[:, :, h:h + 1],
                                 vs[:, :, h:h + 1], oracle.FMT_INT8, lens, 0.0883883)
        assert np.array_equal(one[:, 0], full[:, hq])


def test_ragged_equals_per_row_and_ignores_tail():
    q, kc, ks, vc, vs = small_case(5, B=3, T=40)
    lens = np.array([40, 7, 1], np.int32)
    full = oracle.decode_attn(q, kc, vc, ks, vs, oracle.FMT_INT8, lens, 0.0883883)
    kc2, vc2 = kc.copy(), vc.copy()
    for b, n in enumerate(lens):  # poison everything past the valid length
        kc2[b, n:] = 127
        vc2[b, n:] = -127
    assert np.array_equal(full, oracle.decode_attn(q, kc2, vc2, ks, vs, oracle.FMT_INT8, lens, 0.0883883))
    for b, n in enumerate(lens):
        row = oracle.decode_attn(q[b:b + 1], kc[b:b + 1, :n], vc[b:b + 1, :n], ks[b:b + 1, :n], vs[b:b + 1, :n],
                                 oracle.FMT_INT8, np.array([n], np.int32), 0.0883883)
        assert np.array_equal(row[0], full[b])
    # a single cached token: the output is exactly that token's dequantized V
    assert np.allclose(full[2], np.repeat(oracle.dequant_int8(vc, vs)[2, 0], 4, 0), atol=1e-6)


def test_split_k_merge_identity():
    """Merging per-chunk (m, l, o) partials reproduces the single pass: the rule the GPU kernel relies on."""
    q, kc, ks, vc, vs = small_case(6, B=1, T=96, Hq=4, Hkv=1)
    kd, vd = oracle.dequant_int8(kc, ks)[0, :, 0], oracle.dequant_int8(vc, vs)[0, :, 0]
    want = oracle.decode_attn(q, kc, vc, ks, vs, oracle.FMT_INT8, np.array([96], np.int32), 0.0883883)[0]
    s = (q[0].astype(np.float64) @ kd.T.astype(np.float64)) * 0.0883883
    parts = []
    for lo, hi in [(0, 16), (16, 80), (80, 96)]:
        m = s[:, lo:hi].max(1)
        p = np.exp(s[:, lo:hi] - m[:, None])
        parts.append((m, p.sum(1), p @ vd[lo:hi].astype(np.float64)))
    M = np.max([p[0] for p in parts], 0)
    L = sum(np.exp(m - M) * l for m, l, _ in parts)
    O = sum(np.exp(m - M)[:, None] * o for m, _, o in parts)
    assert np.abs(O / L[:, None] - want).max() < 1e-6


def test_two_token_cached_forward_equals_two_serial_decode_steps():
    """The reference's own equivalence test (llama.rs:3746-3785): a 2-token cached forward must equal
    two single-token steps; this pins the tril(k_len - q_len) offset."""
    r = philox(7)
    B, T, Hq, Hkv, D = 1, 12, 4, 2, 64
    q = r.standard_normal((B, 2, Hq, D)).astype(np.float32)
    k = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    v = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    two = oracle.prefill_attn(q, k, v, None, None, oracle.FMT_DENSE, np.array([T], np.int32), 0.125)
    s1 = oracle.prefill_attn(q[:, :1], k[:, :T - 1], v[:, :T - 1], None, None, oracle.FMT_DENSE,
                             np.array([T - 1], np.int32), 0.125)
    s2 = oracle.prefill_attn(q[:, 1:], k, v, None, None, oracle.FMT_DENSE, np.array([T], np.int32), 0.125)
    assert np.array_equal(two[:, 0], s1[:, 0]) and np.array_equal(two[:, 1], s2[:, 0])


def test_chunked_prefill_equals_unchunked():
    r = philox(8)
    B, T, Hq, Hkv, D, C = 1, 48, 4, 2, 64, 16
    q = r.standard_normal((B, T, Hq, D)).astype(np.float32)
    k = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    v = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    whole = oracle.prefill_attn(q, k, v, None, None, oracle.FMT_DENSE, np.array([T], np.int32), 0.125)
    for c in range(T // C):
        part = oracle.prefill_attn(q[:, c * C:(c + 1) * C], k[:, :(c + 1) * C], v[:, :(c + 1) * C], None, None,
                                   oracle.FMT_DENSE, np.array([(c + 1) * C], np.int32), 0.125)
        assert np.array_equal(part, whole[:, c * C:(c + 1) * C])


def test_fp8_decode_vs_live_qwen35_op_sequence():
    r = philox(9)
    B, T, Hq, Hkv, D = 2, 130, 16, 2, 128
    q = oracle.round_bf16(r.standard_normal((B, Hq, D)).astype(np.float32))
    k = (r.standard_normal((B, T, Hkv, D)) * 0.5).astype(np.float32)
    v = (r.standard_normal((B, T, Hkv, D)) * 0.5).astype(np.float32)
    ks, vs = oracle.fp8_calibrate(k), oracle.fp8_calibrate(v)
    kc, vc = oracle.quant_fp8(k, ks), oracle.quant_fp8(v, vs)
    mine = oracle.decode_attn(q, kc, vc, ks, vs, oracle.FMT_FP8, np.full(B, T, np.int32), 1 / np.sqrt(128.0))
    theirs = ref.decode_attention_fp8(torch.from_numpy(q).to(torch.bfloat16)[:, None], torch.from_numpy(kc),
                                      torch.from_numpy(vc), torch.from_numpy(ks), torch.from_numpy(vs))
    d = np.abs(mine - theirs.float().numpy()[:, 0])
    assert d.max() < TOL_MAX and d.mean() < TOL_MEAN


# ---------------------------------------------------------------- sliding window (local layers)
def test_windowed_prompt_matches_reference_op_sequence_golden():
    """apply_sliding_window_mask on a prompt over an empty cache (llama.rs:1086-1091, 1123-1155), libtorch ops."""
    g = np.load(os.path.join(GOLDEN, "attention_window.npz"))
    for tag in "abcde":
        q, k, v, W = g[tag + "_q"], g[tag + "_k"], g[tag + "_v"], int(g[tag + "_window"])
        B, S = q.shape[:2]
        out = oracle.prefill_attn(q, k, v, None, None, oracle.FMT_DENSE, np.full(B, S, np.int32),
                                  1.0 / np.sqrt(q.shape[-1]), window=W)
        assert np.abs(out - g[tag + "_out"]).max() < 2e-6, tag


def test_window_at_least_the_length_is_no_window_and_window_one_is_the_own_value_row():
    r = np.random.default_rng(31)
    B, T, S, Hq, Hkv, D = 2, 29, 11, 4, 2, 64
    q = r.standard_normal((B, S, Hq, D)).astype(np.float32)
    k = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    v = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    lens = np.full(B, T, np.int32)
    plain = oracle.prefill_attn(q, k, v, None, None, oracle.FMT_DENSE, lens, 0.125)
    for W in (T, T + 1, 10 ** 6):
        assert np.array_equal(oracle.prefill_attn(q, k, v, None, None, oracle.FMT_DENSE, lens, 0.125, window=W), plain)
    one = oracle.prefill_attn(q, k, v, None, None, oracle.FMT_DENSE, lens, 0.125, window=1)
    own = np.repeat(v[:, T - S:], Hq // Hkv, axis=2)  # query i sees only the key at its own position
    assert np.abs(one - own).max() < 1e-6


def test_window_with_history_is_attention_over_the_last_window_keys():
    """Brute force: for every query, cut the keys to (p - W, p] and run the unwindowed oracle on that slice."""
    r = np.random.default_rng(32)
    B, T, S, Hq, Hkv, D, W = 1, 37, 6, 2, 1, 64, 9
    q = r.standard_normal((B, S, Hq, D)).astype(np.float32)
    k = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    v = r.standard_normal((B, T, Hkv, D)).astype(np.float32)
    got = oracle.prefill_attn(q, k, v, None, None, oracle.FMT_DENSE, np.array([T], np.int32), 0.125, window=W)
    for i in range(S):
        p = T - S + i
        lo = max(0, p - W + 1)
        want = oracle.prefill_attn(q[:, i:i + 1], k[:, lo:p + 1], v[:, lo:p + 1], None, None, oracle.FMT_DENSE,
                                   np.array([p + 1 - lo], np.int32), 0.125)
        assert np.abs(got[:, i] - want[:, 0]).max() < 1e-6


def test_output_gate_matches_the_libtorch_ops_of_the_qwen35_layer():
    """ctx * gate.sigmoid() on bf16 tensors (qwen3_5.rs:1056-1059), live: the oracle's restatement gives libtorch's bits
    except where libm's and libtorch's exp differ in the last fp32 bit and that flips a bf16 rounding (rare, one ulp);
    closed forms: gate 0 halves the output exactly, a large gate leaves it, a very negative one gives a signed zero."""
    r = np.random.Generator(np.random.Philox(4242))
    ctx = (r.standard_normal((7, 5, 128)) * 2).astype(np.float32)
    gate = torch.from_numpy((r.standard_normal((7, 5, 128)) * 3).astype(np.float32)).to(torch.bfloat16)
    gate_bits = gate.view(torch.int16).numpy().view(np.uint16)
    got = oracle.output_gate_bf16(ctx, gate_bits)
    want = (torch.from_numpy(ctx).to(torch.bfloat16) * gate.sigmoid()).view(torch.int16).numpy().view(np.uint16)
    key = lambda u: np.where(u.astype(np.int32) & 0x8000, -(u.astype(np.int32) & 0x7fff), u.astype(np.int32) & 0x7fff)
    d = np.abs(key(got) - key(want))
    assert d.max() <= 1 and (d != 0).mean() < 2e-3
    o = np.array([1.5, -3.0, 0.25], np.float32)
    z = np.zeros(3, np.uint16)
    assert np.array_equal(oracle.bf16_to_f32(oracle.output_gate_bf16(o, z)), o * 0.5)
    big = oracle.f32_to_bf16(np.full(3, 40.0, np.float32))
    assert np.array_equal(oracle.bf16_to_f32(oracle.output_gate_bf16(o, big)), o)
    neg = oracle.f32_to_bf16(np.full(3, -200.0, np.float32))
    assert np.all(oracle.bf16_to_f32(oracle.output_gate_bf16(o, neg)) == 0.0)
