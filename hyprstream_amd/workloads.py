"""Seeded synthetic inputs for the attention hot path (the five benchmark configurations).

Small cases are drawn on the host with numpy's counter-based Philox generator so that the CPU
checker and the GPU box regenerate identical bytes from the seed alone; full-size cases are drawn
on the device with torch's seeded generator (nothing is shipped as data).
"""
import numpy as np

SEED = 0x5EED


def philox(stream, seed=SEED):
    return np.random.Generator(np.random.Philox(key=seed, counter=stream))


def to_bf16_bits(x):
    """fp32 numpy -> bf16 bit patterns (uint16), round-to-nearest-even."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def decode_case(stream, B, Hq, Hkv, D, T, ragged=False, outliers=False, sigma=1.0, bf16_source=True, min_len=1):
    """One decode-attention problem.  Returns a dict of numpy arrays:
    q_bits [B,Hq,D] uint16 (bf16), k/v [B,T,Hkv,D] fp32 (bf16-representable when bf16_source),
    seq_lens [B] int32 (T everywhere unless ragged)."""
    r = philox(stream)
    q = r.standard_normal((B, Hq, D)).astype(np.float32)
    k = (r.standard_normal((B, T, Hkv, D)) * sigma).astype(np.float32)
    v = (r.standard_normal((B, T, Hkv, D)) * sigma).astype(np.float32)
    if outliers:  # 1 % of the elements replaced by +-8 sigma
        for a in (k, v):
            m = r.random(a.shape) < 0.01
            a[m] = np.sign(a[m]) * 8.0 * sigma
    if bf16_source:
        k, v = bf16_bits_to_f32(to_bf16_bits(k)), bf16_bits_to_f32(to_bf16_bits(v))
    lens = r.integers(min_len, T + 1, B).astype(np.int32) if ragged else np.full(B, T, np.int32)
    return dict(q_bits=to_bf16_bits(q), k=k, v=v, seq_lens=lens)


def deltanet_case(stream, B, T, nk, nv, dk, dv):
    """q,k bf16 N(0,1) L2-normalised per head, v bf16 N(0,1), g = -softplus(N(0,1)), beta = sigmoid(N(0,1))."""
    r = philox(stream)
    q = r.standard_normal((B, T, nk, dk)).astype(np.float32)
    k = r.standard_normal((B, T, nk, dk)).astype(np.float32)
    q /= np.maximum(np.linalg.norm(q, axis=-1, keepdims=True), 1e-3)
    k /= np.maximum(np.linalg.norm(k, axis=-1, keepdims=True), 1e-3)
    v = r.standard_normal((B, T, nv, dv)).astype(np.float32)
    g = -np.log1p(np.exp(r.standard_normal((B, T, nv)))).astype(np.float32)
    beta = (1.0 / (1.0 + np.exp(-r.standard_normal((B, T, nv))))).astype(np.float32)
    return dict(q_bits=to_bf16_bits(q), k_bits=to_bf16_bits(k), v_bits=to_bf16_bits(v), g=g, beta=beta)


# Algorithmic HBM bytes of one decode call (int8 cache): K+V codes, their scales, Q and O in bf16,
# and the one new token per sequence that is read in bf16 and written as codes + scales.
def decode_bytes_int8(seq_lens, Hq, Hkv, D):
    tot = int(np.sum(seq_lens))
    B = len(seq_lens)
    return 2 * tot * Hkv * D + 2 * tot * Hkv * 4 + 2 * B * Hq * D * 2 + B * Hkv * D * (2 * 2 + 2 * 1) + B * Hkv * 2 * 4


def decode_bytes_fp8(seq_lens, Hq, Hkv, D):
    tot = int(np.sum(seq_lens))
    B = len(seq_lens)
    return 2 * tot * Hkv * D + 2 * B * Hkv * 4 + 2 * B * Hq * D * 2 + B * Hkv * D * (2 * 2 + 2 * 1)
