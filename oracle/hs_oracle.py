"""numpy front end of the C oracle (libhs_oracle.so).  Test infrastructure only.

Canonical layouts (the reference's own, kv_cache.rs:513-514): K/V and their
codes are [B, T, Hkv, D]; int8 scales are [B, T, Hkv]; fp8 scales are [B, Hkv].
bf16 tensors travel as numpy uint16 arrays holding the raw bit patterns.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhs_oracle.so")
_lib = None

FMT_INT8 = 0
FMT_FP8 = 1
FMT_DENSE = 2


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            from . import build as _build  # build on first use (gcc only)
            _build.build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_f32_to_bf16.restype = ctypes.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.orc_fp8_e4m3fn_from_f32.restype = ctypes.c_uint8
        _lib.orc_fp8_e4m3fn_from_f32.argtypes = [ctypes.c_float]
        _lib.orc_fp8_e4m3fn_to_f32.restype = ctypes.c_float
        _lib.orc_fp8_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


# ----------------------------------------------------------------- bf16 helpers
def f32_to_bf16(x):
    """fp32 -> bf16 bit patterns (uint16), round-to-nearest-even."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_f32_to_bf16_array(_p(x), ctypes.c_int64(x.size), _p(out))
    return out


def bf16_to_f32(x):
    x = _c(x, np.uint16)
    return (x.astype(np.uint32) << 16).view(np.float32)


def round_bf16(x):
    """fp32 -> nearest bf16 value, returned as fp32."""
    return bf16_to_f32(f32_to_bf16(x))


# ------------------------------------------------------------------------ int8
def quant_int8(x):
    """x: [..., D] fp32 -> (codes int8 [..., D], scales fp32 [...])."""
    x = _c(x, np.float32)
    D = x.shape[-1]
    rows = x.size // D if D else 0
    codes = np.empty(x.shape, np.int8)
    scales = np.empty(x.shape[:-1], np.float32)
    lib().orc_quant_int8_f32(_p(x), ctypes.c_int64(rows), ctypes.c_int(D), _p(codes), _p(scales))
    return codes, scales


def quant_int8_bf16(x_bits):
    """x_bits: [..., D] uint16 bf16 patterns -> (codes, scales)."""
    x = _c(x_bits, np.uint16)
    D = x.shape[-1]
    rows = x.size // D if D else 0
    codes = np.empty(x.shape, np.int8)
    scales = np.empty(x.shape[:-1], np.float32)
    lib().orc_quant_int8_bf16(_p(x), ctypes.c_int64(rows), ctypes.c_int(D), _p(codes), _p(scales))
    return codes, scales


def dequant_int8(codes, scales):
    codes = _c(codes, np.int8)
    scales = _c(scales, np.float32)
    D = codes.shape[-1]
    out = np.empty(codes.shape, np.float32)
    lib().orc_dequant_int8(_p(codes), _p(scales), ctypes.c_int64(codes.size // D), ctypes.c_int(D), _p(out))
    return out


# ------------------------------------------------------------------------- fp8
def fp8_encode(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    lib().orc_fp8_encode_array(_p(x), ctypes.c_int64(x.size), _p(out))
    return out


def fp8_decode(b):
    b = _c(b, np.uint8)
    out = np.empty(b.shape, np.float32)
    lib().orc_fp8_decode_array(_p(b), ctypes.c_int64(b.size), _p(out))
    return out


def fp8_calibrate(x):
    """x: [B, S, H, D] fp32 -> scales [B, H] = amax/448."""
    x = _c(x, np.float32)
    B, S, H, D = x.shape
    out = np.empty((B, H), np.float32)
    lib().orc_fp8_calibrate(_p(x), B, S, H, D, _p(out))
    return out


def quant_fp8(x, scales):
    """x: [B, S, H, D] fp32, scales [B, H] -> e4m3fn codes uint8 [B, S, H, D]."""
    x = _c(x, np.float32)
    scales = _c(scales, np.float32)
    B, S, H, D = x.shape
    assert scales.shape == (B, H)
    out = np.empty(x.shape, np.uint8)
    lib().orc_quant_fp8_f32(_p(x), _p(scales), B, S, H, D, _p(out))
    return out


def dequant_fp8(codes, scales):
    """codes [B, T, H, D] uint8, scales [B, H] -> fp32."""
    return fp8_decode(codes) * _c(scales, np.float32)[:, None, :, None]


# ------------------------------------------------------------------- attention
def _kv_args(kc, vc, ks, vs, fmt):
    if fmt == FMT_INT8:
        kc, vc = _c(kc, np.int8), _c(vc, np.int8)
        ks, vs = _c(ks, np.float32), _c(vs, np.float32)
        assert ks.shape == kc.shape[:3] and vs.shape == vc.shape[:3]
    elif fmt == FMT_FP8:
        kc, vc = _c(kc, np.uint8), _c(vc, np.uint8)
        ks, vs = _c(ks, np.float32), _c(vs, np.float32)
        assert ks.shape == (kc.shape[0], kc.shape[2])
    else:
        kc, vc = _c(kc, np.float32), _c(vc, np.float32)
        ks = vs = np.zeros(1, np.float32)
    return kc, vc, ks, vs


def prefill_attn(q, kc, vc, ks, vs, fmt, kv_lens, softmax_scale, window=0):
    """q [B, S, Hq, D] fp32; cache canonical [B, Tcap, Hkv, D]; kv_lens [B].

    Query row i of sequence b sits at absolute position kv_lens[b]-S+i.
    window > 0: sliding window of local layers, a query at position p attends keys in (p - window, p].
    Returns fp32 [B, S, Hq, D] (double accumulation inside).
    """
    q = _c(q, np.float32)
    kc, vc, ks, vs = _kv_args(kc, vc, ks, vs, fmt)
    B, S, Hq, D = q.shape
    _, Tcap, Hkv, D2 = kc.shape
    assert D2 == D and Hq % Hkv == 0 and kc.shape[0] == B
    kv_lens = _c(kv_lens, np.int32)
    assert kv_lens.shape == (B,) and (kv_lens <= Tcap).all()
    out = np.empty(q.shape, np.float32)
    lib().orc_prefill_attn_window(_p(q), _p(kc), _p(vc), _p(ks), _p(vs), fmt, _p(kv_lens), B, S, Hq, Hkv, D, Tcap,
                                  ctypes.c_float(softmax_scale), int(window), _p(out))
    return out


def decode_attn(q, kc, vc, ks, vs, fmt, seq_lens, softmax_scale):
    """q [B, Hq, D] fp32 -> out [B, Hq, D] fp32."""
    q = _c(q, np.float32)
    return prefill_attn(q[:, None], kc, vc, ks, vs, fmt, seq_lens, softmax_scale)[:, 0]


# -------------------------------------------------------------------- DeltaNet
def deltanet_recurrent(q, k, v, g, beta, state, q_scale, l2norm=False):
    """q,k [B,T,nk,dk]; v [B,T,nv,dv]; g,beta [B,T,nv]; state [B,nv,dk,dv] or None.

    Returns (out [B,T,nv,dv] fp32, final state fp32).
    """
    q, k, v = _c(q, np.float32), _c(k, np.float32), _c(v, np.float32)
    g, beta = _c(g, np.float32), _c(beta, np.float32)
    B, T, nk, dk = q.shape
    _, _, nv, dv = v.shape
    assert nv % nk == 0
    st = np.zeros((B, nv, dk, dv), np.float32) if state is None else np.array(state, np.float32, order="C", copy=True)
    out = np.empty((B, T, nv, dv), np.float32)
    lib().orc_deltanet_recurrent(_p(q), _p(k), _p(v), _p(g), _p(beta), _p(st), B, T, nk, nv, dk, dv,
                                 ctypes.c_float(q_scale), int(bool(l2norm)), _p(out))
    return out, st


# ------------------------------------------------------------------------ RoPE
def rope_apply_bf16(x_bits, sin_bits, cos_bits, pos):
    """x_bits: uint16 [rows, H, D] bf16 patterns; sin/cos: uint16 [L, D/2]; pos: int32 [rows] -> uint16 [rows, H, D]."""
    x = _c(x_bits, np.uint16)
    rows, H, D = x.shape
    out = np.empty_like(x)
    lib().orc_rope_apply_bf16(_p(x), _p(_c(sin_bits, np.uint16)), _p(_c(cos_bits, np.uint16)), _p(_c(pos, np.int32)),
                              ctypes.c_int64(rows), ctypes.c_int(H), ctypes.c_int(D), _p(out))
    return out


def rope_apply_f32(x, sin_t, cos_t, pos):
    x = _c(x, np.float32)
    rows, H, D = x.shape
    out = np.empty_like(x)
    lib().orc_rope_apply_f32(_p(x), _p(_c(sin_t, np.float32)), _p(_c(cos_t, np.float32)), _p(_c(pos, np.int32)),
                             ctypes.c_int64(rows), ctypes.c_int(H), ctypes.c_int(D), _p(out))
    return out


def qk_norm_bf16(x_bits, kind, weight, eps):
    """x_bits: uint16 [rows, H, D] bf16 patterns.  kind 1 (Llama/Gemma3, bf16 op by op): weight uint16 bf16 [H, D] or [D];
    kind 2 (Qwen3.5, fp32, (1 + w)): weight fp32 [D] or [H, D].  Returns uint16 [rows, H, D]."""
    x = _c(x_bits, np.uint16)
    rows, H, D = x.shape
    w = _c(weight, np.uint16 if kind == 1 else np.float32)
    assert w.shape in ((D,), (H, D))
    out = np.empty_like(x)
    lib().orc_qk_norm_bf16(_p(x), ctypes.c_int64(rows), ctypes.c_int(H), ctypes.c_int(D), ctypes.c_int(kind), _p(w),
                           ctypes.c_int(D if w.ndim == 2 else 0), ctypes.c_float(eps), _p(out))
    return out


# ------------------------------------------------------- DeltaNet surroundings
def deltanet_conv_silu_bf16(x_bits, w_bits, state_bits):
    """x [B,S,C], w [C,K], state [B,C,K-1] (bf16 patterns) -> (y [B,S,C], new state)."""
    x = _c(x_bits, np.uint16)
    w = _c(w_bits, np.uint16)
    st = _c(state_bits, np.uint16).copy()
    B, S, C = x.shape
    y = np.empty_like(x)
    lib().orc_deltanet_conv_silu_bf16(_p(x), _p(w), _p(st), B, S, C, w.shape[1], _p(y))
    return y, st


def deltanet_gates(a_bits, b_bits, neg_a_exp, dt_bias):
    a = _c(a_bits, np.uint16)
    b = _c(b_bits, np.uint16)
    nv = a.shape[-1]
    g = np.empty(a.shape, np.float32)
    beta = np.empty(a.shape, np.float32)
    lib().orc_deltanet_gates(_p(a), _p(b), _p(_c(neg_a_exp, np.float32)), _p(_c(dt_bias, np.float32)),
                             ctypes.c_int64(a.size // nv), nv, _p(g), _p(beta))
    return g, beta


def gated_rmsnorm(x, z_bits, w, eps):
    x = _c(x, np.float32)
    z = _c(z_bits, np.uint16)
    D = x.shape[-1]
    out = np.empty(x.shape, np.uint16)
    lib().orc_gated_rmsnorm(_p(x), _p(z), _p(_c(w, np.float32)), ctypes.c_float(eps), ctypes.c_int64(x.size // D), D, _p(out))
    return out



def output_gate_bf16(attn, gate_bits):
    """The output gate of the Qwen3.5 full-attention layers (qwen3_5.rs:1056-1059: ctx_flat * gate.sigmoid() on tensors
    of the model dtype): the attention output rounded to bf16, the sigmoid of the bf16 gate computed in fp32 and
    rounded to bf16, their product rounded to bf16.  attn fp32 (any shape), gate_bits uint16 of the same shape;
    returns bf16 bits."""
    o = bf16_to_f32(f32_to_bf16(np.asarray(attn, np.float32)))
    g = bf16_to_f32(np.asarray(gate_bits, np.uint16))
    with np.errstate(over="ignore"):
        sg = (np.float32(1.0) / (np.float32(1.0) + np.exp(-g, dtype=np.float32))).astype(np.float32)
    sg = bf16_to_f32(f32_to_bf16(sg))
    return f32_to_bf16((o * sg).astype(np.float32))
