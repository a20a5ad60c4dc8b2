"""numpy restatement of the reference's chunked gated-delta-rule prefill.

Follows `chunked_delta_rule` (crates/hyprstream/src/runtime/architectures/
qwen3_5.rs:342-498) step for step, in the precision asked for (fp32 as the
reference, or fp64): pad T to a multiple of 64, cumulative log-decay per chunk,
the strictly-lower correction matrix solved row by row (forward substitution,
qwen3_5.rs:423-442), then the chunk loop that carries the [dk, dv] state.
Test infrastructure only.  Pinned by equality with the token-by-token
recurrence (oracle.deltanet_recurrent) and by the delta-rule invariants in
tests/test_oracle_deltanet.py.
"""
import numpy as np

CHUNK = 64


def l2_normalize(x):
    """x / max(||x||_2, 1e-3) over the last axis (qwen3_5.rs:331-335)."""
    n = np.sqrt((x.astype(np.float64) ** 2).sum(-1, keepdims=True))
    return (x / np.maximum(n, 1e-3)).astype(x.dtype)


def chunked_delta_rule(q, k, v, g, beta, initial_state=None, dtype=np.float32):
    """q,k [B,nv,T,dk] (normalised, q pre-scaled); v [B,nv,T,dv]; g,beta [B,nv,T].

    Returns (out [B,nv,T,dv], state [B,nv,dk,dv]).
    """
    q, k, v, g, beta = (np.asarray(a, dtype) for a in (q, k, v, g, beta))
    B, nv, T, dk = q.shape
    dv = v.shape[-1]
    pad = (CHUNK - T % CHUNK) % CHUNK
    if pad:
        zp = lambda a: np.concatenate([a, np.zeros(a.shape[:2] + (pad,) + a.shape[3:], dtype)], 2)
        q, k, v, g, beta = zp(q), zp(k), zp(v), zp(g), zp(beta)
    Tp = T + pad
    nc = Tp // CHUNK
    v_beta = v * beta[..., None]
    k_beta = k * beta[..., None]
    r5 = lambda a: a.reshape(B, nv, nc, CHUNK, a.shape[-1])
    q, k, v, k_beta, v_beta = r5(q), r5(k), r5(v), r5(k_beta), r5(v_beta)
    g = np.cumsum(g.reshape(B, nv, nc, CHUNK), -1, dtype=dtype)
    decay = np.tril(np.exp(g[..., :, None] - g[..., None, :]))
    lower_strict = np.tril(np.ones((CHUNK, CHUNK), bool), -1)
    attn = -(k_beta @ np.swapaxes(k, -1, -2) * decay) * lower_strict
    for i in range(1, CHUNK):
        row = attn[..., i, :i].copy()
        attn[..., i, :i] = row + (row[..., None, :] @ attn[..., :i, :i])[..., 0, :]
    attn = attn + np.eye(CHUNK, dtype=dtype)
    value_t = attn @ v_beta
    k_cumdecay = attn @ (k_beta * np.exp(g)[..., None])
    state = np.zeros((B, nv, dk, dv), dtype) if initial_state is None else np.asarray(initial_state, dtype).copy()
    keep = np.tril(np.ones((CHUNK, CHUNK), bool))  # diagonal kept: triu(1) is what is zeroed
    outs = []
    for i in range(nc):
        q_i, k_i, v_i, g_i = q[:, :, i], k[:, :, i], value_t[:, :, i], g[:, :, i]
        inner = (q_i @ np.swapaxes(k_i, -1, -2) * decay[:, :, i]) * keep
        v_new = v_i - k_cumdecay[:, :, i] @ state
        inter = (q_i * np.exp(g_i)[..., None]) @ state
        outs.append(inter + inner @ v_new)
        g_last = g_i[..., -1:]
        state = state * np.exp(g_last)[..., None] + np.swapaxes(k_i * np.exp(g_last - g_i)[..., None], -1, -2) @ v_new
    out = np.stack(outs, 2).reshape(B, nv, Tp, dv)[:, :, :T]
    return np.ascontiguousarray(out), state
