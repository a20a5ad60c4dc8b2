"""The reference's CPU attention path restated op for op with libtorch CPU ops.

hyprstream runs attention as a sequence of libtorch tensor ops reached through
tch-rs; the same ATen CPU kernels are reached here through PyTorch.  This file
is (a) the CPU baseline timed next to the GPU numbers and (b) a second witness
for the C oracle.  Test infrastructure only.  Citations are relative to
crates/hyprstream/src/runtime/ in the reference checkout.

  dequant_view            kv_cache.rs:1517-1580  get() on quantized storage returns dense K/V in
                                                  the model dtype (codes * scale -> bf16)
  expand_kv_for_gqa       architectures/llama.rs:847-872   unsqueeze + expand + reshape
  compute_attention       architectures/llama.rs:1023-1119 transpose/contiguous, fp32 upcast, matmul,
                                                  scale, mask, softmax, matmul, downcast
  qwen35_attention        architectures/qwen3_5.rs:1001-1053 same, probabilities cast to the model
                                                  dtype before the PV matmul
  batched_mask            architectures/llama.rs:2544-2572 additive -1e9 mask for ragged rows
  deltanet_decode_step    architectures/qwen3_5.rs:725-751
"""
import torch

ATTN_CHUNK = 1024  # llama.rs:1032, qwen3_5.rs:1012


def dequant_view_int8(codes, scales, dtype=torch.bfloat16):
    """codes int8 [B,T,H,D], scales fp32 [B,T,H] -> dense [B,T,H,D] in `dtype`."""
    return (codes.to(torch.float32) * scales.unsqueeze(-1)).to(dtype)


def dequant_view_fp8(codes_u8, scales, dtype=torch.bfloat16):
    """codes uint8 (e4m3fn bit patterns) [B,T,H,D], scales fp32 [B,H]."""
    x = codes_u8.view(torch.float8_e4m3fn).to(torch.float32)
    return (x * scales[:, None, :, None]).to(dtype)


def expand_kv_for_gqa(kv, num_heads):
    B, T, Hkv, D = kv.shape
    rep = num_heads // Hkv
    if rep == 1:
        return kv
    return kv.unsqueeze(3).expand(B, T, Hkv, rep, D).reshape(B, T, num_heads, D)


def sliding_window_mask(seq_len, window, dtype=torch.float32):
    """apply_sliding_window_mask (llama.rs:1123-1155): additive [seq_len, seq_len] mask, 0 where j <= i and
    i - j < window, -10000 elsewhere, built as tril(0) * triu(1 - window)."""
    causal = torch.ones(seq_len, seq_len, dtype=dtype).tril(0)
    win = torch.ones(seq_len, seq_len, dtype=dtype).triu(1 - window)
    return (torch.ones(seq_len, seq_len, dtype=dtype) - causal * win) * (-10000.0)


def compute_attention(q, k, v, attn_mask=None, sliding_window=None):
    """q [B,S,Hq,D], k/v [B,T,Hq,D] (already GQA-expanded) -> [B,Hq,S,D] in q.dtype.
    sliding_window: the local-layer window (llama.rs:1086-1091); like the reference, single-shot and only
    meaningful for q_len == k_len (the mask is [q_len, q_len]) or q_len == 1 (where it is a single zero)."""
    D = q.shape[-1]
    scale = 1.0 / (float(D) ** 0.5)
    kind = q.dtype
    q = q.transpose(1, 2).contiguous()
    k_t = k.transpose(1, 2).transpose(2, 3).contiguous()
    v = v.transpose(1, 2).contiguous()
    if kind != torch.float32:
        q, k_t, v = q.float(), k_t.float(), v.float()
    q_len, k_len = q.shape[2], k_t.shape[3]

    def one(qc, start):
        scores = qc.matmul(k_t) * scale
        if attn_mask is not None:
            scores = scores + attn_mask.float()
        elif q_len > 1:
            m = torch.ones(qc.shape[2], k_len).tril(k_len - q_len + start)
            scores = scores.masked_fill(m.eq(0.0), -10000.0)
        if sliding_window is not None:
            scores = scores + sliding_window_mask(q_len, sliding_window, scores.dtype)  # broadcast_add
        return scores.softmax(-1, dtype=torch.float32).matmul(v)

    if attn_mask is not None or sliding_window is not None or q_len <= ATTN_CHUNK:
        out = one(q, 0)
    else:
        out = torch.cat([one(q[:, :, s:s + ATTN_CHUNK], s) for s in range(0, q_len, ATTN_CHUNK)], 2)
    return out.to(kind)


def qwen35_attention(q, k_full, v_full):
    """q [B,S,Hq,D]; k/v [B,T,Hkv,D]; returns [B,S,Hq,D] in q.dtype (bf16 PV)."""
    dtype = q.dtype
    Hq, Hkv = q.shape[2], k_full.shape[2]
    k_exp = k_full.repeat_interleave(Hq // Hkv, 2)
    v_exp = v_full.repeat_interleave(Hq // Hkv, 2)
    scale = 1.0 / (float(q.shape[-1]) ** 0.5)
    q_p = q.permute(0, 2, 1, 3).float().contiguous()
    k_p = k_exp.permute(0, 2, 3, 1).float().contiguous()
    v_d = v_exp.permute(0, 2, 1, 3).float().contiguous().to(dtype)
    q_len, kv_len = q_p.shape[2], k_p.shape[3]
    outs = []
    for s in range(0, q_len, ATTN_CHUNK):
        qc = q_p[:, :, s:s + ATTN_CHUNK]
        scores = qc.matmul(k_p) * scale
        if q_len > 1:
            m = torch.ones(qc.shape[2], kv_len).tril(kv_len - q_len + s)
            scores = scores.masked_fill(m.eq(0.0), -10000.0)
        outs.append(scores.softmax(-1, dtype=torch.float32).to(dtype).matmul(v_d))
    return torch.cat(outs, 2).permute(0, 2, 1, 3).contiguous()


def batched_mask(start_positions, q_len):
    """Additive mask [B,1,q,kv_max]: 0 where j <= sp_r+i and j < kv_len_r, else -1e9."""
    kv_lens = [sp + q_len for sp in start_positions]
    kv_max = max(kv_lens)
    mask = torch.zeros(len(start_positions), 1, q_len, kv_max)
    cols = torch.arange(kv_max)
    for r, sp in enumerate(start_positions):
        for i in range(q_len):
            valid = cols.le(sp + i).logical_and(cols.lt(kv_lens[r]))
            mask[r, 0, i] = valid.logical_not().float() * -1.0e9
    return mask


def decode_attention_int8(q, k_codes, v_codes, k_scales, v_scales, seq_lens=None):
    """One decode step through the reference's op sequence.

    q [B,1,Hq,D] bf16; codes [B,T,Hkv,D] int8; scales [B,T,Hkv]; seq_lens: list or None
    (None = every row uses all T tokens).  Returns [B,1,Hq,D] in q.dtype.
    Timed region of the CPU baseline: dequant (get), GQA expand, attention.
    """
    k = dequant_view_int8(k_codes, k_scales, q.dtype)
    v = dequant_view_int8(v_codes, v_scales, q.dtype)
    Hq = q.shape[2]
    k, v = expand_kv_for_gqa(k, Hq), expand_kv_for_gqa(v, Hq)
    mask = None
    if seq_lens is not None:
        mask = batched_mask([int(n) - 1 for n in seq_lens], 1)[..., : k.shape[1]]
        if mask.shape[-1] < k.shape[1]:
            k, v = k[:, : mask.shape[-1]], v[:, : mask.shape[-1]]
    return compute_attention(q, k, v, mask).transpose(1, 2)


def decode_attention_fp8(q, k_codes, v_codes, k_scales, v_scales):
    k = dequant_view_fp8(k_codes, k_scales, q.dtype)
    v = dequant_view_fp8(v_codes, v_scales, q.dtype)
    return qwen35_attention(q, k, v)


def deltanet_decode_step(q_t, k_t, v_t, g_t, b_t, state):
    """fp32 tensors: q_t,k_t [B,nv,dk] (expanded, normalised, q scaled); v_t [B,nv,dv];
    g_t,b_t [B,nv]; state [B,nv,dk,dv].  Returns (out [B,nv,dv], new state)."""
    B, nv, dk, dv = state.shape
    state = state * g_t.exp().reshape(B, nv, 1, 1)
    kv_mem = k_t.reshape(B * nv, 1, dk).bmm(state.reshape(B * nv, dk, dv)).reshape(B, nv, dv)
    delta = (v_t - kv_mem) * b_t.unsqueeze(-1)
    state = state + k_t.unsqueeze(-1) * delta.unsqueeze(-2)
    out = q_t.reshape(B * nv, 1, dk).bmm(state.reshape(B * nv, dk, dv)).reshape(B, nv, dv)
    return out, state


def rope_tables(dim, base, length, dtype=torch.bfloat16):
    """sin/cos tables [length, dim/2]: fp32 throughout, cast at the end (rope.rs:100-122)."""
    half = dim // 2
    positions = torch.arange(half, dtype=torch.float32)
    exponents = positions * 2.0 / float(dim)
    inv_freq = torch.full([half], float(base), dtype=torch.float32).pow(-exponents)
    pos = torch.arange(length, dtype=torch.float32)
    angles = pos.unsqueeze(-1).matmul(inv_freq.unsqueeze(0))
    return angles.sin().to(dtype), angles.cos().to(dtype)


def rope_apply(x, sin_full, cos_full, position_ids):
    """x [B, S, H, D] in the tables' dtype; position_ids int64 [S] (rope.rs:150-248): index_select on the
    tables, unsqueeze the head axis, then x1*cos - x2*sin and x1*sin + x2*cos as separate tensor ops."""
    half = x.shape[-1] // 2
    sin = sin_full.index_select(0, position_ids).unsqueeze(1).unsqueeze(0)
    cos = cos_full.index_select(0, position_ids).unsqueeze(1).unsqueeze(0)
    x1 = x.narrow(-1, 0, half)
    x2 = x.narrow(-1, half, half)
    sin_e = sin.expand_as(x1)
    cos_e = cos.expand_as(x1)
    x1r = x1 * cos_e - x2 * sin_e
    x2r = x1 * sin_e + x2 * cos_e
    return torch.cat([x1r, x2r], -1)


def qk_norm_llama(x, weight, eps=1e-6):
    """LlamaAttention::apply_qk_norm (llama.rs:929-991, Gemma3): per-head RMS norm in the tensor dtype, every op a
    separate libtorch op.  x [B, S, H, D]; weight [H * D] (reshaped to [1, 1, H, D]) or [D]."""
    H, D = x.shape[-2], x.shape[-1]
    w = weight.reshape(H, D).unsqueeze(0).unsqueeze(0) if weight.numel() == H * D else weight.reshape(1, 1, 1, D)
    x2 = x.square()
    mean = x2.mean(dim=-1, keepdim=True, dtype=x.dtype)
    rrms = (mean + eps).reciprocal().sqrt()
    return (x * rrms) * w


def qk_norm_qwen35(x, weight_f32, eps):
    """Qwen3_5Model::apply_qknorm (qwen3_5.rs:1077-1091): fp32, (1 + w), one cast back.  x [B, S, H, D]; weight fp32 [D]."""
    shp = x.shape
    D = shp[-1]
    flat = x.reshape(-1, D)
    f = flat.float()
    mean_sq = (f * f).mean(dim=-1, keepdim=True, dtype=torch.float32)
    rrms = (mean_sq + eps).rsqrt()
    normed = f * rrms
    return (normed * (weight_f32.reshape(1, D) + 1.0)).to(x.dtype).reshape(shp)


def deltanet_prepare(mixed_qkv, conv_weight, conv_state, a_in, b_in, neg_a_exp, dt_bias):
    """GatedDeltaNetLayer::forward between the projection and the delta rule (qwen3_5.rs:629-686): depthwise
    causal conv1d over [state | x] + SiLU in the model dtype, g and beta in fp32.  mixed_qkv [B,S,C];
    conv_weight [C,1,K]; conv_state [B,C,K-1] or None.  Returns (conv_out [B,S,C], new_state, g, beta)."""
    B, S, C = mixed_qkv.shape
    ks = conv_weight.shape[-1]
    x_t = mixed_qkv.permute(0, 2, 1)
    if conv_state is None:
        conv_state = torch.zeros(B, C, ks - 1, dtype=mixed_qkv.dtype)
    padded = torch.cat([conv_state, x_t], 2)
    new_state = padded.narrow(2, padded.shape[2] - (ks - 1), ks - 1).contiguous()
    conv_out = torch.nn.functional.conv1d(padded, conv_weight, None, 1, 0, 1, C)
    conv_out = torch.nn.functional.silu(conv_out).permute(0, 2, 1)
    g = neg_a_exp * torch.nn.functional.softplus(a_in.float() + dt_bias)
    beta = b_in.float().sigmoid()
    return conv_out, new_state, g, beta


def gated_rmsnorm(x, gate, weight_f32, eps):
    """RMSNormGated::forward (qwen3_5.rs:305-313)."""
    orig = gate.dtype
    x_f = x.float()
    mean_sq = (x_f * x_f).mean(-1, keepdim=True)
    rrms = (mean_sq + eps).rsqrt()
    return (x_f * rrms * weight_f32 * torch.nn.functional.silu(gate.float())).to(orig)

