"""Regenerate the golden vectors in this folder:  python tests/golden/make_golden.py

The expected outputs are computed with libtorch CPU ops (PyTorch), the same
arithmetic provider the reference reaches through tch-rs -- NOT with the C
oracle and not with anything from this repository's kernels:

  int8_quant.npz   x.abs().amax(-1) / 127, torch.round(x / s) on hand-built hard rows
  fp8_codec.npz    Tensor.to(float8_e4m3fn) over all 65536 bf16 bit patterns, and the
                   fp32 value of each of the 256 codes
  fp8_quant.npz    per-(sequence, head) scale amax/448, clamp, convert
  attention.npz    the reference's op sequence (transpose/contiguous, fp32 upcast, matmul,
                   scale, mask, softmax, matmul; llama.rs:1023-1119) on small cases
  attention_window.npz  the same with the sliding-window mask of local layers (tril(0) * triu(1 - window) turned into
                   an additive -10000 mask and added to the scores; llama.rs:1086-1091, 1123-1155) for prompts on an
                   empty cache, windows 1, 4, 7, 16 and larger than the prompt
  deltanet.npz     the reference's decode-step op sequence (qwen3_5.rs:725-751) iterated
                   over a few tokens
  rope.npz         the reference's table construction and rotation op sequence (rope.rs:100-122,
                   206-248) on bf16 and fp32 tensors, bases 10000 and 1e6, positions up to 8191

  qknorm.npz       the two per-head RMS norms that run on q and k before the rotary embedding: Llama/Gemma3's
                   bf16 op chain (llama.rs:929-991) and Qwen3.5's fp32 (1 + w) form (qwen3_5.rs:1077-1091),
                   head_dim 64 / 128 / 256, per-head and shared weights

Inputs come from numpy's Philox generator so the file is reproducible.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
from oracle import reference_path as ref  # noqa: E402  (torch op sequences only)


def gen(stream):
    return np.random.Generator(np.random.Philox(key=0x5EED, counter=stream))


def torch_quant_int8(x):
    a = x.abs().amax(-1)
    s = a / 127.0
    q = torch.round(x / s.unsqueeze(-1)).clamp(-127, 127)
    q = torch.where(s.unsqueeze(-1) > 0, q, torch.zeros_like(q))
    return q.to(torch.int8), s


def make_int8():
    r = gen(1)
    rows = []
    rows.append(r.standard_normal((24, 128)).astype(np.float32))
    x = r.standard_normal((8, 128)).astype(np.float32)  # 1% outliers at 8 sigma
    idx = r.random((8, 128)) < 0.01
    x[idx] = np.sign(x[idx]) * 8.0
    rows.append(x)
    rows.append(np.zeros((1, 128), np.float32))                          # all-zero row
    rows.append((r.standard_normal((4, 128)) * 1e-30).astype(np.float32))  # tiny: scale is subnormal-ish
    rows.append((r.standard_normal((4, 128)) * 1e30).astype(np.float32))   # huge
    t = np.zeros((1, 128), np.float32)                                   # exact ties: absmax 127 -> s == 1
    t[0, 0] = 127.0
    t[0, 1:] = (np.arange(127) - 63).astype(np.float32) + 0.5
    rows.append(t)
    t2 = t.copy()
    t2[0, 0] = -127.0                                                    # negative extreme element
    rows.append(t2)
    e = np.zeros((1, 128), np.float32)
    e[0, 5] = -3.25                                                      # single non-zero element
    rows.append(e)
    c = np.full((1, 128), 0.1, np.float32)                               # constant row: every element is the max
    rows.append(c)
    x = np.concatenate(rows, 0)
    q, s = torch_quant_int8(torch.from_numpy(x))
    # bf16 sources: widen exactly, then the same ops
    xb = torch.from_numpy(x[:40]).to(torch.bfloat16)
    qb, sb = torch_quant_int8(xb.float())
    np.savez_compressed(os.path.join(HERE, "int8_quant.npz"), x=x, codes=q.numpy(), scales=s.numpy(),
                        x_bf16_bits=xb.view(torch.int16).numpy().view(np.uint16), codes_bf16=qb.numpy(),
                        scales_bf16=sb.numpy())


def make_fp8():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    xb = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    codes = xb.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    all_codes = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    # fp32 inputs that are not bf16-representable: midpoints and near-midpoints between codes
    vals = all_codes[:127].astype(np.float64)  # non-negative finite codes 0..126
    mids = (vals[:-1] + vals[1:]) / 2
    probe = np.concatenate([mids, np.nextafter(mids.astype(np.float32), np.float32(np.inf)),
                            np.nextafter(mids.astype(np.float32), np.float32(-np.inf)),
                            gen(2).standard_normal(4096) * 50]).astype(np.float32)
    probe = np.concatenate([probe, -probe])
    probe_codes = torch.from_numpy(probe).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    np.savez_compressed(os.path.join(HERE, "fp8_codec.npz"), bf16_to_fp8=codes, code_values=all_codes, probe=probe,
                        probe_codes=probe_codes)
    r = gen(3)
    x = (r.standard_normal((2, 9, 3, 128)) * 0.5).astype(np.float32)
    x[1, :, 2] = 0.0  # a head that is all zero
    xt = torch.from_numpy(x)
    amax = xt.abs().amax((1, 3))
    s = amax / 448.0
    y = (xt / s[:, None, :, None]).clamp(-448, 448)
    y = torch.where(s[:, None, :, None] > 0, y, torch.zeros_like(y))
    q = y.to(torch.float8_e4m3fn).view(torch.uint8)
    # later tokens quantized with the calibrated scale must be clamped, not wrapped to NaN
    x2 = (r.standard_normal((2, 2, 3, 128)) * 2.0).astype(np.float32)
    y2 = (torch.from_numpy(x2) / s[:, None, :, None]).clamp(-448, 448)
    y2 = torch.where(s[:, None, :, None] > 0, y2, torch.zeros_like(y2))
    q2 = y2.to(torch.float8_e4m3fn).view(torch.uint8)
    np.savez_compressed(os.path.join(HERE, "fp8_quant.npz"), x=x, scales=s.numpy(), codes=q.numpy(), x_late=x2,
                        codes_late=q2.numpy())


def make_attention():
    r = gen(4)
    out = {}
    # case a: decode, GQA 4, ragged rows through the reference's additive mask
    B, T, Hq, Hkv, D = 3, 41, 8, 2, 128
    q = torch.from_numpy(r.standard_normal((B, 1, Hq, D)).astype(np.float32)).to(torch.bfloat16)
    k = torch.from_numpy(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    v = torch.from_numpy(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    kq, ks = torch_quant_int8(k)
    vq, vs = torch_quant_int8(v)
    lens = [41, 17, 1]
    # dense fp32 dequantized view (no bf16 rounding): isolates the attention math
    kd = kq.float() * ks.unsqueeze(-1)
    vd = vq.float() * vs.unsqueeze(-1)
    mask = ref.batched_mask([n - 1 for n in lens], 1)
    o = ref.compute_attention(q.float(), ref.expand_kv_for_gqa(kd, Hq), ref.expand_kv_for_gqa(vd, Hq), mask)
    out.update(a_q=q.float().numpy(), a_kq=kq.numpy(), a_ks=ks.numpy(), a_vq=vq.numpy(), a_vs=vs.numpy(),
               a_lens=np.array(lens, np.int32), a_out=o.transpose(1, 2).contiguous().numpy())
    # case b: cached prefill, 5 new rows on top of 19 cached, causal tril(k_len - q_len)
    B, T, S, Hq, Hkv, D = 2, 24, 5, 4, 2, 64
    q = torch.from_numpy(r.standard_normal((B, S, Hq, D)).astype(np.float32))
    k = torch.from_numpy(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    v = torch.from_numpy(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    o = ref.compute_attention(q, ref.expand_kv_for_gqa(k, Hq), ref.expand_kv_for_gqa(v, Hq))
    out.update(b_q=q.numpy(), b_k=k.numpy(), b_v=v.numpy(), b_out=o.transpose(1, 2).contiguous().numpy())
    np.savez_compressed(os.path.join(HERE, "attention.npz"), **out)


def make_attention_window():
    r = gen(40)
    out = {}
    for tag, (B, S, Hq, Hkv, D, W) in {"a": (1, 23, 2, 1, 64, 4), "b": (1, 40, 2, 1, 64, 16), "c": (2, 9, 2, 2, 64, 1),
                                          "d": (1, 20, 2, 1, 128, 7), "e": (1, 12, 2, 1, 64, 50)}.items():
        q = torch.from_numpy(r.standard_normal((B, S, Hq, D)).astype(np.float32))
        k = torch.from_numpy(r.standard_normal((B, S, Hkv, D)).astype(np.float32))
        v = torch.from_numpy(r.standard_normal((B, S, Hkv, D)).astype(np.float32))
        o = ref.compute_attention(q, ref.expand_kv_for_gqa(k, Hq), ref.expand_kv_for_gqa(v, Hq), sliding_window=W)
        out.update({tag + "_q": q.numpy(), tag + "_k": k.numpy(), tag + "_v": v.numpy(), tag + "_window": np.int32(W),
                    tag + "_out": o.transpose(1, 2).contiguous().numpy()})
    np.savez_compressed(os.path.join(HERE, "attention_window.npz"), **out)


def make_deltanet():
    r = gen(5)
    B, T, nk, nv, dk, dv = 2, 6, 2, 4, 32, 16
    q = torch.from_numpy(r.standard_normal((B, T, nk, dk)).astype(np.float32))
    k = torch.from_numpy(r.standard_normal((B, T, nk, dk)).astype(np.float32))
    v = torch.from_numpy(r.standard_normal((B, T, nv, dv)).astype(np.float32))
    g = -torch.nn.functional.softplus(torch.from_numpy(r.standard_normal((B, T, nv)).astype(np.float32)))
    beta = torch.sigmoid(torch.from_numpy(r.standard_normal((B, T, nv)).astype(np.float32)))
    state0 = torch.from_numpy(r.standard_normal((B, nv, dk, dv)).astype(np.float32)) * 0.1
    l2 = lambda x: x / x.norm(2.0, -1, True).clamp_min(1e-3)
    qn = l2(q) * (1.0 / dk ** 0.5)
    kn = l2(k)
    rep = nv // nk
    qe, ke = qn.repeat_interleave(rep, 2), kn.repeat_interleave(rep, 2)
    st = state0.clone()
    outs = []
    for t in range(T):
        o, st = ref.deltanet_decode_step(qe[:, t], ke[:, t], v[:, t], g[:, t], beta[:, t], st)
        outs.append(o)
    np.savez_compressed(os.path.join(HERE, "deltanet.npz"), q=q.numpy(), k=k.numpy(), v=v.numpy(), g=g.numpy(),
                        beta=beta.numpy(), state0=state0.numpy(), out=torch.stack(outs, 1).numpy(),
                        state=st.numpy())


def make_rope():
    r = gen(6)
    out = {}
    for tag, base, D in (("a", 10000.0, 128), ("b", 1000000.0, 128), ("c", 10000.0, 64)):
        L = 8192
        pos = np.concatenate([[0, 1, 2, 255, 256, 257], r.integers(0, L, 10), [L - 1]]).astype(np.int64)
        S, H = len(pos), 2
        x = torch.from_numpy(r.standard_normal((1, S, H, D)).astype(np.float32))
        x[0, 0, 0, :4] = torch.tensor([0.0, -0.0, 8.0, -3.5])
        for dt_name, dt in (("bf16", torch.bfloat16), ("f32", torch.float32)):
            sin, cos = ref.rope_tables(D, base, L, dt)
            xd = x.to(dt)
            y = ref.rope_apply(xd, sin, cos, torch.from_numpy(pos))
            sel = torch.from_numpy(pos)
            if dt == torch.bfloat16:
                bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
                out[f"{tag}_{dt_name}_x"], out[f"{tag}_{dt_name}_y"] = bits(xd), bits(y)
                out[f"{tag}_{dt_name}_sin"], out[f"{tag}_{dt_name}_cos"] = bits(sin.index_select(0, sel)), bits(cos.index_select(0, sel))
            else:
                out[f"{tag}_{dt_name}_x"], out[f"{tag}_{dt_name}_y"] = xd.numpy(), y.numpy()
                out[f"{tag}_{dt_name}_sin"], out[f"{tag}_{dt_name}_cos"] = sin.index_select(0, sel).numpy(), cos.index_select(0, sel).numpy()
        out[f"{tag}_pos"] = pos
        out[f"{tag}_base"] = np.float64(base)
    np.savez_compressed(os.path.join(HERE, "rope.npz"), **out)


def make_qknorm():
    r = gen(9)
    out = {}
    for D in (64, 128, 256):
        H, rows = 3, 24
        x = torch.from_numpy((r.standard_normal((1, rows, H, D)) * r.random((1, rows, H, 1)) * 3).astype(np.float32)).to(torch.bfloat16)
        x[0, 0, 0] = 0  # an all-zero head: rrms = 1/sqrt(eps), output zero
        x[0, 1, 1] *= 1e-4
        w1 = torch.from_numpy((1.0 + 0.2 * r.standard_normal((H, D))).astype(np.float32)).to(torch.bfloat16)
        w1s = w1[0].clone()
        w2 = torch.from_numpy((0.05 * r.standard_normal(D)).astype(np.float32))
        bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
        out["x_%d" % D] = bits(x[0])
        out["w1_%d" % D] = bits(w1)
        out["w2_%d" % D] = w2.numpy()
        out["llama_%d" % D] = bits(ref.qk_norm_llama(x, w1.reshape(-1))[0])
        out["llama_shared_%d" % D] = bits(ref.qk_norm_llama(x, w1s)[0])
        out["qwen_%d" % D] = bits(ref.qk_norm_qwen35(x, w2, 1e-6)[0])
    np.savez_compressed(os.path.join(HERE, "qknorm.npz"), **out)


if __name__ == "__main__":
    make_rope()
    make_int8()
    make_fp8()
    make_attention()
    make_attention_window()
    make_deltanet()
    make_qknorm()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))
