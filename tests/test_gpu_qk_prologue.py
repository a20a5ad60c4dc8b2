"""GPU parity of what the reference runs on q and k between the projections and cache.update -- per-head QK-norm
(llama.rs:929-991 for Gemma3-style models, qwen3_5.rs:1077-1091 for Qwen3.5), then the (partial) rotary embedding
(rope.rs:206-248; llama.rs:589-611, qwen3_5.rs:973-990) -- through the C ABI:

  hs_qk_prologue_apply            bit-exact with the oracle's norm followed by its op-by-op rounded rotation
  hs_kv_quantize_int8_prologue    codes / scales of quantizing the oracle's normalised and rotated K
  hs_decode_step_int8_prologue    = hs_qk_prologue_apply + hs_decode_step_int8 bit for bit, and the oracle
  hs_decode_step_fp8_prologue     = hs_qk_prologue_apply + hs_decode_step_fp8 bit for bit, and the oracle
  prologue -> prefill -> cache    rope(q), rope(k) -> hs_prefill_attn_int8(quantize_on_write) against the oracle's
                                  rotation + causal attention; the cache holds the codes of hs_kv_quantize_int8_rope
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import hs_oracle as orc
from oracle import reference_path as ref
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV, DeviceCache

pytestmark = pytest.mark.gpu
TOL_MAX, TOL_MEAN = 2e-2, 2e-3


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _bf(a):
    return torch.from_numpy(np.asarray(a, np.float32)).to(torch.bfloat16)


def _tables(rd, base, L):
    sin, cos = ref.rope_tables(rd, base, L, torch.bfloat16)  # libtorch CPU: test data
    return sin.contiguous(), cos.contiguous()


def _weights(r, kind, H, D, per_head):
    shape = (H, D) if per_head else (D,)
    if kind == hb.QKNORM_LLAMA:
        return _bf(1.0 + 0.2 * r.standard_normal(shape))
    return torch.from_numpy((0.05 * r.standard_normal(shape)).astype(np.float32))


def _w_np(w, kind):
    return _bits(w) if kind == hb.QKNORM_LLAMA else w.numpy()


def oracle_prologue(x_bits, kind, w, eps, sin, cos, pos, rd):
    """x_bits uint16 [rows, H, D] -> normalised then (partially) rotated rows, the oracle's functions in sequence."""
    y = x_bits if kind == hb.QKNORM_NONE else orc.qk_norm_bf16(x_bits, kind, _w_np(w, kind), eps)
    if sin is None:
        return y
    out = y.copy()
    out[..., :rd] = orc.rope_apply_bf16(np.ascontiguousarray(y[..., :rd]), _bits(sin), _bits(cos), pos)
    return out


@pytest.mark.parametrize("kind", [hb.QKNORM_NONE, hb.QKNORM_LLAMA, hb.QKNORM_QWEN35])
@pytest.mark.parametrize("D,rd", [(64, 64), (128, 128), (256, 64), (256, 256), (128, 32), (128, 96), (256, 160), (64, 16)])
def test_prologue_apply_bit_exact(kind, D, rd):
    r = wl.philox(1000 + 10 * D + rd + kind)
    B, S, Hq, Hkv, L = 2, 13, 6, 2, 512
    sin, cos = _tables(rd, 10000.0, L)
    q = _bf(r.standard_normal((B, S, Hq, D)) * 2)
    k = _bf(r.standard_normal((B, S, Hkv, D)) * r.random((B, S, Hkv, 1)) * 3)
    wq = _weights(r, kind, Hq, D, per_head=True) if kind else None
    wk = _weights(r, kind, Hkv, D, per_head=False) if kind else None
    pos0 = np.array([7, 300], np.int32)
    pro = hb.qk_prologue(kind, 1e-6, wq.to(DEV) if kind else None, wk.to(DEV) if kind else None, sin.to(DEV), cos.to(DEV), rd)
    q_out = torch.full_like(q, float("nan"), device=DEV)
    k_out = torch.full_like(k, float("nan"), device=DEV)
    hb.qk_prologue_apply(q.to(DEV), k.to(DEV), pro, q_out, k_out, torch.from_numpy(pos0).to(DEV), start_pos=2)
    torch.cuda.synchronize()
    pos = (pos0[:, None] + 2 + np.arange(S, dtype=np.int32)[None]).reshape(-1)
    wantq = oracle_prologue(_bits(q).reshape(B * S, Hq, D), kind, wq, 1e-6, sin, cos, pos, rd)
    wantk = oracle_prologue(_bits(k).reshape(B * S, Hkv, D), kind, wk, 1e-6, sin, cos, pos, rd)
    assert np.array_equal(_bits(q_out).reshape(B * S, Hq, D), wantq)
    assert np.array_equal(_bits(k_out).reshape(B * S, Hkv, D), wantk)
    # only k, no rotation: the norm alone
    if kind:
        pro2 = hb.qk_prologue(kind, 1e-6, None, wk.to(DEV))
        k2 = torch.empty_like(k_out)
        hb.qk_prologue_apply(None, k.to(DEV), pro2, None, k2)
        torch.cuda.synchronize()
        assert np.array_equal(_bits(k2).reshape(B * S, Hkv, D), orc.qk_norm_bf16(_bits(k).reshape(B * S, Hkv, D), kind, _w_np(wk, kind), 1e-6))


@pytest.mark.parametrize("kind", [hb.QKNORM_NONE, hb.QKNORM_LLAMA, hb.QKNORM_QWEN35])
@pytest.mark.parametrize("D,rd", [(64, 32), (128, 128), (256, 96)])
def test_prologue_kernels_for_aligned_and_unaligned_buffers_agree(kind, D, rd):
    """16-byte-aligned 16-bit tensors take the kernel that packs several rows into a wavefront, anything else the
    one-row-per-wavefront kernel: the same bits from both (here the same data at an address that is 2 mod 16)."""
    r = wl.philox(1500 + D + rd + kind)
    B, S, Hq, Hkv, L = 3, 7, 5, 3, 64
    sin, cos = _tables(rd, 10000.0, L)
    q = _bf(r.standard_normal((B, S, Hq, D)) * 2).to(DEV)
    k = _bf(r.standard_normal((B, S, Hkv, D))).to(DEV)
    wq = _weights(r, kind, Hq, D, per_head=True).to(DEV) if kind else None
    wk = _weights(r, kind, Hkv, D, per_head=False).to(DEV) if kind else None
    pro = hb.qk_prologue(kind, 1e-5, wq, wk, sin.to(DEV), cos.to(DEV), rd)

    def shifted(t):  # the same values in a buffer whose address is 2 bytes past a 16-byte boundary
        flat = torch.empty(t.numel() + 8, dtype=t.dtype, device=DEV)
        v = flat[1:1 + t.numel()].view(t.shape)
        v.copy_(t)
        assert v.data_ptr() % 16 == 2 and v.is_contiguous()
        return v

    qa, ka = torch.empty_like(q), torch.empty_like(k)
    hb.qk_prologue_apply(q, k, pro, qa, ka, None, 3)
    qu, ku = shifted(torch.zeros_like(q)), shifted(torch.zeros_like(k))
    hb.qk_prologue_apply(shifted(q), shifted(k), pro, qu, ku, None, 3)
    torch.cuda.synchronize()
    assert torch.equal(qa.view(torch.int16), qu.view(torch.int16)) and torch.equal(ka.view(torch.int16), ku.view(torch.int16))
    assert qa.float().abs().sum() > 0


def test_prologue_against_libtorch_op_sequences():
    """The second witness: the reference's libtorch op sequences on the CPU (norm, then narrow + rope + cat).  They can
    differ from the kernel in single elements by one bf16 ulp (host-dependent summation order / rsqrt)."""
    r = wl.philox(1100)
    B, S, H, D, rd, L = 1, 64, 8, 256, 64, 256
    sin, cos = _tables(rd, 10000000.0, L)
    x = _bf(r.standard_normal((B, S, H, D)) * 1.5)
    w = torch.from_numpy((0.05 * r.standard_normal(D)).astype(np.float32))
    pro = hb.qk_prologue(hb.QKNORM_QWEN35, 1e-6, w.to(DEV), None, sin.to(DEV), cos.to(DEV), rd)
    out = torch.empty_like(x, device=DEV)
    hb.qk_prologue_apply(x.to(DEV), None, pro, out, None, None, 0)
    torch.cuda.synchronize()
    normed = ref.qk_norm_qwen35(x, w, 1e-6)
    rot = ref.rope_apply(normed.narrow(-1, 0, rd), sin, cos, torch.arange(S))
    want = torch.cat([rot, normed.narrow(-1, rd, D - rd)], -1)
    diff = _bits(out) != _bits(want)
    assert diff.mean() <= 1e-4
    if diff.any():
        assert np.abs(_bits(out)[diff].astype(np.int32) - _bits(want)[diff].astype(np.int32)).max() == 1


@pytest.mark.parametrize("kind,D,rd", [(hb.QKNORM_LLAMA, 128, 128), (hb.QKNORM_QWEN35, 256, 64), (hb.QKNORM_LLAMA, 64, 64)])
def test_quantize_with_prologue_bit_exact(kind, D, rd):
    r = wl.philox(1200 + D + kind)
    B, S, Hkv, L, start = 2, 21, 4, 512, 90
    sin, cos = _tables(rd, 10000.0, L)
    k = _bf(r.standard_normal((B, S, Hkv, D)) * 2)
    v = _bf(r.standard_normal((B, S, Hkv, D)))
    wk = _weights(r, kind, Hkv, D, per_head=True)
    pro = hb.qk_prologue(kind, 1e-6, None, wk.to(DEV), sin.to(DEV), cos.to(DEV), rd)
    c = DeviceCache(B, Hkv, start + S, D)
    hb.kv_quantize_int8_prologue(k.to(DEV), v.to(DEV), pro, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, None, start)
    torch.cuda.synchronize()
    kc, vc, ks, vs = c.canonical(start + S)
    pos = np.tile(start + np.arange(S, dtype=np.int32), B)
    k_fin = oracle_prologue(_bits(k).reshape(B * S, Hkv, D), kind, wk, 1e-6, sin, cos, pos, rd).reshape(B, S, Hkv, D)
    wkc, wks = oracle.quant_int8(oracle.bf16_to_f32(k_fin))
    wvc, wvs = oracle.quant_int8(v.float().numpy())
    assert np.array_equal(kc[:, start:], wkc) and np.array_equal(ks[:, start:].view(np.uint32), wks.view(np.uint32))
    assert np.array_equal(vc[:, start:], wvc) and np.array_equal(vs[:, start:].view(np.uint32), wvs.view(np.uint32))
    assert not kc[:, :start].any()


@pytest.mark.parametrize("kind,D,rd", [(hb.QKNORM_LLAMA, 128, 128), (hb.QKNORM_QWEN35, 256, 64), (hb.QKNORM_QWEN35, 256, 128),
                                       (hb.QKNORM_LLAMA, 64, 64), (hb.QKNORM_NONE, 128, 32), (hb.QKNORM_LLAMA, 256, 256),
                                       (hb.QKNORM_QWEN35, 128, 0),
                                       # lengths with no lane pattern of their own: partners re-read from the q tensor
                                       (hb.QKNORM_LLAMA, 128, 96), (hb.QKNORM_QWEN35, 128, 16), (hb.QKNORM_NONE, 128, 48),
                                       (hb.QKNORM_QWEN35, 256, 192), (hb.QKNORM_LLAMA, 256, 80), (hb.QKNORM_LLAMA, 64, 48),
                                       (hb.QKNORM_NONE, 64, 16), (hb.QKNORM_QWEN35, 64, 32)])
@pytest.mark.parametrize("lens", [[260, 260, 260], [1, 129, 700]])
def test_decode_step_with_prologue_matches_unfused_and_oracle(lens, kind, D, rd):
    """rd = 0 here means no rotation at all (norm only)."""
    r = wl.philox(1300 + len(set(lens)) + D + rd + kind)
    B, Hq, Hkv, L = len(lens), 16, 4, 1024
    T = max(lens)
    rope = rd > 0
    sin, cos = _tables(rd, 500000.0, L) if rope else (None, None)
    hist_k = _bf(r.standard_normal((B, T, Hkv, D))).to(DEV)
    hist_v = _bf(r.standard_normal((B, T, Hkv, D))).to(DEV)
    q = _bf(r.standard_normal((B, Hq, D)) * 1.7).to(DEV)
    k_new = _bf(r.standard_normal((B, 1, Hkv, D)) * 0.6).to(DEV)
    v_new = _bf(r.standard_normal((B, 1, Hkv, D))).to(DEV)
    wq = _weights(r, kind, Hq, D, per_head=False) if kind else None
    wk = _weights(r, kind, Hkv, D, per_head=True) if kind else None
    pro = hb.qk_prologue(kind, 1e-6, wq.to(DEV) if kind else None, wk.to(DEV) if kind else None,
                         sin.to(DEV) if rope else None, cos.to(DEV) if rope else None, rd)
    lens_d = torch.tensor(lens, dtype=torch.int32, device=DEV)
    scale = 1.0 / np.sqrt(D)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)

    def fresh():
        c = DeviceCache(B, Hkv, T, D)
        c.write(hist_k, hist_v)
        return c

    c1 = fresh()
    out1 = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    hb.decode_step_prologue(q, k_new, v_new, pro, c1.k_codes, c1.v_codes, c1.k_scales, c1.v_scales, c1.layout, lens_d,
                            out1, ws, Hkv, T, scale)
    # unfused: the pre-pass over q and k_new, then the plain fused step
    c2 = fresh()
    q2 = torch.empty(B, 1, Hq, D, dtype=torch.bfloat16, device=DEV)
    k2 = torch.empty(B, 1, Hkv, D, dtype=torch.bfloat16, device=DEV)
    pos_new = lens_d - 1
    hb.qk_prologue_apply(q.view(B, 1, Hq, D), k_new, pro, q2, k2, pos_new, 0)
    out2 = torch.empty_like(out1)
    hb.decode_step(q2.view(B, Hq, D), k2, v_new, c2.k_codes, c2.v_codes, c2.k_scales, c2.v_scales, c2.layout, lens_d,
                   out2, ws, Hkv, T, scale)
    torch.cuda.synchronize()
    assert all(bool(torch.equal(a, b)) for a, b in ((c1.k_codes, c2.k_codes), (c1.v_codes, c2.v_codes),
                                                      (c1.k_scales, c2.k_scales), (c1.v_scales, c2.v_scales)))
    assert bool(torch.equal(out1, out2))
    # oracle: its own norm + rotation of q and k_new, its quantizer, its attention
    pos = np.array(lens, np.int32) - 1
    q_fin = oracle_prologue(_bits(q).reshape(B, Hq, D), kind, wq, 1e-6, sin, cos, pos, rd)
    k_fin = oracle_prologue(_bits(k_new).reshape(B, Hkv, D), kind, wk, 1e-6, sin, cos, pos, rd)
    assert np.array_equal(_bits(q2).reshape(B, Hq, D), q_fin)
    kc, vc, ks, vs = c1.canonical(T)
    wkc, wks = oracle.quant_int8(oracle.bf16_to_f32(k_fin))
    for b, n in enumerate(lens):
        assert np.array_equal(kc[b, n - 1], wkc[b]) and np.array_equal(ks[b, n - 1].view(np.uint32), wks[b].view(np.uint32))
    want = oracle.decode_attn(oracle.bf16_to_f32(q_fin), kc, vc, ks, vs, oracle.FMT_INT8, np.array(lens, np.int32), scale)
    err = np.abs(out1.float().cpu().numpy() - want)
    assert err.max() < TOL_MAX and err.mean() < TOL_MEAN


@pytest.mark.parametrize("kind,D,rd", [(hb.QKNORM_LLAMA, 128, 128), (hb.QKNORM_QWEN35, 256, 64), (hb.QKNORM_LLAMA, 64, 64),
                                       (hb.QKNORM_NONE, 128, 32), (hb.QKNORM_QWEN35, 128, 0), (hb.QKNORM_LLAMA, 128, 96),
                                       (hb.QKNORM_QWEN35, 256, 112)])
@pytest.mark.parametrize("lens", [[260, 260, 260], [1, 129, 700]])
def test_fp8_decode_step_with_prologue_matches_unfused_and_oracle(lens, kind, D, rd):
    """The FP8 cache (per-(sequence, head) scales calibrated on the history): hs_decode_step_fp8_prologue against
    hs_qk_prologue_apply + hs_decode_step_fp8 bit for bit, the new token's codes against the oracle's e4m3 encoder
    applied to the oracle's normalised and rotated k_new, the output against the oracle's attention."""
    r = wl.philox(1400 + len(set(lens)) + D + rd + kind)
    B, Hq, Hkv, L = len(lens), 16, 4, 1024
    T = max(lens)
    rope = rd > 0
    sin, cos = _tables(rd, 1000000.0, L) if rope else (None, None)
    hist_k = _bf(r.standard_normal((B, T, Hkv, D)) * 0.8).to(DEV)
    hist_v = _bf(r.standard_normal((B, T, Hkv, D)) * 0.8).to(DEV)
    q = _bf(r.standard_normal((B, Hq, D)) * 1.7).to(DEV)
    k_new = _bf(r.standard_normal((B, 1, Hkv, D)) * 0.6).to(DEV)
    v_new = _bf(r.standard_normal((B, 1, Hkv, D)) * 0.8).to(DEV)
    wq = _weights(r, kind, Hq, D, per_head=False) if kind else None
    wk = _weights(r, kind, Hkv, D, per_head=True) if kind else None
    pro = hb.qk_prologue(kind, 1e-6, wq.to(DEV) if kind else None, wk.to(DEV) if kind else None,
                         sin.to(DEV) if rope else None, cos.to(DEV) if rope else None, rd)
    lens_d = torch.tensor(lens, dtype=torch.int32, device=DEV)
    scale = 1.0 / np.sqrt(D)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)

    def fresh():
        c = DeviceCache(B, Hkv, T, D, fp8=True)
        hb.kv_fp8_calibrate(hist_k, hist_v, c.k_scales, c.v_scales)
        c.write(hist_k, hist_v)
        return c

    c1 = fresh()
    out1 = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    hb.decode_step_prologue(q, k_new, v_new, pro, c1.k_codes, c1.v_codes, c1.k_scales, c1.v_scales, c1.layout, lens_d,
                            out1, ws, Hkv, T, scale, fp8=True)
    c2 = fresh()
    q2 = torch.empty(B, 1, Hq, D, dtype=torch.bfloat16, device=DEV)
    k2 = torch.empty(B, 1, Hkv, D, dtype=torch.bfloat16, device=DEV)
    hb.qk_prologue_apply(q.view(B, 1, Hq, D), k_new, pro, q2, k2, lens_d - 1, 0)
    out2 = torch.empty_like(out1)
    hb.decode_step(q2.view(B, Hq, D), k2, v_new, c2.k_codes, c2.v_codes, c2.k_scales, c2.v_scales, c2.layout, lens_d,
                   out2, ws, Hkv, T, scale, fp8=True)
    torch.cuda.synchronize()
    assert bool(torch.equal(c1.k_codes, c2.k_codes)) and bool(torch.equal(c1.v_codes, c2.v_codes))
    assert bool(torch.equal(out1, out2))
    pos = np.array(lens, np.int32) - 1
    q_fin = oracle_prologue(_bits(q).reshape(B, Hq, D), kind, wq, 1e-6, sin, cos, pos, rd)
    k_fin = oracle_prologue(_bits(k_new).reshape(B, Hkv, D), kind, wk, 1e-6, sin, cos, pos, rd)
    kc, vc, ks, vs = c1.canonical(T)
    wkc = oracle.quant_fp8(oracle.bf16_to_f32(k_fin).reshape(B, 1, Hkv, D), ks)
    wvc = oracle.quant_fp8(v_new.float().cpu().numpy(), vs)
    for b, n in enumerate(lens):
        assert np.array_equal(kc[b, n - 1], wkc[b, 0]) and np.array_equal(vc[b, n - 1], wvc[b, 0])
    want = oracle.decode_attn(oracle.bf16_to_f32(q_fin), kc, vc, ks, vs, oracle.FMT_FP8, np.array(lens, np.int32), scale)
    err = np.abs(out1.float().cpu().numpy() - want)
    assert err.max() < TOL_MAX and err.mean() < TOL_MEAN


@pytest.mark.parametrize("rd", [24, 136, 8])
def test_decode_step_prologue_rejects_bad_rotary_dim(rd):
    """The rotated length is a multiple of 16 within the head, as for hs_rope_apply_partial and hs_qk_prologue_apply."""
    B, Hq, Hkv, D, T = 1, 4, 1, 128, 64
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
    sin = z(8, 128)
    pro = hb.qk_prologue(hb.QKNORM_NONE, 0.0, None, None, sin, sin, rd)
    c = DeviceCache(B, Hkv, T, D)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    with pytest.raises(hb.HsError) as e:
        hb.decode_step_prologue(z(B, Hq, D), z(B, 1, Hkv, D), z(B, 1, Hkv, D), pro, c.k_codes, c.v_codes, c.k_scales,
                                c.v_scales, c.layout, torch.ones(B, dtype=torch.int32, device=DEV), z(B, Hq, D), ws, Hkv,
                                T, 0.1)
    assert e.value.code == 1 and "rotary_dim" in str(e.value)


@pytest.mark.parametrize("D", [64, 128, 256])
def test_rope_then_prefill_then_cache(D):
    """llama.rs:598-636 for a prompt in two chunks: rotate q and k (rope.rs:206-248), cache.update, attention.  The
    prefill call gets the ROTATED q and k; it attends its own chunk in bf16 and the first chunk through the int8 cache,
    and writes the rotated K's codes."""
    r = wl.philox(1400 + D)
    B, Hq, Hkv, L, C = 2, 8, 2, 1024, 192
    S = 2 * C
    sin, cos = _tables(D, 10000.0, L)
    sin_d, cos_d = sin.to(DEV), cos.to(DEV)
    q, k, v = (_bf(r.standard_normal((B, S, H, D))) for H in (Hq, Hkv, Hkv))
    pro = hb.qk_prologue(hb.QKNORM_NONE, 0.0, None, None, sin_d, cos_d, 0)
    c = DeviceCache(B, Hkv, S, D)
    outs = []
    for i in range(0, S, C):
        qc, kc_, vc_ = (t[:, i:i + C].contiguous().to(DEV) for t in (q, k, v))
        q_rot, k_rot = torch.empty_like(qc), torch.empty_like(kc_)
        hb.qk_prologue_apply(qc, kc_, pro, q_rot, k_rot, None, i)
        o = torch.full((B, C, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        hb.prefill_attn(q_rot, k_rot, vc_, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, i, o, 1.0 / np.sqrt(D), True)
        outs.append(o)
    torch.cuda.synchronize()
    out = torch.cat(outs, 1).float().cpu().numpy()
    # the cache holds what the rope-fused writer writes, which is the oracle's quantizer on the oracle's rotation
    c2 = DeviceCache(B, Hkv, S, D)
    hb.kv_quantize_int8_rope(k.to(DEV), v.to(DEV), sin_d, cos_d, c2.k_codes, c2.v_codes, c2.k_scales, c2.v_scales, c2.layout, None, 0)
    torch.cuda.synchronize()
    assert torch.equal(c.k_codes, c2.k_codes) and torch.equal(c.k_scales, c2.k_scales)
    assert torch.equal(c.v_codes, c2.v_codes) and torch.equal(c.v_scales, c2.v_scales)
    pos = np.tile(np.arange(S, dtype=np.int32), B)
    q_rot = oracle.bf16_to_f32(orc.rope_apply_bf16(_bits(q).reshape(B * S, Hq, D), _bits(sin), _bits(cos), pos)).reshape(B, S, Hq, D)
    k_rot = oracle.bf16_to_f32(orc.rope_apply_bf16(_bits(k).reshape(B * S, Hkv, D), _bits(sin), _bits(cos), pos)).reshape(B, S, Hkv, D)
    kc, vc, ks, vs = c.canonical(S)
    wk, wks = oracle.quant_int8(k_rot)
    assert np.array_equal(kc, wk) and np.array_equal(ks.view(np.uint32), wks.view(np.uint32))
    # chunk 2 attends [dequantized chunk 1 | its own exact rows]; chunk 1 attends itself
    vf = v.float().numpy()
    kd = np.concatenate([oracle.dequant_int8(kc[:, :C], ks[:, :C]), k_rot[:, C:]], 1)
    vd = np.concatenate([oracle.dequant_int8(vc[:, :C], vs[:, :C]), vf[:, C:]], 1)
    want1 = oracle.prefill_attn(q_rot[:, :C], k_rot[:, :C], vf[:, :C], None, None, oracle.FMT_DENSE, np.full(B, C, np.int32), 1.0 / np.sqrt(D))
    want2 = oracle.prefill_attn(q_rot[:, C:], kd, vd, None, None, oracle.FMT_DENSE, np.full(B, S, np.int32), 1.0 / np.sqrt(D))
    err = np.abs(out - np.concatenate([want1, want2], 1))
    assert err.max() < TOL_MAX and err.mean() < TOL_MEAN, (err.max(), err.mean())


@pytest.mark.parametrize("columns", [0, 128, 16, "split3", "split2x128"])
@pytest.mark.parametrize("kind", [hb.QKNORM_NONE, hb.QKNORM_LLAMA, hb.QKNORM_QWEN35])
@pytest.mark.parametrize("D,rd,Hq,Hkv", [(64, 64, 8, 2), (128, 128, 8, 2), (128, 64, 6, 2), (128, 32, 4, 4),
                                         (256, 256, 8, 1), (256, 64, 4, 2), (64, 16, 4, 1)])
def test_prefill_with_the_q_prologue_inside_the_launch(D, rd, Hq, Hkv, kind, columns):
    """hs_kv_layout.prefill_q_prologue: q arrives as projected, the prefill launch runs its QK-norm and rotation.
    Outputs and cache equal, bit for bit, those of hs_qk_prologue_apply on q followed by the plain launch -- a prompt in
    two ragged chunks (S not a multiple of the tile; the second chunk over an int8 history), per-head weights, the
    hinted widths (16 = the sixteen-wavefront instance, head_dim 128 only), and with every query tile's keys split into
    runs (each stages its q pieces in its own record of the workspace: `out` belongs to the merging workgroup)."""
    if columns == 16 and D != 128:
        pytest.skip("the sixteen-wavefront instance serves head_dim 128")
    splits = int(columns[5]) if isinstance(columns, str) else 0  # "split3": three runs of full-width tiles; "split2x128": two of half-width
    columns = (128 if columns.endswith("x128") else 0) if splits else columns
    if columns == 128 and D == 256:
        pytest.skip("head_dim 256 has one width")
    r = wl.philox(9100 + D + rd + 7 * kind + columns + splits)
    B, L = 2, 512
    chunks = [(0, 150), (150, 333)]
    T = 333
    sin, cos = _tables(rd, 10000.0, L)
    wq, wk = _weights(r, kind, Hq, D, True), _weights(r, kind, Hkv, D, False)
    pro = hb.qk_prologue(kind, 1e-6, wq.to(DEV) if kind else None, wk.to(DEV) if kind else None, sin.to(DEV), cos.to(DEV), rd)
    q, k, v = (_bf(r.standard_normal((B, T, H, D))) for H in (Hq, Hkv, Hkv))
    fused, plain = DeviceCache(B, Hkv, T, D), DeviceCache(B, Hkv, T, D)
    extra = {}
    for lo, hi in chunks:
        if splits:
            extra = dict(split_workspace=hb.prefill_split_workspace(B, hi - lo, Hq, Hkv, D), key_splits=splits)
        qc, kc_, vc_ = (t[:, lo:hi].contiguous().to(DEV) for t in (q, k, v))
        q_fin, k_fin = torch.empty_like(qc), torch.empty_like(kc_)
        hb.qk_prologue_apply(qc, kc_, pro, q_fin, k_fin, None, lo)
        want = torch.full_like(qc, float("nan"))
        hb.prefill_attn(q_fin, k_fin, vc_, plain.k_codes, plain.v_codes, plain.k_scales, plain.v_scales, plain.layout, lo,
                        want, 1.0 / np.sqrt(D), True, columns=columns, **extra)
        got = torch.full_like(qc, float("nan"))
        q_before = qc.clone()
        hb.prefill_attn(qc, k_fin, vc_, fused.k_codes, fused.v_codes, fused.k_scales, fused.v_scales, fused.layout, lo,
                        got, 1.0 / np.sqrt(D), True, columns=columns, q_prologue=pro, **extra)
        torch.cuda.synchronize()
        assert torch.equal(qc, q_before)  # q is read, never written
        assert not torch.isnan(want.float()).any()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (lo, hi)
    assert torch.equal(fused.k_codes, plain.k_codes) and torch.equal(fused.v_codes, plain.v_codes)
    assert torch.equal(fused.k_scales, plain.k_scales) and torch.equal(fused.v_scales, plain.v_scales)


def test_prefill_q_prologue_on_ragged_rows_and_fp8():
    """Rows at different positions (hist_lens) rotate their q at their own positions; fp8 history."""
    r = wl.philox(9200)
    B, Hq, Hkv, D, Hmax, S, L = 3, 8, 2, 128, 200, 96, 512
    hist = np.array([200, 0, 77], np.int32)
    sin, cos = _tables(D, 10000.0, L)
    wq = _weights(r, hb.QKNORM_LLAMA, Hq, D, False)
    pro = hb.qk_prologue(hb.QKNORM_LLAMA, 1e-6, wq.to(DEV), wq.to(DEV), sin.to(DEV), cos.to(DEV), 0)
    q, k, v = (_bf(r.standard_normal((B, S, H, D))).to(DEV) for H in (Hq, Hkv, Hkv))
    hk, hv = (_bf(r.standard_normal((B, Hmax, Hkv, D))).to(DEV) for _ in range(2))
    hl = torch.from_numpy(hist).to(DEV)
    outs = []
    for fused in (False, True):
        c = DeviceCache(B, Hkv, Hmax + S, D, fp8=True)
        hb.kv_fp8_calibrate(hk, hv, c.k_scales, c.v_scales)
        hb.kv_quantize_fp8(hk, hv, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, None, 0)
        o = torch.full_like(q, float("nan"))
        if fused:
            hb.prefill_attn(q, k, v, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, Hmax, o, 0.088, True, fp8=True,
                            hist_lens=hl, q_prologue=pro)
        else:
            q_fin = torch.empty_like(q)
            hb.qk_prologue_apply(q, None, pro, q_fin, None, hl, 0)  # positions: each row's first position
            hb.prefill_attn(q_fin, k, v, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, Hmax, o, 0.088, True,
                            fp8=True, hist_lens=hl)
        torch.cuda.synchronize()
        outs.append((o, c.k_codes.clone()))
    assert not torch.isnan(outs[0][0].float()).any()
    assert torch.equal(outs[0][0].view(torch.int16), outs[1][0].view(torch.int16))
    assert torch.equal(outs[0][1], outs[1][1])


def test_prefill_q_prologue_rejections():
    B, S, Hq, Hkv, D = 1, 64, 4, 1, 128
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
    c = DeviceCache(B, Hkv, S, D)
    q, k, o = z(B, S, Hq, D), z(B, S, Hkv, D), z(B, S, Hq, D)
    run = lambda pro, q_=q, o_=o, hist=0: hb.prefill_attn(q_, k, k, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout,
                                                           hist, o_, 0.1, False, q_prologue=pro)
    sin = z(64, 48)
    with pytest.raises(hb.HsError) as e:  # 96 of 128 rotated: not one of the served fractions
        run(hb.qk_prologue(hb.QKNORM_NONE, 0.0, None, None, sin, sin, 96))
    assert e.value.code == 1 and "hs_qk_prologue_apply" in str(e.value)
    full = z(32, 64)
    with pytest.raises(hb.HsError) as e:  # tables shorter than the positions
        run(hb.qk_prologue(hb.QKNORM_NONE, 0.0, None, None, full, full, 0))
    assert e.value.code == 1 and "rotary tables" in str(e.value)
    ok = z(64, 64)
    with pytest.raises(hb.HsError) as e:  # the launch stages the finished q in `out`
        run(hb.qk_prologue(hb.QKNORM_NONE, 0.0, None, None, ok, ok, 0), o_=q)
    assert e.value.code == 1 and "different buffers" in str(e.value)
    with pytest.raises(hb.HsError) as e:  # norm asked for, no weight
        run(hb.qk_prologue(hb.QKNORM_LLAMA, 1e-6, None, None, ok, ok, 0))
    assert e.value.code == 1
