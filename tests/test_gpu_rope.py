"""GPU parity of the rotary-embedding entry points (through the C ABI):

  hs_rope_apply               bit-exact with the oracle's op-by-op rounded rotation (bf16 and fp32)
  hs_kv_quantize_int8_rope    codes/scales bit-exact with quantizing the oracle-rotated K; V untouched by RoPE
  hs_decode_step_int8_rope    equals rope_apply(q) + quantize_rope(k_new) + decode attention, and the oracle

Reference: rope.rs:100-122, 206-248 (tables, rotation), llama.rs:598-611 (rotation right before cache.update)."""
import numpy as np
import pytest
import torch

import oracle
from oracle import hs_oracle as orc
from oracle import reference_path as ref
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV, DeviceCache, bf16_from_bits

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _tables(D, base, L, dtype):
    sin, cos = ref.rope_tables(D, base, L, dtype)  # libtorch CPU: test data, not the thing under test
    return sin.contiguous(), cos.contiguous()


@pytest.mark.parametrize("D", [64, 128, 256])
def test_rope_apply_bf16_bit_exact(D):
    r = wl.philox(700 + D)
    B, S, H, L = 2, 19, 5, 1024
    sin, cos = _tables(D, 10000.0, L, torch.bfloat16)
    x = torch.from_numpy(r.standard_normal((B, S, H, D)).astype(np.float32) * 2).to(torch.bfloat16)
    pos0 = np.array([3, 700], np.int32)
    out = torch.empty_like(x, device=DEV)
    hb.rope_apply(x.to(DEV), sin.to(DEV), cos.to(DEV), out, torch.from_numpy(pos0).to(DEV), start_pos=5)
    torch.cuda.synchronize()
    pos = (pos0[:, None] + 5 + np.arange(S, dtype=np.int32)[None]).reshape(-1)
    want = orc.rope_apply_bf16(_bits(x).reshape(B * S, H, D), _bits(sin), _bits(cos), pos).reshape(B, S, H, D)
    assert np.array_equal(_bits(out), want)


def test_rope_apply_f32_bit_exact():
    r = wl.philox(711)
    B, S, H, D, L = 1, 33, 3, 128, 4096
    sin, cos = _tables(D, 1000000.0, L, torch.float32)
    x = torch.from_numpy(r.standard_normal((B, S, H, D)).astype(np.float32))
    out = torch.empty_like(x, device=DEV)
    hb.rope_apply(x.to(DEV), sin.to(DEV), cos.to(DEV), out, None, start_pos=4000)
    torch.cuda.synchronize()
    pos = 4000 + np.arange(S, dtype=np.int32)
    want = orc.rope_apply_f32(x.numpy().reshape(S, H, D), sin.numpy(), cos.numpy(), pos).reshape(B, S, H, D)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("D,rd", [(256, 64), (128, 32), (128, 96), (64, 16)])
def test_partial_rotary_equals_narrow_rope_cat(D, rd):
    """Qwen3.5 rotates the first rotary_dim elements of every head and passes the rest through
    (qwen3_5.rs:977-990: narrow, rope, cat); tables are built for rotary_dim."""
    r = wl.philox(720 + D + rd)
    B, S, H, L = 2, 11, 3, 512
    sin, cos = _tables(rd, 10000000.0, L, torch.bfloat16)
    x = torch.from_numpy(r.standard_normal((B, S, H, D)).astype(np.float32) * 2).to(torch.bfloat16)
    out = torch.full_like(x, float("nan"), device=DEV)
    hb.rope_apply(x.to(DEV), sin.to(DEV), cos.to(DEV), out, None, start_pos=100, rotary_dim=rd)
    # the element-aligned path (one row per wavefront) gives the same bits
    buf = torch.empty(x.numel() + 1, dtype=x.dtype, device=DEV)
    xm = buf[1:].view(x.shape)
    xm.copy_(x)
    out_m = torch.empty_like(out)
    hb.rope_apply(xm, sin.to(DEV), cos.to(DEV), out_m, None, start_pos=100, rotary_dim=rd)
    torch.cuda.synchronize()
    pos = np.tile(100 + np.arange(S, dtype=np.int32), B)
    xb = _bits(x).reshape(B * S, H, D)
    want = xb.copy()
    want[..., :rd] = orc.rope_apply_bf16(np.ascontiguousarray(xb[..., :rd]), _bits(sin), _bits(cos), pos)
    assert np.array_equal(_bits(out).reshape(B * S, H, D), want)
    assert torch.equal(out, out_m)
    # fp32 tensors
    sin32, cos32 = _tables(rd, 10000000.0, L, torch.float32)
    x32 = x.float()
    out32 = torch.empty_like(x32, device=DEV)
    hb.rope_apply(x32.to(DEV), sin32.to(DEV), cos32.to(DEV), out32, None, start_pos=100, rotary_dim=rd)
    torch.cuda.synchronize()
    w32 = x32.numpy().reshape(B * S, H, D).copy()
    w32[..., :rd] = orc.rope_apply_f32(np.ascontiguousarray(w32[..., :rd]), sin32.numpy(), cos32.numpy(), pos)
    assert np.array_equal(out32.cpu().numpy().reshape(B * S, H, D).view(np.uint32), w32.view(np.uint32))


def test_partial_rotary_rejects_bad_rotary_dim():
    x = torch.zeros(1, 2, 2, 128, dtype=torch.bfloat16, device=DEV)
    for rd in (24, 144):
        sin = torch.zeros(8, rd // 2, dtype=torch.bfloat16, device=DEV)
        with pytest.raises(hb.HsError) as e:
            hb.rope_apply(x, sin, sin, torch.empty_like(x), None, 0, rotary_dim=rd)
        assert e.value.code == 1 and "rotary_dim" in str(e.value)


def test_rope_apply_rejects_positions_beyond_the_table():
    x = torch.zeros(1, 4, 2, 128, dtype=torch.bfloat16, device=DEV)
    sin = torch.zeros(6, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(hb.HsError) as e:
        hb.rope_apply(x, sin, sin, torch.empty_like(x), None, start_pos=3)
    assert e.value.code == 1 and "exceed the rotary tables" in str(e.value)


@pytest.mark.parametrize("D", [64, 128])
def test_quantize_with_rope_bit_exact(D):
    r = wl.philox(720 + D)
    B, S, Hkv, L, start = 2, 23, 4, 512, 100
    sin, cos = _tables(D, 10000.0, L, torch.bfloat16)
    k = torch.from_numpy(r.standard_normal((B, S, Hkv, D)).astype(np.float32)).to(torch.bfloat16)
    v = torch.from_numpy(r.standard_normal((B, S, Hkv, D)).astype(np.float32)).to(torch.bfloat16)
    c = DeviceCache(B, Hkv, start + S, D)
    hb.kv_quantize_int8_rope(k.to(DEV), v.to(DEV), sin.to(DEV), cos.to(DEV), c.k_codes, c.v_codes, c.k_scales,
                             c.v_scales, c.layout, None, start)
    torch.cuda.synchronize()
    kc, vc, ks, vs = c.canonical(start + S)
    pos = np.tile(start + np.arange(S, dtype=np.int32), B)
    k_rot = orc.rope_apply_bf16(_bits(k).reshape(B * S, Hkv, D), _bits(sin), _bits(cos), pos).reshape(B, S, Hkv, D)
    wk, wks = oracle.quant_int8(oracle.bf16_to_f32(k_rot))
    wv, wvs = oracle.quant_int8(k.float().numpy() * 0 + v.float().numpy())
    assert np.array_equal(kc[:, start:], wk) and np.array_equal(ks[:, start:].view(np.uint32), wks.view(np.uint32))
    assert np.array_equal(vc[:, start:], wv) and np.array_equal(vs[:, start:].view(np.uint32), wvs.view(np.uint32))
    assert not kc[:, :start].any()  # nothing before start_pos is touched


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("lens", [[300, 300, 300], [1, 129, 700]])
def test_decode_step_with_rope_matches_unfused_and_oracle(lens, D):
    r = wl.philox(740 + len(set(lens)) + D)
    B, Hq, Hkv, L = len(lens), 16, 4, 1024
    T = max(lens)
    sin, cos = _tables(D, 500000.0, L, torch.bfloat16)
    sin_d, cos_d = sin.to(DEV), cos.to(DEV)
    hist_k = torch.from_numpy(r.standard_normal((B, T, Hkv, D)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    hist_v = torch.from_numpy(r.standard_normal((B, T, Hkv, D)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    q = torch.from_numpy(r.standard_normal((B, Hq, D)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    k_new = torch.from_numpy(r.standard_normal((B, 1, Hkv, D)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    v_new = torch.from_numpy(r.standard_normal((B, 1, Hkv, D)).astype(np.float32)).to(torch.bfloat16).to(DEV)
    lens_d = torch.tensor(lens, dtype=torch.int32, device=DEV)
    scale = 1.0 / np.sqrt(D)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)

    def fresh():
        c = DeviceCache(B, Hkv, T, D)
        c.write(hist_k, hist_v)  # history (already "rotated" as far as this test cares)
        return c

    # fused: one call
    c1 = fresh()
    out1 = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=DEV)
    hb.decode_step_rope(q, k_new, v_new, sin_d, cos_d, c1.k_codes, c1.v_codes, c1.k_scales, c1.v_scales, c1.layout,
                        lens_d, out1, ws, Hkv, T, scale)
    # unfused: rotate q, write rotated k at position len-1, plain decode
    c2 = fresh()
    q_rot = torch.empty(B, 1, Hq, D, dtype=torch.bfloat16, device=DEV)
    pos_new = lens_d - 1
    hb.rope_apply(q.view(B, 1, Hq, D), sin_d, cos_d, q_rot, pos_new, 0)
    hb.kv_quantize_int8_rope(k_new, v_new, sin_d, cos_d, c2.k_codes, c2.v_codes, c2.k_scales, c2.v_scales, c2.layout,
                             pos_new, 0)
    out2 = torch.empty_like(out1)
    hb.decode_attn(q_rot.view(B, Hq, D).contiguous(), c2.k_codes, c2.v_codes, c2.k_scales, c2.v_scales, c2.layout, lens_d,
                   out2, ws, Hkv, T, scale)
    torch.cuda.synchronize()
    assert all(bool(torch.equal(a, b)) for a, b in ((c1.k_codes, c2.k_codes), (c1.v_codes, c2.v_codes),
                                                      (c1.k_scales, c2.k_scales), (c1.v_scales, c2.v_scales)))
    assert bool(torch.equal(out1, out2))
    # oracle: rotated q over the caches just checked
    kc, vc, ks, vs = c1.canonical(T)
    q_rot_bits = orc.rope_apply_bf16(_bits(q).reshape(B, Hq, D), _bits(sin), _bits(cos), np.array(lens, np.int32) - 1)
    want = oracle.decode_attn(oracle.bf16_to_f32(q_rot_bits), kc, vc, ks, vs, oracle.FMT_INT8, np.array(lens, np.int32), scale)
    err = np.abs(out1.float().cpu().numpy() - want)
    assert err.max() < 2e-2 and err.mean() < 2e-3
    # and the new token's codes are those of the oracle-rotated k_new
    k_rot = orc.rope_apply_bf16(_bits(k_new).reshape(B, Hkv, D), _bits(sin), _bits(cos), np.array(lens, np.int32) - 1)
    wk, wks = oracle.quant_int8(oracle.bf16_to_f32(k_rot))
    for b, n in enumerate(lens):
        assert np.array_equal(kc[b, n - 1], wk[b]) and np.array_equal(ks[b, n - 1].view(np.uint32), wks[b].view(np.uint32))
