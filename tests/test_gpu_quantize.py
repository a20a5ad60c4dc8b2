"""GPU parity: quantize-on-write codes and scales must be BIT-EXACT with the CPU oracle."""
import os

import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from conftest import GOLDEN
from gpu_util import DEV, DeviceCache, bf16_from_bits

pytestmark = pytest.mark.gpu


def quant_roundtrip(x, dtype, D, positions=None, start_pos=0, cap=None):
    """x: [B,S,Hkv,D] fp32 numpy (representable in dtype) -> canonical codes/scales from the GPU."""
    B, S, Hkv, _ = x.shape
    cap = cap or (start_pos + S)
    c = DeviceCache(B, Hkv, cap, D)
    src = torch.from_numpy(x).to(DEV).to(dtype).contiguous()
    c.write(src, src.clone(), positions, start_pos)
    torch.cuda.synchronize()
    return c, c.canonical(cap)


def test_golden_rows_fp32_source():
    g = np.load(os.path.join(GOLDEN, "int8_quant.npz"))
    x = g["x"][None, :, None, :]  # [1, rows, 1, 128]
    _, (kc, vc, ks, vs) = quant_roundtrip(x, torch.float32, 128)
    assert np.array_equal(kc[0, :, 0], g["codes"]) and np.array_equal(vc[0, :, 0], g["codes"])
    assert np.array_equal(ks[0, :, 0].view(np.uint32), g["scales"].view(np.uint32))
    assert np.array_equal(vs[0, :, 0].view(np.uint32), g["scales"].view(np.uint32))


def test_golden_rows_bf16_source():
    g = np.load(os.path.join(GOLDEN, "int8_quant.npz"))
    x = oracle.bf16_to_f32(g["x_bf16_bits"])[None, :, None, :]
    _, (kc, _, ks, _) = quant_roundtrip(x, torch.bfloat16, 128)
    assert np.array_equal(kc[0, :, 0], g["codes_bf16"])
    assert np.array_equal(ks[0, :, 0].view(np.uint32), g["scales_bf16"].view(np.uint32))


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_random_with_outliers_bit_exact(D, dtype):
    r = wl.philox(100 + D)
    x = r.standard_normal((3, 37, 4, D)).astype(np.float32)
    m = r.random(x.shape) < 0.01
    x[m] = np.sign(x[m]) * 8
    x = torch.from_numpy(x).to(dtype).float().numpy()  # make it representable in the source dtype
    _, (kc, vc, ks, vs) = quant_roundtrip(x, dtype, D)
    wc, ws = oracle.quant_int8(x)
    assert np.array_equal(kc, wc) and np.array_equal(vc, wc)
    assert np.array_equal(ks.view(np.uint32), ws.view(np.uint32))
    assert np.array_equal(vs.view(np.uint32), ws.view(np.uint32))


def test_extreme_magnitudes_bit_exact():
    r = wl.philox(7)
    x = r.standard_normal((1, 64, 2, 128)).astype(np.float32)
    x[0, :16] *= 1e-30
    x[0, 16:32] *= 1e30
    x[0, 32:40] *= 1e-38  # scales fall into the fp32 subnormal range
    x[0, 40] = 0
    _, (kc, _, ks, _) = quant_roundtrip(x, torch.float32, 128)
    wc, ws = oracle.quant_int8(x)
    assert np.array_equal(ks.view(np.uint32), ws.view(np.uint32))
    assert np.array_equal(kc, wc)


def test_write_positions_only_touch_new_tokens():
    """Quantize-on-write: a decode step writes exactly one token per sequence at its own position."""
    B, Hkv, D, cap = 4, 2, 128, 40
    r = wl.philox(8)
    prompt = r.standard_normal((B, 24, Hkv, D)).astype(np.float32)
    c = DeviceCache(B, Hkv, cap, D, fill=0)
    p = torch.from_numpy(prompt).to(DEV).bfloat16()
    c.write(p, p, None, 0)
    before = [t.clone() for t in (c.k_codes, c.v_codes, c.k_scales, c.v_scales)]
    pos = np.array([24, 3, 39, 0], np.int32)
    new = torch.from_numpy(r.standard_normal((B, 1, Hkv, D)).astype(np.float32)).to(DEV).bfloat16()
    c.write(new, new, torch.from_numpy(pos).to(DEV), 0)
    torch.cuda.synchronize()
    wc, ws = oracle.quant_int8(new.float().cpu().numpy())
    for b in range(B):
        assert np.array_equal(c.k_codes[b, :, pos[b]].cpu().numpy(), wc[b, 0])
        assert np.array_equal(c.k_scales[b, :, pos[b]].cpu().numpy(), ws[b, 0])
        keep = torch.ones(cap, dtype=torch.bool, device=DEV)
        keep[pos[b]] = False
        assert torch.equal(c.k_codes[b][:, keep], before[0][b][:, keep])
        assert torch.equal(c.v_codes[b][:, keep], before[1][b][:, keep])
        assert torch.equal(c.k_scales[b][:, :cap][:, keep], before[2][b][:, :cap][:, keep])


def test_device_positions_past_capacity_are_skipped():
    B, Hkv, D, cap = 2, 2, 128, 8
    c = DeviceCache(B, Hkv, cap, D, fill=5)
    new = torch.ones(B, 2, Hkv, D, device=DEV, dtype=torch.bfloat16)
    c.write(new, new, torch.tensor([7, 8], dtype=torch.int32, device=DEV), 0)  # row 0: slot 7 ok, 8 skipped
    torch.cuda.synchronize()
    assert (c.k_codes[0, :, 7] == 127).all() and (c.k_codes[0, :, :7] == 5).all()
    assert (c.k_codes[1] == 5).all()


def test_scalar_overflow_is_an_error():
    c = DeviceCache(1, 2, 8, 128)
    new = torch.ones(1, 4, 2, 128, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(hb.HsError) as e:
        c.write(new, new, None, 6)
    assert e.value.code == hb.HS_ERR_OVERFLOW and "Cache overflow" in str(e.value)


def test_dense_view_matches_oracle_dequant():
    r = wl.philox(9)
    x = r.standard_normal((2, 19, 3, 128)).astype(np.float32)
    c, (kc, vc, ks, vs) = quant_roundtrip(x, torch.float32, 128)
    out = torch.empty(2, 19, 3, 128, dtype=torch.float32, device=DEV)
    hb.kv_dequantize(c.k_codes, c.k_scales, False, c.layout, 0, out)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), oracle.dequant_int8(kc, ks))
    outb = torch.empty(2, 19, 3, 128, dtype=torch.bfloat16, device=DEV)
    hb.kv_dequantize(c.k_codes, c.k_scales, False, c.layout, 0, outb)
    want = torch.from_numpy(oracle.dequant_int8(kc, ks)).bfloat16()
    assert torch.equal(outb.cpu(), want)


# ------------------------------------------------------------------ fp8
def test_fp8_golden_and_calibration():
    g = np.load(os.path.join(GOLDEN, "fp8_quant.npz"))
    x = g["x"]
    B, S, H, D = x.shape
    c = DeviceCache(B, H, S + 2, D, fp8=True)
    src = torch.from_numpy(x).to(DEV)
    hb.kv_fp8_calibrate(src, src, c.k_scales, c.v_scales)
    c.write(src, src, None, 0)
    late = torch.from_numpy(g["x_late"]).to(DEV)
    c.write(late, late, None, S)
    torch.cuda.synchronize()
    kc, vc, ks, vs = c.canonical(S + 2)
    assert np.array_equal(ks.view(np.uint32), g["scales"].view(np.uint32))
    assert np.array_equal(kc[:, :S], g["codes"]) and np.array_equal(vc[:, :S], g["codes"])
    assert np.array_equal(kc[:, S:], g["codes_late"])


def test_fp8_all_bf16_inputs_bit_exact():
    """Every bf16 bit pattern through the device encoder (scale 1.0 -> clamp to +-448 then convert)."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = oracle.bf16_to_f32(bits)
    finite = np.isfinite(x)
    x = x[finite].reshape(1, -1, 1, 128)  # 65280 finite patterns = 510 rows
    S = x.shape[1]
    c = DeviceCache(1, 1, S, 128, fp8=True)
    c.k_scales.fill_(1.0)
    c.v_scales.fill_(0.37)
    src = torch.from_numpy(x).to(DEV).bfloat16()
    c.write(src, src, None, 0)
    torch.cuda.synchronize()
    kc, vc, _, _ = c.canonical(S)
    assert np.array_equal(kc, oracle.quant_fp8(x, np.array([[1.0]], np.float32)))
    assert np.array_equal(vc, oracle.quant_fp8(x, np.array([[0.37]], np.float32)))


def test_fp8_dense_view():
    r = wl.philox(10)
    x = (r.standard_normal((2, 9, 2, 128)) * 0.5).astype(np.float32)
    c = DeviceCache(2, 2, 9, 128, fp8=True)
    src = torch.from_numpy(x).to(DEV)
    hb.kv_fp8_calibrate(src, src, c.k_scales, c.v_scales)
    c.write(src, src, None, 0)
    out = torch.empty(2, 9, 2, 128, dtype=torch.float32, device=DEV)
    hb.kv_dequantize(c.v_codes, c.v_scales, True, c.layout, 1, out)
    torch.cuda.synchronize()
    kc, vc, ks, vs = c.canonical(9)
    assert np.array_equal(out.cpu().numpy(), oracle.dequant_fp8(vc, vs))


def _misaligned(t):
    """The same values in a contiguous tensor whose address is only element-aligned (not 16-byte aligned)."""
    buf = torch.empty(t.numel() + 1, dtype=t.dtype, device=t.device)
    out = buf[1:].view(t.shape)
    out.copy_(t)
    assert out.is_contiguous() and out.data_ptr() % 16 != 0
    return out


@pytest.mark.parametrize("fp8", [False, True])
def test_sources_without_16_byte_alignment_give_the_same_bits(fp8):
    """Tensors that do not meet the wide kernels' alignment take the one-row-per-wavefront kernels: same cache."""
    B, S, Hkv, D = 2, 21, 3, 128
    r = wl.philox(31)
    k = torch.from_numpy(r.standard_normal((B, S, Hkv, D)).astype(np.float32)).to(DEV).bfloat16()
    v = torch.from_numpy(r.standard_normal((B, S, Hkv, D)).astype(np.float32)).to(DEV).bfloat16()
    caches = []
    for ks, vs in ((k, v), (_misaligned(k), _misaligned(v))):
        c = DeviceCache(B, Hkv, S, D, fp8=fp8)
        if fp8:
            hb.kv_fp8_calibrate(ks, vs, c.k_scales, c.v_scales)
        c.write(ks, vs)
        caches.append(c)
    torch.cuda.synchronize()
    a, m = caches
    for name in ("k_codes", "v_codes", "k_scales", "v_scales"):
        assert torch.equal(getattr(a, name), getattr(m, name)), name
    # dense view into an output that is not 16-byte aligned
    want = torch.empty(B, S, Hkv, D, dtype=torch.bfloat16, device=DEV)
    got = _misaligned(want)
    hb.kv_dequantize(a.k_codes, a.k_scales, fp8, a.layout, 0, want)
    hb.kv_dequantize(a.k_codes, a.k_scales, fp8, a.layout, 0, got)
    torch.cuda.synchronize()
    assert torch.equal(want, got)


def test_rope_without_16_byte_alignment_gives_the_same_bits():
    B, S, H, D = 2, 9, 4, 128
    r = wl.philox(32)
    x = torch.from_numpy(r.standard_normal((B, S, H, D)).astype(np.float32)).to(DEV).bfloat16()
    ang = torch.from_numpy(r.random((S, D // 2)).astype(np.float32) * 6.0).to(DEV)
    sin, cos = ang.sin().bfloat16().contiguous(), ang.cos().bfloat16().contiguous()
    want = torch.empty_like(x)
    hb.rope_apply(x, sin, cos, want)
    got = _misaligned(want)
    hb.rope_apply(_misaligned(x), sin, cos, got)
    torch.cuda.synchronize()
    assert torch.equal(want, got)
