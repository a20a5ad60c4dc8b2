"""Edge cases through the C ABI: empty problems are accepted and touch nothing; rows holding NaN or infinities
quantize exactly as the oracle says (a NaN never becomes the row maximum and maps to code 0)."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from gpu_util import DEV, DeviceCache

pytestmark = pytest.mark.gpu


def test_empty_problems_are_no_ops():
    Hkv, D, Hq = 2, 128, 8
    c = DeviceCache(1, Hkv, 64, D, fill=7)
    e4 = lambda *s: torch.empty(*s, dtype=torch.bfloat16, device=DEV)
    hb.kv_quantize_int8(e4(1, 0, Hkv, D), e4(1, 0, Hkv, D), c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, None, 0)
    hb.kv_quantize_int8(e4(0, 5, Hkv, D), e4(0, 5, Hkv, D), c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, None, 0)
    out = torch.full((0, Hq, D), 1.0, dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(256, dtype=torch.uint8, device=DEV)
    hb.decode_attn(e4(0, Hq, D), c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout,
                   torch.empty(0, dtype=torch.int32, device=DEV), out, ws, Hkv, 64, 0.1)
    hb.prefill_attn(e4(1, 0, Hq, D), e4(1, 0, Hkv, D), e4(1, 0, Hkv, D), c.k_codes, c.v_codes, c.k_scales, c.v_scales,
                    c.layout, 0, e4(1, 0, Hq, D), 0.1, True)
    st = torch.zeros(1, 2, 128, 128, device=DEV)
    hb.deltanet_forward(e4(1, 0, 1, 128), e4(1, 0, 1, 128), e4(1, 0, 2, 128), torch.empty(1, 0, 2, device=DEV),
                        torch.empty(1, 0, 2, device=DEV), st, torch.empty(1, 0, 2, 128, device=DEV), 0.1, False)
    torch.cuda.synchronize()
    assert bool((c.k_codes == 7).all()) and bool((c.v_codes == 7).all()) and bool((st == 0).all())


def test_rows_with_nan_and_inf_match_the_oracle():
    D = 128
    x = np.random.default_rng(3).standard_normal((1, 6, 1, D)).astype(np.float32)
    x[0, 0, 0, 5] = np.nan                      # NaN among finite values: ignored by the max, code 0
    x[0, 1, 0, :] = np.nan                      # all NaN: scale 0, codes 0
    x[0, 2, 0, 7] = np.inf                      # +inf: scale inf, finite elements -> 0, inf/inf = NaN -> 0
    x[0, 3, 0, 9] = -np.inf
    x[0, 4, 0, 3], x[0, 4, 0, 4] = np.inf, np.nan
    c = DeviceCache(1, 1, 6, D)
    src = torch.from_numpy(x).to(DEV)
    c.write(src, src.clone())
    torch.cuda.synchronize()
    kc, vc, ks, vs = c.canonical(6)
    wc, ws = oracle.quant_int8(x)
    assert np.array_equal(kc, wc) and np.array_equal(vc, wc)
    assert np.array_equal(ks.view(np.uint32), ws.view(np.uint32)) and np.array_equal(vs.view(np.uint32), ws.view(np.uint32))
    assert ws[0, 1, 0] == 0.0 and np.isinf(ws[0, 2, 0]) and not wc[0, 1].any()


def test_decode_ignores_sequences_marked_empty_or_negative():
    B, Hq, Hkv, D, T = 3, 8, 2, 128, 40
    c = DeviceCache(B, Hkv, T, D)
    r = torch.Generator(device=DEV).manual_seed(1)
    k = torch.randn(B, T, Hkv, D, generator=r, device=DEV).to(torch.bfloat16)
    c.write(k, k.clone())
    q = torch.randn(B, Hq, D, generator=r, device=DEV).to(torch.bfloat16)
    out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    lens = torch.tensor([0, -3, T], dtype=torch.int32, device=DEV)
    hb.decode_attn(q, c.k_codes, c.v_codes, c.k_scales, c.v_scales, c.layout, lens, out, ws, Hkv, T, 0.1)
    torch.cuda.synchronize()
    assert bool((out[:2] == 0).all()) and bool(torch.isfinite(out[2].float()).all()) and bool(out[2].float().abs().sum() > 0)
