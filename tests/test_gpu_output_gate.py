"""The output gate of the Qwen3.5 full-attention layers inside the attention launches (hs_kv_layout.out_gate;
qwen3_5.rs:1056-1059: ctx * gate.sigmoid() on bf16 tensors).  Each case runs the call without the gate, applies the
oracle's gate to its bf16 output on the CPU, and compares with the gated call: the same bits, except where the device's
and libm's exp differ in the last fp32 bit of a sigmoid and that flips a bf16 rounding (one ulp, rare)."""
import numpy as np
import pytest
import torch

import oracle
from hyprstream_amd import bindings as hb
from hyprstream_amd import workloads as wl
from gpu_util import DEV, bf16_from_bits
from test_gpu_decode import build_cache

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _check(gated, plain, gate):
    want = oracle.output_gate_bf16(plain.float().cpu().numpy(), _bits(gate))
    got = _bits(gated)
    key = lambda u: np.where(u.astype(np.int32) & 0x8000, -(u.astype(np.int32) & 0x7fff), u.astype(np.int32) & 0x7fff)
    d = np.abs(key(got) - key(want))
    assert d.max() <= 1 and (d != 0).mean() < 5e-3, (int(d.max()), float((d != 0).mean()))
    assert not np.array_equal(got, _bits(plain))  # the gate did something


def _clone(layout):
    return type(layout).from_buffer_copy(layout)


def _with_gate(layout, gate):
    lay = _clone(layout)
    lay.out_gate = gate.data_ptr()
    return lay


@pytest.mark.parametrize("B,T,hint,D,fp8", [(64, 300, False, 128, False),   # one chunk: written by the attention kernel
                                             (3, 2500, False, 128, False),   # split: written by the merge kernel
                                             (9, 1800, True, 128, False),    # balanced split
                                             (4, 900, False, 256, True), (5, 700, False, 64, False)])
def test_decode(B, T, hint, D, fp8):
    Hq, Hkv = 8, 2
    case = wl.decode_case(5100 + B, B, Hq, Hkv, D, T, ragged=True, min_len=1)
    c = build_cache(case, Hkv, D, fp8=fp8)
    lens_np = case["seq_lens"]
    lens = torch.from_numpy(lens_np).to(DEV)
    q = bf16_from_bits(case["q_bits"]).to(DEV)
    gate = (2 * torch.randn(B, Hq, D, generator=torch.Generator().manual_seed(B))).to(torch.bfloat16).to(DEV)
    lay = _clone(c.layout)
    if hint:
        lay.total_tokens_hint = int(lens_np.sum())
        assert hb.decode_num_chunks(B, Hkv, T, lay.total_tokens_hint) > 1
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, T), dtype=torch.uint8, device=DEV)
    outs = []
    for layout in (lay, _with_gate(lay, gate)):
        out = torch.full((B, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        hb.decode_attn(q, c.k_codes, c.v_codes, c.k_scales, c.v_scales, layout, lens, out, ws, Hkv, T, 1.0 / np.sqrt(D), fp8=fp8)
        torch.cuda.synchronize()
        outs.append(out)
    _check(outs[1], outs[0], gate)


@pytest.mark.parametrize("mode", ["plain", "key-split", "bf16-copy"])
@pytest.mark.parametrize("D,Hq,Hkv,hist,S", [(128, 8, 2, 0, 70), (128, 32, 8, 200, 130), (256, 8, 2, 64, 64), (64, 6, 2, 33, 100)])
def test_prefill(D, Hq, Hkv, hist, S, mode):
    """The gate is applied by whichever workgroup stores the output: the tile's own, the one that merges a key split's
    runs, or the instance that reads the history from the bf16 copy."""
    if mode == "bf16-copy" and D != 128:
        pytest.skip("the copy serves head_dim 128")
    B, T = 2, hist + S
    extra = lambda: {}
    if mode == "key-split":
        extra = lambda: dict(columns=0, key_splits=3, split_workspace=hb.prefill_split_workspace(B, max(S, hist, 1), Hq, Hkv, D))
    elif mode == "bf16-copy":
        extra = lambda: dict(columns=256, key_splits=1, shadow=shadows[-1])
    shadows = []
    r = wl.philox(5200 + D)
    t = lambda *s: torch.from_numpy(r.standard_normal(s).astype(np.float32)).to(torch.bfloat16).to(DEV)
    q, k, v = t(B, T, Hq, D), t(B, T, Hkv, D), t(B, T, Hkv, D)
    gate = 2 * t(B, S, Hq, D)
    lay = hb.contiguous_layout(Hkv, T, D)
    outs = []
    for use_gate in (False, True):
        kc = torch.zeros(B, Hkv, T, D, dtype=torch.int8, device=DEV)
        vc = torch.zeros_like(kc)
        ks = torch.zeros(B, Hkv, lay.scale_stride_head, dtype=torch.float32, device=DEV)
        vs = torch.zeros_like(ks)
        if mode == "bf16-copy":
            shadows.append(hb.prefill_shadow(B, Hkv, D, T))
        if hist:
            o0 = torch.empty(B, hist, Hq, D, dtype=torch.bfloat16, device=DEV)
            hb.prefill_attn(q[:, :hist].contiguous(), k[:, :hist].contiguous(), v[:, :hist].contiguous(), kc, vc, ks, vs, lay, 0, o0,
                            1.0 / np.sqrt(D), True, **extra())
        out = torch.full((B, S, Hq, D), float("nan"), dtype=torch.bfloat16, device=DEV)
        hb.prefill_attn(q[:, hist:].contiguous(), k[:, hist:].contiguous(), v[:, hist:].contiguous(), kc, vc, ks, vs,
                        _with_gate(lay, gate) if use_gate else lay, hist, out, 1.0 / np.sqrt(D), True, **extra())
        torch.cuda.synchronize()
        outs.append((out, kc.clone(), ks.clone()))
    _check(outs[1][0], outs[0][0], gate)
    assert torch.equal(outs[0][1], outs[1][1]) and torch.equal(outs[0][2], outs[1][2])  # the cache write is unaffected
