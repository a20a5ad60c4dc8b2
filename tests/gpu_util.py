"""Helpers shared by the GPU parity tests: device cache allocation in the library's head-major
layout and conversion to/from the canonical [B, T, Hkv, D] layout the oracle speaks."""
import numpy as np
import torch

from hyprstream_amd import bindings as hb

DEV = "cuda:0"


def bf16_from_bits(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16)


def bf16_to_f32_np(t):
    return t.detach().float().cpu().numpy()


class DeviceCache:
    """Contiguous (non-paged) int8 or fp8 cache buffers on the GPU."""

    def __init__(self, B, Hkv, cap, D, fp8=False, fill=None):
        self.B, self.Hkv, self.cap, self.D, self.fp8 = B, Hkv, cap, D, fp8
        self.layout = hb.contiguous_layout(Hkv, cap, D)
        cap_s = self.layout.scale_stride_head
        cdt = torch.uint8 if fp8 else torch.int8
        mk = (lambda *s, dtype: torch.zeros(*s, dtype=dtype, device=DEV)) if fill is None else \
             (lambda *s, dtype: torch.full(s, fill, dtype=dtype, device=DEV))
        self.k_codes = mk(B, Hkv, cap, D, dtype=cdt)
        self.v_codes = mk(B, Hkv, cap, D, dtype=cdt)
        if fp8:
            self.k_scales = torch.zeros(B, Hkv, dtype=torch.float32, device=DEV)
            self.v_scales = torch.zeros(B, Hkv, dtype=torch.float32, device=DEV)
        else:
            self.k_scales = torch.zeros(B, Hkv, cap_s, dtype=torch.float32, device=DEV)
            self.v_scales = torch.zeros(B, Hkv, cap_s, dtype=torch.float32, device=DEV)

    def write(self, k_src, v_src, positions=None, start_pos=0):
        fn = hb.kv_quantize_fp8 if self.fp8 else hb.kv_quantize_int8
        fn(k_src, v_src, self.k_codes, self.v_codes, self.k_scales, self.v_scales, self.layout, positions, start_pos)

    def canonical(self, T):
        """(k_codes, v_codes, k_scales, v_scales) as numpy in the oracle's layout, first T tokens."""
        kc = self.k_codes[:, :, :T].permute(0, 2, 1, 3).contiguous().cpu().numpy()
        vc = self.v_codes[:, :, :T].permute(0, 2, 1, 3).contiguous().cpu().numpy()
        if self.fp8:
            return kc, vc, self.k_scales.cpu().numpy(), self.v_scales.cpu().numpy()
        ks = self.k_scales[:, :, :T].permute(0, 2, 1).contiguous().cpu().numpy()
        vs = self.v_scales[:, :, :T].permute(0, 2, 1).contiguous().cpu().numpy()
        return kc, vc, ks, vs

    def load_canonical(self, kc, vc, ks, vs):
        """Upload oracle-made codes/scales ([B,T,Hkv,D], [B,T,Hkv] or [B,Hkv])."""
        T = kc.shape[1]
        self.k_codes[:, :, :T] = torch.from_numpy(kc).to(DEV).permute(0, 2, 1, 3)
        self.v_codes[:, :, :T] = torch.from_numpy(vc).to(DEV).permute(0, 2, 1, 3)
        if self.fp8:
            self.k_scales.copy_(torch.from_numpy(ks))
            self.v_scales.copy_(torch.from_numpy(vs))
        else:
            self.k_scales[:, :, :T] = torch.from_numpy(ks).to(DEV).permute(0, 2, 1)
            self.v_scales[:, :, :T] = torch.from_numpy(vs).to(DEV).permute(0, 2, 1)


def run_decode(cache, q_bits, seq_lens, Hq, max_seq_len=None, softmax_scale=None, layout=None):
    B = cache.B
    q = bf16_from_bits(q_bits).to(DEV)
    lens = torch.from_numpy(np.ascontiguousarray(seq_lens, np.int32)).to(DEV)
    out = torch.full((B, Hq, cache.D), float("nan"), dtype=torch.bfloat16, device=DEV)
    max_seq_len = int(max(1, seq_lens.max())) if max_seq_len is None else max_seq_len
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, cache.Hkv, cache.D, max_seq_len), dtype=torch.uint8, device=DEV)
    scale = 1.0 / np.sqrt(cache.D) if softmax_scale is None else softmax_scale
    hb.decode_attn(q, cache.k_codes, cache.v_codes, cache.k_scales, cache.v_scales, layout or cache.layout, lens, out,
                   ws, cache.Hkv, max_seq_len, scale, fp8=cache.fp8)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()
