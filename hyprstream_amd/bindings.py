"""ctypes binding of libhs_attn.so: the same C ABI a Rust `-sys` crate would bind.

This module is plumbing for tests, the smoke check and the benchmark: torch supplies device
memory and the current stream, every call goes through the extern "C" entry points declared
in include/hs_attn.h.  There is no fallback: if the shared library is missing the import of
`lib()` raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libhs_attn.so")

HS_OK = 0
HS_ERR_INVALID_ARGUMENT = 1
HS_ERR_OVERFLOW = 2
HS_ERR_WORKSPACE = 3
HS_ERR_LAUNCH = 4
HS_ERR_POOL_EXHAUSTED = 5
HS_ERR_BUSY = 6
HS_BF16, HS_F32, HS_F16 = 0, 1, 2

EXPORTS = [
    "hs_attn_last_error", "hs_attn_abi_version",
    "hs_kv_quantize_int8", "hs_kv_fp8_calibrate", "hs_kv_quantize_fp8", "hs_kv_dequantize",
    "hs_decode_attn_workspace_bytes", "hs_decode_attn_int8", "hs_decode_attn_fp8", "hs_decode_attn_phases",
    "hs_decode_step_int8", "hs_decode_step_fp8", "hs_prefill_attn_int8", "hs_prefill_attn_fp8", "hs_deltanet_forward",
    "hs_kv_quantize_int8_rope", "hs_rope_apply", "hs_rope_apply_partial", "hs_decode_step_int8_rope", "hs_decode_attn_num_chunks",
    "hs_decode_attn_int8_static", "hs_qk_prologue_apply", "hs_kv_quantize_int8_prologue", "hs_decode_step_int8_prologue", "hs_decode_step_fp8_prologue",
    "hs_deltanet_prepare", "hs_deltanet_gated_norm", "hs_deltanet_decode_layer", "hs_deltanet_forward_chunked", "hs_deltanet_forward_chunked_gated_norm", "hs_deltanet_prefill_layer", "hs_deltanet_prefill_layer_workspace_bytes", "hs_prefill_attn_int8_ragged", "hs_prefill_attn_fp8_ragged", "hs_deltanet_chunked_workspace_bytes",
    "hs_deltanet_chunked_gated_norm_workspace_bytes", "hs_prefill_attn_split_workspace_bytes", "hs_prefill_attn_split_workspace_init", "hs_prefill_shadow_bytes", "hs_prefill_shadow_init",
]


class KvLayout(ctypes.Structure):
    """Mirror of `struct hs_kv_layout`."""
    _fields_ = [
        ("code_stride_seq", ctypes.c_int64),
        ("code_stride_head", ctypes.c_int64),
        ("scale_stride_seq", ctypes.c_int64),
        ("scale_stride_head", ctypes.c_int64),
        ("capacity_tokens", ctypes.c_int32),
        ("block_table_stride", ctypes.c_int32),
        ("k_block_table", ctypes.c_void_p),
        ("v_block_table", ctypes.c_void_p),
        ("total_tokens_hint", ctypes.c_int64),
        ("prefill_columns_hint", ctypes.c_int32),
        ("prefill_window", ctypes.c_int32),
        ("out_gate", ctypes.c_void_p),
        ("prefill_q_prologue", ctypes.c_void_p),
        ("prefill_split_workspace", ctypes.c_void_p),
        ("prefill_split_workspace_bytes", ctypes.c_int64),
        ("prefill_key_splits", ctypes.c_int32),
        ("reserved0", ctypes.c_int32),
        ("prefill_shadow", ctypes.c_void_p),
        ("prefill_shadow_bytes", ctypes.c_int64),
        ("prefill_shadow_tokens", ctypes.c_int32),
        ("reserved1", ctypes.c_int32),
    ]


QKNORM_NONE, QKNORM_LLAMA, QKNORM_QWEN35 = 0, 1, 2


class QkPrologue(ctypes.Structure):
    """Mirror of `struct hs_qk_prologue`."""
    _fields_ = [
        ("norm_kind", ctypes.c_int32),
        ("norm_eps", ctypes.c_float),
        ("q_norm_weight", ctypes.c_void_p),
        ("k_norm_weight", ctypes.c_void_p),
        ("q_norm_head_stride", ctypes.c_int32),
        ("k_norm_head_stride", ctypes.c_int32),
        ("rope_sin", ctypes.c_void_p),
        ("rope_cos", ctypes.c_void_p),
        ("rope_len", ctypes.c_int32),
        ("rotary_dim", ctypes.c_int32),
    ]


def qk_prologue(norm_kind=QKNORM_NONE, eps=0.0, q_weight=None, k_weight=None, rope_sin=None, rope_cos=None, rotary_dim=0):
    """Build an hs_qk_prologue from torch tensors (weights [H, D] or [D]; tables [rope_len, rotary_dim/2])."""
    p = QkPrologue()
    p.norm_kind, p.norm_eps = norm_kind, eps
    keep = [q_weight, k_weight, rope_sin, rope_cos]
    if q_weight is not None:
        assert q_weight.is_contiguous()
        p.q_norm_weight, p.q_norm_head_stride = q_weight.data_ptr(), (q_weight.shape[-1] if q_weight.dim() == 2 else 0)
    if k_weight is not None:
        assert k_weight.is_contiguous()
        p.k_norm_weight, p.k_norm_head_stride = k_weight.data_ptr(), (k_weight.shape[-1] if k_weight.dim() == 2 else 0)
    if rope_sin is not None:
        assert rope_sin.is_contiguous() and rope_cos.is_contiguous() and rope_sin.shape == rope_cos.shape
        p.rope_sin, p.rope_cos, p.rope_len = rope_sin.data_ptr(), rope_cos.data_ptr(), rope_sin.shape[0]
    p.rotary_dim = rotary_dim
    p._keep = keep  # the struct holds raw addresses
    return p


class HsError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("hs_attn error %d: %s" % (code, msg))
        self.code = code


_lib = None


def lib():
    """Load libhs_attn.so (built by `python -m hyprstream_amd.build`); raises if absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("libhs_attn.so not built: run `python -m hyprstream_amd.build` (%s)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.hs_attn_last_error.restype = ctypes.c_char_p
        L.hs_decode_attn_workspace_bytes.restype = ctypes.c_size_t
        L.hs_decode_attn_workspace_bytes.argtypes = [ctypes.c_int32] * 5
        L.hs_prefill_shadow_bytes.restype = ctypes.c_size_t
        L.hs_prefill_shadow_bytes.argtypes = [ctypes.c_int32] * 4
        L.hs_prefill_attn_split_workspace_bytes.restype = ctypes.c_size_t
        L.hs_prefill_attn_split_workspace_bytes.argtypes = [ctypes.c_int32] * 5
        _lib = L
    return _lib


def check(rc):
    if rc != HS_OK:
        raise HsError(rc, lib().hs_attn_last_error().decode())


def contiguous_layout(Hkv, capacity_tokens, D, scale_pad=4):
    """Head-major cache of one buffer per tensor: codes [B, Hkv, cap, D], scales [B, Hkv, cap_padded]."""
    cap_s = (capacity_tokens + scale_pad - 1) // scale_pad * scale_pad
    return KvLayout(Hkv * capacity_tokens * D, capacity_tokens * D, Hkv * cap_s, cap_s, capacity_tokens, 0, None, None, 0, 0, 0)


def paged_layout(Hkv, block_tokens, D, k_table, v_table):
    """Pool of blocks [nblocks, Hkv, block_tokens, D]; tables are int32 device tensors [B, max_blocks]."""
    assert k_table.dtype.is_signed and k_table.element_size() == 4 and k_table.is_contiguous()
    lay = KvLayout(Hkv * block_tokens * D, block_tokens * D, Hkv * block_tokens, block_tokens, block_tokens,
                   k_table.shape[1], k_table.data_ptr(), v_table.data_ptr(), 0, 0, 0)
    lay._tables = (k_table, v_table)  # the struct holds raw addresses: the tensors must live as long as it does
    return lay


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else None)


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dtype_code(t):
    import torch
    return {torch.bfloat16: HS_BF16, torch.float32: HS_F32, torch.float16: HS_F16}[t.dtype]


def kv_quantize_int8(k_src, v_src, k_codes, v_codes, k_scales, v_scales, layout, positions=None, start_pos=0):
    B, S, Hkv, D = k_src.shape
    assert k_src.is_contiguous() and v_src.is_contiguous()
    check(lib().hs_kv_quantize_int8(_ptr(k_src), _ptr(v_src), _dtype_code(k_src), _ptr(k_codes), _ptr(v_codes),
                                    _ptr(k_scales), _ptr(v_scales), ctypes.byref(layout), _ptr(positions),
                                    ctypes.c_int32(start_pos), B, S, Hkv, D, _stream()))


def kv_quantize_int8_rope(k_src, v_src, rope_sin, rope_cos, k_codes, v_codes, k_scales, v_scales, layout,
                          positions=None, start_pos=0):
    """As kv_quantize_int8 with K rotated on the way in; rope_sin/rope_cos: [rope_len, D/2] in k_src's dtype."""
    B, S, Hkv, D = k_src.shape
    assert k_src.is_contiguous() and v_src.is_contiguous() and rope_sin.is_contiguous() and rope_cos.is_contiguous()
    assert rope_sin.dtype == k_src.dtype and rope_sin.shape[1] == D // 2
    check(lib().hs_kv_quantize_int8_rope(_ptr(k_src), _ptr(v_src), _dtype_code(k_src), _ptr(rope_sin), _ptr(rope_cos),
                                         ctypes.c_int32(rope_sin.shape[0]), _ptr(k_codes), _ptr(v_codes),
                                         _ptr(k_scales), _ptr(v_scales), ctypes.byref(layout), _ptr(positions),
                                         ctypes.c_int32(start_pos), B, S, Hkv, D, _stream()))


def rope_apply(x, rope_sin, rope_cos, out, positions=None, start_pos=0, rotary_dim=None):
    """Half-split rotary embedding of x [B, S, H, D] into out (same shape and dtype).  rotary_dim < D rotates only the
    leading rotary_dim elements of each head (tables [rope_len, rotary_dim/2]) and copies the rest."""
    B, S, H, D = x.shape
    assert x.is_contiguous() and out.is_contiguous() and out.dtype == x.dtype and rope_sin.dtype == x.dtype
    rd = D if rotary_dim is None else rotary_dim
    assert rope_sin.shape[1] == rd // 2 and rope_sin.is_contiguous() and rope_cos.is_contiguous()
    check(lib().hs_rope_apply_partial(_ptr(x), _dtype_code(x), _ptr(rope_sin), _ptr(rope_cos), ctypes.c_int32(rope_sin.shape[0]),
                                      _ptr(positions), ctypes.c_int32(start_pos), _ptr(out), B, S, H, D, ctypes.c_int32(rd),
                                      _stream()))


def qk_prologue_apply(q, k, prologue, q_out, k_out, positions=None, start_pos=0):
    """QK-norm + rotary embedding of q [B,S,Hq,D] and k [B,S,Hkv,D] in one launch (either pair may be None)."""
    ref_t = q if q is not None else k
    B, S, _, D = ref_t.shape
    Hq = q.shape[2] if q is not None else 0
    Hkv = k.shape[2] if k is not None else 0
    for t in (q, k, q_out, k_out):
        assert t is None or t.is_contiguous()
    check(lib().hs_qk_prologue_apply(_ptr(q), _ptr(k), _dtype_code(ref_t), ctypes.byref(prologue), _ptr(positions),
                                     ctypes.c_int32(start_pos), _ptr(q_out), _ptr(k_out), B, S, Hq, Hkv, D, _stream()))


def kv_quantize_int8_prologue(k_src, v_src, prologue, k_codes, v_codes, k_scales, v_scales, layout, positions=None,
                              start_pos=0):
    """kv_quantize_int8 with K normalised and rotated on the way in."""
    B, S, Hkv, D = k_src.shape
    assert k_src.is_contiguous() and v_src.is_contiguous()
    check(lib().hs_kv_quantize_int8_prologue(_ptr(k_src), _ptr(v_src), _dtype_code(k_src), ctypes.byref(prologue),
                                             _ptr(k_codes), _ptr(v_codes), _ptr(k_scales), _ptr(v_scales),
                                             ctypes.byref(layout), _ptr(positions), ctypes.c_int32(start_pos), B, S,
                                             Hkv, D, _stream()))


def decode_step_prologue(q, k_new, v_new, prologue, k_codes, v_codes, k_scales, v_scales, layout, seq_lens, out,
                         workspace, Hkv, max_seq_len, softmax_scale, fp8=False):
    """decode_step (int8, or fp8 with calibrated scales) with the QK-norm and the rotation of q and k_new inside the
    launch."""
    B, Hq, D = q.shape
    assert k_new.shape == (B, 1, Hkv, D) and k_new.is_contiguous() and v_new.is_contiguous()
    fn = lib().hs_decode_step_fp8_prologue if fp8 else lib().hs_decode_step_int8_prologue
    check(fn(_ptr(q), _ptr(k_new), _ptr(v_new), ctypes.byref(prologue), _ptr(k_codes), _ptr(v_codes), _ptr(k_scales),
             _ptr(v_scales), ctypes.byref(layout), _ptr(seq_lens), _ptr(out), _ptr(workspace),
             ctypes.c_size_t(workspace.numel() * workspace.element_size()), B, Hq, Hkv, D,
             ctypes.c_int32(max_seq_len), ctypes.c_float(softmax_scale), _stream()))


def kv_fp8_calibrate(k_src, v_src, k_scales, v_scales):
    B, S, Hkv, D = k_src.shape
    check(lib().hs_kv_fp8_calibrate(_ptr(k_src), _ptr(v_src), _dtype_code(k_src), _ptr(k_scales), _ptr(v_scales),
                                    B, S, Hkv, D, _stream()))


def kv_quantize_fp8(k_src, v_src, k_codes, v_codes, k_scales, v_scales, layout, positions=None, start_pos=0):
    B, S, Hkv, D = k_src.shape
    assert k_src.is_contiguous() and v_src.is_contiguous()
    check(lib().hs_kv_quantize_fp8(_ptr(k_src), _ptr(v_src), _dtype_code(k_src), _ptr(k_codes), _ptr(v_codes),
                                   _ptr(k_scales), _ptr(v_scales), ctypes.byref(layout), _ptr(positions),
                                   ctypes.c_int32(start_pos), B, S, Hkv, D, _stream()))


def kv_dequantize(codes, scales, fp8, layout, which_table, out):
    B, T, Hkv, D = out.shape
    check(lib().hs_kv_dequantize(_ptr(codes), _ptr(scales), int(fp8), ctypes.byref(layout), int(which_table),
                                 _ptr(out), _dtype_code(out), B, T, Hkv, D, _stream()))


def decode_num_chunks(B, Hkv, max_seq_len, total_tokens_hint=0):
    return lib().hs_decode_attn_num_chunks(B, Hkv, max_seq_len, ctypes.c_int64(total_tokens_hint))


def decode_workspace_bytes(B, Hq, Hkv, D, max_seq_len):
    return lib().hs_decode_attn_workspace_bytes(B, Hq, Hkv, D, max_seq_len)


def decode_attn(q, k_codes, v_codes, k_scales, v_scales, layout, seq_lens, out, workspace, Hkv, max_seq_len,
                softmax_scale, fp8=False, phases=3):
    B, Hq, D = q.shape
    if phases != 3:
        fn0 = lib().hs_decode_attn_phases
        fn = lambda *a: fn0(int(fp8), int(phases), *a)
    else:
        fn = lib().hs_decode_attn_fp8 if fp8 else lib().hs_decode_attn_int8
    check(fn(_ptr(q), _ptr(k_codes), _ptr(v_codes), _ptr(k_scales), _ptr(v_scales), ctypes.byref(layout),
             _ptr(seq_lens), _ptr(out), _ptr(workspace),
             ctypes.c_size_t(workspace.numel() * workspace.element_size() if workspace is not None else 0),
             B, Hq, Hkv, D, ctypes.c_int32(max_seq_len), ctypes.c_float(softmax_scale), _stream()))


def decode_attn_static(q, k_codes, v_codes, k_scales, v_scales, layout, seq_lens, out, Hkv, max_seq_len, softmax_scale):
    """hs_decode_attn_int8 without a workspace argument: the split-K partials use the library's built-in scratch."""
    B, Hq, D = q.shape
    check(lib().hs_decode_attn_int8_static(_ptr(q), _ptr(k_codes), _ptr(v_codes), _ptr(k_scales), _ptr(v_scales),
                                           ctypes.byref(layout), _ptr(seq_lens), _ptr(out), B, Hq, Hkv, D,
                                           ctypes.c_int32(max_seq_len), ctypes.c_float(softmax_scale), _stream()))


def decode_step(q, k_new, v_new, k_codes, v_codes, k_scales, v_scales, layout, seq_lens, out, workspace, Hkv,
                max_seq_len, softmax_scale, fp8=False):
    """Quantize-on-write of one new token per sequence (at seq_lens-1) + decode attention, one call."""
    B, Hq, D = q.shape
    assert k_new.shape == (B, 1, Hkv, D) and k_new.is_contiguous() and v_new.is_contiguous()
    fn = lib().hs_decode_step_fp8 if fp8 else lib().hs_decode_step_int8
    check(fn(_ptr(q), _ptr(k_new), _ptr(v_new), _dtype_code(k_new), _ptr(k_codes), _ptr(v_codes), _ptr(k_scales),
             _ptr(v_scales), ctypes.byref(layout), _ptr(seq_lens), _ptr(out), _ptr(workspace),
             ctypes.c_size_t(workspace.numel() * workspace.element_size()), B, Hq, Hkv, D,
             ctypes.c_int32(max_seq_len), ctypes.c_float(softmax_scale), _stream()))


def decode_step_rope(q, k_new, v_new, rope_sin, rope_cos, k_codes, v_codes, k_scales, v_scales, layout, seq_lens, out,
                     workspace, Hkv, max_seq_len, softmax_scale):
    """decode_step (int8) with q and k_new arriving unrotated; bf16 tables [rope_len, D/2]."""
    B, Hq, D = q.shape
    assert k_new.shape == (B, 1, Hkv, D) and k_new.is_contiguous() and v_new.is_contiguous()
    check(lib().hs_decode_step_int8_rope(_ptr(q), _ptr(k_new), _ptr(v_new), _ptr(rope_sin), _ptr(rope_cos),
                                         ctypes.c_int32(rope_sin.shape[0]), _ptr(k_codes), _ptr(v_codes),
                                         _ptr(k_scales), _ptr(v_scales), ctypes.byref(layout), _ptr(seq_lens),
                                         _ptr(out), _ptr(workspace),
                                         ctypes.c_size_t(workspace.numel() * workspace.element_size()), B, Hq, Hkv, D,
                                         ctypes.c_int32(max_seq_len), ctypes.c_float(softmax_scale), _stream()))


def prefill_split_workspace(B, S, Hq, Hkv, D, device="cuda:0"):
    """Scratch for the key split of small prefill calls of at most B x S new tokens, counters cleared."""
    import torch
    n = lib().hs_prefill_attn_split_workspace_bytes(B, S, Hq, Hkv, D)
    ws = torch.empty(n, dtype=torch.uint8, device=device)
    check(lib().hs_prefill_attn_split_workspace_init(_ptr(ws), ctypes.c_size_t(n), _stream()))
    return ws


def prefill_shadow(B, Hkv, D, max_tokens, device="cuda:0"):
    """(buffer, tokens) for prefill_attn's `shadow`: the cleared bf16 copy for prompts of at most max_tokens tokens."""
    import torch
    tokens = (max_tokens + 63) // 64 * 64
    n = lib().hs_prefill_shadow_bytes(B, Hkv, D, tokens)
    buf = torch.empty(n, dtype=torch.uint8, device=device)
    check(lib().hs_prefill_shadow_init(_ptr(buf), ctypes.c_size_t(n), _stream()))
    return buf, tokens


PREFILL_KEY_SPLITS = 0  # tests: force this many key runs per query tile on every prefill_attn call (with a scratch of their own)
_split_scratch = {}


PREFILL_COLUMNS = 0  # default for prefill_attn's `columns` (tests set it to run every case at each workgroup width)


def prefill_attn(q, k_new, v_new, k_codes, v_codes, k_scales, v_scales, layout, hist_len, out, softmax_scale,
                 quantize_on_write=True, fp8=False, hist_lens=None, columns=None, window=0, q_prologue=None,
                 split_workspace=None, key_splits=0, shadow=None):
    """Causal attention of S new tokens over [int8 or fp8 history | their own bf16 K/V]; optionally caches them.
    hist_lens (int32 device tensor [B]): rows at different positions; hist_len is then their upper bound.
    columns: 0 = the library's choice of workgroup width, 256 or 128 fixes it (layout.prefill_columns_hint).
    window: sliding window of local layers (layout.prefill_window), 0 = none.
    q_prologue (QkPrologue): q arrives as projected and the launch normalises and rotates it
    (layout.prefill_q_prologue); k_new arrives normalised and rotated either way.
    split_workspace (uint8 device tensor from prefill_split_workspace()): lets a call with few query tiles split their
    keys over several workgroups; key_splits 0 = the library decides, 1 = never, 2..8 = forced.
    shadow ((uint8 device tensor, tokens) from prefill_shadow()): the bf16 operand-order copy of the prompt's K/V that
    every call appends to and calls with history read instead of the codes (layout.prefill_shadow)."""
    B, S, Hq, D = q.shape
    layout.prefill_columns_hint = PREFILL_COLUMNS if columns is None else columns
    layout.prefill_window = window
    layout.prefill_q_prologue = ctypes.addressof(q_prologue) if q_prologue is not None else None
    if split_workspace is None and key_splits == 0 and PREFILL_KEY_SPLITS > 1:
        key = (B, S, Hq, k_new.shape[2], D)
        if key not in _split_scratch:
            _split_scratch[key] = prefill_split_workspace(*key)
        split_workspace, key_splits = _split_scratch[key], PREFILL_KEY_SPLITS
    layout.prefill_split_workspace = split_workspace.data_ptr() if split_workspace is not None else None
    layout.prefill_split_workspace_bytes = split_workspace.numel() if split_workspace is not None else 0
    layout.prefill_key_splits = key_splits
    layout.prefill_shadow = shadow[0].data_ptr() if shadow is not None else None
    layout.prefill_shadow_bytes = shadow[0].numel() if shadow is not None else 0
    layout.prefill_shadow_tokens = shadow[1] if shadow is not None else 0
    Hkv = k_new.shape[2]
    assert q.is_contiguous() and k_new.is_contiguous() and v_new.is_contiguous() and out.is_contiguous()
    if hist_lens is not None:
        assert str(hist_lens.dtype) == "torch.int32" and hist_lens.numel() == B and hist_lens.is_contiguous()
        fn = lib().hs_prefill_attn_fp8_ragged if fp8 else lib().hs_prefill_attn_int8_ragged
        check(fn(_ptr(q), _ptr(k_new), _ptr(v_new), _ptr(k_codes), _ptr(v_codes), _ptr(k_scales), _ptr(v_scales),
                 ctypes.byref(layout), _ptr(hist_lens), ctypes.c_int32(hist_len), _ptr(out), B, S, Hq, Hkv, D,
                 ctypes.c_float(softmax_scale), int(bool(quantize_on_write)), _stream()))
        return
    fn = lib().hs_prefill_attn_fp8 if fp8 else lib().hs_prefill_attn_int8
    check(fn(_ptr(q), _ptr(k_new), _ptr(v_new), _ptr(k_codes), _ptr(v_codes), _ptr(k_scales),
                                     _ptr(v_scales), ctypes.byref(layout), ctypes.c_int32(hist_len), _ptr(out),
                                     B, S, Hq, Hkv, D, ctypes.c_float(softmax_scale), int(bool(quantize_on_write)),
                                     _stream()))


def deltanet_forward(q, k, v, g, beta, state, out, q_scale, l2norm=False):
    """Gated delta rule over T tokens; q,k bf16 [B,T,nk,128], v bf16 [B,T,nv,128], g,beta fp32 [B,T,nv],
    state fp32 [B,nv,128,128] (updated in place), out fp32 [B,T,nv,128]."""
    B, T, nk, dk = q.shape
    nv, dv = v.shape[2], v.shape[3]
    for t in (q, k, v, g, beta, state, out):
        assert t.is_contiguous()
    check(lib().hs_deltanet_forward(_ptr(q), _ptr(k), _ptr(v), _ptr(g), _ptr(beta), _ptr(state), _ptr(out),
                                    B, T, nk, nv, dk, dv, ctypes.c_float(q_scale), int(bool(l2norm)), _stream()))


def deltanet_chunked_workspace_bytes(B, T, nk, nv):
    lib().hs_deltanet_chunked_workspace_bytes.restype = ctypes.c_size_t
    return int(lib().hs_deltanet_chunked_workspace_bytes(B, T, nk, nv))


def deltanet_chunked_gated_norm_workspace_bytes(B, T, nk, nv):
    lib().hs_deltanet_chunked_gated_norm_workspace_bytes.restype = ctypes.c_size_t
    return int(lib().hs_deltanet_chunked_gated_norm_workspace_bytes(B, T, nk, nv))


def deltanet_forward_chunked(q, k, v, g, beta, state, out, q_scale, l2norm=False, workspace=None):
    """The same over a prompt in 64-token chunks on the matrix pipe (fp16 operands, fp32 accumulation and state)."""
    import torch
    B, T, nk, dk = q.shape
    nv, dv = v.shape[2], v.shape[3]
    for t in (q, k, v, g, beta, state, out):
        assert t.is_contiguous()
    lib().hs_deltanet_chunked_workspace_bytes.restype = ctypes.c_size_t
    need = lib().hs_deltanet_chunked_workspace_bytes(B, T, nk, nv)
    if workspace is None:
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    check(lib().hs_deltanet_forward_chunked(_ptr(q), _ptr(k), _ptr(v), _ptr(g), _ptr(beta), _ptr(state), _ptr(out),
                                            B, T, nk, nv, dk, dv, ctypes.c_float(q_scale), int(bool(l2norm)),
                                            _ptr(workspace), ctypes.c_size_t(workspace.numel()), _stream()))
    return workspace


def deltanet_forward_chunked_gated_norm(q, k, v, g, beta, state, z, norm_weight, eps, out, q_scale, l2norm=False, workspace=None):
    """deltanet_forward_chunked + the gated RMSNorm, one call: out bf16 [B, T, nv, dv]."""
    import torch
    B, T, nk, dk = q.shape
    nv, dv = v.shape[2], v.shape[3]
    for t in (q, k, v, g, beta, state, z, out):
        assert t.is_contiguous()
    lib().hs_deltanet_chunked_gated_norm_workspace_bytes.restype = ctypes.c_size_t
    need = lib().hs_deltanet_chunked_gated_norm_workspace_bytes(B, T, nk, nv)
    if workspace is None:
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    check(lib().hs_deltanet_forward_chunked_gated_norm(_ptr(q), _ptr(k), _ptr(v), _ptr(g), _ptr(beta), _ptr(state), _ptr(z),
                                                       _ptr(norm_weight), ctypes.c_float(eps), _ptr(out), B, T, nk, nv, dk, dv,
                                                       ctypes.c_float(q_scale), int(bool(l2norm)), _ptr(workspace),
                                                       ctypes.c_size_t(workspace.numel()), _stream()))
    return workspace


def deltanet_prepare(mixed_qkv, conv_weight, conv_state_in, a_in, b_in, neg_a_exp, dt_bias, nk, nv, dk, dv):
    """conv1d(k=4)+SiLU with carried state, q/k/v split, g and beta.  Returns (q, k, v, g, beta, new_conv_state)."""
    import torch
    B, S, C = mixed_qkv.shape
    assert C == 2 * nk * dk + nv * dv and mixed_qkv.is_contiguous() and conv_weight.is_contiguous()
    dev = mixed_qkv.device
    q = torch.empty(B, S, nk, dk, dtype=torch.bfloat16, device=dev)
    k = torch.empty(B, S, nk, dk, dtype=torch.bfloat16, device=dev)
    v = torch.empty(B, S, nv, dv, dtype=torch.bfloat16, device=dev)
    g = torch.empty(B, S, nv, dtype=torch.float32, device=dev)
    beta = torch.empty(B, S, nv, dtype=torch.float32, device=dev)
    state_out = torch.empty(B, C, 3, dtype=torch.bfloat16, device=dev)
    check(lib().hs_deltanet_prepare(_ptr(mixed_qkv), _ptr(conv_weight), _ptr(conv_state_in), _ptr(state_out),
                                    _ptr(a_in.contiguous()), _ptr(b_in.contiguous()), _ptr(neg_a_exp), _ptr(dt_bias),
                                    _ptr(q), _ptr(k), _ptr(v), _ptr(g), _ptr(beta), B, S, nk, nv, dk, dv, _stream()))
    return q, k, v, g, beta, state_out


def deltanet_decode_layer(mixed_qkv, conv_weight, conv_state_in, a_in, b_in, neg_a_exp, dt_bias, z, norm_weight, eps,
                          state, nk, nv, dk, dv, q_scale, l2norm=True, out=None, conv_state_out=None):
    """One decode step of a gated-DeltaNet layer between its projections, one launch.  mixed_qkv [B, 1, C];
    `state` is updated in place.  Returns (out bf16 [B, 1, nv, dv], new_conv_state)."""
    import torch
    B, S, C = mixed_qkv.shape
    assert S == 1 and C == 2 * nk * dk + nv * dv and mixed_qkv.is_contiguous() and conv_weight.is_contiguous()
    dev = mixed_qkv.device
    if out is None:
        out = torch.empty(B, 1, nv, dv, dtype=torch.bfloat16, device=dev)
    if conv_state_out is None:
        conv_state_out = torch.empty(B, C, 3, dtype=torch.bfloat16, device=dev)
    check(lib().hs_deltanet_decode_layer(_ptr(mixed_qkv), _ptr(conv_weight), _ptr(conv_state_in), _ptr(conv_state_out),
                                         _ptr(a_in), _ptr(b_in), _ptr(neg_a_exp), _ptr(dt_bias), _ptr(z), _ptr(norm_weight),
                                         ctypes.c_float(eps), _ptr(state), _ptr(out), B, nk, nv, dk, dv,
                                         ctypes.c_float(q_scale), int(bool(l2norm)), _stream()))
    return out, conv_state_out


def deltanet_prefill_layer(mixed_qkv, conv_weight, conv_state_in, a_in, b_in, neg_a_exp, dt_bias, z, norm_weight, eps,
                           state, nk, nv, dk, dv, q_scale, l2norm=True, workspace=None):
    """The prompt branch of a gated-DeltaNet layer between its projections in one call.  `state` is updated in place.
    Returns (out bf16 [B, S, nv, dv], new_conv_state, workspace)."""
    import torch
    B, S, C = mixed_qkv.shape
    assert C == 2 * nk * dk + nv * dv and mixed_qkv.is_contiguous() and conv_weight.is_contiguous() and z.is_contiguous()
    dev = mixed_qkv.device
    lib().hs_deltanet_prefill_layer_workspace_bytes.restype = ctypes.c_size_t
    need = lib().hs_deltanet_prefill_layer_workspace_bytes(B, S, nk, nv, dk, dv)
    if workspace is None:
        workspace = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
    out = torch.empty(B, S, nv, dv, dtype=torch.bfloat16, device=dev)
    conv_state_out = torch.empty(B, C, 3, dtype=torch.bfloat16, device=dev)
    check(lib().hs_deltanet_prefill_layer(_ptr(mixed_qkv), _ptr(conv_weight), _ptr(conv_state_in), _ptr(conv_state_out),
                                          _ptr(a_in.contiguous()), _ptr(b_in.contiguous()), _ptr(neg_a_exp), _ptr(dt_bias),
                                          _ptr(z), _ptr(norm_weight), ctypes.c_float(eps), _ptr(state), _ptr(out), B, S, nk, nv,
                                          dk, dv, ctypes.c_float(q_scale), int(bool(l2norm)), _ptr(workspace),
                                          ctypes.c_size_t(workspace.numel()), _stream()))
    return out, conv_state_out, workspace


def deltanet_gated_norm(x, z, weight, eps):
    """x fp32 [..., D], z bf16 [..., D], weight fp32 [D] -> bf16 [..., D]."""
    import torch
    D = x.shape[-1]
    out = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
    check(lib().hs_deltanet_gated_norm(_ptr(x.contiguous()), _ptr(z.contiguous()), _ptr(weight), ctypes.c_float(eps),
                                       _ptr(out), ctypes.c_int64(x.numel() // D), D, _stream()))
    return out

