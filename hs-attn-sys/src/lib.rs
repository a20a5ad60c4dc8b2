//! hs-attn-sys: the thin `-sys` crate through which hyprstream reaches the MI355X attention kernels, in the
//! style of bitsandbytes-sys (crates/bitsandbytes-sys/src/lib.rs): `bindings` is the raw `extern "C"` surface,
//! this file adds an error type and `unsafe fn ..._gpu` wrappers over raw device pointers that turn the status
//! code into a `Result` (the counterpart of `BnbError`, bitsandbytes-sys/src/lib.rs:48-74, and of the `_gpu`
//! functions at lib.rs:443-506).  Nothing here allocates: every buffer is a tensor the caller owns
//! (`tensor.data_ptr()`), as in kv_cache.rs:797-865.
//!
//! This crate is text in the kernel repository: it is compiled in hyprstream's tree, not here.
pub mod bindings;

use std::ffi::{c_int, c_void, CStr};
use std::fmt;

pub use bindings::{hs_kv_layout, hs_qk_prologue, hs_stream_t};

/// A failed call: the status code (`HS_ERR_*`) and the library's message for this thread.
#[derive(Debug, Clone, PartialEq, Eq)]
pub struct HsAttnError {
    pub code: c_int,
    pub message: String,
}

impl fmt::Display for HsAttnError {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result {
        write!(f, "hs_attn error {}: {}", self.code, self.message)
    }
}
impl std::error::Error for HsAttnError {}

pub type Result<T> = std::result::Result<T, HsAttnError>;

/// Status code -> `Result`, reading `hs_attn_last_error()` on failure.
pub fn check(rc: c_int) -> Result<()> {
    if rc == bindings::HS_OK {
        return Ok(());
    }
    // SAFETY: the library returns a pointer to a thread-local, NUL-terminated buffer that lives until the next call.
    let message = unsafe { CStr::from_ptr(bindings::hs_attn_last_error()) }.to_string_lossy().into_owned();
    Err(HsAttnError { code: rc, message })
}

/// Refuses a library whose ABI differs from the one these bindings were generated for.
pub fn check_abi() -> Result<()> {
    let v = unsafe { bindings::hs_attn_abi_version() };
    if v == bindings::HS_ATTN_ABI_VERSION {
        Ok(())
    } else {
        Err(HsAttnError { code: bindings::HS_ERR_INVALID_ARGUMENT, message: format!("libhs_attn ABI {v}, bindings {}", bindings::HS_ATTN_ABI_VERSION) })
    }
}

/// Layout of one contiguous head-major cache: codes `[B, Hkv, cap, D]`, int8 scales `[B, Hkv, cap rounded up to 4]`.
pub fn contiguous_layout(hkv: i32, capacity_tokens: i32, d: i32) -> hs_kv_layout {
    let cap_s = (capacity_tokens as i64 + 3) / 4 * 4;
    hs_kv_layout {
        code_stride_seq: hkv as i64 * capacity_tokens as i64 * d as i64,
        code_stride_head: capacity_tokens as i64 * d as i64,
        scale_stride_seq: hkv as i64 * cap_s,
        scale_stride_head: cap_s,
        capacity_tokens,
        block_table_stride: 0,
        k_block_table: std::ptr::null(),
        v_block_table: std::ptr::null(),
        total_tokens_hint: 0,
        prefill_columns_hint: 0,
        prefill_window: 0,
        out_gate: std::ptr::null(),
        prefill_q_prologue: std::ptr::null(),
        prefill_split_workspace: std::ptr::null_mut(),
        prefill_split_workspace_bytes: 0,
        prefill_key_splits: 0,
        reserved0: 0,
        prefill_shadow: std::ptr::null_mut(),
        prefill_shadow_bytes: 0,
        prefill_shadow_tokens: 0,
        reserved1: 0,
    }
}

/// Shape of one attention problem, as the entry points take it.
#[derive(Clone, Copy, Debug)]
pub struct AttnShape {
    pub b: i32,
    pub hq: i32,
    pub hkv: i32,
    pub d: i32,
}

/// Quantize-on-write of `s` new tokens per sequence into the int8 cache (`LayerKVCache::update`, kv_cache.rs:1275-1432).
///
/// # Safety
/// Every pointer is a device pointer of the current device, valid for the sizes the header states.
#[allow(clippy::too_many_arguments)]
pub unsafe fn kv_quantize_int8_gpu(k_src: *const c_void, v_src: *const c_void, src_dtype: c_int, k_codes: *mut i8,
                                   v_codes: *mut i8, k_scales: *mut f32, v_scales: *mut f32, layout: &hs_kv_layout,
                                   positions: *const i32, start_pos: i32, b: i32, s: i32, hkv: i32, d: i32,
                                   stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_kv_quantize_int8(k_src, v_src, src_dtype, k_codes, v_codes, k_scales, v_scales, layout, positions,
                                        start_pos, b, s, hkv, d, stream))
}

/// One decode step: the new token's K/V quantized on write at `seq_lens[b] - 1`, then attention over the cache
/// (cache.update + cache.get + compute_attention of `LlamaAttention::forward`, llama.rs:605-636).
///
/// # Safety
/// As above; `workspace` holds at least `decode_workspace_bytes(..)` bytes, 256-byte aligned.
#[allow(clippy::too_many_arguments)]
pub unsafe fn decode_step_int8_gpu(q: *const c_void, k_new: *const c_void, v_new: *const c_void, src_dtype: c_int,
                                   k_codes: *mut i8, v_codes: *mut i8, k_scales: *mut f32, v_scales: *mut f32,
                                   layout: &hs_kv_layout, seq_lens: *const i32, out: *mut c_void,
                                   workspace: *mut c_void, workspace_bytes: usize, shape: AttnShape, max_seq_len: i32,
                                   softmax_scale: f32, stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_decode_step_int8(q, k_new, v_new, src_dtype, k_codes, v_codes, k_scales, v_scales, layout, seq_lens,
                                        out, workspace, workspace_bytes, shape.b, shape.hq, shape.hkv, shape.d,
                                        max_seq_len, softmax_scale, stream))
}

/// The same step with QK-norm and rotary embedding of q and k_new inside the launch (llama.rs:589-611).
///
/// # Safety
/// As `decode_step_int8_gpu`; the tables and weights named by `prologue` are device pointers.
#[allow(clippy::too_many_arguments)]
pub unsafe fn decode_step_int8_prologue_gpu(q: *const c_void, k_new: *const c_void, v_new: *const c_void,
                                            prologue: &hs_qk_prologue, k_codes: *mut i8, v_codes: *mut i8,
                                            k_scales: *mut f32, v_scales: *mut f32, layout: &hs_kv_layout,
                                            seq_lens: *const i32, out: *mut c_void, workspace: *mut c_void,
                                            workspace_bytes: usize, shape: AttnShape, max_seq_len: i32,
                                            softmax_scale: f32, stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_decode_step_int8_prologue(q, k_new, v_new, prologue, k_codes, v_codes, k_scales, v_scales, layout,
                                                 seq_lens, out, workspace, workspace_bytes, shape.b, shape.hq, shape.hkv,
                                                 shape.d, max_seq_len, softmax_scale, stream))
}

/// Decode attention over an int8 cache without a new token (q_len == 1 branch of compute_attention_masked, llama.rs:1066-1093).
///
/// # Safety
/// As `decode_step_int8_gpu`.
#[allow(clippy::too_many_arguments)]
pub unsafe fn decode_attn_int8_gpu(q: *const c_void, k_codes: *const i8, v_codes: *const i8, k_scales: *const f32,
                                   v_scales: *const f32, layout: &hs_kv_layout, seq_lens: *const i32, out: *mut c_void,
                                   workspace: *mut c_void, workspace_bytes: usize, shape: AttnShape, max_seq_len: i32,
                                   softmax_scale: f32, stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_decode_attn_int8(q, k_codes, v_codes, k_scales, v_scales, layout, seq_lens, out, workspace,
                                        workspace_bytes, shape.b, shape.hq, shape.hkv, shape.d, max_seq_len, softmax_scale,
                                        stream))
}

/// FP8 e4m3fn cache: decode attention with per-(sequence, kv-head) scales.
///
/// # Safety
/// As `decode_step_int8_gpu`.
#[allow(clippy::too_many_arguments)]
pub unsafe fn decode_step_fp8_gpu(q: *const c_void, k_new: *const c_void, v_new: *const c_void, src_dtype: c_int,
                                  k_codes: *mut u8, v_codes: *mut u8, k_scales: *const f32, v_scales: *const f32,
                                  layout: &hs_kv_layout, seq_lens: *const i32, out: *mut c_void, workspace: *mut c_void,
                                  workspace_bytes: usize, shape: AttnShape, max_seq_len: i32, softmax_scale: f32,
                                  stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_decode_step_fp8(q, k_new, v_new, src_dtype, k_codes, v_codes, k_scales, v_scales, layout, seq_lens,
                                       out, workspace, workspace_bytes, shape.b, shape.hq, shape.hkv, shape.d, max_seq_len,
                                       softmax_scale, stream))
}

/// `decode_step_fp8_gpu` with QK-norm and rotary embedding of q and k_new inside the launch (qwen3_5.rs:1077-1091,
/// rope.rs:206-248).
///
/// # Safety
/// As `decode_step_int8_prologue_gpu`.
#[allow(clippy::too_many_arguments)]
pub unsafe fn decode_step_fp8_prologue_gpu(q: *const c_void, k_new: *const c_void, v_new: *const c_void,
                                           prologue: &hs_qk_prologue, k_codes: *mut u8, v_codes: *mut u8,
                                           k_scales: *const f32, v_scales: *const f32, layout: &hs_kv_layout,
                                           seq_lens: *const i32, out: *mut c_void, workspace: *mut c_void,
                                           workspace_bytes: usize, shape: AttnShape, max_seq_len: i32,
                                           softmax_scale: f32, stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_decode_step_fp8_prologue(q, k_new, v_new, prologue, k_codes, v_codes, k_scales, v_scales, layout,
                                                seq_lens, out, workspace, workspace_bytes, shape.b, shape.hq, shape.hkv,
                                                shape.d, max_seq_len, softmax_scale, stream))
}

/// Causal prefill of `s` new tokens over [int8 history | their own bf16 K/V], caching them (q_len > 1 branch,
/// llama.rs:1066-1112).  q and k_new arrive rotated (`qk_prologue_apply_gpu` is the one-launch pre-pass).
///
/// # Safety
/// As above.
#[allow(clippy::too_many_arguments)]
pub unsafe fn prefill_attn_int8_gpu(q: *const c_void, k_new: *const c_void, v_new: *const c_void, k_codes: *mut i8,
                                    v_codes: *mut i8, k_scales: *mut f32, v_scales: *mut f32, layout: &hs_kv_layout,
                                    hist_len: i32, out: *mut c_void, s: i32, shape: AttnShape, softmax_scale: f32,
                                    quantize_on_write: bool, stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_prefill_attn_int8(q, k_new, v_new, k_codes, v_codes, k_scales, v_scales, layout, hist_len, out,
                                         shape.b, s, shape.hq, shape.hkv, shape.d, softmax_scale,
                                         quantize_on_write as c_int, stream))
}

/// QK-norm + rotary embedding of q and k in one launch (apply_qk_norm / apply_qknorm then apply_rope).
///
/// # Safety
/// As above; `q_out` / `k_out` are buffers of their own (the rotation does not run in place).
#[allow(clippy::too_many_arguments)]
pub unsafe fn qk_prologue_apply_gpu(q: *const c_void, k: *const c_void, dtype: c_int, prologue: &hs_qk_prologue,
                                    positions: *const i32, start_pos: i32, q_out: *mut c_void, k_out: *mut c_void,
                                    s: i32, shape: AttnShape, stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_qk_prologue_apply(q, k, dtype, prologue, positions, start_pos, q_out, k_out, shape.b, s, shape.hq,
                                         shape.hkv, shape.d, stream))
}

/// Gated delta rule over `t` tokens (decode branch qwen3_5.rs:725-751 for t == 1, chunked_delta_rule otherwise).
///
/// # Safety
/// As above.
#[allow(clippy::too_many_arguments)]
pub unsafe fn deltanet_forward_gpu(q: *const c_void, k: *const c_void, v: *const c_void, g: *const f32, beta: *const f32,
                                   state: *mut f32, out: *mut f32, b: i32, t: i32, nk: i32, nv: i32, dk: i32, dv: i32,
                                   q_scale: f32, l2norm: bool, stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_deltanet_forward(q, k, v, g, beta, state, out, b, t, nk, nv, dk, dv, q_scale, l2norm as c_int, stream))
}

/// chunked_delta_rule (qwen3_5.rs:342-498) followed by RMSNormGated (qwen3_5.rs:305-313) in one call: `out` is the
/// bf16 normed tensor, the fp32 rows between the two pass through the workspace.
///
/// # Safety
/// As above; `workspace` holds at least `hs_deltanet_chunked_gated_norm_workspace_bytes(b, t, nk, nv)` bytes.
#[allow(clippy::too_many_arguments)]
pub unsafe fn deltanet_forward_chunked_gated_norm_gpu(q: *const c_void, k: *const c_void, v: *const c_void, g: *const f32,
                                                      beta: *const f32, state: *mut f32, z: *const c_void,
                                                      norm_weight: *const f32, norm_eps: f32, out: *mut c_void, b: i32, t: i32,
                                                      nk: i32, nv: i32, dk: i32, dv: i32, q_scale: f32, l2norm: bool,
                                                      workspace: *mut c_void, workspace_bytes: usize,
                                                      stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_deltanet_forward_chunked_gated_norm(q, k, v, g, beta, state, z, norm_weight, norm_eps, out, b, t, nk, nv,
                                                           dk, dv, q_scale, l2norm as c_int, workspace, workspace_bytes,
                                                           stream))
}

/// The prompt branch of a gated-DeltaNet layer between its projections in one call (conv1d + SiLU + gates, the chunked
/// delta rule, RMSNormGated: GatedDeltaNetLayer::forward, qwen3_5.rs:629-786 with seq > 1).
///
/// # Safety
/// As above; `workspace` holds at least `hs_deltanet_prefill_layer_workspace_bytes(..)` bytes, 256-byte aligned.
#[allow(clippy::too_many_arguments)]
pub unsafe fn deltanet_prefill_layer_gpu(mixed_qkv: *const c_void, conv_weight: *const c_void, conv_state_in: *const c_void,
                                         conv_state_out: *mut c_void, a_in: *const c_void, b_in: *const c_void,
                                         neg_a_exp: *const f32, dt_bias: *const f32, z: *const c_void, norm_weight: *const f32,
                                         norm_eps: f32, state: *mut f32, out: *mut c_void, b: i32, s: i32, nk: i32, nv: i32,
                                         dk: i32, dv: i32, q_scale: f32, l2norm: bool, workspace: *mut c_void,
                                         workspace_bytes: usize, stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_deltanet_prefill_layer(mixed_qkv, conv_weight, conv_state_in, conv_state_out, a_in, b_in, neg_a_exp,
                                              dt_bias, z, norm_weight, norm_eps, state, out, b, s, nk, nv, dk, dv, q_scale,
                                              l2norm as c_int, workspace, workspace_bytes, stream))
}

/// One decode step of a gated-DeltaNet layer between its projections in a single launch (conv1d + SiLU + gates,
/// the recurrent step, RMSNormGated: GatedDeltaNetLayer::forward, qwen3_5.rs:629-786 with seq == 1).
///
/// # Safety
/// As above; `conv_state_out` must not alias `conv_state_in`.
#[allow(clippy::too_many_arguments)]
pub unsafe fn deltanet_decode_layer_gpu(mixed_qkv: *const c_void, conv_weight: *const c_void, conv_state_in: *const c_void,
                                        conv_state_out: *mut c_void, a_in: *const c_void, b_in: *const c_void,
                                        neg_a_exp: *const f32, dt_bias: *const f32, z: *const c_void, norm_weight: *const f32,
                                        norm_eps: f32, state: *mut f32, out: *mut c_void, b: i32, nk: i32, nv: i32, dk: i32,
                                        dv: i32, q_scale: f32, l2norm: bool, stream: hs_stream_t) -> Result<()> {
    check(bindings::hs_deltanet_decode_layer(mixed_qkv, conv_weight, conv_state_in, conv_state_out, a_in, b_in, neg_a_exp,
                                             dt_bias, z, norm_weight, norm_eps, state, out, b, nk, nv, dk, dv, q_scale,
                                             l2norm as c_int, stream))
}

/// Bytes of split-K workspace a decode call of this shape may need.
pub fn decode_workspace_bytes(shape: AttnShape, max_seq_len: i32) -> usize {
    unsafe { bindings::hs_decode_attn_workspace_bytes(shape.b, shape.hq, shape.hkv, shape.d, max_seq_len) }
}

/// Bytes of workspace of the chunked delta rule (`deltanet_forward_chunked*`): the per-chunk factors, and with
/// `with_gated_norm` also the fp32 rows between the walk and the norm.
pub fn deltanet_chunked_workspace_bytes(b: i32, t: i32, nk: i32, nv: i32, with_gated_norm: bool) -> usize {
    unsafe {
        if with_gated_norm {
            bindings::hs_deltanet_chunked_gated_norm_workspace_bytes(b, t, nk, nv)
        } else {
            bindings::hs_deltanet_chunked_workspace_bytes(b, t, nk, nv)
        }
    }
}

/// Bytes of workspace of `deltanet_prefill_layer_gpu` (256-byte aligned).
pub fn deltanet_prefill_layer_workspace_bytes(b: i32, s: i32, nk: i32, nv: i32, dk: i32, dv: i32) -> usize {
    unsafe { bindings::hs_deltanet_prefill_layer_workspace_bytes(b, s, nk, nv, dk, dv) }
}
