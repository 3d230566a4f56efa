//! Raw bindings to `libhf2q_hip.so` (`include/hf2q_hip.h`), plus a few thin safe helpers.
//!
//! The `extern "C"` block below mirrors the header entry for entry, in the header's order, with the header's
//! parameter names.  Every function that returns `c_int` returns an `HqStatus` value; `hq_last_error()` holds the
//! message of the calling thread's last failure.  `stream` is a `hipStream_t` (null = the default stream); every
//! pointer named x, w, y, codes, norms, ... is DEVICE memory unless its comment in the header says otherwise.
//!
//! This crate is source only: the image this library is developed in has no Rust toolchain.  A test of the
//! repository (`tests/test_bindings.py`) checks that the block declares exactly the header's functions with the
//! header's parameter names and that the `#[repr(C)]` structs list the header's fields in order.
#![allow(non_camel_case_types)]

use core::ffi::{c_char, c_int, c_void};

/// `hq_status`
#[repr(C)]
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum HqStatus {
    Ok = 0,
    InvalidArgument = 1,
    Unsupported = 2,
    Hip = 3,
}

/// `hq_ggml_type`: GGML's own type ids.
#[repr(C)]
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum hq_ggml_type {
    HQ_Q4_0 = 2,
    HQ_Q8_0 = 8,
    HQ_Q4_K = 12,
    HQ_Q5_K = 13,
    HQ_Q6_K = 14,
}

/// `hq_act_dtype`; `HQ_F16` is an output type of `hq_dequant_ggml` only.
#[repr(C)]
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum hq_act_dtype {
    HQ_F32 = 0,
    HQ_BF16 = 1,
    HQ_F16 = 2,
}

pub const HQ_QMATMUL_BATCH_MAX_JOBS: u32 = 4;
pub const HQ_TQ_STATIC_TMP_BYTES: usize = 4 << 20;
pub const HQ_TQP_HEADER_BYTES: usize = 40;
pub const HQ_TQP_FLAG_HADAMARD_ROTATED: u32 = 1;
pub const HQ_TQP_FLAG_SPLIT_CHANNEL_25BIT: u32 = 2;

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct hq_qmatmul_job {
    pub x: *const c_void,
    pub x_up: *const c_void,
    pub w: *const c_void,
    pub ids: *const u32,
    pub y: *mut f32,
    pub rows: u32,
    pub top_k: u32,
    pub n: u32,
    pub k: u32,
    pub n_experts: u32,
    pub expert_stride: u64,
    pub route_logits: *const f32,
    pub route_ids: *mut u32,
    pub route_weights: *mut f32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct hq_moe_ffn_layer {
    pub router: *const c_void,
    pub shared_gate_logit: *const c_void,
    pub expert_gate: *const c_void,
    pub expert_up: *const c_void,
    pub expert_down: *const c_void,
    pub shared_gate: *const c_void,
    pub shared_up: *const c_void,
    pub shared_down: *const c_void,
    pub hidden: u32,
    pub n_experts: u32,
    pub top_k: u32,
    pub inter: u32,
    pub shared_inter: u32,
    pub ggml_type: hq_ggml_type,
    pub expert_stride_gate_up: u64,
    pub expert_stride_down: u64,
    pub down_type: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct hq_moe_ffn_row_scales {
    pub expert_gate: *const f32,
    pub expert_up: *const f32,
    pub expert_down: *const f32,
    pub shared_gate: *const f32,
    pub shared_up: *const f32,
    pub shared_down: *const f32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct hq_tq_attn_params {
    pub num_heads: u32,
    pub num_kv_heads: u32,
    pub head_dim: u32,
    pub kv_seq_len: u32,
    pub kv_capacity: u32,
    pub scale: f32,
    pub mask_type: u32,
    pub sliding_window: u32,
    pub softcap: f32,
    pub ring_start: u32,
    pub scale_factor_d512: f32,
    pub codebook_bits: u32,
    pub fuse_fwht_pre: u32,
    pub nsg: u32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct hq_tqp_header {
    pub codec_version: u32,
    pub bits_per_coord: u32,
    pub head_dim: u32,
    pub n_kv_heads: u32,
    pub n_tokens: u32,
    pub flags: u32,
    pub scale: f64,
}

/// Opaque handle of an open GGUF file.
#[repr(C)]
pub struct hq_gguf {
    _private: [u8; 0],
}

#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct hq_gguf_tensor_info {
    pub ggml_type: u32,
    pub n_dims: u32,
    pub dims: [u64; 4],
    pub data_offset: u64,
    pub byte_len: u64,
}

extern "C" {
    pub fn hq_last_error() -> *const c_char;
    pub fn hq_version() -> c_int;
    pub fn hq_block_elems(t: hq_ggml_type) -> u32;
    pub fn hq_block_bytes(t: hq_ggml_type) -> u32;
    pub fn hq_dequant_ggml(stream: *mut c_void, w_blocks: *const c_void, out: *mut c_void, out_dtype: hq_act_dtype, n_elems: u64, t: hq_ggml_type) -> c_int;
    pub fn hq_quantize_ggml(stream: *mut c_void, src: *const f32, n_elems: u64, n_per_row: u64, t: hq_ggml_type, out_blocks: *mut c_void) -> c_int;
    pub fn hq_quantize_ggml_imatrix_scratch_bytes(n_elems: u64, n_per_row: u64, t: hq_ggml_type) -> usize;
    pub fn hq_quantize_ggml_imatrix(stream: *mut c_void, src: *const f32, n_elems: u64, n_per_row: u64, t: hq_ggml_type, imatrix: *const f32, out_blocks: *mut c_void, scratch: *mut c_void, scratch_bytes: usize) -> c_int;
    pub fn hq_qmatmul_ggml(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_blocks: *const c_void, y: *mut f32, m: u32, n: u32, k: u32, t: hq_ggml_type) -> c_int;
    pub fn hq_qmatmul_ggml_k_slices(m: u32, n: u32, k: u32, t: hq_ggml_type, slices: *mut u32, blocks_per_slice: *mut u32) -> c_int;
    pub fn hq_gemv_flat_plan(n: u32, k: u32, t: hq_ggml_type, waves: u32, units_per_row: *mut u32, rows_per_task: *mut u32, windows_per_task: *mut u32, units_per_window: *mut u32, window_capacity: *mut u32) -> c_int;
    pub fn hq_qmatmul_ggml_workspace_bytes(m: u32, n: u32, k: u32, xdt: hq_act_dtype, t: hq_ggml_type) -> usize;
    pub fn hq_qmatmul_ggml_ws(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_blocks: *const c_void, y: *mut f32, m: u32, n: u32, k: u32, t: hq_ggml_type, workspace: *mut c_void, workspace_bytes: usize) -> c_int;
    pub fn hq_qmatmul_gated_ggml_workspace_bytes(m: u32, n: u32, k: u32, xdt: hq_act_dtype, t: hq_ggml_type) -> usize;
    pub fn hq_qmatmul_gated_ggml_ws(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_blocks: *const c_void, w_row_scales: *const f32, gate: *const f32, y: *mut f32, m: u32, n: u32, k: u32, t: hq_ggml_type, workspace: *mut c_void, workspace_bytes: usize) -> c_int;
    pub fn hq_qmatmul_swiglu_ggml_workspace_bytes(m: u32, n: u32, k: u32, xdt: hq_act_dtype, t: hq_ggml_type) -> usize;
    pub fn hq_qmatmul_swiglu_ggml_ws(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_gate: *const c_void, w_up: *const c_void, gate_row_scales: *const f32, up_row_scales: *const f32, y: *mut f32, m: u32, n: u32, k: u32, t: hq_ggml_type, workspace: *mut c_void, workspace_bytes: usize) -> c_int;
    pub fn hq_qmatmul_swiglu_decode_supported(n: u32, k: u32, t: hq_ggml_type, xdt: hq_act_dtype) -> c_int;
    pub fn hq_qmatmul_swiglu_decode(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_gate: *const c_void, w_up: *const c_void, y: *mut f32, m: u32, n: u32, k: u32, t: hq_ggml_type) -> c_int;
    pub fn hq_qmatmul_perm021_ggml_workspace_bytes(m: u32, n: u32, k: u32, xdt: hq_act_dtype, t: hq_ggml_type) -> usize;
    pub fn hq_qmatmul_perm021_ggml_ws(stream: *mut c_void, x_perm: *const c_void, xdt: hq_act_dtype, w_blocks: *const c_void, y: *mut f32, m: u32, n: u32, k: u32, head_dim: u32, t: hq_ggml_type, workspace: *mut c_void, workspace_bytes: usize) -> c_int;
    pub fn hq_qmatmul_id_ggml(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_stack: *const c_void, ids: *const u32, y: *mut f32, scratch: *mut c_void, scratch_bytes: usize, n_tokens: u32, top_k: u32, n: u32, k: u32, n_experts: u32, expert_stride: u64, t: hq_ggml_type) -> c_int;
    pub fn hq_weight_row_scales_ggml(stream: *mut c_void, w_blocks: *const c_void, scales: *mut f32, n_rows: u64, k: u32, t: hq_ggml_type) -> c_int;
    pub fn hq_qmatmul_ggml_ws_prepared(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_blocks: *const c_void, w_row_scales: *const f32, y: *mut f32, m: u32, n: u32, k: u32, t: hq_ggml_type, workspace: *mut c_void, workspace_bytes: usize) -> c_int;
    pub fn hq_qmatmul_id_ggml_prepared(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_stack: *const c_void, w_row_scales: *const f32, ids: *const u32, y: *mut f32, scratch: *mut c_void, scratch_bytes: usize, n_tokens: u32, top_k: u32, n: u32, k: u32, n_experts: u32, expert_stride: u64, t: hq_ggml_type) -> c_int;
    pub fn hq_qmatmul_id_swiglu_ggml_workspace_bytes(n_tokens: u32, top_k: u32, n: u32, k: u32, n_experts: u32, expert_stride: u64, t: hq_ggml_type) -> usize;
    pub fn hq_qmatmul_id_swiglu_ggml(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_gate_stack: *const c_void, w_up_stack: *const c_void, gate_row_scales: *const f32, up_row_scales: *const f32, ids: *const u32, y: *mut f32, scratch: *mut c_void, scratch_bytes: usize, n_tokens: u32, top_k: u32, n: u32, k: u32, n_experts: u32, expert_stride: u64, t: hq_ggml_type) -> c_int;
    pub fn hq_qmatmul_id_scratch_bytes(n_experts: u32, max_rows: u32) -> usize;
    pub fn hq_qmatmul_id_ggml_workspace_bytes(n_tokens: u32, top_k: u32, n: u32, k: u32, n_experts: u32, expert_stride: u64, t: hq_ggml_type) -> usize;
    pub fn hq_qmatmul_batch_ggml(stream: *mut c_void, jobs: *const hq_qmatmul_job, n_jobs: u32, xdt: hq_act_dtype, t: hq_ggml_type) -> c_int;
    pub fn hq_dense_gemv_bf16(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_bf16: *const c_void, y: *mut f32, m: u32, n: u32, k: u32) -> c_int;
    pub fn hq_dense_gemv_bf16_pair(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_a: *const c_void, y_a: *mut f32, n_a: u32, w_b: *const c_void, y_b: *mut f32, n_b: u32, m: u32, k: u32) -> c_int;
    pub fn hq_moe_softmax_topk(stream: *mut c_void, logits: *const f32, ids: *mut u32, weights: *mut f32, n_tokens: u32, n_experts: u32, top_k: u32) -> c_int;
    pub fn hq_silu_mul(stream: *mut c_void, gate: *const f32, up: *const f32, out: *mut f32, n: u64) -> c_int;
    pub fn hq_moe_weighted_reduce(stream: *mut c_void, y: *const f32, w: *const f32, shared: *const f32, shared_logit: *const f32, residual: *const f32, out: *mut f32, n_tokens: u32, top_k: u32, hidden: u32) -> c_int;
    pub fn hq_moe_ffn_decode_scratch_bytes(n_tokens: u32, hidden: u32, n_experts: u32, top_k: u32, inter: u32, shared_inter: u32, t: hq_ggml_type, xdt: hq_act_dtype) -> usize;
    pub fn hq_moe_ffn_decode_layer_scratch_bytes(layer: *const hq_moe_ffn_layer, n_tokens: u32, xdt: hq_act_dtype) -> usize;
    pub fn hq_moe_ffn_decode(stream: *mut c_void, layer: *const hq_moe_ffn_layer, x: *const c_void, xdt: hq_act_dtype, residual: *const f32, out: *mut f32, n_tokens: u32, scratch: *mut c_void, scratch_bytes: usize, route_ids: *mut u32, route_weights: *mut f32) -> c_int;
    pub fn hq_handover_status(stream: *mut c_void, scratch: *const c_void, error: *mut u32) -> c_int;
    pub fn hq_set_handover_spin_limit(limit: u32);
    pub fn hq_dense_ffn_decode_scratch_bytes(hidden: u32, inter: u32, t_gate_up: hq_ggml_type, t_down: hq_ggml_type, xdt: hq_act_dtype) -> usize;
    pub fn hq_dense_ffn_decode(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_gate: *const c_void, w_up: *const c_void, w_down: *const c_void, t_gate_up: hq_ggml_type, t_down: hq_ggml_type, residual: *const f32, out: *mut f32, hidden: u32, inter: u32, scratch: *mut c_void, scratch_bytes: usize) -> c_int;
    pub fn hq_moe_ffn_prefill_scratch_bytes(layer: *const hq_moe_ffn_layer, n_tokens: u32, xdt: hq_act_dtype) -> usize;
    pub fn hq_moe_ffn_prefill(stream: *mut c_void, layer: *const hq_moe_ffn_layer, row_scales: *const hq_moe_ffn_row_scales, x: *const c_void, xdt: hq_act_dtype, residual: *const f32, out: *mut f32, n_tokens: u32, scratch: *mut c_void, scratch_bytes: usize, route_ids: *mut u32, route_weights: *mut f32) -> c_int;
    pub fn hq_dense_ffn_scratch_bytes(m: u32, hidden: u32, inter: u32, t_gate_up: hq_ggml_type, t_down: hq_ggml_type, xdt: hq_act_dtype) -> usize;
    pub fn hq_dense_ffn(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_gate: *const c_void, w_up: *const c_void, w_down: *const c_void, t_gate_up: hq_ggml_type, t_down: hq_ggml_type, gate_row_scales: *const f32, up_row_scales: *const f32, down_row_scales: *const f32, out: *mut f32, m: u32, hidden: u32, inter: u32, scratch: *mut c_void, scratch_bytes: usize) -> c_int;
    pub fn hq_fwht_sign_premult_f32(stream: *mut c_void, buf: *mut f32, n_heads: u32, head_dim: u32) -> c_int;
    pub fn hq_fwht_sign_undo_f32(stream: *mut c_void, buf: *mut f32, n_heads: u32, head_dim: u32) -> c_int;
    pub fn hq_tq_encode_kv(stream: *mut c_void, src: *const f32, codes: *mut u8, norms: *mut f32, n_tokens: u32, n_kv_heads: u32, head_dim: u32, capacity: u32, write_pos: u32) -> c_int;
    pub fn hq_tq_dequantize_kv_seq(stream: *mut c_void, codes: *const u8, norms: *const f32, lut256: *const f32, dst: *mut f32, n_kv_heads: u32, head_dim: u32, capacity: u32, start_pos: u32, n_tokens: u32, scale_factor_d512: f32, codebook_bits: u32, unrotate: c_int) -> c_int;
    pub fn hq_flash_attn_vec_tq(stream: *mut c_void, q: *const f32, k_codes: *const u8, k_norms: *const f32, v_codes: *const u8, v_norms: *const f32, lut256: *const f32, out: *mut f32, tmp: *mut c_void, tmp_bytes: usize, p: *const hq_tq_attn_params) -> c_int;
    pub fn hq_flash_attn_vec_tq_undo(stream: *mut c_void, q: *const f32, k_codes: *const u8, k_norms: *const f32, v_codes: *const u8, v_norms: *const f32, lut256: *const f32, out: *mut f32, tmp: *mut c_void, tmp_bytes: usize, p: *const hq_tq_attn_params) -> c_int;
    pub fn hq_flash_attn_vec_tq_tmp_bytes(num_heads: u32, head_dim: u32, kv_seq_len: u32) -> usize;
    pub fn hq_flash_attn_vec_tq_static(stream: *mut c_void, q: *const f32, k_codes: *const u8, k_norms: *const f32, v_codes: *const u8, v_norms: *const f32, lut256: *const f32, out: *mut f32, p: *const hq_tq_attn_params, undo_rotation: c_int) -> c_int;
    pub fn hq_tqp_indices_bytes(h: *const hq_tqp_header) -> usize;
    pub fn hq_tqp_norms_bytes(h: *const hq_tqp_header) -> usize;
    pub fn hq_tqp_total_bytes(h: *const hq_tqp_header) -> usize;
    pub fn hq_tqp_pack(h: *const hq_tqp_header, indices: *const c_void, indices_len: usize, norms_le: *const c_void, norms_len: usize, out: *mut c_void, out_capacity: usize) -> c_int;
    pub fn hq_tqp_unpack(payload: *const c_void, len: usize, h: *mut hq_tqp_header, indices_offset: *mut usize, norms_offset: *mut usize) -> c_int;
    pub fn hq_tq_kv_capture_bytes(n_kv_heads: u32, head_dim: u32, n_tokens: u32) -> usize;
    pub fn hq_tq_kv_capture(stream: *mut c_void, codes: *const u8, norms: *const f32, n_kv_heads: u32, head_dim: u32, capacity: u32, start_pos: u32, n_tokens: u32, payload: *mut c_void, payload_capacity: usize) -> c_int;
    pub fn hq_tq_kv_restore(stream: *mut c_void, payload: *const c_void, len: usize, codes: *mut u8, norms: *mut f32, n_kv_heads: u32, head_dim: u32, capacity: u32, start_pos: u32) -> c_int;
    pub fn hq_matmul_f16_shadow_workspace_bytes(m: u32, n: u32, k: u32) -> usize;
    pub fn hq_matmul_f16_shadow(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_f16: *const c_void, y: *mut f32, m: u32, n: u32, k: u32, workspace: *mut c_void, workspace_bytes: usize) -> c_int;
    pub fn hq_dense_matmul_workspace_bytes(m: u32, n: u32, k: u32, xdt: hq_act_dtype, wdt: hq_act_dtype) -> usize;
    pub fn hq_dense_matmul(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w: *const c_void, wdt: hq_act_dtype, y: *mut f32, m: u32, n: u32, k: u32, workspace: *mut c_void, workspace_bytes: usize) -> c_int;
    pub fn hq_stream_read_probe(stream: *mut c_void, buf: *const c_void, bytes: usize, sink: *mut u32) -> c_int;
    pub fn hq_gguf_open(path: *const c_char, out: *mut *mut hq_gguf) -> c_int;
    pub fn hq_gguf_close(g: *mut hq_gguf);
    pub fn hq_gguf_tensor_count(g: *const hq_gguf) -> u64;
    pub fn hq_gguf_metadata_count(g: *const hq_gguf) -> u64;
    pub fn hq_gguf_alignment(g: *const hq_gguf) -> u64;
    pub fn hq_gguf_tensor_name(g: *const hq_gguf, index: u64) -> *const c_char;
    pub fn hq_gguf_metadata_key(g: *const hq_gguf, index: u64) -> *const c_char;
    pub fn hq_gguf_tensor_info_by_name(g: *const hq_gguf, name: *const c_char, out: *mut hq_gguf_tensor_info) -> c_int;
    pub fn hq_gguf_metadata_u64(g: *const hq_gguf, key: *const c_char, out: *mut u64) -> c_int;
    pub fn hq_gguf_metadata_f64(g: *const hq_gguf, key: *const c_char, out: *mut f64) -> c_int;
    pub fn hq_gguf_metadata_string(g: *const hq_gguf, key: *const c_char, out: *mut *const c_char, len: *mut u64) -> c_int;
    pub fn hq_gguf_tensor_data(g: *const hq_gguf, name: *const c_char, byte_len: *mut u64) -> *const c_void;
    pub fn hq_gguf_load_tensor(g: *const hq_gguf, name: *const c_char, stream: *mut c_void, dev_dst: *mut c_void, dst_bytes: usize) -> c_int;
}

/// A failed call: the status code and the library's message for it.
#[derive(Debug, Clone)]
pub struct HqError {
    pub status: c_int,
    pub message: String,
}

impl core::fmt::Display for HqError {
    fn fmt(&self, f: &mut core::fmt::Formatter<'_>) -> core::fmt::Result {
        write!(f, "hf2q_hip status {}: {}", self.status, self.message)
    }
}

impl std::error::Error for HqError {}

/// Turns a status code into a `Result`, reading `hq_last_error()` on failure.
pub fn check(status: c_int) -> Result<(), HqError> {
    if status == HqStatus::Ok as c_int {
        return Ok(());
    }
    // SAFETY: hq_last_error returns a NUL-terminated string owned by the library (thread-local, valid until the
    // thread's next failing call).
    let message = unsafe {
        let p = hq_last_error();
        if p.is_null() { String::new() } else { std::ffi::CStr::from_ptr(p).to_string_lossy().into_owned() }
    };
    Err(HqError { status, message })
}

/// Bytes of `n_elems` weights of type `t` (`n_elems` a multiple of the block size).
pub fn ggml_bytes(t: hq_ggml_type, n_elems: u64) -> u64 {
    // SAFETY: pure functions of the enum.
    let (be, bb) = unsafe { (hq_block_elems(t) as u64, hq_block_bytes(t) as u64) };
    n_elems / be * bb
}

/// The dense product `y[m, n] = x[m, k] . W[n, k]^T` with caller-owned scratch: the form for prefill call sites
/// (`quantized_matmul_ggml` with m > 8), which must not allocate inside a captured graph.
///
/// # Safety
/// All pointers are device pointers of at least the sizes the header states; `workspace` holds
/// `hq_qmatmul_ggml_workspace_bytes(m, n, k, xdt, t)` bytes, 256-byte aligned (null when that is 0).
#[allow(clippy::too_many_arguments)]
pub unsafe fn qmatmul_ggml_ws(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_blocks: *const c_void, y: *mut f32, m: u32, n: u32, k: u32, t: hq_ggml_type, workspace: *mut c_void, workspace_bytes: usize) -> Result<(), HqError> {
    check(hq_qmatmul_ggml_ws(stream, x, xdt, w_blocks, y, m, n, k, t, workspace, workspace_bytes))
}

/// The weight-row scales of the f16 tile kernels (`n_rows` floats; a contiguous expert stack counts its experts' rows
/// in order).  They depend on the weights alone: compute them once after a tensor's blocks are uploaded, keep the
/// buffer beside the weight and pass it to the `_prepared` calls, whose pre-pass then skips the scan of the block
/// headers (same results to the bit).
///
/// # Safety
/// Device pointers: `w_blocks` holds `n_rows` rows of `k` weights of type `t`, `scales` has room for `n_rows` floats.
pub unsafe fn weight_row_scales_ggml(stream: *mut c_void, w_blocks: *const c_void, scales: *mut f32, n_rows: u64, k: u32, t: hq_ggml_type) -> Result<(), HqError> {
    check(hq_weight_row_scales_ggml(stream, w_blocks, scales, n_rows, k, t))
}

/// `qmatmul_ggml_ws` with the weight's row scales from `weight_row_scales_ggml`.
///
/// # Safety
/// As `qmatmul_ggml_ws`; `w_row_scales` holds the `n` floats computed for exactly these `w_blocks`.
#[allow(clippy::too_many_arguments)]
pub unsafe fn qmatmul_ggml_ws_prepared(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_blocks: *const c_void, w_row_scales: *const f32, y: *mut f32, m: u32, n: u32, k: u32, t: hq_ggml_type, workspace: *mut c_void, workspace_bytes: usize) -> Result<(), HqError> {
    check(hq_qmatmul_ggml_ws_prepared(stream, x, xdt, w_blocks, w_row_scales, y, m, n, k, t, workspace, workspace_bytes))
}

/// `qmatmul_id_ggml` with the stack's row scales (`n_experts * n` floats) from `weight_row_scales_ggml`.
///
/// # Safety
/// As `qmatmul_id_ggml`; `w_row_scales` holds the floats computed for exactly this `w_stack`.
#[allow(clippy::too_many_arguments)]
pub unsafe fn qmatmul_id_ggml_prepared(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_stack: *const c_void, w_row_scales: *const f32, ids: *const u32, y: *mut f32, scratch: *mut c_void, scratch_bytes: usize, n_tokens: u32, top_k: u32, n: u32, k: u32, n_experts: u32, expert_stride: u64, t: hq_ggml_type) -> Result<(), HqError> {
    check(hq_qmatmul_id_ggml_prepared(stream, x, xdt, w_stack, w_row_scales, ids, y, scratch, scratch_bytes, n_tokens, top_k, n, k, n_experts, expert_stride, t))
}

/// `quantized_matmul_id_ggml`: one product per (token, slot) with the slot's expert.  `scratch` = null keeps the
/// per-row GEMV form; with `hq_qmatmul_id_ggml_workspace_bytes(..)` bytes of scratch, prefill-sized inputs are
/// sorted by expert and multiplied as tiles.
///
/// # Safety
/// Device pointers as the header states; ids outside `0..n_experts` give NaN rows, not an error.
#[allow(clippy::too_many_arguments)]
pub unsafe fn qmatmul_id_ggml(stream: *mut c_void, x: *const c_void, xdt: hq_act_dtype, w_stack: *const c_void, ids: *const u32, y: *mut f32, scratch: *mut c_void, scratch_bytes: usize, n_tokens: u32, top_k: u32, n: u32, k: u32, n_experts: u32, expert_stride: u64, t: hq_ggml_type) -> Result<(), HqError> {
    check(hq_qmatmul_id_ggml(stream, x, xdt, w_stack, ids, y, scratch, scratch_bytes, n_tokens, top_k, n, k, n_experts, expert_stride, t))
}

/// The MoE FFN block of a decode step (1..8 tokens) as one launch.  `scratch` holds
/// `hq_moe_ffn_decode_scratch_bytes(..)` bytes that were zeroed once when they were allocated; the library keeps
/// its call counter there, so the same scratch must not serve two calls that overlap in time.
///
/// # Safety
/// Device pointers as the header states.
#[allow(clippy::too_many_arguments)]
pub unsafe fn moe_ffn_decode(stream: *mut c_void, layer: &hq_moe_ffn_layer, x: *const c_void, xdt: hq_act_dtype, residual: *const f32, out: *mut f32, n_tokens: u32, scratch: *mut c_void, scratch_bytes: usize, route_ids: *mut u32, route_weights: *mut f32) -> Result<(), HqError> {
    check(hq_moe_ffn_decode(stream, layer, x, xdt, residual, out, n_tokens, scratch, scratch_bytes, route_ids, route_weights))
}

/// TurboQuant decode attention with the library's own static scratch (no allocation, no scratch argument): for
/// callers that cannot allocate.  Fails when the shape needs more than `HQ_TQ_STATIC_TMP_BYTES`; calls that
/// overlap on one GPU race on that scratch.
///
/// # Safety
/// Device pointers as the header states.
#[allow(clippy::too_many_arguments)]
pub unsafe fn flash_attn_vec_tq_static(stream: *mut c_void, q: *const f32, k_codes: *const u8, k_norms: *const f32, v_codes: *const u8, v_norms: *const f32, lut256: *const f32, out: *mut f32, p: &hq_tq_attn_params, undo_rotation: bool) -> Result<(), HqError> {
    check(hq_flash_attn_vec_tq_static(stream, q, k_codes, k_norms, v_codes, v_norms, lut256, out, p, undo_rotation as c_int))
}

/// An open GGUF file; closed on drop.
pub struct Gguf(*mut hq_gguf);

impl Gguf {
    pub fn open(path: &std::ffi::CStr) -> Result<Self, HqError> {
        let mut g: *mut hq_gguf = core::ptr::null_mut();
        // SAFETY: path is NUL-terminated, g receives an owned handle on success.
        check(unsafe { hq_gguf_open(path.as_ptr(), &mut g) })?;
        Ok(Gguf(g))
    }
    pub fn tensor_count(&self) -> u64 {
        // SAFETY: self.0 is a live handle.
        unsafe { hq_gguf_tensor_count(self.0) }
    }
    pub fn tensor_info(&self, name: &std::ffi::CStr) -> Result<hq_gguf_tensor_info, HqError> {
        let mut info = hq_gguf_tensor_info::default();
        // SAFETY: live handle, NUL-terminated name, info is writable.
        check(unsafe { hq_gguf_tensor_info_by_name(self.0, name.as_ptr(), &mut info) })?;
        Ok(info)
    }
    /// Copies the tensor's bytes to device memory on `stream`.
    ///
    /// # Safety
    /// `dev_dst` is device memory of `dst_bytes` bytes.
    pub unsafe fn load_tensor(&self, name: &std::ffi::CStr, stream: *mut c_void, dev_dst: *mut c_void, dst_bytes: usize) -> Result<(), HqError> {
        check(hq_gguf_load_tensor(self.0, name.as_ptr(), stream, dev_dst, dst_bytes))
    }
    pub fn as_ptr(&self) -> *const hq_gguf {
        self.0
    }
}

impl Drop for Gguf {
    fn drop(&mut self) {
        // SAFETY: the handle came from hq_gguf_open and is closed once.
        unsafe { hq_gguf_close(self.0) }
    }
}
