//! Raw declarations of the C ABI of `libizwi_qmm.so`: every function of `include/izwi_qmm.h`,
//! `include/izwi_gguf.h` and `include/izwi_decode_ops.h`, with the same names, argument order and
//! pointer constness.  `tests/test_rust_binding.py` compares this block with the headers
//! mechanically (symbol set, argument count, pointer-ness of every argument and result), so the
//! two cannot drift apart unnoticed.  Semantics, sizes and error behaviour: the comments in the
//! headers.  Safe wrappers live in the `izwi-qmm` crate next to this one.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

/// `izwi_qmm_status`
pub const IZWI_QMM_OK: c_int = 0;
pub const IZWI_QMM_ERR_INVALID: c_int = -1;
pub const IZWI_QMM_ERR_UNSUPPORTED: c_int = -2;
pub const IZWI_QMM_ERR_HIP: c_int = -3;
pub const IZWI_QMM_ERR_NO_DEVICE: c_int = -4;

/// `izwi_qmm_mem_space`
pub const IZWI_QMM_DEVICE: c_int = 0;
pub const IZWI_QMM_HOST: c_int = 1;

/// `izwi_qmm_out_dtype`
pub const IZWI_QMM_OUT_F32: c_int = 0;
pub const IZWI_QMM_OUT_BF16: c_int = 1;

/// ggml type ids of the block formats the library multiplies (`GgmlDType`)
pub const IZWI_QMM_Q8_0: c_int = 8;
pub const IZWI_QMM_Q4_K: c_int = 12;
pub const IZWI_QMM_Q6_K: c_int = 14;

/// `izwi_qmm_large_m`
pub const IZWI_QMM_LARGE_M_BF16: c_int = 0;
pub const IZWI_QMM_LARGE_M_INT8: c_int = 1;

/// `izwi_qmm_prefill_form`
pub const IZWI_QMM_PREFILL_AUTO: c_int = -1;
pub const IZWI_QMM_PREFILL_LDS: c_int = 0;
pub const IZWI_QMM_PREFILL_PLANE: c_int = 1;

/// `izwi_gguf_mmap_mode` / `izwi_gguf_reader_kind`
pub const IZWI_GGUF_MMAP_AUTO: c_int = 0;
pub const IZWI_GGUF_MMAP_ON: c_int = 1;
pub const IZWI_GGUF_MMAP_OFF: c_int = 2;
pub const IZWI_GGUF_READER_BUFFERED: c_int = 0;
pub const IZWI_GGUF_READER_MAPPED: c_int = 1;

pub const IZWI_GGUF_MAX_DIMS: usize = 8;

/// Opaque: a `QTensor` + `QMatMul` on the device.
#[repr(C)]
pub struct IzwiQmmWeight {
    _private: [u8; 0],
}

/// Opaque: a chain of dependent one-row projection steps (experimental).
#[repr(C)]
pub struct IzwiQmmChain {
    _private: [u8; 0],
}

/// Opaque: an open GGUF file (`GgufLoader`).
#[repr(C)]
pub struct IzwiGguf {
    _private: [u8; 0],
}

/// `izwi_qmm_weight_info`
#[repr(C)]
#[derive(Debug, Default, Clone, Copy)]
pub struct IzwiQmmWeightInfo {
    pub ggml_dtype: i32,
    pub n_stacked: i32,
    pub n: i64,
    pub k: i64,
    pub nbytes: u64,
    pub device: i32,
    pub reserved: i32,
}

/// `izwi_qmm_profile_snapshot` == `Qwen3RuntimeProfileSnapshot` (qwen3/core.rs:571-582)
#[repr(C)]
#[derive(Debug, Default, Clone, Copy)]
pub struct IzwiQmmProfileSnapshot {
    pub qmatmul_calls: u64,
    pub qmatmul_ns: u64,
    pub qmatmul_input_casts: u64,
    pub qmatmul_input_cast_ns: u64,
    pub qmatmul_output_casts: u64,
    pub qmatmul_output_cast_ns: u64,
    pub lm_head_calls: u64,
    pub lm_head_ns: u64,
    pub silu_mul_fused_calls: u64,
    pub silu_mul_fallback_calls: u64,
}

/// `izwi_qmm_chain_step`
#[repr(C)]
#[derive(Clone, Copy)]
pub struct IzwiQmmChainStep {
    pub weights: [*const IzwiQmmWeight; 4],
    pub n_weights: i32,
    pub reserved: i32,
    pub x: *const f32,
    pub ys: [*mut f32; 4],
}

/// `izwi_gguf_tensor_info`
#[repr(C)]
#[derive(Clone, Copy)]
pub struct IzwiGgufTensorInfo {
    pub ggml_dtype: i32,
    pub n_dims: i32,
    pub dims: [i64; IZWI_GGUF_MAX_DIMS],
    pub offset: u64,
    pub nbytes: u64,
    pub data: *const c_void,
}

#[link(name = "izwi_qmm")]
extern "C" {
    // ---- include/izwi_qmm.h
    pub fn izwi_qmm_abi_version() -> c_int;
    pub fn izwi_qmm_init(device: c_int) -> c_int;
    pub fn izwi_qmm_last_error() -> *const c_char;
    pub fn izwi_qmm_storage_bytes(ggml_dtype: c_int, rows: i64, cols: i64, out_bytes: *mut u64) -> c_int;
    pub fn izwi_qmm_weight_create(ggml_dtype: c_int, n: i64, k: i64, blocks: *const c_void, nbytes: u64,
        mem_space: c_int, out: *mut *mut IzwiQmmWeight) -> c_int;
    pub fn izwi_qmm_weight_create_packed(ggml_dtype: c_int, n_parts: i32, part_rows: *const i64, k: i64,
        part_blocks: *const *const c_void, part_nbytes: *const u64, mem_space: c_int, out: *mut *mut IzwiQmmWeight) -> c_int;
    pub fn izwi_qmm_weight_create_stacked(ggml_dtype: c_int, n_experts: i32, n: i64, k: i64, blocks: *const c_void,
        nbytes: u64, mem_space: c_int, out: *mut *mut IzwiQmmWeight) -> c_int;
    pub fn izwi_qmm_quantize_weights_f32(ggml_dtype: c_int, w: *const f32, n: i64, k: i64, out_blocks: *mut c_void,
        mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_weight_destroy(w: *mut IzwiQmmWeight);
    pub fn izwi_qmm_weight_get_info(w: *const IzwiQmmWeight, out: *mut IzwiQmmWeightInfo) -> c_int;
    pub fn izwi_qmm_set_large_m_arithmetic(mode: c_int) -> c_int;
    pub fn izwi_qmm_get_large_m_arithmetic() -> c_int;
    pub fn izwi_qmm_set_prefill_form(form: c_int) -> c_int;
    pub fn izwi_qmm_get_prefill_form() -> c_int;
    pub fn izwi_qmm_set_moe_expert_form(enabled: c_int) -> c_int;
    pub fn izwi_qmm_scratch_reserve(bytes: u64, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_weight_data(w: *const IzwiQmmWeight, out_blocks: *mut c_void, nbytes: u64, mem_space: c_int,
        stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_dequantize_f32(w: *const IzwiQmmWeight, out: *mut f32, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_dequantize_rows(w: *const IzwiQmmWeight, row_ids: *const i32, n_rows: i64,
        ids_mem_space: c_int, out: *mut c_void, out_dtype: c_int, out_mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_forward_f32(w: *const IzwiQmmWeight, x: *const f32, m: i64, y: *mut f32, mem_space: c_int,
        stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_forward_rows_f32(w: *const IzwiQmmWeight, row_ids: *const u32, n_rows: i64, x: *const f32,
        m: i64, y: *mut f32, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_records_bytes(ggml_weight_dtype: c_int, m: i64, k: i64) -> u64;
    pub fn izwi_qmm_quantize_records_f32(ggml_weight_dtype: c_int, x: *const f32, m: i64, k: i64,
        records: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_silu_mul_quantize_records_f32(ggml_weight_dtype: c_int, gate: *const f32, up: *const f32,
        m: i64, k: i64, records: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_forward_group_records_f32(weights: *const *const IzwiQmmWeight, n_weights: i32,
        records: *const c_void, m: i64, ys: *const *mut f32, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_chain_create(steps: *const IzwiQmmChainStep, n_steps: i32, out: *mut *mut IzwiQmmChain) -> c_int;
    pub fn izwi_qmm_chain_destroy(chain: *mut IzwiQmmChain);
    pub fn izwi_qmm_chain_run(chain: *mut IzwiQmmChain, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_chain_status(chain: *mut IzwiQmmChain, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_chain_set_spin_limit(chain: *mut IzwiQmmChain, polls: u32) -> c_int;
    pub fn izwi_qmm_forward_f32_noalloc(w: *const IzwiQmmWeight, x: *const f32, m: i64, y: *mut f32,
        stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_forward_group_f32(weights: *const *const IzwiQmmWeight, n_weights: i32, x: *const f32, m: i64,
        ys: *const *mut f32, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_forward_group_bf16(weights: *const *const IzwiQmmWeight, n_weights: i32, x_bf16: *const u16,
        m: i64, ys: *const *mut c_void, out_dtype: c_int, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_forward_gate_up_silu_f32(gate: *const IzwiQmmWeight, up: *const IzwiQmmWeight, x: *const f32,
        m: i64, h: *mut f32, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_mlp_forward_f32(gate: *const IzwiQmmWeight, up: *const IzwiQmmWeight,
        down: *const IzwiQmmWeight, x: *const f32, m: i64, y: *mut f32, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_forward_bf16(w: *const IzwiQmmWeight, x_bf16: *const u16, m: i64, y: *mut c_void,
        out_dtype: c_int, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_forward_fused(w: *const IzwiQmmWeight, x: *const c_void, x_dtype: c_int, m: i64,
        residual: *const c_void, y: *mut c_void, y_dtype: c_int, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_forward_normed_f32(w: *const IzwiQmmWeight, x: *const f32, m: i64, norm_weight: *const f32,
        eps: f32, y: *mut f32, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_forward_group_normed_f32(weights: *const *const IzwiQmmWeight, n_weights: i32, x: *const f32,
        m: i64, norm_weight: *const f32, eps: f32, ys: *const *mut f32, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_forward_gate_up_silu_normed_f32(gate: *const IzwiQmmWeight, up: *const IzwiQmmWeight,
        x: *const f32, m: i64, norm_weight: *const f32, eps: f32, h: *mut f32, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_quantize_activations(ggml_weight_dtype: c_int, x: *const f32, m: i64, k: i64,
        out_blocks: *mut c_void, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_moe_route(logits: *const f32, t: i64, n_experts: i32, top_k: i32, ids: *mut i32, weights: *mut f32,
        mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_moe_sort(ids: *const i32, t: i64, top_k: i32, n_experts: i32, perm: *mut i32, offsets: *mut i32,
        mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_moe_forward_f32(gate: *const IzwiQmmWeight, up: *const IzwiQmmWeight, down: *const IzwiQmmWeight,
        x: *const f32, t: i64, ids: *const i32, weights: *const f32, top_k: i32, perm: *const i32,
        offsets: *const i32, out: *mut f32, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_moe_layer_f32(gate: *const IzwiQmmWeight, up: *const IzwiQmmWeight, down: *const IzwiQmmWeight,
        logits: *const f32, x: *const f32, t: i64, top_k: i32, out: *mut f32, ids_out: *mut i32,
        weights_out: *mut f32, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qmm_profile_enable(enabled: c_int) -> c_int;
    pub fn izwi_qmm_profile_enabled() -> c_int;
    pub fn izwi_qmm_profile_snapshot_get(out: *mut IzwiQmmProfileSnapshot) -> c_int;
    pub fn izwi_qmm_profile_reset() -> c_int;
    pub fn izwi_qmm_profile_argmax_get(calls: *mut u64, ns: *mut u64) -> c_int;
    pub fn izwi_qmm_weight_set_lm_head(w: *mut IzwiQmmWeight, is_lm_head: c_int) -> c_int;
    // ---- include/izwi_gguf.h
    pub fn izwi_gguf_is_gguf_file(path: *const c_char) -> c_int;
    pub fn izwi_gguf_open(path: *const c_char, out: *mut *mut IzwiGguf) -> c_int;
    pub fn izwi_gguf_close(g: *mut IzwiGguf);
    pub fn izwi_gguf_open_with_mode(path: *const c_char, mmap_mode: c_int, out: *mut *mut IzwiGguf) -> c_int;
    pub fn izwi_gguf_parse_mmap_mode(raw: *const c_char) -> c_int;
    pub fn izwi_gguf_resolve_mmap_mode(configured: c_int) -> c_int;
    pub fn izwi_gguf_reader_kind(g: *const IzwiGguf) -> c_int;
    pub fn izwi_gguf_header(g: *const IzwiGguf, version: *mut u32, alignment: *mut u32, data_offset: *mut u64) -> c_int;
    pub fn izwi_gguf_tensor_count(g: *const IzwiGguf) -> i64;
    pub fn izwi_gguf_tensor_name(g: *const IzwiGguf, index: i64, name: *mut *const c_char) -> c_int;
    pub fn izwi_gguf_tensor_info_get(g: *const IzwiGguf, name: *const c_char, out: *mut IzwiGgufTensorInfo) -> c_int;
    pub fn izwi_gguf_metadata_count(g: *const IzwiGguf) -> i64;
    pub fn izwi_gguf_metadata_key(g: *const IzwiGguf, index: i64, key: *mut *const c_char) -> c_int;
    pub fn izwi_gguf_metadata_type(g: *const IzwiGguf, key: *const c_char) -> c_int;
    pub fn izwi_gguf_metadata_string(g: *const IzwiGguf, key: *const c_char, str: *mut *const c_char, len: *mut u64) -> c_int;
    pub fn izwi_gguf_metadata_u64(g: *const IzwiGguf, key: *const c_char, value: *mut u64) -> c_int;
    pub fn izwi_gguf_metadata_f64(g: *const IzwiGguf, key: *const c_char, value: *mut f64) -> c_int;
    pub fn izwi_gguf_metadata_array(g: *const IzwiGguf, key: *const c_char, elem_type: *mut i32, count: *mut u64,
        data: *mut *const c_void) -> c_int;
    pub fn izwi_gguf_metadata_array_string(g: *const IzwiGguf, key: *const c_char, index: u64,
        str: *mut *const c_char, len: *mut u64) -> c_int;
    pub fn izwi_gguf_load_weight(g: *const IzwiGguf, name: *const c_char, out: *mut *mut IzwiQmmWeight) -> c_int;
    pub fn izwi_gguf_load_packed(g: *const IzwiGguf, names: *const *const c_char, n_names: i32,
        out: *mut *mut IzwiQmmWeight) -> c_int;
    pub fn izwi_gguf_load_tensor_f32(g: *const IzwiGguf, name: *const c_char, out: *mut f32, count: u64,
        mem_space: c_int, stream: *mut c_void) -> c_int;
    // ---- include/izwi_decode_ops.h
    pub fn izwi_rms_norm_f32(x: *const f32, weight: *const f32, rows: i64, hidden: i64, eps: f32, y: *mut f32,
        mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qk_rms_norm_f32(q: *const f32, k: *const f32, qk_weight: *const f32, q_rows: i64, k_rows: i64,
        head_dim: i64, eps: f32, q_out: *mut f32, k_out: *mut f32, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_rope_pair_bshd_f32(q: *const f32, k: *const f32, cos_sin: *const f32, batch: i64, seq: i64,
        q_heads: i64, k_heads: i64, head_dim: i64, q_out: *mut f32, k_out: *mut f32, mem_space: c_int,
        stream: *mut c_void) -> c_int;
    pub fn izwi_rms_norm_f16(x: *const u16, weight: *const u16, rows: i64, hidden: i64, eps: f32, y: *mut u16,
        mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_rms_norm_quantize_records_f32(ggml_weight_dtype: c_int, x: *const f32, weight: *const f32,
        rows: i64, hidden: i64, eps: f32, records: *mut c_void, stream: *mut c_void) -> c_int;
    pub fn izwi_qk_rms_norm_f16(q: *const u16, k: *const u16, qk_weight: *const u16, q_rows: i64, k_rows: i64,
        head_dim: i64, eps: f32, q_out: *mut u16, k_out: *mut u16, mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_rope_pair_bshd_f16(q: *const u16, k: *const u16, cos_sin: *const u16, batch: i64, seq: i64,
        q_heads: i64, k_heads: i64, head_dim: i64, q_out: *mut u16, k_out: *mut u16, mem_space: c_int,
        stream: *mut c_void) -> c_int;
    pub fn izwi_decode_gqa_attention_f16(q: *const u16, k: *const u16, v: *const u16, num_heads: i64,
        num_kv_heads: i64, head_dim: i64, kv_len: i64, kv_capacity: i64, scale: f32, out: *mut u16,
        mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_qk_norm_rope_append_f32(q: *const f32, k: *const f32, v: *const f32, qk_weight: *const f32,
        cos_sin: *const f32, num_heads: i64, num_kv_heads: i64, head_dim: i64, eps: f32, q_out: *mut f32,
        k_cache: *mut f32, v_cache: *mut f32, kv_capacity: i64, pos: i64, stream: *mut c_void) -> c_int;
    pub fn izwi_decode_attention_step_f32(q: *const f32, k: *const f32, v: *const f32, qk_weight: *const f32,
        cos_sin: *const f32, num_heads: i64, num_kv_heads: i64, head_dim: i64, eps: f32, k_cache: *mut f32,
        v_cache: *mut f32, kv_capacity: i64, pos: i64, scale: f32, out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn izwi_decode_gqa_attention_f32(q: *const f32, k: *const f32, v: *const f32, num_heads: i64,
        num_kv_heads: i64, head_dim: i64, kv_len: i64, kv_capacity: i64, scale: f32, out: *mut f32,
        mem_space: c_int, stream: *mut c_void) -> c_int;
    pub fn izwi_argmax_f32(logits: *const f32, rows: i64, n: i64, out: *mut u32, mem_space: c_int,
        stream: *mut c_void) -> c_int;
}
