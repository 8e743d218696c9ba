//! Raw Rust bindings of `libfusor_hip.so` (`fusor_hip.h`), one declaration per C entry point.
//!
//! This is the `-sys` half of the `Hip` arm a maintainer adds next to `Tensor::{Cpu,Gpu}`
//! (fusor-ml/fusor/src/lib.rs:91-94), `QMatrix::{Cpu*,Gpu}` (fusor-ml/fusor/src/quantized.rs:80-99) and
//! `Device::{Cpu,Gpu}` (fusor-ml/fusor/src/device.rs:7-13): drop the file into a crate as `src/lib.rs`, link with
//! `cargo:rustc-link-lib=dylib=fusor_hip` from `build.rs`, and build the safe wrappers on top.  It has no
//! dependencies.  It was written without a Rust toolchain at hand; a test of the repository checks that every
//! function of the header is declared here with the same number of parameters.
//!
//! Conventions of the C side: every call returns `FhStatus` (0 = ok, negative = error, message from
//! `fh_last_error()` on the calling thread); `*_dev` pointers are device memory from `fh_malloc`; calls on one
//! `FhDevice` must be serialised by the caller; nothing unwinds across the boundary.
#![allow(non_camel_case_types, clippy::too_many_arguments)]

use core::ffi::{c_char, c_void};

pub type FhStatus = i32;
pub const FH_OK: FhStatus = 0;
pub const FH_ERR_INVALID: FhStatus = -1;
pub const FH_ERR_HIP: FhStatus = -2;
/// `GgufReadError::UnsupportedDType`, and `None` from `QMatrix::concat_rows`
pub const FH_ERR_UNSUPPORTED: FhStatus = -3;
pub const FH_ERR_OOM: FhStatus = -4;
/// `Device::gpu()` found no gfx950 device
pub const FH_ERR_NO_DEVICE: FhStatus = -5;
/// `GgufReadError::Io`
pub const FH_ERR_IO: FhStatus = -6;
/// a metadata key or tensor name that the file does not hold
pub const FH_ERR_NOT_FOUND: FhStatus = -7;

/// `GgmlType` ids (fusor-ml/gguf/src/lib.rs:35-50) the library takes
pub const FH_GGML_F32: u32 = 0;
pub const FH_GGML_F16: u32 = 1;
pub const FH_Q4_0: u32 = 2;
pub const FH_Q5_0: u32 = 6;
pub const FH_Q8_0: u32 = 8;
pub const FH_Q4_K: u32 = 12;
pub const FH_Q5_K: u32 = 13;
pub const FH_Q6_K: u32 = 14;

/// `MaskKind` (fusor-ml/fusor/src/composite/flash_attention.rs:12-24)
pub const FH_MASK_NONE: i32 = 0;
pub const FH_MASK_CAUSAL: i32 = 1;
pub const FH_MASK_ADDITIVE: i32 = 2;
/// `MaskKind::BatchKeyMask`: additive [batch, kv_len] mask
pub const FH_MASK_BATCH_KEY: i32 = 3;

/// element types of attention operands and of the KV cache
pub const FH_F32: i32 = 0;
pub const FH_F16: i32 = 1;

/// `GgufMetadataValueType` ids (fusor-ml/gguf/src/lib.rs:349-379)
pub const FH_GGUF_U8: u32 = 0;
pub const FH_GGUF_I8: u32 = 1;
pub const FH_GGUF_U16: u32 = 2;
pub const FH_GGUF_I16: u32 = 3;
pub const FH_GGUF_U32: u32 = 4;
pub const FH_GGUF_I32: u32 = 5;
pub const FH_GGUF_F32: u32 = 6;
pub const FH_GGUF_BOOL: u32 = 7;
pub const FH_GGUF_STRING: u32 = 8;
pub const FH_GGUF_ARRAY: u32 = 9;
pub const FH_GGUF_U64: u32 = 10;
pub const FH_GGUF_I64: u32 = 11;
pub const FH_GGUF_F64: u32 = 12;
pub const FH_GGUF_MAX_RANK: usize = 8;

macro_rules! opaque {
    ($($name:ident),*) => { $(#[repr(C)] pub struct $name { _private: [u8; 0] })* };
}
opaque!(FhDevice, FhQMatrix, FhKvCache, FhLlama, FhGraph, FhGguf);

/// `fh_llama_config`
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct FhLlamaConfig {
    pub n_layers: i32,
    pub d_model: i32,
    pub n_heads: i32,
    pub n_kv_heads: i32,
    pub head_dim: i32,
    pub ffn: i32,
    pub vocab: i32,
    pub ctx: i32,
    pub eps: f32,
    pub theta: f32,
    pub kv_dtype: i32,
    pub fuse_qkv: i32,
    pub fuse_gate_up: i32,
    pub use_graph: i32,
}

/// `fh_finite_stats` (what `debug_check_nan_f32` logs, models/kalosm-llama/src/raw/mod.rs:9-58)
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct FhFiniteStats {
    pub nan: u64,
    pub pos_inf: u64,
    pub neg_inf: u64,
    pub max_abs: f32,
    pub first_nan_count: u32,
    pub first_nan: [u64; 4],
}

/// `fh_rope_scaling` (`RopeScalingConfig`, models/kalosm-llama/src/raw/mod.rs:163-169)
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct FhRopeScaling {
    pub factor: f32,
    pub high_freq_factor: f32,
    pub low_freq_factor: f32,
    pub original_max_position_embeddings: i32,
}

/// `fh_sampler_params` (`GpuStandardSamplerParams` / `GpuMirostat2SamplerParams`, fusor-ml/core/src/sampling/mod.rs:96-114)
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct FhSamplerParams {
    pub kind: u32,
    pub top_k: u32,
    pub temperature: f32,
    pub repetition_penalty: f32,
    pub top_p: f32,
    pub min_p: f32,
    pub tau: f32,
    pub eta: f32,
    pub random: f32,
}

/// `fh_gguf_tensor`: `name` is owned by the `FhGguf` handle
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct FhGgufTensor {
    pub name: *const c_char,
    pub ggml_type: u32,
    pub rank: i32,
    pub shape: [i64; FH_GGUF_MAX_RANK],
    pub offset: u64,
}

extern "C" {
    pub fn fh_last_error() -> *const c_char;
    pub fn fh_version() -> *const c_char;
    pub fn fh_device_count(count: *mut i32) -> FhStatus;
    pub fn fh_device_create(ordinal: i32, out: *mut *mut FhDevice) -> FhStatus;
    pub fn fh_device_destroy(dev: *mut FhDevice) -> FhStatus;
    pub fn fh_device_sync(dev: *mut FhDevice) -> FhStatus;
    pub fn fh_device_info(dev: *mut FhDevice, name: *mut c_char, name_cap: usize, compute_units: *mut i32, total_mem_bytes: *mut u64) -> FhStatus;
    pub fn fh_malloc(dev: *mut FhDevice, bytes: usize, out_dev: *mut *mut c_void) -> FhStatus;
    pub fn fh_free(dev: *mut FhDevice, ptr_dev: *mut c_void) -> FhStatus;
    pub fn fh_memset(dev: *mut FhDevice, ptr_dev: *mut c_void, byte: i32, bytes: usize) -> FhStatus;
    pub fn fh_upload(dev: *mut FhDevice, dst_dev: *mut c_void, src_host: *const c_void, bytes: usize) -> FhStatus;
    pub fn fh_download(dev: *mut FhDevice, dst_host: *mut c_void, src_dev: *const c_void, bytes: usize) -> FhStatus;
    pub fn fh_copy(dev: *mut FhDevice, dst_dev: *mut c_void, src_dev: *const c_void, bytes: usize) -> FhStatus;
    pub fn fh_timer_start(dev: *mut FhDevice) -> FhStatus;
    pub fn fh_timer_stop(dev: *mut FhDevice, elapsed_ms: *mut f32) -> FhStatus;
    pub fn fh_check_finite(dev: *mut FhDevice, x_dev: *const f32, count: i64, out_host: *mut FhFiniteStats) -> FhStatus;
    pub fn fh_graph_begin(dev: *mut FhDevice) -> FhStatus;
    pub fn fh_graph_end(dev: *mut FhDevice, out: *mut *mut FhGraph) -> FhStatus;
    pub fn fh_graph_launch(g: *mut FhGraph) -> FhStatus;
    pub fn fh_graph_free(g: *mut FhGraph) -> FhStatus;
    pub fn fh_qmatrix_from_gguf_bytes(dev: *mut FhDevice, ggml_type: u32, n: i64, k: i64, bytes: *const c_void, len: usize, out: *mut *mut FhQMatrix) -> FhStatus;
    pub fn fh_qmatrix_concat_rows(dev: *mut FhDevice, parts: *const *const FhQMatrix, count: i32, out: *mut *mut FhQMatrix) -> FhStatus;
    pub fn fh_qmatrix_free(q: *mut FhQMatrix) -> FhStatus;
    pub fn fh_qmatrix_info(q: *const FhQMatrix, ggml_type: *mut u32, n: *mut i64, k: *mut i64, device_bytes: *mut u64) -> FhStatus;
    pub fn fh_qmatrix_dequantize(q: *const FhQMatrix, out_dev: *mut f32) -> FhStatus;
    pub fn fh_embed_rows(q: *const FhQMatrix, ids_dev: *const u32, ids_host: *const u32, count: i32, out_dev: *mut f32) -> FhStatus;
    pub fn fh_qmatmul(q: *const FhQMatrix, x_dev: *const f32, m: i32, y_dev: *mut f32) -> FhStatus;
    pub fn fh_qmatmul_add2(q: *const FhQMatrix, x_dev: *const f32, m: i32, a_dev: *const f32, b_dev: *const f32, y_dev: *mut f32) -> FhStatus;
    pub fn fh_qmatmul_swiglu(q: *const FhQMatrix, x_dev: *const f32, m: i32, y_dev: *mut f32) -> FhStatus;
    pub fn fh_qmatmul_bf16(q: *const FhQMatrix, x_bf16_dev: *const u16, m: i32, y_dev: *mut f32) -> FhStatus;
    pub fn fh_qmatmul_q8(q: *const FhQMatrix, x_dev: *const f32, m: i32, y_dev: *mut f32, isums_dev: *mut i32) -> FhStatus;
    pub fn fh_q8_0_quantize(dev: *mut FhDevice, x_dev: *const f32, count: i64, out_dev: *mut c_void) -> FhStatus;
    pub fn fh_set_option(dev: *mut FhDevice, key: *const c_char, value: i64) -> FhStatus;
    pub fn fh_rms_norm(dev: *mut FhDevice, x_dev: *const f32, residual_dev: *const f32, w_dev: *const f32, bias_dev: *const f32, eps: f32, rows: i32, cols: i32, y_dev: *mut f32) -> FhStatus;
    pub fn fh_rope_tables(dev: *mut FhDevice, head_dim: i32, ctx: i32, theta: f32, cos_dev: *mut f32, sin_dev: *mut f32) -> FhStatus;
    pub fn fh_rope_tables_weighted(dev: *mut FhDevice, head_dim: i32, ctx: i32, theta: f32, freq_weight_host: *const f32, cos_dev: *mut f32, sin_dev: *mut f32) -> FhStatus;
    pub fn fh_rope_tables_scaled(dev: *mut FhDevice, head_dim: i32, ctx: i32, theta: f32, scaling: *const FhRopeScaling, freq_weight_host: *const f32, cos_dev: *mut f32, sin_dev: *mut f32) -> FhStatus;
    pub fn fh_rope_pair(dev: *mut FhDevice, q_dev: *const f32, q_sb: i64, q_sh: i64, q_st: i64, k_dev: *const f32, k_sb: i64, k_sh: i64, k_st: i64, b: i32, hq: i32, hk: i32, s: i32, d: i32, cos_dev: *const f32, sin_dev: *const f32, table_rows: i32, start_pos: i32, interleaved: i32, q_out_dev: *mut f32, k_out_dev: *mut f32) -> FhStatus;
    pub fn fh_kvcache_create(dev: *mut FhDevice, layers: i32, kv_heads: i32, head_dim: i32, max_len: i32, dtype: i32, out: *mut *mut FhKvCache) -> FhStatus;
    pub fn fh_kvcache_destroy(c: *mut FhKvCache) -> FhStatus;
    pub fn fh_kvcache_set_sliding(c: *mut FhKvCache, on: i32) -> FhStatus;
    pub fn fh_kvcache_reset(c: *mut FhKvCache) -> FhStatus;
    pub fn fh_kvcache_append(c: *mut FhKvCache, layer: i32, k_dev: *const f32, v_dev: *const f32, sh: i64, st: i64, s: i32) -> FhStatus;
    pub fn fh_kvcache_view(c: *const FhKvCache, layer: i32, len: *mut i32, capacity: *mut i32, k_dev: *mut *const c_void, v_dev: *mut *const c_void) -> FhStatus;
    pub fn fh_matmul(dev: *mut FhDevice, dtype: i32, a_dev: *const c_void, a_sb: i64, a_sr: i64, a_sc: i64, b_dev: *const c_void, b_sb: i64, b_sr: i64, b_sc: i64, batch: i32, m: i32, k: i32, n: i32, c_dev: *mut c_void) -> FhStatus;
    pub fn fh_flash_attention(dev: *mut FhDevice, dtype: i32, q_dev: *const c_void, q_sb: i64, q_sh: i64, q_st: i64, k_dev: *const c_void, v_dev: *const c_void, kv_sb: i64, kv_sh: i64, kv_st: i64, b: i32, hq: i32, hkv: i32, sq: i32, skv: i32, d: i32, scale: f32, mask_kind: i32, mask_dev: *const f32, out_dev: *mut c_void) -> FhStatus;
    pub fn fh_flash_attention_ex(dev: *mut FhDevice, q_dtype: i32, kv_dtype: i32, q_dev: *const c_void, q_sb: i64, q_sh: i64, q_st: i64, k_dev: *const c_void, v_dev: *const c_void, kv_sb: i64, kv_sh: i64, kv_st: i64, b: i32, hq: i32, hkv: i32, sq: i32, skv: i32, d: i32, scale: f32, mask_kind: i32, mask_dev: *const f32, out_dev: *mut c_void) -> FhStatus;
    pub fn fh_flash_attention_decode_static(dev: *mut FhDevice, q_dtype: i32, kv_dtype: i32, q_dev: *const c_void, k_dev: *const c_void, v_dev: *const c_void, kv_sh: i64, kv_st: i64, hq: i32, hkv: i32, d: i32, scale: f32, skv: i32, out_dev: *mut c_void) -> FhStatus;
    pub fn fh_swiglu(dev: *mut FhDevice, gate_dev: *const f32, up_dev: *const f32, y_dev: *mut f32, count: i64) -> FhStatus;
    pub fn fh_add3(dev: *mut FhDevice, a_dev: *const f32, b_dev: *const f32, c_dev: *const f32, y_dev: *mut f32, count: i64) -> FhStatus;
    pub fn fh_transpose_shd(dev: *mut FhDevice, x_dev: *const f32, s: i32, h: i32, d: i32, y_dev: *mut f32) -> FhStatus;
    pub fn fh_cast_f32_f16(dev: *mut FhDevice, x_dev: *const f32, y_f16_dev: *mut c_void, count: i64) -> FhStatus;
    pub fn fh_cast_f16_f32(dev: *mut FhDevice, x_f16_dev: *const c_void, y_dev: *mut f32, count: i64) -> FhStatus;
    pub fn fh_cast_f32_bf16(dev: *mut FhDevice, x_dev: *const f32, y_bf16_dev: *mut c_void, count: i64) -> FhStatus;
    pub fn fh_argmax(dev: *mut FhDevice, x_dev: *const f32, count: i64, id_dev: *mut u32) -> FhStatus;
    pub fn fh_top_k(dev: *mut FhDevice, x_dev: *const f32, count: i64, k: i32, ids_dev: *mut u32, values_dev: *mut f32, found_dev: *mut u32) -> FhStatus;
    pub fn fh_sample_token(dev: *mut FhDevice, logits_dev: *const f32, count: i64, params: *const FhSamplerParams, previous_host: *const u32, n_previous: u32, previous_tail_dev: *const u32, mu_dev: *mut f32, result_dev: *mut u32, ids_dev: *mut u32, values_dev: *mut f32) -> FhStatus;
    pub fn fh_gguf_open(path: *const c_char, out: *mut *mut FhGguf) -> FhStatus;
    pub fn fh_gguf_open_memory(bytes: *const c_void, len: usize, out: *mut *mut FhGguf) -> FhStatus;
    pub fn fh_gguf_close(g: *mut FhGguf) -> FhStatus;
    pub fn fh_gguf_info(g: *const FhGguf, version: *mut u32, tensor_count: *mut u64, metadata_count: *mut u64, alignment: *mut u64, tensor_data_offset: *mut u64) -> FhStatus;
    pub fn fh_gguf_meta_key(g: *const FhGguf, index: u64, key: *mut *const c_char, value_type: *mut u32) -> FhStatus;
    pub fn fh_gguf_meta_find(g: *const FhGguf, key: *const c_char, full_key: *mut *const c_char, value_type: *mut u32) -> FhStatus;
    pub fn fh_gguf_meta_int(g: *const FhGguf, key: *const c_char, out: *mut i64) -> FhStatus;
    pub fn fh_gguf_meta_float(g: *const FhGguf, key: *const c_char, out: *mut f64) -> FhStatus;
    pub fn fh_gguf_meta_bool(g: *const FhGguf, key: *const c_char, out: *mut i32) -> FhStatus;
    pub fn fh_gguf_meta_string(g: *const FhGguf, key: *const c_char, bytes: *mut *const c_char, len: *mut u64) -> FhStatus;
    pub fn fh_gguf_meta_array(g: *const FhGguf, key: *const c_char, elem_type: *mut u32, count: *mut u64, packed: *mut *const c_void) -> FhStatus;
    pub fn fh_gguf_meta_array_int(g: *const FhGguf, key: *const c_char, index: u64, out: *mut i64) -> FhStatus;
    pub fn fh_gguf_meta_array_float(g: *const FhGguf, key: *const c_char, index: u64, out: *mut f64) -> FhStatus;
    pub fn fh_gguf_meta_array_string(g: *const FhGguf, key: *const c_char, index: u64, bytes: *mut *const c_char, len: *mut u64) -> FhStatus;
    pub fn fh_gguf_tensor_info(g: *const FhGguf, index: u64, out: *mut FhGgufTensor) -> FhStatus;
    pub fn fh_gguf_tensor_find(g: *const FhGguf, name: *const c_char, index: *mut u64) -> FhStatus;
    pub fn fh_gguf_tensor_data(g: *const FhGguf, index: u64, bytes: *mut *const c_void, len: *mut usize) -> FhStatus;
    pub fn fh_qmatrix_from_gguf_tensor(dev: *mut FhDevice, g: *const FhGguf, name: *const c_char, out: *mut *mut FhQMatrix) -> FhStatus;
    pub fn fh_llama_create(dev: *mut FhDevice, cfg: *const FhLlamaConfig, out: *mut *mut FhLlama) -> FhStatus;
    pub fn fh_llama_destroy(m: *mut FhLlama) -> FhStatus;
    pub fn fh_llama_load_tensor(m: *mut FhLlama, name: *const c_char, ggml_type: u32, n: i64, k: i64, bytes: *const c_void, len: usize) -> FhStatus;
    pub fn fh_llama_set_rope_scaling(m: *mut FhLlama, scaling: *const FhRopeScaling) -> FhStatus;
    pub fn fh_llama_finalize(m: *mut FhLlama) -> FhStatus;
    pub fn fh_llama_reset(m: *mut FhLlama) -> FhStatus;
    pub fn fh_llama_forward(m: *mut FhLlama, tokens_host: *const u32, count: i32, logits_host: *mut f32, hidden_host: *mut f32) -> FhStatus;
    pub fn fh_llama_trace_text(m: *const FhLlama, buf: *mut c_char, capacity: usize, length: *mut usize) -> FhStatus;
    pub fn fh_llama_decode_greedy(m: *mut FhLlama, first_token: u32, steps: i32, out_tokens_host: *mut u32, elapsed_ms: *mut f32) -> FhStatus;
    pub fn fh_llama_decode_sampled(m: *mut FhLlama, first_token: u32, steps: i32, params: *const FhSamplerParams, randoms_host: *const f32, previous_host: *const u32, n_previous: u32, repetition_range: u32, mu: *mut f32, out_tokens_host: *mut u32, elapsed_ms: *mut f32) -> FhStatus;
    pub fn fh_llama_weight_bytes(m: *const FhLlama, bytes: *mut u64) -> FhStatus;
    pub fn fh_llama_config_from_gguf(g: *const FhGguf, cfg: *mut FhLlamaConfig) -> FhStatus;
    pub fn fh_llama_load_gguf(m: *mut FhLlama, g: *const FhGguf) -> FhStatus;
}

/// The message of the last failed call on this thread.
pub fn last_error() -> String {
    unsafe { core::ffi::CStr::from_ptr(fh_last_error()) }.to_string_lossy().into_owned()
}

/// `Ok(())` for `FH_OK`, otherwise the status with its message.
pub fn check(status: FhStatus) -> Result<(), (FhStatus, String)> {
    if status == FH_OK { Ok(()) } else { Err((status, last_error())) }
}
