// Generated from include/lumen_hip.h by rust/gen_ffi.py -- do not edit.
// Rust binding of liblumen_hip.so: src/ffi.rs + `mod ffi;` in the reference crate; link the library from build.rs.
#![allow(non_camel_case_types, dead_code)]
use std::os::raw::{c_char, c_float, c_int, c_void};

#[repr(C)] pub struct lumen_ctx { _private: [u8; 0] }
#[repr(C)] pub struct lumen_rope { _private: [u8; 0] }
#[repr(C)] pub struct lumen_kv_cache { _private: [u8; 0] }
#[repr(C)] pub struct lumen_llama { _private: [u8; 0] }

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct lumen_llama_config {
    pub vocab_size: c_int,
    pub hidden_size: c_int,
    pub intermediate_size: c_int,
    pub num_hidden_layers: c_int,
    pub num_attention_heads: c_int,
    pub num_key_value_heads: c_int,
    pub rms_norm_eps: c_float,
    pub max_seq_len: c_int,
    pub rope_theta: c_float,
    pub head_dim: c_int,
    pub qk_norm: c_int,
    pub tie_embeddings: c_int,
    pub weight_dtype: c_int,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct lumen_sampling {
    pub temperature: c_float,
    pub top_p: c_float,
    pub repetition_penalty: c_float,
    pub recent_window: c_int,
    pub max_gen: c_int,
    pub seed: u64,
}

pub const LUMEN_OK: c_int = 0;
pub const LUMEN_ERR_SHAPE: c_int = 1;
pub const LUMEN_ERR_KV_OVERFLOW: c_int = 2;
pub const LUMEN_ERR_ROPE_RANGE: c_int = 3;
pub const LUMEN_ERR_EMBED_OOB: c_int = 4;
pub const LUMEN_ERR_CACHE_COUNT: c_int = 5;
pub const LUMEN_ERR_INVALID: c_int = 6;
pub const LUMEN_ERR_HIP: c_int = 7;
pub const LUMEN_ERR_NO_DEVICE: c_int = 8;
pub const LUMEN_ERR_UNSUPPORTED: c_int = 9;
pub const LUMEN_DTYPE_F32: c_int = 0;
pub const LUMEN_DTYPE_BF16: c_int = 1;
pub const LUMEN_GEMV_EPI_STORE: c_int = 0;
pub const LUMEN_GEMV_EPI_RESIDUAL: c_int = 1;
pub const LUMEN_GEMV_EPI_SWIGLU: c_int = 2;
pub const LUMEN_GEMV_EPI_ARGMAX: c_int = 3;
pub const LUMEN_GEMV_EPI_ROPE_QKV: c_int = 4;
pub const LUMEN_DECODE_EAGER: c_int = 0;
pub const LUMEN_DECODE_GRAPH: c_int = 1;
pub const LUMEN_DECODE_PERSISTENT: c_int = 2;

extern "C" {
    pub fn lumen_last_error() -> *const c_char;
    pub fn lumen_version() -> *const c_char;
    pub fn lumen_ctx_create(device: c_int, out: *mut *mut lumen_ctx) -> c_int;
    pub fn lumen_ctx_destroy(ctx: *mut lumen_ctx) -> c_int;
    pub fn lumen_ctx_set_stream(ctx: *mut lumen_ctx, hip_stream: *mut c_void) -> c_int;
    pub fn lumen_ctx_synchronize(ctx: *mut lumen_ctx) -> c_int;
    pub fn lumen_ctx_num_cus(ctx: *const lumen_ctx, num_cus_out: *mut c_int) -> c_int;
    pub fn lumen_timer_start(ctx: *mut lumen_ctx) -> c_int;
    pub fn lumen_timer_stop(ctx: *mut lumen_ctx, ms_out: *mut c_float) -> c_int;
    pub fn lumen_malloc(ctx: *mut lumen_ctx, bytes: usize, dev_out: *mut *mut c_void) -> c_int;
    pub fn lumen_free(ctx: *mut lumen_ctx, dev: *mut c_void) -> c_int;
    pub fn lumen_upload(ctx: *mut lumen_ctx, dst_dev: *mut c_void, src_host: *const c_void, bytes: usize) -> c_int;
    pub fn lumen_download(ctx: *mut lumen_ctx, dst_host: *mut c_void, src_dev: *const c_void, bytes: usize) -> c_int;
    pub fn lumen_copy_d2d(ctx: *mut lumen_ctx, dst_dev: *mut c_void, src_dev: *const c_void, bytes: usize) -> c_int;
    pub fn lumen_matmul_f32(ctx: *mut lumen_ctx, A_dev: *const c_float, W_dev: *const c_float, C_dev: *mut c_float, M: c_int, N: c_int, K_a: c_int, K_w: c_int) -> c_int;
    pub fn lumen_gemv_f32(ctx: *mut lumen_ctx, W_dev: *const c_float, x_dev: *const c_float, y_dev: *mut c_float, N: c_int, K: c_int) -> c_int;
    pub fn lumen_gemm_f32(ctx: *mut lumen_ctx, A_dev: *const c_float, W_dev: *const c_float, C_dev: *mut c_float, M: c_int, N: c_int, K: c_int) -> c_int;
    pub fn lumen_gemv_fused_f32(ctx: *mut lumen_ctx, W_dev: *const c_void, w_bf16: c_int, x_dev: *const c_float, y_dev: *mut c_float, N: c_int, K: c_int, norm_w_dev: *const c_float, eps: c_float, epilogue: c_int, residual_dev: *const c_float) -> c_int;
    pub fn lumen_interleave_rows(ctx: *mut lumen_ctx, a_dev: *const c_void, b_dev: *const c_void, out_dev: *mut c_void, rows: c_int, row_bytes: usize) -> c_int;
    pub fn lumen_gemv_kernel_name(num_cus: c_int, N: c_int, K: c_int, w_bf16: c_int, rmsnorm: c_int, epilogue: c_int, buf: *mut c_char, buf_len: c_int) -> c_int;
    pub fn lumen_gemv_bf16w(ctx: *mut lumen_ctx, W_dev: *const u16, x_dev: *const c_float, y_dev: *mut c_float, N: c_int, K: c_int) -> c_int;
    pub fn lumen_gemm_bf16w(ctx: *mut lumen_ctx, A_dev: *const c_float, W_dev: *const u16, C_dev: *mut c_float, M: c_int, N: c_int, K: c_int) -> c_int;
    pub fn lumen_gemv_bench(ctx: *mut lumen_ctx, W_base_dev: *const c_void, stride_elems: usize, ncopies: c_int, w_bf16: c_int, x_dev: *const c_float, y_dev: *mut c_float, N: c_int, K: c_int, iters: c_int, ms_out: *mut c_float) -> c_int;
    pub fn lumen_rmsnorm_f32(ctx: *mut lumen_ctx, x_dev: *const c_float, w_dev: *const c_float, out_dev: *mut c_float, rows: c_int, dim: c_int, eps: c_float) -> c_int;
    pub fn lumen_silu_f32(ctx: *mut lumen_ctx, x_dev: *const c_float, out_dev: *mut c_float, n: usize) -> c_int;
    pub fn lumen_copy_f32(ctx: *mut lumen_ctx, x_dev: *const c_float, out_dev: *mut c_float, n: usize) -> c_int;
    pub fn lumen_add_f32(ctx: *mut lumen_ctx, a_dev: *const c_float, b_dev: *const c_float, out_dev: *mut c_float, n: usize) -> c_int;
    pub fn lumen_mul_f32(ctx: *mut lumen_ctx, a_dev: *const c_float, b_dev: *const c_float, out_dev: *mut c_float, n: usize) -> c_int;
    pub fn lumen_swiglu_f32(ctx: *mut lumen_ctx, gate_dev: *const c_float, up_dev: *const c_float, out_dev: *mut c_float, n: usize) -> c_int;
    pub fn lumen_embedding_f32(ctx: *mut lumen_ctx, W_dev: *const c_float, ids_host: *const c_float, n_ids: c_int, vocab: c_int, dim: c_int, out_dev: *mut c_float) -> c_int;
    pub fn lumen_argmax_f32(ctx: *mut lumen_ctx, x_dev: *const c_float, n: c_int, index_host_out: *mut c_int) -> c_int;
    pub fn lumen_rope_create(ctx: *mut lumen_ctx, dim: c_int, max_seq: c_int, theta: c_float, out: *mut *mut lumen_rope) -> c_int;
    pub fn lumen_rope_destroy(rope: *mut lumen_rope) -> c_int;
    pub fn lumen_rope_tables_download(rope: *mut lumen_rope, cos_host: *mut c_float, sin_host: *mut c_float) -> c_int;
    pub fn lumen_rope_forward_f32(rope: *mut lumen_rope, x_dev: *const c_float, out_dev: *mut c_float, b: c_int, h: c_int, s: c_int, d: c_int, offset: c_int) -> c_int;
    pub fn lumen_rope_1token_copy_f32(rope: *mut lumen_rope, src_dev: *const c_float, dst_dev: *mut c_float, d: c_int, pos: c_int) -> c_int;
    pub fn lumen_kv_cache_create(ctx: *mut lumen_ctx, b: c_int, h_kv: c_int, max_seq: c_int, d: c_int, out: *mut *mut lumen_kv_cache) -> c_int;
    pub fn lumen_kv_cache_destroy(cache: *mut lumen_kv_cache) -> c_int;
    pub fn lumen_kv_cache_reset(cache: *mut lumen_kv_cache) -> c_int;
    pub fn lumen_kv_cache_len(cache: *const lumen_kv_cache, len_out: *mut c_int) -> c_int;
    pub fn lumen_kv_cache_set_len(cache: *mut lumen_kv_cache, len: c_int) -> c_int;
    pub fn lumen_kv_cache_ptrs(cache: *const lumen_kv_cache, k_dev_out: *mut *mut c_float, v_dev_out: *mut *mut c_float) -> c_int;
    pub fn lumen_kv_cache_update(cache: *mut lumen_kv_cache, k_dev: *const c_float, v_dev: *const c_float, s: c_int, start_pos: c_int) -> c_int;
    pub fn lumen_kv_cache_get_view(cache: *const lumen_kv_cache, current_len: c_int, k_out_dev: *mut c_float, v_out_dev: *mut c_float) -> c_int;
    pub fn lumen_attn_decode_f32(cache: *mut lumen_kv_cache, rope: *mut lumen_rope, q3_dev: *const c_float, k3_dev: *const c_float, v3_dev: *const c_float, out_dev: *mut c_float, h: c_int, scale: c_float, causal: c_int) -> c_int;
    pub fn lumen_qkv_rope_append_f32(cache: *mut lumen_kv_cache, rope: *mut lumen_rope, Wqkv_dev: *const c_void, w_bf16: c_int, x_dev: *const c_float, K: c_int, norm_w_dev: *const c_float, eps: c_float, q_rot_out_dev: *mut c_float, n_head: c_int) -> c_int;
    pub fn lumen_attn_decode_prerotated_f32(cache: *mut lumen_kv_cache, q_rot_dev: *const c_float, out_dev: *mut c_float, n_head: c_int, scale: c_float) -> c_int;
    pub fn lumen_attn_decode_static_f32(cache: *mut lumen_kv_cache, rope: *mut lumen_rope, q3_dev: *const c_float, k3_dev: *const c_float, v3_dev: *const c_float, out_dev: *mut c_float, h: c_int, scale: c_float, causal: c_int) -> c_int;
    pub fn lumen_attn_prefill_f32(cache: *mut lumen_kv_cache, rope: *mut lumen_rope, q_dev: *const c_float, k_dev: *const c_float, v_dev: *const c_float, out_dev: *mut c_float, s: c_int, h: c_int, scale: c_float, causal: c_int) -> c_int;
    pub fn lumen_llama_create(ctx: *mut lumen_ctx, cfg: *const lumen_llama_config, out: *mut *mut lumen_llama) -> c_int;
    pub fn lumen_llama_destroy(model: *mut lumen_llama) -> c_int;
    pub fn lumen_llama_set_param(model: *mut lumen_llama, name: *const c_char, data_host: *const c_void, dtype: c_int, shape: *const i64, ndim: c_int) -> c_int;
    pub fn lumen_llama_load_safetensors(model: *mut lumen_llama, path: *const c_char, n_loaded_out: *mut c_int, n_missing_out: *mut c_int) -> c_int;
    pub fn lumen_safetensors_find(path: *const c_char, name: *const c_char, dtype_out: *mut c_int, shape_out: *mut i64, ndim_inout: *mut c_int, begin_out: *mut u64, end_out: *mut u64) -> c_int;
    pub fn lumen_llama_forward(model: *mut lumen_llama, ids_host: *const c_float, s: c_int, logits_host: *mut c_float, all_rows: c_int) -> c_int;
    pub fn lumen_llama_decode_greedy(model: *mut lumen_llama, first_id: c_int, n: c_int, ids_out_host: *mut i32, logits_out_host: *mut c_float) -> c_int;
    pub fn lumen_sample_top_p_f32(logits_host: *const c_float, n: c_int, temperature: c_float, top_p: c_float, repetition_penalty: c_float, recent_tokens: *const i32, n_recent: c_int, r: c_float, index_out: *mut i32) -> c_int;
    pub fn lumen_rand01(state: *mut u64) -> c_float;
    pub fn lumen_llama_generate_turn(model: *mut lumen_llama, new_tokens: *const i32, n_new: c_int, history: *const i32, n_history: c_int, sampling: *const lumen_sampling, stop_ids: *const i32, n_stop: c_int, out_ids: *mut i32, out_cap: c_int, n_out: *mut c_int) -> c_int;
    pub fn lumen_llama_get_config(model: *const lumen_llama, cfg_out: *mut lumen_llama_config) -> c_int;
    pub fn lumen_llama_decode_profile(model: *mut lumen_llama, first_id: c_int, n: c_int, ms_sum_out: *mut f64, count_out: *mut c_int, n_classes: c_int) -> c_int;
    pub fn lumen_llama_set_decode_mode(model: *mut lumen_llama, mode: c_int) -> c_int;
    pub fn lumen_llama_profile_kernel_name(model: *const lumen_llama, kernel_class: c_int, buf: *mut c_char, buf_len: c_int) -> c_int;
    pub fn lumen_llama_set_handover(model: *mut lumen_llama, enable: c_int, spin_limit: i64, pre_sleep: c_int, poll_delay: c_int, poll_gap: c_int) -> c_int;
    pub fn lumen_llama_get_decode_mode(model: *const lumen_llama, mode_out: *mut c_int) -> c_int;
    pub fn lumen_llama_reset(model: *mut lumen_llama) -> c_int;
    pub fn lumen_llama_kv_len(model: *const lumen_llama, len_out: *mut c_int) -> c_int;
    pub fn lumen_llama_set_kv_len(model: *mut lumen_llama, len: c_int) -> c_int;
    pub fn lumen_llama_cache_download(model: *mut lumen_llama, layer: c_int, k_host: *mut c_float, v_host: *mut c_float) -> c_int;
    pub fn lumen_llama_cache_upload(model: *mut lumen_llama, layer: c_int, k_host: *const c_float, v_host: *const c_float) -> c_int;
    pub fn lumen_llama_decode_bytes(model: *const lumen_llama, len: c_int, bytes_out: *mut f64) -> c_int;
    pub fn lumen_decoder_layer_create(ctx: *mut lumen_ctx, cfg: *const lumen_llama_config, out: *mut *mut lumen_decoder_layer) -> c_int;
    pub fn lumen_decoder_layer_destroy(layer: *mut lumen_decoder_layer) -> c_int;
    pub fn lumen_decoder_layer_decode_f32(layer: *mut lumen_decoder_layer, cache: *mut lumen_kv_cache, wqkv_dev: *const c_void, wo_dev: *const c_void, wgu_dev: *const c_void, wdown_dev: *const c_void, input_norm_dev: *const c_float, post_norm_dev: *const c_float, q_norm_dev: *const c_float, k_norm_dev: *const c_float, x_dev: *const c_float, y_dev: *mut c_float) -> c_int;
}

/// status -> panic with the library's message: the reference's own error behaviour (Cargo.toml: panic = "abort")
pub fn check(rc: c_int) {
    if rc != 0 {
        let msg = unsafe { std::ffi::CStr::from_ptr(lumen_last_error()) }.to_string_lossy().into_owned();
        panic!("{msg}");
    }
}
