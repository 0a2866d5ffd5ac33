//! Raw bindings to `librllama_hip.so`: rllama's per-token transformer forward path on one MI355X (gfx950).
//!
//! GENERATED from `include/rllama_hip.h` by `gen_bindings.py`; edit the header and run the generator, not this file.
//! The header's comments say what each call replaces in rllama (`OpenCL`, `OpenCLTensor`, `Transformer::forward`, ...).
#![allow(non_camel_case_types, non_snake_case)]

use std::os::raw::{c_char, c_double, c_float, c_int, c_void};

pub const RLH_ABI_VERSION: c_int = 1;

#[repr(C)]
pub struct rlh_ctx {
    _private: [u8; 0],
}
#[repr(C)]
pub struct rlh_model {
    _private: [u8; 0],
}
#[repr(C)]
pub struct rlh_caches {
    _private: [u8; 0],
}
#[repr(C)]
pub struct rlh_tensor {
    _private: [u8; 0],
}
#[repr(C)]
pub struct rlh_event {
    _private: [u8; 0],
}

// rlh_status
pub const RLH_OK: c_int = 0;
pub const RLH_ERR_INVALID: c_int = 1;
pub const RLH_ERR_NO_DEVICE: c_int = 2;
pub const RLH_ERR_HIP: c_int = 3;
pub const RLH_ERR_OOM: c_int = 4;
pub const RLH_ERR_STATE: c_int = 5;
pub const RLH_ERR_UNSUPPORTED: c_int = 6;

// rlh_dtype
pub const RLH_F16: c_int = 0;
pub const RLH_F32: c_int = 1;

// rlh_tensor_kind
pub const RLH_TOK_EMB: c_int = 0;
pub const RLH_WQ: c_int = 1;
pub const RLH_WK: c_int = 2;
pub const RLH_WV: c_int = 3;
pub const RLH_WO: c_int = 4;
pub const RLH_W1: c_int = 5;
pub const RLH_W2: c_int = 6;
pub const RLH_W3: c_int = 7;
pub const RLH_ATTN_NORM: c_int = 8;
pub const RLH_FFN_NORM: c_int = 9;
pub const RLH_NORM: c_int = 10;
pub const RLH_OUTPUT: c_int = 11;

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct rlh_model_params {
    pub dim: i32,
    pub n_layers: i32,
    pub n_heads: i32,
    pub ffn_hidden: i32,
    pub vocab_size: i32,
    pub max_seq_len: i32,
    pub norm_eps: c_double,
    pub force_f16: i32,
    pub percentage_to_gpu: c_float,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct rlh_sampler_params {
    pub temperature: c_float,
    pub top_p: c_float,
    pub top_k: i32,
    pub repetition_penalty: c_float,
}

#[link(name = "rllama_hip")]
extern "C" {
    pub fn rlh_init(device_ordinal: c_int, verbose: c_int, out: *mut *mut rlh_ctx) -> c_int;
    pub fn rlh_shutdown(ctx: *mut rlh_ctx);
    pub fn rlh_sync(ctx: *mut rlh_ctx) -> c_int;
    pub fn rlh_last_error() -> *const c_char;
    pub fn rlh_set_option(ctx: *mut rlh_ctx, name: *const c_char, value: *const c_char) -> c_int;
    pub fn rlh_device_info(ctx: *mut rlh_ctx, name: *mut c_char, cap: c_int, compute_units: *mut c_int, hbm_bytes: *mut u64) -> c_int;
    pub fn rlh_model_create(ctx: *mut rlh_ctx, params: *const rlh_model_params, out: *mut *mut rlh_model) -> c_int;
    pub fn rlh_model_free(model: *mut rlh_model);
    pub fn rlh_model_set_tensor(model: *mut rlh_model, kind: c_int, layer: c_int, host: *const c_void, rows: c_int, cols: c_int, src_dtype: c_int) -> c_int;
    pub fn rlh_model_get_tensor(model: *mut rlh_model, kind: c_int, layer: c_int, host_out: *mut c_void, rows: c_int, cols: c_int, dst_dtype: c_int) -> c_int;
    pub fn rlh_model_fill_synthetic(model: *mut rlh_model, seed: u64, std: c_double) -> c_int;
    pub fn rlh_model_set_prefill_mode(model: *mut rlh_model, mode: c_int) -> c_int;
    pub fn rlh_model_layers_on_gpu(model: *const rlh_model, last_layer_on_gpu: *mut c_int) -> c_int;
    pub fn rlh_model_decode_bytes(model: *const rlh_model, T: c_int, bytes: *mut u64) -> c_int;
    pub fn rlh_caches_create(model: *mut rlh_model, out: *mut *mut rlh_caches) -> c_int;
    pub fn rlh_caches_true_clone(src: *const rlh_caches, out: *mut *mut rlh_caches) -> c_int;
    pub fn rlh_caches_shift_left(caches: *mut rlh_caches, shifts: c_int) -> c_int;
    pub fn rlh_caches_free(caches: *mut rlh_caches);
    pub fn rlh_caches_read(caches: *const rlh_caches, layer: c_int, head: c_int, which: c_int, host_out: *mut c_float) -> c_int;
    pub fn rlh_forward(model: *mut rlh_model, caches: *mut rlh_caches, tokens: *const i32, n: c_int, start_pos: c_int, logits_out: *mut c_float) -> c_int;
    pub fn rlh_forward_layers(model: *mut rlh_model, caches: *mut rlh_caches, x_in: *const c_float, n: c_int, start_pos: c_int, first_layer: c_int, last_layer: c_int, x_out: *mut c_float) -> c_int;
    pub fn rlh_forward_greedy(model: *mut rlh_model, caches: *mut rlh_caches, tokens: *const i32, n: c_int, start_pos: c_int, next_token: *mut i32) -> c_int;
    pub fn rlh_generate_greedy(model: *mut rlh_model, caches: *mut rlh_caches, prompt: *const i32, n_prompt: c_int, n_new: c_int, out_tokens: *mut i32, ms_first: *mut c_float, ms_per_token: *mut c_float) -> c_int;
    pub fn rlh_decode_greedy(model: *mut rlh_model, caches: *mut rlh_caches, n_steps: c_int, out_tokens: *mut i32, ms_total: *mut c_float) -> c_int;
    pub fn rlh_sampler_default(p: *mut rlh_sampler_params);
    pub fn rlh_sample_candidates(logits: *const c_float, vocab: c_int, p: *const rlh_sampler_params, existing_tokens: *const i32, n_existing: c_int, out_ids: *mut i32, out_probs: *mut c_float, cap: c_int, n_out: *mut c_int, total_p: *mut c_float) -> c_int;
    pub fn rlh_sample(logits: *const c_float, vocab: c_int, p: *const rlh_sampler_params, existing_tokens: *const i32, n_existing: c_int, u: c_float, token: *mut i32, prob: *mut c_float) -> c_int;
    pub fn rlh_forward_sample(model: *mut rlh_model, caches: *mut rlh_caches, tokens: *const i32, n: c_int, start_pos: c_int, p: *const rlh_sampler_params, existing_tokens: *const i32, n_existing: c_int, u: c_float, token: *mut i32, prob: *mut c_float) -> c_int;
    pub fn rlh_tensor_upload(ctx: *mut rlh_ctx, host: *const c_void, rows: c_int, cols: c_int, cols_capacity: c_int, dtype: c_int, out: *mut *mut rlh_tensor) -> c_int;
    pub fn rlh_tensor_alloc(ctx: *mut rlh_ctx, rows: c_int, cols: c_int, dtype: c_int, out: *mut *mut rlh_tensor) -> c_int;
    pub fn rlh_tensor_download(t: *mut rlh_tensor, host: *mut c_void, cols_capacity: c_int, ev: *mut *mut rlh_event) -> c_int;
    pub fn rlh_tensor_free(t: *mut rlh_tensor);
    pub fn rlh_tensor_shape(t: *const rlh_tensor, rows: *mut c_int, cols: *mut c_int, dtype: *mut c_int) -> c_int;
    pub fn rlh_event_wait(ev: *mut rlh_event) -> c_int;
    pub fn rlh_event_record(ctx: *mut rlh_ctx, out: *mut *mut rlh_event) -> c_int;
    pub fn rlh_event_elapsed_ms(start: *mut rlh_event, stop: *mut rlh_event, ms: *mut c_float) -> c_int;
    pub fn rlh_event_free(ev: *mut rlh_event);
    pub fn rlh_copy_inplace(dst: *mut rlh_tensor, src: *const rlh_tensor) -> c_int;
    pub fn rlh_transpose_from(dst: *mut rlh_tensor, src: *const rlh_tensor) -> c_int;
    pub fn rlh_hadamard_product_inplace(dst: *mut rlh_tensor, src: *const rlh_tensor) -> c_int;
    pub fn rlh_silu_inplace(t: *mut rlh_tensor) -> c_int;
    pub fn rlh_matrix_mul_inplace_transposed(dst: *mut rlh_tensor, src: *const rlh_tensor, other: *const rlh_tensor) -> c_int;
    pub fn rlh_gemv(y: *mut rlh_tensor, w: *const rlh_tensor, x: *const rlh_tensor, round_x: c_int, round_y: c_int) -> c_int;
    pub fn rlh_rmsnorm(y: *mut rlh_tensor, x: *const rlh_tensor, w: *const rlh_tensor, eps: c_double, round_y: c_int) -> c_int;
    pub fn rlh_rope_inplace(x: *mut rlh_tensor, n_heads: c_int, head_dim: c_int, pos: c_int) -> c_int;
    pub fn rlh_add(dst: *mut rlh_tensor, a: *const rlh_tensor, b: *const rlh_tensor) -> c_int;
    pub fn rlh_silu_mul(dst: *mut rlh_tensor, gate: *const rlh_tensor, up: *const rlh_tensor) -> c_int;
    pub fn rlh_ffn_gate(dst: *mut rlh_tensor, x: *const rlh_tensor, w1: *const rlh_tensor, w3: *const rlh_tensor) -> c_int;
    pub fn rlh_rope_kvwrite(q: *mut rlh_tensor, k: *const rlh_tensor, v: *const rlh_tensor, cache_k: *mut rlh_tensor, cache_v: *mut rlh_tensor, n_heads: c_int, max_seq_len: c_int, pos: c_int) -> c_int;
    pub fn rlh_attn_decode(out: *mut rlh_tensor, q: *const rlh_tensor, cache_k: *const rlh_tensor, cache_v: *const rlh_tensor, n_heads: c_int, max_seq_len: c_int, T: c_int, n_splits: c_int, round_out: c_int) -> c_int;
    pub fn rlh_attn_decode_noalloc(out: *mut rlh_tensor, q: *const rlh_tensor, cache_k: *const rlh_tensor, cache_v: *const rlh_tensor, n_heads: c_int, max_seq_len: c_int, T: c_int, n_splits: c_int, round_out: c_int) -> c_int;
    pub fn rlh_attn_prefill(out: *mut rlh_tensor, qkv: *const rlh_tensor, cache_k: *mut rlh_tensor, cache_v: *mut rlh_tensor, n_heads: c_int, max_seq_len: c_int) -> c_int;
    pub fn rlh_argmax_greedy(logits: *const rlh_tensor, temperature: c_float, token: *mut i32) -> c_int;
    pub fn rlh_model_time_kernel(model: *mut rlh_model, caches: *mut rlh_caches, which: c_int, T: c_int, iters: c_int, us_per_launch: *mut c_float, bytes_per_launch: *mut u64) -> c_int;
    pub fn rlh_time_gemv(ctx: *mut rlh_ctx, rows: c_int, k: c_int, w_dtype: c_int, round_x: c_int, round_y: c_int, n_buffers: c_int, iters: c_int, us_per_launch: *mut c_float) -> c_int;
    pub fn rlh_probe_gemv_phases(ctx: *mut rlh_ctx, rows: c_int, k: c_int, n_buffers: c_int, launches: c_int, out_us: *mut c_float) -> c_int;
    pub fn rlh_synth_normal_f16(seed: u64, kind: c_int, layer: c_int, first_index: u64, count: u64, std: c_double, out: *mut u16);
    pub fn rlh_synth_tokens(seed: u64, first_index: u64, count: u64, lo: i32, hi: i32, out: *mut i32);
    pub fn rlh_abi_version() -> c_int;
}
