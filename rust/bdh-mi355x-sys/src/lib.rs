//! Raw bindings to `libbdh_mi355x.so`, the MI355X (gfx950) implementation of the BDH cached-inference hot path.
//!
//! One declaration per entry point of `include/bdh_mi355x.h`, in the header's order; the header documents each
//! argument and names the reference function an entry point replaces.  All data pointers are caller-owned DEVICE
//! memory unless the parameter name ends in `_host`; calls are asynchronous on the context's HIP stream; every
//! function returns 0 or a negative `bdh_status` and never unwinds.
//!
//! This crate is source only here: the environment this repository is built and tested in has no Rust toolchain.
//! `tests/test_rust_binding.py` checks every name and argument count below against the C header.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};

#[cfg(feature = "burn-wrappers")]
pub mod wrappers;

/// opaque: device, stream, workspace
#[repr(C)]
pub struct bdh_ctx {
    _private: [u8; 0],
}
/// opaque: weights view + per-model tables
#[repr(C)]
pub struct bdh_model {
    _private: [u8; 0],
}

/// opaque: pending rank-1 updates of one state tensor (the deferred decode step)
#[repr(C)]
pub struct bdh_state_log {
    _private: [u8; 0],
}

/// opaque: one bdh_state_log per layer of a model (the deferred decode step of a whole model)
#[repr(C)]
pub struct bdh_model_logs {
    _private: [u8; 0],
}

pub const BDH_OK: c_int = 0;
pub const BDH_E_INVAL: c_int = -1;
pub const BDH_E_SHAPE: c_int = -2;
pub const BDH_E_ALIGN: c_int = -3;
pub const BDH_E_HIP: c_int = -4;
pub const BDH_E_NOMEM: c_int = -5;
pub const BDH_E_UNSUPPORTED: c_int = -6;

/// src/positional.rs:8-15
pub const BDH_ROPE: c_int = 0;
pub const BDH_ALIBI: c_int = 1;
pub const BDH_POPE: c_int = 2;

/// storage type of the recurrent state
pub const BDH_F32: c_int = 0;
pub const BDH_BF16: c_int = 1;

/// flags of bdh_prefill_chunked
pub const BDH_PREFILL_STATE_IS_ZERO: c_int = 1;
pub const BDH_PREFILL_STATE_HILO: c_int = 2;
pub const BDH_PREFILL_ALL_SCORES: c_int = 4;
pub const BDH_PREFILL_ROW_NORMALIZE: c_int = 8;

/// src/model/config.rs:113-164 (BDHConfig) + :10-31 (FusedKernelConfig), as plain scalars
#[repr(C)]
pub struct bdh_model_config {
    pub n_layer: i32,
    pub n_embd: i32,
    pub n_head: i32,
    pub latent: i32,
    pub vocab: i32,
    pub rotary: i32,
    pub rope_theta: f32,
    pub relu_threshold: f32,
    pub alibi_slopes_host: *const f32,
}

/// device pointers, in the record order of the reference module (src/model/bdh.rs:27-33)
#[repr(C)]
pub struct bdh_model_weights {
    pub embed: *const f32,
    pub encoder: *const f32,
    pub encoder_v: *const f32,
    pub decoder: *const f32,
    pub lm_head: *const f32,
}

extern "C" {
    pub fn bdh_version() -> *const c_char;
    pub fn bdh_status_string(status: c_int) -> *const c_char;
    pub fn bdh_ctx_create(device_id: c_int, hip_stream: *mut c_void, out: *mut *mut bdh_ctx) -> c_int;
    pub fn bdh_ctx_destroy(ctx: *mut bdh_ctx) -> c_int;
    pub fn bdh_ctx_set_stream(ctx: *mut bdh_ctx, hip_stream: *mut c_void) -> c_int;
    pub fn bdh_ctx_synchronize(ctx: *mut bdh_ctx) -> c_int;
    pub fn bdh_last_error(ctx: *const bdh_ctx) -> *const c_char;
    pub fn bdh_ctx_set_option(ctx: *mut bdh_ctx, name: *const c_char, value: c_int) -> c_int;
    pub fn bdh_build_freqs(latent: c_int, theta: f32, rotary: c_int, freqs_host: *mut f32) -> c_int;
    pub fn bdh_default_alibi_slopes(n_head: c_int, slopes_host: *mut f32) -> c_int;
    pub fn bdh_rotate(ctx: *mut bdh_ctx, b: c_int, h: c_int, t: c_int, n: c_int, rotary: c_int,
        x: *const f32, freqs: *const f32, position: i64, positions_dev: *const i32, q: *mut f32) -> c_int;
    pub fn bdh_recurrent_attention(ctx: *mut bdh_ctx, b: c_int, h: c_int, t: c_int, n: c_int, d: c_int,
        rotary: c_int, x: *const f32, v: *const f32, freqs: *const f32, position: i64,
        positions_dev: *const i32, alibi_slopes_host: *const f32, rho: *mut c_void, rho_dtype: c_int,
        out: *mut f32, active_bitmask: *mut u64, rows_touched: *mut i32) -> c_int;
    pub fn bdh_state_step(ctx: *mut bdh_ctx, b: c_int, h: c_int, n: c_int, d: c_int, rotary: c_int,
        x: *const f32, v: *const f32, freqs: *const f32, position: i64, positions_dev: *const i32,
        alibi_slopes_host: *const f32, rho: *mut c_void, rho_dtype: c_int, out: *mut f32,
        active_bitmask: *mut u64, rows_touched: *mut i32) -> c_int;
    pub fn bdh_state_step_noalloc(ctx: *mut bdh_ctx, b: c_int, h: c_int, n: c_int, d: c_int, rotary: c_int,
        x: *const f32, v: *const f32, freqs: *const f32, position: i64, positions_dev: *const i32,
        alibi_slopes_host: *const f32, rho: *mut c_void, rho_dtype: c_int, out: *mut f32,
        active_bitmask: *mut u64, rows_touched: *mut i32) -> c_int;
    pub fn bdh_state_log_create(ctx: *mut bdh_ctx, b: c_int, h: c_int, n: c_int, d: c_int, rho_dtype: c_int,
        capacity: c_int, out: *mut *mut bdh_state_log) -> c_int;
    pub fn bdh_state_log_destroy(ctx: *mut bdh_ctx, log: *mut bdh_state_log) -> c_int;
    pub fn bdh_state_log_pending(log: *const bdh_state_log) -> c_int;
    pub fn bdh_state_log_bytes(log: *const bdh_state_log) -> usize;
    pub fn bdh_state_step_deferred(ctx: *mut bdh_ctx, log: *mut bdh_state_log, x: *const f32, v: *const f32,
        freqs: *const f32, position: i64, positions_dev: *const i32, rho: *mut c_void, out: *mut f32,
        active_bitmask: *mut u64, rows_touched: *mut i32) -> c_int;
    pub fn bdh_state_flush(ctx: *mut bdh_ctx, log: *mut bdh_state_log, rho: *mut c_void) -> c_int;
    pub fn bdh_relu_lowrank(ctx: *mut bdh_ctx, b: c_int, h_in: c_int, t: c_int, d: c_int, h: c_int, n: c_int,
        input: *const f32, weight: *const f32, bias: *const f32, threshold: f32, block_size: c_int,
        active_blocks_host: *const u8, n_blocks: c_int, gate: *const f32, out: *mut f32) -> c_int;
    pub fn bdh_layer_norm(ctx: *mut bdh_ctx, rows: i64, d: c_int, input: *const f32,
        out: *mut f32) -> c_int;
    pub fn bdh_fused_state_aligned(ctx: *mut bdh_ctx, b: c_int, h: c_int, t: c_int, n: c_int, dv: c_int,
        query: *const f32, value: *const f32, freqs: *const f32, alibi_slopes_host: *const f32,
        block_size: c_int, block_pairs_host: *const i32, n_pairs: c_int, rotary: c_int, row_normalize: c_int,
        out: *mut f32) -> c_int;
    pub fn bdh_prefill_chunked(ctx: *mut bdh_ctx, b: c_int, h: c_int, t: c_int, n: c_int, d: c_int,
        x_bf16: *const u16, v_bf16: *const u16, freqs: *const f32, position: i64, chunk: c_int, flags: c_int,
        rho: *mut f32, out: *mut f32) -> c_int;
    pub fn bdh_prefill_chunked_ex(ctx: *mut bdh_ctx, b: c_int, h: c_int, t: c_int, n: c_int, d: c_int, rotary: c_int,
        x_bf16: *const u16, v_bf16: *const u16, freqs: *const f32, alibi_slopes_host: *const f32, position: i64,
        chunk: c_int, flags: c_int, block_size: c_int, rho: *mut f32, out: *mut f32) -> c_int;
    pub fn bdh_model_create(ctx: *mut bdh_ctx, config: *const bdh_model_config,
        weights: *const bdh_model_weights, out: *mut *mut bdh_model) -> c_int;
    pub fn bdh_model_destroy(model: *mut bdh_model) -> c_int;
    pub fn bdh_model_state_bytes(model: *const bdh_model, b: c_int, rho_dtype: c_int) -> usize;
    pub fn bdh_model_forward(model: *mut bdh_model, tokens: *const i64, b: c_int, t: c_int, rho: *mut c_void,
        rho_dtype: c_int, position: i64, logits: *mut f32, next_tokens: *mut i64, x_tap: *mut f32) -> c_int;
    pub fn bdh_model_forward_ex(model: *mut bdh_model, tokens: *const i64, b: c_int, t: c_int,
        rho: *mut c_void, rho_dtype: c_int, position: i64, positions_dev: *const i32, logits: *mut f32,
        next_tokens: *mut i64, x_tap: *mut f32) -> c_int;
    pub fn bdh_model_forward_fast(model: *mut bdh_model, tokens: *const i64, b: c_int, t: c_int,
        time_block_size: c_int, logits: *mut f32) -> c_int;
    pub fn bdh_model_forward_fast_ex(model: *mut bdh_model, tokens: *const i64, b: c_int, t: c_int,
        time_block_size: c_int, time_pairs_host: *const i32, n_time_pairs: c_int, latent_block_size: c_int,
        latent_blocks_host: *const u8, n_latent_blocks: c_int, logits: *mut f32) -> c_int;
    pub fn bdh_advance_positions(ctx: *mut bdh_ctx, positions_dev: *mut i32, b: c_int,
        delta: c_int) -> c_int;
    pub fn bdh_recurrent_attention_lazy_alibi(ctx: *mut bdh_ctx, b: c_int, h: c_int, t: c_int, n: c_int,
        d: c_int, x: *const f32, v: *const f32, clock: i64, clocks_dev: *const i32,
        alibi_slopes_host: *const f32, rho: *mut c_void, rho_dtype: c_int, stamps: *mut i32, out: *mut f32,
        active_bitmask: *mut u64, rows_touched: *mut i32) -> c_int;
    pub fn bdh_alibi_materialize(ctx: *mut bdh_ctx, b: c_int, h: c_int, n: c_int, d: c_int, clock: i64,
        clocks_dev: *const i32, alibi_slopes_host: *const f32, rho: *mut c_void, rho_dtype: c_int,
        stamps: *mut i32) -> c_int;
    pub fn bdh_model_forward_lazy(model: *mut bdh_model, tokens: *const i64, b: c_int, t: c_int,
        rho: *mut c_void, rho_dtype: c_int, stamps: *mut i32, position: i64, positions_dev: *const i32,
        logits: *mut f32, next_tokens: *mut i64, x_tap: *mut f32) -> c_int;
    pub fn bdh_model_forward_layers(model: *mut bdh_model, tokens: *const i64, b: c_int, t: c_int,
        rho_layers_host: *const *mut c_void, rho_dtype: c_int, stamps_layers_host: *const *mut i32, position: i64,
        positions_dev: *const i32, logits: *mut f32, next_tokens: *mut i64, x_tap: *mut f32) -> c_int;
    pub fn bdh_rho_energy(ctx: *mut bdh_ctx, b: c_int, h: c_int, n: c_int, d: c_int, rho: *const c_void,
        rho_dtype: c_int, stamps: *const i32, clock: i64, clocks_dev: *const i32,
        alibi_slopes_host: *const f32, out: *mut f32) -> c_int;
    pub fn bdh_model_forward_viz(model: *mut bdh_model, tokens: *const i64, b: c_int, t: c_int,
        rho: *mut c_void, rho_dtype: c_int, stamps: *mut i32, position: i64, positions_dev: *const i32,
        logits: *mut f32, next_tokens: *mut i64, x_tap: *mut f32, viz: *mut f32) -> c_int;
    pub fn bdh_model_logs_create(model: *mut bdh_model, b: c_int, rho_dtype: c_int, capacity: c_int,
        out: *mut *mut bdh_model_logs) -> c_int;
    pub fn bdh_model_logs_destroy(model: *mut bdh_model, logs: *mut bdh_model_logs) -> c_int;
    pub fn bdh_model_logs_pending(logs: *const bdh_model_logs) -> c_int;
    pub fn bdh_model_forward_deferred(model: *mut bdh_model, logs: *mut bdh_model_logs, tokens: *const i64, b: c_int,
        rho: *mut c_void, rho_dtype: c_int, position: i64, positions_dev: *const i32, logits: *mut f32,
        next_tokens: *mut i64) -> c_int;
    pub fn bdh_model_flush(model: *mut bdh_model, logs: *mut bdh_model_logs, rho: *mut c_void) -> c_int;
    pub fn bdh_model_forward_deferred_layers(model: *mut bdh_model, logs: *mut bdh_model_logs, tokens: *const i64,
        b: c_int, rho_layers_host: *const *mut c_void, rho_dtype: c_int, position: i64, positions_dev: *const i32,
        logits: *mut f32, next_tokens: *mut i64) -> c_int;
    pub fn bdh_model_flush_layers(model: *mut bdh_model, logs: *mut bdh_model_logs,
        rho_layers_host: *const *mut c_void) -> c_int;
    pub fn bdh_sample_top_k(ctx: *mut bdh_ctx, b: c_int, v: c_int, logits: *const f32, row_stride: i64,
        temperature: f32, top_k: c_int, uniforms: *const f32, next_tokens: *mut i64) -> c_int;
    pub fn bdh_probe_chunks(ctx: *mut bdh_ctx, region: *mut c_void, region_bytes: usize,
        chunk_index: *const i32, n_chunks: c_int, chunk_kib: c_int, mode: c_int,
        workgroups: c_int) -> c_int;
}
