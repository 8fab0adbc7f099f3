//! Raw FFI for include/qproj.h (libqproj.so: GGUF Q8_0 / Q4_K / Q6_K projections on one MI355X).
//! Every function returns 0 (QPROJ_OK) on success; nothing aborts or unwinds across the boundary.
//! Not for direct use by workspace crates: depend on the safe `qproj` crate instead.
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_int, c_void};
#[repr(C)] pub struct qproj_ctx { _p: [u8; 0] }
#[repr(C)] pub struct qproj_weight { _p: [u8; 0] }
pub const QPROJ_TYPE_Q8_0: c_int = 8; pub const QPROJ_TYPE_Q4_K: c_int = 12; pub const QPROJ_TYPE_Q6_K: c_int = 14;
pub const QPROJ_ACT_GGML: c_int = 0;  pub const QPROJ_ACT_F32: c_int = 1;   pub const QPROJ_ACT_Q8X32: c_int = 2;
pub const QPROJ_OK: c_int = 0;
pub const QPROJ_ERR_INVALID_ARG: c_int = 1;
pub const QPROJ_ERR_HIP: c_int = 2;
pub const QPROJ_ERR_OOM: c_int = 3;
pub const QPROJ_ERR_UNSUPPORTED: c_int = 4;
pub const QPROJ_ERR_NO_DEVICE: c_int = 5;
pub const QPROJ_NOALLOC_SCRATCH_BYTES: usize = 64 << 20;
pub const QPROJ_PROBE_MAX_DEVICES: usize = 16;
pub const QPROJ_ELIGIBILITY_USABLE: c_int = 0;
pub const QPROJ_ELIGIBILITY_ABSENT: c_int = 1;
pub const QPROJ_ELIGIBILITY_FAILED: c_int = 2;

/// struct qproj_eligibility of include/qproj.h
#[repr(C)]
pub struct qproj_eligibility {
    pub state: c_int,
    pub driver_api: c_int,
    pub runtime_api: c_int,
    pub n_devices: c_int,
    pub architectures: [[c_char; 32]; QPROJ_PROBE_MAX_DEVICES],
    pub hardware_labels: [[c_char; 256]; QPROJ_PROBE_MAX_DEVICES],
    pub runtime_library: [c_char; 1024],
    pub diagnostic: [c_char; 244],
}

extern "C" {
    pub fn qproj_device_count(count: *mut c_int) -> c_int;
    pub fn qproj_ctx_create(device: c_int, stream: *mut c_void, out: *mut *mut qproj_ctx) -> c_int;
    pub fn qproj_ctx_destroy(ctx: *mut qproj_ctx) -> c_int;
    pub fn qproj_sync(ctx: *mut qproj_ctx) -> c_int;
    pub fn qproj_last_error(ctx: *const qproj_ctx) -> *const c_char;
    pub fn qproj_stream(ctx: *const qproj_ctx) -> *mut c_void;
    pub fn qproj_row_bytes(ty: c_int, k: i64) -> usize;
    pub fn qproj_upload(ctx: *mut qproj_ctx, ty: c_int, k: i64, n: i64, n_expert: i64,
                        gguf_bytes: *const c_void, out: *mut *mut qproj_weight) -> c_int;
    pub fn qproj_upload_from_device(ctx: *mut qproj_ctx, ty: c_int, k: i64, n: i64, n_expert: i64,
                        gguf_bytes_dev: *const c_void, out: *mut *mut qproj_weight) -> c_int;
    pub fn qproj_download(ctx: *mut qproj_ctx, w: *const qproj_weight, out: *mut c_void) -> c_int;
    pub fn qproj_weight_free(ctx: *mut qproj_ctx, w: *mut qproj_weight) -> c_int;
    pub fn qproj_weight_info(w: *const qproj_weight, ty: *mut c_int, k: *mut i64, n: *mut i64,
                             n_expert: *mut i64, gguf_bytes: *mut usize) -> c_int;
    pub fn qproj_dequantize(ctx: *mut qproj_ctx, w: *const qproj_weight, out_dev: *mut f32) -> c_int;
    pub fn qproj_act_bytes(kind: c_int, wtype: c_int, m: i64, k: i64) -> usize;
    pub fn qproj_quantize_activations(ctx: *mut qproj_ctx, kind: c_int, wtype: c_int, x_dev: *const f32,
                                      m: i64, k: i64, out_dev: *mut c_void) -> c_int;
    pub fn qproj_rms_norm(ctx: *mut qproj_ctx, x_dev: *const f32, gamma_dev: *const f32, eps: f32,
                          m: i64, k: i64, y_dev: *mut f32) -> c_int;
    pub fn qproj_rms_norm_quantize(ctx: *mut qproj_ctx, kind: c_int, wtype: c_int, x_dev: *const f32,
                                   gamma_dev: *const f32, eps: f32, m: i64, k: i64,
                                   out_dev: *mut c_void) -> c_int;
    pub fn qproj_rms_norm_mul_mat(ctx: *mut qproj_ctx, n: c_int, w: *const *const qproj_weight,
                                  x_dev: *const f32, gamma_dev: *const f32, eps: f32, m: i64,
                                  y_dev: *const *mut f32, act: c_int) -> c_int;
    pub fn qproj_ffn_gate_up(ctx: *mut qproj_ctx, gate: *const qproj_weight, up: *const qproj_weight,
                             x_dev: *const f32, m: i64, h_dev: *mut f32, act: c_int) -> c_int;
    pub fn qproj_rms_norm_ffn_gate_up(ctx: *mut qproj_ctx, gate: *const qproj_weight,
                                      up: *const qproj_weight, x_dev: *const f32, gamma_dev: *const f32,
                                      eps: f32, m: i64, h_dev: *mut f32, act: c_int) -> c_int;
    pub fn qproj_ffn(ctx: *mut qproj_ctx, gate: *const qproj_weight, up: *const qproj_weight,
                     down: *const qproj_weight, x_dev: *const f32, gamma_dev: *const f32, eps: f32,
                     use_norm: c_int, m: i64, y_dev: *mut f32, act: c_int) -> c_int;
    pub fn qproj_mul_mat(ctx: *mut qproj_ctx, w: *const qproj_weight, x_dev: *const f32, m: i64,
                         y_dev: *mut f32, act: c_int) -> c_int;
    pub fn qproj_mul_mat_multi(ctx: *mut qproj_ctx, n: c_int, w: *const *const qproj_weight,
                               x_dev: *const f32, m: i64, y_dev: *const *mut f32, act: c_int) -> c_int;
    pub fn qproj_mul_mat_multi_noalloc(ctx: *mut qproj_ctx, n: c_int, w: *const *const qproj_weight,
                                       x_dev: *const f32, m: i64, y_dev: *const *mut f32, act: c_int) -> c_int;
    pub fn qproj_workspace_bytes(ty: c_int, k: i64, n: c_int, rows: *const i64, m: i64, act: c_int,
                                 status: *mut c_int) -> usize;
    pub fn qproj_plan_mul_mat(ty: c_int, k: i64, n: c_int, rows: *const i64, m: i64, act: c_int, with_norm: c_int,
                              buf: *mut c_char, buf_bytes: usize) -> c_int;
    pub fn qproj_plan_moe_ffn(gate_ty: c_int, down_ty: c_int, d_model: i64, d_ff: i64, n_expert: i64, n_used: i64,
                              b: i64, buf: *mut c_char, buf_bytes: usize) -> c_int;
    pub fn qproj_mul_mat_quantized(ctx: *mut qproj_ctx, n: c_int, w: *const *const qproj_weight,
                                   act_dev: *const c_void, kind: c_int, m: i64, y_dev: *const *mut f32) -> c_int;
    pub fn qproj_mul_mat_id(ctx: *mut qproj_ctx, w: *const qproj_weight, x_dev: *const f32, nb1: i64,
                            ids_dev: *const i32, n_used: i64, b: i64, y_dev: *mut f32, act: c_int) -> c_int;
    pub fn qproj_moe_ffn(ctx: *mut qproj_ctx, gate: *const qproj_weight, up: *const qproj_weight,
                         down: *const qproj_weight, x_dev: *const f32, ids_dev: *const i32,
                         weights_dev: *const f32, n_used: i64, b: i64, y_dev: *mut f32, act: c_int) -> c_int;
    pub fn qproj_version() -> *const c_char;
    pub fn qproj_probe_eligibility(out: *mut qproj_eligibility) -> c_int;
}
