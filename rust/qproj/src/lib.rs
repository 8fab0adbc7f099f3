//! Safe wrapper over `qproj-sys`, the crate an engine depends on.
//!
//! Mirrors how the reference reaches its native code: one owner thread makes every call
//! (design/inference/engine.md:49-50), errors come back as values and the caller recovers the way
//! `icn-engine` recovers from a failed `llama_decode` (icn-engine/src/lib.rs:1597-1617): synchronize, drop the
//! batch, fail the active requests.  Device buffers for activations and outputs belong to the caller and are passed
//! as raw device pointers wrapped in `DevicePtr`; weights belong to the library.
use std::ffi::CStr;
use std::marker::PhantomData;
use std::os::raw::{c_int, c_void};
use std::ptr;

use qproj_sys as sys;

#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum WeightType {
    Q8_0 = 8,
    Q4K = 12,
    Q6K = 14,
}

#[derive(Debug, Clone, Copy, PartialEq, Eq)]
pub enum Activation {
    /// ggml's own arithmetic: activations to Q8_0 / Q8_K, integer dot products
    Ggml = 0,
    F32 = 1,
    /// per-32 int8 blocks with an fp32 scale (prefill)
    Q8x32 = 2,
}

#[derive(Debug, Clone, PartialEq, Eq)]
pub struct QprojError {
    pub status: i32,
    pub message: String,
}

impl std::fmt::Display for QprojError {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "qproj status {}: {}", self.status, self.message)
    }
}
impl std::error::Error for QprojError {}

pub type Result<T> = std::result::Result<T, QprojError>;

/// A device address owned by the caller (f32 unless said otherwise).
#[derive(Debug, Clone, Copy)]
pub struct DevicePtr(pub *mut c_void);

/// One device + one HIP stream.  Not `Sync`: a context is used from one thread, like the engine's executor.
pub struct Context {
    raw: *mut sys::qproj_ctx,
    _not_sync: PhantomData<*mut ()>,
}

unsafe impl Send for Context {}

pub struct Weight<'c> {
    raw: *mut sys::qproj_weight,
    ctx: &'c Context,
    pub k: i64,
    pub n: i64,
    pub n_expert: i64,
}

impl Context {
    /// `stream`: an existing `hipStream_t`, or null for a stream of the context's own.
    pub fn new(device: i32, stream: *mut c_void) -> Result<Context> {
        let mut raw = ptr::null_mut();
        let st = unsafe { sys::qproj_ctx_create(device as c_int, stream, &mut raw) };
        if st != sys::QPROJ_OK {
            return Err(QprojError { status: st, message: "qproj_ctx_create".into() });
        }
        Ok(Context { raw, _not_sync: PhantomData })
    }

    fn check(&self, st: c_int) -> Result<()> {
        if st == sys::QPROJ_OK {
            return Ok(());
        }
        let message = unsafe { CStr::from_ptr(sys::qproj_last_error(self.raw)) }.to_string_lossy().into_owned();
        Err(QprojError { status: st, message })
    }

    /// Waits for the stream and reports errors kernels met on the device (a bad expert id).
    pub fn synchronize(&self) -> Result<()> {
        self.check(unsafe { sys::qproj_sync(self.raw) })
    }

    /// GGUF bytes of `n_expert * n` rows of `k` weights (host memory) -> a resident weight.
    pub fn upload(&self, ty: WeightType, k: i64, n: i64, n_expert: i64, gguf_bytes: &[u8]) -> Result<Weight<'_>> {
        let row = unsafe { sys::qproj_row_bytes(ty as c_int, k) };
        if row == 0 || gguf_bytes.len() != row * (n * n_expert) as usize {
            return Err(QprojError { status: sys::QPROJ_ERR_INVALID_ARG, message: "byte count does not fit the shape".into() });
        }
        let mut raw = ptr::null_mut();
        self.check(unsafe { sys::qproj_upload(self.raw, ty as c_int, k, n, n_expert, gguf_bytes.as_ptr().cast(), &mut raw) })?;
        Ok(Weight { raw, ctx: self, k, n, n_expert })
    }

    /// GGML_OP_MUL_MAT for one to four tensors that share the activation rows (q/k/v, gate/up).
    pub fn mul_mat(&self, w: &[&Weight<'_>], x: DevicePtr, m: i64, y: &[DevicePtr], act: Activation) -> Result<()> {
        self.mul_mat_with(w, x, m, y, act, false)
    }

    /// The same without any device allocation (scratch in the library's fixed buffer): for graph capture.
    pub fn mul_mat_noalloc(&self, w: &[&Weight<'_>], x: DevicePtr, m: i64, y: &[DevicePtr], act: Activation) -> Result<()> {
        self.mul_mat_with(w, x, m, y, act, true)
    }

    fn mul_mat_with(&self, w: &[&Weight<'_>], x: DevicePtr, m: i64, y: &[DevicePtr], act: Activation, noalloc: bool) -> Result<()> {
        if w.is_empty() || w.len() > 4 || w.len() != y.len() {
            return Err(QprojError { status: sys::QPROJ_ERR_INVALID_ARG, message: "one to four tensors, one output each".into() });
        }
        let ws: Vec<*const sys::qproj_weight> = w.iter().map(|t| t.raw as *const _).collect();
        let ys: Vec<*mut f32> = y.iter().map(|p| p.0.cast()).collect();
        let st = unsafe {
            if noalloc {
                sys::qproj_mul_mat_multi_noalloc(self.raw, ws.len() as c_int, ws.as_ptr(), x.0.cast(), m, ys.as_ptr(), act as c_int)
            } else {
                sys::qproj_mul_mat_multi(self.raw, ws.len() as c_int, ws.as_ptr(), x.0.cast(), m, ys.as_ptr(), act as c_int)
            }
        };
        self.check(st)
    }

    /// GGML_OP_MUL_MAT_ID: ids `[b][n_used]` i32 on the device, x `[b][nb1][K]`, y `[b][n_used][N]`.
    pub fn mul_mat_id(&self, w: &Weight<'_>, x: DevicePtr, nb1: i64, ids: DevicePtr, n_used: i64, b: i64, y: DevicePtr) -> Result<()> {
        self.check(unsafe {
            sys::qproj_mul_mat_id(self.raw, w.raw, x.0.cast(), nb1, ids.0.cast(), n_used, b, y.0.cast(), Activation::Ggml as c_int)
        })
    }

    /// llama.cpp's build_moe_ffn: gate/up, SwiGLU, down and the weighted sum over a token's experts.
    #[allow(clippy::too_many_arguments)]
    pub fn moe_ffn(&self, gate: &Weight<'_>, up: &Weight<'_>, down: &Weight<'_>, x: DevicePtr, ids: DevicePtr,
                   weights: DevicePtr, n_used: i64, b: i64, y: DevicePtr) -> Result<()> {
        self.check(unsafe {
            sys::qproj_moe_ffn(self.raw, gate.raw, up.raw, down.raw, x.0.cast(), ids.0.cast(), weights.0.cast(), n_used, b,
                               y.0.cast(), Activation::Ggml as c_int)
        })
    }

    /// RMS norm (llama.cpp's `build_norm`, `LLM_NORM_RMS`) followed by the projections that read the normalised rows.
    #[allow(clippy::too_many_arguments)]
    pub fn rms_norm_mul_mat(&self, w: &[&Weight<'_>], x: DevicePtr, gamma: DevicePtr, eps: f32, m: i64, y: &[DevicePtr],
                            act: Activation) -> Result<()> {
        if w.is_empty() || w.len() > 4 || w.len() != y.len() {
            return Err(QprojError { status: sys::QPROJ_ERR_INVALID_ARG, message: "one to four tensors, one output each".into() });
        }
        let ws: Vec<*const sys::qproj_weight> = w.iter().map(|t| t.raw as *const _).collect();
        let ys: Vec<*mut f32> = y.iter().map(|p| p.0.cast()).collect();
        self.check(unsafe {
            sys::qproj_rms_norm_mul_mat(self.raw, ws.len() as c_int, ws.as_ptr(), x.0.cast(), gamma.0.cast(), eps, m, ys.as_ptr(),
                                        act as c_int)
        })
    }

    /// llama.cpp's `build_ffn` of a dense layer: (norm,) gate, up, swiglu, down.  `gamma`: the norm weights, or `None`
    /// for rows that are already normalised.
    #[allow(clippy::too_many_arguments)]
    pub fn ffn(&self, gate: &Weight<'_>, up: &Weight<'_>, down: &Weight<'_>, x: DevicePtr, gamma: Option<DevicePtr>, eps: f32,
               m: i64, y: DevicePtr) -> Result<()> {
        let (g, use_norm) = match gamma {
            Some(p) => (p.0 as *const f32, 1),
            None => (ptr::null(), 0),
        };
        self.check(unsafe {
            sys::qproj_ffn(self.raw, gate.raw, up.raw, down.raw, x.0.cast(), g, eps, use_norm, m, y.0.cast(),
                           Activation::Ggml as c_int)
        })
    }
}

/// Scratch bytes a `mul_mat` of this shape needs at most (what `mul_mat_noalloc` holds against its fixed buffer).
pub fn workspace_bytes(ty: WeightType, k: i64, rows: &[i64], m: i64, act: Activation) -> Result<usize> {
    let mut st: c_int = sys::QPROJ_OK;
    let bytes = unsafe { sys::qproj_workspace_bytes(ty as c_int, k, rows.len() as c_int, rows.as_ptr(), m, act as c_int, &mut st) };
    if st != sys::QPROJ_OK {
        return Err(QprojError { status: st, message: "qproj_workspace_bytes".into() });
    }
    Ok(bytes)
}

/// Which kernels a `mul_mat` of this shape would launch, one launch a line; needs no GPU.
pub fn plan_mul_mat(ty: WeightType, k: i64, rows: &[i64], m: i64, act: Activation, with_norm: bool) -> Result<String> {
    let mut buf = vec![0u8; 4096];
    let st = unsafe {
        sys::qproj_plan_mul_mat(ty as c_int, k, rows.len() as c_int, rows.as_ptr(), m, act as c_int, with_norm as c_int,
                                buf.as_mut_ptr().cast(), buf.len())
    };
    let text = CStr::from_bytes_until_nul(&buf).map(|c| c.to_string_lossy().into_owned()).unwrap_or_default();
    if st != sys::QPROJ_OK {
        return Err(QprojError { status: st, message: text });
    }
    Ok(text)
}

impl Drop for Context {
    fn drop(&mut self) {
        unsafe { sys::qproj_ctx_destroy(self.raw) };
    }
}

impl Drop for Weight<'_> {
    fn drop(&mut self) {
        unsafe { sys::qproj_weight_free(self.ctx.raw, self.raw) };
    }
}
