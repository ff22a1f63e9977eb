//! `engine::backend::mi355x` — `impl Backend` over `liborangu_mi355x.so`, meant to take
//! `engine/backend/rocm.rs`'s place behind the `rocm` feature (`src/bin/orangu-server/main.rs:3662-3681`).
//!
//! Source only: the build image that produced the library has no Rust toolchain, so this file has
//! not been compiled.  It declares exactly the symbols `include/orangu_mi355x.h` exports and maps the
//! trait (`engine/backend/mod.rs:309-496`) onto them one to one.  Link with
//! `cargo:rustc-link-lib=dylib=orangu_mi355x`.
//!
//! Error convention, as `RocmBackend` (`rocm.rs:168-173, 333-347`): `try_init_on` returns `None`
//! and never panics; a failure inside a matmul panics with the library's message and is caught per
//! request by `panic_capture`.

use std::ffi::{c_char, c_int, c_void, CStr};

use crate::engine::backend::{max_multi_token_phase_tokens, Backend, MatmulOp, MATMUL_ONLY_SURFACE};
use crate::engine::loader::QuantMatrix;

#[repr(C)]
pub struct OgmCtx {
    _private: [u8; 0],
}
#[repr(C)]
pub struct OgmWeight {
    _private: [u8; 0],
}
#[repr(C)]
struct OgmOp {
    w: *const OgmWeight,
    x: *const f32,
    n_tokens: u32,
    y: *mut f32,
}

extern "C" {
    fn ogm_init(device: c_int, out: *mut *mut OgmCtx) -> c_int;
    fn ogm_destroy(ctx: *mut OgmCtx);
    fn ogm_last_error(ctx: *mut OgmCtx) -> *const c_char;
    fn ogm_device_name(ctx: *mut OgmCtx, buf: *mut c_char, len: usize) -> c_int;
    fn ogm_supports_type(ggml_type: u32) -> c_int;
    fn ogm_supports(ggml_type: u32, in_dim: u32) -> c_int;
    fn ogm_weight_upload(
        ctx: *mut OgmCtx,
        ggml_type: u32,
        raw: *const c_void,
        row_bytes: usize,
        in_dim: u32,
        out_dim: u32,
        key_addr: u64,
        key_len: u64,
        out: *mut *mut OgmWeight,
    ) -> c_int;
    fn ogm_matmul(ctx: *mut OgmCtx, w: *const OgmWeight, x: *const f32, n_tokens: u32, y: *mut f32) -> c_int;
    fn ogm_matmul_decode(ctx: *mut OgmCtx, w: *const OgmWeight, x: *const f32, n_tokens: u32, y: *mut f32) -> c_int;
    fn ogm_matmul_batch(ctx: *mut OgmCtx, ops: *const OgmOp, n_ops: usize, decode: c_int, max_tokens: u32) -> c_int;
}

/// The MI355X backend.  The context serialises calls on its own mutex (one stream, one set of
/// scratch buffers), as `RocmBackend`'s `Mutex<RocmState>` does (`rocm.rs:30-41`), so sharing it
/// between the scheduler's blocking-pool threads (`scheduler.rs:16-22`) is safe.
pub struct Mi355xBackend {
    ctx: *mut OgmCtx,
    /// For the startup banner, like `RocmBackend::device_name`.
    pub device_name: String,
}

unsafe impl Send for Mi355xBackend {}
unsafe impl Sync for Mi355xBackend {}

impl Mi355xBackend {
    /// `None` when there is no gfx950 device or the HIP runtime is missing; never panics.
    pub fn try_init_on(device: usize) -> Option<Self> {
        let mut ctx = std::ptr::null_mut();
        if unsafe { ogm_init(device as c_int, &mut ctx) } != 0 || ctx.is_null() {
            return None;
        }
        let mut buf = [0 as c_char; 256];
        unsafe { ogm_device_name(ctx, buf.as_mut_ptr(), buf.len()) };
        let device_name = unsafe { CStr::from_ptr(buf.as_ptr()) }.to_string_lossy().into_owned();
        Some(Self { ctx, device_name })
    }

    pub fn try_init() -> Option<Self> {
        Self::try_init_on(0)
    }

    fn err(&self) -> String {
        unsafe { CStr::from_ptr(ogm_last_error(self.ctx)) }.to_string_lossy().into_owned()
    }

    fn check(&self, rc: c_int, what: &str) {
        assert_eq!(rc, 0, "mi355x {what}: {}", self.err());
    }

    /// Uploads on first sight of the matrix's cache key and reuses the device copy afterwards
    /// (`rocm.rs:329-350`); the library repacks the rows into its tile-planar layout once.
    fn weight(&self, w: &QuantMatrix) -> *const OgmWeight {
        let (addr, len) = w.cache_key(); // loader.rs:674-679
        let raw = w.raw_bytes(); // loader.rs:608-610
        let mut h = std::ptr::null_mut();
        let rc = unsafe {
            ogm_weight_upload(
                self.ctx,
                w.ggml_type(),
                raw.as_ptr().cast(),
                w.row_bytes(),
                w.in_dim as u32,
                w.out_dim as u32,
                addr as u64,
                len as u64,
                &mut h,
            )
        };
        self.check(rc, "weight upload");
        h
    }

    fn batch(&self, outs: &mut Vec<Vec<f32>>, ops: &[MatmulOp<'_>], decode: bool) {
        outs.resize_with(ops.len(), Vec::new);
        let mut raw_ops = Vec::with_capacity(ops.len());
        for (op, out) in ops.iter().zip(outs.iter_mut()) {
            debug_assert_eq!(op.x.len(), op.n_tokens * op.w.in_dim);
            out.resize(op.n_tokens * op.w.out_dim, 0.0);
            raw_ops.push(OgmOp {
                w: self.weight(op.w),
                x: op.x.as_ptr(),
                n_tokens: op.n_tokens as u32,
                y: out.as_mut_ptr(),
            });
        }
        // The library applies guarded_matmul_op's token stripes (mod.rs:154-172), groups ops that
        // read the same x (q/k/v, gate/up) into one launch, and synchronises once.
        let rc = unsafe {
            ogm_matmul_batch(
                self.ctx,
                raw_ops.as_ptr(),
                raw_ops.len(),
                decode as c_int,
                max_multi_token_phase_tokens() as u32,
            )
        };
        self.check(rc, "matmul_batch");
    }
}

impl Drop for Mi355xBackend {
    fn drop(&mut self) {
        unsafe { ogm_destroy(self.ctx) }
    }
}

impl Backend for Mi355xBackend {
    fn matmul(&self, x: &[f32], n_tokens: usize, w: &QuantMatrix) -> Vec<f32> {
        let mut out = Vec::new();
        self.matmul_into(&mut out, x, n_tokens, w);
        out
    }

    fn matmul_into(&self, out: &mut Vec<f32>, x: &[f32], n_tokens: usize, w: &QuantMatrix) {
        debug_assert_eq!(x.len(), n_tokens * w.in_dim);
        out.resize(n_tokens * w.out_dim, 0.0);
        let rc = unsafe { ogm_matmul(self.ctx, self.weight(w), x.as_ptr(), n_tokens as u32, out.as_mut_ptr()) };
        self.check(rc, "matmul");
    }

    /// Row `t` equals decoding token `t` alone, bit for bit (mod.rs:368-388).
    fn matmul_decode_into(&self, out: &mut Vec<f32>, x: &[f32], n_tokens: usize, w: &QuantMatrix) {
        debug_assert_eq!(x.len(), n_tokens * w.in_dim);
        out.resize(n_tokens * w.out_dim, 0.0);
        let rc =
            unsafe { ogm_matmul_decode(self.ctx, self.weight(w), x.as_ptr(), n_tokens as u32, out.as_mut_ptr()) };
        self.check(rc, "matmul_decode");
    }

    fn matmul_decode(&self, x: &[f32], n_tokens: usize, w: &QuantMatrix) -> Vec<f32> {
        let mut out = Vec::new();
        self.matmul_decode_into(&mut out, x, n_tokens, w);
        out
    }

    fn matmul_batch(&self, ops: &[MatmulOp<'_>]) -> Vec<Vec<f32>> {
        let mut outs = Vec::new();
        self.batch(&mut outs, ops, false);
        outs
    }

    fn matmul_batch_into(&self, outs: &mut Vec<Vec<f32>>, ops: &[MatmulOp<'_>]) {
        self.batch(outs, ops, false);
    }

    fn matmul_batch_decode(&self, ops: &[MatmulOp<'_>]) -> Vec<Vec<f32>> {
        let mut outs = Vec::new();
        self.batch(&mut outs, ops, true);
        outs
    }

    /// Q8_0, Q5_0, Q4_0, IQ4_NL, Q3_K, Q4_K, Q5_K, Q6_K; anything else is a start-up error through `unsupported_tensor_types`
    /// (mod.rs:522-533).
    fn supports_type(&self, ggml_type: u32) -> bool {
        unsafe { ogm_supports_type(ggml_type) != 0 }
    }

    fn reduced_surface(&self) -> Option<&'static str> {
        Some(MATMUL_ONLY_SURFACE)
    }
}

/// Whether a matrix of this type and row length has a kernel (`vecdot::supports`,
/// vecdot.rs:274-283): K-quants need `in_dim % 256 == 0`, Q8_0 `in_dim % 32 == 0`.
pub fn supports(ggml_type: u32, in_dim: usize) -> bool {
    unsafe { ogm_supports(ggml_type, in_dim as u32) != 0 }
}
