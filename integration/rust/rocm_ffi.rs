//! FFI layer of the `rocm` backend: the kernel-level C ABI of libmni_rocm.so
//! (include/mni_rocm.h, section 1) as Rust declarations, plus the two helpers
//! every arm uses (`check`, `DeviceBuf`).
//!
//! Goes to src/native/src/rocm_ffi.rs; `mod rocm_ffi;` in lib.rs under
//! `#[cfg(feature = "rocm")]`.  Nothing here computes: every function forwards
//! pointers and sizes to the library.  The reference's arms `unwrap()` /
//! `expect()` their driver calls (src/native/src/tensor.rs:364, ops/matmul.rs:172),
//! i.e. misuse panics; `check` keeps that behaviour with the library's message.
#![allow(dead_code)]

use std::ffi::CStr;
use std::os::raw::{c_char, c_int, c_uint, c_void};
use std::rc::Rc;

pub const MNI_OK: c_int = 0;
pub const MNI_ERR_INVALID: c_int = 1;
pub const MNI_ERR_FREED: c_int = 2;
pub const MNI_ERR_HIP: c_int = 3;
pub const MNI_ERR_NOMEM: c_int = 4;

pub const MNI_EPI_NONE: i32 = 0;
pub const MNI_EPI_BIAS: i32 = 1;
pub const MNI_EPI_BIAS_RELU: i32 = 2;
pub const MNI_EPI_BIAS_GELU: i32 = 3;
pub const MNI_EPI_BIAS_GELU_DUAL: i32 = 4;
pub const MNI_EPI_DGELU: i32 = 5;

pub const MNI_ALGO_AUTO: i32 = 0;

/// One operand of a product: element (batch b, row r, col c) lives at
/// ptr[(b % batch_count) * batch_stride + r * row_stride + c * col_stride].
#[repr(C)]
#[derive(Clone, Copy)]
pub struct MniOperand {
    pub ptr: *const f32,
    pub row_stride: i64,
    pub col_stride: i64,
    pub batch_stride: i64,
    pub batch_count: i64,
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct MniGemmDesc {
    pub m: i64,
    pub n: i64,
    pub k: i64,
    pub batch: i64,
    pub a: MniOperand,
    pub b: MniOperand,
    pub c: *mut f32,
    pub ldc: i64,
    pub c_batch_stride: i64,
    pub bias: *const f32,
    pub epilogue: i32,
    pub accumulate: i32,
    pub split_k: i32,
    pub algo: i32,
    pub aux: *mut f32,
    pub colsum_part: *mut f32,
}

#[link(name = "mni_rocm")]
extern "C" {
    pub fn mni_rocm_init(device: c_int) -> c_int;
    pub fn mni_rocm_device_info(name: *mut c_char, name_cap: usize, compute_units: *mut c_int, clock_khz: *mut c_int) -> c_int;
    pub fn mni_rocm_device_xcds() -> c_int;
    pub fn mni_rocm_last_error() -> *const c_char;
    pub fn mni_rocm_malloc(ptr: *mut *mut c_void, bytes: usize) -> c_int;
    pub fn mni_rocm_free(ptr: *mut c_void) -> c_int;
    pub fn mni_rocm_clear_cache() -> c_int;
    pub fn mni_rocm_h2d(dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn mni_rocm_d2h(dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn mni_rocm_d2d(dst: *mut c_void, src: *const c_void, bytes: usize) -> c_int;
    pub fn mni_rocm_sync() -> c_int;
    pub fn mni_rocm_test_raise_device_status(code: c_uint) -> c_int;
    pub fn mni_rocm_launch_count() -> u64;
    pub fn mni_rocm_sgemm(desc: *const MniGemmDesc) -> c_int;
    pub fn mni_rocm_sgemm_pair(first: *const MniGemmDesc, second: *const MniGemmDesc) -> c_int;
    pub fn mni_rocm_sgemm_colsum_rows(m: i64, batch: i64) -> i64;
    pub fn mni_rocm_sgemm_noalloc(desc: *const MniGemmDesc) -> c_int;
    pub fn mni_rocm_sgemm_noalloc_workspace_bytes() -> usize;
    pub fn mni_rocm_strided_copy(dst: *mut f32, src: *const f32, shape: *const i64, src_strides: *const i64, ndim: c_int) -> c_int;
    pub fn mni_rocm_add_bias(out: *mut f32, a: *const f32, bias: *const f32, rows: i64, cols: i64) -> c_int;
    pub fn mni_rocm_colsum(out: *mut f32, a: *const f32, rows: i64, cols: i64) -> c_int;
    pub fn mni_rocm_unbroadcast(out: *mut f32, g: *const f32, g_shape: *const i64, g_ndim: c_int, to_shape: *const i64, to_ndim: c_int) -> c_int;
    pub fn mni_rocm_axpy(dst: *mut f32, src: *const f32, alpha: f32, n: i64) -> c_int;
    pub fn mni_rocm_fill(dst: *mut f32, value: f32, n: i64) -> c_int;
}

/// Non-zero status -> panic carrying the library's message, as the reference's
/// own arms panic on a failed driver call.
pub fn check(rc: c_int) {
    if rc != MNI_OK {
        let msg = unsafe { CStr::from_ptr(mni_rocm_last_error()) }.to_string_lossy().into_owned();
        panic!("{}", msg);
    }
}

/// A device allocation of `len` floats owned by the library's caching
/// allocator; returned to it on drop.  Tensors hold it behind an `Rc`, so a
/// permuted view and its source share one buffer.
pub struct DeviceBuf {
    ptr: *mut f32,
    len: usize,
}

impl DeviceBuf {
    /// Contents undefined.
    pub fn uninit(len: usize) -> Rc<Self> {
        let mut p: *mut c_void = std::ptr::null_mut();
        check(unsafe { mni_rocm_malloc(&mut p, len.max(1) * std::mem::size_of::<f32>()) });
        Rc::new(Self { ptr: p as *mut f32, len })
    }
    pub fn filled(len: usize, value: f32) -> Rc<Self> {
        let b = Self::uninit(len);
        check(unsafe { mni_rocm_fill(b.ptr, value, len as i64) });
        b
    }
    pub fn from_host(src: &[f32]) -> Rc<Self> {
        let b = Self::uninit(src.len());
        check(unsafe { mni_rocm_h2d(b.ptr as *mut c_void, src.as_ptr() as *const c_void, src.len() * 4) });
        b
    }
    pub fn to_host(&self) -> Vec<f32> {
        let mut out = vec![0.0f32; self.len];
        check(unsafe { mni_rocm_d2h(out.as_mut_ptr() as *mut c_void, self.ptr as *const c_void, self.len * 4) });
        out
    }
    pub fn as_ptr(&self) -> *const f32 {
        self.ptr
    }
    pub fn as_mut_ptr(&self) -> *mut f32 {
        self.ptr
    }
    pub fn len(&self) -> usize {
        self.len
    }
}

impl Drop for DeviceBuf {
    fn drop(&mut self) {
        // A failed free while unwinding must not panic again.
        let _ = unsafe { mni_rocm_free(self.ptr as *mut c_void) };
    }
}
