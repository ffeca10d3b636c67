//! `rocm` arm of src/native/src/device.rs (the cuda arm is device.rs:29-48 and
//! the kernel table behind it).  There is nothing to compile or look up at run
//! time: the kernels are code objects inside libmni_rocm.so, and the stream is
//! the library's own.  What remains of `GpuDevice` is "initialise once".
#![allow(dead_code)]

use crate::rocm_ffi::{check, mni_rocm_device_info, mni_rocm_init, mni_rocm_sync};
use std::os::raw::c_int;
use std::sync::OnceLock;

pub struct GpuDevice {
    pub name: String,
    pub compute_units: i32,
}

static GPU: OnceLock<GpuDevice> = OnceLock::new();

impl GpuDevice {
    /// One device, as in the reference (`CudaContext::new(0)`, device.rs:35).
    pub fn instance() -> &'static Self {
        GPU.get_or_init(|| {
            check(unsafe { mni_rocm_init(0) });
            let mut name = vec![0u8; 256];
            let mut cus: c_int = 0;
            check(unsafe { mni_rocm_device_info(name.as_mut_ptr() as *mut _, name.len(), &mut cus, std::ptr::null_mut()) });
            let end = name.iter().position(|&b| b == 0).unwrap_or(name.len());
            GpuDevice { name: String::from_utf8_lossy(&name[..end]).into_owned(), compute_units: cus }
        })
    }

    /// Waits for everything issued so far (the reference synchronises only
    /// through its blocking copies; exposed for tests and timing).
    pub fn synchronize(&self) {
        check(unsafe { mni_rocm_sync() });
    }
}
