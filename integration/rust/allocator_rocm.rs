//! `rocm` arm of src/native/src/allocator.rs (cuda arm: allocator.rs:46-84).
//! The exact-size free lists live inside libmni_rocm.so (mni_rocm_malloc /
//! mni_rocm_free / mni_rocm_clear_cache), shared with the library's own
//! workspaces, so this type only keeps the reference's interface and its
//! byte count.  Unlike the cuda arm, `alloc` hands out zeroed memory also when
//! a block is recycled (`zeros()` relies on that, tensor.rs:412-420).
#![allow(dead_code)]

use crate::rocm_ffi::{check, mni_rocm_clear_cache, DeviceBuf};
use std::rc::Rc;

pub struct CachingAllocator {
    total_allocated: usize,
}

impl CachingAllocator {
    pub fn new() -> Self {
        Self { total_allocated: 0 }
    }

    /// `size` floats, all zero.
    pub fn alloc(&mut self, size: usize) -> Rc<DeviceBuf> {
        self.total_allocated += size * 4;
        DeviceBuf::filled(size, 0.0)
    }

    /// `size` floats, contents undefined (for outputs that are fully written).
    pub fn alloc_uninit(&mut self, size: usize) -> Rc<DeviceBuf> {
        self.total_allocated += size * 4;
        DeviceBuf::uninit(size)
    }

    /// Dropping the last reference returns the block to the library's free list.
    pub fn dealloc(&mut self, buf: Rc<DeviceBuf>) {
        drop(buf);
    }

    pub fn clear_cache(&mut self) {
        check(unsafe { mni_rocm_clear_cache() });
    }

    pub fn allocated_bytes(&self) -> usize {
        self.total_allocated
    }
}
