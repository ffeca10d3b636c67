//! `rocm` arm of `GpuTensor` and of the backend-specific half of `TensorStore`
//! in src/native/src/tensor.rs (cuda arm: tensor.rs:60-93 and 325-540).  The
//! shared half (`insert`, `get`, `shape`, `ensure_grad`, ... tensor.rs:96-153)
//! is backend-agnostic and stays as it is.
//!
//! Differences from the cuda arm, all invisible through values:
//!  * `data` is an `Rc<DeviceBuf>`: a permuted view shares its source's buffer
//!    (the cuda arm clones it, ops/layout.rs:125); `offset` is always 0 here
//!    but lets a future slice view share storage too;
//!  * `ensure_contiguous` gathers on the device (mni_rocm_strided_copy) instead
//!    of the device -> host -> device round trip of tensor.rs:510-517;
//!  * in-place writers (`accumulate_grad`, `add_inplace`, `zero_grad`) first make
//!    the destination's buffer unique, so a view never sees the write.
#![allow(dead_code)]

use crate::allocator::CachingAllocator;
use crate::rocm_ffi::*;
use crate::tensor::{compute_strides, shape_size, TensorId, TensorStore};
use std::rc::Rc;

pub struct GpuTensor {
    pub data: Rc<DeviceBuf>,
    pub shape: Vec<usize>,
    pub strides: Vec<usize>,
    pub size: usize,
    pub requires_grad: bool,
    pub grad: Option<TensorId>,
    pub adam_m: Option<Rc<DeviceBuf>>,
    pub adam_v: Option<Rc<DeviceBuf>>,
}

impl GpuTensor {
    /// Same rule as the other arms (tensor.rs:41-53): every dim is compared,
    /// size-1 dims included.
    pub fn is_contiguous(&self) -> bool {
        let mut expected = 1usize;
        for i in (0..self.shape.len()).rev() {
            if self.strides[i] != expected {
                return false;
            }
            expected *= self.shape[i];
        }
        true
    }

    fn fresh(data: Rc<DeviceBuf>, shape: &[usize]) -> Self {
        GpuTensor {
            data,
            shape: shape.to_vec(),
            strides: compute_strides(shape),
            size: shape_size(shape),
            requires_grad: false,
            grad: None,
            adam_m: None,
            adam_v: None,
        }
    }
}

impl TensorStore {
    pub fn new() -> Self {
        let _ = crate::device::GpuDevice::instance();
        Self { tensors: Vec::new(), free_ids: Vec::new(), alloc: CachingAllocator::new() }
    }

    /// tensor.rs:350-355: the slot is emptied and its id recycled LIFO; the
    /// buffer goes back to the allocator when its last sharer is gone.
    pub fn free(&mut self, id: TensorId) {
        if let Some(t) = self.tensors[id].take() {
            self.alloc.dealloc(t.data);
            self.free_ids.push(id);
        }
    }

    pub fn dev_ptr(&self, id: TensorId) -> *const f32 {
        self.get(id).data.as_ptr()
    }

    pub fn dev_ptr_mut(&self, id: TensorId) -> *mut f32 {
        self.get(id).data.as_mut_ptr()
    }

    /// Values in the tensor's own (logical) order.
    pub fn to_host(&mut self, id: TensorId) -> Vec<f32> {
        let c = self.ensure_contiguous(id);
        let out = {
            let t = self.get(c);
            let mut v = t.data.to_host();
            v.truncate(t.size);
            v
        };
        if c != id {
            self.free(c);
        }
        out
    }

    pub fn get_scalar(&self, id: TensorId) -> f32 {
        let mut v = [0.0f32; 1];
        check(unsafe { mni_rocm_d2h(v.as_mut_ptr() as *mut _, self.dev_ptr(id) as *const _, 4) });
        v[0]
    }

    pub fn zeros(&mut self, shape: &[usize]) -> TensorId {
        let data = self.alloc.alloc(shape_size(shape));
        self.insert(GpuTensor::fresh(data, shape))
    }

    /// For outputs that a kernel writes in full (not in the reference: its
    /// `zeros` doubles as "allocate").
    pub fn uninit(&mut self, shape: &[usize]) -> TensorId {
        let data = self.alloc.alloc_uninit(shape_size(shape));
        self.insert(GpuTensor::fresh(data, shape))
    }

    pub fn ones(&mut self, shape: &[usize]) -> TensorId {
        let size = shape_size(shape);
        self.insert(GpuTensor::fresh(DeviceBuf::filled(size, 1.0), shape))
    }

    pub fn from_slice(&mut self, src: &[f32], shape: &[usize]) -> TensorId {
        let size = shape_size(shape);
        self.insert(GpuTensor::fresh(DeviceBuf::from_host(&src[..size]), shape))
    }

    pub fn from_vec(&mut self, src: Vec<f32>, shape: &[usize]) -> TensorId {
        self.from_slice(&src, shape)
    }

    /// A view: same buffer, other shape / strides (what `permute` returns).
    pub fn insert_view(&mut self, of: TensorId, shape: Vec<usize>, strides: Vec<usize>) -> TensorId {
        let data = Rc::clone(&self.get(of).data);
        let size = shape_size(&shape);
        self.insert(GpuTensor { data, shape, strides, size, requires_grad: false, grad: None, adam_m: None, adam_v: None })
    }

    /// Gather on the device (replaces tensor.rs:510-517).
    pub fn ensure_contiguous(&mut self, id: TensorId) -> TensorId {
        if self.get(id).is_contiguous() {
            return id;
        }
        let (shape, strides) = {
            let t = self.get(id);
            (t.shape.clone(), t.strides.clone())
        };
        let out = self.uninit(&shape);
        let shape_i: Vec<i64> = shape.iter().map(|&d| d as i64).collect();
        let strides_i: Vec<i64> = strides.iter().map(|&s| s as i64).collect();
        check(unsafe {
            mni_rocm_strided_copy(self.dev_ptr_mut(out), self.dev_ptr(id), shape_i.as_ptr(), strides_i.as_ptr(), shape.len() as i32)
        });
        out
    }

    /// Same data under a new shape, copied on the device (tensor.rs:519-536).
    pub fn clone_device(&mut self, src: TensorId, new_shape: &[usize]) -> TensorId {
        let c = self.ensure_contiguous(src);
        let size = self.get(c).size;
        let out = self.uninit(new_shape);
        check(unsafe { mni_rocm_d2d(self.dev_ptr_mut(out) as *mut _, self.dev_ptr(c) as *const _, size * 4) });
        if c != src {
            self.free(c);
        }
        out
    }

    /// Before writing in place: if a view shares the buffer, take a private copy.
    fn make_unique(&mut self, id: TensorId) {
        if Rc::strong_count(&self.get(id).data) > 1 {
            let len = self.get(id).data.len();
            let copy = DeviceBuf::uninit(len);
            check(unsafe { mni_rocm_d2d(copy.as_mut_ptr() as *mut _, self.dev_ptr(id) as *const _, len * 4) });
            self.get_mut(id).data = copy;
        }
    }

    /// grad(dst) += src  (tensor.rs:475-492)
    pub fn accumulate_grad(&mut self, dst: TensorId, src: TensorId) {
        let grad_id = self.ensure_grad(dst);
        self.add_inplace(grad_id, src);
    }

    /// dst += src  (tensor.rs:494-508)
    pub fn add_inplace(&mut self, dst: TensorId, src: TensorId) {
        let s = self.ensure_contiguous(src);
        self.make_unique(dst);
        let n = self.get(s).size as i64;
        check(unsafe { mni_rocm_axpy(self.dev_ptr_mut(dst), self.dev_ptr(s), 1.0, n) });
        if s != src {
            self.free(s);
        }
    }

    /// tensor.rs:395-410
    pub fn zero_grad(&mut self, id: TensorId) {
        if let Some(grad_id) = self.get(id).grad {
            self.make_unique(grad_id);
            let n = self.get(grad_id).size as i64;
            check(unsafe { mni_rocm_fill(self.dev_ptr_mut(grad_id), 0.0, n) });
        }
    }

    pub fn clear_alloc_cache(&mut self) {
        self.alloc.clear_cache();
    }

    /// The last two dims of tensor `id` as a GEMM operand: rows x cols with
    /// their strides, the leading dims collapsed into one batch stride.  The
    /// leading dims of every tensor the path produces nest (row-major or a
    /// permutation that keeps them in order); one that does not is gathered
    /// first, `scratch` then names the temporary to free after the launch.
    pub fn operand(&mut self, id: TensorId, scratch: &mut Option<TensorId>) -> MniOperand {
        let nests = {
            let t = self.get(id);
            let nd = t.shape.len();
            let mut ok = true;
            let mut expect: Option<usize> = None;
            for d in (0..nd.saturating_sub(2)).rev() {
                if t.shape[d] == 1 {
                    continue;
                }
                if let Some(e) = expect {
                    ok &= t.strides[d] == e;
                }
                expect = Some(t.strides[d] * t.shape[d]);
            }
            ok
        };
        let src = if nests {
            id
        } else {
            let c = self.ensure_contiguous(id);
            *scratch = Some(c);
            c
        };
        let t = self.get(src);
        let nd = t.shape.len();
        let batch_count: usize = t.shape[..nd - 2].iter().product::<usize>().max(1);
        let batch_stride = (0..nd - 2).rev().find(|&d| t.shape[d] > 1).map(|d| t.strides[d]).unwrap_or(0);
        MniOperand {
            ptr: t.data.as_ptr(),
            row_stride: t.strides[nd - 2] as i64,
            col_stride: t.strides[nd - 1] as i64,
            batch_stride: batch_stride as i64,
            batch_count: batch_count as i64,
        }
    }
}

/// The operand with rows and columns exchanged: what `transpose_last2`
/// (ops/matmul.rs:258-326) materialises in the other arms.
pub fn transposed(o: MniOperand) -> MniOperand {
    MniOperand { row_stride: o.col_stride, col_stride: o.row_stride, ..o }
}
