//! `rocm` arms of `add` and `add_backward` in src/native/src/ops/elementwise.rs
//! (cuda arms :76-197 and :213-231): the Linear layer's bias add and its
//! gradient.  Equal shapes and `[.., C] + [C]` run on the device; any other
//! broadcast pattern takes the CPU arm's `broadcast_binary` on host copies, as
//! the cuda arm's last branch does.
#![allow(dead_code)]

use crate::autograd::{BackwardOp, SavedContext, Tape, TapeEntry};
use crate::rocm_ffi::*;
use crate::tensor::{shape_size, TensorId, TensorStore};
use crate::utils::broadcast_shape;
use smallvec::smallvec;

pub fn add(a: TensorId, b: TensorId, store: &mut TensorStore, tape: &mut Tape) -> TensorId {
    let a_shape = store.shape(a).to_vec();
    let b_shape = store.shape(b).to_vec();
    let out_shape = broadcast_shape(&a_shape, &b_shape);
    let out = if a_shape == b_shape {
        // out = a, then out += b
        let out = store.clone_device(a, &out_shape);
        store.add_inplace(out, b);
        out
    } else if b_shape.len() == 1 && *a_shape.last().unwrap() == b_shape[0] {
        let ca = store.ensure_contiguous(a);
        let out = store.uninit(&out_shape);
        let cols = b_shape[0];
        let rows = shape_size(&a_shape) / cols;
        check(unsafe { mni_rocm_add_bias(store.dev_ptr_mut(out), store.dev_ptr(ca), store.dev_ptr(b), rows as i64, cols as i64) });
        if ca != a {
            store.free(ca);
        }
        out
    } else {
        // `broadcast_binary` (elementwise.rs:20-56) only needs `to_host`; the patch widens its
        // `cfg` from cpu / webgpu to rocm as well
        let (data, shape) = crate::ops::elementwise::broadcast_binary(a, b, store, |x, y| x + y);
        store.from_vec(data, &shape)
    };
    tape.record(TapeEntry {
        op: BackwardOp::Add,
        output_id: out,
        input_ids: smallvec![a, b],
        saved: SavedContext::TensorsAndShape(smallvec![a, b], out_shape),
    });
    out
}

pub fn add_backward(grad: TensorId, saved: &SavedContext, store: &mut TensorStore) -> Vec<Option<TensorId>> {
    if let SavedContext::TensorsAndShape(ids, _) = saved {
        let a_shape = store.shape(ids[0]).to_vec();
        let b_shape = store.shape(ids[1]).to_vec();
        let grad_shape = store.shape(grad).to_vec();
        let one = |store: &mut TensorStore, shape: &[usize]| -> TensorId {
            if shape == grad_shape.as_slice() {
                return store.clone_device(grad, shape);
            }
            // every broadcast dim summed on the device (the bias case [rows, C] -> [C] is the library's column sum;
            // interior dims of extent 1 go through its general form): utils::unbroadcast (utils.rs:39-66)
            let g = store.ensure_contiguous(grad);
            let out = store.uninit(shape);
            let from64: Vec<i64> = grad_shape.iter().map(|&d| d as i64).collect();
            let to64: Vec<i64> = shape.iter().map(|&d| d as i64).collect();
            check(unsafe {
                mni_rocm_unbroadcast(store.dev_ptr_mut(out), store.dev_ptr(g), from64.as_ptr(), from64.len() as i32, to64.as_ptr(), to64.len() as i32)
            });
            if g != grad {
                store.free(g);
            }
            out
        };
        let ga = one(store, &a_shape);
        let gb = one(store, &b_shape);
        vec![Some(ga), Some(gb)]
    } else {
        vec![None, None]
    }
}
