//! `rocm` arms of src/native/src/ops/matmul.rs: `matmul` (cuda arm :82-197),
//! `matmul_backward` (:224-255) and `matmul_no_grad` (:329-333).
//! `transpose_last2` (:287-326) has no rocm arm: a transposed operand is the
//! same buffer with its two strides exchanged.
#![allow(dead_code)]

use crate::autograd::{BackwardOp, SavedContext, Tape, TapeEntry};
use crate::rocm_ffi::*;
use crate::tensor::{shape_size, TensorId, TensorStore};
use crate::tensor_rocm::transposed;
use smallvec::smallvec;

/// out[..., M, N] = op_a[..., M, K] * op_b[..., K, N]; batch b of an operand
/// with fewer batches reads batch `b % count` (the CPU arm's rule, :55-56).
fn product(store: &mut TensorStore, a: MniOperand, b: MniOperand, m: usize, n: usize, k: usize, batch: usize, out_shape: &[usize]) -> TensorId {
    let (out, desc) = describe(store, a, b, m, n, k, batch, out_shape);
    check(unsafe { mni_rocm_sgemm(&desc) });
    out
}

/// A result tensor and the descriptor of the product that fills it; nothing is launched.
fn describe(store: &mut TensorStore, a: MniOperand, b: MniOperand, m: usize, n: usize, k: usize, batch: usize, out_shape: &[usize]) -> (TensorId, MniGemmDesc) {
    let out = store.uninit(out_shape);
    let desc = MniGemmDesc {
        m: m as i64,
        n: n as i64,
        k: k as i64,
        batch: batch as i64,
        a,
        b,
        c: store.dev_ptr_mut(out),
        ldc: n as i64,
        c_batch_stride: (m * n) as i64,
        bias: std::ptr::null(),
        epilogue: MNI_EPI_NONE,
        accumulate: 0,
        split_k: 0,
        algo: MNI_ALGO_AUTO,
        aux: std::ptr::null_mut(),
        colsum_part: std::ptr::null_mut(),
    };
    (out, desc)
}

struct Dims {
    m: usize,
    k: usize,
    n: usize,
    batch: usize,
    out_shape: Vec<usize>,
}

fn dims(store: &TensorStore, a: TensorId, b: TensorId) -> Dims {
    let a_shape = store.shape(a).to_vec();
    let b_shape = store.shape(b).to_vec();
    assert!(a_shape.len() >= 2 && b_shape.len() >= 2, "matmul requires at least 2D tensors");
    let (m, k) = (a_shape[a_shape.len() - 2], a_shape[a_shape.len() - 1]);
    let (k2, n) = (b_shape[b_shape.len() - 2], b_shape[b_shape.len() - 1]);
    assert_eq!(k, k2, "matmul inner dimensions must match: {} vs {}", k, k2);
    let out_batch = crate::utils::broadcast_shape(&a_shape[..a_shape.len() - 2], &b_shape[..b_shape.len() - 2]);
    let batch = shape_size(&out_batch);
    let mut out_shape = out_batch;
    out_shape.push(m);
    out_shape.push(n);
    Dims { m, k, n, batch, out_shape }
}

fn forward(a: TensorId, b: TensorId, store: &mut TensorStore) -> TensorId {
    let d = dims(store, a, b);
    let (mut ta, mut tb) = (None, None);
    let oa = store.operand(a, &mut ta);
    let ob = store.operand(b, &mut tb);
    let out = product(store, oa, ob, d.m, d.n, d.k, d.batch, &d.out_shape);
    for t in [ta, tb].into_iter().flatten() {
        store.free(t);
    }
    out
}

pub fn matmul(a: TensorId, b: TensorId, store: &mut TensorStore, tape: &mut Tape) -> TensorId {
    let out = forward(a, b, store);
    // the tape names the caller's ids, views included (:73-76)
    tape.record(TapeEntry {
        op: BackwardOp::MatMul,
        output_id: out,
        input_ids: smallvec![a, b],
        saved: SavedContext::Tensors(smallvec![a, b]),
    });
    out
}

pub fn matmul_no_grad(a: TensorId, b: TensorId, store: &mut TensorStore) -> TensorId {
    forward(a, b, store)
}

/// Sum a gradient down to the shape of the operand it belongs to: every dim that the batch broadcast had stretched,
/// the missing leading ones and interior ones of extent 1 alike (`a[2,1,M,K] * b[2,3,K,N]` sums dim 1 of the
/// `[2,3,M,K]` gradient).  `utils::unbroadcast` (utils.rs:39-66) on the device.
pub(crate) fn unbroadcast_device(store: &mut TensorStore, g: TensorId, to: &[usize]) -> TensorId {
    let from = store.shape(g).to_vec();
    if from == to {
        return g;
    }
    let gc = store.ensure_contiguous(g);
    let out = store.uninit(to);
    let from64: Vec<i64> = from.iter().map(|&d| d as i64).collect();
    let to64: Vec<i64> = to.iter().map(|&d| d as i64).collect();
    check(unsafe {
        mni_rocm_unbroadcast(store.dev_ptr_mut(out), store.dev_ptr(gc), from64.as_ptr(), from64.len() as i32, to64.as_ptr(), to64.len() as i32)
    });
    if gc != g {
        store.free(gc);
    }
    store.free(g);
    out
}

/// dA = unbroadcast(dC * B^T), dB = unbroadcast(A^T * dC); always both (:199-222).
pub fn matmul_backward(grad: TensorId, saved: &SavedContext, store: &mut TensorStore) -> Vec<Option<TensorId>> {
    if let SavedContext::Tensors(ids) = saved {
        let (a, b) = (ids[0], ids[1]);
        let a_shape = store.shape(a).to_vec();
        let b_shape = store.shape(b).to_vec();
        let d = dims(store, a, b);
        let (mut ta, mut tb, mut tg) = (None, None, None);
        let oa = store.operand(a, &mut ta);
        let ob = store.operand(b, &mut tb);
        let og = store.operand(grad, &mut tg);

        // dA[.., M, K] = dC[.., M, N] * B^T[.., N, K]
        let mut ga_shape = d.out_shape.clone();
        let nd = ga_shape.len();
        ga_shape[nd - 1] = d.k;
        let (ga, desc_a) = describe(store, og, transposed(ob), d.m, d.k, d.n, d.batch, &ga_shape);
        // dB[.., K, N] = A^T[.., K, M] * dC[.., M, N]
        let mut gb_shape = d.out_shape.clone();
        gb_shape[nd - 2] = d.k;
        let (gb, desc_b) = describe(store, transposed(oa), og, d.k, d.n, d.m, d.batch, &gb_shape);
        // the two products do not depend on each other: issued together, in one launch where the library pairs them
        check(unsafe { mni_rocm_sgemm_pair(&desc_a, &desc_b) });
        for t in [ta, tb, tg].into_iter().flatten() {
            store.free(t);
        }
        // a broadcast operand receives the sum over the batches it served
        let ga = unbroadcast_device(store, ga, &a_shape);
        let gb = unbroadcast_device(store, gb, &b_shape);
        vec![Some(ga), Some(gb)]
    } else {
        vec![None, None]
    }
}
