"""Pins the oracle's autograd tape, backward functions, losses and optimiser
WITHOUT a GPU: reference-held gradient values (test/autograd.test.ts,
test/nn.test.ts, test/module.test.ts), closed forms evaluated in float64 with
numpy, and central finite differences."""
import math

import numpy as np
import pytest

from framework_amd import synth
from helpers import max_err


def _t(api, a, grad=False):
    a = np.asarray(a, dtype=np.float32)
    t = api.Tensor.fromFloat32(a, list(a.shape))
    return t.setRequiresGrad(True) if grad else t


# ---- reference-held gradient checks (test/autograd.test.ts) -----------------

def test_mul_and_add_gradients(orc):
    a = _t(orc, [[1, 2], [3, 4]], True)
    b = _t(orc, [[5, 6], [7, 8]], True)
    a.mul(b).sum(0).sum(0).backward()
    assert list(a.grad.toFloat32()) == [5, 6, 7, 8]  # autograd.test.ts:19-30
    assert list(b.grad.toFloat32()) == [1, 2, 3, 4]
    x = _t(orc, [2, 3], True)
    y = _t(orc, [4, 5], True)
    x.add(y).sum().backward()
    assert list(x.grad.toFloat32()) == [1, 1] and list(y.grad.toFloat32()) == [1, 1]  # :32-39


def test_matmul_gradient_closed_form(orc):
    # autograd.test.ts:42-46 only asserts existence; the values follow from
    # dX = G Y^T, dY = X^T G with G = ones.
    x = _t(orc, [[1, 0], [0, 1]], True)
    y = _t(orc, [[3, 4], [5, 6]], True)
    x.matmul(y).sum().backward()
    assert list(x.grad.toFloat32()) == [7, 11, 7, 11]
    assert list(y.grad.toFloat32()) == [1, 1, 1, 1]


# ---- matmul backward: closed form, finite differences, broadcast ------------

def _loss_weights(shape, seed):
    return synth.normal(seed, shape, stream=7)


@pytest.mark.parametrize("m,k,n", [(3, 4, 5), (8, 8, 8), (1, 6, 2)])
def test_matmul_backward_vs_closed_form_and_fd(orc, m, k, n):
    a = synth.normal(1, (m, k))
    b = synth.normal(2, (k, n), stream=1)
    r = _loss_weights((m, n), 3)
    A, B = _t(orc, a, True), _t(orc, b, True)
    A.matmul(B).mul(_t(orc, r)).sum().backward()  # loss = sum(R * (A B))
    ga, gb = A.grad.numpy(), B.grad.numpy()
    a64, b64, r64 = a.astype(np.float64), b.astype(np.float64), r.astype(np.float64)
    assert max_err(ga, r64 @ b64.T) < 1e-5
    assert max_err(gb, a64.T @ r64) < 1e-5
    # central differences in float64 on the closed-form loss
    f = lambda aa, bb: float(np.sum(r64 * (aa @ bb)))
    eps = 1e-5
    for (i, j) in [(0, 0), (m - 1, k - 1)]:
        d = np.zeros_like(a64); d[i, j] = eps
        assert abs((f(a64 + d, b64) - f(a64 - d, b64)) / (2 * eps) - ga[i, j]) < 1e-4
    for (i, j) in [(0, 0), (k - 1, n - 1)]:
        d = np.zeros_like(b64); d[i, j] = eps
        assert abs((f(a64, b64 + d) - f(a64, b64 - d)) / (2 * eps) - gb[i, j]) < 1e-4


def test_matmul_backward_sums_broadcast_batch(orc):
    # [B, M, K] x [K, N]: dW is summed over the batch (utils::unbroadcast)
    x = synth.normal(4, (3, 4, 5))
    w = synth.normal(5, (5, 2), stream=1)
    r = _loss_weights((3, 4, 2), 6)
    X, W = _t(orc, x, True), _t(orc, w, True)
    X.matmul(W).mul(_t(orc, r)).sum().backward()
    x64, w64, r64 = x.astype(np.float64), w.astype(np.float64), r.astype(np.float64)
    assert W.grad.shape == [5, 2] and X.grad.shape == [3, 4, 5]
    assert max_err(W.grad.numpy(), np.einsum("bmk,bmn->kn", x64, r64)) < 1e-5
    assert max_err(X.grad.numpy(), r64 @ w64.T) < 1e-5
    # the other way round: [M, K] x [B, K, N]
    a = synth.normal(7, (4, 5))
    bb = synth.normal(8, (3, 5, 2), stream=1)
    A, Bt = _t(orc, a, True), _t(orc, bb, True)
    A.matmul(Bt).mul(_t(orc, r)).sum().backward()
    assert max_err(A.grad.numpy(), np.einsum("bmn,bkn->mk", r64, bb.astype(np.float64))) < 1e-5
    assert max_err(Bt.grad.numpy(), np.einsum("mk,bmn->bkn", a.astype(np.float64), r64)) < 1e-5


def test_attention_scores_through_permuted_view(orc):
    # Q K^T with K^T a permuted view; gradients reach K in K's own layout
    q = synth.normal(2, (2, 6, 4))
    k = synth.normal(2, (2, 6, 4), stream=1)
    ds = _loss_weights((2, 6, 6), 9)
    Q, K = _t(orc, q, True), _t(orc, k, True)
    Q.matmul(K.permute(0, 2, 1)).mul(_t(orc, ds)).sum().backward()
    q64, k64, g = q.astype(np.float64), k.astype(np.float64), ds.astype(np.float64)
    assert K.grad.shape == [2, 6, 4]
    assert max_err(Q.grad.numpy(), g @ k64) < 1e-5                       # dQ = dS K
    assert max_err(K.grad.numpy(), g.transpose(0, 2, 1) @ q64) < 1e-5    # dK = dS^T Q


def test_permute_backward_general(orc):
    x = synth.normal(3, (2, 3, 4))
    r = _loss_weights((4, 2, 3), 4)
    X = _t(orc, x, True)
    X.permute(2, 0, 1).mul(_t(orc, r)).sum().backward()
    assert np.array_equal(X.grad.numpy(), r.transpose(1, 2, 0))


# ---- tape rules ---------------------------------------------------------------

def test_same_tensor_twice_adds_both_grads(orc):
    d = _t(orc, [[1, -2], [3, 4]], True)
    d.mul(d).sum().backward()  # the diff.mul(diff) of mseLoss: grad 2 d
    assert list(d.grad.toFloat32()) == [2, -4, 6, 8]


def test_seed_is_ones_for_non_scalar_loss(orc):
    x = _t(orc, [[1, 2], [3, 4]], True)
    x.mul(3.0).backward()  # autograd.rs:143 seeds ones_like(loss)
    assert list(x.grad.toFloat32()) == [3, 3, 3, 3]


def test_grad_accumulates_across_backwards_and_zero_grad(orc):
    x = _t(orc, [1, 2], True)
    x.mul(2.0).sum().backward()
    x.mul(2.0).sum().backward()
    assert list(x.grad.toFloat32()) == [4, 4]
    orc.native.zeroGrad([x._id])
    assert list(x.grad.toFloat32()) == [0, 0]
    assert _t(orc, [1.0]).grad is None


def test_no_grad_and_backward_reenables_tape(orc):
    x = _t(orc, [1, 2], True)
    orc.native.noGradStart()
    y = x.mul(2.0).sum()
    orc.native.noGradEnd()
    y.backward()
    assert x.grad is None  # nothing recorded
    orc.native.noGradStart()
    x.mul(1.0).sum().backward()  # backward installs a fresh *enabled* tape (lib.rs:135)
    z = x.mul(5.0).sum()
    z.backward()
    assert list(x.grad.toFloat32()) == [5, 5]


# ---- bias add / unbroadcast -----------------------------------------------------

def test_linear_forward_backward_closed_form(orc):
    x = synth.normal(1, (4, 3))
    w = synth.normal(2, (3, 2), stream=1)
    b = synth.normal(3, (2,), stream=2)
    r = _loss_weights((4, 2), 5)
    lin = orc.Linear(3, 2, weight=w, bias=b)
    out = lin.forward(_t(orc, x))
    assert out.shape == [4, 2] and len(lin.parameters()) == 2  # test/nn.test.ts:217-226
    assert max_err(out.numpy(), x.astype(np.float64) @ w + b) < 1e-5
    out.mul(_t(orc, r)).sum().backward()
    assert max_err(lin.weight.value.grad.numpy(), x.astype(np.float64).T @ r) < 1e-5
    assert max_err(lin.bias.value.grad.numpy(), r.astype(np.float64).sum(0)) < 1e-5


def test_broadcast_add_mul_values(orc):
    a = _t(orc, [[1, 2, 3], [4, 5, 6]])
    b = _t(orc, [10, 20, 30])
    assert list(a.add(b).toFloat32()) == [11, 22, 33, 14, 25, 36]  # test/tensor.test.ts:248-256
    assert list(a.mul(b).toFloat32()) == [10, 40, 90, 40, 100, 180]
    col = _t(orc, [[1], [2]])
    assert list(a.sub(col).toFloat32()) == [0, 1, 2, 2, 3, 4]
    assert list(a.add(5).toFloat32()) == [6, 7, 8, 9, 10, 11]


def test_unbroadcast_patterns(orc):
    g = _loss_weights((2, 3, 4), 11)
    for shape, axes in [([4], (0, 1)), ([3, 1], (0, 2)), ([1, 3, 4], (0,)), ([2, 1, 4], (1,)), ([1], (0, 1, 2))]:
        orc.native.resetEngine()
        a = _t(orc, np.zeros((2, 3, 4)), True)
        b = _t(orc, np.zeros(shape), True)
        a.add(b).mul(_t(orc, g)).sum().backward()
        want = g.astype(np.float64).sum(axis=axes, keepdims=True).reshape(shape)
        assert b.grad.shape == shape
        assert max_err(b.grad.numpy(), want) < 1e-5
        orc.native.resetEngine()
        a = _t(orc, np.zeros((2, 3, 4)), True)
        b = _t(orc, np.zeros(shape), True)
        a.sub(b).mul(_t(orc, g)).sum().backward()
        assert max_err(b.grad.numpy(), -want) < 1e-5


# ---- reductions, mseLoss quirks ------------------------------------------------------

def test_sum_mean_values_and_backward(orc):
    x = synth.normal(1, (2, 3, 4))
    X = _t(orc, x)
    for d in (0, 1, 2, -1):
        assert max_err(X.sum(d).numpy(), x.astype(np.float64).sum(d, keepdims=True)) < 1e-5
        assert max_err(X.mean(d).numpy(), x.astype(np.float64).mean(d, keepdims=True)) < 1e-5
    assert X.sum().shape == [1, 1, 1]
    Y = _t(orc, x, True)
    Y.mean(1).sum().backward()
    assert np.allclose(Y.grad.numpy(), 1.0 / 3.0)


def test_mse_loss_reference_semantics(orc):
    p = _t(orc, [[1, 2], [3, 4]])
    assert orc.mseLoss(p, _t(orc, [[1, 2], [3, 4]])).toFloat32()[0] == 0  # test/nn.test.ts:78-81
    l = orc.mseLoss(p, _t(orc, [[2, 3], [4, 5]]))
    assert abs(l.toFloat32()[0] - 1.0) < 1e-6  # :83-86
    # mean(-1) twice: a [rows, 1] tensor, not a scalar (src/nn.ts:161-165)
    assert l.shape == [2, 1]
    pred = synth.normal(1, (5, 8))
    tgt = synth.normal(2, (5, 8), stream=1)
    P = _t(orc, pred, True)
    L = orc.mseLoss(P, _t(orc, tgt))
    assert max_err(L.numpy()[:, 0], ((pred.astype(np.float64) - tgt) ** 2).mean(1)) < 1e-6
    L.backward()  # seeds ones over every row
    assert max_err(P.grad.numpy(), 2 * (pred.astype(np.float64) - tgt) / 8) < 1e-6


def test_mean_backward_divisor_rule(orc):
    # divisor = extent of the LAST dim with grad 1 and orig > 1, else 1 (reduce.rs:242-247)
    x = _t(orc, np.ones((3, 1)), True)
    x.mean(-1).sum().backward()  # reduced dim has extent 1: divisor 1
    assert list(x.grad.toFloat32()) == [1, 1, 1]


# ---- activations -------------------------------------------------------------------------

def test_relu_gelu_anchors_and_grads(orc):
    x = np.array([-2.0, -0.5, 0.0, 0.5, 2.0], dtype=np.float32)
    assert list(_t(orc, x).relu().toFloat32()) == [0, 0, 0, 0.5, 2.0]
    g = _t(orc, x).gelu().numpy()
    x64 = x.astype(np.float64)
    ref = 0.5 * x64 * (1 + np.tanh(math.sqrt(2 / math.pi) * (x64 + 0.044715 * x64 ** 3)))
    assert max_err(g, ref) < 1e-6
    assert g[2] == 0 and abs(g[4] - 1.9546) < 1e-3  # test/nn.test.ts:17-27 anchors
    X = _t(orc, x, True)
    X.relu().sum().backward()
    assert list(X.grad.toFloat32()) == [0, 0, 0, 1, 1]  # x > 0 strictly
    X2 = _t(orc, x, True)
    X2.gelu().sum().backward()
    eps = 1e-6
    f = lambda v: 0.5 * v * (1 + np.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3)))
    fd = (f(x64 + eps) - f(x64 - eps)) / (2 * eps)
    assert max_err(X2.grad.numpy(), fd) < 1e-5


# ---- cross entropy ----------------------------------------------------------------------------

def test_cross_entropy_closed_form(orc):
    logits = synth.normal(1, (6, 5), std=2.0)
    targets = synth.integers(2, (6,), 0, 5)
    L = _t(orc, logits, True)
    loss = orc.crossEntropyLoss(L, [[int(t)] for t in targets])
    assert loss.shape == [1]
    z = logits.astype(np.float64)
    lse = np.log(np.exp(z - z.max(1, keepdims=True)).sum(1)) + z.max(1)
    want = float(np.mean(lse - z[np.arange(6), targets]))
    assert abs(loss.toFloat32()[0] - want) < 1e-5
    loss.backward()
    sm = np.exp(z - lse[:, None])
    sm[np.arange(6), targets] -= 1
    assert max_err(L.grad.numpy(), sm / 6) < 1e-6
    # test/nn.test.ts:70-76: a perfect prediction scores lower
    perfect = orc.crossEntropyLoss(_t(orc, [[100, -100, -100], [-100, -100, 100]]), [[0], [2]]).toFloat32()[0]
    assert perfect < loss.toFloat32()[0]


# ---- Adam ------------------------------------------------------------------------------------------

def test_adam_steps_closed_form(orc):
    p0 = np.array([5.0, -3.0, 0.5, 2.0], dtype=np.float32)
    P = orc.Parameter(_t(orc, p0, True))
    opt = orc.Adam([P], lr=0.01)  # defaults beta1 .9, beta2 .95, eps 1e-8 (src/optimizer.ts:46-56)
    assert (opt.beta1, opt.beta2, opt.eps, opt.weightDecay) == (0.9, 0.95, 1e-8, 0.0)
    p = p0.astype(np.float64)
    m = np.zeros(4); v = np.zeros(4)
    for t in (1, 2, 3):
        opt.zeroGrad()
        P.value.mul(P.value).sum().backward()  # grad = 2 p
        norm = opt.step()
        g = 2 * p
        assert abs(norm - np.linalg.norm(g)) < 1e-4 * np.linalg.norm(g)
        m = 0.9 * m + 0.1 * g
        v = 0.95 * v + 0.05 * g * g
        p = p - 0.01 * (m / (1 - 0.9 ** t)) / (np.sqrt(v / (1 - 0.95 ** t)) + 1e-8)
        assert max_err(P.value.toFloat32(), p) < 1e-5
    # first step moves every element by ~lr * sign(g)
    assert abs((p0[0] - 0.01) - (p0.astype(np.float64) - 0.01 * np.sign(p0))[0]) < 1e-6


def test_clip_scales_grads_before_step(orc):
    P = orc.Parameter(_t(orc, [3.0, 4.0], True))
    P.value.mul(1.0).sum().backward()  # grad = [1, 1], norm sqrt(2)
    opt = orc.Adam([P], lr=0.1)
    norm = opt.step(0.5)  # clip to 0.5
    assert abs(norm - math.sqrt(2)) < 1e-6
    assert max_err(P.value.grad.toFloat32(), np.array([0.5, 0.5]) / math.sqrt(2)) < 1e-6


def test_regression_converges_like_reference_suite(orc):
    # test/module.test.ts:113-130 with a seeded init instead of thread_rng
    X = _t(orc, [[0], [1], [2], [3], [4], [5]])
    Y = _t(orc, [[1], [3], [5], [7], [9], [11]])
    net = orc.Linear(1, 1, weight=synth.uniform(1, (1, 1), -1, 1), bias=synth.uniform(2, (1,), -1, 1))
    opt = orc.Adam(net.parameters(), lr=0.05)
    early = None
    for i in range(200):
        opt.zeroGrad()
        loss = orc.mseLoss(net.forward(X), Y)
        if i == 10:
            early = loss.toFloat32()[0]
        loss.backward()
        opt.step()
    final = orc.mseLoss(net.forward(X), Y).toFloat32()[0]
    assert final < early and final < 1.0


def test_gc_keeps_listed_tensors(orc):
    a = _t(orc, [1, 2])
    b = _t(orc, [3, 4])
    orc.native.gcTensors([a._id])
    assert list(a.toFloat32()) == [1, 2]
    from oracle.native import OracleError
    with pytest.raises(OracleError):
        b.toFloat32()


def test_view_copies_and_backward_restores_shape(orc):
    x = synth.normal(1, (2, 6))
    X = _t(orc, x, True)
    v = X.view(3, 4)
    assert v.shape == [3, 4] and np.array_equal(v.numpy().ravel(), x.ravel())
    v.mul(2.0).sum().backward()
    assert X.grad.shape == [2, 6] and np.all(X.grad.numpy() == 2)
