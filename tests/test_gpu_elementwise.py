"""exp / log / sigmoid / pow / div / comparisons / max / layernorm on the GPU
against the CPU oracle through the engine-level C ABI.  Transcendentals may
differ from glibc's by a few ulp, hence relative tolerances of 2e-6 on values;
comparisons, max and division are exact."""
import math

import numpy as np
import pytest

from framework_amd import synth
from framework_amd.api import bind
from helpers import max_err

pytestmark = pytest.mark.gpu


def _t(api, a, grad=False):
    a = np.asarray(a, dtype=np.float32)
    t = api.Tensor.fromFloat32(a, list(a.shape))
    return t.setRequiresGrad(True) if grad else t


@pytest.fixture()
def both(rocm_native, oracle_native):
    gpu, cpu = bind(rocm_native), bind(oracle_native)
    yield gpu, cpu
    rocm_native.resetEngine()
    oracle_native.resetEngine()


def test_reference_assertions_on_the_gpu(both):
    gpu, _ = both
    a, b = _t(gpu, [1, 2, 3]), _t(gpu, [4, 5, 6])
    assert list(_t(gpu, [6, 10, 15]).div(_t(gpu, [2, 5, 3])).toFloat32()) == [3, 2, 5]      # test/tensor.test.ts:84-87
    assert max_err(a.pow(2).numpy(), np.array([1, 4, 9])) < 1e-4                             # :92-95
    assert all(v == 1 for v in a.lt(b).toFloat32()) and all(v == 0 for v in a.lt(a).toFloat32())
    assert all(v == 1 for v in b.gt(a).toFloat32()) and all(v == 1 for v in a.eq(a).toFloat32())
    assert all(v == 0 for v in a.eq(b).toFloat32()) and all(v == 1 for v in a.isClose(a).toFloat32())
    assert all(v == 1 for v in a.isClose(_t(gpu, [1.000001, 2.000001, 3.000001]), 1e-4).toFloat32())
    e = _t(gpu, [0, 1, 2]).exp().toFloat32()
    assert abs(e[0] - 1) < 1e-4 and abs(e[1] - math.e) < 1e-4 and abs(e[2] - math.e ** 2) < 1e-3
    sg = _t(gpu, [0, 100, -100]).sigmoid().toFloat32()
    assert abs(sg[0] - 0.5) < 1e-4 and abs(sg[1] - 1) < 1e-2 and abs(sg[2]) < 1e-2
    mat = _t(gpu, [[1, 2, 3], [4, 5, 6]])
    assert list(mat.max(1).toFloat32()) == [3, 6] and list(mat.max(0).toFloat32()) == [4, 5, 6]  # :180-187
    x = _t(gpu, [3], True)
    x.pow(2).backward()
    assert abs(x.grad.toFloat32()[0] - 6) < 1e-3                                              # test/autograd.test.ts:10-16
    ln = gpu.layerNorm(_t(gpu, [[1, 2, 3], [4, 5, 6]]), gpu.Tensor.ones([3]), gpu.Tensor.zeros([3])).toFloat32()
    assert abs(sum(ln[:3]) / 3) < 1e-3 and abs(sum(ln[3:]) / 3) < 1e-3                        # test/nn.test.ts:94-105


@pytest.mark.parametrize("shape", [(7,), (300, 257), (4, 5, 64)])
def test_unary_math_matches_the_oracle(both, shape):
    gpu, cpu = both
    x = synth.uniform(1, shape, 0.2, 3.0)
    w = synth.normal(2, shape, stream=1)
    fns = {"exp": lambda t: t.exp(), "log": lambda t: t.log(), "sigmoid": lambda t: t.sigmoid(),
           "pow2.5": lambda t: t.pow(2.5), "pow-1": lambda t: t.pow(-1.0), "pow2": lambda t: t.pow(2.0)}
    for name, fn in fns.items():
        res = []
        for api in (gpu, cpu):
            X = _t(api, x, True)
            y = fn(X)
            y.mul(_t(api, w)).sum().backward()
            res.append((y.numpy(), X.grad.numpy()))
        assert max_err(res[0][0], res[1][0]) <= 2e-6 * max(1.0, float(np.abs(res[1][0]).max())), name
        assert max_err(res[0][1], res[1][1]) <= 4e-6 * max(1.0, float(np.abs(res[1][1]).max())), name


def test_div_and_comparisons_match_the_oracle_exactly(both):
    gpu, cpu = both
    a = synth.normal(3, (40, 1, 50))
    b = synth.uniform(4, (30, 50), 0.5, 2.0, stream=1)
    w = synth.normal(5, (40, 30, 50), stream=2)
    res = []
    for api in (gpu, cpu):
        A, B = _t(api, a, True), _t(api, b, True)
        q = A.div(B)
        q.mul(_t(api, w)).sum().backward()
        res.append((q.numpy(), A.grad.numpy(), B.grad.numpy()))
    assert np.array_equal(res[0][0], res[1][0])  # one correctly rounded division per element
    assert max_err(res[0][1], res[1][1]) <= 1e-4 * math.sqrt(30) * 2 * float(np.abs(w).max())
    assert max_err(res[0][2], res[1][2]) <= 1e-4 * math.sqrt(40) * 4 * float(np.abs(w).max() * np.abs(a).max())
    c = synth.small_ints(6, (40, 30, 50), 2)
    d = synth.small_ints(7, (30, 50), 2, stream=1)
    for name in ("lt", "gt", "eq"):
        assert np.array_equal(getattr(_t(gpu, c), name)(_t(gpu, d)).numpy(), getattr(_t(cpu, c), name)(_t(cpu, d)).numpy())
    assert np.array_equal(_t(gpu, c).isClose(_t(gpu, d), 1.5).numpy(), (np.abs(c - d) < 1.5).astype(np.float32))
    # same-shape fast path and a permuted (non-contiguous) operand
    e = synth.normal(8, (64, 48))
    f = synth.uniform(9, (48, 64), 0.5, 2.0, stream=1)
    got = _t(gpu, e).div(_t(gpu, f).permute(1, 0)).numpy()
    assert np.array_equal(got, e / f.T)


@pytest.mark.parametrize("shape,dim", [((5, 7), 1), ((5, 7), 0), ((3, 40, 6), 1), ((3, 4, 600), -1), ((2000,), 0)])
def test_max_matches_the_oracle_exactly(both, shape, dim):
    gpu, cpu = both
    x = synth.small_ints(8, shape, 3)  # many ties: every one of them receives the gradient
    wshape = tuple(1 if i == (dim % len(shape)) else s for i, s in enumerate(shape))
    w = synth.normal(9, wshape, stream=1)
    res = []
    for api in (gpu, cpu):
        X = _t(api, x, True)
        m = X.max(dim)
        m.mul(_t(api, w)).sum().backward()
        res.append((m.numpy(), X.grad.numpy()))
    assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1], res[1][1])
    assert np.array_equal(res[0][0], x.max(axis=dim, keepdims=True))


@pytest.mark.parametrize("shape", [(1 << 22,), (8, 1 << 18), (3, 32768 + 5), (2048, 2048), (2, 50000, 7), (100000, 3), (1, 33000), (300, 40), (8, 16384), (5, 9000)])
def test_sums_and_means_over_long_axes_and_of_whole_tensors(both, shape):
    # sum / mean (src/native/src/ops/reduce.rs:13-46,169-184) where the reduced axis is long and the outputs few: a
    # row of millions is summed chunk by chunk over the whole device, the column sums of a tall matrix in two passes
    # (a wavefront per row, or a thread per output, took 58 ms for one row of 16 M elements).  Against float64; the
    # oracle too where it is quick.
    gpu, cpu = both
    a = synth.normal(sum(shape), shape)
    a64 = a.astype(np.float64)
    t = _t(gpu, a)
    for dim in (None, -1, 0):
        for mean in (False, True):
            got = (t.mean() if mean else t.sum()) if dim is None else (t.mean(dim) if mean else t.sum(dim))
            want = (a64.mean(keepdims=True) if mean else a64.sum(keepdims=True)) if dim is None else \
                   (a64.mean(dim, keepdims=True) if mean else a64.sum(dim, keepdims=True))
            nred = a.size / want.size
            tol = 1e-5 * math.sqrt(nred) * float(np.abs(a).max()) / (nred if mean else 1.0) + 1e-7
            assert list(got.shape) == list(want.shape), (dim, mean)
            assert max_err(got.numpy(), want) <= tol, (dim, mean)
    if a.size <= 1 << 19:
        tc = _t(cpu, a)
        for dim in (-1, 0):
            assert max_err(t.sum(dim).numpy(), tc.sum(dim).numpy()) <= 1e-5 * math.sqrt(a.size) * float(np.abs(a).max())
    # backward of a whole-tensor mean: every element gets 1 / n
    X = _t(gpu, a, True)
    X.mean().backward()
    assert np.allclose(X.grad.numpy(), 1.0 / a.size, rtol=1e-6, atol=0)


@pytest.mark.parametrize("shape,dim", [((4, 1 << 18), -1), ((1, 1 << 20), -1), ((2048, 2048), 0), ((1 << 18, 4), 0), ((2, 3, 1 << 16), -1),
                                       ((2, 40000, 5), 1), ((3, 32768 + 5), 1), ((8, 16384), 1), ((5, 9000), -1)])
def test_max_over_a_long_axis_under_few_outputs_is_exact(gpu, shape, dim):
    # taken in two levels (chunks of a long row, blocks of a tall matrix): a maximum is exact whatever the order
    a = synth.normal(sum(shape), shape)
    assert np.array_equal(_t(gpu, a).max(dim).numpy(), a.max(axis=dim, keepdims=True))


@pytest.mark.parametrize("shape", [(8, 50304), (5, 50257), (3, 70000), (100000, 4), (5000, 13), (300, 4096), (64, 8192), (7, 1030)])
def test_softmax_and_cross_entropy_over_long_and_short_lines(both, shape):
    # softmax over the last axis (src/native/src/ops/reduce.rs softmax) and the cross-entropy on top of it
    # (src/native/src/ops/loss.rs:24-67) for lines of vocabulary length under a handful of rows (a workgroup per
    # line; a wavefront per line took 624 us for 8 x 50304), lines held in registers, and lines of a few values
    # (a thread per line).  Against float64, and against the oracle where it is quick.
    gpu, cpu = both
    a = synth.normal(shape[0] + shape[1], shape, 3.0)
    a64 = a.astype(np.float64)
    e = np.exp(a64 - a64.max(-1, keepdims=True))
    want = e / e.sum(-1, keepdims=True)
    got = gpu.softmax(_t(gpu, a), -1).numpy()
    assert max_err(got, want) <= 2e-6
    assert np.abs(got.astype(np.float64).sum(-1) - 1.0).max() <= 1e-4
    if shape[0] <= 5000:   # its gradient: p * (w - sum(p * w)) per line (the axis given as 1: the reference reads -1 back as 0)
        w = synth.normal(3, shape, stream=2)
        X = _t(gpu, a, True)
        gpu.softmax(X, 1).mul(_t(gpu, w)).sum().backward()
        w64 = w.astype(np.float64)
        assert max_err(X.grad.numpy(), want * (w64 - (want * w64).sum(-1, keepdims=True))) <= 1e-5 * float(np.abs(w).max())
    if shape[0] <= 5000:
        targets = [int(t) for t in (np.arange(shape[0]) * 7919) % shape[1]]
        want_loss = float(np.mean(-np.log(want[np.arange(shape[0]), targets])))
        L = _t(gpu, a, True)
        loss = gpu.crossEntropyLoss(L, targets)
        assert abs(float(loss.numpy().ravel()[0]) - want_loss) <= 1e-5 * max(1.0, abs(want_loss))
        loss.backward()
        onehot = np.zeros(shape); onehot[np.arange(shape[0]), targets] = 1.0
        assert max_err(L.grad.numpy(), (want - onehot) / shape[0]) <= 2e-6
        if a.size <= 1 << 19:
            Lc = _t(cpu, a, True)
            assert abs(float(cpu.crossEntropyLoss(Lc, targets).numpy().ravel()[0]) - float(loss.numpy().ravel()[0])) <= 1e-5 * max(1.0, abs(want_loss))


def test_layernorm_backward_of_more_rows_than_one_grid_axis_of_row_blocks(gpu):
    # 1.2 M rows of 8: the column sums for gamma and beta run over more 16-row blocks than the second grid axis holds,
    # so a block takes more rows; checked against float64 (the oracle would need minutes)
    rows, c = 1_200_000, 8
    x = synth.normal(20, (rows, c), 2.0)
    g = synth.uniform(21, (c,), 0.5, 1.5, stream=1)
    b = synth.normal(22, (c,), stream=2)
    w = synth.normal(23, (rows, c), stream=3)
    X, G, B = _t(gpu, x, True), _t(gpu, g, True), _t(gpu, b, True)
    gpu.layerNorm(X, G, B, 1e-5).mul(_t(gpu, w)).sum().backward()
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    xhat = (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-5)
    assert max_err(G.grad.numpy(), (w64 * xhat).sum(0)) <= 1e-4 * math.sqrt(rows) * float(np.abs(w).max()) * 3
    assert max_err(B.grad.numpy(), w64.sum(0)) <= 1e-4 * math.sqrt(rows) * float(np.abs(w).max())


@pytest.mark.parametrize("shape", [(2, 3), (64, 768), (4, 33, 100), (5000, 16), (8, 4096), (3, 1024), (2, 8192), (5, 2052), (2, 8196), (3, 16384), (2, 16388)])
def test_layernorm_matches_the_oracle(both, shape):
    gpu, cpu = both
    c = shape[-1]
    rows = int(np.prod(shape[:-1]))
    x = synth.normal(10, shape, 2.0)
    g = synth.uniform(11, (c,), 0.5, 1.5, stream=1)
    b = synth.normal(12, (c,), stream=2)
    w = synth.normal(13, shape, stream=3)
    res = []
    for api in (gpu, cpu):
        X, G, B = _t(api, x, True), _t(api, g, True), _t(api, b, True)
        y = api.layerNorm(X, G, B, 1e-5)
        y.mul(_t(api, w)).sum().backward()
        res.append((y.numpy(), X.grad.numpy(), G.grad.numpy(), B.grad.numpy()))
    mw = float(np.abs(w).max())
    assert max_err(res[0][0], res[1][0]) <= 1e-5 * float(np.abs(res[1][0]).max())
    assert max_err(res[0][1], res[1][1]) <= 2e-5 * max(1.0, float(np.abs(res[1][1]).max()))
    assert max_err(res[0][2], res[1][2]) <= 1e-4 * math.sqrt(rows) * mw * 6   # column sums over `rows` terms of g * xhat
    assert max_err(res[0][3], res[1][3]) <= 1e-4 * math.sqrt(rows) * mw
