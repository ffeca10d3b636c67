"""softmax and flash_attention on the GPU against the CPU oracle, through the
engine-level C ABI.  Tolerances: softmax outputs and attention weights live in
[0, 1] and are compared to 2e-6 absolute; attention outputs are convex
combinations of rows of v, compared to 1e-5 * max|v|; gradients are sums of s
products, compared to 1e-4 * sqrt(s) * (product of the operand maxima)."""
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


@pytest.mark.parametrize("shape,dim", [((2, 3), 1), ((64, 1000), 1), ((64, 1000), 0), ((3, 50, 7), 1), ((3, 50, 7), -1),
                                       ((5,), 0), ((2, 3, 4, 5), 2), ((1, 4097), 1)])
def test_softmax_forward_and_backward_match_the_oracle(both, shape, dim):
    gpu, cpu = both
    x = synth.normal(1, shape, 2.0)
    w = synth.normal(2, shape, stream=1)
    res = []
    for api in (gpu, cpu):
        X = _t(api, x, True)
        y = api.softmax(X, dim)
        y.mul(_t(api, w)).sum().backward()
        res.append((y.numpy(), X.grad.numpy()))
    assert max_err(res[0][0], res[1][0]) <= 2e-6
    assert max_err(res[0][1], res[1][1]) <= 1e-5 * float(np.abs(w).max())


def test_softmax_negative_dim_gradient_is_the_reference_one(both):
    # dim = -1 is saved as -1.0 and read back as 0 by the reference's backward
    gpu, cpu = both
    x, w = synth.normal(3, (6, 9)), synth.normal(4, (6, 9), stream=1)
    grads = []
    for api in (gpu, cpu):
        X = _t(api, x, True)
        api.softmax(X, -1).mul(_t(api, w)).sum().backward()
        grads.append(X.grad.numpy())
    assert max_err(grads[0], grads[1]) <= 1e-5
    x64 = x.astype(np.float64)
    s = np.exp(x64 - x64.max(1, keepdims=True))
    s /= s.sum(1, keepdims=True)
    assert max_err(grads[0], s * (w - (w * s).sum(0, keepdims=True))) <= 1e-5


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("bh,s,d", [(2, 4, 8), (3, 37, 20), (1, 1, 4), (4, 130, 64), (2, 1100, 16),
                                    # head dims of the one-kernel forward: key / query tails, one block, several blocks
                                    (2, 300, 32), (1, 257, 96), (2, 129, 128), (1, 31, 64), (3, 1, 32), (1, 640, 64),
                                    # around the edges of the two key halves of a 64-key tile (split forward)
                                    (2, 33, 32), (1, 64, 64), (2, 97, 64), (3, 32, 32)])
def test_attention_forward_and_backward_match_the_oracle(both, bh, s, d, causal):
    gpu, cpu = both
    q, k, v = (synth.normal(5, (bh, s, d), stream=i) for i in range(3))
    w = synth.normal(5, (bh, s, d), stream=4)
    scale = 1.0 / math.sqrt(d)
    res = []
    for api in (gpu, cpu):
        Q, K, V = _t(api, q, True), _t(api, k, True), _t(api, v, True)
        out = api.flashAttention(Q, K, V, scale, causal)
        assert out.shape == [bh, s, d]
        out.mul(_t(api, w)).sum().backward()
        res.append([out.numpy(), Q.grad.numpy(), K.grad.numpy(), V.grad.numpy()])
    mq, mk, mv, mw = (float(np.abs(a).max()) for a in (q, k, v, w))
    assert max_err(res[0][0], res[1][0]) <= 1e-5 * mv
    gtol = 1e-4 * math.sqrt(s)
    assert max_err(res[0][3], res[1][3]) <= gtol * mw                      # dv = P^T dO
    assert max_err(res[0][1], res[1][1]) <= gtol * mw * mv * mk * scale * 2  # dq = dS k
    assert max_err(res[0][2], res[1][2]) <= gtol * mw * mv * mq * scale * 2  # dk = dS^T q


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("bh,s,d", [(2, 4096, 64), (1, 3001, 128), (3, 1000, 32)])
def test_long_attention_forward_against_float64(rocm_native, bh, s, d, causal):
    """Sequences of thousands of positions through the one-kernel forward (dozens of key steps, query and key
    tails, every wavefront's diagonal) against a float64 softmax(q k^T) v."""
    rocm_native.resetEngine()
    gpu = bind(rocm_native)
    q, k, v = (synth.normal(9, (bh, s, d), stream=i) for i in range(3))
    scale = 1.0 / math.sqrt(d)
    got = gpu.flashAttention(_t(gpu, q), _t(gpu, k), _t(gpu, v), scale, causal).numpy()
    for b in range(bh):
        sc = (q[b].astype(np.float64) @ k[b].astype(np.float64).T) * scale
        if causal:
            sc = np.where(np.tri(s, dtype=bool), sc, -np.inf)
        p = np.exp(sc - sc.max(1, keepdims=True))
        want = (p / p.sum(1, keepdims=True)) @ v[b].astype(np.float64)
        assert max_err(got[b], want) <= 1e-5 * float(np.abs(v).max())


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("bh,s,d", [(2, 1500, 64), (1, 1031, 128), (2, 700, 32)])
def test_long_attention_backward_against_float64(rocm_native, bh, s, d, causal):
    """The two backward kernels over dozens of key / query steps against the closed form in float64:
    dV = P^T dO, dP = dO V^T, dS = P (dP - rowsum(dO O)) scale, dQ = dS K, dK = dS^T Q."""
    rocm_native.resetEngine()
    gpu = bind(rocm_native)
    q, k, v, w = (synth.normal(10, (bh, s, d), stream=i) for i in range(4))
    scale = 1.0 / math.sqrt(d)
    Q, K, V = (_t(gpu, a, True) for a in (q, k, v))
    gpu.flashAttention(Q, K, V, scale, causal).mul(_t(gpu, w)).sum().backward()
    got = [T.grad.numpy() for T in (Q, K, V)]
    for b in range(bh):
        q64, k64, v64, w64 = (a[b].astype(np.float64) for a in (q, k, v, w))
        sc = (q64 @ k64.T) * scale
        if causal:
            sc = np.where(np.tri(s, dtype=bool), sc, -np.inf)
        p = np.exp(sc - sc.max(1, keepdims=True))
        p /= p.sum(1, keepdims=True)
        o = p @ v64
        dp = w64 @ v64.T
        ds = p * (dp - (w64 * o).sum(1, keepdims=True)) * scale
        tol = 1e-4 * math.sqrt(s) * float(np.abs(w).max()) * float(np.abs(v).max())
        assert max_err(got[2][b], p.T @ w64) <= tol
        assert max_err(got[0][b], ds @ k64) <= tol * float(np.abs(k).max()) * scale * 2
        assert max_err(got[1][b], ds.T @ q64) <= tol * float(np.abs(q).max()) * scale * 2


@pytest.mark.parametrize("bh,s,d", [(75, 512, 32), (40, 1000, 64), (64, 1024, 32), (50, 1750, 32), (65, 512, 32), (9, 3800, 32),
                                    (70, 512, 96), (33, 1024, 128), (70, 1024, 64),
                                    # the last grids that still take the split forms: 511 blocks at 64, 256 at 128
                                    (73, 896, 64), (32, 1024, 128)])
def test_attention_grids_beyond_one_workgroup_per_cu_against_float64(rocm_native, bh, s, d):
    """More workgroups than the 256 CUs: the kernels then hand out the causal blocks in folded order (the
    lightest blocks as second workgroups of the CUs that hold the matching heavy ones), for grids of 300, 320,
    512, 700, 260 and 270 workgroups -- a partly filled second row, a full one, and a tail past it -- and for
    head dims 96 and 128, whose backward kernels fit one workgroup per CU and take the blocks in falling order.
    Below 512 blocks of 128 queries at head dims 32 and 64, and up to 256 at 96 and 128, all three kernels run
    in their split forms (64 queries or keys per workgroup, a tile shared between two wavefronts); the grids
    beyond take the unsplit ones.
    Every block must still be computed exactly once: forward and all three gradients against the closed form in
    float64."""
    rocm_native.resetEngine()
    gpu = bind(rocm_native)
    q, k, v, w = (synth.normal(11, (bh, s, d), stream=i) for i in range(4))
    scale = 1.0 / math.sqrt(d)
    Q, K, V = (_t(gpu, a, True) for a in (q, k, v))
    out = gpu.flashAttention(Q, K, V, scale, True)
    got_out = out.numpy()
    out.mul(_t(gpu, w)).sum().backward()
    got = [T.grad.numpy() for T in (Q, K, V)]
    tol = 1e-4 * math.sqrt(s) * float(np.abs(w).max()) * float(np.abs(v).max())
    mask = np.tri(s, dtype=bool)
    for b in range(bh):
        q64, k64, v64, w64 = (a[b].astype(np.float64) for a in (q, k, v, w))
        sc = np.where(mask, (q64 @ k64.T) * scale, -np.inf)
        p = np.exp(sc - sc.max(1, keepdims=True))
        p /= p.sum(1, keepdims=True)
        o = p @ v64
        assert max_err(got_out[b], o) <= 1e-5 * float(np.abs(v).max()), b
        dp = w64 @ v64.T
        ds = p * (dp - (w64 * o).sum(1, keepdims=True)) * scale
        assert max_err(got[2][b], p.T @ w64) <= tol, b
        assert max_err(got[0][b], ds @ k64) <= tol * float(np.abs(k).max()) * scale * 2, b
        assert max_err(got[1][b], ds.T @ q64) <= tol * float(np.abs(q).max()) * scale * 2, b


def test_attention_known_answers_on_the_gpu(both):
    gpu, _ = both
    bh, s, d = 2, 70, 8
    q, k = synth.normal(6, (bh, s, d)), synth.normal(6, (bh, s, d), stream=1)
    v = synth.normal(6, (bh, s, d), stream=2)
    ones = np.ones((bh, s, d), np.float32)
    assert max_err(gpu.flashAttention(_t(gpu, q), _t(gpu, k), _t(gpu, ones), 0.3, False).numpy(), ones) <= 2e-6
    out = gpu.flashAttention(_t(gpu, q), _t(gpu, k), _t(gpu, v), 0.3, True).numpy()
    assert max_err(out[:, 0, :], v[:, 0, :]) <= 1e-6
    zero = np.zeros_like(q)
    prefix = np.cumsum(v.astype(np.float64), axis=1) / np.arange(1, s + 1)[None, :, None]
    assert max_err(gpu.flashAttention(_t(gpu, zero), _t(gpu, k), _t(gpu, v), 0.3, True).numpy(), prefix) <= 1e-5


def test_attention_config3_shape_against_the_oracle(both):
    # batch 32, 512 x 64: the attention-score shapes of the measured configuration
    gpu, cpu = both
    bh, s, d = 32, 512, 64
    q, k = synth.normal(2, (bh, s, d)) / np.float32(8), synth.normal(2, (bh, s, d), stream=1) / np.float32(8)
    v = synth.normal(2, (bh, s, d), stream=2)
    w = synth.normal(2, (bh, s, d), stream=3)
    res = []
    for api in (gpu, cpu):
        Q, K, V = _t(api, q, True), _t(api, k, True), _t(api, v, True)
        out = api.flashAttention(Q, K, V, 0.125, True)
        out.mul(_t(api, w)).sum().backward()
        res.append([out.numpy(), Q.grad.numpy(), K.grad.numpy(), V.grad.numpy()])
    mq, mk, mv, mw = (float(np.abs(a).max()) for a in (q, k, v, w))
    assert max_err(res[0][0], res[1][0]) <= 1e-5 * mv
    gtol = 1e-4 * math.sqrt(s)
    assert max_err(res[0][3], res[1][3]) <= gtol * mw
    assert max_err(res[0][1], res[1][1]) <= gtol * mw * mv * mk * 0.125 * 2
    assert max_err(res[0][2], res[1][2]) <= gtol * mw * mv * mq * 0.125 * 2


def test_attention_misuse_is_an_error(rocm_native):
    from framework_amd import native as N
    T = rocm_native
    q = T.fromFloat32(np.zeros(8, np.float32), [2, 4])
    with pytest.raises(N.MniError, match="bh, s, d"):
        T.flashAttention(q, q, q, 1.0, True)
    q3 = T.fromFloat32(np.zeros(24, np.float32), [2, 3, 4])
    short = T.fromFloat32(np.zeros(12, np.float32), [1, 3, 4])
    with pytest.raises(N.MniError, match="fewer than"):
        T.flashAttention(q3, short, q3, 1.0, True)
    with pytest.raises(N.MniError, match="out of range"):
        T.softmaxOp(q3, 3)
    T.resetEngine()


def test_attention_golden_fixtures_on_the_gpu(rocm_native):
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_cases.json")) as f:
        g = json.load(f)
    api = bind(rocm_native)
    v = g["softmax_rows_123"]
    sm = api.softmax(api.Tensor.fromFloat32(v["input"], v["shape"]), v["dim"]).toFloat32()
    assert np.allclose(sm, v["out"], rtol=0, atol=2e-6)
    for c in g["cases"]:
        bh, s, d = c["bh"], c["s"], c["d"]
        q, k, vv, w = (synth.normal(c["seed"], (bh, s, d), 1.0, st) for st in range(4))
        Q, K, V = (_t(api, a, True) for a in (q, k, vv))
        out = api.flashAttention(Q, K, V, c["scale"], c["causal"])
        out.mul(_t(api, w)).sum().backward()
        mv, mw = float(np.abs(vv).max()), float(np.abs(w).max())
        assert max_err(out.numpy().ravel(), np.array(c["out"])) <= 1e-5 * mv
        for key, T in (("dq", Q), ("dk", K), ("dv", V)):
            assert max_err(T.grad.numpy().ravel(), np.array(c[key])) <= 1e-4 * math.sqrt(s) * mw * mv * 4, (c["seed"], key)
    rocm_native.resetEngine()


@pytest.mark.parametrize("shape", [(2, 4), (300, 257), (4096, 1024), (3, 50, 8), (7,)])
def test_bias_gelu_forward_and_backward_match_the_oracle(both, shape):
    gpu, cpu = both
    x = synth.normal(7, shape, 1.5)
    b = synth.normal(8, (shape[-1],), 1.0, stream=1)
    w = synth.normal(9, shape, 1.0, stream=2)
    res = []
    for api in (gpu, cpu):
        X, B = _t(api, x, True), _t(api, b, True)
        out = api.biasGelu(X, B)
        out.mul(_t(api, w)).sum().backward()
        res.append((out.numpy(), X.grad.numpy(), B.grad.numpy()))
    rows = int(np.prod(shape[:-1])) if len(shape) > 1 else 1
    mw = float(np.abs(w).max())
    assert max_err(res[0][0], res[1][0]) <= 1e-5 * float(np.abs(x).max() + np.abs(b).max())
    assert max_err(res[0][1], res[1][1]) <= 1e-5 * mw * 1.2
    assert max_err(res[0][2], res[1][2]) <= 1e-4 * math.sqrt(rows) * mw * 1.2  # column sums over `rows` terms


def test_fused_linear_gelu_equals_the_unfused_chain(both):
    # Linear(fused) with GELU = matmul, then bias + GELU in one pass; its backward
    # takes dGELU and the bias gradient in one pass.  Same values as matmul -> add -> gelu.
    gpu, cpu = both
    x = synth.normal(1, (130, 70))
    wt = synth.uniform(2, (70, 90), -0.2, 0.2, stream=1)
    b = synth.normal(3, (90,), 0.3, stream=2)
    r = synth.normal(4, (130, 90), 1.0, stream=3)
    grads = []
    for api, fused in ((gpu, True), (gpu, False), (cpu, False)):
        X, W, B = _t(api, x, True), _t(api, wt, True), _t(api, b, True)
        if fused:
            y = api.Tensor(api.native.linear(X._id, W._id, B._id, 3))
        else:
            y = X.matmul(W).add(B).gelu()
        y.mul(_t(api, r)).sum().backward()
        grads.append([y.numpy(), X.grad.numpy(), W.grad.numpy(), B.grad.numpy()])
    for other in (1, 2):
        assert max_err(grads[0][0], grads[other][0]) <= 1e-4 * math.sqrt(70) * 0.2 * 4
        assert max_err(grads[0][1], grads[other][1]) <= 1e-4 * math.sqrt(90) * 0.2 * 5
        assert max_err(grads[0][2], grads[other][2]) <= 1e-4 * math.sqrt(130) * 4 * 5
        assert max_err(grads[0][3], grads[other][3]) <= 1e-4 * math.sqrt(130) * 5
