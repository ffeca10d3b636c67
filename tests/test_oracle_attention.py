"""Pins the oracle's softmax and flash_attention (forward and backward) WITHOUT
a GPU: the reference's own softmax assertions (test/nn.test.ts:46-54), float64
closed forms, special cases with known answers, and finite differences."""
import math

import numpy as np
import pytest

from framework_amd import synth
from helpers import max_err


def _t(api, a, grad=False):
    a = np.asarray(a, dtype=np.float32)
    t = api.Tensor.fromFloat32(a, list(a.shape))
    return t.setRequiresGrad(True) if grad else t


def _softmax64(x, axis):
    x = x.astype(np.float64)
    e = np.exp(x - x.max(axis=axis, keepdims=True))
    return e / e.sum(axis=axis, keepdims=True)


def _attention64(q, k, v, scale, causal):
    q, k, v = (a.astype(np.float64) for a in (q, k, v))
    s = np.einsum("bid,bjd->bij", q, k) * scale
    if causal:
        n = s.shape[1]
        s = np.where(np.tril(np.ones((n, n), bool))[None], s, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    e = np.exp(s - m)
    z = e.sum(axis=-1, keepdims=True)
    return np.einsum("bij,bjd->bid", e / z, v), (m + np.log(z))[..., 0]


# ---- softmax ----------------------------------------------------------------

def test_softmax_reference_assertions(orc):
    sm = orc.softmax(_t(orc, [[1, 2, 3], [1, 2, 3]]), 1).toFloat32()  # nn.test.ts:46-54
    assert abs(sm[0] + sm[1] + sm[2] - 1.0) < 1e-4 and abs(sm[3] + sm[4] + sm[5] - 1.0) < 1e-4
    assert all(v > 0 for v in sm) and sm[2] > sm[1] > sm[0]
    want = [math.exp(i - 3) / (math.exp(-2) + math.exp(-1) + 1) for i in (1, 2, 3)]
    assert max_err(np.array(sm[:3]), np.array(want)) < 1e-7


@pytest.mark.parametrize("shape,dim", [((5, 7), 1), ((5, 7), 0), ((3, 4, 6), 1), ((3, 4, 6), -1), ((9,), 0), ((2, 3, 4, 5), 2)])
def test_softmax_vs_float64_and_shift_invariance(orc, shape, dim):
    x = synth.normal(1, shape, 3.0)
    got = orc.softmax(_t(orc, x), dim).numpy()
    assert max_err(got, _softmax64(x, dim)) < 2e-7
    shifted = orc.softmax(_t(orc, x + np.float32(100.0)), dim).numpy()
    assert max_err(shifted, got) < 2e-5  # x + c only changes the rounding of the inputs


@pytest.mark.parametrize("shape,dim", [((4, 6), 1), ((4, 6), 0), ((2, 5, 3), 1), ((2, 5, 3), 2)])
def test_softmax_backward_vs_float64_jacobian(orc, shape, dim):
    x = synth.normal(2, shape)
    w = synth.normal(3, shape, stream=1)
    X = _t(orc, x, True)
    orc.softmax(X, dim).mul(_t(orc, w)).sum().backward()
    s = _softmax64(x, dim)
    w64 = w.astype(np.float64)
    want = s * (w64 - (w64 * s).sum(axis=dim, keepdims=True))
    assert max_err(X.grad.numpy(), want) < 1e-6


def test_softmax_backward_of_a_negative_dim_follows_the_reference_cast(orc):
    # The tape stores `dim as f32` as passed and the backward reads it back with
    # `as usize`, which saturates -1.0 to 0 (ops/norm.rs:47, :98): for dim = -1
    # the reference's gradient is the dim-0 formula applied to the dim -1 output.
    x = synth.normal(4, (3, 5))
    w = synth.normal(5, (3, 5), stream=1)
    X = _t(orc, x, True)
    orc.softmax(X, -1).mul(_t(orc, w)).sum().backward()
    s = _softmax64(x, 1)
    w64 = w.astype(np.float64)
    as_reference = s * (w64 - (w64 * s).sum(axis=0, keepdims=True))
    as_intended = s * (w64 - (w64 * s).sum(axis=1, keepdims=True))
    got = X.grad.numpy()
    assert max_err(got, as_reference) < 1e-6
    assert max_err(got, as_intended) > 1e-3  # and the two really differ on this input
    # on a 1-D tensor the cast changes nothing
    v = synth.normal(6, (7,))
    V = _t(orc, v, True)
    orc.softmax(V, -1).mul(_t(orc, w[0, :1].repeat(7) * np.arange(7, dtype=np.float32))).sum().backward()
    s1 = _softmax64(v, 0)
    w1 = (w[0, :1].repeat(7) * np.arange(7, dtype=np.float32)).astype(np.float64)
    assert max_err(V.grad.numpy(), s1 * (w1 - (w1 * s1).sum())) < 1e-6


# ---- flash attention -----------------------------------------------------------

@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("bh,s,d", [(2, 4, 8), (3, 17, 5), (1, 1, 4), (2, 33, 16)])
def test_attention_forward_vs_float64(orc, bh, s, d, causal):
    q, k, v = (synth.normal(7, (bh, s, d), stream=i) for i in range(3))
    scale = 1.0 / math.sqrt(d)
    out = orc.flashAttention(_t(orc, q), _t(orc, k), _t(orc, v), scale, causal)
    assert out.shape == [bh, s, d]  # native.test.ts:19-23 checks only the shape
    want, _ = _attention64(q, k, v, scale, causal)
    assert max_err(out.numpy(), want) < 5e-6


def test_attention_special_cases_with_known_answers(orc):
    bh, s, d = 2, 6, 4
    q, k = synth.normal(8, (bh, s, d)), synth.normal(8, (bh, s, d), stream=1)
    v = synth.normal(8, (bh, s, d), stream=2)
    ones = np.ones((bh, s, d), np.float32)
    # the weights of a row sum to one: v = 1 gives exactly-one-ish outputs
    assert max_err(orc.flashAttention(_t(orc, q), _t(orc, k), _t(orc, ones), 0.5, False).numpy(), ones) < 1e-6
    # causal: row 0 sees only column 0
    out = orc.flashAttention(_t(orc, q), _t(orc, k), _t(orc, v), 0.5, True).numpy()
    assert max_err(out[:, 0, :], v[:, 0, :]) < 1e-6
    # equal scores (q = 0): plain mean of v, or of the causal prefix
    zero = np.zeros_like(q)
    out = orc.flashAttention(_t(orc, zero), _t(orc, k), _t(orc, v), 0.5, False).numpy()
    assert max_err(out, np.broadcast_to(v.astype(np.float64).mean(axis=1, keepdims=True), v.shape)) < 1e-6
    out = orc.flashAttention(_t(orc, zero), _t(orc, k), _t(orc, v), 0.5, True).numpy()
    prefix = np.cumsum(v.astype(np.float64), axis=1) / np.arange(1, s + 1)[None, :, None]
    assert max_err(out, prefix) < 1e-6
    # scale = 0 is the same thing
    out0 = orc.flashAttention(_t(orc, q), _t(orc, k), _t(orc, v), 0.0, True).numpy()
    assert max_err(out0, prefix) < 1e-6


@pytest.mark.parametrize("causal", [False, True])
def test_attention_backward_vs_float64_finite_differences(orc, causal):
    bh, s, d = 2, 5, 3
    q, k, v = (synth.normal(9, (bh, s, d), stream=i) for i in range(3))
    w = synth.normal(9, (bh, s, d), stream=5)
    scale = 0.7
    Q, K, V = _t(orc, q, True), _t(orc, k, True), _t(orc, v, True)
    orc.flashAttention(Q, K, V, scale, causal).mul(_t(orc, w)).sum().backward()

    def loss(q_, k_, v_):
        return float((_attention64(q_, k_, v_, scale, causal)[0] * w.astype(np.float64)).sum())

    eps = 1e-5
    for name, T, idx in (("q", Q, 0), ("k", K, 1), ("v", V, 2)):
        base = [q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)]
        fd = np.zeros((bh, s, d))
        for pos in np.ndindex(bh, s, d):
            hi = [a.copy() for a in base]
            lo = [a.copy() for a in base]
            hi[idx][pos] += eps
            lo[idx][pos] -= eps
            fd[pos] = (loss(*hi) - loss(*lo)) / (2 * eps)
        assert max_err(T.grad.numpy(), fd) < 2e-5, name


def test_attention_key_gradient_vanishes_for_constant_keys(orc):
    # With every key equal, the weights do not depend on q: dq = 0 exactly-ish,
    # and dv is the column sum of the (uniform) weights times dO.
    bh, s, d = 1, 4, 3
    q = synth.normal(10, (bh, s, d))
    k = np.broadcast_to(synth.normal(10, (bh, 1, d), stream=1), (bh, s, d)).copy()
    v = synth.normal(10, (bh, s, d), stream=2)
    Q, K, V = _t(orc, q, True), _t(orc, k, True), _t(orc, v, True)
    orc.flashAttention(Q, K, V, 1.0, False).sum().backward()
    assert max_err(Q.grad.numpy(), np.zeros((bh, s, d))) < 1e-6
    assert max_err(V.grad.numpy(), np.ones((bh, s, d))) < 1e-6  # each column gets s * (1/s)


# ---- fused bias + GELU (ops/fused.rs:247-273, 316-351) -------------------------

def _gelu64(z):
    return 0.5 * z * (1 + np.tanh(np.sqrt(2 / np.pi) * (z + 0.044715 * z ** 3)))


def _dgelu64(z):
    s = np.sqrt(2 / np.pi)
    th = np.tanh(s * (z + 0.044715 * z ** 3))
    return 0.5 * (1 + th) + 0.5 * z * (1 - th * th) * s * (1 + 3 * 0.044715 * z * z)


@pytest.mark.parametrize("shape", [(2, 4), (5, 7), (3, 4, 6), (9,)])
def test_bias_gelu_forward_vs_float64_and_composition(orc, shape):
    x = synth.normal(11, shape, 2.0)
    b = synth.normal(12, (shape[-1],), 1.0, stream=1)
    out = orc.biasGelu(_t(orc, x), _t(orc, b))
    assert out.shape == list(shape)  # test/native.test.ts:39-43 checks the shape only
    z = x.astype(np.float64) + b.astype(np.float64)
    assert max_err(out.numpy(), _gelu64(z)) < 1e-6
    composed = _t(orc, x).add(_t(orc, b)).gelu().numpy()  # the unfused path of the same oracle
    assert max_err(out.numpy(), composed) < 5e-7


def test_bias_gelu_backward_vs_float64_and_column_sums(orc):
    x = synth.normal(13, (6, 5), 1.5)
    b = synth.normal(14, (5,), 1.0, stream=1)
    w = synth.normal(15, (6, 5), 1.0, stream=2)
    X, B = _t(orc, x, True), _t(orc, b, True)
    orc.biasGelu(X, B).mul(_t(orc, w)).sum().backward()
    z = x.astype(np.float64) + b.astype(np.float64)
    dx = w.astype(np.float64) * _dgelu64(z)
    assert max_err(X.grad.numpy(), dx) < 1e-6
    assert max_err(B.grad.numpy(), dx.sum(axis=0)) < 1e-5
    # dbias is exactly the f32 column sum of dx taken down the rows
    got_dx = X.grad.numpy()
    col = np.zeros(5, np.float32)
    for r in range(6):
        col = col + got_dx[r]
    assert np.array_equal(B.grad.numpy(), col)
    # finite differences of the float64 closed form, as a check on the closed form itself
    eps = 1e-6
    fd = ((_gelu64(z + eps) - _gelu64(z - eps)) / (2 * eps)) * w
    assert max_err(dx, fd) < 1e-6
