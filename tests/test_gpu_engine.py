"""Engine-level parity: the same script runs on the HIP engine (through the
C ABI) and on the CPU oracle, and every output and gradient must agree within
the path's bound 1e-4 * sqrt(K) * max|a| * max|b| (bit for bit where the
arithmetic is exact)."""
import math

import numpy as np
import pytest

from framework_amd import native as N
from framework_amd import synth
from helpers import gemm_tol, max_err

pytestmark = pytest.mark.gpu


def T(api, a, grad=False):
    a = np.asarray(a, dtype=np.float32)
    t = api.Tensor.fromFloat32(a, list(a.shape))
    return t.setRequiresGrad(True) if grad else t


def both(gpu, orc, script):
    return script(gpu), script(orc)


def assert_close(got, want, tol, what=""):
    assert np.shape(got) == np.shape(want), what
    err = max_err(got, want)
    assert err <= tol, "%s: max err %g > tol %g" % (what, err, tol)


# ---- the reference suite's own assertions, on the GPU --------------------------------

def test_reference_matmul_vectors(gpu):
    Tn = gpu.Tensor
    mm = Tn.fromFloat32([1, 2, 3, 4], [2, 2]).matmul(Tn.fromFloat32([5, 6, 7, 8], [2, 2])).toFloat32()
    assert list(mm) == [19, 22, 43, 50]  # test/tensor.test.ts:222-228
    out = Tn.fromFloat32([1, 2, 3, 4, 5, 6], [2, 3]).matmul(Tn.fromFloat32([1, 2, 3, 4, 5, 6], [3, 2]))
    assert out.shape == [2, 2] and list(out.toFloat32()) == [22, 28, 49, 64]  # :230-235
    a = T(gpu, synth.uniform(1, (4, 3, 5)))
    b = T(gpu, synth.uniform(2, (4, 5, 2)))
    assert a.matmul(b).shape == [4, 3, 2]  # :237-240


def test_reference_autograd_and_losses(gpu):
    x = T(gpu, [[1, 0], [0, 1]], True)
    y = T(gpu, [[3, 4], [5, 6]], True)
    x.matmul(y).sum().backward()  # test/autograd.test.ts:42-46
    assert list(x.grad.toFloat32()) == [7, 11, 7, 11] and list(y.grad.toFloat32()) == [1, 1, 1, 1]
    a = T(gpu, [[1, 2], [3, 4]], True)
    b = T(gpu, [[5, 6], [7, 8]], True)
    a.mul(b).sum(0).sum(0).backward()  # :19-30
    assert list(a.grad.toFloat32()) == [5, 6, 7, 8]
    p = T(gpu, [[1, 2], [3, 4]])
    assert gpu.mseLoss(p, T(gpu, [[1, 2], [3, 4]])).toFloat32()[0] == 0  # test/nn.test.ts:78-86
    l = gpu.mseLoss(p, T(gpu, [[2, 3], [4, 5]]))
    assert l.shape == [2, 1] and abs(l.toFloat32()[0] - 1.0) < 1e-6
    lin = gpu.Linear(3, 2)
    assert lin.forward(T(gpu, synth.uniform(3, (4, 3)))).shape == [4, 2] and len(lin.parameters()) == 2  # :217-226
    assert list(T(gpu, [[1, 2, 3], [4, 5, 6]]).add(T(gpu, [10, 20, 30])).toFloat32()) == [11, 22, 33, 14, 25, 36]


def test_reference_regression_converges(gpu):
    # test/module.test.ts:113-130
    X = T(gpu, [[0], [1], [2], [3], [4], [5]])
    Y = T(gpu, [[1], [3], [5], [7], [9], [11]])
    net = gpu.Linear(1, 1, weight=synth.uniform(1, (1, 1), -1, 1), bias=synth.uniform(2, (1,), -1, 1))
    opt = gpu.Adam(net.parameters(), lr=0.05)
    early = None
    for i in range(200):
        opt.zeroGrad()
        loss = gpu.mseLoss(net.forward(X), Y)
        if i == 10:
            early = loss.toFloat32()[0]
        loss.backward()
        opt.step()
        gpu.native.gcTensors([X._id, Y._id] + [p.value._id for p in net.parameters()] +
                             [p.value.grad._id for p in net.parameters()])
    final = gpu.mseLoss(net.forward(X), Y).toFloat32()[0]
    assert final < early and final < 1.0


# ---- matmul forward / backward against the oracle ------------------------------------------

CASES = [
    ((5, 7), (7, 3)),
    ((64, 96), (96, 48)),
    ((130, 65), (65, 257)),
    ((4, 3, 5), (4, 5, 2)),
    ((3, 40, 24), (24, 56)),          # broadcast weight: dW summed over the batch (folded into K)
    ((40, 24), (3, 24, 56)),          # broadcast left operand
    ((2, 3, 16, 8), (2, 3, 8, 12)),
    ((2, 1, 6, 4), (1, 3, 4, 5)),     # the modulo batch rule
    ((2, 300), (300, 512)),           # skinny
    ((600, 32), (32, 3)),             # few output columns
    ((6, 2048), (2048, 4096)),        # a small batch under a wide layer: dA = dC B^T reads B K-contiguous, K = 4096 in slices
    ((3, 1024), (1024, 1280)),        # the same with a K of 1280: all of it per wavefront
]


@pytest.mark.parametrize("sa,sb", CASES)
def test_matmul_forward_backward_vs_oracle(gpu, orc, sa, sb):
    a = synth.normal(1, sa)
    b = synth.normal(2, sb, stream=1)

    def script(api):
        A, B = T(api, a, True), T(api, b, True)
        out = A.matmul(B)
        r = synth.normal(3, tuple(out.shape), stream=2)
        out.mul(T(api, r)).sum().backward()
        return {"out": out.numpy(), "ga": A.grad.numpy(), "gb": B.grad.numpy(), "r": r}

    g, o = both(gpu, orc, script)
    K = sa[-1]
    assert_close(g["out"], o["out"], gemm_tol(K, a, b), "forward")
    nbatch = int(np.prod(g["out"].shape[:-2])) if g["out"].ndim > 2 else 1
    assert_close(g["ga"], o["ga"], gemm_tol(sb[-1] * nbatch, g["r"], b), "dA")
    assert_close(g["gb"], o["gb"], gemm_tol(sa[-2] * nbatch, a, g["r"]), "dB")


def test_integer_inputs_are_bit_exact(gpu, orc):
    a = synth.small_ints(1, (3, 70, 50), 3)
    b = synth.small_ints(2, (50, 90), 3, stream=1)
    r = synth.small_ints(3, (3, 70, 90), 2, stream=2)

    def script(api):
        A, B = T(api, a, True), T(api, b, True)
        out = A.matmul(B)
        out.mul(T(api, r)).sum().backward()
        return out.numpy(), A.grad.numpy(), B.grad.numpy()

    g, o = both(gpu, orc, script)
    for x, y in zip(g, o):
        assert np.array_equal(x, y)


def test_permuted_and_non_collapsible_views(gpu, orc):
    x = synth.normal(1, (2, 6, 3, 8))  # [B, T, H, D]
    y = synth.normal(2, (2, 6, 3, 8), stream=1)

    def script(api):
        X, Y = T(api, x, True), T(api, y, True)
        q = X.permute(0, 2, 1, 3)            # [B, H, T, D]: batch dims do not collapse
        kt = Y.permute(0, 2, 3, 1)           # [B, H, D, T]
        s = q.matmul(kt)
        r = synth.normal(3, tuple(s.shape), stream=2)
        s.mul(T(api, r)).sum().backward()
        return {"s": s.numpy(), "gx": X.grad.numpy(), "gy": Y.grad.numpy(), "kt": kt.numpy()}

    g, o = both(gpu, orc, script)
    assert np.array_equal(g["kt"], o["kt"])
    for k in ("s", "gx", "gy"):
        assert_close(g[k], o[k], gemm_tol(8, x, y) * 4, k)


# ---- configuration 3: attention scores through a permuted view, full size -------------------

def test_config3_attention_scores(gpu, orc):
    q = synth.normal(2, (32, 512, 64)) / np.float32(8)
    k = synth.normal(2, (32, 512, 64), stream=1) / np.float32(8)
    ds = synth.normal(2, (32, 512, 512), stream=2)

    def script(api):
        Q, K = T(api, q, True), T(api, k, True)
        kt = K.permute(0, 2, 1)
        assert kt.shape == [32, 64, 512]
        s = Q.matmul(kt)
        # upstream gradient dS: loss = sum(S * dS)
        s.mul(T(api, ds)).sum().backward()
        return {"s": s.numpy(), "dq": Q.grad.numpy(), "dk": K.grad.numpy()}

    g, o = both(gpu, orc, script)
    assert_close(g["s"], o["s"], gemm_tol(64, q, k), "scores")
    assert_close(g["dq"], o["dq"], gemm_tol(512, ds, k), "dQ")
    assert_close(g["dk"], o["dk"], gemm_tol(512, ds, q), "dK")
    assert g["dk"].shape == (32, 512, 64)


# ---- Linear: composed, fused, and the bias gradient -----------------------------------------------

@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("xshape", [(32, 10), (3, 50, 64), (300, 128)])
def test_linear_forward_backward(gpu, orc, fused, xshape):
    fin, fout = xshape[-1], 96
    x = synth.normal(1, xshape)
    w = synth.uniform(2, (fin, fout), -1 / math.sqrt(fin), 1 / math.sqrt(fin))
    b = synth.uniform(3, (fout,), -1 / math.sqrt(fin), 1 / math.sqrt(fin))
    r = synth.normal(4, xshape[:-1] + (fout,), stream=2)

    def script(api, use_fused):
        lin = api.Linear(fin, fout, weight=w, bias=b, fused=use_fused)
        X = T(api, x, True)
        out = lin.forward(X)
        out.mul(T(api, r)).sum().backward()
        return {"out": out.numpy(), "gx": X.grad.numpy(), "gw": lin.weight.value.grad.numpy(),
                "gb": lin.bias.value.grad.numpy()}

    g = script(gpu, fused)
    o = script(orc, False)
    rows = int(np.prod(xshape[:-1]))
    assert_close(g["out"], o["out"], gemm_tol(fin, x, w), "out")
    assert_close(g["gx"], o["gx"], gemm_tol(fout, r, w), "dX")
    assert_close(g["gw"], o["gw"], gemm_tol(rows, x, r), "dW")
    assert_close(g["gb"], o["gb"], gemm_tol(rows, r, np.ones(1)), "db")


@pytest.mark.parametrize("act", [N.EPI_BIAS_RELU, N.EPI_BIAS_GELU])
def test_fused_linear_activation(gpu, orc, act):
    x = synth.normal(1, (70, 40))
    w = synth.uniform(2, (40, 56), -0.2, 0.2)
    b = synth.uniform(3, (56,), -0.2, 0.2)
    r = synth.normal(4, (70, 56), stream=2)
    X, W, B = T(gpu, x, True), T(gpu, w, True), T(gpu, b, True)
    out = gpu.Tensor(gpu.native.linear(X._id, W._id, B._id, act))
    out.mul(T(gpu, r)).sum().backward()
    Xo, Wo, Bo = T(orc, x, True), T(orc, w, True), T(orc, b, True)
    z = Xo.matmul(Wo).add(Bo)
    oo = z.relu() if act == N.EPI_BIAS_RELU else z.gelu()
    oo.mul(T(orc, r)).sum().backward()
    assert_close(out.numpy(), oo.numpy(), gemm_tol(40, x, w), "out")
    assert_close(X.grad.numpy(), Xo.grad.numpy(), gemm_tol(56, r, w) * 2, "dX")
    assert_close(W.grad.numpy(), Wo.grad.numpy(), gemm_tol(70, x, r) * 2, "dW")
    assert_close(B.grad.numpy(), Bo.grad.numpy(), gemm_tol(70, r, np.ones(1)) * 2, "db")


# ---- configuration 1: README MLP step (cross-entropy + Adam) ----------------------------------------

def test_config1_readme_mlp_step(gpu, orc):
    x = synth.uniform(0, (32, 10))
    w1 = synth.uniform(0, (10, 64), -1 / math.sqrt(10), 1 / math.sqrt(10), stream=1)
    b1 = synth.uniform(0, (64,), -1 / math.sqrt(10), 1 / math.sqrt(10), stream=2)
    w2 = synth.uniform(0, (64, 3), -1 / 8, 1 / 8, stream=3)
    b2 = synth.uniform(0, (3,), -1 / 8, 1 / 8, stream=4)
    targets = [[int(t)] for t in synth.integers(0, (32,), 0, 3, stream=5)]

    def script(api):
        l1 = api.Linear(10, 64, weight=w1, bias=b1)
        l2 = api.Linear(64, 3, weight=w2, bias=b2)
        params = l1.parameters() + l2.parameters()
        opt = api.Adam(params, lr=1e-3)
        out = {}
        for step in range(3):
            opt.zeroGrad()
            logits = l2.forward(l1.forward(T(api, x)).relu())
            loss = api.crossEntropyLoss(logits, targets)
            loss.backward()
            out["loss%d" % step] = loss.toFloat32().copy()
            if step == 0:
                out["logits"] = logits.numpy()
                out["grads"] = [p.value.grad.numpy() for p in params]
            out["norm%d" % step] = opt.step()
        out["params"] = [p.value.numpy() for p in params]
        return out

    g, o = both(gpu, orc, script)
    assert_close(g["logits"], o["logits"], 1e-5, "logits")
    for s in range(3):
        assert abs(g["loss%d" % s][0] - o["loss%d" % s][0]) <= 1e-5
        assert abs(g["norm%d" % s] - o["norm%d" % s]) <= 1e-5
    for gg, og in zip(g["grads"], o["grads"]):
        assert_close(gg, og, 1e-5, "grad")
    for gp, op in zip(g["params"], o["params"]):
        assert_close(gp, op, 1e-5, "param after 3 Adam steps")


# ---- configuration 4: FFN step (bias, GELU, reference mseLoss), reduced and full size -------------------

def ffn_inputs(rows, d, h):
    x = synth.normal(3, (rows, d))
    w1 = synth.uniform(3, (d, h), -1 / math.sqrt(d), 1 / math.sqrt(d), stream=1)
    w2 = synth.uniform(3, (h, d), -1 / math.sqrt(h), 1 / math.sqrt(h), stream=2)
    t = synth.normal(3, (rows, d), stream=3)
    return x, w1, w2, t


def ffn_script(api, x, w1, w2, t, fused=False, fused_gelu=False, b1=None, fused_mse=False):
    """fused: each Linear is one product with a bias epilogue.  fused_gelu: the first Linear also carries
    its GELU (two outputs from one epilogue), and in the backward the second Linear's product hands dX
    straight through gelu' to the first (no pre-activation tensor is visible then: hpre is None)."""
    d, h = w1.shape
    b1 = np.zeros(h, np.float32) if b1 is None else b1
    l1 = api.Linear(d, h, weight=w1, bias=b1, fused=fused or fused_gelu, activation="gelu" if fused_gelu else None)
    l2 = api.Linear(h, d, weight=w2, bias=np.zeros(d, np.float32), fused=fused or fused_gelu)
    X = T(api, x, True)
    hpre = None if fused_gelu else l1.forward(X)
    hact = l1.forward(X) if fused_gelu else hpre.gelu()
    y = l2.forward(hact)
    loss = api.mseLoss(y, T(api, t), fused=True) if fused_mse else api.mseLoss(y, T(api, t))
    loss.backward()
    return {"hpre": hpre, "hact": hact, "y": y, "loss": loss, "X": X, "l1": l1, "l2": l2}


def test_config4_ffn_step_reduced_vs_oracle(gpu, orc):
    x, w1, w2, t = ffn_inputs(256, 128, 512)
    b1 = synth.uniform(3, (512,), -0.3, 0.3, stream=4)   # the benchmark's bias is zero; a non-zero one exercises z + b
    for fused, fused_gelu, bias1, fused_mse in ((False, False, None, False), (True, False, None, False), (True, True, None, False), (True, True, b1, False),
                                                (True, True, b1, True)):
        gpu.native.resetEngine()
        orc.native.resetEngine()
        g = ffn_script(gpu, x, w1, w2, t, fused, fused_gelu, bias1, fused_mse)
        o = ffn_script(orc, x, w1, w2, t, b1=bias1)
        assert g["loss"].shape == [256, 1]
        assert_close(g["y"].numpy(), o["y"].numpy(), gemm_tol(512, o["hact"].numpy(), w2), "y")
        assert_close(g["loss"].numpy(), o["loss"].numpy(), 1e-4, "loss")
        dy = 2 * (o["y"].numpy() - t) / 128
        assert_close(g["l2"].weight.value.grad.numpy(), o["l2"].weight.value.grad.numpy(), gemm_tol(256, o["hact"].numpy(), dy), "dW2")
        assert_close(g["l2"].bias.value.grad.numpy(), o["l2"].bias.value.grad.numpy(), gemm_tol(256, dy, np.ones(1)), "db2")
        dh = dy.astype(np.float64) @ w2.T.astype(np.float64)
        assert_close(g["l1"].weight.value.grad.numpy(), o["l1"].weight.value.grad.numpy(), gemm_tol(256, x, dh) * 2, "dW1")
        assert_close(g["l1"].bias.value.grad.numpy(), o["l1"].bias.value.grad.numpy(), gemm_tol(256, dh, np.ones(1)) * 2, "db1")
        assert_close(g["X"].grad.numpy(), o["X"].grad.numpy(), gemm_tol(512, dh, w1) * 2, "dX")


@pytest.mark.parametrize("fused_gelu", [False, True])
def test_config4_ffn_step_full_size_relations(gpu, fused_gelu):
    # X[4096,1024] -> 4096 -> 1024: too slow for the scalar oracle, so every
    # product of the step is checked on sampled rows/columns in float64 from
    # the tensors the GPU itself produced.  fused_gelu: the step the benchmark
    # times as "fused" (GELU and its backward inside the products' epilogues).
    x, w1, w2, t = ffn_inputs(4096, 1024, 4096)
    g = ffn_script(gpu, x, w1, w2, t, fused_gelu, fused_gelu, fused_mse=fused_gelu)
    hact, y = g["hact"].numpy(), g["y"].numpy()
    rows = np.array([0, 1, 2047, 4095])
    x64, w164, w264 = x.astype(np.float64), w1.astype(np.float64), w2.astype(np.float64)
    gelu = lambda v: 0.5 * v * (1 + np.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3)))
    if fused_gelu:
        # the pre-activation never leaves the engine: take it in float64 where it is needed
        class Pre:
            def __getitem__(self, idx):
                r, c = idx if isinstance(idx, tuple) else (idx, slice(None))
                return (x64[r] @ w164[:, c]).astype(np.float64)
        hpre = Pre()
        assert_close(hact[rows], gelu(hpre[rows]), gemm_tol(1024, x, w1), "gelu(X W1)")
    else:
        hpre = g["hpre"].numpy()
        assert_close(hpre[rows], x64[rows] @ w164, gemm_tol(1024, x, w1), "X W1")
        assert_close(hact[rows], gelu(hpre[rows].astype(np.float64)), 1e-5, "gelu")
    assert_close(y[rows], hact[rows].astype(np.float64) @ w264, gemm_tol(4096, hact, w2), "H W2")
    loss = g["loss"].numpy()
    assert loss.shape == (4096, 1)
    assert_close(loss[rows, 0], ((y[rows].astype(np.float64) - t[rows]) ** 2).mean(1), 1e-4, "mseLoss rows")
    dy = 2 * (y.astype(np.float64) - t) / 1024
    cols = np.array([0, 5, 1023])
    gw2 = g["l2"].weight.value.grad.numpy()
    assert_close(gw2[:, cols], hact.astype(np.float64).T @ dy[:, cols], gemm_tol(4096, hact, dy), "dW2 = H^T dY")
    assert_close(g["l2"].bias.value.grad.numpy(), dy.sum(0), gemm_tol(4096, dy, np.ones(1)), "db2")
    dh_rows = dy[rows] @ w264.T
    gelu_grad_rows = np.zeros_like(dh_rows)
    v = hpre[rows].astype(np.float64)
    s = math.sqrt(2 / math.pi)
    th = np.tanh(s * (v + 0.044715 * v ** 3))
    gelu_grad_rows = 0.5 * (1 + th) + 0.5 * v * (1 - th * th) * s * (1 + 3 * 0.044715 * v * v)
    dz_rows = dh_rows * gelu_grad_rows
    assert_close(g["X"].grad.numpy()[rows], dz_rows @ w164.T, gemm_tol(4096, dz_rows, w1) * 2, "dX = dZ W1^T")
    gw1 = g["l1"].weight.value.grad.numpy()
    assert gw1.shape == (1024, 4096) and np.isfinite(gw1).all()
    # dW1[:, c] = X^T dZ[:, c] needs dZ for all rows at a few columns
    hc = np.array([0, 7, 4095])
    dh_cols = dy @ w264[hc].T
    vc = hpre[:, hc].astype(np.float64)
    thc = np.tanh(s * (vc + 0.044715 * vc ** 3))
    dz_cols = dh_cols * (0.5 * (1 + thc) + 0.5 * vc * (1 - thc * thc) * s * (1 + 3 * 0.044715 * vc * vc))
    assert_close(gw1[:, hc], x64.T @ dz_cols, gemm_tol(4096, x, dz_cols) * 2, "dW1 = X^T dZ")
    assert_close(g["l1"].bias.value.grad.numpy()[hc], dz_cols.sum(0), gemm_tol(4096, dz_cols, np.ones(1)) * 2, "db1")


@pytest.mark.parametrize("shape", [(256, 128), (7, 33), (3, 5, 40), (1, 1), (64, 4096)])
def test_fused_mse_loss_is_the_composition_in_one_pass(gpu, orc, shape):
    # forward: one mean of squared differences per row of the last dim, shape [..., 1] like the composition's two
    # mean(-1) calls; backward: the composition's own arithmetic ((g / dim) d + (g / dim) d), so the same bits
    p, t = synth.normal(11, shape), synth.normal(12, shape, stream=1)
    up = synth.normal(13, shape[:-1] + (1,), stream=2)
    res = {}
    for name, api, fused in (("fused", gpu, True), ("composed", gpu, False), ("oracle", orc, False)):
        api.native.resetEngine()
        P, Tt = T(api, p, True), T(api, t, True)
        loss = api.mseLoss(P, Tt, fused=True) if fused else api.mseLoss(P, Tt)
        loss.mul(T(api, up)).backward()  # (a different upstream gradient for every row)
        res[name] = (loss.shape, loss.numpy(), P.grad.numpy(), Tt.grad.numpy())
    assert res["fused"][0] == res["composed"][0] == list(shape[:-1]) + [1]
    assert_close(res["fused"][1], res["oracle"][1], 1e-5 * max(1.0, float(np.abs(res["oracle"][1]).max())), "loss")
    assert_close(res["fused"][1], res["composed"][1], 1e-5 * max(1.0, float(np.abs(res["oracle"][1]).max())), "loss vs composed")
    assert np.array_equal(res["fused"][2], res["composed"][2]) and np.array_equal(res["fused"][3], res["composed"][3])
    assert_close(res["fused"][2], res["oracle"][2], 1e-6 * max(1.0, float(np.abs(res["oracle"][2]).max())), "dpred")
    assert np.array_equal(res["fused"][3], -res["fused"][2])


@pytest.mark.parametrize("shape", [(256, 128), (7, 33), (1, 5), (4096, 1024)])
def test_fused_mse_loss_rooted_backward_takes_the_gradient_the_forward_pass_left(gpu, shape):
    # backward() rooted at the loss starts from ones: the forward pass has already written the gradient for that case,
    # with the arithmetic of the backward kernel, so the bits are those of the composition and nothing is launched for
    # it; a target that wants a gradient, or a second use of the loss, takes the backward kernel
    p, t = synth.normal(31, shape), synth.normal(32, shape, stream=1)
    res = {}
    for fused in (True, False):
        gpu.native.resetEngine()
        P = T(gpu, p, True)
        loss = gpu.mseLoss(P, T(gpu, t), fused=True) if fused else gpu.mseLoss(P, T(gpu, t))
        before = int(gpu.native.lib.mni_rocm_launch_count())
        loss.backward()
        res[fused] = (P.grad.numpy(), int(gpu.native.lib.mni_rocm_launch_count()) - before)
    assert np.array_equal(res[True][0], res[False][0])
    assert_close(res[True][0], 2 * (p.astype(np.float64) - t) / shape[-1], 1e-6 * max(1.0, float(np.abs(p - t).max())), "dpred")
    assert res[True][1] <= 1   # (at most the fill of a seed of a new size)
    gpu.native.resetEngine()
    P, Tt = T(gpu, p, True), T(gpu, t, True)
    gpu.mseLoss(P, Tt, fused=True).backward()
    assert np.array_equal(P.grad.numpy(), res[False][0]) and np.array_equal(Tt.grad.numpy(), -res[False][0])
    gpu.native.resetEngine()
    gpu.native.noGradStart()
    try:
        loss = gpu.mseLoss(T(gpu, p), T(gpu, t), fused=True)
    finally:
        gpu.native.noGradEnd()
    assert_close(loss.numpy(), ((p.astype(np.float64) - t) ** 2).mean(-1, keepdims=True), 1e-5, "loss without a tape")


def test_fused_mse_loss_views_plain_targets_and_errors(gpu):
    # a permuted prediction is gathered first; a target that asks for no gradient gets none; shapes must be equal
    p, t = synth.normal(21, (40, 24)), synth.normal(22, (24, 40), stream=1)
    P, Tt = T(gpu, p, True), T(gpu, t)
    loss = gpu.mseLoss(P.permute(1, 0), Tt, fused=True)
    loss.backward()
    want = ((p.T.astype(np.float64) - t) ** 2).mean(1, keepdims=True)
    assert_close(loss.numpy(), want, 1e-5, "loss of a permuted view")
    assert_close(P.grad.numpy(), (2 * (p.T.astype(np.float64) - t) / 40).T, 1e-6, "gradient through the view")
    assert Tt.grad is None
    with pytest.raises(Exception, match="same non-empty shape"):
        gpu.native.mseLoss(P._id, T(gpu, synth.normal(23, (24,)))._id)
    # broadcasting keeps the composition
    l2 = gpu.mseLoss(T(gpu, t), T(gpu, t[0]), fused=True)
    assert l2.shape == [24, 1]


# ---- configuration 5 through the engine ------------------------------------------------------------------

def test_config5a_through_engine(gpu):
    x = synth.normal(4, (4, 4096), 0.02)
    w = synth.normal(4, (4096, 4096), 0.02, stream=1)
    out = T(gpu, x).matmul(T(gpu, w)).numpy()
    assert_close(out, x.astype(np.float64) @ w.astype(np.float64), gemm_tol(4096, x, w), "x W")


def test_config5b_weight_gradient_through_matmul_backward(gpu, orc):
    # reduced K for the oracle; the full-size kernel is covered in test_gpu_sgemm.py
    x = synth.normal(5, (8192, 96))
    w = synth.normal(5, (96, 64), stream=1)
    dy = synth.normal(5, (8192, 64), stream=2)

    def script(api):
        X, W = T(api, x), T(api, w, True)
        X.matmul(W).mul(T(api, dy)).sum().backward()
        return W.grad.numpy()

    g, o = both(gpu, orc, script)
    assert_close(g, o, gemm_tol(8192, x, dy), "dW = X^T dY")


# ---- store / tape behaviour ---------------------------------------------------------------------------------

def test_views_keep_their_values_when_the_parameter_is_updated(gpu):
    w = T(gpu, [[1, 2, 3], [4, 5, 6]], True)
    v = w.permute(1, 0)  # shares w's buffer
    w.mul(w).sum().backward()
    gpu.Adam([gpu.Parameter(w)], lr=0.5).step()
    assert list(v.toFloat32()) == [1, 4, 2, 5, 3, 6]      # the reference's permute cloned the data
    assert not np.array_equal(w.toFloat32(), [1, 2, 3, 4, 5, 6])


def test_grad_accumulation_zero_grad_no_grad(gpu):
    x = T(gpu, [1, 2], True)
    x.mul(2.0).sum().backward()
    x.mul(2.0).sum().backward()
    assert list(x.grad.toFloat32()) == [4, 4]
    gpu.native.zeroGrad([x._id])
    assert list(x.grad.toFloat32()) == [0, 0]
    gpu.native.noGradStart()
    x.mul(3.0).sum().backward()
    z = x.mul(5.0).sum()  # backward re-enabled the tape (lib.rs:135)
    z.backward()
    assert list(x.grad.toFloat32()) == [5, 5]


def test_same_tensor_twice_and_non_scalar_seed(gpu):
    d = T(gpu, [[1, -2], [3, 4]], True)
    d.mul(d).sum().backward()
    assert list(d.grad.toFloat32()) == [2, -4, 6, 8]
    x = T(gpu, [[1, 2], [3, 4]], True)
    x.mul(3.0).backward()
    assert list(x.grad.toFloat32()) == [3, 3, 3, 3]


def test_id_recycling_free_and_gc(gpu):
    Tn = gpu.Tensor
    a, b, c = Tn.ones([1]), Tn.ones([1]), Tn.ones([1])
    b.free()
    c.free()
    assert Tn.ones([1])._id == c._id and Tn.ones([1])._id == b._id  # LIFO, tensor.rs:104-113
    keep = T(gpu, [1, 2])
    drop = T(gpu, [3, 4])
    gpu.native.gcTensors([keep._id])
    assert list(keep.toFloat32()) == [1, 2]
    with pytest.raises(N.MniError, match="already freed"):
        drop.toFloat32()


def test_unbroadcast_patterns_vs_oracle(gpu, orc):
    g = synth.normal(11, (2, 3, 4), stream=7)
    for shape in ([4], [3, 1], [1, 3, 4], [2, 1, 4], [1]):
        def script(api):
            a = T(api, np.zeros((2, 3, 4)), True)
            b = T(api, np.zeros(shape), True)
            a.sub(b).mul(T(api, g)).sum().backward()
            return b.grad.numpy()
        x, y = both(gpu, orc, script)
        assert_close(x, y, 1e-5, str(shape))


@pytest.mark.parametrize("full,small", [((512, 2048), (512, 1)), ((16, 256, 96), (1, 256, 1)), ((4, 1 << 18), (4, 1)),
                                        ((8, 6, 128, 128), (8, 1, 1, 128)), ((8, 6, 128, 128), (1, 6, 1, 1)), ((3, 70, 5000), (70, 1)),
                                        ((2, 300, 40), (2, 1, 40))])
def test_unbroadcast_of_few_outputs_under_many_values(gpu, orc, full, small):
    # utils::unbroadcast (src/native/src/utils.rs:39-66) where the operand's gradient has few elements, each the sum
    # of many: one reduced axis after the other (row sums of a matrix, a mask broadcast over heads and queries, ...),
    # not one thread per output.  Against float64; against the oracle too where it is quick.
    x, y, w = synth.normal(1, full), synth.normal(2, small, stream=1), synth.normal(3, full, stream=2)
    X, Y = T(gpu, x, True), T(gpu, y, True)
    X.mul(Y).mul(T(gpu, w)).sum().backward()
    nd = len(full)
    al = (1,) * (nd - len(small)) + tuple(small)
    axes = tuple(i for i in range(nd) if al[i] == 1 and full[i] != 1)
    want = (x.astype(np.float64) * w.astype(np.float64)).sum(axis=axes, keepdims=True).reshape(small)
    nred = int(np.prod([full[i] for i in axes]))
    assert max_err(Y.grad.numpy(), want) <= 1e-5 * math.sqrt(nred) * float(np.abs(x).max()) * float(np.abs(w).max())
    if int(np.prod(full)) <= 1 << 20:
        def script(api):
            a, b = T(api, x, True), T(api, y, True)
            a.mul(b).mul(T(api, w)).sum().backward()
            return b.grad.numpy()
        assert_close(script(gpu), script(orc), 1e-5 * math.sqrt(nred) * 16, str(small))


def test_scalar_and_bias_gradients_of_large_tensors_vs_oracle(gpu, orc):
    # a broadcast operand's gradient is a sum over every element of a [3000, 1024] tensor (3.07M rows of one
    # column: more row blocks than one grid axis holds), and over its 3000 rows for a [1024] operand
    x = synth.normal(21, (3000, 1024))
    g = synth.normal(22, (3000, 1024), stream=1)

    def script(api):
        a = T(api, x, True)
        c, d, e = T(api, np.array([1.0]), True), T(api, np.zeros(1024), True), T(api, np.full((1, 1), 0.5), True)
        a.add(c).sub(d).mul(e).mul(T(api, g)).sum().backward()
        return [c.grad.numpy(), d.grad.numpy(), e.grad.numpy(), a.grad.numpy()]
    for (got, want), k in zip(zip(*both(gpu, orc, script)), (3072000, 3000, 3072000, 1)):
        assert got.shape == want.shape
        # the oracle adds in flat order in float32; bound both against the float64 sum
        tol = 1e-4 * np.sqrt(k) * 4.0 * 5.0
        assert max_err(got, want) <= tol


def test_reductions_views_and_activations_vs_oracle(gpu, orc):
    x = synth.normal(1, (3, 5, 300))

    def script(api):
        X = T(api, x, True)
        out = {"sum0": X.sum(0).numpy(), "mean1": X.mean(1).numpy(), "meanl": X.mean(-1).numpy(),
               "relu": X.relu().numpy(), "gelu": X.gelu().numpy(), "view": X.permute(2, 0, 1).view(300, 15).numpy()}
        X.permute(1, 0, 2).gelu().mean(-1).sum().backward()
        out["grad"] = X.grad.numpy()
        return out

    g, o = both(gpu, orc, script)
    for k in g:
        assert_close(g[k], o[k], 2e-5, k)
    assert np.array_equal(g["relu"], o["relu"]) and np.array_equal(g["view"], o["view"])


def test_errors_where_the_reference_panics(gpu):
    Tn = gpu.Tensor
    with pytest.raises(N.MniError, match="at least 2D"):
        Tn.ones([2]).matmul(Tn.ones([2]))
    with pytest.raises(N.MniError, match="inner dimensions"):
        Tn.ones([2, 3]).matmul(Tn.ones([4, 2]))
    with pytest.raises(N.MniError, match="broadcastable"):
        Tn.ones([2, 2, 3]).matmul(Tn.ones([3, 3, 2]))
    with pytest.raises(N.MniError, match="broadcastable"):
        Tn.ones([2, 3]).add(Tn.ones([4]))
    other = Tn.ones([2, 2])
    t = Tn.ones([2, 2])
    t.free()
    with pytest.raises(N.MniError, match="already freed"):
        t.matmul(other)
    with pytest.raises(N.MniError, match="out of range"):
        gpu.crossEntropyLoss(Tn.ones([2, 3]), [[0], [3]])


def test_entry_points_serialise_concurrent_callers(rocm_native):
    # The reference funnels every export through one mutex (src/native/src/lib.rs:27-39);
    # ctypes drops the GIL during a call, so these threads really do race into the library.
    import threading
    T = rocm_native
    errors = []

    def worker(seed):
        try:
            for it in range(40):
                a = synth.small_ints(seed + it, (17, 9), 3)
                b = synth.small_ints(seed + it, (9, 23), 3, stream=1)
                ia, ib = T.fromFloat32(a.ravel(), [17, 9]), T.fromFloat32(b.ravel(), [9, 23])
                ic = T.matmul(ia, ib)
                got = np.asarray(T.toFloat32(ic)).reshape(17, 23)
                if not np.array_equal(got, (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)):
                    errors.append((seed, it))
                for i in (ia, ib, ic):
                    T.freeTensor(i)
        except Exception as e:  # noqa: BLE001 - reported through the assertion below
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(100 * k,)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert errors == []


@pytest.mark.parametrize("sizes", [[5], [640, 64, 192, 3], [4096 * 16], [4096 * 16 + 1], [100000, 7], [33] * 49, [4096] * 16 + [1]])
def test_grad_norm_small_models_in_one_launch_and_large_ones_in_two(gpu, sizes):
    # up to sixteen 4096-value chunks of gradients are summed by one workgroup in one launch; beyond that (or with more
    # tensors than one launch's table holds) by a launch of partial sums and one that adds them.  Either way the
    # norm reaches the host through pinned memory; the value is checked against float64.
    Tn = gpu.Tensor
    ws, want = [], 0.0
    for i, n in enumerate(sizes):
        x = synth.normal(n + i, (n,), stream=i)
        w = Tn.fromFloat32(np.zeros(n, np.float32), [n]).setRequiresGrad(True)
        w.mul(Tn.fromFloat32(x, [n])).sum().backward()
        ws.append(w)
        want += float(np.sum(x.astype(np.float64) ** 2))
    ids = [w._id for w in ws]
    got = gpu.native.gradNorm(ids)
    assert abs(got - np.sqrt(want)) <= 2e-7 * np.sqrt(want)
    assert gpu.native.gradNorm(ids) == got          # the same sums in the same order
    # a step without clipping returns the same norm (its update is queued before the host looks at the norm) and
    # moves every parameter by lr (Adam's first step is lr * g / (|g| + eps))
    opt = gpu.Adam([gpu.Parameter(w) for w in ws], lr=0.01)
    assert opt.step() == got
    assert all(np.mean(np.abs(w.numpy()) > 0.009) > 0.999 for w in ws)
    # with clipping: the norm is read first, the gradients are scaled to the limit, then the update
    assert opt.step(maxGradNorm=got / 4) == got
    assert abs(gpu.native.gradNorm(ids) - got / 4) <= 1e-6 * got


def test_cleared_gradients_read_as_zeros_and_accumulate_from_zero(gpu):
    # zeroGrad only marks a gradient; the zeros appear when it is read, and the first accumulation replaces them
    Tn = gpu.Tensor
    w = Tn.fromFloat32(np.arange(6, dtype=np.float32).reshape(2, 3), [2, 3]).setRequiresGrad(True)
    u = Tn.fromFloat32(np.ones((2, 3), np.float32), [2, 3]).setRequiresGrad(True)
    x = Tn.fromFloat32(np.array([[1, 2, 3], [4, 5, 6]], np.float32), [2, 3])
    w.mul(x).sum().backward()
    assert np.array_equal(w.grad.numpy(), x.numpy()) and u.grad is None
    gpu.native.zeroGrad([w._id, u._id])
    assert not np.any(w.grad.numpy())                                    # read before any accumulation: zeros
    gview = w.grad.permute(1, 0)                                         # a view of the cleared gradient
    w.mul(x).sum().backward()
    w.mul(x).sum().backward()                                            # second accumulation adds
    assert np.array_equal(w.grad.numpy(), 2 * x.numpy())
    assert not np.any(gview.numpy())                                     # the view kept the zeros it was taken from
    gpu.native.zeroGrad([w._id])
    gpu.native.zeroGrad([w._id])                                         # twice in a row
    assert gpu.native.gradNorm([w._id, u._id]) == 0.0                    # a reader other than toFloat32
    w.mul(x).sum().backward()
    assert np.array_equal(w.grad.numpy(), x.numpy())
    # a gradient shared with the tape's tensor is not corrupted by scaling it in place afterwards
    gpu.native.zeroGrad([w._id])
    loss = w.mul(x).sum()
    loss.backward()
    assert gpu.native.scaleGrads([w._id], 0.5) is False
    assert np.array_equal(w.grad.numpy(), 0.5 * x.numpy()) and np.array_equal(x.numpy(), np.array([[1, 2, 3], [4, 5, 6]], np.float32))
    # an optimiser step on a parameter whose gradient stayed cleared leaves it alone (zero gradient, zero moments)
    opt = gpu.Adam([gpu.Parameter(w), gpu.Parameter(u)], lr=0.1)
    before = u.numpy().copy()
    opt.zeroGrad()
    w.mul(x).sum().backward()
    opt.step()
    assert np.array_equal(u.numpy(), before) and not np.array_equal(w.numpy(), np.arange(6, dtype=np.float32).reshape(2, 3))
