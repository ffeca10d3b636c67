"""The committed golden fixtures against the CPU oracle (no GPU)."""
import json
import os

import numpy as np

from framework_amd import synth

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


def case_inputs(c):
    gen = (lambda s, sh, st: synth.small_ints(s, sh, 4, st)) if c["kind"] == "int" else (lambda s, sh, st: synth.normal(s, sh, 1.0, st))
    return gen(c["seed"], (c["m"], c["k"]), 0), gen(c["seed"], (c["k"], c["n"]), 1)


def test_reference_vectors_on_oracle(orc):
    ref = load("reference_vectors.json")
    T = orc.Tensor
    v = ref["matmul_2x2"]
    assert list(T.fromFloat32(v["a"], v["a_shape"]).matmul(T.fromFloat32(v["b"], v["b_shape"])).toFloat32()) == v["out"]
    v = ref["matmul_2x3_3x2"]
    out = T.fromFloat32(v["a"], v["a_shape"]).matmul(T.fromFloat32(v["b"], v["b_shape"]))
    assert out.shape == v["out_shape"] and out.toFloat32()[0] == v["out00"]
    v = ref["matmul_grad"]
    x = T.fromFloat32(v["x"], v["shape"]).setRequiresGrad(True)
    y = T.fromFloat32(v["y"], v["shape"]).setRequiresGrad(True)
    x.matmul(y).sum().backward()
    assert list(x.grad.toFloat32()) == v["dx"] and list(y.grad.toFloat32()) == v["dy"]
    v = ref["mse"]
    p = T.fromFloat32(v["pred"], v["shape"])
    assert orc.mseLoss(p, T.fromFloat32(v["target_same"], v["shape"])).toFloat32()[0] == v["loss_same"]
    assert abs(orc.mseLoss(p, T.fromFloat32(v["target_off1"], v["shape"])).toFloat32()[0] - v["loss_off1"]) < 1e-6


def test_matmul_cases_on_oracle(oracle_native):
    for c in load("matmul_cases.json")["cases"]:
        a, b = case_inputs(c)
        got = oracle_native.sgemm_ikj(a, b)
        assert np.array_equal(got.ravel(), np.array(c["out"], dtype=np.float32)), c["seed"]
        if c["kind"] == "int":  # exact in integers too
            assert np.array_equal(got, (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32))


def _attention_case(api, c):
    bh, s, d = c["bh"], c["s"], c["d"]
    q, k, v, w = (synth.normal(c["seed"], (bh, s, d), 1.0, st) for st in range(4))
    T = api.Tensor
    Q, K, V = (T.fromFloat32(a, [bh, s, d]).setRequiresGrad(True) for a in (q, k, v))
    out = api.flashAttention(Q, K, V, c["scale"], c["causal"])
    out.mul(T.fromFloat32(w, [bh, s, d])).sum().backward()
    return {"out": out.toFloat32(), "dq": Q.grad.toFloat32(), "dk": K.grad.toFloat32(), "dv": V.grad.toFloat32()}


def test_attention_fixtures_on_oracle(orc):
    g = load("attention_cases.json")
    v = g["softmax_rows_123"]
    sm = orc.softmax(orc.Tensor.fromFloat32(v["input"], v["shape"]), v["dim"]).toFloat32()
    assert np.allclose(sm, v["out"], rtol=0, atol=1e-7)
    assert abs(sum(v["out"][:3]) - 1.0) < 1e-6 and v["out"][2] > v["out"][1] > v["out"][0]  # test/nn.test.ts:51-54
    for c in g["cases"]:
        got = _attention_case(orc, c)
        for key in ("out", "dq", "dk", "dv"):  # libm's expf may differ in the last place between machines
            assert np.allclose(got[key], c[key], rtol=0, atol=2e-6), (c["seed"], key)
