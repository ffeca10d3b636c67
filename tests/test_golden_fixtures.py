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
