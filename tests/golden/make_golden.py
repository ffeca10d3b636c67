"""Writes the golden fixtures of this directory.

    python tests/golden/make_golden.py

* reference_vectors.json -- the matmul values the reference's own test suite
  holds (test/tensor.test.ts:222-240, test/autograd.test.ts:42-46,
  test/nn.test.ts:78-86), typed in from those files: data, not code.
* matmul_cases.json -- small seeded cases (inputs are regenerated from the
  seed by framework_amd.synth; expected outputs computed by the CPU oracle),
  including integer-valued cases whose result is exact in any summation order.
* config_samples.json -- for each benchmark configuration, sampled rows of the
  full-size product computed by the CPU oracle's i-k-j loop: per row the f64
  sum, the f64 sum of squares and the first 8 values.

* attention_cases.json -- the reference's softmax assertion input
  (test/nn.test.ts:46-54) and small seeded flash_attention cases: outputs and
  the gradients of sum(w * out), computed by the CPU oracle
  (`python tests/golden/make_golden.py attention` writes only this file).

Nothing here executes reference code; the oracle is this repository's own C
restatement (oracle/mni_oracle.c).
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from framework_amd import synth  # noqa: E402
from oracle.native import OracleNative  # noqa: E402


def dump(name, obj):
    with open(os.path.join(HERE, name), "w") as f:
        json.dump(obj, f, indent=1)
    print("wrote", name)


def row_stats(rows):
    return [{"sum": float(np.sum(r.astype(np.float64))), "sumsq": float(np.sum(r.astype(np.float64) ** 2)),
             "head": [float(x) for x in r[:8]]} for r in rows]


def attention_cases(orc):
    from framework_amd.api import bind
    api = bind(orc)
    T = api.Tensor
    sm = api.softmax(T.fromFloat32(np.array([1, 2, 3, 1, 2, 3], np.float32), [2, 3]), 1).toFloat32()
    cases = []
    for i, (bh, s, d, causal) in enumerate([(2, 4, 8, True), (1, 7, 3, False), (2, 19, 8, True)]):
        seed = 200 + i
        q, k, v, w = (synth.normal(seed, (bh, s, d), 1.0, st) for st in range(4))
        scale = 1.0 / float(np.sqrt(d))
        Q, K, V = (T.fromFloat32(a, [bh, s, d]).setRequiresGrad(True) for a in (q, k, v))
        out = api.flashAttention(Q, K, V, scale, causal)
        out.mul(T.fromFloat32(w, [bh, s, d])).sum().backward()
        cases.append({"bh": bh, "s": s, "d": d, "causal": causal, "scale": scale, "seed": seed,
                      "out": [float(x) for x in out.toFloat32()], "dq": [float(x) for x in Q.grad.toFloat32()],
                      "dk": [float(x) for x in K.grad.toFloat32()], "dv": [float(x) for x in V.grad.toFloat32()]})
        orc.resetEngine()
    dump("attention_cases.json", {
        "softmax_rows_123": {"input": [1, 2, 3, 1, 2, 3], "shape": [2, 3], "dim": 1, "out": [float(x) for x in sm],
                             "source": "input of test/nn.test.ts:46-54; values from the oracle"},
        "generator": "framework_amd.synth.normal(seed, (bh, s, d), 1, stream): q, k, v, w = streams 0..3; loss = sum(w * out)",
        "cases": cases})


def main():
    orc = OracleNative()
    if sys.argv[1:] == ["attention"]:
        attention_cases(orc)
        return
    attention_cases(orc)

    dump("reference_vectors.json", {
        "matmul_2x2": {"a": [1, 2, 3, 4], "a_shape": [2, 2], "b": [5, 6, 7, 8], "b_shape": [2, 2],
                       "out": [19, 22, 43, 50], "source": "test/tensor.test.ts:222-228"},
        "matmul_2x3_3x2": {"a": [1, 2, 3, 4, 5, 6], "a_shape": [2, 3], "b": [1, 2, 3, 4, 5, 6], "b_shape": [3, 2],
                           "out_shape": [2, 2], "out00": 22, "source": "test/tensor.test.ts:230-235"},
        "batched_shape": {"a_shape": [4, 3, 5], "b_shape": [4, 5, 2], "out_shape": [4, 3, 2],
                          "source": "test/tensor.test.ts:237-240"},
        "matmul_grad": {"x": [1, 0, 0, 1], "y": [3, 4, 5, 6], "shape": [2, 2], "dx": [7, 11, 7, 11],
                        "dy": [1, 1, 1, 1], "source": "test/autograd.test.ts:42-46 (values derived: G = ones)"},
        "mse": {"pred": [1, 2, 3, 4], "target_same": [1, 2, 3, 4], "target_off1": [2, 3, 4, 5], "shape": [2, 2],
                "loss_same": 0.0, "loss_off1": 1.0, "source": "test/nn.test.ts:78-86"},
        "linear_shape": {"in": 3, "out": 2, "x_shape": [4, 3], "out_shape": [4, 2], "n_params": 2,
                         "source": "test/nn.test.ts:217-226"},
    })

    cases = []
    for i, (m, n, k, kind) in enumerate([(1, 1, 1, "int"), (3, 5, 7, "int"), (17, 63, 65, "int"), (33, 31, 130, "int"),
                                         (8, 8, 64, "normal"), (5, 40, 19, "normal"), (64, 48, 96, "normal")]):
        seed = 100 + i
        gen = (lambda s, sh, st: synth.small_ints(s, sh, 4, st)) if kind == "int" else (lambda s, sh, st: synth.normal(s, sh, 1.0, st))
        a, b = gen(seed, (m, k), 0), gen(seed, (k, n), 1)
        out = orc.sgemm_ikj(a, b)
        cases.append({"m": m, "n": n, "k": k, "kind": kind, "seed": seed, "out": [float(x) for x in out.ravel()]})
    dump("matmul_cases.json", {"generator": "framework_amd.synth: small_ints(seed, shape, 4, stream) or normal(seed, shape, 1, stream); A stream 0, B stream 1",
                              "cases": cases})

    samples = {}
    # config 2: A[4096,4096] B[4096,4096] ~ N(0,1), seed 1
    a = synth.normal(1, (4096, 4096)); b = synth.normal(1, (4096, 4096), stream=1)
    rows = [0, 1, 127, 128, 2047, 4095]
    samples["config2"] = {"rows": rows, "stats": row_stats(orc.sgemm_ikj(a[rows], b))}
    # config 5a: x[4,4096] W[4096,4096] ~ N(0, 0.02), seed 4
    x = synth.normal(4, (4, 4096), 0.02); w = synth.normal(4, (4096, 4096), 0.02, stream=1)
    samples["config5a"] = {"rows": [0, 1, 2, 3], "stats": row_stats(orc.sgemm_ikj(x, w))}
    # config 5b: X[65536,1024]^T dY[65536,1024] ~ N(0,1), seed 5: sampled rows of X^T
    X = synth.normal(5, (65536, 1024)); dY = synth.normal(5, (65536, 1024), stream=1)
    rows = [0, 1, 511, 1023]
    samples["config5b"] = {"rows": rows, "stats": row_stats(orc.sgemm_ikj(np.ascontiguousarray(X[:, rows].T), dY))}
    dump("config_samples.json", samples)


if __name__ == "__main__":
    main()
