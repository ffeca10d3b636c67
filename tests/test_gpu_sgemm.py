"""Kernel-level parity of mni_rocm_sgemm (through the C ABI) with the CPU
oracle's i-k-j loop.  Integer-valued inputs must match bit for bit (any
summation order is exact), normal inputs within
1e-4 * sqrt(K) * max|a| * max|b|."""
import json
import os

import numpy as np
import pytest

from framework_amd import native as N
from framework_amd import synth
from helpers import gemm_tol, max_err

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


class Dev:
    """Device buffers freed at the end of a test."""

    def __init__(self, r):
        self.r, self.ptrs = r, []

    def put(self, a):
        p = self.r.to_device(a)
        self.ptrs.append(p)
        return p

    def empty(self, n, fill=None):
        p = self.r.malloc(max(n, 1) * 4)
        self.ptrs.append(p)
        if fill is not None:
            self.r.fill(p, fill, n)
        return p

    def close(self):
        for p in self.ptrs:
            self.r.free(p)


@pytest.fixture()
def dev(rocm):
    d = Dev(rocm)
    yield d
    d.close()


def run_gemm(dev, a, b, ta=False, tb=False, **kw):
    """a, b are the arrays as stored; op(A) = a.T when ta."""
    r = dev.r
    batch = a.shape[0] if a.ndim == 3 else 1
    a3 = a.reshape((batch,) + a.shape[-2:])
    b3 = b.reshape((-1,) + b.shape[-2:])
    M, K = (a3.shape[2], a3.shape[1]) if ta else (a3.shape[1], a3.shape[2])
    Nn = b3.shape[1] if tb else b3.shape[2]
    batch = max(a3.shape[0], b3.shape[0])
    dA, dB = dev.put(a3), dev.put(b3)
    dC = dev.empty(batch * M * Nn, fill=-7.0)
    r.sgemm(M, Nn, K, dA, dB, dC, batch=batch,
            a_strides=(1, a3.shape[2]) if ta else (a3.shape[2], 1),
            b_strides=(1, b3.shape[2]) if tb else (b3.shape[2], 1),
            a_batch=(a3.shape[1] * a3.shape[2], a3.shape[0]), b_batch=(b3.shape[1] * b3.shape[2], b3.shape[0]), **kw)
    return r.to_host(dC, (batch, M, Nn))


SHAPES = [(1, 1, 1), (3, 5, 7), (17, 63, 65), (64, 64, 16), (128, 128, 32), (129, 127, 33), (256, 384, 160), (1000, 300, 200)]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_mfma_integer_exact_all_layouts(dev, m, n, k, ta, tb):
    a = synth.small_ints(m + k, (k, m) if ta else (m, k), 4)
    b = synth.small_ints(n + k, (n, k) if tb else (k, n), 4, stream=1)
    got = run_gemm(dev, a, b, ta, tb, algo=N.ALGO_MFMA)[0]
    want = ((a.T if ta else a).astype(np.int64) @ (b.T if tb else b).astype(np.int64)).astype(np.float32)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("m,n,k", [(300, 50, 200), (50, 300, 200), (256, 384, 160), (512, 512, 64)])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("algo", [N.ALGO_MFMA, N.ALGO_MFMA_SMALL])
def test_mfma_tile_shapes_integer_exact(dev, m, n, k, ta, tb, algo):
    # 128x64 / 64x128 tiles (an extent <= 64), forced 64x64 tiles, short K
    a = synth.small_ints(m + k, (k, m) if ta else (m, k), 4)
    b = synth.small_ints(n + k, (n, k) if tb else (k, n), 4, stream=1)
    got = run_gemm(dev, a, b, ta, tb, algo=algo)[0]
    want = ((a.T if ta else a).astype(np.int64) @ (b.T if tb else b).astype(np.int64)).astype(np.float32)
    assert np.array_equal(got, want)
    got = run_gemm(dev, a, b, ta, tb, algo=algo, split_k=2)[0]
    assert np.array_equal(got, want)


@pytest.mark.parametrize("m,n,k", [(64, 48, 96), (300, 200, 1000), (512, 512, 512)])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_mfma_normal_inputs_vs_oracle(dev, oracle_native, m, n, k, ta, tb):
    a = synth.normal(m, (k, m) if ta else (m, k))
    b = synth.normal(n, (n, k) if tb else (k, n), stream=1)
    got = run_gemm(dev, a, b, ta, tb, algo=N.ALGO_MFMA)[0]
    want = oracle_native.sgemm_ikj(a.T if ta else a, b.T if tb else b)
    assert max_err(got, want) <= gemm_tol(k, a, b)


@pytest.mark.parametrize("m,n,k,lda,ldb", [
    (1004, 300, 200, 200, 300),    # both edges on a multiple of 4: fast loads, rows beyond the edge re-read
    (1001, 302, 200, 200, 320),    # B is a view into wider rows, its edge (46 columns) is not a multiple of 4
    (1002, 300, 203, 208, 300),    # K tail inside padded rows of A
    (1000, 1004, 517, 520, 1004),  # long enough for the steady K loop before the tail
])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_edge_tiles_in_padded_buffers(dev, m, n, k, lda, ldb, ta, tb):
    """Edge tiles and K tails of operands that sit in wider (16-byte aligned) rows: the extent is smaller than the
    leading dimension, so the 16-byte load paths are eligible and have to stop at the edge by themselves.  The
    padding holds a large value that must not leak into the result."""
    r = dev.r
    # op(A) is m x k; stored k x m (leading dimension padded) when ta
    ea, eb = (k, m) if ta else (m, k), (n, k) if tb else (k, n)
    pa = lda if not ta else ((m + 3) // 4 * 4 + 4)
    pb = ldb if not tb else ((k + 3) // 4 * 4 + 4)
    a = np.full((ea[0], pa), 1e30, dtype=np.float32)
    b = np.full((eb[0], pb), 1e30, dtype=np.float32)
    a[:, :ea[1]] = synth.small_ints(m + k, ea, 4)
    b[:, :eb[1]] = synth.small_ints(n + k, eb, 4, stream=1)
    dA, dB = dev.put(a), dev.put(b)
    dC = dev.empty(m * n, fill=-7.0)
    want = ((a[:, :ea[1]].T if ta else a[:, :ea[1]]).astype(np.int64) @ (b[:, :eb[1]].T if tb else b[:, :eb[1]]).astype(np.int64)).astype(np.float32)
    for algo in (N.ALGO_AUTO, N.ALGO_MFMA, N.ALGO_MFMA_SMALL):
        r.fill(dC, -7.0, m * n)
        r.sgemm(m, n, k, dA, dB, dC, a_strides=(1, pa) if ta else (pa, 1), b_strides=(1, pb) if tb else (pb, 1), algo=algo)
        assert np.array_equal(r.to_host(dC, (m, n)), want), algo


@pytest.mark.parametrize("ld", [4194300, 4194308])
@pytest.mark.parametrize("ta", [False, True])
def test_row_pitches_at_the_limit_of_32_bit_byte_offsets(dev, rocm, ld, ta):
    """The steady K loop addresses a tile through 32-bit byte offsets from the tile's base (buffer loads); a
    128-row tile side at a pitch of 2^22 floats is where they stop fitting.  Just below the limit the offsets
    reach 2.13e9; just above it the tile takes the loop with 64-bit addresses (64-row tiles still fit).  A sits
    in rows of `ld` floats (16 MiB apart), everything between the rows is never touched."""
    m, n, k = 130, 70, 96
    rows = k if ta else m            # stored rows of A
    a = synth.small_ints(ld % 97, (rows, m if ta else k), 4)
    b = synth.small_ints(5, (k, n), 4, stream=1)
    dA = rocm.malloc(rows * ld * 4)
    try:
        for i in range(rows):
            rocm._check(rocm.lib.mni_rocm_h2d(dA + i * ld * 4, a[i].ctypes.data, a[i].nbytes))
        dB, dC = dev.put(b), dev.empty(m * n)
        want = ((a.T if ta else a).astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
        for algo in (N.ALGO_MFMA, N.ALGO_MFMA_SMALL, N.ALGO_AUTO):
            rocm.fill(dC, -7.0, m * n)
            rocm.sgemm(m, n, k, dA, dB, dC, a_strides=(1, ld) if ta else (ld, 1), algo=algo)
            assert np.array_equal(rocm.to_host(dC, (m, n)), want), algo
    finally:
        rocm.free(dA)


@pytest.mark.parametrize("m,n,k", [(257, 259, 261), (1000, 1001, 515)])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_odd_leading_dimensions_and_offset_bases(dev, m, n, k, ta, tb):
    """Rows that start on no 16-byte boundary (odd leading dimensions; operands that begin one, two or three floats
    into their allocation) still take the 16-byte load paths; the result must not change."""
    r = dev.r
    a = synth.small_ints(m + k, (k, m) if ta else (m, k), 4)
    b = synth.small_ints(n + k, (n, k) if tb else (k, n), 4, stream=1)
    want = ((a.T if ta else a).astype(np.int64) @ (b.T if tb else b).astype(np.int64)).astype(np.float32)
    for off_a, off_b in ((0, 0), (1, 2), (3, 1)):
        fa = np.concatenate([np.full(off_a, 1e30, np.float32), a.ravel()])
        fb = np.concatenate([np.full(off_b, 1e30, np.float32), b.ravel()])
        dA, dB = dev.put(fa), dev.put(fb)
        dC = dev.empty(m * n, fill=-7.0)
        for algo in (N.ALGO_AUTO, N.ALGO_MFMA_SMALL):
            r.fill(dC, -7.0, m * n)
            r.sgemm(m, n, k, dA + 4 * off_a, dB + 4 * off_b, dC, a_strides=(1, a.shape[1]) if ta else (a.shape[1], 1),
                    b_strides=(1, b.shape[1]) if tb else (b.shape[1], 1), algo=algo)
            assert np.array_equal(r.to_host(dC, (m, n)), want), (off_a, off_b, algo)


def test_golden_cases(dev):
    with open(os.path.join(GOLDEN, "matmul_cases.json")) as f:
        cases = json.load(f)["cases"]
    for c in cases:
        gen = (lambda s, sh, st: synth.small_ints(s, sh, 4, st)) if c["kind"] == "int" else (lambda s, sh, st: synth.normal(s, sh, 1.0, st))
        a, b = gen(c["seed"], (c["m"], c["k"]), 0), gen(c["seed"], (c["k"], c["n"]), 1)
        want = np.array(c["out"], dtype=np.float32).reshape(c["m"], c["n"])
        for algo in (N.ALGO_AUTO, N.ALGO_MFMA):
            got = run_gemm(dev, a, b, algo=algo)[0]
            if c["kind"] == "int":
                assert np.array_equal(got, want), (c["seed"], algo)
            else:
                assert max_err(got, want) <= gemm_tol(c["k"], a, b), (c["seed"], algo)


@pytest.mark.parametrize("split", [2, 3, 7, 16])
def test_split_k_equals_unsplit(dev, split):
    a = synth.small_ints(1, (1000, 200), 4)  # stored K x M: TN like a weight gradient
    b = synth.small_ints(2, (1000, 130), 4, stream=1)
    base = run_gemm(dev, a, b, ta=True, algo=N.ALGO_MFMA, split_k=1)[0]
    got = run_gemm(dev, a, b, ta=True, algo=N.ALGO_MFMA, split_k=split)[0]
    assert np.array_equal(got, base)
    an, bn = synth.normal(3, (4096, 96)), synth.normal(4, (4096, 80), stream=1)
    base = run_gemm(dev, an, bn, ta=True, algo=N.ALGO_MFMA, split_k=1)[0]
    got = run_gemm(dev, an, bn, ta=True, algo=N.ALGO_MFMA, split_k=split)[0]
    assert max_err(got, base) <= gemm_tol(4096, an, bn)


def test_auto_split_k_on_tall_k(dev, oracle_native):
    a = synth.normal(5, (8192, 128))
    b = synth.normal(5, (8192, 256), stream=1)
    got = run_gemm(dev, a, b, ta=True)[0]  # 2 tiles only: the planner must split
    want = oracle_native.sgemm_ikj(a.T, b)
    assert max_err(got, want) <= gemm_tol(8192, a, b)


def test_batched_and_batch_broadcast(dev):
    a = synth.small_ints(1, (5, 70, 40), 4)
    b = synth.small_ints(2, (5, 40, 90), 4, stream=1)
    got = run_gemm(dev, a, b, algo=N.ALGO_MFMA)
    assert np.array_equal(got, np.matmul(a.astype(np.int64), b.astype(np.int64)).astype(np.float32))
    w = synth.small_ints(3, (1, 40, 90), 4, stream=2)  # batch_count 1: reused by every batch
    got = run_gemm(dev, a, w, algo=N.ALGO_MFMA)
    assert np.array_equal(got, np.matmul(a.astype(np.int64), w.astype(np.int64)).astype(np.float32))


def test_batch_modulo_rule(dev, rocm):
    # operand batch index = b % batch_count (src/native/src/ops/matmul.rs:55-56)
    a = synth.small_ints(1, (2, 8, 6), 4)
    b = synth.small_ints(2, (3, 6, 5), 4, stream=1)
    dA, dB, dC = dev.put(a), dev.put(b), dev.empty(6 * 8 * 5)
    rocm.sgemm(8, 5, 6, dA, dB, dC, batch=6, a_batch=(48, 2), b_batch=(30, 3), algo=N.ALGO_MFMA)
    got = rocm.to_host(dC, (6, 8, 5))
    for i in range(6):
        assert np.array_equal(got[i], a[i % 2] @ b[i % 3])


def test_arbitrary_strides_and_unaligned_pointers(dev, rocm):
    big_a = synth.small_ints(1, (2 * 37, 2 * 29 + 1), 4)
    big_b = synth.small_ints(2, (3 * 29, 3 * 41 + 2), 4, stream=1)
    a = big_a[::2, 1::2][:37, :29]   # row stride 2*ld, col stride 2, offset 1 element
    b = big_b[::3, 2::3][:29, :41]
    dA, dB, dC = dev.put(big_a), dev.put(big_b), dev.empty(37 * 41)
    rocm.sgemm(37, 41, 29, dA + 4, dB + 8, dC, a_strides=(2 * big_a.shape[1], 2), b_strides=(3 * big_b.shape[1], 3))
    assert np.array_equal(rocm.to_host(dC, (37, 41)), (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32))
    # contiguous but based 4 bytes off a 16-byte boundary, odd leading dimension
    a2 = synth.small_ints(3, (130 * 131 + 1,), 4)
    b2 = synth.small_ints(4, (131 * 129 + 1,), 4, stream=1)
    dA, dB, dC = dev.put(a2), dev.put(b2), dev.empty(130 * 129)
    rocm.sgemm(130, 129, 131, dA + 4, dB + 4, dC)
    want = a2[1:].reshape(130, 131).astype(np.int64) @ b2[1:].reshape(131, 129).astype(np.int64)
    assert np.array_equal(rocm.to_host(dC, (130, 129)), want.astype(np.float32))


@pytest.mark.parametrize("algo", [N.ALGO_MFMA, N.ALGO_SKINNY])
@pytest.mark.parametrize("epi", [N.EPI_BIAS, N.EPI_BIAS_RELU, N.EPI_BIAS_GELU])
def test_bias_epilogues(dev, rocm, algo, epi):
    m = 130 if algo == N.ALGO_MFMA else 7
    a = synth.small_ints(1, (m, 64), 3)
    b = synth.small_ints(2, (64, 256), 3, stream=1)
    bias = synth.small_ints(3, (256,), 3, stream=2)
    dbias = dev.put(bias)
    got = run_gemm(dev, a, b, algo=algo, bias=dbias, epilogue=epi)[0]
    z = (a.astype(np.int64) @ b.astype(np.int64) + bias.astype(np.int64)).astype(np.float64)
    if epi == N.EPI_BIAS:
        assert np.array_equal(got, z.astype(np.float32))
    elif epi == N.EPI_BIAS_RELU:
        assert np.array_equal(got, np.maximum(z, 0).astype(np.float32))
    else:
        want = 0.5 * z * (1 + np.tanh(np.sqrt(2 / np.pi) * (z + 0.044715 * z ** 3)))
        assert max_err(got, want) <= 1e-5 * max(1.0, np.abs(z).max())
    # split-K applies the epilogue once, in the reduction
    if algo == N.ALGO_MFMA:
        got2 = run_gemm(dev, a, b, algo=algo, bias=dbias, epilogue=epi, split_k=2)[0]
        assert max_err(got2, got) <= 1e-6 * max(1.0, np.abs(z).max())


def _gelu64(v):
    return 0.5 * v * (1 + np.tanh(np.sqrt(2 / np.pi) * (v + 0.044715 * v ** 3)))


def _gelu_grad64(v):
    s = np.sqrt(2 / np.pi)
    th = np.tanh(s * (v + 0.044715 * v ** 3))
    return 0.5 * (1 + th) + 0.5 * v * (1 - th * th) * s * (1 + 3 * 0.044715 * v * v)


@pytest.mark.parametrize("m,n,k,batch,algo", [(256, 384, 160, 1, N.ALGO_AUTO), (130, 70, 96, 3, N.ALGO_AUTO), (70, 200, 64, 2, N.ALGO_MFMA_SMALL),
                                              (1, 5, 8, 1, N.ALGO_AUTO)])
def test_two_output_gelu_epilogue(dev, rocm, m, n, k, batch, algo):
    # C = product, aux = gelu(product + bias): the forward of a fused GELU Linear
    a = synth.normal(1, (batch, m, k))
    b = synth.normal(2, (k, n), 0.3, stream=1)
    bias = synth.normal(3, (n,), stream=2)
    dA, dB, dbias = dev.put(a), dev.put(b), dev.put(bias)
    dC, dH = dev.empty(batch * m * n, fill=-7.0), dev.empty(batch * m * n, fill=-7.0)
    rocm.sgemm(m, n, k, dA, dB, dC, batch=batch, a_batch=(m * k, batch), bias=dbias, epilogue=N.EPI_BIAS_GELU_DUAL, aux=dH, algo=algo)
    z = a.astype(np.float64) @ b.astype(np.float64)
    assert max_err(rocm.to_host(dC, (batch, m, n)), z) <= gemm_tol(k, a, b)
    assert max_err(rocm.to_host(dH, (batch, m, n)), _gelu64(z + bias)) <= gemm_tol(k, a, b)


@pytest.mark.parametrize("m,n,k,batch,algo,strips", [(256, 384, 160, 1, N.ALGO_AUTO, True), (130, 70, 96, 3, N.ALGO_AUTO, True),
                                                     (70, 200, 64, 2, N.ALGO_MFMA_SMALL, False), (40, 36, 200, 1, N.ALGO_AUTO, True)])
def test_gelu_backward_epilogue_with_strip_sums(dev, rocm, m, n, k, batch, algo, strips):
    # C = product * gelu'(z + bias) and the column sums of C per strip of rows: the gradient of a Linear's
    # input taken through the GELU of the layer that produced it, with that layer's bias gradient
    g = synth.normal(1, (batch, m, k))
    wt = synth.normal(2, (n, k), 0.3, stream=1)          # the weight [n, k] used transposed
    z = synth.normal(3, (batch, m, n), stream=2)
    bias = synth.normal(4, (n,), stream=3)
    dG, dW, dZ, dbias = dev.put(g), dev.put(wt), dev.put(z), dev.put(bias)
    dC = dev.empty(batch * m * n, fill=-7.0)
    rows = rocm.sgemm_colsum_rows(m, batch)
    assert rows == batch * ((m + 127) // 128) * 2
    dP = dev.empty(rows * n, fill=-7.0) if strips else None
    rocm.sgemm(m, n, k, dG, dW, dC, batch=batch, a_batch=(m * k, batch), b_strides=(1, k), bias=dbias, epilogue=N.EPI_DGELU, aux=dZ,
               colsum_part=dP, algo=algo)
    want = (g.astype(np.float64) @ wt.T.astype(np.float64)) * _gelu_grad64(z.astype(np.float64) + bias)
    got = rocm.to_host(dC, (batch, m, n))
    tol = gemm_tol(k, g, wt) * 1.2
    assert max_err(got, want) <= tol
    if strips:
        part = rocm.to_host(dP, (rows, n))
        assert max_err(part.astype(np.float64).sum(0), want.sum((0, 1))) <= tol * np.sqrt(batch * m)
        # strip r holds rows 64 r' .. of its batch: each strip is the sum of exactly its own rows
        per_batch = rows // batch
        for bi in range(batch):
            for st in range(per_batch):
                lo, hi = 64 * st, min(m, 64 * (st + 1))
                exp = got[bi, lo:hi].astype(np.float64).sum(0) if lo < m else np.zeros(n)
                assert max_err(part[bi * per_batch + st], exp) <= 1e-4 * max(1.0, np.abs(got).max()) * 8


def test_fused_gelu_epilogues_reject_what_they_cannot_do(dev, rocm):
    a, b = dev.put(np.ones((64, 64), np.float32)), dev.put(np.ones((64, 64), np.float32))
    c, bias = dev.empty(64 * 64), dev.put(np.zeros(64, np.float32))
    with pytest.raises(N.MniError, match="needs the aux pointer"):
        rocm.sgemm(64, 64, 64, a, b, c, bias=bias, epilogue=N.EPI_BIAS_GELU_DUAL)
    with pytest.raises(N.MniError, match="neither accumulate nor split_k"):
        rocm.sgemm(64, 64, 64, a, b, c, bias=bias, epilogue=N.EPI_DGELU, aux=c, split_k=2)
    with pytest.raises(N.MniError, match="MFMA tile kernel only"):
        rocm.sgemm(4, 64, 64, a, b, c, bias=bias, epilogue=N.EPI_DGELU, aux=c, algo=N.ALGO_SKINNY)
    with pytest.raises(N.MniError, match="colsum_part goes with the DGELU epilogue"):
        rocm.sgemm(64, 64, 64, a, b, c, bias=bias, epilogue=N.EPI_BIAS, colsum_part=c)


def test_accumulate(dev, rocm):
    a = synth.small_ints(1, (100, 50), 3)
    b = synth.small_ints(2, (50, 60), 3, stream=1)
    c0 = synth.small_ints(3, (100, 60), 3, stream=2)
    dA, dB, dC = dev.put(a), dev.put(b), dev.put(c0)
    rocm.sgemm(100, 60, 50, dA, dB, dC, accumulate=True, algo=N.ALGO_MFMA)
    assert np.array_equal(rocm.to_host(dC, (100, 60)), c0 + (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32))


def test_ldc_padding_is_untouched(dev, rocm):
    a = synth.small_ints(1, (33, 20), 3)
    b = synth.small_ints(2, (20, 45), 3, stream=1)
    dA, dB = dev.put(a), dev.put(b)
    dC = dev.empty(33 * 64, fill=-7.0)
    rocm.sgemm(33, 45, 20, dA, dB, dC, ldc=64, algo=N.ALGO_MFMA)
    got = rocm.to_host(dC, (33, 64))
    assert np.array_equal(got[:, :45], (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32))
    assert np.all(got[:, 45:] == -7.0)


def test_empty_and_zero_k(dev, rocm):
    dC = dev.empty(12, fill=5.0)
    rocm.sgemm(3, 4, 0, None, None, dC)  # K = 0: an empty sum
    assert np.all(rocm.to_host(dC, (3, 4)) == 0.0)
    rocm.sgemm(0, 4, 3, None, None, None)  # nothing to do
    rocm.sgemm(3, 0, 3, None, None, None)


# ---- stream-K distribution of the tile kernel -------------------------------------------
# Shapes that land in each form of the stream-K grid on a 256-CU / 8-XCD device:
# a pure stream-K region (fewer tiles than resident workgroups), whole rounds plus a
# region, ragged tile counts per XCD, edge tiles and K tails, 64 x 64 tiles.
STREAMK_SHAPES = [(768, 776, 1000), (1000, 1000, 1000), (1500, 1300, 520), (4096, 768, 768), (2100, 2050, 300), (640, 3000, 777),
                  (520, 260, 4100)]


@pytest.mark.parametrize("m,n,k", STREAMK_SHAPES)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_streamk_integer_exact_all_layouts(dev, m, n, k, ta, tb):
    a = synth.small_ints(m + k, (k, m) if ta else (m, k), 3)
    b = synth.small_ints(n + k, (n, k) if tb else (k, n), 3, stream=1)
    want = ((a.T if ta else a).astype(np.int64) @ (b.T if tb else b).astype(np.int64)).astype(np.float32)
    for algo in (N.ALGO_MFMA_STREAMK, N.ALGO_AUTO):
        assert np.array_equal(run_gemm(dev, a, b, ta, tb, algo=algo)[0], want), algo


def test_streamk_normal_inputs_batched_epilogue_accumulate(dev, rocm, oracle_native):
    a = synth.normal(1, (3, 700, 900))
    b = synth.normal(2, (1, 900, 650), stream=1)                      # one B for every batch (batch % 1)
    bias = synth.normal(3, (650,), stream=2)
    got = run_gemm(dev, a, b, algo=N.ALGO_MFMA_STREAMK, bias=dev.put(bias), epilogue=N.EPI_BIAS_RELU)
    for i in range(3):
        want = np.maximum(oracle_native.sgemm_ikj(a[i], b[0]) + bias, 0)
        assert max_err(got[i], want) <= gemm_tol(900, a, b)
    # accumulate: C += A B, with a padded ldc that must stay untouched
    a2, b2 = synth.small_ints(4, (1100, 600), 3), synth.small_ints(5, (600, 1030), 3, stream=1)
    c0 = synth.small_ints(6, (1100, 1040), 3, stream=2)
    dA, dB, dC = dev.put(a2), dev.put(b2), dev.put(c0)
    rocm.sgemm(1100, 1030, 600, dA, dB, dC, ldc=1040, accumulate=True, algo=N.ALGO_MFMA_STREAMK)
    out = rocm.to_host(dC, (1100, 1040))
    assert np.array_equal(out[:, :1030], c0[:, :1030] + (a2.astype(np.int64) @ b2.astype(np.int64)).astype(np.float32))
    assert np.array_equal(out[:, 1030:], c0[:, 1030:])


def test_streamk_repeats_and_agrees_with_the_tile_per_workgroup_form(dev, rocm):
    # every launch marks arrivals with a fresh value, so back-to-back launches (also of
    # other shapes and of the skinny kernel, which shares the marks) cannot see old ones
    a, b = synth.normal(7, (1300, 1100)), synth.normal(8, (1100, 900), stream=1)
    base = run_gemm(dev, a, b, algo=N.ALGO_MFMA)[0]
    dA, dB = dev.put(a), dev.put(b)
    dC = dev.empty(1300 * 900)
    x, w = dev.put(synth.normal(9, (4, 4096))), dev.put(synth.normal(10, (4096, 512), stream=1))
    dY = dev.empty(4 * 512)
    for it in range(6):
        rocm.fill(dC, -3.0, 1300 * 900)
        rocm.sgemm(1300, 900, 1100, dA, dB, dC, algo=N.ALGO_MFMA_STREAMK)
        if it % 2:
            rocm.sgemm(4, 512, 4096, x, w, dY)                                 # skinny single-launch kernel in between
        got = rocm.to_host(dC, (1300, 900))
        assert max_err(got, base) <= gemm_tol(1100, a, b) * 1e-2              # same products, another order of the K sum
        assert np.all(np.isfinite(got))
    first = rocm.to_host(dC, (1300, 900)).copy()
    rocm.sgemm(1300, 900, 1100, dA, dB, dC, algo=N.ALGO_MFMA_STREAMK)
    assert np.array_equal(rocm.to_host(dC, (1300, 900)), first)              # the sum order is fixed by the shape


def test_streamk_is_refused_where_it_cannot_work(dev, rocm):
    a, b = dev.put(np.ones((64, 64), np.float32)), dev.put(np.ones((64, 64), np.float32))
    c = dev.empty(64 * 64)
    with pytest.raises(N.MniError, match="too small"):
        rocm.sgemm(64, 64, 64, a, b, c, algo=N.ALGO_MFMA_STREAMK)
    with pytest.raises(N.MniError, match="split_k"):
        rocm.sgemm(64, 64, 64, a, b, c, algo=N.ALGO_MFMA_STREAMK, split_k=2)
    rocm.sgemm(64, 64, 64, a, b, c)                                           # the planner falls back by itself
    assert np.all(rocm.to_host(c, (64, 64)) == 64.0)


# ---- skinny kernels ----------------------------------------------------------------

# ---- register-direct kernel (batched products of many small tiles) ------------------------------

DIRECT_SHAPES = [(64, 64, 64), (512, 512, 64), (130, 70, 64), (100, 64, 512), (64, 200, 520), (34, 36, 36), (2, 2, 4),
                 (192, 128, 128), (66, 130, 1000)]


@pytest.mark.parametrize("m,n,k", DIRECT_SHAPES)
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("parts", [1, 4])
def test_direct_integer_exact_all_layouts(dev, m, n, k, ta, tb, parts):
    # every extent is even and K a multiple of 4, so all four layouts are eligible; edges inside tiles,
    # K tails inside phases, wavefronts without any K of their own (K = 4 split four ways)
    a = synth.small_ints(m + k, (3, k, m) if ta else (3, m, k), 4)
    b = synth.small_ints(n + k, (3, n, k) if tb else (3, k, n), 4, stream=1)
    got = run_gemm(dev, a, b, ta, tb, algo=N.ALGO_DIRECT, split_k=parts)
    A = a.transpose(0, 2, 1) if ta else a
    B = b.transpose(0, 2, 1) if tb else b
    assert np.array_equal(got, np.einsum("bmk,bkn->bmn", A.astype(np.int64), B.astype(np.int64)).astype(np.float32))


@pytest.mark.parametrize("parts", [1, 4])
def test_direct_odd_extents_where_the_layout_allows(dev, parts):
    # an operand that is contiguous along K may have any number of rows
    a = synth.small_ints(1, (77, 40), 4)
    bt = synth.small_ints(2, (51, 40), 4, stream=1)
    got = run_gemm(dev, a, bt, False, True, algo=N.ALGO_DIRECT, split_k=parts)[0]
    assert np.array_equal(got, (a.astype(np.int64) @ bt.T.astype(np.int64)).astype(np.float32))


@pytest.mark.parametrize("parts", [1, 4])
def test_direct_normal_inputs_batch_rule_epilogue_accumulate(dev, rocm, oracle_native, parts):
    a = synth.normal(1, (6, 96, 200))
    w = synth.normal(2, (2, 200, 72), stream=1)   # batch b reads w[b % 2]
    bias = synth.normal(3, (72,), stream=2)
    c0 = synth.normal(4, (6, 96, 72), stream=3)
    dA, dW, dbias, dC = dev.put(a), dev.put(w), dev.put(bias), dev.put(c0)
    rocm.sgemm(96, 72, 200, dA, dW, dC, batch=6, a_batch=(96 * 200, 6), b_batch=(200 * 72, 2), bias=dbias,
               epilogue=N.EPI_BIAS_RELU, accumulate=True, algo=N.ALGO_DIRECT, split_k=parts)
    got = rocm.to_host(dC, (6, 96, 72))
    for b in range(6):
        want = np.maximum(oracle_native.sgemm_ikj(a[b], w[b % 2]) + bias, 0) + c0[b]
        assert max_err(got[b], want) <= gemm_tol(200, a, w)


def test_direct_is_refused_for_layouts_it_cannot_read(dev, rocm):
    a, b = synth.small_ints(1, (64, 30), 3), synth.small_ints(2, (30, 64), 3, stream=1)
    dA, dB, dC = dev.put(a), dev.put(b), dev.empty(64 * 64)
    with pytest.raises(N.MniError, match="not eligible for the direct kernel"):
        rocm.sgemm(64, 64, 30, dA, dB, dC, algo=N.ALGO_DIRECT)  # A contiguous along K, K % 4 != 0
    with pytest.raises(N.MniError, match="split_k 0, 1 or 4"):
        rocm.sgemm(64, 64, 28, dA, dB, dC, a_strides=(30, 1), algo=N.ALGO_DIRECT, split_k=3)
    with pytest.raises(N.MniError, match="not eligible for the direct kernel"):
        rocm.sgemm(64, 64, 15, dA, dB, dC, a_strides=(2, 128), algo=N.ALGO_DIRECT)  # neither axis contiguous


# ---- short-K panel kernel (two K-contiguous operands, all of K at once) ---------------------------

@pytest.mark.parametrize("m,n,k,batch", [(128, 128, 64, 1), (512, 512, 64, 3), (200, 150, 64, 2), (130, 257, 48, 1), (64, 40, 32, 2),
                                         (300, 129, 20, 1), (1, 1, 4, 1), (129, 3, 36, 1)])
def test_panel_integer_exact(dev, m, n, k, batch):
    # edges inside tiles (rows beyond them re-read the last row), K below the kernel's 32 / 64 (zero quads)
    a = synth.small_ints(m + k, (batch, m, k), 4)
    bt = synth.small_ints(n + k, (batch, n, k), 4, stream=1)
    got = run_gemm(dev, a, bt, False, True, algo=N.ALGO_PANEL)
    assert np.array_equal(got, np.einsum("bmk,bnk->bmn", a.astype(np.int64), bt.astype(np.int64)).astype(np.float32))


def test_panel_normal_inputs_batch_rule_epilogue_accumulate(dev, rocm, oracle_native):
    a = synth.normal(1, (5, 140, 64))
    wt = synth.normal(2, (2, 136, 64), stream=1)   # batch b reads wt[b % 2]
    bias = synth.normal(3, (136,), stream=2)
    c0 = synth.normal(4, (5, 140, 136), stream=3)
    for epi, f in ((N.EPI_NONE, lambda z: z), (N.EPI_BIAS_RELU, lambda z: np.maximum(z + bias, 0))):
        dA, dW, dbias, dC = dev.put(a), dev.put(wt), dev.put(bias), dev.put(c0)
        rocm.sgemm(140, 136, 64, dA, dW, dC, batch=5, a_batch=(140 * 64, 5), b_strides=(1, 64), b_batch=(136 * 64, 2),
                   bias=dbias if epi else None, epilogue=epi, accumulate=True, algo=N.ALGO_PANEL)
        got = rocm.to_host(dC, (5, 140, 136))
        for b in range(5):
            want = f(oracle_native.sgemm_ikj(a[b], wt[b % 2].T.copy())) + c0[b]
            assert max_err(got[b], want) <= gemm_tol(64, a, wt)


def test_panel_is_refused_for_shapes_it_cannot_take(dev, rocm):
    a, b = synth.small_ints(1, (64, 68), 3), synth.small_ints(2, (68, 64), 3, stream=1)
    dA, dB, dC = dev.put(a), dev.put(b), dev.empty(64 * 64)
    with pytest.raises(N.MniError, match="short-K panel kernel takes two K-contiguous operands"):
        rocm.sgemm(64, 64, 68, dA, dB, dC, b_strides=(1, 68), algo=N.ALGO_PANEL)   # K > 64
    with pytest.raises(N.MniError, match="short-K panel kernel takes two K-contiguous operands"):
        rocm.sgemm(64, 64, 64, dA, dB, dC, a_strides=(68, 1), algo=N.ALGO_PANEL)   # B contiguous along N
    with pytest.raises(N.MniError, match="no split_k"):
        rocm.sgemm(64, 64, 64, dA, dB, dC, a_strides=(68, 1), b_strides=(1, 68), algo=N.ALGO_PANEL, split_k=2)


def test_planner_choices_for_attention_shaped_products(dev, rocm):
    # scores (short K, both operands K-contiguous) go to the panel kernel by themselves; the two backward
    # products (about one 64 x 64 tile per CU, a long thin operand) to the tile kernel's 64 x 64 tiles in one K
    # slice, one launch each; the results must be the forced plans' bits
    q = synth.normal(1, (16, 512, 64), 0.125)
    ds = synth.normal(2, (16, 512, 512), stream=1)
    dQ, dS = dev.put(q), dev.put(ds)
    outs = []
    for algo, split in ((N.ALGO_AUTO, 0), (N.ALGO_PANEL, 0)):
        dC = dev.empty(16 * 512 * 512)
        rocm.sgemm(512, 512, 64, dQ, dQ, dC, batch=16, a_batch=(512 * 64, 16), b_strides=(1, 64), b_batch=(512 * 64, 16), algo=algo, split_k=split)
        outs.append(rocm.to_host(dC, (16, 512, 512)))
    assert np.array_equal(outs[0], outs[1])
    assert max_err(outs[0][3], q[3].astype(np.float64) @ q[3].T.astype(np.float64)) <= gemm_tol(64, q, q)
    outs, launches = [], []
    for algo, split in ((N.ALGO_AUTO, 0), (N.ALGO_MFMA_SMALL, 1), (N.ALGO_DIRECT, 4)):
        dC = dev.empty(16 * 512 * 64)
        before = rocm.launch_count()
        rocm.sgemm(512, 64, 512, dS, dQ, dC, batch=16, a_batch=(512 * 512, 16), b_batch=(512 * 64, 16), algo=algo, split_k=split)
        launches.append(rocm.launch_count() - before)
        outs.append(rocm.to_host(dC, (16, 512, 64)))
    assert np.array_equal(outs[0], outs[1]) and launches[0] == 1
    for got in outs:
        assert max_err(got[5], ds[5].astype(np.float64) @ q[5].astype(np.float64)) <= gemm_tol(512, ds, q)
    # its transposed twin, dK^T = Q^T dS
    outs = []
    for algo, split in ((N.ALGO_AUTO, 0), (N.ALGO_MFMA_SMALL, 1)):
        dC = dev.empty(16 * 64 * 512)
        rocm.sgemm(64, 512, 512, dQ, dS, dC, batch=16, a_strides=(1, 64), a_batch=(512 * 64, 16), b_batch=(512 * 512, 16), algo=algo, split_k=split)
        outs.append(rocm.to_host(dC, (16, 64, 512)))
    assert np.array_equal(outs[0], outs[1])
    assert max_err(outs[0][7], q[7].T.astype(np.float64) @ ds[7].astype(np.float64)) <= gemm_tol(512, q, ds)


@pytest.mark.parametrize("m,n,k,batch", [(16, 64, 16, 1024), (48, 256, 16, 512), (33, 70, 12, 600)])
@pytest.mark.parametrize("tb", [False, True])
def test_planner_gives_many_batches_of_few_rows_and_one_k_phase_to_the_direct_kernel(dev, rocm, m, n, k, batch, tb):
    # three quarters of a 64 x 64 tile would be padding: the register-direct kernel, one wavefront per tile, takes them;
    # the bits are the forced plan's, the values exact on small integers
    a = synth.small_ints(m + n, (batch, m, k), 4)
    b = synth.small_ints(k + batch, (batch, n, k) if tb else (batch, k, n), 4, stream=1)
    got = run_gemm(dev, a, b, False, tb)
    forced = run_gemm(dev, a, b, False, tb, algo=N.ALGO_DIRECT, split_k=1)
    B = b.transpose(0, 2, 1) if tb else b
    assert np.array_equal(got, np.einsum("bmk,bkn->bmn", a.astype(np.int64), B.astype(np.int64)).astype(np.float32))
    assert np.array_equal(got, forced)


@pytest.mark.parametrize("m,n,k", [(33, 4096, 4096), (64, 2048, 8192), (50, 8192, 2048), (64, 16384, 1024), (96, 4096, 8192), (128, 8192, 8192),
                                   (70, 4096, 11008)])
def test_planner_gives_33_to_64_rows_against_a_large_weight_wide_tiles_in_k_slices(dev, rocm, m, n, k):
    # 64 x 128 tiles (128 x 128 from 65 rows, for a long K) in 256 / (N / 128) K slices, one workgroup per CU, and their reduction pass:
    # exact on small integers, with and without the bias epilogue, and the bits of the forced plan
    a = synth.small_ints(m + n, (m, k), 3)
    b = synth.small_ints(k + m, (k, n), 3, stream=1)
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)  # (exact: the sums stay far below 2^53)
    got = run_gemm(dev, a, b)[0]
    assert np.array_equal(got, want)
    assert np.array_equal(got, run_gemm(dev, a, b, algo=N.ALGO_MFMA, split_k=256 // (n // 128))[0])
    bias = synth.small_ints(n, (n,), 5, stream=2)
    dA, dB, dBias, dC = dev.put(a), dev.put(b), dev.put(bias), dev.empty(m * n, fill=-3.0)
    rocm.sgemm(m, n, k, dA, dB, dC, bias=dBias, epilogue=N.EPI_BIAS_RELU)
    assert np.array_equal(rocm.to_host(dC, (m, n)), np.maximum(want + bias, 0.0).astype(np.float32))


# ---- tiny products: one thread per output, the reference CPU arm's own sum ---------------------------

@pytest.mark.parametrize("m,n,k", [(32, 64, 10), (32, 3, 64), (32, 64, 3), (32, 10, 64), (64, 3, 32), (10, 64, 32), (1, 1, 1), (7, 5, 3),
                                   (64, 64, 64), (33, 17, 130), (100, 60, 7)])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_tiny_products_are_the_reference_sum_bit_for_bit(dev, oracle_native, m, n, k, ta, tb):
    # the README example's six products among them; normal inputs: every output must be the oracle's i-k-j sum
    # (products rounded, added in k order) to the last bit, whatever the layout, forced and chosen by the planner
    a = synth.normal(m + k, (k, m) if ta else (m, k))
    b = synth.normal(n + k, (n, k) if tb else (k, n), stream=1)
    want = oracle_native.sgemm_ikj(np.ascontiguousarray(a.T) if ta else a, np.ascontiguousarray(b.T) if tb else b)
    for algo in (N.ALGO_TINY, N.ALGO_AUTO):
        got = run_gemm(dev, a, b, ta, tb, algo=algo)[0]
        assert np.array_equal(got, want), algo


def test_tiny_products_batch_rule_strides_epilogues_accumulate(dev, rocm, oracle_native):
    a = synth.normal(1, (6, 20, 12))
    w = synth.normal(2, (2, 12, 9), stream=1)     # batch b reads w[b % 2]
    bias = synth.normal(3, (9,), stream=2)
    c0 = synth.normal(4, (6, 20, 11), stream=3)   # C sits in rows of 11 floats
    for epi, f in ((N.EPI_NONE, lambda z: z), (N.EPI_BIAS, lambda z: z + bias), (N.EPI_BIAS_RELU, lambda z: np.maximum(z + bias, 0)),
                   (N.EPI_BIAS_GELU, lambda z: None)):   # tanh-approximation GELU, in float64 below
        dA, dW, dbias, dC = dev.put(a), dev.put(w), dev.put(bias), dev.put(c0)
        before = rocm.launch_count()
        rocm.sgemm(20, 9, 12, dA, dW, dC, batch=6, a_batch=(20 * 12, 6), b_batch=(12 * 9, 2), ldc=11, c_batch_stride=20 * 11,
                   bias=dbias if epi else None, epilogue=epi, accumulate=True)
        assert rocm.launch_count() - before == 1
        got = rocm.to_host(dC, (6, 20, 11))
        assert np.array_equal(got[:, :, 9:], c0[:, :, 9:])   # the padding of C is untouched
        for bb in range(6):
            z = oracle_native.sgemm_ikj(a[bb], w[bb % 2])
            want = f(z)
            if want is None:
                s_ = np.float32(0.7978845608028654)
                zb = (z + bias).astype(np.float64)
                want = (0.5 * zb * (1.0 + np.tanh(s_ * (zb + 0.044715 * zb ** 3)))).astype(np.float32)
            assert max_err(got[bb, :, :9], want + c0[bb, :, :9]) <= 2e-6 * max(1.0, float(np.abs(want).max()))
    # neither axis of A contiguous, B a column slice of a wider matrix
    wide_a = synth.small_ints(5, (16, 2 * 24), 4)
    wide_b = synth.small_ints(6, (24, 40), 4, stream=1)
    dA, dB, dC = dev.put(wide_a), dev.put(wide_b), dev.empty(16 * 8)
    rocm.sgemm(16, 8, 24, dA, dB + 4 * 5, dC, a_strides=(48, 2), b_strides=(40, 1), algo=N.ALGO_TINY)
    want = wide_a[:, ::2].astype(np.int64) @ wide_b[:, 5:13].astype(np.int64)
    assert np.array_equal(rocm.to_host(dC, (16, 8)), want.astype(np.float32))
    with pytest.raises(N.MniError, match="no split_k and no fused GELU"):
        rocm.sgemm(16, 8, 24, dA, dB, dC, algo=N.ALGO_TINY, split_k=2)


# ---- two independent products in one launch (the backward pair of a batched matmul) ----------------

def _pair_descs(rocm, dev, batch, t, d, kview, ds, q, k):
    """dQ = dS K and dK^T = Q^T dS for S = Q K^T; kview: K^T given as a permuted view (the forward's B
    operand), so dQ's B is K row-major; else the forward's B is K^T stored [d, t] and dQ's B is its transpose."""
    dDS, dQm, dKm = dev.put(ds), dev.put(q), dev.put(k)
    o0, o1 = dev.empty(batch * t * d), dev.empty(batch * t * d)
    if kview:
        d0 = rocm.gemm_desc(t, d, t, dDS, dKm, o0, batch=batch, a_batch=(t * t, batch), b_batch=(t * d, batch))
        d1 = rocm.gemm_desc(d, t, t, dQm, dDS, o1, batch=batch, a_strides=(1, d), a_batch=(t * d, batch), b_batch=(t * t, batch))
    else:
        d0 = rocm.gemm_desc(t, d, t, dDS, dKm, o0, batch=batch, a_batch=(t * t, batch), b_strides=(1, t), b_batch=(t * d, batch))
        d1 = rocm.gemm_desc(d, t, t, dQm, dDS, o1, batch=batch, a_batch=(t * d, batch), b_batch=(t * t, batch))
    return d0, d1, o0, o1


@pytest.mark.parametrize("batch,t,d,kview", [(16, 512, 64, True), (16, 512, 64, False), (32, 256, 128, True), (20, 500, 62, True), (20, 448, 64, True),
                                             (64, 512, 64, True)])
def test_pair_launch_gives_the_bits_of_separate_launches(dev, rocm, batch, t, d, kview):
    # sizes at which each product alone is planned as 64 x 64 tiles, one workgroup per tile, so the pair goes out as
    # one launch (the fourth with edges inside tiles and a K tail; the fifth with a tile count that is no multiple
    # of 8, so that padding workgroups exist; the last with two tiles per CU each); integer
    # inputs pin the values, normal inputs the order of the K sum
    for make in (lambda s, shape, st: synth.small_ints(s, shape, 3, stream=st), lambda s, shape, st: synth.normal(s, shape, stream=st)):
        ds = make(1, (batch, t, t), 0)
        q = make(2, (batch, t, d) if kview else (batch, d, t), 1)
        k = make(3, (batch, t, d) if kview else (batch, d, t), 2)
        d0, d1, o0, o1 = _pair_descs(rocm, dev, batch, t, d, kview, ds, q, k)
        before = rocm.launch_count()
        rocm.sgemm_pair(d0, d1)
        launches = rocm.launch_count() - before
        got0, got1 = rocm.to_host(o0, (batch, t, d)), rocm.to_host(o1, (batch, d, t))
        rocm.fill(o0, -1.0, batch * t * d)
        rocm.fill(o1, -1.0, batch * t * d)
        rocm._check(rocm.lib.mni_rocm_sgemm(d0))
        rocm._check(rocm.lib.mni_rocm_sgemm(d1))
        assert np.array_equal(got0, rocm.to_host(o0, (batch, t, d)))
        assert np.array_equal(got1, rocm.to_host(o1, (batch, d, t)))
        assert launches == 1
        if np.all(ds == np.round(ds)):
            K = k if kview else k.transpose(0, 2, 1)
            Q = q if kview else q.transpose(0, 2, 1)
            assert np.array_equal(got0, np.einsum("bij,bjd->bid", ds.astype(np.int64), K.astype(np.int64)).astype(np.float32))
            assert np.array_equal(got1, np.einsum("bid,bij->bdj", Q.astype(np.int64), ds.astype(np.int64)).astype(np.float32))


def test_pair_launch_of_small_and_of_big_products(dev, rocm, oracle_native):
    # a pair of small products (a few tiles each) may share a launch too; either way the values are right
    a = synth.normal(1, (96, 200))
    b = synth.normal(2, (200, 72), stream=1)
    g = synth.normal(3, (96, 72), stream=2)
    dA, dB, dG = dev.put(a), dev.put(b), dev.put(g)
    oa, ob = dev.empty(96 * 200), dev.empty(200 * 72)
    d0 = rocm.gemm_desc(96, 200, 72, dG, dB, oa, b_strides=(1, 72))
    d1 = rocm.gemm_desc(200, 72, 96, dA, dG, ob, a_strides=(1, 200))
    rocm.sgemm_pair(d0, d1)
    assert max_err(rocm.to_host(oa, (96, 200)), oracle_native.sgemm_ikj(g, b.T.copy())) <= gemm_tol(72, g, b)
    assert max_err(rocm.to_host(ob, (200, 72)), oracle_native.sgemm_ikj(a.T.copy(), g)) <= gemm_tol(96, a, g)
    with pytest.raises(N.MniError, match="null descriptor"):
        rocm._check(rocm.lib.mni_rocm_sgemm_pair(None, None))
    # a pair with an extent off a multiple of 4 (its edge tiles could not be read in 16-byte pieces along that axis: sgemm cuts
    # such a product up first): each product is launched by itself
    n = 2048
    big = synth.normal(4, (n, n))
    odd = synth.normal(5, (n - 2, n), stream=1)
    dBig, dOdd, o2, o3 = dev.put(big), dev.put(odd), dev.empty((n - 2) * n), dev.empty(n * n)
    before = rocm.launch_count()
    rocm.sgemm_pair(rocm.gemm_desc(n - 2, n, n, dOdd, dBig, o2, b_strides=(1, n)), rocm.gemm_desc(n, n, n - 2, dOdd, dOdd, o3, a_strides=(1, n)))
    assert rocm.launch_count() - before >= 2
    assert max_err(rocm.to_host(o2, (n - 2, n)), odd.astype(np.float64) @ big.T.astype(np.float64)) <= gemm_tol(n, odd, big)
    assert max_err(rocm.to_host(o3, (n, n)), odd.T.astype(np.float64) @ odd.astype(np.float64)) <= gemm_tol(n, odd, odd)


def _linear_backward_descs(rocm, dev, M, K, Nn, g, x, w, **first):
    """dx = g . w^T and dw = x^T . g of y[M, Nn] = x[M, K] . w[K, Nn]."""
    dG, dX, dW = dev.put(g), dev.put(x), dev.put(w)
    o0, o1 = dev.empty(M * K, fill=-3.0), dev.empty(K * Nn, fill=-3.0)
    d0 = rocm.gemm_desc(M, K, Nn, dG, dW, o0, b_strides=(1, Nn), **first)
    d1 = rocm.gemm_desc(K, Nn, M, dX, dG, o1, a_strides=(1, K))
    return d0, d1, o0, o1


@pytest.mark.parametrize("M,K,Nn", [(2048, 2048, 2048), (2044, 2048, 2040), (1920, 2176, 1920), (4096, 4096, 1024), (1024, 4096, 2048)])
def test_pair_launch_of_big_tiles_gives_the_bits_of_separate_launches(dev, rocm, M, K, Nn):
    # the two gradients of a Linear layer, each planned alone as whole 128 x 128 tiles: one launch (the second with edges
    # inside tiles; the third with 255 tiles each, so that a padding workgroup exists; the fourth with 1024 tiles of
    # K = 1024 behind 256 of K = 4096, which lead, four short tiles to a workgroup; the last with the first product
    # leading and two tiles to a workgroup of the second); integer inputs pin the values, normal inputs the order of the K sum
    for make in (lambda s, shape, st: synth.small_ints(s, shape, 3, stream=st), lambda s, shape, st: synth.normal(s, shape, stream=st)):
        g, x, w = make(1, (M, Nn), 0), make(2, (M, K), 1), make(3, (K, Nn), 2)
        d0, d1, o0, o1 = _linear_backward_descs(rocm, dev, M, K, Nn, g, x, w)
        before = rocm.launch_count()
        rocm.sgemm_pair(d0, d1)
        launches = rocm.launch_count() - before
        got0, got1 = rocm.to_host(o0, (M, K)), rocm.to_host(o1, (K, Nn))
        rocm.fill(o0, -1.0, M * K)
        rocm.fill(o1, -1.0, K * Nn)
        rocm._check(rocm.lib.mni_rocm_sgemm(d0))
        rocm._check(rocm.lib.mni_rocm_sgemm(d1))
        assert np.array_equal(got0, rocm.to_host(o0, (M, K)))
        assert np.array_equal(got1, rocm.to_host(o1, (K, Nn)))
        assert launches == 1
        if np.all(g == np.round(g)):
            assert np.array_equal(got0, (g.astype(np.float64) @ w.T.astype(np.float64)).astype(np.float32))
            assert np.array_equal(got1, (x.T.astype(np.float64) @ g.astype(np.float64)).astype(np.float32))


def test_pair_launch_of_big_tiles_with_the_gelu_backward_epilogue(dev, rocm):
    # the same pair behind a GELU Linear: the first product scales by gelu'(z + bias) and leaves strip sums for that layer's
    # bias gradient; still one launch, and the bits of the two products launched apart
    M, K, Nn = 2048, 2048, 2048
    g, x, w = synth.normal(1, (M, Nn)), synth.normal(2, (M, K), stream=1), synth.normal(3, (K, Nn), 0.3, stream=2)
    z, bias = synth.normal(4, (M, K), stream=3), synth.normal(5, (K,), stream=4)
    dZ, dbias = dev.put(z), dev.put(bias)
    rows = rocm.sgemm_colsum_rows(M, 1)
    dP = dev.empty(rows * K, fill=-7.0)
    d0, d1, o0, o1 = _linear_backward_descs(rocm, dev, M, K, Nn, g, x, w, bias=dbias, epilogue=N.EPI_DGELU, aux=dZ, colsum_part=dP)
    before = rocm.launch_count()
    rocm.sgemm_pair(d0, d1)
    assert rocm.launch_count() - before == 1
    got0, got1, part = rocm.to_host(o0, (M, K)), rocm.to_host(o1, (K, Nn)), rocm.to_host(dP, (rows, K))
    rocm.fill(o0, -1.0, M * K)
    rocm.fill(o1, -1.0, K * Nn)
    rocm.fill(dP, -1.0, rows * K)
    rocm._check(rocm.lib.mni_rocm_sgemm(d0))
    rocm._check(rocm.lib.mni_rocm_sgemm(d1))
    assert np.array_equal(got0, rocm.to_host(o0, (M, K)))
    assert np.array_equal(got1, rocm.to_host(o1, (K, Nn)))
    assert np.array_equal(part, rocm.to_host(dP, (rows, K)))
    want = (g.astype(np.float64) @ w.T.astype(np.float64)) * _gelu_grad64(z.astype(np.float64) + bias)
    assert max_err(got0, want) <= gemm_tol(Nn, g, w) * 1.2
    assert max_err(part.astype(np.float64).sum(0), want.sum(0)) <= gemm_tol(Nn, g, w) * 1.2 * np.sqrt(M)
    assert max_err(got1, x.T.astype(np.float64) @ g.astype(np.float64)) <= gemm_tol(M, x, g)


@pytest.mark.parametrize("m,n,k", [(24, 4096, 4096), (96, 4096, 4096), (128, 1024, 4096), (192, 4096, 1024), (48, 11008, 1024), (64, 512, 16384),
                                   (200, 1000, 3000)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
def test_products_of_few_tiles_in_planned_k_slices_integer_exact(dev, rocm, m, n, k, ta, tb):
    # 17 to a few hundred rows against a large operand: fewer 64 x 64 tiles than CUs, so the planner's cost model
    # picks the number of K slices (1 to 16 over these shapes); whatever it picks, the sums are exact and the
    # launches are the product and at most one reduction
    a = synth.small_ints(m + k, (k, m) if ta else (m, k), 3)
    b = synth.small_ints(n + k, (n, k) if tb else (k, n), 3, stream=1)
    want = ((a.T if ta else a).astype(np.int64) @ (b.T if tb else b).astype(np.int64)).astype(np.float32)
    before = rocm.launch_count()
    got = run_gemm(dev, a, b, ta, tb)[0]
    assert np.array_equal(got, want)
    assert rocm.launch_count() - before <= 3   # (the output buffer's fill, the product, the reduction)


@pytest.mark.parametrize("m,n,k,split", [(32, 256, 256, 0), (17, 128, 64, 0), (32, 4096, 4096, 0), (24, 1000, 520, 0), (32, 512, 1024, 1), (20, 640, 2056, 3),
                                         (32, 4096, 1024, 16), (31, 132, 72, 0), (29, 11008, 512, 0), (32, 2048, 8192, 5), (18, 50304, 256, 0),
                                         (9, 512, 512, 0), (12, 8192, 2048, 0), (16, 4096, 4096, 0)])
def test_fewrows_integer_exact(dev, rocm, m, n, k, split):
    # 9 to 32 rows against a wide N-contiguous operand: W straight into MFMA registers, K slices summed by the last
    # workgroup of a column group to arrive.  Edges in M and N, slices that do not divide K, one slice, more slices
    # than CUs per column group; forced and (where the planner picks it) by itself, twice in a row (the arrival
    # counters must be back at zero).
    a = synth.small_ints(m + k, (m, k), 3)
    b = synth.small_ints(n + k, (k, n), 3, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    for _ in range(2):
        assert np.array_equal(run_gemm(dev, a, b, algo=N.ALGO_FEWROWS, split_k=split)[0], want)
    assert np.array_equal(run_gemm(dev, a, b)[0], want)


def test_fewrows_normal_inputs_batch_epilogues_accumulate(dev, rocm, oracle_native):
    m, n, k, batch = 27, 640, 1024, 3
    a = synth.normal(1, (batch, m, k))
    w = synth.normal(2, (1, k, n), stream=1)          # one W for all batches (the reference's broadcast rule)
    bias = synth.normal(3, (n,), stream=2)
    tol = gemm_tol(k, a, w)
    want = np.stack([oracle_native.sgemm_ikj(a[b], w[0]) for b in range(batch)])
    for algo in (N.ALGO_FEWROWS, N.ALGO_AUTO):
        assert max_err(run_gemm(dev, a, w, algo=algo), want) <= tol
    dBias = dev.put(bias)
    for epi, f in ((N.EPI_BIAS, lambda z: z), (N.EPI_BIAS_RELU, lambda z: np.maximum(z, 0)),
                   (N.EPI_BIAS_GELU, lambda z: 0.5 * z * (1 + np.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3))))):
        for split in (1, 0):
            got = run_gemm(dev, a, w, algo=N.ALGO_FEWROWS, split_k=split, bias=dBias, epilogue=epi)
            assert max_err(got, f(want.astype(np.float64) + bias[None, None, :])) <= tol + 1e-5
    # accumulate: C += A W on a C that holds something
    dA, dW = dev.put(a), dev.put(w)
    dC = dev.put(want.copy())
    rocm.sgemm(m, n, k, dA, dW, dC, batch=batch, a_batch=(m * k, batch), b_batch=(k * n, 1), accumulate=True, algo=N.ALGO_FEWROWS)
    assert max_err(rocm.to_host(dC, (batch, m, n)), 2.0 * want.astype(np.float64)) <= 2 * tol
    # what it does not take is refused when forced
    with pytest.raises(N.MniError, match="few-rows kernel takes 9 to 32 rows"):
        run_gemm(dev, synth.normal(1, (40, 256)), synth.normal(2, (256, 256)), algo=N.ALGO_FEWROWS)
    with pytest.raises(N.MniError, match="few-rows kernel takes 9 to 32 rows"):
        run_gemm(dev, synth.normal(1, (256, 32)), synth.normal(2, (256, 256)), ta=True, algo=N.ALGO_FEWROWS)


@pytest.mark.parametrize("m,h,c", [(32, 64, 3), (32, 10, 64), (7, 5, 3), (128, 64, 64), (33, 257, 9)])
def test_pair_of_tiny_products_is_one_launch_with_the_reference_sums(dev, rocm, oracle_native, m, h, c):
    # the backward pair of a small Linear (x [m, h] . w [h, c]; dx = g . w^T, dw = x^T . g): products the tiny-product
    # kernel takes go out as one launch, each output still the reference CPU arm's sum bit for bit
    x = synth.normal(m, (m, h))
    w = synth.normal(h, (h, c), stream=1)
    g = synth.normal(c, (m, c), stream=2)
    dX, dW, dG = dev.put(x), dev.put(w), dev.put(g)
    ox, ow = dev.empty(m * h), dev.empty(h * c)
    d0 = rocm.gemm_desc(m, h, c, dG, dW, ox, b_strides=(1, c))   # g . w^T
    d1 = rocm.gemm_desc(h, c, m, dX, dG, ow, a_strides=(1, h))   # x^T . g
    before = rocm.launch_count()
    rocm.sgemm_pair(d0, d1)
    assert rocm.launch_count() - before == 1
    got0, got1 = rocm.to_host(ox, (m, h)), rocm.to_host(ow, (h, c))
    assert np.array_equal(got0, oracle_native.sgemm_ikj(g, w.T.copy()))
    assert np.array_equal(got1, oracle_native.sgemm_ikj(x.T.copy(), g))
    # accumulate on one side, a bias on the other: the two products keep their own epilogues
    bias = synth.normal(3, (c,), stream=3)
    dBias = dev.put(bias)
    d2 = rocm.gemm_desc(m, h, c, dG, dW, ox, b_strides=(1, c), accumulate=1)
    d3 = rocm.gemm_desc(h, c, m, dX, dG, ow, a_strides=(1, h), bias=dBias, epilogue=N.EPI_BIAS)
    rocm.sgemm_pair(d2, d3)
    assert np.array_equal(rocm.to_host(ox, (m, h)), got0 + got0)
    assert np.array_equal(rocm.to_host(ow, (h, c)), got1 + bias[None, :])


def test_single_launch_skinny_path_is_available(rocm):
    # MI355X deals workgroups over its 8 XCDs round-robin; were the probe to fail,
    # ALGO_SKINNY would quietly run as ALGO_SKINNY_TWO_PASS and the tests below
    # would cover one path twice.
    assert rocm.device_xcds() == 8


SKINNY_ALGOS = [N.ALGO_SKINNY, N.ALGO_SKINNY_TWO_PASS]  # slices summed inside the launch / by a second launch


@pytest.mark.parametrize("algo", SKINNY_ALGOS)
@pytest.mark.parametrize("m", [1, 2, 4, 5, 8, 13, 16])
def test_skinny_cols_integer_exact(dev, m, algo):
    a = synth.small_ints(m, (m, 700), 4)
    b = synth.small_ints(m + 1, (700, 520), 4, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a, b, algo=algo)[0], want)
    for split in (1, 3, 11):  # 3 slices < 13 rows: reducers take several rows each
        assert np.array_equal(run_gemm(dev, a, b, algo=algo, split_k=split)[0], want)


@pytest.mark.parametrize("m,n,k", [(12, 8192, 2048), (12, 11008, 1024), (8, 50304, 768), (13, 4096, 4096), (16, 50304, 256), (5, 32000, 512), (9, 2048, 8192)])
def test_skinny_cols_wide_outputs_integer_exact(dev, rocm, m, n, k):
    # Many column groups: the reducers of the single-launch form (the workgroups of a unit's last min(rows, slices)
    # K slices, which wait for all of its slices) must all fit on their XCD together, or the first ones fill it and
    # wait for slices that are never dispatched.  The 16-row general form fits one workgroup per CU (253 VGPRs): at
    # 12 x 8192 x 8192 its 48 reducers per XCD met 32 places, gave up and wrote NaN.  The host now takes the
    # two-launch form whenever the reducers would not fit.
    a = synth.small_ints(m + n, (m, k), 3)
    b = synth.small_ints(n + k, (k, n), 3, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    for algo in (N.ALGO_AUTO, N.ALGO_SKINNY):
        assert np.array_equal(run_gemm(dev, a, b, algo=algo)[0], want)
    rocm.sync()   # (a wait that expired would be reported here)


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 6, 7, 8, 16])
def test_skinny_cols_decode_shape_integer_exact(dev, m):
    # whole column groups, plain output: the single-launch kernel specialised for the row count
    a = synth.small_ints(m, (m, 2048), 4)
    b = synth.small_ints(m + 1, (2048, 768), 4, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a, b, algo=N.ALGO_SKINNY)[0], want)
    assert np.array_equal(run_gemm(dev, a, b, algo=N.ALGO_SKINNY, split_k=5)[0], want)
    assert np.array_equal(run_gemm(dev, a, b)[0], want)  # (what the planner picks for the shape)


@pytest.mark.parametrize("m", [1, 4, 6, 16])
def test_skinny_cols_decode_shape_epilogues_and_accumulate(dev, rocm, m):
    # bias, activation and accumulation in the kernels specialised for a row count (the bias and, without an
    # activation, the old output enter the sum with the first K slice)
    k, n = 1024, 512
    a = synth.small_ints(m, (m, k), 3); b = synth.small_ints(m + 1, (k, n), 3, stream=1)
    bias = synth.small_ints(m + 2, (n,), 5, stream=2); old = synth.small_ints(m + 3, (m, n), 9, stream=3)
    prod = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float64)
    dA, dB, dBias = dev.put(a), dev.put(b), dev.put(bias)
    for epi, accumulate in [(N.EPI_NONE, True), (N.EPI_BIAS, False), (N.EPI_BIAS, True), (N.EPI_BIAS_RELU, False),
                            (N.EPI_BIAS_RELU, True), (N.EPI_BIAS_GELU, False), (N.EPI_BIAS_GELU, True)]:
        z = prod + (bias if epi != N.EPI_NONE else 0.0)
        if epi == N.EPI_BIAS_RELU: z = np.maximum(z, 0.0)
        if epi == N.EPI_BIAS_GELU: z = 0.5 * z * (1.0 + np.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        want = z + (old if accumulate else 0.0)
        for algo in (N.ALGO_AUTO, N.ALGO_SKINNY, N.ALGO_SKINNY_TWO_PASS):
            dC = dev.put(old)
            rocm.sgemm(m, n, k, dA, dB, dC, bias=dBias if epi != N.EPI_NONE else None, epilogue=epi, accumulate=accumulate, algo=algo)
            got = rocm.to_host(dC, (m, n))
            if epi == N.EPI_BIAS_GELU:
                assert np.abs(got - want).max() <= 1e-4 * max(1.0, np.abs(want).max()), (epi, accumulate, algo)
            else:
                assert np.array_equal(got, want.astype(np.float32)), (epi, accumulate, algo)


# ---- the decode product kernel (one workgroup per CU, tagged K-slice partials, the last wavefront to arrive adds) ----
def _gemv_gemm(dev, a, b, ldb=None, **kw):
    """a [m, k] against b [k, n] stored with row pitch ldb."""
    r = dev.r
    m, k = a.shape
    n = b.shape[1]
    ldb = ldb or n
    store = np.zeros((k, ldb), np.float32)
    store[:, :n] = b
    dA, dB = dev.put(a), dev.put(store)
    dC = dev.empty(m * n, fill=-7.0)
    r.sgemm(m, n, k, dA, dB, dC, b_strides=(ldb, 1), **kw)
    return r.to_host(dC, (m, n))


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 6, 7, 8])
def test_decode_product_kernel_integer_exact(dev, rocm, m):
    # 4096 x 4096: 32 units x 8 K slices of one trip (the form fixed at compile time); forced and as the planner's choice,
    # and repeated: every launch must find the counters of the last one back at zero
    a = synth.small_ints(m, (m, 4096), 3)
    b = synth.small_ints(m + 1, (4096, 4096), 3, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    for algo in (N.ALGO_GEMV, N.ALGO_AUTO, N.ALGO_GEMV):
        assert np.array_equal(_gemv_gemm(dev, a, b, algo=algo), want), algo
    rocm.sync()   # (an adding wavefront's expired wait would be reported here)


@pytest.mark.parametrize("m,n,k", [(4, 4096, 8192), (3, 8192, 2048), (8, 8192, 4096), (5, 16384, 1024), (2, 32768, 512), (7, 32768, 1024),
                                   (1, 4096, 16384), (6, 16384, 2048)])
def test_decode_product_kernel_other_plans_integer_exact(dev, rocm, m, n, k):
    # 8, 4, 2 slices and none at all (32768 columns: every workgroup owns its columns outright), one and several trips
    a = synth.small_ints(m, (m, k), 3)
    b = synth.small_ints(m + 1, (k, n), 3, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    assert np.array_equal(_gemv_gemm(dev, a, b, algo=N.ALGO_GEMV), want)
    assert np.array_equal(_gemv_gemm(dev, a, b), want)  # (the planner's choice, whichever kernel that is)
    rocm.sync()


@pytest.mark.parametrize("m,n,k", [(4, 4096, 4096), (1, 8192, 2048), (6, 32768, 512)])
def test_decode_product_kernel_epilogues_accumulate_and_pitch(dev, rocm, m, n, k):
    a = synth.small_ints(m, (m, k), 3); b = synth.small_ints(m + 1, (k, n), 3, stream=1)
    bias = synth.small_ints(m + 2, (n,), 5, stream=2); old = synth.small_ints(m + 3, (m, n), 9, stream=3)
    prod = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float64)
    ldb = n + 12  # rows of W 48 bytes apart from a power of two
    store = np.zeros((k, ldb), np.float32); store[:, :n] = b
    dA, dB, dBias = dev.put(a), dev.put(store), dev.put(bias)
    for epi, accumulate in [(N.EPI_NONE, False), (N.EPI_NONE, True), (N.EPI_BIAS, False), (N.EPI_BIAS, True), (N.EPI_BIAS_RELU, False),
                            (N.EPI_BIAS_GELU, False)]:
        z = prod + (bias if epi != N.EPI_NONE else 0.0)
        if epi == N.EPI_BIAS_RELU: z = np.maximum(z, 0.0)
        if epi == N.EPI_BIAS_GELU: z = 0.5 * z * (1.0 + np.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        want = z + (old if accumulate else 0.0)
        dC = dev.put(old)
        rocm.sgemm(m, n, k, dA, dB, dC, b_strides=(ldb, 1), bias=dBias if epi != N.EPI_NONE else None, epilogue=epi, accumulate=accumulate,
                   algo=N.ALGO_GEMV)
        got = rocm.to_host(dC, (m, n))
        if epi == N.EPI_BIAS_GELU:
            assert np.abs(got - want).max() <= 1e-4 * max(1.0, np.abs(want).max()), (epi, accumulate)
        else:
            assert np.array_equal(got, want.astype(np.float32)), (epi, accumulate)
    # an activation together with accumulate is not this kernel's: refused when forced, taken by another under the planner
    dC = dev.put(old)
    with pytest.raises(N.MniError):
        rocm.sgemm(m, n, k, dA, dB, dC, b_strides=(ldb, 1), bias=dBias, epilogue=N.EPI_BIAS_RELU, accumulate=True, algo=N.ALGO_GEMV)
    rocm.sgemm(m, n, k, dA, dB, dC, b_strides=(ldb, 1), bias=dBias, epilogue=N.EPI_BIAS_RELU, accumulate=True)
    assert np.array_equal(rocm.to_host(dC, (m, n)), (np.maximum(prod + bias, 0.0) + old).astype(np.float32))


def test_decode_product_kernel_normal_inputs_and_repeats(dev, rocm):
    # within the tolerance of a float64 product and of the column kernel; the same bits launch after launch (the sums
    # are formed in a fixed order whichever wavefront adds the slices up)
    m, k, n = 4, 4096, 4096
    a = synth.normal(31, (m, k), 0.02); b = synth.normal(32, (k, n), 0.02, stream=1)
    want = a.astype(np.float64) @ b.astype(np.float64)
    first = _gemv_gemm(dev, a, b, algo=N.ALGO_GEMV)
    assert max_err(first, want) <= gemm_tol(k, a, b)
    assert max_err(_gemv_gemm(dev, a, b, algo=N.ALGO_SKINNY), want) <= gemm_tol(k, a, b)
    dA, dB = dev.put(a), dev.put(b)
    dC = dev.empty(m * n, fill=-7.0)
    for _ in range(50):
        rocm.sgemm(m, n, k, dA, dB, dC, algo=N.ALGO_GEMV)
    assert np.array_equal(rocm.to_host(dC, (m, n)), first)


def test_decode_product_kernel_ineligible_is_an_error_only_when_forced(dev, rocm):
    a = synth.small_ints(1, (4, 1024), 3); b = synth.small_ints(2, (1024, 768), 3, stream=1)  # 6 units: not a multiple of 8
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    with pytest.raises(N.MniError):
        _gemv_gemm(dev, a, b, algo=N.ALGO_GEMV)
    assert np.array_equal(_gemv_gemm(dev, a, b), want)
    a33 = synth.small_ints(3, (33, 4096), 3); b33 = synth.small_ints(4, (4096, 4096), 3, stream=1)  # 33 rows
    with pytest.raises(N.MniError):
        _gemv_gemm(dev, a33, b33, algo=N.ALGO_GEMV)


@pytest.mark.parametrize("m,n,k", [(7, 4096, 4096), (8, 4096, 4096), (4, 8192, 8192), (8, 16384, 1024), (5, 32768, 512)])
def test_decode_product_both_forms_give_exact_sums(dev, rocm, m, n, k):
    # from 7 rows, or beyond 4096 columns, the 16-row form is preferred; an X whose pitch is not a whole number of 16-byte
    # pieces is outside that form and keeps the per-row-count kernels in use for these shapes
    a = synth.small_ints(m, (m, k), 3)
    b = synth.small_ints(m + 1, (k, n), 3, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    assert np.array_equal(_gemv_gemm(dev, a, b, algo=N.ALGO_GEMV), want)
    lda = k + 1
    sa = np.zeros((m, lda), np.float32); sa[:, :k] = a
    dA, dB, dC = dev.put(sa), dev.put(b), dev.empty(m * n, fill=-7.0)
    before = rocm.launch_count()
    rocm.sgemm(m, n, k, dA, dB, dC, a_strides=(lda, 1), algo=N.ALGO_GEMV)
    assert rocm.launch_count() - before == 1
    assert np.array_equal(rocm.to_host(dC, (m, n)), want)
    rocm.sync()


@pytest.mark.parametrize("m", [9, 10, 13, 16])
def test_decode_product_16_row_form_integer_exact(dev, rocm, m):
    # 4096 x 4096: 64 units of 64 columns x 4 K slices of one trip; forced and as the planner's choice, and repeated
    a = synth.small_ints(m, (m, 4096), 3)
    b = synth.small_ints(m + 1, (4096, 4096), 3, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    for algo in (N.ALGO_GEMV, N.ALGO_AUTO, N.ALGO_GEMV):
        assert np.array_equal(_gemv_gemm(dev, a, b, algo=algo), want), algo
    rocm.sync()   # (an adding wavefront's expired wait would be reported here)


@pytest.mark.parametrize("m,n,k", [(16, 8192, 8192), (12, 16384, 4096), (9, 16384, 1024), (16, 4096, 8192), (11, 2048, 8192), (16, 8192, 2048)])
def test_decode_product_16_row_form_other_plans_integer_exact(dev, rocm, m, n, k):
    # 8, 4, 2 slices and none at all (16384 columns: every workgroup owns its columns outright), one and several trips
    a = synth.small_ints(m, (m, k), 3)
    b = synth.small_ints(m + 1, (k, n), 3, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    assert np.array_equal(_gemv_gemm(dev, a, b, algo=N.ALGO_GEMV), want)
    assert np.array_equal(_gemv_gemm(dev, a, b), want)  # (the planner's choice, whichever kernel that is)
    rocm.sync()


@pytest.mark.parametrize("m,n,k", [(13, 4096, 4096), (11, 16384, 2048)])   # (K slices summed by the last arrival; no slices: every workgroup finishes its own)
def test_decode_product_16_row_form_epilogues_accumulate_pitches_and_repeats(dev, rocm, m, n, k):
    a = synth.small_ints(m, (m, k), 3); b = synth.small_ints(m + 1, (k, n), 3, stream=1)
    bias = synth.small_ints(m + 2, (n,), 5, stream=2); old = synth.small_ints(m + 3, (m, n), 9, stream=3)
    prod = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float64)
    lda, ldb, ldc = k + 8, n + 12, n + 4
    sa = np.zeros((m, lda), np.float32); sa[:, :k] = a
    sb = np.zeros((k, ldb), np.float32); sb[:, :n] = b
    dA, dB, dBias = dev.put(sa), dev.put(sb), dev.put(bias)
    for epi, accumulate in [(N.EPI_NONE, False), (N.EPI_NONE, True), (N.EPI_BIAS, False), (N.EPI_BIAS, True), (N.EPI_BIAS_RELU, False),
                            (N.EPI_BIAS_GELU, False)]:
        z = prod + (bias if epi != N.EPI_NONE else 0.0)
        if epi == N.EPI_BIAS_RELU: z = np.maximum(z, 0.0)
        if epi == N.EPI_BIAS_GELU: z = 0.5 * z * (1.0 + np.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        want = z + (old if accumulate else 0.0)
        sc = np.full((m, ldc), -5.0, np.float32); sc[:, :n] = old
        dC = dev.put(sc)
        rocm.sgemm(m, n, k, dA, dB, dC, a_strides=(lda, 1), b_strides=(ldb, 1), ldc=ldc, bias=dBias if epi != N.EPI_NONE else None, epilogue=epi,
                   accumulate=accumulate, algo=N.ALGO_GEMV)
        got = rocm.to_host(dC, (m, ldc))
        assert np.all(got[:, n:] == -5.0), "the padding of C was written"
        if epi == N.EPI_BIAS_GELU:
            assert np.abs(got[:, :n] - want).max() <= 1e-4 * max(1.0, np.abs(want).max()), (epi, accumulate)
        else:
            assert np.array_equal(got[:, :n], want.astype(np.float32)), (epi, accumulate)
    # normal inputs: within tolerance, and the same bits launch after launch
    an = synth.normal(61, (16, k), 0.02); bn = synth.normal(62, (k, n), 0.02, stream=1)
    first = _gemv_gemm(dev, an, bn, algo=N.ALGO_GEMV)
    assert max_err(first, an.astype(np.float64) @ bn.astype(np.float64)) <= gemm_tol(k, an, bn)
    dA2, dB2 = dev.put(an), dev.put(bn)
    dC2 = dev.empty(16 * n, fill=-7.0)
    for _ in range(50):
        rocm.sgemm(16, n, k, dA2, dB2, dC2, algo=N.ALGO_GEMV)
    assert np.array_equal(rocm.to_host(dC2, (16, n)), first)
    rocm.sync()


@pytest.mark.parametrize("m,n,k", [(17, 4096, 4096), (32, 4096, 4096), (24, 4096, 4096), (32, 8192, 8192), (20, 16384, 1024), (31, 16384, 4096),
                                   (32, 2048, 8192), (19, 8192, 2048), (32, 4096, 16384)])
def test_decode_product_two_sets_of_rows_integer_exact(dev, rocm, m, n, k):
    # 17 to 32 rows: the same loads of W multiplied with two sets of 16 rows; 8, 4, 2 slices and none, one and several trips
    a = synth.small_ints(m, (m, k), 3)
    b = synth.small_ints(m + 1, (k, n), 3, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    for algo in (N.ALGO_GEMV, N.ALGO_AUTO, N.ALGO_GEMV):
        assert np.array_equal(_gemv_gemm(dev, a, b, algo=algo), want), algo
    rocm.sync()


@pytest.mark.parametrize("m,n,k", [(27, 4096, 4096), (21, 16384, 1024)])
def test_decode_product_two_sets_of_rows_epilogues_accumulate_pitches_and_repeats(dev, rocm, m, n, k):
    a = synth.small_ints(m, (m, k), 3); b = synth.small_ints(m + 1, (k, n), 3, stream=1)
    bias = synth.small_ints(m + 2, (n,), 5, stream=2); old = synth.small_ints(m + 3, (m, n), 9, stream=3)
    prod = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float64)
    lda, ldb, ldc = k + 8, n + 12, n + 4
    sa = np.zeros((m, lda), np.float32); sa[:, :k] = a
    sb = np.zeros((k, ldb), np.float32); sb[:, :n] = b
    dA, dB, dBias = dev.put(sa), dev.put(sb), dev.put(bias)
    for epi, accumulate in [(N.EPI_NONE, False), (N.EPI_NONE, True), (N.EPI_BIAS, False), (N.EPI_BIAS, True), (N.EPI_BIAS_RELU, False),
                            (N.EPI_BIAS_GELU, False)]:
        z = prod + (bias if epi != N.EPI_NONE else 0.0)
        if epi == N.EPI_BIAS_RELU: z = np.maximum(z, 0.0)
        if epi == N.EPI_BIAS_GELU: z = 0.5 * z * (1.0 + np.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        want = z + (old if accumulate else 0.0)
        sc = np.full((m, ldc), -5.0, np.float32); sc[:, :n] = old
        dC = dev.put(sc)
        rocm.sgemm(m, n, k, dA, dB, dC, a_strides=(lda, 1), b_strides=(ldb, 1), ldc=ldc, bias=dBias if epi != N.EPI_NONE else None, epilogue=epi,
                   accumulate=accumulate, algo=N.ALGO_GEMV)
        got = rocm.to_host(dC, (m, ldc))
        assert np.all(got[:, n:] == -5.0), "the padding of C was written"
        if epi == N.EPI_BIAS_GELU:
            assert np.abs(got[:, :n] - want).max() <= 1e-4 * max(1.0, np.abs(want).max()), (epi, accumulate)
        else:
            assert np.array_equal(got[:, :n], want.astype(np.float32)), (epi, accumulate)
    # normal inputs: within tolerance, the same bits launch after launch, also with other decode launches in between
    an = synth.normal(71, (32, k), 0.02); bn = synth.normal(72, (k, n), 0.02, stream=1)
    first = _gemv_gemm(dev, an, bn, algo=N.ALGO_GEMV)
    assert max_err(first, an.astype(np.float64) @ bn.astype(np.float64)) <= gemm_tol(k, an, bn)
    dA2, dB2 = dev.put(an), dev.put(bn)
    dC2 = dev.empty(32 * n, fill=-7.0)
    dC4 = dev.empty(4 * n, fill=-7.0)
    for i in range(50):
        rocm.sgemm(32, n, k, dA2, dB2, dC2, algo=N.ALGO_GEMV)
        if i % 3 == 0: rocm.sgemm(4, n, k, dA2, dB2, dC4, algo=N.ALGO_GEMV)   # (the other forms share the partial sums' buffer)
        if i % 5 == 0: rocm.sgemm(16, n, k, dA2, dB2, dC2, algo=N.ALGO_GEMV)
    rocm.sgemm(32, n, k, dA2, dB2, dC2, algo=N.ALGO_GEMV)
    assert np.array_equal(rocm.to_host(dC2, (32, n)), first)
    rocm.sync()


@pytest.mark.parametrize("m", [12, 29])
def test_decode_product_16_row_forms_take_operands_off_a_128_byte_boundary(dev, rocm, m):
    # X, W and C 16 bytes (X: 48) past a 128-byte boundary, as rows of a larger tensor are: the loads of X into LDS then start in
    # the middle of a cache line; several trips and K slices (8192 x 8192: 2 slices of 4 trips)
    for n, k in ((4096, 4096), (8192, 8192)):
        a = synth.small_ints(m, (m, k), 3); b = synth.small_ints(m + 1, (k, n), 3, stream=1)
        want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
        fa = np.zeros(m * k + 12, np.float32); fa[12:] = a.ravel()
        fb = np.zeros(k * n + 4, np.float32); fb[4:] = b.ravel()
        dA, dB = dev.put(fa), dev.put(fb)
        dC = dev.empty(m * n + 4, fill=-7.0)
        before = rocm.launch_count()
        rocm.sgemm(m, n, k, dA + 4 * 12, dB + 4 * 4, dC + 4 * 4, algo=N.ALGO_GEMV)
        assert rocm.launch_count() - before == 1
        got = rocm.to_host(dC, (m * n + 4,))
        assert np.all(got[:4] == -7.0)
        assert np.array_equal(got[4:].reshape(m, n), want)
    rocm.sync()


# ---- few rows against a wide K-contiguous operand (a weight stored [out, in]): a wavefront per 16 columns, all of K ----
@pytest.mark.parametrize("m,n,k", [(16, 50304, 768), (9, 20000, 256), (32, 16400, 512), (17, 16384, 960), (12, 33000, 1984), (1, 4096, 64),
                                   (8, 1000, 128), (32, 70, 320), (16, 16, 1984), (5, 4099, 768), (3, 9001, 512), (8, 16384, 768),
                                   (4, 5000, 8192), (8, 6144, 4096), (2, 300, 4096), (16, 5120, 2048), (7, 2052, 4032)])
def test_fewrows_nt_kernel_integer_exact(dev, rocm, m, n, k):
    # one to eight sets of four rows, column counts off a multiple of 16, K at both ends of what fits LDS (8192 values of 4 rows,
    # 4096 of 8, 2048 of 16), K off a multiple of the ring of loads, fewer column groups than CUs; forced and as the planner's choice
    a = synth.small_ints(m + n, (m, k), 3)
    bt = synth.small_ints(n + k, (n, k), 3, stream=1)
    want = (a.astype(np.int64) @ bt.T.astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a, bt, False, True, algo=N.ALGO_FEWROWS_NT)[0], want)
    assert np.array_equal(run_gemm(dev, a, bt, False, True)[0], want)  # (the planner's choice, whichever kernel that is)


@pytest.mark.parametrize("m,n,k", [(16, 20000, 768), (24, 16390, 256)])
def test_fewrows_nt_kernel_epilogues_accumulate_and_pitches(dev, rocm, m, n, k):
    a = synth.small_ints(m, (m, k), 3); bt = synth.small_ints(m + 1, (n, k), 3, stream=1)
    bias = synth.small_ints(m + 2, (n,), 5, stream=2); old = synth.small_ints(m + 3, (m, n), 9, stream=3)
    prod = (a.astype(np.int64) @ bt.T.astype(np.int64)).astype(np.float64)
    lda, ldb, ldc = k + 8, k + 12, n + 3  # pitches off their extents (operands in whole 16-byte pieces, C any)
    sa = np.zeros((m, lda), np.float32); sa[:, :k] = a
    sb = np.zeros((n, ldb), np.float32); sb[:, :k] = bt
    dA, dB, dBias = dev.put(sa), dev.put(sb), dev.put(bias)
    for epi, accumulate in [(N.EPI_NONE, False), (N.EPI_NONE, True), (N.EPI_BIAS, False), (N.EPI_BIAS, True), (N.EPI_BIAS_RELU, True),
                            (N.EPI_BIAS_GELU, False)]:
        z = prod + (bias if epi != N.EPI_NONE else 0.0)
        if epi == N.EPI_BIAS_RELU: z = np.maximum(z, 0.0)
        if epi == N.EPI_BIAS_GELU: z = 0.5 * z * (1.0 + np.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        want = z + (old if accumulate else 0.0)
        sc = np.full((m, ldc), -5.0, np.float32); sc[:, :n] = old
        dC = dev.put(sc)
        rocm.sgemm(m, n, k, dA, dB, dC, a_strides=(lda, 1), b_strides=(1, ldb), ldc=ldc, bias=dBias if epi != N.EPI_NONE else None, epilogue=epi,
                   accumulate=accumulate, algo=N.ALGO_FEWROWS_NT)
        got = rocm.to_host(dC, (m, ldc))
        assert np.all(got[:, n:] == -5.0), "the padding of C was written"
        if epi == N.EPI_BIAS_GELU:
            assert np.abs(got[:, :n] - want).max() <= 1e-4 * max(1.0, np.abs(want).max()), (epi, accumulate)
        else:
            assert np.array_equal(got[:, :n], want.astype(np.float32)), (epi, accumulate)


def test_fewrows_nt_kernel_normal_inputs_and_what_it_refuses(dev, rocm):
    m, n, k = 16, 50304, 768
    a = synth.normal(51, (m, k), 0.05); bt = synth.normal(52, (n, k), 0.05, stream=1)
    want = a.astype(np.float64) @ bt.T.astype(np.float64)
    got = run_gemm(dev, a, bt, False, True, algo=N.ALGO_FEWROWS_NT)[0]
    assert max_err(got, want) <= gemm_tol(k, a, bt)
    assert np.array_equal(got, run_gemm(dev, a, bt, False, True, algo=N.ALGO_FEWROWS_NT)[0])
    # 40 rows; K off a multiple of 64; a row-major B  (a K beyond what LDS holds of A goes to the form with K in slices)
    for mm, kk, tb in ((40, 256, True), (16, 208, True), (16, 256, False)):
        aa = synth.small_ints(1, (mm, kk), 3)
        bb = synth.small_ints(2, (20000, kk) if tb else (kk, 20000), 3, stream=1)
        with pytest.raises(N.MniError, match="few-rows kernel for a K-contiguous B"):
            run_gemm(dev, aa, bb, False, tb, algo=N.ALGO_FEWROWS_NT)


@pytest.mark.parametrize("m,n,k,split", [(16, 4096, 4096, 0), (16, 4096, 4096, 8), (16, 4096, 4096, 16), (9, 1000, 2048, 0), (1, 4096, 4096, 0),
                                          (4, 2050, 5120, 5), (8, 11008, 4096, 0), (12, 192, 2816, 3), (16, 64, 512, 2), (32, 4096, 4096, 0),
                                          (17, 1111, 1536, 2), (24, 8192, 3072, 0), (3, 70, 1024, 4), (13, 3000, 2112, 0), (32, 500, 1088, 0),
                                          (7, 4096, 2240, 3)])
def test_fewrows_nt_kernel_in_k_slices_integer_exact(dev, rocm, m, n, k, split):
    # K beyond what LDS holds of A: workgroups of 64 columns x one K slice, the last slice of a column block to arrive adds
    # them.  Even and uneven slices, column counts off a multiple of 64 and under one block, 1 to 32 rows; forced (with
    # and without a slice count) and as the planner's choice; twice in a row (the counters wrap back to zero)
    a = synth.small_ints(m + n, (m, k), 3)
    bt = synth.small_ints(n + k, (n, k), 3, stream=1)
    want = (a.astype(np.int64) @ bt.T.astype(np.int64)).astype(np.float32)
    for _ in range(2):
        assert np.array_equal(run_gemm(dev, a, bt, False, True, algo=N.ALGO_FEWROWS_NT, split_k=split)[0], want)
    assert np.array_equal(run_gemm(dev, a, bt, False, True)[0], want)  # (the planner's choice, whichever kernel that is)


@pytest.mark.parametrize("m,n,k,split", [(16, 4100, 2048, 2), (30, 2000, 1536, 3)])
def test_fewrows_nt_kernel_in_k_slices_epilogues_accumulate_and_pitches(dev, rocm, m, n, k, split):
    a = synth.small_ints(m, (m, k), 3); bt = synth.small_ints(m + 1, (n, k), 3, stream=1)
    bias = synth.small_ints(m + 2, (n,), 5, stream=2); old = synth.small_ints(m + 3, (m, n), 9, stream=3)
    prod = (a.astype(np.int64) @ bt.T.astype(np.int64)).astype(np.float64)
    lda, ldb, ldc = k + 8, k + 12, n + 3  # pitches off their extents (operands in whole 16-byte pieces, C any)
    sa = np.zeros((m, lda), np.float32); sa[:, :k] = a
    sb = np.zeros((n, ldb), np.float32); sb[:, :k] = bt
    dA, dB, dBias = dev.put(sa), dev.put(sb), dev.put(bias)
    for epi, accumulate in [(N.EPI_NONE, False), (N.EPI_NONE, True), (N.EPI_BIAS, False), (N.EPI_BIAS, True), (N.EPI_BIAS_RELU, True),
                            (N.EPI_BIAS_GELU, False)]:
        z = prod + (bias if epi != N.EPI_NONE else 0.0)
        if epi == N.EPI_BIAS_RELU: z = np.maximum(z, 0.0)
        if epi == N.EPI_BIAS_GELU: z = 0.5 * z * (1.0 + np.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
        want = z + (old if accumulate else 0.0)
        sc = np.full((m, ldc), -5.0, np.float32); sc[:, :n] = old
        dC = dev.put(sc)
        rocm.sgemm(m, n, k, dA, dB, dC, a_strides=(lda, 1), b_strides=(1, ldb), ldc=ldc, bias=dBias if epi != N.EPI_NONE else None, epilogue=epi,
                   accumulate=accumulate, algo=N.ALGO_FEWROWS_NT, split_k=split)
        got = rocm.to_host(dC, (m, ldc))
        assert np.all(got[:, n:] == -5.0), "the padding of C was written"
        if epi == N.EPI_BIAS_GELU:
            assert np.abs(got[:, :n] - want).max() <= 1e-4 * max(1.0, np.abs(want).max()), (epi, accumulate)
        else:
            assert np.array_equal(got[:, :n], want.astype(np.float32)), (epi, accumulate)


def test_fewrows_nt_kernel_in_k_slices_normal_inputs_and_what_it_refuses(dev, rocm):
    m, n, k = 16, 4096, 4096
    a = synth.normal(61, (m, k), 0.05); bt = synth.normal(62, (n, k), 0.05, stream=1)
    want = a.astype(np.float64) @ bt.T.astype(np.float64)
    got = run_gemm(dev, a, bt, False, True)[0]
    assert max_err(got, want) <= gemm_tol(k, a, bt)
    for _ in range(3):  # the same bits whoever of a column block's slices arrives last
        assert np.array_equal(got, run_gemm(dev, a, bt, False, True)[0])
    assert np.array_equal(got, run_gemm(dev, a, bt, False, True, algo=N.ALGO_FEWROWS_NT, split_k=4)[0])
    # slices longer than 16 steps of 64; more slices than steps; more than 16 slices; K off a multiple of 64; 32 rows of a K
    # that 16 slices of 12 steps do not cover
    for mm, kk, split in ((16, 4096, 2), (16, 256, 5), (16, 8192, 17), (16, 2400, 3), (32, 12352, 0)):
        aa = synth.small_ints(1, (mm, kk), 3)
        bb = synth.small_ints(2, (512, kk), 3, stream=1)
        with pytest.raises(N.MniError, match="few-rows kernel for a K-contiguous B"):
            run_gemm(dev, aa, bb, False, True, algo=N.ALGO_FEWROWS_NT, split_k=split)


def test_fewrows_kernels_share_their_counters_launch_after_launch(dev, rocm):
    # the sliced kernel for a K-contiguous B and the few-rows kernel for a row-major B count their K slices in at the same
    # array of counters (every count wraps back to zero with its last arrival): products of different unit and slice counts
    # one after the other, ten rounds, every result integer-exact
    cases = []
    for m, n, k, tb, split, algo in ((16, 4096, 4096, True, 4, N.ALGO_FEWROWS_NT), (8, 1000, 2048, True, 2, N.ALGO_FEWROWS_NT),
                                     (24, 1280, 4096, False, 0, N.ALGO_FEWROWS), (5, 2112, 3072, True, 3, N.ALGO_FEWROWS_NT),
                                     (12, 640, 8192, False, 0, N.ALGO_FEWROWS), (3, 520, 4096, True, 16, N.ALGO_FEWROWS_NT)):
        a = synth.small_ints(m + n, (m, k), 3)
        b = synth.small_ints(n + k, (n, k) if tb else (k, n), 3, stream=1)
        want = (a.astype(np.int64) @ (b.T if tb else b).astype(np.int64)).astype(np.float32)
        cases.append((m, n, k, dev.put(a), dev.put(b), dev.empty(m * n, fill=-7.0), tb, split, algo, want))
    for _ in range(10):
        for m, n, k, dA, dB, dC, tb, split, algo, want in cases:
            rocm.sgemm(m, n, k, dA, dB, dC, b_strides=(1, k) if tb else (n, 1), algo=algo, split_k=split)
    for m, n, k, dA, dB, dC, tb, split, algo, want in cases:
        assert np.array_equal(rocm.to_host(dC, (m, n)), want), (m, n, k)


@pytest.mark.parametrize("m", [1, 3, 5, 7])
def test_skinny_cols_decode_shape_normal_inputs(dev, m):
    # the kernels specialised for a row count: within tolerance of a float64 product and of the two-launch form,
    # and the same bits launch after launch
    k, n = 4096, 1024
    a = synth.normal(m, (m, k)); b = synth.normal(m + 1, (k, n), stream=1)
    one = run_gemm(dev, a, b, algo=N.ALGO_SKINNY)[0]
    assert np.array_equal(one, run_gemm(dev, a, b, algo=N.ALGO_SKINNY)[0])
    ref = a.astype(np.float64) @ b.astype(np.float64)
    assert np.abs(one - ref).max() <= gemm_tol(k, a, b)
    assert max_err(one, run_gemm(dev, a, b, algo=N.ALGO_SKINNY_TWO_PASS)[0]) <= gemm_tol(k, a, b)


@pytest.mark.parametrize("algo", SKINNY_ALGOS)
def test_skinny_cols_many_slices_few_columns(dev, algo):
    # one column group, hundreds of K slices: more arrival flags than lanes
    a = synth.small_ints(1, (4, 32768), 2)
    b = synth.small_ints(2, (32768, 96), 2, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a, b, algo=algo)[0], want)
    assert np.array_equal(run_gemm(dev, a, b, algo=algo, split_k=200)[0], want)


@pytest.mark.parametrize("algo", SKINNY_ALGOS)
def test_skinny_cols_batched_units_epilogue_accumulate(dev, rocm, algo):
    # 5 batches x 3 column groups = 15 units over the XCDs; bias + ReLU and accumulate in the slice reduction
    a = synth.small_ints(1, (5, 6, 1024), 3)
    w = synth.small_ints(2, (5, 1024, 640), 3, stream=1)
    bias = synth.small_ints(3, (640,), 3, stream=2)
    c0 = synth.small_ints(4, (5, 6, 640), 3, stream=3)
    dA, dW, dbias, dC = dev.put(a), dev.put(w), dev.put(bias), dev.put(c0)
    rocm.sgemm(6, 640, 1024, dA, dW, dC, batch=5, a_batch=(6 * 1024, 5), b_batch=(1024 * 640, 5),
               bias=dbias, epilogue=N.EPI_BIAS_RELU, accumulate=True, split_k=7, algo=algo)
    z = np.einsum("bmk,bkn->bmn", a.astype(np.int64), w.astype(np.int64)) + bias.astype(np.int64)
    assert np.array_equal(rocm.to_host(dC, (5, 6, 640)), (np.maximum(z, 0) + c0).astype(np.float32))


def test_skinny_single_launch_repeats_and_matches_two_pass(dev, rocm):
    # the arrival flags are reused launch after launch (fresh epoch each time)
    a = synth.normal(1, (4, 4096), 1.0)
    w = synth.normal(2, (4096, 1024), 0.05, stream=1)
    two = run_gemm(dev, a, w, algo=N.ALGO_SKINNY_TWO_PASS)[0]
    dA, dW, dC = dev.put(a), dev.put(w), dev.empty(4 * 1024)
    first = None
    for _ in range(50):
        rocm.sgemm(4, 1024, 4096, dA, dW, dC, algo=N.ALGO_SKINNY)
        got = rocm.to_host(dC, (4, 1024))
        first = got if first is None else first
        assert np.array_equal(got, first)  # fixed summation order: the same bits every launch
    assert max_err(first, two) <= gemm_tol(4096, a, w)


@pytest.mark.parametrize("nin,nout,rows,batch", [(128, 128, 8, 1), (100, 132, 7, 1), (33, 4, 1, 1), (300, 260, 33, 2), (257, 516, 128, 3),
                                                 (64, 64, 2, 1), (1000, 640, 5, 1), (31, 1028, 19, 4), (260, 132, 301, 1), (128, 256, 512, 2)])
def test_outer_product_kernel_integer_exact(dev, rocm, nin, nout, rows, batch):
    # dW[b] = X[b]^T dY[b] of a small batch: K = its rows, A the transposed view of X, both operands contiguous along
    # the output axes.  Forced and as planned; overwriting and accumulating; edges in both extents, odd K.
    x = synth.small_ints(rows + nin, (batch, rows, nin), 3); dy = synth.small_ints(rows + nout, (batch, rows, nout), 3, stream=1)
    old = synth.small_ints(5, (batch, nin, nout), 7, stream=2)
    want = np.einsum("bki,bkn->bin", x.astype(np.int64), dy.astype(np.int64)).astype(np.float32)
    dX, dY = dev.put(x), dev.put(dy)
    for algo in (N.ALGO_OUTER, N.ALGO_AUTO, N.ALGO_MFMA_SMALL):
        for accumulate in (False, True):
            dC = dev.put(old)
            rocm.sgemm(nin, nout, rows, dX, dY, dC, batch=batch, a_strides=(1, nin), a_batch=(rows * nin, batch),
                       b_batch=(rows * nout, batch), accumulate=accumulate, algo=algo)
            assert np.array_equal(rocm.to_host(dC, (batch, nin, nout)), want + (old if accumulate else 0)), (algo, accumulate)
    # one X against a dY per batch (X's batch count 1), into a padded C
    dC = dev.empty(batch * nin * (nout + 4), fill=-7.0)
    rocm.sgemm(nin, nout, rows, dX, dY, dC, batch=batch, a_strides=(1, nin), a_batch=(0, 1), b_batch=(rows * nout, batch),
               ldc=nout + 4, c_batch_stride=nin * (nout + 4), algo=N.ALGO_OUTER)
    got = rocm.to_host(dC, (batch, nin, nout + 4))
    want1 = np.einsum("ki,bkn->bin", x[0].astype(np.int64), dy.astype(np.int64)).astype(np.float32)
    assert np.array_equal(got[:, :, :nout], want1) and np.all(got[:, :, nout:] == -7.0)


def test_more_batches_than_a_grid_dimension_holds_go_to_the_tile_kernel(dev, rocm):
    # 70000 x (32 x 64 x 32) with A given as its transpose: what the outer-product kernel would take but for its batch in
    # grid dimension z (65535); the planner must fall through to the tile kernel instead of failing, and a forced
    # outer-product launch must say why it cannot
    batch, m, n, k = 70000, 32, 64, 32
    x = synth.small_ints(1, (1, k, m), 3); dy = synth.small_ints(2, (1, k, n), 3, stream=1)
    want = (x[0].astype(np.int64).T @ dy[0].astype(np.int64)).astype(np.float32)
    dX, dY = dev.put(x), dev.put(dy)
    dC = dev.empty(batch * m * n, fill=-7.0)
    rocm.sgemm(m, n, k, dX, dY, dC, batch=batch, a_strides=(1, m), a_batch=(0, 1), b_batch=(0, 1))
    got = rocm.to_host(dC, (batch, m, n))
    assert np.array_equal(got[0], want) and np.array_equal(got[65535], want) and np.array_equal(got[-1], want)
    assert np.all(got == want[None])
    with pytest.raises(N.MniError):
        rocm.sgemm(m, n, k, dX, dY, dC, batch=batch, a_strides=(1, m), a_batch=(0, 1), b_batch=(0, 1), algo=N.ALGO_OUTER)


def test_outer_product_kernel_is_the_plan_for_a_small_batch_weight_gradient_and_refuses_other_layouts(dev, rocm):
    rows, nin, nout = 16, 2048, 4096
    x = synth.normal(1, (rows, nin)); dy = synth.normal(2, (rows, nout), stream=1)
    dX, dY, dC = dev.put(x), dev.put(dy), dev.empty(nin * nout)
    before = rocm.launch_count()
    rocm.sgemm(nin, nout, rows, dX, dY, dC, a_strides=(1, nin))
    assert rocm.launch_count() - before == 1
    got = rocm.to_host(dC, (nin, nout))
    ref = x.astype(np.float64).T @ dy.astype(np.float64)
    assert np.abs(got - ref).max() <= gemm_tol(rows, x, dy)
    forced = dev.empty(nin * nout)
    rocm.sgemm(nin, nout, rows, dX, dY, forced, a_strides=(1, nin), algo=N.ALGO_OUTER)
    assert np.array_equal(rocm.to_host(forced, (nin, nout)), got)  # the planner's choice was this kernel
    bias = dev.put(np.zeros(nout, np.float32))
    for kw in (dict(), dict(a_strides=(1, nin), bias=bias, epilogue=N.EPI_BIAS), dict(a_strides=(1, nin), split_k=2)):
        with pytest.raises(N.MniError):   # K-contiguous A; an epilogue; K slices
            rocm.sgemm(nin, nout, rows, dX, dY, dC, algo=N.ALGO_OUTER, **kw)
    with pytest.raises(N.MniError):       # K beyond the kernel's limit
        rocm.sgemm(32, 32, 600, dX, dY, dC, a_strides=(1, 32), algo=N.ALGO_OUTER)


@pytest.mark.parametrize("batch,m,n,k", [(4096, 8, 8, 64), (20000, 3, 3, 3), (300, 16, 16, 128), (2048, 1, 64, 64), (2048, 64, 1, 64), (70, 2, 100, 7)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, True)])
def test_large_batches_of_tiny_products_integer_exact(dev, batch, m, n, k, ta, tb):
    # thousands of products of at most 256 outputs each: one thread per output over the whole batch, not a padded
    # 64 x 64 tile per product (65536 x (4 x 4 x 4): 223 us -> 6)
    a = synth.small_ints(batch + m, (batch, k, m) if ta else (batch, m, k), 3)
    b = synth.small_ints(batch + n, (batch, n, k) if tb else (batch, k, n), 3, stream=1)
    opa = a.transpose(0, 2, 1) if ta else a
    opb = b.transpose(0, 2, 1) if tb else b
    want = np.einsum("bmk,bkn->bmn", opa.astype(np.int64), opb.astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a, b, ta=ta, tb=tb), want)


@pytest.mark.parametrize("batch,m,n,k", [(256, 1, 4096, 128), (32, 1, 8192, 64), (1024, 1, 512, 64), (16, 1, 1000, 100), (40, 1, 333, 7), (64, 1, 2048, 4),
                                         (4, 1, 65536, 64), (32, 1, 4096, 256), (16, 1, 4096, 384), (128, 2, 4096, 64), (64, 2, 1024, 128),
                                         (16, 64, 4096, 64), (16, 4096, 32, 64), (16, 96, 1024, 64)])
def test_few_rows_per_batch_against_k_contiguous_b_integer_exact(dev, batch, m, n, k):
    # q[B, 1, d] . K[B, n, d]^T, the scores of one new token per head: a thread per score reads its own row of K
    # (256 x (1 x 4096 x 128): 166 us through tiles -> 122); K = 384 goes to the dots kernel, two rows of K <= 64 to the
    # thread-per-output kernel, up to 64 rows or columns of K <= 64 to 64 x 64 tiles rather than 128 x 128 panels
    a = synth.small_ints(batch + k, (batch, m, k), 3)
    b = synth.small_ints(batch + n, (batch, n, k), 3, stream=1)
    want = np.einsum("bmk,bnk->bmn", a.astype(np.int64), b.astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a, b, tb=True), want)


@pytest.mark.parametrize("batch,m,n,k,ta,tb", [(512, 64, 64, 64, True, False), (512, 64, 32, 64, True, False), (256, 80, 80, 80, True, False),
                                               (512, 32, 64, 32, True, False), (1024, 16, 64, 16, False, False), (1024, 16, 64, 16, True, False),
                                               (256, 16, 256, 32, True, False), (256, 16, 256, 32, False, False), (2048, 16, 16, 64, False, True),
                                               (1024, 16, 16, 32, False, True), (300, 12, 100, 20, False, False), (3, 4096, 4160, 16, True, False)])
def test_many_small_products_under_the_planner_integer_exact(dev, batch, m, n, k, ta, tb):
    # attention-sized products of short sequences, forward and backward: which of the outer-product kernel (32 x 128 blocks),
    # 64 x 64 tiles, the 16-row column kernel and the thread-per-output kernel takes them depends on how much each would pad
    a = synth.small_ints(batch + m, (batch, k, m) if ta else (batch, m, k), 3)
    b = synth.small_ints(batch + n, (batch, n, k) if tb else (batch, k, n), 3, stream=1)
    opa = a.transpose(0, 2, 1) if ta else a
    opb = b.transpose(0, 2, 1) if tb else b
    want = np.einsum("bmk,bkn->bmn", opa.astype(np.int64), opb.astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a, b, ta=ta, tb=tb), want)


@pytest.mark.parametrize("m,n,k,ta,tb", [(16384, 16, 16, False, False), (16384, 16, 16, False, True), (784, 128, 64, True, False), (1024, 256, 32, False, False),
                                         (4096, 10, 128, False, False), (4096, 64, 10, False, True), (64, 256, 256, False, True), (64, 512, 512, False, True),
                                         (256, 512, 512, False, False), (64, 1024, 256, False, True), (16, 16, 16384, True, False), (64, 10, 16384, True, False),
                                         (128, 10, 1024, True, False), (300, 300, 64, True, False)])
def test_small_layers_under_the_planner_integer_exact(dev, m, n, k, ta, tb):
    # the products of Linear layers of 10 to 512 features under batches of 64 to 16384 rows (forward, dX, dW): thread-per-output
    # kernel up to 2^18 outputs, short K slices for a handful of 64 x 64 tiles, no 16-row column kernel under 256 columns
    a = synth.small_ints(m + k, (k, m) if ta else (m, k), 2)
    b = synth.small_ints(n + k, (n, k) if tb else (k, n), 2, stream=1)
    want = ((a.T if ta else a).astype(np.int64) @ (b.T if tb else b).astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a, b, ta, tb)[0], want)


@pytest.mark.parametrize("batch,m,n,k", [(64, 16, 132, 256), (100, 1, 64, 512), (7, 33, 260, 100), (3, 128, 128, 64), (40, 5, 1024, 768)])
def test_batches_of_a_against_one_shared_b_integer_exact(dev, rocm, batch, m, n, k):
    # x[B, T, d] . W[d, n]: the batches of A are stacked at a uniform pitch, as are those of C, so the library runs one
    # product of B x T rows (1024 products of one row each took 6.5 ms against 0.3).  Same values as batch by batch; not
    # collapsed when C's batches are padded apart or A is itself broadcast.
    a = synth.small_ints(batch + m, (batch, m, k), 3); b = synth.small_ints(n + k, (1, k, n), 3, stream=1)
    want = np.einsum("bmk,kn->bmn", a.astype(np.int64), b[0].astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a, b), want)
    bias = synth.small_ints(9, (n,), 5, stream=2)
    dA, dB, dBias = dev.put(a), dev.put(b), dev.put(bias)
    pad = m * n + 8                                        # C's batches apart: stays a batch of products
    dC = dev.empty(batch * pad, fill=-7.0)
    rocm.sgemm(m, n, k, dA, dB, dC, batch=batch, a_batch=(m * k, batch), b_batch=(0, 1), c_batch_stride=pad, bias=dBias, epilogue=N.EPI_BIAS)
    got = rocm.to_host(dC, (batch, pad))
    assert np.array_equal(got[:, :m * n].reshape(batch, m, n), want + bias) and np.all(got[:, m * n:] == -7.0)
    dC2 = dev.empty(batch * m * n, fill=-7.0)             # the same, C contiguous: one product
    before = rocm.launch_count()
    rocm.sgemm(m, n, k, dA, dB, dC2, batch=batch, a_batch=(m * k, batch), b_batch=(0, 1), bias=dBias, epilogue=N.EPI_BIAS)
    assert rocm.launch_count() - before <= 3
    assert np.array_equal(rocm.to_host(dC2, (batch, m, n)), want + bias)


@pytest.mark.parametrize("m,n,k", [(1001, 1003, 999), (1538, 1537, 1400), (2048, 1027, 1500), (1281, 2050, 1300)])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_big_products_with_edges_off_a_multiple_of_four_integer_exact(dev, rocm, m, n, k, ta, tb):
    # An operand contiguous along M or N with that extent off a multiple of 4: the product is cut into the part that
    # ends on a multiple of 4 and a strip of 1 to 3 rows / columns (both, and their corner, when both operands are
    # such).  Same sums; with a bias and accumulation across the cut as well.
    a = synth.small_ints(m + k, (k, m) if ta else (m, k), 3)
    b = synth.small_ints(n + k, (n, k) if tb else (k, n), 3, stream=1)
    opa = a.T if ta else a
    opb = b.T if tb else b
    want = (opa.astype(np.int64) @ opb.astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a, b, ta=ta, tb=tb)[0], want)
    bias = synth.small_ints(7, (n,), 5, stream=2); old = synth.small_ints(8, (m, n), 9, stream=3)
    dA, dB, dBias, dC = dev.put(a), dev.put(b), dev.put(bias), dev.put(old)
    rocm.sgemm(m, n, k, dA, dB, dC, a_strides=(1, m) if ta else None, b_strides=(1, k) if tb else None, bias=dBias,
               epilogue=N.EPI_BIAS_RELU, accumulate=True)
    z = np.maximum(want.astype(np.float64) + bias, 0.0) + old
    assert np.array_equal(rocm.to_host(dC, (m, n)), z.astype(np.float32))


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 7, 8, 9, 10, 13, 17])
def test_few_output_columns_under_a_tall_operand_integer_exact(dev, rocm, n):
    # A head with a few outputs: the [K, n] weight is small and, for most n, not laid out for 16-byte loads.  The
    # planner copies it into a K-contiguous layout first (for the dots kernel up to 8 columns, for the tile
    # kernel beyond) when the tall operand is big enough to pay for the extra launch; same sums either way.
    m, k = 2048, 640
    a = synth.small_ints(n, (m, k), 3); b = synth.small_ints(n + 1, (k, n), 3, stream=1)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a, b)[0], want)
    # batched, with one weight per batch and with a shared one
    a3 = synth.small_ints(n + 2, (3, 1024, 512), 3); b3 = synth.small_ints(n + 3, (3, 512, n), 3, stream=1)
    want3 = np.einsum("bmk,bkn->bmn", a3.astype(np.int64), b3.astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a3, b3), want3)
    want1 = np.einsum("bmk,kn->bmn", a3.astype(np.int64), b3[0].astype(np.int64)).astype(np.float32)
    assert np.array_equal(run_gemm(dev, a3, b3[:1]), want1)
    # with a bias along the few columns, accumulating
    bias = synth.small_ints(n + 4, (n,), 5, stream=2); old = synth.small_ints(n + 5, (m, n), 9, stream=3)
    dA, dB, dBias, dC = dev.put(a), dev.put(b), dev.put(bias), dev.put(old)
    rocm.sgemm(m, n, k, dA, dB, dC, bias=dBias, epilogue=N.EPI_BIAS_RELU, accumulate=True)
    z = np.maximum(want.astype(np.float64) + bias, 0.0) + old
    assert np.array_equal(rocm.to_host(dC, (m, n)), z.astype(np.float32))


@pytest.mark.parametrize("m", [1, 4, 16])
def test_skinny_dots_integer_exact(dev, m):
    a = synth.small_ints(m, (m, 1024), 4)
    bt = synth.small_ints(m + 1, (300, 1024), 4, stream=1)  # B stored as its transpose: K contiguous
    got = run_gemm(dev, a, bt, tb=True, algo=N.ALGO_SKINNY)[0]
    assert np.array_equal(got, (a.astype(np.int64) @ bt.T.astype(np.int64)).astype(np.float32))


@pytest.mark.parametrize("algo", SKINNY_ALGOS)
def test_skinny_few_output_columns(dev, algo):
    # [rows, K] x [K, 4]: the few columns become the skinny side (C^T = B^T A^T)
    at = synth.small_ints(1, (64, 1000), 4)  # A stored K x M
    b = synth.small_ints(2, (64, 4), 4, stream=1)
    got = run_gemm(dev, at, b, ta=True, algo=algo)[0]
    assert np.array_equal(got, (at.T.astype(np.int64) @ b.astype(np.int64)).astype(np.float32))
    a = synth.small_ints(3, (1000, 64), 4)
    bt = synth.small_ints(4, (4, 64), 4, stream=1)
    got = run_gemm(dev, a, bt, tb=True, algo=N.ALGO_SKINNY)[0]
    assert np.array_equal(got, (a.astype(np.int64) @ bt.T.astype(np.int64)).astype(np.float32))


def test_skinny_batched_and_vs_oracle(dev, oracle_native):
    a = synth.normal(1, (3, 2, 4096), 0.02)
    w = synth.normal(2, (1, 4096, 512), 0.02, stream=1)
    got = run_gemm(dev, a, w, algo=N.ALGO_SKINNY)
    for i in range(3):
        assert max_err(got[i], oracle_native.sgemm_ikj(a[i], w[0])) <= gemm_tol(4096, a, w)


@pytest.mark.parametrize("algo", SKINNY_ALGOS)
def test_skinny_cols_units_sharing_a_cache_line(dev, algo):
    # N = 2100: 9 column groups, and rows of the partials that are not whole
    # 128-byte lines, so the end of one unit's row shares a line with the
    # start of another unit's row (both units on the same XCD: groups 0 and 8)
    a = synth.normal(1, (4, 4096), 0.02)
    w = synth.normal(2, (4096, 2100), 0.02, stream=1)
    want = a.astype(np.float64) @ w.astype(np.float64)
    first = run_gemm(dev, a, w, algo=algo)[0]
    assert max_err(first, want) <= gemm_tol(4096, a, w)
    for _ in range(20):
        assert np.array_equal(run_gemm(dev, a, w, algo=algo)[0], first)
    ai = synth.small_ints(3, (4, 4096), 3)
    wi = synth.small_ints(4, (4096, 2100), 3, stream=1)
    assert np.array_equal(run_gemm(dev, ai, wi, algo=algo)[0], (ai.astype(np.int64) @ wi.astype(np.int64)).astype(np.float32))


def test_skinny_ineligible_is_an_error_only_when_forced(dev, rocm):
    a = synth.small_ints(1, (40, 30), 3)
    b = synth.small_ints(2, (30, 50), 3, stream=1)
    with pytest.raises(N.MniError, match="not eligible"):
        run_gemm(dev, a, b, algo=N.ALGO_SKINNY)
    a = synth.small_ints(1, (3, 30), 3)
    b = synth.small_ints(2, (30, 50), 3, stream=1)  # N % 4 != 0: auto falls back to MFMA
    got = run_gemm(dev, a, b)[0]
    assert np.array_equal(got, (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32))


# ---- argument checking: status codes, never an abort --------------------------------------

def test_invalid_arguments_are_reported(dev, rocm):
    dC = dev.empty(16)
    dA = dev.put(np.zeros((4, 4), np.float32))
    with pytest.raises(N.MniError, match="negative"):
        rocm.sgemm(-1, 4, 4, dA, dA, dC)
    with pytest.raises(N.MniError, match="ldc"):
        rocm.sgemm(4, 4, 4, dA, dA, dC, ldc=2)
    with pytest.raises(N.MniError, match="null"):
        rocm.sgemm(4, 4, 4, None, dA, dC)
    with pytest.raises(N.MniError, match="bias"):
        rocm.sgemm(4, 4, 4, dA, dA, dC, epilogue=N.EPI_BIAS)
    with pytest.raises(N.MniError, match="batch_count"):
        rocm.sgemm(4, 4, 4, dA, dA, dC, a_batch=(0, 0))


# ---- support kernels of the C ABI ----------------------------------------------------------

def test_strided_copy_add_bias_colsum_axpy_fill(dev, rocm):
    x = synth.normal(1, (3, 40, 50))
    src = dev.put(x)
    dst = dev.empty(x.size)
    rocm.strided_copy(dst, src, [3, 50, 40], [2000, 1, 50])  # swap last two dims
    assert np.array_equal(rocm.to_host(dst, (3, 50, 40)), x.transpose(0, 2, 1))
    rocm.strided_copy(dst, src, [50, 3, 40], [1, 2000, 50])  # general permutation
    assert np.array_equal(rocm.to_host(dst, (50, 3, 40)), x.transpose(2, 0, 1))
    a = synth.small_ints(2, (300, 96), 5)
    bias = synth.small_ints(3, (96,), 5, stream=1)
    da, db, out = dev.put(a), dev.put(bias), dev.empty(a.size)
    rocm.add_bias(out, da, db, 300, 96)
    assert np.array_equal(rocm.to_host(out, (300, 96)), a + bias)
    cs = dev.empty(96)
    rocm.colsum(cs, da, 300, 96)
    assert np.array_equal(rocm.to_host(cs, (96,)), a.sum(0))
    big = synth.normal(4, (5000, 33))
    dbig, cs2 = dev.put(big), dev.empty(33)
    rocm.colsum(cs2, dbig, 5000, 33)
    assert max_err(rocm.to_host(cs2, (33,)), big.astype(np.float64).sum(0)) <= gemm_tol(5000, big, np.ones(1))
    # more row blocks than the second grid axis holds (2.2M rows of 4 columns, in both forms), and few
    # columns against many rows (the row-lane form): integer inputs, so any summation order is exact
    tall = synth.small_ints(5, (2200000, 4), 3)
    dtall, cs3 = dev.put(tall), dev.empty(128)
    for rows, cols in ((2200000, 4), (100000, 88), (2200000 * 4, 1), (275000, 32), (200, 44)):
        rocm.colsum(cs3, dtall, rows, cols)
        assert np.array_equal(rocm.to_host(cs3, (cols,)), tall.ravel()[:rows * cols].reshape(rows, cols).astype(np.int64).sum(0).astype(np.float32))
    rocm.axpy(out, da, 2.0, a.size)
    assert np.array_equal(rocm.to_host(out, (300, 96)), a + bias + 2 * a)
    rocm.fill(out, 3.5, 7)
    assert np.all(rocm.to_host(out, (7,)) == 3.5)


# ---- benchmark configurations at full size ---------------------------------------------------

def _check_rows(got_rows, stats, K, amax, bmax):
    tol = 1e-4 * np.sqrt(K) * amax * bmax
    for row, st in zip(got_rows, stats):
        assert max_err(row[:8], st["head"]) <= tol
        # |sum of N errors| <= N * tol
        assert abs(float(row.astype(np.float64).sum()) - st["sum"]) <= tol * row.size
        assert abs(float((row.astype(np.float64) ** 2).sum()) - st["sumsq"]) <= 2 * tol * np.abs(row).max() * row.size


def test_config2_4096_cubed(dev, rocm, oracle_native):
    with open(os.path.join(GOLDEN, "config_samples.json")) as f:
        gold = json.load(f)["config2"]
    a = synth.normal(1, (4096, 4096))
    b = synth.normal(1, (4096, 4096), stream=1)
    got = run_gemm(dev, a, b)[0]
    _check_rows(got[gold["rows"]], gold["stats"], 4096, np.abs(a).max(), np.abs(b).max())
    # live oracle on another 16 rows, every element
    rows = list(range(1000, 1016))
    assert max_err(got[rows], oracle_native.sgemm_ikj(a[rows], b)) <= gemm_tol(4096, a, b)
    # C 1 = A (B 1) in float64: touches every element of C
    ones = np.ones(4096)
    lhs = got.astype(np.float64) @ ones
    rhs = a.astype(np.float64) @ (b.astype(np.float64) @ ones)
    assert np.max(np.abs(lhs - rhs)) <= 4096 * gemm_tol(4096, a, b)


@pytest.mark.parametrize("m,n,k,ta,tb", [(4096, 768, 3072, False, False), (768, 3072, 4096, True, False), (4096, 768, 768, False, True),
                                          (3000, 3000, 1000, False, False)])
def test_streamk_at_training_sizes(dev, oracle_native, m, n, k, ta, tb):
    # the mid-size products of a transformer step, which the planner hands to stream-K (128 x 128 and 64 x 64 tiles)
    a = synth.normal(m, (k, m) if ta else (m, k))
    b = synth.normal(n, (n, k) if tb else (k, n), stream=1)
    A, B = (a.T if ta else a), (b.T if tb else b)
    got = run_gemm(dev, a, b, ta, tb)[0]
    rows = [0, 1, 127, 128, m // 2, m - 1]
    assert max_err(got[rows], oracle_native.sgemm_ikj(np.ascontiguousarray(A[rows]), np.ascontiguousarray(B))) <= gemm_tol(k, a, b)
    ones = np.ones(n)
    lhs = got.astype(np.float64) @ ones                                        # C 1 = A (B 1): touches every element of C
    rhs = A.astype(np.float64) @ (B.astype(np.float64) @ ones)
    assert np.max(np.abs(lhs - rhs)) <= n * gemm_tol(k, a, b)
    forced = run_gemm(dev, a, b, ta, tb, algo=N.ALGO_MFMA_STREAMK)[0]
    assert max_err(forced, got) <= gemm_tol(k, a, b)


@pytest.mark.parametrize("m,n,k,ta,tb", [(2048, 2048, 1536, False, False), (2048, 2048, 1536, False, True), (2048, 2048, 1536, True, False),
                                          (4096, 3072, 768, False, False), (4096, 3072, 776, False, True)])
def test_planner_half_width_tiles(dev, m, n, k, ta, tb):
    """Products whose 128 x 128 tiles fill their rounds badly while 64 x 128 / 128 x 64 tiles fill theirs: with a
    K-contiguous operand the planner takes the half-width tiles (whole tiles, steady K loop, the last case with a
    K tail), otherwise stream-K; every choice must give the integer-exact result, and so must the forced ones."""
    a = synth.small_ints(m + k, (k, m) if ta else (m, k), 3)
    b = synth.small_ints(n + k, (n, k) if tb else (k, n), 3, stream=1)
    # float64 holds these sums of small integers exactly (and runs on the host BLAS, unlike an int64 product)
    want = ((a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)).astype(np.float32)
    for algo in (N.ALGO_AUTO, N.ALGO_MFMA, N.ALGO_MFMA_SMALL, N.ALGO_MFMA_STREAMK):
        assert np.array_equal(run_gemm(dev, a, b, ta, tb, algo=algo)[0], want), algo


def test_config5a_decode_gemv(dev, rocm):
    with open(os.path.join(GOLDEN, "config_samples.json")) as f:
        gold = json.load(f)["config5a"]
    x = synth.normal(4, (4, 4096), 0.02)
    w = synth.normal(4, (4096, 4096), 0.02, stream=1)
    got = run_gemm(dev, x, w)[0]
    _check_rows(got, gold["stats"], 4096, np.abs(x).max(), np.abs(w).max())
    want = x.astype(np.float64) @ w.astype(np.float64)
    assert max_err(got, want) <= gemm_tol(4096, x, w)


def test_config5b_tall_k_weight_gradient(dev, rocm):
    with open(os.path.join(GOLDEN, "config_samples.json")) as f:
        gold = json.load(f)["config5b"]
    X = synth.normal(5, (65536, 1024))
    dY = synth.normal(5, (65536, 1024), stream=1)
    got = run_gemm(dev, X, dY, ta=True)[0]  # X^T as a view: strides (1, 1024)
    _check_rows(got[gold["rows"]], gold["stats"], 65536, np.abs(X).max(), np.abs(dY).max())
    # a sampled block in float64
    rows, cols = slice(100, 116), slice(900, 932)
    want = X[:, rows].astype(np.float64).T @ dY[:, cols].astype(np.float64)
    assert max_err(got[rows, cols], want) <= gemm_tol(65536, X, dY)


def test_device_status_word_makes_the_next_wait_fail(dev, rocm):
    # What a kernel does when its bounded wait for another workgroup expires (NaN into the output, a code
    # into the status word) cannot be provoked without hanging a kernel; the host side can: set the word
    # the way such a kernel would and see that every waiting call reports it once and then recovers.
    x = dev.put(np.ones(8, np.float32))
    for code, text in ((1, "stream-K"), (2, "skinny_cols_kernel")):
        rocm.test_raise_device_status(code)
        with pytest.raises(N.MniError, match=text):
            rocm.sync()
        rocm.sync()  # cleared by the report
        rocm.test_raise_device_status(code)
        with pytest.raises(N.MniError, match="device status %d" % code):
            rocm.to_host(x, (8,))
        assert np.array_equal(rocm.to_host(x, (8,)), np.ones(8, np.float32))
    rocm.test_raise_device_status(2)
    e0, e1 = rocm.event(), rocm.event()
    rocm.record(e0)
    rocm.record(e1)
    with pytest.raises(N.MniError, match="device status 2"):
        rocm.elapsed_ms(e0, e1)
    assert rocm.elapsed_ms(e0, e1) >= 0.0
    rocm.event_destroy(e0)
    rocm.event_destroy(e1)
    # the engine's read-backs go through the same check
    from framework_amd.native import Native
    nat = Native()
    t = nat.fromFloat32(np.arange(4, dtype=np.float32), [4])
    rocm.test_raise_device_status(1)
    with pytest.raises(N.MniError, match="device status 1"):
        nat.toFloat32(t)
    assert np.array_equal(nat.toFloat32(t), np.arange(4, dtype=np.float32))
    nat.freeTensor(t)


def test_sgemm_timed_runs_the_products_and_reports_a_duration(dev, rocm):
    a = synth.small_ints(1, (64, 48), 3)
    bs = [synth.small_ints(2 + i, (48, 80), 3, stream=1) for i in range(3)]
    dA, dBs = dev.put(a), [dev.put(b) for b in bs]
    dCs = [dev.empty(64 * 80) for _ in bs]
    descs = [rocm.gemm_desc(64, 80, 48, dA, dB, dC) for dB, dC in zip(dBs, dCs)]
    ms = rocm.sgemm_timed(descs, 2, 7)  # 9 launches cycle over the 3 products
    assert np.isfinite(ms) and ms > 0.0
    for b, dC in zip(bs, dCs):
        assert np.array_equal(rocm.to_host(dC, (64, 80)), (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32))
    with pytest.raises(N.MniError):
        rocm.sgemm_timed(descs, 0, 0)


def test_mfma_yardstick_runs_and_shows_what_a_register_move_costs(dev, rocm):
    pure = rocm.mfma_yardstick(0, mfmas_per_wave=8192)
    moved = rocm.mfma_yardstick(2, mfmas_per_wave=8192)
    assert moved < pure                  # vector-ALU instructions take their issue time from the MFMAs
    # the yardstick is a ceiling for products on the same card at the same clocks: a 2048^3 product stays below it,
    # and not by an order of magnitude
    n = 2048
    dA, dB, dC = dev.empty(n * n, fill=0.5), dev.empty(n * n, fill=0.25), dev.empty(n * n)
    product = 2.0 * n ** 3 / (rocm.sgemm_timed([rocm.gemm_desc(n, n, n, dA, dB, dC)], 5, 20) * 1e-3) / 1e12
    assert 0.1 * pure < product < pure
    with pytest.raises(N.MniError, match="bad arguments"):
        rocm.mfma_yardstick(3)


# ---- the kernel-level ABI driven the way the Rust `rocm` arm of matmul_backward drives it ----------------------------
def _rust_arm_matmul_backward(dev, a, b, g):
    """dA, dB of C = A B for an upstream gradient g, through mni_rocm_sgemm_pair and mni_rocm_unbroadcast exactly as
    integration/rust/ops/matmul_rocm.rs issues them: the two products with the transposed operand as a stride swap
    and the batch rule `b % count`, then each gradient summed down to its operand's shape."""
    r = dev.r
    m, k = a.shape[-2:]
    n = b.shape[-1]
    out_batch = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
    batch = int(np.prod(out_batch, dtype=np.int64))
    a_count, b_count = int(np.prod(a.shape[:-2], dtype=np.int64)), int(np.prod(b.shape[:-2], dtype=np.int64))
    dA, dB, dG = dev.put(a), dev.put(b), dev.put(g)
    ga_full, gb_full = dev.empty(batch * m * k), dev.empty(batch * k * n)
    first = r.gemm_desc(m, k, n, dG, dB, ga_full, batch=batch, a_strides=(n, 1), a_batch=(m * n, batch),
                        b_strides=(1, n), b_batch=(k * n, b_count))          # dA = dC * B^T
    second = r.gemm_desc(k, n, m, dA, dG, gb_full, batch=batch, a_strides=(1, k), a_batch=(m * k, a_count),
                         b_strides=(n, 1), b_batch=(m * n, batch))           # dB = A^T * dC
    r.sgemm_pair(first, second)
    ga, gb = dev.empty(a.size), dev.empty(b.size)
    r.unbroadcast(ga, ga_full, list(out_batch) + [m, k], list(a.shape))
    r.unbroadcast(gb, gb_full, list(out_batch) + [k, n], list(b.shape))
    return r.to_host(ga, a.shape), r.to_host(gb, b.shape)


@pytest.mark.parametrize("a_shape,b_shape", [((2, 1, 5, 7), (2, 3, 7, 4)), ((1, 6, 9), (4, 9, 5)), ((3, 8, 6), (6, 10)),
                                             ((2, 3, 4, 6), (1, 3, 6, 5)), ((4, 1, 1, 3, 8), (4, 2, 5, 8, 2))])
def test_rust_arm_call_sequence_gradients_vs_oracle(dev, orc, a_shape, b_shape):
    # an interior batch dim of extent 1 (a[2,1,M,K] against b[2,3,K,N]) is summed along that dim, not along the
    # leading one; the oracle's matmul_backward (ops/matmul.rs:199-222 with utils.rs:39-66) is the reference
    a = synth.small_ints(1, a_shape, 3); b = synth.small_ints(2, b_shape, 3, stream=1)
    out_batch = np.broadcast_shapes(a_shape[:-2], b_shape[:-2])
    # (an operand with fewer batches is read at batch % count, the reference's rule (ops/matmul.rs:55-56), by the
    # oracle and by the kernel alike; test_oracle_matmul pins the rule itself)
    g = synth.small_ints(3, tuple(out_batch) + (a_shape[-2], b_shape[-1]), 2, stream=2)
    A = orc.Tensor.fromFloat32(a, list(a_shape)).setRequiresGrad(True)
    B = orc.Tensor.fromFloat32(b, list(b_shape)).setRequiresGrad(True)
    A.matmul(B).mul(orc.Tensor.fromFloat32(g, list(g.shape))).sum().backward()
    want_a, want_b = A.grad.numpy(), B.grad.numpy()
    ga, gb = _rust_arm_matmul_backward(dev, a, b, g)
    assert np.array_equal(ga, want_a) and np.array_equal(gb, want_b)


def test_kernel_level_unbroadcast_patterns_and_errors(dev, rocm):
    g = synth.small_ints(4, (2, 3, 4, 5), 4)
    dG = dev.put(g)
    for to, axes in (([2, 1, 4, 5], (1,)), ([3, 1, 5], (0, 2)), ([5], (0, 1, 2)), ([1], (0, 1, 2, 3)), ([2, 3, 4, 5], ()), ([1, 1, 4, 1], (0, 1, 3)),
                     ([4, 5], (0, 1))):
        out = dev.empty(int(np.prod(to)))
        rocm.unbroadcast(out, dG, list(g.shape), to)
        want = g.astype(np.int64).sum(axis=axes, keepdims=True).reshape(to).astype(np.float32) if axes else g
        assert np.array_equal(rocm.to_host(out, tuple(to)), want), to
    out = dev.empty(40)
    with pytest.raises(N.MniError):
        rocm.unbroadcast(out, dG, list(g.shape), [2, 4, 5])      # 2 does not broadcast against 3
    with pytest.raises(N.MniError):
        rocm.unbroadcast(out, dG, [4, 5], [2, 4, 5])             # more dims than the gradient has
