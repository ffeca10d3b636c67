"""Seeded random sweep of mni_rocm_sgemm through the C ABI: shapes around the tile and K-step sizes, padded leading
dimensions, operands that start 1-3 floats into their allocation, transposes, batches with the reference's modulo
rule, epilogues, accumulation, requested K splits and every tile algorithm.  Inputs are small integers, so any
summation order gives the exact result and float64 on the host is the reference; the padding of A and B holds a
huge value that must never reach C, and the padding columns of C must keep what they held."""
import random

import numpy as np
import pytest

from framework_amd import native as N

pytestmark = pytest.mark.gpu

M_CHOICES = [1, 3, 17, 64, 65, 100, 128, 129, 200, 256, 300, 333, 512, 700]
N_CHOICES = [1, 4, 20, 63, 64, 96, 128, 130, 192, 257, 320, 500, 640]
K_CHOICES = [1, 5, 31, 32, 33, 64, 70, 96, 100, 128, 160, 200, 256, 300, 515, 1024, 2051]
HUGE = 7e29


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_products_are_integer_exact(rocm, seed):
    r = rocm
    rng = random.Random(seed)
    gen = np.random.default_rng(seed)
    ran = 0
    for case in range(150):
        m, n, k = rng.choice(M_CHOICES), rng.choice(N_CHOICES), rng.choice(K_CHOICES)
        ta, tb = rng.random() < 0.5, rng.random() < 0.5
        batch = rng.choice([1, 1, 1, 2, 3, 5])
        ab, bb = rng.choice([1, batch]), rng.choice([1, batch])
        pad_a, pad_b = rng.choice([0, 0, 1, 3, 4, 8]), rng.choice([0, 0, 1, 2, 4, 12])
        off_a, off_b = rng.choice([0, 0, 1, 2, 3]), rng.choice([0, 0, 1, 2, 3])
        sa, sb = ((k, m) if ta else (m, k)), ((n, k) if tb else (k, n))
        lda, ldb = sa[1] + pad_a, sb[1] + pad_b
        a = np.full((ab, sa[0], lda), HUGE, np.float32)
        b = np.full((bb, sb[0], ldb), HUGE, np.float32)
        a[:, :, :sa[1]] = gen.integers(-3, 4, (ab,) + sa)
        b[:, :, :sb[1]] = gen.integers(-3, 4, (bb,) + sb)
        ldc = n + rng.choice([0, 0, 1, 5])
        c0 = gen.integers(-3, 4, (batch, m, ldc)).astype(np.float32)
        bias = gen.integers(-3, 4, n).astype(np.float32)
        epi = rng.choice([N.EPI_NONE, N.EPI_NONE, N.EPI_BIAS, N.EPI_BIAS_RELU])
        acc = rng.random() < 0.25
        algo = rng.choice([N.ALGO_AUTO, N.ALGO_AUTO, N.ALGO_MFMA, N.ALGO_MFMA_SMALL, N.ALGO_MFMA_STREAMK])
        split = rng.choice([0, 0, 0, 2, 3]) if algo != N.ALGO_MFMA_STREAMK else 0
        what = dict(case=case, m=m, n=n, k=k, ta=ta, tb=tb, batch=batch, ab=ab, bb=bb, lda=lda, ldb=ldb, off_a=off_a,
                    off_b=off_b, ldc=ldc, epi=epi, acc=acc, algo=algo, split=split)
        d_a = r.to_device(np.concatenate([np.full(off_a, HUGE, np.float32), a.ravel()]))
        d_b = r.to_device(np.concatenate([np.full(off_b, HUGE, np.float32), b.ravel()]))
        d_c, d_bias = r.to_device(c0), r.to_device(bias)
        try:
            try:
                r.sgemm(m, n, k, d_a + 4 * off_a, d_b + 4 * off_b, d_c, batch=batch,
                        a_strides=(1, lda) if ta else (lda, 1), b_strides=(1, ldb) if tb else (ldb, 1),
                        a_batch=(sa[0] * lda, ab), b_batch=(sb[0] * ldb, bb), ldc=ldc, c_batch_stride=m * ldc,
                        epilogue=epi, bias=d_bias if epi != N.EPI_NONE else None, accumulate=acc, split_k=split, algo=algo)
            except N.MniError as e:
                # forced stream-K refuses products that cannot fill its grid: that is its documented answer
                assert algo == N.ALGO_MFMA_STREAMK and "stream-K" in str(e), (what, str(e))
                continue
            got = r.to_host(d_c, (batch, m, ldc))
        finally:
            for p in (d_a, d_b, d_c, d_bias):
                r.free(p)
        want = c0.astype(np.float64)
        for i in range(batch):
            a2, b2 = a[i % ab, :, :sa[1]].astype(np.float64), b[i % bb, :, :sb[1]].astype(np.float64)
            p = (a2.T if ta else a2) @ (b2.T if tb else b2)
            if epi != N.EPI_NONE:
                p = p + bias
            if epi == N.EPI_BIAS_RELU:
                p = np.maximum(p, 0)
            want[i, :, :n] = p + (want[i, :, :n] if acc else 0)
        assert np.array_equal(got.astype(np.float64), want), what
        ran += 1
    assert ran >= 100


FEW_M = [1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 17, 24, 32]
FEW_N = [64, 65, 132, 1003, 1024, 2048, 2050, 4096, 4100, 8192]
FEW_K = [64, 256, 512, 640, 768, 960, 1024, 1088, 1984, 2048, 2112, 3072, 4096]


@pytest.mark.parametrize("seed", [21, 22])
def test_random_few_rows_against_wide_operands_are_integer_exact(rocm, seed):
    # the decode family under the planner: 1 to 32 rows against a wide B, three times in four stored K-contiguous (a weight kept
    # [out, in]); pitches off their extents (whole 16 bytes or not), operands that start 1 or 4 floats into their allocation,
    # epilogues, accumulation.  The padding of A and B holds a huge value that must never reach C.
    r = rocm
    rng = random.Random(seed)
    gen = np.random.default_rng(seed)
    for case in range(60):
        m, n, k = rng.choice(FEW_M), rng.choice(FEW_N), rng.choice(FEW_K)
        while n * k > (1 << 24):
            n = rng.choice(FEW_N)
        tb = rng.random() < 0.75
        pad_a, pad_b = rng.choice([0, 0, 4, 8, 3]), rng.choice([0, 0, 4, 12, 1])
        off_a, off_b = rng.choice([0, 0, 4, 1]), rng.choice([0, 0, 4, 2])
        sb = (n, k) if tb else (k, n)
        lda, ldb = k + pad_a, sb[1] + pad_b
        a = np.full((m, lda), HUGE, np.float32)
        b = np.full((sb[0], ldb), HUGE, np.float32)
        a[:, :k] = gen.integers(-3, 4, (m, k))
        b[:, :sb[1]] = gen.integers(-3, 4, sb)
        ldc = n + rng.choice([0, 0, 1, 5])
        c0 = gen.integers(-3, 4, (m, ldc)).astype(np.float32)
        bias = gen.integers(-3, 4, n).astype(np.float32)
        epi = rng.choice([N.EPI_NONE, N.EPI_NONE, N.EPI_BIAS, N.EPI_BIAS_RELU])
        acc = rng.random() < 0.25
        what = dict(case=case, m=m, n=n, k=k, tb=tb, lda=lda, ldb=ldb, off_a=off_a, off_b=off_b, ldc=ldc, epi=epi, acc=acc)
        d_a = r.to_device(np.concatenate([np.full(off_a, HUGE, np.float32), a.ravel()]))
        d_b = r.to_device(np.concatenate([np.full(off_b, HUGE, np.float32), b.ravel()]))
        d_c, d_bias = r.to_device(c0), r.to_device(bias)
        try:
            r.sgemm(m, n, k, d_a + 4 * off_a, d_b + 4 * off_b, d_c, a_strides=(lda, 1), b_strides=(1, ldb) if tb else (ldb, 1), ldc=ldc,
                    epilogue=epi, bias=d_bias if epi != N.EPI_NONE else None, accumulate=acc)
            got = r.to_host(d_c, (m, ldc))
        finally:
            for ptr in (d_a, d_b, d_c, d_bias):
                r.free(ptr)
        opb = b[:, :sb[1]].T if tb else b[:, :sb[1]]
        want = a[:, :k].astype(np.float64) @ opb.astype(np.float64)
        if epi != N.EPI_NONE:
            want = want + bias
        if epi == N.EPI_BIAS_RELU:
            want = np.maximum(want, 0.0)
        if acc:
            want = want + c0[:, :n]
        assert np.array_equal(got[:, :n], want.astype(np.float32)), what
        assert np.array_equal(got[:, n:], c0[:, n:]), ("the padding of C was written", what)
