"""mni_rocm_sgemm_noalloc: the product for callers that cannot allocate.  Its
results must be the bits mni_rocm_sgemm gives (same kernels, same plan; only
the home of the partial sums differs), call after call on the one shared
workspace, also when a smaller product follows a larger one, and the
library's allocator must not be asked for anything meanwhile."""
import numpy as np
import pytest

from framework_amd import native as N
from framework_amd import synth
from helpers import gemm_tol, max_err

pytestmark = pytest.mark.gpu

# (M, N, K, a_strides, algo, split_k): plans that keep partial sums in a workspace
STREAMK = (1300, 900, 1100, None, N.ALGO_MFMA_STREAMK, 0)   # stream-K forced: ragged tiles, one tile-sized slot per workgroup in the workspace
STREAMK_AUTO = (2560, 2560, 2560, None, N.ALGO_AUTO, 0)     # no tile shape deals 256 CUs equal loads: the planner's own stream-K
SPLITK = (1024, 1024, 8192, (1, 1024), N.ALGO_AUTO, 0)  # A^T view, 8 K slices of a 4 MiB result
GEMV = (4, 4096, 4096, None, N.ALGO_AUTO, 0)            # skinny kernel, 64 K slices reduced inside the launch
SMALL_SPLIT = (200, 136, 1000, None, N.ALGO_MFMA, 5)    # ragged edges, explicit split
NO_WORKSPACE = (512, 512, 64, None, N.ALGO_AUTO, 0)     # one workgroup per tile: no partials at all
FEWROWS = (24, 4096, 2048, None, N.ALGO_AUTO, 0)        # few-rows kernel: 8 K slices summed by the last workgroup to arrive


def _operands(rocm, case, seed):
    M, Nn, K, a_strides, _, _ = case
    a = synth.normal(seed, (K, M) if a_strides else (M, K), 0.5)
    b = synth.normal(seed, (K, Nn), 0.5, stream=1)
    return a, b, rocm.to_device(a), rocm.to_device(b)


def _run(rocm, fn, case, dA, dB, dC):
    M, Nn, K, a_strides, algo, split = case
    rocm.fill(dC, -3.0, M * Nn)
    fn(M, Nn, K, dA, dB, dC, a_strides=a_strides, algo=algo, split_k=split)
    return rocm.to_host(dC, (M, Nn))


@pytest.mark.parametrize("first,second", [(STREAMK, GEMV), (SPLITK, SMALL_SPLIT), (GEMV, NO_WORKSPACE), (STREAMK, SPLITK), (SPLITK, FEWROWS),
                                          (FEWROWS, GEMV), (STREAMK_AUTO, STREAMK)])
def test_two_calls_in_a_row_match_the_allocating_entry_point(rocm, first, second):
    bufs = []
    try:
        cases = []
        for seed, case in enumerate((first, second)):
            a, b, dA, dB = _operands(rocm, case, 40 + seed)
            dC = rocm.malloc(case[0] * case[1] * 4)
            bufs += [dA, dB, dC]
            cases.append((case, a, b, dA, dB, dC))
        want = [_run(rocm, rocm.sgemm, c, dA, dB, dC) for c, _, _, dA, dB, dC in cases]
        # the larger product, then the smaller one on the workspace the first left behind, then both again
        for _ in range(2):
            for (c, a, b, dA, dB, dC), w in zip(cases, want):
                rocm.fill(dC, -3.0, c[0] * c[1])
                before = rocm.alloc_stats()
                rocm.sgemm_noalloc(c[0], c[1], c[2], dA, dB, dC, a_strides=c[3], algo=c[4], split_k=c[5])
                assert rocm.alloc_stats() == before, "the allocator was used during the call"
                got = rocm.to_host(dC, (c[0], c[1]))
                assert np.array_equal(got, w), "case %r differs from mni_rocm_sgemm" % (c,)
                A = a.T if c[3] else a
                rows = [0, c[0] // 2, c[0] - 1]
                assert max_err(got[rows], A[rows].astype(np.float64) @ b.astype(np.float64)) <= gemm_tol(c[2], a, b)
    finally:
        for p in bufs:
            rocm.free(p)


def test_a_plan_beyond_the_workspace_is_refused_with_both_sizes(rocm):
    cap = rocm.sgemm_noalloc_workspace_bytes()
    assert cap == 32 << 20
    M = Nn = 2048
    K = 2048
    a, b = synth.small_ints(1, (M, K), 2), synth.small_ints(2, (K, Nn), 2, stream=1)
    dA, dB, dC = rocm.to_device(a), rocm.to_device(b), rocm.malloc(M * Nn * 4)
    try:
        with pytest.raises(N.MniError, match=r"needs %d bytes of workspace, the fixed scratch holds %d" % (4 * M * Nn * 4, cap)):
            rocm.sgemm_noalloc(M, Nn, K, dA, dB, dC, split_k=4, algo=N.ALGO_MFMA)
        # the library is unharmed: two slices fit (2 x 16 MiB) and give the exact integer result
        rocm.sgemm_noalloc(M, Nn, K, dA, dB, dC, split_k=2, algo=N.ALGO_MFMA)
        got = rocm.to_host(dC, (M, Nn))
        assert np.array_equal(got[:64], (a[:64].astype(np.int64) @ b.astype(np.int64)).astype(np.float32))
    finally:
        for p in (dA, dB, dC):
            rocm.free(p)
