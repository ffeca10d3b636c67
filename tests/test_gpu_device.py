"""Copies and waits of the device layer (mni_rocm_h2d / d2h / sync and the engine's small uploads).

Small reads come to the host through pinned memory that a kernel writes, waits watch a word a marker kernel
writes, small uploads inside the engine are queued through pinned staging slots; each has a fallback on the
runtime's own copy or wait.  These tests check the bytes on both sides of every size limit and with work of
every length queued in front.
"""
import ctypes as C

import numpy as np
import pytest

from framework_amd import synth

pytestmark = pytest.mark.gpu

STAGE = 16384  # bytes: the limit of the pinned paths


@pytest.mark.parametrize("nbytes", [4, 8, 252, 4096, STAGE - 4, STAGE, STAGE + 4, 3 * STAGE, 1 << 20])
def test_reads_of_every_size_return_the_bytes(rocm, nbytes):
    words = np.random.default_rng(nbytes).integers(0, 2**32, size=nbytes // 4 + 2, dtype=np.uint32)
    p = rocm.to_device(words)
    assert np.array_equal(rocm.to_host(p, (nbytes // 4,), np.uint32), words[:nbytes // 4])
    # from an address that is 4-byte but not 16-byte aligned
    assert np.array_equal(rocm.to_host(p + 4, (nbytes // 4,), np.uint32), words[1:nbytes // 4 + 1])
    # a size that is no multiple of 4 takes the runtime's copy
    assert np.array_equal(rocm.to_host(p + 4, (nbytes + 3,), np.uint8), words.view(np.uint8)[4:nbytes + 7])
    rocm.free(p)


def test_small_reads_and_waits_behind_long_and_short_work(rocm):
    # behind a product that runs for milliseconds the watch for the marker gives up and the runtime's wait takes
    # over; behind a short one the marker arrives within the watch.  The values read are the finished ones.
    n = 4096
    a = rocm.to_device(np.full((n, n), 0.5, np.float32))
    c = rocm.malloc(n * n * 4)
    d = rocm.gemm_desc(n, n, n, a, a, c)
    for launches in (12, 1):
        rocm.fill(c, -1.0, n * n)
        for _ in range(launches):
            rocm._check(rocm.lib.mni_rocm_sgemm(C.byref(d)))
        assert np.array_equal(rocm.to_host(c + 4 * (n * n - 8), (8,)), np.full(8, 0.25 * n, np.float32))   # small read
        rocm.fill(c, -1.0, n * n)
        for _ in range(launches):
            rocm._check(rocm.lib.mni_rocm_sgemm(C.byref(d)))
        rocm.sync()
        got = np.empty(8, np.float32)
        # (after the wait the copy below finds the stream idle; the value must be the product's)
        rocm._check(rocm.lib.mni_rocm_d2h(got.ctypes.data, c, 32))
        assert np.array_equal(got, np.full(8, 0.25 * n, np.float32))
    rocm.free(a)
    rocm.free(c)


def test_many_small_uploads_in_a_row_keep_their_own_data(gpu):
    # more uploads than there are staging slots, none waited for in between: a slot is reused only when its
    # transfer has left it
    Tn = gpu.Tensor
    rows = [synth.normal(i, (4096,), stream=i) for i in range(50)]           # 16 KB each: the largest staged size
    small = [np.float32(i) * np.ones(3, np.float32) for i in range(50)]
    ts = [Tn.fromFloat32(r, [4096]) for r in rows]
    ss = [Tn.fromFloat32(s, [3]) for s in small]
    big = Tn.fromFloat32(synth.normal(99, (4097,)), [4097])                  # one float over: the waiting copy
    total = ts[0]
    for t in ts[1:]:
        total = total.add(t)                                                 # queued behind the uploads
    want = rows[0].copy()
    for r in rows[1:]:
        want = (want + r).astype(np.float32)
    assert np.array_equal(total.numpy(), want)
    for t, r in zip(ts, rows):
        assert np.array_equal(t.numpy(), r)
    for t, s in zip(ss, small):
        assert np.array_equal(t.numpy(), s)
    assert np.array_equal(big.numpy(), synth.normal(99, (4097,)))


def test_targets_of_a_small_cross_entropy_reach_the_backward_pass(gpu, orc):
    # up to 64 rows: the targets travel in the kernel arguments and the kernel stores them for backward();
    # a scaled loss takes the backward kernel, which reads them from there
    logits = synth.normal(5, (64, 7)) * 2.0
    targets = [[int(t)] for t in np.random.default_rng(5).integers(0, 7, size=64)]
    res = []
    for api in (gpu, orc):
        lg = api.Tensor.fromFloat32(logits, [64, 7]).setRequiresGrad(True)
        api.crossEntropyLoss(lg, targets).mul(0.5).backward()
        res.append(lg.grad.numpy())
    assert np.max(np.abs(res[0] - res[1])) < 1e-7
    onehot_rows = np.argmin(res[0], axis=1)                                  # the only negative entry of a row is its target's
    assert onehot_rows.tolist() == [t[0] for t in targets]
