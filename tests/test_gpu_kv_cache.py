"""The device-resident KV cache against the CPU oracle through the C ABI:
the reference suite's behaviours (test/native.test.ts:48-151), step-by-step
parity of fp32 and int8 decoding, long histories that need several workgroups
per head, and the error texts."""
import math

import numpy as np
import pytest

from framework_amd import native as N
from framework_amd import synth
from framework_amd.api import bind
from helpers import max_err

pytestmark = pytest.mark.gpu


def _t(api, a):
    a = np.asarray(a, dtype=np.float32)
    return api.Tensor.fromFloat32(a, list(a.shape))


@pytest.fixture()
def both(rocm_native, oracle_native):
    gpu, cpu = bind(rocm_native), bind(oracle_native)
    yield gpu, cpu
    rocm_native.resetEngine()
    oracle_native.resetEngine()


def test_reference_suite_behaviours_on_the_gpu(both):
    gpu, _ = both
    batch, heads, d, max_seq, steps = 1, 2, 8, 16, 6
    scale = 1.0 / math.sqrt(d)
    fp, qc = gpu.KvCache(batch, heads, d, max_seq, False), gpu.KvCache(batch, heads, d, max_seq, True)
    assert qc.isQuantized() and not fp.isQuantized()
    ap = gpu.KvCache(batch, heads, d, max_seq, False)
    ap.append(_t(gpu, synth.uniform(1, (batch, heads, 1, d), 0, 1)), _t(gpu, synth.uniform(2, (batch, heads, 1, d), 0, 1)))
    assert ap.length() == 1
    ap.free()
    worst = 0.0
    for t in range(steps):
        q, k, v = (_t(gpu, synth.uniform(10 + t, (batch, heads, 1, d), 0, 1, stream=i)) for i in range(3))
        a, b = fp.decodeStep(q, k, v, scale), qc.decodeStep(q, k, v, scale)
        assert a.shape == [batch, heads, 1, d] and a.size == batch * heads * d
        worst = max(worst, max_err(a.numpy(), b.numpy()))
    assert fp.length() == steps and qc.length() == steps
    assert 0 < worst < 0.15
    bad = gpu.KvCache(batch, heads, d, max_seq, False)
    two = _t(gpu, np.zeros((batch, heads, 2, d)))
    with pytest.raises(N.MniError, match="kv cache decode failed: kv cache decode expects seq_len=1, got 2"):
        bad.decodeStep(two, two, two, scale)
    one, wide = _t(gpu, np.zeros((batch, heads, 1, d))), _t(gpu, np.zeros((batch, heads, 1, d + 1)))
    with pytest.raises(N.MniError, match="q/k/v shapes must match for kv cache decode"):
        bad.decodeStep(one, wide, wide, scale)
    with pytest.raises(N.MniError, match=r"shape mismatch: expected \[B=1, H=2, S=1, D=8\], got \[B=1, H=2, S=1, D=9\]"):
        bad.decodeStep(wide, wide, wide, scale)
    flat = _t(gpu, np.zeros((2, 8)))
    with pytest.raises(N.MniError, match=r"kv cache append failed: expected \[B,H,S,D\] or \[BH,S,D\], got shape \[2, 8\]"):
        bad.append(flat, flat)
    assert bad.length() == 0
    over = gpu.KvCache(batch, heads, d, 2, False)
    over.append(one, one)
    over.append(one, one)
    with pytest.raises(N.MniError, match=r"kv cache append failed: kv cache is full \(len=2, max_seq_len=2\)"):
        over.append(one, one)
    fp.reset()
    assert fp.length() == 0
    fp.free()
    assert fp.length() == 0
    with pytest.raises(N.MniError, match="invalid kv cache id"):
        fp.decodeStep(one, one, one, scale)
    first = gpu.KvCache(1, 1, 4, 4, False).cacheId
    gpu.native.resetEngine()
    assert gpu.KvCache(1, 1, 4, 4, False).cacheId == 1 and first > 1


@pytest.mark.parametrize("quantized", [False, True])
@pytest.mark.parametrize("batch,heads,d,shape4", [(2, 3, 16, True), (1, 6, 64, False), (1, 2, 5, True), (3, 4, 300, True),
                                                 (1, 2, 8, True), (2, 2, 128, True), (1, 3, 4, False), (1, 2, 256, True), (1, 2, 36, False)])
def test_decode_steps_match_the_oracle(both, batch, heads, d, shape4, quantized):
    gpu, cpu = both
    bh = batch * heads
    shp = (batch, heads, 1, d) if shape4 else (bh, 1, d)
    caches = [api.KvCache(batch if shape4 else 1, heads if shape4 else bh, d, 40, quantized) for api in (gpu, cpu)]
    for t in range(33):
        q, k, v = (synth.normal(50 + t, shp, 1.0, stream=i) for i in range(3))
        outs = [c.decodeStep(_t(api, q), _t(api, k), _t(api, v), 1.0 / math.sqrt(d)) for api, c in zip((gpu, cpu), caches)]
        assert outs[0].shape == outs[1].shape == list(shp)
        assert max_err(outs[0].numpy(), outs[1].numpy()) <= 1e-5 * float(np.abs(v).max()) * 4
    assert caches[0].length() == caches[1].length() == 33
    # reset, then reuse: the old contents must not leak into the new sequence
    for c in caches:
        c.reset()
    q, k, v = (synth.normal(99, shp, 1.0, stream=i) for i in range(3))
    outs = [c.decodeStep(_t(api, q), _t(api, k), _t(api, v), 0.5) for api, c in zip((gpu, cpu), caches)]
    assert max_err(outs[0].numpy(), outs[1].numpy()) <= 1e-5 and caches[0].length() == 1


@pytest.mark.parametrize("quantized", [False, True])
def test_long_history_uses_several_workgroups_per_head(both, quantized):
    # 5000 cached positions for 2 heads: the history is split over many workgroups and merged
    gpu, cpu = both
    bh, d, n = 2, 64, 5000
    caches = [api.KvCache(1, bh, d, n + 8, quantized) for api in (gpu, cpu)]
    hist_k, hist_v = synth.normal(7, (n, bh, 1, d)), synth.normal(8, (n, bh, 1, d), stream=1)
    for api, c in zip((gpu, cpu), caches):
        for t in range(n):
            c.append(_t(api, hist_k[t]), _t(api, hist_v[t]))
        api.native.gcTensors([])
    assert caches[0].length() == caches[1].length() == n
    q, k, v = (synth.normal(9, (bh, 1, d), 1.0, stream=i) for i in range(3))
    outs = [c.decodeStep(_t(api, q), _t(api, k), _t(api, v), 0.125) for api, c in zip((gpu, cpu), caches)]
    assert max_err(outs[0].numpy(), outs[1].numpy()) <= 2e-5
    if not quantized:  # and against float64 directly
        ks = np.concatenate([hist_k, k[None]]).reshape(n + 1, bh, d).transpose(1, 0, 2).astype(np.float64)
        vs = np.concatenate([hist_v, v[None]]).reshape(n + 1, bh, d).transpose(1, 0, 2).astype(np.float64)
        s = np.einsum("bd,bld->bl", q.reshape(bh, d).astype(np.float64), ks) * 0.125
        e = np.exp(s - s.max(1, keepdims=True))
        want = np.einsum("bl,bld->bd", e / e.sum(1, keepdims=True), vs)
        assert max_err(outs[0].numpy().reshape(bh, d), want) <= 2e-5
