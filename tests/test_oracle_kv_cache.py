"""Pins the oracle's KV cache (ops/kv_cache.rs, cpu arm) WITHOUT a GPU: the
behaviours the reference's suite asserts (test/native.test.ts:48-151), float64
softmax attention over the appended history, and the int8 row quantisation in
exact arithmetic."""
import math

import numpy as np
import pytest

from framework_amd import synth
from helpers import max_err


def _t(api, a):
    a = np.asarray(a, dtype=np.float32)
    return api.Tensor.fromFloat32(a, list(a.shape))


def _attend64(q, ks, vs, scale):
    # q [bh, d]; ks, vs [bh, len, d]
    s = np.einsum("bd,bld->bl", q.astype(np.float64), ks.astype(np.float64)) * scale
    e = np.exp(s - s.max(axis=1, keepdims=True))
    return np.einsum("bl,bld->bd", e / e.sum(axis=1, keepdims=True), vs.astype(np.float64))


def _quantize64(rows):
    # the reference's quantize_row_i8 restated with numpy float32 scalars
    out = np.empty_like(rows)
    for i, r in enumerate(rows):
        scale = max(np.float32(np.abs(r).max()) / np.float32(127.0), np.float32(1e-8))
        inv = np.float32(1.0) / scale
        q = np.clip(np.sign(r * inv) * np.floor(np.abs(r * inv) + np.float32(0.5)), -127, 127)  # round half away from zero
        out[i] = (q * scale).astype(np.float32)
    return out


def test_reference_suite_behaviours(orc, oracle_native):
    batch, heads, d, max_seq, steps = 1, 2, 8, 16, 6                      # native.test.ts:51-56
    scale = 1.0 / math.sqrt(d)
    fp, qc = orc.KvCache(batch, heads, d, max_seq, False), orc.KvCache(batch, heads, d, max_seq, True)
    assert qc.isQuantized() and not fp.isQuantized()                       # :60
    ap = orc.KvCache(batch, heads, d, max_seq, False)
    ap.append(_t(orc, synth.uniform(1, (batch, heads, 1, d), 0, 1)), _t(orc, synth.uniform(2, (batch, heads, 1, d), 0, 1)))
    assert ap.length() == 1                                                # :73-78
    ap.free()
    worst = 0.0
    for t in range(steps):                                                 # :82-99
        q, k, v = (_t(orc, synth.uniform(10 + t, (batch, heads, 1, d), 0, 1, stream=i)) for i in range(3))
        a, b = fp.decodeStep(q, k, v, scale), qc.decodeStep(q, k, v, scale)
        assert a.shape == [batch, heads, 1, d] and a.size == batch * heads * d
        worst = max(worst, max_err(a.numpy(), b.numpy()))
    assert fp.length() == steps and qc.length() == steps                   # :101-102
    assert 0 < worst < 0.15                                                # :103 (and the quantised path does differ)
    OracleError = type(oracle_native._err())
    bad = orc.KvCache(batch, heads, d, max_seq, False)                     # :114-121
    two = _t(orc, np.zeros((batch, heads, 2, d)))
    with pytest.raises(OracleError, match="kv cache decode failed: kv cache decode expects seq_len=1, got 2"):
        bad.decodeStep(two, two, two, scale)
    one, wide = _t(orc, np.zeros((batch, heads, 1, d))), _t(orc, np.zeros((batch, heads, 1, d + 1)))
    with pytest.raises(OracleError, match="q/k/v shapes must match for kv cache decode"):  # :123-130
        bad.decodeStep(one, wide, wide, scale)
    with pytest.raises(OracleError, match=r"shape mismatch: expected \[B=1, H=2, S=1, D=8\], got \[B=1, H=2, S=1, D=9\]"):
        bad.decodeStep(wide, wide, wide, scale)
    with pytest.raises(OracleError, match=r"expected \[B,H,S,D\] or \[BH,S,D\], got shape \[2, 8\]"):
        flat = _t(orc, np.zeros((2, 8)))
        bad.append(flat, flat)
    assert bad.length() == 0
    over = orc.KvCache(batch, heads, d, 2, False)                          # :132-138
    over.append(one, one)
    over.append(one, one)
    with pytest.raises(OracleError, match=r"kv cache append failed: kv cache is full \(len=2, max_seq_len=2\)"):
        over.append(one, one)
    fp.reset()
    assert fp.length() == 0                                                # :140-141
    fp.free()
    assert fp.length() == 0                                                # freed handle: len reads 0 ...
    with pytest.raises(OracleError, match="invalid kv cache id"):          # ... and decode throws, :145-151
        fp.decodeStep(one, one, one, scale)
    first = orc.KvCache(1, 1, 4, 4, False).cacheId
    oracle_native.resetEngine()
    assert orc.KvCache(1, 1, 4, 4, False).cacheId == 1 and first > 1       # reset_engine restarts the ids at 1


@pytest.mark.parametrize("shape4", [True, False])
def test_fp32_decode_vs_float64_attention(orc, shape4):
    batch, heads, d, steps = 2, 3, 16, 9
    bh = batch * heads
    shp = (batch, heads, 1, d) if shape4 else (bh, 1, d)
    cache = orc.KvCache(batch if shape4 else 1, heads if shape4 else bh, d, 12, False)
    ks, vs = [], []
    for t in range(steps):
        q, k, v = (synth.normal(20 + t, shp, 1.0, stream=i) for i in range(3))
        ks.append(k.reshape(bh, d)); vs.append(v.reshape(bh, d))
        out = cache.decodeStep(_t(orc, q), _t(orc, k), _t(orc, v), 0.3)
        assert out.shape == list(shp)
        want = _attend64(q.reshape(bh, d), np.stack(ks, 1), np.stack(vs, 1), 0.3)
        assert max_err(out.numpy().reshape(bh, d), want) < 2e-6
    assert cache.length() == steps
    # the first step sees a single key: the output is exactly that value row
    c2 = orc.KvCache(1, 2, 4, 4, False)
    v1 = synth.normal(30, (2, 1, 4))
    assert np.array_equal(c2.decodeStep(_t(orc, v1), _t(orc, v1), _t(orc, v1), 1.0).numpy(), v1)


def test_quantised_decode_equals_attention_over_the_dequantised_rows(orc):
    bh, d, steps = 4, 8, 7
    cache = orc.KvCache(1, bh, d, 8, True)
    ks, vs = [], []
    for t in range(steps):
        q, k, v = (synth.normal(40 + t, (bh, 1, d), 1.0, stream=i) for i in range(3))
        ks.append(_quantize64(k.reshape(bh, d))); vs.append(_quantize64(v.reshape(bh, d)))
        out = cache.decodeStep(_t(orc, q), _t(orc, k), _t(orc, v), 0.35)
        want = _attend64(q.reshape(bh, d), np.stack(ks, 1), np.stack(vs, 1), 0.35)
        assert max_err(out.numpy().reshape(bh, d), want) < 2e-6
        # and each stored row is within half a quantisation step of the original
        assert np.all(np.abs(ks[-1] - k.reshape(bh, d)) <= np.abs(k.reshape(bh, d)).max(axis=1, keepdims=True) / 127 / 2 * 1.0001)
    # hand-picked row: max 127 -> scale exactly 1; .5 rounds away from zero; an all-zero row takes the 1e-8 floor
    c = orc.KvCache(1, 1, 4, 2, True)
    row = np.array([[[127.0, 2.5, -2.5, 0.4]]], np.float32)
    out = c.decodeStep(_t(orc, row), _t(orc, row), _t(orc, row), 0.0)
    assert np.array_equal(out.numpy(), np.array([[[127.0, 3.0, -3.0, 0.0]]], np.float32))
    z = np.zeros((1, 1, 4), np.float32)
    c0 = orc.KvCache(1, 1, 4, 2, True)
    assert np.array_equal(c0.decodeStep(_t(orc, z), _t(orc, z), _t(orc, z), 1.0).numpy(), z)
