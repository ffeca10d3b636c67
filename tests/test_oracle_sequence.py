"""Pins the oracle's token-side ops WITHOUT a GPU: the Philox generator against
its published known-answer vectors, rand / randn by their distribution,
dropout, dataset windows, embedding (forward, ordered scatter-add backward),
tile, residual + layernorm, cross-entropy with buffered targets and gradient
unscaling, each against the reference's own assertions
(test/nn.test.ts:176-251, test/module.test.ts:97-105, test/native.test.ts:28-36),
numpy and closed forms."""
import numpy as np
import pytest

from framework_amd import synth
from helpers import max_err


def _t(api, a, grad=False):
    a = np.asarray(a, dtype=np.float32)
    t = api.Tensor.fromFloat32(a, list(a.shape))
    return t.setRequiresGrad(True) if grad else t


# Random123's kat_vectors for philox4x32-10: counter, key, expected output
PHILOX_KAT = [
    ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
    ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
    ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
     [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
]


def test_philox_known_answers(oracle_native):
    for ctr, key, want in PHILOX_KAT:
        assert oracle_native.philox(ctr, key) == want
    # the stream form: word i is word i % 4 of the block with counter (offset + i / 4, 0, 0), key = seed
    seed, offset = 0x299f31d0a4093822, 0x85a308d3243f6a88
    words = oracle_native.philoxWords(seed, offset, 10)
    for blk in range(3):
        c = offset + blk
        want = oracle_native.philox([c & 0xffffffff, c >> 32, 0, 0], [seed & 0xffffffff, seed >> 32])
        assert list(words[4 * blk:4 * blk + 4]) == want[:len(words[4 * blk:4 * blk + 4])]
    assert list(oracle_native.philoxWords(0, 0, 4)) == PHILOX_KAT[0][2]


def test_rand_is_uniform_on_24_bit_fractions(orc):
    orc.native.seed(7)
    u = orc.Tensor.rand([200, 500]).numpy().astype(np.float64).ravel()
    assert u.min() >= 0.0 and u.max() < 1.0                      # rand in [0, 1), tensor.rs:228-238
    assert np.all(u * 2 ** 24 == np.round(u * 2 ** 24))          # multiples of 2^-24 like rand's f32 sampling
    n = u.size
    assert abs(u.mean() - 0.5) < 4 * np.sqrt(1 / 12 / n)
    assert abs(u.var() - 1 / 12) < 0.002
    hist = np.histogram(u, bins=16, range=(0, 1))[0]
    assert np.all(np.abs(hist - n / 16) < 5 * np.sqrt(n / 16))
    # same seed, same stream; the next tensor continues it
    orc.native.seed(7)
    again = orc.Tensor.rand([200, 500]).numpy().ravel()
    assert np.array_equal(again.astype(np.float64), u)
    nxt = orc.Tensor.rand([200, 500]).numpy().ravel()
    assert not np.array_equal(nxt, again)
    assert abs(np.corrcoef(nxt, again)[0, 1]) < 0.02


def test_randn_moments(orc):
    orc.native.seed(11)
    z = orc.Tensor.randn([100000]).numpy().astype(np.float64)
    assert np.all(np.isfinite(z))
    assert abs(z.mean()) < 4 / np.sqrt(z.size)
    assert abs(z.var() - 1.0) < 0.02
    assert abs((z ** 3).mean()) < 0.05 and abs((z ** 4).mean() - 3.0) < 0.15
    assert abs(np.mean(np.abs(z) < 1.0) - 0.6827) < 0.01
    assert orc.Tensor.randn([3]).shape == [3] and orc.Tensor.randn([2, 0, 3]).size in (0, 1)


def test_randrange_like_the_reference(orc):
    # nn.ts:238-249 randRange = rand * (max - min) + min; test/nn.test.ts:249-251
    r = orc.Tensor.rand([100]).numpy() * 4.0 - 2.0
    assert np.all((r >= -2) & (r <= 2))


def test_dropout_reference_assertions(orc):
    x = _t(orc, [1, 2, 3, 4])
    assert orc.dropout(x, 0.5, True) is x                        # inference passthrough, nn.test.ts:229-233
    assert orc.dropout(x, 0.0, False) is x                       # rate 0 passthrough, :235-237
    assert orc.native.dropoutOp(x._id, 0.5, False) == x._id      # the op returns the same id, dropout.rs:30-32
    assert orc.native.dropoutOp(x._id, 0.0, True) == x._id
    d = orc.dropout(orc.Tensor.ones([1000]), 0.5, False).toFloat32()
    zeros = int(np.sum(d == 0))
    assert 100 < zeros < 900                                     # :239-244
    assert set(np.unique(d)) <= {0.0, 2.0}                       # kept values are x / (1 - rate)


@pytest.mark.parametrize("rate", [0.1, 0.5, 0.9])
def test_dropout_forward_backward_share_one_mask(orc, rate):
    orc.native.seed(3)
    xv = synth.uniform(5, (64, 257), 0.5, 2.0)
    x = _t(orc, xv, True)
    y = orc.dropout(x, rate)
    yv = y.numpy()
    scale = np.float32(1.0) / (np.float32(1.0) - np.float32(rate))
    kept = yv != 0
    assert np.array_equal(yv[kept], (xv * np.float32(1.0) * scale)[kept])
    assert abs(kept.mean() - (1 - rate)) < 4 * np.sqrt(rate * (1 - rate) / xv.size)
    w = synth.normal(6, xv.shape)
    y.mul(_t(orc, w)).sum().backward()
    g = x.grad.numpy()
    assert np.array_equal(g != 0, kept)                          # the same mask
    assert np.array_equal(g[kept], (w * np.float32(1.0) * scale)[kept])
    # E[dropout(x)] = x
    orc.native.seed(9)
    acc = np.zeros(4096)
    ones = orc.Tensor.ones([4096])
    for _ in range(64):
        acc += orc.dropout(ones, rate).numpy()
    assert abs(acc.mean() / 64 - 1.0) < 0.05


def test_dataset_windows(orc):
    n = orc.native
    data = (np.arange(1000) * 7 % 1009).astype(np.int32)
    ds = n.createDataset(data)
    starts = [0, 5, 990, 123]
    inp, tgt = n.sampleBatchAt(ds, 8, 4, starts)
    a, b = n.intBufferToHost(inp).reshape(4, 8), n.intBufferToHost(tgt).reshape(4, 8)
    for r, s in enumerate(starts):
        assert np.array_equal(a[r], data[s:s + 8]) and np.array_equal(b[r], data[s + 1:s + 9])
    assert np.array_equal(a[:, 1:], b[:, :-1])                   # targets are the inputs shifted by one
    with pytest.raises(Exception):
        n.sampleBatchAt(ds, 8, 1, [991])                         # gen_range(0..len - block - 1) excludes 991
    with pytest.raises(Exception):
        n.sampleBatchAt(n.createDataset(np.arange(9, dtype=np.int32)), 8, 1, [0])   # empty range
    # ids are recycled last-freed-first, data.rs:37-47
    n.freeIntBuffer(inp)
    n.freeIntBuffer(tgt)
    assert n.createDataset(np.zeros(3, np.int32)) == tgt
    assert n.createDataset(np.zeros(3, np.int32)) == inp
    with pytest.raises(Exception):
        n.intBufferToHost(99)


def test_embedding_reference_assertions(orc):
    emb = orc.Embedding(10, 4)                                   # test/nn.test.ts:197-211
    out = emb.forward([[0, 1, 2], [3, 4, 5]])
    assert out.shape == [2, 3, 4]
    same = emb.forward([[0, 0], [0, 0]]).toFloat32()
    assert same[0] == same[4]
    assert len(emb.parameters()) == 1
    with pytest.raises(Exception):
        emb.forward([[10]])


def test_embedding_forward_and_ordered_backward(orc):
    vocab, dim, batch, seq = 37, 24, 5, 19
    w = synth.normal(1, (vocab, dim))
    rng = np.random.default_rng(2)
    idx = rng.integers(0, 6, size=(batch, seq))                  # few distinct rows: long same-row runs
    idx[0, :4] = [36, 36, 0, 36]
    emb = orc.Embedding(vocab, dim, weight=w)
    out = emb.forward(idx.tolist())
    assert np.array_equal(out.numpy(), w[idx])
    g = synth.normal(3, (batch, seq, dim))
    out.mul(_t(orc, g)).sum().backward()
    dw = emb.weight.value.grad.numpy()
    want = np.zeros((vocab, dim), np.float32)                    # embedding.rs:104-128: += in token order
    for t, v in enumerate(idx.ravel()):
        want[v] += g.reshape(-1, dim)[t]
    assert np.array_equal(dw, want)
    ref64 = np.zeros((vocab, dim))
    np.add.at(ref64, idx.ravel(), g.reshape(-1, dim).astype(np.float64))
    assert max_err(dw, ref64) < 1e-5
    assert np.all(dw[7:36] == 0)                                 # rows nobody used


def test_embedding_from_an_int_buffer_equals_the_host_index_form(orc):
    n = orc.native
    vocab, dim = 50, 8
    w = synth.normal(4, (vocab, dim))
    data = (np.arange(400) * 13 % vocab).astype(np.int32)
    ds = n.createDataset(data)
    inp, tgt = n.sampleBatchAt(ds, 16, 3, [2, 100, 383 - 1])
    emb = orc.Embedding(vocab, dim, weight=w)
    a = emb.forwardGpu(inp, 3, 16).numpy()
    b = emb.forward(n.intBufferToHost(inp).reshape(3, 16).tolist()).numpy()
    assert np.array_equal(a, b) and a.shape == (3, 16, dim)
    # cross-entropy with buffered targets == the host-target form on the viewed logits (lib.rs:679-691)
    logits = synth.normal(5, (3, 16, vocab))
    l1 = _t(orc, logits, True)
    loss1 = orc.crossEntropyLossGpu(l1, tgt)
    loss1.backward()
    l2 = _t(orc, logits, True)
    loss2 = orc.crossEntropyLoss(l2, n.intBufferToHost(tgt).reshape(3, 16).tolist())
    loss2.backward()
    assert loss1.shape == [1] and loss1.item() == loss2.item()
    assert np.array_equal(l1.grad.numpy(), l2.grad.numpy())
    lp = logits.astype(np.float64).reshape(-1, vocab)
    lse = np.log(np.exp(lp - lp.max(1, keepdims=True)).sum(1)) + lp.max(1)
    want = np.mean(lse - lp[np.arange(48), n.intBufferToHost(tgt)])
    assert abs(loss1.item() - want) < 1e-5


def test_tile_reference_assertions_and_numpy(orc):
    t = orc.tile(_t(orc, [[1, 2, 3]]), [2, 1])                   # test/nn.test.ts:181-190
    assert t.shape == [2, 3]
    d = t.toFloat32()
    assert d[0] == 1 and d[3] == 1 and d[5] == 3
    assert orc.tile(_t(orc, [[1, 2]]), [3, 2]).shape == [3, 4]
    for shape, reps in [((2, 3), (2, 2)), ((3,), (4,)), ((2, 1, 3), (1, 5, 2)), ((2, 3, 4, 2), (2, 1, 3, 2))]:
        a = synth.normal(1, shape)
        got = orc.tile(_t(orc, a), list(reps))
        assert got.shape == list(np.tile(a, reps).shape) and np.array_equal(got.numpy(), np.tile(a, reps))
    # a permuted view is tiled by its logical contents
    a = synth.normal(2, (3, 4))
    assert np.array_equal(orc.tile(_t(orc, a).permute(1, 0), [2, 2]).numpy(), np.tile(a.T, (2, 2)))
    with pytest.raises(Exception):
        orc.tile(_t(orc, a), [2])
    # not differentiable in the reference: nothing reaches x through it
    x = _t(orc, a, True)
    orc.tile(x, [2, 1]).sum().backward()
    assert x.grad is None or not np.any(x.grad.numpy())


def test_residual_layernorm_equals_layernorm_of_the_sum(orc):
    rows, c = 33, 70
    xv, rv = synth.normal(1, (rows, c)), synth.normal(2, (rows, c), stream=1)
    gv, bv = synth.uniform(3, (c,), 0.5, 1.5), synth.normal(4, (c,), stream=2)
    wv = synth.normal(5, (rows, c), stream=3)

    x, r, g, b = _t(orc, xv, True), _t(orc, rv, True), _t(orc, gv, True), _t(orc, bv, True)
    out = orc.residualLayerNorm(x, r, g, b, 1e-5)
    out.mul(_t(orc, wv)).sum().backward()
    x2, r2, g2, b2 = _t(orc, xv, True), _t(orc, rv, True), _t(orc, gv, True), _t(orc, bv, True)
    out2 = orc.layerNorm(x2.add(r2), g2, b2, 1e-5)
    out2.mul(_t(orc, wv)).sum().backward()
    assert np.array_equal(out.numpy(), out2.numpy())
    for a, a2 in ((x, x2), (r, r2), (g, g2), (b, b2)):
        assert np.array_equal(a.grad.numpy(), a2.grad.numpy())
    assert np.array_equal(x.grad.numpy(), r.grad.numpy())       # one dx for both, fused.rs:176-181
    s = (xv + rv).astype(np.float64)
    want = (s - s.mean(1, keepdims=True)) / np.sqrt(s.var(1, keepdims=True) + 1e-5) * gv + bv
    assert max_err(out.numpy(), want) < 1e-5
    o = orc.residualLayerNorm(orc.Tensor.rand([2, 4]), orc.Tensor.rand([2, 4]), orc.Tensor.ones([4]).setRequiresGrad(True),
                              orc.Tensor.zeros([4]).setRequiresGrad(True))
    assert o.shape == [2, 4]                                     # test/native.test.ts:28-34


def test_scale_grads_and_grad_scaler(orc):
    p = _t(orc, [1.0, 2.0, 3.0], True)
    p.mul(_t(orc, [4.0, 8.0, 16.0])).sum().mul(1024.0).backward()
    assert orc.native.scaleGrads([p._id], 1.0 / 1024.0) is False
    assert list(p.grad.toFloat32()) == [4.0, 8.0, 16.0]
    assert orc.native.scaleGrads([p._id], float("inf")) is True          # mixed_precision.rs:24-26
    q = _t(orc, [1.0], True)
    q.mul(_t(orc, [float("nan")])).sum().backward()
    assert orc.native.scaleGrads([q._id], 1.0) is True
    assert orc.native.scaleGrads([_t(orc, [1.0])._id], 2.0) is False       # no gradient: nothing to scale

    scaler = orc.GradScaler(initScale=1024)                      # test/module.test.ts:97-105
    assert scaler.getScale() == 1024
    sl = scaler.scaleLoss(_t(orc, [2, 3])).toFloat32()
    assert abs(sl[0] - 2048) < 0.1 and abs(sl[1] - 3072) < 0.1
    # a finite step updates, an overflowing one halves the scale and skips (optimizer.ts:98-120)
    lin = orc.Linear(2, 1, weight=np.ones((2, 1), np.float32), bias=np.zeros(1, np.float32))
    opt = orc.Adam(lin.parameters(), lr=0.1)
    scaler.scaleLoss(lin.forward(_t(orc, [[1.0, 2.0]])).sum()).backward()
    r = scaler.unscaleAndStep(opt)
    assert r["skipped"] is False and abs(r["gradNorm"] - np.sqrt(1 + 4 + 1)) < 1e-5
    w_after = lin.weight.value.numpy().copy()
    opt.zeroGrad()
    lin.forward(_t(orc, [[1.0, 2.0]])).sum().mul(float("inf")).backward()
    r = scaler.unscaleAndStep(opt)
    assert r["skipped"] is True and scaler.getScale() == 512
    assert np.array_equal(lin.weight.value.numpy(), w_after)
    assert not np.any(lin.weight.value.grad.numpy())
