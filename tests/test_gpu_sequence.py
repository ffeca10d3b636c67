"""Token-side ops on the GPU against the CPU oracle through the engine-level C
ABI: the Philox stream (bit for bit), rand (bit for bit) / randn (1e-5: device
log / sin / cos), dropout (same seed, same mask, bit for bit), dataset windows,
embedding forward and its ordered scatter-add backward (bit for bit), tile,
residual + layernorm (2e-6 relative: wavefront sums), cross-entropy with
buffered targets, gradient unscaling, and one language-model training step end
to end."""
import math

import numpy as np
import pytest

from framework_amd import synth
from framework_amd.api import bind
from helpers import max_err

pytestmark = pytest.mark.gpu


def _t(api, a, grad=False):
    a = np.asarray(a, dtype=np.float32)
    t = api.Tensor.fromFloat32(a, list(a.shape))
    return t.setRequiresGrad(True) if grad else t


@pytest.fixture()
def both(rocm_native, oracle_native):
    gpu, cpu = bind(rocm_native), bind(oracle_native)
    yield gpu, cpu
    rocm_native.resetEngine()
    oracle_native.resetEngine()


def test_philox_stream_is_bit_exact(both):
    gpu, cpu = both
    assert list(gpu.native.philoxWords(0, 0, 4)) == [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]   # Random123 kat_vectors
    for seed, offset, n in [(0, 0, 4), (0x299f31d0a4093822, 0x85a308d3243f6a88, 4099), (2 ** 64 - 1, 2 ** 32 - 2, 1030)]:
        assert np.array_equal(gpu.native.philoxWords(seed, offset, n), cpu.native.philoxWords(seed, offset, n))


def test_rand_and_randn_follow_the_seeded_stream(both):
    gpu, cpu = both
    for api in both:
        api.native.seed(12345)
    for shape in ([7], [300, 257], [2, 3, 5]):
        assert np.array_equal(gpu.Tensor.rand(shape).numpy(), cpu.Tensor.rand(shape).numpy())
        assert max_err(gpu.Tensor.randn(shape).numpy(), cpu.Tensor.randn(shape).numpy()) < 1e-5
    u = gpu.Tensor.rand([1 << 20]).numpy().astype(np.float64)
    assert u.min() >= 0 and u.max() < 1 and abs(u.mean() - 0.5) < 2e-3 and abs(u.var() - 1 / 12) < 1e-3
    z = gpu.Tensor.randn([1 << 20]).numpy().astype(np.float64)
    assert np.all(np.isfinite(z)) and abs(z.mean()) < 5e-3 and abs(z.var() - 1) < 1e-2
    # unseeded engines still produce a valid stream (the reference's thread RNG is unseedable)
    gpu.native.resetEngine()
    assert 0.4 < gpu.Tensor.rand([4096]).numpy().mean() < 0.6


@pytest.mark.parametrize("shape,rate", [((1000,), 0.5), ((64, 257), 0.1), ((3, 5, 7), 0.9), ((1 << 20,), 0.25)])
def test_dropout_matches_the_oracle_under_one_seed(both, shape, rate):
    gpu, cpu = both
    xv = synth.uniform(5, shape, 0.5, 2.0) * np.where(synth.normal(6, shape) > 0, 1, -1).astype(np.float32)
    wv = synth.normal(7, shape, stream=1)
    res = []
    for api in both:
        api.native.seed(99)
        api.Tensor.rand([5])                                    # move the stream off its origin
        x = _t(api, xv, True)
        y = api.dropout(x, rate)
        y.mul(_t(api, wv)).sum().backward()
        res.append((y.numpy(), x.grad.numpy()))
    assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1], res[1][1])
    kept = res[0][0] != 0
    assert abs(kept.mean() - (1 - rate)) < 5 * math.sqrt(rate * (1 - rate) / xv.size) + 1e-9
    assert np.array_equal(res[0][1] != 0, kept)


def test_dropout_passthrough_and_reference_assertions(both):
    gpu, _ = both
    x = _t(gpu, [1, 2, 3, 4])
    assert gpu.native.dropoutOp(x._id, 0.5, False) == x._id and gpu.native.dropoutOp(x._id, 0.0, True) == x._id
    d = gpu.dropout(gpu.Tensor.ones([1000]), 0.5, False).toFloat32()             # test/nn.test.ts:239-244
    zeros = int(np.sum(d == 0))
    assert 100 < zeros < 900 and set(np.unique(d)) <= {0.0, 2.0}
    # a permuted view is dropped by its logical contents
    a = synth.normal(3, (5, 6))
    gpu.native.seed(4)
    y1 = gpu.dropout(_t(gpu, a).permute(1, 0), 0.5).numpy()
    gpu.native.seed(4)
    y2 = gpu.dropout(_t(gpu, np.ascontiguousarray(a.T)), 0.5).numpy()
    assert np.array_equal(y1, y2)


def test_dataset_windows_on_the_device(both):
    gpu, _ = both
    n = gpu.native
    data = np.arange(5000, dtype=np.int32)                      # value == position: a window names its start
    ds = n.createDataset(data)
    n.seed(1)
    seen = set()
    for _ in range(20):
        inp, tgt = n.sampleBatch(ds, 64, 16)
        a, b = n.intBufferToHost(inp).reshape(16, 64), n.intBufferToHost(tgt).reshape(16, 64)
        assert np.array_equal(a, a[:, :1] + np.arange(64)) and np.array_equal(b, a + 1)
        assert a[:, 0].min() >= 0 and a[:, 0].max() < 5000 - 64 - 1         # gen_range(0..len - block - 1)
        seen.update(a[:, 0].tolist())
        n.freeIntBuffer(inp)
        n.freeIntBuffer(tgt)
    assert len(seen) > 250                                       # 320 draws out of 4935 starts
    starts = np.array(sorted(seen))
    assert starts.min() < 500 and starts.max() > 4400            # spread over the whole range
    with pytest.raises(Exception):
        n.sampleBatch(n.createDataset(np.arange(65, dtype=np.int32)), 64, 1)     # empty range
    with pytest.raises(Exception):
        n.sampleBatch(99, 8, 1)
    n.seed(1)
    first = n.intBufferToHost(n.sampleBatch(ds, 64, 16)[0])
    n.seed(1)
    assert np.array_equal(first, n.intBufferToHost(n.sampleBatch(ds, 64, 16)[0]))


@pytest.mark.parametrize("vocab,dim,batch,seq,distinct", [(37, 24, 5, 19, 6), (1000, 64, 8, 128, 1000), (50, 7, 3, 11, 50),
                                                          (300, 768, 4, 256, 40), (5, 4, 1, 1, 1)])
def test_embedding_matches_the_oracle_bit_for_bit(both, vocab, dim, batch, seq, distinct):
    rng = np.random.default_rng(vocab + dim)
    idx = rng.integers(0, distinct, size=(batch, seq))
    idx.flat[0] = vocab - 1
    w, g = synth.normal(1, (vocab, dim)), synth.normal(3, (batch, seq, dim))
    res = []
    for api in both:
        emb = api.Embedding(vocab, dim, weight=w)
        out = emb.forward(idx.tolist())
        out.mul(_t(api, g)).sum().backward()
        res.append((out.numpy(), emb.weight.value.grad.numpy()))
    assert np.array_equal(res[0][0], w[idx]) and np.array_equal(res[0][0], res[1][0])
    assert np.array_equal(res[0][1], res[1][1])                  # same additions in the same (token) order


def test_embedding_one_row_used_by_every_token(both):
    gpu, cpu = both                                              # the longest possible bucket: all 4096 tokens hit row 2
    w, g = synth.normal(1, (4, 32)), synth.normal(3, (8, 512, 32))
    idx = np.full((8, 512), 2)
    res = []
    for api in both:
        emb = api.Embedding(4, 32, weight=w)
        emb.forward(idx.tolist()).mul(_t(api, g)).sum().backward()
        res.append(emb.weight.value.grad.numpy())
    assert np.array_equal(res[0], res[1]) and not np.any(res[0][[0, 1, 3]])


def test_embedding_errors(both):
    gpu, _ = both
    emb = gpu.Embedding(10, 4)
    assert emb.forward([[0, 1, 2], [3, 4, 5]]).shape == [2, 3, 4]                # test/nn.test.ts:197-203
    same = emb.forward([[0, 0], [0, 0]]).toFloat32()
    assert same[0] == same[4]
    with pytest.raises(Exception, match="out of range"):
        emb.forward([[10]])
    with pytest.raises(Exception, match="out of range"):
        emb.forward([[-1]])
    with pytest.raises(Exception):
        gpu.native.embeddingForward(emb.weight.value._id, [1, 2, 3], 2, 2)       # 3 indices for 4 tokens
    ds = gpu.native.createDataset(np.array([1, 2, 30, 4, 5, 6, 7, 8], dtype=np.int32))
    with pytest.raises(Exception, match="out of range"):
        emb.forwardGpu(ds, 2, 2)                                                 # the buffer can hold 30 >= 10 rows


def test_int_buffer_forms_equal_the_host_forms(both):
    vocab, dim = 50, 8
    w = synth.normal(4, (vocab, dim))
    data = (np.arange(400) * 13 % vocab).astype(np.int32)
    logits = synth.normal(5, (3, 16, vocab))
    res = []
    for api in both:
        n = api.native
        ds = n.createDataset(data)
        if n.name == "rocm":
            n.seed(5)
            inp, tgt = n.sampleBatch(ds, 16, 3)
            # recover each window's start from the data it copied
            pos = [next(s for s in range(383) if np.array_equal(data[s:s + 16], row)) for row in n.intBufferToHost(inp).reshape(3, 16)]
        else:
            inp, tgt = n.sampleBatchAt(ds, 16, 3, pos)
        emb = api.Embedding(vocab, dim, weight=w)
        e = emb.forwardGpu(inp, 3, 16)
        lg = _t(api, logits, True)
        loss = api.crossEntropyLossGpu(lg, tgt)
        loss.backward()
        res.append((n.intBufferToHost(inp), n.intBufferToHost(tgt), e.numpy(), loss.item(), lg.grad.numpy()))
    assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1], res[1][1])
    assert np.array_equal(res[0][2], res[1][2])
    assert abs(res[0][3] - res[1][3]) < 2e-6 * abs(res[1][3])
    assert max_err(res[0][4], res[1][4]) < 1e-7
    gpu = both[0]
    bad = gpu.native.createDataset(np.array([0, 1, 2, 3, 99], dtype=np.int32))
    with pytest.raises(Exception, match="out of range"):
        gpu.crossEntropyLossGpu(_t(gpu, np.zeros((4, 50))), bad)


@pytest.mark.parametrize("n,v", [(5, 3), (33, 512), (17, 516), (64, 2048), (9, 2050), (12, 4100), (40, 8192), (6, 8196), (3, 20000),
                                 (1, 2), (32, 3), (64, 3), (65, 3), (33, 496), (64, 256), (16, 1001), (2, 8190)])
def test_cross_entropy_row_kernels_match_the_oracle(both, n, v):
    # every row-kernel variant: scalar rows, rows cached in registers at two depths, a workgroup per row, long rows;
    # from (1, 2) on, batches small enough for the single launch (rows and their mean by one workgroup) and
    # their neighbours just outside it
    logits = synth.normal(n + v, (n, v)) * 3.0
    targets = [[int(t)] for t in np.random.default_rng(v).integers(0, v, size=n)]
    res = []
    for api in both:
        lg = _t(api, logits, True)
        loss = api.crossEntropyLoss(lg, targets)
        loss.mul(3.0).backward()
        res.append((loss.item(), lg.grad.numpy()))
    assert abs(res[0][0] - res[1][0]) < 4e-6 * abs(res[1][0])
    assert max_err(res[0][1], res[1][1]) < 4e-6 * float(np.abs(res[1][1]).max())   # the row sum runs in another order
    # backward() from the loss itself (a small batch's gradient for that case is written by the forward launch)
    direct = []
    for api in both:
        lg = _t(api, logits, True)
        api.crossEntropyLoss(lg, targets).backward()
        direct.append(lg.grad.numpy())
    assert max_err(direct[0], direct[1]) < 4e-6 * float(np.abs(direct[1]).max())
    assert max_err(direct[0] * np.float32(3.0), res[0][1]) < 1e-6 * float(np.abs(res[0][1]).max())
    lp = logits.astype(np.float64)
    want = np.mean(np.log(np.exp(lp - lp.max(1, keepdims=True)).sum(1)) + lp.max(1) - lp[np.arange(n), [t[0] for t in targets]])
    assert abs(res[0][0] - want) < 1e-5 * abs(want)


def test_tile_matches_numpy_and_the_oracle(both):
    gpu, cpu = both
    t = gpu.tile(_t(gpu, [[1, 2, 3]]), [2, 1])                   # test/nn.test.ts:181-190
    assert t.shape == [2, 3] and list(t.toFloat32()) == [1, 2, 3, 1, 2, 3]
    assert gpu.tile(_t(gpu, [[1, 2]]), [3, 2]).shape == [3, 4]
    for shape, reps in [((2, 3), (2, 2)), ((3,), (4,)), ((2, 1, 3), (1, 5, 2)), ((2, 3, 4, 2), (2, 1, 3, 2)), ((64, 257), (3, 2))]:
        a = synth.normal(1, shape)
        got = gpu.tile(_t(gpu, a), list(reps))
        assert got.shape == list(np.tile(a, reps).shape) and np.array_equal(got.numpy(), np.tile(a, reps))
        assert np.array_equal(got.numpy(), cpu.tile(_t(cpu, a), list(reps)).numpy())
    a = synth.normal(2, (3, 4))
    assert np.array_equal(gpu.tile(_t(gpu, a).permute(1, 0), [2, 2]).numpy(), np.tile(a.T, (2, 2)))
    with pytest.raises(Exception, match="reps must match"):
        gpu.tile(_t(gpu, a), [2])


@pytest.mark.parametrize("rows,c", [(33, 70), (4, 4), (512, 768), (7, 1), (1, 1000), (8, 4096), (3, 1024), (2, 8192), (5, 2052)])
def test_residual_layernorm_matches_the_oracle(both, rows, c):
    xv, rv = synth.normal(1, (rows, c)), synth.normal(2, (rows, c), stream=1)
    gv, bv = synth.uniform(3, (c,), 0.5, 1.5), synth.normal(4, (c,), stream=2)
    wv = synth.normal(5, (rows, c), stream=3)
    res = []
    for api in both:
        x, r, g, b = _t(api, xv, True), _t(api, rv, True), _t(api, gv, True), _t(api, bv, True)
        out = api.residualLayerNorm(x, r, g, b, 1e-5)
        out.mul(_t(api, wv)).sum().backward()
        res.append([out.numpy()] + [t.grad.numpy() for t in (x, r, g, b)])
    for got, want in zip(res[0], res[1]):
        scale = max(1.0, float(np.abs(want).max()))
        # column sums over `rows` terms in another order than the oracle's: rounding grows like sqrt(rows)
        assert max_err(got, want) < 4e-6 * scale * max(1.0, math.sqrt(rows) / 4)
    assert np.array_equal(res[0][1], res[0][2])                  # one dx for x and the residual


def test_scale_grads_and_grad_scaler_on_the_gpu(both):
    gpu, cpu = both
    for api in both:
        p = _t(api, synth.normal(1, (300, 33)), True)
        p.mul(_t(api, synth.normal(2, (300, 33)))).sum().mul(1024.0).backward()
        assert api.native.scaleGrads([p._id], 1.0 / 1024.0) is False
        assert np.array_equal(p.grad.numpy(), synth.normal(2, (300, 33)))
    p = _t(gpu, np.ones(5000), True)
    v = np.ones(5000, np.float32)
    v[4321] = np.inf
    p.mul(_t(gpu, v)).sum().backward()
    assert gpu.native.scaleGrads([p._id], 0.5) is True
    q = _t(gpu, [1.0, 2.0], True)
    q.mul(_t(gpu, [float("nan"), 1.0])).sum().backward()
    assert gpu.native.scaleGrads([q._id], 1.0) is True
    assert gpu.native.scaleGrads([_t(gpu, [1.0])._id], 2.0) is False
    r = _t(gpu, [1e30, 1.0], True)
    r.mul(_t(gpu, [1.0, 1.0])).sum().mul(1e30).backward()          # 1e30 finite, its product with 1e30 is not
    assert gpu.native.scaleGrads([r._id], 1e30) is True

    scaler = gpu.GradScaler(initScale=1024)
    lin = gpu.Linear(2, 1, weight=np.ones((2, 1), np.float32), bias=np.zeros(1, np.float32))
    opt = gpu.Adam(lin.parameters(), lr=0.1)
    scaler.scaleLoss(lin.forward(_t(gpu, [[1.0, 2.0]])).sum()).backward()
    out = scaler.unscaleAndStep(opt)
    assert out["skipped"] is False and abs(out["gradNorm"] - math.sqrt(6)) < 1e-5
    w_after = lin.weight.value.numpy().copy()
    opt.zeroGrad()
    lin.forward(_t(gpu, [[1.0, 2.0]])).sum().mul(float("inf")).backward()
    out = scaler.unscaleAndStep(opt)
    assert out["skipped"] is True and scaler.getScale() == 512 and np.array_equal(lin.weight.value.numpy(), w_after)


def _lm_step(api, cfg, weights, data, starts=None):
    """One training step of a small pre-norm-free GPT block the way the reference's ops compose it:
    embeddings from an int buffer, attention, residual + layernorm, dropout, GELU MLP, tied-free head,
    cross-entropy on buffered targets, clipped AdamW."""
    n = api.native
    V, D, H, T, B = cfg
    n.seed(2024)
    tok = api.Embedding(V, D, weight=weights["tok"])
    pos = api.Embedding(T, D, weight=weights["pos"])
    P = lambda k: api.Parameter(_t(api, weights[k], True))
    qkv_w, proj_w, fc_w, out_w, head_w = P("qkv"), P("proj"), P("fc"), P("out"), P("head")
    fc_b, out_b = P("fc_b"), P("out_b")
    g1, b1, g2, b2 = P("g1"), P("b1"), P("g2"), P("b2")
    params = [tok.weight, pos.weight, qkv_w, proj_w, fc_w, out_w, head_w, fc_b, out_b, g1, b1, g2, b2]
    opt = api.Adam(params, lr=1e-2)
    ds = n.createDataset(data)
    losses = []
    picked = []
    for step in range(2):
        if n.name == "rocm":
            inp, tgt = n.sampleBatch(ds, T, B)
            a, b = n.intBufferToHost(inp).reshape(B, T), n.intBufferToHost(tgt).reshape(B, T)
            picked.append(np.concatenate([a, b[:, -1:]], axis=1))                  # each window and the token after it
        else:
            inp, tgt = n.sampleBatchAt(ds, T, B, starts[step])
        h0 = tok.forwardGpu(inp, B, T).add(pos.forward([list(range(T))] * B))
        h0 = api.dropout(h0, 0.1)
        qkv = h0.matmul(qkv_w.value)                                               # [B, T, 3D]
        heads = lambda i: _slice_heads(api, qkv, i, B, T, D, H)
        att = api.flashAttention(heads(0), heads(1), heads(2), 1.0 / math.sqrt(D // H), True)   # [B*H, T, D/H]
        att = att.view(B, H, T, D // H).permute(0, 2, 1, 3).contiguous().view(B, T, D)
        h1 = api.residualLayerNorm(att.matmul(proj_w.value), h0, g1.value, b1.value)
        mlp = api.biasGelu(h1.matmul(fc_w.value), fc_b.value).matmul(out_w.value).add(out_b.value)
        h2 = api.residualLayerNorm(api.dropout(mlp, 0.1), h1, g2.value, b2.value)
        loss = api.crossEntropyLossGpu(h2.matmul(head_w.value), tgt)
        opt.zeroGrad()
        loss.backward()
        norm = opt.step(1.0)
        losses.append((loss.item(), norm))
        n.freeIntBuffer(inp)
        n.freeIntBuffer(tgt)
    return losses, [p.value.numpy() for p in params], picked


def _slice_heads(api, qkv, i, B, T, D, H):
    # column block i of [B, T, 3D] as [B*H, T, D/H]: a selection matmul keeps everything on the tape
    sel = np.zeros((3 * D, D), np.float32)
    sel[i * D:(i + 1) * D] = np.eye(D, dtype=np.float32)
    x = qkv.matmul(_t(api, sel))
    return x.view(B, T, H, D // H).permute(0, 2, 1, 3).contiguous().view(B * H, T, D // H)


def test_language_model_step_end_to_end(both):
    gpu, cpu = both
    V, D, H, T, B = 67, 32, 4, 16, 3
    cfg = (V, D, H, T, B)
    u = lambda seed, shape, bound: synth.uniform(seed, shape, -bound, bound)
    weights = {"tok": u(1, (V, D), 0.2), "pos": u(2, (T, D), 0.2), "qkv": u(3, (D, 3 * D), 0.18), "proj": u(4, (D, D), 0.18),
               "fc": u(5, (D, 4 * D), 0.18), "out": u(6, (4 * D, D), 0.09), "head": u(7, (D, V), 0.18),
               "fc_b": u(8, (4 * D,), 0.1), "out_b": u(9, (D,), 0.1), "g1": 1 + u(10, (D,), 0.1), "b1": u(11, (D,), 0.1),
               "g2": 1 + u(12, (D,), 0.1), "b2": u(13, (D,), 0.1)}
    data = ((np.arange(600) * 31 + (np.arange(600) // 7)) % V).astype(np.int32)
    g_losses, g_params, picked = _lm_step(gpu, cfg, weights, data)
    # the oracle takes the window starts as an argument: find where the windows the GPU run sampled lie in the data
    starts = [[next(s for s in range(len(data) - T - 1) if np.array_equal(data[s:s + T + 1], row)) for row in rows]
              for rows in picked]
    c_losses, c_params, _ = _lm_step(cpu, cfg, weights, data, starts)
    for (gl, gn), (cl, cn) in zip(g_losses, c_losses):
        assert abs(gl - cl) < 2e-5 * abs(cl) and abs(gn - cn) < 2e-4 * abs(cn)
    assert g_losses[0][0] > math.log(V) * 0.8
    # AdamW's first steps move a weight by about lr * sign(g): where g is within rounding of zero the two runs
    # may step in opposite directions, so a handful of entries may differ by up to 2 lr per step; the rest agree.
    for gp, cp in zip(g_params, c_params):
        d = np.abs(gp.astype(np.float64) - cp)
        assert np.mean(d > 2e-4) < 2e-3 and d.max() <= 4.1e-2 and d.mean() < 2e-5
