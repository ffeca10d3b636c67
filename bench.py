#!/usr/bin/env python3
"""Benchmark of the fp32 matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extras]

A step is one pass of the hot path over one batch of synthetic input: the
single fp32 product A[4096,4096] x B[4096,4096] (A, B ~ N(0,1), seed 1,
row-major, forward only), with A and B resident in HBM before the timed region.
One JSON line is printed:

* value       TFLOP/s over the K timed steps (wall clock between two stream
              synchronisations), algorithmic flops = 2 * 4096^3 per step;
* roofline    the dominant kernel (gemm_mfma_kernel) against the MI355X fp32
              matrix peak of 157.3 TFLOP/s; `achieved` uses the kernel's
              average launch duration measured with HIP events recorded on the
              stream the kernel runs on;
* cpu_baseline  the CPU oracle (a C restatement of the reference's
              single-threaded CPU backend) timed on this host on a bounded
              sample of the same product (the first 2048 rows of A);
* extra       the other configurations of the path, for information: the
              decode-shaped GEMV against HBM bandwidth, the tall-K weight
              gradient, attention-shaped batched products, and the README-MLP
              and FFN training steps in ms.

Only one GPU is used; --gpus above 1 is refused.
"""
import argparse
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from framework_amd import synth  # noqa: E402
from framework_amd import native as N  # noqa: E402

PEAK_FP32_MATRIX_TFLOPS = 157.3  # MI355X dense fp32 MFMA: 256 CU x 256 FLOP/clk x 2.4 GHz
PEAK_HBM_GBPS = 8000.0

# HBM bytes per gemm_mfma_kernel launch at 4096^3, from the rocprofv3 --pmc
# runs summarised in profiles/gemm_mfma_4096_pmc.txt (FETCH_SIZE + WRITE_SIZE,
# scaled by a copy kernel of known size).  None until measured.
MEASURED_HBM_BYTES_4096 = 797.2e6


def time_launches(r, fn, warmup, iters):
    """Average duration in ms of fn() between two HIP events on the library's stream."""
    for _ in range(warmup):
        fn()
    e0, e1 = r.event(), r.event()
    r.record(e0)
    for _ in range(iters):
        fn()
    r.record(e1)
    ms = r.elapsed_ms(e0, e1) / iters
    r.event_destroy(e0)
    r.event_destroy(e1)
    return ms


def bench_headline(r, steps, warmup):
    M = Nn = K = 4096
    a = synth.normal(1, (M, K))
    b = synth.normal(1, (K, Nn), stream=1)
    dA, dB = r.to_device(a), r.to_device(b)
    dC = r.malloc(M * Nn * 4)
    step = lambda: r.sgemm(M, Nn, K, dA, dB, dC)
    # The uploads above leave the GPU idle, and its clocks need ~20 ms of work to settle
    # (the first launches after an idle spell run 10 % slow): settle first, then the W warm-up steps.
    for _ in range(25):
        step()
    for _ in range(warmup):
        step()
    r.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    r.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    kernel_ms = time_launches(r, step, 2, max(steps, 10))
    # spot check against float64 so that a wrong kernel cannot post a number
    c = r.to_host(dC, (M, Nn))
    rows = [0, 2047, 4095]
    err = float(np.max(np.abs(c[rows] - a[rows].astype(np.float64) @ b.astype(np.float64))))
    tol = 1e-4 * math.sqrt(K) * float(np.abs(a).max()) * float(np.abs(b).max())
    if not err <= tol:
        raise SystemExit("bench: 4096^3 result outside tolerance (%g > %g)" % (err, tol))
    for p in (dA, dB, dC):
        r.free(p)
    return wall_ms, kernel_ms, 2.0 * M * Nn * K, (a, b), err


def bench_extras(r):
    out = {}
    # config 5a: decode-shaped GEMV x[4,4096] W[4096,4096], HBM-bound
    x = synth.normal(4, (4, 4096), 0.02)
    w = synth.normal(4, (4096, 4096), 0.02, stream=1)
    dx, dw, dy = r.to_device(x), r.to_device(w), r.malloc(4 * 4096 * 4)
    # launches of a few microseconds are issued from C (mni_rocm_sgemm_timed) so that the host stays ahead
    ms = r.sgemm_timed([r.gemm_desc(4, 4096, 4096, dx, dw, dy)], 10, 200)
    by = 4.0 * (4096 * 4096 + 2 * 4 * 4096)
    out["config5a_gemv"] = {"us": ms * 1e3, "GB/s": by / ms / 1e6, "frac_hbm": by / ms / 1e6 / PEAK_HBM_GBPS,
                            "note": "W (64 MiB) is re-read every launch and fits the 256 MiB Infinity Cache"}
    # the same after 3000 launches (~40 ms) of it: memory-bound work runs ~5 % slower once the part has been
    # streaming for a while than in a short burst
    ms = r.sgemm_timed([r.gemm_desc(4, 4096, 4096, dx, dw, dy)], 3000, 1000)
    out["config5a_gemv_sustained"] = {"us": ms * 1e3, "GB/s": by / ms / 1e6, "frac_hbm": by / ms / 1e6 / PEAK_HBM_GBPS}
    # the same product over 8 different W in turn (512 MiB working set): HBM-resident
    ws = [r.to_device(w) for _ in range(8)]
    ms = r.sgemm_timed([r.gemm_desc(4, 4096, 4096, dx, p, dy) for p in ws], 16, 200)
    out["config5a_gemv_cold"] = {"us": ms * 1e3, "GB/s": by / ms / 1e6, "frac_hbm": by / ms / 1e6 / PEAK_HBM_GBPS}
    for p in ws + [dx, dw, dy]:
        r.free(p)
    # config 5b: X^T[1024,65536] dY[65536,1024], X^T as a view, split-K
    X = synth.normal(5, (65536, 1024))
    dX, dG, dO = r.to_device(X), r.to_device(X), r.malloc(1024 * 1024 * 4)
    # (30 launches of warm-up: the upload above leaves the GPU idle and its clocks take ~20 ms to settle)
    ms = time_launches(r, lambda: r.sgemm(1024, 1024, 65536, dX, dG, dO, a_strides=(1, 1024)), 30, 20)
    fl = 2.0 * 1024 * 1024 * 65536
    out["config5b_tall_k"] = {"us": ms * 1e3, "TFLOP/s": fl / ms / 1e9, "frac_mfma": fl / ms / 1e9 / PEAK_FP32_MATRIX_TFLOPS}
    for p in (dX, dG, dO):
        r.free(p)
    del X
    # config 3: Q K^T (K^T a permuted view), dQ, dK^T -- batched, near the ridge
    q = synth.normal(2, (32, 512, 64)) / np.float32(8)
    ds = synth.normal(2, (32, 512, 512), stream=2)
    dq, dk, dds = r.to_device(q), r.to_device(q), r.to_device(ds)
    s_out, g_out = r.malloc(32 * 512 * 512 * 4), r.malloc(32 * 512 * 64 * 4)
    fl = 2.0 * 32 * 512 * 512 * 64
    ms_f = r.sgemm_timed([r.gemm_desc(512, 512, 64, dq, dk, s_out, batch=32, a_batch=(512 * 64, 32),
                                      b_strides=(1, 64), b_batch=(512 * 64, 32))], 5, 100)
    ms_q = r.sgemm_timed([r.gemm_desc(512, 64, 512, dds, dk, g_out, batch=32, a_batch=(512 * 512, 32),
                                      b_batch=(512 * 64, 32))], 5, 100)
    ms_k = r.sgemm_timed([r.gemm_desc(64, 512, 512, dq, dds, g_out, batch=32, a_strides=(1, 64),
                                      a_batch=(512 * 64, 32), b_batch=(512 * 512, 32))], 5, 100)
    by = 4.0 * 32 * (512 * 64 * 2 + 512 * 512)
    out["config3_attention_scores"] = {
        "fwd_us": ms_f * 1e3, "dq_us": ms_q * 1e3, "dkT_us": ms_k * 1e3,
        "TFLOP/s": 3 * fl / (ms_f + ms_q + ms_k) / 1e9, "GB/s": 3 * by / (ms_f + ms_q + ms_k) / 1e6}
    for p in (dq, dk, dds, s_out, g_out):
        r.free(p)
    # configs 1 and 4: training steps through the engine (wall clock, trailing sync)
    from framework_amd.api import bind
    api = bind(N.Native())

    def T(a, grad=False):
        t = api.Tensor.fromFloat32(a, list(a.shape))
        return t.setRequiresGrad(True) if grad else t

    def time_step(step, keep, n, warm):
        for _ in range(warm):
            step()
            api.native.gcTensors(keep())
        r.sync()
        total = 0.0
        for _ in range(n):
            t0 = time.perf_counter()
            step()
            r.sync()
            total += time.perf_counter() - t0
            api.native.gcTensors(keep())
        return total * 1e3 / n

    # config 4: FFN step X[4096,1024] -> 4096 (GELU) -> 1024, reference mseLoss, fwd + bwd
    for fused in (False, True):
        api.native.resetEngine()
        d, h, rows = 1024, 4096, 4096
        x = T(synth.normal(3, (rows, d)), True)
        tg = T(synth.normal(3, (rows, d), stream=3))
        l1 = api.Linear(d, h, weight=synth.uniform(3, (d, h), -1 / 32, 1 / 32, stream=1), bias=np.zeros(h, np.float32), fused=fused, activation="gelu")
        l2 = api.Linear(h, d, weight=synth.uniform(3, (h, d), -1 / 64, 1 / 64, stream=2), bias=np.zeros(d, np.float32), fused=fused)
        params = l1.parameters() + l2.parameters()

        def step4():
            api.native.zeroGrad([x._id] + [p.value._id for p in params])
            api.mseLoss(l2.forward(l1.forward(x)), tg).backward()

        def keep4():
            ids = [x._id, tg._id] + [p.value._id for p in params]
            for t in [x] + [p.value for p in params]:
                g = api.native.getGrad(t._id)
                if g is not None:
                    ids.append(g)
            return ids
        ms = time_step(step4, keep4, 20, 15)  # 30 ms of warm-up: the clocks take tens of milliseconds to settle after an idle spell
        out["config4_ffn_step" + ("_fused_linear" if fused else "")] = {
            "ms": ms, "gemm_TFLOP/s_if_all_gemm": 6 * 2.0 * rows * d * h / ms / 1e9}
    # config 1: README MLP step (32x10 -> 64 -> 3, cross-entropy, Adam): launch-latency bound
    api.native.resetEngine()
    x1 = T(synth.uniform(0, (32, 10)))
    m1 = api.Linear(10, 64, weight=synth.uniform(0, (10, 64), -0.316, 0.316, stream=1), bias=synth.uniform(0, (64,), -0.316, 0.316, stream=2))
    m2 = api.Linear(64, 3, weight=synth.uniform(0, (64, 3), -0.125, 0.125, stream=3), bias=synth.uniform(0, (3,), -0.125, 0.125, stream=4))
    params1 = m1.parameters() + m2.parameters()
    targets = [[int(t)] for t in synth.integers(0, (32,), 0, 3, stream=5)]
    opt = api.Adam(params1, lr=1e-3)

    def step1():
        opt.zeroGrad()
        api.crossEntropyLoss(m2.forward(m1.forward(x1).relu()), targets).backward()
        opt.step()

    def keep1():
        ids = [x1._id] + [p.value._id for p in params1]
        ids += [g for g in (api.native.getGrad(p.value._id) for p in params1) if g is not None]
        return ids
    out["config1_readme_mlp_step"] = {"ms": time_step(step1, keep1, 20, 5)}
    # attention on the batched GEMM at the config-3 shapes: flashAttention(q, k, v) [32, 512, 64], causal
    api.native.resetEngine()
    bh, s, d = 32, 512, 64
    qa, ka, va = (T(synth.normal(2, (bh, s, d), stream=i) / np.float32(8 if i < 2 else 1), True) for i in range(3))
    wa = T(synth.normal(2, (bh, s, d), stream=3))

    def keep_att():
        ids = [t._id for t in (qa, ka, va, wa)]
        return ids + [g for g in (api.native.getGrad(t._id) for t in (qa, ka, va)) if g is not None]
    ms_fwd = time_step(lambda: api.flashAttention(qa, ka, va, 0.125, True), keep_att, 20, 5)

    def att_step():
        api.native.zeroGrad([qa._id, ka._id, va._id])
        api.flashAttention(qa, ka, va, 0.125, True).mul(wa).sum().backward()
    ms_all = time_step(att_step, keep_att, 20, 5)
    # the one-kernel forward on long sequences ([8, 8192, 64] and [16, 4096, 128], causal): useful flops = half of dense
    for lb, ls, ld in ((8, 8192, 64), (16, 4096, 128)):
        ql, kl, vl = (T(synth.normal(2, (lb, ls, ld), stream=i)) for i in range(3))
        keep_long = lambda: [ql._id, kl._id, vl._id] + keep_att()
        ms_long = time_step(lambda: api.flashAttention(ql, kl, vl, 1.0 / math.sqrt(ld), True), keep_long, 10, 3)
        out["attention_fwd_%dx%dx%d_causal" % (lb, ls, ld)] = {"ms": ms_long, "useful_TFLOP/s": 2.0 * lb * ls * ls * ld / ms_long / 1e9}
        api.native.gcTensors(keep_att())
    dense = 2.0 * bh * s * s * d  # one s x s x d product, mask not exploited
    out["attention_32x512x64_causal"] = {"fwd_ms": ms_fwd, "fwd_bwd_ms": ms_all,
                                         "fwd_TFLOP/s_dense_count": 2 * dense / ms_fwd / 1e9,
                                         "fwd_bwd_TFLOP/s_dense_count": 7 * dense / ms_all / 1e9,
                                         "note": "wall clock per call incl. host issue and a trailing sync; 2 products forward, 5 backward"}
    # KV-cache decode: 8 x 32 heads of 128, 4096 cached positions, one new token per call
    api.native.resetEngine()
    bsz, nh, hd, hist = 8, 32, 128, 4096
    for quantized in (False, True):
        cache = api.KvCache(bsz, nh, hd, hist + 64, quantized)
        kk = T(synth.normal(6, (bsz, nh, 1, hd)))
        for _ in range(hist):
            cache.append(kk, kk)
        qq = T(synth.normal(6, (bsz, nh, 1, hd), stream=1))
        for _ in range(3):
            cache.decodeStep(qq, kk, kk, 0.088)
        r.sync()
        t0 = time.perf_counter()
        for _ in range(20):
            cache.decodeStep(qq, kk, kk, 0.088)
        r.sync()
        us = (time.perf_counter() - t0) / 20 * 1e6
        by = 2.0 * bsz * nh * (hist + 12) * hd * (1 if quantized else 4)
        out["kv_decode_8x32x128_hist4096_" + ("int8" if quantized else "fp32")] = {"us": us, "GB/s": by / us / 1e3}
        cache.free()
        api.native.gcTensors([])
    # language-model training step: 2 blocks of width 768 (12 heads), 8 x 512 tokens, vocabulary 8192;
    # dataset windows, embeddings, dropout, attention, residual + layernorm, GELU MLP, cross-entropy on
    # buffered targets, clipped AdamW -- everything device-resident
    api.native.resetEngine()
    nat = api.native
    V, D, H, Tn, Bn, L = 8192, 768, 12, 512, 8, 2
    hd_ = D // H
    nat.seed(1)
    u = lambda seed, shape, b: synth.uniform(seed, shape, -b, b)
    lin = lambda sd, i, o, act=None: api.Linear(i, o, weight=u(sd, (i, o), 1 / math.sqrt(i)), bias=np.zeros(o, np.float32), fused=True, activation=act)
    tok, pos = api.Embedding(V, D, weight=u(1, (V, D), 0.05)), api.Embedding(Tn, D, weight=u(2, (Tn, D), 0.05))
    layers = [dict(q=lin(10 + l, D, D), k=lin(20 + l, D, D), v=lin(30 + l, D, D), proj=lin(40 + l, D, D), fc=lin(50 + l, D, 4 * D, "gelu"),
                   out=lin(60 + l, 4 * D, D), g1=api.Parameter(T(np.ones(D, np.float32), True)), b1=api.Parameter(T(np.zeros(D, np.float32), True)),
                   g2=api.Parameter(T(np.ones(D, np.float32), True)), b2=api.Parameter(T(np.zeros(D, np.float32), True))) for l in range(L)]
    head = lin(3, D, V)
    lm_params = [tok.weight, pos.weight] + head.parameters()
    for ly in layers:
        for kname in ("q", "k", "v", "proj", "fc", "out"):
            lm_params += ly[kname].parameters()
        lm_params += [ly["g1"], ly["b1"], ly["g2"], ly["b2"]]
    lm_opt = api.Adam(lm_params, lr=1e-3)
    ds = nat.createDataset((np.arange(1 << 20, dtype=np.int64) * 2654435761 % V).astype(np.int32))
    posidx = [list(range(Tn))] * Bn
    heads = lambda t: t.view(Bn, Tn, H, hd_).permute(0, 2, 1, 3).contiguous().view(Bn * H, Tn, hd_)

    def lm_step():
        inp, tgt = nat.sampleBatch(ds, Tn, Bn)
        h = api.dropout(tok.forwardGpu(inp, Bn, Tn).add(pos.forward(posidx)), 0.1)
        for ly in layers:
            att = api.flashAttention(heads(ly["q"].forward(h)), heads(ly["k"].forward(h)), heads(ly["v"].forward(h)), 1 / math.sqrt(hd_), True)
            att = att.view(Bn, H, Tn, hd_).permute(0, 2, 1, 3).contiguous().view(Bn, Tn, D)
            h1 = api.residualLayerNorm(api.dropout(ly["proj"].forward(att), 0.1), h, ly["g1"].value, ly["b1"].value)
            h = api.residualLayerNorm(api.dropout(ly["out"].forward(ly["fc"].forward(h1)), 0.1), h1, ly["g2"].value, ly["b2"].value)
        loss = api.crossEntropyLossGpu(head.forward(h), tgt)
        lm_opt.zeroGrad()
        loss.backward()
        lm_opt.step(1.0)
        nat.freeIntBuffer(inp)
        nat.freeIntBuffer(tgt)

    def keep_lm():
        ids = [p.value._id for p in lm_params]
        return ids + [g for g in (nat.getGrad(p.value._id) for p in lm_params) if g is not None]
    ms = time_step(lm_step, keep_lm, 15, 6)
    per_tok = 6.0 * (L * 12 * D * D + D * V) + L * 3.5 * 4 * Tn * D  # matmul FLOPs per token, fwd + bwd (attention counted dense)
    out["lm_step_2x768_8x512_vocab8192"] = {"ms": ms, "tokens/s": Bn * Tn / ms * 1e3, "matmul_TFLOP/s": per_tok * Bn * Tn / ms / 1e9}
    # token-side kernels on their own (wall clock per call incl. host issue; bytes = algorithmic)
    api.native.resetEngine()
    xt, rt = T(synth.normal(7, (8192, 768))), T(synth.normal(7, (8192, 768), stream=1))
    gm, bt = T(np.ones(768, np.float32)), T(np.zeros(768, np.float32))
    wemb = T(u(8, (32768, 768), 0.05), True)
    idx = np.asarray(synth.integers(9, (8192,), 0, 32768), dtype=np.int64)

    def keep_tok():
        g = nat.getGrad(wemb._id)
        return [t._id for t in (xt, rt, gm, bt, wemb)] + ([g] if g is not None else [])

    def timed(fn, n=20):
        # every call is followed by a collection (untimed), as in a training loop, so buffers come from the allocator's cache
        total = 0.0
        for it in range(n + 3):
            r.sync()
            t0 = time.perf_counter()
            fn()
            r.sync()
            if it >= 3:
                total += time.perf_counter() - t0
            nat.gcTensors(keep_tok())
        return total / n * 1e6
    nb = 8192 * 768 * 4.0
    us_d = timed(lambda: nat.dropoutOp(xt._id, 0.1, True))
    us_l = timed(lambda: nat.residualLayernorm(xt._id, rt._id, gm._id, bt._id, 1e-5))
    us_e = timed(lambda: nat.embeddingForward(wemb._id, idx, 8, 1024))

    def emb_fb():
        nat.zeroGrad([wemb._id])
        api.Tensor(nat.embeddingForward(wemb._id, idx, 8, 1024)).mul(xt.view(8, 1024, 768)).sum().backward()
    us_eb = timed(emb_fb, 10)
    out["token_ops_8192x768"] = {
        "dropout_us": us_d, "dropout_GB/s": 2 * nb / us_d / 1e3,
        "residual_layernorm_us": us_l, "residual_layernorm_GB/s": 4 * nb / us_l / 1e3,
        "embedding_forward_us": us_e, "embedding_forward_GB/s": 2 * nb / us_e / 1e3,
        "embedding_forward_backward_vocab32768_us": us_eb,
        "note": "one call, then a sync; embedding_forward includes the host-to-device copy of 8192 indices"}
    api.native.resetEngine()
    return out


def run_for_counters(r, which):
    """Launch sequence for hardware-counter runs: the strided-copy kernel x3 on
    a contiguous 16M-float buffer (64 MiB read, 64 MiB written: the yardstick
    the counters are scaled by), then the product x5."""
    n = 4096 * 4096
    src = r.to_device(synth.normal(9, (n,)))
    dst = r.malloc(n * 4)
    for _ in range(3):
        r.strided_copy(dst, src, [n], [1])
    if which == "gemm":
        a, b = r.to_device(synth.normal(1, (4096, 4096))), r.to_device(synth.normal(1, (4096, 4096), stream=1))
        for _ in range(5):
            r.sgemm(4096, 4096, 4096, a, b, dst)
    elif which == "streamk":
        # a mid-size product whose 192 tiles do not fill a round: the planner deals its K steps (stream-K)
        a, b = r.to_device(synth.normal(1, (4096, 3072))), r.to_device(synth.normal(1, (3072, 768), stream=1))
        for _ in range(5):
            r.sgemm(4096, 768, 3072, a, b, dst)
    elif which == "attention":
        # the one-kernel attention forward on [8, 8192, 64], causal, through the engine entry point
        from framework_amd.api import bind
        api = bind(N.Native())
        q, k, v = (api.Tensor.fromFloat32(synth.normal(2, (8, 8192, 64), stream=i), [8, 8192, 64]) for i in range(3))
        for _ in range(5):
            api.flashAttention(q, k, v, 0.125, True)
            api.native.gcTensors([q._id, k._id, v._id])
    elif which == "attention_bwd":
        # forward + backward of the same attention: the query-owned and the key-owned backward kernels
        from framework_amd.api import bind
        api = bind(N.Native())
        mk = lambda i, g: api.Tensor.fromFloat32(synth.normal(2, (8, 8192, 64), stream=i), [8, 8192, 64]).setRequiresGrad(g)
        q, k, v, w = mk(0, True), mk(1, True), mk(2, True), mk(3, False)
        for _ in range(3):
            api.native.zeroGrad([t._id for t in (q, k, v)])
            api.flashAttention(q, k, v, 0.125, True).mul(w).sum().backward()
            grads = [g for g in (api.native.getGrad(t._id) for t in (q, k, v)) if g is not None]
            api.native.gcTensors([t._id for t in (q, k, v, w)] + grads)
    else:
        x, w = r.to_device(synth.normal(4, (4, 4096), 0.02)), r.to_device(synth.normal(4, (4096, 4096), 0.02, stream=1))
        for _ in range(5):
            r.sgemm(4, 4096, 4096, x, w, dst)
    r.sync()
    print(json.dumps({"counters_run": which, "copy_bytes_read": n * 4, "copy_bytes_written": n * 4}))


def cpu_baseline(a, b, target_seconds):
    """The CPU oracle's matmul (clones and i-k-j loop, one thread) on the first
    rows of A against all of B; the row count is chosen from a short
    calibration run so that the sample takes about `target_seconds`."""
    from framework_amd.api import bind
    from oracle.native import OracleNative
    orc = bind(OracleNative())
    orc.native.resetEngine()
    B0 = orc.Tensor.fromFloat32(b, list(b.shape))
    t0 = time.perf_counter()
    orc.Tensor.fromFloat32(a[:128], [128, a.shape[1]]).matmul(B0)
    per_row = (time.perf_counter() - t0) / 128
    orc.native.resetEngine()
    sample_rows = int(min(a.shape[0], max(128, (target_seconds / per_row) // 128 * 128)))
    A = orc.Tensor.fromFloat32(a[:sample_rows], [sample_rows, a.shape[1]])
    B = orc.Tensor.fromFloat32(b, list(b.shape))
    t0 = time.perf_counter()
    C = A.matmul(B)
    dt = time.perf_counter() - t0
    del C
    orc.native.resetEngine()
    fl = 2.0 * sample_rows * a.shape[1] * b.shape[1]
    return {"value": fl / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": "first %d of 4096 rows of A against all of B (%.1f GFLOP, %.1f s), oracle/mni_oracle.c "
                      "built -O3 -ffp-contract=off without -march=native; host has %d logical cores, 1 used"
                      % (sample_rows, fl / 1e9, dt, os.cpu_count() or 0)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip the other configurations")
    ap.add_argument("--cpu-sample-seconds", type=float, default=12.0, help="target CPU time of the baseline sample")
    ap.add_argument("--counters", choices=["gemm", "gemv", "streamk", "attention", "attention_bwd"], default=None,
                    help="for rocprofv3 --pmc runs: launch a copy kernel of known size (64 MiB read + 64 MiB "
                         "written) 3 times, then the chosen product 5 times, and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (got --gpus %d)" % args.gpus)

    r = N.Rocm()
    r.init(0)
    info = r.device_info()
    if args.counters:
        run_for_counters(r, args.counters)
        return
    wall_ms, kernel_ms, flops, (a, b), err = bench_headline(r, args.steps, args.warmup)
    value = flops / wall_ms / 1e9
    achieved = flops / kernel_ms / 1e9
    line = {
        "metric": "fp32 matmul TFLOP/s", "value": value, "unit": "TFLOP/s",
        "pct_of_fp32_matrix_peak": 100.0 * value / PEAK_FP32_MATRIX_TFLOPS,
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "single fp32 matmul A[4096,4096] x B[4096,4096], A,B ~ N(0,1) seed 1, row-major, forward only",
                   "M": 4096, "N": 4096, "K": 4096, "device": info["name"].strip(), "compute_units": info["compute_units"],
                   "max_err_vs_f64_sample": err},
        "roofline": {"bound": "mfma", "kernel": "gemm_mfma_kernel<0, 1, 2, 2, false>", "achieved": achieved,
                     "peak": PEAK_FP32_MATRIX_TFLOPS, "unit": "TFLOP/s", "frac": achieved / PEAK_FP32_MATRIX_TFLOPS,
                     "kernel_ms": kernel_ms, "algorithmic_flops": flops, "traffic": MEASURED_HBM_BYTES_4096},
    }
    if not args.no_extras:
        line["extra"] = bench_extras(r)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(a, b, args.cpu_sample_seconds)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
