#!/usr/bin/env python3
"""Benchmark of the fp32 matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extras]
    python bench.py --planner-check        (MNI_ALGO_AUTO against the recorded best forced plan per shape)

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
* other       rows that are not among the configurations the metric is quoted
              on (what the device gives a kernel that only streams or only
              multiplies, batched decoding, small-batch weight gradients,
              attention, the KV cache) -- printed first;
* extra       the other four configurations, printed LAST and kept short so
              that they survive in a record that keeps the end of the line:
              config1 (README MLP step: ms through a plain-C loop over the
              engine ABI, the ctypes figure beside it, launches per step),
              config3 (the three attention-shaped batched products), config4
              (FFN training step), config5a (decode GEMV against HBM
              bandwidth, weights cold) and config5b (tall-K weight gradient),
              each with `frac` against the roof that bounds it, `traffic`
              from the committed counter summaries, and a `cpu_baseline`.

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

SETTLE_LAUNCHES = 25  # untimed launches ahead of the --warmup steps (see bench_headline)


def profile_traffic(name):
    """HBM-side bytes per launch of a kernel as its committed rocprofv3 --pmc summary under profiles/ states them
    (FETCH_SIZE + WRITE_SIZE, each scaled by what the same counter reads for a copy kernel of known size): the
    line `traffic = <x> MB`.  None when the summary is absent."""
    import re
    try:
        text = open(os.path.join(ROOT, "profiles", name)).read()
    except OSError:
        return None
    m = re.search(r"traffic = ([0-9.]+) MB", text)
    return float(m.group(1)) * 1e6 if m else None


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
    for _ in range(SETTLE_LAUNCHES):
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


def roofline(bound, kernel, seconds, flops, nbytes, traffic=None):
    """Roofline object of one kernel launch (or one step): algorithmic flops and bytes against the datasheet
    peaks; `frac` is taken against the roof that bounds the work."""
    tf, gb = flops / seconds / 1e12, nbytes / seconds / 1e9
    out = {"bound": bound, "kernel": kernel, "us": seconds * 1e6, "algorithmic_flops": flops, "algorithmic_bytes": nbytes,
           "TFLOP/s": tf, "GB/s": gb, "frac_mfma": tf / PEAK_FP32_MATRIX_TFLOPS, "frac_hbm": gb / PEAK_HBM_GBPS, "traffic": traffic}
    if bound == "mfma":
        out.update(achieved=tf, peak=PEAK_FP32_MATRIX_TFLOPS, unit="TFLOP/s", frac=tf / PEAK_FP32_MATRIX_TFLOPS)
    else:
        out.update(achieved=gb, peak=PEAK_HBM_GBPS, unit="GB/s", frac=gb / PEAK_HBM_GBPS)
    return out


def sig(x, digits=4):
    """x rounded to a few significant digits (the record keeps the end of the line: every byte counts)."""
    if isinstance(x, float):
        return float("%.*g" % (digits, x))
    if isinstance(x, dict):
        return {k: sig(v, digits) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [sig(v, digits) for v in x]
    return x


def brief(roof, **more):
    """The fields of a roofline object that a reader of the record needs."""
    out = {k: roof[k] for k in ("us", "frac", "bound", "kernel", "achieved", "peak", "unit", "traffic") if k in roof}
    out.update(more)
    return sig(out)


def brief_cpu(cpu):
    return sig({k: cpu[k] for k in ("value", "unit", "cores", "kind", "sample") if k in cpu})


def profile_value(name, label):
    """A figure from a committed profile summary: the number on the line `<label> = <x>`."""
    import re
    try:
        text = open(os.path.join(ROOT, "profiles", name)).read()
    except OSError:
        return None
    m = re.search(re.escape(label) + r" = ([0-9.]+)", text)
    return float(m.group(1)) if m else None


def c_loop_step(fused):
    """The README step driven from plain C over the engine ABI (framework_amd/lib/mlp_step_bench, built with the library):
    its JSON line, or None when the program is not there."""
    import subprocess
    exe = os.path.join(ROOT, "framework_amd", "lib", "mlp_step_bench")
    if not os.path.exists(exe):
        return None
    p = subprocess.run([exe, "1" if fused else "0", "1000", "100"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    if p.returncode != 0:
        return {"error": (p.stderr or p.stdout).strip()[-200:]}
    return json.loads(p.stdout.strip().splitlines()[-1])


def oracle_api():
    from framework_amd.api import bind
    from oracle.native import OracleNative
    orc = bind(OracleNative())
    orc.native.resetEngine()
    return orc


def cpu_time(fn, reps=1):
    """Wall clock of fn() on this host (the oracle is single-threaded), best of `reps`."""
    best = None
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    return best


def cpu_note(sample):
    return {"cores": 1, "kind": "port", "sample": sample + "; oracle/mni_oracle.c (-O3 -ffp-contract=off, no -march=native), "
            "1 of %d logical cores" % (os.cpu_count() or 0)}


def bench_yardsticks(r):
    """What the device gives a kernel that only streams, measured in this run: the figures the bandwidth-bound
    rows below are to be read against, next to the datasheet's 8 TB/s."""
    MB = 1 << 20
    bufs = [r.malloc(64 * MB) for _ in range(9)]
    for b in bufs:
        r.fill(b, 1.0, 16 * MB)
    out = {"empty_launch_us": r.yardstick_timed("empty", 0, iters=500) * 1e3}

    def line(ms, nbytes):
        return {"us": ms * 1e3, "GB/s": nbytes / ms / 1e6, "frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBPS}
    n = 64 * MB
    out["hbm_read_yardstick_warm"] = dict(line(r.yardstick_timed("read", n, srcs=bufs[:1], iters=200), n),
                                          note="the same 64 MiB every launch: served by the 256 MiB Infinity Cache")
    out["hbm_read_yardstick_cold"] = dict(line(r.yardstick_timed("read", n, srcs=bufs[:8], iters=200), n),
                                          note="eight 64 MiB buffers in rotation (512 MiB working set): served by HBM")
    out["hbm_write_yardstick_32MiB"] = line(r.yardstick_timed("write", 32 * MB, dst=bufs[8], iters=200), 32 * MB)
    out["hbm_copy_yardstick_64MiB"] = line(r.yardstick_timed("copy", n, dst=bufs[8], srcs=bufs[:1], iters=100), 2 * n)
    for b in bufs:
        r.free(b)
    # What the matrix pipe gives a loop of nothing but fp32 MFMAs (two wavefronts per SIMD, as the tile kernel has),
    # and with one or two register moves behind every MFMA: the vector ALU's issue time comes out of the MFMAs'.
    r.mfma_yardstick(0, warmup=20, iters=1)  # ~40 ms of nothing but MFMAs first: the clocks take that long to settle
    tf = [r.mfma_yardstick(v, warmup=3, iters=10) for v in (0, 1, 2)]
    out["mfma_yardstick"] = {"TFLOP/s": tf[0], "frac_mfma": tf[0] / PEAK_FP32_MATRIX_TFLOPS,
                             "with_1_v_mov_per_mfma": tf[1], "with_2_v_mov_per_mfma": tf[2],
                             "note": "v_mfma_f32_32x32x2_f32 on four independent accumulators per wavefront, nothing else in the loop"}
    return out


def bench_extras(r, with_cpu):
    out = bench_yardsticks(r)
    # ---- config 5a: decode-shaped GEMV x[4,4096] W[4096,4096], HBM-bound --------------------------------------
    x = synth.normal(4, (4, 4096), 0.02)
    w = synth.normal(4, (4096, 4096), 0.02, stream=1)
    dx, dw, dy = r.to_device(x), r.to_device(w), r.malloc(4 * 4096 * 4)
    by = 4.0 * (4096 * 4096 + 2 * 4 * 4096)
    fl = 2.0 * 4 * 4096 * 4096
    kern = "gemv_units_kernel<4, false, true>"
    # launches of a few microseconds are issued from C (mni_rocm_sgemm_timed) so that the host stays ahead
    ms_warm = r.sgemm_timed([r.gemm_desc(4, 4096, 4096, dx, dw, dy)], 10, 200)
    ms_sus = r.sgemm_timed([r.gemm_desc(4, 4096, 4096, dx, dw, dy)], 3000, 1000)
    ws = [r.to_device(w) for _ in range(8)]
    ms_cold = r.sgemm_timed([r.gemm_desc(4, 4096, 4096, dx, p, dy) for p in ws], 16, 200)
    r.sgemm(4, 4096, 4096, dx, dw, dy)
    got = r.to_host(dy, (4, 4096))
    c5a = {"roofline": dict(roofline("hbm", kern, ms_cold * 1e-3, fl, by, traffic=profile_traffic("gemv_units_4x4096x4096.txt")),
                            note="cold: eight different W in rotation (512 MiB working set), every byte comes from HBM"),
           "warm": dict(roofline("hbm", kern, ms_warm * 1e-3, fl, by),
                        note="the same W (64 MiB) every launch: it stays in the 256 MiB Infinity Cache, so this is not an HBM figure"),
           "warm_sustained": dict(roofline("hbm", kern, ms_sus * 1e-3, fl, by), note="the same after 3000 launches (~40 ms) of it"),
           "vs_read_yardstick": {"cold": out["hbm_read_yardstick_cold"]["us"] / (ms_cold * 1e3),
                                 "warm": out["hbm_read_yardstick_warm"]["us"] / (ms_warm * 1e3),
                                 "note": "time of a pure read of the same 64 MiB / time of the product"}}
    if with_cpu:
        orc = oracle_api()
        X, W = orc.Tensor.fromFloat32(x, [4, 4096]), orc.Tensor.fromFloat32(w, [4096, 4096])
        res = []
        dt = cpu_time(lambda: res.append(X.matmul(W)), reps=3)
        ref = res[-1].numpy()
        c5a["max_err_vs_oracle"] = float(np.max(np.abs(got.astype(np.float64) - ref)))
        c5a["cpu_baseline"] = dict(cpu_note("the whole product, best of 3"), value=dt * 1e3, unit="ms", **{"GB/s": by / dt / 1e9})
        orc.native.resetEngine()
    out["config5a_gemv"] = c5a
    # the same W against batches of token rows (batched decoding): up to 32 rows through the decode kernel (a form per
    # row count up to 6 rows, one or two sets of 16 rows on the 16 x 16 x 4 MFMA beyond), 64 through the tile kernel;
    # W cold (eight in rotation) -- not a BASELINE config
    rows_out = {}
    for mrows in (1, 2, 8, 16, 32, 64):
        xb = r.to_device(synth.normal(5, (mrows, 4096)))
        yb = r.malloc(mrows * 4096 * 4)
        descs = [r.gemm_desc(mrows, 4096, 4096, xb, wp, yb) for wp in ws]
        r.sgemm_timed(descs, 300, 200)
        us = min(r.sgemm_timed(descs, 20, 200) for _ in range(3)) * 1e3  # (the smallest of three: one in ten single runs reads 2 us high)
        byb = 4.0 * (4096 * 4096 + 2 * mrows * 4096)
        rows_out["%d_rows" % mrows] = {"us": us, "GB/s": byb / us / 1e3, "frac_hbm": byb / us / 1e3 / PEAK_HBM_GBPS,
                                       "TFLOP/s": 2.0 * mrows * 4096 * 4096 / us / 1e6}
        r.free(xb)
        r.free(yb)
    out["decode_batch_rows_x_4096x4096_cold"] = rows_out
    # the same buffers read as W stored [out, in]: rows . W^T, the layout of dX = dY W^T under a small batch (matmul_backward's
    # first product against a weight kept [in, out]) and of a Linear whose weight is kept transposed -- not a BASELINE config
    rows_t = {}
    for mrows in (1, 4, 8, 16):
        xb = r.to_device(synth.normal(5, (mrows, 4096)))
        yb = r.malloc(mrows * 4096 * 4)
        descs = [r.gemm_desc(mrows, 4096, 4096, xb, wp, yb, b_strides=(1, 4096)) for wp in ws]
        r.sgemm_timed(descs, 100, 200)
        us = min(r.sgemm_timed(descs, 20, 200) for _ in range(3)) * 1e3
        byb = 4.0 * (4096 * 4096 + 2 * mrows * 4096)
        rows_t["%d_rows" % mrows] = {"us": us, "GB/s": byb / us / 1e3, "frac_hbm": byb / us / 1e3 / PEAK_HBM_GBPS}
        r.free(xb)
        r.free(yb)
    out["rows_x_transposed_4096x4096_weight_cold"] = rows_t
    # the decode product against larger row-major weights (the shapes of a 7B-class model's layers), 4 rows, cold (two or three
    # weights in rotation, more than the Infinity Cache holds): what the launch, the first access and the sum of the K slices cost
    # weighs less the longer the stream is -- not a BASELINE config
    big_out = {}
    for (n_, k_) in ((11008, 4096), (8192, 8192), (32000, 4096)):
        nbuf = 3 if n_ * k_ * 4 < (200 << 20) else 2
        wb = [r.malloc(n_ * k_ * 4) for _ in range(nbuf)]
        for w_ in wb:
            r.fill(w_, 0.01, n_ * k_)
        xb = r.to_device(synth.normal(5, (4, k_)))
        yb = r.malloc(4 * n_ * 4)
        descs = [r.gemm_desc(4, n_, k_, xb, w_, yb) for w_ in wb]
        r.sgemm_timed(descs, 20, 60)
        us = min(r.sgemm_timed(descs, 10, 60) for _ in range(3)) * 1e3
        byb = 4.0 * (n_ * k_ + 4 * k_ + 4 * n_)
        big_out["4x%dx%d" % (n_, k_)] = {"us": us, "GB/s": byb / us / 1e3, "frac_hbm": byb / us / 1e3 / PEAK_HBM_GBPS}
        r.free(xb)
        r.free(yb)
        for w_ in wb:
            r.free(w_)
    out["decode_gemv_larger_weights_cold"] = big_out
    # token rows against a weight stored [out, in] (a tied language-model head: logits = x E^T with E [50304, 768]), E cold
    # (four in rotation, 618 MB) -- not a BASELINE config
    head_out = {}
    vocab, dm = 50304, 768
    es = [r.malloc(vocab * dm * 4) for _ in range(4)]
    for e in es:
        r.fill(e, 0.01, vocab * dm)
    for mrows in (1, 8, 16):
        xb = r.to_device(synth.normal(7, (mrows, dm)))
        yb = r.malloc(mrows * vocab * 4)
        descs = [r.gemm_desc(mrows, vocab, dm, xb, e, yb, b_strides=(1, dm)) for e in es]
        us = r.sgemm_timed(descs, 100, 200) * 1e3
        byb = 4.0 * (vocab * dm + mrows * dm + mrows * vocab)
        head_out["%d_rows" % mrows] = {"us": us, "GB/s": byb / us / 1e3, "frac_hbm": byb / us / 1e3 / PEAK_HBM_GBPS}
        r.free(xb)
        r.free(yb)
    for e in es:
        r.free(e)
    out["rows_x_transposed_50304x768_weight_cold"] = head_out
    # the weight gradient of the same layer under a small batch: dW[4096,4096] = X^T[4096,rows] dY[rows,4096], X^T as a
    # view (matmul_backward's second product with K = the batch's rows): bound by writing dW -- not a BASELINE config
    grad_out = {}
    dwg = r.malloc(4096 * 4096 * 4)
    for mrows in (8, 32):
        xb = r.to_device(synth.normal(6, (mrows, 4096)))
        gb = r.to_device(synth.normal(7, (mrows, 4096)))
        for accumulate in (False, True):
            d = r.gemm_desc(4096, 4096, mrows, xb, gb, dwg, a_strides=(1, 4096), accumulate=accumulate)
            us = r.sgemm_timed([d], 300, 200) * 1e3
            byb = 4.0 * (4096 * 4096 * (2 if accumulate else 1) + 2 * mrows * 4096)
            grad_out["%d_rows%s" % (mrows, "_accumulating" if accumulate else "")] = {
                "us": us, "GB/s": byb / us / 1e3, "frac_hbm": byb / us / 1e3 / PEAK_HBM_GBPS, "TFLOP/s": 2.0 * mrows * 4096 * 4096 / us / 1e6}
        r.free(xb)
        r.free(gb)
    r.free(dwg)
    out["weight_gradient_4096x4096_of_a_small_batch"] = grad_out
    for p in ws + [dx, dw, dy]:
        r.free(p)
    # ---- config 5b: X^T[1024,65536] dY[65536,1024], X^T as a view, split-K -------------------------------------
    X = synth.normal(5, (65536, 1024))
    dX, dG, dO = r.to_device(X), r.to_device(X), r.malloc(1024 * 1024 * 4)
    # (30 launches of warm-up: the upload above leaves the GPU idle and its clocks take ~20 ms to settle)
    ms = time_launches(r, lambda: r.sgemm(1024, 1024, 65536, dX, dG, dO, a_strides=(1, 1024)), 30, 20)
    fl = 2.0 * 1024 * 1024 * 65536
    by = 4.0 * (2 * 65536 * 1024 + 1024 * 1024)
    c5b = {"roofline": roofline("mfma", "gemm_mfma_kernel<1, 1, 2, 2, false> + splitk_reduce_kernel", ms * 1e-3, fl, by,
                                traffic=profile_traffic("config5b_tall_k_1024x1024x65536.txt"))}
    if with_cpu:
        rows = 8192  # an eighth of K: the oracle gathers X^T into a contiguous copy, then runs its i-k-j loop
        orc = oracle_api()
        Xs = orc.Tensor.fromFloat32(X[:rows], [rows, 1024])
        dt = cpu_time(lambda: Xs.permute(1, 0).matmul(Xs))
        c5b["cpu_baseline"] = dict(cpu_note("the first %d of 65536 K rows (%.1f GFLOP), gather of the transposed view included" % (rows, 2.0 * 1024 * 1024 * rows / 1e9)),
                                   value=2.0 * 1024 * 1024 * rows / dt / 1e12, unit="TFLOP/s", seconds=dt)
        orc.native.resetEngine()
    out["config5b_tall_k"] = c5b
    for p in (dX, dG, dO):
        r.free(p)
    del X
    # ---- config 3: Q K^T (K^T a permuted view), dQ, dK^T -- batched, near the ridge -------------------------------
    q = synth.normal(2, (32, 512, 64)) / np.float32(8)
    kk = synth.normal(2, (32, 512, 64), stream=1) / np.float32(8)
    ds = synth.normal(2, (32, 512, 512), stream=2)
    dq, dk, dds = r.to_device(q), r.to_device(kk), r.to_device(ds)
    s_out, g_out = r.malloc(32 * 512 * 512 * 4), r.malloc(32 * 512 * 64 * 4)
    fl = 2.0 * 32 * 512 * 512 * 64
    by = 4.0 * 32 * (512 * 64 * 2 + 512 * 512)
    prods = [("scores", "gemm_panel_kernel<8>", r.gemm_desc(512, 512, 64, dq, dk, s_out, batch=32, a_batch=(512 * 64, 32),
                                                             b_strides=(1, 64), b_batch=(512 * 64, 32))),
             ("dQ", "gemm_mfma_kernel<0, 1, 1, 1, false>", r.gemm_desc(512, 64, 512, dds, dk, g_out, batch=32, a_batch=(512 * 512, 32),
                                                                  b_batch=(512 * 64, 32))),
             ("dKT", "gemm_mfma_kernel<1, 1, 1, 1, false>", r.gemm_desc(64, 512, 512, dq, dds, g_out, batch=32, a_strides=(1, 64),
                                                                   a_batch=(512 * 64, 32), b_batch=(512 * 512, 32)))]
    c3 = {}
    each = {}
    # 1500 untimed launches (~25 ms) first: after the host-side work above the clocks are down, and the first ~20 ms of
    # any timing run 10 % slow (the headline's settle launches and config 4's warm-up steps are there for the same reason)
    C3_WARM = 1500
    for name, kern, desc in prods:
        each[name] = r.sgemm_timed([desc], C3_WARM, 200)
        # each product moves 41.9 MB and 1.07 GFLOP: the matrix pipe needs 6.8 us for it, HBM 5.2 us
        c3[name] = roofline("mfma", kern, each[name] * 1e-3, fl, by)
    # the two gradients as the engine's matmul backward issues them: one paired launch (mni_rocm_sgemm_pair)
    g_out2 = r.malloc(32 * 512 * 64 * 4)
    pair = [prods[1][2], r.gemm_desc(64, 512, 512, dq, dds, g_out2, batch=32, a_strides=(1, 64), a_batch=(512 * 64, 32), b_batch=(512 * 512, 32))]
    ms_pair = r.sgemm_pair_timed(pair, C3_WARM, 200)
    c3["dQ_and_dKT_paired"] = dict(roofline("mfma", "gemm_mfma_pair_kernel<0, 1, 1, 1>", ms_pair * 1e-3, 2 * fl, 2 * by),
                                   note="both gradients in one launch; one after the other they take %.1f us" % ((each["dQ"] + each["dKT"]) * 1e3))
    total = each["scores"] + ms_pair
    c3["roofline"] = dict(roofline("mfma", "the three products (scores, then both gradients in one launch)", total * 1e-3, 3 * fl, 3 * by,
                                   traffic=profile_traffic("config3_attention_products_32x512x64.txt")),
                          note="arithmetic intensity 25.6 flop/B against a ridge of 19.7: the matrix pipe bounds it (20.5 us for all "
                               "three), HBM is close behind (15.7 us); an empty launch in the same sequence takes "
                               "%.2f us; three separate launches take %.1f us" % (out["empty_launch_us"], sum(each.values()) * 1e3))
    r.free(g_out2)
    if with_cpu:
        nb = 2  # batches of the 32
        orc = oracle_api()
        Q = orc.Tensor.fromFloat32(q[:nb], [nb, 512, 64]).setRequiresGrad(True)
        K = orc.Tensor.fromFloat32(kk[:nb], [nb, 512, 64]).setRequiresGrad(True)
        G = orc.Tensor.fromFloat32(ds[:nb], [nb, 512, 512])
        dt = cpu_time(lambda: Q.matmul(K.permute(0, 2, 1)).mul(G).sum().backward())
        c3["cpu_baseline"] = dict(cpu_note("%d of 32 batches: forward through the permuted view, backward to dQ and dK (incl. the oracle's "
                                           "transposes, clones and the mul/sum that seed the gradient)" % nb),
                                  value=dt * 1e3 * 32 / nb, unit="ms (scaled to 32 batches)", seconds=dt)
        orc.native.resetEngine()
    out["config3_attention_scores"] = c3
    for p in (dq, dk, dds, s_out, g_out):
        r.free(p)
    # ---- configs 1 and 4: training steps through the engine (wall clock, trailing sync) -------------------------
    from framework_amd.api import bind
    api = bind(N.Native())

    def T(a, grad=False, on=None):
        t = (on or api).Tensor.fromFloat32(a, list(a.shape))
        return t.setRequiresGrad(True) if grad else t

    def time_step(step, keep, n, warm):
        for _ in range(warm):
            step()
            api.native.gcTensors(keep())
        r.sync()
        total, launches = 0.0, 0
        for _ in range(n):
            l0 = r.launch_count()
            t0 = time.perf_counter()
            step()
            r.sync()
            total += time.perf_counter() - t0
            launches = r.launch_count() - l0
            api.native.gcTensors(keep())
        return total * 1e3 / n, launches

    def time_steps_back_to_back(step, keep, n):
        """n steps issued one after the other (the bookkeeping between them included), one wait at the end."""
        r.sync()
        t0 = time.perf_counter()
        for _ in range(n):
            step()
            api.native.gcTensors(keep())
        r.sync()
        return (time.perf_counter() - t0) * 1e3 / n

    # config 4: FFN step X[4096,1024] -> 4096 (GELU) -> 1024, reference mseLoss, fwd + bwd
    d, h, rows = 1024, 4096, 4096
    x4, t4 = synth.normal(3, (rows, d)), synth.normal(3, (rows, d), stream=3)
    w1, w2 = synth.uniform(3, (d, h), -1 / 32, 1 / 32, stream=1), synth.uniform(3, (h, d), -1 / 64, 1 / 64, stream=2)
    gemm_flops = 6 * 2.0 * rows * d * h
    gemm_bytes = 4.0 * (2 * (rows * d + d * h + rows * h) + (rows * h + h * d + rows * d) + (rows * h + rows * d + h * d)
                        + (rows * d + d * h + rows * h) + (rows * d + rows * h + d * h))  # operands + result of the six products
    for fused in (False, True):
        api.native.resetEngine()
        x = T(x4, True)
        tg = T(t4)
        l1 = api.Linear(d, h, weight=w1, bias=np.zeros(h, np.float32), fused=fused, activation="gelu")
        l2 = api.Linear(h, d, weight=w2, bias=np.zeros(d, np.float32), fused=fused)
        params = l1.parameters() + l2.parameters()

        def step4():
            api.native.zeroGrad([x._id] + [p.value._id for p in params])
            api.mseLoss(l2.forward(l1.forward(x)), tg, fused=fused).backward()

        def keep4():
            ids = [x._id, tg._id] + [p.value._id for p in params]
            for t in [x] + [p.value for p in params]:
                g = api.native.getGrad(t._id)
                if g is not None:
                    ids.append(g)
            return ids
        ms, launches = time_step(step4, keep4, 20, 15)  # 30 ms of warm-up: the clocks take tens of milliseconds to settle after an idle spell
        ms_loop = time_steps_back_to_back(step4, keep4, 15)
        out["config4_ffn_step" + ("_fused_linear" if fused else "")] = {
            "ms": ms, "launches_per_step": launches, "ms_in_a_loop_without_waits": ms_loop,
            "roofline": dict(roofline("mfma", "whole step (six gemm_mfma_kernel launches + elementwise)", ms * 1e-3, gemm_flops, gemm_bytes,
                                      traffic=profile_traffic("config4_ffn_step.txt") if fused else None),
                             note="flops and bytes of the six products only; the step's elementwise kernels add ~0.7 GB of traffic and no counted flops")}
    if with_cpu:
        rs = 256  # rows of the 4096
        orc = oracle_api()
        xo = T(x4[:rs], True, orc)
        to = T(t4[:rs], False, orc)
        o1 = orc.Linear(d, h, weight=w1, bias=np.zeros(h, np.float32))
        o2 = orc.Linear(h, d, weight=w2, bias=np.zeros(d, np.float32))
        dt = cpu_time(lambda: orc.mseLoss(o2.forward(o1.forward(xo).gelu()), to).backward())
        out["config4_ffn_step"]["cpu_baseline"] = dict(cpu_note("the first %d of 4096 rows of X (%.1f GFLOP of the 206.2), forward + backward" % (rs, gemm_flops * rs / rows / 1e9)),
                                                       value=gemm_flops * rs / rows / dt / 1e12, unit="TFLOP/s", seconds=dt,
                                                       ms_scaled_to_4096_rows=dt * 1e3 * rows / rs)
        orc.native.resetEngine()
    # config 1: README MLP step (32x10 -> 64 -> 3, cross-entropy, Adam): launch-latency bound
    api.native.resetEngine()
    c1 = dict(x=synth.uniform(0, (32, 10)), w1=synth.uniform(0, (10, 64), -0.316, 0.316, stream=1), b1=synth.uniform(0, (64,), -0.316, 0.316, stream=2),
              w2=synth.uniform(0, (64, 3), -0.125, 0.125, stream=3), b2=synth.uniform(0, (3,), -0.125, 0.125, stream=4))
    targets = [[int(t)] for t in synth.integers(0, (32,), 0, 3, stream=5)]

    def build1(a, fused=False):
        x1 = T(c1["x"], False, a)
        m1 = a.Linear(10, 64, weight=c1["w1"], bias=c1["b1"], fused=fused, activation="relu")
        m2 = a.Linear(64, 3, weight=c1["w2"], bias=c1["b2"], fused=fused)
        ps = m1.parameters() + m2.parameters()
        opt = a.Adam(ps, lr=1e-3)

        def step():
            opt.zeroGrad()
            a.crossEntropyLoss(m2.forward(m1.forward(x1)), targets).backward()
            opt.step()

        def keep():
            ids = [x1._id] + [p.value._id for p in ps]
            return ids + [g for g in (a.native.getGrad(p.value._id) for p in ps) if g is not None]
        return step, keep
    for fused in (False, True):
        api.native.resetEngine()
        step1, keep1 = build1(api, fused)
        ms, launches = time_step(step1, keep1, 200, 20)
        # the same steps without a wait after each: what a training loop that does not read the loss sees
        r.sync()
        t0 = time.perf_counter()
        for _ in range(200):
            step1()
            api.native.gcTensors(keep1())
        r.sync()
        ms_loop = (time.perf_counter() - t0) / 200 * 1e3
        out["config1_readme_mlp_step" + ("_fused_linear" if fused else "")] = {
            "ms": ms, "ms_per_step_in_a_loop_of_200": ms_loop, "launches_per_step": launches,
            "roofline": {"bound": "launch latency", "kernel": "%d kernel launches per step" % launches,
                         "us_per_launch": ms * 1e3 / max(launches, 1), "empty_launch_us": out["empty_launch_us"],
                         "algorithmic_flops": 0.16e6, "frac": None,
                         "note": "0.16 MFLOP and < 0.1 MB per step: neither roof applies; the step is the sum of its launch "
                                 "latencies and of the host's own work per op.  ms: each step followed by a wait for the device"}}
    api.native.resetEngine()
    # the same step driven from plain C over the engine ABI (no language binding in the loop)
    for fused in (False, True):
        out["config1_readme_mlp_step" + ("_fused_linear" if fused else "")]["c_loop"] = c_loop_step(fused)
    if with_cpu:
        orc = oracle_api()
        so, ko = build1(orc)
        for _ in range(3):
            so()
            orc.native.gcTensors(ko())
        t0 = time.perf_counter()
        for _ in range(50):
            so()
            orc.native.gcTensors(ko())
        out["config1_readme_mlp_step"]["cpu_baseline"] = dict(cpu_note("the whole step, mean of 50 (through the same Python binding)"),
                                                              value=(time.perf_counter() - t0) / 50 * 1e3, unit="ms")
        orc.native.resetEngine()
    # ---- "next" rows: attention on the batched GEMM shapes, KV-cache decode ---------------------------------------
    api.native.resetEngine()
    bh, s, d = 32, 512, 64
    qa, ka, va = (T(synth.normal(2, (bh, s, d), stream=i) / np.float32(8 if i < 2 else 1), True) for i in range(3))
    wa = T(synth.normal(2, (bh, s, d), stream=3))

    def keep_att():
        ids = [t._id for t in (qa, ka, va, wa)]
        return ids + [g for g in (api.native.getGrad(t._id) for t in (qa, ka, va)) if g is not None]
    ms_fwd, _ = time_step(lambda: api.flashAttention(qa, ka, va, 0.125, True), keep_att, 20, 5)

    def att_step():
        api.native.zeroGrad([qa._id, ka._id, va._id])
        api.flashAttention(qa, ka, va, 0.125, True).mul(wa).sum().backward()
    ms_all, _ = time_step(att_step, keep_att, 20, 5)
    # the one-kernel forward on long sequences ([8, 8192, 64] and [16, 4096, 128], causal): useful flops = half of dense
    for lb, ls, ld in ((8, 8192, 64), (16, 4096, 128)):
        ql, kl, vl = (T(synth.normal(2, (lb, ls, ld), stream=i)) for i in range(3))
        keep_long = lambda: [ql._id, kl._id, vl._id] + keep_att()
        ms_long, _ = time_step(lambda: api.flashAttention(ql, kl, vl, 1.0 / math.sqrt(ld), True), keep_long, 10, 3)
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
        out["kv_decode_8x32x128_hist4096_" + ("int8" if quantized else "fp32")] = {"us": us, "GB/s": by / us / 1e3, "frac_hbm": by / us / 1e3 / PEAK_HBM_GBPS}
        cache.free()
        api.native.gcTensors([])
    api.native.resetEngine()
    return out


def split_extras(out):
    """(other, extra): `extra` holds the configurations BASELINE names, in short form; `other` everything else."""
    ex = {}
    c1f, c1 = out.pop("config1_readme_mlp_step_fused_linear"), out.pop("config1_readme_mlp_step")
    cf, cc = c1f.get("c_loop") or {}, c1.get("c_loop") or {}
    ms1 = cf.get("ms_per_step_with_a_wait_after_each", c1f["ms"])
    ex["config1"] = sig({
        "ms": ms1, "measured": "plain-C loop over the engine ABI, fused Linear, a wait for the device after every step" if cf.get("steps") else "ctypes binding",
        "launches_per_step": cf.get("launches_per_step", c1f["launches_per_step"]), "ms_in_a_loop_without_waits": cf.get("ms_per_step_in_a_loop"),
        "composed_matmul_then_add": {"ms": cc.get("ms_per_step_with_a_wait_after_each"), "launches_per_step": cc.get("launches_per_step", c1["launches_per_step"])},
        "through_the_ctypes_binding": {"fused_ms": c1f["ms"], "composed_ms": c1["ms"]},
        "bound": "launch latency", "us_per_launch": ms1 * 1e3 / max(cf.get("launches_per_step", c1f["launches_per_step"]), 1),
        "empty_launch_us": out["empty_launch_us"], "frac": None, "traffic": None})
    if "cpu_baseline" in c1:
        ex["config1"]["cpu_baseline"] = brief_cpu(c1["cpu_baseline"])
    c3 = out.pop("config3_attention_scores")
    ex["config3"] = brief(c3["roofline"], scores_us=c3["scores"]["us"], dQ_us=c3["dQ"]["us"], dKT_us=c3["dKT"]["us"],
                          gradients_in_one_launch_us=c3["dQ_and_dKT_paired"]["us"], GBps=c3["roofline"]["GB/s"])
    if "cpu_baseline" in c3:
        ex["config3"]["cpu_baseline"] = brief_cpu(c3["cpu_baseline"])
    c4f, c4 = out.pop("config4_ffn_step_fused_linear"), out.pop("config4_ffn_step")
    ex["config4"] = brief(c4f["roofline"], ms=c4f["ms"], launches_per_step=c4f["launches_per_step"], kernel="whole step, fused Linear + GELU epilogues: six products + elementwise",
                          ms_in_a_loop_without_waits=c4f["ms_in_a_loop_without_waits"],
                          composed=sig({"ms": c4["ms"], "frac": c4["roofline"]["frac"], "launches_per_step": c4["launches_per_step"]}))
    if "cpu_baseline" in c4:
        ex["config4"]["cpu_baseline"] = brief_cpu(c4["cpu_baseline"])
    c5a = out.pop("config5a_gemv")
    ex["config5a"] = brief(c5a["roofline"], weights="cold: eight W in rotation, every byte from HBM", warm_us=c5a["warm"]["us"], warm_frac=c5a["warm"]["frac"],
                           read_yardstick_cold_us=out["hbm_read_yardstick_cold"]["us"], vs_read_yardstick_cold=c5a["vs_read_yardstick"]["cold"])
    if "max_err_vs_oracle" in c5a:
        ex["config5a"]["max_err_vs_oracle"] = sig(c5a["max_err_vs_oracle"])
    if "cpu_baseline" in c5a:
        ex["config5a"]["cpu_baseline"] = brief_cpu(c5a["cpu_baseline"])
    c5b = out.pop("config5b_tall_k")
    ex["config5b"] = brief(c5b["roofline"])
    if "cpu_baseline" in c5b:
        ex["config5b"]["cpu_baseline"] = brief_cpu(c5b["cpu_baseline"])
    return sig(out), ex


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
    elif which == "config3":
        # the three attention-shaped batched products of configuration 3 (scores through the panel kernel, dQ and
        # dK^T through the tile kernel's 64 x 64 tiles), 5 launches each, then the two gradients as one paired launch
        q, ds = synth.normal(2, (32, 512, 64)) / np.float32(8), synth.normal(2, (32, 512, 512), stream=2)
        dq, dk, dds = r.to_device(q), r.to_device(q), r.to_device(ds)
        g_out = r.malloc(32 * 512 * 64 * 4)
        for _ in range(5):
            r.sgemm(512, 512, 64, dq, dk, dst, batch=32, a_batch=(512 * 64, 32), b_strides=(1, 64), b_batch=(512 * 64, 32))
        for _ in range(5):
            r.sgemm(512, 64, 512, dds, dk, g_out, batch=32, a_batch=(512 * 512, 32), b_batch=(512 * 64, 32))
        for _ in range(5):
            r.sgemm(64, 512, 512, dq, dds, g_out, batch=32, a_strides=(1, 64), a_batch=(512 * 64, 32), b_batch=(512 * 512, 32))
        g_out2 = r.malloc(32 * 512 * 64 * 4)
        for _ in range(5):
            r.sgemm_pair(r.gemm_desc(512, 64, 512, dds, dk, g_out, batch=32, a_batch=(512 * 512, 32), b_batch=(512 * 64, 32)),
                         r.gemm_desc(64, 512, 512, dq, dds, g_out2, batch=32, a_strides=(1, 64), a_batch=(512 * 64, 32), b_batch=(512 * 512, 32)))
    elif which == "config5b":
        # the tall-K weight gradient X^T[1024, 65536] dY[65536, 1024] (X^T a view): K slices and their reduction pass
        X = r.to_device(synth.normal(5, (65536, 1024)))
        G = r.to_device(synth.normal(5, (65536, 1024), stream=1))
        for _ in range(5):
            r.sgemm(1024, 1024, 65536, X, G, dst, a_strides=(1, 1024))
    elif which == "config4":
        # 24 FFN training steps with the fused Linear and the fused loss (forward + backward through the engine)
        from framework_amd.api import bind
        api = bind(N.Native())
        d, h, rows = 1024, 4096, 4096
        T = lambda a, g=False: (api.Tensor.fromFloat32(a, list(a.shape)).setRequiresGrad(True) if g else api.Tensor.fromFloat32(a, list(a.shape)))
        x, tg = T(synth.normal(3, (rows, d)), True), T(synth.normal(3, (rows, d), stream=3))
        l1 = api.Linear(d, h, weight=synth.uniform(3, (d, h), -1 / 32, 1 / 32, stream=1), bias=np.zeros(h, np.float32), fused=True, activation="gelu")
        l2 = api.Linear(h, d, weight=synth.uniform(3, (h, d), -1 / 64, 1 / 64, stream=2), bias=np.zeros(d, np.float32), fused=True)
        params = l1.parameters() + l2.parameters()
        for _ in range(24):  # (the clocks settle over the first twenty: the last steps of the trace are the ones to read)
            api.native.zeroGrad([x._id] + [p.value._id for p in params])
            api.mseLoss(l2.forward(l1.forward(x)), tg, fused=True).backward()
            keep = [x._id, tg._id] + [p.value._id for p in params]
            keep += [g for g in (api.native.getGrad(t._id) for t in [x] + [p.value for p in params]) if g is not None]
            api.native.gcTensors(keep)
    elif which == "fewrows":
        # 32 token rows against a [4096, 4096] weight (the few-rows kernel) and against an [8192, 8192] one, 5 launches each
        x = r.to_device(synth.normal(4, (32, 8192), 0.02))
        w = r.to_device(synth.normal(4, (8192, 8192), 0.02, stream=1))
        for _ in range(5):
            r.sgemm(32, 4096, 4096, x, w, dst)
        for _ in range(5):
            r.sgemm(32, 8192, 8192, x, w, dst)
    elif which == "decode_rows":
        # 16 and 32 token rows against a [4096, 4096] weight, eight weights in rotation (every byte of W from HBM): the
        # decode product's 16 x 16 x 4 form with one and with two sets of rows, 16 launches each
        x = r.to_device(synth.normal(4, (32, 4096), 0.02))
        ws = [r.to_device(synth.normal(4, (4096, 4096), 0.02, stream=1 + i)) for i in range(8)]
        for mrows in (16, 32):
            for i in range(16):
                r.sgemm(mrows, 4096, 4096, x, ws[i % 8], dst)
    elif which == "nt_rows":
        # 4 and 16 token rows against a [4096, 4096] weight stored [out, in] (rows . W^T: dX = dY W^T of a small batch), eight weights
        # in rotation (every byte of W from HBM): the few-rows kernel for a K-contiguous weight with K in slices, 16 launches each
        x = r.to_device(synth.normal(4, (16, 4096), 0.02))
        ws = [r.to_device(synth.normal(4, (4096, 4096), 0.02, stream=1 + i)) for i in range(8)]
        for mrows in (4, 16):
            for i in range(16):
                r.sgemm(mrows, 4096, 4096, x, ws[i % 8], dst, b_strides=(1, 4096))
        # ... and 1 and 8 rows against a [14336, 4096] weight of the same layout, two in rotation (470 MB): the unsliced form (all of K
        # per wavefront, no partial sums), 8 launches each
        for w in ws:
            r.free(w)
        wl = [r.malloc(14336 * 4096 * 4) for _ in range(2)]
        for w in wl:
            r.fill(w, 0.01, 14336 * 4096)
        for mrows in (1, 8):
            for i in range(8):
                r.sgemm(mrows, 14336, 4096, x, wl[i % 2], dst, b_strides=(1, 4096))
    elif which == "outer":
        # the weight gradient of a [4096, 4096] layer under 8 rows (the outer-product kernel), overwriting and
        # accumulating, 5 launches each
        x, gy = r.to_device(synth.normal(6, (8, 4096))), r.to_device(synth.normal(7, (8, 4096)))
        for accumulate in (False, True):
            for _ in range(5):
                r.sgemm(4096, 4096, 8, x, gy, dst, a_strides=(1, 4096), accumulate=accumulate)
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


# ---- the planner held against forced plans -----------------------------------------------------------------------------
# (M, N, K, batch, A given as its transpose, B given as its transpose): the configurations, the products of batched
# decoding, small and transformer-sized Linear layers with their backward products, weight gradients of small batches,
# batches of small products, edges off a multiple of four.
PLANNER_SHAPES = [
    (4096, 4096, 4096, 1, 0, 0), (4096, 4096, 1024, 1, 0, 0), (4096, 4096, 1024, 1, 0, 1), (4096, 1024, 4096, 1, 1, 0), (1024, 4096, 4096, 1, 1, 0),
    (1024, 1024, 65536, 1, 1, 0), (512, 512, 64, 32, 0, 1), (512, 64, 512, 32, 0, 0), (64, 512, 512, 32, 1, 0),
    (1, 4096, 4096, 1, 0, 0), (4, 4096, 4096, 1, 0, 0), (8, 4096, 4096, 1, 0, 0), (16, 4096, 4096, 1, 0, 0), (32, 4096, 4096, 1, 0, 0),
    (64, 4096, 4096, 1, 0, 0), (128, 4096, 4096, 1, 0, 0), (192, 4096, 4096, 1, 0, 0), (4, 8192, 8192, 1, 0, 0), (4, 4096, 16384, 1, 0, 0),
    (4, 16384, 4096, 1, 0, 0), (8, 50304, 768, 1, 0, 0), (12, 8192, 8192, 1, 0, 0), (16, 50304, 768, 1, 0, 1), (1, 50304, 768, 1, 0, 1),
    (24, 11008, 4096, 1, 0, 0), (64, 4096, 11008, 1, 0, 0), (8, 50304, 768, 1, 0, 1), (16, 32000, 1024, 1, 0, 1), (32, 64, 10, 1, 0, 0), (32, 3, 64, 1, 0, 0), (64, 512, 512, 1, 0, 0),
    (256, 512, 512, 1, 0, 0), (16384, 16, 16, 1, 0, 0), (784, 128, 64, 1, 1, 0), (4096, 768, 3072, 1, 0, 0), (4096, 3072, 768, 1, 0, 0),
    (4096, 2304, 768, 1, 0, 0), (2048, 2048, 2048, 1, 0, 0), (3000, 3000, 3000, 1, 0, 0), (1001, 1003, 999, 1, 0, 0), (2048, 2050, 2048, 1, 0, 0),
    (4096, 4096, 8, 1, 1, 0), (4096, 4096, 32, 1, 1, 0), (4096, 11008, 64, 1, 1, 0), (768, 3072, 256, 1, 1, 0), (4096, 11008, 64, 1, 0, 0),
    (8192, 8192, 128, 1, 0, 0), (2048, 8192, 32, 1, 0, 0), (64, 64, 64, 2048, 1, 0), (16, 64, 16, 8192, 0, 0), (4, 4, 4, 65536, 0, 0),
    (1, 512, 64, 1024, 0, 1), (128, 128, 512, 32, 0, 0), (1024, 64, 1024, 16, 0, 0), (65536, 2, 768, 1, 0, 0), (4096, 10, 4096, 1, 0, 0),
    (512, 512, 4096, 1, 0, 0), (768, 768, 4096, 1, 1, 0), (6144, 1024, 2048, 1, 0, 0), (8192, 8192, 8192, 1, 0, 0),
]


def planner_plans():
    P = [("mfma128", N.ALGO_MFMA, 1), ("mfma128_s2", N.ALGO_MFMA, 2), ("mfma128_s4", N.ALGO_MFMA, 4), ("mfma128_s8", N.ALGO_MFMA, 8),
         ("mfma64", N.ALGO_MFMA_SMALL, 1), ("mfma64_s2", N.ALGO_MFMA_SMALL, 2), ("mfma64_s4", N.ALGO_MFMA_SMALL, 4), ("mfma64_s8", N.ALGO_MFMA_SMALL, 8),
         ("mfma64_s16", N.ALGO_MFMA_SMALL, 16), ("streamk", N.ALGO_MFMA_STREAMK, 0), ("skinny", N.ALGO_SKINNY, 0), ("skinny_two_pass", N.ALGO_SKINNY_TWO_PASS, 0),
         ("direct", N.ALGO_DIRECT, 0), ("direct_s4", N.ALGO_DIRECT, 4), ("panel", N.ALGO_PANEL, 0), ("tiny", N.ALGO_TINY, 0), ("fewrows", N.ALGO_FEWROWS, 0),
         ("outer", N.ALGO_OUTER, 0), ("gemv", N.ALGO_GEMV, 0), ("fewrows_nt", N.ALGO_FEWROWS_NT, 0)]
    return {name: (algo, split) for name, algo, split in P}


def planner_time(r, shape, bufs, algo, split, iters):
    M, Nn, K, batch, ta, tb = shape
    dA, dB, dC = bufs
    desc = r.gemm_desc(M, Nn, K, dA, dB, dC, batch=batch, a_strides=(1, M) if ta else (K, 1), b_strides=(1, K) if tb else (Nn, 1),
                       a_batch=(M * K, batch), b_batch=(K * Nn, batch), algo=algo, split_k=split)
    try:
        return r.sgemm_timed([desc], max(5, iters // 4), iters) * 1e3
    except N.MniError:
        return None  # the plan does not take this shape or layout


def planner_bufs(r, shape):
    """Operands of normally distributed values (the matrix pipe's power, and with it the clock, depends on the bits that
    toggle: a product of constants runs faster than the same product of real data, and ranks the tile shapes differently;
    4096 x 4096 x 1024 takes 242 us on constants with 64 x 64 or 128 x 128 tiles alike, 262 and 248 on normal values)."""
    M, Nn, K, batch, _, _ = shape
    sizes = (M * K * batch, K * Nn * batch, M * Nn * batch)
    rng = np.random.default_rng(M * 7 + Nn * 3 + K)
    bufs = []
    for i, n in enumerate(sizes):
        if i < 2:
            host = rng.standard_normal(max(n, 1), dtype=np.float32) * np.float32(1.0 if i == 0 else 1.0 / 32)
            bufs.append(r.to_device(host))
        else:
            bufs.append(r.malloc(max(n, 1) * 4))
    return bufs


def planner_iters(shape):
    M, Nn, K, batch, _, _ = shape
    return 40 if 2.0 * M * Nn * K * batch > 2e10 else 200


def planner_sweep(r, path):
    """Every forced plan on every shape of PLANNER_SHAPES: writes the best plan and its time per shape (the data
    --planner-check holds the planner against)."""
    plans = planner_plans()
    rows = []
    for shape in PLANNER_SHAPES:
        bufs = planner_bufs(r, shape)
        it = planner_iters(shape)
        planner_time(r, shape, bufs, N.ALGO_AUTO, 0, it)  # (clocks)
        heavy = 2.0 * shape[0] * shape[1] * shape[2] * shape[3] > 2e10  # no thread-per-output kernels on the large products
        times = {name: planner_time(r, shape, bufs, algo, split, it) for name, (algo, split) in plans.items()
                 if not (heavy and name in ("direct", "direct_s4", "tiny", "outer"))}
        times = {k: round(v, 2) for k, v in times.items() if v is not None}
        auto = min(planner_time(r, shape, bufs, N.ALGO_AUTO, 0, it) for _ in range(3))  # (a figure of a few microseconds moves with the clocks)
        best = min(times, key=times.get)
        rows.append({"M": shape[0], "N": shape[1], "K": shape[2], "batch": shape[3], "a_transposed": shape[4], "b_transposed": shape[5],
                     "auto_us": round(auto, 2), "best_plan": best, "best_us": times[best], "plans_us": times})
        print("%-40s auto %9.2f  best %-16s %9.2f" % (str(shape), auto, best, times[best]), file=sys.stderr, flush=True)
        for p in bufs:
            r.free(p)
    with open(path, "w") as f:
        json.dump({"device": r.device_info()["name"].strip(), "unit": "us per launch, mni_rocm_sgemm_timed (HIP events, launches back to back)",
                   "shapes": rows}, f, indent=1)


def planner_check(r, path):
    """Re-times every shape of the recorded sweep under MNI_ALGO_AUTO and under its recorded best plan, one right
    after the other, and reports the shapes where the planner's choice is more than 10 % behind."""
    plans = planner_plans()
    data = json.load(open(path))
    behind, lines = [], []
    for row in data["shapes"]:
        shape = (row["M"], row["N"], row["K"], row["batch"], row["a_transposed"], row["b_transposed"])
        bufs = planner_bufs(r, shape)
        it = planner_iters(shape)
        algo, split = plans[row["best_plan"]]
        planner_time(r, shape, bufs, N.ALGO_AUTO, 0, it)
        best, auto = float("inf"), float("inf")
        for _ in range(3):  # in turns, the smallest of three each: a figure of a few microseconds moves with the clocks
            best = min(best, planner_time(r, shape, bufs, algo, split, it))
            auto = min(auto, planner_time(r, shape, bufs, N.ALGO_AUTO, 0, it))
        for p in bufs:
            r.free(p)
        rec = {"shape": list(shape), "auto_us": round(auto, 2), "best_plan": row["best_plan"], "best_us": round(best, 2),
               "recorded_best_us": row["best_us"], "auto_over_best": round(auto / best, 3)}
        lines.append(rec)
        if auto > 1.10 * best:
            behind.append(rec)
        print("%-40s auto %9.2f  %-16s %9.2f  x%.3f%s" % (str(shape), auto, row["best_plan"], best, auto / best, "   <-- behind" if auto > 1.10 * best else ""),
              file=sys.stderr, flush=True)
    ratios = [l["auto_over_best"] for l in lines]
    print(json.dumps({"planner_check": {"shapes": len(lines), "more_than_10_percent_behind": behind, "worst_ratio": max(ratios),
                                        "mean_ratio": round(sum(ratios) / len(ratios), 4)}, "rows": lines}))


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
    ap.add_argument("--counters", choices=["gemm", "gemv", "streamk", "config3", "config4", "config5b", "fewrows", "decode_rows", "nt_rows", "outer", "attention", "attention_bwd"], default=None,
                    help="for rocprofv3 --pmc runs: launch a copy kernel of known size (64 MiB read + 64 MiB "
                         "written) 3 times, then the chosen product 5 times, and exit")
    ap.add_argument("--planner-sweep", metavar="JSON", default=None, help="time every forced plan on the planner's shape list and write the best per shape")
    ap.add_argument("--planner-check", action="store_true", help="hold MNI_ALGO_AUTO against the recorded best plan of tests/golden/planner_sweep.json")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (got --gpus %d)" % args.gpus)

    r = N.Rocm()
    r.init(0)
    info = r.device_info()
    if args.counters:
        run_for_counters(r, args.counters)
        return
    if args.planner_sweep:
        planner_sweep(r, args.planner_sweep)
        return
    if args.planner_check:
        planner_check(r, os.path.join(ROOT, "tests", "golden", "planner_sweep.json"))
        return
    wall_ms, kernel_ms, flops, (a, b), err = bench_headline(r, args.steps, args.warmup)
    value = flops / wall_ms / 1e9
    achieved = flops / kernel_ms / 1e9
    line = {
        "metric": "fp32 matmul TFLOP/s", "value": value, "unit": "TFLOP/s",
        "pct_of_fp32_matrix_peak": 100.0 * value / PEAK_FP32_MATRIX_TFLOPS,
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_launches": SETTLE_LAUNCHES, "ms_per_step": wall_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "single fp32 matmul A[4096,4096] x B[4096,4096], A,B ~ N(0,1) seed 1, row-major, forward only",
                   "M": 4096, "N": 4096, "K": 4096, "device": info["name"].strip(), "compute_units": info["compute_units"],
                   "max_err_vs_f64_sample": err},
        "roofline": {"bound": "mfma", "kernel": "gemm_mfma_kernel<0, 1, 2, 2, false>", "achieved": achieved,
                     "peak": PEAK_FP32_MATRIX_TFLOPS, "unit": "TFLOP/s", "frac": achieved / PEAK_FP32_MATRIX_TFLOPS,
                     "kernel_ms": kernel_ms, "algorithmic_flops": flops, "traffic": profile_traffic("gemm_mfma_4096_pmc.txt")},
    }
    extra = None
    if not args.no_extras:
        line["other"], extra = split_extras(bench_extras(r, not args.no_cpu))
    # the headline's own objects and the BASELINE configurations close the line
    line["roofline"] = line.pop("roofline")
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(a, b, args.cpu_sample_seconds)
    if extra is not None:
        line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
