#!/usr/bin/env python3
"""Benchmark of the matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one launch of the fused GEMM + bias + ReLU at M = N = K = 8192 (fp32, row-major
A[M,K] . B[K,N], inputs resident in HBM).  Prints one JSON line: `value` is the GEMM rate in
TFLOP/s over the K timed steps; `roofline` prices the same kernel against the fp32 MFMA peak;
`gemv` carries the second half of the headline metric, the batch-1 4096 x 4096 product in GB/s
against the HBM peak (cold: rotating over weight buffers larger than the 256 MB last-level
cache); `cpu_baseline` is the CPU restatement of the reference's host loop timed on this box.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def hbm_traffic_from_profile(summary_name):
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE and WRITE_SIZE, scaled by what the
    same counters read for a plain copy of known size), as recorded in the kernel's summary under
    profiles/; None if no summary holds the figure."""
    import re
    try:
        with open(os.path.join(ROOT, "profiles", summary_name)) as f:
            m = re.search(r"HBM_TRAFFIC_BYTES_PER_LAUNCH\s*=\s*([0-9.eE+]+)", f.read())
        return float(m.group(1)) if m else None
    except OSError:
        return None


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def usable_cores():
    """Host threads this process may use: its CPU affinity, capped by OMP_NUM_THREADS where the box sets it."""
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    cap = os.environ.get("OMP_NUM_THREADS", "")
    if cap.isdigit() and int(cap) > 0:
        n = min(n, int(cap))
    return max(1, n)


def cpu_baseline(a_rows, bt, bias, seconds_hint=10.0):
    """Times the oracle (the reference's host loop restated in C) on a bounded sample of rows of the same
    8192^3 product: on ONE thread, as the reference's host path runs (`value`), and with the rows spread
    over all usable cores (`all_cores`; every output element is still summed sequentially, so the results are
    bit-identical to the single-thread run, which is checked)."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as ko
    n = bt.shape[0]
    k = bt.shape[1]
    t0 = time.perf_counter()
    ko.matmul(bt, a_rows[:4])
    per_row = (time.perf_counter() - t0) / 4
    rows = int(max(8, min(a_rows.shape[0], seconds_hint / max(per_row, 1e-9))))
    t0 = time.perf_counter()
    y = ko.matmul(bt, a_rows[:rows])
    y = ko.activate(ko.add_bias(y, bias), "relu")
    dt = time.perf_counter() - t0
    flops = 2.0 * rows * n * k
    threads = usable_cores()
    prow = int(min(a_rows.shape[0], max(threads, rows * min(threads, 8))))
    t0 = time.perf_counter()
    yp = ko.matmul_parallel(bt, a_rows[:prow], threads)
    yp = ko.activate(ko.add_bias(yp, bias), "relu")
    dtp = time.perf_counter() - t0
    return {
        "value": flops / dt * 1e-12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
        "sample": "%d of %d rows of the same 8192^3 GEMM+bias+ReLU, %.1f s, oracle/kai_oracle.c "
                  "(gcc -O2 -ffp-contract=off), extrapolates to %.0f s for the full product" % (
                      rows, n, dt, dt * n / rows),
        "all_cores": {"value": 2.0 * prow * n * k / dtp * 1e-12, "unit": "TFLOP/s", "cores": threads,
                      "sample": "%d rows spread over %d threads, %.1f s, extrapolates to %.0f s" % (
                          prow, threads, dtp, dtp * n / prow),
                      "bit_identical_to_one_thread": bool(np.array_equal(yp[:rows], y))},
        "nproc": os.cpu_count(), "cpu_model": cpu_model(),
    }, y, rows


def per_config_table(torch, kai, stream, dev, with_cpu, warm_ms=40.0, only=None):
    """The other BASELINE configurations (they are parity cases; reported here for completeness): GPU time
    per call from HIP events over back-to-back launches (after about 40 ms of the same call untimed; the median
    of three runs of `iters` launches), achieved rate, and the oracle's single-thread time."""
    import ctypes
    L = kai.load()
    g = torch.Generator(device=dev)
    g.manual_seed(11)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    I = ctypes.c_int64
    if with_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import oracle as ko

    def gpu_us(fn, iters=50, prep=None):
        # untimed warm-up: the same call back to back for about 40 ms, so that the clocks have come up from idle
        # (in a fresh process 144 x 4096 x 4096 measures 61, 58, 55, 53 ... us over the first 20 ms and 50 from
        # then on); an in-place op works on one spare copy of its input meanwhile
        spare = prep() if prep else None
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < warm_ms * 1e-3:
            for _ in range(20):
                if prep:
                    fn(spare)
                else:
                    fn()
            torch.cuda.synchronize()
        del spare
        if prep is None:
            reps = []
            for _ in range(3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(iters):
                    fn()
                e1.record(stream)
                torch.cuda.synchronize()
                reps.append(e0.elapsed_time(e1) * 1e3 / iters)
            return sorted(reps)[1]
        # in-place ops: every launch works on a fresh copy of the input (prep() returns it), the launches go
        # back to back between one pair of events like every other row; the copies (iters x the operand, beyond
        # the last-level cache) are made outside the timed span
        bufs = [prep() for _ in range(iters)]
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for b in bufs:
            fn(b)
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / iters

    def cpu_us(f):
        if not with_cpu:
            return None
        t0 = time.perf_counter()
        f()
        return (time.perf_counter() - t0) * 1e6

    rows = []

    def row(name, fn, iters=50, prep=None, flops=None, nbytes=None, cpu=None):
        """One row: `fn` timed on the GPU (see gpu_us), `cpu` (a callable) the oracle's time for the same work."""
        if only and not any(o in name for o in only):
            return
        us = gpu_us(fn, iters, prep)
        cpu = cpu_us(cpu) if cpu is not None else None
        r = {"case": name, "gpu_us": round(us, 2)}
        if flops:
            r["tflops"] = round(flops / us * 1e-6, 2)
            r["frac_fp32_mfma_peak"] = round(flops / us * 1e-6 / PEAK_FP32_MFMA_TFLOPS, 4)
        if nbytes:
            r["gbs"] = round(nbytes / us * 1e-3, 1)
            r["frac_hbm_peak"] = round(nbytes / us * 1e-3 / PEAK_HBM_GBS, 4)
        if cpu is not None:
            r["cpu_us_1_thread"] = round(cpu, 1)
        rows.append(r)

    relu = kai.ACT["relu"]
    # the headline product in the ENGINE's operand forms (weights stored [out, in]): forward NT with bias + ReLU in
    # one launch, the input gradient NN, the weight gradient TN
    n8 = 8192
    x8 = torch.rand((n8, n8), device=dev, generator=g) * 2 - 1
    w8 = torch.rand((n8, n8), device=dev, generator=g) * 2 - 1
    b8 = torch.randn(n8, device=dev, generator=g)
    o8 = torch.empty((n8, n8), device=dev)
    f8 = 2.0 * n8 ** 3
    row("8192^3 NT  Y = relu(X.W^T + b)  (kai_dense_forward)",
        lambda: L.kai_dense_forward(0, P(o8), None, P(w8), P(b8), P(x8), I(n8), I(n8), I(n8), relu, None), iters=10,
        flops=f8)
    row("8192^3 NT  Y = X.W^T  (kai_matmul)",
        lambda: L.kai_matmul(0, P(o8), P(w8), P(x8), I(n8), I(n8), I(n8), 0), iters=10, flops=f8)
    row("8192^3 NN  dX = dY.W  (kai_matmul_backward_x)",
        lambda: L.kai_matmul_backward_x(0, P(o8), P(x8), P(w8), I(n8), I(n8), I(n8), 0), iters=10, flops=f8)
    row("8192^3 TN  dW = dY^T.X  (kai_matmul_backward_w)",
        lambda: L.kai_matmul_backward_w(0, P(o8), P(x8), P(w8), I(n8), I(n8), I(n8), 0), iters=10, flops=f8)
    # the same launch with a transcendental activation: applied to the accumulators in registers, one store
    row("8192^3 NT  Y = gelu(X.W^T + b)  (kai_dense_forward)",
        lambda: L.kai_dense_forward(0, P(o8), None, P(w8), P(b8), P(x8), I(n8), I(n8), I(n8), kai.ACT["gelu"], None), iters=10,
        flops=f8)
    del x8, w8, b8, o8
    # a product whose operands and output (1.5 GiB) exceed the 256 MB last-level cache: the HBM-side traffic of the
    # 256 x 256 tiling is priced against HBM here (the summary under profiles/ holds the counters)
    mb, nb, kb_ = 16384, 16384, 4096
    xb = torch.rand((mb, kb_), device=dev, generator=g) * 2 - 1
    wb = torch.rand((nb, kb_), device=dev, generator=g) * 2 - 1
    bb = torch.randn(nb, device=dev, generator=g)
    ob = torch.empty((mb, nb), device=dev)
    row("16384 x 16384 x 4096 NT  Y = relu(X.W^T + b), operands and output beyond the last-level cache (kai_dense_forward)",
        lambda: L.kai_dense_forward(0, P(ob), None, P(wb), P(bb), P(xb), I(nb), I(mb), I(kb_), relu, None), iters=5,
        flops=2.0 * mb * nb * kb_)
    del xb, wb, bb, ob
    # cfg1: dense forward 64 x 784 -> 512, fused
    x = torch.randn((64, 784), device=dev, generator=g)
    w = (torch.rand((512, 784), device=dev, generator=g) * 2 - 1) / 28.0
    b = torch.zeros(512, device=dev)
    y = torch.empty((64, 512), device=dev)
    us = lambda: L.kai_dense_forward(0, P(y), None, P(w), P(b), P(x), I(512), I(64), I(784), relu, None)
    xc, wc, bc = x.cpu().numpy(), w.cpu().numpy(), b.cpu().numpy()
    row("cfg1 dense fwd 64x784->512 +bias+relu (1 launch)", us, flops=2.0 * 64 * 784 * 512,
        cpu=lambda: ko.activate(ko.add_bias(ko.matmul(wc, xc), bc), "relu"))
    # cfg2: batch 256, 1024 -> 1024
    x = torch.randn((256, 1024), device=dev, generator=g)
    w = (torch.rand((1024, 1024), device=dev, generator=g) * 2 - 1) / 32.0
    b = torch.randn(1024, device=dev, generator=g)
    gy = torch.randn((256, 1024), device=dev, generator=g) * 0.01
    y, gx, gw, gb = (torch.empty_like(x), torch.empty_like(x), torch.empty_like(w), torch.empty_like(b))
    f = 2.0 * 256 * 1024 * 1024
    xc, wc, bc, gyc = x.cpu().numpy(), w.cpu().numpy(), b.cpu().numpy(), gy.cpu().numpy()
    row("cfg2 Y = X.W^T + b (fused)", lambda: L.kai_dense_forward(0, P(y), None, P(w), P(b), P(x), I(1024), I(256), I(1024), 0, None),
        flops=f, cpu=lambda: ko.add_bias(ko.matmul(wc, xc), bc))
    alpha = torch.tensor([0.1], device=dev)
    for name in ("relu", "leaky", "sigmoid", "tanh", "gelu", "selu", "mish", "swish"):
        row("cfg2 Y = %s(X.W^T + b) (fused)" % name,
            lambda: L.kai_dense_forward(0, P(y), None, P(w), P(b), P(x), I(1024), I(256), I(1024), kai.ACT[name], P(alpha)),
            flops=f)
    row("cfg2 dX = dY.W", lambda: L.kai_matmul_backward_x(0, P(gx), P(gy), P(w), I(1024), I(256), I(1024), 0),
        flops=f, cpu=lambda: ko.matmul_backward_x(gyc, wc))
    row("cfg2 dW = dY^T.X", lambda: L.kai_matmul_backward_w(0, P(gw), P(gy), P(x), I(1024), I(256), I(1024), 0),
        flops=f, cpu=lambda: ko.matmul_backward_w(gyc, xc, 1024, 1024))
    row("cfg2 db = colsum(dY)", lambda: L.kai_add_bias_backward_b(0, P(gb), P(gy), I(256), I(1024), 0),
        nbytes=4.0 * 256 * 1024, cpu=lambda: ko.add_bias_backward_b(gyc, 1024))
    pre = torch.randn((256, 1024), device=dev, generator=g)
    work = torch.empty_like(pre)
    row("cfg2 dense backward with ReLU: dX, dW, db from dY and the pre-activation (kai_dense_backward)",
        lambda: L.kai_dense_backward(0, P(gx), P(gw), P(gb), P(work), P(gy), P(w), P(x), P(pre), I(1024), I(256),
                                            I(1024), relu, None, 0),
        flops=2 * f)
    # cfg4: attention, both mappings of 32 batch x heads, seq 512, head dim 64
    for nbat, nhead, nvec in ((32, 1, 64), (4, 8, 512)):
        T, D = 512, 64
        q, k, v = (torch.randn((nbat, T, nvec), device=dev, generator=g) for _ in range(3))
        s0 = torch.empty((nbat, T, T, nhead), device=dev)
        pbuf = torch.empty_like(s0)
        o = torch.empty((nbat, T, nvec), device=dev)
        coef = torch.tensor([0.125], device=dev)
        tag = "cfg4 nbat=%d nhead=%d " % (nbat, nhead)
        fl = 2.0 * 32 * T * T * D
        qc, kc, vc = q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy()
        row(tag + "S = Q.K^T/8 (mult_on_heads)",
            lambda: L.kai_mult_on_heads(0, P(s0), P(k), P(q), I(nbat), I(T), I(nvec), I(nhead), I(D), P(coef)),
            flops=fl, cpu=lambda: ko.mult_on_heads(kc, qc, nhead, 0.125))
        row(tag + "softmax_direct_on_axis (in place)",
            lambda b: L.kai_softmax_direct_on_axis(0, P(b), I(nbat * T), I(T), I(nhead)), iters=20,
                   prep=lambda: s0.clone(),
            nbytes=8.0 * 32 * T * T, cpu=lambda: ko.softmax_direct_on_axis(s0.cpu().numpy(), nbat * T, T, nhead))
        pbuf.copy_(s0)
        L.kai_softmax_direct_on_axis(0, P(pbuf), I(nbat * T), I(T), I(nhead))
        row(tag + "O = P.V (mix_values)",
            lambda: L.kai_mix_values(0, P(o), P(pbuf), P(v), I(nbat), I(T), I(nvec), I(nhead), I(D)),
            flops=fl, cpu=lambda: ko.mix_values(pbuf.cpu().numpy(), vc, nhead))
        def three_calls():
            L.kai_mult_on_heads(0, P(pbuf), P(k), P(q), I(nbat), I(T), I(nvec), I(nhead), I(D), P(coef))
            L.kai_softmax_direct_on_axis(0, P(pbuf), I(nbat * T), I(T), I(nhead))
            L.kai_mix_values(0, P(o), P(pbuf), P(v), I(nbat), I(T), I(nvec), I(nhead), I(D))

        row(tag + "the three calls back to back", three_calls, flops=2 * fl)
        row(tag + "all three fused, forward only (kai_attention_forward)",
            lambda: L.kai_attention_forward(0, P(o), P(q), P(k), P(v), I(nbat), I(T), I(nvec), I(nhead), I(D),
                                                   P(coef), 0),
            flops=2 * fl)
        row(tag + "all three in one launch, probabilities stored (kai_attention_forward_train)",
            lambda: L.kai_attention_forward_train(0, P(o), P(pbuf), P(q), P(k), P(v), I(nbat), I(T), I(nvec), I(nhead), I(D),
                                                  P(coef), 0),
            flops=2 * fl)
        # the backward calls of the same block (vtensor.cpp:3142-3166 of the reference)
        go = torch.randn((nbat, T, nvec), device=dev, generator=g)
        gp = torch.empty_like(s0)
        gv = torch.empty_like(v)
        gq = torch.empty_like(q)
        goc = go.cpu().numpy() if with_cpu else None
        row(tag + "gP = gO.V^T (mix_values_backward_prop)",
            lambda: L.kai_mix_values_backward_prop(0, P(gp), P(go), P(v), I(nbat), I(T), I(nvec), I(nhead), I(D)),
            flops=fl, cpu=lambda: ko.mix_values_backward_prop(goc, vc, nhead))
        row(tag + "gV = P^T.gO (mix_values_backward_value)",
            lambda: L.kai_mix_values_backward_value(0, P(gv), P(go), P(pbuf), I(nbat), I(T), I(nvec), I(nhead), I(D)),
            flops=fl, cpu=lambda: ko.mix_values_backward_value(goc, pbuf.cpu().numpy(), nhead))
        gp0 = gp.clone()
        row(tag + "softmax_direct_on_axis_backward (in place)",
            lambda b: L.kai_softmax_direct_on_axis_backward(0, P(b), P(pbuf), I(nbat), I(T), I(nhead), P(coef)),
                   iters=20, prep=lambda: gp0.clone(),
            nbytes=12.0 * 32 * T * T,
            cpu=lambda: ko.softmax_direct_on_axis_backward(gp0.cpu().numpy(), pbuf.cpu().numpy(), 0.125))
        row(tag + "gQ = gS.K (mult_on_heads_backward)",
            lambda: L.kai_mult_on_heads_backward(0, P(gq), P(gp), P(k), I(nbat), I(T), I(nvec), I(nhead), I(D)),
            flops=fl, cpu=lambda: ko.mult_on_heads_backward(gp.cpu().numpy(), kc, nhead))
        # the same backward middle (vtensor.cpp:3145-3154) as the reference's five calls back to back, and as one call
        mo = torch.empty_like(o)
        L.kai_mix_values(0, P(mo), P(pbuf), P(v), I(nbat), I(T), I(nvec), I(nhead), I(D))
        gk = torch.empty_like(q)

        def five_calls():
            L.kai_mix_values_backward_prop(0, P(gp), P(go), P(v), I(nbat), I(T), I(nvec), I(nhead), I(D))
            L.kai_mix_values_backward_value(0, P(gv), P(go), P(pbuf), I(nbat), I(T), I(nvec), I(nhead), I(D))
            L.kai_softmax_direct_on_axis_backward(0, P(gp), P(pbuf), I(nbat), I(T), I(nhead), P(coef))
            L.kai_mult_on_heads_backward(0, P(gk), P(gp), P(q), I(nbat), I(T), I(nvec), I(nhead), I(D))
            L.kai_mult_on_heads_backward(0, P(gq), P(gp), P(k), I(nbat), I(T), I(nvec), I(nhead), I(D))

        row(tag + "backward: the five calls back to back", five_calls, flops=4 * fl)
        row(tag + "backward: gQ, gK, gV in one call (kai_attention_backward: %s)"
            % kai.VMath.attention_plan("backward", nbat, T, nvec, nhead, D),
            lambda: L.kai_attention_backward(0, P(gq), P(gk), P(gv), P(go), P(pbuf), P(mo), P(q), P(k), P(v), I(nbat), I(T),
                                             I(nvec), I(nhead), I(D), P(coef), 0),
            flops=4 * fl)
        row(tag + "backward: the same without the mixed output (row sums in a first pass)",
            lambda: L.kai_attention_backward(0, P(gq), P(gk), P(gv), P(go), P(pbuf), None, P(q), P(k), P(v), I(nbat), I(T),
                                             I(nvec), I(nhead), I(D), P(coef), 0),
            flops=5 * fl)
    # a BERT-base sized block: 2 x 384 tokens, 12 heads of 64 (the head count is no power of two)
    nbat, T, nhead, D = 2, 384, 12, 64
    nvec = nhead * D
    q, k, v, go = (torch.randn((nbat, T, nvec), device=dev, generator=g) for _ in range(4))
    pbuf = torch.empty((nbat, T, T, nhead), device=dev)
    o, gq, gk, gv = (torch.empty_like(q) for _ in range(4))
    coef = torch.tensor([0.125], device=dev)
    fl = 2.0 * nbat * nhead * T * T * D
    tag = "attention 2 x 384 x 12 heads of 64: "

    def three_calls_12():
        L.kai_mult_on_heads(0, P(pbuf), P(k), P(q), I(nbat), I(T), I(nvec), I(nhead), I(D), P(coef))
        L.kai_softmax_direct_on_axis(0, P(pbuf), I(nbat * T), I(T), I(nhead))
        L.kai_mix_values(0, P(o), P(pbuf), P(v), I(nbat), I(T), I(nvec), I(nhead), I(D))

    row(tag + "the three forward calls back to back", three_calls_12, flops=2 * fl)
    row(tag + "forward only, one launch (kai_attention_forward, %s)" % kai.VMath.attention_plan("forward", nbat, T, nvec, nhead, D),
        lambda: L.kai_attention_forward(0, P(o), P(q), P(k), P(v), I(nbat), I(T), I(nvec), I(nhead), I(D), P(coef), 0),
        flops=2 * fl)
    row(tag + "forward with the probabilities stored (kai_attention_forward_train, %s)" % kai.VMath.attention_plan("forward_train", nbat, T, nvec, nhead, D),
        lambda: L.kai_attention_forward_train(0, P(o), P(pbuf), P(q), P(k), P(v), I(nbat), I(T), I(nvec), I(nhead), I(D),
                                              P(coef), 0),
        flops=2 * fl)
    row(tag + "backward (kai_attention_backward, %s)" % kai.VMath.attention_plan("backward", nbat, T, nvec, nhead, D),
        lambda: L.kai_attention_backward(0, P(gq), P(gk), P(gv), P(go), P(pbuf), P(o), P(q), P(k), P(v), I(nbat), I(T),
                                         I(nvec), I(nhead), I(D), P(coef), 0),
        flops=4 * fl)
    del q, k, v, go, pbuf, o, gq, gk, gv
    # cfg5: skinny (cold: six rotating weight buffers) and ragged
    K = N = 4096
    ws = [torch.rand((N, K), device=dev, generator=g) * 0.1 - 0.05 for _ in range(6)]
    for m in (1, 4, 16):
        x = torch.randn((m, K), device=dev, generator=g)
        y = torch.empty((m, N), device=dev)
        it = [0]

        def call():
            it[0] += 1
            L.kai_matmul(0, P(y), P(ws[it[0] % 6]), P(x), I(N), I(m), I(K), 0)

        wc = ws[0].cpu().numpy() if with_cpu else None
        xc = x.cpu().numpy()
        row("cfg5 M=%d x 4096 x 4096 (cold)" % m, call, iters=120, flops=2.0 * m * N * K,
            nbytes=4.0 * (K * N + m * K + m * N), cpu=lambda: ko.matmul(wc, xc))
    del ws
    m, k, n = 1000, 777, 333
    x = torch.randn((m, k), device=dev, generator=g)
    w = torch.rand((n, k), device=dev, generator=g) * 0.1 - 0.05
    y = torch.empty((m, n), device=dev)
    xc, wc = x.cpu().numpy(), w.cpu().numpy()
    row("cfg5 ragged 1000x777x333", lambda: L.kai_matmul(0, P(y), P(w), P(x), I(n), I(m), I(k), 0),
        flops=2.0 * m * n * k, cpu=lambda: ko.matmul(wc, xc))
    # batches of a per-shard size against a wide weight matrix (kai_matmul, the matrix warm in the caches)
    for m, n, k in ((32, 4096, 4096), (64, 4096, 4096), (96, 4096, 4096), (144, 4096, 4096), (256, 2048, 2048),
                    (16, 11008, 4096), (32, 11008, 4096), (48, 11008, 4096), (48, 8192, 4096), (96, 4096, 11008), (144, 5120, 4096),
                    (200, 6656, 4096)):
        x = torch.randn((m, k), device=dev, generator=g)
        w = torch.rand((n, k), device=dev, generator=g) * 0.1 - 0.05
        y = torch.empty((m, n), device=dev)
        row("batch of %d rows: Y = X.W^T, W %d x %d (%s)" % (m, n, k, kai.VMath.gemm_plan(0, 1, m, n, k)),
            lambda: L.kai_matmul(0, P(y), P(w), P(x), I(n), I(m), I(k), 0), flops=2.0 * m * n * k)
    # shapes off the configurations' grid that the sweep over row counts (--rows-sweep) brought rules for: W from HBM
    # (rotating buffers beyond the last-level cache)
    for m, n, k in ((1, 4096, 11008), (4, 3072, 4096), (16, 4352, 4096), (24, 4096, 2048), (1, 50257, 768)):
        nb = max(2, min(24, (520 << 20) // (n * k * 4)))
        ws2 = [torch.rand((n, k), device=dev, generator=g) * 0.1 - 0.05 for _ in range(nb)]
        x = torch.randn((m, k), device=dev, generator=g)
        y = torch.empty((m, n), device=dev)
        cnt = [0]

        def call_cold(ws2=ws2, x=x, y=y, m=m, n=n, k=k, nb=nb, cnt=cnt):
            cnt[0] += 1
            L.kai_matmul(0, P(y), P(ws2[cnt[0] % nb]), P(x), I(n), I(m), I(k), 0)

        row("%d row%s: Y = X.W^T, W %d x %d from HBM (%s)" % (m, "" if m == 1 else "s", n, k, kai.VMath.gemm_plan(0, 1, m, n, k)),
            call_cold, iters=48, flops=2.0 * m * n * k, nbytes=4.0 * (k * n + m * k + m * n))
        del ws2
    # the score softmax for a head count outside the four-heads layout, short sequences (one row of the scores per wave)
    sp = torch.randn((64, 128, 128, 12), device=dev, generator=g)
    row("softmax_direct_on_axis [64,128,128,12] (in place)", lambda: L.kai_softmax_direct_on_axis(0, P(sp), I(64 * 128), I(128), I(12)),
        nbytes=2.0 * sp.numel() * 4)
    del sp
    # a dense layer's whole backward at a training batch (the bias gradient on a kernel of its own from here on)
    yv_, nd2_, xv_ = 4096, 512, 1024
    gy_ = torch.randn((nd2_, yv_), device=dev, generator=g) * 0.01
    x_ = torch.randn((nd2_, xv_), device=dev, generator=g)
    w_ = torch.rand((yv_, xv_), device=dev, generator=g) * 0.1 - 0.05
    pre_ = torch.randn((nd2_, yv_), device=dev, generator=g)
    gx_, gw_, gb_ = torch.empty((nd2_, xv_), device=dev), torch.empty((yv_, xv_), device=dev), torch.empty((yv_,), device=dev)
    row("dense backward with ReLU, 512 x (1024 -> 4096): dX, dW, db in one call (kai_dense_backward)",
        lambda: L.kai_dense_backward(0, P(gx_), P(gw_), P(gb_), None, P(gy_), P(w_), P(x_), P(pre_), I(yv_), I(nd2_), I(xv_), 1, None, 0),
        iters=20, flops=4.0 * yv_ * nd2_ * xv_)
    # one LSTM layer forward as the engine's loop issues it (vtensor.cpp:2455-2492): 32 steps of 64 x 256 -> 4 x 256
    nt_, nd_, ni_, nr_ = 32, 64, 256, 256
    xs = torch.randn((nt_, nd_, ni_), device=dev, generator=g)
    wi = torch.randn((4 * nr_, ni_), device=dev, generator=g) / 32
    wr = torch.randn((4 * nr_, nr_), device=dev, generator=g) / 32
    bi = torch.zeros(4 * nr_, device=dev)
    aff = torch.zeros((nt_, nd_, 4 * nr_), device=dev)
    rec = torch.zeros((nt_, nd_, nr_), device=dev)
    sta = torch.zeros((nt_, nd_, nr_), device=dev)

    def lstm_layer(batched, fused=False):
        L.kai_set_zero(0, P(aff), I(aff.numel() * 4))
        if batched:
            L.kai_matmul(0, P(aff), P(wi), P(xs), I(4 * nr_), I(nt_ * nd_), I(ni_), 0)
        for t in range(nt_ if fused else 0):
            L.kai_lstm_step(0, P(rec[t]), P(sta[t]), P(sta[t - 1]) if t > 0 else None, P(aff[t]), P(wr),
                            P(rec[t - 1]) if t > 0 else None, P(bi), None, I(nd_), I(nr_))
        for t in range(0 if fused else nt_):
            if t > 0:
                L.kai_matmul(0, P(aff[t]), P(wr), P(rec[t - 1]), I(4 * nr_), I(nd_), I(nr_), int(batched))
            if not batched:
                L.kai_matmul(0, P(aff[t]), P(wi), P(xs[t]), I(4 * nr_), I(nd_), I(ni_), 1)
            L.kai_add_bias(0, P(aff[t]), P(aff[t]), P(bi), I(nd_), I(4 * nr_))
            L.kai_lstm_process(0, P(rec[t]), P(sta[t]), P(sta[t - 1]) if t > 0 else None, P(aff[t]), I(nd_), I(nr_), I(ni_))

    lstm_flops = 2.0 * nt_ * nd_ * 4 * nr_ * (ni_ + nr_)
    row("lstm layer forward, 32 steps x (64 x 256 -> 4 x 256), per-step calls", lambda: lstm_layer(False), iters=10,
        flops=lstm_flops)
    row("lstm layer forward, same, input products of all steps in one call", lambda: lstm_layer(True), iters=10,
        flops=lstm_flops)
    row("lstm layer forward, same, one kai_lstm_step per step", lambda: lstm_layer(True, True), iters=10,
        flops=lstm_flops)
    # the same calls recorded once into a HIP graph and replayed (the counterpart of the engine's call replay)
    side = torch.cuda.Stream()
    for fused, name in ((False, "three calls per step"), (True, "one kai_lstm_step per step")):
        kai.set_stream(side.cuda_stream)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            lstm_layer(True, fused)
        kai.set_stream(stream.cuda_stream)
        row("lstm layer forward, %s, replayed from a HIP graph" % name, graph.replay, iters=10, flops=lstm_flops)
        del graph
    # transposes next to the path: the head split [4,512,8,64] -> [4,8,512,64] of configuration 4 and a plain 4096^2
    shape, axes = (4, 512, 8, 64), (0, 2, 1, 3)
    x = torch.randn(shape, device=dev, generator=g)
    y = torch.empty_like(x)
    # the engine's table: per output axis (source axis, output elements per step), per source axis its source step
    info = torch.tensor([[0, 512 * 8 * 64, 512 * 8 * 64], [2, 512 * 64, 8 * 64], [1, 64, 64], [3, 1, 1]],
                        dtype=torch.int32, device=dev)
    xc = x.cpu().numpy()
    row("transpose [4,512,8,64] -> [4,8,512,64]",
        lambda: L.kai_transpose(0, P(y), P(x), P(info), I(4), I(x.numel())),
        nbytes=8.0 * x.numel(), cpu=lambda: ko.transpose(xc, axes))
    # the innermost axis changes (keys to the last axis): tiles through LDS inside the general entry point
    x = torch.randn((16, 512, 12, 64), device=dev, generator=g)
    y = torch.empty_like(x)
    info = torch.tensor([[0, 12 * 64 * 512, 512 * 12 * 64], [2, 64 * 512, 12 * 64], [3, 512, 64], [1, 1, 1]],
                        dtype=torch.int32, device=dev)
    xc = x.cpu().numpy()
    row("transpose [16,512,12,64] -> [16,12,64,512]",
        lambda: L.kai_transpose(0, P(y), P(x), P(info), I(4), I(x.numel())),
        nbytes=8.0 * x.numel(), cpu=lambda: ko.transpose(xc, (0, 2, 3, 1)))
    x = torch.randn((4096, 4096), device=dev, generator=g)
    y = torch.empty_like(x)
    xc = x.cpu().numpy()
    row("transpose_bin 4096 x 4096", lambda: L.kai_transpose_bin(0, P(y), P(x), I(4096), I(4096)),
        nbytes=8.0 * x.numel(), cpu=lambda: ko.transpose_bin(xc, 4096, 4096))
    return rows


def plan_audit(torch, kai, stream, dev, out_path, shapes_text=None):
    """Times the dispatcher's choice against every alternative it could have made (forced through
    kai_gemm_force_plan) on shapes that sit on both sides of the thresholds coded in csrc/gemm_dispatch.hip, in the
    three operand forms of the dense layer, and writes a table: chosen plan, its time, the fastest alternative, the
    ratio.  A ratio above 1.08 marks a shape where the fitted rules have gone stale."""
    import ctypes
    L = kai.load()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    I = ctypes.c_int64
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    shapes = []
    for nk in ((4096, 4096), (3584, 4096), (5120, 4096), (6656, 4096), (11008, 4096)):
        for m in (128, 129, 160, 161, 192, 193, 224, 225):
            shapes.append((m,) + nk)
    for nk in ((2048, 2047), (2048, 2048), (4096, 2048)):
        for m in (64, 144, 256):
            shapes.append((m,) + nk)
    shapes += [(64, 512, 784), (256, 1024, 1024), (1000, 333, 777), (512, 2048, 2048), (1024, 1024, 1024),
               (32, 4096, 4096), (33, 4096, 4096), (96, 4096, 11008), (200, 6656, 4096), (144, 5120, 4096)]
    if shapes_text:   # "M,N,K;M,N,K;...": the caller's own shapes instead of the built-in list
        shapes = [tuple(int(v) for v in item.split(",")) for item in shapes_text.split(";") if item.strip()]
    tiles = ("large", "medium", "wide", "small", "flat")
    splits = (1, 2, 3, 4, 6, 8, 12, 16)
    forms = (("NT", 0, 1), ("NN", 0, 0), ("TN", 1, 0))

    def time_us(call, iters=20):
        for _ in range(5):
            call()
        torch.cuda.synchronize()
        reps = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(iters):
                call()
            e1.record(stream)
            torch.cuda.synchronize()
            reps.append(e0.elapsed_time(e1) * 1e3 / iters)
        return sorted(reps)[1]

    rows = []
    for m, n, k in shapes:
        for form, ta, tb in forms:
            a = torch.randn((k, m) if ta else (m, k), device=dev, generator=g)
            b = torch.randn((n, k) if tb else (k, n), device=dev, generator=g) * 0.05
            c = torch.empty((m, n), device=dev)
            lda, ldb = (m if ta else k), (k if tb else n)

            def call():
                rc = L.kai_gemm_f32(0, ta, tb, I(m), I(n), I(k), P(a), I(lda), P(b), I(ldb), P(c), I(n), None, 0, None, 0)
                if rc != 0:
                    raise RuntimeError(L.kai_last_error().decode())

            kai.VMath.gemm_force_plan(None)
            chosen = kai.VMath.gemm_plan(ta, tb, m, n, k)
            t_chosen = time_us(call)
            call()
            torch.cuda.synchronize()
            want = c.clone()
            seen = {chosen: t_chosen}
            cands = ["%s split %d" % (t, sp) for t in tiles for sp in splits] + ["wavesplit 16", "wavesplit 32"]
            for cand in cands:
                kai.VMath.gemm_force_plan(cand)
                text = kai.VMath.gemm_plan(ta, tb, m, n, k)
                if text in seen:
                    continue
                seen[text] = time_us(call)
                # a forced plan is a different order of the same sums: it must still be the same product
                call()
                torch.cuda.synchronize()
                err = float(torch.linalg.norm((c - want).double()) / torch.linalg.norm(want.double()))
                if not err <= 1e-5:
                    raise RuntimeError("forced plan %r gives another result for %s %dx%dx%d: %.2e" % (text, form, m, n, k, err))
            kai.VMath.gemm_force_plan(None)
            # the audit times every candidate twice as often as the chosen plan was timed: time the chosen one again
            seen[chosen] = min(seen[chosen], time_us(call))
            best = min(seen, key=seen.get)
            rows.append({"form": form, "M": m, "N": n, "K": k, "chosen": chosen, "chosen_us": round(seen[chosen], 2),
                         "best": best, "best_us": round(seen[best], 2), "ratio": round(seen[chosen] / seen[best], 3),
                         "candidates": len(seen)})
    rows.sort(key=lambda r: -r["ratio"])
    worst = rows[0]["ratio"]
    geo = float(np.exp(np.mean([np.log(r["ratio"]) for r in rows])))
    lines = ["| form | M x N x K | chosen plan | us | fastest alternative | us | chosen / fastest |", "|---|---|---|---|---|---|---|"]
    for r in rows:
        if r["ratio"] > 1.03 or r is rows[0]:
            lines.append("| %s | %d x %d x %d | %s | %.2f | %s | %.2f | %.3f |" % (
                r["form"], r["M"], r["N"], r["K"], r["chosen"], r["chosen_us"], r["best"], r["best_us"], r["ratio"]))
    summary = {"cases": len(rows), "worst_ratio": worst, "geomean_ratio": round(geo, 4),
               "over_1_08": sum(r["ratio"] > 1.08 for r in rows), "over_1_03": sum(r["ratio"] > 1.03 for r in rows)}
    with open(out_path, "w") as f:
        f.write(json.dumps(summary) + "\n\n" + "\n".join(lines) + "\n\n" + "\n".join(json.dumps(r) for r in rows) + "\n")
    print(json.dumps({"plan_audit": summary, "written_to": out_path}))


def stream_audit(torch, kai, stream, dev, out_path):
    """The same audit for the rules of the skinny streaming kernel (csrc/skinny_stream.hip: which row counts and
    matrices stream, and on workgroups of how many rows of W): 9..64 rows against wide weight matrices stored [N, K],
    the matrix streamed from HBM (rotating buffers beyond the last-level cache), the chosen plan against workgroups of
    16 / 32 / 48 rows of W and against the tiled kernels with 1..8 parts of the reduction."""
    import ctypes
    L = kai.load()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    I = ctypes.c_int64
    g = torch.Generator(device=dev)
    g.manual_seed(6)
    mats = ((4096, 4096), (6144, 4096), (8192, 4096), (10240, 4096), (11008, 4096), (12288, 4096), (14336, 4096),
            (16384, 4096), (4096, 8192), (8192, 8192), (11008, 8192))
    row_counts = (12, 16, 24, 32, 48, 64)
    cands = ["stream 16", "stream 32", "stream 48"] + ["%s split %d" % (t, sp) for t in ("flat", "small", "wide") for sp in (1, 2, 3, 4, 6, 8)]
    rows = []
    for n, k in mats:
        nb = max(2, (640 << 20) // (n * k * 4))
        ws = [torch.rand((n, k), device=dev, generator=g) * 0.1 - 0.05 for _ in range(nb)]
        for m in row_counts:
            x = torch.randn((m, k), device=dev, generator=g)
            y = torch.empty((m, n), device=dev)

            def time_us(iters=30):
                for i in range(max(nb, 4)):
                    L.kai_matmul(0, P(y), P(ws[i % nb]), P(x), I(n), I(m), I(k), 0)
                torch.cuda.synchronize()
                reps = []
                for _ in range(3):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(stream)
                    for i in range(iters):
                        if L.kai_matmul(0, P(y), P(ws[i % nb]), P(x), I(n), I(m), I(k), 0) != 0:
                            raise RuntimeError(L.kai_last_error().decode())
                    e1.record(stream)
                    torch.cuda.synchronize()
                    reps.append(e0.elapsed_time(e1) * 1e3 / iters)
                return sorted(reps)[1]

            kai.VMath.gemm_force_plan(None)
            chosen = kai.VMath.gemm_plan(0, 1, m, n, k)
            seen = {chosen: time_us()}
            want = (x.double() @ ws[29 % nb].double().T)
            for cand in cands:
                kai.VMath.gemm_force_plan(cand)
                text = kai.VMath.gemm_plan(0, 1, m, n, k)
                if text in seen:
                    continue
                seen[text] = time_us()
                err = float(torch.linalg.norm(y.double() - want) / torch.linalg.norm(want))
                if not err <= 1e-5:
                    raise RuntimeError("forced plan %r gives another result for %dx%dx%d: %.2e" % (text, m, n, k, err))
            kai.VMath.gemm_force_plan(None)
            seen[chosen] = min(seen[chosen], time_us())
            best = min(seen, key=seen.get)
            rows.append({"M": m, "N": n, "K": k, "chosen": chosen, "chosen_us": round(seen[chosen], 2), "best": best,
                         "best_us": round(seen[best], 2), "ratio": round(seen[chosen] / seen[best], 3), "candidates": len(seen)})
        del ws
    geo = float(np.exp(np.mean([np.log(r["ratio"]) for r in rows])))
    summary = {"cases": len(rows), "worst_ratio": max(r["ratio"] for r in rows), "geomean_ratio": round(geo, 4),
               "over_1_08": sum(r["ratio"] > 1.08 for r in rows), "over_1_03": sum(r["ratio"] > 1.03 for r in rows)}
    lines = ["| M x N x K | chosen plan | us | fastest alternative | us | chosen / fastest |", "|---|---|---|---|---|---|"]
    for r in rows:
        lines.append("| %d x %d x %d | %s | %.2f | %s | %.2f | %.3f |" % (r["M"], r["N"], r["K"], r["chosen"], r["chosen_us"],
                                                                        r["best"], r["best_us"], r["ratio"]))
    with open(out_path, "w") as f:
        f.write(json.dumps(summary) + "\n\n" + "\n".join(lines) + "\n")
    print(json.dumps({"stream_audit": summary, "written_to": out_path}))


def rows_sweep(torch, kai, stream, dev, out_path):
    """An audit that needs no forced plan: Y = X.W^T for 1..65 rows of X against weight matrices of many widths and
    reduction lengths, W streamed from HBM (rotating buffers beyond the last-level cache).  More rows never do less
    work, so a row count that takes longer than a LARGER one at the same matrix marks a kernel or a dispatch rule
    that leaves time on the table there; the table lists every such case beyond 7 %."""
    import ctypes
    L = kai.load()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    I = ctypes.c_int64
    g = torch.Generator(device=dev)
    g.manual_seed(8)
    row_counts = (1, 2, 3, 4, 5, 8, 9, 12, 16, 17, 24, 32, 33, 48, 64, 65)
    widths = (1024, 2048, 2304, 3072, 4096, 4352, 5120, 8192, 8704, 11008)
    lengths = (1024, 2048, 3072, 4096, 5120, 8192, 11008)
    lines, flagged, worst = [], [], 1.0
    for k in lengths:
        for n in widths:
            nb = max(2, min(24, (520 << 20) // (n * k * 4)))
            ws = [torch.rand((n, k), device=dev, generator=g) * 0.1 - 0.05 for _ in range(nb)]
            ts = {}
            for m in row_counts:
                x = torch.randn((m, k), device=dev, generator=g)
                y = torch.empty((m, n), device=dev)

                def call(i):
                    rc = L.kai_matmul(0, P(y), P(ws[i % nb]), P(x), I(n), I(m), I(k), 0)
                    if rc != 0:
                        raise RuntimeError(L.kai_last_error().decode())

                for i in range(max(nb, 6)):
                    call(i)
                torch.cuda.synchronize()
                reps = []
                for _ in range(5):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(stream)
                    for i in range(48):
                        call(i)
                    e1.record(stream)
                    torch.cuda.synchronize()
                    reps.append(e0.elapsed_time(e1) * 1e3 / 48)
                ts[m] = sorted(reps)[2]
                ref = x.double() @ ws[47 % nb].double().T
                err = float(torch.linalg.norm(y.double() - ref) / torch.linalg.norm(ref))
                if not err <= 1e-5:
                    raise RuntimeError("%d x %d x %d: relative error %.2e" % (m, n, k, err))
            marks = []
            for j, m in enumerate(row_counts):
                later = min(ts[mm] for mm in row_counts[j:])
                worst = max(worst, ts[m] / later)
                if ts[m] > 1.07 * later:
                    marks.append("%d rows %.2f > %.2f" % (m, ts[m], later))
                    flagged.append((round(ts[m] / later, 3), m, n, k))
            lines.append("| %d x %d | %s | %s |" % (n, k, " ".join("%d:%.1f" % (m, ts[m]) for m in row_counts), "; ".join(marks)))
            del ws
    summary = {"matrices": len(lines), "row_counts": len(row_counts), "flagged_over_1_07": len(flagged),
               "worst_ratio": round(worst, 3)}
    with open(out_path, "w") as f:
        f.write(json.dumps(summary) + "\n\n| W (N x K) | us per call by row count | slower than a larger row count by > 7 % |\n|---|---|---|\n"
                + "\n".join(lines) + "\n")
    print(json.dumps({"rows_sweep": summary, "written_to": out_path}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--headline-only", action="store_true", help="skip the table of the other configurations")
    ap.add_argument("--plan-audit", metavar="FILE", default=None,
                    help="instead of the benchmark: time the dispatcher's choice against every forced alternative on "
                         "shapes around its thresholds and write the table to FILE")
    ap.add_argument("--plan-audit-shapes", metavar="M,N,K;...", default=None,
                    help="with --plan-audit: audit these shapes instead of the built-in list")
    ap.add_argument("--stream-audit", metavar="FILE", default=None,
                    help="instead of the benchmark: the same audit for the skinny streaming kernel's rules (9..64 rows "
                         "against wide weight matrices streamed from HBM), table written to FILE")
    ap.add_argument("--rows-sweep", metavar="FILE", default=None,
                    help="instead of the benchmark: 1..65 rows against 70 weight matrices streamed from HBM; a row count "
                         "slower than a larger one marks a kernel or dispatch rule that leaves time on the table")
    ap.add_argument("--only", action="append", default=None, metavar="TEXT",
                    help="measure only the rows of the table whose name contains TEXT (may be given several times)")
    ap.add_argument("--row-warmup-ms", type=float, default=40.0,
                    help="untimed warm-up before each row of the table (a profiler run passes a small value to keep its trace short)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path is built and measured on a single MI355X "
              "(--gpus %d is not supported)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch   # device memory and synchronisation only
    from deep_learning_framework_amd import kai
    from deep_learning_framework_amd.kai import VMath

    kai.load()
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    kai.set_device(0)
    stream = torch.cuda.current_stream()
    kai.set_stream(stream.cuda_stream)
    dev = torch.device("cuda:0")

    if args.plan_audit:
        plan_audit(torch, kai, stream, dev, args.plan_audit, args.plan_audit_shapes)
        return
    if args.stream_audit:
        stream_audit(torch, kai, stream, dev, args.stream_audit)
        return
    if args.rows_sweep:
        rows_sweep(torch, kai, stream, dev, args.rows_sweep)
        return

    n = 8192
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    a = torch.rand((n, n), device=dev, generator=g) * 2 - 1
    b = torch.rand((n, n), device=dev, generator=g) * 2 - 1
    bias = torch.randn((n,), device=dev, generator=g)
    c = torch.empty((n, n), device=dev)
    relu = kai.ACT["relu"]

    def step():
        VMath.gemm_f32(0, 0, 0, n, n, n, a.data_ptr(), n, b.data_ptr(), n, c.data_ptr(), n, bias.data_ptr(), relu,
                       None, False)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # events between the steps as well: the average over the timed region prices the roofline, the per-step
    # durations give the median
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    evs[0].record(stream)
    for i in range(args.steps):
        step()
        evs[i + 1].record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kernel_ms = evs[0].elapsed_time(evs[-1]) / args.steps
    step_ms = sorted(evs[i].elapsed_time(evs[i + 1]) for i in range(args.steps))
    kernel_ms_median = step_ms[len(step_ms) // 2] if len(step_ms) % 2 else 0.5 * (step_ms[len(step_ms) // 2 - 1] + step_ms[len(step_ms) // 2])
    flops = 2.0 * n * n * n
    tflops = flops / (wall_ms * 1e-3) * 1e-12
    achieved = flops / (kernel_ms * 1e-3) * 1e-12

    # parity spot check on the timed output: a row sample against float64
    rows = torch.tensor([0, 1234, 4095, 8191], device=dev)
    ref = torch.relu(a[rows].double() @ b.double() + bias.double())
    err = float(torch.linalg.norm(c[rows].double() - ref) / torch.linalg.norm(ref))

    # one plain 256 MiB device-to-device copy: the yardstick the FETCH_SIZE / WRITE_SIZE counters of a
    # profiling run are scaled by (its true traffic is 256 MiB read + 256 MiB written)
    calib = torch.empty_like(a)
    VMath.copy_data(0, 0, calib.data_ptr(), a.data_ptr(), n * n * 4)
    torch.cuda.synchronize()
    del calib

    # ---- batch-1 GEMV, engine layout W[N,K]: y = x . W^T -------------------------------------------
    kk = nn = 4096
    nbuf = 6   # 6 x 64 MiB > 256 MB last-level cache
    ws = [torch.rand((nn, kk), device=dev, generator=g) * 0.1 - 0.05 for _ in range(nbuf)]
    x = torch.randn((1, kk), device=dev, generator=g)
    y = torch.empty((1, nn), device=dev)
    gemv_bytes = 4.0 * (kk * nn + kk + nn)

    # raw ctypes calls with pre-built arguments: the Python wrapper costs more than the kernel runs
    import ctypes
    fn = kai.load().kai_matmul
    argsets = [(0, ctypes.c_void_p(y.data_ptr()), ctypes.c_void_p(w.data_ptr()), ctypes.c_void_p(x.data_ptr()),
                ctypes.c_int64(nn), ctypes.c_int64(1), ctypes.c_int64(kk), 0) for w in ws]

    def gemv_time(cold, iters=120, repeats=7, warm_launches=60):
        """Median (and the extremes) over `repeats` measurements of `iters` back-to-back launches each."""
        for i in range(warm_launches):
            fn(*argsets[i % nbuf if cold else 0])
        torch.cuda.synchronize()
        times = []
        for _ in range(repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for i in range(iters):
                fn(*argsets[i % nbuf if cold else 0])
            e1.record(stream)
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) / iters)
        times.sort()
        return times[len(times) // 2], times[0], times[-1]

    cold_ms, cold_min, cold_max = gemv_time(True)
    warm_ms, warm_min, warm_max = gemv_time(False)
    gemv_ref = (x.double() @ ws[0].double().T)   # the warm pass ran last, on buffer 0
    gemv_err = float(torch.linalg.norm(y.double() - gemv_ref) / torch.linalg.norm(gemv_ref))
    gemv_gbs = gemv_bytes / (cold_ms * 1e-3) * 1e-9

    out = {
        "metric": "GEMM TFLOP/s (% fp32 MFMA peak) at 8192^3; HBM GB/s for batch-1 GEMV",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "fp32 GEMM M=N=K=8192 row-major A.B + bias + ReLU fused (BASELINE configs[2]); "
                               "A,B~U(-1,1), bias~N(0,1)", "entry_point": "kai_gemm_f32"},
        "pct_of_fp32_mfma_peak": 100.0 * tflops / PEAK_FP32_MFMA_TFLOPS,
        "rel_fro_err_vs_f64_rows": err,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_FP32_MFMA_TFLOPS, "traffic": hbm_traffic_from_profile("gemm_mfma_kernel_8192_gemm_bias_relu.md"),
                     "kernel": "gemm_mfma_kernel", "kernel_ms": kernel_ms, "kernel_ms_median": kernel_ms_median,
                     "kernel_ms_min_max": [step_ms[0], step_ms[-1]], "flops_per_launch": flops},
        "gemv": {"workload": "batch-1 y = x . W^T, W[4096,4096] fp32 (BASELINE configs[4], M=1), kai_matmul",
                 "value": gemv_gbs, "unit": "GB/s", "us_per_call_cold": cold_ms * 1e3,
                 "us_per_call_cold_min_max": [cold_min * 1e3, cold_max * 1e3],
                 "us_per_call_warm": warm_ms * 1e3, "us_per_call_warm_min_max": [warm_min * 1e3, warm_max * 1e3],
                 "warm_gbs": gemv_bytes / (warm_ms * 1e-3) * 1e-9,
                 "timing": "median of 7 measurements of 120 back-to-back launches after 60 warm-up launches; cold = six "
                           "rotating 64 MiB weight buffers (384 MiB > the 256 MB last-level cache)",
                 "rel_fro_err_vs_f64": gemv_err,
                 "roofline": {"bound": "hbm", "achieved": gemv_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                              "frac": gemv_gbs / PEAK_HBM_GBS, "traffic": hbm_traffic_from_profile("gemv_rows_kernel_4096x4096_batch1.md"),
                              "kernel": "gemv_rows_kernel", "bytes_per_launch": gemv_bytes}},
    }

    if not args.no_cpu_baseline:
        a_rows = a[:2048].cpu().numpy()
        bt = np.ascontiguousarray(b.cpu().numpy().T)
        base, y_cpu, nrows = cpu_baseline(a_rows, bt, bias.cpu().numpy())
        got = c[:nrows].cpu().numpy()
        base["gpu_vs_oracle_rel_fro"] = float(np.linalg.norm((got - y_cpu).astype(np.float64)) /
                                              np.linalg.norm(y_cpu.astype(np.float64)))
        out["cpu_baseline"] = base
    else:
        out["cpu_baseline"] = None
    if not args.headline_only:
        out["per_config"] = per_config_table(torch, kai, stream, dev, not args.no_cpu_baseline, args.row_warmup_ms, args.only)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
