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


def cpu_baseline(a_rows, bt, bias, seconds_hint=15.0):
    """Times the oracle (the reference's host loop restated in C, one thread as in the reference) on
    a bounded sample of rows of the same 8192^3 product."""
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
    return {
        "value": flops / dt * 1e-12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
        "sample": "%d of %d rows of the same 8192^3 GEMM+bias+ReLU, %.1f s, oracle/kai_oracle.c "
                  "(gcc -O2 -ffp-contract=off), extrapolates to %.0f s for the full product" % (
                      rows, n, dt, dt * n / rows),
    }, y, rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
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
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for _ in range(args.steps):
        step()
    ev1.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kernel_ms = ev0.elapsed_time(ev1) / args.steps
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

    def gemv_time(cold, iters=120):
        for i in range(nbuf):
            fn(*argsets[i if cold else 0])
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(iters):
            fn(*argsets[i % nbuf if cold else 0])
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters

    cold_ms = gemv_time(True)
    warm_ms = gemv_time(False)
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
                     "kernel": "gemm_mfma_kernel", "kernel_ms": kernel_ms, "flops_per_launch": flops},
        "gemv": {"workload": "batch-1 y = x . W^T, W[4096,4096] fp32 (BASELINE configs[4], M=1), kai_matmul",
                 "value": gemv_gbs, "unit": "GB/s", "us_per_call_cold": cold_ms * 1e3,
                 "us_per_call_warm": warm_ms * 1e3, "warm_gbs": gemv_bytes / (warm_ms * 1e-3) * 1e-9,
                 "rel_fro_err_vs_f64": gemv_err,
                 "roofline": {"bound": "hbm", "achieved": gemv_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                              "frac": gemv_gbs / PEAK_HBM_GBS, "traffic": hbm_traffic_from_profile("gemv_rows_kernel_4096x4096_batch1.md"),
                              "kernel": "gemv_rows_kernel", "bytes_per_launch": gemv_bytes}},
    }

    if not args.no_cpu_baseline:
        a_rows = a[:768].cpu().numpy()
        bt = np.ascontiguousarray(b.cpu().numpy().T)
        base, y_cpu, nrows = cpu_baseline(a_rows, bt, bias.cpu().numpy())
        base["host_cores_available"] = os.cpu_count()
        got = c[:nrows].cpu().numpy()
        base["gpu_vs_oracle_rel_fro"] = float(np.linalg.norm((got - y_cpu).astype(np.float64)) /
                                              np.linalg.norm(y_cpu.astype(np.float64)))
        out["cpu_baseline"] = base
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
