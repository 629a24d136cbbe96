#!/usr/bin/env python3
"""Benchmark of the int8 FullyConnected_q forward at M=N=K=4096 on one MI355X.

A step is one lten_hip_quantized_matmul call (the whole FC forward: MFMA GEMM with the
zero-point correction and the requantize fused in) over one synthetic batch whose operands
are already resident in HBM.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from __graft_entry__ import load_package  # noqa: E402

INT8_MFMA_PEAK_TOPS = 5000.0   # MI355X dense int8 MFMA, published: 5.0 POP/s
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published: 8 TB/s

# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs,
# scaled by the same counters on a plain copy kernel; None until such a run is on file under profiles/.
TRAFFIC_BYTES = {"qgemm_nt_256x256x64": None}


def cpu_baseline(X, W, sc, zp, budget_s=15.0):
    """l-ten's own quantized_matmul (compiled reference) or, where that library is absent, the C port,
    on the first rows of the same workload, single thread as in l-ten."""
    from oracle import bindings as ob
    ref = ob.ref()
    N, K = W.shape

    def run(rows):
        A = np.ascontiguousarray(X[:rows])
        t0 = time.perf_counter()
        if ref is not None:
            ob.ref_quantized_matmul(A, W, sc, zp)
        else:
            ob.quantized_matmul(A, W, sc, zp, want_acc=False)
        return time.perf_counter() - t0

    probe_rows = 16
    t_probe = run(probe_rows)
    rows = int(min(X.shape[0], max(probe_rows, budget_s / max(t_probe, 1e-6) * probe_rows)))
    rows = max(16, rows // 16 * 16)
    t = run(rows)
    tops = 2.0 * rows * N * K / t / 1e12
    return {"value": tops, "unit": "TOPS", "cores": 1, "kind": "reference" if ref is not None else "port",
            "sample": f"first {rows} of {X.shape[0]} activation rows against the full {N}x{K} weight matrix "
                      f"({t:.1f} s single-threaded quantized_matmul)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-verify", action="store_true", help="skip the post-run output check")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (the path has no collective to scale); use --gpus 1")

    lt = load_package()
    from light_tensor_amd import workloads as wl
    lt.init(0)

    M = N = K = 4096
    X, W, sc, zp = wl.cfg3()
    dA, dB = lt.DeviceBuffer.from_numpy(X), lt.DeviceBuffer.from_numpy(W)
    dC = lt.DeviceBuffer(M * N)
    ws = lt.DeviceBuffer(4 * (M + N))
    qp = lt.qparams3(sc, zp)

    def step():
        lt.quantized_matmul(False, True, M, N, K, dA, dB, dC, qp, None, ws)

    for _ in range(args.warmup):
        step()
    lt.sync()
    timer = lt.Timer()
    t0 = time.perf_counter()
    timer.start()
    for _ in range(args.steps):
        step()
    kernel_ms = timer.stop_ms() / args.steps   # HIP events on the stream the kernel runs on
    lt.sync()
    wall = time.perf_counter() - t0
    kernel = lt.last_kernel()

    ops = 2.0 * M * N * K
    ms_per_step = wall / args.steps * 1e3
    value = ops / (ms_per_step * 1e-3) / 1e12
    achieved = ops / (kernel_ms * 1e-3) / 1e12

    verified = None
    if not args.no_verify:
        acc = ((X.astype(np.float64) - float(zp[0])) @ (W.astype(np.float64) - float(zp[1])).T)
        mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
        s = (acc.astype(np.float32) * mult).astype(np.float32) + np.float32(zp[2])
        want = (np.trunc(s).astype(np.int64) & 0xFF).astype(np.uint8)
        verified = bool(np.array_equal(dC.numpy(np.uint8, (M, N)), want))

    out = {
        "metric": "int8_fc_forward_tops_4096",
        "value": round(value, 2),
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "cfg3 int8 FullyConnected_q forward M=N=K=4096: uint8 activations (zero point 128) x "
                               "8-bit weights (N(0,40) clipped, zero point 128) -> int32 -> fused requantize to uint8",
                   "M": M, "N": N, "K": K, "input_digest": wl.digest(X, W)},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": INT8_MFMA_PEAK_TOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / INT8_MFMA_PEAK_TOPS, 4), "traffic": TRAFFIC_BYTES.get(kernel),
                     "kernel": kernel, "kernel_us": round(kernel_ms * 1e3, 2),
                     "note": "int8 multiply-add counted as 2 ops; achieved/peak in tera-ops per second"},
        "verified_bit_exact": verified,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(X, W, sc, zp)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
