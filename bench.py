#!/usr/bin/env python3
"""Benchmark of the int8 FullyConnected_q forward at M=N=K=4096 on one MI355X.

A step is one FullyConnected_q forward (lten_hip_fcq_forward_prepared: MFMA GEMM with the
zero-point correction and the requantize fused in) over one synthetic batch whose operands
are already resident in HBM; the layer's weights were converted to int8 once, when the layer
was set up, as the host-side FullyConnected_q does in to(GPU).  The same step on l-ten's raw
uint8 weight bytes (lten_hip_quantized_matmul) is timed beside it.  Prints ONE JSON line.  The headline fields describe config 3;
"configs" adds one record per other benchmark configuration (1, 2, 4, 5) and three for the Conv2d_q
forward, each with its own roofline figure and the CPU path timed beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-verify] [--no-extra] [--no-vendor] [--copy-calibration MiB]
"""
import argparse
import ctypes as C
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
FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 MFMA, published
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published: 8 TB/s

# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs scaled by the
# same counters on the plain copy kernel (--copy-calibration): FETCH_SIZE reads half the bytes
# the copy kernel is known to fetch (factor 2.0), WRITE_SIZE reads them exactly (factor 1.0).
# Source of the figures: profiles/qgemm_fast_256x256x128_w4x2_cfg3_4096.md (KiB per dispatch as rocprofv3 printed them).
TRAFFIC_KIB = {"qgemm_fast_256x256x128_w4x2_s2_wpre": {"FETCH_SIZE": 49240, "WRITE_SIZE": 16384},
               "qgemm_fast_256x256x128_w4x2_s2": {"FETCH_SIZE": 49240, "WRITE_SIZE": 16384}}


def traffic_bytes(kernel):
    t = TRAFFIC_KIB.get(kernel)
    if not t or t["FETCH_SIZE"] is None or t["WRITE_SIZE"] is None:
        return None
    return t["FETCH_SIZE"] * 1024 * 2.0 + t["WRITE_SIZE"] * 1024 * 1.0


VENDOR_SCRIPT = r"""
import json, sys, torch
n = 4096
a = torch.randint(0, 256, (n, n), device="cuda").sub(128).to(torch.int8)
w = (torch.randn(n, n, device="cuda") * 40).round().clamp(-127, 127).to(torch.int8)
b = w.t()   # the FullyConnected layout: weights [N, K], K contiguous
for _ in range(300): torch._int_mm(a, b)
torch.cuda.synchronize()
e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
e0.record()
for _ in range(300): torch._int_mm(a, b)
e1.record(); torch.cuda.synchronize()
us = e0.elapsed_time(e1) / 300 * 1e3
print(json.dumps({"us": round(us, 2), "tops": round(2 * n ** 3 / us / 1e6, 1), "torch": torch.__version__}))
"""


def vendor_int8(timeout_s=240):
    """The vendor's int8 GEMM (torch._int_mm, i.e. hipBLASLt) on the same shape and value distributions, in a
    process of its own: a calibration of what the part sustains, not part of the product.  None when torch
    cannot run here."""
    import subprocess
    try:
        r = subprocess.run([sys.executable, "-c", VENDOR_SCRIPT], capture_output=True, text=True, timeout=timeout_s)
        line = [l for l in r.stdout.splitlines() if l.startswith("{")]
        return json.loads(line[-1]) if r.returncode == 0 and line else {"error": (r.stderr or r.stdout)[-300:]}
    except Exception as e:  # noqa: BLE001
        return {"error": repr(e)[:300]}


SETTLE_S = 0.06


def telemetry(lt, fn, seconds=2.0):
    """Socket power, power cap and shader clock while `fn` is launched back to back for `seconds`: a side thread reads
    the amdgpu hwmon files (power1_input, power1_cap, in microwatts) and the current level of pp_dpm_sclk every 20 ms,
    and asks amd-smi once, a second into the run, for the socket power and the clock of each of the eight XCDs (a child
    process; it never touches this process's GPU state).  The hwmon power figure is a filtered one that takes about
    half a second to follow a load step, so the reported values are medians over the second half of the run.  Fields
    the box does not offer are None."""
    import glob
    import re
    import subprocess
    import threading
    power_f = (glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input") +
               glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average") + [None])[0]
    cap_f = (glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap") + [None])[0]
    sclk_f = (glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk") + [None])[0]
    samples, smi, stop = [], {}, threading.Event()
    t0 = time.perf_counter()

    def sampler():
        while not stop.is_set():
            rec = [time.perf_counter() - t0, None, None]
            try:
                if power_f:
                    rec[1] = int(open(power_f).read()) / 1e6
                if sclk_f:
                    cur = [ln for ln in open(sclk_f).read().splitlines() if "*" in ln]
                    m = re.search(r"(\d+)\s*[Mm][Hh]z", cur[0]) if cur else None
                    rec[2] = int(m.group(1)) if m else None
            except (OSError, ValueError):
                pass
            samples.append(rec)
            time.sleep(0.02)

    def ask_smi():
        # not under a profiler: its preloaded tool library would come up inside the child as well
        if "ROCP_TOOL_LIBRARIES" in os.environ or "rocprofiler" in os.environ.get("LD_PRELOAD", ""):
            smi["error"] = "skipped under a profiler"
            return
        time.sleep(min(1.0, seconds / 2))
        try:
            r = subprocess.run(["amd-smi", "metric", "-p", "-c", "--json"], capture_output=True, text=True, timeout=20)
            d = json.loads(r.stdout)
            g = (d["gpu_data"] if isinstance(d, dict) else d)[0]
            smi["socket_power_w"] = g["power"]["socket_power"]["value"]
            smi["xcd_clk_mhz"] = [g["clock"][k]["clk"]["value"] for k in sorted(g["clock"]) if k.startswith("gfx_")]
        except Exception as e:  # noqa: BLE001  (no tool, another format: the fields stay absent)
            smi["error"] = repr(e)[:120]

    threads = [threading.Thread(target=sampler), threading.Thread(target=ask_smi)]
    for t in threads:
        t.start()
    n = 0
    timer = lt.Timer()
    timer.start()
    while time.perf_counter() - t0 < seconds:
        for _ in range(200):
            fn()
        lt.sync()
        n += 200
    kernel_us = timer.stop_ms() / n * 1e3
    stop.set()
    for t in threads:
        t.join()

    def median_late(idx):
        v = sorted(r[idx] for r in samples if r[idx] is not None and r[0] >= seconds / 2)
        return v[len(v) // 2] if v else None
    cap = None
    try:
        cap = int(open(cap_f).read()) / 1e6 if cap_f else None
    except (OSError, ValueError):
        pass
    p = median_late(1)
    return {"power_w": None if p is None else round(p), "power_cap_w": None if cap is None else round(cap),
            "sclk_mhz": median_late(2), "sclk_max_mhz": 2400, "xcd_clk_mhz": smi.get("xcd_clk_mhz"),
            "socket_power_w_amd_smi": smi.get("socket_power_w"), "kernel_us_during": round(kernel_us, 2),
            "seconds": seconds, "launches": n}


def timed(lt, fn, iters, warmup=3):
    """Average milliseconds per call of fn over `iters` back-to-back calls (HIP events on the library's stream), in the
    steady state: after an idle spell the part needs tens of milliseconds of load before its clocks settle (the first
    launches of an MFMA-bound kernel run up to 1.5x slower), so the same call is repeated for SETTLE_S seconds first."""
    t_end = time.perf_counter() + SETTLE_S
    n = 0
    while n < warmup or time.perf_counter() < t_end:
        fn()
        n += 1
        if n % 100 == 0:
            lt.sync()
    lt.sync()
    t = lt.Timer()
    t.start()
    for _ in range(iters):
        fn()
    return t.stop_ms() / iters


def best_of(fn, reps):
    best = float("inf")
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t0)
    return best


def cpu_int8(ob, X, W, sc, zp, rows=None):
    ref = ob.ref()
    A = np.ascontiguousarray(X if rows is None else X[:rows])
    t0 = time.perf_counter()
    if ref is not None:
        ob.ref_quantized_matmul(A, W, sc, zp)
    else:
        ob.quantized_matmul(A, W, sc, zp, want_acc=False)
    return time.perf_counter() - t0, ("reference" if ref is not None else "port")


def cpu_baseline(X, W, sc, zp, budget_s=15.0):
    """l-ten's own quantized_matmul (compiled reference) or, where that library is absent, the C port,
    on the first rows of the same workload, single thread as in l-ten."""
    from oracle import bindings as ob
    N, K = W.shape
    probe_rows = 16
    t_probe, kind = cpu_int8(ob, X, W, sc, zp, probe_rows)
    rows = int(min(X.shape[0], max(probe_rows, budget_s / max(t_probe, 1e-6) * probe_rows)))
    rows = max(16, rows // 16 * 16)
    t, kind = cpu_int8(ob, X, W, sc, zp, rows)
    tops = 2.0 * rows * N * K / t / 1e12
    return {"value": tops, "unit": "TOPS", "cores": 1, "kind": kind,
            "sample": f"first {rows} of {X.shape[0]} activation rows against the full {N}x{K} weight matrix "
                      f"({t:.1f} s single-threaded quantized_matmul)"}


def cpu_sgemm(ob, tA, tB, M, N, K, A, B, Cm, beta, threads):
    """One fp32 GEMM on the CPU path: l-ten's cpu_gemm<float> (threadpool + AVX build) where compiled, else the port."""
    ref = ob.ref()
    if ref is not None and (N < 16 or N % 8 == 0):
        rc = ref.ref_cpu_gemm_f32(int(tA), int(tB), M, N, K, 1.0, A.reshape(-1), B.reshape(-1), beta, Cm.reshape(-1))
        assert rc == 0
        return "reference"
    ob.oracle().oracle_sgemm_mt(int(tA), int(tB), M, N, K, 1.0, A.reshape(-1), M if tA else K, B.reshape(-1),
                                K if tB else N, beta, Cm.reshape(-1), N, threads)
    return "port"


def extra_configs(lt, wl, with_cpu):
    """Configs 1, 2, 4, 5: GPU time per pass (HIP events), rate against the bound that applies, CPU path beside it."""
    from oracle import bindings as ob
    D = lt.DeviceBuffer
    l = lt.lib()
    threads = os.cpu_count() or 1
    if ob.ref() is not None:
        threads = int(ob.ref().ref_hardware_threads())
    out = []

    # ---- config 1: int8 FC 64x512x784 (latency bound)
    X, W, sc, zp = wl.cfg1()
    M, K = X.shape
    N = W.shape[0]
    dA, dB, dC, ws, qp = D.from_numpy(X), D.from_numpy(W), D(M * N), D(4 * (M + N)), lt.qparams3(sc, zp)
    ms = timed(lt, lambda: lt.quantized_matmul(False, True, M, N, K, dA, dB, dC, qp, None, ws), 200)
    rec = {"config": "cfg1 int8 FC 64x512x784 (zero point 0, zero-point row-sum correction active)", "gpu_us": round(ms * 1e3, 2),
           "kernel": lt.last_kernel(), "gops": round(2.0 * M * N * K / ms / 1e6, 1), "bound": "launch latency",
           "algorithmic_bytes": M * K + N * K + M * N}
    if with_cpu:
        t = min(cpu_int8(ob, X, W, sc, zp)[0] for _ in range(5))
        rec.update(cpu_ms=round(t * 1e3, 3), cpu_cores=1, cpu_kind=cpu_int8(ob, X, W, sc, zp)[1], speedup=round(t * 1e3 / ms, 1))
    out.append(rec)

    # ---- config 4: skinny weight streaming, M in {1, 4, 16}, K = N = 8192 (HBM bound)
    for M in (1, 4, 16):
        X, W, sc, zp = wl.cfg4(M)
        N, K = W.shape
        dA, dB, dC, ws, qp = D.from_numpy(X), D.from_numpy(W), D(M * N), D(4 * (M + N)), lt.qparams3(sc, zp)
        ms = timed(lt, lambda: lt.quantized_matmul(False, True, M, N, K, dA, dB, dC, qp, None, ws), 100)
        nbytes = N * K + M * K + M * N
        gbs = nbytes / ms / 1e6
        rec = {"config": f"cfg4 int8 FC skinny M={M} K=N=8192", "gpu_us": round(ms * 1e3, 2), "kernel": lt.last_kernel(),
               "algorithmic_bytes": nbytes,
               "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                            "frac": round(gbs / HBM_PEAK_GBS, 4)}}
        if with_cpu:
            t, kind = cpu_int8(ob, X, W, sc, zp)
            rec.update(cpu_ms=round(t * 1e3, 2), cpu_cores=1, cpu_kind=kind, speedup=round(t * 1e3 / ms, 1))
        out.append(rec)
        del dA, dB, dC, ws

    # ---- config 2: fp32 MLP 784-1024-1024-10, batch 128, one training step resident on the device: 3 forward GEMMs with
    # bias, relu after the first two, log_softmax + nll_loss, their backward, then per layer the data-gradient GEMM,
    # the weight-gradient GEMM (which also sums the bias gradient) and relu_backward.
    X, Ws, bs, labels = wl.cfg2()
    B_ = X.shape[0]
    sizes = [X.shape[1]] + [w.shape[0] for w in Ws]
    pre = [None] + [D(4 * B_ * n) for n in sizes[1:]]
    acts = [D.from_numpy(X)] + [D(4 * B_ * n) for n in sizes[1:-1]] + [pre[-1]]
    grads = [D(4 * B_ * n, zero=True) for n in sizes]
    tmpg = [D(4 * B_ * n, zero=True) for n in sizes]
    dWs, dbs = [D.from_numpy(w) for w in Ws], [D.from_numpy(b) for b in bs]
    gWs, gbs_ = [D(w.nbytes) for w in Ws], [D(b.nbytes, zero=True) for b in bs]
    dT = D.from_numpy(np.eye(sizes[-1], dtype=np.float32)[labels])
    logp, gl, loss = D(4 * B_ * sizes[-1]), D(4 * B_ * sizes[-1]), D(4)

    def mlp_step():
        for i in range(3):
            lt.check(l.lten_hip_fc_forward_f32(B_, sizes[i], sizes[i + 1], acts[i].ptr, dWs[i].ptr, dbs[i].ptr, pre[i + 1].ptr))
            if i < 2:
                lt.check(l.lten_hip_relu_f32(acts[i + 1].ptr, pre[i + 1].ptr, B_ * sizes[i + 1]))
        lt.check(l.lten_hip_log_softmax_f32(B_, sizes[-1], pre[3].ptr, logp.ptr))
        lt.check(l.lten_hip_nll_loss_f32(logp.ptr, dT.ptr, loss.ptr, B_ * sizes[-1], B_))
        lt.check(l.lten_hip_scale_f32(B_ * sizes[-1], -1.0 / B_, dT.ptr, gl.ptr))
        lt.check(l.lten_hip_log_softmax_backward_f32(B_, sizes[-1], logp.ptr, gl.ptr, grads[3].ptr))
        for i in (2, 1, 0):
            lt.check(l.lten_hip_fc_backward_f32(B_, sizes[i], sizes[i + 1], acts[i].ptr, dWs[i].ptr, grads[i + 1].ptr,
                                                tmpg[i].ptr, gWs[i].ptr, gbs_[i].ptr))
            if i > 0:
                lt.check(l.lten_hip_relu_backward_f32(grads[i].ptr, tmpg[i].ptr, pre[i].ptr, B_ * sizes[i]))
    def mlp_step_fused(input_gradient=True):
        for i in range(3):
            if i < 2:
                lt.check(l.lten_hip_fc_forward_relu_f32(B_, sizes[i], sizes[i + 1], acts[i].ptr, dWs[i].ptr, dbs[i].ptr, pre[i + 1].ptr, acts[i + 1].ptr))
            else:
                lt.check(l.lten_hip_fc_forward_f32(B_, sizes[i], sizes[i + 1], acts[i].ptr, dWs[i].ptr, dbs[i].ptr, pre[i + 1].ptr))
        lt.check(l.lten_hip_fc_backward_log_softmax_nll_loss_f32(B_, sizes[2], sizes[3], acts[2].ptr, dWs[2].ptr, pre[3].ptr, dT.ptr, -1.0 / B_,
                                                                 logp.ptr, loss.ptr, grads[3].ptr, pre[2].ptr, grads[2].ptr, gWs[2].ptr, gbs_[2].ptr))
        for i in (1, 0):
            if i > 0:
                lt.check(l.lten_hip_fc_backward_relu_f32(B_, sizes[i], sizes[i + 1], acts[i].ptr, dWs[i].ptr, grads[i + 1].ptr, pre[i].ptr,
                                                         grads[i].ptr, gWs[i].ptr, gbs_[i].ptr))
            else:
                lt.check(l.lten_hip_fc_backward_f32(B_, sizes[i], sizes[i + 1], acts[i].ptr, dWs[i].ptr, grads[i + 1].ptr,
                                                    tmpg[i].ptr if input_gradient else None, gWs[i].ptr, gbs_[i].ptr))
    unfused_ms = timed(lt, mlp_step, 100)
    ms = timed(lt, mlp_step_fused, 100)
    # l-ten's backward pass also works out the gradient with respect to the network's input (its traversal calls
    # fc_backward for every child, l-ten/backprop.cpp:312-349) and drops it when the input tensor takes no gradient;
    # the step without that product is timed beside the one above
    no_dx_ms = timed(lt, lambda: mlp_step_fused(False), 100)
    no_dx_kernel = lt.last_kernel()
    # The same launches recorded once and replayed with one submit.  Not under a profiler: rocprofv3's interception of
    # graph launches segfaulted in its own code in about half of the runs of this loop on this image.
    graph_ms = None
    if "ROCP_TOOL_LIBRARIES" not in os.environ and "rocprofiler" not in os.environ.get("LD_PRELOAD", ""):
        with lt.Graph() as step_graph:
            mlp_step()
        graph_ms = timed(lt, step_graph.launch, 100)
    flops = sum(3 * 2.0 * B_ * sizes[i] * sizes[i + 1] for i in range(3))
    tf = flops / ms / 1e9
    rec = {"config": "cfg2 fp32 MLP 784-1024-1024-10 batch 128, one training step on the device: 9 GEMMs, bias adds, bias gradients, "
                     "relu x2, log_softmax, nll_loss and their backward in 6 launches (relu and relu_backward in the GEMM stores, "
                     "dX and dW of a layer in one, log_softmax, the loss and its gradient inside the last layer's backward launch)",
           "gpu_us": round(ms * 1e3, 2), "unfused_entry_points_us": round(unfused_ms * 1e3, 2), "unfused_graph_replay_us": None if graph_ms is None else round(graph_ms * 1e3, 2),
           "gflop_per_step": round(flops / 1e9, 3),
           "without_the_gradient_of_the_input_us": round(no_dx_ms * 1e3, 2), "without_the_gradient_of_the_input_last_kernel": no_dx_kernel,
           "roofline": {"bound": "mfma", "achieved": round(tf, 2), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                        "frac": round(tf / FP32_MFMA_PEAK_TFLOPS, 4)},
           "note": "six dependent launches; the launch-to-launch latency (3 to 4.4 us from box to box for a kernel that does nothing), not the MFMA rate, sets this time (GEMM flops "
                   "only in the rate); unfused_entry_points_us = the same step through the 14 separate calls l-ten's op chain maps to, "
                   "unfused_graph_replay_us = those 14 recorded once and replayed with one submit"}
    if with_cpu:
        # The CPU step on the configuration's own data: activations and gradients of the real network.  Two columns:
        # l-ten's default build multiplies with OpenBLAS (makefile USE_OPENBLAS=1; numpy's matmul is its bundled
        # OpenBLAS sgemm), its other build with its own threadpool + AVX cpu_gemm (compiled from l-ten's sources where
        # present).  Bias add, relu, log_softmax, the loss and their backward run in numpy in both.
        onehot = np.eye(sizes[-1], dtype=np.float32)[labels]

        def cpu_step(gemm):
            acts_h, pre_h = [X], [None]
            for i in range(3):
                y = gemm(acts_h[i], Ws[i], "nt") + bs[i]
                pre_h.append(y)
                acts_h.append(np.maximum(y, 0) if i < 2 else y)
            z = pre_h[3] - pre_h[3].max(axis=1, keepdims=True)
            logp_h = z - np.log(np.exp(z).sum(axis=1, keepdims=True))
            loss_h = -(logp_h * onehot).sum() / B_
            g = (np.exp(logp_h) - onehot) / np.float32(B_)
            for i in (2, 1, 0):
                dw_h = gemm(g, acts_h[i], "tn")
                db_h = g.sum(axis=0)
                if i > 0:
                    g = gemm(g, Ws[i], "nn") * (pre_h[i] > 0)
            return loss_h, dw_h, db_h

        def gemm_openblas(a, b, mode):
            return a @ b.T if mode == "nt" else (a.T @ b if mode == "tn" else a @ b)

        kinds = set()

        def gemm_lten(a, b, mode):
            a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
            if mode == "nt":
                Mg, Kg, Ng = a.shape[0], a.shape[1], b.shape[0]
                tA, tB = 0, 1
            elif mode == "tn":
                Kg, Mg, Ng = a.shape[0], a.shape[1], b.shape[1]
                tA, tB = 1, 0
            else:
                Mg, Kg, Ng = a.shape[0], a.shape[1], b.shape[1]
                tA, tB = 0, 0
            c = np.empty((Mg, Ng), np.float32)
            kinds.add(cpu_sgemm(ob, tA, tB, Mg, Ng, Kg, a, b, c, 0.0, threads))
            return c

        cpu_step(gemm_openblas)
        t_blas = best_of(lambda: cpu_step(gemm_openblas), 7)
        cpu_step(gemm_lten)
        t_lten = best_of(lambda: cpu_step(gemm_lten), 5)
        try:
            from threadpoolctl import threadpool_info
            blas = [f"{i.get('internal_api')} {i.get('version')} x{i.get('num_threads')}" for i in threadpool_info() if i.get("user_api") == "blas"]
        except Exception:  # noqa: BLE001
            blas = []
        t = min(t_blas, t_lten)
        rec.update(cpu_ms=round(t * 1e3, 2), cpu_cores=threads, speedup=round(t * 1e3 / ms, 1),
                   cpu_openblas_ms=round(t_blas * 1e3, 2), cpu_openblas=blas or "numpy matmul",
                   cpu_lten_threadpool_avx_ms=round(t_lten * 1e3, 2), cpu_kind="+".join(sorted(kinds)),
                   cpu_note="one training step on the configuration's own activations, GEMMs through numpy's OpenBLAS sgemm (l-ten's "
                            "default backend) and through l-ten's threadpool + AVX cpu_gemm; speedup is quoted against the faster of the two")
    out.append(rec)
    del acts, pre, grads, tmpg, dWs, dbs, gWs, gbs_

    # ---- config 5: Conv2d 3x3 s1 p1, 32x1x128x128 -> 32 ch -> 64 ch: forward + weight gradient of both layers
    x, cws, dyshapes = wl.cfg5()
    Nimg, H, Wd = x.shape[0], x.shape[2], x.shape[3]
    chans = [x.shape[1]] + [w.shape[0] for w in cws]
    dx = [D.from_numpy(x)] + [D(4 * Nimg * c * H * Wd) for c in chans[1:]]
    dw_ = [D.from_numpy(w) for w in cws]
    ddy = [D.from_numpy(wl.cfg5_dy(s, layer=i)) for i, s in enumerate(dyshapes)]
    ddw = [D(w.nbytes) for w in cws]
    geos = [(Nimg, chans[i], H, Wd, chans[i + 1], 3, 3, 1, 1, 1, 1) for i in range(2)]
    wss = [D(max(int(l.lten_hip_conv2d_wgrad_workspace_bytes(*g)), 4)) for g in geos]
    wsx = D(x.nbytes)  # the data gradient of layer 1 (not part of the configuration's timed pair) lands here
    for i, g in enumerate(geos):
        Cin, Cout = g[1], g[4]
        fl = 2.0 * Nimg * Cout * H * Wd * Cin * 9
        ms_f = timed(lt, lambda: lt.check(l.lten_hip_conv2d_forward_f32(*g, dx[i].ptr, dw_[i].ptr, None, dx[i + 1].ptr)), 30)
        kf = lt.last_kernel()
        ms_w = timed(lt, lambda: lt.check(l.lten_hip_conv2d_wgrad_f32(*g, dx[i].ptr, ddy[i].ptr, ddw[i].ptr, wss[i].ptr)), 30)
        kw = lt.last_kernel()
        wsd = D(max(int(l.lten_hip_conv2d_dgrad_workspace_bytes(*g)), 4))
        ms_d = timed(lt, lambda: lt.check(l.lten_hip_conv2d_dgrad_f32(*g, dw_[i].ptr, ddy[i].ptr, dx[i].ptr if i else wsx.ptr, wsd.ptr)), 30)
        kd = lt.last_kernel()
        in_b, out_b = 4 * Nimg * Cin * H * Wd, 4 * Nimg * Cout * H * Wd
        rec = {"config": f"cfg5 Conv2d layer {i + 1}: {Cin}->{Cout} ch 3x3 s1 p1 on 32x{Cin}x128x128, forward + weight gradient",
               "forward_us": round(ms_f * 1e3, 1), "wgrad_us": round(ms_w * 1e3, 1), "kernels": [kf, kw],
               "dgrad_us": round(ms_d * 1e3, 1), "dgrad_kernel": kd,
               "gflop": round(2 * fl / 1e9, 2)}
        if Cin * 9 >= 64:
            tf = 2 * fl / (ms_f + ms_w) / 1e9
            rec["roofline"] = {"bound": "mfma", "achieved": round(tf, 2), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                               "frac": round(tf / FP32_MFMA_PEAK_TFLOPS, 4)}
        else:
            gbs = 2.0 * (in_b + out_b) / (ms_f + ms_w) / 1e6
            rec["roofline"] = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                               "frac": round(gbs / HBM_PEAK_GBS, 4), "algorithmic_bytes": 2 * (in_b + out_b)}
        if with_cpu:
            # l-ten's own loop (im2col + cpu_gemm per image) over the whole batch
            sample = Nimg
            Kc, HW = Cin * 9, H * Wd
            xin = x if i == 0 else np.random.default_rng(3).standard_normal((sample, Cin, H, Wd)).astype(np.float32)
            wmat = np.ascontiguousarray(cws[i].reshape(Cout, Kc))
            dyh = wl.cfg5_dy((sample, Cout, H, Wd), layer=i)
            col = np.empty((Kc, HW), np.float32)
            yimg = np.empty((Cout, HW), np.float32)
            dwh = np.zeros((Cout, Kc), np.float32)
            kinds = set()
            im2col = ob.ref().ref_im2col_f32 if ob.ref() is not None else ob.oracle().oracle_im2col_f32

            def cpu_pass():
                for n in range(sample):
                    im2col(xin[n].reshape(-1), Cin, H, Wd, 3, 3, 1, 1, 1, 1, col.reshape(-1))
                    kinds.add(cpu_sgemm(ob, 0, 0, Cout, HW, Kc, wmat, col, yimg, 0.0, threads))
                for n in range(sample):
                    im2col(xin[n].reshape(-1), Cin, H, Wd, 3, 3, 1, 1, 1, 1, col.reshape(-1))
                    kinds.add(cpu_sgemm(ob, 0, 1, Cout, Kc, HW, np.ascontiguousarray(dyh[n].reshape(Cout, HW)), col, dwh, 1.0, threads))
            cpu_pass()
            t_lten = best_of(cpu_pass, 2) * (Nimg / sample)

            def cpu_pass_openblas():  # the same loop with the products through numpy's OpenBLAS sgemm (l-ten's default backend)
                col2 = col.reshape(Kc, HW)
                for n in range(sample):
                    im2col(xin[n].reshape(-1), Cin, H, Wd, 3, 3, 1, 1, 1, 1, col.reshape(-1))
                    np.matmul(wmat, col2, out=yimg)
                for n in range(sample):
                    im2col(xin[n].reshape(-1), Cin, H, Wd, 3, 3, 1, 1, 1, 1, col.reshape(-1))
                    dwh[...] += dyh[n].reshape(Cout, HW) @ col2.T
            cpu_pass_openblas()
            t_blas = best_of(cpu_pass_openblas, 2) * (Nimg / sample)
            t = min(t_lten, t_blas)
            rec.update(cpu_ms=round(t * 1e3, 1), cpu_cores=threads, cpu_kind="+".join(sorted(kinds)),
                       cpu_openblas_ms=round(t_blas * 1e3, 1), cpu_lten_threadpool_avx_ms=round(t_lten * 1e3, 1),
                       cpu_sample=f"all {Nimg} images; speedup against the faster of the two CPU columns",
                       speedup=round(t * 1e3 / (ms_f + ms_w), 1))
        out.append(rec)

    # ---- beyond the five configs: Conv2d_q forward, the 1 -> 10 channel 5x5 layer of l-ten's quantized MNIST network
    geo = (64, 1, 28, 28, 10, 5, 5, 0, 0, 1, 1)
    rng = np.random.default_rng(7)
    xq = rng.integers(0, 256, (64, 1, 28, 28), dtype=np.uint8)
    wq = rng.integers(0, 256, (10, 1, 5, 5), dtype=np.uint8)
    sc, zp = [1.0 / 255.0, 0.01, 0.05], [0, 128, 128]
    dxq, dwq, dyq = D.from_numpy(xq), D.from_numpy(wq), D(64 * 10 * 24 * 24)
    wsq = D(max(int(l.lten_hip_conv2dq_workspace_bytes(*geo)), 16))
    qpq = lt.qparams3(sc, zp)
    ms = timed(lt, lambda: lt.check(l.lten_hip_conv2dq_forward(*geo, dxq.ptr, dwq.ptr, None, qpq, dyq.ptr, wsq.ptr)), 100)
    nbytes = xq.nbytes + wq.nbytes + 64 * 10 * 24 * 24
    rec = {"config": "Conv2d_q forward 64x1x28x28 -> 10 ch 5x5 (l-ten's quantized MNIST conv1, batch 64)", "gpu_us": round(ms * 1e3, 2),
           "kernel": lt.last_kernel(), "bound": "launch latency", "algorithmic_bytes": nbytes}
    if with_cpu:
        f = (lambda: ob.ref_conv2dq_forward(geo, xq, wq, sc, zp)) if ob.ref() is not None else (lambda: ob.conv2dq_forward(geo, xq, wq, sc, zp, want_acc=False))
        t = best_of(f, 3)
        rec.update(cpu_ms=round(t * 1e3, 3), cpu_cores=1, cpu_kind="reference" if ob.ref() is not None else "port",
                   speedup=round(t * 1e3 / ms, 1))
    out.append(rec)

    # ---- the second conv of that network, 10 -> 20 channels 5x5 on the pooled 12x12 maps: 250 taps, one launch from the
    # image in LDS
    geo2 = (64, 10, 12, 12, 20, 5, 5, 0, 0, 1, 1)
    xq2 = rng.integers(0, 256, (64, 10, 12, 12), dtype=np.uint8)
    wq2 = rng.integers(0, 256, (20, 10, 5, 5), dtype=np.uint8)
    dxq2, dwq2, dyq2 = D.from_numpy(xq2), D.from_numpy(wq2), D(64 * 20 * 8 * 8)
    wsq2 = D(max(int(l.lten_hip_conv2dq_workspace_bytes(*geo2)), 16))
    ms2 = timed(lt, lambda: lt.check(l.lten_hip_conv2dq_forward(*geo2, dxq2.ptr, dwq2.ptr, None, qpq, dyq2.ptr, wsq2.ptr)), 100)
    rec = {"config": "Conv2d_q forward 64x10x12x12 -> 20 ch 5x5 (l-ten's quantized MNIST conv2, batch 64)", "gpu_us": round(ms2 * 1e3, 2),
           "kernel": lt.last_kernel(), "bound": "launch latency", "algorithmic_bytes": xq2.nbytes + wq2.nbytes + 64 * 20 * 8 * 8}
    if with_cpu:
        f2 = (lambda: ob.ref_conv2dq_forward(geo2, xq2, wq2, sc, zp)) if ob.ref() is not None else (lambda: ob.conv2dq_forward(geo2, xq2, wq2, sc, zp, want_acc=False))
        t2 = best_of(f2, 3)
        rec.update(cpu_ms=round(t2 * 1e3, 3), cpu_cores=1, cpu_kind="reference" if ob.ref() is not None else "port",
                   speedup=round(t2 * 1e3 / ms2, 1))
    out.append(rec)

    # ---- a quantized layer of the size of a ResNet block, 64 -> 64 channels 3x3 on 56x56 maps, batch 32: one launch, a band
    # of output rows per workgroup (checked against the three-launch route of the same library, option conv_variant 2)
    geo3 = (32, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1)
    xq3 = rng.integers(0, 256, (32, 64, 56, 56), dtype=np.uint8)
    wq3 = rng.integers(0, 256, (64, 64, 3, 3), dtype=np.uint8)
    qpq3 = lt.qparams3([0.02, 0.013, 0.9], [17, 250, 100])
    dxq3, dwq3, dyq3, dyq3b = D.from_numpy(xq3), D.from_numpy(wq3), D(xq3.size), D(xq3.size)
    wsq3 = D(max(int(l.lten_hip_conv2dq_workspace_bytes(*geo3)), 16))
    run3 = lambda dy: lt.check(l.lten_hip_conv2dq_forward(*geo3, dxq3.ptr, dwq3.ptr, None, qpq3, dy.ptr, wsq3.ptr))
    ms3 = timed(lt, lambda: run3(dyq3), 100)
    k3 = lt.last_kernel()
    lt.set_option("conv_variant", 2)
    try:
        ms3b = timed(lt, lambda: run3(dyq3b), 20)
    finally:
        lt.set_option("conv_variant", 0)
    same3 = bool(np.array_equal(dyq3.numpy(np.uint8, (xq3.size,)), dyq3b.numpy(np.uint8, (xq3.size,))))
    ops3 = 2.0 * 32 * 64 * 56 * 56 * 64 * 9
    out.append({"config": "Conv2d_q forward 32x64x56x56 -> 64 ch 3x3, pad 1 (beyond l-ten's networks)", "gpu_us": round(ms3 * 1e3, 2), "kernel": k3,
                "three_launch_route_us": round(ms3b * 1e3, 2), "same_bytes_as_three_launch_route": same3,
                "achieved_TOPs": round(ops3 / ms3 / 1e9, 1), "bound": "LDS reads; memory latency at the start",
                "algorithmic_bytes": xq3.nbytes + wq3.nbytes + xq3.size})
    del dxq3, dwq3, dyq3, dyq3b, wsq3

    # ---- fp32 Conv2d layers of many channels on small maps (the late stages of a ResNet-like network), where no patch
    # kernel applies: the batch's column matrices in library memory and the direct-to-LDS GEMM tiles, against the implicit
    # GEMM (forward) and l-ten's GEMM + col2im image by image (data gradient) of the same library (option conv_variant 1)
    # on the same operands
    for geo4, what in (((32, 256, 14, 14, 256, 3, 3, 1, 1, 1, 1), "256 -> 256 ch 3x3 on 32x256x14x14"),
                       ((32, 128, 28, 28, 256, 3, 3, 1, 1, 2, 2), "128 -> 256 ch 3x3 stride 2 on 32x128x28x28")):
        N4, Ci4, H4, W4, Co4, kh4, kw4, ph4, pw4, sh4, sw4 = geo4
        Ho4, Wo4 = (H4 + 2 * ph4 - kh4) // sh4 + 1, (W4 + 2 * pw4 - kw4) // sw4 + 1
        rng4 = np.random.default_rng(sum(geo4))
        x4 = D.from_numpy(rng4.standard_normal((N4, Ci4, H4, W4)).astype(np.float32))
        w4 = D.from_numpy((rng4.standard_normal((Co4, Ci4 * kh4 * kw4)) * 0.05).astype(np.float32))
        b4 = D.from_numpy(rng4.standard_normal(Co4).astype(np.float32))
        dy4 = D.from_numpy(rng4.standard_normal((N4, Co4, Ho4, Wo4)).astype(np.float32))
        ny, nx = N4 * Co4 * Ho4 * Wo4, N4 * Ci4 * H4 * W4
        y4, y4b, dx4, dx4b = D(4 * ny), D(4 * ny), D(4 * nx), D(4 * nx)
        ws4 = D(max(int(l.lten_hip_conv2d_dgrad_workspace_bytes(*geo4)), 16))
        fwd = lambda y: lt.check(l.lten_hip_conv2d_forward_f32(*geo4, x4.ptr, w4.ptr, b4.ptr, y.ptr))
        bwd = lambda dx: lt.check(l.lten_hip_conv2d_dgrad_f32(*geo4, w4.ptr, dy4.ptr, dx.ptr, ws4.ptr))
        ms_f = timed(lt, lambda: fwd(y4), 50)
        kf4 = lt.last_kernel()
        ms_d = timed(lt, lambda: bwd(dx4), 50)
        kd4 = lt.last_kernel()
        lt.set_option("conv_variant", 1)
        try:
            ms_f1 = timed(lt, lambda: fwd(y4b), 20)
            ms_d1 = timed(lt, lambda: bwd(dx4b), 20)
        finally:
            lt.set_option("conv_variant", 0)
        ya, yb = y4.numpy(np.float32, (ny,)), y4b.numpy(np.float32, (ny,))
        da, db_ = dx4.numpy(np.float32, (nx,)), dx4b.numpy(np.float32, (nx,))
        fl4 = 2.0 * ny * Ci4 * kh4 * kw4
        out.append({"config": f"Conv2d fp32 {what} (beyond l-ten's networks), forward with bias + data gradient",
                    "forward_us": round(ms_f * 1e3, 1), "forward_kernel": kf4, "dgrad_us": round(ms_d * 1e3, 1), "dgrad_kernel": kd4,
                    "implicit_gemm_forward_us": round(ms_f1 * 1e3, 1), "dgrad_image_by_image_gemm_col2im_us": round(ms_d1 * 1e3, 1),
                    "max_rel_diff_to_those": float(max(np.abs(ya - yb).max() / np.abs(yb).max(), np.abs(da - db_).max() / np.abs(db_).max())),
                    "roofline": {"bound": "mfma", "achieved": round(fl4 / ms_f / 1e9, 1), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                                 "frac": round(fl4 / ms_f / 1e9 / FP32_MFMA_PEAK_TFLOPS, 4)}})
        del x4, w4, dy4, y4, y4b, dx4, dx4b, ws4

    # ---- int8 layers whose sizes are no multiples of the kernels' vector widths: in_features no multiple of 16 (the rows
    # are copied into padded ones first; prepared weights are padded once), out_features no multiple of 4 (byte stores).
    # Prepared weights, zero points (17, 250, 100); the first rows (2^30 multiply-adds' worth) against the oracle.
    for (Mo, No, Ko, what) in ((4096, 4096, 4100, "in_features = 4100, no multiple of 16"), (4096, 1001, 4096, "out_features = 1001, no multiple of 4"),
                               (64, 500, 1000, "a 1000 -> 500 layer at batch 64")):
        rngo = np.random.default_rng(Mo + No + Ko)
        Xo = rngo.integers(0, 256, (Mo, Ko), dtype=np.uint8)
        Wo_ = (np.clip(np.round(rngo.normal(0, 40, (No, Ko))), -127, 127).astype(np.int16) + 128).astype(np.uint8)
        Kp = (Ko + 15) // 16 * 16
        dXo, dWo, dWp, dSo, dYo, wso = D.from_numpy(Xo), D.from_numpy(Wo_), D(No * Kp), D(4 * No), D(Mo * No), D(4 * (Mo + No))
        lt.check(l.lten_hip_fcq_prepare_weights(dWo.ptr, dWp.ptr, No, Ko, dSo.ptr))
        sco, zpo = [0.02, 0.01, 3.0 * Ko / 4096], [17, 250, 100]
        qpo = lt.qparams3(sco, zpo)
        fo = lambda: lt.check(l.lten_hip_fcq_forward_prepared(1, Mo, Ko, No, dXo.ptr, dWp.ptr, dSo.ptr, None, qpo, dYo.ptr, wso.ptr))
        mso = timed(lt, fo, 100)
        rec = {"config": f"int8 FC {Mo}x{No}x{Ko} ({what}), prepared weights, zero points (17, 250, 100)", "gpu_us": round(mso * 1e3, 2),
               "kernel": lt.last_kernel(), "achieved_TOPs": round(2.0 * Mo * No * Ko / mso / 1e9, 1)}
        if with_cpu:
            rows = max(1, min(Mo, (1 << 30) // (No * Ko)))
            want_o, _ = ob.quantized_matmul(Xo[:rows], Wo_, np.array(sco, np.float32), np.array(zpo, np.uint8))
            rec["verified_bit_exact_rows"] = rows if np.array_equal(dYo.numpy(np.uint8, (Mo, No))[:rows], want_o) else 0
        out.append(rec)
        del dXo, dWo, dWp, dSo, dYo, wso

    # ---- beyond the five configs: a large fp32 product in the three layouts l-ten's layers use (FullyConnected forward
    # NT, data gradient NN, weight gradient TN), synthetic N(0,1) operands
    n = 4096
    ga = D.from_numpy(np.random.default_rng(11).standard_normal((n, n)).astype(np.float32))
    gb = D.from_numpy(np.random.default_rng(12).standard_normal((n, n)).astype(np.float32))
    gc = D(4 * n * n)
    per_layout = {}
    for name, (ta, tb) in (("NT", (0, 1)), ("NN", (0, 0)), ("TN", (1, 0))):
        ms = timed(lt, lambda: lt.sgemm(ta, tb, n, n, n, 1.0, ga, n, gb, n, 0.0, gc, n), 10, warmup=10)
        per_layout[name] = round(ms * 1e3, 1)
    kname = lt.last_kernel()
    ms = sum(per_layout.values()) / 3e3
    tf = 2.0 * n ** 3 / ms / 1e9
    out.append({"config": "fp32 sgemm 4096^3 (Tensor::matmul / FullyConnected at scale), mean of NT, NN, TN", "gpu_us": round(ms * 1e3, 1),
                "per_layout_us": per_layout, "kernel": kname,
                "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                             "frac": round(tf / FP32_MFMA_PEAK_TFLOPS, 4)}})
    del ga, gb, gc

    # ---- beyond the five configs: one GRU time step's two M = 1 products (l-ten/gru.cpp:267-268), input = hidden = 1024
    hid = 1024
    gx = D.from_numpy(np.random.default_rng(13).standard_normal(hid).astype(np.float32))
    gu = D.from_numpy(np.random.default_rng(14).standard_normal((hid, 3 * hid)).astype(np.float32))
    gy = D(4 * 3 * hid)
    ms = timed(lt, lambda: lt.sgemm(0, 0, 1, 3 * hid, hid, 1.0, gx, hid, gu, 3 * hid, 0.0, gy, 3 * hid), 100)
    nbytes = 4 * (hid + hid * 3 * hid + 3 * hid)
    out.append({"config": "GRU step product 1 x 1024 times 1024 x 3072 (fp32, M = 1)", "gpu_us": round(ms * 1e3, 2), "kernel": lt.last_kernel(),
                "algorithmic_bytes": nbytes,
                "roofline": {"bound": "hbm", "achieved": round(nbytes / ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}})
    # both products of the time step (x U and h W, l-ten/gru.cpp:358-361) as one strided batch of two: one launch
    gxh = D.from_numpy(np.random.default_rng(15).standard_normal((2, hid)).astype(np.float32))
    guw = D.from_numpy(np.random.default_rng(16).standard_normal((2, hid, 3 * hid)).astype(np.float32))
    gy2 = D(4 * 2 * 3 * hid)
    ms = timed(lt, lambda: lt.check(l.lten_hip_sgemm_strided_batched(0, 0, 1, 3 * hid, hid, 1.0, gxh.ptr, hid, hid, guw.ptr, 3 * hid, hid * 3 * hid,
                                                                     0.0, gy2.ptr, 3 * hid, 3 * hid, 2)), 100)
    out.append({"config": "GRU time step, both products (x U and h W, 1 x 1024 times 1024 x 3072 each) in one batched launch", "gpu_us": round(ms * 1e3, 2),
                "kernel": lt.last_kernel(), "algorithmic_bytes": 2 * nbytes,
                "roofline": {"bound": "hbm", "achieved": round(2 * nbytes / ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": round(2 * nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}})
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-verify", action="store_true", help="skip the post-run output check")
    ap.add_argument("--no-extra", action="store_true", help="skip the per-config records for configs 1, 2, 4, 5")
    ap.add_argument("--no-vendor", action="store_true", help="skip the torch._int_mm (hipBLASLt) calibration leg")
    ap.add_argument("--no-telemetry", action="store_true", help="skip the two-second power / clock reading")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="run only the plain copy kernel on buffers of this size (what FETCH_SIZE / WRITE_SIZE "
                         "counters are scaled against) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (the path has no collective to scale); use --gpus 1")

    lt = load_package()
    from light_tensor_amd import workloads as wl
    lt.init(0)

    if args.copy_calibration:
        nbytes = args.copy_calibration << 20
        src, dst = lt.DeviceBuffer(nbytes), lt.DeviceBuffer(nbytes)
        lt.check(lt.lib().lten_hip_zero(src.ptr, nbytes))
        for _ in range(max(args.warmup, 1)):
            lt.measure_copy(src, dst, nbytes)
        lt.sync()
        timer = lt.Timer()
        timer.start()
        for _ in range(args.steps):
            lt.measure_copy(src, dst, nbytes)
        ms = timer.stop_ms() / args.steps
        print(json.dumps({"copy_bytes_read": nbytes, "copy_bytes_written": nbytes, "us": round(ms * 1e3, 2),
                          "GB_per_s": round(2 * nbytes / ms / 1e6, 1)}))
        return

    M = N = K = 4096
    X, W, sc, zp = wl.cfg3()
    l = lt.lib()
    dA, dB = lt.DeviceBuffer.from_numpy(X), lt.DeviceBuffer.from_numpy(W)
    dBp, dBs = lt.DeviceBuffer(N * K), lt.DeviceBuffer(4 * N)
    lt.check(l.lten_hip_fcq_prepare_weights(dB.ptr, dBp.ptr, N, K, dBs.ptr))   # once per layer, as FullyConnected_q::to(GPU) does
    dC = lt.DeviceBuffer(M * N)
    ws = lt.DeviceBuffer(4 * (M + N))
    qp = lt.qparams3(sc, zp)

    def step():
        lt.check(l.lten_hip_fcq_forward_prepared(1, M, K, N, dA.ptr, dBp.ptr, dBs.ptr, None, qp, dC.ptr, ws.ptr))

    def step_raw():
        lt.quantized_matmul(False, True, M, N, K, dA, dB, dC, qp, None, ws)

    # The sustained figure: clocks settle only after tens of milliseconds of load, so the roofline fraction is taken
    # from 300 back-to-back launches that follow at least 60 ms of the same launches.  It runs before the timed region,
    # which therefore starts on a part that is already in its steady state.
    def sustained(fn):
        t_end = time.perf_counter() + 0.06
        n = 0
        while time.perf_counter() < t_end or n < 600:
            fn()
            n += 1
            if n % 100 == 0:
                lt.sync()
        lt.sync()
        t = lt.Timer()
        t.start()
        for _ in range(300):
            fn()
        return t.stop_ms() / 300

    ops = 2.0 * M * N * K
    raw_ms = sustained(step_raw)
    raw_kernel = lt.last_kernel()
    # what the part draws and clocks at while it runs the headline kernel (two seconds of it)
    tele = None if args.no_telemetry else telemetry(lt, step)

    # The same product with zero points that need the correction terms: a post-relu activation tensor (zero point 0)
    # against symmetric weights, and a general triple.  On prepared weights both stay one launch.
    general_zp = []
    for zps in ((0, 128, 128), (17, 250, 100)):
        qpz = lt.qparams3(sc, zps)

        def step_zp():
            lt.check(l.lten_hip_fcq_forward_prepared(1, M, K, N, dA.ptr, dBp.ptr, dBs.ptr, None, qpz, dC.ptr, ws.ptr))

        def step_zp_raw():
            lt.quantized_matmul(False, True, M, N, K, dA, dB, dC, qpz, None, ws)
        zms = sustained(step_zp)
        zkern = lt.last_kernel()
        ok = None
        if not args.no_verify:
            acc = ((X.astype(np.float64) - float(zps[0])) @ (W.astype(np.float64) - float(zps[1])).T)
            mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
            sfl = (acc.astype(np.float32) * mult).astype(np.float32) + np.float32(zps[2])
            ok = bool(np.array_equal(dC.numpy(np.uint8, (M, N)), (np.trunc(sfl).astype(np.int64) & 0xFF).astype(np.uint8)))
        zraw_ms = sustained(step_zp_raw)
        general_zp.append({"zero_points_in_wt_out": list(zps), "kernel": zkern, "launches": 1, "sustained_kernel_us": round(zms * 1e3, 2),
                           "tops": round(ops / (zms * 1e-3) / 1e12, 1),
                           "roofline": {"bound": "mfma", "achieved": round(ops / (zms * 1e-3) / 1e12, 1), "peak": INT8_MFMA_PEAK_TOPS,
                                        "unit": "TOP/s", "frac": round(ops / (zms * 1e-3) / 1e12 / INT8_MFMA_PEAK_TOPS, 4)},
                           "raw_uint8_weights_two_launches_us": round(zraw_ms * 1e3, 2), "verified_bit_exact": ok})
    sustained_ms = sustained(step)
    achieved = ops / (sustained_ms * 1e-3) / 1e12

    # The synchronisation that closes the timed region polls the stream (hipStreamQuery on the library's stream, the
    # null stream here) instead of sleeping in hipStreamSynchronize: a blocked host thread is woken tens of microseconds
    # after the last kernel has finished, which at 20 steps of 55 us is 2 % of the region.
    hip = C.CDLL("libamdhip64.so")

    def spin_sync():
        while True:
            rc = hip.hipStreamQuery(None)
            if rc == 0:
                return
            if rc != 600:   # hipErrorNotReady
                raise RuntimeError(f"hipStreamQuery: error {rc}")

    for _ in range(args.warmup):
        step()
    spin_sync()
    timer = lt.Timer()
    t0 = time.perf_counter()
    timer.start()
    for _ in range(args.steps):
        step()
    timer.record_stop()
    spin_sync()
    wall = time.perf_counter() - t0
    kernel_ms = timer.elapsed_ms() / args.steps   # HIP events on the stream the kernel runs on
    kernel = lt.last_kernel()

    ms_per_step = wall / args.steps * 1e3
    value = ops / (ms_per_step * 1e-3) / 1e12

    # The same call as an l-ten caller without device-resident tensors sees it: synchronous upload of both operands,
    # the product, synchronous download of the output (never the reported value).
    host_out = np.empty((M, N), np.uint8)

    def with_copies():
        dA.upload(X)
        dB.upload(W)
        step_raw()
        lt.check(lt.lib().lten_hip_copy_from_gpu(host_out.ctypes.data, dC.ptr, host_out.nbytes))
    with_copies()
    copies_ms = best_of(with_copies, 3) * 1e3

    # and through the host-side mirror of l-ten's layer API (lten::Tensor::to, lten::FullyConnected_q::forward, C++)
    host_api = None
    host_exe = os.path.join(ROOT, "light-tensor_amd", "host", "test_host")
    if os.path.exists(host_exe):
        import subprocess
        try:
            r = subprocess.run([host_exe, "bench"], capture_output=True, text=True, timeout=120)
            lines = [ln for ln in r.stdout.splitlines() if ln.startswith("{")]
            host_api = json.loads(lines[-1]) if r.returncode == 0 and lines else {"error": (r.stdout + r.stderr)[-300:]}
        except Exception as e:  # noqa: BLE001
            host_api = {"error": repr(e)[:300]}

    verified = None
    if not args.no_verify:
        acc = ((X.astype(np.float64) - float(zp[0])) @ (W.astype(np.float64) - float(zp[1])).T)
        mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
        sfl = (acc.astype(np.float32) * mult).astype(np.float32) + np.float32(zp[2])
        want = (np.trunc(sfl).astype(np.int64) & 0xFF).astype(np.uint8)
        step()
        ok_prepared = bool(np.array_equal(dC.numpy(np.uint8, (M, N)), want))
        lt.check(l.lten_hip_zero(dC.ptr, M * N))
        step_raw()
        verified = ok_prepared and bool(np.array_equal(dC.numpy(np.uint8, (M, N)), want))

    # MFMA-only ceilings of this part: constant operands, and operands that change like a GEMM's, at 1, 2 and 4
    # wavefronts per SIMD
    measured_peak = lt.measure_mfma_peak(0, 1)
    _, shader_mhz = lt.measure_last_clocks()
    data_peaks, data_mhz = {}, {}
    for wps in (1, 2, 4):
        data_peaks[wps] = lt.measure_mfma_peak(2, wps)
        data_mhz[wps] = lt.measure_last_clocks()[1]
    measured_peak_data = max(data_peaks.values())
    # and on operands taken from this very product's matrices (uniform bytes against N(0,40) bytes): its own ceiling
    own_peaks, own_mhz = {}, {}
    for wps in (1, 2, 4):
        own_peaks[wps] = lt.measure_mfma_peak_operands(dA, dBp, M * K, wps)
        own_mhz[wps] = lt.measure_last_clocks()[1]
    measured_peak_own = max(own_peaks.values())
    vendor = None if args.no_vendor else vendor_int8()

    out = {
        "metric": "int8_fc_forward_tops_4096",
        "value": round(value, 2),
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "value_raw_uint8_weights": round(ops / (raw_ms * 1e-3) / 1e12, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "cfg3 int8 FullyConnected_q forward M=N=K=4096: uint8 activations (zero point 128) x "
                               "8-bit weights (N(0,40) clipped, zero point 128) -> int32 -> fused requantize to uint8; the layer's "
                               "weights were converted to int8 once outside the timed region (lten_hip_fcq_prepare_weights), "
                               "value_raw_uint8_weights is the same product on l-ten's uint8 weight bytes",
                   "M": M, "N": N, "K": K, "input_digest": wl.digest(X, W)},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOP/s",
                     "frac": round(achieved / INT8_MFMA_PEAK_TOPS, 4), "traffic": traffic_bytes(kernel),
                     "kernel": kernel, "sustained_kernel_us": round(sustained_ms * 1e3, 2),
                     "timed_region_kernel_us": round(kernel_ms * 1e3, 2), "algorithmic_bytes": 3 * M * N,
                     "raw_uint8_weights": {"kernel": raw_kernel, "sustained_kernel_us": round(raw_ms * 1e3, 2),
                                           "tops": round(ops / (raw_ms * 1e-3) / 1e12, 1)},
                     "measured_mfma_only_tops": round(measured_peak, 1), "measured_mfma_only_shader_mhz": round(shader_mhz),
                     "measured_mfma_only_data_operands_tops": {str(k): round(v, 1) for k, v in data_peaks.items()},
                     "measured_mfma_only_data_operands_shader_mhz": {str(k): round(v) for k, v in data_mhz.items()},
                     "frac_of_measured_mfma_only_data_operands": round(achieved / measured_peak_data, 4),
                     "measured_mfma_only_cfg3_operands_tops": {str(k): round(v, 1) for k, v in own_peaks.items()},
                     "measured_mfma_only_cfg3_operands_shader_mhz": {str(k): round(v) for k, v in own_mhz.items()},
                     "frac_of_measured_mfma_only_cfg3_operands": round(achieved / measured_peak_own, 4),
                     "frac_driver_timed": round(value / INT8_MFMA_PEAK_TOPS, 4),
                     "power_w": tele and tele["power_w"], "power_cap_w": tele and tele["power_cap_w"],
                     "sclk_mhz": tele and tele["sclk_mhz"], "telemetry": tele,
                     "vendor_int8_gemm_same_shape": vendor,
                     "same_shape_other_zero_points": general_zp,
                     "note": "int8 multiply-add counted as 2 ops; achieved = 2*4096^3 / sustained_kernel_us (300 back-to-back "
                             "launches after at least 60 ms of the same load, HIP events on the library's stream); "
                             "timed_region_kernel_us = the same over the --steps launches; measured_mfma_only = a kernel that "
                             "issues nothing but 32x32x32 int8 MFMAs on constant operands; _data_operands = the same with "
                             "pseudo-random operands that change with every MFMA, per wavefronts per SIMD (the part lowers its "
                             "clock under that load although nothing but the matrix pipes is busy); _cfg3_operands = the same loop on "
                             "operands loaded from this product's own activation and weight matrices; frac = achieved / peak on the "
                             "sustained figure, frac_driver_timed = value / peak on the --steps launches (wall clock); power_w / "
                             "power_cap_w / sclk_mhz = socket power, its cap and the shader clock during two seconds of the headline "
                             "kernel (amdgpu hwmon and pp_dpm_sclk; per-XCD clocks from amd-smi under telemetry); vendor_int8_gemm_same_shape = "
                             "torch._int_mm (hipBLASLt) at 4096^3 in a process of its own, a calibration only"},
        "verified_bit_exact": verified,
        "with_pcie_copies": {"ms_per_step": round(copies_ms, 3), "tops": round(ops / (copies_ms * 1e-3) / 1e12, 2),
                             "note": "operands uploaded and the output downloaded with the library's synchronous copies around "
                                     "the same call, pageable host memory; for reference only",
                             "through_host_layer_api": host_api},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(X, W, sc, zp)
    del dA, dB, dBp, dBs, dC, ws
    if not args.no_extra:
        out["configs"] = extra_configs(lt, wl, not args.no_cpu)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
