"""Writes the golden vectors under tests/golden/ from the compiled l-ten CPU path.

Run in a container that has the l-ten sources, after `make -C oracle ref`:
    python tests/golden/make_golden.py
Every expected output below is produced by l-ten's own code (oracle/_ref/liblten_ref.so);
inputs come from the repo's counter-based generator or numpy's PCG64.  The files hold data
only (inputs and expected outputs).
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from conftest import load_package  # noqa: E402
from oracle import bindings as ob  # noqa: E402

load_package()
from light_tensor_amd import workloads as wl  # noqa: E402

ref = ob.ref()
assert ref is not None, "build the reference first: make -C oracle ref"
fp = C.POINTER(C.c_float)


def fptr(a):
    return None if a is None else a.ctypes.data_as(fp)


def requant_sweep():
    """Requantize alone: M=1, K=1, A=0, zero points 0 make `element` equal to bias[j]
    (l-ten/math_fns.cpp:1469-1473), so any int32 accumulator can be fed through :1474."""
    rng = np.random.default_rng(1234)
    acc = np.concatenate([
        np.arange(-70000, 70000, 7, dtype=np.int64),
        np.array([0, 1, -1, 255, 256, -255, -256, 2**24 - 1, 2**24, 2**24 + 1, -(2**24) - 1, 2**31 - 1, -(2**31),
                  2**31 - 128, 2**30, -(2**30), 16777217, 33554433, -33554433], dtype=np.int64),
        (2 ** np.arange(8, 31)).astype(np.int64) + rng.integers(-3, 4, 23),
        -(2 ** np.arange(8, 31)).astype(np.int64) + rng.integers(-3, 4, 23),
        rng.integers(-(2**31), 2**31, 6000),
        rng.integers(-400000, 400000, 6000),
    ]).astype(np.int32)
    mults = np.array([np.float32(1 / 255.0) * np.float32(0.01) / np.float32(0.05), 4e-4, 2.8e-4, 1.0, 0.5, 1e-3, 0.33333334,
                      3.0, 1e10, -0.25, 1.1920929e-07, 255.0], dtype=np.float32)
    zps = np.array([0, 128, 255, 1], dtype=np.uint8)
    n = len(acc)
    out = np.empty((len(mults), len(zps), n), dtype=np.uint8)
    A = np.zeros(1, np.uint8)
    B = np.zeros(n, np.uint8)
    ws = np.empty(1 + n, np.int32)
    for i, m in enumerate(mults):
        for j, z in enumerate(zps):
            # scale_a * scale_b / scale_c with scale_b = scale_c = 1 gives exactly m
            sc = np.array([m, 1.0, 1.0], np.float32)
            zp = np.array([0, 0, z], np.uint8)
            rc = ref.ref_quantized_matmul(0, 1, 1, n, 1, 1, A, B, 0, out[i, j], sc, zp,
                                          acc.ctypes.data_as(C.POINTER(C.c_int32)), ws)
            assert rc == 0
    np.savez_compressed(os.path.join(HERE, "requant_sweep.npz"), acc=acc, mults=mults, zps=zps, expected=out)
    print("requant_sweep", out.shape)


def qmm_cases():
    rng = np.random.default_rng(99)
    cases = {}
    idx = 0
    for (M, N, K) in [(1, 1, 1), (5, 3, 2), (37, 53, 91), (64, 48, 160), (16, 130, 257)]:
        for tA in (0, 1):
            for tB in (0, 1):
                A = rng.integers(0, 256, M * K, dtype=np.uint8)
                B = rng.integers(0, 256, N * K, dtype=np.uint8)
                zp = rng.integers(0, 256, 3).astype(np.uint8)
                sc = np.array([0.021, 0.013, 0.61], np.float32)
                bias = rng.integers(-50000, 50000, N).astype(np.int32) if (idx % 2) else None
                Cq = ob.ref_quantized_matmul(A, B, sc, zp, tA=bool(tA), tB=bool(tB), bias=bias, M=M, N=N, K=K)
                pre = f"c{idx}_"
                cases[pre + "dims"] = np.array([M, N, K, tA, tB], np.int64)
                cases[pre + "A"] = A
                cases[pre + "B"] = B
                cases[pre + "zp"] = zp
                cases[pre + "sc"] = sc
                if bias is not None:
                    cases[pre + "bias"] = bias
                cases[pre + "C"] = Cq
                idx += 1
    cases["count"] = np.array(idx)
    np.savez_compressed(os.path.join(HERE, "qmm_cases.npz"), **cases)
    print("qmm_cases", idx)


def cfg1_expected():
    X, W, sc, zp = wl.cfg1()
    Cq = ob.ref_quantized_matmul(X, W, sc, zp)
    # FullyConnected_q layer path on a {2, 32, 784} view of the same input (leading dim looped)
    Y = np.empty((2, 32, 512), np.uint8)
    rc = ref.ref_fcq_u8(2, 32, 784, 512, X.reshape(-1), W.reshape(-1), None, sc, zp, Y.reshape(-1))
    assert rc == 0 and np.array_equal(Y.reshape(64, 512), Cq)
    np.savez_compressed(os.path.join(HERE, "cfg1_expected.npz"), C=Cq, input_digest=np.array(wl.digest(X, W)))
    print("cfg1", wl.digest(X, W), wl.digest(Cq))


def sgemm_cases():
    """cpu_gemm<float> (threadpool + AVX build).  N is below 16 (scalar path only) or a multiple of 8:
    full 16-column blocks are stored with aligned 32-byte stores (l-ten/math_fns.cpp:994-1002)."""
    rng = np.random.default_rng(7)
    cases = {}
    idx = 0
    for (M, N, K) in [(4, 8, 3), (5, 16, 7), (33, 24, 129), (64, 48, 100), (3, 8, 300), (7, 13, 5), (9, 1, 20), (1, 15, 33)]:
        for (tA, tB) in [(0, 0), (0, 1), (1, 0)]:
            for (alpha, beta) in [(1.0, 0.0), (1.0, 1.0), (0.5, 2.0)]:
                A = rng.standard_normal(M * K).astype(np.float32)
                B = rng.standard_normal(N * K).astype(np.float32)
                C0 = rng.standard_normal(M * N).astype(np.float32)
                Cm = C0.copy()
                rc = ref.ref_cpu_gemm_f32(tA, tB, M, N, K, alpha, A, B, beta, Cm)
                assert rc == 0
                pre = f"c{idx}_"
                cases[pre + "dims"] = np.array([M, N, K, tA, tB], np.int64)
                cases[pre + "ab"] = np.array([alpha, beta], np.float32)
                cases[pre + "A"], cases[pre + "B"], cases[pre + "C0"], cases[pre + "C"] = A, B, C0, Cm
                idx += 1
    cases["count"] = np.array(idx)
    np.savez_compressed(os.path.join(HERE, "sgemm_cases.npz"), **cases)
    print("sgemm_cases", idx)


def layer_cases():
    rng = np.random.default_rng(21)
    out = {}
    # The layer classes allocate their own outputs, whose alignment the caller does not control, so
    # every GEMM N dimension in these cases stays below 16: l-ten then runs its scalar loops only
    # (the aligned-store AVX block needs N >= 16, l-ten/math_fns.cpp:1016).
    # FullyConnected forward + backward (bias on and off).
    idx = 0
    for (M, fin, fout, use_bias) in [(8, 12, 15, 1), (6, 14, 8, 0), (32, 9, 11, 1), (3, 5, 7, 1)]:
        x = rng.standard_normal(M * fin).astype(np.float32)
        w = (rng.standard_normal(fout * fin) * 0.2).astype(np.float32)
        b = (rng.standard_normal(fout) * 0.2).astype(np.float32) if use_bias else None
        dy = rng.standard_normal(M * fout).astype(np.float32)
        y = np.empty(M * fout, np.float32)
        dx = np.empty(M * fin, np.float32)
        dw = np.empty(fout * fin, np.float32)
        db = np.zeros(fout, np.float32)
        rc = ref.ref_fc_f32(M, fin, fout, x, w, fptr(b), fptr(dy), fptr(y), fptr(dx), fptr(dw), fptr(db))
        assert rc == 0
        pre = f"fc{idx}_"
        out[pre + "dims"] = np.array([M, fin, fout, use_bias], np.int64)
        out[pre + "x"], out[pre + "w"], out[pre + "dy"] = x, w, dy
        if use_bias:
            out[pre + "b"], out[pre + "db"] = b, db
        out[pre + "y"], out[pre + "dx"], out[pre + "dw"] = y, dx, dw
        idx += 1
    out["fc_count"] = np.array(idx)

    # Tensor::matmul with leading-dim broadcast + backward
    idx = 0
    for (ad, bd) in [((2, 1, 4, 8), (1, 1, 8, 15)), ((3, 5, 8), (3, 8, 8)), ((1, 2, 6, 13), (4, 2, 13, 8)),
                     ((2, 3, 4, 8), (2, 3, 8, 12)), ((2, 1, 3, 9, 5), (1, 4, 3, 5, 7))]:
        ad, bd = np.array(ad, np.uint64), np.array(bd, np.uint64)
        cd = [int(max(a, b)) for a, b in zip(ad[:-2], bd[:-2])] + [int(ad[-2]), int(bd[-1])]
        a = rng.standard_normal(int(np.prod(ad))).astype(np.float32)
        b = rng.standard_normal(int(np.prod(bd))).astype(np.float32)
        dc = rng.standard_normal(int(np.prod(cd))).astype(np.float32)
        c = np.empty(int(np.prod(cd)), np.float32)
        da = np.empty_like(a)
        db = np.empty_like(b)
        rc = ref.ref_matmul_f32(len(ad), ad, bd, a, b, fptr(dc), fptr(c), fptr(da), fptr(db))
        assert rc == 0
        pre = f"mm{idx}_"
        out[pre + "adims"], out[pre + "bdims"] = ad, bd
        out[pre + "a"], out[pre + "b"], out[pre + "dc"] = a, b, dc
        out[pre + "c"], out[pre + "da"], out[pre + "db"] = c, da, db
        idx += 1
    out["mm_count"] = np.array(idx)

    # Conv2d forward, weight gradient, data gradient; Hout*Wout and Cin*kh*kw below 16 (see above).
    idx = 0
    for (N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw) in [
            (2, 1, 3, 5, 4, 3, 3, 1, 1, 1, 1),      # 3x3 s1 p1: 3x5 out, K=9
            (3, 2, 4, 6, 5, 2, 2, 0, 0, 1, 1),      # no pad: 3x5 out, K=8
            (2, 1, 5, 7, 6, 3, 2, 1, 1, 2, 2),      # stride 2, kh != kw: 3x4 out, K=6
            (2, 3, 5, 5, 3, 5, 1, 2, 0, 1, 2),      # 5x1 kernel, mixed pad/stride: 5x3 out, K=15
            (1, 1, 7, 7, 2, 3, 3, 0, 0, 2, 2)]:     # stride 2 no pad: 3x3 out
        Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
        assert Ho * Wo < 16 and Cin * kh * kw < 16, (Ho, Wo, Cin * kh * kw)
        x = rng.standard_normal(N * Cin * H * W).astype(np.float32)
        w = (rng.standard_normal(Cout * Cin * kh * kw) * 0.3).astype(np.float32)
        dy = rng.standard_normal(N * Cout * Ho * Wo).astype(np.float32)
        y = np.empty(N * Cout * Ho * Wo, np.float32)
        dw = np.empty_like(w)
        dx = np.empty_like(x)
        rc = ref.ref_conv2d_f32(N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, x, w, fptr(dy), fptr(y), fptr(dw), fptr(dx))
        assert rc == 0
        pre = f"cv{idx}_"
        out[pre + "geo"] = np.array([N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw], np.int64)
        out[pre + "x"], out[pre + "w"], out[pre + "dy"] = x, w, dy
        out[pre + "y"], out[pre + "dw"], out[pre + "dx"] = y, dw, dx
        idx += 1
    out["conv_count"] = np.array(idx)
    np.savez_compressed(os.path.join(HERE, "layer_cases.npz"), **out)
    print("layer_cases ok")


def conv2dq_cases():
    """The compiled lten::Conv2d_q forward (no bias), including the 1 -> 10 channel 5x5 layer of l-ten's quantized
    MNIST network (tests/nn_tests.cpp:625), padded / strided / multi-channel windows and zero points that make
    every correction term non-zero."""
    rng = np.random.default_rng(77)
    geos = [(2, 1, 28, 28, 10, 5, 5, 0, 0, 1, 1), (3, 3, 9, 11, 4, 3, 3, 1, 1, 1, 1), (1, 2, 10, 7, 5, 3, 2, 0, 1, 2, 1),
            (2, 4, 6, 6, 3, 1, 1, 0, 0, 1, 1), (1, 8, 12, 12, 6, 3, 3, 2, 2, 1, 1), (2, 1, 9, 140, 33, 3, 3, 1, 1, 1, 1)]
    qps = [([1 / 255, 0.01, 0.05], [0, 128, 128]), ([0.02, 0.013, 0.9], [17, 250, 100]), ([0.5, 0.5, 0.1], [128, 128, 0])]
    out, idx = {}, 0
    for geo in geos:
        N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
        x = rng.integers(0, 256, (N, Cin, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (Cout, Cin, kh, kw), dtype=np.uint8)
        for sc, zp in qps:
            pre = f"q{idx}_"
            out[pre + "geo"] = np.array(geo, np.int64)
            out[pre + "x"], out[pre + "w"] = x, w
            out[pre + "scales"], out[pre + "zps"] = np.array(sc, np.float32), np.array(zp, np.uint8)
            out[pre + "y"] = ob.ref_conv2dq_forward(geo, x, w, sc, zp)
            idx += 1
    out["count"] = np.array(idx)
    np.savez_compressed(os.path.join(HERE, "conv2dq_cases.npz"), **out)
    print("conv2dq_cases", idx)


def mlp_step_case():
    """One training step of the compiled l-ten network FullyConnected(+bias) -> relu -> FullyConnected -> relu ->
    FullyConnected -> log_softmax -> nll_loss.  Every GEMM dimension stays below 16 (the compiled cpu_gemm's AVX
    block needs 32-byte aligned outputs from 16 columns on)."""
    rng = np.random.default_rng(31)
    sizes, B = [13, 12, 9, 10], 6
    X = rng.random((B, sizes[0])).astype(np.float32)
    Ws = [(rng.standard_normal((sizes[i + 1], sizes[i])) * 0.3).astype(np.float32) for i in range(3)]
    bs = [(rng.standard_normal(sizes[i + 1]) * 0.3).astype(np.float32) for i in range(3)]
    T = np.eye(10, dtype=np.float32)[rng.integers(0, 10, B)]
    # l-ten's threaded cpu_gemm multiplies a fresh output buffer by beta = 0 (l-ten/math_fns.cpp:1168-1171), so a NaN
    # that happens to sit in that uninitialised memory survives: repeat until the run is clean
    for attempt in range(50):
        r = ob.mlp_step(X, Ws, bs, T, use_ref=True)
        if all(np.isfinite(a).all() for a in [r["logp"], r["dX"]] + r["dW"] + r["db"]):
            break
    else:
        raise RuntimeError("no NaN-free run of the compiled network")
    out = {"X": X, "T": T, "loss": np.float32(r["loss"]), "logp": r["logp"], "dX": r["dX"]}
    for l in range(3):
        out[f"W{l}"], out[f"b{l}"], out[f"dW{l}"], out[f"db{l}"] = Ws[l], bs[l], r["dW"][l], r["db"][l]
    np.savez_compressed(os.path.join(HERE, "mlp_step_case.npz"), **out)
    print("mlp_step_case loss", r["loss"])


def quant_inputs():
    """Values that exercise the helpers' corners: ties at .5 after the scale, both clamps, zeros of both signs,
    infinities, NaN, magnitudes beyond int range."""
    rng = np.random.default_rng(55)
    special = np.array([0.0, -0.0, 0.5, -0.5, 1.5, 2.5, -1.5, 127.5, 128.5, 254.5, 255.5, 1e-30, -1e-30, 1e9, -1e9, 3e9, -3e9,
                        2147483520.0, 2147483648.0, -2147483648.0, np.inf, -np.inf, np.nan, 1e38, -1e38], np.float32)
    return np.concatenate([special, (rng.standard_normal(3000) * 3).astype(np.float32),
                           (rng.integers(-600, 600, 500) * 0.25).astype(np.float32),
                           (rng.standard_normal(200) * 1e10).astype(np.float32)])


def quant_cases():
    """Quantize (uint8 and int), Dequantize, GetMinMax and ComputeQuantizationParams of the compiled l-ten."""
    data = quant_inputs()
    out = {"data": data}
    qps = [(0.5, 0), (0.25, 128), (1.0, 255), (0.0123, 17), (3.7, 200), (1e-3, 1)]
    out["qps"] = np.array(qps, np.float64)
    r = ob.ref()
    for i, (sc, zp) in enumerate(qps):
        q8, q32 = np.empty(data.size, np.uint8), np.empty(data.size, np.int32)
        r.ref_quantize_u8(data, q8, data.size, sc, zp)
        r.ref_quantize_i32(data, q32, data.size, sc, zp)
        codes = np.arange(256, dtype=np.uint8)
        dq = np.empty(256, np.float32)
        r.ref_dequantize_u8(dq, codes, 256, sc, zp)
        out[f"q8_{i}"], out[f"q32_{i}"], out[f"dq_{i}"] = q8, q32, dq
    ranges = [(-1.0, 1.0), (0.0, 6.0), (-3.5, 0.0), (0.2, 0.9), (-7.25, 12.5), (-1e-3, 2e-3)]
    res = []
    for lo, hi in ranges:
        sc, zp = C.c_float(), C.c_uint8()
        r.ref_compute_qparams(lo, hi, C.byref(sc), C.byref(zp))
        res.append((lo, hi, sc.value, zp.value))
    out["qparam_cases"] = np.array(res, np.float64)
    finite = data[np.isfinite(data)]
    lo, hi = C.c_float(), C.c_float()
    r.ref_min_max(finite, finite.size, C.byref(lo), C.byref(hi))
    out["minmax"] = np.array([lo.value, hi.value], np.float32)
    np.savez_compressed(os.path.join(HERE, "quant_cases.npz"), **out)
    print("quant_cases", data.size)


def optimizer_cases():
    """Five steps of the compiled SGDOptimizer and AdamOptimizer on one parameter tensor with a fixed gradient."""
    rng = np.random.default_rng(66)
    n = 1000
    w0 = rng.standard_normal(n).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    g[:10] = 0.0
    out = {"w0": w0, "g": g}
    for name, kind, p in (("sgd", 0, [0.9, 0.0005, 0.01]), ("sgd_plain", 0, [0.0, 0.0, 0.1]), ("adam", 1, [0.01, 0.9, 0.999]),
                          ("adam_fast", 1, [0.1, 0.5, 0.9])):
        w = w0.copy()
        assert ob.ref().ref_optimizer_steps(kind, n, 5, np.array(p, np.float32), w, g) == 0
        out[name + "_p"], out[name + "_w"] = np.array(p, np.float32), w
    np.savez_compressed(os.path.join(HERE, "optimizer_cases.npz"), **out)
    print("optimizer_cases ok")


if __name__ == "__main__":
    requant_sweep()
    qmm_cases()
    cfg1_expected()
    sgemm_cases()
    layer_cases()
    conv2dq_cases()
    mlp_step_case()
    quant_cases()
    optimizer_cases()
