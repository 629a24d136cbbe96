"""Seeded sweeps of random shapes through the C ABI: whatever route the dispatch rules pick for a shape (tile sizes, split
reductions, weight-streaming kernels, column matrices), the result must not depend on it.  Operands are small integers, so
every fp32 sum is exact in any order and the comparison is bit for bit; the int8 path is bit-exact by construction."""
import numpy as np
import pytest

from conftest import exact_acc, requant_numpy

pytestmark = pytest.mark.gpu

DIMS = [1, 2, 3, 4, 5, 8, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 96, 100, 127, 128, 129, 192, 196, 200, 255, 256, 257, 320, 384, 500, 512, 513,
        640, 768, 1000, 1024, 1025, 1536, 2048, 2304, 3000, 4096, 4100, 6272, 8192, 8200, 12288, 16384, 20000, 20011, 25088, 32000, 34815, 100000]
DIMS_ALIGNED = [d for d in DIMS if d % 4 == 0] + [12, 20, 160, 1280, 3072, 34812, 65536 + 2044]


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_sgemm_random_shapes_exact(gpu, seed):
    """lten_hip_sgemm / _strided_batched in random layouts, leading dimensions, alpha and beta (NaN in C under beta = 0), and the
    same product through lten_hip_fc_forward_f32 with a bias; even seeds draw sizes that are multiples of four (the routes
    with 16-byte loads), odd seeds any size."""
    rng = np.random.default_rng(seed)
    pool = DIMS_ALIGNED if seed % 2 == 0 else DIMS
    D, l = gpu.DeviceBuffer, gpu.lib()
    for it in range(160):
        while True:
            M, N, K = (int(rng.choice(pool)) for _ in range(3))
            batch = 1 if rng.random() < 0.75 else int(rng.choice([2, 3, 8, 12, 24]))
            if max(M * K, K * N, M * N) * batch <= 2e7 and M * N * K * batch <= 1.5e9:
                break
        tA, tB = int(rng.random() < 0.4), int(rng.random() < 0.45)
        pads = [0, 0, 0, 4, 8] if seed % 2 == 0 else [0, 0, 0, 4, 3, 8]
        lda, ldb, ldc = (M if tA else K) + int(rng.choice(pads)), (K if tB else N) + int(rng.choice(pads)), N + int(rng.choice(pads))
        alpha, beta = float(rng.choice([1.0, 2.0, -1.0, 0.5])), float(rng.choice([0.0, 0.0, 1.0, -1.0]))
        a = rng.integers(-3, 4, (batch, M, K)).astype(np.float32)
        b = rng.integers(-3, 4, (batch, K, N)).astype(np.float32)
        c0 = rng.integers(-9, 10, (batch, M, N)).astype(np.float32)
        want = (alpha * (a.astype(np.float64) @ b.astype(np.float64)) + beta * c0).astype(np.float32)
        ra, rb = (K if tA else M), (N if tB else K)
        As = np.zeros((batch, ra, lda), np.float32)
        As[:, :, :(M if tA else K)] = a.transpose(0, 2, 1) if tA else a
        Bs = np.zeros((batch, rb, ldb), np.float32)
        Bs[:, :, :(K if tB else N)] = b.transpose(0, 2, 1) if tB else b
        Cs = np.full((batch, M, ldc), 7.0, np.float32)
        Cs[:, :, :N] = np.nan if beta == 0.0 and rng.random() < 0.3 else c0
        dA, dB, dC = D.from_numpy(As), D.from_numpy(Bs), D.from_numpy(Cs)
        case = (seed, it, tA, tB, M, N, K, batch, lda, ldb, ldc, alpha, beta)
        if batch == 1:
            gpu.check(l.lten_hip_sgemm(tA, tB, M, N, K, alpha, dA.ptr, lda, dB.ptr, ldb, beta, dC.ptr, ldc))
        else:
            gpu.check(l.lten_hip_sgemm_strided_batched(tA, tB, M, N, K, alpha, dA.ptr, lda, ra * lda, dB.ptr, ldb, rb * ldb, beta, dC.ptr, ldc,
                                                       M * ldc, batch))
        got = dC.numpy(np.float32, Cs.shape)
        assert np.array_equal(got[:, :, :N], want), (case, gpu.last_kernel())
        assert (got[:, :, N:] == 7.0).all(), (case, gpu.last_kernel())
        if batch == 1 and not tA and rng.random() < 0.4:
            X, W = np.ascontiguousarray(a[0]), np.ascontiguousarray(b[0].T)
            bias = rng.integers(-9, 10, N).astype(np.float32)
            dX, dW, dBias, dY = D.from_numpy(X), D.from_numpy(W), D.from_numpy(bias), D(4 * M * N)
            gpu.check(l.lten_hip_fc_forward_f32(M, K, N, dX.ptr, dW.ptr, dBias.ptr, dY.ptr))
            wantf = (a[0].astype(np.float64) @ b[0].astype(np.float64) + bias[None, :]).astype(np.float32)
            assert np.array_equal(dY.numpy(np.float32, (M, N)), wantf), (case, gpu.last_kernel())


@pytest.mark.parametrize("seed", [21, 22])
def test_fcq_random_shapes_bit_exact(gpu, seed):
    """FullyConnected_q forward on l-ten's uint8 weights, on prepared weights and through the entry point that allocates
    nothing, random zero points and bias, and the other transpose modes of quantized_matmul on the smaller cases: the exact
    accumulator (every product and sum fits a double) requantized by l-ten's five steps."""
    rng = np.random.default_rng(seed)
    Ms = [1, 2, 3, 4, 7, 8, 15, 16, 17, 24, 31, 32, 33, 48, 63, 64, 65, 100, 127, 128, 129, 192, 255, 256, 257, 384, 500, 512, 1000, 1024, 2048]
    Ns = [1, 2, 5, 10, 16, 17, 50, 64, 100, 128, 250, 256, 500, 512, 1000, 1001, 1024, 2000, 2048, 4096]
    Ks = [1, 3, 16, 33, 64, 100, 127, 128, 256, 300, 512, 784, 1000, 1024, 2048, 4000, 4096, 5760, 8192, 9216, 12288, 16384, 16392, 16400, 20003, 25088, 32768]
    D, l = gpu.DeviceBuffer, gpu.lib()
    for it in range(120):
        while True:
            M, N, K = int(rng.choice(Ms)), int(rng.choice(Ns)), int(rng.choice(Ks))
            if M * N * K <= 6e9 and max(M * K, N * K) <= 7e7 and M * N <= 5e6:
                break
        zp = rng.integers(0, 256, 3).astype(np.uint8)
        if rng.random() < 0.3:
            zp[:] = 128
        if rng.random() < 0.2:
            zp[0] = 0
        sc = np.array([0.02, 0.01, 0.02 * 0.01 * np.sqrt(K) * 40], np.float32)
        A = rng.integers(0, 256, (M, K), dtype=np.uint8)
        B = rng.integers(0, 256, (N, K), dtype=np.uint8)
        bias = rng.integers(-100000, 100000, N).astype(np.int32) if rng.random() < 0.6 else None
        acc = exact_acc(A, B, zp[0], zp[1]) + (bias[None, :].astype(np.int64) if bias is not None else 0)
        mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
        want = requant_numpy(acc, mult, zp[2])
        case = (seed, it, M, N, K, zp.tolist(), bias is not None)
        qp = gpu.qparams3(sc, zp)
        dX, dW, dY, ws = D.from_numpy(A), D.from_numpy(B), D(M * N), D(4 * (M + N))
        db = D.from_numpy(bias) if bias is not None else None
        gpu.check(l.lten_hip_fcq_forward(1, M, K, N, dX.ptr, dW.ptr, db.ptr if db else None, qp, dY.ptr, ws.ptr))
        assert np.array_equal(dY.numpy(np.uint8, (M, N)), want), (case, "raw", gpu.last_kernel())
        Kp = (K + 15) // 16 * 16
        dWp, dS, dY2 = D(N * Kp + 16), D(4 * N + 16), D(M * N)
        gpu.check(l.lten_hip_fcq_prepare_weights(dW.ptr, dWp.ptr, N, K, dS.ptr))
        gpu.check(l.lten_hip_fcq_forward_prepared(1, M, K, N, dX.ptr, dWp.ptr, dS.ptr, db.ptr if db else None, qp, dY2.ptr, ws.ptr))
        assert np.array_equal(dY2.numpy(np.uint8, (M, N)), want), (case, "prepared", gpu.last_kernel())
        dY3 = D(M * N)
        if l.lten_hip_fcq_forward_static(1, M, K, N, dX.ptr, dW.ptr, db.ptr if db else None, qp, dY3.ptr) == 0:   # (declines what exceeds its array)
            assert np.array_equal(dY3.numpy(np.uint8, (M, N)), want), (case, "static", gpu.last_kernel())
        if M * K + N * K <= 2e6:
            for tA, tB in ((0, 0), (1, 1), (1, 0)):
                As = np.ascontiguousarray(A.T) if tA else A
                Bs = B if tB else np.ascontiguousarray(B.T)
                got, _ = gpu.qgemm_host(As, Bs, sc, zp, tA=bool(tA), tB=bool(tB), bias=bias, M=M, N=N, K=K)
                assert np.array_equal(got, want), (case, tA, tB, gpu.last_kernel())


@pytest.mark.parametrize("seed", [31, 32])
def test_conv2d_random_geometries_exact(gpu, ob, seed):
    """Conv2d forward (with and without bias), weight gradient and data gradient on random geometries against the oracle;
    even seeds draw network-like layers (square maps, 1 x 1 / 3 x 3 / 5 x 5 windows, wide channels), odd seeds anything."""
    rng = np.random.default_rng(seed)
    D, l = gpu.DeviceBuffer, gpu.lib()
    for it in range(60):
        while True:
            N = int(rng.choice([1, 1, 2, 3, 4, 8, 16, 32, 64]))
            Cin = int(rng.choice([1, 2, 3, 4, 5, 8, 10, 16, 20, 24, 32, 48, 64, 96, 128, 256]))
            Cout = int(rng.choice([1, 2, 3, 4, 6, 8, 10, 16, 20, 32, 33, 48, 64, 96, 128, 256]))
            H = int(rng.choice([4, 5, 7, 8, 12, 13, 14, 16, 24, 28, 29, 32, 48, 56, 64]))
            W = H if rng.random() < 0.6 else int(rng.choice([4, 6, 7, 8, 12, 14, 16, 20, 28, 30, 32, 50, 56, 64, 100]))
            kh = int(rng.choice([1, 1, 2, 3, 3, 3, 4, 5, 5, 7]))
            kw = kh if rng.random() < 0.8 else int(rng.choice([1, 2, 3, 4, 5]))
            ph = int(rng.integers(0, kh)) if rng.random() < 0.7 else 0
            pw = int(rng.integers(0, kw)) if rng.random() < 0.7 else 0
            sh = int(rng.choice([1, 1, 1, 2, 2, 3]))
            sw = sh if rng.random() < 0.85 else int(rng.choice([1, 2]))
            if seed % 2 == 0:
                Cin, Cout = int(rng.choice([3, 8, 16, 32, 64, 96, 128, 256, 512])), int(rng.choice([16, 32, 64, 96, 128, 256, 512]))
                H = W = int(rng.choice([7, 8, 13, 14, 16, 28, 32, 56]))
                kh = kw = int(rng.choice([1, 3, 3, 3, 5]))
                ph = pw = kh // 2 if rng.random() < 0.85 else 0
                sh = sw = int(rng.choice([1, 1, 1, 2]))
            if H + 2 * ph < kh or W + 2 * pw < kw:
                continue
            Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
            if 2.0 * N * Cout * Ho * Wo * Cin * kh * kw <= 4e8 and N * Cin * H * W <= 4e6 and N * Cout * Ho * Wo <= 4e6:
                break
        geo = (N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw)
        x = rng.integers(-2, 3, (N, Cin, H, W)).astype(np.float32)
        w = rng.integers(-2, 3, (Cout, Cin, kh, kw)).astype(np.float32)
        dy = rng.integers(-2, 3, (N, Cout, Ho, Wo)).astype(np.float32)
        bias = rng.integers(-9, 10, Cout).astype(np.float32) if rng.random() < 0.5 else None
        col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
        want_y, want_dw, want_dx = np.empty_like(dy), np.empty_like(w), np.empty_like(x)
        o = ob.oracle()
        o.oracle_conv2d_forward(*geo, x.reshape(-1), w.reshape(-1), want_y.reshape(-1), col)
        if bias is not None:
            want_y += bias[None, :, None, None]
        o.oracle_conv2d_wgrad(*geo, x.reshape(-1), dy.reshape(-1), want_dw.reshape(-1), col)
        o.oracle_conv2d_dgrad(*geo, w.reshape(-1), dy.reshape(-1), want_dx.reshape(-1), col)
        dX, dW, dDY, dY = D.from_numpy(x), D.from_numpy(w), D.from_numpy(dy), D(dy.nbytes)
        dB = D.from_numpy(bias) if bias is not None else None
        gpu.check(l.lten_hip_conv2d_forward_f32(*geo, dX.ptr, dW.ptr, dB.ptr if dB else None, dY.ptr))
        assert np.array_equal(dY.numpy(np.float32, dy.shape), want_y), (seed, it, geo, "forward", gpu.last_kernel())
        ws, dDW = D(max(int(l.lten_hip_conv2d_wgrad_workspace_bytes(*geo)), 4)), D(w.nbytes)
        gpu.check(l.lten_hip_conv2d_wgrad_f32(*geo, dX.ptr, dDY.ptr, dDW.ptr, ws.ptr))
        assert np.array_equal(dDW.numpy(np.float32, w.shape), want_dw), (seed, it, geo, "wgrad", gpu.last_kernel())
        wsd, dDX = D(max(int(l.lten_hip_conv2d_dgrad_workspace_bytes(*geo)), 4)), D(x.nbytes)
        gpu.check(l.lten_hip_conv2d_dgrad_f32(*geo, dW.ptr, dDY.ptr, dDX.ptr, wsd.ptr))
        assert np.array_equal(dDX.numpy(np.float32, x.shape), want_dx), (seed, it, geo, "dgrad", gpu.last_kernel())


@pytest.mark.parametrize("seed", [41, 42])
def test_conv2dq_random_geometries_bit_exact(gpu, ob, seed):
    """Conv2d_q forward on random geometries, zero points and (l-ten's per-pixel) bias: accumulators and requantized outputs
    bit for bit against the oracle; even seeds draw network-like layers, odd seeds anything."""
    rng = np.random.default_rng(seed)
    for it in range(60):
        while True:
            N = int(rng.choice([1, 1, 2, 3, 4, 8, 16, 32]))
            Cin = int(rng.choice([1, 2, 3, 4, 5, 8, 10, 16, 20, 24, 32, 48, 64, 96, 128, 256]))
            Cout = int(rng.choice([1, 2, 3, 4, 6, 8, 10, 16, 20, 32, 33, 48, 64, 96, 128, 256]))
            H = int(rng.choice([4, 5, 7, 8, 12, 13, 14, 16, 24, 28, 29, 32, 48, 56, 64]))
            W = H if rng.random() < 0.6 else int(rng.choice([4, 6, 7, 8, 12, 14, 16, 20, 28, 30, 32, 50, 56, 64, 100]))
            kh = int(rng.choice([1, 1, 2, 3, 3, 3, 4, 5, 5, 7]))
            kw = kh if rng.random() < 0.8 else int(rng.choice([1, 2, 3, 4, 5]))
            ph = int(rng.integers(0, kh)) if rng.random() < 0.7 else 0
            pw = int(rng.integers(0, kw)) if rng.random() < 0.7 else 0
            sh = int(rng.choice([1, 1, 1, 2, 2, 3]))
            sw = sh if rng.random() < 0.85 else int(rng.choice([1, 2]))
            if seed % 2 == 0:
                Cin, Cout = int(rng.choice([3, 8, 16, 32, 64, 128, 256, 512, 1024])), int(rng.choice([16, 32, 64, 128, 256, 512]))
                H = W = int(rng.choice([7, 8, 14, 16, 28, 32, 56]))
                kh = kw = int(rng.choice([1, 3, 3, 3, 5]))
                ph = pw = kh // 2 if rng.random() < 0.85 else 0
                sh = sw = int(rng.choice([1, 1, 1, 2]))
            if H + 2 * ph < kh or W + 2 * pw < kw:
                continue
            Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
            if 1.0 * N * Cout * Ho * Wo * Cin * kh * kw <= 1e9 and N * Cin * H * W <= 4e6 and N * Cout * Ho * Wo <= 4e6:
                break
        geo = (N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw)
        x = rng.integers(0, 256, (N, Cin, H, W), dtype=np.uint8)
        w = rng.integers(0, 256, (Cout, Cin, kh, kw), dtype=np.uint8)
        zp = rng.integers(0, 256, 3).astype(np.uint8)
        if rng.random() < 0.3:
            zp[:] = 128
        if rng.random() < 0.2:
            zp[0] = 0
        sc = [0.02, 0.01, 0.02 * 0.01 * float(np.sqrt(Cin * kh * kw)) * 40]
        bias = rng.integers(-9999, 9999, Ho * Wo).astype(np.int32) if rng.random() < 0.5 else None
        want_y, want_acc = ob.conv2dq_forward(geo, x, w, sc, zp, bias=bias)
        y, acc = gpu.conv2dq_host(geo, x, w, sc, zp, bias=bias, want_acc=True)
        case = (seed, it, geo, zp.tolist(), bias is not None, gpu.last_kernel())
        assert np.array_equal(acc, want_acc), case
        assert np.array_equal(y, want_y), case


@pytest.mark.parametrize("seed", [51, 52])
def test_fc_backward_random_shapes_exact(gpu, seed):
    """FullyConnected backward (dX = dY W, dW = dY^T X, db += column sums of dY), plain and with the relu's backward pass folded
    in, over random batch sizes and layer widths (the paired launch, the weight-streaming kernels, split reductions, rank-1
    updates at batch 1); any of the three outputs may be left out."""
    rng = np.random.default_rng(seed)
    D, l = gpu.DeviceBuffer, gpu.lib()
    Ms = [1, 2, 3, 4, 8, 15, 16, 17, 32, 33, 64, 100, 128, 256, 257, 512, 1000, 2048, 4096, 16384]
    widths = [1, 2, 5, 10, 16, 50, 64, 100, 128, 250, 256, 500, 512, 784, 1000, 1024, 2048, 4096, 5760, 8192, 25088, 32000]
    if seed % 2 == 0:
        widths = [w for w in widths if w % 4 == 0]
    for it in range(70):
        while True:
            M, n_in, n_out = int(rng.choice(Ms)), int(rng.choice(widths)), int(rng.choice(widths))
            if max(M * n_in, M * n_out, n_in * n_out) <= 2e7 and M * n_in * n_out <= 1.5e9:
                break
        X = rng.integers(-3, 4, (M, n_in)).astype(np.float32)
        W = rng.integers(-3, 4, (n_out, n_in)).astype(np.float32)
        dY = rng.integers(-3, 4, (M, n_out)).astype(np.float32)
        db0 = rng.integers(-9, 10, n_out).astype(np.float32)
        relu_in = rng.integers(-2, 3, (M, n_in)).astype(np.float32) if rng.random() < 0.4 else None
        want_dx = (dY.astype(np.float64) @ W.astype(np.float64)).astype(np.float32)
        if relu_in is not None:
            want_dx = np.where(relu_in > 0, want_dx, np.float32(0.0))
        want_dw = (dY.astype(np.float64).T @ X.astype(np.float64)).astype(np.float32)
        want_db = (db0 + dY.astype(np.float64).sum(axis=0)).astype(np.float32)
        wants = [rng.random() < 0.85 for _ in range(3)]
        dXb, dWb, dDY, dR = D.from_numpy(X), D.from_numpy(W), D.from_numpy(dY), D.from_numpy(relu_in) if relu_in is not None else None
        dDX, dDW, dDB = D(X.nbytes) if wants[0] else None, D(W.nbytes) if wants[1] else None, D.from_numpy(db0) if wants[2] else None
        args = (dDX.ptr if dDX else None, dDW.ptr if dDW else None, dDB.ptr if dDB else None)
        if relu_in is None:
            gpu.check(l.lten_hip_fc_backward_f32(M, n_in, n_out, dXb.ptr, dWb.ptr, dDY.ptr, *args))
        else:
            gpu.check(l.lten_hip_fc_backward_relu_f32(M, n_in, n_out, dXb.ptr, dWb.ptr, dDY.ptr, dR.ptr, *args))
        case = (seed, it, M, n_in, n_out, relu_in is not None, wants, gpu.last_kernel())
        if dDX:
            assert np.array_equal(dDX.numpy(np.float32, X.shape), want_dx), ("dX", case)
        if dDW:
            assert np.array_equal(dDW.numpy(np.float32, W.shape), want_dw), ("dW", case)
        if dDB:
            assert np.array_equal(dDB.numpy(np.float32, (n_out,)), want_db), ("db", case)
