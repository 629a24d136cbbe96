"""GPU parity tests of the fp32 GEMM path through the C ABI.  Tolerance (north star): max relative
error 1e-4, measured as max |got - want| / max(|want|, rms(want)) (conftest.rel_err); integer-valued
inputs must come out exactly (any summation order is exact), which checks layouts and transposes bit for bit."""
import json

import numpy as np
import pytest

from conftest import golden_path, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4


def gpu_sgemm(gpu, tA, tB, M, N, K, alpha, A, lda, B, ldb, beta, C0, ldc, tile=0):
    dA, dB, dC = gpu.DeviceBuffer.from_numpy(A), gpu.DeviceBuffer.from_numpy(B), gpu.DeviceBuffer.from_numpy(C0)
    gpu.set_option("sgemm_tile", tile)
    try:
        gpu.sgemm(tA, tB, M, N, K, alpha, dA, lda, dB, ldb, beta, dC, ldc)
    finally:
        gpu.set_option("sgemm_tile", 0)
    return dC.numpy(np.float32, C0.shape)


def test_sgemm_golden_cases(gpu):
    g = np.load(golden_path("sgemm_cases.npz"))
    for i in range(int(g["count"])):
        pre = f"c{i}_"
        M, N, K, tA, tB = (int(v) for v in g[pre + "dims"])
        alpha, beta = (float(v) for v in g[pre + "ab"])
        got = gpu_sgemm(gpu, tA, tB, M, N, K, alpha, g[pre + "A"], M if tA else K, g[pre + "B"], K if tB else N, beta,
                        g[pre + "C0"], N)
        assert rel_err(got, g[pre + "C"]) < TOL, (i, M, N, K, tA, tB, alpha, beta, gpu.last_kernel())


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4])  # 1-3: LDS-tiled kernels, 4: direct (intra-workgroup split-K) kernel
@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_integer_valued_exact_with_leading_dims(gpu, tile, tA, tB):
    rng = np.random.default_rng(40 + 2 * tA + tB + 10 * tile)
    M, N, K = 77, 139, 101
    A = rng.integers(-8, 9, (M, K)).astype(np.float32)
    B = rng.integers(-8, 9, (K, N)).astype(np.float32)
    want = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)
    lda, ldb, ldc = (M if tA else K) + 3, (K if tB else N) + 5, N + 2
    As = np.zeros(((K if tA else M), lda), np.float32)
    As[:, :(M if tA else K)] = A.T if tA else A
    Bs = np.zeros(((N if tB else K), ldb), np.float32)
    Bs[:, :(K if tB else N)] = B.T if tB else B
    C0 = np.full((M, ldc), 7.0, np.float32)
    got = gpu_sgemm(gpu, tA, tB, M, N, K, 1.0, As, lda, Bs, ldb, 0.0, C0, ldc, tile)
    assert np.array_equal(got[:, :N], want)
    assert (got[:, N:] == 7.0).all()
    got2 = gpu_sgemm(gpu, tA, tB, M, N, K, 2.0, As, lda, Bs, ldb, -1.0, got, ldc, tile)
    assert np.array_equal(got2[:, :N], want)


@pytest.mark.parametrize("tA,tB,M,N,K", [(1, 0, 128, 128, 16384), (1, 0, 10, 32, 20011), (0, 0, 64, 200, 8200), (0, 1, 100, 37, 4099 + 2),
                                          (1, 1, 256, 256, 4096), (1, 0, 64, 64, 65536),
                                          (1, 0, 16, 16, 34815), (1, 0, 10, 32, 100000)])   # 64 slices of 512 leave 2047, which is split itself: its partial sums must not land on the first split's
def test_long_reduction_into_a_small_output_is_split(gpu, tA, tB, M, N, K):
    """The weight gradient of a small layer over a large batch: K is cut into slices that run as a batch into partial
    matrices, added in slice order by a second launch.  Integer-valued operands come out exactly whatever the order;
    alpha, beta and padded leading dimensions as in every other route; two runs give the same bits."""
    rng = np.random.default_rng(M + N + K + 2 * tA + tB)
    A = rng.integers(-4, 5, (M, K)).astype(np.float32)
    B = rng.integers(-4, 5, (K, N)).astype(np.float32)
    want = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)
    lda, ldb, ldc = (M if tA else K) + 4, (K if tB else N) + 8, N + 3
    As = np.zeros(((K if tA else M), lda), np.float32)
    As[:, :(M if tA else K)] = A.T if tA else A
    Bs = np.zeros(((N if tB else K), ldb), np.float32)
    Bs[:, :(K if tB else N)] = B.T if tB else B
    C0 = np.full((M, ldc), 7.0, np.float32)
    got = gpu_sgemm(gpu, tA, tB, M, N, K, 1.0, As, lda, Bs, ldb, 0.0, C0, ldc)
    assert gpu.last_kernel() == "sgemm_split_k", gpu.last_kernel()
    assert np.array_equal(got[:, :N], want)
    assert (got[:, N:] == 7.0).all()
    got2 = gpu_sgemm(gpu, tA, tB, M, N, K, 2.0, As, lda, Bs, ldb, -1.0, got, ldc)
    assert np.array_equal(got2[:, :N], want)
    # real-valued operands: within the tolerance of every other route, and the same bits on a second run
    Ar = rng.standard_normal(As.shape).astype(np.float32)
    Br = rng.standard_normal(Bs.shape).astype(np.float32)
    a64 = (Ar[:, :M].T if tA else Ar[:, :K]).astype(np.float64)
    b64 = (Br[:, :K].T if tB else Br[:, :N]).astype(np.float64)
    r1 = gpu_sgemm(gpu, tA, tB, M, N, K, 1.0, Ar, lda, Br, ldb, 0.0, C0, ldc)
    r2 = gpu_sgemm(gpu, tA, tB, M, N, K, 1.0, Ar, lda, Br, ldb, 0.0, C0, ldc)
    assert np.array_equal(r1, r2)
    assert rel_err(r1[:, :N], (a64 @ b64).astype(np.float32)) < TOL


@pytest.mark.parametrize("K", [12, 24, 32, 52])   # (up to 8 rows: the stream over C, tested below)
def test_short_reduction_into_a_large_output_on_the_large_tiles(gpu, K):
    """The weight gradient of a wide layer at a small batch, dW = dY^T X with fewer than 64 rows to reduce over and 512 or more
    tiles of 128 x 128 to write: the operands are copied into 64 rows (the rest zero) for the direct-to-LDS tiles.
    Integer-valued operands come out exactly; alpha, beta and padded leading dimensions as in every other route."""
    M, N = 2048, 4096
    rng = np.random.default_rng(K)
    A = rng.integers(-4, 5, (K, M + 4)).astype(np.float32)   # stored [K][M], leading dimension M + 4
    B = rng.integers(-4, 5, (K, N + 8)).astype(np.float32)
    want = (A[:, :M].astype(np.int64).T @ B[:, :N].astype(np.int64)).astype(np.float32)
    C0 = np.full((M, N + 4), 7.0, np.float32)
    got = gpu_sgemm(gpu, 1, 0, M, N, K, 1.0, A, M + 4, B, N + 8, 0.0, C0, N + 4)
    assert gpu.last_kernel().startswith("sgemm_fast_128x128x32"), gpu.last_kernel()
    assert np.array_equal(got[:, :N], want)
    assert (got[:, N:] == 7.0).all()
    got2 = gpu_sgemm(gpu, 1, 0, M, N, K, 2.0, A, M + 4, B, N + 8, -1.0, got, N + 4)
    assert np.array_equal(got2[:, :N], want)


@pytest.mark.parametrize("tB,K", [(0, 12), (0, 50), (1, 9), (1, 33)])
def test_short_reduction_of_row_major_operands_into_a_large_output(gpu, tB, K):
    """A B and A B^T over 9 to 63 columns of A into 512 or more tiles of 128 x 128: the operands that are contiguous along K are
    copied into rows of 64 (zeros behind) for the direct-to-LDS tiles.  Odd row counts and padded leading dimensions;
    integer-valued operands, exact; alpha and beta."""
    M, N = 2051, 4100
    rng = np.random.default_rng(K + tB)
    A = rng.integers(-4, 5, (M, K + 3)).astype(np.float32)            # leading dimension K + 3
    B = rng.integers(-4, 5, (N, K + 5) if tB else (K, N + 8)).astype(np.float32)
    b = B[:, :K].T if tB else B[:, :N]
    want = (A[:, :K].astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    C0 = np.full((M, N + 4), 7.0, np.float32)
    got = gpu_sgemm(gpu, 0, tB, M, N, K, 1.0, A, K + 3, B, K + 5 if tB else N + 8, 0.0, C0, N + 4)
    assert gpu.last_kernel().startswith("sgemm_fast_128x128x32"), gpu.last_kernel()
    assert np.array_equal(got[:, :N], want)
    assert (got[:, N:] == 7.0).all()
    got2 = gpu_sgemm(gpu, 0, tB, M, N, K, 2.0, A, K + 3, B, K + 5 if tB else N + 8, -1.0, got, N + 4)
    assert np.array_equal(got2[:, :N], want)


@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_long_reduction_into_a_mid_size_output_is_split(gpu, tA, tB):
    """65 to 255 tiles of 64 x 64 under a reduction of 4096 or more: K is cut until the slices give the direct-to-LDS tiles
    about 512 workgroups, the partial matrices are added in slice order.  Integer-valued operands come out exactly; alpha,
    beta and padded leading dimensions as in every other route; FullyConnected's bias rides on the adding launch."""
    M, N, K = 320, 1280, 4096 + 64
    rng = np.random.default_rng(7 + 2 * tA + tB)
    A = rng.integers(-4, 5, (M, K)).astype(np.float32)
    B = rng.integers(-4, 5, (K, N)).astype(np.float32)
    want = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)
    lda, ldb, ldc = (M if tA else K) + 4, (K if tB else N) + 8, N + 4
    As = np.zeros(((K if tA else M), lda), np.float32)
    As[:, :(M if tA else K)] = A.T if tA else A
    Bs = np.zeros(((N if tB else K), ldb), np.float32)
    Bs[:, :(K if tB else N)] = B.T if tB else B
    C0 = np.full((M, ldc), 7.0, np.float32)
    got = gpu_sgemm(gpu, tA, tB, M, N, K, 1.0, As, lda, Bs, ldb, 0.0, C0, ldc)
    assert gpu.last_kernel() == "sgemm_split_k", gpu.last_kernel()
    assert np.array_equal(got[:, :N], want)
    assert (got[:, N:] == 7.0).all()
    got2 = gpu_sgemm(gpu, tA, tB, M, N, K, 2.0, As, lda, Bs, ldb, -1.0, got, ldc)
    assert np.array_equal(got2[:, :N], want)
    if not tA and tB:   # the same product as a FullyConnected forward pass with a bias
        D = gpu.DeviceBuffer
        X, W = np.ascontiguousarray(A), np.ascontiguousarray(B.T)
        b = rng.integers(-9, 10, N).astype(np.float32)
        dX, dW, dB, dY = D.from_numpy(X), D.from_numpy(W), D.from_numpy(b), D(4 * M * N)
        gpu.check(gpu.lib().lten_hip_fc_forward_f32(M, K, N, dX.ptr, dW.ptr, dB.ptr, dY.ptr))
        assert gpu.last_kernel() == "sgemm_split_k", gpu.last_kernel()
        assert np.array_equal(dY.numpy(np.float32, (M, N)), want + b[None, :])


@pytest.mark.parametrize("rows", [1, 8])
def test_fc_forward_of_few_rows_onto_few_outputs_over_a_long_reduction_is_split(gpu, rows):
    """A classifier behind a flattened feature map (1 x 25088 -> 1000): one workgroup per 16 outputs of the streaming NT
    kernel would leave most CUs idle, so the reduction of 8192 or more is cut into slices instead.  Integer-valued operands
    come out exactly, bias included; one more column group (1040 outputs at 8 rows is still under 128 groups) too."""
    K, N = 8192 + 64, 1000
    rng = np.random.default_rng(31 + rows)
    X = rng.integers(-4, 5, (rows, K)).astype(np.float32)
    W = rng.integers(-4, 5, (N, K)).astype(np.float32)
    b = rng.integers(-9, 10, N).astype(np.float32)
    want = (X.astype(np.float64) @ W.astype(np.float64).T).astype(np.float32) + b[None, :]
    D = gpu.DeviceBuffer
    dX, dW, dB, dY = D.from_numpy(X), D.from_numpy(W), D.from_numpy(b), D(4 * rows * N)
    gpu.check(gpu.lib().lten_hip_fc_forward_f32(rows, K, N, dX.ptr, dW.ptr, dB.ptr, dY.ptr))
    assert gpu.last_kernel() == "sgemm_split_k", gpu.last_kernel()
    assert np.array_equal(dY.numpy(np.float32, (rows, N)), want)


def test_beta_zero_overwrites_nan(gpu):
    A = np.ones((5, 3), np.float32)
    B = np.ones((3, 6), np.float32)
    got = gpu_sgemm(gpu, 0, 0, 5, 6, 3, 1.0, A, 3, B, 6, 0.0, np.full((5, 6), np.nan, np.float32), 6)
    assert np.array_equal(got, np.full((5, 6), 3.0, np.float32))


@pytest.mark.parametrize("shape", [(128, 1024, 784), (128, 1024, 1024), (128, 10, 1024)])
def test_cfg2_gemm_shapes_all_layouts(gpu, ob, shape):
    """The nine GEMMs of the MLP step: forward NT, data gradient NN, weight gradient TN."""
    M, N, K = shape  # forward: Y[M x N] = X[M x K] W[N x K]^T
    rng = np.random.default_rng(M + N + K)
    X = rng.uniform(0, 1, (M, K)).astype(np.float32)
    W = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    dY = rng.standard_normal((M, N)).astype(np.float32)
    for (tA, tB, m, n, k, A, B) in [(0, 1, M, N, K, X, W), (0, 0, M, K, N, dY, W), (1, 0, N, K, M, dY, X)]:
        lda, ldb = A.shape[1], B.shape[1]
        want = np.zeros((m, n), np.float32)
        ob.sgemm(tA, tB, m, n, k, 1.0, A, lda, B, ldb, 0.0, want, n, f64=True)
        got = gpu_sgemm(gpu, tA, tB, m, n, k, 1.0, A, lda, B, ldb, 0.0, np.zeros((m, n), np.float32), n)
        err = rel_err(got, want)
        print(f"  {'TN'[tA]}{'NT'[tB]} {m}x{n}x{k} via {gpu.last_kernel()}: max rel err {err:.2e}")
        assert err < TOL


@pytest.mark.parametrize("tile,name", [(4, "sgemm_staged"), (5, "sgemm_direct")])
def test_small_output_kernels_are_deterministic_and_repeatable(gpu, tile, name):
    """The small-output kernels (LDS-staged and direct operand loads) add their wavefronts' partial tiles in wavefront
    order: bitwise equal results run after run; all layouts, ragged M / N / K, beta, batches."""
    rng = np.random.default_rng(3)
    if True:
        M, N, K = 128, 1024, 1024   # the data-gradient product of a 1024-wide layer at batch 128 (NN)
        A = rng.standard_normal((M, K)).astype(np.float32)
        B = rng.standard_normal((K, N)).astype(np.float32)
        z = np.zeros((M, N), np.float32)
        first = gpu_sgemm(gpu, 0, 0, M, N, K, 1.0, A, K, B, N, 0.0, z, N, tile=tile)
        assert gpu.last_kernel().startswith(name)
        for _ in range(5):
            assert np.array_equal(gpu_sgemm(gpu, 0, 0, M, N, K, 1.0, A, K, B, N, 0.0, z, N, tile=tile), first)
        want = A.astype(np.float64) @ B.astype(np.float64)
        assert rel_err(first, want) < TOL
        for (tA, tB, m, n, k) in [(0, 0, 70, 100, 532), (0, 1, 33, 47, 788), (1, 0, 100, 36, 660), (1, 1, 20, 65, 596)]:
            a = rng.standard_normal((k, m) if tA else (m, k)).astype(np.float32)
            b = rng.standard_normal((n, k) if tB else (k, n)).astype(np.float32)
            c0 = rng.standard_normal((m, n)).astype(np.float32)
            got = gpu_sgemm(gpu, tA, tB, m, n, k, 0.5, a, a.shape[1], b, b.shape[1], 2.0, c0, n, tile=tile)
            assert gpu.last_kernel().startswith(name), gpu.last_kernel()
            opa, opb = (a.T if tA else a).astype(np.float64), (b.T if tB else b).astype(np.float64)
            assert rel_err(got, 0.5 * opa @ opb + 2.0 * c0) < TOL, (tA, tB, m, n, k)


def test_classifier_head_on_the_weight_streaming_kernel(gpu):
    """NT products with few output columns (a classifier head: 128 x 10 x 1024; l-ten's 5760 -> 50 layer) run on the
    16-column weight-streaming kernel: ragged column block, ragged rows, alpha and beta, repeatable bit for bit."""
    rng = np.random.default_rng(21)
    for (m, n, k) in [(128, 10, 1024), (33, 31, 788), (200, 16, 256), (5, 1, 512), (64, 50, 5760), (130, 300, 1024), (7, 511, 260)]:
        a = rng.standard_normal((m, k)).astype(np.float32)
        b = rng.standard_normal((n, k)).astype(np.float32)
        c0 = rng.standard_normal((m, n)).astype(np.float32)
        got = gpu_sgemm(gpu, 0, 1, m, n, k, 0.5, a, k, b, k, 2.0, c0, n)
        assert gpu.last_kernel().startswith("sgemm_skinny_nt"), gpu.last_kernel()
        assert np.array_equal(got, gpu_sgemm(gpu, 0, 1, m, n, k, 0.5, a, k, b, k, 2.0, c0, n))
        assert rel_err(got, 0.5 * a.astype(np.float64) @ b.astype(np.float64).T + 2.0 * c0) < TOL, (m, n, k)


def test_data_gradient_on_the_weight_streaming_kernel(gpu):
    """NN products with few rows against a wide weight matrix (dX = dY W of a FullyConnected layer at batch 128) run
    on the 16-column weight-streaming tiles with the weights read along n: ragged row blocks, a ragged last column
    block, K that is no multiple of 32, alpha and beta, repeatable bit for bit."""
    rng = np.random.default_rng(22)
    for (m, n, k) in [(128, 1024, 1024), (128, 784, 1024), (40, 520, 260), (17, 512, 1000)]:
        a = rng.standard_normal((m, k)).astype(np.float32)
        b = rng.standard_normal((k, n)).astype(np.float32)
        c0 = rng.standard_normal((m, n)).astype(np.float32)
        got = gpu_sgemm(gpu, 0, 0, m, n, k, 0.5, a, k, b, n, 2.0, c0, n)
        assert gpu.last_kernel().startswith("sgemm_skinny_nn"), gpu.last_kernel()
        assert np.array_equal(got, gpu_sgemm(gpu, 0, 0, m, n, k, 0.5, a, k, b, n, 2.0, c0, n))
        assert rel_err(got, 0.5 * a.astype(np.float64) @ b.astype(np.float64) + 2.0 * c0) < TOL, (m, n, k)


def test_rank1_and_rowvec_shapes(gpu, ob):
    rng = np.random.default_rng(9)
    M, N = 128, 1024
    ones = np.ones((M, 1), np.float32)
    bias = rng.standard_normal((1, N)).astype(np.float32)
    Y0 = rng.standard_normal((M, N)).astype(np.float32)
    # l-ten/fully_connected.cpp:165: Y += ones[M x 1] bias[1 x N]
    got = gpu_sgemm(gpu, 0, 0, M, N, 1, 1.0, ones, 1, bias, N, 1.0, Y0, N)
    assert gpu.last_kernel() == "sgemm_rank1"
    assert np.array_equal(got, Y0 + bias)
    # the weight gradient of a layer at batch 1, dW = dy^T x (A stored [1][M]), alpha and beta at work: the four-column form
    # (M * N >= 2^16, N a multiple of 4) and the one-column form (N = 1023) give the same rounding, alpha * (a * b) + beta * c
    dyv = rng.standard_normal((1, M)).astype(np.float32)
    for n in (N, N - 1):
        xv = rng.standard_normal((1, n)).astype(np.float32)
        C0 = rng.standard_normal((M, n)).astype(np.float32)
        got = gpu_sgemm(gpu, 1, 0, M, n, 1, 0.5, dyv, M, xv, n, -2.0, C0, n)
        assert gpu.last_kernel() == "sgemm_rank1"
        assert np.array_equal(got, np.float32(0.5) * (dyv.T * xv) + np.float32(-2.0) * C0)
    # l-ten/backprop.cpp:2267: db[1 x N] += ones[1 x M] dY[M x N]
    db0 = rng.standard_normal((1, N)).astype(np.float32)
    got = gpu_sgemm(gpu, 0, 0, 1, N, M, 1.0, np.ones((1, M), np.float32), M, Y0, N, 1.0, db0, N)
    assert gpu.last_kernel() == "sgemm_rowvec"
    assert rel_err(got, db0 + Y0.astype(np.float64).sum(0, keepdims=True)) < TOL


def test_gru_step_products(gpu, ob):
    """The two M = 1 products of a GRU time step (l-ten/gru.cpp:267-268, 358-361: a 1 x K row times K x 3H, not
    transposed) at input = hidden = 1024, and at a ragged size, against the oracle's GEMM."""
    rng = np.random.default_rng(21)
    for K, N in ((1024, 3072), (1000, 300), (3, 3072)):
        x = rng.standard_normal((1, K)).astype(np.float32)
        u = (rng.standard_normal((K, N)) * 0.05).astype(np.float32)
        want = np.zeros((1, N), np.float32)
        ob.sgemm(0, 0, 1, N, K, 1.0, x, K, u, N, 0.0, want, N)
        got = gpu_sgemm(gpu, 0, 0, 1, N, K, 1.0, x, K, u, N, 0.0, np.zeros((1, N), np.float32), N)
        assert gpu.last_kernel() == "sgemm_rowvec"
        assert rel_err(got, want) < TOL, (K, N)
        assert rel_err(got, x.astype(np.float64) @ u.astype(np.float64)) < TOL, (K, N)
    # small integers: exact in any order
    x = rng.integers(-3, 4, (1, 1024)).astype(np.float32)
    u = rng.integers(-3, 4, (1024, 3072)).astype(np.float32)
    got = gpu_sgemm(gpu, 0, 0, 1, 3072, 1024, 1.0, x, 1024, u, 3072, 0.0, np.zeros((1, 3072), np.float32), 3072)
    assert np.array_equal(got, x @ u)


def test_gru_step_both_products_in_one_launch(gpu, ob):
    """x U and h W of one GRU time step (l-ten/gru.cpp:358-361) as one strided batch of two M = 1 products: one launch
    of the row-vector kernel; each product equal to the single call (same kernel, same order) and to the oracle.
    The two operand pairs sit in separate allocations: the strides are the distances between them."""
    rng = np.random.default_rng(22)
    H = 1024
    K, N = H, 3 * H
    D = gpu.DeviceBuffer
    xh = rng.standard_normal((2, K)).astype(np.float32)                  # x_t and h_{t-1}
    uw = (rng.standard_normal((2, K, N)) * 0.05).astype(np.float32)      # weights_u and weights_w
    dX, dU, dOut = D.from_numpy(xh), D.from_numpy(uw), D(2 * N * 4, zero=True)
    gpu.check(gpu.lib().lten_hip_sgemm_strided_batched(0, 0, 1, N, K, 1.0, dX.ptr, K, K, dU.ptr, N, K * N, 0.0, dOut.ptr, N, N, 2))
    assert gpu.last_kernel() == "sgemm_rowvec_batched", gpu.last_kernel()
    got = dOut.numpy(np.float32, (2, N))
    for i in range(2):
        want = np.zeros((1, N), np.float32)
        ob.sgemm(0, 0, 1, N, K, 1.0, xh[i:i + 1], K, uw[i], N, 0.0, want, N)
        assert rel_err(got[i:i + 1], want) < TOL, i
        single = gpu_sgemm(gpu, 0, 0, 1, N, K, 1.0, xh[i:i + 1], K, uw[i], N, 0.0, np.zeros((1, N), np.float32), N)
        assert np.array_equal(got[i:i + 1], single), i
    # beta = 1 accumulates per product, a broadcast input row (stride 0) is allowed
    gpu.check(gpu.lib().lten_hip_sgemm_strided_batched(0, 0, 1, N, K, 2.0, dX.ptr, K, 0, dU.ptr, N, K * N, 1.0, dOut.ptr, N, N, 2))
    again = dOut.numpy(np.float32, (2, N))
    for i in range(2):
        want = got[i].astype(np.float64) + 2.0 * (xh[0].astype(np.float64) @ uw[i].astype(np.float64))
        assert rel_err(again[i], want) < TOL, i


def test_strided_batched_and_broadcast(gpu, ob):
    g = np.load(golden_path("layer_cases.npz"))
    # case 0: a{2,1,4,8} x b{1,1,8,15}: b broadcast over the leading index (stride 0)
    a, b, c = g["mm0_a"], g["mm0_b"], g["mm0_c"]
    dA, dB, dC = gpu.DeviceBuffer.from_numpy(a), gpu.DeviceBuffer.from_numpy(b), gpu.DeviceBuffer(c.nbytes)
    gpu.check(gpu.lib().lten_hip_sgemm_strided_batched(0, 0, 4, 15, 8, 1.0, dA.ptr, 8, 32, dB.ptr, 15, 0, 0.0, dC.ptr, 15,
                                                       60, 2))
    assert rel_err(dC.numpy(np.float32, c.shape), c) < TOL
    # its weight gradient: dB += A_i^T dC_i over the batch, all into one dB (stride_c = 0, beta = 1)
    dc, db = g["mm0_dc"], g["mm0_db"]
    dDC, dDB = gpu.DeviceBuffer.from_numpy(dc), gpu.DeviceBuffer(db.nbytes, zero=True)
    gpu.check(gpu.lib().lten_hip_sgemm_strided_batched(1, 0, 8, 15, 4, 1.0, dA.ptr, 8, 32, dDC.ptr, 15, 60, 1.0, dDB.ptr,
                                                       15, 0, 2))
    assert rel_err(dDB.numpy(np.float32, db.shape), db) < TOL


@pytest.mark.parametrize("batch,M,K,N", [(64, 100, 96, 80), (7, 33, 50, 20), (512, 64, 32, 48)])
def test_gradient_of_a_broadcast_matrix_over_a_stack(gpu, batch, M, K, N):
    """dB = sum_i A_i^T dC_i for a[batch, M, K] x b[K, N] (b shared by the stack): the stack lies along the reduction, so the
    batch that all writes one C runs as a single product over batch * M rows; with beta = 1 on top of what dB held."""
    rng = np.random.default_rng(batch + M + K + N)
    a = rng.standard_normal((batch, M, K)).astype(np.float32)
    dc = rng.standard_normal((batch, M, N)).astype(np.float32)
    db0 = rng.standard_normal((K, N)).astype(np.float32)
    D = gpu.DeviceBuffer
    dA, dDC, dDB = D.from_numpy(a), D.from_numpy(dc), D.from_numpy(db0)
    gpu.check(gpu.lib().lten_hip_sgemm_strided_batched(1, 0, K, N, M, 1.0, dA.ptr, K, M * K, dDC.ptr, N, M * N, 1.0, dDB.ptr, N, 0, batch))
    want = db0.astype(np.float64) + np.einsum("bmk,bmn->kn", a.astype(np.float64), dc.astype(np.float64))
    assert rel_err(dDB.numpy(np.float32, (K, N)), want.astype(np.float32)) < TOL, gpu.last_kernel()


@pytest.mark.parametrize("tB", [0, 1])
@pytest.mark.parametrize("batch,M,K,N", [(64, 10, 96, 80), (7, 33, 50, 20), (300, 16, 128, 128)])
def test_stack_against_one_shared_matrix(gpu, batch, M, K, N, tB):
    """a[batch, M, K] x b[K, N] (or b^T given as [N, K]) with b shared by the stack (stride 0) and the stack's matrices one
    behind the other in a and c: runs as one product with batch * M rows; alpha, beta as in every route."""
    rng = np.random.default_rng(batch + M + K + N + tB)
    a = rng.standard_normal((batch, M, K)).astype(np.float32)
    b = rng.standard_normal((N, K) if tB else (K, N)).astype(np.float32)
    c0 = rng.standard_normal((batch, M, N)).astype(np.float32)
    D = gpu.DeviceBuffer
    dA, dB, dC = D.from_numpy(a), D.from_numpy(b), D.from_numpy(c0)
    gpu.check(gpu.lib().lten_hip_sgemm_strided_batched(0, tB, M, N, K, 0.5, dA.ptr, K, M * K, dB.ptr, K if tB else N, 0, 2.0, dC.ptr, N, M * N, batch))
    b64 = (b.T if tB else b).astype(np.float64)
    want = 0.5 * a.astype(np.float64) @ b64 + 2.0 * c0
    assert rel_err(dC.numpy(np.float32, c0.shape), want.astype(np.float32)) < TOL, gpu.last_kernel()


@pytest.mark.parametrize("layout", [(0, 0), (0, 1), (1, 0)])
@pytest.mark.parametrize("batch,M,N,K,tile", [(24, 256, 512, 64, "sgemm_fast_128x128"),    # 8 tiles of 128 x 128 a product: 192
                                              (13, 256, 320, 128, "sgemm_fast_64x64"),     # 20 tiles of 64 x 64 a product: 260
                                              (6, 260, 516, 96, "sgemm_fast_64x64")])      # ragged last tiles, K = 96: three k-steps
def test_stack_of_products_over_a_short_reduction(gpu, batch, M, N, K, tile, layout):
    """A batch of attention-head-sized products (K of 64 to 255 in whole steps of 32): on the direct-to-LDS tiles from 192 tiles
    of 128 x 128 (K = 64) or 256 tiles of 64 x 64 (K >= 96) on.  Integer-valued operands come out exactly in every layout;
    alpha and beta as everywhere."""
    tA, tB = layout
    rng = np.random.default_rng(batch + M + N + K + 2 * tA + tB)
    a = rng.integers(-4, 5, (batch, M, K)).astype(np.float32)
    b = rng.integers(-4, 5, (batch, K, N)).astype(np.float32)
    c0 = rng.integers(-9, 10, (batch, M, N)).astype(np.float32)
    want = 2.0 * (a.astype(np.float64) @ b.astype(np.float64)) - c0
    D = gpu.DeviceBuffer
    dA = D.from_numpy(np.ascontiguousarray(a.transpose(0, 2, 1)) if tA else a)
    dB = D.from_numpy(np.ascontiguousarray(b.transpose(0, 2, 1)) if tB else b)
    dC = D.from_numpy(c0)
    gpu.check(gpu.lib().lten_hip_sgemm_strided_batched(tA, tB, M, N, K, 2.0, dA.ptr, M if tA else K, M * K, dB.ptr, K if tB else N, K * N,
                                                       -1.0, dC.ptr, N, M * N, batch))
    assert gpu.last_kernel().startswith(tile), gpu.last_kernel()
    assert np.array_equal(dC.numpy(np.float32, c0.shape), want.astype(np.float32))


@pytest.mark.parametrize("batch,M,N,K", [(5, 7, 100, 1028), (64, 16, 128, 512), (300, 1, 33, 260)])
def test_stack_of_few_row_products_against_transposed_matrices(gpu, batch, M, N, K):
    """A strided batch of NT products with at most 16 rows each (the slices of a split reduction are one): the weight-streaming
    kernel with one grid plane per problem.  Integer-valued operands, exact; alpha and beta as everywhere."""
    rng = np.random.default_rng(batch + M + N + K)
    a = rng.integers(-4, 5, (batch, M, K)).astype(np.float32)
    b = rng.integers(-4, 5, (batch, N, K)).astype(np.float32)
    c0 = rng.integers(-9, 10, (batch, M, N)).astype(np.float32)
    want = (0.5 * (a.astype(np.float64) @ b.astype(np.float64).transpose(0, 2, 1)) + 2.0 * c0).astype(np.float32)
    D = gpu.DeviceBuffer
    dA, dB, dC = D.from_numpy(a), D.from_numpy(b), D.from_numpy(c0)
    gpu.check(gpu.lib().lten_hip_sgemm_strided_batched(0, 1, M, N, K, 0.5, dA.ptr, K, M * K, dB.ptr, K, N * K, 2.0, dC.ptr, N, M * N, batch))
    assert gpu.last_kernel() == "sgemm_skinny_nt_16x16", gpu.last_kernel()
    assert np.array_equal(dC.numpy(np.float32, c0.shape), want)


@pytest.mark.parametrize("tA,tB", [(1, 0), (0, 0)])
def test_small_stack_of_long_reductions_is_split_one_by_one(gpu, tA, tB):
    """matmul's gradient for a stack of tall matrices: a few products with a small output each under a reduction of 8192 or more
    run one after the other, each cut into slices; integer-valued operands, exact, C's padding untouched."""
    batch, M, N, K = 3, 40, 72, 8192 + 96
    rng = np.random.default_rng(5 + tA)
    a = rng.integers(-3, 4, (batch, M, K)).astype(np.float32)
    b = rng.integers(-3, 4, (batch, K, N)).astype(np.float32)
    c0 = rng.integers(-9, 10, (batch, M, N + 4)).astype(np.float32)
    want = (2.0 * (a.astype(np.float64) @ b.astype(np.float64)) - c0[:, :, :N]).astype(np.float32)
    D = gpu.DeviceBuffer
    dA, dB, dC = D.from_numpy(np.ascontiguousarray(a.transpose(0, 2, 1)) if tA else a), D.from_numpy(b), D.from_numpy(c0)
    gpu.check(gpu.lib().lten_hip_sgemm_strided_batched(tA, tB, M, N, K, 2.0, dA.ptr, M if tA else K, M * K, dB.ptr, N, K * N, -1.0, dC.ptr, N + 4,
                                                       M * (N + 4), batch))
    assert gpu.last_kernel() == "sgemm_split_k", gpu.last_kernel()
    got = dC.numpy(np.float32, c0.shape)
    assert np.array_equal(got[:, :, :N], want)
    assert np.array_equal(got[:, :, N:], c0[:, :, N:])


@pytest.mark.parametrize("M,N,K", [(1027, 512, 2), (640, 1000, 5), (513, 2052, 8)])
def test_weight_gradient_over_a_batch_of_2_to_8_is_a_stream_over_c(gpu, M, N, K):
    """A^T B over 2 to 8 rows into a large output (dW of a wide layer at a batch that small): four rows by four columns per
    thread, the products added in the order of k.  Row counts that are no multiple of four, padded leading dimensions, alpha
    and beta; integer-valued operands, exact, C's padding untouched."""
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(-4, 5, (K, M)).astype(np.float32)
    B = rng.integers(-4, 5, (K, N)).astype(np.float32)
    want = (A.astype(np.float64).T @ B.astype(np.float64)).astype(np.float32)
    lda, ldb, ldc = M + 3, N + 4, N + 8
    As = np.zeros((K, lda), np.float32)
    As[:, :M] = A
    Bs = np.zeros((K, ldb), np.float32)
    Bs[:, :N] = B
    C0 = np.full((M, ldc), 7.0, np.float32)
    got = gpu_sgemm(gpu, 1, 0, M, N, K, 1.0, As, lda, Bs, ldb, 0.0, C0, ldc)
    assert gpu.last_kernel() == "sgemm_tn_few_rows", gpu.last_kernel()
    assert np.array_equal(got[:, :N], want)
    assert (got[:, N:] == 7.0).all()
    got2 = gpu_sgemm(gpu, 1, 0, M, N, K, 2.0, As, lda, Bs, ldb, -1.0, got, ldc)
    assert np.array_equal(got2[:, :N], want)
    assert (got2[:, N:] == 7.0).all()
    nan0 = np.full((M, ldc), np.nan, np.float32)
    assert np.array_equal(gpu_sgemm(gpu, 1, 0, M, N, K, 1.0, As, lda, Bs, ldb, 0.0, nan0, ldc)[:, :N], want)


def test_fc_forward_backward_golden_and_lten_vectors(gpu):
    g = np.load(golden_path("layer_cases.npz"))
    cases = []
    for i in range(int(g["fc_count"])):
        pre = f"fc{i}_"
        M, fin, fout, use_bias = (int(v) for v in g[pre + "dims"])
        cases.append((M, fin, fout, g[pre + "x"], g[pre + "w"], g[pre + "b"] if use_bias else None, g[pre + "dy"],
                      g[pre + "y"], g[pre + "dx"], g[pre + "dw"], g[pre + "db"] if use_bias else None, TOL, True))
    v = json.load(open(golden_path("lten_unit_test_vectors.json")))["fc_test"]   # tests/unit_tests.cpp fc_test
    dy = np.zeros((2, 1, 4, 8), np.float32)
    dy[tuple(v["backward_from"])] = 1.0
    cases.append((8, 3, 8, np.array(v["x"], np.float32), np.array(v["weights"], np.float32), None, dy.reshape(-1),
                  np.array(v["z"], np.float32), np.array(v["x_grad"], np.float32), np.array(v["w_grad"], np.float32),
                  None, v["tolerance"], False))
    for (M, fin, fout, x, w, b, dy, y, dx, dw, db, tol, relative) in cases:
        D = gpu.DeviceBuffer
        dX, dW, dDY = D.from_numpy(x), D.from_numpy(w), D.from_numpy(dy)
        dB = D.from_numpy(b) if b is not None else None
        dYo, dDX, dDW = D(4 * M * fout), D(4 * M * fin), D(4 * fout * fin)
        dDB = D(4 * fout, zero=True) if b is not None else None
        gpu.check(gpu.lib().lten_hip_fc_forward_f32(M, fin, fout, dX.ptr, dW.ptr, dB.ptr if dB else None, dYo.ptr))
        gpu.check(gpu.lib().lten_hip_fc_backward_f32(M, fin, fout, dX.ptr, dW.ptr, dDY.ptr, dDX.ptr, dDW.ptr,
                                                     dDB.ptr if dDB else None))
        for got, want in ((dYo.numpy(np.float32, y.shape), y), (dDX.numpy(np.float32, dx.shape), dx),
                          (dDW.numpy(np.float32, dw.shape), dw)) + (((dDB.numpy(np.float32, db.shape), db),) if b is not None else ()):
            if relative:
                assert rel_err(got, want) < tol
            else:
                assert np.abs(got - want).max() <= tol   # l-ten's own abs tolerance for fc_test


@pytest.mark.parametrize("M,fin,fout,kernels", [
    (128, 200, 75, ("sgemm_fc_backward_pair_32x32_w8",)),            # both products in one launch, bias gradient inside it
    (37, 33, 10, ("sgemm_fc_backward_pair_32x32_w8",)),              # ragged in every dimension
    (100, 530, 490, ("sgemm_fc_backward_pair_32x32_shortk",)),       # many weight-gradient tiles, short K: a whole-K tile per wavefront, ragged
    (300, 600, 500, ("sgemm_fc_backward_pair_32x32_w8",)),           # batch above 256: the weight gradient cuts K over the wavefronts
    (777, 96, 132, ("sgemm_staged_32x32_w8",)),                      # batch >= 512: two launches, dW with whole-line loads, ragged K
    (128, 784, 1024, ("sgemm_fc_backward_pair_wide",)),              # config 2, layer 1: both products on 16-byte loads, each on a workgroup per CU
    (100, 1024, 516, ("sgemm_fc_backward_pair_wide",)),              # the same with a ragged batch (two halves of 64 and 36 rows) and ragged tiles
    (128, 786, 1024, ("sgemm_fc_backward_pair_32x32_shortk",)),      # rows of X that allow no 16-byte loads: whole-K tiles from dword loads
    (511, 64, 2048, ("sgemm_fc_backward_pair_32x32_w8",)),           # the largest batch the paired launch takes
    (8, 1024, 1024, ("sgemm_fc_backward_pair_wide",)),               # fewer rows than a block of the data-gradient tiles
    (20, 2048, 2048, ("sgemm_fc_backward_pair_wide",)),              # 4096 tiles of dW: a whole-K tile per wavefront, eight per workgroup
    (70, 2052, 2060, ("sgemm_fc_backward_pair_wide",)),              # the same with ragged tiles on every side and a ragged batch
    (3, 512, 4096, ("sgemm_fc_backward_pair_wide",)),                # 4096 outputs wide, 2048 tiles: four per workgroup
    (128, 1024, 10, ("sgemm_fc_backward_pair_32x32_w8",)),           # config 2, last layer
    (1024, 2048, 2048, ("sgemm_rowvec",)),                           # direct-to-LDS tiles, then the column-sum kernel
    (640, 1101, 999, ("sgemm_rowvec",)),                             # unaligned rows, many tiles: LDS-tiled GEMM, then the column sum
    (128, 2048, 8192, ("sgemm_rowvec",)),                            # a wide layer at a small batch: dW on the 128 x 128 tiles, no paired launch
])
def test_fc_backward_bias_gradient_accumulates_on_every_route(gpu, M, fin, fout, kernels):
    """db += column sums of dY (l-ten/backprop.cpp:2267, beta = 1) whichever kernel computes dW: integer-valued
    inputs make the sums exact in any order, so db must equal its start value plus the sum, bit for bit."""
    rng = np.random.default_rng(M + fin)
    x = rng.integers(-3, 4, (M, fin)).astype(np.float32)
    w = rng.integers(-3, 4, (fout, fin)).astype(np.float32)
    dy = rng.integers(-4, 5, (M, fout)).astype(np.float32)
    db0 = rng.integers(-50, 50, fout).astype(np.float32)
    D = gpu.DeviceBuffer
    dX, dW, dDY, dDB = D.from_numpy(x), D.from_numpy(w), D.from_numpy(dy), D.from_numpy(db0)
    dDX, dDW = D(x.nbytes), D(w.nbytes)
    gpu.check(gpu.lib().lten_hip_fc_backward_f32(M, fin, fout, dX.ptr, dW.ptr, dDY.ptr, dDX.ptr, dDW.ptr, dDB.ptr))
    assert gpu.last_kernel() in kernels
    assert np.array_equal(dDB.numpy(np.float32, (fout,)), db0 + dy.sum(axis=0))
    assert np.array_equal(dDW.numpy(np.float32, w.shape), dy.T @ x)
    assert np.array_equal(dDX.numpy(np.float32, x.shape), dy @ w)
    # one product at a time goes through the GEMM entry's own choice of kernel
    dDX2, dDW2, dDB3 = D(x.nbytes), D(w.nbytes), D.from_numpy(db0)
    gpu.check(gpu.lib().lten_hip_fc_backward_f32(M, fin, fout, dX.ptr, dW.ptr, dDY.ptr, dDX2.ptr, None, None))
    assert not gpu.last_kernel().startswith("sgemm_fc_backward_pair")
    gpu.check(gpu.lib().lten_hip_fc_backward_f32(M, fin, fout, dX.ptr, dW.ptr, dDY.ptr, None, dDW2.ptr, dDB3.ptr))
    assert np.array_equal(dDX2.numpy(np.float32, x.shape), dy @ w)
    assert np.array_equal(dDW2.numpy(np.float32, w.shape), dy.T @ x)
    assert np.array_equal(dDB3.numpy(np.float32, (fout,)), db0 + dy.sum(axis=0))
    # without dW the column-sum kernel still serves db
    dDB2 = D.from_numpy(db0)
    gpu.check(gpu.lib().lten_hip_fc_backward_f32(M, fin, fout, dX.ptr, dW.ptr, dDY.ptr, None, None, dDB2.ptr))
    assert np.array_equal(dDB2.numpy(np.float32, (fout,)), db0 + dy.sum(axis=0))


def test_lten_matmul_test_vectors(gpu):
    """tests/unit_tests.cpp matmul_test through the strided-batched entry point: exact values."""
    v = json.load(open(golden_path("lten_unit_test_vectors.json")))["matmul_test"]
    a, b = np.array(v["x"], np.float32), np.array(v["w"], np.float32)
    D = gpu.DeviceBuffer
    dA, dB, dC = D.from_numpy(a), D.from_numpy(b), D(4 * 32)
    l = gpu.lib()
    gpu.check(l.lten_hip_sgemm_strided_batched(0, 0, 4, 4, 3, 1.0, dA.ptr, 3, 12, dB.ptr, 4, 0, 0.0, dC.ptr, 4, 16, 2))
    assert np.array_equal(dC.numpy(np.float32, (32,)), np.array(v["z"], np.float32))
    dc = np.zeros((2, 1, 4, 4), np.float32)
    dc[tuple(v["backward_from"])] = 1.0
    dDC, dDA, dDB = D.from_numpy(dc), D(4 * 24, zero=True), D(4 * 12, zero=True)
    # l-ten/backprop.cpp:562  dA_i += dC_i B^T ; :580  dB += A_i^T dC_i (B broadcast: one dB for both i)
    gpu.check(l.lten_hip_sgemm_strided_batched(0, 1, 4, 3, 4, 1.0, dDC.ptr, 4, 16, dB.ptr, 4, 0, 1.0, dDA.ptr, 3, 12, 2))
    gpu.check(l.lten_hip_sgemm_strided_batched(1, 0, 3, 4, 4, 1.0, dA.ptr, 3, 12, dDC.ptr, 4, 16, 1.0, dDB.ptr, 4, 0, 2))
    assert np.array_equal(dDA.numpy(np.float32, (24,)), np.array(v["x_grad"], np.float32))
    assert np.array_equal(dDB.numpy(np.float32, (12,)), np.array(v["w_grad"], np.float32))


def test_large_gemm_linearity_property(gpu):
    """2048^3: too large for the scalar oracle; check (A1 + A2) B == A1 B + A2 B on integer-valued data
    (exact in fp32 at these magnitudes) and a sampled fp64 comparison on random data."""
    n = 2048
    rng = np.random.default_rng(1)
    A1 = rng.integers(-4, 5, (n, n)).astype(np.float32)
    A2 = rng.integers(-4, 5, (n, n)).astype(np.float32)
    B = rng.integers(-4, 5, (n, n)).astype(np.float32)
    z = np.zeros((n, n), np.float32)
    c1 = gpu_sgemm(gpu, 0, 0, n, n, n, 1.0, A1, n, B, n, 0.0, z, n)
    c12 = gpu_sgemm(gpu, 0, 0, n, n, n, 1.0, A2, n, B, n, 1.0, c1, n)
    cs = gpu_sgemm(gpu, 0, 0, n, n, n, 1.0, A1 + A2, n, B, n, 0.0, z, n)
    assert np.array_equal(c12, cs)
    R = rng.standard_normal((n, n)).astype(np.float32)
    S = rng.standard_normal((n, n)).astype(np.float32)
    got = gpu_sgemm(gpu, 0, 1, n, n, n, 1.0, R, n, S, n, 0.0, z, n)
    rows = rng.integers(0, n, 64)
    want = R[rows].astype(np.float64) @ S.astype(np.float64).T
    assert rel_err(got[rows], want) < TOL


FAST_TILES = {11: "sgemm_fast_256x256x32_w2x4_s2", 12: "sgemm_fast_256x256x32_w4x2_s2", 21: "sgemm_fast_128x128x32_w2x2_s2",
              22: "sgemm_fast_128x128x32_w2x2_s3", 23: "sgemm_fast_128x128x32_w2x2_s4", 31: "sgemm_fast_64x64x32_w2x2_s2"}


@pytest.mark.parametrize("tile", sorted(FAST_TILES))
@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_direct_to_lds_tiles_exact_all_layouts(gpu, tile, tA, tB):
    """The direct-to-LDS tiles by number: integer-valued operands make every summation order exact, so the result
    must equal the int64 product bit for bit, with padded leading dimensions, alpha / beta and an untouched pad."""
    rng = np.random.default_rng(500 + 10 * tile + 2 * tA + tB)
    M, N, K = (512, 256, 160) if tile < 20 else (256, 384, 96)   # K / 32 = 5 or 3 k-steps: prologue, steady state, drain
    A = rng.integers(-8, 9, (M, K)).astype(np.float32)
    B = rng.integers(-8, 9, (K, N)).astype(np.float32)
    want = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)
    lda, ldb, ldc = (M if tA else K) + 4, (K if tB else N) + 8, N + 3
    As = np.zeros(((K if tA else M), lda), np.float32)
    As[:, :(M if tA else K)] = A.T if tA else A
    Bs = np.zeros(((N if tB else K), ldb), np.float32)
    Bs[:, :(K if tB else N)] = B.T if tB else B
    C0 = np.full((M, ldc), 7.0, np.float32)
    got = gpu_sgemm(gpu, tA, tB, M, N, K, 1.0, As, lda, Bs, ldb, 0.0, C0, ldc, tile)
    assert gpu.last_kernel() == FAST_TILES[tile]
    assert np.array_equal(got[:, :N], want)
    assert (got[:, N:] == 7.0).all()
    got2 = gpu_sgemm(gpu, tA, tB, M, N, K, 2.0, As, lda, Bs, ldb, -1.0, got, ldc, tile)
    assert np.array_equal(got2[:, :N], want)


def test_direct_to_lds_tiles_are_the_default_for_large_aligned_problems(gpu):
    """Heuristic, long K (many trips round the stage ring), FullyConnected bias, and a strided batch; an unaligned
    operand must fall back to the general kernels and still be right."""
    rng = np.random.default_rng(9)
    D, l = gpu.DeviceBuffer, gpu.lib()
    M, fin, fout = 4096, 1024, 4096
    x = rng.integers(-4, 5, (M, fin)).astype(np.float32)
    w = rng.integers(-4, 5, (fout, fin)).astype(np.float32)
    b = rng.integers(-9, 10, fout).astype(np.float32)
    dX, dW, dB, dY = D.from_numpy(x), D.from_numpy(w), D.from_numpy(b), D(4 * M * fout)
    gpu.check(l.lten_hip_fc_forward_f32(M, fin, fout, dX.ptr, dW.ptr, dB.ptr, dY.ptr))
    assert gpu.last_kernel() == FAST_TILES[12]
    assert np.array_equal(dY.numpy(np.float32, (M, fout)), x @ w.T + b)
    # 2048 x 2048 output: too few 256-tiles, so 128-tiles
    gpu.check(l.lten_hip_fc_forward_f32(2048, fin, 2048, dX.ptr, dW.ptr, None, dY.ptr))
    assert gpu.last_kernel() == FAST_TILES[21]
    assert np.array_equal(dY.numpy(np.float32, (2048, 2048)), x[:2048] @ w[:2048].T)
    # 2048 x 1024 and 300 x 3400 outputs (NT): 128-tiles would leave CUs without a workgroup, 64-tiles do not
    gpu.check(l.lten_hip_fc_forward_f32(2048, fin, 1024, dX.ptr, dW.ptr, dB.ptr, dY.ptr))
    assert gpu.last_kernel() == FAST_TILES[31]
    assert np.array_equal(dY.numpy(np.float32, (2048, 1024)), x[:2048] @ w[:1024].T + b[:1024])
    gpu.check(l.lten_hip_fc_forward_f32(300, fin, 3400, dX.ptr, dW.ptr, dB.ptr, dY.ptr))
    assert gpu.last_kernel() == FAST_TILES[31]
    assert np.array_equal(dY.numpy(np.float32, (300, 3400)), x[:300] @ w[:3400].T + b[:3400])
    # strided batch of 4 (Tensor::matmul over a leading dimension), NN: 128 tiles of 128 x 128 in all, so 64-tiles here too
    a4 = rng.integers(-4, 5, (4, 512, 256)).astype(np.float32)
    b4 = rng.integers(-4, 5, (4, 256, 1024)).astype(np.float32)
    dA4, dB4, dC4 = D.from_numpy(a4), D.from_numpy(b4), D(4 * 4 * 512 * 1024)
    gpu.check(l.lten_hip_sgemm_strided_batched(0, 0, 512, 1024, 256, 1.0, dA4.ptr, 256, 512 * 256, dB4.ptr, 1024, 256 * 1024, 0.0,
                                               dC4.ptr, 1024, 512 * 1024, 4))
    assert gpu.last_kernel() == FAST_TILES[31]
    assert np.array_equal(dC4.numpy(np.float32, (4, 512, 1024)), a4 @ b4)
    # an operand base that is not 16-byte aligned: general kernel
    dXo = D(x.nbytes + 16)
    dXo.upload(x, offset=4)
    gpu.check(l.lten_hip_fc_forward_f32(M, fin, fout, dXo.ptr + 4, dW.ptr, dB.ptr, dY.ptr))
    assert not gpu.last_kernel().startswith("sgemm_fast")
    assert np.array_equal(dY.numpy(np.float32, (M, fout)), x @ w.T + b)
    # ragged M: still the tiles (edge rows are fetched twice and not stored)
    gpu.check(l.lten_hip_fc_forward_f32(M - 1, fin, fout, dX.ptr, dW.ptr, dB.ptr, dY.ptr))
    assert gpu.last_kernel() == FAST_TILES[12]
    assert np.array_equal(dY.numpy(np.float32, (M - 1, fout)), x[:-1] @ w.T + b)


@pytest.mark.parametrize("tA,tB,M,N,K", [(0, 1, 1999, 2001, 1000), (0, 0, 1501, 2004, 488), (1, 0, 2000, 1532, 520),
                                         (1, 1, 1796, 1801, 1032), (0, 1, 129, 16385, 256)])
def test_direct_to_lds_tiles_ragged_sizes(gpu, tA, tB, M, N, K):
    """Sizes that are no multiple of the tile or of the k-step: edge tiles fetch an existing row twice and store only
    what exists; the k remainder is added by a second launch.  Exact on integer-valued data, pad columns untouched."""
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(-4, 5, (M, K)).astype(np.float32)
    B = rng.integers(-4, 5, (K, N)).astype(np.float32)
    want = A @ B   # exact: |sum| < 2^24
    lda, ldb, ldc = (M if tA else K), (K if tB else N), N + 1
    As = np.ascontiguousarray(A.T if tA else A)
    Bs = np.ascontiguousarray(B.T if tB else B)
    C0 = np.full((M, ldc), 3.0, np.float32)
    D = gpu.DeviceBuffer
    dA, dB, dC = D.from_numpy(As), D.from_numpy(Bs), D.from_numpy(C0)
    gpu.sgemm(tA, tB, M, N, K, 1.0, dA, lda, dB, ldb, 0.0, dC, ldc)
    first = gpu.last_kernel()
    got = dC.numpy(np.float32, C0.shape)
    assert np.array_equal(got[:, :N], want), first
    assert (got[:, N:] == 3.0).all()
    gpu.set_option("sgemm_tile", 21)
    try:
        gpu.sgemm(tA, tB, M, N, K & ~31, 0.5, dA, lda, dB, ldb, 2.0, dC, ldc)
        assert gpu.last_kernel() == FAST_TILES[21]
    finally:
        gpu.set_option("sgemm_tile", 0)
    Am, Bm = A[:, :K & ~31], B[:K & ~31]
    assert np.array_equal(dC.numpy(np.float32, C0.shape)[:, :N], 0.5 * (Am @ Bm) + 2.0 * want)


@pytest.mark.parametrize("M,N,K", [(1, 512, 256), (5, 1000, 1024), (16, 4096, 512), (17, 520, 4100), (32, 2048, 2048), (29, 1001, 300)])
def test_small_batch_weight_stream(gpu, M, N, K):
    """FullyConnected forward with at most 32 rows: the streaming kernel (16 columns per workgroup, 16x16x4 tiles).
    Integer-valued data make the sums exact in any order; bias, alpha / beta and a padded C are covered."""
    rng = np.random.default_rng(M * 3 + N + K)
    x = rng.integers(-4, 5, (M, K)).astype(np.float32)
    w = rng.integers(-4, 5, (N, K)).astype(np.float32)
    b = rng.integers(-9, 10, N).astype(np.float32)
    D, l = gpu.DeviceBuffer, gpu.lib()
    dX, dW, dB, dY = D.from_numpy(x), D.from_numpy(w), D.from_numpy(b), D(4 * M * N)
    gpu.check(l.lten_hip_fc_forward_f32(M, K, N, dX.ptr, dW.ptr, dB.ptr, dY.ptr))
    assert gpu.last_kernel().startswith("sgemm_skinny_nt"), gpu.last_kernel()
    assert np.array_equal(dY.numpy(np.float32, (M, N)), x @ w.T + b)
    ldc = N + 3
    C0 = np.full((M, ldc), 2.0, np.float32)
    got = gpu_sgemm(gpu, 0, 1, M, N, K, 0.5, x, K, w, K, 3.0, C0, ldc)
    assert gpu.last_kernel().startswith("sgemm_skinny_nt")
    assert np.array_equal(got[:, :N], 0.5 * (x @ w.T) + 6.0)
    assert (got[:, N:] == 2.0).all()


def test_seeded_sweep_over_dispatch_boundaries(gpu):
    """Fifty seeded products in all four layouts around the limits at which the library changes kernels (1 / 32 rows,
    few and many 32x32 tiles, 128-tile counts, leading dimensions that do and do not allow 16-byte loads, K = 1, K a
    multiple of 32 or not), random alpha / beta, against an fp64 product within 1e-4."""
    rng = np.random.default_rng(777)
    seen = set()
    Ms = [1, 3, 16, 32, 33, 100, 128, 256, 500, 1024, 1536]
    Ns = [1, 10, 31, 64, 130, 512, 1000, 1024, 2048]
    Ks = [1, 2, 33, 64, 100, 256, 300, 512, 1000, 1024, 2080]
    larger = [(2048, 1024, 256), (1030, 2052, 288), (2048, 1024, 300)]   # enough 128 x 128 tiles for the direct-to-LDS kernels
    for case in range(50 + 4 * len(larger)):
        if case < 50:
            M, N, K = int(rng.choice(Ms)), int(rng.choice(Ns)), int(rng.choice(Ks))
            while M * N * K > 3e8:
                M = max(1, M // 2)
            tA, tB = int(rng.integers(0, 2)), int(rng.integers(0, 2))
            pad_a, pad_b = int(rng.choice([0, 0, 1, 4])), int(rng.choice([0, 0, 3, 4]))
        else:
            M, N, K = larger[(case - 50) // 4]
            tA, tB = (case - 50) % 4 // 2, (case - 50) % 2
            pad_a, pad_b = 4, 0
        A = rng.standard_normal((M, K)).astype(np.float32)
        B = rng.standard_normal((K, N)).astype(np.float32)
        lda, ldb, ldc = (M if tA else K) + pad_a, (K if tB else N) + pad_b, N + int(rng.choice([0, 5]))
        As = np.zeros(((K if tA else M), lda), np.float32)
        As[:, :(M if tA else K)] = A.T if tA else A
        Bs = np.zeros(((N if tB else K), ldb), np.float32)
        Bs[:, :(K if tB else N)] = B.T if tB else B
        alpha, beta = float(rng.choice([1.0, 0.5, -2.0])), float(rng.choice([0.0, 0.0, 1.0, 0.25]))
        C0 = rng.standard_normal((M, ldc)).astype(np.float32)
        got = gpu_sgemm(gpu, tA, tB, M, N, K, alpha, As, lda, Bs, ldb, beta, C0, ldc)
        name = gpu.last_kernel()
        seen.add(name.split("_")[1])
        want = alpha * (A.astype(np.float64) @ B.astype(np.float64)) + beta * C0[:, :N].astype(np.float64)
        assert rel_err(got[:, :N], want) < TOL, (case, tA, tB, M, N, K, lda, ldb, alpha, beta, name)
        assert np.array_equal(got[:, N:], C0[:, N:]), (case, name)
    assert {"fast", "staged", "direct", "rowvec", "rank1"} <= seen, seen
