"""The entry point that allocates nothing, lten_hip_fcq_forward_static, against lten_hip_fcq_forward (bit-exact),
through the C ABI: two calls in a row, the second on a smaller problem, on shapes that use the static scratch both
for the zero-point terms and for the split-K partial sums; then sizes beyond the limit."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def both(gpu, X, W, sc, zp, bias):
    l, D = gpu.lib(), gpu.DeviceBuffer
    M, K = X.shape
    N = W.shape[0]
    dX, dW = D.from_numpy(X), D.from_numpy(W)
    db = D.from_numpy(bias)
    qp = gpu.qparams3(sc, zp)
    y_ref, y_new = D(M * N, zero=True), D(M * N, zero=True)
    ws = D(4 * (M + N))
    gpu.check(l.lten_hip_fcq_forward(1, M, K, N, dX.ptr, dW.ptr, db.ptr, qp, y_ref.ptr, ws.ptr))
    k_ref = gpu.last_kernel()
    gpu.check(l.lten_hip_fcq_forward_static(1, M, K, N, dX.ptr, dW.ptr, db.ptr, qp, y_new.ptr))
    k_new = gpu.last_kernel()
    return y_ref.numpy(np.uint8, (M, N)), y_new.numpy(np.uint8, (M, N)), k_ref, k_new


def test_static_entry_point_matches_twice_in_a_row(gpu, ob):
    rng = np.random.default_rng(2024)
    sc, zp = [0.02, 0.013, 3.0], [3, 250, 77]
    first = True
    for M, N, K in ((256, 1024, 4096), (128, 512, 4096), (200, 300, 784), (4096, 512, 256)):
        X = rng.integers(0, 256, (M, K), dtype=np.uint8)
        W = rng.integers(0, 256, (N, K), dtype=np.uint8)
        bias = rng.integers(-5000, 5000, N).astype(np.int32)
        want, got, k_ref, k_new = both(gpu, X, W, sc, zp, bias)
        print(f"  {M}x{N}x{K}: {k_ref} / {k_new}", flush=True)
        assert k_ref == k_new
        if first:
            assert "splitk" in k_new   # the first pair exercises the partial sums and counters in the static array
            first = False
        assert np.array_equal(got, want), (M, N, K)
        if M * N * K <= 256 * 1024 * 4096:
            Co, _ = ob.quantized_matmul(X, W, np.array(sc, np.float32), np.array(zp, np.uint8), bias=bias)
            assert np.array_equal(want, Co)


def test_static_entry_point_rejects_sizes_beyond_its_scratch(gpu):
    l, D = gpu.lib(), gpu.DeviceBuffer
    M, N, K = 65536, 64, 16
    dX, dW, dY = D(M * K, zero=True), D(N * K, zero=True), D(M * N)
    rc = l.lten_hip_fcq_forward_static(1, M, K, N, dX.ptr, dW.ptr, None, gpu.qparams3([1, 1, 1], [0, 0, 0]), dY.ptr)
    assert rc != 0 and b"exceeds the limit" in l.lten_hip_last_error()
