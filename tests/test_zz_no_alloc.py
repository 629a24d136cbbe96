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


def test_static_entry_point_inside_a_recording_and_without_allocation(gpu):
    """The call recorded into a launch graph, where lten_hip_alloc is refused (first use of the entry point in this
    process when the file runs alone): every replay, with eager work and waits between them, returns the eager
    result; and a call leaves the device's free memory as it found it."""
    import ctypes as C
    l, D = gpu.lib(), gpu.DeviceBuffer
    rng = np.random.default_rng(7)
    M, N, K = 256, 1024, 4096   # split-K: zero-point terms, partial sums and counters all in the static array
    X = rng.integers(0, 256, (M, K), dtype=np.uint8)
    W = rng.integers(0, 256, (N, K), dtype=np.uint8)
    bias = rng.integers(-5000, 5000, N).astype(np.int32)
    sc, zp = [0.02, 0.013, 3.0], [3, 250, 77]
    dX, dW, db, ws = D.from_numpy(X), D.from_numpy(W), D.from_numpy(bias), D(4 * (M + N))
    y_ref, y_new = D(M * N, zero=True), D(M * N, zero=True)
    qp = gpu.qparams3(sc, zp)
    with gpu.Graph() as g:
        p = C.c_void_p()
        assert l.lten_hip_alloc(C.byref(p), 1024, 0) != 0        # a recording cannot allocate ...
        gpu.check(l.lten_hip_fcq_forward_static(1, M, K, N, dX.ptr, dW.ptr, db.ptr, qp, y_new.ptr))   # ... this call need not
    assert "splitk" in gpu.last_kernel()
    gpu.check(l.lten_hip_fcq_forward(1, M, K, N, dX.ptr, dW.ptr, db.ptr, qp, y_ref.ptr, ws.ptr))
    want = y_ref.numpy(np.uint8, (M, N))
    for rep in range(3):
        gpu.check(l.lten_hip_zero(y_new.ptr, M * N))
        g.launch()
        assert np.array_equal(y_new.numpy(np.uint8, (M, N)), want), rep
        gpu.check(l.lten_hip_fcq_forward(1, M, K, N, dX.ptr, dW.ptr, db.ptr, qp, y_ref.ptr, ws.ptr))   # eager work between replays
        gpu.sync()
    hip = C.CDLL("libamdhip64.so")
    free0, free1, total = C.c_size_t(), C.c_size_t(), C.c_size_t()
    gpu.sync()
    assert hip.hipMemGetInfo(C.byref(free0), C.byref(total)) == 0
    gpu.check(l.lten_hip_fcq_forward_static(1, M, K, N, dX.ptr, dW.ptr, db.ptr, qp, y_new.ptr))
    gpu.sync()
    assert hip.hipMemGetInfo(C.byref(free1), C.byref(total)) == 0
    assert free1.value == free0.value
    assert np.array_equal(y_new.numpy(np.uint8, (M, N)), want)


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


def test_static_entry_point_on_a_long_reduction_stays_off_library_memory(gpu, ob):
    """Four rows against K = 20000: lten_hip_fcq_forward runs the weight-streaming kernel in chunks of K with their sums in
    memory the library allocates; the static entry point must not, takes another kernel, and returns the same bytes."""
    import ctypes as C
    rng = np.random.default_rng(99)
    M, N, K = 4, 256, 20000
    X = rng.integers(0, 256, (M, K), dtype=np.uint8)
    W = rng.integers(0, 256, (N, K), dtype=np.uint8)
    bias = rng.integers(-5000, 5000, N).astype(np.int32)
    sc, zp = [0.02, 0.013, 3.0], [3, 250, 77]
    hip = C.CDLL("libamdhip64.so")
    free0, free1, total = C.c_size_t(), C.c_size_t(), C.c_size_t()
    l, D = gpu.lib(), gpu.DeviceBuffer
    dX, dW, db, y = D.from_numpy(X), D.from_numpy(W), D.from_numpy(bias), D(M * N, zero=True)
    qp = gpu.qparams3(sc, zp)
    gpu.sync()
    assert hip.hipMemGetInfo(C.byref(free0), C.byref(total)) == 0
    gpu.check(l.lten_hip_fcq_forward_static(1, M, K, N, dX.ptr, dW.ptr, db.ptr, qp, y.ptr))
    k_new = gpu.last_kernel()
    gpu.sync()
    assert hip.hipMemGetInfo(C.byref(free1), C.byref(total)) == 0
    assert free1.value == free0.value
    assert k_new != "qskinny_mfma_kchunks", k_new
    got = y.numpy(np.uint8, (M, N)).copy()
    want, _, k_ref, _ = both(gpu, X, W, sc, zp, bias)
    assert k_ref == "qskinny_mfma_kchunks", k_ref
    assert np.array_equal(got, want)
    Co, _ = ob.quantized_matmul(X, W, np.array(sc, np.float32), np.array(zp, np.uint8), bias=bias)
    assert np.array_equal(want, Co)
