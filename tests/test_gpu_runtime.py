"""GPU tests of the context / memory entry points and of work on a caller-created stream (all through the C ABI)."""
import ctypes as C

import numpy as np
import pytest

from conftest import rel_err

pytestmark = pytest.mark.gpu


def test_fill_zero_copy_and_get_device(gpu):
    l, D = gpu.lib(), gpu.DeviceBuffer
    dev = C.c_int(-1)
    gpu.check(l.lten_hip_get_device(C.byref(dev)))
    assert dev.value == 0
    assert l.lten_hip_get_device(None) != 0 and b"null" in l.lten_hip_last_error()
    n = 100003
    a = D(4 * n)
    gpu.check(l.lten_hip_fill_i32(a.ptr, n, -123456789))
    assert (a.numpy(np.int32, (n,)) == -123456789).all()
    gpu.check(l.lten_hip_fill_f32(a.ptr, n, 2.5))
    assert (a.numpy(np.float32, (n,)) == 2.5).all()
    gpu.check(l.lten_hip_fill_u8(a.ptr, 4 * n, 0xAB))
    assert (a.numpy(np.uint8, (4 * n,)) == 0xAB).all()
    # zero: word-sized and byte-sized paths, and only the named range
    gpu.check(l.lten_hip_zero(a.ptr + 4, 4 * 10))
    gpu.check(l.lten_hip_zero(a.ptr + 101, 7))
    h = a.numpy(np.uint8, (4 * n,))
    want = np.full(4 * n, 0xAB, np.uint8)
    want[4:44] = 0
    want[101:108] = 0
    assert np.array_equal(h, want)
    # device-to-device copy is stream ordered: the read-back behind it sees the copied bytes
    src = D.from_numpy(np.arange(n, dtype=np.int32))
    gpu.check(l.lten_hip_copy_gpu_to_gpu(a.ptr, src.ptr, 4 * n))
    assert np.array_equal(a.numpy(np.int32, (n,)), np.arange(n, dtype=np.int32))
    # alloc with zero_memory hands out zeros, also when the block comes back from the pool with old contents
    for _ in range(3):
        z = D(4096 + 3, zero=True)
        assert not z.numpy(np.uint8, (4099,)).any()
        gpu.check(l.lten_hip_fill_u8(z.ptr, 4099, 0x5A))
        z.free()
    # the pool hands a freed block of the same rounded size out again; freeing twice is an error
    p1, p2 = C.c_void_p(), C.c_void_p()
    gpu.check(l.lten_hip_alloc(C.byref(p1), 3000000, 0))
    gpu.check(l.lten_hip_free(p1))
    gpu.check(l.lten_hip_alloc(C.byref(p2), 2500000, 0))   # both round to 4 MiB
    assert p2.value == p1.value
    gpu.check(l.lten_hip_free(p2))
    assert l.lten_hip_free(p2) != 0 and b"freed already" in l.lten_hip_last_error()


def test_pool_release_and_stream_change(gpu):
    """lten_hip_pool_release gives the cached blocks back (free device memory grows by at least their size, a later
    allocation of that size works and is usable); lten_hip_set_stream waits for the work pending on the stream it
    leaves, so a block freed behind pending work there is safe to reuse on the next stream."""
    l, D = gpu.lib(), gpu.DeviceBuffer
    hip = C.CDLL("libamdhip64.so")
    free0, free1, total = C.c_size_t(), C.c_size_t(), C.c_size_t()
    size = 96 << 20                      # rounds to 128 MiB (a multiple of 64 MiB)
    p = C.c_void_p()
    gpu.check(l.lten_hip_alloc(C.byref(p), size, 0))
    gpu.check(l.lten_hip_free(p))        # cached now
    gpu.sync()
    assert hip.hipMemGetInfo(C.byref(free0), C.byref(total)) == 0
    gpu.check(l.lten_hip_pool_release())
    assert hip.hipMemGetInfo(C.byref(free1), C.byref(total)) == 0
    assert free1.value >= free0.value + (128 << 20), (free0.value, free1.value)
    z = D(size, zero=True)               # a fresh block after the release
    assert not z.numpy(np.uint8, (4096,)).any()
    z.free()
    # a long fill on a caller's stream, the block freed behind it, the stream changed: the fill must have finished
    # by the time lten_hip_set_stream returns (the next user of the block may run on the other stream)
    st = C.c_void_p()
    assert hip.hipStreamCreate(C.byref(st)) == 0
    try:
        gpu.check(l.lten_hip_set_stream(st))
        n = 64 << 20
        q = C.c_void_p()
        gpu.check(l.lten_hip_alloc(C.byref(q), 4 * n, 0))
        for v in range(8):
            gpu.check(l.lten_hip_fill_i32(q, n, v))
        gpu.check(l.lten_hip_free(q))
        gpu.check(l.lten_hip_set_stream(None))
        assert hip.hipStreamQuery(st) == 0   # hipSuccess: nothing pending on the stream that was left
        r = C.c_void_p()
        gpu.check(l.lten_hip_alloc(C.byref(r), 4 * n, 0))
        assert r.value == q.value            # the same block, now used on the null stream
        gpu.check(l.lten_hip_fill_i32(r, n, -1))
        out = np.empty(n, np.int32)
        gpu.check(l.lten_hip_copy_from_gpu(out.ctypes.data, r, 4 * n))
        assert (out == -1).all()
        gpu.check(l.lten_hip_free(r))
    finally:
        gpu.check(l.lten_hip_set_stream(None))
        hip.hipStreamDestroy(st)


def test_calls_that_cannot_be_recorded_fail_with_a_message(gpu):
    """Between graph_begin and graph_end, allocation, freeing, copies, waits and the range search return an error
    that names the call; the recording survives and replays."""
    l, D = gpu.lib(), gpu.DeviceBuffer
    n = 4096
    x = D.from_numpy(np.linspace(-1, 1, n, dtype=np.float32))
    y = D(4 * n)
    host = np.empty(n, np.float32)
    p = C.c_void_p()
    lo, hi = C.c_float(), C.c_float()
    ev0, ev1 = C.c_void_p(), C.c_void_p()
    gpu.check(l.lten_hip_event_create(C.byref(ev0)))
    gpu.check(l.lten_hip_event_create(C.byref(ev1)))
    g = gpu.Graph()
    with g:
        gpu.check(l.lten_hip_relu_f32(y.ptr, x.ptr, n))
        for name, call in (("lten_hip_alloc", lambda: l.lten_hip_alloc(C.byref(p), 64, 1)),
                           ("lten_hip_free", lambda: l.lten_hip_free(x.ptr)),
                           ("lten_hip_copy_to_gpu", lambda: l.lten_hip_copy_to_gpu(y.ptr, host.ctypes.data, 4 * n)),
                           ("lten_hip_copy_from_gpu", lambda: l.lten_hip_copy_from_gpu(host.ctypes.data, y.ptr, 4 * n)),
                           ("lten_hip_copy_gpu_to_gpu", lambda: l.lten_hip_copy_gpu_to_gpu(y.ptr, x.ptr, 4 * n)),
                           ("lten_hip_sync", lambda: l.lten_hip_sync()),
                           ("lten_hip_set_stream", lambda: l.lten_hip_set_stream(None)),
                           ("lten_hip_event_elapsed_ms", lambda: l.lten_hip_event_elapsed_ms(ev0, ev1, C.byref(lo))),
                           ("lten_hip_get_min_max", lambda: l.lten_hip_get_min_max(x.ptr, n, C.byref(lo), C.byref(hi)))):
            assert call() != 0, name
            assert name.encode() in l.lten_hip_last_error(), (name, l.lten_hip_last_error())
    for _ in range(2):
        gpu.check(l.lten_hip_zero(y.ptr, 4 * n))
        g.launch()
        gpu.sync()
        assert np.array_equal(y.numpy(np.float32, (n,)), np.maximum(np.linspace(-1, 1, n, dtype=np.float32), 0))
    l.lten_hip_event_destroy(ev0)
    l.lten_hip_event_destroy(ev1)


def test_work_on_a_caller_created_stream(gpu, ob, wl):
    """lten_hip_set_stream with a real stream: one int8, one fp32 and one conv call plus a graph record / replay run on
    it and match the oracle; the null stream is restored afterwards."""
    hip = C.CDLL("libamdhip64.so")
    stream = C.c_void_p()
    assert hip.hipStreamCreate(C.byref(stream)) == 0
    l, D = gpu.lib(), gpu.DeviceBuffer
    gpu.check(l.lten_hip_set_stream(stream))
    try:
        X, W, sc, zp = wl.cfg1()
        Cg, acc = gpu.qgemm_host(X, W, sc, zp, want_acc=True)
        Co, acco = ob.quantized_matmul(X, W, sc, zp)
        assert np.array_equal(Cg, Co) and np.array_equal(acc, acco)

        rng = np.random.default_rng(3)
        A = rng.integers(-4, 5, (96, 200)).astype(np.float32)
        B = rng.integers(-4, 5, (200, 72)).astype(np.float32)
        dA, dB, dC = D.from_numpy(A), D.from_numpy(B), D(4 * 96 * 72)
        gpu.sgemm(0, 0, 96, 72, 200, 1.0, dA, 200, dB, 72, 0.0, dC, 72)
        assert np.array_equal(dC.numpy(np.float32, (96, 72)), A @ B)   # small integers: exact in any order

        geo = (2, 3, 12, 10, 5, 3, 3, 1, 1, 1, 1)
        x = rng.standard_normal((2, 3, 12, 10)).astype(np.float32)
        w = rng.standard_normal((5, 27)).astype(np.float32)
        dx, dw, dy = D.from_numpy(x), D.from_numpy(w), D(4 * 2 * 5 * 12 * 10)
        gpu.check(l.lten_hip_conv2d_forward_f32(*geo, dx.ptr, dw.ptr, None, dy.ptr))
        want = np.empty((2, 5, 12, 10), np.float32)
        col = np.empty(27 * 12 * 10, np.float32)
        ob.oracle().oracle_conv2d_forward(*geo, x.reshape(-1), w.reshape(-1), want.reshape(-1), col)
        assert rel_err(dy.numpy(np.float32, want.shape), want) < 1e-4   # the fp32 bar of the conv tests

        # record on the caller's stream, replay twice with eager work and a wait between the replays
        with gpu.Graph() as g:
            gpu.sgemm(0, 0, 96, 72, 200, 1.0, dA, 200, dB, 72, 0.0, dC, 72)
            gpu.check(l.lten_hip_relu_f32(dC.ptr, dC.ptr, 96 * 72))
        for _ in range(2):
            gpu.check(l.lten_hip_zero(dC.ptr, 4 * 96 * 72))
            g.launch()
            gpu.sync()
            assert np.array_equal(dC.numpy(np.float32, (96, 72)), np.maximum(A @ B, 0))
    finally:
        gpu.sync()
        gpu.check(l.lten_hip_set_stream(None))
        assert hip.hipStreamDestroy(stream) == 0
