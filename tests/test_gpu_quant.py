"""GPU parity tests of the quantization helpers (C ABI), bit-exact against the golden outputs of the compiled l-ten
functions and the oracle, and of a whole quantized forward pass that stays on the device."""
import ctypes as C

import numpy as np
import pytest

from conftest import golden_path

pytestmark = pytest.mark.gpu


def one_qp(gpu, scale, zp):
    return gpu.qparams3([scale, 1, 1], [int(zp), 0, 0])


def test_quantize_dequantize_golden(gpu):
    g = np.load(golden_path("quant_cases.npz"))
    data = g["data"]
    D, l = gpu.DeviceBuffer, gpu.lib()
    dd, d8, d32 = D.from_numpy(data), D(data.size), D(4 * data.size)
    codes, ddq = D.from_numpy(np.arange(256, dtype=np.uint8)), D(4 * 256)
    for i, (sc, zp) in enumerate(g["qps"]):
        qp = one_qp(gpu, sc, zp)
        gpu.check(l.lten_hip_quantize_u8(dd.ptr, d8.ptr, data.size, qp))
        gpu.check(l.lten_hip_quantize_i32(dd.ptr, d32.ptr, data.size, qp))
        gpu.check(l.lten_hip_dequantize_u8(ddq.ptr, codes.ptr, 256, qp))
        assert np.array_equal(d8.numpy(np.uint8, (data.size,)), g[f"q8_{i}"]), i
        assert np.array_equal(d32.numpy(np.int32, (data.size,)), g[f"q32_{i}"]), i
        assert np.array_equal(ddq.numpy(np.float32, (256,)), g[f"dq_{i}"]), i


def test_min_max(gpu, ob):
    rng = np.random.default_rng(4)
    D, l = gpu.DeviceBuffer, gpu.lib()
    for n in (1, 5, 1000, 1 << 20, (1 << 22) + 77):
        x = rng.standard_normal(n).astype(np.float32)
        if n > 100:
            x[7], x[n // 2] = np.nan, np.inf          # NaN elements are skipped, as in l-ten's comparisons
        lo, hi = C.c_float(), C.c_float()
        gpu.check(l.lten_hip_get_min_max(D.from_numpy(x).ptr, n, C.byref(lo), C.byref(hi)))
        wlo, whi = C.c_float(), C.c_float()
        ob.oracle().oracle_min_max(x, n, C.byref(wlo), C.byref(whi))
        assert lo.value == wlo.value and hi.value == whi.value, n
    x = np.array([np.nan, 1.0, -2.0], np.float32)     # a NaN first element stays, as in l-ten
    lo, hi = C.c_float(), C.c_float()
    gpu.check(l.lten_hip_get_min_max(D.from_numpy(x).ptr, 3, C.byref(lo), C.byref(hi)))
    assert np.isnan(lo.value) and np.isnan(hi.value)


def test_quantized_network_forward_on_device(gpu, ob):
    """The forward pass of l-ten's quantized MNIST network (tests/nn_tests.cpp:620-641, :940-942): Quantize the float
    input, Conv2d_q 1 -> 10 channels 5x5, FullyConnected_q 5760 -> 50, FullyConnected_q 50 -> 10, Dequantize; every
    tensor stays on the device.  Against the same chain of oracle functions, bit-exact."""
    rng = np.random.default_rng(12)
    B = 16
    x = rng.random((B, 1, 28, 28)).astype(np.float32)
    wc = rng.integers(0, 256, (10, 1, 5, 5), dtype=np.uint8)
    w1 = rng.integers(0, 256, (50, 5760), dtype=np.uint8)
    w2 = rng.integers(0, 256, (10, 50), dtype=np.uint8)
    b1 = rng.integers(-3000, 3000, 50).astype(np.int32)
    b2 = rng.integers(-300, 300, 10).astype(np.int32)
    q_in, q_c, q_1, q_2 = (1 / 255, 0), (0.02, 120), (0.9, 131), (7.0, 99)      # activations
    qw_c, qw_1, qw_2 = (0.01, 128), (0.004, 125), (0.01, 130)                    # weights
    geo = (B, 1, 28, 28, 10, 5, 5, 0, 0, 1, 1)
    # oracle chain
    xq = np.empty(x.size, np.uint8)
    ob.oracle().oracle_quantize_u8(x.reshape(-1), xq, x.size, ob.qparams3([q_in[0], 1, 1], [q_in[1], 0, 0]))
    yc, _ = ob.conv2dq_forward(geo, xq.reshape(x.shape), wc, [q_in[0], qw_c[0], q_c[0]], [q_in[1], qw_c[1], q_c[1]], want_acc=False)
    h1, _ = ob.quantized_matmul(yc.reshape(B, 5760), w1, [q_c[0], qw_1[0], q_1[0]], [q_c[1], qw_1[1], q_1[1]], bias=b1)
    h2, _ = ob.quantized_matmul(h1, w2, [q_1[0], qw_2[0], q_2[0]], [q_1[1], qw_2[1], q_2[1]], bias=b2)
    want = np.empty(h2.size, np.float32)
    ob.oracle().oracle_dequantize_u8(want, np.ascontiguousarray(h2).reshape(-1), h2.size, ob.qparams3([q_2[0], 1, 1], [q_2[1], 0, 0]))
    # device chain
    D, l = gpu.DeviceBuffer, gpu.lib()
    dx, dxq = D.from_numpy(x), D(x.size)
    dwc, dw1, dw2, db1, db2 = D.from_numpy(wc), D.from_numpy(w1), D.from_numpy(w2), D.from_numpy(b1), D.from_numpy(b2)
    dyc, dh1, dh2, dout = D(B * 5760), D(B * 50), D(B * 10), D(4 * B * 10)
    wsc = D(max(int(l.lten_hip_conv2dq_workspace_bytes(*geo)), 16))
    ws = D(4 * (B + 5760))
    gpu.check(l.lten_hip_quantize_u8(dx.ptr, dxq.ptr, x.size, one_qp(gpu, *q_in)))
    gpu.check(l.lten_hip_conv2dq_forward(*geo, dxq.ptr, dwc.ptr, None, gpu.qparams3([q_in[0], qw_c[0], q_c[0]], [q_in[1], qw_c[1], q_c[1]]), dyc.ptr, wsc.ptr))
    gpu.check(l.lten_hip_fcq_forward(1, B, 5760, 50, dyc.ptr, dw1.ptr, db1.ptr, gpu.qparams3([q_c[0], qw_1[0], q_1[0]], [q_c[1], qw_1[1], q_1[1]]), dh1.ptr, ws.ptr))
    gpu.check(l.lten_hip_fcq_forward(1, B, 50, 10, dh1.ptr, dw2.ptr, db2.ptr, gpu.qparams3([q_1[0], qw_2[0], q_2[0]], [q_1[1], qw_2[1], q_2[1]]), dh2.ptr, ws.ptr))
    gpu.check(l.lten_hip_dequantize_u8(dout.ptr, dh2.ptr, B * 10, one_qp(gpu, *q_2)))
    assert np.array_equal(dxq.numpy(np.uint8, (x.size,)), xq)
    assert np.array_equal(dyc.numpy(np.uint8, yc.shape), yc)
    assert np.array_equal(dh1.numpy(np.uint8, h1.shape), h1)
    assert np.array_equal(dh2.numpy(np.uint8, h2.shape), h2)
    assert np.array_equal(dout.numpy(np.float32, (B * 10,)), want)
