"""CPU tests of the oracle's quantization helpers (l-ten/utils.cpp:198-286) against the golden outputs of the compiled
l-ten functions and against closed forms."""
import ctypes as C

import numpy as np

from conftest import golden_path


def test_quantize_dequantize_golden(ob):
    g = np.load(golden_path("quant_cases.npz"))
    data = g["data"]
    for i, (sc, zp) in enumerate(g["qps"]):
        qp = ob.qparams3([sc, 1, 1], [int(zp), 0, 0])
        q8, q32 = np.empty(data.size, np.uint8), np.empty(data.size, np.int32)
        ob.oracle().oracle_quantize_u8(data, q8, data.size, qp)
        ob.oracle().oracle_quantize_i32(data, q32, data.size, qp)
        assert np.array_equal(q8, g[f"q8_{i}"]), i
        assert np.array_equal(q32, g[f"q32_{i}"]), i
        dq = np.empty(256, np.float32)
        ob.oracle().oracle_dequantize_u8(dq, np.arange(256, dtype=np.uint8), 256, qp)
        assert np.array_equal(dq, g[f"dq_{i}"]), i


def test_qparams_and_minmax_golden(ob):
    g = np.load(golden_path("quant_cases.npz"))
    for lo, hi, sc, zp in g["qparam_cases"]:
        qp = ob.qparams3([1, 1, 1], [0, 0, 0])
        ob.oracle().oracle_compute_qparams(float(lo), float(hi), qp)
        assert qp[0].scale == np.float32(sc) and qp[0].zero_point == int(zp), (lo, hi)
    data = g["data"]
    finite = np.ascontiguousarray(data[np.isfinite(data)])
    lo, hi = C.c_float(), C.c_float()
    ob.oracle().oracle_min_max(finite, finite.size, C.byref(lo), C.byref(hi))
    assert lo.value == g["minmax"][0] == finite.min() and hi.value == g["minmax"][1] == finite.max()


def test_quantize_closed_forms(ob):
    # scale 1, zero point 0: round half away from zero, clamped to [0, 255]
    x = np.array([0.49, 0.5, 1.5, 2.5, 254.4, 254.5, 300.0, -0.4, -0.6, -5.0], np.float32)
    q = np.empty(x.size, np.uint8)
    ob.oracle().oracle_quantize_u8(x, q, x.size, ob.qparams3([1, 1, 1], [0, 0, 0]))
    assert q.tolist() == [0, 1, 2, 3, 254, 255, 255, 0, 0, 0]
    # dequantize(quantize(x)) is within half a step for in-range x
    rng = np.random.default_rng(1)
    x = rng.uniform(-3, 5, 2000).astype(np.float32)
    qp = ob.qparams3([1, 1, 1], [0, 0, 0])
    ob.oracle().oracle_compute_qparams(-3.0, 5.0, qp)
    q, back = np.empty(x.size, np.uint8), np.empty(x.size, np.float32)
    ob.oracle().oracle_quantize_u8(x, q, x.size, qp)
    ob.oracle().oracle_dequantize_u8(back, q, x.size, qp)
    assert np.abs(back - x).max() <= qp[0].scale * 0.5001 + qp[0].scale   # zero point rounding adds at most one step
