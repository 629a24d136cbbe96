"""ctypes front of liblten_hip.so — the C ABI declared in include/lten_hip.h.

This module is plumbing for tests and measurements: it owns no arithmetic.  Every
function here ends in a call through the C ABI into the HIP library; there is no CPU
fallback, and importing `lib()` fails loudly when the library has not been built.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liblten_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(HERE), "include", "lten_hip.h")


class LtenHipError(RuntimeError):
    """A non-zero status from the C ABI (what the C++ glue turns into LTEN_ERR)."""


class QParams(C.Structure):
    """l-ten's QuantizationParams (l-ten/math_fns.h:12-16)."""
    _fields_ = [("scale", C.c_float), ("zero_point", C.c_uint8)]


u64 = C.c_uint64
i64 = C.c_int64
vp = C.c_void_p

_SIGNATURES = {
    "lten_hip_init": (C.c_int, [C.c_int]),
    "lten_hip_last_error": (C.c_char_p, []),
    "lten_hip_last_kernel": (C.c_char_p, []),
    "lten_hip_get_device": (C.c_int, [C.POINTER(C.c_int)]),
    "lten_hip_set_stream": (C.c_int, [vp]),
    "lten_hip_sync": (C.c_int, []),
    "lten_hip_alloc": (C.c_int, [C.POINTER(vp), u64, C.c_int]),
    "lten_hip_pool_release": (C.c_int, []),
    "lten_hip_free": (C.c_int, [vp]),
    "lten_hip_zero": (C.c_int, [vp, C.c_size_t]),
    "lten_hip_copy_to_gpu": (C.c_int, [vp, vp, C.c_size_t]),
    "lten_hip_copy_from_gpu": (C.c_int, [vp, vp, C.c_size_t]),
    "lten_hip_copy_gpu_to_gpu": (C.c_int, [vp, vp, C.c_size_t]),
    "lten_hip_fill_f32": (C.c_int, [vp, u64, C.c_float]),
    "lten_hip_fill_i32": (C.c_int, [vp, u64, C.c_int32]),
    "lten_hip_fill_u8": (C.c_int, [vp, u64, C.c_uint8]),
    "lten_hip_sgemm": (C.c_int, [C.c_int, C.c_int, u64, u64, u64, C.c_float, vp, u64, vp, u64, C.c_float, vp, u64]),
    "lten_hip_sgemm_strided_batched": (C.c_int, [C.c_int, C.c_int, u64, u64, u64, C.c_float, vp, u64, i64, vp, u64,
                                                 i64, C.c_float, vp, u64, i64, u64]),
    "lten_hip_fc_forward_f32": (C.c_int, [u64, u64, u64, vp, vp, vp, vp]),
    "lten_hip_fc_backward_f32": (C.c_int, [u64, u64, u64, vp, vp, vp, vp, vp, vp]),
    "lten_hip_quantized_matmul": (C.c_int, [C.c_int, C.c_int, u64, u64, u64, C.c_uint8, vp, vp, C.c_uint8, vp,
                                            C.POINTER(QParams), vp, vp]),
    "lten_hip_quantized_matmul_acc": (C.c_int, [C.c_int, C.c_int, u64, u64, u64, vp, vp, vp, C.POINTER(QParams), vp,
                                                vp]),
    "lten_hip_fcq_forward": (C.c_int, [u64, u64, u64, u64, vp, vp, vp, C.POINTER(QParams), vp, vp]),
    "lten_hip_fcq_forward_prepared": (C.c_int, [u64, u64, u64, u64, vp, vp, vp, vp, C.POINTER(QParams), vp, vp]),
    "lten_hip_fcq_prepare_weights": (C.c_int, [vp, vp, u64, u64, vp]),
    "lten_hip_fcq_forward_static": (C.c_int, [u64, u64, u64, u64, vp, vp, vp, C.POINTER(QParams), vp]),
    "lten_hip_im2col_f32": (C.c_int, [vp] + [C.c_int] * 11 + [vp]),
    "lten_hip_im2col_i32": (C.c_int, [vp] + [C.c_int] * 11 + [vp]),
    "lten_hip_col2im_i32": (C.c_int, [vp] + [C.c_int] * 11 + [vp]),
    "lten_hip_col2im_u8": (C.c_int, [vp] + [C.c_int] * 11 + [vp]),
    "lten_hip_im2col_u8": (C.c_int, [vp] + [C.c_int] * 11 + [vp]),
    "lten_hip_col2im_f32": (C.c_int, [vp] + [C.c_int] * 11 + [vp]),
    "lten_hip_conv2d_forward_f32": (C.c_int, [u64] * 5 + [C.c_int] * 6 + [vp, vp, vp, vp]),
    "lten_hip_conv2d_wgrad_f32": (C.c_int, [u64] * 5 + [C.c_int] * 6 + [vp, vp, vp, vp]),
    "lten_hip_conv2d_wgrad_workspace_bytes": (u64, [u64] * 5 + [C.c_int] * 6),
    "lten_hip_conv2d_dgrad_f32": (C.c_int, [u64] * 5 + [C.c_int] * 6 + [vp, vp, vp, vp]),
    "lten_hip_conv2d_dgrad_workspace_bytes": (u64, [u64] * 5 + [C.c_int] * 6),
    "lten_hip_conv2dq_workspace_bytes": (u64, [u64] * 5 + [C.c_int] * 6),
    "lten_hip_conv2dq_forward": (C.c_int, [u64] * 5 + [C.c_int] * 6 + [vp, vp, vp, C.POINTER(QParams), vp, vp]),
    "lten_hip_conv2dq_forward_acc": (C.c_int, [u64] * 5 + [C.c_int] * 6 + [vp, vp, vp, C.POINTER(QParams), vp, vp]),
    "lten_hip_fc_forward_relu_f32": (C.c_int, [u64, u64, u64, vp, vp, vp, vp, vp]),
    "lten_hip_fc_backward_relu_f32": (C.c_int, [u64, u64, u64, vp, vp, vp, vp, vp, vp, vp]),
    "lten_hip_log_softmax_nll_loss_f32": (C.c_int, [u64, u64, vp, vp, vp, vp]),
    "lten_hip_nll_log_softmax_backward_f32": (C.c_int, [u64, u64, vp, vp, C.c_float, vp]),
    "lten_hip_log_softmax_nll_loss_grad_f32": (C.c_int, [u64, u64, vp, vp, C.c_float, vp, vp, vp]),
    "lten_hip_fc_backward_log_softmax_nll_loss_f32": (C.c_int, [u64, u64, u64, vp, vp, vp, vp, C.c_float, vp, vp, vp, vp, vp, vp, vp]),
    "lten_hip_relu_f32": (C.c_int, [vp, vp, u64]),
    "lten_hip_relu_backward_f32": (C.c_int, [vp, vp, vp, u64]),
    "lten_hip_scale_f32": (C.c_int, [u64, C.c_float, vp, vp]),
    "lten_hip_axpy_f32": (C.c_int, [u64, C.c_float, vp, vp]),
    "lten_hip_log_softmax_f32": (C.c_int, [u64, u64, vp, vp]),
    "lten_hip_log_softmax_backward_f32": (C.c_int, [u64, u64, vp, vp, vp]),
    "lten_hip_nll_loss_f32": (C.c_int, [vp, vp, vp, u64, u64]),
    "lten_hip_sgd_step_f32": (C.c_int, [vp, vp, vp, u64, C.c_float, C.c_float, C.c_float]),
    "lten_hip_adam_step_f32": (C.c_int, [vp, vp, vp, vp, u64, C.c_float, C.c_float, C.c_float, u64]),
    "lten_hip_quantize_u8": (C.c_int, [vp, vp, u64, C.POINTER(QParams)]),
    "lten_hip_quantize_i32": (C.c_int, [vp, vp, u64, C.POINTER(QParams)]),
    "lten_hip_dequantize_u8": (C.c_int, [vp, vp, u64, C.POINTER(QParams)]),
    "lten_hip_get_min_max": (C.c_int, [vp, u64, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "lten_hip_conv2d_bias_grad_f32": (C.c_int, [u64, u64, u64, vp, vp, C.c_int]),
    "lten_hip_graph_begin": (C.c_int, []),
    "lten_hip_graph_end": (C.c_int, [C.POINTER(vp)]),
    "lten_hip_graph_launch": (C.c_int, [vp]),
    "lten_hip_graph_destroy": (C.c_int, [vp]),
    "lten_hip_event_create": (C.c_int, [C.POINTER(vp)]),
    "lten_hip_event_record": (C.c_int, [vp]),
    "lten_hip_event_elapsed_ms": (C.c_int, [vp, vp, C.POINTER(C.c_float)]),
    "lten_hip_event_destroy": (C.c_int, [vp]),
    "lten_hip_set_option": (C.c_int, [C.c_char_p, C.c_int]),
}

# The calibration library (include/lten_hip_measure.h): not part of the drop-in surface, loaded on first use.
MEASURE_LIB_PATH = os.path.join(HERE, "liblten_hip_measure.so")
MEASURE_HEADER_PATH = os.path.join(os.path.dirname(HERE), "include", "lten_hip_measure.h")
_MEASURE_SIGNATURES = {
    "lten_measure_last_error": (C.c_char_p, []),
    "lten_measure_mfma_peak": (C.c_int, [C.c_int, C.c_int, C.POINTER(C.c_float)]),
    "lten_measure_mfma_peak_operands": (C.c_int, [vp, vp, u64, C.c_int, C.POINTER(C.c_float)]),
    "lten_measure_last_clocks": (C.c_int, [C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "lten_measure_copy": (C.c_int, [vp, vp, u64]),
}
_measure_lib = None


def measure_lib():
    global _measure_lib
    if _measure_lib is None:
        if not os.path.exists(MEASURE_LIB_PATH):
            raise LtenHipError(f"{MEASURE_LIB_PATH} is missing: build it with `python light-tensor_amd/build.py`")
        m = C.CDLL(MEASURE_LIB_PATH)
        for name, (res, args) in _MEASURE_SIGNATURES.items():
            fn = getattr(m, name)
            fn.restype, fn.argtypes = res, args
        _measure_lib = m
    return _measure_lib


def _mcheck(rc):
    if rc != 0:
        raise LtenHipError(measure_lib().lten_measure_last_error().decode())

_lib = None


def declared_symbols():
    """Names of the functions include/lten_hip.h declares."""
    import re
    text = open(HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lten_hip_[a-z0-9_]+)\s*\(", text)))


def lib():
    """The loaded C-ABI library.  Raises when it has not been built: there is no other path."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LtenHipError(f"{LIB_PATH} is missing: build it with `python light-tensor_amd/build.py` "
                           "(there is no CPU fallback)")
    l = C.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(l, name)  # AttributeError here = the library is older than the header
        fn.restype = res
        fn.argtypes = args
    _lib = l
    return l


def check(rc):
    if rc != 0:
        raise LtenHipError(lib().lten_hip_last_error().decode())


def init(device=0):
    check(lib().lten_hip_init(device))


def sync():
    check(lib().lten_hip_sync())


def last_kernel():
    return lib().lten_hip_last_kernel().decode()


def set_option(name, value):
    check(lib().lten_hip_set_option(name.encode(), int(value)))


def measure_mfma_peak(kind=0, waves_per_simd=1):
    out = C.c_float()
    _mcheck(measure_lib().lten_measure_mfma_peak(kind, waves_per_simd, C.byref(out)))
    return out.value


def measure_mfma_peak_operands(a_u8, b_i8, nbytes, waves_per_simd=1):
    """int8 MFMA-only rate on operands drawn from two device buffers (uint8 activations, prepared int8 weights)."""
    out = C.c_float()
    _mcheck(measure_lib().lten_measure_mfma_peak_operands(a_u8.ptr, b_i8.ptr, nbytes, waves_per_simd, C.byref(out)))
    return out.value


def measure_last_clocks():
    a, b = C.c_double(), C.c_double()
    _mcheck(measure_lib().lten_measure_last_clocks(C.byref(a), C.byref(b)))
    return a.value, b.value


def measure_copy(src, dst, nbytes):
    _mcheck(measure_lib().lten_measure_copy(src.ptr, dst.ptr, nbytes))


def qparams3(scales, zps):
    arr = (QParams * 3)()
    for i in range(3):
        arr[i].scale = float(np.float32(scales[i]))
        arr[i].zero_point = int(zps[i])
    return arr


class DeviceBuffer:
    """A device allocation owned by Python; `.ptr` is the raw device address."""

    def __init__(self, nbytes, zero=False):
        p = vp()
        check(lib().lten_hip_alloc(C.byref(p), int(nbytes), int(zero)))
        self.ptr = p.value
        self.nbytes = int(nbytes)

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        check(lib().lten_hip_copy_to_gpu(buf.ptr, a.ctypes.data, a.nbytes))
        return buf

    def upload(self, a, offset=0):
        a = np.ascontiguousarray(a)
        assert offset + a.nbytes <= self.nbytes
        check(lib().lten_hip_copy_to_gpu(self.ptr + offset, a.ctypes.data, a.nbytes))

    def numpy(self, dtype, shape, offset=0):
        out = np.empty(shape, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        check(lib().lten_hip_copy_from_gpu(out.ctypes.data, self.ptr + offset, out.nbytes))
        return out

    def at(self, offset):
        return self.ptr + offset

    def free(self):
        if self.ptr:
            lib().lten_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Timer:
    """HIP events on the library's stream."""

    def __init__(self):
        self.e0, self.e1 = vp(), vp()
        check(lib().lten_hip_event_create(C.byref(self.e0)))
        check(lib().lten_hip_event_create(C.byref(self.e1)))

    def start(self):
        check(lib().lten_hip_event_record(self.e0))

    def stop_ms(self):
        check(lib().lten_hip_event_record(self.e1))
        return self.elapsed_ms()

    def record_stop(self):
        check(lib().lten_hip_event_record(self.e1))

    def elapsed_ms(self):
        """Milliseconds between the two recorded events (waits for the second one)."""
        ms = C.c_float()
        check(lib().lten_hip_event_elapsed_ms(self.e0, self.e1, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            lib().lten_hip_event_destroy(self.e0)
            lib().lten_hip_event_destroy(self.e1)
        except Exception:
            pass


class Graph:
    """A recorded sequence of compute calls: `with Graph() as g: <calls>` records, g.launch() replays.
    The buffers the calls named must stay allocated at the same addresses."""

    def __init__(self):
        self.handle = vp()

    def __enter__(self):
        check(lib().lten_hip_graph_begin())
        return self

    def __exit__(self, exc_type, exc, tb):
        rc = lib().lten_hip_graph_end(C.byref(self.handle))
        if exc_type is None:
            check(rc)
        return False

    def launch(self):
        check(lib().lten_hip_graph_launch(self.handle))

    def __del__(self):
        try:
            if self.handle:
                lib().lten_hip_graph_destroy(self.handle)
        except Exception:
            pass


# ----------------------------------------------------------------------- thin call wrappers

def _p(x):
    if x is None:
        return None
    return x.ptr if isinstance(x, DeviceBuffer) else x


def quantized_matmul(tA, tB, M, N, K, A, B, Cq, qp, bias=None, workspace=None, alpha=1, beta=0):
    check(lib().lten_hip_quantized_matmul(int(tA), int(tB), M, N, K, alpha, _p(A), _p(B), beta, _p(Cq), qp, _p(bias),
                                          _p(workspace)))


def quantized_matmul_acc(tA, tB, M, N, K, A, B, acc, qp, bias=None, workspace=None):
    check(lib().lten_hip_quantized_matmul_acc(int(tA), int(tB), M, N, K, _p(A), _p(B), _p(acc), qp, _p(bias),
                                              _p(workspace)))


def sgemm(tA, tB, M, N, K, alpha, A, lda, B, ldb, beta, Cm, ldc):
    check(lib().lten_hip_sgemm(int(tA), int(tB), M, N, K, alpha, _p(A), lda, _p(B), ldb, beta, _p(Cm), ldc))


def qgemm_host(A, B, scales, zps, tA=False, tB=True, bias=None, want_acc=False, M=None, N=None, K=None):
    """numpy in / numpy out convenience around lten_hip_quantized_matmul[_acc] (copies included)."""
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    if M is None:
        M, K = (A.shape[1], A.shape[0]) if tA else A.shape
        N = B.shape[0] if tB else B.shape[1]
    dA, dB = DeviceBuffer.from_numpy(A), DeviceBuffer.from_numpy(B)
    dbias = DeviceBuffer.from_numpy(np.asarray(bias, dtype=np.int32)) if bias is not None else None
    ws = DeviceBuffer(4 * (M + N))
    qp = qparams3(scales, zps)
    dC = DeviceBuffer(max(M * N, 1))
    quantized_matmul(tA, tB, M, N, K, dA, dB, dC, qp, dbias, ws)
    out = dC.numpy(np.uint8, (M, N))
    acc = None
    if want_acc:
        dacc = DeviceBuffer(max(4 * M * N, 4))
        quantized_matmul_acc(tA, tB, M, N, K, dA, dB, dacc, qp, dbias, ws)
        acc = dacc.numpy(np.int32, (M, N))
    return out, acc


def conv2dq_host(geo, x, w, scales, zps, bias=None, want_acc=False):
    """numpy in / numpy out convenience around lten_hip_conv2dq_forward[_acc]; scales / zps ordered (input, weights,
    output); geo = (N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw).  Copies included."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    Ho, Wo = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    dx = DeviceBuffer.from_numpy(np.ascontiguousarray(x, dtype=np.uint8))
    dw = DeviceBuffer.from_numpy(np.ascontiguousarray(w, dtype=np.uint8))
    db = DeviceBuffer.from_numpy(np.asarray(bias, dtype=np.int32)) if bias is not None else None
    ws = DeviceBuffer(max(int(lib().lten_hip_conv2dq_workspace_bytes(*geo)), 16))
    qp = qparams3(scales, zps)
    count = N * Cout * Ho * Wo
    dy = DeviceBuffer(max(count, 1))
    check(lib().lten_hip_conv2dq_forward(*geo, dx.ptr, dw.ptr, _p(db), qp, dy.ptr, ws.ptr))
    out = dy.numpy(np.uint8, (N, Cout, Ho, Wo))
    acc = None
    if want_acc:
        dacc = DeviceBuffer(max(4 * count, 4))
        check(lib().lten_hip_conv2dq_forward_acc(*geo, dx.ptr, dw.ptr, _p(db), qp, dacc.ptr, ws.ptr))
        acc = dacc.numpy(np.int32, (N, Cout, Ho, Wo))
    return out, acc
