"""TEST INFRASTRUCTURE ONLY: ctypes doors into the CPU oracle and the compiled reference.

`oracle()` loads oracle/liblten_oracle.so (built by `make -C oracle`); `ref()` loads
oracle/_ref/liblten_ref.so when it exists (built by `make -C oracle ref` where the l-ten
sources are present) and returns None otherwise.  Only tests/, the smoke check and the
benchmark's cpu_baseline leg import this module; the product package never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "liblten_oracle.so")
REF_SO = os.path.join(HERE, "_ref", "liblten_ref.so")

u8p = np.ctypeslib.ndpointer(dtype=np.uint8, flags="C_CONTIGUOUS")
i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
u64p = np.ctypeslib.ndpointer(dtype=np.uint64, flags="C_CONTIGUOUS")
u64 = C.c_uint64


class QParams(C.Structure):
    """Layout of l-ten's QuantizationParams (l-ten/math_fns.h:12-16)."""
    _fields_ = [("scale", C.c_float), ("zero_point", C.c_uint8)]


def qparams3(scales, zps):
    arr = (QParams * 3)()
    for i in range(3):
        arr[i].scale = float(np.float32(scales[i]))
        arr[i].zero_point = int(zps[i])
    return arr


_FPP = C.POINTER(C.POINTER(C.c_float))
_MLP_ARGS = [C.c_uint64, C.c_int, C.POINTER(C.c_uint64), C.POINTER(C.c_float), _FPP, _FPP, C.POINTER(C.c_float),
             C.POINTER(C.c_float), C.POINTER(C.c_float), _FPP, _FPP, C.POINTER(C.c_float)]


def _opt(a, ctype):
    return None if a is None else a.ctypes.data_as(C.POINTER(ctype))


def build_oracle():
    subprocess.run(["make", "-C", HERE, "-s"], check=True)


_oracle = None
_ref = None
_ref_tried = False


def oracle():
    global _oracle
    if _oracle is not None:
        return _oracle
    if not os.path.exists(ORACLE_SO):
        build_oracle()
    lib = C.CDLL(ORACLE_SO)
    lib.oracle_requantize.restype = C.c_uint8
    lib.oracle_requantize.argtypes = [C.c_float, C.c_int32, C.c_uint8]
    lib.oracle_real_multiplier.restype = C.c_float
    lib.oracle_real_multiplier.argtypes = [C.c_float] * 3
    lib.oracle_quantized_matmul.restype = C.c_int
    lib.oracle_quantized_matmul.argtypes = [C.c_int, C.c_int, u64, u64, u64, C.c_uint8, u8p, u8p, C.c_uint8, u8p,
                                            C.POINTER(QParams), C.POINTER(C.c_int32), i32p, C.POINTER(C.c_int32)]
    sg = [C.c_int, C.c_int, u64, u64, u64, C.c_float, f32p, u64, f32p, u64, C.c_float, f32p, u64]
    lib.oracle_sgemm.restype = None
    lib.oracle_sgemm.argtypes = sg
    lib.oracle_sgemm_f64.restype = None
    lib.oracle_sgemm_f64.argtypes = sg
    lib.oracle_sgemm_mt.restype = None
    lib.oracle_sgemm_mt.argtypes = sg + [C.c_int]
    geo = [u64] * 9
    lib.oracle_im2col_f32.restype = None
    lib.oracle_im2col_f32.argtypes = [f32p] + geo + [f32p]
    lib.oracle_im2col_u8.restype = None
    lib.oracle_im2col_u8.argtypes = [u8p] + geo + [u8p]
    lib.oracle_col2im_f32.restype = None
    lib.oracle_col2im_f32.argtypes = [f32p] + geo + [f32p]
    fp = C.POINTER(C.c_float)
    lib.oracle_fc_forward.restype = None
    lib.oracle_fc_forward.argtypes = [u64, u64, u64, f32p, f32p, fp, f32p]
    lib.oracle_fc_backward.restype = None
    lib.oracle_fc_backward.argtypes = [u64, u64, u64, f32p, f32p, f32p, fp, fp, fp]
    lib.oracle_fcq_forward.restype = C.c_int
    lib.oracle_fcq_forward.argtypes = [u64, u64, u64, u64, u8p, u8p, C.POINTER(C.c_int32), C.POINTER(QParams), u8p]
    lib.oracle_matmul.restype = C.c_int
    lib.oracle_matmul.argtypes = [C.c_int, u64p, u64p, f32p, f32p, u64p, f32p]
    lib.oracle_matmul_backward.restype = C.c_int
    lib.oracle_matmul_backward.argtypes = [C.c_int, u64p, u64p, f32p, f32p, f32p, fp, fp]
    conv = [u64] * 11
    for name in ("oracle_conv2d_forward", "oracle_conv2d_wgrad", "oracle_conv2d_dgrad"):
        getattr(lib, name).restype = None
        getattr(lib, name).argtypes = conv + [f32p, f32p, f32p, f32p]
    lib.oracle_relu.restype = None
    lib.oracle_relu.argtypes = [f32p, f32p, u64]
    lib.oracle_relu_backward.restype = None
    lib.oracle_relu_backward.argtypes = [f32p, f32p, f32p, u64]
    lib.oracle_log_softmax.restype = None
    lib.oracle_log_softmax.argtypes = [u64, u64, f32p, f32p]
    lib.oracle_log_softmax_backward.restype = None
    lib.oracle_log_softmax_backward.argtypes = [u64, u64, f32p, f32p, f32p]
    lib.oracle_nll_loss.restype = C.c_float
    lib.oracle_nll_loss.argtypes = [f32p, f32p, u64, u64]
    lib.oracle_nll_backward.restype = None
    lib.oracle_nll_backward.argtypes = [f32p, u64, u64, C.c_float, f32p]
    lib.oracle_mlp_step.restype = C.c_int
    lib.oracle_mlp_step.argtypes = _MLP_ARGS
    lib.oracle_min_max.restype = None
    lib.oracle_min_max.argtypes = [f32p, u64, C.POINTER(C.c_float), C.POINTER(C.c_float)]
    lib.oracle_compute_qparams.restype = None
    lib.oracle_compute_qparams.argtypes = [C.c_float, C.c_float, C.POINTER(QParams)]
    lib.oracle_quantize_u8.restype = None
    lib.oracle_quantize_u8.argtypes = [f32p, u8p, u64, C.POINTER(QParams)]
    lib.oracle_quantize_i32.restype = None
    lib.oracle_quantize_i32.argtypes = [f32p, i32p, u64, C.POINTER(QParams)]
    lib.oracle_dequantize_u8.restype = None
    lib.oracle_dequantize_u8.argtypes = [f32p, u8p, u64, C.POINTER(QParams)]
    lib.oracle_sgd_step.restype = None
    lib.oracle_sgd_step.argtypes = [f32p, f32p, f32p, u64, C.c_float, C.c_float, C.c_float]
    lib.oracle_adam_step.restype = None
    lib.oracle_adam_step.argtypes = [f32p, f32p, f32p, f32p, u64, C.c_float, C.c_float, C.c_float, u64]
    lib.oracle_conv2dq_forward.restype = C.c_int
    lib.oracle_conv2dq_forward.argtypes = conv + [u8p, u8p, C.POINTER(C.c_int32), C.POINTER(QParams), u8p, C.POINTER(C.c_int32)]
    _oracle = lib
    return lib


def ref():
    """The compiled l-ten CPU path, or None where it has not been built."""
    global _ref, _ref_tried
    if _ref_tried:
        return _ref
    _ref_tried = True
    if not os.path.exists(REF_SO):
        return None
    lib = C.CDLL(REF_SO)
    lib.ref_quantized_matmul.restype = C.c_int
    lib.ref_quantized_matmul.argtypes = [C.c_int, C.c_int, u64, u64, u64, C.c_uint8, u8p, u8p, C.c_uint8, u8p,
                                         f32p, u8p, C.POINTER(C.c_int32), i32p]
    lib.ref_cpu_gemm_f32.restype = C.c_int
    lib.ref_cpu_gemm_f32.argtypes = [C.c_int, C.c_int, u64, u64, u64, C.c_float, f32p, f32p, C.c_float, f32p]
    geo = [u64] * 9
    lib.ref_im2col_f32.restype = None
    lib.ref_im2col_f32.argtypes = [f32p] + geo + [f32p]
    lib.ref_col2im_f32.restype = None
    lib.ref_col2im_f32.argtypes = [f32p] + geo + [f32p]
    lib.ref_im2col_u8.restype = None
    lib.ref_im2col_u8.argtypes = [u8p] + geo + [u8p]
    fp = C.POINTER(C.c_float)
    lib.ref_fc_f32.restype = C.c_int
    lib.ref_fc_f32.argtypes = [u64, u64, u64, f32p, f32p, fp, fp, fp, fp, fp, fp]
    lib.ref_fcq_u8.restype = C.c_int
    lib.ref_fcq_u8.argtypes = [u64, u64, u64, u64, u8p, u8p, C.POINTER(C.c_int32), f32p, u8p, u8p]
    lib.ref_conv2d_f32.restype = C.c_int
    lib.ref_conv2d_f32.argtypes = [u64] * 5 + [C.c_int] * 6 + [f32p, f32p, fp, fp, fp, fp]
    lib.ref_min_max.restype = None
    lib.ref_min_max.argtypes = [f32p, u64, C.POINTER(C.c_float), C.POINTER(C.c_float)]
    lib.ref_compute_qparams.restype = None
    lib.ref_compute_qparams.argtypes = [C.c_float, C.c_float, C.POINTER(C.c_float), C.POINTER(C.c_uint8)]
    lib.ref_quantize_u8.restype = None
    lib.ref_quantize_u8.argtypes = [f32p, u8p, u64, C.c_float, C.c_uint8]
    lib.ref_quantize_i32.restype = None
    lib.ref_quantize_i32.argtypes = [f32p, i32p, u64, C.c_float, C.c_uint8]
    lib.ref_dequantize_u8.restype = None
    lib.ref_dequantize_u8.argtypes = [f32p, u8p, u64, C.c_float, C.c_uint8]
    lib.ref_optimizer_steps.restype = C.c_int
    lib.ref_optimizer_steps.argtypes = [C.c_int, u64, C.c_int, f32p, f32p, f32p]
    lib.ref_mlp_step.restype = C.c_int
    lib.ref_mlp_step.argtypes = _MLP_ARGS
    lib.ref_conv2dq_u8.restype = C.c_int
    lib.ref_conv2dq_u8.argtypes = [u64] * 5 + [C.c_int] * 6 + [u8p, u8p, f32p, u8p, u8p]
    lib.ref_matmul_f32.restype = C.c_int
    lib.ref_matmul_f32.argtypes = [C.c_int, u64p, u64p, f32p, f32p, fp, fp, fp, fp]
    lib.ref_hardware_threads.restype = C.c_int
    _ref = lib
    return lib


# ----------------------------------------------------------------- numpy-level helpers

def quantized_matmul(A, B, scales, zps, tA=False, tB=True, bias=None, M=None, N=None, K=None, want_acc=True):
    """Oracle quantized_matmul on numpy arrays; returns (C u8 [M,N], acc i32 [M,N] or None)."""
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    if M is None:
        M, K = (A.shape[1], A.shape[0]) if tA else A.shape
        N = B.shape[0] if tB else B.shape[1]
    Cq = np.empty((M, N), dtype=np.uint8)
    acc = np.empty((M, N), dtype=np.int32) if want_acc else None
    ws = np.empty(M + N, dtype=np.int32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    rc = oracle().oracle_quantized_matmul(int(tA), int(tB), M, N, K, 1, A.reshape(-1), B.reshape(-1), 0,
                                          Cq.reshape(-1), qparams3(scales, zps), _opt(b, C.c_int32), ws,
                                          _opt(acc, C.c_int32))
    assert rc == 0
    return Cq, acc


def ref_quantized_matmul(A, B, scales, zps, tA=False, tB=True, bias=None, M=None, N=None, K=None):
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    if M is None:
        M, K = (A.shape[1], A.shape[0]) if tA else A.shape
        N = B.shape[0] if tB else B.shape[1]
    Cq = np.empty((M, N), dtype=np.uint8)
    ws = np.empty(M + N, dtype=np.int32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    rc = ref().ref_quantized_matmul(int(tA), int(tB), M, N, K, 1, A.reshape(-1), B.reshape(-1), 0, Cq.reshape(-1),
                                    np.asarray(scales, dtype=np.float32), np.asarray(zps, dtype=np.uint8),
                                    _opt(b, C.c_int32), ws)
    assert rc == 0
    return Cq


def sgemm(tA, tB, M, N, K, alpha, A, lda, B, ldb, beta, Cm, ldc, f64=False):
    """In-place oracle sgemm on flat fp32 arrays; returns Cm."""
    fn = oracle().oracle_sgemm_f64 if f64 else oracle().oracle_sgemm
    fn(int(tA), int(tB), M, N, K, alpha, A.reshape(-1), lda, B.reshape(-1), ldb, beta, Cm.reshape(-1), ldc)
    return Cm


def conv_out_hw(H, W, kh, kw, ph, pw, sh, sw):
    return (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1


def conv2dq_forward(geo, x, w, scales, zps, bias=None, want_acc=True):
    """oracle_conv2dq_forward on numpy arrays; scales / zps ordered (input, weights, output).  Returns (y, acc)."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    Ho, Wo = conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    x = np.ascontiguousarray(x, np.uint8)
    w = np.ascontiguousarray(w, np.uint8)
    y = np.empty((N, Cout, Ho, Wo), np.uint8)
    acc = np.empty((N, Cout, Ho, Wo), np.int32) if want_acc else None
    b = None
    if bias is not None:
        b = np.ascontiguousarray(bias, np.int32)
        assert b.size >= Ho * Wo
    rc = oracle().oracle_conv2dq_forward(*geo, x.reshape(-1), w.reshape(-1),
                                         b.ctypes.data_as(C.POINTER(C.c_int32)) if b is not None else None,
                                         qparams3(scales, zps), y.reshape(-1),
                                         acc.ctypes.data_as(C.POINTER(C.c_int32)) if acc is not None else None)
    assert rc == 0
    return y, acc


def ref_conv2dq_forward(geo, x, w, scales, zps):
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    Ho, Wo = conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    y = np.empty((N, Cout, Ho, Wo), np.uint8)
    rc = ref().ref_conv2dq_u8(*geo, np.ascontiguousarray(x, np.uint8).reshape(-1), np.ascontiguousarray(w, np.uint8).reshape(-1),
                              np.asarray(scales, np.float32), np.asarray(zps, np.uint8), y.reshape(-1))
    assert rc == 0
    return y


def mlp_step(X, Ws, bs, target, use_ref=False):
    """One training step of the FullyConnected/relu/log_softmax/nll network (oracle_mlp_step, or the compiled l-ten
    network with use_ref).  Returns dict(loss, logp, dW[], db[], dX)."""
    fpc = C.POINTER(C.c_float)
    X = np.ascontiguousarray(X, np.float32)
    Ws = [np.ascontiguousarray(w, np.float32) for w in Ws]
    bs = [np.ascontiguousarray(b, np.float32) for b in bs] if bs is not None else None
    target = np.ascontiguousarray(target, np.float32)
    layers, batch = len(Ws), X.shape[0]
    sizes = (C.c_uint64 * (layers + 1))(*([X.shape[1]] + [w.shape[0] for w in Ws]))
    dW = [np.zeros_like(w) for w in Ws]
    db = [np.zeros_like(b) for b in bs] if bs is not None else None
    dX, logp, loss = np.zeros_like(X), np.zeros_like(target), C.c_float()

    def arr(lst):
        return (fpc * layers)(*[a.ctypes.data_as(fpc) for a in lst])
    fn = ref().ref_mlp_step if use_ref else oracle().oracle_mlp_step
    rc = fn(batch, layers, sizes, X.ctypes.data_as(fpc), arr(Ws), arr(bs) if bs is not None else None,
            target.ctypes.data_as(fpc), C.byref(loss), logp.ctypes.data_as(fpc), arr(dW),
            arr(db) if db is not None else None, dX.ctypes.data_as(fpc))
    assert rc == 0
    return dict(loss=float(loss.value), logp=logp, dW=dW, db=db, dX=dX)
