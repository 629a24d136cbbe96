"""No-GPU checks of the C-ABI library: it loads, exports every symbol include/lten_hip.h declares,
and its argument validation (which runs before any HIP call) reports errors the way the header says."""
import ctypes as C
import os

import numpy as np


def test_library_is_built_in_tree(lt):
    assert os.path.exists(lt.LIB_PATH), "build with: python light-tensor_amd/build.py"
    assert os.path.dirname(lt.LIB_PATH).endswith("light-tensor_amd")


def test_every_declared_symbol_is_exported(lt):
    raw = C.CDLL(lt.LIB_PATH)
    declared = lt.declared_symbols()
    assert len(declared) >= 30
    missing = [s for s in declared if not hasattr(raw, s)]
    assert not missing, missing
    # and the Python signature table covers exactly the declared surface
    assert sorted(lt._SIGNATURES) == declared


def test_calibration_library_is_separate(lt):
    """The calibration kernels live in a library of their own: it exports what include/lten_hip_measure.h declares,
    and the product library exports none of it."""
    import re
    text = re.sub(r"/\*.*?\*/", "", open(lt.MEASURE_HEADER_PATH).read(), flags=re.S)
    declared = sorted(set(re.findall(r"\b(lten_measure_[a-z0-9_]+)\s*\(", text)))
    assert declared == sorted(lt._MEASURE_SIGNATURES)
    m, raw = C.CDLL(lt.MEASURE_LIB_PATH), C.CDLL(lt.LIB_PATH)
    assert all(hasattr(m, s) for s in declared)
    assert not any(hasattr(raw, s) for s in declared)
    assert not any("measure" in s or "copy_kernel" in s for s in lt.declared_symbols())


def test_qparams_layout_matches_lten(lt):
    # l-ten/math_fns.h:12-16: float scale; uint8_t zero_point -> 8 bytes, zero_point at offset 4
    assert C.sizeof(lt.QParams) == 8 and lt.QParams.zero_point.offset == 4


def test_alpha_beta_rejected_like_lten(lt):
    # l-ten/math_fns.cpp:1331-1334; checked on the host before anything touches the GPU
    qp = lt.qparams3([1, 1, 1], [0, 0, 0])
    l = lt.lib()
    assert l.lten_hip_quantized_matmul(0, 1, 4, 4, 4, 2, None, None, 0, None, qp, None, None) != 0
    assert b"alpha != 1 and beta != 0" in l.lten_hip_last_error()
    assert l.lten_hip_quantized_matmul(0, 1, 4, 4, 4, 1, None, None, 1, None, qp, None, None) != 0


def test_argument_validation_without_gpu(lt):
    l = lt.lib()
    qp = lt.qparams3([1, 1, 1], [0, 0, 0])
    # null matrices
    assert l.lten_hip_quantized_matmul(0, 1, 4, 4, 4, 1, None, None, 0, None, qp, None, None) != 0
    assert b"null" in l.lten_hip_last_error()
    # K beyond the reference's int accumulator range
    assert l.lten_hip_quantized_matmul(0, 1, 4, 4, 40000, 1, 16, 16, 0, 16, qp, None, None) != 0
    assert b"overflows" in l.lten_hip_last_error()
    # empty problem is a no-op
    assert l.lten_hip_quantized_matmul(0, 1, 0, 4, 4, 1, None, None, 0, None, qp, None, None) == 0
    assert l.lten_hip_set_option(b"no_such_option", 1) != 0
    assert l.lten_hip_set_option(b"qgemm_tile", 0) == 0


def test_product_does_not_reference_the_oracle(lt):
    """The shipped sources never name the oracle: no CPU fallback can hide behind the C ABI."""
    pkg = os.path.dirname(lt.LIB_PATH)
    for root, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".hip", ".h", ".cpp", ".py")):
                text = open(os.path.join(root, f), errors="ignore").read()
                assert "oracle" not in text.lower(), os.path.join(root, f)
