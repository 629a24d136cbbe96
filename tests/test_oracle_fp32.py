"""CPU tests that pin the fp32 oracle: l-ten's own unit-test vectors (matmul_test, fc_test),
golden outputs of the compiled cpu_gemm<float> / layer classes, integer-valued exactness
(any summation order is exact, so layout and transposes are checked bit for bit) and the
fp64 bound."""
import ctypes as C
import json

import numpy as np
import pytest

from conftest import golden_path, rel_err

fp = C.POINTER(C.c_float)


def fptr(a):
    return None if a is None else a.ctypes.data_as(fp)


def test_sgemm_golden_cases(ob):
    g = np.load(golden_path("sgemm_cases.npz"))
    for i in range(int(g["count"])):
        pre = f"c{i}_"
        M, N, K, tA, tB = (int(v) for v in g[pre + "dims"])
        alpha, beta = (float(v) for v in g[pre + "ab"])
        lda = M if tA else K
        ldb = K if tB else N
        Cm = g[pre + "C0"].copy()
        ob.sgemm(tA, tB, M, N, K, alpha, g[pre + "A"], lda, g[pre + "B"], ldb, beta, Cm, N)
        # l-ten sums 128-wide k blocks in AVX lanes, the oracle sums k in order: same value up to fp32 reassociation (north-star bound 1e-4)
        assert rel_err(Cm, g[pre + "C"]) < 1e-4, (i, M, N, K, tA, tB, alpha, beta)
        C64 = g[pre + "C0"].copy()
        ob.sgemm(tA, tB, M, N, K, alpha, g[pre + "A"], lda, g[pre + "B"], ldb, beta, C64, N, f64=True)
        assert rel_err(C64, g[pre + "C"]) < 1e-4


@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_sgemm_integer_valued_is_exact(ob, tA, tB):
    rng = np.random.default_rng(40 + 2 * tA + tB)
    M, N, K = 19, 27, 45
    A = rng.integers(-8, 9, (M, K)).astype(np.float32)
    B = rng.integers(-8, 9, (K, N)).astype(np.float32)
    want = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)
    # leading dimensions larger than the logical width
    lda, ldb, ldc = (M if tA else K) + 3, (K if tB else N) + 5, N + 2
    As = np.zeros(((K if tA else M), lda), np.float32)
    As[:, :(M if tA else K)] = A.T if tA else A
    Bs = np.zeros(((N if tB else K), ldb), np.float32)
    Bs[:, :(K if tB else N)] = B.T if tB else B
    Cm = np.full((M, ldc), 7.0, np.float32)
    ob.sgemm(tA, tB, M, N, K, 1.0, As, lda, Bs, ldb, 0.0, Cm, ldc)
    assert np.array_equal(Cm[:, :N], want)
    assert (Cm[:, N:] == 7.0).all()  # padding columns untouched
    ob.sgemm(tA, tB, M, N, K, 2.0, As, lda, Bs, ldb, -1.0, Cm, ldc)
    assert np.array_equal(Cm[:, :N], want)  # 2*AB - AB


def test_beta_zero_overwrites_nan(ob):
    A = np.ones((2, 3), np.float32)
    B = np.ones((3, 2), np.float32)
    Cm = np.full((2, 2), np.nan, np.float32)
    ob.sgemm(0, 0, 2, 2, 3, 1.0, A, 3, B, 2, 0.0, Cm, 2)
    assert np.array_equal(Cm, np.full((2, 2), 3.0, np.float32))


def test_sgemm_mt_equals_single_thread(ob):
    rng = np.random.default_rng(2)
    M, N, K = 37, 40, 51
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((N, K)).astype(np.float32)
    C1 = np.zeros((M, N), np.float32)
    C2 = np.zeros((M, N), np.float32)
    ob.sgemm(0, 1, M, N, K, 1.0, A, K, B, K, 0.0, C1, N)
    ob.oracle().oracle_sgemm_mt(0, 1, M, N, K, 1.0, A.reshape(-1), K, B.reshape(-1), K, 0.0, C2.reshape(-1), N, 5)
    assert np.array_equal(C1, C2)


def test_lten_matmul_test_vectors(ob):
    """tests/unit_tests.cpp matmul_test: exact forward values and gradients of z[1][0][3][1]."""
    v = json.load(open(golden_path("lten_unit_test_vectors.json")))["matmul_test"]
    ad, bd = np.array(v["x_dims"], np.uint64), np.array(v["w_dims"], np.uint64)
    a, b = np.array(v["x"], np.float32), np.array(v["w"], np.float32)
    cd = np.zeros(4, np.uint64)
    c = np.zeros(32, np.float32)
    assert ob.oracle().oracle_matmul(4, ad, bd, a, b, cd, c) == 0
    assert list(cd) == [2, 1, 4, 4]
    assert np.array_equal(c, np.array(v["z"], np.float32))
    dc = np.zeros((2, 1, 4, 4), np.float32)
    dc[tuple(v["backward_from"])] = 1.0
    assert c.reshape(2, 1, 4, 4)[tuple(v["backward_from"])] == v["picked_value"]
    da, db = np.empty_like(a), np.empty_like(b)
    assert ob.oracle().oracle_matmul_backward(4, ad, bd, a, b, dc.reshape(-1), fptr(da), fptr(db)) == 0
    assert np.array_equal(da, np.array(v["x_grad"], np.float32))
    assert np.array_equal(db, np.array(v["w_grad"], np.float32))


def test_lten_fc_test_vectors(ob):
    """tests/unit_tests.cpp fc_test: FullyConnected(3, 8) without bias, abs tolerance 1e-3."""
    v = json.load(open(golden_path("lten_unit_test_vectors.json")))["fc_test"]
    x, w = np.array(v["x"], np.float32), np.array(v["weights"], np.float32)
    M, fin, fout = 8, v["in_features"], v["out_features"]
    y = np.empty(M * fout, np.float32)
    ob.oracle().oracle_fc_forward(M, fin, fout, x, w, None, y)
    assert np.abs(y - np.array(v["z"], np.float32)).max() <= v["tolerance"]
    dy = np.zeros((2, 1, 4, 8), np.float32)
    dy[tuple(v["backward_from"])] = 1.0
    assert abs(y.reshape(2, 1, 4, 8)[tuple(v["backward_from"])] - v["picked_value"]) <= v["tolerance"]
    dx, dw = np.empty_like(x), np.empty_like(w)
    ob.oracle().oracle_fc_backward(M, fin, fout, x, w, dy.reshape(-1), fptr(dx), fptr(dw), None)
    assert np.abs(dx - np.array(v["x_grad"], np.float32)).max() <= v["tolerance"]
    assert np.abs(dw - np.array(v["w_grad"], np.float32)).max() <= v["tolerance"]


def test_layer_golden_fc(ob):
    g = np.load(golden_path("layer_cases.npz"))
    for i in range(int(g["fc_count"])):
        pre = f"fc{i}_"
        M, fin, fout, use_bias = (int(v) for v in g[pre + "dims"])
        b = g[pre + "b"] if use_bias else None
        y = np.empty(M * fout, np.float32)
        ob.oracle().oracle_fc_forward(M, fin, fout, g[pre + "x"], g[pre + "w"], fptr(b), y)
        # same scalar loops on both sides (all N < 16): bit-exact
        assert np.array_equal(y, g[pre + "y"]), i
        dx, dw = np.empty(M * fin, np.float32), np.empty(fout * fin, np.float32)
        db = np.zeros(fout, np.float32)
        ob.oracle().oracle_fc_backward(M, fin, fout, g[pre + "x"], g[pre + "w"], g[pre + "dy"], fptr(dx), fptr(dw),
                                       fptr(db) if use_bias else None)
        assert np.array_equal(dx, g[pre + "dx"]) and np.array_equal(dw, g[pre + "dw"]), i
        if use_bias:
            assert np.array_equal(db, g[pre + "db"]), i


def test_layer_golden_matmul_broadcast(ob):
    g = np.load(golden_path("layer_cases.npz"))
    for i in range(int(g["mm_count"])):
        pre = f"mm{i}_"
        ad, bd = g[pre + "adims"], g[pre + "bdims"]
        nd = len(ad)
        cd = np.zeros(nd, np.uint64)
        c = np.empty_like(g[pre + "c"])
        assert ob.oracle().oracle_matmul(nd, ad, bd, g[pre + "a"], g[pre + "b"], cd, c) == 0
        assert np.array_equal(c, g[pre + "c"]), i
        da, db = np.empty_like(g[pre + "a"]), np.empty_like(g[pre + "b"])
        assert ob.oracle().oracle_matmul_backward(nd, ad, bd, g[pre + "a"], g[pre + "b"], g[pre + "dc"], fptr(da),
                                                  fptr(db)) == 0
        assert np.array_equal(da, g[pre + "da"]) and np.array_equal(db, g[pre + "db"]), i


def test_matmul_rejects_bad_shapes(ob):
    # l-ten/md_array.h:985,1234: inner dims must agree, leading dims must match or be 1
    a = np.zeros(24, np.float32)
    cd = np.zeros(3, np.uint64)
    c = np.zeros(64, np.float32)
    f = ob.oracle().oracle_matmul
    assert f(3, np.array([2, 3, 4], np.uint64), np.array([2, 5, 2], np.uint64), a, a, cd, c) == -1
    assert f(3, np.array([2, 3, 4], np.uint64), np.array([3, 4, 2], np.uint64), a, a, cd, c) == -1
