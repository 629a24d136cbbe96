"""GPU parity tests of the int8 path, through the C ABI, against the oracle and the golden vectors.
Bar: bit-exact int32 accumulators and bit-exact requantized uint8 outputs."""
import numpy as np
import pytest

from conftest import exact_acc, golden_path, requant_numpy

pytestmark = pytest.mark.gpu

TILES = {0: "heuristic", 1: "256x256", 2: "128x128", 3: "guard 64x64", 4: "guard 32x32"}


def run_case(gpu, ob, A, B, sc, zp, tA=False, tB=True, bias=None, M=None, N=None, K=None, tile=0):
    gpu.set_option("qgemm_tile", tile)
    try:
        Cg, accg = gpu.qgemm_host(A, B, sc, zp, tA=tA, tB=tB, bias=bias, want_acc=True, M=M, N=N, K=K)
    finally:
        gpu.set_option("qgemm_tile", 0)
    Co, acco = ob.quantized_matmul(A, B, sc, zp, tA=tA, tB=tB, bias=bias, M=M, N=N, K=K)
    assert np.array_equal(accg, acco), "int32 accumulators differ"
    assert np.array_equal(Cg, Co), "requantized outputs differ"
    return Cg


def test_cfg1_bit_exact_and_golden(gpu, ob, wl):
    X, W, sc, zp = wl.cfg1()
    want = np.load(golden_path("cfg1_expected.npz"))["C"]
    for tile in (0, 3, 4):
        Cg = run_case(gpu, ob, X, W, sc, zp, tile=tile)
        assert np.array_equal(Cg, want)


def test_golden_cases_all_transpose_modes(gpu):
    g = np.load(golden_path("qmm_cases.npz"))
    for i in range(int(g["count"])):
        pre = f"c{i}_"
        M, N, K, tA, tB = (int(v) for v in g[pre + "dims"])
        bias = g[pre + "bias"] if pre + "bias" in g.files else None
        Cg, _ = gpu.qgemm_host(g[pre + "A"], g[pre + "B"], g[pre + "sc"], g[pre + "zp"], tA=bool(tA), tB=bool(tB),
                               bias=bias, M=M, N=N, K=K)
        assert np.array_equal(Cg, g[pre + "C"]), (i, M, N, K, tA, tB)


@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 5, 7), (33, 65, 100), (64, 64, 64), (100, 200, 300), (17, 512, 784),
                                   (300, 257, 1000), (1, 300, 33), (130, 1, 2000)])
def test_ragged_shapes_random_zero_points(gpu, ob, shape):
    M, N, K = shape
    rng = np.random.default_rng(M * 1000003 + N * 1009 + K)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    zp = rng.integers(0, 256, 3).astype(np.uint8)
    sc = np.array([0.02, 0.01, 0.7], np.float32)
    bias = rng.integers(-100000, 100000, N).astype(np.int32)
    for tile in (0, 3, 4):
        run_case(gpu, ob, A, B, sc, zp, bias=bias, tile=tile)


@pytest.mark.parametrize("tile,shape", [(1, (256, 256, 64)), (1, (512, 768, 320)), (2, (128, 128, 64)),
                                        (2, (384, 256, 448)), (1, (256, 512, 1024))])
def test_fast_tiles(gpu, ob, tile, shape):
    M, N, K = shape
    rng = np.random.default_rng(M + N + K + tile)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    for zp in ([128, 128, 128], [0, 128, 3], [255, 1, 200]):
        run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array(zp, np.uint8),
                 bias=rng.integers(-5000, 5000, N).astype(np.int32) if zp[0] else None, tile=tile)


@pytest.mark.parametrize("variant", [33, 34, 41])
@pytest.mark.parametrize("shape", [(256, 256, 128), (512, 768, 640), (256, 1024, 2048), (256, 512, 256), (200, 260, 384), (256, 256, 400)])
def test_direct_to_lds_tiles(gpu, ob, variant, shape):
    """The direct-to-LDS tiles (256 x 256 in both wavefront layouts, 128 x 128): with and without zero-point terms
    and bias, one to sixteen k-steps (prologue, the half-open refill at the end of the steady loop, drain), ragged
    M and N, a K that is no multiple of the k-step."""
    M, N, K = shape
    rng = np.random.default_rng(M + N + K + variant)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    if K % 128 != 0 and variant == 34:
        pytest.skip("this layout takes whole k-steps only")
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([128, 128, 128], np.uint8), tile=variant)
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([3, 250, 77], np.uint8),
             bias=rng.integers(-5000, 5000, N).astype(np.int32), tile=variant)


@pytest.mark.parametrize("variant", [33, 41, 51])
@pytest.mark.parametrize("shape", [(300, 1001, 512), (256, 258, 640), (130, 4099, 256), (257, 129, 400), (512, 50257 // 16, 768)])
def test_direct_to_lds_tiles_with_any_number_of_columns(gpu, ob, variant, shape):
    """out_features that are no multiple of 4 (1001 classes, a vocabulary of 50257): rows of the output then start on any
    byte, and the zero-point vectors end inside a group of four.  Raw and prepared weights, int32 and uint8 outputs,
    with every term and a bias, on each tile family."""
    M, N, K = shape
    rng = np.random.default_rng(M + N + K + variant)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    l = gpu.lib()
    for zp, with_bias in (([128, 128, 128], False), ([0, 128, 3], True), ([3, 250, 77], True)):
        bias = rng.integers(-5000, 5000, N).astype(np.int32) if with_bias else None
        sc = [0.02, 0.013, 0.9]
        run_case(gpu, ob, A, B, sc, np.array(zp, np.uint8), bias=bias, tile=variant)
        assert gpu.last_kernel().startswith("qgemm_fast"), gpu.last_kernel()
        gpu.set_option("qgemm_tile", variant)
        try:
            got, k1 = fcq(gpu, l.lten_hip_fcq_forward_prepared, A, B, sc, zp, bias, prepared=True)
        finally:
            gpu.set_option("qgemm_tile", 0)
        assert k1.startswith("qgemm_fast") and "wpre" in k1, k1
        Co, _ = ob.quantized_matmul(A, B, np.array(sc, np.float32), np.array(zp, np.uint8), bias=bias)
        assert np.array_equal(got, Co), (shape, zp, k1)


def test_requantize_exact_epilogue_in_tiled_kernels(gpu, ob):
    """Multipliers above 1 select the epilogue that spells out the x86 conversion (out-of-range -> 0x80000000)."""
    rng = np.random.default_rng(4)
    A = rng.integers(0, 256, (256, 256), dtype=np.uint8)
    B = rng.integers(0, 256, (256, 256), dtype=np.uint8)
    for scales in ([300.0, 500.0, 1.0], [1.0, 1.0, 1e-6]):
        for tile in (0, 1, 3, 33, 41):
            run_case(gpu, ob, A, B, scales, np.array([128, 128, 9], np.uint8), tile=tile)


@pytest.mark.parametrize("tA,tB", [(0, 0), (1, 0), (1, 1)])
def test_other_transpose_modes(gpu, ob, tA, tB):
    rng = np.random.default_rng(77 + tA * 2 + tB)
    M, N, K = 70, 130, 150
    A = rng.integers(0, 256, M * K, dtype=np.uint8)
    B = rng.integers(0, 256, N * K, dtype=np.uint8)
    run_case(gpu, ob, A, B, [0.02, 0.01, 0.5], np.array([7, 99, 128], np.uint8), tA=bool(tA), tB=bool(tB), M=M, N=N, K=K)


def test_extreme_values_and_zero_point_invariants(gpu, ob):
    M, N, K = 64, 96, 2048
    for a, b in ((255, 255), (0, 0), (255, 0)):
        A = np.full((M, K), a, np.uint8)
        B = np.full((N, K), b, np.uint8)
        run_case(gpu, ob, A, B, [0.001, 0.001, 1.0], np.array([0, 0, 0], np.uint8))       # largest accumulators
        run_case(gpu, ob, A, B, [0.001, 0.001, 1.0], np.array([255, 255, 9], np.uint8))   # most negative terms
    rng = np.random.default_rng(0)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    Bc = np.full((N, K), 77, np.uint8)
    Cg = run_case(gpu, ob, A, Bc, [0.3, 0.2, 0.1], np.array([5, 77, 200], np.uint8))
    assert (Cg == 200).all()   # B == zpB: accumulator 0, output = output zero point


def test_requantize_sweep_on_gpu(gpu):
    """Arbitrary int32 accumulators through the GPU epilogue: A = 0, zero points 0 make `element`
    equal to bias[n] (l-ten/math_fns.cpp:1469-1473).  Expected bytes come from l-ten's own code."""
    g = np.load(golden_path("requant_sweep.npz"))
    acc, mults, zps, expected = g["acc"], g["mults"], g["zps"], g["expected"]
    n = len(acc)
    A = np.zeros((1, 1), np.uint8)
    B = np.zeros((n, 1), np.uint8)
    for i, m in enumerate(mults):
        for j, z in enumerate(zps):
            Cg, _ = gpu.qgemm_host(A, B, [m, 1.0, 1.0], [0, 0, z], bias=acc)
            assert np.array_equal(Cg.reshape(-1), expected[i, j]), (float(m), int(z))


def test_fcq_forward_leading_dims(gpu, ob, wl):
    """FullyConnected_q on a {2, 32, 784} input (l-ten/fully_connected.cpp:364-396) in one call."""
    X, W, sc, zp = wl.cfg1()
    dX, dW = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer.from_numpy(W)
    dY = gpu.DeviceBuffer(64 * 512)
    ws = gpu.DeviceBuffer(4 * (64 + 512))
    gpu.check(gpu.lib().lten_hip_fcq_forward(2, 32, 784, 512, dX.ptr, dW.ptr, None, gpu.qparams3(sc, zp), dY.ptr, ws.ptr))
    assert np.array_equal(dY.numpy(np.uint8, (64, 512)), np.load(golden_path("cfg1_expected.npz"))["C"])


@pytest.mark.parametrize("variant", [41])
@pytest.mark.parametrize("shape", [(128, 128, 128), (384, 640, 640), (128, 1152, 2048),
                                   # ragged M and N (N a multiple of 16): edge tiles fetch the last row again and store what exists
                                   (33, 144, 512), (200, 656, 1152), (1, 16, 128),
                                   # N a multiple of 4 only: output rows are stored four bytes at a time
                                   (130, 1000, 256), (64, 12, 640)])
def test_direct_to_lds_128_tiles(gpu, ob, variant, shape):
    """The 128x128 form of the direct-to-LDS tiles (what the library picks when 256x256 tiles would leave CUs idle):
    with and without zero-point terms and bias, short and long K; int32 and u8."""
    M, N, K = shape
    rng = np.random.default_rng(M + N + K + variant)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([128, 128, 128], np.uint8), tile=variant)
    assert gpu.last_kernel().startswith("qgemm_fast_128x128")
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([3, 250, 77], np.uint8),
             bias=rng.integers(-5000, 5000, N).astype(np.int32), tile=variant)
    run_case(gpu, ob, A, B, [0.5, 0.5, 0.2], np.array([128, 128, 9], np.uint8), tile=variant)   # multiplier > 0.99: exact-convert epilogue


@pytest.mark.parametrize("variant,shape", [(41, (128, 128, 144)), (41, (200, 272, 784)), (41, (64, 160, 2064)), (33, (300, 272, 400)),
                                           (33, (256, 512, 912)), (33, (256, 256, 128 + 16))])
def test_direct_to_lds_tiles_partial_last_k_step(gpu, ob, variant, shape):
    """K a multiple of 16 but not of the 128-byte k-step: the last step loads only what exists and pads the A tile
    with bytes that the sign flip turns into zeros; with and without zero-point terms, exact-convert epilogue."""
    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([128, 128, 128], np.uint8), tile=variant)
    assert gpu.last_kernel().endswith("ktail"), gpu.last_kernel()
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([3, 250, 77], np.uint8), bias=rng.integers(-5000, 5000, N).astype(np.int32), tile=variant)
    run_case(gpu, ob, A, B, [0.5, 0.5, 0.2], np.array([128, 128, 9], np.uint8), tile=variant)


@pytest.mark.parametrize("shape", [(256, 128, 128), (512, 384, 640), (300, 272, 400), (520, 392, 2064), (1, 16, 256), (257, 132, 1152)])
def test_direct_to_lds_256x128_tiles(gpu, ob, shape):
    """The 256 x 128 form (four wavefronts of 64 x 128, three stages), forced by option on shapes the oracle finishes:
    whole and ragged tiles, K with and without a partial last k-step, N a multiple of 16 or of 4 only; with and
    without zero-point terms and bias, exact-convert epilogue; prepared weights give the same bytes."""
    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([128, 128, 128], np.uint8), tile=51)
    assert gpu.last_kernel() == "qgemm_fast_256x128x128_w4x1_s3" + ("_ktail" if K % 128 else ""), gpu.last_kernel()
    bias = rng.integers(-5000, 5000, N).astype(np.int32)
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([3, 250, 77], np.uint8), bias=bias, tile=51)
    run_case(gpu, ob, A, B, [0.5, 0.5, 0.2], np.array([128, 128, 9], np.uint8), tile=51)
    l = gpu.lib()
    gpu.set_option("qgemm_tile", 51)
    try:
        sc, zp = [0.02, 0.013, 0.9 * K / 512], [200, 17, 99]
        want, k0 = fcq(gpu, l.lten_hip_fcq_forward, A, B, sc, zp, bias)
        got, k1 = fcq(gpu, l.lten_hip_fcq_forward_prepared, A, B, sc, zp, bias, prepared=True)
    finally:
        gpu.set_option("qgemm_tile", 0)
    # prepared weights: the tiles work out the zero-point terms themselves (the name says which), no launch before them
    assert k0.startswith("qgemm_fast_256x128") and k1 == k0 + "_wpre+zpcol+zprow", (k0, k1)
    assert np.array_equal(got, want)


def test_256x128_tiles_are_picked_for_about_one_tile_per_cu(gpu):
    """2048 x 2688 x 2048: 88 tiles of 256 x 256 would leave most CUs idle, 336 of 128 x 128 bring more operand bytes
    per MFMA; the library takes 168 tiles of 256 x 128.  Closed form in fp64 (exact) as the check."""
    M, N, K = 2048, 2688, 2048
    rng = np.random.default_rng(51)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    zp, sc = [11, 140, 120], [0.02, 0.02, 3.0]
    bias = rng.integers(-9000, 9000, N).astype(np.int32)
    dA, dB, dBias = gpu.DeviceBuffer.from_numpy(A), gpu.DeviceBuffer.from_numpy(B), gpu.DeviceBuffer.from_numpy(bias)
    dC, ws = gpu.DeviceBuffer(M * N), gpu.DeviceBuffer(4 * (M + N))
    gpu.quantized_matmul(False, True, M, N, K, dA, dB, dC, gpu.qparams3(sc, zp), dBias, ws)
    assert gpu.last_kernel() == "qgemm_fast_256x128x128_w4x1_s3", gpu.last_kernel()
    want = exact_acc(A, B, zp[0], zp[1]) + bias[None, :]
    mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
    assert np.array_equal(dC.numpy(np.uint8, (M, N)), requant_numpy(want, mult, zp[2]))


@pytest.mark.parametrize("variant", [33, 34])
def test_direct_to_lds_256_tiles_ragged(gpu, ob, variant):
    """300 x 272 x 640 on 256 x 256 tiles: two row tiles and two column tiles, all of them edge tiles."""
    rng = np.random.default_rng(variant)
    A = rng.integers(0, 256, (300, 640), dtype=np.uint8)
    B = rng.integers(0, 256, (272, 640), dtype=np.uint8)
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([3, 250, 77], np.uint8), bias=rng.integers(-5000, 5000, 272).astype(np.int32), tile=variant)
    assert gpu.last_kernel().startswith("qgemm_fast_256x256")
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([128, 128, 128], np.uint8), tile=variant)


def test_batch_sizes_between_the_tile_sizes(gpu):
    """M = 65, 100, 200 against 4096 x 4096 or 2048 x 4096 weights (more rows than the streaming kernel takes, no multiple of 128): the
    tiles with K split, checked against the closed form; M = 200 against 4096 x 1024 (no split)."""
    rng = np.random.default_rng(3)
    for (M, N, K, split) in ((65, 4096, 4096, True), (100, 2048, 4096, True), (200, 2048, 4096, True), (200, 4096, 1024, False)):
        A = rng.integers(0, 256, (M, K), dtype=np.uint8)
        B = rng.integers(0, 256, (N, K), dtype=np.uint8)
        zp, sc = [11, 140, 120], [0.02, 0.02, 3.0]
        bias = rng.integers(-9000, 9000, N).astype(np.int32)
        dA, dB, dBias = gpu.DeviceBuffer.from_numpy(A), gpu.DeviceBuffer.from_numpy(B), gpu.DeviceBuffer.from_numpy(bias)
        dC, dacc, ws = gpu.DeviceBuffer(M * N), gpu.DeviceBuffer(4 * M * N), gpu.DeviceBuffer(4 * (M + N))
        qp = gpu.qparams3(sc, zp)
        gpu.quantized_matmul_acc(False, True, M, N, K, dA, dB, dacc, qp, dBias, ws)
        assert gpu.last_kernel().startswith("qgemm_fast_128x128") and gpu.last_kernel().endswith("splitk") == split, gpu.last_kernel()
        want = exact_acc(A, B, zp[0], zp[1]) + bias[None, :]
        assert np.array_equal(dacc.numpy(np.int32, (M, N)), want)
        gpu.quantized_matmul(False, True, M, N, K, dA, dB, dC, qp, dBias, ws)
        mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
        assert np.array_equal(dC.numpy(np.uint8, (M, N)), requant_numpy(want, mult, zp[2]))


@pytest.mark.parametrize("shape", [
    (384, 1536, 4096, "qgemm_fast_128x128x128_w2x2_s4"),          # 36 tiles, one per CU: the ring of four stages
    (300, 1540, 4112, "qgemm_fast_128x128x128_w2x2_s4_ktail"),    # the same with ragged edges and a partial last k-step
    (384, 1536, 8192, "qgemm_fast_128x128x128_w2x2_s4_splitk"),   # 36 tiles, K in two shares of 4096
    (130, 2048, 512 * 5, "qgemm_fast_128x128x128_w2x2_s2"),       # K below 4096: two stages
    (1024, 4096, 640, "qgemm_fast_128x128x128_w2x2_s2"),          # five k-steps, one workgroup per CU
])
def test_128_tiles_ring_depth(gpu, shape):
    """Where a CU holds a single 128 x 128 tile and K is at least 4096 the stages form a ring of four (three k-steps
    in flight), otherwise of two: int32 sums against the closed form, bytes against the requantize of those sums."""
    M, N, K, kernel = shape
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    zp, sc = [11, 140, 120], [0.02, 0.02, 3.0]
    bias = rng.integers(-9000, 9000, N).astype(np.int32)
    dA, dB, dBias = gpu.DeviceBuffer.from_numpy(A), gpu.DeviceBuffer.from_numpy(B), gpu.DeviceBuffer.from_numpy(bias)
    dC, dacc, ws = gpu.DeviceBuffer(M * N), gpu.DeviceBuffer(4 * M * N), gpu.DeviceBuffer(4 * (M + N))
    qp = gpu.qparams3(sc, zp)
    gpu.quantized_matmul_acc(False, True, M, N, K, dA, dB, dacc, qp, dBias, ws)
    assert gpu.last_kernel() == kernel, gpu.last_kernel()
    want = exact_acc(A, B, zp[0], zp[1]) + bias[None, :]
    assert np.array_equal(dacc.numpy(np.int32, (M, N)), want)
    gpu.quantized_matmul(False, True, M, N, K, dA, dB, dC, qp, dBias, ws)
    mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
    assert np.array_equal(dC.numpy(np.uint8, (M, N)), requant_numpy(want, mult, zp[2]))


def test_medium_batch_picks_128_tiles(gpu, ob):
    """512 x 1024 x 1024: 8 tiles of 256x256 would occupy 8 CUs; the library takes 32 tiles of 128x128."""
    rng = np.random.default_rng(77)
    A = rng.integers(0, 256, (512, 1024), dtype=np.uint8)
    B = rng.integers(0, 256, (1024, 1024), dtype=np.uint8)
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([9, 131, 100], np.uint8), bias=rng.integers(-5000, 5000, 1024).astype(np.int32))
    assert gpu.last_kernel().startswith("qgemm_fast_128x128x128")


@pytest.mark.parametrize("splits", [2, 4, 8])
def test_split_k_tiles_forced(gpu, ob, splits):
    """Several workgroups per 128 x 128 tile, each with a share of K, the last to arrive adds the shares: forced by
    option on a shape the oracle still finishes (10 tiles, K = 2048), with zero-point terms, bias, the exact-convert
    epilogue, int32 and u8 outputs; repeated launches check that the arrival counters return to zero."""
    rng = np.random.default_rng(splits)
    M, N, K = 256, 640, 2048
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    gpu.set_option("qgemm_split", splits)
    try:
        for rep in range(3):
            run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([128, 128, 128], np.uint8))
            assert gpu.last_kernel().endswith("splitk")
        run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([3, 250, 77], np.uint8), bias=rng.integers(-5000, 5000, N).astype(np.int32))
        assert gpu.last_kernel().endswith("splitk")
        run_case(gpu, ob, A, B, [0.5, 0.5, 0.2], np.array([128, 128, 9], np.uint8))
    finally:
        gpu.set_option("qgemm_split", 0)


@pytest.mark.parametrize("splits,K", [(4, 128 * 13), (8, 128 * 21), (2, 128 * 5)])
def test_split_k_shares_of_unequal_length(gpu, ob, splits, K):
    """A number of k-steps that the shares do not divide (13 steps over 4 workgroups: 4, 3, 3, 3): the first shares are a
    step longer.  Zero-point terms, bias, int32 and u8 outputs against the oracle."""
    rng = np.random.default_rng(splits + K)
    M, N = 200, 384
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    gpu.set_option("qgemm_split", splits)
    try:
        run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([128, 128, 128], np.uint8))
        assert gpu.last_kernel().endswith("splitk")
        run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([3, 250, 77], np.uint8), bias=rng.integers(-5000, 5000, N).astype(np.int32))
        assert gpu.last_kernel().endswith("splitk")
    finally:
        gpu.set_option("qgemm_split", 0)


@pytest.mark.parametrize("M,N,K", [(1, 1000, 25088), (4, 300, 33024), (16, 130, 20000), (7, 64, 16400), (20, 200, 12000), (32, 100, 30000)])
def test_few_rows_against_a_reduction_beyond_16384(gpu, ob, M, N, K):
    """The weight-streaming kernel holds the activations of at most 16384 k (8192 from 17 rows on) in the registers of its
    wavefronts: a longer K (a 25088 -> 1000 layer at batch 1) runs in chunks of K, a launch each into int32 sums, and a last launch adds them and
    requantizes.  Zero points, bias, int32 and u8 outputs against the oracle; the chunks are not equal (K = 16400)."""
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    run_case(gpu, ob, A, B, [0.02, 0.013, 3.0], np.array([128, 128, 128], np.uint8))
    assert gpu.last_kernel() == "qskinny_mfma_kchunks", gpu.last_kernel()
    run_case(gpu, ob, A, B, [0.02, 0.013, 3.0], np.array([3, 250, 77], np.uint8), bias=rng.integers(-5000, 5000, N).astype(np.int32))
    assert gpu.last_kernel() == "qskinny_mfma_kchunks", gpu.last_kernel()
    run_case(gpu, ob, A, B, [0.5, 0.5, 0.2], np.array([128, 0, 9], np.uint8))


@pytest.mark.parametrize("M,N,K", [(16, 8192, 16392), (3, 600, 20003)])
def test_long_reduction_that_is_no_multiple_of_16_keeps_its_padded_copies(gpu, ob, M, N, K):
    """in_features beyond 16384 and no multiple of 16: the operands are first copied into padded rows in memory the library
    owns, and the K-chunks of the streaming kernel then take their int32 sums from the same block: behind the copies, not
    on top of them.  Also with both operands transposed (copies of both).  Bit-exact against the closed form."""
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    zp, sc = np.array([3, 250, 77], np.uint8), [0.02, 0.013, 3.0]
    bias = rng.integers(-5000, 5000, N).astype(np.int32)
    mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
    want = requant_numpy(exact_acc(A, B, zp[0], zp[1]) + bias[None, :], mult, zp[2])
    got, k0 = fcq(gpu, gpu.lib().lten_hip_fcq_forward, A, B, sc, zp, bias)
    assert k0 == "qskinny_mfma_kchunks", k0
    assert np.array_equal(got, want)
    if N <= 1024:
        got_t, _ = gpu.qgemm_host(np.ascontiguousarray(A.T), np.ascontiguousarray(B.T), sc, zp, tA=True, tB=False, bias=bias, M=M, N=N, K=K)
        assert gpu.last_kernel() == "qskinny_mfma_kchunks", gpu.last_kernel()
        assert np.array_equal(got_t, want)


@pytest.mark.parametrize("M,N,K", [(2048, 8192, 64), (2048, 2048, 32), (2048, 4096, 48), (1000, 8190, 80), (2048, 4096, 112)])
def test_reduction_shorter_than_a_k_step_on_the_direct_to_lds_tiles(gpu, ob, M, N, K):
    """in_features of 32 to 112 against an output of 64 tiles or more: one partial k-step of the direct-to-LDS tiles (the
    activation tile padded with the zero point's image, whatever the weight tile holds there multiplied by zero).  l-ten's
    uint8 weights and prepared weights, with and without zero-point terms and bias, int32 accumulators and uint8 outputs."""
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    bias = rng.integers(-5000, 5000, N).astype(np.int32)
    for zp, b in (([128, 128, 128], None), ([0, 128, 3], bias), ([17, 250, 100], bias)):
        zp, sc = np.array(zp, np.uint8), [0.02, 0.013, 0.9]
        acc = exact_acc(A, B, zp[0], zp[1]) + (b[None, :] if b is not None else 0)
        mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
        want = requant_numpy(acc, mult, zp[2])
        got, k0 = fcq(gpu, gpu.lib().lten_hip_fcq_forward, A, B, sc, zp, b)
        assert k0.startswith("qgemm_fast_") and "ktail" in k0, k0
        assert np.array_equal(got, want), (zp.tolist(), k0)
        got, k1 = fcq(gpu, gpu.lib().lten_hip_fcq_forward_prepared, A, B, sc, zp, b, prepared=True)
        assert k1.startswith("qgemm_fast_") and "ktail" in k1, k1
        assert np.array_equal(got, want), (zp.tolist(), k1)
        _, accg = gpu.qgemm_host(A, B, sc, zp, bias=b, want_acc=True)
        assert np.array_equal(accg, acc)


@pytest.mark.parametrize("M,N,K", [(4096, 100, 9216), (8192, 66, 1024)])
def test_many_rows_onto_64_to_127_outputs_take_the_128_column_tiles(gpu, ob, M, N, K):
    """A layer of 64 to 127 outputs at a large batch: half-empty 128-column tiles (split over K where the tiles are few) are
    ahead of the 16 x 16 kernel; bit-exact on raw and prepared weights with zero points and bias."""
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    bias = rng.integers(-5000, 5000, N).astype(np.int32)
    zp, sc = np.array([17, 250, 100], np.uint8), [0.02, 0.013, 2.0]
    mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
    want = requant_numpy(exact_acc(A, B, zp[0], zp[1]) + bias[None, :], mult, zp[2])
    got, k0 = fcq(gpu, gpu.lib().lten_hip_fcq_forward, A, B, sc, zp, bias)
    assert k0.startswith("qgemm_fast_128x128"), k0
    assert np.array_equal(got, want)
    got, k1 = fcq(gpu, gpu.lib().lten_hip_fcq_forward_prepared, A, B, sc, zp, bias, prepared=True)
    assert k1.startswith("qgemm_fast_128x128"), k1
    assert np.array_equal(got, want)


def test_split_k_is_the_default_for_few_tiles_and_long_k(gpu):
    """256 x 1024 x 4096 (16 tiles): the library splits K in two; the closed form in int64 is the check.  With the
    option at 1 the unsplit tiles run and give the same bytes; a launch recorded into a graph also matches."""
    rng = np.random.default_rng(5)
    M, N, K = 256, 1024, 4096
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    zp = [7, 200, 128]
    sc = [0.02, 0.02, 2.5]
    dA, dB = gpu.DeviceBuffer.from_numpy(A), gpu.DeviceBuffer.from_numpy(B)
    dC, dacc, ws = gpu.DeviceBuffer(M * N), gpu.DeviceBuffer(4 * M * N), gpu.DeviceBuffer(4 * (M + N))
    qp = gpu.qparams3(sc, zp)
    gpu.quantized_matmul_acc(False, True, M, N, K, dA, dB, dacc, qp, None, ws)
    assert gpu.last_kernel().endswith("splitk")
    want = exact_acc(A, B, zp[0], zp[1])
    assert np.array_equal(dacc.numpy(np.int32, (M, N)), want)
    gpu.quantized_matmul(False, True, M, N, K, dA, dB, dC, qp, None, ws)
    assert gpu.last_kernel().endswith("splitk")
    mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
    split_out = dC.numpy(np.uint8, (M, N)).copy()
    assert np.array_equal(split_out, requant_numpy(want, mult, zp[2]))
    gpu.set_option("qgemm_split", 1)
    try:
        gpu.quantized_matmul(False, True, M, N, K, dA, dB, dC, qp, None, ws)
        assert not gpu.last_kernel().endswith("splitk")
        assert np.array_equal(dC.numpy(np.uint8, (M, N)), split_out)
    finally:
        gpu.set_option("qgemm_split", 0)
    gpu.check(gpu.lib().lten_hip_fill_u8(dC.ptr, M * N, 0))
    with gpu.Graph() as graph:
        gpu.quantized_matmul(False, True, M, N, K, dA, dB, dC, qp, None, ws)
    for _ in range(3):
        gpu.check(gpu.lib().lten_hip_fill_u8(dC.ptr, M * N, 0))
        graph.launch()
        assert np.array_equal(dC.numpy(np.uint8, (M, N)), split_out)


def test_cfg3_full_size_properties(gpu, wl):
    """4096^3: exact closed form of every accumulator (fp64 BLAS holds these integers exactly),
    then the requantize rule on top; plus linearity in the bias."""
    X, W, sc, zp = wl.cfg3()
    M = N = K = 4096
    dA, dB = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer.from_numpy(W)
    dC, dacc = gpu.DeviceBuffer(M * N), gpu.DeviceBuffer(4 * M * N)
    ws = gpu.DeviceBuffer(4 * (M + N))
    qp = gpu.qparams3(sc, zp)
    gpu.quantized_matmul(False, True, M, N, K, dA, dB, dC, qp, None, ws)
    assert gpu.last_kernel().startswith("qgemm_fast_256x256x128")
    gpu.quantized_matmul_acc(False, True, M, N, K, dA, dB, dacc, qp, None, ws)
    acc = dacc.numpy(np.int32, (M, N))
    want = exact_acc(X, W, int(zp[0]), int(zp[1]))
    assert np.array_equal(acc, want)
    mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
    out = dC.numpy(np.uint8, (M, N))
    assert np.array_equal(out, requant_numpy(want, mult, int(zp[2])))
    s = want * float(mult) + float(zp[2])
    assert 0.03 < ((s < 0) | (s >= 256)).mean() < 0.25   # some outputs wrap, most do not


@pytest.mark.parametrize("shape", [(1, 16, 2048), (4, 48, 4096), (7, 160, 8192), (16, 64, 8192), (13, 32, 2048),
                                   (17, 64, 2048), (32, 320, 8192), (25, 112, 4096)])
def test_weight_streaming_kernel(gpu, ob, shape):
    """M <= 32 (one or two blocks of 16 activation rows): the streaming kernel with in-kernel zero-point sums, every combination of needed terms,
    checked against the oracle and against the tiled kernels (option qskinny = 2 switches it off)."""
    M, N, K = shape
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    for zp in ([128, 128, 128], [3, 128, 9], [128, 200, 0], [17, 250, 100]):
        bias = rng.integers(-9999, 9999, N).astype(np.int32) if zp[0] != 128 else None
        gpu.set_option("qskinny", 1)   # stream whatever the size of the weights
        try:
            Cg = run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array(zp, np.uint8), bias=bias)
            assert gpu.last_kernel().startswith("qskinny_mfma")
            gpu.set_option("qskinny", 2)
            Ct = run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array(zp, np.uint8), bias=bias)
            assert not gpu.last_kernel().startswith("qskinny")
        finally:
            gpu.set_option("qskinny", 0)
        assert np.array_equal(Cg, Ct)


@pytest.mark.parametrize("shape", [(5, 50, 5760), (32, 999, 3072), (16, 520, 16384), (1, 2048, 5760), (20, 1000, 784), (8, 64, 64),
                                   (3, 17, 80), (16, 4100, 1024), (31, 33, 8176), (9, 300, 8208), (2, 70, 12304), (16, 48, 2048 + 16)])
def test_weight_streaming_any_k_any_n(gpu, ob, shape):
    """The streaming kernel on reductions that are no multiple of a wavefront's slab (K = 5760 of l-ten's quantized MNIST
    layer, 784, 3072, a partial last 64-byte step, a last wavefront with a short or empty share, two slab passes above
    8192) and on row counts N that are no multiple of 16: int32 and u8 against the oracle, all zero-point patterns."""
    M, N, K = shape
    rng = np.random.default_rng(M * 5 + N * 3 + K)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    gpu.set_option("qskinny", 1)
    try:
        for zp in ([128, 128, 128], [3, 128, 9], [128, 200, 0], [17, 250, 100]):
            bias = rng.integers(-9999, 9999, N).astype(np.int32) if zp[0] != 128 else None
            run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array(zp, np.uint8), bias=bias)
            assert gpu.last_kernel().startswith("qskinny_mfma"), gpu.last_kernel()
    finally:
        gpu.set_option("qskinny", 0)


@pytest.mark.parametrize("M", [33, 47, 64])
def test_33_to_64_rows_on_the_tiles(gpu, ob, M):
    """33 to 64 activation rows against 2048 x 2048 weights: beyond the streaming kernel's 32 rows the one-launch kernel or
    the 128 x 128 tiles take over (two streaming passes were slower); with zero-point terms and bias, u8 and int32
    outputs, against the oracle."""
    rng = np.random.default_rng(M)
    A = rng.integers(0, 256, (M, 2048), dtype=np.uint8)
    B = rng.integers(0, 256, (2048, 2048), dtype=np.uint8)
    for zp in ([128, 128, 128], [17, 250, 100]):
        bias = rng.integers(-9999, 9999, 2048).astype(np.int32) if zp[0] != 128 else None
        run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array(zp, np.uint8), bias=bias)
        assert gpu.last_kernel().startswith(("qgemm_fast_128x128x128", "qdirect_16x16")), gpu.last_kernel()   # (whichever the cost model puts ahead)


@pytest.mark.parametrize("shape", [(64, 512, 784), (1, 10, 16), (17, 33, 48), (100, 70, 1040), (16, 16, 16384), (33, 250, 2064),
                                   (2100, 50, 784), (600, 210, 1040)])
def test_small_output_kernel(gpu, ob, shape):
    """At most 512 output tiles of 16x16 (8192 when N is no multiple of 4: 528 and 532 tiles in the last two), K % 16 == 0: the one-launch kernel with in-kernel zero-point sums (ragged
    M and N, K tails inside a 64-byte step, both wavefront counts), against the oracle and the tiled kernels."""
    M, N, K = shape
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    for zp, scales in (([128, 128, 128], [0.02, 0.013, 0.9]), ([0, 128, 128], [1 / 255, 0.01, 0.05]),
                       ([128, 200, 0], [0.02, 0.013, 0.9]), ([17, 250, 100], [0.5, 0.5, 0.2])):
        bias = rng.integers(-9999, 9999, N).astype(np.int32) if zp[0] != 128 else None
        Cg = run_case(gpu, ob, A, B, scales, np.array(zp, np.uint8), bias=bias)
        assert gpu.last_kernel().startswith("qdirect_16x16"), gpu.last_kernel()
        gpu.set_option("qskinny", 2)
        try:
            Ct = run_case(gpu, ob, A, B, scales, np.array(zp, np.uint8), bias=bias)
            assert not gpu.last_kernel().startswith("qdirect")
        finally:
            gpu.set_option("qskinny", 0)
        assert np.array_equal(Cg, Ct)


@pytest.mark.parametrize("M", [5, 29])
def test_weight_streaming_many_row_groups(gpu, ob, M):
    """More groups of 16 weight rows than workgroups (600 against 256): a workgroup walks two or three groups
    with the activations kept in registers; zero-point sums and bias active; one and two activation row blocks."""
    N, K = 9600, 8192
    rng = np.random.default_rng(11 + M)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K), dtype=np.uint8)
    bias = rng.integers(-9999, 9999, N).astype(np.int32)
    run_case(gpu, ob, A, B, [0.02, 0.013, 0.9], np.array([17, 250, 100], np.uint8), bias=bias)
    assert gpu.last_kernel().startswith("qskinny_mfma_w8")


@pytest.mark.parametrize("M", [1, 4, 16])
def test_cfg4_skinny(gpu, wl, M):
    X, W, sc, zp = wl.cfg4(M)
    N = K = 8192
    Cg, accg = gpu.qgemm_host(X, W, sc, zp, want_acc=True)
    assert gpu.last_kernel() == "qskinny_mfma_w8"
    want = exact_acc(X, W, int(zp[0]), int(zp[1]))
    assert np.array_equal(accg, want)
    mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
    assert np.array_equal(Cg, requant_numpy(want, mult, int(zp[2])))


def test_seeded_sweep_over_dispatch_boundaries(gpu, ob):
    """Sixty seeded shapes around the limits at which the library changes kernels (32 / 64 rows, 128-tile edges, N a
    multiple of 4 or not, K a multiple of 16 / 128 or not, short and long K), each with random zero points, with and
    without bias, u8 and int32 outputs against the oracle; the kernel names show that every family took part."""
    rng = np.random.default_rng(20240607)
    seen, seen_prepared = set(), set()
    Ms = [1, 2, 15, 16, 17, 31, 32, 33, 47, 63, 64, 65, 100, 127, 128, 129, 200, 255, 257, 300]
    Ns = [1, 10, 16, 36, 100, 128, 130, 132, 256, 500, 512, 1000, 1024, 2048, 2052]
    Ks = [1, 7, 16, 48, 100, 128, 144, 512, 528, 784, 1000, 1024, 2048, 2064, 4096]
    larger = [(1024, 1000, 1024), (520, 2052, 784), (1025, 516, 2064), (2100, 2048, 144)]   # where the 128 x 128 tiles are ahead of the one-launch kernel
    for case in range(60 + len(larger)):
        if case < 60:
            M, N, K = int(rng.choice(Ms)), int(rng.choice(Ns)), int(rng.choice(Ks))
            while M * N * K > 6e7:
                M = max(1, M // 2)
        else:
            M, N, K = larger[case - 60]
        A = rng.integers(0, 256, (M, K), dtype=np.uint8)
        B = rng.integers(0, 256, (N, K), dtype=np.uint8)
        zp = np.array([rng.choice([0, 128, int(rng.integers(0, 256))]) for _ in range(3)], np.uint8)
        sc = [0.02, 0.013, float(rng.choice([0.9, 0.05, 7.0]))]
        bias = rng.integers(-20000, 20000, N).astype(np.int32) if rng.integers(0, 2) else None
        Cg = run_case(gpu, ob, A, B, sc, zp, bias=bias)
        seen.add(gpu.last_kernel().split("_")[0] + "_" + gpu.last_kernel().split("_")[1])
        # the same layer on prepared weights with their kept sums: the same bytes, whatever kernel the shape selects
        Cp, kp = fcq(gpu, gpu.lib().lten_hip_fcq_forward_prepared, A, B, sc, zp, bias, prepared=True)
        assert np.array_equal(Cp, Cg), (M, N, K, zp, kp)
        seen_prepared.add(kp.split("_")[0] + "_" + kp.split("_")[1] + ("+zp" if "+zp" in kp else ""))
    assert {"qskinny_mfma", "qdirect_16x16", "qgemm_fast", "qgemm_guard"} <= seen, seen
    # (prepared weights keep their rows on 16-byte boundaries, so the guarded kernel no longer sees them)
    assert {"qgemm_fast+zp", "qdirect_16x16", "qskinny_mfma"} <= seen_prepared, seen_prepared


def fcq(gpu, entry, X, W, sc, zp, bias=None, prepared=False):
    """One FullyConnected_q forward through `entry` (lten_hip_fcq_forward or _prepared); numpy in, numpy out."""
    D = gpu.DeviceBuffer
    M, K = X.shape
    N = W.shape[0]
    dX, dW, dY, ws = D.from_numpy(X), D.from_numpy(W), D(M * N), D(4 * (M + N))
    db = D.from_numpy(np.asarray(bias, np.int32)) if bias is not None else None
    if prepared:
        Kp = (K + 15) // 16 * 16   # rows of the prepared form start on 16-byte boundaries, zeros behind the weights
        dWp, dS = D(N * Kp + 16), D(4 * N + 16)
        gpu.check(gpu.lib().lten_hip_fcq_prepare_weights(dW.ptr, dWp.ptr, N, K, dS.ptr))
        Wp = dWp.numpy(np.uint8, (N, Kp))
        assert np.array_equal(Wp[:, :K], W ^ 0x80) and not Wp[:, K:].any()
        assert np.array_equal(dS.numpy(np.int32, (N,)), W.sum(axis=1, dtype=np.int64))
        gpu.check(entry(1, M, K, N, dX.ptr, dWp.ptr, dS.ptr, db.ptr if db else None, gpu.qparams3(sc, zp), dY.ptr, ws.ptr))
    else:
        gpu.check(entry(1, M, K, N, dX.ptr, dW.ptr, db.ptr if db else None, gpu.qparams3(sc, zp), dY.ptr, ws.ptr))
    return dY.numpy(np.uint8, (M, N)), gpu.last_kernel()


@pytest.mark.parametrize("shape", [(64, 512, 784), (16, 2048, 2048), (40, 4096, 2048), (256, 512, 640), (128, 1024, 4096),
                                   (512, 8192, 512), (300, 260, 400), (70, 50, 5760), (33, 65, 100)])
def test_prepared_weights_match_unprepared(gpu, ob, shape):
    """lten_hip_fcq_forward_prepared on int8 weights (w - 128) returns what lten_hip_fcq_forward returns on l-ten's
    uint8 weights, on every kernel family the shapes select (one-launch, streaming, split-K, 128 and 256 tiles with and
    without a partial k-step, the guarded general kernel), with all three zero-point patterns and a bias; the
    unprepared result is checked against the oracle."""
    M, N, K = shape
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    X = rng.integers(0, 256, (M, K), dtype=np.uint8)
    W = rng.integers(0, 256, (N, K), dtype=np.uint8)
    l = gpu.lib()
    for zp, with_bias in (([128, 128, 128], False), ([0, 128, 3], True), ([200, 17, 99], True)):
        bias = rng.integers(-5000, 5000, N).astype(np.int32) if with_bias else None
        sc = [0.02, 0.013, 0.9 * K / 512]
        want, k0 = fcq(gpu, l.lten_hip_fcq_forward, X, W, sc, zp, bias)
        got, k1 = fcq(gpu, l.lten_hip_fcq_forward_prepared, X, W, sc, zp, bias, prepared=True)
        assert np.array_equal(got, want), (shape, zp, k0, k1)
        # the direct-to-LDS tiles on prepared weights take the zero-point terms in the same launch
        # (the name says which terms the launch took on; the unfused form is a launch of qgemm_terms_kernel before it)
        if k1.startswith("qgemm_fast"):
            assert k1.endswith("" if zp == [128, 128, 128] and not with_bias else "+zpcol" if zp[1] == 128 else "+zpcol+zprow"), k1
        Co, _ = ob.quantized_matmul(X, W, np.array(sc, np.float32), np.array(zp, np.uint8), bias=bias)
        assert np.array_equal(want, Co), (shape, zp, k0)


@pytest.mark.parametrize("shape", [(1, 4096, 4100), (16, 512, 1000), (64, 512, 1000), (128, 1000, 1000), (300, 260, 401), (1024, 1024, 1000),
                                   (512, 10, 50), (700, 520, 2050), (33, 65, 100), (40, 4096, 1937)])
def test_rows_that_are_no_multiple_of_16_bytes(gpu, ob, shape):
    """A layer whose in_features is no multiple of 16 (l-ten's own quantized MNIST network has one of 50): the product runs on
    copies with padded rows, through the kernels of the padded shape instead of the guarded general kernel, and returns
    the oracle's bytes and int32 sums through every entry point, with every zero-point pattern and a bias."""
    M, N, K = shape
    rng = np.random.default_rng(M * 11 + N * 5 + K)
    X = rng.integers(0, 256, (M, K), dtype=np.uint8)
    W = rng.integers(0, 256, (N, K), dtype=np.uint8)
    l = gpu.lib()
    for zp, with_bias in (([128, 128, 128], False), ([0, 128, 3], True), ([200, 17, 99], True), ([255, 0, 255], False)):
        bias = rng.integers(-5000, 5000, N).astype(np.int32) if with_bias else None
        sc = [0.02, 0.013, 0.9 * K / 512]
        Co, acco = ob.quantized_matmul(X, W, np.array(sc, np.float32), np.array(zp, np.uint8), bias=bias)
        raw, k0 = fcq(gpu, l.lten_hip_fcq_forward, X, W, sc, zp, bias)
        got, k1 = fcq(gpu, l.lten_hip_fcq_forward_prepared, X, W, sc, zp, bias, prepared=True)
        _, accg = gpu.qgemm_host(X, W, np.array(sc, np.float32), np.array(zp, np.uint8), bias=bias, want_acc=True)
        assert np.array_equal(raw, Co), (shape, zp, k0)
        assert np.array_equal(got, Co), (shape, zp, k1)
        assert np.array_equal(accg, acco), (shape, zp)
        if N % 4 == 0 and M * N * K >= 1 << 20:
            assert "guard" not in k0 and "guard" not in k1, (k0, k1)
    # the entry point that allocates nothing has no memory for such copies and keeps the guarded kernel: same bytes
    D = gpu.DeviceBuffer
    dX, dW, dY = D.from_numpy(X), D.from_numpy(W), D(M * N)
    db = D.from_numpy(bias) if bias is not None else None
    gpu.check(l.lten_hip_fcq_forward_static(1, M, K, N, dX.ptr, dW.ptr, db.ptr if db else None, gpu.qparams3(sc, zp), dY.ptr))
    assert np.array_equal(dY.numpy(np.uint8, (M, N)), Co)


@pytest.mark.parametrize("tA,tB", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("shape", [(300, 260, 400), (200, 130, 1000), (65, 1030, 333), (1024, 512, 512)])
def test_operands_that_lie_with_k_outermost(gpu, ob, shape, tA, tB):
    """quantized_matmul with a transposed A ([K x M] in memory) or an untransposed B ([K x N], how l-ten's Conv2d_q calls
    it): the operands are copied into the layers' layout (rows contiguous in K, padded to a multiple of 16 bytes) and the
    product runs on the kernels of that layout; int32 sums and bytes against the oracle."""
    M, N, K = shape
    rng = np.random.default_rng(M + 3 * N + 7 * K + 2 * tA + tB)
    A = rng.integers(0, 256, (K, M) if tA else (M, K), dtype=np.uint8)
    B = rng.integers(0, 256, (N, K) if tB else (K, N), dtype=np.uint8)
    for zp, with_bias in (([128, 128, 128], False), ([7, 201, 99], True)):
        bias = rng.integers(-5000, 5000, N).astype(np.int32) if with_bias else None
        run_case(gpu, ob, A, B, [0.02, 0.013, 0.9 * K / 512], np.array(zp, np.uint8), tA=tA, tB=tB, bias=bias, M=M, N=N, K=K)
        assert "guard" not in gpu.last_kernel(), gpu.last_kernel()


def test_padded_rows_inside_a_recorded_launch_graph(gpu, ob):
    """A prepared layer of 1000 inputs run once eagerly (which allocates the memory of the padded copy) and then
    recorded: the copy and the product both land in the graph, and every replay on new activations matches the oracle."""
    l, D = gpu.lib(), gpu.DeviceBuffer
    rng = np.random.default_rng(1000)
    M, N, K = 96, 512, 1000
    Kp = (K + 15) // 16 * 16
    W = rng.integers(0, 256, (N, K), dtype=np.uint8)
    sc, zp = [0.02, 0.013, 0.9], [5, 200, 90]
    dX, dW, dWp, dS, dY, ws = D(M * K), D.from_numpy(W), D(N * Kp), D(4 * N), D(M * N), D(4 * (M + N))
    gpu.check(l.lten_hip_fcq_prepare_weights(dW.ptr, dWp.ptr, N, K, dS.ptr))
    qp = gpu.qparams3(sc, zp)
    call = lambda: gpu.check(l.lten_hip_fcq_forward_prepared(1, M, K, N, dX.ptr, dWp.ptr, dS.ptr, None, qp, dY.ptr, ws.ptr))
    dX.upload(rng.integers(0, 256, (M, K), dtype=np.uint8))
    call()
    with gpu.Graph() as g:
        call()
    for rep in range(3):
        X = rng.integers(0, 256, (M, K), dtype=np.uint8)
        dX.upload(X)
        gpu.check(l.lten_hip_zero(dY.ptr, M * N))
        g.launch()
        want, _ = ob.quantized_matmul(X, W, np.array(sc, np.float32), np.array(zp, np.uint8))
        assert np.array_equal(dY.numpy(np.uint8, (M, N)), want), rep
        if rep == 1:
            # an eager call that needs far more of that memory than anything before it: the library takes a new block,
            # and the one whose address the recording holds must stay where it is for the replay that follows
            Mb, Nb = 60000, 16
            Xb = rng.integers(0, 256, (Mb, K), dtype=np.uint8)
            Wb = rng.integers(0, 256, (Nb, K), dtype=np.uint8)
            dXb, dWb, dYb, wsb = D.from_numpy(Xb), D.from_numpy(Wb), D(Mb * Nb), D(4 * (Mb + Nb))
            gpu.check(l.lten_hip_fcq_forward(1, Mb, K, Nb, dXb.ptr, dWb.ptr, None, qp, dYb.ptr, wsb.ptr))
            wb, _ = ob.quantized_matmul(Xb[:500], Wb, np.array(sc, np.float32), np.array(zp, np.uint8))
            assert np.array_equal(dYb.numpy(np.uint8, (Mb, Nb))[:500], wb)


def test_prepare_weights_in_place_and_odd_count(gpu):
    rng = np.random.default_rng(5)
    for n in (16, 4096, 1 << 20):   # rows that are multiples of 16 bytes: in place
        w = rng.integers(0, 256, n, dtype=np.uint8)
        d = gpu.DeviceBuffer.from_numpy(w)
        gpu.check(gpu.lib().lten_hip_fcq_prepare_weights(d.ptr, d.ptr, 1, n, None))
        assert np.array_equal(d.numpy(np.uint8, (n,)), w ^ 0x80)
    # with and without the row sums, on rows of any length (16-byte loads only where every row allows them); rows that are
    # no multiple of 16 bytes are padded with zeros to the next one, which cannot happen in place
    for rows, cols in ((1, 1), (1, 15), (1, 17), (1, 4099), (3, 15), (5, 16), (7, 100), (130, 784), (64, 4099), (33, 4096)):
        w = rng.integers(0, 256, (rows, cols), dtype=np.uint8)
        cp = (cols + 15) // 16 * 16
        for with_sums in (True, False):
            d, sums = gpu.DeviceBuffer.from_numpy(w), gpu.DeviceBuffer(4 * rows + 16)
            out = d if cp == cols else gpu.DeviceBuffer(rows * cp, zero=False)
            gpu.check(gpu.lib().lten_hip_fcq_prepare_weights(d.ptr, out.ptr, rows, cols, sums.ptr if with_sums else None))
            got = out.numpy(np.uint8, (rows, cp))
            assert np.array_equal(got[:, :cols], w ^ 0x80) and not got[:, cols:].any()
            if with_sums:
                assert np.array_equal(sums.numpy(np.int32, (rows,)), w.sum(axis=1, dtype=np.int64))
        if cp != cols:
            d = gpu.DeviceBuffer.from_numpy(np.concatenate([w.ravel(), np.zeros(rows * (cp - cols), np.uint8)]))
            assert gpu.lib().lten_hip_fcq_prepare_weights(d.ptr, d.ptr, rows, cols, None) != 0
            assert b"must not overlap" in gpu.lib().lten_hip_last_error()


def test_cfg3_prepared_weights_full_size(gpu, wl):
    """Config 3 at full size through the prepared-weights entry point: bit-identical to the plain entry point."""
    X, W, sc, zp = wl.cfg3()
    l = gpu.lib()
    want, k0 = fcq(gpu, l.lten_hip_fcq_forward, X, W, sc, zp)
    got, k1 = fcq(gpu, l.lten_hip_fcq_forward_prepared, X, W, sc, zp, prepared=True)
    assert k1.endswith("_wpre") and not k0.endswith("_wpre"), (k0, k1)
    assert np.array_equal(got, want)


ZP_FUSED = ([0, 128, 128], [17, 250, 100])   # a post-relu activation tensor against symmetric weights; every term needed


@pytest.mark.parametrize("tile", [33, 41, 51, 0])
@pytest.mark.parametrize("shape", [(512, 512, 512), (300, 260, 400), (256, 384, 4096), (130, 1024, 8192)])
def test_prepared_forward_takes_zero_point_terms_in_the_gemm_launch(gpu, ob, shape, tile):
    """Prepared weights with their row sums: the direct-to-LDS tiles (256 x 256, 128 x 128, 256 x 128, forced by option,
    and whatever the heuristic picks, split-K included) work out the column term from the kept sums and the row term
    from the activation fragments, in the one launch, with and without a bias (16-byte aligned and not), whole and
    ragged tiles and a partial last k-step.  Checked against the oracle."""
    M, N, K = shape
    rng = np.random.default_rng(M * 5 + N * 3 + K + tile)
    X = rng.integers(0, 256, (M, K), dtype=np.uint8)
    W = rng.integers(0, 256, (N, K), dtype=np.uint8)
    l, D = gpu.lib(), gpu.DeviceBuffer
    dX, dW, dWp, dS, dY, ws = D.from_numpy(X), D.from_numpy(W), D(W.size), D(4 * N), D(M * N), D(4 * (M + N))
    gpu.check(l.lten_hip_fcq_prepare_weights(dW.ptr, dWp.ptr, N, K, dS.ptr))
    bias = rng.integers(-5000, 5000, N + 1).astype(np.int32)
    dbias = D.from_numpy(bias)
    gpu.set_option("qgemm_tile", tile)
    seen_fast = False
    try:
        for zp in ZP_FUSED:
            for bias_off in (None, 0, 1):
                sc = [0.02, 0.013, 0.9 * K / 512]
                b = None if bias_off is None else bias[bias_off:bias_off + N]
                gpu.check(l.lten_hip_fcq_forward_prepared(1, M, K, N, dX.ptr, dWp.ptr, dS.ptr, None if b is None else dbias.ptr + 4 * bias_off,
                                                          gpu.qparams3(sc, zp), dY.ptr, ws.ptr))
                kern = gpu.last_kernel()
                assert tile == 0 or kern.startswith("qgemm_fast"), kern   # (small outputs go to the one-launch kernel by themselves)
                if kern.startswith("qgemm_fast"):
                    assert kern.endswith("+zpcol" if zp[1] == 128 else "+zpcol+zprow"), kern
                    seen_fast = True
                want, _ = ob.quantized_matmul(X, W, np.array(sc, np.float32), np.array(zp, np.uint8), bias=b)
                assert np.array_equal(dY.numpy(np.uint8, (M, N)), want), (shape, tile, zp, bias_off, kern)
    finally:
        gpu.set_option("qgemm_tile", 0)
    assert seen_fast or shape in ((300, 260, 400), (256, 384, 4096), (512, 512, 512)), shape


@pytest.mark.parametrize("zp", ZP_FUSED)
def test_cfg3_shape_with_general_zero_points_full_size(gpu, wl, zp):
    """4096^3 with zero points other than 128 on prepared weights: one launch (the name says so), every output equal to
    the requantize rule applied to the exact closed form of the accumulator."""
    X, W, sc, _ = wl.cfg3()
    M = N = K = 4096
    l, D = gpu.lib(), gpu.DeviceBuffer
    dX, dW, dWp, dS, dY = D.from_numpy(X), D.from_numpy(W), D(W.size), D(4 * N), D(M * N)
    gpu.check(l.lten_hip_fcq_prepare_weights(dW.ptr, dWp.ptr, N, K, dS.ptr))
    gpu.check(l.lten_hip_fcq_forward_prepared(1, M, K, N, dX.ptr, dWp.ptr, dS.ptr, None, gpu.qparams3(sc, zp), dY.ptr, None))
    assert gpu.last_kernel() == "qgemm_fast_256x256x128_w4x2_s2_wpre" + ("+zpcol" if zp[1] == 128 else "+zpcol+zprow"), gpu.last_kernel()
    want = exact_acc(X, W, zp[0], zp[1])
    mult = np.float32(np.float32(sc[0]) * np.float32(sc[1])) / np.float32(sc[2])
    assert np.array_equal(dY.numpy(np.uint8, (M, N)), requant_numpy(want, mult, zp[2]))
