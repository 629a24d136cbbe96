"""GPU parity tests of im2col / col2im and the fused Conv2d forward + weight gradient (C ABI).
im2col and col2im are data movement / fixed-order sums: bit-exact.  Convolutions: max relative error 1e-4
(conftest.rel_err)."""
import numpy as np
import pytest

from conftest import golden_path, rel_err
from test_oracle_conv import GEOS, direct_conv

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.mark.parametrize("geo", GEOS + [(3, 33, 47, 3, 3, 1, 1, 1, 1), (2, 64, 64, 5, 3, 2, 1, 2, 2)])
def test_im2col_col2im_bit_exact(gpu, ob, geo):
    C, H, W, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    im = rng.standard_normal((C, H, W)).astype(np.float32)
    col = np.empty((C * kh * kw, Ho * Wo), np.float32)
    ob.oracle().oracle_im2col_f32(im.reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, col.reshape(-1))
    D = gpu.DeviceBuffer
    dIm, dCol = D.from_numpy(im), D(col.nbytes)
    gpu.check(gpu.lib().lten_hip_im2col_f32(dIm.ptr, C, H, W, kh, kw, ph, pw, sh, sw, 1, 1, dCol.ptr))
    assert np.array_equal(dCol.numpy(np.float32, col.shape), col)
    # uint8 flavour (Conv2d_q's operand)
    imu = rng.integers(0, 256, (C, H, W), dtype=np.uint8)
    colu = np.empty((C * kh * kw, Ho * Wo), np.uint8)
    ob.oracle().oracle_im2col_u8(imu.reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, colu.reshape(-1))
    dImu, dColu = D.from_numpy(imu), D(colu.nbytes)
    gpu.check(gpu.lib().lten_hip_im2col_u8(dImu.ptr, C, H, W, kh, kw, ph, pw, sh, sw, 1, 1, dColu.ptr))
    assert np.array_equal(dColu.numpy(np.uint8, colu.shape), colu)
    # col2im: same taps in the same order as the CPU scatter-add -> identical floats
    c = rng.standard_normal(col.shape).astype(np.float32)
    back = np.zeros_like(im)
    ob.oracle().oracle_col2im_f32(c.reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, back.reshape(-1))
    dC, dBack = D.from_numpy(c), D(im.nbytes)
    gpu.check(gpu.lib().lten_hip_col2im_f32(dC.ptr, C, H, W, kh, kw, ph, pw, sh, sw, 1, 1, dBack.ptr))
    assert np.array_equal(dBack.numpy(np.float32, im.shape), back)
    # the int and uint8 instantiations (l-ten/im_col.cu:199-218): integers small enough to be exact as floats go through
    # the same oracle functions; uint8 sums wrap modulo 256 as the template's `+=` on uint8_t does
    imi = rng.integers(-100000, 100000, (C, H, W)).astype(np.int32)
    coli = np.empty(col.shape, np.float32)
    ob.oracle().oracle_im2col_f32(imi.astype(np.float32).reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, coli.reshape(-1))
    dImi, dColi = D.from_numpy(imi), D(4 * col.size)
    gpu.check(gpu.lib().lten_hip_im2col_i32(dImi.ptr, C, H, W, kh, kw, ph, pw, sh, sw, 1, 1, dColi.ptr))
    assert np.array_equal(dColi.numpy(np.int32, col.shape), coli.astype(np.int32))
    ci = rng.integers(-1000, 1000, col.shape).astype(np.int32)
    backi = np.zeros(im.shape, np.float32)
    ob.oracle().oracle_col2im_f32(ci.astype(np.float32).reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, backi.reshape(-1))
    dCi, dBacki = D.from_numpy(ci), D(4 * im.size)
    gpu.check(gpu.lib().lten_hip_col2im_i32(dCi.ptr, C, H, W, kh, kw, ph, pw, sh, sw, 1, 1, dBacki.ptr))
    assert np.array_equal(dBacki.numpy(np.int32, im.shape), backi.astype(np.int32))
    cu = rng.integers(0, 256, col.shape, dtype=np.uint8)
    backu = np.zeros(im.shape, np.float32)
    ob.oracle().oracle_col2im_f32(cu.astype(np.float32).reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, backu.reshape(-1))
    dCu, dBacku = D.from_numpy(cu), D(im.size)
    gpu.check(gpu.lib().lten_hip_col2im_u8(dCu.ptr, C, H, W, kh, kw, ph, pw, sh, sw, 1, 1, dBacku.ptr))
    assert np.array_equal(dBacku.numpy(np.uint8, im.shape), (backu.astype(np.int64) % 256).astype(np.uint8))


def gpu_conv(gpu, geo, x, w, dy=None, bias=None):
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    Ho, Wo = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    D = gpu.DeviceBuffer
    dX, dW = D.from_numpy(x), D.from_numpy(w)
    dB = D.from_numpy(bias) if bias is not None else None
    dY = D(4 * N * Cout * Ho * Wo)
    l = gpu.lib()
    gpu.check(l.lten_hip_conv2d_forward_f32(*geo, dX.ptr, dW.ptr, dB.ptr if dB else None, dY.ptr))
    fk = gpu.last_kernel()
    y = dY.numpy(np.float32, (N, Cout, Ho, Wo))
    dw = None
    if dy is not None:
        dDY = D.from_numpy(dy)
        ws = D(max(int(l.lten_hip_conv2d_wgrad_workspace_bytes(*geo)), 4))
        dDW = D(w.nbytes)
        gpu.check(l.lten_hip_conv2d_wgrad_f32(*geo, dX.ptr, dDY.ptr, dDW.ptr, ws.ptr))
        dw = dDW.numpy(np.float32, w.shape)
    return y, dw, fk


def gpu_dgrad(gpu, geo, w, dy):
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    D, l = gpu.DeviceBuffer, gpu.lib()
    dW, dDY, dDX = D.from_numpy(w), D.from_numpy(dy), D(4 * N * Cin * H * W)
    ws = D(max(int(l.lten_hip_conv2d_dgrad_workspace_bytes(*geo)), 4))
    gpu.check(l.lten_hip_conv2d_dgrad_f32(*geo, dW.ptr, dDY.ptr, dDX.ptr, ws.ptr))
    return dDX.numpy(np.float32, (N, Cin, H, W))


def test_conv_layer_golden(gpu):
    g = np.load(golden_path("layer_cases.npz"))
    for i in range(int(g["conv_count"])):
        pre = f"cv{i}_"
        geo = tuple(int(v) for v in g[pre + "geo"])
        y, dw, _ = gpu_conv(gpu, geo, g[pre + "x"], g[pre + "w"], g[pre + "dy"])
        assert rel_err(y.reshape(-1), g[pre + "y"]) < TOL, i
        assert rel_err(dw.reshape(-1), g[pre + "dw"]) < TOL, i
        assert rel_err(gpu_dgrad(gpu, geo, g[pre + "w"], g[pre + "dy"]).reshape(-1), g[pre + "dx"]) < TOL, i


@pytest.mark.parametrize("geo", [(2, 3, 9, 8, 4, 3, 3, 1, 1, 1, 1), (1, 2, 10, 7, 3, 3, 2, 0, 1, 2, 1),
                                 (2, 4, 6, 6, 5, 5, 5, 2, 2, 1, 1), (3, 16, 33, 29, 40, 3, 3, 1, 1, 1, 1),
                                 (2, 8, 40, 40, 70, 3, 3, 1, 1, 2, 2), (2, 1, 64, 64, 32, 3, 3, 1, 1, 1, 1),
                                 # 3x3 stride 1 (LDS patch kernels): several column tiles and channel blocks, rows
                                 # that are / are not a multiple of four floats, pad 0 / 1 / 2, ragged channel counts
                                 (2, 20, 17, 136, 70, 3, 3, 1, 1, 1, 1), (1, 37, 12, 64, 33, 3, 3, 0, 0, 1, 1),
                                 (2, 9, 8, 20, 8, 3, 3, 2, 2, 1, 1), (1, 64, 5, 260, 130, 3, 3, 1, 0, 1, 1), (2, 12, 10, 36, 96, 3, 3, 1, 1, 1, 1),
                                 # input channels a multiple of four (patch filled by direct-to-LDS loads): 64-channel
                                 # workgroups with a ragged second column tile, ragged channel count with pad 2, one chunk pair
                                 (2, 8, 9, 132, 64, 3, 3, 1, 1, 1, 1), (1, 16, 6, 128, 100, 3, 3, 2, 2, 1, 1), (1, 32, 7, 12, 128, 3, 3, 0, 1, 1, 1),
                                 # pad 1 and rows of whole 64-pixel chunks (weight gradient with both tiles filled by
                                 # direct-to-LDS loads): ragged channel blocks on both sides with one column tile, a
                                 # single image row (halo above and below at once), three column tiles (the middle
                                 # one has no halo outside the image), two full blocks each way
                                 (2, 40, 5, 64, 70, 3, 3, 1, 1, 1, 1), (1, 32, 1, 64, 64, 3, 3, 1, 1, 1, 1),
                                 (3, 12, 3, 192, 33, 3, 3, 1, 1, 1, 1), (2, 64, 6, 128, 128, 3, 3, 1, 1, 1, 1),
                                 # at most four output channels (forward) or input channels (data gradient) with column
                                 # pad 1: the streaming kernel on the vector ALUs; ragged tiles both ways, row pad 0 / 1 / 2
                                 (2, 8, 9, 132, 3, 3, 3, 1, 1, 1, 1), (1, 4, 5, 8, 1, 3, 3, 0, 1, 1, 1), (2, 12, 17, 260, 4, 3, 3, 2, 1, 1, 1),
                                 (2, 2, 10, 64, 16, 3, 3, 1, 1, 1, 1), (1, 4, 7, 36, 8, 3, 3, 0, 1, 1, 1), (3, 1, 20, 128, 32, 3, 3, 1, 1, 1, 1),
                                 # one or two input channels at the smallest sizes: a single quad of pixels, one row, row pad 2,
                                 # a channel count that is no multiple of the groups of eight
                                 (1, 1, 1, 4, 1, 3, 3, 1, 1, 1, 1), (2, 2, 3, 4, 5, 3, 3, 2, 1, 1, 1), (1, 1, 9, 260, 19, 3, 3, 0, 1, 1, 1),
                                 # stride 1 with Cin*kh*kw <= 32 (first-layer kernels): ragged widths, two column
                                 # tiles, more than 32 output channels, 5x5 and 1x1 windows, pad 0 / 1 / 2
                                 (2, 1, 11, 200, 40, 3, 3, 1, 1, 1, 1), (3, 1, 9, 131, 7, 5, 5, 2, 2, 1, 1),
                                 (1, 20, 9, 132, 33, 1, 1, 0, 0, 1, 1), (2, 3, 16, 36, 64, 3, 3, 0, 0, 1, 1),
                                 (5, 2, 7, 9, 3, 2, 7, 1, 4, 1, 1),
                                 # at most 16 taps with rows that allow 16-byte loads: the weight gradient on 16x16x4 MFMA
                                 # tiles (12 taps of a 4x3 window, 15 taps of five channels with a 1x3 window; 33 and 40
                                 # output channels: a ragged second block of 32)
                                 (2, 1, 12, 64, 40, 4, 3, 1, 1, 1, 1), (2, 5, 9, 128, 33, 1, 3, 0, 1, 1, 1)])
@pytest.mark.parametrize("variant", [0, 1, 2, 3, 5])
def test_conv_vs_oracle(gpu, ob, geo, variant):
    """variant 0: the kernel the library picks; 1: the implicit-GEMM kernels for every shape; 2: the register-staged
    patch kernel also where the direct-to-LDS one would run; 3: also the unpipelined weight-gradient kernel; 5: the
    direct-to-LDS forward kernel with four-row tiles also where it would pick two-row tiles."""
    try:
        gpu.set_option("conv_variant", variant)
        _conv_vs_oracle(gpu, ob, geo)
    finally:
        gpu.set_option("conv_variant", 0)


@pytest.mark.parametrize("geo", [(41, 8, 37, 132, 64, 3, 3, 1, 1, 1, 1), (40, 8, 37, 132, 128, 3, 3, 1, 1, 1, 1),
                                 (60, 8, 37, 132, 32, 3, 3, 1, 1, 1, 1)])
def test_conv_many_tiles(gpu, ob, geo):
    """Many tiles of the direct-to-LDS forward kernel in one launch (820, 1600 and 1200, more than the chip holds at a
    time), with a ragged last row tile, a ragged second column tile and several images."""
    _conv_vs_oracle(gpu, ob, geo)


@pytest.mark.parametrize("geo", [(3, 8, 28, 28, 64, 3, 3, 1, 1, 1, 1),      # MNIST-sized: one column tile, two row tiles (the second 12 rows of 16)
                                 (2, 12, 37, 44, 70, 3, 3, 2, 1, 1, 1),     # two column tiles, three row tiles, ragged on every side, row pad 2
                                 (1, 16, 16, 32, 32, 3, 3, 0, 0, 1, 1),     # no padding: 14 x 30 outputs, 32 channels per workgroup
                                 (2, 8, 50, 96, 33, 3, 3, 1, 1, 1, 1),      # the widest image that takes these tiles: three column tiles, ragged channels
                                 (5, 64, 9, 8, 128, 3, 3, 1, 1, 1, 1)])     # a quarter of a tile's columns, two channel blocks of 64
def test_conv_narrow_images_on_16x32_tiles(gpu, ob, geo):
    """Images of at most 96 columns: forward (and the stride-1 data gradient through it) on the direct-to-LDS kernel
    with tiles of 16 rows x 32 columns, against the oracle."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    gpu.set_option("conv_variant", 6)   # these tiles however few workgroups the small test shapes give
    try:
        y, _, fk = gpu_conv(gpu, geo, x, w, dy, bias)
        assert fk.startswith("conv2d_patch_fast_forward_3x3_") and fk.endswith("x16x32"), fk
        _conv_vs_oracle(gpu, ob, geo)
    finally:
        gpu.set_option("conv_variant", 0)


@pytest.mark.parametrize("geo", [(3, 16, 27, 28, 64, 3, 3, 1, 1, 1, 1),      # MNIST-sized with an odd number of rows: the last chunk has one
                                 (2, 40, 9, 96, 33, 3, 3, 0, 1, 1, 1),      # three chunk columns, no row padding, ragged channel blocks
                                 (4, 9, 5, 20, 5, 3, 3, 1, 1, 1, 1),        # 20 of a chunk's 32 columns, the fewest input channels
                                 (2, 70, 30, 32, 130, 3, 3, 2, 1, 1, 1)])   # exactly one chunk column, row pad 2, three channel blocks each way
def test_conv_weight_gradient_on_two_row_chunks(gpu, ob, geo):
    """Narrow images whose rows allow 16-byte loads: the weight gradient walks chunks of two rows x 32 columns."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    gpu_conv(gpu, geo, x, w, dy, None)
    assert gpu.last_kernel() == "conv2d_patch_wgrad_3x3_64x32_2x32", gpu.last_kernel()
    _conv_vs_oracle(gpu, ob, geo)


@pytest.mark.parametrize("geo", [(64, 1, 28, 28, 10, 5, 5, 0, 0, 1, 1),      # l-ten's MNIST conv layer at batch 64: 24 x 24 outputs
                                 (3, 1, 28, 28, 32, 3, 3, 0, 0, 1, 1),      # 26 columns: no 16-byte loads of dy; 8-row patch variant
                                 (5, 3, 33, 32, 40, 3, 3, 1, 1, 1, 1),      # three channels, a ragged last chunk row, two channel blocks
                                 (2, 1, 9, 68, 16, 4, 3, 1, 1, 1, 1)])      # three chunk columns (68 of 96), 12 taps: the 16x16x4 weight gradient
def test_conv_first_layers_of_narrow_images_on_four_row_chunks(gpu, ob, geo):
    """Short reductions (Cin * kh * kw <= 32) on images where chunks of four rows x 32 columns waste fewer pixels than 128
    columns of one row: forward and weight gradient against the oracle."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    _, _, fk = gpu_conv(gpu, geo, x, w, dy, None)
    assert fk.startswith("conv2d_smallk_forward_32x4x32"), fk
    assert gpu.last_kernel().startswith("conv2d_smallk_wgrad_32x4x32"), gpu.last_kernel()
    _conv_vs_oracle(gpu, ob, geo)


@pytest.mark.parametrize("geo", [
    (64, 1, 28, 28, 10, 5, 5, 0, 0, 1, 1),   # l-ten's MNIST layer: eight threads an element, 250 products padded to 256
    (3, 1, 28, 28, 32, 3, 3, 0, 0, 1, 1),    # elements not a multiple of the 32 a workgroup holds
    (2, 4, 19, 23, 7, 4, 2, 2, 1, 1, 1),     # four input channels, even window, padding on both sides
    (32, 2, 64, 64, 3, 4, 4, 1, 1, 1, 1),    # 2^18 elements: one thread an element (three output channels: too few for the GEMM + col2im route that takes larger batches)
    (1, 3, 9, 300, 5, 1, 7, 0, 3, 1, 1),     # one-row window on a wide image
])
def test_conv_data_gradient_of_first_layers(gpu, ob, geo):
    """Data gradient for at most four input channels and a short reduction, outside the 3 x 3 same-size case that the
    few-output kernel takes: one kernel, products shared by the threads of an element, against the oracle."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
    want_dx = np.empty((N, Cin, H, W), np.float32)
    ob.oracle().oracle_conv2d_dgrad(*geo, w.reshape(-1), dy.reshape(-1), want_dx.reshape(-1), col)
    dx = gpu_dgrad(gpu, geo, w, dy)
    assert gpu.last_kernel() == "conv2d_dgrad_direct", gpu.last_kernel()
    assert rel_err(dx, want_dx) < TOL


@pytest.mark.parametrize("geo", [
    (2, 5, 9, 11, 7, 3, 3, 1, 1, 2, 2),       # stride 2, odd sizes
    (3, 16, 12, 10, 40, 5, 3, 2, 1, 2, 3),    # strides 2 x 3, oblong window
    (1, 70, 8, 8, 3, 1, 1, 0, 0, 2, 2),       # 1 x 1 at stride 2: three pixels in four get no gradient
    (2, 8, 15, 15, 8, 4, 4, 1, 1, 3, 3),      # stride 3, even window
    (5, 33, 7, 6, 65, 3, 3, 1, 1, 2, 1),      # two row tiles, columns that cross images
    (2, 4, 1, 9, 6, 1, 3, 0, 1, 3, 2),        # one image row at stride 3: two of the three row classes hold no pixel
])
def test_conv_data_gradient_with_strides(gpu, ob, geo):
    """Data gradient at strides above 1: one implicit-GEMM launch for the batch (rows = input channels, columns = the input
    pixels of one class (y mod sh, x mod sw) per grid row, reduction over the taps that reach that class, per-column
    tables of the output rows and columns each tap reaches), against the oracle."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
    want_dx = np.empty((N, Cin, H, W), np.float32)
    ob.oracle().oracle_conv2d_dgrad(*geo, w.reshape(-1), dy.reshape(-1), want_dx.reshape(-1), col)
    dx = gpu_dgrad(gpu, geo, w, dy)
    assert gpu.last_kernel() == "conv2d_dgrad_64x64x32", gpu.last_kernel()
    assert rel_err(dx, want_dx) < TOL


@pytest.mark.parametrize("geo", [(3, 64, 20, 20, 48, 1, 1, 0, 0, 1, 1), (2, 100, 13, 17, 70, 1, 1, 0, 0, 1, 1), (5, 40, 56, 56, 256, 1, 1, 0, 0, 1, 1)])
def test_conv_1x1_layers_as_batched_products(gpu, ob, geo):
    """A 1 x 1 layer without bias, and its data gradient, run as a strided batch of plain products on the images as they
    lie in memory; with a bias only where a pass over y that adds it pays (not at these sizes: the convolution kernels).
    Both against the oracle."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, 1, 1)) * 0.2).astype(np.float32)
    dy = rng.standard_normal((N, Cout, H, W)).astype(np.float32)
    col = np.empty(Cin * H * W, np.float32)
    want_y = np.empty((N, Cout, H, W), np.float32)
    ob.oracle().oracle_conv2d_forward(*geo, x.reshape(-1), w.reshape(-1), want_y.reshape(-1), col)
    y, _, fk = gpu_conv(gpu, geo, x, w)
    assert fk == "conv2d_1x1_batched_gemm", fk
    assert rel_err(y, want_y) < TOL
    want_dx = np.empty_like(x)
    ob.oracle().oracle_conv2d_dgrad(*geo, w.reshape(-1), dy.reshape(-1), want_dx.reshape(-1), col)
    dx = gpu_dgrad(gpu, geo, w, dy)
    assert gpu.last_kernel() == "conv2d_1x1_batched_gemm", gpu.last_kernel()
    assert rel_err(dx, want_dx) < TOL
    _conv_vs_oracle(gpu, ob, geo)   # with a bias: the convolution kernels


@pytest.mark.parametrize("geo", [(1, 96, 12, 12, 96, 3, 3, 1, 1, 1, 1),       # one image: a single product on the 32 x 32 tiles; its data gradient the same way
                                 (1, 192, 10, 10, 96, 3, 3, 1, 1, 1, 1),     # one image, K = 1728: the product splits its reduction, partial sums behind the columns
                                 (3, 64, 16, 12, 130, 3, 3, 1, 1, 2, 1),     # strides (2, 1), ragged channel blocks
                                 (2, 60, 12, 12, 100, 3, 3, 1, 1, 1, 1),     # K = 540: whole k-steps, then the rest in a second pass
                                 (16, 64, 16, 16, 128, 3, 3, 1, 1, 1, 1),    # enough tiles for the 64 x 64 direct-to-LDS kernel
                                 (4, 512, 7, 7, 256, 1, 1, 0, 0, 1, 1),      # 1 x 1 on 7 x 7 maps: 49 pixels, rows of the columns padded to 52
                                 (3, 64, 9, 9, 100, 3, 3, 1, 1, 1, 1),       # 81 pixels
                                 (63, 96, 7, 7, 128, 3, 3, 1, 1, 1, 1),      # 63 images of 49 pixels: one product with 3087 columns (images start off 16-byte boundaries)
                                 (64, 96, 14, 14, 128, 3, 3, 1, 1, 1, 1)])   # 64 images of 196 pixels: one product with 12544 columns, no tile padded per image
def test_conv_deep_layers_on_small_images_by_column_matrices(gpu, ob, geo):
    """Many channels on images too small for the patch tiles: the batch's column matrices go to memory of the library in one
    launch, one product over all pixels of the batch (or a strided batch of products, one per image) writes y, a pass adds
    the bias.  Forward (with and without bias), and the gradients
    on their own routes, against the oracle."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
    want_y = np.empty((N, Cout, Ho, Wo), np.float32)
    ob.oracle().oracle_conv2d_forward(*geo, x.reshape(-1), w.reshape(-1), want_y.reshape(-1), col)
    # one product over the pixels of the whole batch, stored image by image, where its tiles fill more of the chip than a
    # product per image does (the last two geometries here)
    route = "conv2d_im2col_gemm" if N >= 63 else "conv2d_im2col_batched_gemm"
    y, _, fk = gpu_conv(gpu, geo, x, w)
    assert fk == route, fk
    assert rel_err(y, want_y) < TOL
    bias = rng.standard_normal(Cout).astype(np.float32)
    yb, _, fk = gpu_conv(gpu, geo, x, w, None, bias)
    assert fk == route, fk
    assert rel_err(yb, want_y + bias[None, :, None, None]) < TOL
    if geo[0] == 1:
        dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
        gpu_dgrad(gpu, geo, w, dy)
        assert gpu.last_kernel() == "conv2d_im2col_batched_gemm", gpu.last_kernel()
    if geo[0] < 64:   # (the gradients of the largest layer would take the oracle a while)
        _conv_vs_oracle(gpu, ob, geo)


@pytest.mark.parametrize("geo", [(1, 512, 7, 7, 512, 3, 3, 1, 1, 1, 1),       # one image of 49 pixels: the product on the 32 x 32 tiles
                                 (2, 2048, 7, 7, 510, 1, 1, 0, 0, 1, 1),      # a 1 x 1 layer; 510 channels: dy's pixel-major rows padded to 512
                                 (16, 512, 7, 7, 256, 3, 3, 1, 1, 1, 1)])     # 784 pixels: the 64 x 64 direct-to-LDS tiles, K = 784 in two passes
def test_conv_weight_gradient_over_few_pixels_by_column_matrices(gpu, ob, geo):
    """Few output pixels in the whole batch and many channels: the columns and dy are copied with a row per pixel into memory
    of the library and the weight gradient is one plain TN product over the pixels; against the oracle."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = np.zeros((Cout, Cin, kh, kw), np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
    want_dw = np.empty_like(w)
    ob.oracle().oracle_conv2d_wgrad(*geo, x.reshape(-1), dy.reshape(-1), want_dw.reshape(-1), col)
    _, dw, _ = gpu_conv(gpu, geo, x, w, dy)
    assert gpu.last_kernel() == "conv2d_wgrad_columns_gemm", gpu.last_kernel()
    assert rel_err(dw, want_dw) < TOL


def test_conv_by_column_matrices_inside_a_recorded_launch_graph(gpu):
    """The column routes keep their matrices in memory of the library, which is only allocated outside a recording: a layer
    that ran once before is recorded with that route and replays to the same values (also after a larger eager call has made
    the library take a new block); forward, strided data gradient and few-pixel weight gradient."""
    D, l = gpu.DeviceBuffer, gpu.lib()
    rng = np.random.default_rng(11)
    fgeo = (16, 64, 16, 16, 128, 3, 3, 1, 1, 1, 1)      # forward by columns
    dgeo = (8, 32, 40, 48, 48, 3, 3, 1, 1, 2, 2)        # strided data gradient by columns
    wgeo = (2, 2048, 7, 7, 512, 1, 1, 0, 0, 1, 1)       # weight gradient over 98 pixels
    def operands(geo):
        N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
        Ho, Wo = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
        x = D.from_numpy(rng.standard_normal((N, Cin, H, W)).astype(np.float32))
        w = D.from_numpy((rng.standard_normal((Cout, Cin * kh * kw)) * 0.1).astype(np.float32))
        dy = D.from_numpy(rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32))
        return x, w, dy, N * Cout * Ho * Wo, N * Cin * H * W, Cout * Cin * kh * kw
    fx, fw, _, fny, _, _ = operands(fgeo)
    _, dw_, ddy, _, dnx, _ = operands(dgeo)
    wx, _, wdy, _, _, wnw = operands(wgeo)
    fb = D.from_numpy(rng.standard_normal(fgeo[4]).astype(np.float32))
    y, dx, dwt = D(4 * fny), D(4 * dnx), D(4 * wnw)
    dws = D(max(int(l.lten_hip_conv2d_dgrad_workspace_bytes(*dgeo)), 16))
    wws = D(max(int(l.lten_hip_conv2d_wgrad_workspace_bytes(*wgeo)), 16))
    names = []
    def step():
        gpu.check(l.lten_hip_conv2d_forward_f32(*fgeo, fx.ptr, fw.ptr, fb.ptr, y.ptr)); names.append(gpu.last_kernel())
        gpu.check(l.lten_hip_conv2d_dgrad_f32(*dgeo, dw_.ptr, ddy.ptr, dx.ptr, dws.ptr)); names.append(gpu.last_kernel())
        gpu.check(l.lten_hip_conv2d_wgrad_f32(*wgeo, wx.ptr, wdy.ptr, dwt.ptr, wws.ptr)); names.append(gpu.last_kernel())
    step()
    assert names == ["conv2d_im2col_batched_gemm", "conv2d_dgrad_batched_gemm_col2im", "conv2d_wgrad_columns_gemm"], names
    want = [y.numpy(np.float32, (fny,)).copy(), dx.numpy(np.float32, (dnx,)).copy(), dwt.numpy(np.float32, (wnw,)).copy()]
    del names[:]
    with gpu.Graph() as graph:
        step()
    assert names == ["conv2d_im2col_batched_gemm", "conv2d_dgrad_batched_gemm_col2im", "conv2d_wgrad_columns_gemm"], names
    for rep in range(3):
        for buf, n in ((y, fny), (dx, dnx), (dwt, wnw)):
            gpu.check(l.lten_hip_zero(buf.ptr, 4 * n))
        graph.launch()
        got = [y.numpy(np.float32, (fny,)), dx.numpy(np.float32, (dnx,)), dwt.numpy(np.float32, (wnw,))]
        for g_, w_ in zip(got, want):
            assert np.array_equal(g_, w_)
        if rep == 0:   # a larger layer, eagerly: the library needs a bigger block and must leave the recorded one alone
            big = (32, 128, 16, 16, 128, 3, 3, 1, 1, 1, 1)
            bx, bw, _, bny, _, _ = operands(big)
            by = D(4 * bny)
            gpu.check(l.lten_hip_conv2d_forward_f32(*big, bx.ptr, bw.ptr, None, by.ptr))
            assert gpu.last_kernel().startswith("conv2d_im2col_"), gpu.last_kernel()


def test_conv_data_gradient_of_a_strided_first_layer_with_a_large_window(gpu, ob):
    """Three input channels fill three of the 64 rows of the implicit GEMM's tiles; with a 7 x 7 window on a large image that
    padding costs more than l-ten's own decomposition (GEMM + col2im), which the library then takes: once for the batch,
    with the columns in memory of its own; image by image in the caller's workspace when that memory cannot be had."""
    geo = (2, 3, 128, 128, 64, 7, 7, 3, 3, 2, 2)
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
    want_dx = np.empty((N, Cin, H, W), np.float32)
    ob.oracle().oracle_conv2d_dgrad(*geo, w.reshape(-1), dy.reshape(-1), want_dx.reshape(-1), col)
    dx = gpu_dgrad(gpu, geo, w, dy)
    assert gpu.last_kernel() == "conv2d_dgrad_batched_gemm_col2im", gpu.last_kernel()
    assert rel_err(dx, want_dx) < TOL


@pytest.mark.parametrize("geo", [(256, 10, 12, 12, 20, 5, 5, 0, 0, 1, 1),     # l-ten's MNIST conv2 at batch 256: 10 input channels
                                 (32, 2, 64, 64, 24, 4, 4, 1, 1, 1, 1),       # a first layer with 2^18 input elements
                                 (64, 20, 8, 8, 50, 5, 5, 0, 0, 1, 1),        # 50 output channels (dy's rows as they lie), 64 tiles under K = 1250
                                 (64, 6, 14, 14, 16, 5, 5, 0, 0, 1, 1)])      # LeNet's second layer
def test_conv_data_gradient_of_few_channels_by_column_matrices(gpu, ob, geo):
    """Stride 1 with few input channels (or few tiles under a long reduction): as a convolution of dy the gradient would fill a
    fraction of its tiles, and the GEMM + col2im decomposition done once for the batch runs instead; against the oracle."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
    want_dx = np.empty((N, Cin, H, W), np.float32)
    ob.oracle().oracle_conv2d_dgrad(*geo, w.reshape(-1), dy.reshape(-1), want_dx.reshape(-1), col)
    dx = gpu_dgrad(gpu, geo, w, dy)
    assert gpu.last_kernel() == "conv2d_dgrad_batched_gemm_col2im", gpu.last_kernel()
    assert rel_err(dx, want_dx) < TOL


@pytest.mark.parametrize("geo,route", [((4, 256, 8, 8, 64, 5, 5, 2, 2, 2, 2), "conv2d_im2col"),           # 16 output pixels an image under K = 6400
                                       ((8, 128, 7, 7, 8, 7, 7, 3, 3, 2, 2), "conv2d_im2col")])            # 8 output channels under K = 6272
def test_conv_forward_of_tiny_outputs_under_a_long_reduction_by_column_matrices(gpu, ob, geo, route):
    """Few output channels or pixels under a reduction of 2048 or more: the implicit GEMM's handful of tiles would walk it one
    after another, the column matrices hand it to the GEMM entry (which splits it); forward with bias against the oracle."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
    want_y = np.empty((N, Cout, Ho, Wo), np.float32)
    ob.oracle().oracle_conv2d_forward(*geo, x.reshape(-1), w.reshape(-1), want_y.reshape(-1), col)
    want_y += bias[None, :, None, None]
    y, _, fk = gpu_conv(gpu, geo, x, w, None, bias)
    assert fk.startswith(route), fk
    assert rel_err(y, want_y) < TOL


@pytest.mark.parametrize("geo,route", [((16, 16, 64, 64, 16, 3, 3, 1, 1, 1, 1), "conv2d_patch"),     # 3 x 3 on wide rows: the patch kernels
                                       ((64, 8, 32, 32, 8, 3, 3, 1, 1, 1, 1), "conv2d_forward"),     # a short reduction: the implicit GEMM
                                       ((64, 16, 16, 16, 128, 3, 3, 1, 1, 1, 1), "conv2d_dgrad_batched_gemm_col2im"),    # a long one: the columns
                                       ((4, 3, 14, 14, 512, 7, 7, 3, 3, 1, 1), "conv2d_dgrad_batched_gemm_col2im")])     # a small input under many channels: 13 tiles would walk K = 25088
def test_conv_data_gradient_of_few_channels_takes_the_cheaper_route(gpu, ob, geo, route):
    """Few input channels at stride 1: an estimate decides between the column matrices and the convolution of dy with the
    flipped weights (which runs 3 x 3 windows on the patch kernels); whichever it picks, against the oracle."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
    want_dx = np.empty((N, Cin, H, W), np.float32)
    ob.oracle().oracle_conv2d_dgrad(*geo, w.reshape(-1), dy.reshape(-1), want_dx.reshape(-1), col)
    dx = gpu_dgrad(gpu, geo, w, dy)
    assert gpu.last_kernel().startswith(route), gpu.last_kernel()
    assert rel_err(dx, want_dx) < TOL


@pytest.mark.parametrize("geo", [(8, 32, 40, 48, 48, 3, 3, 1, 1, 2, 2),       # 3 x 3 at stride 2
                                 (4, 24, 34, 30, 36, 5, 4, 2, 1, 3, 2),       # strides 3 x 2, oblong window
                                 (3, 5, 40, 40, 32, 7, 7, 3, 3, 2, 2),        # K = 245: the weights' rows are padded to a multiple of four floats
                                 (8, 40, 32, 32, 64, 2, 2, 0, 0, 2, 2),       # windows that do not overlap
                                 (6, 32, 25, 29, 64, 3, 3, 1, 1, 2, 2),       # 13 x 15 = 195 output pixels: dy is copied into rows of 196 floats
                                 (32, 5, 29, 29, 36, 3, 3, 1, 1, 2, 2),       # K = 45 and 225 output pixels: both operands copied into padded rows
                                 (6, 256, 28, 29, 512, 1, 1, 0, 0, 2, 2)])    # 1 x 1 at stride 2 between wide layers (a residual network's shortcut): the columns are dy
def test_conv_strided_data_gradient_by_column_matrices(gpu, ob, geo):
    """With a stride and a megabyte or more of columns, l-ten's GEMM + col2im runs once for the batch: a strided batch of
    TN products into memory of the library, one col2im launch; against the oracle, and against the implicit GEMM."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    assert N * Cin * kh * kw * Ho * Wo >= 1 << 18
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
    want_dx = np.empty((N, Cin, H, W), np.float32)
    ob.oracle().oracle_conv2d_dgrad(*geo, w.reshape(-1), dy.reshape(-1), want_dx.reshape(-1), col)
    dx = gpu_dgrad(gpu, geo, w, dy)
    assert gpu.last_kernel() == "conv2d_dgrad_batched_gemm_col2im", gpu.last_kernel()
    assert rel_err(dx, want_dx) < TOL
    gpu.set_option("conv_variant", 1)
    try:
        dx1 = gpu_dgrad(gpu, geo, w, dy)
        assert gpu.last_kernel() != "conv2d_dgrad_batched_gemm_col2im"
    finally:
        gpu.set_option("conv_variant", 0)
    assert rel_err(dx, dx1) < TOL


@pytest.mark.parametrize("geo", [(3, 16, 20, 30, 64, 3, 3, 1, 1, 1, 1),      # 30 columns: rows start 8 bytes off 16-byte boundaries
                                 (2, 8, 17, 26, 33, 3, 3, 0, 0, 1, 1),      # MNIST after one unpadded 3x3: 26 columns, no padding
                                 (2, 12, 33, 50, 130, 3, 3, 1, 1, 1, 1),    # two column tiles, three tile rows, three channel blocks
                                 (5, 64, 15, 15, 64, 3, 3, 1, 1, 1, 1),     # odd width: every row starts at another offset
                                 (1, 8, 7, 95, 40, 3, 3, 2, 1, 1, 1)])      # three column tiles, the last 31 columns wide, row pad 2
def test_conv_narrow_images_with_unaligned_rows(gpu, ob, geo):
    """The 16 x 32 tiles with the patch fetched four bytes per lane: input widths that are no multiple of four, where
    rows do not start on 16-byte boundaries; forward, and the stride-1 data gradient through it, against the oracle."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    gpu.set_option("conv_variant", 6)   # these tiles however few workgroups the small test shapes give
    try:
        y, _, fk = gpu_conv(gpu, geo, x, w, dy, rng.standard_normal(Cout).astype(np.float32))
        assert fk.startswith("conv2d_patch_fast_forward_3x3_") and fk.endswith("x16x32_e4"), fk
        _conv_vs_oracle(gpu, ob, geo)
    finally:
        gpu.set_option("conv_variant", 0)


def _conv_vs_oracle(gpu, ob, geo):
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
    want_y = np.empty((N, Cout, Ho, Wo), np.float32)
    ob.oracle().oracle_conv2d_forward(*geo, x.reshape(-1), w.reshape(-1), want_y.reshape(-1), col)
    want_dw = np.empty_like(w)
    ob.oracle().oracle_conv2d_wgrad(*geo, x.reshape(-1), dy.reshape(-1), want_dw.reshape(-1), col)
    y, dw, fk = gpu_conv(gpu, geo, x, w, dy, bias)
    print(f"  {geo}: forward via {fk}, wgrad via {gpu.last_kernel()}", flush=True)
    assert rel_err(y, want_y + bias[None, :, None, None]) < TOL, fk
    assert rel_err(dw, want_dw) < TOL, gpu.last_kernel()
    want_dx = np.empty_like(x)
    ob.oracle().oracle_conv2d_dgrad(*geo, w.reshape(-1), dy.reshape(-1), want_dx.reshape(-1), col)
    dx = gpu_dgrad(gpu, geo, w, dy)
    print(f"  {geo}: dgrad via {gpu.last_kernel()}", flush=True)
    assert rel_err(dx, want_dx) < TOL, gpu.last_kernel()
    assert rel_err(y, direct_conv(x, w, ph, pw, sh, sw) + bias[None, :, None, None]) < TOL


def test_cfg5_full_size(gpu, wl):
    """32x1x128x128 -> 32 channels -> 64 channels, 3x3 s1 p1: forward of both layers and both weight gradients,
    checked in fp64 on sampled outputs (forward) and in full (weight gradients are only 288 / 18432 numbers)."""
    x, ws, dyshapes = wl.cfg5()
    rng = np.random.default_rng(0)
    inp = x
    for layer, w in enumerate(ws):
        N, Cin, H, W = inp.shape
        Cout = w.shape[0]
        geo = (N, Cin, H, W, Cout, 3, 3, 1, 1, 1, 1)
        dy = wl.cfg5_dy(dyshapes[layer], layer=layer)
        y, dw, fk = gpu_conv(gpu, geo, inp, w, dy)
        # forward: sampled output positions against a direct fp64 sum
        xp = np.pad(inp.astype(np.float64), ((0, 0), (0, 0), (1, 1), (1, 1)))
        idx = [(int(rng.integers(0, N)), int(rng.integers(0, Cout)), int(rng.integers(0, H)), int(rng.integers(0, W)))
               for _ in range(400)] + [(0, 0, 0, 0), (N - 1, Cout - 1, H - 1, W - 1), (1, 1, 0, W - 1), (2, 0, H - 1, 0)]
        want = np.array([(xp[n, :, h:h + 3, ww:ww + 3] * w[c].astype(np.float64)).sum() for (n, c, h, ww) in idx])
        got = np.array([y[i] for i in idx])
        scale = float(np.sqrt((y.astype(np.float64) ** 2).mean()))
        assert (np.abs(got - want) / np.maximum(np.abs(want), scale)).max() < TOL, fk
        # weight gradient in full: dw[c, ci, i, j] = sum_{n,h,w} dy[n,c,h,w] * xpad[n,ci,h+i,w+j]
        want_dw = np.empty(w.shape, np.float64)
        dy64 = dy.astype(np.float64)
        for i in range(3):
            for j in range(3):
                want_dw[:, :, i, j] = np.einsum("nchw,ndhw->cd", dy64, xp[:, :, i:i + H, j:j + W], optimize=True)
        assert rel_err(dw, want_dw) < TOL
        print(f"  layer {layer + 1}: forward via {fk}, wgrad via {gpu.last_kernel()}, "
              f"dw max rel err {rel_err(dw, want_dw):.2e}")
        # data gradient on sampled input positions: dx[n,ci,y,x] = sum_{c,i,j} dy[n,c,y+1-i,x+1-j] * w[c,ci,i,j]
        dx = gpu_dgrad(gpu, geo, w, dy)
        dyp = np.pad(dy64, ((0, 0), (0, 0), (1, 1), (1, 1)))
        wf = w.astype(np.float64)[:, :, ::-1, ::-1]
        pts = [(int(rng.integers(0, N)), int(rng.integers(0, Cin)), int(rng.integers(0, H)), int(rng.integers(0, W)))
               for _ in range(200)] + [(0, 0, 0, 0), (N - 1, Cin - 1, H - 1, W - 1)]
        want_dx = np.array([(dyp[n, :, yy:yy + 3, xx:xx + 3] * wf[:, ci]).sum() for (n, ci, yy, xx) in pts])
        got_dx = np.array([dx[p] for p in pts])
        sc = float(np.sqrt((dx.astype(np.float64) ** 2).mean()))
        assert (np.abs(got_dx - want_dx) / np.maximum(np.abs(want_dx), sc)).max() < TOL, gpu.last_kernel()
        inp = y


def test_seeded_sweep_over_geometries(gpu, ob):
    """Forty seeded geometries (channel counts on both sides of the kernels' limits, 1x1 / 3x3 / 5x5 / oblong windows,
    stride 1 and 2, pad 0..2, widths that are and are not multiples of four): forward, weight gradient and data gradient
    against the oracle, with whatever kernel the library picks."""
    rng = np.random.default_rng(31415)
    seen = set()
    for case in range(40):
        Cin = int(rng.choice([1, 2, 3, 4, 8, 12, 16, 20, 33]))
        Cout = int(rng.choice([1, 7, 16, 32, 40, 64, 70]))
        kh, kw = [(1, 1), (3, 3), (3, 3), (3, 3), (5, 5), (2, 3), (3, 1)][int(rng.integers(0, 7))]
        sh = sw = int(rng.choice([1, 1, 1, 2]))
        ph, pw = int(rng.integers(0, min(kh, 3))), int(rng.integers(0, min(kw, 3)))
        H, W = int(rng.integers(kh + 1, 24)), int(rng.choice([8, 12, 17, 20, 36, 132, 140]))
        N = int(rng.integers(1, 4))
        geo = (N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw)
        _conv_vs_oracle(gpu, ob, geo)
        seen.add(gpu.last_kernel())
    print(sorted(seen))


@pytest.mark.parametrize("geo", [(2, 16, 6, 128, 64, 3, 3, 1, 1, 1, 1), (1, 12, 5, 64, 40, 3, 3, 1, 1, 1, 1)])
def test_conv_operands_aligned_to_four_bytes_only(gpu, ob, geo):
    """x, w, dy and y that start 4 bytes into their allocations (views into larger tensors, as l-ten's per-image
    offsets produce): the kernels that need 16-byte aligned operands must step aside, the results stay the same."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo) + 1)
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * 0.2).astype(np.float32)
    dy = rng.standard_normal((N, Cout, H, W)).astype(np.float32)
    col = np.empty(Cin * kh * kw * H * W, np.float32)
    want_y, want_dw, want_dx = np.empty_like(dy), np.empty_like(w), np.empty_like(x)
    ob.oracle().oracle_conv2d_forward(*geo, x.reshape(-1), w.reshape(-1), want_y.reshape(-1), col)
    ob.oracle().oracle_conv2d_wgrad(*geo, x.reshape(-1), dy.reshape(-1), want_dw.reshape(-1), col)
    ob.oracle().oracle_conv2d_dgrad(*geo, w.reshape(-1), dy.reshape(-1), want_dx.reshape(-1), col)
    D, l = gpu.DeviceBuffer, gpu.lib()
    dX, dW, dDY = D(x.nbytes + 16), D(w.nbytes + 16), D(dy.nbytes + 16)
    dX.upload(x, offset=4); dW.upload(w, offset=4); dDY.upload(dy, offset=4)
    dY, dDW, dDX = D(dy.nbytes + 16), D(w.nbytes + 16), D(x.nbytes + 16)
    gpu.check(l.lten_hip_conv2d_forward_f32(*geo, dX.ptr + 4, dW.ptr + 4, None, dY.ptr + 4))
    fk = gpu.last_kernel()
    ws = D(max(int(l.lten_hip_conv2d_wgrad_workspace_bytes(*geo)), int(l.lten_hip_conv2d_dgrad_workspace_bytes(*geo)), 4))
    gpu.check(l.lten_hip_conv2d_wgrad_f32(*geo, dX.ptr + 4, dDY.ptr + 4, dDW.ptr + 4, ws.ptr))
    wk = gpu.last_kernel()
    gpu.check(l.lten_hip_conv2d_dgrad_f32(*geo, dW.ptr + 4, dDY.ptr + 4, dDX.ptr + 4, ws.ptr))
    print(f"  {geo}: forward via {fk}, wgrad via {wk}, dgrad via {gpu.last_kernel()}", flush=True)
    assert "fast" not in fk and "fast" not in wk
    got = lambda buf, shape: buf.numpy(np.uint8, (buf.nbytes,))[4:4 + 4 * int(np.prod(shape))].view(np.float32).reshape(shape)
    assert rel_err(got(dY, dy.shape), want_y) < TOL, fk
    assert rel_err(got(dDW, w.shape), want_dw) < TOL, wk
    assert rel_err(got(dDX, x.shape), want_dx) < TOL, gpu.last_kernel()


def test_seeded_sweep_over_chunked_rows(gpu, ob):
    """Sixteen seeded 3x3, stride 1, pad 1 geometries whose rows are whole 64-pixel chunks (the shapes the
    direct-to-LDS weight-gradient kernel takes), channel counts on both sides of its 64 x 32 blocks, images of one row
    up to 40 (a workgroup's run of chunks then starts anywhere in a 64-column strip and crosses strips and images)."""
    rng = np.random.default_rng(2718)
    seen = set()
    for case in range(16):
        Cin = int(rng.choice([9, 16, 31, 32, 33, 48, 64, 70]))
        Cout = int(rng.choice([1, 16, 63, 64, 65, 100, 128]))
        H, W = int(rng.choice([1, 2, 3, 5, 8, 17, 40])), int(rng.choice([64, 64, 128, 192]))
        N = int(rng.integers(1, 4))
        _conv_vs_oracle(gpu, ob, (N, Cin, H, W, Cout, 3, 3, 1, 1, 1, 1))
        seen.add(gpu.last_kernel())
    print(sorted(seen))


@pytest.mark.parametrize("shape", [(1, 1, 1), (2, 5, 7), (3, 70, 33 * 29), (32, 64, 128 * 128), (4, 4096, 6), (5, 3, 1000)])
def test_conv_bias_gradient(gpu, shape):
    """db[c] = sum over n, h, w of dy: integer-valued data make the sum exact in any order; then random data against
    an fp64 sum, overwrite and accumulate."""
    N, C, HW = shape
    rng = np.random.default_rng(N + C + HW)
    dy = rng.integers(-3, 4, (N, C, HW)).astype(np.float32)
    db0 = rng.integers(-20, 20, C).astype(np.float32)
    D, l = gpu.DeviceBuffer, gpu.lib()
    dDY, dDB = D.from_numpy(dy), D.from_numpy(db0)
    gpu.check(l.lten_hip_conv2d_bias_grad_f32(N, C, HW, dDY.ptr, dDB.ptr, 1))
    assert np.array_equal(dDB.numpy(np.float32, (C,)), db0 + dy.sum(axis=(0, 2)))
    gpu.check(l.lten_hip_conv2d_bias_grad_f32(N, C, HW, dDY.ptr, dDB.ptr, 0))
    assert np.array_equal(dDB.numpy(np.float32, (C,)), dy.sum(axis=(0, 2)))
    r = rng.standard_normal((N, C, HW)).astype(np.float32)
    dR = D.from_numpy(r)
    gpu.check(l.lten_hip_conv2d_bias_grad_f32(N, C, HW, dR.ptr, dDB.ptr, 0))
    assert rel_err(dDB.numpy(np.float32, (C,)), r.astype(np.float64).sum(axis=(0, 2))) < TOL
    assert l.lten_hip_conv2d_bias_grad_f32(1, 5000, 4, dR.ptr, dDB.ptr, 0) != 0   # more channels than the library's partial array
