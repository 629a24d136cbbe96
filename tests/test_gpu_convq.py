"""GPU parity tests of the Conv2d_q forward (C ABI): int32 accumulators and requantized uint8 outputs bit-exact against
the oracle, the golden outputs of l-ten's compiled Conv2d_q layer, and the int64 closed form."""
import numpy as np
import pytest

from conftest import golden_path
from test_oracle_conv import conv2dq_closed_form

pytestmark = pytest.mark.gpu


def test_conv2dq_golden_from_compiled_layer(gpu):
    g = np.load(golden_path("conv2dq_cases.npz"))
    for variant in (0, 1):   # 0: the library's choice (one launch up to 64 taps); 1: im2col + GEMM per image
        gpu.set_option("conv_variant", variant)
        try:
            for i in range(int(g["count"])):
                pre = f"q{i}_"
                geo = tuple(int(v) for v in g[pre + "geo"])
                y, acc = gpu.conv2dq_host(geo, g[pre + "x"], g[pre + "w"], g[pre + "scales"], g[pre + "zps"], want_acc=True)
                assert np.array_equal(y, g[pre + "y"]), (variant, i, gpu.last_kernel())
                want = conv2dq_closed_form(geo, g[pre + "x"], g[pre + "w"], int(g[pre + "zps"][0]), int(g[pre + "zps"][1]))
                assert np.array_equal(acc, want), (variant, i)
        finally:
            gpu.set_option("conv_variant", 0)


@pytest.mark.parametrize("geo", [(64, 1, 28, 28, 10, 5, 5, 0, 0, 1, 1),      # l-ten's quantized MNIST conv1 at batch 64
                                 (3, 7, 13, 17, 70, 3, 3, 1, 1, 1, 1),       # 63 taps, two channel blocks
                                 (2, 16, 20, 22, 24, 3, 3, 1, 1, 2, 1),      # 144 taps: patch rows + GEMM + finish
                                 (5, 10, 12, 12, 20, 5, 5, 0, 0, 1, 1),      # l-ten's quantized MNIST conv2: 250 taps (padded to 256)
                                 (3, 8, 9, 7, 10, 3, 3, 1, 1, 1, 1),         # 72 taps, 63 positions an image
                                 (3, 15, 9, 7, 10, 3, 3, 1, 1, 1, 1),        # 135 taps, 10 channels (padded to 12), 63 positions an image
                                 (2, 64, 6, 10, 70, 3, 3, 1, 1, 1, 1),       # 576 taps, two channel blocks of the finish pass
                                 (4, 128, 5, 5, 33, 1, 1, 0, 0, 1, 1),       # 1x1 with 128 channels
                                 (2, 6, 14, 14, 16, 5, 5, 2, 2, 1, 1),       # 150 taps, padding 2
                                 (1, 20, 17, 9, 6, 3, 5, 0, 2, 2, 2),        # 300 taps, strides, oblong window
                                 (1, 3, 33, 300, 5, 7, 3, 3, 0, 2, 3),       # 63 taps, strides, ragged
                                 (2, 32, 9, 9, 40, 1, 1, 0, 0, 1, 1),        # 1x1
                                 (2, 5, 11, 13, 9, 3, 3, 1, 0, 1, 2),        # 45 taps: twelve packed dwords
                                 (1, 4, 8, 8, 3, 2, 2, 1, 1, 1, 1),          # 16 taps: four dwords, all full
                                 (2, 11, 7, 9, 5, 1, 3, 0, 1, 1, 1),         # 33 taps: one tap in the ninth dword
                                 (1, 3, 12, 10, 7, 4, 4, 1, 2, 1, 1),        # 48 taps
                                 (64, 10, 12, 12, 20, 5, 5, 0, 0, 1, 1),     # l-ten's quantized MNIST conv2 at batch 64
                                 (3, 9, 15, 11, 64, 3, 3, 1, 1, 1, 1),       # 81 taps, four blocks of 16 channels, 165 positions
                                 (2, 16, 28, 32, 17, 3, 3, 2, 2, 1, 1),      # 144 taps, 1020 positions an image: 64 workgroups each
                                 (2, 40, 5, 5, 30, 5, 5, 2, 2, 1, 1),        # 1000 taps, most of them outside the image
                                 (2, 40, 5, 5, 50, 5, 5, 2, 2, 1, 1),        # the same with 50 channels: weights beyond the 64 KB of LDS the route allows
                                 (1, 33, 31, 31, 3, 2, 2, 0, 0, 3, 3),       # 132 taps, image of 31.7 KB, stride 3
                                 (1, 65, 9, 9, 70, 1, 1, 0, 0, 1, 1),        # 65 taps but 70 channels: not for the one-launch route
                                 (2, 16, 40, 40, 24, 3, 3, 1, 1, 1, 1),      # 1600 positions an image: bands of output rows
                                 (1, 8, 50, 70, 64, 5, 3, 2, 1, 2, 1),       # bands with a row stride of 2, 64 channels, 120 taps
                                 (1, 3, 100, 37, 9, 5, 5, 0, 0, 1, 1),       # rows of 37 bytes: the region is filled byte by byte
                                 (3, 12, 33, 41, 20, 3, 3, 0, 2, 1, 3),      # column stride 3, padding 2 on the columns only
                                 (1, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1),      # 576 taps, 64 channels: several passes of blocks per band
                                 (3, 8, 44, 36, 16, 5, 5, 2, 2, 1, 1),       # bands, 5 x 5 windows of 8 channels (weights permuted in registers, 25 taps)
                                 (2, 4, 67, 70, 12, 7, 7, 3, 3, 2, 2),       # bands, 7 x 7 windows of 4 channels, stride 2 (49 taps)
                                 (19, 12, 36, 36, 40, 3, 3, 1, 1, 1, 1),     # 19 images x 9 bands = 171 workgroups: not a multiple of the 8 XCDs
                                 (2, 16, 20, 24, 80, 3, 3, 1, 1, 1, 1),      # 80 channels: a block of 64 and one of 16 per band
                                 (1, 128, 14, 14, 136, 3, 3, 1, 1, 1, 1),    # 1152 taps: weights of 32 channels at a time fit LDS, 5 blocks
                                 (1, 400, 9, 9, 40, 3, 3, 0, 0, 1, 1),       # 3600 taps: the weights of 32 channels do not fit, three launches
                                 (1, 200, 9, 9, 30, 3, 3, 0, 0, 1, 1),       # 1800 taps, 30 channels: two blocks of 16 channels
                                 (3, 96, 20, 20, 72, 1, 1, 0, 0, 1, 1),      # a 1 x 1 layer of 96 channels: the weights are copied as they lie
                                 (2, 68, 21, 22, 40, 1, 1, 1, 0, 2, 1),      # 1 x 1 with a row stride of 2 and padded rows
                                 (8, 16, 20, 24, 64, 2, 2, 0, 0, 2, 2),      # 64 taps, 64 channels: short windows on the band kernel
                                 (2, 3, 40, 44, 64, 3, 3, 1, 1, 1, 1),       # 27 taps of 3 channels (padded to 4), one k-step
                                 (2, 64, 12, 12, 80, 1, 1, 0, 0, 1, 1),      # 1 x 1 with 64 channels in, 80 out
                                 (3, 5, 17, 19, 50, 3, 3, 2, 2, 1, 2)])      # 45 taps, 50 channels, ragged everything
def test_conv2dq_vs_oracle(gpu, ob, geo):
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.integers(0, 256, (N, Cin, H, W), dtype=np.uint8)
    w = rng.integers(0, 256, (Cout, Cin, kh, kw), dtype=np.uint8)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    K = Cin * kh * kw
    for sc, zp, with_bias in (([1 / 255, 0.01, 0.05], [0, 128, 128], False), ([0.02, 0.013, 0.9], [17, 250, 100], True),
                              ([0.5, 0.5, 0.2], [128, 128, 0], False)):
        bias = rng.integers(-9999, 9999, Ho * Wo).astype(np.int32) if with_bias else None
        want_y, want_acc = ob.conv2dq_forward(geo, x, w, sc, zp, bias=bias)
        y, acc = gpu.conv2dq_host(geo, x, w, sc, zp, bias=bias, want_acc=True)
        kern = gpu.last_kernel()
        # up to 64 taps: one launch from registers; longer windows on small images: one launch from the image in LDS;
        # else patch rows + GEMM + finish
        Kp, ncb = (K + 63) // 64 * 64, (Cout + 15) // 16
        lds = (Cin * H * W + 15) // 16 * 16 + ncb * 16 * (Kp + 16) + 4 * Kp
        small = (Cin * H * W <= 32768 and Cout <= 64 and K <= 1024 and Ho * Wo <= 1024 and lds <= 65536 and
                 N * ((Ho * Wo + 15) // 16) <= 4096)
        # larger images with at most 64 channels: a band of output rows per workgroup, as long as one row's region fits LDS
        PL = (pw + 3) // 4 * 4
        RW = (PL + max((Wo - 1) * sw + kw - pw, W) + 3) // 4 * 4
        CP = 4 if Cin <= 4 else 8 if Cin <= 8 else 16
        CPtot = (Cin + CP - 1) // CP * CP
        PP = CPtot + (16 if CPtot % 32 == 0 else 0)
        Kb = (kh * kw * CPtot + 63) // 64 * 64      # the band kernel reduces over (tap, channel padded to a multiple of CP)
        # (blocks of 64 output channels per workgroup, or 32 where the weights of 64 leave no room for one window's rows; 16
        # only for layers of at most 32 channels)
        band = (pw <= 64 and kh * kw * CPtot <= 4096 and
                kh * RW * PP + (1 if ncb <= 2 else 2) * 16 * (Kb + 16) + 4 * (Kb // CP) + 2 * K + 32 <= 65536)
        # (where the band kernel applies, the small-image kernel only while its workgroups stage at most 16 MB in all and
        # the window is none of those whose weights the band kernel permutes in registers)
        staged = N * ((Ho * Wo + 15) // 16) * ((Cin * H * W + 15) // 16 * 16 + ncb * 16 * Kp)
        permuted = Cin % 4 == 0 and kh * kw in (1, 9, 25, 49)
        small = small and not (band and (permuted or staged > 16 << 20))
        # (windows of at most 64 taps: the band kernel from 48 output channels on, else one launch from registers)
        assert kern == (("conv2dq_band" if Cout >= 48 and band else "conv2dq_direct") if K <= 64 else
                        "conv2dq_image" if small else "conv2dq_band" if band else "conv2dq_rows_gemm_finish"), kern
        assert np.array_equal(acc, want_acc), kern
        assert np.array_equal(y, want_y), kern
        if kern in ("conv2dq_image", "conv2dq_band"):   # the three-launch route on the same shape gives the same bytes
            gpu.set_option("conv_variant", 2)
            try:
                y2, acc2 = gpu.conv2dq_host(geo, x, w, sc, zp, bias=bias, want_acc=True)
                assert gpu.last_kernel() == ("conv2dq_direct" if K <= 64 else "conv2dq_rows_gemm_finish")
            finally:
                gpu.set_option("conv_variant", 0)
            assert np.array_equal(acc2, want_acc) and np.array_equal(y2, want_y)
        if kern == "conv2dq_image" and band:   # and so does the band kernel where both one-launch kernels apply
            gpu.set_option("conv_variant", 3)
            try:
                y3, acc3 = gpu.conv2dq_host(geo, x, w, sc, zp, bias=bias, want_acc=True)
                assert gpu.last_kernel() == "conv2dq_band"
            finally:
                gpu.set_option("conv_variant", 0)
            assert np.array_equal(acc3, want_acc) and np.array_equal(y3, want_y)
    if K > 64:   # l-ten's decomposition image by image (what a workspace beyond 2 GiB falls back to) gives the same bytes
        gpu.set_option("conv_variant", 1)
        try:
            y1, acc1 = gpu.conv2dq_host(geo, x, w, sc, zp, bias=bias, want_acc=True)
            assert gpu.last_kernel() != "conv2dq_rows_gemm_finish"
        finally:
            gpu.set_option("conv_variant", 0)
        assert np.array_equal(acc1, want_acc) and np.array_equal(y1, want_y)


def test_conv2dq_long_windows_on_small_maps_take_the_three_launches(gpu, ob):
    """A 1 x 1 layer of 1024 channels on 14 x 14 maps: the band kernel has a plan (one output row and 32 channels per
    workgroup), but its workgroups would stage more than they compute, and the library's estimate sends the layer to patch
    rows + GEMM + finish.  Both routes give the oracle's bytes."""
    geo = (16, 1024, 14, 14, 256, 1, 1, 0, 0, 1, 1)
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.integers(0, 256, (N, Cin, H, W), dtype=np.uint8)
    w = rng.integers(0, 256, (Cout, Cin, kh, kw), dtype=np.uint8)
    sc, zp = [0.02, 0.013, 0.9], [17, 250, 100]
    want_y, want_acc = ob.conv2dq_forward(geo, x, w, sc, zp)
    y, acc = gpu.conv2dq_host(geo, x, w, sc, zp, want_acc=True)
    assert gpu.last_kernel() == "conv2dq_rows_gemm_finish", gpu.last_kernel()
    assert np.array_equal(acc, want_acc) and np.array_equal(y, want_y)
    gpu.set_option("conv_variant", 3)   # the band kernel whatever the estimate says
    try:
        y3, acc3 = gpu.conv2dq_host(geo, x, w, sc, zp, want_acc=True)
        assert gpu.last_kernel() == "conv2dq_band", gpu.last_kernel()
    finally:
        gpu.set_option("conv_variant", 0)
    assert np.array_equal(acc3, want_acc) and np.array_equal(y3, want_y)
