"""CPU tests that pin the im2col / conv oracle: the compiled l-ten templates where present,
golden outputs of l-ten's Conv2d layer (forward, weight gradient, data gradient), a direct
seven-loop convolution, the im2col/col2im adjoint identity and finite differences."""
import numpy as np
import pytest

from conftest import golden_path

GEOS = [  # C, H, W, kh, kw, ph, pw, sh, sw
    (1, 5, 5, 3, 3, 1, 1, 1, 1), (3, 7, 9, 3, 2, 0, 1, 2, 1), (2, 8, 6, 5, 5, 2, 2, 1, 1),
    (4, 6, 6, 1, 1, 0, 0, 1, 1), (2, 9, 11, 3, 3, 1, 0, 2, 3), (1, 4, 4, 4, 4, 0, 0, 1, 1),
]


def direct_conv(x, w, ph, pw, sh, sw):
    """out[n,co,ho,wo] = sum_{ci,i,j} w[co,ci,i,j] * xpad[n,ci,ho*sh+i,wo*sw+j], in fp64."""
    N, Cin, H, W = x.shape
    Cout, _, kh, kw = w.shape
    Ho, Wo = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    xp = np.zeros((N, Cin, H + 2 * ph, W + 2 * pw), np.float64)
    xp[:, :, ph:ph + H, pw:pw + W] = x
    out = np.zeros((N, Cout, Ho, Wo), np.float64)
    for i in range(kh):
        for j in range(kw):
            patch = xp[:, :, i:i + (Ho - 1) * sh + 1:sh, j:j + (Wo - 1) * sw + 1:sw]
            out += np.einsum("ncxy,oc->noxy", patch, w[:, :, i, j].astype(np.float64))
    return out


@pytest.mark.parametrize("geo", GEOS)
def test_im2col_closed_form_and_reference(ob, geo):
    C, H, W, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    im = rng.standard_normal((C, H, W)).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    col = np.empty((C * kh * kw, Ho * Wo), np.float32)
    ob.oracle().oracle_im2col_f32(im.reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, col.reshape(-1))
    # closed form: col[(c*kh+i)*kw+j, h*Wo+w] = im[c, h*sh-ph+i, w*sw-pw+j] or 0
    for r in range(C * kh * kw):
        c, i, j = r // (kh * kw), (r // kw) % kh, r % kw
        for h in range(Ho):
            for w in range(Wo):
                y, x = h * sh - ph + i, w * sw - pw + j
                want = im[c, y, x] if 0 <= y < H and 0 <= x < W else 0.0
                assert col[r, h * Wo + w] == want
    if ob.ref() is not None:
        col2 = np.empty_like(col)
        ob.ref().ref_im2col_f32(im.reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, col2.reshape(-1))
        assert np.array_equal(col, col2)
        back = np.zeros_like(im)
        back2 = np.zeros_like(im)
        ob.oracle().oracle_col2im_f32(col.reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, back.reshape(-1))
        ob.ref().ref_col2im_f32(col.reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, back2.reshape(-1))
        assert np.array_equal(back, back2)
    imu = rng.integers(0, 256, (C, H, W), dtype=np.uint8)
    colu = np.empty((C * kh * kw, Ho * Wo), np.uint8)
    ob.oracle().oracle_im2col_u8(imu.reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, colu.reshape(-1))
    colf = np.empty_like(col)
    ob.oracle().oracle_im2col_f32(imu.astype(np.float32).reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, colf.reshape(-1))
    assert np.array_equal(colu.astype(np.float32), colf)


@pytest.mark.parametrize("geo", GEOS)
def test_col2im_is_adjoint_of_im2col(ob, geo):
    C, H, W, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(1 + sum(geo))
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    x = rng.integers(-4, 5, (C, H, W)).astype(np.float32)   # integer valued: both inner products exact
    c = rng.integers(-4, 5, (C * kh * kw, Ho * Wo)).astype(np.float32)
    col = np.empty_like(c)
    ob.oracle().oracle_im2col_f32(x.reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, col.reshape(-1))
    im = np.zeros_like(x)
    ob.oracle().oracle_col2im_f32(c.reshape(-1), C, H, W, kh, kw, ph, pw, sh, sw, im.reshape(-1))
    assert float((col * c).sum()) == float((x * im).sum())


def test_conv_layer_golden(ob):
    g = np.load(golden_path("layer_cases.npz"))
    for i in range(int(g["conv_count"])):
        pre = f"cv{i}_"
        N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = (int(v) for v in g[pre + "geo"])
        Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
        col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
        y = np.empty(N * Cout * Ho * Wo, np.float32)
        args = (N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw)
        ob.oracle().oracle_conv2d_forward(*args, g[pre + "x"], g[pre + "w"], y, col)
        assert np.array_equal(y, g[pre + "y"]), i   # scalar loops on both sides: bit-exact
        dw = np.empty(Cout * Cin * kh * kw, np.float32)
        ob.oracle().oracle_conv2d_wgrad(*args, g[pre + "x"], g[pre + "dy"], dw, col)
        assert np.array_equal(dw, g[pre + "dw"]), i
        dx = np.empty(N * Cin * H * W, np.float32)
        ob.oracle().oracle_conv2d_dgrad(*args, g[pre + "w"], g[pre + "dy"], dx, col)
        assert np.array_equal(dx, g[pre + "dx"]), i


@pytest.mark.parametrize("geo", [(2, 3, 9, 8, 4, 3, 3, 1, 1, 1, 1), (1, 2, 10, 7, 3, 3, 2, 0, 1, 2, 1),
                                 (2, 4, 6, 6, 5, 5, 5, 2, 2, 1, 1)])
def test_conv_forward_and_wgrad_vs_direct(ob, geo):
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    rng = np.random.default_rng(sum(geo))
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = rng.standard_normal((Cout, Cin, kh, kw)).astype(np.float32)
    Ho, Wo = ob.conv_out_hw(H, W, kh, kw, ph, pw, sh, sw)
    col = np.empty(Cin * kh * kw * Ho * Wo, np.float32)
    y = np.empty((N, Cout, Ho, Wo), np.float32)
    ob.oracle().oracle_conv2d_forward(*geo, x.reshape(-1), w.reshape(-1), y.reshape(-1), col)
    want = direct_conv(x, w, ph, pw, sh, sw)
    assert np.abs(y - want).max() < 1e-4 * max(1.0, np.abs(want).max())
    # weight gradient: d/dw <dy, conv(x, w)> is linear in w, so finite differences are exact up to rounding
    dy = rng.standard_normal((N, Cout, Ho, Wo)).astype(np.float32)
    dw = np.empty((Cout, Cin, kh, kw), np.float32)
    ob.oracle().oracle_conv2d_wgrad(*geo, x.reshape(-1), dy.reshape(-1), dw.reshape(-1), col)
    for _ in range(6):
        idx = tuple(int(rng.integers(0, s)) for s in w.shape)
        e = np.zeros_like(w)
        e[idx] = 1.0
        want_g = float((dy.astype(np.float64) * direct_conv(x, e, ph, pw, sh, sw)).sum())
        assert abs(dw[idx] - want_g) < 1e-3 * max(1.0, abs(want_g))
    # data gradient likewise, linear in x
    dx = np.empty_like(x)
    ob.oracle().oracle_conv2d_dgrad(*geo, w.reshape(-1), dy.reshape(-1), dx.reshape(-1), col)
    for _ in range(6):
        idx = tuple(int(rng.integers(0, s)) for s in x.shape)
        e = np.zeros_like(x)
        e[idx] = 1.0
        want_g = float((dy.astype(np.float64) * direct_conv(e, w, ph, pw, sh, sw)).sum())
        assert abs(dx[idx] - want_g) < 1e-3 * max(1.0, abs(want_g))


# ----------------------------------------------------------------------------------------- Conv2d_q

def conv2dq_closed_form(geo, x, w, zp_in, zp_w):
    """sum over the window of (w - zpW) * (x_or_0 - zpIn) in int64: positions outside the image hold the byte 0
    (l-ten/im_col.h:24-27 pads the column buffer with T(0), not with the zero point)."""
    N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw = geo
    Ho, Wo = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    xp = np.pad(x.astype(np.int64), ((0, 0), (0, 0), (ph, ph), (pw, pw))) - zp_in
    wz = w.astype(np.int64) - zp_w
    acc = np.zeros((N, Cout, Ho, Wo), np.int64)
    for i in range(kh):
        for j in range(kw):
            win = xp[:, :, i:i + (Ho - 1) * sh + 1:sh, j:j + (Wo - 1) * sw + 1:sw]
            acc += np.einsum("nchw,oc->nohw", win, wz[:, :, i, j])
    return acc


def test_conv2dq_golden_from_compiled_layer(ob):
    g = np.load(golden_path("conv2dq_cases.npz"))
    for i in range(int(g["count"])):
        pre = f"q{i}_"
        geo = tuple(int(v) for v in g[pre + "geo"])
        y, acc = ob.conv2dq_forward(geo, g[pre + "x"], g[pre + "w"], g[pre + "scales"], g[pre + "zps"])
        assert np.array_equal(y, g[pre + "y"]), i
        want = conv2dq_closed_form(geo, g[pre + "x"], g[pre + "w"], int(g[pre + "zps"][0]), int(g[pre + "zps"][1]))
        assert np.array_equal(acc, want), i


def test_conv2dq_bias_is_per_output_position_and_invariants(ob):
    geo = (2, 2, 7, 6, 3, 3, 3, 1, 1, 1, 1)
    rng = np.random.default_rng(5)
    x = rng.integers(0, 256, (2, 2, 7, 6), dtype=np.uint8)
    w = rng.integers(0, 256, (3, 2, 3, 3), dtype=np.uint8)
    bias = rng.integers(-5000, 5000, 42).astype(np.int32)
    _, acc0 = ob.conv2dq_forward(geo, x, w, [0.02, 0.02, 1.0], [9, 200, 3])
    _, acc1 = ob.conv2dq_forward(geo, x, w, [0.02, 0.02, 1.0], [9, 200, 3], bias=bias)
    assert np.array_equal(acc1 - acc0, np.broadcast_to(bias.reshape(1, 1, 7, 6), acc0.shape))
    # weights equal to their zero point: every accumulator is 0, the output is the output zero point
    wz = np.full_like(w, 200)
    y, acc = ob.conv2dq_forward(geo, x, wz, [0.02, 0.02, 1.0], [9, 200, 3])
    assert not acc.any() and (y == 3).all()
