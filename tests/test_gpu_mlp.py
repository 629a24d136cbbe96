"""GPU parity tests of the element-wise / loss kernels and of a whole MLP training step on the device (C ABI):
FullyConnected(+bias) -> relu -> FullyConnected -> relu -> FullyConnected -> log_softmax -> nll_loss, then backward.
fp32: max relative error 1e-4 (conftest.rel_err); relu and its backward are selections and must match exactly."""
import numpy as np
import pytest

from conftest import golden_path, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4


def gpu_mlp_step(gpu, X, Ws, bs, T, fused=False):
    """The step through the C ABI, every intermediate resident on the device.  Returns what ob.mlp_step returns.
    fused: the entry points that fold relu, relu_backward, the loss and nll_backward into their neighbours; "head": the
    loss and its gradient as one call; "tail": the loss, its gradient and the last layer's backward as one call."""
    if fused:
        return gpu_mlp_step_fused(gpu, X, Ws, bs, T, head=fused if fused in ("head", "tail") else False)
    D, l = gpu.DeviceBuffer, gpu.lib()
    B, layers = X.shape[0], len(Ws)
    sizes = [X.shape[1]] + [w.shape[0] for w in Ws]
    dW_, db_ = [D.from_numpy(w) for w in Ws], [D.from_numpy(b) for b in bs]
    pre = [None] + [D(4 * B * n) for n in sizes[1:]]
    act = [D.from_numpy(X)] + [D(4 * B * n) for n in sizes[1:-1]] + [None]
    act[layers] = pre[layers]
    for i in range(layers):
        gpu.check(l.lten_hip_fc_forward_f32(B, sizes[i], sizes[i + 1], act[i].ptr, dW_[i].ptr, db_[i].ptr, pre[i + 1].ptr))
        if i + 1 < layers:
            gpu.check(l.lten_hip_relu_f32(act[i + 1].ptr, pre[i + 1].ptr, B * sizes[i + 1]))
    dT, logp, loss = D.from_numpy(T), D(4 * B * sizes[-1]), D(4)
    gpu.check(l.lten_hip_log_softmax_f32(B, sizes[-1], pre[layers].ptr, logp.ptr))
    gpu.check(l.lten_hip_nll_loss_f32(logp.ptr, dT.ptr, loss.ptr, B * sizes[-1], B))
    # backward from the loss: nll_backward (top = 1), log_softmax backward, then the layers
    g = [D(4 * B * n) for n in sizes]
    gl = D(4 * B * sizes[-1])
    gpu.check(l.lten_hip_scale_f32(B * sizes[-1], -1.0 / B, dT.ptr, gl.ptr))
    gpu.check(l.lten_hip_log_softmax_backward_f32(B, sizes[-1], logp.ptr, gl.ptr, g[layers].ptr))
    gW, gb = [D(w.nbytes) for w in Ws], [D(b.nbytes, zero=True) for b in bs]
    tmp = [D(4 * B * n) for n in sizes]
    for i in range(layers - 1, -1, -1):
        gpu.check(l.lten_hip_fc_backward_f32(B, sizes[i], sizes[i + 1], act[i].ptr, dW_[i].ptr, g[i + 1].ptr, tmp[i].ptr, gW[i].ptr, gb[i].ptr))
        if i > 0:
            gpu.check(l.lten_hip_relu_backward_f32(g[i].ptr, tmp[i].ptr, pre[i].ptr, B * sizes[i]))
    return dict(loss=float(loss.numpy(np.float32, (1,))[0]), logp=logp.numpy(np.float32, T.shape),
                pre=[pre[i + 1].numpy(np.float32, (B, sizes[i + 1])) for i in range(layers)],
                dW=[gW[i].numpy(np.float32, Ws[i].shape) for i in range(layers)],
                db=[gb[i].numpy(np.float32, bs[i].shape) for i in range(layers)], dX=tmp[0].numpy(np.float32, X.shape))


def gpu_mlp_step_fused(gpu, X, Ws, bs, T, head=False):
    D, l = gpu.DeviceBuffer, gpu.lib()
    B, layers = X.shape[0], len(Ws)
    sizes = [X.shape[1]] + [w.shape[0] for w in Ws]
    dW_, db_ = [D.from_numpy(w) for w in Ws], [D.from_numpy(b) for b in bs]
    pre = [None] + [D(4 * B * n) for n in sizes[1:]]
    act = [D.from_numpy(X)] + [D(4 * B * n) for n in sizes[1:-1]] + [None]
    dT, logp, loss = D.from_numpy(T), D(4 * B * sizes[-1]), D(4)
    g = [D(4 * B * n) for n in sizes]
    for i in range(layers):
        if i + 1 < layers:
            gpu.check(l.lten_hip_fc_forward_relu_f32(B, sizes[i], sizes[i + 1], act[i].ptr, dW_[i].ptr, db_[i].ptr, pre[i + 1].ptr, act[i + 1].ptr))
        else:
            gpu.check(l.lten_hip_fc_forward_f32(B, sizes[i], sizes[i + 1], act[i].ptr, dW_[i].ptr, db_[i].ptr, pre[i + 1].ptr))
    gW, gb = [D(w.nbytes) for w in Ws], [D(b.nbytes, zero=True) for b in bs]
    last = layers - 1
    if head == "tail":
        i = last  # a single layer has no relu in front of it
        gpu.check(l.lten_hip_fc_backward_log_softmax_nll_loss_f32(B, sizes[i], sizes[i + 1], act[i].ptr, dW_[i].ptr, pre[layers].ptr, dT.ptr,
                                                                  -1.0 / B, logp.ptr, loss.ptr, g[layers].ptr, pre[i].ptr if i > 0 else None,
                                                                  g[i].ptr, gW[i].ptr, gb[i].ptr))
        last -= 1
    elif head:
        gpu.check(l.lten_hip_log_softmax_nll_loss_grad_f32(B, sizes[-1], pre[layers].ptr, dT.ptr, -1.0 / B, logp.ptr, loss.ptr, g[layers].ptr))
    else:
        gpu.check(l.lten_hip_log_softmax_nll_loss_f32(B, sizes[-1], pre[layers].ptr, dT.ptr, logp.ptr, loss.ptr))
        gpu.check(l.lten_hip_nll_log_softmax_backward_f32(B, sizes[-1], logp.ptr, dT.ptr, -1.0 / B, g[layers].ptr))
    for i in range(last, -1, -1):
        if i > 0:
            gpu.check(l.lten_hip_fc_backward_relu_f32(B, sizes[i], sizes[i + 1], act[i].ptr, dW_[i].ptr, g[i + 1].ptr, pre[i].ptr,
                                                      g[i].ptr, gW[i].ptr, gb[i].ptr))
        else:
            gpu.check(l.lten_hip_fc_backward_f32(B, sizes[i], sizes[i + 1], act[i].ptr, dW_[i].ptr, g[i + 1].ptr, g[i].ptr, gW[i].ptr, gb[i].ptr))
    return dict(loss=float(loss.numpy(np.float32, (1,))[0]), logp=logp.numpy(np.float32, T.shape),
                pre=[pre[i + 1].numpy(np.float32, (B, sizes[i + 1])) for i in range(layers)],
                dW=[gW[i].numpy(np.float32, Ws[i].shape) for i in range(layers)],
                db=[gb[i].numpy(np.float32, bs[i].shape) for i in range(layers)], dX=g[0].numpy(np.float32, X.shape))


def check_step(got, want, tag):
    assert abs(got["loss"] - want["loss"]) < 1e-5 * max(1.0, abs(want["loss"])), tag
    assert rel_err(got["logp"], want["logp"]) < TOL, tag
    assert rel_err(got["dX"], want["dX"]) < TOL, tag
    for i in range(len(want["dW"])):
        assert rel_err(got["dW"][i], want["dW"][i]) < TOL, (tag, i)
        assert rel_err(got["db"][i], want["db"][i]) < TOL, (tag, i)


def test_mlp_step_golden_from_compiled_network(gpu):
    g = np.load(golden_path("mlp_step_case.npz"))
    Ws, bs = [g[f"W{i}"] for i in range(3)], [g[f"b{i}"] for i in range(3)]
    got = gpu_mlp_step(gpu, g["X"], Ws, bs, g["T"])
    want = dict(loss=float(g["loss"]), logp=g["logp"], dX=g["dX"], dW=[g[f"dW{i}"] for i in range(3)], db=[g[f"db{i}"] for i in range(3)])
    check_step(got, want, "golden")


def mlp_step_fp64(X, Ws, bs, T, masks=None):
    """The same step in fp64.  masks (one boolean array per hidden layer) replace the step's own relu decisions."""
    X, T = X.astype(np.float64), T.astype(np.float64)
    Ws, bs = [w.astype(np.float64) for w in Ws], [b.astype(np.float64) for b in bs]
    acts, pres, used = [X], [], []
    for i in range(len(Ws)):
        pres.append(acts[-1] @ Ws[i].T + bs[i])
        if i + 1 < len(Ws):
            used.append(masks[i] if masks is not None else pres[-1] > 0)
            acts.append(np.where(used[-1], pres[-1], 0.0))
    z = pres[-1] - pres[-1].max(axis=1, keepdims=True)
    logp = z - np.log(np.exp(z).sum(axis=1, keepdims=True))
    loss = -(logp * T).sum() / X.shape[0]
    g = (np.exp(logp) - T) / X.shape[0]
    dW, db = [None] * len(Ws), [None] * len(Ws)
    for i in range(len(Ws) - 1, -1, -1):
        dW[i], db[i] = g.T @ acts[i], g.sum(axis=0)
        g = g @ Ws[i]
        if i > 0:
            g = np.where(used[i - 1], g, 0.0)
    return dict(loss=loss, logp=logp, dW=dW, db=db, dX=g, pre=pres)


def test_cfg2_training_step_full_size(gpu, ob, wl):
    """784 -> 1024 -> 1024 -> 10 with bias and relu at batch 128, loss = nll(log_softmax).  The forward pass is held
    against the oracle's step.  Among the 262 144 hidden pre-activations a few lie within fp32 rounding of zero, where
    the summation order of a GEMM decides relu's branch; so the gradients are held against an fp64 evaluation of the
    same network that takes the device's relu decisions, after checking that those differ from the fp64 ones only
    where the pre-activation is that close to zero.  When the oracle took the same decisions it is compared as well."""
    X, Ws, bs, labels = wl.cfg2()
    T = np.eye(10, dtype=np.float32)[labels]
    want = ob.mlp_step(X, Ws, bs, T)
    got = gpu_mlp_step(gpu, X, Ws, bs, T)
    assert abs(got["loss"] - want["loss"]) < 1e-5 * max(1.0, abs(want["loss"]))
    assert rel_err(got["logp"], want["logp"]) < TOL
    free = mlp_step_fp64(X, Ws, bs, T)
    masks = [got["pre"][i] > 0 for i in range(2)]
    flips = 0
    for i in range(2):
        assert rel_err(got["pre"][i], free["pre"][i]) < TOL
        differ = masks[i] != (free["pre"][i] > 0)
        flips += int(differ.sum())
        assert np.abs(free["pre"][i][differ]).max(initial=0.0) < 1e-5, i
    ref = mlp_step_fp64(X, Ws, bs, T, masks)
    check_step(got, ref, "cfg2 vs fp64 with the device's relu decisions")
    if flips == 0:
        check_step(got, want, "cfg2 vs oracle")
    errs = [rel_err(got["dW"][i], ref["dW"][i]) for i in range(3)]
    print(f"  loss {got['loss']:.6f} (oracle {want['loss']:.6f}); relu decisions that differ from fp64: {flips}; "
          f"dW max rel err {max(errs):.2e}")
    # the route with the fused entry points (8 launches instead of 14) computes the same values bit for bit
    fused = gpu_mlp_step(gpu, X, Ws, bs, T, fused=True)
    assert fused["loss"] == got["loss"]
    for key in ("logp", "dX"):
        assert np.array_equal(fused[key], got[key]), key
    for key in ("pre", "dW", "db"):
        for a, b in zip(fused[key], got[key]):
            assert np.array_equal(a, b), key
    # and with the loss and its gradient as one call (7 launches)
    headed = gpu_mlp_step(gpu, X, Ws, bs, T, fused="head")
    assert headed["loss"] == got["loss"]
    for key in ("logp", "dX"):
        assert np.array_equal(headed[key], got[key]), key
    for key in ("pre", "dW", "db"):
        for a, b in zip(headed[key], got[key]):
            assert np.array_equal(a, b), key
    # and with the last layer's backward in that call as well (6 launches)
    tailed = gpu_mlp_step(gpu, X, Ws, bs, T, fused="tail")
    assert tailed["loss"] == got["loss"]
    for key in ("logp", "dX"):
        assert np.array_equal(tailed[key], got[key]), key
    for key in ("pre", "dW", "db"):
        for a, b in zip(tailed[key], got[key]):
            assert np.array_equal(a, b), key


@pytest.mark.parametrize("shape", [(128, 784, 1024), (7, 33, 50), (20, 2048, 640), (600, 96, 200), (300, 2048, 4096), (1, 64, 32)])
def test_fused_fc_relu_entry_points_match_the_unfused_calls(gpu, shape):
    """lten_hip_fc_forward_relu_f32 / lten_hip_fc_backward_relu_f32 against fc_forward + relu / fc_backward + relu_backward
    on shapes that reach every GEMM family (32x32 tiles, weight stream, LDS tiles, the large direct-to-LDS tiles, M = 1):
    bit-identical, whether the relu rides on the store or runs as a launch of its own."""
    M, fin, fout = shape
    rng = np.random.default_rng(M + fin + fout)
    D, l = gpu.DeviceBuffer, gpu.lib()
    X = rng.standard_normal((M, fin)).astype(np.float32)
    W = (rng.standard_normal((fout, fin)) * 0.05).astype(np.float32)
    b = rng.standard_normal(fout).astype(np.float32)
    dY = rng.standard_normal((M, fout)).astype(np.float32)
    Rin = rng.standard_normal((M, fin)).astype(np.float32)
    Rin[::3] = 0.0
    dX_, dW_, db_, ddY, dR = D.from_numpy(X), D.from_numpy(W), D.from_numpy(b), D.from_numpy(dY), D.from_numpy(Rin)
    y0, a0, y1, a1 = (D(4 * M * fout) for _ in range(4))
    gpu.check(l.lten_hip_fc_forward_f32(M, fin, fout, dX_.ptr, dW_.ptr, db_.ptr, y0.ptr))
    gpu.check(l.lten_hip_relu_f32(a0.ptr, y0.ptr, M * fout))
    gpu.check(l.lten_hip_fc_forward_relu_f32(M, fin, fout, dX_.ptr, dW_.ptr, db_.ptr, y1.ptr, a1.ptr))
    k_fwd = gpu.last_kernel()
    assert np.array_equal(y0.numpy(np.float32, (M, fout)), y1.numpy(np.float32, (M, fout)))
    assert np.array_equal(a0.numpy(np.float32, (M, fout)), a1.numpy(np.float32, (M, fout)))
    t0, g0, g1 = (D(4 * M * fin) for _ in range(3))
    w0, w1 = D(W.nbytes), D(W.nbytes)
    b0, b1 = D(b.nbytes, zero=True), D(b.nbytes, zero=True)
    gpu.check(l.lten_hip_fc_backward_f32(M, fin, fout, dX_.ptr, dW_.ptr, ddY.ptr, t0.ptr, w0.ptr, b0.ptr))
    gpu.check(l.lten_hip_relu_backward_f32(g0.ptr, t0.ptr, dR.ptr, M * fin))
    gpu.check(l.lten_hip_fc_backward_relu_f32(M, fin, fout, dX_.ptr, dW_.ptr, ddY.ptr, dR.ptr, g1.ptr, w1.ptr, b1.ptr))
    print(f"  {shape}: forward via {k_fwd}, backward via {gpu.last_kernel()}", flush=True)
    assert np.array_equal(g0.numpy(np.float32, (M, fin)), g1.numpy(np.float32, (M, fin)))
    assert np.array_equal(w0.numpy(np.float32, W.shape), w1.numpy(np.float32, W.shape))
    assert np.array_equal(b0.numpy(np.float32, b.shape), b1.numpy(np.float32, b.shape))


@pytest.mark.parametrize("rows,cols", [(2000, 16), (5000, 10), (3000, 32), (4001, 20), (1024, 1), (64, 50257), (7, 1024), (300, 2048), (9, 8192),
                                       (3, 70000), (2, 8193), (33, 1500), (1023, 16), (100, 1023), (500, 256), (40, 255), (2000, 1000)])
def test_log_softmax_on_narrow_and_wide_rows(gpu, rows, cols):
    """Rows of at most 32 values share a wavefront, rows of 256 and more take a workgroup each: forward and backward
    against float64 within the fp32 tolerance, the same bits on a second run, and rows that hold large and equal values."""
    rng = np.random.default_rng(rows * 3 + cols)
    D, l = gpu.DeviceBuffer, gpu.lib()
    x = (rng.standard_normal((rows, cols)) * 4).astype(np.float32)
    x[0, :] = 80.0                       # equal values: log(1 / cols)
    if cols > 1:
        x[-1, 0] = 300.0                 # one dominant value: exp of the others underflows
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    dx_, dg = D.from_numpy(x), D.from_numpy(dy)
    y0, y1, g0 = D(x.nbytes), D(x.nbytes), D(x.nbytes)
    gpu.check(l.lten_hip_log_softmax_f32(rows, cols, dx_.ptr, y0.ptr))
    gpu.check(l.lten_hip_log_softmax_f32(rows, cols, dx_.ptr, y1.ptr))
    y = y0.numpy(np.float32, x.shape)
    assert np.array_equal(y, y1.numpy(np.float32, x.shape))
    x64 = x.astype(np.float64)
    m = x64.max(axis=1, keepdims=True)
    e = np.exp(x64 - m)
    with np.errstate(divide="ignore"):
        want = np.log(e.astype(np.float32).astype(np.float64) / e.sum(axis=1, keepdims=True))   # l-ten's chain: log(exp(x - max) / sum)
    finite = np.isfinite(want)
    assert np.array_equal(np.isfinite(y), finite)
    assert np.abs(y[finite] - want[finite]).max() < 1e-4 * max(1.0, np.abs(want[finite]).max())
    gpu.check(l.lten_hip_log_softmax_backward_f32(rows, cols, y0.ptr, dg.ptr, g0.ptr))
    g = g0.numpy(np.float32, x.shape)
    want_g = dy.astype(np.float64) - np.exp(y.astype(np.float64)) * dy.astype(np.float64).sum(axis=1, keepdims=True)
    assert np.abs(g - want_g).max() < 1e-4 * max(1.0, np.abs(want_g).max())


@pytest.mark.parametrize("rows,cols", [(4096, 1000), (64, 50257), (1 << 18, 16), (700, 100), (65537, 1)])
def test_nll_loss_over_long_arrays(gpu, rows, cols):
    """Beyond 65536 values the loss is summed share by share on many workgroups and the shares in index order: against
    float64, twice the same bits, and through the entry points that stand for several launches."""
    rng = np.random.default_rng(rows + cols)
    D, l = gpu.DeviceBuffer, gpu.lib()
    x = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    labels = rng.integers(0, cols, rows)
    t = np.zeros((rows, cols), np.float32)
    t[np.arange(rows), labels] = 1.0
    dx_, dt, y, l0, l1, l2, g = D.from_numpy(x), D.from_numpy(t), D(x.nbytes), D(4), D(4), D(4), D(x.nbytes)
    gpu.check(l.lten_hip_log_softmax_f32(rows, cols, dx_.ptr, y.ptr))
    gpu.check(l.lten_hip_nll_loss_f32(y.ptr, dt.ptr, l0.ptr, rows * cols, rows))
    gpu.check(l.lten_hip_nll_loss_f32(y.ptr, dt.ptr, l1.ptr, rows * cols, rows))
    logp = y.numpy(np.float32, x.shape)
    want = -logp[np.arange(rows), labels].astype(np.float64).sum() / rows
    got = float(l0.numpy(np.float32, (1,))[0])
    assert got == float(l1.numpy(np.float32, (1,))[0])
    assert abs(got - want) < 1e-4 * max(1.0, abs(want)), (got, want)
    gpu.check(l.lten_hip_log_softmax_nll_loss_grad_f32(rows, cols, dx_.ptr, dt.ptr, -1.0 / rows, y.ptr, l2.ptr, g.ptr))
    assert float(l2.numpy(np.float32, (1,))[0]) == got


def test_fused_loss_entry_points_match_the_unfused_calls(gpu):
    rng = np.random.default_rng(11)
    D, l = gpu.DeviceBuffer, gpu.lib()
    for rows, cols in ((1, 1), (128, 10), (1024, 16), (1000, 7), (3, 16), (1025, 16), (37, 400), (16, 1024), (5, 4097), (64, 17)):
        x = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
        t = np.eye(cols, dtype=np.float32)[rng.integers(0, cols, rows)]
        dx, dt = D.from_numpy(x), D.from_numpy(t)
        y0, y1, l0, l1, s0, g0, g1 = D(x.nbytes), D(x.nbytes), D(4), D(4), D(x.nbytes), D(x.nbytes), D(x.nbytes)
        gpu.check(l.lten_hip_log_softmax_f32(rows, cols, dx.ptr, y0.ptr))
        gpu.check(l.lten_hip_nll_loss_f32(y0.ptr, dt.ptr, l0.ptr, rows * cols, rows))
        gpu.check(l.lten_hip_log_softmax_nll_loss_f32(rows, cols, dx.ptr, dt.ptr, y1.ptr, l1.ptr))
        assert np.array_equal(y0.numpy(np.float32, x.shape), y1.numpy(np.float32, x.shape)), (rows, cols)
        assert l0.numpy(np.float32, (1,))[0] == l1.numpy(np.float32, (1,))[0], (rows, cols)
        gpu.check(l.lten_hip_scale_f32(rows * cols, -1.0 / rows, dt.ptr, s0.ptr))
        gpu.check(l.lten_hip_log_softmax_backward_f32(rows, cols, y0.ptr, s0.ptr, g0.ptr))
        gpu.check(l.lten_hip_nll_log_softmax_backward_f32(rows, cols, y0.ptr, dt.ptr, -1.0 / rows, g1.ptr))
        assert np.array_equal(g0.numpy(np.float32, x.shape), g1.numpy(np.float32, x.shape)), (rows, cols)
        y2, l2, g2 = D(x.nbytes), D(4), D(x.nbytes)
        gpu.check(l.lten_hip_log_softmax_nll_loss_grad_f32(rows, cols, dx.ptr, dt.ptr, -1.0 / rows, y2.ptr, l2.ptr, g2.ptr))
        assert np.array_equal(y0.numpy(np.float32, x.shape), y2.numpy(np.float32, x.shape)), (rows, cols)
        assert l0.numpy(np.float32, (1,))[0] == l2.numpy(np.float32, (1,))[0], (rows, cols)
        assert np.array_equal(g0.numpy(np.float32, x.shape), g2.numpy(np.float32, x.shape)), (rows, cols)


@pytest.mark.parametrize("shape", [(128, 1024, 10), (2, 40, 2), (100, 516, 16), (255, 33, 16), (409, 64, 10), (300, 128, 16), (64, 9000, 10),
                                   (511, 20, 8), (128, 1024, 17), (1, 64, 10), (512, 64, 8), (37, 12, 1)])
def test_loss_with_the_last_layers_backward_matches_the_separate_calls(gpu, shape):
    """lten_hip_fc_backward_log_softmax_nll_loss_f32 against lten_hip_log_softmax_nll_loss_grad_f32 followed by
    lten_hip_fc_backward_f32: log-probabilities, loss, gradient of the logits, dX, dW and db bit-identical, on shapes the
    one-launch kernel takes (ragged tiles, full LDS, a wide input) and on shapes it hands to the separate launches."""
    M, fin, fout = shape
    rng = np.random.default_rng(M * 7 + fin + fout)
    D, l = gpu.DeviceBuffer, gpu.lib()
    X = rng.standard_normal((M, fin)).astype(np.float32)
    W = (rng.standard_normal((fout, fin)) * 0.05).astype(np.float32)
    logits = (rng.standard_normal((M, fout)) * 3).astype(np.float32)
    T = np.eye(fout, dtype=np.float32)[rng.integers(0, fout, M)]
    b = rng.standard_normal(fout).astype(np.float32)
    dX_, dW_, dL, dT = D.from_numpy(X), D.from_numpy(W), D.from_numpy(logits), D.from_numpy(T)
    out = []
    for fused in (False, True):
        y, loss, gl, gx, gw, gb = D(logits.nbytes), D(4), D(logits.nbytes), D(X.nbytes), D(W.nbytes), D.from_numpy(b)
        if fused:
            gpu.check(l.lten_hip_fc_backward_log_softmax_nll_loss_f32(M, fin, fout, dX_.ptr, dW_.ptr, dL.ptr, dT.ptr, -1.0 / M, y.ptr, loss.ptr,
                                                                      gl.ptr, None, gx.ptr, gw.ptr, gb.ptr))
            print(f"  {shape}: {gpu.last_kernel()}", flush=True)
        else:
            gpu.check(l.lten_hip_log_softmax_nll_loss_grad_f32(M, fout, dL.ptr, dT.ptr, -1.0 / M, y.ptr, loss.ptr, gl.ptr))
            gpu.check(l.lten_hip_fc_backward_f32(M, fin, fout, dX_.ptr, dW_.ptr, gl.ptr, gx.ptr, gw.ptr, gb.ptr))
        out.append([y.numpy(np.float32, logits.shape), loss.numpy(np.float32, (1,)), gl.numpy(np.float32, logits.shape),
                    gx.numpy(np.float32, X.shape), gw.numpy(np.float32, W.shape), gb.numpy(np.float32, b.shape)])
    if shape == (128, 1024, 10):
        assert gpu.last_kernel() == "sgemm_fc_backward_pair_loss"
    for name, a, c in zip(("log_probs", "loss", "dlogits", "dX", "dW", "db"), out[0], out[1]):
        assert np.array_equal(a, c), (shape, name)
    # against numpy in fp64
    z = logits.astype(np.float64) - logits.max(axis=1, keepdims=True)
    lp = z - np.log(np.exp(z).sum(axis=1, keepdims=True))
    g = (np.exp(lp) - T) / M
    assert rel_err(out[1][0], lp) < TOL and rel_err(out[1][2], g) < TOL
    assert abs(out[1][1][0] + (lp * T).sum() / M) < 1e-5 * max(1.0, abs((lp * T).sum() / M))
    assert rel_err(out[1][3], g @ W) < TOL and rel_err(out[1][4], g.T @ X) < TOL and rel_err(out[1][5], b + g.sum(axis=0)) < TOL


def test_elementwise_kernels(gpu, ob):
    rng = np.random.default_rng(9)
    D, l = gpu.DeviceBuffer, gpu.lib()
    for n in (1, 63, 1000, 1 << 20):
        x = rng.standard_normal(n).astype(np.float32)
        x[::5] = 0.0
        top = rng.standard_normal(n).astype(np.float32)
        dx, dt, dy, db = D.from_numpy(x), D.from_numpy(top), D(4 * n), D(4 * n)
        gpu.check(l.lten_hip_relu_f32(dy.ptr, dx.ptr, n))
        gpu.check(l.lten_hip_relu_backward_f32(db.ptr, dt.ptr, dx.ptr, n))
        assert np.array_equal(dy.numpy(np.float32, (n,)), np.where(x > 0, x, np.float32(0)))
        assert np.array_equal(db.numpy(np.float32, (n,)), np.where(x > 0, top, np.float32(0)))
        gpu.check(l.lten_hip_scale_f32(n, -0.37, dx.ptr, dy.ptr))
        assert np.array_equal(dy.numpy(np.float32, (n,)), np.float32(-0.37) * x)
        gpu.check(l.lten_hip_axpy_f32(n, 1.0, dt.ptr, dy.ptr))
        assert np.array_equal(dy.numpy(np.float32, (n,)), np.float32(-0.37) * x + top)
    for rows, cols in ((1, 1), (128, 10), (37, 1000), (5, 4097)):
        z = (rng.standard_normal((rows, cols)) * 4).astype(np.float32)
        dyv = rng.standard_normal((rows, cols)).astype(np.float32)
        T = np.zeros((rows, cols), np.float32)
        T[np.arange(rows), rng.integers(0, cols, rows)] = 1
        want_lp, want_dx = np.empty_like(z), np.empty_like(z)
        ob.oracle().oracle_log_softmax(rows, cols, z.reshape(-1), want_lp.reshape(-1))
        ob.oracle().oracle_log_softmax_backward(rows, cols, want_lp.reshape(-1), dyv.reshape(-1), want_dx.reshape(-1))
        dz, dlp, ddy, ddx, dT, dl = D.from_numpy(z), D(z.nbytes), D.from_numpy(dyv), D(z.nbytes), D.from_numpy(T), D(4)
        gpu.check(l.lten_hip_log_softmax_f32(rows, cols, dz.ptr, dlp.ptr))
        gpu.check(l.lten_hip_log_softmax_backward_f32(rows, cols, dlp.ptr, ddy.ptr, ddx.ptr))
        gpu.check(l.lten_hip_nll_loss_f32(dlp.ptr, dT.ptr, dl.ptr, rows * cols, rows))
        assert rel_err(dlp.numpy(np.float32, z.shape), want_lp) < 1e-5
        assert rel_err(ddx.numpy(np.float32, z.shape), want_dx) < TOL
        want_loss = ob.oracle().oracle_nll_loss(want_lp.reshape(-1), T.reshape(-1), rows * cols, rows)
        assert abs(dl.numpy(np.float32, (1,))[0] - want_loss) < 1e-5 * max(1.0, abs(want_loss))


def test_optimizer_steps(gpu, ob):
    """Five SGD / Adam steps on the device against the golden weights of the compiled l-ten optimizers: SGD bit-exact
    (every operation rounded on its own, as on the CPU), Adam within 1e-6 (its powf comes from a different libm)."""
    g = np.load(golden_path("optimizer_cases.npz"))
    D, l = gpu.DeviceBuffer, gpu.lib()
    n = g["w0"].size
    for name in ("sgd", "sgd_plain", "adam", "adam_fast"):
        p = [float(v) for v in g[name + "_p"]]
        dw, dv, ds = D.from_numpy(g["w0"]), D(4 * n, zero=True), D(4 * n, zero=True)
        for it in range(1, 6):
            dg = D.from_numpy(g["g"])
            if name.startswith("sgd"):
                gpu.check(l.lten_hip_sgd_step_f32(dw.ptr, dg.ptr, dv.ptr, n, p[0], p[1], p[2]))
            else:
                gpu.check(l.lten_hip_adam_step_f32(dw.ptr, dg.ptr, dv.ptr, ds.ptr, n, p[0], p[1], p[2], it))
        got = dw.numpy(np.float32, (n,))
        if name.startswith("sgd"):
            assert np.array_equal(got, g[name + "_w"]), name
        else:
            assert np.abs(got - g[name + "_w"]).max() < 1e-6 * max(1.0, np.abs(g[name + "_w"]).max()), name


def test_recorded_step_replays_like_the_eager_step(gpu):
    """Two FullyConnected layers with relu, forward and backward, recorded once and replayed four times with new
    inputs, eager work and synchronisation between the replays: every replay must equal the eager calls bit for bit
    (same kernels, same order)."""
    D, l = gpu.DeviceBuffer, gpu.lib()
    rng = np.random.default_rng(77)
    B, n0, n1, n2 = 64, 200, 320, 48
    W1, b1 = rng.standard_normal((n1, n0)).astype(np.float32) * 0.1, rng.standard_normal(n1).astype(np.float32)
    W2, b2 = rng.standard_normal((n2, n1)).astype(np.float32) * 0.1, rng.standard_normal(n2).astype(np.float32)
    dW1, db1, dW2, db2 = D.from_numpy(W1), D.from_numpy(b1), D.from_numpy(W2), D.from_numpy(b2)
    x, h, a, y = D(4 * B * n0), D(4 * B * n1), D(4 * B * n1), D(4 * B * n2)
    gy, ga, gh, gx = D(4 * B * n2), D(4 * B * n1), D(4 * B * n1), D(4 * B * n0)
    gW1, gb1, gW2, gb2 = D(W1.nbytes), D(b1.nbytes), D(W2.nbytes), D(b2.nbytes)
    outs = [(y, (B, n2)), (gx, (B, n0)), (gW1, W1.shape), (gb1, b1.shape), (gW2, W2.shape), (gb2, b2.shape)]

    def step():
        gpu.check(l.lten_hip_fill_f32(gb1.ptr, n1, 0.0))
        gpu.check(l.lten_hip_fill_f32(gb2.ptr, n2, 0.0))
        gpu.check(l.lten_hip_fc_forward_f32(B, n0, n1, x.ptr, dW1.ptr, db1.ptr, h.ptr))
        gpu.check(l.lten_hip_relu_f32(a.ptr, h.ptr, B * n1))
        gpu.check(l.lten_hip_fc_forward_f32(B, n1, n2, a.ptr, dW2.ptr, db2.ptr, y.ptr))
        gpu.check(l.lten_hip_fc_backward_f32(B, n1, n2, a.ptr, dW2.ptr, gy.ptr, ga.ptr, gW2.ptr, gb2.ptr))
        gpu.check(l.lten_hip_relu_backward_f32(gh.ptr, ga.ptr, h.ptr, B * n1))
        gpu.check(l.lten_hip_fc_backward_f32(B, n0, n1, x.ptr, dW1.ptr, gh.ptr, gx.ptr, gW1.ptr, gb1.ptr))

    def load_inputs(seed):
        r = np.random.default_rng(seed)
        x.upload(r.standard_normal((B, n0)).astype(np.float32))
        gy.upload(r.standard_normal((B, n2)).astype(np.float32))

    def read():
        return [buf.numpy(np.float32, shape).copy() for buf, shape in outs]

    load_inputs(0)
    step()
    with gpu.Graph() as graph:
        step()
    for replay in range(4):
        load_inputs(100 + replay)
        step()
        want = read()
        for buf, shape in outs:  # eager work between the replays: wipe what the replay has to rewrite
            gpu.check(l.lten_hip_fill_f32(buf.ptr, int(np.prod(shape)), -7.0))
        gpu.sync()
        graph.launch()
        got = read()
        for w, g_ in zip(want, got):
            assert np.array_equal(w, g_), replay
    # misuse is reported, not recorded
    assert l.lten_hip_graph_launch(None) != 0
    import ctypes
    p = ctypes.c_void_p()
    assert l.lten_hip_graph_end(ctypes.byref(p)) != 0 and b"no capture" in l.lten_hip_last_error()
