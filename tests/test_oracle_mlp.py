"""CPU tests of the oracle's element-wise pieces (relu, log_softmax, nll_loss and their backward) and of the whole MLP
training step they form with the FullyConnected GEMMs."""
import numpy as np

from conftest import golden_path, rel_err


def load_case():
    g = np.load(golden_path("mlp_step_case.npz"))
    Ws, bs = [g[f"W{l}"] for l in range(3)], [g[f"b{l}"] for l in range(3)]
    return g, Ws, bs


def test_mlp_step_golden_from_compiled_network(ob):
    g, Ws, bs = load_case()
    r = ob.mlp_step(g["X"], Ws, bs, g["T"])
    assert abs(r["loss"] - float(g["loss"])) < 1e-6
    assert rel_err(r["logp"], g["logp"]) < 1e-6
    assert rel_err(r["dX"], g["dX"]) < 1e-5
    for l in range(3):
        assert rel_err(r["dW"][l], g[f"dW{l}"]) < 1e-5, l
        assert rel_err(r["db"][l], g[f"db{l}"]) < 1e-5, l


def test_mlp_step_gradients_by_finite_differences(ob):
    """d loss / d parameter from central differences of an fp64 evaluation of the same network."""
    g, Ws, bs = load_case()
    X, T = g["X"].astype(np.float64), g["T"].astype(np.float64)

    def loss64(Ws64, bs64):
        h = X
        for l in range(3):
            h = h @ Ws64[l].T + bs64[l]
            if l < 2:
                h = np.maximum(h, 0)
        z = h - h.max(axis=1, keepdims=True)
        logp = z - np.log(np.exp(z).sum(axis=1, keepdims=True))
        return -(logp * T).sum() / X.shape[0]

    r = ob.mlp_step(g["X"], Ws, bs, g["T"])
    W64, b64 = [w.astype(np.float64) for w in Ws], [b.astype(np.float64) for b in bs]
    assert abs(r["loss"] - loss64(W64, b64)) < 1e-6
    rng = np.random.default_rng(0)
    eps = 1e-5
    for l in range(3):
        for _ in range(6):
            i, j = int(rng.integers(0, Ws[l].shape[0])), int(rng.integers(0, Ws[l].shape[1]))
            Wp, Wm = [w.copy() for w in W64], [w.copy() for w in W64]
            Wp[l][i, j] += eps
            Wm[l][i, j] -= eps
            fd = (loss64(Wp, b64) - loss64(Wm, b64)) / (2 * eps)
            assert abs(fd - r["dW"][l][i, j]) < 2e-5, (l, i, j)
        k = int(rng.integers(0, bs[l].shape[0]))
        bp, bm = [b.copy() for b in b64], [b.copy() for b in b64]
        bp[l][k] += eps
        bm[l][k] -= eps
        fd = (loss64(W64, bp) - loss64(W64, bm)) / (2 * eps)
        assert abs(fd - r["db"][l][k]) < 2e-5, (l, k)


def test_elementwise_closed_forms(ob):
    rng = np.random.default_rng(3)
    x = rng.standard_normal(1000).astype(np.float32)
    x[::7] = 0.0
    y = np.empty_like(x)
    ob.oracle().oracle_relu(x, y, x.size)
    assert np.array_equal(y, np.where(x > 0, x, np.float32(0)))
    top = rng.standard_normal(1000).astype(np.float32)
    bot = np.empty_like(x)
    ob.oracle().oracle_relu_backward(top, x, bot, x.size)
    assert np.array_equal(bot, np.where(x > 0, top, np.float32(0)))   # gradient 0 at x == 0, as l-ten's `> 0`
    # log_softmax: rows sum to 1 after exp, shift invariance, fp64 agreement
    z = (rng.standard_normal((37, 10)) * 5).astype(np.float32)
    lp = np.empty_like(z)
    ob.oracle().oracle_log_softmax(37, 10, z.reshape(-1), lp.reshape(-1))
    z64 = z.astype(np.float64)
    want = z64 - z64.max(1, keepdims=True) - np.log(np.exp(z64 - z64.max(1, keepdims=True)).sum(1, keepdims=True))
    assert np.abs(lp - want).max() < 2e-6
    assert np.abs(np.exp(lp.astype(np.float64)).sum(1) - 1).max() < 1e-6
    # its backward against the Jacobian of the fp64 function
    dy = rng.standard_normal((37, 10)).astype(np.float32)
    dx = np.empty_like(z)
    ob.oracle().oracle_log_softmax_backward(37, 10, lp.reshape(-1), dy.reshape(-1), dx.reshape(-1))
    want_dx = dy.astype(np.float64) - np.exp(want) * dy.astype(np.float64).sum(1, keepdims=True)
    assert np.abs(dx - want_dx).max() < 1e-5
    # nll: one-hot targets pick -mean(logp[label]); backward is -target / batch * top
    T = np.eye(10, dtype=np.float32)[rng.integers(0, 10, 37)]
    loss = ob.oracle().oracle_nll_loss(lp.reshape(-1), T.reshape(-1), 370, 37)
    assert abs(loss + float((want * T).sum() / 37)) < 1e-6
    g = np.empty_like(T)
    ob.oracle().oracle_nll_backward(T.reshape(-1), 370, 37, 2.0, g.reshape(-1))
    assert np.array_equal(g, np.float32(np.float32(-1.0 / 37) * np.float32(2.0)) * T)


# ----------------------------------------------------------------------------------------- optimizer steps

def run_oracle_optimizer(ob, kind, p, w0, g, steps=5):
    w, v, s = w0.copy(), np.zeros_like(w0), np.zeros_like(w0)
    for it in range(1, steps + 1):
        if kind == "sgd":
            gg = g.copy()    # the step overwrites the gradient with the decayed one
            ob.oracle().oracle_sgd_step(w, gg, v, w.size, float(p[0]), float(p[1]), float(p[2]))
        else:
            ob.oracle().oracle_adam_step(w, g, v, s, w.size, float(p[0]), float(p[1]), float(p[2]), it)
    return w


def test_optimizer_steps_golden_from_compiled_optimizers(ob):
    g = np.load(golden_path("optimizer_cases.npz"))
    for name in ("sgd", "sgd_plain", "adam", "adam_fast"):
        w = run_oracle_optimizer(ob, "sgd" if name.startswith("sgd") else "adam", g[name + "_p"], g["w0"], g["g"])
        assert np.array_equal(w, g[name + "_w"]), name   # same libm on both sides: bit-exact


def test_optimizer_closed_forms(ob):
    w0 = np.array([1.0, -2.0, 0.5], np.float32)
    g = np.array([0.5, 0.25, -1.0], np.float32)
    # no momentum, no decay: plain gradient descent
    w = run_oracle_optimizer(ob, "sgd", [0.0, 0.0, 0.1], w0, g, steps=1)
    assert np.allclose(w, w0 - 0.1 * g, rtol=1e-6)
    # Adam's first step moves every weight by lr * sign(g) (bias corrections cancel the history factors)
    w = run_oracle_optimizer(ob, "adam", [0.01, 0.9, 0.999], w0, g, steps=1)
    assert np.allclose(w, w0 - 0.01 * np.sign(g), rtol=0, atol=1e-6)
