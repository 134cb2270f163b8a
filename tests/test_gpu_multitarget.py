"""Several targets at once (a matrix target: src/init.jl:11-16, src/loss.jl:49-50, :100-111, :219-236; the reference's
test/multi-target.jl): K outputs for mse / logloss / poisson / gamma / tweedie, 2 per target for gaussian_mle.  Gradients,
trees (bit for bit against the fixed-point oracle, structure and 1e-5 against the Float64 one), node ids, the updated
prediction, the evaluation metric and whole-model inference, all through the C ABI."""
import numpy as np
import pytest

from oracle import oracle as orc
from test_gpu_parity import RTOL, assert_tree_bits, setup_pair

pytestmark = pytest.mark.gpu


def make_targets(seed, N, F, B, loss, T, weights):
    rng = np.random.default_rng(seed)
    x_bin = rng.integers(1, B + 1, size=(F, N), dtype=np.uint8)
    y = np.empty((N, T), np.float32)
    for t in range(T):
        f1, f2 = (3 * t) % F, (5 * t + 1) % F
        y[:, t] = rng.random(N) + 0.6 * (x_bin[f1] / B) + 0.3 * (x_bin[f2] > (B * (t + 1)) // (T + 1))
    if loss == "logloss":
        y = (y > np.median(y, axis=0)).astype(np.float32)
    elif loss == "poisson":
        y = np.floor(y * 3).astype(np.float32)
    elif loss in ("gamma", "tweedie"):
        y = (y + 0.1).astype(np.float32)
    elif loss == "quantile":
        y = (y - 0.95).astype(np.float32)  # residuals of both signs against the starting prediction near zero
    K = 2 * T if loss in ("gaussian_mle", "logistic_mle") else T
    w = (rng.random(N).astype(np.float32) + 0.5) if weights else None
    mu = (rng.standard_normal(K) * 0.1).astype(np.float32)
    return x_bin, y, w, mu


CASES = [
    # loss, targets, weights, N, F, B, D, tree_type, n_js, rowsample, categorical
    ("mse", 2, False, 20000, 12, 32, 5, "binary", 12, 1.0, False),
    ("mse", 5, True, 9000, 100, 64, 4, "binary", 50, 0.5, False),
    ("logloss", 3, True, 15000, 20, 16, 5, "binary", 20, 1.0, True),
    ("poisson", 2, False, 8000, 9, 64, 4, "binary", 9, 0.5, False),
    ("gamma", 4, True, 7000, 33, 8, 3, "oblivious", 20, 1.0, False),
    ("tweedie", 2, False, 6000, 17, 128, 4, "binary", 17, 1.0, True),
    ("gaussian_mle", 2, True, 16000, 14, 32, 5, "binary", 14, 1.0, False),
    ("gaussian_mle", 3, False, 9000, 50, 64, 4, "oblivious", 30, 0.5, False),
    ("mse", 16, False, 3000, 6, 16, 3, "binary", 6, 1.0, False),
    ("gaussian_mle", 8, True, 3000, 6, 255, 3, "binary", 6, 1.0, False),
    ("logistic_mle", 2, True, 12000, 14, 32, 5, "binary", 14, 1.0, False),
    ("logistic_mle", 3, False, 9000, 40, 64, 4, "oblivious", 25, 0.5, True),
    ("mae", 3, True, 12000, 14, 32, 5, "binary", 14, 1.0, False),
    ("mae", 2, False, 9000, 40, 64, 4, "oblivious", 25, 0.5, True),
    ("cred_var", 2, True, 12000, 14, 32, 5, "binary", 10, 1.0, True),
    ("cred_std", 4, False, 9000, 20, 16, 4, "binary", 20, 0.5, False),
    ("quantile", 3, True, 12000, 14, 32, 5, "binary", 14, 1.0, False),
    ("quantile", 2, False, 9000, 20, 16, 4, "oblivious", 20, 0.5, True),
]


@pytest.mark.parametrize("loss,T,weights,N,F,B,D,tt,n_js,rowsample,cat", CASES)
def test_multi_target_tree_against_the_oracle(evt, loss, T, weights, N, F, B, D, tt, n_js, rowsample, cat):
    rng = np.random.default_rng(31)
    x_bin, y, w, mu = make_targets(900, N, F, B, loss, T, weights)
    K = mu.shape[0]
    feattypes = (rng.random(F) > 0.3).astype(np.uint8) if cat else None
    min_weight = 8.0 if loss in ("gaussian_mle", "logistic_mle") else 1.0
    h, o, op, gp, pred0, grad0 = setup_pair(evt, loss, x_bin, y, w, mu, B, D, tt, feattypes=feattypes, min_weight=min_weight, L2=0.1)
    # gradients: the kernel against the oracle (mse is exact Float32 arithmetic)
    grad = grad0.copy()
    orc.update_grads(op, pred0, y, grad)
    h.update_grads()
    g_dev = h.get_grads()
    if loss in ("mse", "mae", "cred_var", "cred_std", "quantile"):
        assert np.array_equal(g_dev.view(np.uint32), grad.view(np.uint32))
    else:
        # (1 - r^2 / s^2) and (1 - z tanh(z / 2)) cancel, which magnifies the last-bit differences between two libm's exp / tanh:
        # the absolute bound scales with the largest gradient
        np.testing.assert_allclose(g_dev, grad, rtol=2e-6, atol=1e-6 * float(np.abs(grad[:, :2 * K]).max()))
    assert np.array_equal(g_dev[:, 2 * K], grad[:, 2 * K])
    # one tree on identical gradients
    h.set_grads(grad)
    h.set_option("record_nidx", 1)
    js = (np.sort(rng.choice(F, n_js, replace=False)) + 1).astype(np.uint32)
    if rowsample < 1.0:
        mask = rng.integers(0, 256, N, dtype=np.uint8)
        cond = int(np.rint(255 * rowsample))
        rows = orc.subsample(mask, cond)
    else:
        mask, cond, rows = None, 255, np.arange(N, dtype=np.uint32)
    t_gpu = h.grow_tree(js, gp, mask=mask, cond=cond)
    qb, qe = h.get_quant()
    o.set_quant(grad, qb)
    assert np.array_equal(o.get_quant()[1], qe)
    t_fx, nidx_fx = o.grow_tree(grad, rows, js, mode=1)
    assert_tree_bits(t_gpu, t_fx)
    assert t_gpu.pred.shape == (t_gpu.feat.shape[0], K)
    if D > 1 and N >= 3000:
        assert t_gpu.split[0]
    assert np.array_equal(h.get_nidx(), nidx_fx)
    p_orc = pred0.copy()
    o.predict_tree(t_fx, p_orc)
    assert np.array_equal(h.get_pred().view(np.uint32), p_orc.view(np.uint32))
    # histograms of the split nodes, every output's gradient and hessian row
    H_gpu, Hq = h.get_hist(), o.hist(fixed=True)
    scale = np.ldexp(1.0, (qe - qb).astype(np.int64))
    for n0 in np.flatnonzero(t_gpu.split)[:6]:
        assert np.array_equal(H_gpu[n0][js - 1], Hq[n0][js - 1].astype(np.float64) * scale), n0
    # Float64 reference arithmetic
    t_ref, _ = o.grow_tree(grad, rows, js, mode=0)
    same = np.array_equal(t_gpu.feat, t_ref.feat) and np.array_equal(t_gpu.cond_bin, t_ref.cond_bin)
    if same:
        np.testing.assert_allclose(t_gpu.pred, t_ref.pred, rtol=RTOL, atol=1e-7)
        np.testing.assert_allclose(t_gpu.gain, t_ref.gain, rtol=RTOL, atol=1e-7)
    else:
        n0 = int(np.flatnonzero((t_gpu.feat != t_ref.feat) | (t_gpu.cond_bin != t_ref.cond_bin))[0])
        assert abs(float(t_gpu.gain[n0]) - float(t_ref.gain[n0])) <= 1e-6 * abs(float(t_ref.gain[n0])) + 1e-12
    # the evaluation metric on the updated prediction
    metric = {"mse": "mse", "logloss": "logloss", "poisson": "poisson", "gamma": "gamma", "tweedie": "tweedie",
              "gaussian_mle": "gaussian_mle", "logistic_mle": "logistic_mle", "mae": "mae", "cred_var": "mae", "cred_std": "mae", "quantile": "quantile"}[loss]
    got = h.eval_metric(metric)
    want = orc.eval_metric(metric, K, p_orc, y, w, alphas=[0.5])
    assert abs(got - want) <= 1e-5 * abs(want) + 1e-9
    if loss == "mse":
        assert abs(h.eval_metric("rmse") - np.sqrt(want)) <= 1e-5 * np.sqrt(want)
        # closed form, independent of the oracle: mean over rows of w * mean_k (p - y)^2 / mean w
        ww = np.ones(N, np.float32) if w is None else w
        cf = float((ww.astype(np.float64) * ((p_orc.astype(np.float64) - y) ** 2).mean(axis=1)).sum() / ww.astype(np.float64).sum())
        assert abs(got - cf) <= 1e-5 * cf
    # whole-model inference: the bias tree and this tree
    bias = orc.Tree(K, 1)
    bias.pred[0] = mu
    raw = evt._lib.predict_model(x_bin, feattypes, loss, K, [bias, t_gpu], apply_link=False)
    want_raw = np.zeros((N, K), np.float32)
    for t in (bias, t_gpu):
        orc.predict_tree(orc.LOSS_IDS[loss], K, x_bin, feattypes if feattypes is not None else np.ones(F, np.uint8), t, want_raw)
    assert np.array_equal(raw.view(np.uint32), want_raw.view(np.uint32))
    h.close()
    o.close()


def test_multi_target_free_running_rounds(evt):
    """Ten rounds without teacher forcing, two mse targets: gradients, trees and predictions bit-equal to the oracle's."""
    N, F, B, D, T = 30000, 10, 32, 5, 2
    x_bin, y, w, mu = make_targets(5, N, F, B, "mse", T, True)
    h, o, op, gp, pred, grad = setup_pair(evt, "mse", x_bin, y, w, mu, B, D, eta=0.3)
    js = np.arange(1, F + 1, dtype=np.uint32)
    rows = np.arange(N, dtype=np.uint32)
    for r in range(10):
        h.update_grads()
        orc.update_grads(op, pred, y, grad)
        t_gpu = h.grow_tree(js, gp)
        qb, _ = h.get_quant()
        o.set_quant(grad, qb)
        t_fx, _ = o.grow_tree(grad, rows, js, mode=1)
        assert_tree_bits(t_gpu, t_fx)
        o.predict_tree(t_fx, pred)
    assert np.array_equal(h.get_pred().view(np.uint32), pred.view(np.uint32))
    # the fit explains both targets down to their noise (uniform, variance 1/12 of 0.132 in total)
    assert ((pred - y) ** 2).mean(axis=0).max() < 0.7 * y.var(axis=0).min()
    h.close()
    o.close()


def test_multi_target_limits(evt):
    with pytest.raises(evt.EvtError):
        evt.Handle(100, 3, 8, 17, 3, "mse")  # more than 16 outputs
    with pytest.raises(evt.EvtError):
        evt.Handle(100, 3, 8, 3, 3, "gaussian_mle")  # two outputs per target
    h = evt.Handle(100, 3, 8, 2, 3, "mse")
    with pytest.raises(evt.EvtError, match="more than one target"):
        h.set_feature_meta(None, np.array([1, 0, 0], np.int32))
    h.set_feature_meta(None, np.zeros(3, np.int32))
    h.close()


def test_multi_target_fit_as_the_reference_tests_it(evt):
    """test/multi-target.jl through the host mirror: two targets on one feature, every in-scope loss; predictions come
    back as nobs x outputs, finite, and each target's squared error is below 90 % of its variance; the scale columns of
    gaussian_mle are positive; an eval set with a matrix target feeds the logger."""
    rng = np.random.default_rng(123)
    nobs = 10_000
    x_num = rng.random(nobs) * 5
    sig = lambda z: 1 / (1 + np.exp(-z))
    logit = lambda p: np.log(p / (1 - p))
    y1 = sig(logit(np.sin(x_num) * 0.5 + 0.5) + rng.standard_normal(nobs) * 0.5)
    y2 = sig(logit(np.sin(2 * x_num - 2) * 0.5 + 0.5) + rng.standard_normal(nobs) * 0.5)
    idx = rng.permutation(nobs)
    tr, ev = idx[:8000], idx[8000:]
    X = x_num.reshape(-1, 1)
    Y = np.stack([y1, y2])  # targets x observations
    base = (y1[tr].var(), y2[tr].var())
    for loss in ("mse", "logloss", "gamma", "poisson", "tweedie"):
        cfg = evt.EvoTreeRegressor(loss=loss, nrounds=200, nbins=64, L2=0.1, gamma=0.05, eta=0.05, max_depth=6, min_weight=1.0,
                                   rowsample=0.5, seed=123)
        # The gamma deviance has hessian 2y / pred: with targets down to 1e-8 (the troughs of the sines) the first tree's leaf
        # there is -0.05 * n / (sum(y) / mean(y) + 0.05) ~ -70, after which those rows' gradients (~1e28) swamp every node total
        # and the trees stop splitting - in Float64 row-order arithmetic (the oracle's mode 0) just as on the device.  The
        # gamma case therefore runs on the targets shifted away from zero.
        shift = 0.25 if loss == "gamma" else 0.0
        m = evt.fit(cfg, x_train=X[tr], y_train=Y[:, tr] + shift, x_eval=X[ev], y_eval=Y[:, ev] + shift, verbosity=0)
        logger = m.info["logger"]
        pred = m(X[tr]) - shift
        assert pred.shape == (8000, 2) and np.isfinite(pred).all()
        assert np.mean((pred[:, 0] - y1[tr]) ** 2) < base[0] * 0.9, loss
        assert np.mean((pred[:, 1] - y2[tr]) ** 2) < base[1] * 0.9, loss
        assert len(logger["metrics"]) == 201 and logger["metrics"][-1] < logger["metrics"][0]
    cfg = evt.EvoTreeMLE(nrounds=200, nbins=64, L2=0.1, gamma=0.05, eta=0.05, max_depth=6, min_weight=1.0, rowsample=0.5, seed=123)
    m = evt.fit(cfg, x_train=X[tr], y_train=Y[:, tr])
    pred = m(X[tr])
    assert pred.shape == (8000, 4) and np.isfinite(pred).all()
    assert (pred[:, 1] > 0).all() and (pred[:, 3] > 0).all()
    assert np.mean((pred[:, 0] - y1[tr]) ** 2) < base[0] * 0.9
    assert np.mean((pred[:, 2] - y2[tr]) ** 2) < base[1] * 0.9
    with pytest.raises(RuntimeError, match="Multi-target"):
        evt.fit(evt.EvoTreeClassifier(nrounds=2), x_train=X[tr], y_train=(Y[:, tr] > 0.5).astype(np.int64))


def test_multi_target_mle_eval_offset(evt):
    """test/multi-target.jl:57-77: every scale column of an offset is unconstrained, not only the second one."""
    n = 200
    rng = np.random.default_rng(9)
    x = rng.random((n, 1))
    Y = np.stack([rng.random(n), rng.random(n)])
    s1, s2 = 1.2, 1.5
    off = np.column_stack([np.full(n, 0.1), np.full(n, s1), np.full(n, -0.2), np.full(n, s2)])
    cfg = evt.EvoTreeMLE(nrounds=0, max_depth=3, metric="gaussian_mle")
    m = evt.fit(cfg, x_train=x, y_train=Y, offset_train=off.copy())
    cb = evt.CallBack(cfg, m, x, Y, offset_eval=off.copy())
    p = cb.handle.get_pred()
    inv = lambda s: s + np.log(-np.expm1(-s))
    assert abs(p[0, 1] - inv(s1)) < 1e-5 and abs(p[0, 3] - inv(s2)) < 1e-5
    assert abs(p[0, 0] - 0.1) < 1e-6 and abs(p[0, 2] + 0.2) < 1e-6
    cb.close()
    off1 = np.column_stack([np.full(n, 0.1), np.full(n, s1)])
    m1 = evt.fit(cfg, x_train=x, y_train=Y[0], offset_train=off1.copy())
    cb1 = evt.CallBack(cfg, m1, x, Y[0], offset_eval=off1.copy())
    assert abs(cb1.handle.get_pred()[0, 1] - inv(s1)) < 1e-5
    cb1.close()
