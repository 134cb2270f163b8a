"""GPU parity tests of the rows next to the tree builder: the eval CallBack's metric on the device,
the logger / early stopping driven by it, the exp-link losses end to end, and inference from raw
Float64 features (device binarize + traversal)."""
import numpy as np
import pytest

from oracle import oracle as orc
from test_gpu_parity import RTOL, make_data, setup_pair

pytestmark = pytest.mark.gpu

METRICS_OF = {
    "mse": ["mse", "rmse", "mae"],
    "logloss": ["logloss", "mse"],
    "gaussian_mle": ["gaussian_mle"],
    "logistic_mle": ["logistic_mle"],
    "poisson": ["poisson", "mae"],
    "gamma": ["gamma"],
    "tweedie": ["tweedie", "rmse"],
    "mlogloss": ["mlogloss"],
    "quantile": ["quantile", "mae", "mse"],
    "multiquantile": ["multiquantile"],
}


@pytest.mark.parametrize("loss,weights", [("mse", True), ("logloss", False), ("gaussian_mle", True), ("poisson", True),
                                          ("gamma", False), ("tweedie", True), ("mlogloss", True), ("logistic_mle", True),
                                          ("quantile", True), ("multiquantile", False)])
def test_eval_metric_matches_oracle(evt, loss, weights):
    N, F, B, D = 70001, 6, 32, 4
    x_bin, y, w, mu = make_data(41, N, F, B, loss, weights)
    if loss == "poisson":
        y = y + 1.0  # the metric's log(y / pred + eps) amplifies ulp differences of exp at y = 0; covered separately below
    pk = dict(min_weight=8.0) if loss in ("gaussian_mle", "logistic_mle") else {}
    h, o, op, gp, pred0, grad0 = setup_pair(evt, loss, x_bin, y, w, mu, B, D, **pk)
    js = np.arange(1, F + 1, dtype=np.uint32)
    for r in range(3):
        h.update_grads()
        h.grow_tree(js, gp)
        pred = h.get_pred()
        for metric in METRICS_OF[loss]:
            got = h.eval_metric(metric)
            want = orc.eval_metric(metric, op.K, pred, y, w, alphas=list(op.alphas[:op.n_alphas]))
            exact_rows = metric in ("mse", "rmse", "mae")  # per-row Float32 values identical, only the Float64 sum order differs
            np.testing.assert_allclose(got, want, rtol=1e-12 if exact_rows else RTOL)
            assert got == h.eval_metric(metric)  # fixed summation order: reproducible to the bit
    if loss != "multiquantile":
        with pytest.raises(evt.EvtError):
            h.eval_metric("multiquantile")
    if loss not in ("gaussian_mle", "mlogloss", "logistic_mle"):
        with pytest.raises(evt.EvtError):
            h.eval_metric("gaussian_mle")
        with pytest.raises(evt.EvtError):
            h.eval_metric("logistic_mle")
        with pytest.raises(evt.EvtError):
            h.eval_metric("mlogloss")
    else:
        with pytest.raises(evt.EvtError):
            h.eval_metric("mse")
    h.close()
    o.close()


def test_poisson_metric_with_zero_counts(evt):
    N, F, B = 5000, 3, 8
    x_bin, y, w, mu = make_data(42, N, F, B, "poisson", False)
    assert (y == 0).any()
    h, o, op, gp, pred0, grad0 = setup_pair(evt, "poisson", x_bin, y, w, mu, B, 3)
    got = h.eval_metric("poisson")
    want = orc.eval_metric("poisson", 1, pred0, y, None)
    np.testing.assert_allclose(got, want, rtol=1e-4)
    h.close()
    o.close()


def test_eval_metric_small_and_state_errors(evt):
    h = evt.Handle(3, 1, 4, 1, 2, "mse")
    with pytest.raises(evt.EvtError) as ei:
        h.eval_metric("mse")
    assert ei.value.code == evt._lib.EVT_ERR_STATE
    h.set_target(np.float32([1, 2, 4]), np.float32([1, 1, 2]), np.float32([1.0]))
    assert h.eval_metric("mse") == (0 + 1 + 2 * 9) / 4
    assert h.eval_metric("rmse") == np.sqrt(19 / 4)
    assert h.eval_metric("mae") == (0 + 1 + 2 * 3) / 4
    h.close()


def _sinus(rng, n):
    feats = rng.random(n) * 5
    Y = np.sin(feats) * 0.5 + 0.5
    Y = 1 / (1 + np.exp(-(np.log(Y / (1 - Y)) + rng.standard_normal(n))))
    return feats.reshape(-1, 1), Y


@pytest.mark.parametrize("cfg_kw", [dict(loss="mse", metric="mae"), dict(loss="logloss"), dict(loss="gamma"), dict(loss="tweedie"),
                                    dict(loss="poisson", learner="count"), dict(loss="gaussian_mle", learner="mle"),
                                    dict(loss="logistic_mle", learner="mle"), dict(loss="mae"), dict(loss="cred_var"),
                                    dict(loss="cred_std", metric="rmse"), dict(loss="quantile", alpha=0.8),
                                    dict(loss="multiquantile", alphas=[0.2, 0.5, 0.8])])
def test_fit_with_eval_logger_matches_oracle_replay(evt, cfg_kw):
    # every logged value equals the oracle's metric of the oracle's own replay of the model on the eval rows
    rng = np.random.default_rng(7)
    X, Y = _sinus(rng, 1200)
    tr, ev = np.arange(900), np.arange(900, 1200)
    kw = dict(cfg_kw)
    if kw["loss"] == "gamma":
        Y = Y + 0.5  # targets near zero make the first Newton steps of the gamma deviance overshoot
    learner = {"count": evt.EvoTreeCount, "mle": evt.EvoTreeMLE}.get(kw.pop("learner", None), evt.EvoTreeRegressor)
    cfg = learner(nrounds=12, nbins=16, eta=0.2, max_depth=4, **kw)
    w_ev = (rng.random(len(ev)) + 0.5).astype(np.float32)
    m = evt.fit(cfg, x_train=X[tr], y_train=Y[tr], x_eval=X[ev], y_eval=Y[ev], w_eval=w_ev, verbosity=0)
    lg = m.info["logger"]
    assert lg["name"] == cfg.metric and lg["iter"] == list(range(13)) and lg["nrounds"] == 12
    if cfg.loss in ("mae", "cred_var"):
        assert cfg.metric == "mae"  # the credibility losses are tracked by mae unless told otherwise (src/learners.jl:76-81)
    assert lg["maximise"] == (cfg.loss in ("gaussian_mle", "logistic_mle"))
    xb = evt.binarize(X[ev], m.info["edges"])
    ft = np.ones(1, np.uint8)
    p = np.zeros((len(ev), m.K), np.float32)
    y32 = Y[ev].astype(np.float32)
    for i, t in enumerate(m.trees):
        orc.predict_tree(orc.LOSS_IDS[cfg.loss], m.K, xb, ft, t, p)
        # a mean log-likelihood can pass through zero: the absolute bound is 1e-6 of the per-row values' scale (~1)
        al = list(cfg.alphas) if cfg.loss == "multiquantile" else [getattr(cfg, "alpha", 0.5)]
        np.testing.assert_allclose(lg["metrics"][i], orc.eval_metric(cfg.metric, m.K, p, y32, w_ev, alphas=al), rtol=RTOL, atol=1e-6)
    best = int(np.argmax(lg["metrics"]) if lg["maximise"] else np.argmin(lg["metrics"]))
    assert lg["best_iter"] == best and lg["best_metric"] == lg["metrics"][best]
    better = lg["metrics"][-1] > lg["metrics"][0] if lg["maximise"] else lg["metrics"][-1] < lg["metrics"][0]
    assert better


def test_early_stopping_and_offsets(evt):
    rng = np.random.default_rng(8)
    X, Y = _sinus(rng, 1000)
    tr, ev = np.arange(800), np.arange(800, 1000)
    noise = rng.random(len(ev))  # an eval target the model cannot learn: the metric stops improving at once
    cfg = evt.EvoTreeRegressor(nrounds=200, nbins=16, eta=0.5, max_depth=5, early_stopping_rounds=4)
    m = evt.fit(cfg, x_train=X[tr], y_train=Y[tr], x_eval=X[ev], y_eval=noise, verbosity=0)
    lg = m.info["logger"]
    assert lg["nrounds"] < 200 and lg["iter_since_best"] == 4 and lg["nrounds"] == lg["best_iter"] + 4
    assert len(m.trees) == lg["nrounds"] + 1
    # tolerance: an improvement smaller than the tolerance does not count
    cfg2 = evt.EvoTreeRegressor(nrounds=50, nbins=16, eta=0.1, max_depth=4, early_stopping_rounds=3, early_stopping_tolerance=1e9)
    m2 = evt.fit(cfg2, x_train=X[tr], y_train=Y[tr], x_eval=X[ev], y_eval=Y[ev], verbosity=0)
    assert m2.info["logger"]["nrounds"] == 3 and m2.info["logger"]["best_iter"] == 0
    # offsets: given on the response scale, moved to the linear one on both the training and the eval side
    off_tr = np.full(len(tr), 0.5, np.float32)
    off_ev = np.full(len(ev), 0.5, np.float32)
    cfg3 = evt.EvoTreeRegressor(loss="poisson", nrounds=3, nbins=16, max_depth=3)
    m3 = evt.fit(cfg3, x_train=X[tr], y_train=Y[tr], offset_train=off_tr, x_eval=X[ev], y_eval=Y[ev], offset_eval=off_ev, verbosity=0)
    assert np.all(m3.trees[0].pred == 0)  # neutral bias with an offset
    p0 = np.full((len(ev), 1), np.log(np.float32(0.5)), np.float32)
    np.testing.assert_allclose(m3.info["logger"]["metrics"][0], orc.eval_metric("poisson", 1, p0, Y[ev].astype(np.float32)), rtol=RTOL)
    # only one of x_eval / y_eval: no logger, a warning
    with pytest.warns(UserWarning):
        m4 = evt.fit(evt.EvoTreeRegressor(nrounds=2, max_depth=2), x_train=X[tr], y_train=Y[tr], x_eval=X[ev], verbosity=0)
    assert m4.info["logger"] is None


@pytest.mark.parametrize("N,F", [((1 << 22) + 12345, 3), (700001, 7)])
def test_predict_f64_equals_host_binarize_then_predict(evt, N, F):
    # the Float64 matrix goes up in pieces of 2^22 values: a long column is cut into row ranges (first shape: two pieces per
    # column, more pieces than upload buffers), short columns share a piece (second shape: five columns, then two); ragged
    # edge counts
    rng = np.random.default_rng(9)
    X = rng.standard_normal((N, F))
    edges = [np.sort(rng.standard_normal(k)) for k in (31, 1, 254, 7, 100, 2, 63)[:F]]
    X[:1000, 0] = edges[0][rng.integers(0, 31, 1000)]  # values equal to an edge fall in that edge's bin
    X[5, 1], X[6, 1] = np.inf, -np.inf
    X[N - 1, F - 1] = np.nan
    xb = evt.binarize(X, edges)
    trees = []
    K = 1
    for s in range(4):
        t = orc.Tree(K, 7)
        t.feat[:3] = rng.integers(1, F + 1, 3)
        t.cond_bin[:3] = [rng.integers(1, len(edges[f - 1]) + 1) for f in t.feat[:3]]
        t.split[:3] = 1
        t.pred[3:, 0] = rng.standard_normal(4).astype(np.float32)
        trees.append(t)
    ft = np.ones(F, np.uint8)
    for loss, link in (("mse", True), ("gamma", True), ("logloss", False)):
        want = evt._lib.predict_model(xb, ft, loss, K, trees, apply_link=link)
        got = evt._lib.predict_model_f64(np.ascontiguousarray(X.T), edges, ft, loss, K, trees, apply_link=link)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    with pytest.raises(evt.EvtError):
        evt._lib.predict_model_f64(np.ascontiguousarray(X[:10].T), [np.zeros(0)] * F, ft, "mse", K, trees)
    # the training cache takes the same way up: evt_binarize_f64 leaves the bins the host computes
    h = evt.Handle(N, F, 255, 1, 2, "mse")
    h.binarize(np.ascontiguousarray(X.T), edges)
    assert np.array_equal(h.get_xbin(), xb)
    h.close()


def test_classifier_fit_levels_logger_and_errors(evt):
    # three classes cut from a noisy function of two features; labels are strings, levels are sorted(unique)
    rng = np.random.default_rng(10)
    N = 3000
    X = rng.random((N, 4))
    score = X[:, 0] + 0.5 * X[:, 1] + 0.05 * rng.standard_normal(N)
    lab = np.where(score < 0.5, "low", np.where(score < 0.95, "mid", "top"))
    tr, ev = np.arange(2400), np.arange(2400, N)
    cfg = evt.EvoTreeClassifier(nrounds=30, nbins=32, eta=0.3, max_depth=4)
    m = evt.fit(cfg, x_train=X[tr], y_train=lab[tr], x_eval=X[ev], y_eval=lab[ev], verbosity=0)
    assert m.K == 3 and list(m.info["target_levels"]) == ["low", "mid", "top"]
    # bias: log(proportions) shifted by its maximum (src/init.jl:63-64)
    prop = np.array([(lab[tr] == l).mean() for l in ("low", "mid", "top")])
    np.testing.assert_allclose(m.trees[0].pred[0], np.log(prop) - np.log(prop).max(), rtol=1e-6, atol=1e-7)
    p = m(X[ev])
    assert p.shape == (len(ev), 3)
    np.testing.assert_allclose(p.sum(axis=1), 1.0, rtol=1e-5)
    acc = (np.array(["low", "mid", "top"])[p.argmax(axis=1)] == lab[ev]).mean()
    assert acc > 0.8, acc
    lg = m.info["logger"]
    assert lg["name"] == "mlogloss" and lg["metrics"][-1] < 0.6 * lg["metrics"][0]
    # the logged values equal the oracle's metric of the oracle's replay
    xb = evt.binarize(X[ev], m.info["edges"])
    codes = np.searchsorted(np.array(["low", "mid", "top"]), lab[ev]).astype(np.float32) + 1
    pr = np.zeros((len(ev), 3), np.float32)
    for i, t in enumerate(m.trees):
        orc.predict_tree(orc.LOSS_IDS["mlogloss"], 3, xb, np.ones(4, np.uint8), t, pr)
        np.testing.assert_allclose(lg["metrics"][i], orc.eval_metric("mlogloss", 3, pr, codes), rtol=RTOL)
    # an eval set with a level the model never saw is an error, as is a single-class or a Float target
    bad = lab[ev].copy()
    bad[0] = "unseen"
    with pytest.raises(RuntimeError, match="absent from `y_train`"):
        evt.fit(evt.EvoTreeClassifier(nrounds=1), x_train=X[tr], y_train=lab[tr], x_eval=X[ev], y_eval=bad, verbosity=0)
    with pytest.raises(RuntimeError, match="at least 2 levels"):
        evt.fit(evt.EvoTreeClassifier(nrounds=1), x_train=X[:50], y_train=np.array(["a"] * 50))
    with pytest.raises(RuntimeError, match="Invalid target eltype"):
        evt.fit(evt.EvoTreeClassifier(nrounds=1), x_train=X[:50], y_train=X[:50, 0])
    # class codes outside 1..K and monotone constraints are refused by the library itself
    h = evt.Handle(10, 2, 8, 3, 2, "mlogloss")
    with pytest.raises(evt.EvtError):
        h.set_target(np.float32([1, 2, 3, 4, 1, 2, 3, 1, 2, 3]), None, np.zeros(3, np.float32))
    with pytest.raises(evt.EvtError):
        h.set_target(np.float32([1, 2, 2.5, 3, 1, 2, 3, 1, 2, 3]), None, np.zeros(3, np.float32))
    with pytest.raises(evt.EvtError):
        h.set_feature_meta(None, np.int32([1, 0]))
    h.close()
    with pytest.raises(evt.EvtError):
        evt.Handle(10, 2, 8, 17, 2, "mlogloss")


@pytest.mark.parametrize("kw", [dict(rowsample=0.6, colsample=0.5), dict(bagging_size=3, rowsample=0.8), dict()])
def test_fit_running_one_tree_ahead_equals_fit_in_turn(evt, kw):
    # without an eval set the device is given the next tree before the last one is collected (two trees in flight, also
    # across rounds); with one, every tree is collected before the next call.  Same generator draws, same trees.
    rng = np.random.default_rng(3)
    X = rng.random((4000, 6))
    Y = X[:, 0] * 2 + np.sin(6 * X[:, 1]) + 0.1 * rng.standard_normal(4000)
    cfg = evt.EvoTreeRegressor(nrounds=9, nbins=32, eta=0.3, max_depth=5, seed=42, **kw)
    m_ahead = evt.fit(cfg, x_train=X, y_train=Y)
    m_turn = evt.fit(cfg, x_train=X, y_train=Y, x_eval=X[:500], y_eval=Y[:500], verbosity=0)
    assert len(m_ahead.trees) == len(m_turn.trees) == 1 + 9 * cfg.bagging_size
    for a, b in zip(m_ahead.trees, m_turn.trees):
        for name in ("feat", "cond_bin", "split", "w", "gain", "pred"):
            assert getattr(a, name).tobytes() == getattr(b, name).tobytes(), name


def test_update_continues_on_the_kept_handle(evt):
    # MMI.update (src/MLJ.jl:38-57): only a larger nrounds continues; the result equals a single longer fit
    rng = np.random.default_rng(11)
    X, Y = _sinus(rng, 600)
    kw = dict(nbins=16, eta=0.2, max_depth=4, rowsample=0.7, colsample=1.0, seed=5)
    m, cache = evt.fit(evt.EvoTreeRegressor(nrounds=5, **kw), x_train=X, y_train=Y, return_cache=True)
    m, cache = evt.update(evt.EvoTreeRegressor(nrounds=12, **kw), m, cache)
    assert m.info["nrounds"] == 12 and len(m.trees) == 13
    m_ref = evt.fit(evt.EvoTreeRegressor(nrounds=12, **kw), x_train=X, y_train=Y)
    assert np.array_equal(m(X), m_ref(X))
    assert not evt.okay_to_continue(evt.EvoTreeRegressor(nrounds=20, **dict(kw, eta=0.1)), m, cache)
    assert not evt.okay_to_continue(evt.EvoTreeRegressor(nrounds=3, **kw), m, cache)
    m2, cache2 = evt.update(evt.EvoTreeRegressor(nrounds=4, **dict(kw, eta=0.1)), m, cache, x_train=X, y_train=Y)
    assert m2.info["nrounds"] == 4 and len(m2.trees) == 5
    cache2.handle.close()
