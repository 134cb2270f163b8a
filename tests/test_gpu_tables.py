"""fit / predict on Tables input through the host mirror: Bool and categorical columns reach the kernels' `==` splits,
ordered levels and Real columns the `<=` ones (src/fit-utils.jl:26-92, src/fit.jl:302-345, src/callback.jl:31-80)."""
import numpy as np
import pandas as pd
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def _frame(n, seed):
    rng = np.random.default_rng(seed)
    cat = rng.choice(["red", "green", "blue", "grey", "pink"], n)
    flag = rng.random(n) > 0.4
    num = rng.standard_normal(n)
    ordl = rng.choice(["s", "m", "l", "xl"], n)
    y = (2.0 * (cat == "blue") - 1.0 * (cat == "red") + 0.7 * flag + 0.5 * np.tanh(num) + 0.3 * np.isin(ordl, ["l", "xl"]) + 0.05 * rng.standard_normal(n))
    return pd.DataFrame({"num": num, "flag": flag, "cat": pd.Categorical(cat), "noise": rng.random(n),
                         "ord": pd.Categorical(ordl, categories=["s", "m", "l", "xl"], ordered=True), "y": y.astype(np.float32),
                         "w": (rng.random(n) + 0.5).astype(np.float32)})


def test_fit_on_a_table_with_categorical_features(evt):
    dtrain, deval = _frame(40000, 1), _frame(8000, 2)
    cfg = evt.EvoTreeRegressor(nrounds=30, max_depth=5, nbins=32, eta=0.3, early_stopping_rounds=10)
    m = evt.fit(cfg, dtrain=dtrain, target_name="y", weight_name="w", deval=deval, verbosity=0)
    names = m.info["feature_names"]
    assert names == ["num", "flag", "cat", "noise", "ord"] and m.info["target_names"] == ["y"]
    assert m.info["feattypes"].tolist() == [1, 0, 0, 1, 1] and m.info["featbins"].tolist() == [32, 2, 5, 32, 4]
    # the unordered levels are separated by `==` splits: "blue" (level code 1) and "red" (4) carry the largest effects
    cat_splits = [(int(t.cond_bin[n]),) for t in m.trees[1:] for n in np.flatnonzero(t.split) if t.feat[n] == 3]
    assert len(cat_splits) >= 10
    assert {1, 4} <= {c[0] for c in cat_splits}
    assert any(t.feat[n] == 2 for t in m.trees[1:] for n in np.flatnonzero(t.split))  # the Bool column
    # eval metric from the device, through the Tables CallBack: weighted mse falls by more than 90 %
    lg = m.info["logger"]
    assert lg["metrics"][-1] < 0.1 * lg["metrics"][0]
    # predictions: the device walk of the host-binned table equals the oracle's walk of the same trees
    x_bin = evt.binarize_table(deval, names, m.info["edges"])
    want = np.zeros((len(deval), 1), np.float32)
    for t in m.trees:
        orc.predict_tree(orc.LOSS_IDS["mse"], 1, x_bin, m.info["feattypes"], t, want)
    got = evt.predict(m, deval)
    assert np.array_equal(got, want[:, 0])
    assert np.array_equal(m(deval), got)  # the functor
    mse = float(np.mean((got - deval["y"].to_numpy()) ** 2))
    assert mse < 0.05 * float(np.var(deval["y"].to_numpy()))
    leaves = evt.predict_leaf_idx(m, deval, ntree_limit=5)
    for j in range(5):
        assert np.array_equal(leaves[:, j], orc.predict_leaf_idx(x_bin, m.info["feattypes"], m.trees[j]))
    # a dict of columns trains the same model (same seed, same host RNG stream)
    m2 = evt.fit(cfg, dtrain={k: dtrain[k] for k in dtrain.columns}, target_name="y", weight_name="w", verbosity=0)
    for a, b in zip(m.trees[:6], m2.trees[:6]):
        assert np.array_equal(a.feat, b.feat) and np.array_equal(a.cond_bin, b.cond_bin) and np.array_equal(a.pred, b.pred)
