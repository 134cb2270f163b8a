"""Host-side handling of Tables input (no GPU): feature typing, edges and binning follow src/fit-utils.jl:26-92."""
import numpy as np
import pandas as pd
import pytest


def _frame(n=3000, seed=0):
    rng = np.random.default_rng(seed)
    return pd.DataFrame({
        "num": rng.standard_normal(n),
        "flag": rng.random(n) > 0.3,
        "cat": pd.Categorical(rng.choice(["red", "green", "blue", "grey", "pink"], n)),
        "ord": pd.Categorical(rng.choice(["s", "m", "l", "xl"], n), categories=["s", "m", "l", "xl"], ordered=True),
        "count": rng.integers(0, 4, n),
        "y": rng.random(n),
        "w": rng.random(n) + 0.5,
    })


def test_feature_types_edges_and_bins(evt):
    df = _frame()
    names = ["num", "flag", "cat", "ord", "count"]
    edges, featbins, feattypes = evt.get_edges_table(df, names, 16, np.random.default_rng(1))
    # Real -> `<=` on unique quantiles; Bool and unordered levels -> `==`; ordered levels -> `<=`
    assert feattypes.tolist() == [1, 0, 0, 1, 1]
    assert featbins.tolist() == [16, 2, 5, 4, len(edges[4]) + 1]
    assert list(edges[1]) == [False, True] and list(edges[2]) == list(df["cat"].cat.categories) and list(edges[3]) == ["s", "m", "l", "xl"]
    assert len(edges[4]) <= 4 and np.all(np.diff(edges[4]) > 0)  # unique(): four distinct values cannot give 15 distinct quantiles
    x_bin = evt.binarize_table(df, names, edges)
    assert x_bin.shape == (5, len(df)) and x_bin.dtype == np.uint8
    assert np.array_equal(x_bin[1], df["flag"].to_numpy().astype(np.uint8) + 1)          # col .+ 1
    assert np.array_equal(x_bin[2], df["cat"].cat.codes.to_numpy() + 1)                   # levelcode
    assert np.array_equal(x_bin[3], df["ord"].cat.codes.to_numpy() + 1)
    assert np.array_equal(x_bin[0], np.searchsorted(edges[0], df["num"].to_numpy(), side="left") + 1)  # searchsortedfirst
    assert x_bin.min() >= 1 and (x_bin.max(axis=1) <= featbins).all()
    # a frame whose categorical column lists its levels in another order is coded by the TRAINING levels
    df2 = df.copy()
    df2["cat"] = df2["cat"].cat.reorder_categories(["pink", "grey", "blue", "green", "red"])
    assert np.array_equal(evt.binarize_table(df2, names, edges), x_bin)
    # a dict of columns is a table too
    assert np.array_equal(evt.binarize_table({k: df[k] for k in df.columns}, names, edges), x_bin)


def test_table_errors(evt):
    df = _frame(500)
    with pytest.raises(RuntimeError, match="Max categorical levels"):
        evt.get_edges_table(df, ["cat"], 4, np.random.default_rng(0))
    df["txt"] = "a"
    with pytest.raises(RuntimeError, match="Invalid feature eltype"):
        evt.get_edges_table(df, ["txt"], 8, np.random.default_rng(0))
    edges, _, _ = evt.get_edges_table(df, ["cat"], 8, np.random.default_rng(0))
    bad = df.copy()
    bad["cat"] = pd.Categorical(["violet"] * len(bad))
    with pytest.raises(RuntimeError, match="not trained on"):
        evt.binarize_table(bad, ["cat"], edges)
    # default feature set: every Real / Bool / categorical column but the target, the weight and the offset
    from evotrees_jl_amd import _table_features
    assert _table_features(df, ["y"], "w", None, None) == ["num", "flag", "cat", "ord", "count"]
