"""Pins the CPU oracle (oracle/evo_oracle.c) without running the reference.

The reference holds no golden vectors for this path (its tests are behavioural), so the
oracle is anchored on: brute-force numpy re-derivations on small inputs (tests/brute.py),
closed forms, the invariants the reference's own tests state (test/predict-leaf-idx.jl:25-49,
test/metrics.jl:160-204, docs/src/overview.md tie rule) and hand-built edge cases chosen so
that a dropped term, a wrong inequality or a transposed index fails.
"""
import numpy as np
import pytest

import brute
from oracle import oracle as orc


def make_data(seed, N, F, nbins, loss="mse", weights=False):
    rng = np.random.default_rng(seed)
    x_bin = rng.integers(1, nbins + 1, size=(F, N), dtype=np.uint8)
    K = 2 if loss == "gaussian_mle" else (3 if loss == "mlogloss" else 1)
    NK = 2 * K + 1
    y = rng.random(N).astype(np.float32)
    if loss == "logloss":
        y = (y > 0.5).astype(np.float32)
    elif loss == "mlogloss":
        y = (np.floor(y * K) + 1).astype(np.float32)  # 1-based class
    pred = (rng.standard_normal((N, K)) * 0.3).astype(np.float32)
    grad = np.zeros((N, NK), np.float32)
    grad[:, NK - 1] = (rng.random(N).astype(np.float32) + 0.5) if weights else 1.0
    return x_bin, y, pred, grad


def trees_equal_struct(t, T):
    return (np.array_equal(t.feat, T["feat"]) and np.array_equal(t.cond_bin, T["cond_bin"])
            and np.array_equal(t.split, T["split"]))


# ---------------------------------------------------------------- gradients
def test_grads_mse_closed_form():
    x_bin, y, pred, grad = make_data(1, 500, 3, 8, weights=True)
    p = orc.make_params("mse")
    w = grad[:, 2].copy()
    orc.update_grads(p, pred, y, grad)
    assert np.array_equal(grad[:, 0], (np.float32(2) * (pred[:, 0] - y)) * w)
    assert np.array_equal(grad[:, 1], np.float32(2) * w)
    assert np.array_equal(grad[:, 2], w)  # the weight row is only read


def test_grads_logloss_vs_float64():
    x_bin, y, pred, grad = make_data(2, 500, 3, 8, loss="logloss", weights=True)
    p = orc.make_params("logloss")
    w = grad[:, 2].astype(np.float64)
    orc.update_grads(p, pred, y, grad)
    s = 1.0 / (1.0 + np.exp(-pred[:, 0].astype(np.float64)))
    np.testing.assert_allclose(grad[:, 0], (s - y) * w, rtol=0, atol=2e-7)
    np.testing.assert_allclose(grad[:, 1], s * (1 - s) * w, rtol=2e-6)


def test_grads_gaussian_fisher_and_finite_difference():
    # test/metrics.jl:160-204: -d(logpdf)/d(loc) == g1, -d(logpdf)/d(raw) == g2, Fisher hessians
    # 1/scale^2 and 2 (sigmoid(raw)/scale)^2 do not depend on the residual; link is softplus.
    def lpdf(yv, loc, raw):
        scale = np.log1p(np.exp(raw))
        return -(np.log(scale) + (yv - loc) ** 2 / (2 * scale ** 2))

    p = orc.make_params("gaussian_mle")
    cases = [(0.5, 0.3, 1.5), (0.5, 0.3, 4.0), (-1.0, -0.7, -3.0), (0.0, 1.2, 0.0)]
    N = len(cases)
    pred = np.array([[c[0], c[1]] for c in cases], np.float32)
    y = np.array([c[2] for c in cases], np.float32)
    grad = np.zeros((N, 5), np.float32)
    grad[:, 4] = 1.0
    orc.update_grads(p, pred, y, grad)
    h = 1e-6
    for i, (loc, raw, yv) in enumerate(cases):
        loc, raw, yv = float(np.float32(loc)), float(np.float32(raw)), float(np.float32(yv))
        dloc = (lpdf(yv, loc + h, raw) - lpdf(yv, loc - h, raw)) / (2 * h)
        draw = (lpdf(yv, loc, raw + h) - lpdf(yv, loc, raw - h)) / (2 * h)
        assert abs(-dloc - grad[i, 0]) < 2e-5 * max(1, abs(dloc))
        assert abs(-draw - grad[i, 1]) < 2e-5 * max(1, abs(draw))
        scale = np.log1p(np.exp(raw))
        ds = 1 / (1 + np.exp(-raw))
        np.testing.assert_allclose(grad[i, 2], 1 / scale ** 2, rtol=1e-5)
        np.testing.assert_allclose(grad[i, 3], 2 * (ds / scale) ** 2, rtol=1e-5)
    # cases 0 and 1 share (loc, raw): hessians identical although residuals differ
    assert grad[0, 2] == grad[1, 2] and grad[0, 3] == grad[1, 3]


def test_grads_gaussian_weight_scales_all_rows():
    p = orc.make_params("gaussian_mle")
    pred = np.array([[0.2, -0.4]] * 2, np.float32)
    y = np.array([1.0, 1.0], np.float32)
    grad = np.zeros((2, 5), np.float32)
    grad[:, 4] = [1.0, 3.0]
    orc.update_grads(p, pred, y, grad)
    np.testing.assert_allclose(grad[1, :4], 3 * grad[0, :4], rtol=1e-6)


# ---------------------------------------------------------------- binarize / subsample
def test_binarize_searchsortedfirst():
    rng = np.random.default_rng(3)
    edges = np.sort(rng.random(15))
    x = np.concatenate([rng.random(200), edges, [-1.0, 2.0]])  # values equal to an edge go to that edge's bin
    got = orc.binarize(x, edges)
    want = np.searchsorted(edges, x, side="left") + 1
    assert np.array_equal(got, want.astype(np.uint8))
    assert got.min() >= 1 and got.max() <= 16


def test_binarize_orders_values_as_julia_isless():
    """searchsortedfirst's default order is isless (src/fit-utils.jl:69 passes none): NaN after everything, Inf included,
    and -0.0 before 0.0.  Known answers worked by hand from that definition, and numpy's own NaN-last ordering."""
    edges = np.array([-1.0, -0.0, 0.0, 1.0])
    x = np.array([-np.inf, -1.0, -0.5, -0.0, 0.0, 0.5, 1.0, 2.0, np.inf, np.nan])
    #             first index whose edge is not isless than x
    want = np.array([1, 1, 2, 2, 3, 4, 4, 5, 5, 5], np.uint8)
    assert np.array_equal(orc.binarize(x, edges), want)
    rng = np.random.default_rng(5)
    e2 = np.sort(rng.standard_normal(31))
    x2 = rng.standard_normal(500)
    x2[::7] = np.nan
    assert np.array_equal(orc.binarize(x2, e2), (np.searchsorted(e2, x2, side="left") + 1).astype(np.uint8))
    assert (orc.binarize(x2, e2)[::7] == 32).all()


def test_subsample_threshold_rule():
    mask = np.arange(256, dtype=np.uint8)
    # src/subsample.jl:9: cond = round(UInt8, 255*rowsample), half-to-even: 0.5 -> 128
    cond = int(np.rint(255 * 0.5))
    assert cond == 128
    got = orc.subsample(mask, cond)
    assert np.array_equal(got, np.arange(129, dtype=np.uint32))
    assert orc.subsample(mask, 255).shape[0] == 256
    assert orc.subsample(np.full(10, 7, np.uint8), 3).shape[0] == 0


# ---------------------------------------------------------------- histogram
@pytest.mark.parametrize("loss,weights", [("mse", False), ("mse", True), ("logloss", True), ("gaussian_mle", False)])
def test_hist_against_dense_bruteforce_and_invariants(loss, weights):
    N, F, B, D = 700, 5, 8, 4
    x_bin, y, pred, grad = make_data(10, N, F, B, loss, weights)
    p = orc.make_params(loss, nbins=B, max_depth=D, min_weight=1.0)
    orc.update_grads(p, pred, y, grad)
    rng = np.random.default_rng(11)
    rows = np.sort(rng.choice(N, 500, replace=False)).astype(np.uint32)
    js = np.array([1, 2, 4, 5], np.uint32)
    o = orc.Oracle(p, x_bin)
    t, nidx = o.grow_tree(grad, rows, js, mode=0)
    H = o.hist()
    S = o.node_sums()
    K, NK = p.K, 2 * p.K + 1
    # walk the tree the oracle produced; every split node's histogram must equal the dense one of its rows
    label = np.zeros(N, np.int64)
    label[rows] = 1
    checked = 0
    for n in range(1, 2 ** (D - 1)):
        if not t.split[n - 1]:
            continue
        r = np.flatnonzero(label == n)
        dense = brute.dense_hist(x_bin, grad, r, B)
        for j in js:
            np.testing.assert_allclose(H[n - 1, j - 1], dense[j - 1], rtol=1e-12, atol=1e-12)
            # sum over bins == node sums, for every sampled feature
            np.testing.assert_allclose(H[n - 1, j - 1].sum(axis=0), S[n], rtol=1e-11, atol=1e-11)
            if not weights:
                cnt = np.bincount(x_bin[j - 1, r].astype(np.int64) - 1, minlength=B)
                assert np.array_equal(H[n - 1, j - 1][:, NK - 1], cnt.astype(np.float64))
        f, b = int(t.feat[n - 1]), int(t.cond_bin[n - 1])
        go = x_bin[f - 1, r] <= b
        label[r[go]] = 2 * n
        label[r[~go]] = 2 * n + 1
        checked += 1
        # parent == left + right wherever both children were scanned
        if 2 * n + 1 < 2 ** (D - 1) and (t.split[2 * n - 1] or t.split[2 * n]):
            for j in js:
                np.testing.assert_allclose(H[n - 1, j - 1], H[2 * n - 1, j - 1] + H[2 * n, j - 1], rtol=1e-11, atol=1e-11)
    assert checked >= 3
    o.close()


# ---------------------------------------------------------------- split search / full tree vs brute force
@pytest.mark.parametrize("loss,weights,lam,gamma,minw", [
    ("mse", False, 0.0, 0.0, 1.0),
    ("mse", True, 0.5, 0.1, 2.0),
    ("logloss", False, 0.0, 0.0, 1.0),
    ("logloss", True, 0.3, 0.0, 1.0),
    ("gaussian_mle", False, 0.0, 0.0, 8.0),
    ("gaussian_mle", True, 0.2, 0.05, 4.0),
    ("mlogloss", False, 0.0, 0.0, 1.0),
    ("mlogloss", True, 0.4, 0.02, 2.0),
])
def test_tree_against_bruteforce(loss, weights, lam, gamma, minw):
    N, F, B, D = 900, 6, 16, 5
    x_bin, y, pred, grad = make_data(20, N, F, B, loss, weights)
    p = orc.make_params(loss, nbins=B, max_depth=D, lambda_=lam, gamma=gamma, min_weight=minw, eta=0.3, K=pred.shape[1])
    orc.update_grads(p, pred, y, grad)
    rng = np.random.default_rng(21)
    rows = np.sort(rng.choice(N, 640, replace=False)).astype(np.uint32)
    js = np.array([1, 3, 4, 6], np.uint32)
    o = orc.Oracle(p, x_bin)
    t, nidx = o.grow_tree(grad, rows, js, mode=0)
    T, label, hists, sums = brute.grow(x_bin, grad, rows, js, p.K, B, D, eta=0.3, lam=lam, L2=1.0, gamma=gamma, min_weight=minw)
    assert trees_equal_struct(t, T)
    assert t.split.sum() >= 3
    np.testing.assert_allclose(t.gain, T["gain"], rtol=1e-5)
    np.testing.assert_allclose(t.pred, T["pred"], rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(t.w, T["w"], rtol=1e-6)
    assert np.array_equal(nidx.astype(np.int64), label)  # node each sampled row ends in; 0 for unsampled rows
    o.close()


def test_root_gain_closed_form_unit_weights():
    # w == 1, lambda == 0, mse => h = 2n: gain = GL^2/(2(2nL+L2)) + GR^2/(2(2nR+L2)) - G^2/(2(2n+L2))
    N, F, B = 400, 3, 8
    x_bin, y, pred, grad = make_data(30, N, F, B)
    p = orc.make_params("mse", nbins=B, max_depth=2, L2=1.0)
    orc.update_grads(p, pred, y, grad)
    rows = np.arange(N, dtype=np.uint32)
    js = np.arange(1, F + 1, dtype=np.uint32)
    o = orc.Oracle(p, x_bin)
    t, _ = o.grow_tree(grad, rows, js)
    g = grad[:, 0].astype(np.float64)
    best = (-1.0, 0, 0)
    for j in range(F):
        for b in range(1, B):
            L = x_bin[j] <= b
            nL, nR = L.sum(), N - L.sum()
            if not (nL > 1.0 and nR > 1.0):
                continue
            GL, GR, G = g[L].sum(), g[~L].sum(), g.sum()
            gain = GL ** 2 / (2 * (2 * nL + 1)) + GR ** 2 / (2 * (2 * nR + 1)) - G ** 2 / (2 * (2 * N + 1))
            if gain > best[0]:
                best = (gain, j + 1, b)
    assert (int(t.feat[0]), int(t.cond_bin[0])) == best[1:]
    np.testing.assert_allclose(t.gain[0], best[0], rtol=1e-6)
    # leaf value closed form and w == row count
    for child in (2, 3):
        sel = (x_bin[best[1] - 1] <= best[2]) if child == 2 else (x_bin[best[1] - 1] > best[2])
        assert t.w[child - 1] == sel.sum()
        np.testing.assert_allclose(t.pred[child - 1, 0], -0.1 * g[sel].sum() / (2 * sel.sum() + 1.0), rtol=1e-6)
    o.close()


def test_tie_rule_duplicate_columns_and_empty_bins():
    # "the first one will be selected": duplicated columns give identical gains -> earliest feature in js;
    # an empty bin repeats the previous cumulative sums -> identical gain -> lowest bin wins.
    N, B = 300, 16
    rng = np.random.default_rng(40)
    col = rng.integers(1, B + 1, N).astype(np.uint8)
    col[col == 7] = 8  # bin 7 empty: candidates at bin 6 and 7 have the same left set
    noise = rng.integers(1, B + 1, N).astype(np.uint8)
    x_bin = np.stack([noise, col, col.copy(), col.copy()])
    y = (col > 6).astype(np.float32) + 0.01 * rng.random(N).astype(np.float32)
    pred = np.zeros((N, 1), np.float32)
    grad = np.zeros((N, 3), np.float32)
    grad[:, 2] = 1
    p = orc.make_params("mse", nbins=B, max_depth=2)
    orc.update_grads(p, pred, y, grad)
    rows = np.arange(N, dtype=np.uint32)
    o = orc.Oracle(p, x_bin)
    t, _ = o.grow_tree(grad, rows, np.array([1, 2, 3, 4], np.uint32))
    assert (int(t.feat[0]), int(t.cond_bin[0])) == (2, 6)
    t, _ = o.grow_tree(grad, rows, np.array([1, 3, 4], np.uint32))
    assert (int(t.feat[0]), int(t.cond_bin[0])) == (3, 6)
    o.close()


def test_min_weight_is_strict_and_gamma_is_strict():
    # 4 rows, one feature: the only balanced split has w_l == w_r == 2.
    x_bin = np.array([[1, 1, 2, 2]], np.uint8)
    grad = np.array([[-1, 2, 1], [-1, 2, 1], [1, 2, 1], [1, 2, 1]], np.float32)
    rows = np.arange(4, dtype=np.uint32)
    js = np.array([1], np.uint32)
    for minw, expect in [(1.999, 1), (2.0, 0), (2.5, 0)]:
        p = orc.make_params("mse", nbins=4, max_depth=2, min_weight=minw)
        o = orc.Oracle(p, x_bin)
        t, _ = o.grow_tree(grad, rows, js)
        assert int(t.split[0]) == expect, minw
        o.close()
    # gain of that split: 2 * (2^2 / (4+1) / 2) - 0 = 0.8 ; accepted only if gain > gamma
    for gamma, expect in [(0.79, 1), (0.8, 0), (0.9, 0)]:
        p = orc.make_params("mse", nbins=4, max_depth=2, min_weight=1.0, gamma=gamma)
        o = orc.Oracle(p, x_bin)
        t, _ = o.grow_tree(grad, rows, js)
        assert int(t.split[0]) == expect, gamma
        if expect:
            np.testing.assert_allclose(t.gain[0], 0.8, rtol=1e-6)
        o.close()


def test_numeric_scan_excludes_last_bin_uses_nbins_param():
    # all rows in bins {B-1, B}: the only separating split is at bin B-1 (allowed, <= B-1)
    B = 8
    x_bin = np.array([[B - 1] * 5 + [B] * 5], np.uint8)
    grad = np.zeros((10, 3), np.float32)
    grad[:, 2] = 1
    grad[:, 1] = 2
    grad[:5, 0] = -1
    grad[5:, 0] = 1
    p = orc.make_params("mse", nbins=B, max_depth=2)
    o = orc.Oracle(p, x_bin)
    t, _ = o.grow_tree(grad, np.arange(10, dtype=np.uint32), np.array([1], np.uint32))
    assert int(t.cond_bin[0]) == B - 1 and t.split[0] == 1
    o.close()


def test_categorical_and_monotone_against_bruteforce():
    N, F, B, D = 800, 4, 8, 4
    x_bin, y, pred, grad = make_data(50, N, F, B, "mse", True)
    y = (y + 0.3 * (x_bin[0] / B)).astype(np.float32)
    feattypes = np.array([1, 0, 1, 0], np.uint8)
    mono = np.array([1, 0, -1, 0], np.int32)
    p = orc.make_params("mse", nbins=B, max_depth=D)
    orc.update_grads(p, pred, y, grad)
    rows = np.arange(N, dtype=np.uint32)
    js = np.arange(1, F + 1, dtype=np.uint32)
    o = orc.Oracle(p, x_bin, feattypes, mono)
    t, nidx = o.grow_tree(grad, rows, js)
    T, label, _, _ = brute.grow(x_bin, grad, rows, js, 1, B, D, feattypes=feattypes, mono=mono)
    assert trees_equal_struct(t, T)
    assert any(t.split[n] and feattypes[t.feat[n] - 1] == 0 for n in range(len(t.split)))
    assert np.array_equal(nidx.astype(np.int64), label)
    for i in (0, 6, 122, N - 1):
        assert brute.walk(x_bin, feattypes, T, i) == nidx[i]
    o.close()


# ---------------------------------------------------------------- node index / traversal / predict
def test_nidx_equals_independent_walk_and_leaves_are_not_split():
    N, F, B, D = 1000, 5, 16, 5
    x_bin, y, pred, grad = make_data(60, N, F, B)
    p = orc.make_params("mse", nbins=B, max_depth=D, eta=0.2)
    orc.update_grads(p, pred, y, grad)
    rows = np.arange(N, dtype=np.uint32)
    js = np.arange(1, F + 1, dtype=np.uint32)
    o = orc.Oracle(p, x_bin)
    t, nidx = o.grow_tree(grad, rows, js)
    ft = np.ones(F, np.uint8)
    T = dict(feat=t.feat, cond_bin=t.cond_bin, split=t.split)
    leaf = orc.predict_leaf_idx(x_bin, ft, t)
    for i in range(N):
        assert brute.walk(x_bin, ft, T, i) == leaf[i]
    assert np.array_equal(leaf, nidx)
    assert not t.split[leaf - 1].any()
    # stable partition property: rows of each node, in the oracle's work buffer order, are ascending
    before = pred.copy()
    o.predict_tree(t, pred)
    np.testing.assert_array_equal(pred[:, 0], before[:, 0] + t.pred[leaf - 1, 0])
    o.close()


def test_max_depth_one_is_a_single_leaf():
    N, F, B = 200, 3, 8
    x_bin, y, pred, grad = make_data(61, N, F, B)
    p = orc.make_params("mse", nbins=B, max_depth=1)
    orc.update_grads(p, pred, y, grad)
    o = orc.Oracle(p, x_bin)
    t, nidx = o.grow_tree(grad, np.arange(N, dtype=np.uint32), np.arange(1, F + 1, dtype=np.uint32))
    assert t.split.shape == (1,) and t.split[0] == 0 and (nidx == 1).all()
    g = grad[:, 0].astype(np.float64).sum()
    np.testing.assert_allclose(t.pred[0, 0], -0.1 * g / (2 * N + 1.0), rtol=1e-6)
    o.close()


def test_predict_clamps():
    x_bin = np.array([[1, 2, 2]], np.uint8)
    ft = np.ones(1, np.uint8)
    t = orc.Tree(1, 3)
    t.feat[0], t.cond_bin[0], t.split[0] = 1, 1, 1
    t.pred[1, 0], t.pred[2, 0] = 20.0, -20.0
    pred = np.array([[1.0], [1.0], [-14.0]], np.float32)
    orc.predict_tree(orc.LOSS_IDS["logloss"], 1, x_bin, ft, t, pred)
    assert pred[:, 0].tolist() == [15.0, -15.0, -15.0]
    pred = np.array([[1.0], [1.0], [-14.0]], np.float32)
    orc.predict_tree(orc.LOSS_IDS["mse"], 1, x_bin, ft, t, pred)
    assert pred[:, 0].tolist() == [21.0, -19.0, -34.0]
    t2 = orc.Tree(2, 3)
    t2.feat[0], t2.cond_bin[0], t2.split[0] = 1, 1, 1
    t2.pred[1] = [100.0, 100.0]
    t2.pred[2] = [-100.0, -100.0]
    pred = np.zeros((3, 2), np.float32)
    orc.predict_tree(orc.LOSS_IDS["gaussian_mle"], 2, x_bin, ft, t2, pred)
    assert pred.tolist() == [[100.0, 100.0], [-100.0, -15.0], [-100.0, -15.0]]  # only the scale row has a floor
    # link: sigmoid for logloss, softplus on the scale row only (test/metrics.jl:200-204)
    pr = np.array([[0.0, -2.0], [1.0, 0.5]], np.float32)
    orc.apply_link(orc.LOSS_IDS["gaussian_mle"], 2, pr)
    assert pr[:, 0].tolist() == [0.0, 1.0]
    np.testing.assert_allclose(pr[:, 1], np.log1p(np.exp(np.array([-2.0, 0.5]))), rtol=1e-6)


# ---------------------------------------------------------------- oblivious
@pytest.mark.parametrize("loss", ["mse", "gaussian_mle"])
def test_oblivious_against_bruteforce(loss):
    N, F, B, D = 1500, 5, 8, 4
    x_bin, y, pred, grad = make_data(70, N, F, B, loss)
    y = (y + 0.5 * (x_bin[1] > 4) + 0.3 * (x_bin[3] > 2)).astype(np.float32)
    p = orc.make_params(loss, nbins=B, max_depth=D, tree_type="oblivious", min_weight=4.0)
    orc.update_grads(p, pred, y, grad)
    rows = np.arange(N, dtype=np.uint32)
    js = np.arange(1, F + 1, dtype=np.uint32)
    o = orc.Oracle(p, x_bin)
    t, nidx = o.grow_tree(grad, rows, js)
    T, label, _, _ = brute.grow(x_bin, grad, rows, js, p.K, B, D, min_weight=4.0, oblivious=True)
    assert trees_equal_struct(t, T)
    assert t.split[:3].all()
    for d in range(D - 1):  # every split node of a depth shares (feat, bin, gain)
        lvl = slice(2 ** d - 1, 2 ** (d + 1) - 1)
        s = t.split[lvl].astype(bool)
        if s.any():
            assert s.all()
            assert len(set(t.feat[lvl])) == 1 and len(set(t.cond_bin[lvl])) == 1 and len(set(t.gain[lvl])) == 1
    np.testing.assert_allclose(t.gain, T["gain"], rtol=1e-5)
    np.testing.assert_allclose(t.pred, T["pred"], rtol=1e-5, atol=1e-9)
    assert np.array_equal(nidx.astype(np.int64), label)
    o.close()


# ---------------------------------------------------------------- fixed-point mode vs reference arithmetic
@pytest.mark.parametrize("loss,weights", [("mse", False), ("logloss", True), ("gaussian_mle", False)])
def test_fixed_point_mode_matches_f64_mode(loss, weights):
    N, F, B, D = 3000, 8, 32, 6
    x_bin, y, pred, grad = make_data(80, N, F, B, loss, weights)
    p = orc.make_params(loss, nbins=B, max_depth=D)
    orc.update_grads(p, pred, y, grad)
    rows = np.arange(N, dtype=np.uint32)
    js = np.arange(1, F + 1, dtype=np.uint32)
    o = orc.Oracle(p, x_bin)
    t0, n0 = o.grow_tree(grad, rows, js, mode=0)
    H0 = o.hist().copy()
    NK = 2 * p.K + 1
    qbits = np.full(NK, 38, np.int32)
    qbits[0] = 30
    o.set_quant(grad, qbits)
    qb, qe = o.get_quant()
    for k in range(NK):
        m = np.abs(grad[:, k]).max()
        assert m < 2.0 ** qe[k] and (m == 0 or m >= 2.0 ** (qe[k] - 1))
    t1, n1 = o.grow_tree(grad, rows, js, mode=1)
    assert np.array_equal(t0.feat, t1.feat) and np.array_equal(t0.cond_bin, t1.cond_bin) and np.array_equal(t0.split, t1.split)
    assert np.array_equal(n0, n1)
    np.testing.assert_allclose(t1.gain, t0.gain, rtol=1e-5)
    np.testing.assert_allclose(t1.pred, t0.pred, rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(t1.w, t0.w, rtol=1e-6)
    Hq = o.hist(fixed=True)
    scale = np.ldexp(1.0, (qe - qb).astype(np.int64))
    root = Hq[0].astype(np.float64) * scale
    np.testing.assert_allclose(root, H0[0], rtol=0, atol=1e-5 * np.abs(grad).max())
    # exact integer invariants of the fixed-point histogram
    tot = Hq[0].sum(axis=1)
    assert (tot == tot[0]).all()  # every feature's bins sum to the same node total, exactly
    if t1.split[0]:
        assert np.array_equal(Hq[0], Hq[1] + Hq[2])
    o.close()


# ---------------------------------------------------------------- exp-link losses and metrics
def _deviance64(name, p, y):
    """Unit deviances in float64 from the textbook forms (McCullagh & Nelder), mu = exp(p)."""
    mu = np.exp(p)
    if name == "poisson":
        return 2 * (y * np.log(y / mu) + mu - y)
    if name == "gamma":
        return 2 * (np.log(mu / y) + y / mu - 1)
    rho = 1.5
    return 2 * (y ** (2 - rho) / ((1 - rho) * (2 - rho)) - y * mu ** (1 - rho) / (1 - rho) + mu ** (2 - rho) / (2 - rho))


@pytest.mark.parametrize("loss", ["poisson", "gamma", "tweedie"])
def test_exp_link_grads_are_derivatives_of_the_deviance(loss):
    # gamma and tweedie use (D', D''); poisson uses half of them (src/loss.jl:59-76).  Central differences of the
    # float64 textbook deviance pin sign, terms and the role of y in both rows; the weight multiplies both.
    rng = np.random.default_rng(11)
    N = 400
    y = (rng.random(N) * 3 + 0.2).astype(np.float32)
    pred = (rng.standard_normal((N, 1)) * 0.5).astype(np.float32)
    grad = np.zeros((N, 3), np.float32)
    grad[:, 2] = rng.random(N).astype(np.float32) + 0.5
    w = grad[:, 2].astype(np.float64)
    orc.update_grads(orc.make_params(loss), pred, y, grad)
    p64, y64, e = pred[:, 0].astype(np.float64), y.astype(np.float64), 1e-4
    d1 = (_deviance64(loss, p64 + e, y64) - _deviance64(loss, p64 - e, y64)) / (2 * e)
    d2 = (_deviance64(loss, p64 + e, y64) - 2 * _deviance64(loss, p64, y64) + _deviance64(loss, p64 - e, y64)) / e ** 2
    scale = 0.5 if loss == "poisson" else 1.0
    np.testing.assert_allclose(grad[:, 0], scale * d1 * w, rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(grad[:, 1], scale * d2 * w, rtol=2e-4, atol=1e-5)
    assert np.all(grad[:, 1] > 0)


@pytest.mark.parametrize("metric", ["poisson", "gamma", "tweedie"])
def test_deviance_metrics_vs_float64_and_zero_at_perfect_fit(metric):
    rng = np.random.default_rng(12)
    N = 1000
    y = (rng.random(N) * 3 + 0.2).astype(np.float32)
    pred = (rng.standard_normal((N, 1)) * 0.5).astype(np.float32)
    w = (rng.random(N) + 0.5).astype(np.float32)
    ref = np.sum(w.astype(np.float64) * _deviance64(metric, pred[:, 0].astype(np.float64), y.astype(np.float64))) / np.sum(w, dtype=np.float64)
    np.testing.assert_allclose(orc.eval_metric(metric, 1, pred, y, w), ref, rtol=3e-6)
    perfect = np.log(y).reshape(N, 1).astype(np.float32)
    assert abs(orc.eval_metric(metric, 1, perfect, y, w)) < 2e-6
    # y = 0 is a legal count: the poisson value is finite thanks to the epsilon inside the log
    if metric == "poisson":
        v = orc.eval_metric("poisson", 1, np.zeros((4, 1), np.float32), np.zeros(4, np.float32), None)
        np.testing.assert_allclose(v, 2.0, rtol=1e-6)


def test_mse_rmse_mae_logloss_metrics_vs_library_forms():
    from sklearn.metrics import log_loss, mean_absolute_error, mean_squared_error
    rng = np.random.default_rng(13)
    N = 2000
    y = rng.random(N).astype(np.float32)
    pred = rng.standard_normal((N, 1)).astype(np.float32)
    w = (rng.random(N) + 0.5).astype(np.float32)
    mse = mean_squared_error(y, pred[:, 0], sample_weight=w)
    np.testing.assert_allclose(orc.eval_metric("mse", 1, pred, y, w), mse, rtol=2e-6)
    np.testing.assert_allclose(orc.eval_metric("rmse", 1, pred, y, w), np.sqrt(mse), rtol=2e-6)
    np.testing.assert_allclose(orc.eval_metric("mae", 1, pred, y, w), mean_absolute_error(y, pred[:, 0], sample_weight=w), rtol=2e-6)
    np.testing.assert_allclose(orc.eval_metric("mse", 1, pred, y, None), mean_squared_error(y, pred[:, 0]), rtol=2e-6)
    yb = (y > 0.5).astype(np.float32)
    prob = 1 / (1 + np.exp(-pred[:, 0].astype(np.float64)))
    np.testing.assert_allclose(orc.eval_metric("logloss", 1, pred, yb, w), log_loss(yb, prob, sample_weight=w), rtol=1e-5)


def test_gaussian_mle_metric_is_mean_logpdf_up_to_the_constant():
    from scipy.stats import norm
    rng = np.random.default_rng(14)
    N = 2000
    y = rng.standard_normal(N).astype(np.float32)
    pred = np.stack([rng.standard_normal(N) * 0.3, rng.standard_normal(N)], axis=1).astype(np.float32)
    w = (rng.random(N) + 0.5).astype(np.float32)
    scale = np.log1p(np.exp(pred[:, 1].astype(np.float64)))
    lp = norm.logpdf(y.astype(np.float64), pred[:, 0].astype(np.float64), scale) + 0.5 * np.log(2 * np.pi)
    ref = np.sum(w * lp) / np.sum(w, dtype=np.float64)
    np.testing.assert_allclose(orc.eval_metric("gaussian_mle", 2, pred, y, w), ref, rtol=1e-5, atol=1e-6)


def test_exp_link_predict_and_apply_link():
    # predict! adds leaf values without clamping for every GradientRegression loss but logloss (src/predict.jl:1-14);
    # the response is exp of the sum (src/predict.jl:108-109)
    x_bin = np.array([[1, 2, 3, 4]], np.uint8)
    t = orc.Tree(1, 3)
    t.feat[0], t.cond_bin[0], t.split[0] = 1, 2, 1
    t.pred[1, 0], t.pred[2, 0] = 40.0, -40.0
    pred = np.zeros((4, 1), np.float32)
    orc.predict_tree(orc.LOSS_IDS["poisson"], 1, x_bin, np.ones(1, np.uint8), t, pred)
    assert np.array_equal(pred[:, 0], np.float32([40, 40, -40, -40]))
    small = np.float32([[0.5], [-1.25]])
    out = small.copy()
    orc.apply_link(orc.LOSS_IDS["gamma"], 1, out)
    np.testing.assert_allclose(out, np.exp(small.astype(np.float64)), rtol=2e-7)


# ---------------------------------------------------------------- multi-class log loss
def _softmax64(p):
    e = np.exp(p.astype(np.float64) - p.astype(np.float64).max(axis=1, keepdims=True))
    return e / e.sum(axis=1, keepdims=True)


def test_mlogloss_grads_metric_and_link():
    from scipy.special import softmax
    from sklearn.metrics import log_loss
    rng = np.random.default_rng(40)
    N, K = 700, 4
    pred = rng.standard_normal((N, K)).astype(np.float32)
    y = rng.integers(1, K + 1, N).astype(np.float32)
    grad = np.zeros((N, 2 * K + 1), np.float32)
    grad[:, 2 * K] = rng.random(N).astype(np.float32) + 0.5
    w = grad[:, 2 * K].astype(np.float64)
    p = orc.make_params("mlogloss", K=K)
    orc.update_grads(p, pred, y, grad)
    P = _softmax64(pred)
    onehot = np.eye(K)[y.astype(int) - 1]
    np.testing.assert_allclose(grad[:, :K], (P - onehot) * w[:, None], rtol=0, atol=3e-7)   # softmax - onehot
    np.testing.assert_allclose(grad[:, K:2 * K], P * (1 - P) * w[:, None], rtol=3e-6, atol=1e-9)
    assert np.array_equal(grad[:, 2 * K], w.astype(np.float32))
    # the metric is the weighted mean of -log softmax[y]; its derivative in every raw score is the gradient row
    m = orc.eval_metric("mlogloss", K, pred, y, grad[:, 2 * K])
    np.testing.assert_allclose(m, log_loss(y, P, sample_weight=w, labels=np.arange(1, K + 1)), rtol=2e-6)
    i, k, e = 5, 2, 1e-2
    pp, pm = pred.copy(), pred.copy()
    pp[i, k] += e
    pm[i, k] -= e
    wsum = w.sum()
    fd = (orc.eval_metric("mlogloss", K, pp, y, grad[:, 2 * K]) - orc.eval_metric("mlogloss", K, pm, y, grad[:, 2 * K])) / (2 * e) * wsum
    np.testing.assert_allclose(fd, grad[i, k], rtol=2e-3, atol=2e-4)
    # link: softmax of the raw scores
    out = pred.copy()
    orc.apply_link(orc.LOSS_IDS["mlogloss"], K, out)
    np.testing.assert_allclose(out, softmax(pred.astype(np.float64), axis=1), rtol=2e-6)


def test_mlogloss_predict_shifts_by_row_max_and_floors():
    # src/predict.jl:48-62: after adding the leaf, each row is shifted so that its maximum is 0 and floored at -15
    x_bin = np.array([[1, 2, 3]], np.uint8)
    t = orc.Tree(3, 3)
    t.feat[0], t.cond_bin[0], t.split[0] = 1, 1, 1
    t.pred[1] = [1.0, 2.0, 4.0]
    t.pred[2] = [0.0, -30.0, 3.0]
    pred = np.float32([[0.5, 0.5, 0.5], [1.0, 0.0, 0.0], [0.0, 0.0, -1.0]])
    orc.predict_tree(orc.LOSS_IDS["mlogloss"], 3, x_bin, np.ones(1, np.uint8), t, pred)
    assert np.array_equal(pred[0], np.float32([-3.0, -2.0, 0.0]))
    assert np.array_equal(pred[1], np.float32([-2.0, -15.0, 0.0]))
    assert np.array_equal(pred[2], np.float32([-2.0, -15.0, 0.0]))


# ---------------------------------------------------------------- matrix targets
@pytest.mark.parametrize("loss", ["mse", "logloss", "poisson", "gamma", "tweedie", "gaussian_mle"])
def test_matrix_target_grads_and_metric_reduce_to_the_one_target_case(loss):
    """With T targets, output k sees only (pred[k, i], y[k, i]) (src/loss.jl:49-50, :100-111; :219-236 for gaussian_mle,
    whose rows are [g_loc_1, g_scale_1, g_loc_2, ..., h_loc_1, h_scale_1, ..., w]): every gradient / hessian row must equal
    the one-target gradients (pinned above by closed forms and finite differences) of that target alone, bit for bit,
    and the metric is the mean over targets of the one-target metrics (src/metrics.jl:39-45, :105-112)."""
    rng = np.random.default_rng(11)
    N, T = 400, 3
    K = 2 * T if loss == "gaussian_mle" else T
    per = 2 if loss == "gaussian_mle" else 1  # outputs per target
    y = (rng.random((N, T)) + 0.1).astype(np.float32)
    if loss == "logloss":
        y = (y > 0.6).astype(np.float32)
    pred = (rng.standard_normal((N, K)) * 0.4).astype(np.float32)
    w = (rng.random(N) + 0.5).astype(np.float32)
    grad = np.zeros((N, 2 * K + 1), np.float32)
    grad[:, 2 * K] = w
    orc.update_grads(orc.make_params(loss, K=K), pred, y, grad)
    assert np.array_equal(grad[:, 2 * K], w)
    p1 = orc.make_params(loss)
    metrics = []
    for t in range(T):
        pt = np.ascontiguousarray(pred[:, per * t:per * t + per])
        yt = np.ascontiguousarray(y[:, t])
        g1 = np.zeros((N, 2 * per + 1), np.float32)
        g1[:, 2 * per] = w
        orc.update_grads(p1, pt, yt, g1)
        for q in range(per):
            assert np.array_equal(grad[:, per * t + q], g1[:, q]), (t, q)              # gradient rows
            assert np.array_equal(grad[:, K + per * t + q], g1[:, per + q]), (t, q)    # hessian rows
        metrics.append(orc.eval_metric(loss, per, pt, yt, w))
    got = orc.eval_metric(loss, K, pred, y, w)
    assert abs(got - np.mean(metrics)) <= 2e-6 * abs(np.mean(metrics)) + 1e-9


@pytest.mark.parametrize("loss,T", [("mse", 3), ("logloss", 2), ("gaussian_mle", 2)])
def test_matrix_target_tree_against_bruteforce(loss, T):
    """Gains and leaf values sum over the outputs (src/split.jl:58-66, :108-117; src/predict.jl:198-204, :224-234): the tree on
    multi-target gradients against the brute-force search organised differently (node labels, no subtraction trick)."""
    rng = np.random.default_rng(40)
    N, F, B, D = 900, 6, 16, 5
    K = 2 * T if loss == "gaussian_mle" else T
    x_bin = rng.integers(1, B + 1, size=(F, N), dtype=np.uint8)
    y = np.stack([rng.random(N) + 0.5 * (x_bin[t] / B) + 0.3 * (x_bin[(t + 3) % F] > B // 2) for t in range(T)], axis=1).astype(np.float32)
    if loss == "logloss":
        y = (y > np.median(y, axis=0)).astype(np.float32)
    pred = (rng.standard_normal((N, K)) * 0.2).astype(np.float32)
    grad = np.zeros((N, 2 * K + 1), np.float32)
    grad[:, 2 * K] = (rng.random(N) + 0.5).astype(np.float32)
    p = orc.make_params(loss, nbins=B, max_depth=D, lambda_=0.1, gamma=0.01, min_weight=2.0, eta=0.3, K=K)
    orc.update_grads(p, pred, y, grad)
    rows = np.sort(rng.choice(N, 700, replace=False)).astype(np.uint32)
    js = np.array([1, 2, 4, 5, 6], np.uint32)
    o = orc.Oracle(p, x_bin)
    t, nidx = o.grow_tree(grad, rows, js, mode=0)
    Tb, label, hists, sums = brute.grow(x_bin, grad, rows, js, K, B, D, eta=0.3, lam=0.1, L2=1.0, gamma=0.01, min_weight=2.0)
    assert trees_equal_struct(t, Tb)
    assert t.split.sum() >= 3
    np.testing.assert_allclose(t.gain, Tb["gain"], rtol=1e-5)
    np.testing.assert_allclose(t.pred, Tb["pred"], rtol=1e-5, atol=1e-9)
    assert np.array_equal(nidx.astype(np.int64), label)
    o.close()


# ---------------------------------------------------------------- logistic_mle
def test_logistic_mle_grads_are_derivatives_of_the_logpdf_and_fisher_hessians():
    """mle2p_grad_hess(LogisticMLE), src/loss.jl:205-217: g = -d logpdf / d(loc, raw) of the Logistic(loc, softplus(raw))
    density (scipy's logistic.logpdf, central differences in Float64); the hessians are the Fisher information
    1 / (3 s^2) and (pi^2 + 3) / 9 * (sigmoid(raw) / s)^2, which do not depend on the residual."""
    from scipy.stats import logistic
    rng = np.random.default_rng(12)
    N = 300
    pred = np.stack([rng.standard_normal(N), rng.standard_normal(N) * 0.7], axis=1).astype(np.float32)
    y = (rng.standard_normal(N) * 1.5).astype(np.float32)
    w = (rng.random(N) + 0.5).astype(np.float32)
    grad = np.zeros((N, 5), np.float32)
    grad[:, 4] = w
    orc.update_grads(orc.make_params("logistic_mle"), pred, y, grad)
    loc, raw, yy = pred[:, 0].astype(np.float64), pred[:, 1].astype(np.float64), y.astype(np.float64)
    sp = lambda r: np.logaddexp(0.0, r)
    f = lambda l, r: logistic.logpdf(yy, loc=l, scale=sp(r))
    eps = 1e-5
    d_loc = (f(loc + eps, raw) - f(loc - eps, raw)) / (2 * eps)
    d_raw = (f(loc, raw + eps) - f(loc, raw - eps)) / (2 * eps)
    np.testing.assert_allclose(grad[:, 0], -d_loc * w, rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(grad[:, 1], -d_raw * w, rtol=2e-5, atol=2e-6)
    s = sp(raw)
    dsc = 1 / (1 + np.exp(-raw))
    np.testing.assert_allclose(grad[:, 2], w / (3 * s ** 2), rtol=2e-6)
    np.testing.assert_allclose(grad[:, 3], w * (np.pi ** 2 + 3) / 9 * (dsc / s) ** 2, rtol=2e-6)
    # Fisher information = E[score^2] under the model: checked by quadrature for one parameter pair
    l0, r0 = 0.3, -0.2
    s0 = sp(r0)
    grid = np.linspace(l0 - 40 * s0, l0 + 40 * s0, 400001)
    pdf = logistic.pdf(grid, loc=l0, scale=s0)
    z = (grid - l0) / s0
    th = np.tanh(z / 2)
    score_loc = th / s0
    score_raw = -(1 - z * th) * (1 / (1 + np.exp(-r0))) / s0
    dx = grid[1] - grid[0]
    assert abs((pdf * score_loc ** 2).sum() * dx - 1 / (3 * s0 ** 2)) < 1e-6
    assert abs((pdf * score_raw ** 2).sum() * dx - (np.pi ** 2 + 3) / 9 * ((1 / (1 + np.exp(-r0))) / s0) ** 2) < 1e-6


def test_logistic_mle_metric_link_and_predict():
    from scipy.stats import logistic
    rng = np.random.default_rng(13)
    N = 500
    pred = np.stack([rng.standard_normal(N), rng.standard_normal(N)], axis=1).astype(np.float32)
    y = rng.standard_normal(N).astype(np.float32)
    w = (rng.random(N) + 0.5).astype(np.float32)
    got = orc.eval_metric("logistic_mle", 2, pred, y, w)
    s = np.logaddexp(0.0, pred[:, 1].astype(np.float64))
    want = (w * logistic.logpdf(y.astype(np.float64), loc=pred[:, 0].astype(np.float64), scale=s)).sum() / w.astype(np.float64).sum()
    assert abs(got - want) < 2e-6 * abs(want) + 1e-7  # the metric is the weighted mean log-likelihood (src/metrics.jl:92-97)
    linked = pred.copy()
    orc.apply_link(orc.LOSS_IDS["logistic_mle"], 2, linked)
    assert np.array_equal(linked[:, 0], pred[:, 0])
    np.testing.assert_allclose(linked[:, 1], s, rtol=2e-6)
    # predict!: location adds, the raw scale is floored at -15 (src/predict.jl:31-46, the MLE2P method)
    x_bin = np.array([[1, 2]], np.uint8)
    t = orc.Tree(2, 3)
    t.feat[0], t.cond_bin[0], t.split[0] = 1, 1, 1
    t.pred[1] = [2.0, -40.0]
    t.pred[2] = [-3.0, 1.0]
    p = np.zeros((2, 2), np.float32)
    orc.predict_tree(orc.LOSS_IDS["logistic_mle"], 2, x_bin, np.ones(1, np.uint8), t, p)
    assert p.tolist() == [[2.0, -15.0], [-3.0, 1.0]]


# ---------------------------------------------------------------- mae and the credibility losses
KIND = {"mae": "mae", "cred_var": "cred_var", "cred_std": "cred_std"}


@pytest.mark.parametrize("loss", ["mae", "cred_var", "cred_std"])
def test_residual_loss_grads_closed_form(loss):
    """mae: [(y - p) w, 0, w]; credibility: [d w, d^2 w, w] with d = y - p (src/loss.jl:78-83), in Float32."""
    N = 500
    x_bin, y, pred, grad = make_data(61, N, 3, 8, "mse", weights=True)
    w = grad[:, 2].copy()
    p = orc.make_params(loss, nbins=8, max_depth=3)
    orc.update_grads(p, pred, y, grad)
    d = y - pred[:, 0]
    assert np.array_equal(grad[:, 0], d * w)
    assert np.array_equal(grad[:, 1], (np.zeros_like(d) if loss == "mae" else (d * d) * w))
    assert np.array_equal(grad[:, 2], w)


def _stump(loss, x_bin, y, pred, grad, B, lam=0.0, L2=0.0, eta=1.0, min_weight=1.0):
    p = orc.make_params(loss, nbins=B, max_depth=2, lambda_=lam, L2=L2, eta=eta, min_weight=min_weight)
    orc.update_grads(p, pred, y, grad)
    o = orc.Oracle(p, x_bin)
    rows = np.arange(x_bin.shape[1], dtype=np.uint32)
    js = np.arange(1, x_bin.shape[0] + 1, dtype=np.uint32)
    t, nidx = o.grow_tree(grad, rows, js, mode=0)
    o.close()
    return t, nidx


def test_mae_stump_is_the_largest_weighted_shift_of_the_mean_residual():
    """With lambda = L2 = 0 and unit weights the mae gain of a split is nL |mean_L - mean| + nR |mean_R - mean|
    (= 2 nL |mean_L - mean|, the two shifts balance), the parent's gain is zero, and a leaf predicts eta times its mean
    residual: checked from the raw residuals, no histogram."""
    N, F, B = 400, 4, 8
    x_bin, y, pred, grad = make_data(62, N, F, B, "mse", weights=False)
    t, nidx = _stump("mae", x_bin, y, pred, grad, B, eta=0.7)
    d = (y - pred[:, 0]).astype(np.float64)
    best = (-1.0, 0, 0)
    for j in range(F):
        for b in range(1, B):  # numeric: bins 1 .. B-1
            L = x_bin[j] <= b
            nL, nR = L.sum(), (~L).sum()
            if nL > 1 and nR > 1:
                g = nL * abs(d[L].mean() - d.mean()) + nR * abs(d[~L].mean() - d.mean())
                assert abs(g - 2 * nL * abs(d[L].mean() - d.mean())) < 1e-9 * max(1.0, g)
                if g > best[0] * (1 + 1e-12) + 1e-12:
                    best = (g, j + 1, b)
    assert t.split[0] == 1 and (int(t.feat[0]), int(t.cond_bin[0])) == best[1:]
    np.testing.assert_allclose(t.gain[0], best[0], rtol=1e-5)
    L = x_bin[best[1] - 1] <= best[2]
    np.testing.assert_allclose(t.pred[1, 0], 0.7 * d[L].mean(), rtol=1e-5)
    np.testing.assert_allclose(t.pred[2, 0], 0.7 * d[~L].mean(), rtol=1e-5)
    assert np.array_equal(nidx, np.where(L, 2, 3))


@pytest.mark.parametrize("loss", ["cred_var", "cred_std"])
def test_cred_stump_from_raw_residual_moments(loss):
    """Unit weights, L2 = 0: a side's term is Z |sum d| with Z = mean^2 / (mean^2 + var) = mean^2 / mean(d^2) for
    cred_var and |mean| / (|mean| + std) for cred_std (population variance); the recorded gain is left + right - parent;
    a leaf predicts eta * mean residual.  All from numpy's mean / var / std of the raw residuals."""
    N, F, B = 400, 4, 8
    x_bin, y, pred, grad = make_data(63, N, F, B, "mse", weights=False)
    y = (y + 0.8).astype(np.float32)  # residuals with a clear mean
    t, nidx = _stump(loss, x_bin, y, pred, grad, B, eta=0.5)
    d = (y - pred[:, 0]).astype(np.float64)

    def term(v):
        m, var = v.mean(), v.var()
        Z = m * m / (m * m + var) if loss == "cred_var" else abs(m) / (abs(m) + np.sqrt(var))
        return Z * abs(v.sum())

    if loss == "cred_var":  # the same credibility written with the second moment only
        assert abs(term(d) - abs(d.sum()) ** 3 / (len(d) * (d * d).sum())) < 1e-9 * term(d)
    best = (-np.inf, 0, 0)
    for j in range(F):
        for b in range(1, B):
            L = x_bin[j] <= b
            if L.sum() > 1 and (~L).sum() > 1:
                g = term(d[L]) + term(d[~L]) - term(d)
                if g > best[0] + 1e-12 * abs(g):
                    best = (g, j + 1, b)
    assert t.split[0] == 1 and (int(t.feat[0]), int(t.cond_bin[0])) == best[1:]
    np.testing.assert_allclose(t.gain[0], best[0], rtol=1e-5)
    L = x_bin[best[1] - 1] <= best[2]
    np.testing.assert_allclose(t.pred[1, 0], 0.5 * d[L].mean(), rtol=1e-5)
    np.testing.assert_allclose(t.pred[2, 0], 0.5 * d[~L].mean(), rtol=1e-5)


@pytest.mark.parametrize("loss,weights,lam,L2,gamma,minw", [
    ("mae", False, 0.0, 1.0, 0.0, 1.0),
    ("mae", True, 0.5, 0.3, 0.05, 2.0),
    ("cred_var", False, 0.0, 1.0, 0.0, 1.0),
    ("cred_var", True, 0.0, 0.4, 0.01, 2.0),
    ("cred_std", False, 0.0, 0.0, 0.0, 1.0),
    ("cred_std", True, 0.0, 2.0, 0.02, 3.0),
])
def test_residual_loss_tree_against_bruteforce(loss, weights, lam, L2, gamma, minw):
    N, F, B, D = 900, 6, 16, 5
    x_bin, y, pred, grad = make_data(64, N, F, B, "mse", weights)
    p = orc.make_params(loss, nbins=B, max_depth=D, lambda_=lam, L2=L2, gamma=gamma, min_weight=minw, eta=0.3)
    orc.update_grads(p, pred, y, grad)
    rng = np.random.default_rng(65)
    rows = np.sort(rng.choice(N, 640, replace=False)).astype(np.uint32)
    js = np.array([1, 2, 4, 6], np.uint32)
    o = orc.Oracle(p, x_bin)
    t, nidx = o.grow_tree(grad, rows, js, mode=0)
    T, label, hists, sums = brute.grow(x_bin, grad, rows, js, 1, B, D, eta=0.3, lam=lam, L2=L2, gamma=gamma, min_weight=minw, kind=KIND[loss])
    assert trees_equal_struct(t, T)
    assert t.split.sum() >= 3
    np.testing.assert_allclose(t.gain, T["gain"], rtol=1e-5)
    np.testing.assert_allclose(t.pred, T["pred"], rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(t.w, T["w"], rtol=1e-6)
    assert np.array_equal(nidx.astype(np.int64), label)
    # fixed-point mode: same structure on this data, values to 1e-5
    qbits = np.full(3, 38, np.int32)
    qbits[0] = 30
    o.set_quant(grad, qbits)
    t1, nidx1 = o.grow_tree(grad, rows, js, mode=1)
    assert trees_equal_struct(t1, T) and np.array_equal(nidx1, nidx)
    np.testing.assert_allclose(t1.pred, t.pred, rtol=1e-5, atol=1e-9)
    o.close()


@pytest.mark.parametrize("loss", ["mae", "cred_std"])
def test_residual_loss_monotone_and_oblivious_against_bruteforce(loss):
    N, F, B, D = 700, 5, 12, 4
    x_bin, y, pred, grad = make_data(66, N, F, B, "mse", weights=True)
    y = (y + 0.02 * x_bin[0] - 0.03 * x_bin[2]).astype(np.float32)
    mono = np.array([1, 0, -1, 0, 0], np.int32)
    rows = np.arange(N, dtype=np.uint32)
    js = np.arange(1, F + 1, dtype=np.uint32)
    for tt in ("binary", "oblivious"):
        p = orc.make_params(loss, nbins=B, max_depth=D, tree_type=tt, eta=0.2, L2=0.5, min_weight=3.0)
        orc.update_grads(p, pred, y, grad)
        o = orc.Oracle(p, x_bin, monotone=mono)
        t, nidx = o.grow_tree(grad, rows, js, mode=0)
        T, label, _, _ = brute.grow(x_bin, grad, rows, js, 1, B, D, eta=0.2, L2=0.5, min_weight=3.0, mono=mono, oblivious=(tt == "oblivious"),
                                    kind=KIND[loss])
        assert trees_equal_struct(t, T), tt
        assert t.split.sum() >= 1
        np.testing.assert_allclose(t.pred, T["pred"], rtol=1e-5, atol=1e-9)
        assert np.array_equal(nidx.astype(np.int64), label)
        o.close()


def test_residual_loss_predict_adds_and_link_is_identity():
    """The generic predict! (src/predict.jl:68-81) adds the leaf value, no clamp; apply_prediction_link! leaves these
    losses alone (src/predict.jl:105-116)."""
    N, F, B = 50, 3, 4
    rng = np.random.default_rng(67)
    x_bin = rng.integers(1, B + 1, size=(F, N), dtype=np.uint8)
    t = orc.Tree(1, 3)
    t.split[0] = 1; t.feat[0] = 2; t.cond_bin[0] = 2
    t.pred[1, 0] = 40.0; t.pred[2, 0] = -40.0
    for loss in ("mae", "cred_var", "cred_std"):
        pred = np.full((N, 1), 3.0, np.float32)
        orc.predict_tree(orc.LOSS_IDS[loss], 1, x_bin, np.ones(F, np.uint8), t, pred)
        assert np.array_equal(pred[:, 0], np.where(x_bin[1] <= 2, 43.0, -37.0).astype(np.float32))
        q = pred.copy()
        orc.apply_link(orc.LOSS_IDS[loss], 1, q)
        assert np.array_equal(q, pred)


# ---------------------------------------------------------------- quantile losses
def test_quantile_grads_closed_form():
    """Row k: alpha (residual > 0) or alpha - 1, a Float64, times the weight, rounded to Float32; row K + k: the raw
    residual, not weighted (src/loss.jl:85-91, :144-171)."""
    N = 400
    x_bin, y, pred, grad = make_data(71, N, 3, 8, "mse", weights=True)
    w = grad[:, 2].copy()
    p = orc.make_params("quantile", nbins=8, max_depth=3, alpha=0.3)
    orc.update_grads(p, pred, y, grad)
    d = y - pred[:, 0]
    want = (np.where(d > 0, 0.3, 0.3 - 1.0) * w.astype(np.float64)).astype(np.float32)
    assert np.array_equal(grad[:, 0], want) and np.array_equal(grad[:, 1], d) and np.array_equal(grad[:, 2], w)
    # multiquantile: one target, an alpha per output
    al = [0.1, 0.5, 0.9]
    pm = orc.make_params("multiquantile", nbins=8, max_depth=3, alphas=al)
    assert pm.K == 3
    predm = (np.random.default_rng(72).standard_normal((N, 3)) * 0.3).astype(np.float32)
    gm = np.zeros((N, 7), np.float32)
    gm[:, 6] = w
    orc.update_grads(pm, predm, y, gm)
    for k in range(3):
        dk = y - predm[:, k]
        assert np.array_equal(gm[:, k], (np.where(dk > 0, al[k], al[k] - 1.0) * w.astype(np.float64)).astype(np.float32))
        assert np.array_equal(gm[:, 3 + k], dk)


@pytest.mark.parametrize("alpha,n", [(0.5, 1), (0.5, 2), (0.1, 11), (0.9, 11), (0.25, 400), (0.999, 57), (0.0, 9), (1.0, 9)])
def test_leaf_quantile_is_numpys_linear_quantile(alpha, n):
    """A depth-1 tree is one leaf over all rows: its value is eta * quantile(residuals, alpha) (lambda = L2 = 0), with the
    quantile of Hyndman & Fan's definition 7 - numpy's "linear" method on the same Float32 residuals."""
    rng = np.random.default_rng(73)
    x_bin = rng.integers(1, 5, size=(2, n), dtype=np.uint8)
    y = rng.standard_normal(n).astype(np.float32)
    pred = np.zeros((n, 1), np.float32)
    grad = np.zeros((n, 3), np.float32)
    grad[:, 2] = 1.0
    p = orc.make_params("quantile", nbins=4, max_depth=1, eta=0.7, L2=0.0, alpha=alpha)
    orc.update_grads(p, pred, y, grad)
    o = orc.Oracle(p, x_bin)
    t, nidx = o.grow_tree(grad, np.arange(n, dtype=np.uint32), np.array([1, 2], np.uint32), mode=0)
    want = 0.7 * np.quantile(y.astype(np.float64), alpha, method="linear")
    np.testing.assert_allclose(t.pred[0, 0], want, rtol=1e-6, atol=1e-7)
    o.close()


def test_pinball_metric_against_sklearn():
    from sklearn.metrics import mean_pinball_loss
    rng = np.random.default_rng(74)
    N = 3000
    y = rng.standard_normal(N).astype(np.float32)
    p1 = (y + rng.standard_normal(N) * 0.5).astype(np.float32).reshape(N, 1)
    w = (rng.random(N) + 0.5).astype(np.float32)
    for alpha in (0.1, 0.5, 0.8):
        got = orc.eval_metric("quantile", 1, p1, y, w, alphas=[alpha])
        np.testing.assert_allclose(got, mean_pinball_loss(y, p1[:, 0], sample_weight=w, alpha=alpha), rtol=1e-5)
    al = [0.2, 0.5, 0.9]
    p3 = (y[:, None] + rng.standard_normal((N, 3)) * 0.5).astype(np.float32)
    got = orc.eval_metric("multiquantile", 3, p3, y, None, alphas=al)
    want = np.mean([mean_pinball_loss(y, p3[:, k], alpha=al[k]) for k in range(3)])
    np.testing.assert_allclose(got, want, rtol=1e-5)
    # quantile loss with several targets: one alpha, averaged over the outputs
    Y2 = np.stack([y, -y], axis=1).astype(np.float32)
    got = orc.eval_metric("quantile", 2, p3[:, :2].copy(), Y2, w, alphas=[0.3])
    want = np.mean([mean_pinball_loss(Y2[:, k], p3[:, k], sample_weight=w, alpha=0.3) for k in range(2)])
    np.testing.assert_allclose(got, want, rtol=1e-5)


@pytest.mark.parametrize("loss,weights,lam,L2,tt", [
    ("quantile", False, 0.0, 0.0, "binary"),
    ("quantile", True, 0.4, 0.7, "binary"),
    ("quantile", True, 0.0, 1.0, "oblivious"),
    ("multiquantile", False, 0.0, 1.0, "binary"),
    ("multiquantile", True, 0.2, 0.5, "binary"),
])
def test_quantile_tree_against_bruteforce(loss, weights, lam, L2, tt):
    N, F, B, D = 900, 6, 16, 5
    x_bin, y, pred, grad0 = make_data(75, N, F, B, "mse", weights)
    y = (y + 0.03 * x_bin[1]).astype(np.float32)
    if loss == "multiquantile":
        al = [0.15, 0.5, 0.85]
        p = orc.make_params(loss, nbins=B, max_depth=D, tree_type=tt, lambda_=lam, L2=L2, eta=0.3, min_weight=2.0, alphas=al)
        K = 3
        pred = (np.random.default_rng(76).standard_normal((N, K)) * 0.2).astype(np.float32)
    else:
        al = [0.7]
        p = orc.make_params(loss, nbins=B, max_depth=D, tree_type=tt, lambda_=lam, L2=L2, eta=0.3, min_weight=2.0, alpha=0.7)
        K = 1
    grad = np.zeros((N, 2 * K + 1), np.float32)
    grad[:, 2 * K] = grad0[:, 2]
    orc.update_grads(p, pred, y, grad)
    rng = np.random.default_rng(77)
    rows = np.sort(rng.choice(N, 700, replace=False)).astype(np.uint32)
    js = np.array([1, 2, 3, 5], np.uint32)
    o = orc.Oracle(p, x_bin)
    t, nidx = o.grow_tree(grad, rows, js, mode=0)
    T, label, hists, sums = brute.grow(x_bin, grad, rows, js, K, B, D, eta=0.3, lam=lam, L2=L2, min_weight=2.0, oblivious=(tt == "oblivious"),
                                       kind="quantile", alphas=al * (K if len(al) == 1 else 1), clamp_denom=(loss == "quantile"))
    assert trees_equal_struct(t, T)
    assert t.split.sum() >= 3
    np.testing.assert_allclose(t.gain, T["gain"], rtol=1e-5)
    np.testing.assert_allclose(t.pred, T["pred"], rtol=1e-5, atol=1e-7)
    assert np.array_equal(nidx.astype(np.int64), label)
    o.close()
