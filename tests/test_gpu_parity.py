"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle on identical
seeded inputs.

Bars (stated by the hot-path contract):
  * node indices, split features and split bins: bit exact;
  * histograms, gains, leaf values, predictions: relative 1e-5 (Float32 outputs) against the
    oracle's Float64 reference arithmetic (mode 0);
  * in addition, against the oracle's fixed-point mode (mode 1), which specifies the device's
    deterministic integer histogram arithmetic, everything is bit exact when both sides are fed the
    same Float32 gradients.
"""
import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu

RTOL = 1e-5


def n_outputs(loss, K=None):
    return 2 if loss in ("gaussian_mle", "logistic_mle") else ((K or 3) if loss in ("mlogloss", "multiquantile") else 1)


def make_data(seed, N, F, nbins, loss="mse", weights=False, signal=True, K=None):
    rng = np.random.default_rng(seed)
    x_bin = rng.integers(1, nbins + 1, size=(F, N), dtype=np.uint8)
    K = n_outputs(loss, K)
    y = rng.random(N).astype(np.float32)
    if signal:
        y = (y + 0.5 * (x_bin[0] / nbins) + 0.25 * (x_bin[F // 2] > nbins // 3)).astype(np.float32)
    if loss == "logloss":
        y = (y > np.median(y)).astype(np.float32)
    elif loss == "poisson":
        y = np.floor(y * 3).astype(np.float32)  # counts, zeros included
    elif loss in ("gamma", "tweedie"):
        y = (y + 0.1).astype(np.float32)  # strictly positive
    elif loss in ("quantile", "multiquantile"):
        y = (y - 0.85).astype(np.float32)  # residuals of both signs against the starting prediction near zero
    elif loss == "mlogloss":
        y = (np.minimum(np.floor(y / y.max() * K), K - 1) + 1).astype(np.float32)  # 1-based class, tied to the features
    w = (rng.random(N).astype(np.float32) + 0.5) if weights else None
    mu = (rng.standard_normal(K) * 0.1).astype(np.float32)
    if loss == "mlogloss":
        mu = mu - mu.max()  # as _init_target leaves it (src/init.jl:63-64): predict! of the bias tree then changes nothing
    return x_bin, y, w, mu


def setup_pair(evt, loss, x_bin, y, w, mu, nbins, depth, tree_type="binary", feattypes=None, mono=None, **pk):
    F, N = x_bin.shape
    K = mu.shape[0]
    h = evt.Handle(N, F, nbins, K, depth, loss, tree_type)
    h.set_xbin(x_bin)
    h.set_feature_meta(feattypes, mono)
    if loss == "multiquantile":  # one level per output
        pk = dict(pk, alphas=pk.get("alphas", [0.1, 0.5, 0.9]))
        assert len(pk["alphas"]) == K
        h.set_alphas(pk["alphas"])
    elif loss == "quantile":
        pk = dict(pk, alpha=pk.get("alpha", 0.5))
        h.set_alphas([pk["alpha"]])
    h.set_target(y, w, mu)
    op = orc.make_params(loss, nbins=nbins, max_depth=depth, tree_type=tree_type, K=K, **pk)
    o = orc.Oracle(op, x_bin, feattypes, mono)
    gp = evt.make_params(eta=op.eta, L2=op.L2, lambda_=op.lambda_, gamma=op.gamma, min_weight=op.min_weight,
                         bagging_size=op.bagging_size, update_pred=True)
    pred0 = np.tile(mu, (N, 1)).astype(np.float32)
    grad0 = np.zeros((N, 2 * K + 1), np.float32)
    grad0[:, 2 * K] = 1.0 if w is None else w
    return h, o, op, gp, pred0, grad0


def assert_tree_bits(t_gpu, t_orc):
    assert np.array_equal(t_gpu.feat, t_orc.feat)
    assert np.array_equal(t_gpu.cond_bin, t_orc.cond_bin)
    assert np.array_equal(t_gpu.split, t_orc.split)
    assert np.array_equal(t_gpu.gain.view(np.uint32), t_orc.gain.view(np.uint32))
    assert np.array_equal(t_gpu.pred.view(np.uint32), t_orc.pred.view(np.uint32))
    assert np.array_equal(t_gpu.w.view(np.uint32), t_orc.w.view(np.uint32))


def assert_tree_close(t_gpu, t_ref, pred_atol=1e-9):
    assert np.array_equal(t_gpu.feat, t_ref.feat)
    assert np.array_equal(t_gpu.cond_bin, t_ref.cond_bin)
    assert np.array_equal(t_gpu.split, t_ref.split)
    np.testing.assert_allclose(t_gpu.gain, t_ref.gain, rtol=RTOL, atol=1e-7)
    np.testing.assert_allclose(t_gpu.pred, t_ref.pred, rtol=RTOL, atol=pred_atol)
    np.testing.assert_allclose(t_gpu.w, t_ref.w, rtol=RTOL)


# --------------------------------------------------------------------------- gradients
@pytest.mark.parametrize("loss,weights", [("mse", False), ("mse", True), ("logloss", True), ("gaussian_mle", False),
                                          ("gaussian_mle", True), ("poisson", True), ("gamma", False), ("tweedie", True),
                                          ("mlogloss", False), ("mlogloss", True), ("logistic_mle", False), ("logistic_mle", True),
                                          ("mae", False), ("mae", True), ("cred_var", True), ("cred_std", False),
                                          ("quantile", True), ("quantile", False), ("multiquantile", True)])
def test_gradient_kernel(evt, loss, weights):
    N, F, B = 70001, 5, 16
    x_bin, y, w, mu = make_data(1, N, F, B, loss, weights)
    h, o, op, gp, pred0, grad0 = setup_pair(evt, loss, x_bin, y, w, mu, B, 3)
    h.update_grads()
    g_gpu = h.get_grads()
    grad = grad0.copy()
    orc.update_grads(op, pred0, y, grad)
    K = op.K
    assert np.array_equal(g_gpu[:, 2 * K], grad[:, 2 * K])  # weight row untouched
    if loss in ("mse", "mae", "cred_var", "cred_std", "quantile", "multiquantile"):
        assert np.array_equal(g_gpu.view(np.uint32), grad.view(np.uint32))  # exact Float32 arithmetic
    else:
        # terms like (1 - z tanh(z / 2)) cancel: the absolute bound is a few ulp of the largest gradient
        np.testing.assert_allclose(g_gpu, grad, rtol=RTOL, atol=1e-6 * max(1.0, float(np.abs(grad[:, :2 * K]).max())))
    h.close()
    o.close()


# --------------------------------------------------------------------------- one tree, teacher forced
CASES = [
    # loss, weights, N, F, nbins, depth, tree_type, n_js, rowsample, extra params
    ("mse", False, 20000, 10, 64, 6, "binary", 10, 1.0, {}),
    ("mse", True, 30011, 7, 32, 5, "binary", 5, 0.5, dict(lambda_=0.5, gamma=0.05)),
    ("mse", False, 150000, 100, 64, 7, "binary", 100, 1.0, {}),
    ("mse", False, 50000, 100, 64, 6, "binary", 50, 0.5, {}),
    ("logloss", False, 40000, 28, 128, 8, "binary", 28, 0.8, dict(eta=0.05)),
    ("logloss", True, 25000, 33, 255, 5, "binary", 20, 1.0, dict(min_weight=3.0)),
    ("gaussian_mle", False, 40000, 50, 64, 7, "binary", 50, 1.0, dict(min_weight=8.0)),
    ("gaussian_mle", True, 20000, 17, 16, 5, "binary", 9, 0.7, dict(min_weight=8.0, lambda_=0.1)),
    ("gaussian_mle", False, 40000, 50, 64, 7, "oblivious", 50, 1.0, dict(min_weight=8.0)),
    ("mse", False, 30000, 12, 32, 6, "oblivious", 12, 1.0, {}),
    ("logloss", True, 30000, 12, 32, 5, "oblivious", 8, 0.6, {}),
    ("mse", False, 5000, 200, 8, 4, "binary", 200, 1.0, {}),
    ("mse", True, 40000, 120, 32, 6, "binary", 120, 1.0, {}),
    ("logloss", False, 40000, 100, 32, 6, "binary", 70, 0.7, {}),
    ("gaussian_mle", False, 30000, 128, 8, 5, "binary", 128, 1.0, dict(min_weight=8.0)),
    ("logistic_mle", True, 30000, 20, 32, 6, "binary", 20, 1.0, dict(min_weight=8.0)),
    ("logistic_mle", False, 20000, 100, 64, 5, "oblivious", 50, 0.5, dict(min_weight=8.0)),
    ("mse", False, 20000, 300, 16, 5, "binary", 300, 1.0, {}),
    # records whose features are spread over all their pieces: 5, 6 and 7 features per 8-byte piece, 3 per 4-byte piece,
    # 32 lanes per row, with and without a column sample that switches the per-feature test on
    ("mse", False, 30000, 80, 32, 5, "binary", 80, 1.0, {}),
    ("mse", False, 20000, 90, 64, 5, "binary", 40, 1.0, {}),
    ("mse", True, 30000, 40, 32, 5, "binary", 15, 0.8, {}),
    ("logloss", False, 20000, 150, 16, 5, "binary", 150, 1.0, {}),
    ("mse", False, 1000, 3, 4, 1, "binary", 3, 1.0, {}),
    ("mse", False, 300, 1, 2, 3, "binary", 1, 1.0, dict(min_weight=0.0)),
    ("poisson", True, 30000, 12, 32, 6, "binary", 9, 0.8, {}),
    ("gamma", False, 30000, 20, 64, 6, "binary", 20, 1.0, dict(lambda_=0.2)),
    ("tweedie", False, 30000, 12, 32, 5, "oblivious", 12, 1.0, {}),
    ("mlogloss", False, 30000, 12, 32, 5, "binary", 12, 1.0, {}),
    ("mlogloss", True, 20000, 100, 16, 5, "binary", 60, 0.7, dict(lambda_=0.1)),
    ("mlogloss", False, 20000, 100, 16, 4, "binary", 100, 1.0, dict(K=2)),
    ("mlogloss", False, 20000, 10, 32, 4, "oblivious", 10, 1.0, dict(K=5)),
    ("mlogloss", True, 12000, 9, 128, 4, "binary", 9, 1.0, dict(K=16, min_weight=2.0)),
    ("mae", False, 30000, 12, 32, 6, "binary", 12, 1.0, {}),
    ("mae", True, 40000, 100, 64, 6, "binary", 60, 0.6, dict(lambda_=0.3, L2=0.5, gamma=0.01)),
    ("mae", False, 20000, 10, 16, 5, "oblivious", 10, 1.0, {}),
    ("cred_var", False, 30000, 12, 32, 6, "binary", 12, 1.0, {}),
    ("cred_var", True, 40000, 100, 64, 6, "binary", 100, 0.7, dict(L2=2.0, min_weight=4.0)),
    ("cred_std", False, 30000, 20, 64, 6, "binary", 14, 1.0, dict(L2=0.0)),
    ("cred_std", True, 20000, 10, 16, 5, "oblivious", 10, 0.8, {}),
    ("quantile", False, 30000, 12, 32, 6, "binary", 12, 1.0, dict(alpha=0.3)),
    ("quantile", True, 40000, 100, 64, 6, "binary", 60, 0.6, dict(alpha=0.9, lambda_=0.2, L2=0.5, gamma=0.01)),
    ("quantile", False, 20000, 10, 16, 5, "oblivious", 10, 1.0, {}),
    ("quantile", True, 3000, 4, 4, 12, "binary", 4, 0.9, dict(alpha=0.05, min_weight=0.0)),  # leaves of one or two rows
    ("multiquantile", True, 30000, 12, 32, 5, "binary", 12, 0.8, dict(alphas=[0.1, 0.5, 0.9])),
    ("multiquantile", False, 20000, 20, 64, 4, "oblivious", 20, 1.0, dict(alphas=[0.25, 0.75], L2=0.0)),
    # more than 1024 features (the reference takes any number): records of 2 KB and more, four and six column tiles
    ("mse", False, 6000, 2048, 16, 4, "binary", 2048, 1.0, {}),
    ("logloss", True, 5000, 3000, 8, 4, "binary", 1500, 0.7, {}),
    ("mse", False, 60000, 5, 8, 14, "binary", 5, 1.0, dict(min_weight=0.0)),   # deep: most leaves hold a handful of rows
    ("logloss", True, 3000, 4, 4, 16, "binary", 4, 0.9, dict(min_weight=0.0)),  # deepest supported tree, far more nodes than rows
    # 16-byte records and few chunks: the levels below the root get their histograms from the partition's scatter pass
    ("logloss", True, 50000, 13, 64, 7, "binary", 13, 1.0, {}),                          # three channels, weights
    ("gaussian_mle", False, 30000, 16, 64, 5, "binary", 16, 1.0, dict(min_weight=8.0)),  # four channels, all 16 features sampled
    ("gaussian_mle", True, 30000, 9, 32, 6, "binary", 7, 0.8, dict(min_weight=8.0)),     # five channels, row and column samples
]


@pytest.mark.parametrize("loss,weights,N,F,B,D,tt,n_js,rowsample,pk", CASES)
def test_grow_tree_matches_oracle(evt, loss, weights, N, F, B, D, tt, n_js, rowsample, pk):
    print("case", loss, weights, N, F, B, D, tt, n_js, rowsample, pk, flush=True)
    pk = dict(pk)
    x_bin, y, w, mu = make_data(7, N, F, B, loss, weights, K=pk.pop("K", None) or (len(pk["alphas"]) if "alphas" in pk else None))
    h, o, op, gp, pred0, grad0 = setup_pair(evt, loss, x_bin, y, w, mu, B, D, tt, **pk)
    rng = np.random.default_rng(99)
    grad = grad0.copy()
    orc.update_grads(op, pred0, y, grad)
    h.set_grads(grad)  # identical Float32 gradients on both sides
    js = (np.sort(rng.choice(F, n_js, replace=False)) + 1).astype(np.uint32)
    if rowsample < 1.0:
        mask = rng.integers(0, 256, N, dtype=np.uint8)
        cond = int(np.rint(255 * rowsample))
        rows = orc.subsample(mask, cond)
    else:
        mask, cond, rows = None, 255, np.arange(N, dtype=np.uint32)
    h.set_option("record_nidx", 1)  # node ids written by the partition itself while the tree grows
    t_gpu = h.grow_tree(js, gp, mask=mask, cond=cond)
    nidx_gpu = h.get_nidx()
    # fixed-point oracle: bit exact
    qb, qe = h.get_quant()
    o.set_quant(grad, qb)
    assert np.array_equal(o.get_quant()[1], qe)
    t_fx, nidx_fx = o.grow_tree(grad, rows, js, mode=1)
    assert_tree_bits(t_gpu, t_fx)
    assert np.array_equal(nidx_gpu, nidx_fx)
    # histograms of every split node, sampled features: bit exact against the fixed-point oracle
    H_gpu = h.get_hist()
    Hq = o.hist(fixed=True)
    scale = np.ldexp(1.0, (qe - qb).astype(np.int64))
    split_nodes = np.flatnonzero(t_gpu.split)
    # one-output quantile: the second gradient row (the raw residual, read per row when the leaves are valued) has no
    # accumulator on the device and is exported as zero; no gain reads its sum
    chan = [0, 2] if loss in ("quantile", "multiquantile") and op.K == 1 else list(range(2 * op.K + 1))
    for n0 in split_nodes:
        want = Hq[n0][js - 1].astype(np.float64) * scale
        assert np.array_equal(H_gpu[n0][js - 1][..., chan], want[..., chan]), n0
        if len(chan) == 2:
            assert not H_gpu[n0][js - 1][..., 1].any()
    # reference arithmetic (Float64 accumulation in row order): same structure, values within 1e-5
    t_ref, nidx_ref = o.grow_tree(grad, rows, js, mode=0)
    assert_tree_close(t_gpu, t_ref)
    assert np.array_equal(nidx_gpu, nidx_ref)
    H_ref = o.hist()
    gmax = np.abs(grad).max(axis=0)
    for n0 in split_nodes:
        np.testing.assert_allclose(H_gpu[n0][js - 1][..., chan], H_ref[n0][js - 1][..., chan], rtol=RTOL, atol=1e-6 * float(gmax.max()))
    if D > 1 and N >= 5000:
        assert len(split_nodes) >= 1
    # predict! on the cache: all rows (also those outside the sample)
    p_gpu = h.get_pred()
    p_orc = pred0.copy()
    o.predict_tree(t_fx, p_orc)
    assert np.array_equal(p_gpu.view(np.uint32), p_orc.view(np.uint32))
    # without recording, the node ids are derived by walking the finished tree: same answer
    h.set_option("record_nidx", 0)
    t_again = h.grow_tree(js, gp, mask=mask, cond=cond)
    assert_tree_bits(t_again, t_fx)
    assert np.array_equal(h.get_nidx(), nidx_fx)
    # the partition's two decision sources - threshold bit planes (default when they fit) and gathered bin bytes - agree
    h.set_option("bit_planes", 0)
    h.set_option("record_nidx", 1)
    assert_tree_bits(h.grow_tree(js, gp, mask=mask, cond=cond), t_fx)
    assert np.array_equal(h.get_nidx(), nidx_fx)
    h.set_option("bit_planes", 1)
    h.set_option("record_nidx", 0)
    # launch shape must not change a bit of the result (integer accumulation is order independent)
    h.set_option("hist_blocks", 37)
    h.set_option("hist_threads", 256)
    assert_tree_bits(h.grow_tree(js, gp, mask=mask, cond=cond), t_fx)
    # both histogram kernels (generic 16-byte pieces / conflict-free 8-byte pieces) give the same bits; the generic one
    # reads a record with one wavefront instruction, so it is not offered for records wider than 1024 bytes
    generic = 1 if F <= 1024 else 2
    h.set_option("hist_variant", generic)
    assert_tree_bits(h.grow_tree(js, gp, mask=mask, cond=cond), t_fx)
    # the per-node padding of the span space only moves work between blocks
    for variant, cost in ((generic, 0), (2, 7), (generic, 5000)):
        h.set_option("hist_variant", variant)
        h.set_option("hist_seg_cost", cost)
        assert_tree_bits(h.grow_tree(js, gp, mask=mask, cond=cond), t_fx)
    h.close()
    o.close()


def test_categorical_and_monotone(evt):
    N, F, B, D = 30000, 6, 16, 5
    x_bin, y, w, mu = make_data(11, N, F, B, "mse", True)
    feattypes = np.array([1, 0, 1, 0, 1, 1], np.uint8)
    mono = np.array([1, 0, -1, 0, 0, 0], np.int32)
    h, o, op, gp, pred0, grad0 = setup_pair(evt, "mse", x_bin, y, w, mu, B, D, feattypes=feattypes, mono=mono)
    grad = grad0.copy()
    orc.update_grads(op, pred0, y, grad)
    h.set_grads(grad)
    js = np.arange(1, F + 1, dtype=np.uint32)
    rows = np.arange(N, dtype=np.uint32)
    t_gpu = h.grow_tree(js, gp)
    qb, qe = h.get_quant()
    o.set_quant(grad, qb)
    t_fx, nidx_fx = o.grow_tree(grad, rows, js, mode=1)
    assert_tree_bits(t_gpu, t_fx)
    assert np.array_equal(h.get_nidx(), nidx_fx)  # derived by walking the finished tree
    t_ref, _ = o.grow_tree(grad, rows, js, mode=0)
    assert_tree_close(t_gpu, t_ref)
    assert any(t_gpu.split[n] and feattypes[t_gpu.feat[n] - 1] == 0 for n in range(len(t_gpu.split)))
    h.close()
    o.close()


def test_tie_rule_and_empty_bins(evt):
    # duplicated columns: earliest feature of js wins; empty bin: lowest bin wins
    N, B = 4000, 16
    rng = np.random.default_rng(40)
    col = rng.integers(1, B + 1, N).astype(np.uint8)
    col[col == 7] = 8
    noise = rng.integers(1, B + 1, N).astype(np.uint8)
    x_bin = np.ascontiguousarray(np.stack([noise, col, col.copy(), col.copy()]))
    y = ((col > 6).astype(np.float32) + 0.01 * rng.random(N).astype(np.float32)).astype(np.float32)
    mu = np.zeros(1, np.float32)
    h, o, op, gp, pred0, grad0 = setup_pair(evt, "mse", x_bin, y, None, mu, B, 2)
    h.update_grads()
    t = h.grow_tree(np.array([1, 2, 3, 4], np.uint32), gp)
    assert (int(t.feat[0]), int(t.cond_bin[0])) == (2, 6)
    h.update_grads()
    t = h.grow_tree(np.array([1, 3, 4], np.uint32), gp)
    assert (int(t.feat[0]), int(t.cond_bin[0])) == (3, 6)
    h.close()
    o.close()


def test_min_weight_and_gamma_strict(evt):
    x_bin = np.array([[1, 1, 2, 2]], np.uint8)
    grad = np.array([[-1, 2, 1], [-1, 2, 1], [1, 2, 1], [1, 2, 1]], np.float32)
    y = np.zeros(4, np.float32)
    js = np.array([1], np.uint32)
    for minw, gamma, expect in [(1.999, 0.0, 1), (2.0, 0.0, 0), (1.0, 0.79, 1), (1.0, 0.8, 0), (1.0, 0.9, 0)]:
        h = evt.Handle(4, 1, 4, 1, 2, "mse")
        h.set_xbin(x_bin)
        h.set_target(y, None, np.zeros(1, np.float32))
        h.set_grads(grad)
        t = h.grow_tree(js, evt.make_params(min_weight=minw, gamma=gamma))
        assert int(t.split[0]) == expect, (minw, gamma)
        if expect:
            np.testing.assert_allclose(t.gain[0], 0.8, rtol=1e-6)
        h.close()


# --------------------------------------------------------------------------- free running boosting
@pytest.mark.parametrize("loss,tt,rowsample,colsample", [("mse", "binary", 1.0, 1.0), ("mse", "binary", 0.5, 0.5),
                                                         ("mse", "oblivious", 1.0, 1.0)])
def test_free_running_rounds_bit_exact_mse(evt, loss, tt, rowsample, colsample):
    # mse gradients are exact Float32 arithmetic, so GPU and fixed-point oracle stay bit identical
    # round after round without teacher forcing.
    N, F, B, D, R = 60000, 20, 64, 6, 12
    x_bin, y, w, mu = make_data(21, N, F, B, loss, False, signal=True)
    h, o, op, gp, pred0, grad0 = setup_pair(evt, loss, x_bin, y, w, mu, B, D, tt)
    rng = np.random.default_rng(5)
    p_orc = pred0.copy()
    grad = grad0.copy()
    nfs = int(np.ceil(colsample * F))
    for r in range(R):
        h.update_grads()
        orc.update_grads(op, p_orc, y, grad)
        js = (np.sort(rng.choice(F, nfs, replace=False)) + 1).astype(np.uint32)
        if rowsample < 1:
            mask = rng.integers(0, 256, N, dtype=np.uint8)
            cond = int(np.rint(255 * rowsample))
            rows = orc.subsample(mask, cond)
        else:
            mask, cond, rows = None, 255, np.arange(N, dtype=np.uint32)
        t_gpu = h.grow_tree(js, gp, mask=mask, cond=cond)
        qb, qe = h.get_quant()
        o.set_quant(grad, qb)
        t_fx, _ = o.grow_tree(grad, rows, js, mode=1)
        assert_tree_bits(t_gpu, t_fx)
        o.predict_tree(t_fx, p_orc)
    assert np.array_equal(h.get_pred().view(np.uint32), p_orc.view(np.uint32))
    h.close()
    o.close()


@pytest.mark.parametrize("weights", [False, True])
def test_free_running_40_rounds_headline_shape(evt, weights):
    # the headline workload's shape (100 features -> 128-byte records, 64 bins, deep trees) at a size the CPU side
    # finishes in seconds: 40 free-running rounds, every tree and the final predictions bit identical
    N, F, B, D, R = 300000, 100, 64, 9, 40
    x_bin, y, w, mu = make_data(23, N, F, B, "mse", weights, signal=True)
    h, o, op, gp, pred0, grad0 = setup_pair(evt, "mse", x_bin, y, w, mu, B, D, eta=0.3)
    p_orc = pred0.copy()
    grad = grad0.copy()
    js = np.arange(1, F + 1, dtype=np.uint32)
    rows = np.arange(N, dtype=np.uint32)
    nsplit = 0
    for r in range(R):
        h.update_grads()
        orc.update_grads(op, p_orc, y, grad)
        t_gpu = h.grow_tree(js, gp)
        qb, qe = h.get_quant()
        o.set_quant(grad, qb)
        t_fx, _ = o.grow_tree(grad, rows, js, mode=1, want_nidx=False)
        assert_tree_bits(t_gpu, t_fx)
        nsplit += int(t_gpu.split.sum())
        o.predict_tree(t_fx, p_orc)
    assert nsplit > 40 * 100  # the trees are deep ones, not stumps
    assert np.array_equal(h.get_pred().view(np.uint32), p_orc.view(np.uint32))
    h.close()
    o.close()


@pytest.mark.parametrize("loss", ["logloss", "gaussian_mle", "logistic_mle", "poisson", "gamma", "tweedie", "mlogloss"])
def test_free_running_rounds_tolerance(evt, loss):
    # device exp/log1p differ from the host's by an ulp: structure must still agree with the
    # reference arithmetic and predictions stay within 1e-5 over several rounds.
    N, F, B, D, R = 40000, 10, 32, 5, 8
    x_bin, y, w, mu = make_data(22, N, F, B, loss, False)
    pk = dict(min_weight=8.0) if loss in ("gaussian_mle", "logistic_mle") else {}
    h, o, op, gp, pred0, grad0 = setup_pair(evt, loss, x_bin, y, w, mu, B, D, **pk)
    p_orc = pred0.copy()
    grad = grad0.copy()
    js = np.arange(1, F + 1, dtype=np.uint32)
    rows = np.arange(N, dtype=np.uint32)
    for r in range(R):
        h.update_grads()
        orc.update_grads(op, p_orc, y, grad)
        t_gpu = h.grow_tree(js, gp)
        t_ref, _ = o.grow_tree(grad, rows, js, mode=0)
        # here the two sides' gradients already differ by an ulp (device vs host exp), and a leaf whose gradient sum
        # nearly cancels amplifies that: leaf values of ~1e-2 typical size get an absolute floor of 1e-5 of that size
        assert_tree_close(t_gpu, t_ref, pred_atol=1e-7)
        o.predict_tree(t_ref, p_orc)
    np.testing.assert_allclose(h.get_pred(), p_orc, rtol=RTOL, atol=1e-6)
    h.close()
    o.close()


# --------------------------------------------------------------------------- inference
def test_model_predict_and_leaf_idx(evt):
    N, F, B, D, R = 20000, 8, 32, 5, 6
    for loss, Kc in (("mse", None), ("logloss", None), ("gaussian_mle", None), ("poisson", None), ("mlogloss", 3), ("mlogloss", 7)):
        x_bin, y, w, mu = make_data(31, N, F, B, loss, False, K=Kc)
        pk = dict(min_weight=8.0) if loss in ("gaussian_mle", "logistic_mle") else {}
        h, o, op, gp, pred0, grad0 = setup_pair(evt, loss, x_bin, y, w, mu, B, D, **pk)
        js = np.arange(1, F + 1, dtype=np.uint32)
        K = op.K
        bias = orc.Tree(K, 1)
        bias.pred[0] = mu
        trees = [bias]
        for r in range(R):
            h.update_grads()
            trees.append(h.grow_tree(js, gp))
        ft = np.ones(F, np.uint8)
        raw = evt._lib.predict_model(x_bin, ft, loss, K, trees, apply_link=False)
        want = np.zeros((N, K), np.float32)
        for t in trees:
            orc.predict_tree(orc.LOSS_IDS[loss], K, x_bin, ft, t, want)
        assert np.array_equal(raw.view(np.uint32), want.view(np.uint32))
        # the training cache followed the same path
        assert np.array_equal(h.get_pred().view(np.uint32), want.view(np.uint32))
        linked = evt._lib.predict_model(x_bin, ft, loss, K, trees, apply_link=True)
        orc.apply_link(orc.LOSS_IDS[loss], K, want)
        np.testing.assert_allclose(linked, want, rtol=RTOL, atol=1e-7)
        leaves = evt._lib.predict_leaf_idx(x_bin, ft, trees)
        assert leaves.shape == (N, len(trees)) and leaves.dtype == np.uint32
        for j, t in enumerate(trees):
            assert np.array_equal(leaves[:, j], orc.predict_leaf_idx(x_bin, ft, t))
            assert not t.split[leaves[:, j] - 1].any()  # a returned node is never a split node
        assert (leaves[:, 0] == 1).all()
        # ntree_limit prefix property
        assert np.array_equal(evt._lib.predict_leaf_idx(x_bin, ft, trees[:3]), leaves[:, :3])
        h.close()
        o.close()


def _random_tree(rng, depth, F, B, K):
    nn = (1 << depth) - 1
    t = orc.Tree(K, nn)
    for n in range(1, 1 << (depth - 1)):
        if n == 1 or (t.split[(n >> 1) - 1] and rng.random() < 0.8):
            t.feat[n - 1] = rng.integers(1, F + 1)
            t.cond_bin[n - 1] = rng.integers(1, B)
            t.split[n - 1] = 1
    t.pred[:] = (rng.standard_normal((nn, K)) * 0.3).astype(np.float32)
    return t


@pytest.mark.parametrize("N,F,B,depths,K,loss", [
    (3001, 700, 16, [3, 5, 1, 4], 1, "mse"),          # wide matrix
    (70000, 9, 64, [15, 3, 15], 1, "logloss"),        # large trees, trees of different sizes in one model
    (5000, 40, 255, [6, 6, 2], 6, "mlogloss"),        # many outputs
    (1025, 3, 4, [2, 12], 2, "gaussian_mle"),         # odd row count
    (64 * 512, 100, 64, [11] * 5, 1, "mse"),          # the benchmark's shape
    # models that take the kernel walking completed trees in LDS, in each of its launch shapes: 1024 rows x 4 trees side by
    # side, 512 x 2, 512 x 1, 256 x 1; tree counts that do not fill the last group, stumps and bias trees in between,
    # row counts that do not fill the last block, the deepest trees each shape takes
    (4097, 150, 32, [7, 3, 7, 1, 6, 7], 1, "mse"),
    (3000, 150, 32, [10, 10, 2, 10, 10], 2, "gaussian_mle"),
    (2000, 250, 16, [5, 6, 6, 4], 1, "logloss"),
    (100001, 20, 64, [12] * 7 + [1, 12], 1, "mse"),
    (20000, 12, 64, [13, 2, 13, 13, 1], 1, "poisson"),
    (777, 5, 8, [1, 1, 1, 1, 1], 1, "mse"),
    (5000, 33, 16, [6] * 9, 2, "gaussian_mle"),
    (4000, 20, 16, [5, 7, 1, 7], 2, "logistic_mle"),
    (3000, 9, 32, [4] * 5, 6, "logistic_mle"),
    # more than four outputs walked from LDS: two trees side by side up to 8 outputs, one at a time up to 16
    (9000, 100, 64, [11, 11, 3, 11, 11, 11], 8, "mlogloss"),
    (5000, 28, 128, [8] * 7, 16, "mlogloss"),
    (4097, 150, 32, [7, 3, 7, 1, 6, 7], 5, "mse"),
    (3000, 250, 16, [5, 6, 6, 4, 6], 12, "poisson"),
])
@pytest.mark.parametrize("categorical", [True, False])
def test_model_predict_random_trees(evt, N, F, B, depths, K, loss, categorical):
    rng = np.random.default_rng(77)
    x_bin = rng.integers(1, B + 1, size=(F, N), dtype=np.uint8)
    ft = (rng.random(F) > 0.2).astype(np.uint8) if categorical else np.ones(F, np.uint8)
    trees = [_random_tree(rng, d, F, B, K) for d in depths]
    want = np.zeros((N, K), np.float32)
    for t in trees:
        orc.predict_tree(orc.LOSS_IDS[loss], K, x_bin, ft, t, want)
    raw = evt._lib.predict_model(x_bin, ft, loss, K, trees, apply_link=False)
    assert np.array_equal(raw.view(np.uint32), want.view(np.uint32))
    linked = evt._lib.predict_model(x_bin, ft, loss, K, trees, apply_link=True)
    orc.apply_link(orc.LOSS_IDS[loss], K, want)
    np.testing.assert_allclose(linked, want, rtol=RTOL, atol=1e-7)


def test_predict_tree_on_cache_and_clamps(evt):
    x_bin = np.array([[1, 2, 2]], np.uint8)
    t = orc.Tree(1, 3)
    t.feat[0], t.cond_bin[0], t.split[0] = 1, 1, 1
    t.pred[1, 0], t.pred[2, 0] = 20.0, -20.0
    for loss, want in (("logloss", [15.0, -15.0, -15.0]), ("mse", [21.0, -19.0, -19.0])):
        h = evt.Handle(3, 1, 4, 1, 2, loss)
        h.set_xbin(x_bin)
        h.set_target(np.zeros(3, np.float32), None, np.ones(1, np.float32))
        h.predict_tree(t)
        assert h.get_pred()[:, 0].tolist() == want
        h.close()
    t2 = orc.Tree(2, 3)
    t2.feat[0], t2.cond_bin[0], t2.split[0] = 1, 1, 1
    t2.pred[1] = [100.0, 100.0]
    t2.pred[2] = [-100.0, -100.0]
    h = evt.Handle(3, 1, 4, 2, 2, "gaussian_mle")
    h.set_xbin(x_bin)
    h.set_target(np.zeros(3, np.float32), None, np.zeros(2, np.float32))
    h.predict_tree(t2)
    assert h.get_pred().tolist() == [[100.0, 100.0], [-100.0, -15.0], [-100.0, -15.0]]
    h.close()


# --------------------------------------------------------------------------- binarize
def test_device_binarize(evt):
    rng = np.random.default_rng(3)
    N, F, B = 50000, 7, 64
    x = rng.random((F, N))
    edges = [np.sort(rng.random(B - 1)) for _ in range(F)]
    edges[2] = edges[2][:5]
    x[1, :63] = edges[1]  # values equal to an edge
    # the order is Julia's isless: NaN after everything (the last bin), -0.0 before 0.0; infinities at the ends
    edges[3] = np.sort(np.concatenate([-rng.random(30), [-0.0, 0.0], rng.random(31)]))
    x[3] = rng.standard_normal(N)
    x[3, :8] = [np.nan, -0.0, 0.0, np.inf, -np.inf, np.nan, 0.0, -0.0]
    x[4, ::11] = np.nan
    h = evt.Handle(N, F, B, 1, 2, "mse")
    h.binarize(x, edges)
    assert np.array_equal(h.get_xbin(), evt.binarize(x.T, edges))  # the host mirror's binarize (inference inputs) agrees
    assert np.array_equal(h.get_xbin()[3, :8], orc.binarize(x[3, :8], edges[3]))
    assert h.get_xbin()[3, 0] == 64 and h.get_xbin()[3, 2] == h.get_xbin()[3, 1] + 1
    # read the bins back through a one-split tree per feature: compare against the oracle's binarize
    h.set_target(np.zeros(N, np.float32), None, np.zeros(1, np.float32))
    for j in range(F):
        want = orc.binarize(x[j], edges[j])
        assert want.max() <= B
        for cb in (1, len(edges[j]) // 2 + 1, len(edges[j])):
            t = orc.Tree(1, 3)
            t.feat[0], t.cond_bin[0], t.split[0] = j + 1, cb, 1
            t.pred[1, 0], t.pred[2, 0] = 1.0, 0.0
            before = h.get_pred()[:, 0].copy()
            h.predict_tree(t)
            got_left = (h.get_pred()[:, 0] - before) == 1.0
            assert np.array_equal(got_left, want <= cb), (j, cb)
    h.close()


@pytest.mark.parametrize("loss,K", [("logloss", 6), ("gaussian_mle", 8), ("logistic_mle", 16), ("mlogloss", 8), ("mlogloss", 12), ("mlogloss", 16),
                                    ("mse", 5), ("poisson", 16)])
@pytest.mark.parametrize("ntrees", [3, 9])
def test_model_predict_many_outputs_with_clamps(evt, loss, K, ntrees):
    """More than four outputs (multi-class, several targets), with leaf values large enough that the per-tree clamps of
    predict! (src/predict.jl:16-62: [-15, 15] for logloss, floor -15 on the scale outputs and on the shifted mlogloss
    scores) act on most rows: 3 trees take the kernel that gathers from global memory, 9 trees the one that walks
    from LDS; both must equal the oracle's tree-by-tree predict!, bit for bit."""
    rng = np.random.default_rng(1234 + K)
    N, F, B = 6001, 37, 32
    x_bin = rng.integers(1, B + 1, size=(F, N), dtype=np.uint8)
    ft = np.ones(F, np.uint8)
    trees = []
    for d in [7, 4, 9, 1, 7, 8, 9, 3, 9][:ntrees]:
        t = _random_tree(rng, d, F, B, K)
        t.pred[:] = (rng.standard_normal(t.pred.shape) * 9.0).astype(np.float32)
        trees.append(t)
    want = np.zeros((N, K), np.float32)
    for t in trees:
        orc.predict_tree(orc.LOSS_IDS[loss], K, x_bin, ft, t, want)
    if loss in ("logloss", "gaussian_mle", "logistic_mle", "mlogloss"):
        assert (np.abs(want) == 15).any()  # a clamp was hit
    raw = evt._lib.predict_model(x_bin, ft, loss, K, trees, apply_link=False)
    assert np.array_equal(raw.view(np.uint32), want.view(np.uint32))
    if loss != "poisson":  # exp of sums of this size overflows Float32 on both sides
        linked = evt._lib.predict_model(x_bin, ft, loss, K, trees, apply_link=True)
        orc.apply_link(orc.LOSS_IDS[loss], K, want)
        np.testing.assert_allclose(linked, want, rtol=RTOL, atol=1e-7)


# --------------------------------------------------------------------------- error paths (forced from the host)
def test_error_paths(evt):
    N, F, B = 1000, 3, 8
    x_bin, y, w, mu = make_data(50, N, F, B)
    h = evt.Handle(N, F, B, 1, 3, "mse")
    bad = x_bin.copy()
    bad[1, 5] = B + 1
    with pytest.raises(evt.EvtError) as e:
        h.set_xbin(bad)
    assert e.value.code == evt._lib.EVT_ERR_ARG
    bad[1, 5] = 0
    with pytest.raises(evt.EvtError):
        h.set_xbin(bad)
    gp = evt.make_params()
    with pytest.raises(evt.EvtError) as e:  # nothing uploaded yet
        h.grow_tree(np.array([1], np.uint32), gp)
    assert e.value.code == evt._lib.EVT_ERR_STATE
    h.set_xbin(x_bin)
    h.set_target(y, None, mu)
    h.update_grads()
    for js in ([0], [4], [2, 2], [3, 1]):
        with pytest.raises(evt.EvtError) as e:
            h.grow_tree(np.array(js, np.uint32), gp)
        assert e.value.code == evt._lib.EVT_ERR_ARG
    with pytest.raises(evt.EvtError) as e:  # "no subsample observation"
        h.grow_tree(np.array([1, 2, 3], np.uint32), gp, mask=np.full(N, 200, np.uint8), cond=3)
    assert e.value.code == evt._lib.EVT_ERR_EMPTY
    assert "no subsample observation" in str(e.value)
    # the handle is still usable afterwards
    t = h.grow_tree(np.array([1, 2, 3], np.uint32), gp)
    assert t.split[0] == 1
    # gradients handed in from outside: with no weights given to evt_set_target the weight row must be all ones
    g = h.get_grads()
    g[17, 2] = 0.5
    with pytest.raises(evt.EvtError) as e:
        h.set_grads(g)
    assert e.value.code == evt._lib.EVT_ERR_ARG and "weight row" in str(e.value)
    with pytest.raises(evt.EvtError) as e:  # ... and leaves no gradients behind
        h.grow_tree(np.array([1, 2, 3], np.uint32), gp)
    assert e.value.code == evt._lib.EVT_ERR_STATE
    g[17, 2] = 1.0
    h.set_grads(g)
    assert h.grow_tree(np.array([1, 2, 3], np.uint32), gp).split[0] == 1
    h.close()
    # model offsets are checked before anything is sized by them: no exception crosses the C ABI
    import ctypes as C
    L = evt._lib.load()
    P = evt._lib.ptr
    feat = np.zeros(3, np.int64); cb = np.zeros(3, np.uint8); sp = np.zeros(3, np.uint8); pr = np.zeros(3, np.float32)
    out = np.zeros(N, np.float32)
    for off in ([0, -5], [2, 3], [0, 0], [0, 1 << 40], [-(1 << 62), 3]):
        off = np.array(off, np.int64)
        rc = L.evt_predict(N, F, P(x_bin), None, 0, 1, 1, P(off), P(feat), P(cb), P(pr), P(sp), 0, P(out))
        assert rc == evt._lib.EVT_ERR_ARG, (off, rc)
        assert b"tree_off" in L.evt_last_error() or b"2^31" in L.evt_last_error()
    for args in [(0, 3, 8, 1, 3, "mse"), (10, 0, 8, 1, 3, "mse"), (10, 3, 1, 1, 3, "mse"), (10, 3, 256, 1, 3, "mse"),
                 (10, 3, 8, 17, 3, "mse"), (10, 3, 8, 3, 3, "gaussian_mle"), (10, 3, 8, 1, 3, "mlogloss"), (10, 3, 8, 1, 0, "mse"),
                 (10, 3, 8, 1, 17, "mse")]:
        with pytest.raises(evt.EvtError):
            evt.Handle(*args)


# --------------------------------------------------------------------------- host API mirror
def test_fit_and_functor_reduce_error(evt):
    # the reference's own acceptance criterion (test/core.jl:25-57): error drops by >= 75 % on the sinus data
    rng = np.random.default_rng(123)
    feats = rng.random(1000) * 5
    X = feats.reshape(-1, 1)
    Y = np.sin(feats) * 0.5 + 0.5
    Y = 1 / (1 + np.exp(-(np.log(Y / (1 - Y)) + rng.standard_normal(1000))))
    idx = rng.permutation(1000)
    tr, ev = idx[:800], idx[800:]
    for cfg, metric in [
        (evt.EvoTreeRegressor(loss="mse", nrounds=100, nbins=16, lambda_=0.5, gamma=0.1, eta=0.1, max_depth=6, rowsample=0.5), "mse"),
        (evt.EvoTreeRegressor(loss="logloss", nrounds=100, nbins=16, lambda_=0.5, gamma=0.1, eta=0.1, max_depth=6, rowsample=0.5), "mse"),
        (evt.EvoTreeMLE(nrounds=100, nbins=16, lambda_=0.5, gamma=0.1, eta=0.1, max_depth=6, rowsample=0.5), "mse"),
        (evt.EvoTreeMLE(loss="logistic_mle", nrounds=100, nbins=16, lambda_=0.5, gamma=0.1, eta=0.1, max_depth=6, rowsample=0.5), "mse"),
        (evt.EvoTreeRegressor(loss="mse", nrounds=100, nbins=32, eta=0.1, max_depth=4, tree_type="oblivious"), "mse"),
    ]:
        m0, cache = evt.init(cfg, X[tr], Y[tr])
        cache.handle.close()
        p0 = m0(X[ev])
        m = evt.fit(cfg, x_train=X[tr], y_train=Y[tr])
        p = m(X[ev])
        if m.K == 2:
            assert (p[:, 1] > 0).all()
            p0, p = p0[:, 0], p[:, 0]
        e0, e1 = np.mean((p0 - Y[ev]) ** 2), np.mean((p - Y[ev]) ** 2)
        assert e1 / e0 - 1 < -0.75, (cfg.loss, cfg.tree_type, e0, e1)
        assert len(m.trees) == 101 and m.info["nrounds"] == 100
        m2 = evt.fit(cfg, x_train=X[tr], y_train=Y[tr])
        assert np.array_equal(m2(X[ev]), m(X[ev]))  # two fits with one config agree exactly (test/core.jl:101-102)
        assert np.array_equal(evt.predict(m, X[ev], ntree_limit=3), evt.EvoTree(m.loss_type, m.K, m.trees[:3], m.info)(X[ev]))
        with pytest.raises(RuntimeError):
            evt.predict(m, X[ev], ntree_limit=len(m.trees) + 1)
    m1 = evt.fit(evt.EvoTreeRegressor(nrounds=3, max_depth=1), x_train=X[tr], y_train=Y[tr])
    assert (evt.predict_leaf_idx(m1, X[ev]) == 1).all()  # a stump has a single leaf (test/predict-leaf-idx.jl:70-73)
    with pytest.raises(RuntimeError, match="no subsample observation"):
        xs = rng.random((40, 3))
        evt.fit(evt.EvoTreeRegressor(nrounds=5, max_depth=3, rowsample=0.001, min_weight=0.0, seed=1), x_train=xs, y_train=xs[:, 0])
