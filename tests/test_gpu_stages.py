"""A tree grown one kernel stage at a time through the C ABI (evt_tree_open, then per level evt_hist_build,
evt_split_scan, evt_update_nodes_idx, then evt_tree_close): after every stage the device state is read back and checked
against the oracle, so each kernel is pinned on its own and not only through the finished tree.

 * after update_hist! of a level: exactly the smaller child of every pair (ties: the left one, src/fit.jl:123-129)
   carries a histogram, bit-equal to the fixed-point oracle's; the larger children carry none yet;
 * after the split search: every active node of the level has its histogram (parent - sibling materialised) and the
   tree arrays up to this level equal the oracle's, bit for bit;
 * after update_nodes_idx!: the node of every sampled row equals an independent walk of the oracle's tree cut at the
   next level (the rule of test/predict-leaf-idx.jl:34-49, level by level)."""
import numpy as np
import pytest

from oracle import oracle as orc
from test_gpu_parity import assert_tree_bits, make_data, setup_pair

pytestmark = pytest.mark.gpu


def walk_to_depth(t, x_bin, feattypes, rows, depth):
    """1-based node of each row after depth-1 decisions of tree t (rows that reach a leaf earlier stay there)."""
    nid = np.ones(rows.shape[0], np.int64)
    for _ in range(depth - 1):
        sp = t.split[nid - 1].astype(bool)
        f = np.where(sp, t.feat[nid - 1] - 1, 0)
        xb = x_bin[f, rows]
        cb = t.cond_bin[nid - 1]
        numeric = np.ones(rows.shape[0], bool) if feattypes is None else feattypes[f] != 0
        left = np.where(numeric, xb <= cb, xb == cb)
        nid = np.where(sp, 2 * nid + (~left), nid)
    return nid


CASES = [
    # loss, weights, N, F, B, D, tree_type, n_js, rowsample, K, categorical
    ("mse", False, 30011, 20, 32, 5, "binary", 20, 1.0, None, False),
    ("mse", True, 20000, 100, 64, 6, "binary", 50, 0.5, None, False),
    ("logloss", True, 15000, 28, 128, 4, "binary", 28, 0.8, None, True),
    ("gaussian_mle", False, 25000, 50, 64, 5, "binary", 50, 1.0, None, False),
    ("gaussian_mle", True, 12000, 33, 16, 4, "oblivious", 20, 1.0, None, True),
    ("mlogloss", True, 9000, 12, 16, 4, "binary", 12, 0.5, 5, False),
    ("mse", False, 5000, 7, 8, 1, "binary", 7, 1.0, None, False),
    ("poisson", False, 8000, 130, 255, 3, "binary", 130, 1.0, None, False),
]


@pytest.mark.parametrize("loss,weights,N,F,B,D,tt,n_js,rowsample,K,cat", CASES)
def test_every_stage_against_the_oracle(evt, loss, weights, N, F, B, D, tt, n_js, rowsample, K, cat):
    rng = np.random.default_rng(77)
    x_bin, y, w, mu = make_data(4242, N, F, B, loss, weights, K=K)
    feattypes = (rng.random(F) > 0.3).astype(np.uint8) if cat else None
    h, o, op, gp, pred0, grad0 = setup_pair(evt, loss, x_bin, y, w, mu, B, D, tt, feattypes=feattypes, min_weight=1.0)
    grad = grad0.copy()
    orc.update_grads(op, pred0, y, grad)
    h.set_grads(grad)
    js = (np.sort(rng.choice(F, n_js, replace=False)) + 1).astype(np.uint32)
    if rowsample < 1.0:
        mask = rng.integers(0, 256, N, dtype=np.uint8)
        cond = int(np.rint(255 * rowsample))
        rows = orc.subsample(mask, cond)
    else:
        mask, cond, rows = None, 255, np.arange(N, dtype=np.uint32)

    qb, qe = h.get_quant()  # fixed by the gradients, before the tree starts
    h.tree_open(js, gp, mask=mask, cond=cond)
    o.set_quant(grad, qb)
    assert np.array_equal(o.get_quant()[1], qe)
    t_fx, nidx_fx = o.grow_tree(grad, rows, js, mode=1)
    Hq = o.hist(fixed=True).copy()
    scale = np.ldexp(1.0, (qe - qb).astype(np.int64))
    nn = t_fx.feat.shape[0]

    def level_nodes(level):  # 0-based ids of the nodes of a level
        return range((1 << (level - 1)) - 1, min((1 << level) - 1, nn))

    def active(n0):  # visited by the oracle: the root, or a child of a split node
        return n0 == 0 or bool(t_fx.split[(n0 + 1) // 2 - 1])

    last_split = max(1, D - 1)
    for level in range(1, last_split + 1):
        print("level", level, flush=True)
        # ---- update_hist!
        h.hist_build(level)
        Hg = h.get_hist()
        cnt = np.bincount(walk_to_depth(t_fx, x_bin, feattypes, rows, level), minlength=nn + 2)
        for n0 in level_nodes(level):
            n = n0 + 1
            if not active(n0):
                assert not Hg[n0].any(), n
                continue
            if level == 1:
                built = True
            else:
                left, right = n & ~1, n | 1
                built = (n == left) == (cnt[right] >= cnt[left])  # the smaller child is built; a tie builds the left one
            if built:
                assert np.array_equal(Hg[n0][js - 1], Hq[n0][js - 1].astype(np.float64) * scale), ("built", n)
            elif tt == "binary":
                assert not Hg[n0].any(), ("larger child has a histogram before the split search", n)
        # ---- subtract_hist! + split search
        h.split_scan(level)
        Hg = h.get_hist()
        for n0 in level_nodes(level):
            if active(n0):
                assert np.array_equal(Hg[n0][js - 1], Hq[n0][js - 1].astype(np.float64) * scale), ("scanned", n0 + 1)
        t_now = h.peek_tree()
        upto = nn if level == last_split else (1 << level) - 1
        for name in ("feat", "cond_bin", "split"):
            assert np.array_equal(getattr(t_now, name)[:upto], getattr(t_fx, name)[:upto]), (name, level)
        assert np.array_equal(t_now.gain[:upto].view(np.uint32), t_fx.gain[:upto].view(np.uint32))
        assert np.array_equal(t_now.w[:upto].view(np.uint32), t_fx.w[:upto].view(np.uint32))
        leaves = [n0 for n0 in range(upto) if active(n0) and not t_fx.split[n0]]
        assert np.array_equal(t_now.pred[leaves].view(np.uint32), t_fx.pred[leaves].view(np.uint32))
        if level < last_split:
            assert not t_now.split[(1 << level) - 1:].any()  # nothing below this level has been searched yet
        # ---- update_nodes_idx!
        h.update_nodes_idx(level)
        want = np.zeros(N, np.uint32)
        want[rows] = walk_to_depth(t_fx, x_bin, feattypes, rows, min(level + 1, D))
        assert np.array_equal(h.get_nidx(), want), level
    h.tree_close()
    t_gpu = h.grow_tree_end()
    assert_tree_bits(t_gpu, t_fx)
    assert np.array_equal(h.get_nidx(), nidx_fx)
    p_orc = pred0.copy()
    o.predict_tree(t_fx, p_orc)
    assert np.array_equal(h.get_pred().view(np.uint32), p_orc.view(np.uint32))
    h.close()
    o.close()


def test_stage_order_is_enforced(evt):
    N, F, B, D = 4000, 6, 16, 3
    x_bin, y, w, mu = make_data(5, N, F, B, "mse", False)
    h, o, op, gp, pred0, grad0 = setup_pair(evt, "mse", x_bin, y, w, mu, B, D)
    h.update_grads()
    js = np.arange(1, F + 1, dtype=np.uint32)
    with pytest.raises(Exception, match="no tree is open"):
        h.hist_build(1)
    h.tree_open(js, gp)
    with pytest.raises(Exception, match="expects evt_hist_build\\(level 1\\)"):
        h.split_scan(1)
    with pytest.raises(Exception, match="expects evt_hist_build\\(level 1\\)"):
        h.hist_build(2)
    with pytest.raises(Exception, match="has not been closed"):
        h.update_grads()
    with pytest.raises(Exception, match="before the last level"):
        h.tree_close()
    for level in (1, 2):
        h.hist_build(level)
        with pytest.raises(Exception, match="expects evt_split_scan"):
            h.update_nodes_idx(level)
        h.split_scan(level)
        h.update_nodes_idx(level)
    with pytest.raises(Exception, match="expects evt_tree_close"):
        h.hist_build(3)
    h.tree_close()
    t_steps = h.grow_tree_end()
    # the same tree as the one-call form
    h.set_target(y, w, mu)
    h.update_grads()
    t_one = h.grow_tree(js, gp)
    assert_tree_bits(t_steps, t_one)
    h.close()
    o.close()
