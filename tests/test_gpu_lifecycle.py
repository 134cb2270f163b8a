"""Handle life cycle and isolation: handles are independent (own stream, own buffers), can be interleaved call by call,
created and destroyed repeatedly without leaking device memory, and give bit-identical trees whatever ran in between."""
import ctypes as C

import numpy as np
import pytest

from test_gpu_parity import assert_tree_bits, make_data

pytestmark = pytest.mark.gpu


def _free_bytes():
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(0), C.c_size_t(0)
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def _grow(evt, h, rounds, js, gp, mask_rng=None, N=None):
    trees = []
    for _ in range(rounds):
        h.update_grads()
        if mask_rng is None:
            trees.append(h.grow_tree(js, gp))
        else:
            trees.append(h.grow_tree(js, gp, mask=mask_rng.integers(0, 256, N, dtype=np.uint8), cond=150))
    return trees


def test_interleaved_handles_match_isolated_runs(evt):
    cfgs = [("mse", 30000, 12, 32, 6, "binary"), ("logloss", 20000, 100, 16, 5, "binary"), ("gaussian_mle", 15000, 7, 64, 4, "oblivious"),
            ("mlogloss", 10000, 9, 16, 4, "binary")]
    data = [make_data(60 + i, N, F, B, loss, weights=(i % 2 == 1)) for i, (loss, N, F, B, D, tt) in enumerate(cfgs)]

    def make(i):
        loss, N, F, B, D, tt = cfgs[i]
        x_bin, y, w, mu = data[i]
        h = evt.Handle(N, F, B, mu.shape[0], D, loss, tt)
        h.set_xbin(x_bin)
        h.set_target(y, w, mu)
        return h

    gp = evt.make_params(eta=0.2, min_weight=2.0)
    R = 4
    # isolated: one handle at a time
    iso = []
    for i, (loss, N, F, B, D, tt) in enumerate(cfgs):
        h = make(i)
        iso.append((_grow(evt, h, R, np.arange(1, F + 1, dtype=np.uint32), gp, np.random.default_rng(i), N), h.get_pred()))
        h.close()
    # interleaved: all handles alive, one round each in turn
    hs = [make(i) for i in range(len(cfgs))]
    rngs = [np.random.default_rng(i) for i in range(len(cfgs))]
    got = [[] for _ in cfgs]
    for r in range(R):
        for i, (loss, N, F, B, D, tt) in enumerate(cfgs):
            got[i] += _grow(evt, hs[i], 1, np.arange(1, F + 1, dtype=np.uint32), gp, rngs[i], N)
    for i in range(len(cfgs)):
        for a, b in zip(got[i], iso[i][0]):
            assert_tree_bits(a, b)
        assert np.array_equal(hs[i].get_pred().view(np.uint32), iso[i][1].view(np.uint32))
        hs[i].close()


def test_create_destroy_does_not_leak(evt):
    x_bin, y, w, mu = make_data(70, 200000, 50, 64, "mse", False)
    js = np.arange(1, 51, dtype=np.uint32)
    gp = evt.make_params()

    def cycle():
        h = evt.Handle(200000, 50, 64, 1, 7, "mse")
        h.set_xbin(x_bin)
        h.set_target(y, None, mu)
        h.update_grads()
        t = h.grow_tree(js, gp)
        evt._lib.predict_model(x_bin[:, :1000].copy(), None, "mse", 1, [t])
        h.eval_metric("mse")
        h.close()
        return t

    t0 = cycle()
    base = _free_bytes()
    for _ in range(15):
        assert_tree_bits(cycle(), t0)
    assert abs(_free_bytes() - base) < 32 * 1024 * 1024  # allocator granularity, not 15 x 100 MB


def test_calls_on_a_closed_or_null_handle_are_errors(evt):
    L = evt._lib.load()
    for call in (lambda: L.evt_update_grads(None), lambda: L.evt_synchronize(None), lambda: L.evt_eval_metric(None, 0, None),
                 lambda: L.evt_get_pred(None, None), lambda: L.evt_set_option(None, b"hist_blocks", 4)):
        assert call() == evt._lib.EVT_ERR_ARG
    h = evt.Handle(10, 2, 4, 1, 2, "mse")
    with pytest.raises(evt.EvtError):
        h.set_option("no_such_option", 1)
    with pytest.raises(evt.EvtError):
        h.set_option("hist_threads", 100)
    with pytest.raises(evt.EvtError) as ei:
        h.update_grads()  # no target yet
    assert ei.value.code == evt._lib.EVT_ERR_STATE
    h.close()
    h.close()  # idempotent


@pytest.mark.parametrize("loss,K,tt", [("mse", 1, "binary"), ("logloss", 1, "binary"), ("gaussian_mle", 2, "oblivious"), ("mlogloss", 3, "binary"),
                                       ("poisson", 1, "binary")])
def test_deferred_leaf_addition_equals_immediate(evt, loss, K, tt):
    """A tree grown on every row leaves its leaf values pending until the next pass over the rows (the next gradient
    update, or whatever reads the predictions first).  Every consumer must see them applied: predictions, metric,
    node ids, gradients and the following trees are bit-identical to the path that adds the values while growing -
    also with several trees per gradient update (bagging), a tree added from outside in between, and a subsampled
    tree (not deferred) after a deferred one."""
    N, F, B, D = 30000, 9, 32, 5
    x_bin, y, w, mu = make_data(77, N, F, B, loss, weights=True, K=K if loss == "mlogloss" else None)
    js = np.arange(1, F + 1, dtype=np.uint32)
    gp = evt.make_params(eta=0.3, bagging_size=2)
    metric = {"mse": "mse", "logloss": "logloss", "gaussian_mle": "gaussian_mle", "mlogloss": "mlogloss", "poisson": "poisson"}[loss]
    mask = np.random.default_rng(5).integers(0, 256, N, dtype=np.uint8)
    out = []
    for defer in (1, 0):
        h = evt.Handle(N, F, B, mu.shape[0], D, loss, tt)
        h.set_option("defer_pred", defer)
        h.set_xbin(x_bin)
        h.set_target(y, w, mu)
        rec = []
        for r in range(3):
            h.update_grads()
            rec.append(h.get_grads())
            t1 = h.grow_tree(js, gp)
            t2 = h.grow_tree(js, gp)            # second tree of the bag: the first one's values are still pending
            rec += [t1, t2, h.get_nidx(), h.eval_metric(metric)]
            if r == 1:
                h.predict_tree(t1)              # an outside tree on top of a pending one
                t3 = h.grow_tree(js, gp, mask=mask, cond=128)
                rec += [t3, h.get_pred()]
        rec.append(h.get_pred())
        h.set_target(y, w, mu)                  # a new target drops what is pending
        rec.append(h.get_pred())
        h.close()
        out.append(rec)
    for a, b in zip(*out):
        if isinstance(a, np.ndarray):
            assert a.tobytes() == b.tobytes()
        elif isinstance(a, float):
            assert a == b
        else:
            assert_tree_bits(a, b)


def test_mask_staged_while_the_last_tree_grows(evt):
    """evt_stage_mask + evt_grow_tree_begin_staged give the trees of evt_grow_tree with the same masks, bit for bit: the next
    mask is uploaded while a tree is in flight (and the host buffer is free again on return); a staged begin without a
    staged mask is refused; node ids derived afterwards use the mask of the tree they belong to."""
    N, F, B, D = 60000, 9, 32, 6
    x_bin, y, w, mu = make_data(17, N, F, B, "mse", weights=False)
    js = np.arange(1, F + 1, dtype=np.uint32)
    gp = evt.make_params(eta=0.3)
    rng = np.random.default_rng(8)
    masks = [rng.integers(0, 256, N, dtype=np.uint8) for _ in range(5)]
    conds = [128, 40, 255, 200, 128]

    def make():
        h = evt.Handle(N, F, B, 1, D, "mse")
        h.set_xbin(x_bin)
        h.set_target(y, w, mu)
        return h

    ha, hb = make(), make()
    with pytest.raises(evt.EvtError) as ei:
        hb.grow_tree_begin_staged(js, gp, 128)
    assert ei.value.code == evt._lib.EVT_ERR_STATE
    hb.update_grads()
    hb.stage_mask(masks[0].copy())
    for r in range(5):
        ha.update_grads()
        ta = ha.grow_tree(js, gp, mask=masks[r], cond=conds[r])
        if r > 0:
            hb.update_grads()
        hb.grow_tree_begin_staged(js, gp, conds[r])
        if r + 1 < 5:
            m = masks[r + 1].copy()
            hb.stage_mask(m)  # while tree r is in flight
            m[:] = 7          # the buffer is free again when the call returns
        tb = hb.grow_tree_end()
        assert_tree_bits(ta, tb)
        assert np.array_equal(ha.get_nidx(), hb.get_nidx()), r  # walks the tree with the mask of tree r, not of tree r + 1
    assert np.array_equal(ha.get_pred().view(np.uint32), hb.get_pred().view(np.uint32))
    with pytest.raises(evt.EvtError) as ei:
        hb.grow_tree_begin_staged(js, gp, 128)  # the last staged mask has been used
    assert ei.value.code == evt._lib.EVT_ERR_STATE
    ha.close()
    hb.close()


def test_mask_drawn_on_the_device(evt):
    """evt_draw_mask writes the bytes splitmix_mask computes on the host (pinned there by SplitMix64's published outputs):
    the rows in the tree are exactly those with byte <= cond, for thresholds that cut the bytes in different places and a
    row count that is not a multiple of eight, and the trees equal those grown from the same bytes uploaded.  A mask is
    used once."""
    N, F, B, D = 60003, 9, 32, 6
    x_bin, y, w, mu = make_data(23, N, F, B, "mse", weights=False)
    js = np.arange(1, F + 1, dtype=np.uint32)
    gp = evt.make_params(eta=0.3)

    def make():
        h = evt.Handle(N, F, B, 1, D, "mse")
        h.set_xbin(x_bin)
        h.set_target(y, w, mu)
        return h

    ha, hb = make(), make()
    seeds = [0, 1, 0xFFFFFFFFFFFFFFFF, 0x0123456789ABCDEF, 42, 7]
    conds = [128, 0, 254, 1, 77, 200]
    for r, (seed, cond) in enumerate(zip(seeds, conds)):
        mask = evt.splitmix_mask(seed, N)
        ha.update_grads()
        ta = ha.grow_tree(js, gp, mask=mask, cond=cond)
        hb.update_grads()
        hb.draw_mask(seed)
        hb.grow_tree_begin_staged(js, gp, cond)
        if r == 2:
            hb_next = seeds[r + 1]
            hb.draw_mask(hb_next)  # queued behind the tree in flight, used by the next round
        tb = hb.grow_tree_end()
        assert_tree_bits(ta, tb)
        nb = hb.get_nidx()
        assert np.array_equal(nb != 0, mask <= cond), (r, seed, cond)
        assert np.array_equal(ha.get_nidx(), nb)
        if r == 2:  # the mask drawn while tree 2 was in flight serves tree 3
            mask = evt.splitmix_mask(seeds[3], N)
            ha.update_grads()
            ta = ha.grow_tree(js, gp, mask=mask, cond=conds[3])
            hb.update_grads()
            hb.grow_tree_begin_staged(js, gp, conds[3])
            tb = hb.grow_tree_end()
            assert_tree_bits(ta, tb)
            assert np.array_equal(hb.get_nidx() != 0, mask <= conds[3])
    assert np.array_equal(ha.get_pred().view(np.uint32), hb.get_pred().view(np.uint32))
    with pytest.raises(evt.EvtError) as ei:
        hb.grow_tree_begin_staged(js, gp, 128)
    assert ei.value.code == evt._lib.EVT_ERR_STATE
    ha.close()
    hb.close()


def test_grow_tree_in_two_halves(evt):
    """evt_grow_tree_begin / evt_grow_tree_end give the trees and predictions of evt_grow_tree, bit for bit; between
    the two halves the handle refuses every call that reads or rewrites its state (and still answers afterwards); an end
    without a begin and an empty subsample are reported by the half that knows."""
    N, F, B, D = 40000, 11, 32, 6
    x_bin, y, w, mu = make_data(91, N, F, B, "logloss", weights=True)
    js = np.arange(1, F + 1, dtype=np.uint32)
    gp = evt.make_params(eta=0.2)
    rng_a, rng_b = np.random.default_rng(3), np.random.default_rng(3)

    def make():
        h = evt.Handle(N, F, B, 1, D, "logloss")
        h.set_xbin(x_bin)
        h.set_target(y, w, mu)
        return h

    ha, hb = make(), make()
    for r in range(4):
        sub = r % 2 == 1
        ha.update_grads()
        hb.update_grads()
        ma = rng_a.integers(0, 256, N, dtype=np.uint8) if sub else None
        mb = rng_b.integers(0, 256, N, dtype=np.uint8) if sub else None
        ta = ha.grow_tree(js, gp, mask=ma, cond=140)
        hb.grow_tree_begin(js, gp, mask=mb, cond=140)
        if sub:
            mb[:] = 0  # the mask has been read when begin returns
        for call in (hb.get_pred, hb.get_grads, lambda: hb.eval_metric("logloss"), lambda: hb.predict_tree(ta), lambda: hb.set_target(y, w, mu)):
            with pytest.raises(evt.EvtError) as ei:
                call()
            assert ei.value.code == evt._lib.EVT_ERR_STATE
        hb.synchronize()
        tb = hb.grow_tree_end()
        assert_tree_bits(ta, tb)
    assert np.array_equal(ha.get_pred().view(np.uint32), hb.get_pred().view(np.uint32))
    with pytest.raises(evt.EvtError) as ei:
        hb.grow_tree_end()
    assert ei.value.code == evt._lib.EVT_ERR_STATE
    hb.update_grads()
    hb.grow_tree_begin(js, gp, mask=np.full(N, 255, np.uint8), cond=10)  # keeps no row: the count is known at the end
    with pytest.raises(evt.EvtError) as ei:
        hb.grow_tree_end()
    assert ei.value.code == evt._lib.EVT_ERR_EMPTY
    hb.grow_tree(js, gp)  # the handle goes on working
    ha.close()
    hb.close()


@pytest.mark.parametrize("loss,tt,bagging,sub", [("mse", "binary", 1, False), ("mse", "binary", 1, True), ("logloss", "oblivious", 1, True),
                                                 ("gaussian_mle", "binary", 2, False), ("quantile", "binary", 1, True)])
def test_two_trees_in_flight(evt, loss, tt, bagging, sub):
    """The next tree (with its gradient update and its device-drawn mask) may be queued before the last one has been
    collected: evt_grow_tree_end then hands out the older tree.  Trees, gradients and predictions are those of calls
    strictly in turn, bit for bit, with and without the gradients queued ahead; with two trees in flight the handle
    takes nothing but the collection of the older one; per-level row counts in the profile stay those of each tree."""
    N, F, B, D, R = 50000, 10, 32, 6, 7
    x_bin, y, w, mu = make_data(33, N, F, B, loss, weights=(loss == "logloss"))
    rng = np.random.default_rng(5)
    jss = [np.sort(rng.choice(F, 7, replace=False)).astype(np.uint32) + 1 if r % 3 == 1 else np.arange(1, F + 1, dtype=np.uint32) for r in range(R)]
    seeds = [int(s) for s in rng.integers(0, 1 << 62, R)]
    gp = evt.make_params(eta=0.3, bagging_size=bagging, min_weight=8.0 if loss == "gaussian_mle" else 1.0)
    cond = 150

    def make(ahead):
        h = evt.Handle(N, F, B, mu.shape[0], D, loss, tt)
        h.set_option("grads_ahead", ahead)
        h.set_xbin(x_bin)
        h.set_target(y, w, mu)
        if loss == "quantile":
            h.set_alphas([0.3])
        return h

    def begin(h, r):
        if r % bagging == 0:
            h.update_grads()
        if sub:
            h.draw_mask(seeds[r])
            h.grow_tree_begin_staged(jss[r], gp, cond)
        else:
            h.grow_tree_begin(jss[r], gp)

    ha = make(0)
    ref = []
    for r in range(R):
        begin(ha, r)
        ref.append(ha.grow_tree_end())
    ha.update_grads()
    ref_state = [ha.get_grads(), ha.get_pred()]
    ha.close()
    for ahead in (0, 1) if bagging == 1 else (0,):
        hb = make(ahead)
        hb.set_profiling(["hist"])
        got = []
        begin(hb, 0)
        for r in range(1, R):
            begin(hb, r)  # tree r - 1 has not been collected
            if r == 2:
                for call in (hb.update_grads, lambda: hb.grow_tree_begin(jss[r], gp), lambda: hb.draw_mask(1), hb.get_pred,
                             lambda: hb.stage_mask(np.zeros(N, np.uint8)), lambda: hb.set_profiling(False)):
                    with pytest.raises(evt.EvtError) as ei:
                        call()
                    assert ei.value.code == evt._lib.EVT_ERR_STATE
            got.append(hb.grow_tree_end())
            if r == 4:
                with pytest.raises(evt.EvtError) as ei:
                    hb.get_pred()  # one tree is still in flight
                assert ei.value.code == evt._lib.EVT_ERR_STATE
        got.append(hb.grow_tree_end())
        with pytest.raises(evt.EvtError) as ei:
            hb.grow_tree_end()
        assert ei.value.code == evt._lib.EVT_ERR_STATE
        for a, b in zip(ref, got):
            assert_tree_bits(a, b)
        prof = hb.get_profile()["hist"]
        # rows built, as the histogram launches' events were matched with each tree's own per-level counts: the root
        # level of every tree holds the tree's sampled rows (= the root's weight for unit weights)
        if loss == "mse":
            assert prof["launches"] == R  # 16-byte records, few chunks: only the root's histogram is a launch of its own
            assert prof["units"] == sum(int(t.w[0]) for t in got)
        hb.update_grads()
        assert hb.get_grads().tobytes() == ref_state[0].tobytes()
        assert hb.get_pred().tobytes() == ref_state[1].tobytes()
        hb.close()


def test_empty_subsample_with_a_second_tree_in_flight(evt):
    """A tree whose mask keeps no row is reported when it is collected (EVT_ERR_EMPTY), also when the next tree has been
    queued behind it meanwhile; that next tree is collected as usual and equals the tree a handle grows that never saw
    the empty one (a tree on no rows is a single zero leaf: it changes no prediction)."""
    N, F, B, D = 30000, 8, 32, 5
    x_bin, y, w, mu = make_data(12, N, F, B, "mse", weights=False)
    js = np.arange(1, F + 1, dtype=np.uint32)
    gp = evt.make_params(eta=0.3)

    def make():
        h = evt.Handle(N, F, B, 1, D, "mse")
        h.set_xbin(x_bin)
        h.set_target(y, w, mu)
        return h

    ha, hb = make(), make()
    ha.update_grads()
    t0 = ha.grow_tree(js, gp)
    ha.update_grads()
    t1 = ha.grow_tree(js, gp)
    hb.update_grads()
    assert_tree_bits(t0, hb.grow_tree(js, gp))
    hb.update_grads()
    hb.grow_tree_begin(js, gp, mask=np.full(N, 255, np.uint8), cond=10)  # keeps no row
    hb.update_grads()
    hb.grow_tree_begin(js, gp)                                            # queued behind it
    with pytest.raises(evt.EvtError) as ei:
        hb.grow_tree_end()
    assert ei.value.code == evt._lib.EVT_ERR_EMPTY
    assert_tree_bits(t1, hb.grow_tree_end())
    assert ha.get_pred().tobytes() == hb.get_pred().tobytes()
    ha.close()
    hb.close()


@pytest.mark.parametrize("loss,tt", [("mse", "binary"), ("logloss", "oblivious"), ("gaussian_mle", "binary")])
def test_gradients_queued_ahead_change_nothing(evt, loss, tt):
    """With "grads_ahead" the gradient update of the next round is queued behind every tree and the next
    evt_update_grads only takes note; trees, gradients and predictions stay bit-identical, also when the predictions
    are changed from outside in between (evt_predict_tree, evt_set_target) or gradients are injected."""
    N, F, B, D = 30000, 9, 32, 5
    x_bin, y, w, mu = make_data(78, N, F, B, loss, weights=True)
    js = np.arange(1, F + 1, dtype=np.uint32)
    gp = evt.make_params(eta=0.3)
    mask = np.random.default_rng(6).integers(0, 256, N, dtype=np.uint8)
    out = []
    for ahead in (1, 0):
        h = evt.Handle(N, F, B, mu.shape[0], D, loss, tt)
        h.set_option("grads_ahead", ahead)
        h.set_xbin(x_bin)
        h.set_target(y, w, mu)
        rec = []
        for r in range(5):
            h.update_grads()
            rec.append(h.get_grads())
            t = h.grow_tree(js, gp, mask=mask if r == 2 else None, cond=128)
            rec.append(t)
            if r == 1:
                h.predict_tree(t)            # the predictions change after the gradients were queued
            if r == 3:
                g = rec[0].copy()
                h.set_grads(g)               # injected gradients replace the queued ones
                rec.append(h.grow_tree(js, gp))
        h.update_grads()
        rec += [h.get_grads(), h.get_pred()]
        h.set_target(y, w, mu)               # starts over: nothing queued survives
        h.update_grads()
        rec += [h.get_grads(), h.get_pred()]
        h.close()
        out.append(rec)
    for a, b in zip(*out):
        if isinstance(a, np.ndarray):
            assert a.tobytes() == b.tobytes()
        else:
            assert_tree_bits(a, b)


@pytest.mark.parametrize("loss,weights,rowsample", [("mse", False, 1.0), ("mse", True, 0.6), ("gaussian_mle", False, 1.0)])
def test_histograms_built_by_the_scatter_pass_change_nothing(evt, loss, weights, rowsample):
    """With 16-byte records and few chunks the levels below the root get their histograms from the partition's scatter
    pass ("hist_in_scatter", on by default) instead of a histogram kernel per level: trees, histograms, node ids and
    predictions are bit-identical either way over free-running rounds."""
    N, F, B, D, R = 100000, 10, 64, 6, 5
    x_bin, y, w, mu = make_data(91, N, F, B, loss, weights)
    js = np.array([1, 2, 4, 5, 6, 8, 9, 10], np.uint32)
    gp = evt.make_params(eta=0.4, min_weight=8.0 if loss == "gaussian_mle" else 1.0)
    rng = np.random.default_rng(17)
    masks = [None if rowsample >= 1 else rng.integers(0, 256, N, dtype=np.uint8) for _ in range(R)]
    out = []
    for on in (1, 0):
        h = evt.Handle(N, F, B, mu.shape[0], D, loss)
        h.set_option("hist_in_scatter", on)
        h.set_option("record_nidx", 1)
        h.set_xbin(x_bin)
        h.set_target(y, w, mu)
        rec = []
        for r in range(R):
            h.update_grads()
            rec.append(h.grow_tree(js if r % 2 else np.arange(1, F + 1, dtype=np.uint32), gp, mask=masks[r], cond=int(np.rint(255 * rowsample))))
            rec += [h.get_hist(), h.get_nidx()]
        rec.append(h.get_pred())
        h.close()
        out.append(rec)
    for a, b in zip(*out):
        if isinstance(a, np.ndarray):
            assert a.tobytes() == b.tobytes()
        else:
            assert_tree_bits(a, b)


@pytest.mark.parametrize("bagging", [1, 2])
def test_gradients_queued_ahead_with_bagging_and_read_back(evt, bagging):
    """A round of bagging_size trees is grown on ONE set of gradients (src/fit.jl:9-11): "grads_ahead" must not refresh
    them between the trees of a round.  And what describes the tree just grown - its histogram and its fixed-point
    tables - reads the same right after evt_grow_tree whether or not the next round's gradients were queued behind it."""
    N, F, B, D = 30000, 9, 32, 5
    x_bin, y, w, mu = make_data(79, N, F, B, "logloss", weights=True)
    js = np.arange(1, F + 1, dtype=np.uint32)
    gp = evt.make_params(eta=0.3, bagging_size=bagging)
    rng = np.random.default_rng(8)
    masks = [rng.integers(0, 256, N, dtype=np.uint8) for _ in range(8)]
    out = []
    for ahead in (1, 0):
        h = evt.Handle(N, F, B, 1, D, "logloss")
        h.set_option("grads_ahead", ahead)
        h.set_xbin(x_bin)
        h.set_target(y, w, mu)
        rec = []
        for r in range(3):
            h.update_grads()
            for b in range(bagging):
                t = h.grow_tree(js, gp, mask=masks[2 * r + b], cond=200)
                qb, qe = h.get_quant()
                rec += [t, h.get_hist(), qb, qe]
        rec.append(h.get_pred())
        h.close()
        out.append(rec)
    for a, b in zip(*out):
        if isinstance(a, np.ndarray):
            assert a.tobytes() == b.tobytes()
        else:
            assert_tree_bits(a, b)
    assert out[0][0].split.sum() >= 3


def test_two_handles_on_two_threads(evt):
    """Different handles may be driven from different threads at once (each has its own stream; the error message is
    per thread): two threads boost different problems concurrently and get, bit for bit, what a single thread gets."""
    import threading
    specs = [("mse", 60000, 20, 32, 6, 11), ("logloss", 45000, 9, 64, 5, 12)]

    def run(spec, out, k, barrier=None):
        loss, N, F, B, D, seed = spec
        x_bin, y, w, mu = make_data(seed, N, F, B, loss, weights=True)
        h = evt.Handle(N, F, B, 1, D, loss)
        h.set_xbin(x_bin)
        h.set_target(y, w, mu)
        gp = evt.make_params(eta=0.2)
        js = np.arange(1, F + 1, dtype=np.uint32)
        rng = np.random.default_rng(seed)
        trees = []
        if barrier is not None:
            barrier.wait()
        for r in range(12):
            h.update_grads()
            mask = rng.integers(0, 256, N, dtype=np.uint8) if r % 3 == 1 else None
            trees.append(h.grow_tree(js, gp, mask=mask, cond=150))
        try:
            h.grow_tree(np.array([F + 5], np.uint32), gp)  # an error on this thread: its message stays on this thread
        except evt.EvtError as e:
            out[k] = (trees, h.get_pred(), str(e))
        h.close()

    seq, par = {}, {}
    for k, s in enumerate(specs):
        run(s, seq, k)
    barrier = threading.Barrier(2)
    ths = [threading.Thread(target=run, args=(s, par, k, barrier)) for k, s in enumerate(specs)]
    for t in ths:
        t.start()
    for t in ths:
        t.join()
    for k in range(2):
        assert k in par, "thread %d did not finish" % k
        for ta, tb in zip(seq[k][0], par[k][0]):
            assert_tree_bits(ta, tb)
        assert np.array_equal(seq[k][1].view(np.uint32), par[k][1].view(np.uint32))
        assert "js entries" in par[k][2]


def test_size_limits_are_refused_with_a_message(evt):
    """What the library does not take is refused before anything is sized by it, with a message that names the limit:
    more than 16 outputs, trees deeper than 16, and - the one histogram shape without a wide-record kernel - more than 1024
    features when channels x bins exceed 512."""
    for args, word in (((100, 4, 8, 17, 3, "mse"), "16"), ((100, 4, 8, 1, 17, "mse"), "max_depth"), ((100, 65535, 8, 1, 3, "mse"), "nfeats"),
                       ((100, 4, 8, 34, 3, "gaussian_mle"), "16")):
        with pytest.raises(evt.EvtError) as ei:
            evt.Handle(*args)
        assert ei.value.code == evt._lib.EVT_ERR_ARG and word in str(ei.value)
    N, F, B = 2000, 1100, 255
    rng = np.random.default_rng(5)
    x_bin = rng.integers(1, B + 1, size=(F, N), dtype=np.uint8)
    y = rng.random(N).astype(np.float32)
    w = (rng.random(N) + 0.5).astype(np.float32)
    h = evt.Handle(N, F, B, 2, 3, "gaussian_mle")  # five channels x 255 bins: not even a 32-byte column tile fits the LDS
    h.set_xbin(x_bin)
    h.set_target(y, w, np.array([0.5, 0.1], np.float32))
    h.update_grads()
    with pytest.raises(evt.EvtError) as ei:
        h.grow_tree(np.arange(1, F + 1, dtype=np.uint32), evt.make_params(min_weight=8.0))
    assert ei.value.code == evt._lib.EVT_ERR_ARG and "1024 features" in str(ei.value)
    with pytest.raises(evt.EvtError):
        h.set_option("hist_variant", 1)
    # the same shape with unit weights needs four channels and 64 bins fit: it grows
    h.close()
    h = evt.Handle(N, F, 64, 2, 3, "gaussian_mle")
    h.set_xbin(np.minimum(x_bin, 64).astype(np.uint8))
    h.set_target(y, None, np.array([0.5, 0.1], np.float32))
    h.update_grads()
    t = h.grow_tree(np.arange(1, F + 1, dtype=np.uint32), evt.make_params(min_weight=8.0))
    assert t.w[0] == N
    h.close()
