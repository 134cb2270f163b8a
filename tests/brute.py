"""Independent numpy re-derivation used to pin the C oracle on small inputs.

It shares no code with oracle/evo_oracle.c and is organised differently on purpose:
rows carry a node label (no row lists, no stable partition), every node's histogram is
built directly from its rows (no parent-minus-sibling), left sums come from numpy cumsum
and the split search is a dense array expression with a first-occurrence argmax.
"""
import numpy as np

EPS = np.finfo(np.float64).eps


def dense_hist(x_bin_FN, grad, rows, nbins):
    """hist[j, b, k] = sum over rows of grad[row, k] where x_bin[j, row] == b+1 (Float64)."""
    F = x_bin_FN.shape[0]
    NK = grad.shape[1]
    h = np.zeros((F, nbins, NK), np.float64)
    g = grad[rows].astype(np.float64)
    for j in range(F):
        b = x_bin_FN[j, rows].astype(np.int64) - 1
        for k in range(NK):
            np.add.at(h[j, :, k], b, g[:, k])
    return h


def term(g, h, w, lam, L2):
    return g * g / np.maximum(EPS, h + lam * w + L2) / 2.0


def leaf_value(S, K, eta, lam, L2, bagging=1):
    return np.array([-eta / bagging * S[k] / max(EPS, S[K + k] + lam * S[2 * K] + L2) for k in range(K)])


def gains_matrix(h, S, js, feattypes, mono, K, lam, L2, min_weight, eta):
    """Returns gains[jpos, bin] (-inf where not a candidate), for features js (1-based)."""
    nbins = h.shape[1]
    out = np.full((len(js), nbins), -np.inf)
    gp = sum(term(S[k], S[K + k], S[2 * K], lam, L2) for k in range(K))
    for jp, j in enumerate(js):
        hj = h[j - 1]
        if feattypes[j - 1]:
            L = np.cumsum(hj, axis=0)[: nbins - 1]
        else:
            L = hj.copy()
        wl = L[:, 2 * K]
        wr = S[2 * K] - wl
        ok = (wl > min_weight) & (wr > min_weight)
        g = np.zeros(L.shape[0])
        for k in range(K):
            g = g + (term(L[:, k], L[:, K + k], wl, lam, L2) + term(S[k] - L[:, k], S[K + k] - L[:, K + k], wr, lam, L2))
        g = g - gp
        if mono[j - 1] != 0:
            pl = -eta * L[:, 0] / np.maximum(EPS, L[:, K] + lam * wl + L2)
            R = S[None, :] - L
            pr = -eta * R[:, 0] / np.maximum(EPS, R[:, K] + lam * wr + L2)
            ok &= (pl > pr) if mono[j - 1] == -1 else (pl < pr)
        out[jp, : L.shape[0]] = np.where(ok, g, -np.inf)
    return out


def grow(x_bin_FN, grad, rows, js, K, nbins, max_depth, eta=0.1, lam=0.0, L2=1.0, gamma=0.0, min_weight=1.0,
         feattypes=None, mono=None, oblivious=False):
    F, N = x_bin_FN.shape
    feattypes = np.ones(F, bool) if feattypes is None else np.asarray(feattypes, bool)
    mono = np.zeros(F, int) if mono is None else np.asarray(mono, int)
    nn = 2 ** max_depth - 1
    T = dict(feat=np.zeros(nn, np.int64), cond_bin=np.zeros(nn, np.uint8), w=np.zeros(nn, np.float32),
             gain=np.zeros(nn, np.float32), pred=np.zeros((nn, K), np.float32), split=np.zeros(nn, np.uint8))
    label = np.zeros(N, np.int64)
    label[rows] = 1
    sums = {1: grad[rows].astype(np.float64).sum(axis=0)}
    hists = {}
    active = [1]
    for depth in range(1, max_depth + 1):
        if not active:
            break
        if depth == max_depth:
            for n in active:
                T["w"][n - 1] = sums[n][2 * K]
                T["pred"][n - 1] = leaf_value(sums[n], K, eta, lam, L2)
            break
        G = {}
        for n in active:
            r = np.flatnonzero(label == n)
            hists[n] = dense_hist(x_bin_FN, grad, r, nbins)
            T["w"][n - 1] = sums[n][2 * K]
            G[n] = gains_matrix(hists[n], sums[n], js, feattypes, mono, K, lam, L2, min_weight, eta)
        decisions = {}
        if not oblivious:
            for n in active:
                g = G[n]
                flat = g.ravel()  # js-major, bin-minor: first occurrence = first in (js, bin) order
                i = int(np.argmax(flat))
                if flat[i] > gamma:
                    decisions[n] = (float(flat[i]), int(js[i // g.shape[1]]), i % g.shape[1] + 1)
        else:
            tot = np.zeros_like(G[active[0]])
            allpos = np.ones(tot.shape, bool)
            for n in active:
                g0 = np.where(np.isfinite(G[n]), G[n], 0.0)
                tot = tot + g0
                if n > 1:
                    allpos &= g0 > 0
            lvl = np.where(allpos, tot, 0.0)
            i = int(np.argmax(lvl.ravel()))
            if lvl.ravel()[i] > gamma:
                for n in active:
                    decisions[n] = (float(lvl.ravel()[i]), int(js[i // lvl.shape[1]]), i % lvl.shape[1] + 1)
        nxt = []
        for n in active:
            if n in decisions:
                gain, feat, b = decisions[n]
                T["gain"][n - 1] = gain
                T["feat"][n - 1] = feat
                T["cond_bin"][n - 1] = b
                T["split"][n - 1] = 1
                r = np.flatnonzero(label == n)
                xb = x_bin_FN[feat - 1, r]
                goleft = (xb <= b) if feattypes[feat - 1] else (xb == b)
                label[r[goleft]] = 2 * n
                label[r[~goleft]] = 2 * n + 1
                hj = hists[n][feat - 1]
                SL = hj[:b].sum(axis=0) if feattypes[feat - 1] else hj[b - 1].copy()
                sums[2 * n] = SL
                sums[2 * n + 1] = sums[n] - SL
                nxt += [2 * n, 2 * n + 1]
            else:
                T["pred"][n - 1] = leaf_value(sums[n], K, eta, lam, L2)
        active = nxt
    return T, label, hists, sums


def walk(x_bin_FN, feattypes, T, i):
    nid = 1
    while T["split"][nid - 1]:
        f = T["feat"][nid - 1]
        xb = x_bin_FN[f - 1, i]
        cond = xb <= T["cond_bin"][nid - 1] if feattypes[f - 1] else xb == T["cond_bin"][nid - 1]
        nid = 2 * nid + (0 if cond else 1)
    return nid
