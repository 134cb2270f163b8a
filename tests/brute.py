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


def cred_term(kind, m1, m2, w, L2):
    """Credibility-weighted absolute sum: Z |m1| / (1 + L2 / w) with Z = between / (between + within), on variances
    (cred_var) or on standard deviations (cred_std); the within-variance is floored at eps."""
    between = (m1 / w) ** 2
    within = np.maximum(EPS, m2 / w - between)
    if kind == "cred_std":
        between, within = np.sqrt(between), np.sqrt(within)
    return between / (between + within) * np.abs(m1) / (1.0 + L2 / w)


def side_terms(kind, S, L, K, wl, wr, lam, L2):
    """Gain of the two sides summed over the K outputs; L holds the left sums of every candidate (rows)."""
    g = np.zeros(L.shape[0])
    for k in range(K):
        if kind in ("mae", "quantile"):  # absolute shift of each side's mean first-row value from the parent's, weighted
            mu_p = S[k] / S[2 * K]
            dl = np.maximum(EPS, 1.0 + lam + L2 / wl)
            dr = np.maximum(EPS, 1.0 + lam + L2 / wr)
            g = g + (np.abs(L[:, k] / wl - mu_p) * wl / dl + np.abs((S[k] - L[:, k]) / wr - mu_p) * wr / dr)
        elif kind in ("cred_var", "cred_std"):
            g = g + (cred_term(kind, L[:, k], L[:, K + k], wl, L2) + cred_term(kind, S[k] - L[:, k], S[K + k] - L[:, K + k], wr, L2))
        else:
            g = g + (term(L[:, k], L[:, K + k], wl, lam, L2) + term(S[k] - L[:, k], S[K + k] - L[:, K + k], wr, lam, L2))
    return g


def parent_gain(kind, S, K, lam, L2):
    if kind in ("mae", "quantile"):
        return 0.0
    if kind in ("cred_var", "cred_std"):
        return sum(cred_term(kind, S[k], S[K + k], S[2 * K], L2) for k in range(K))
    return sum(term(S[k], S[K + k], S[2 * K], lam, L2) for k in range(K))


def leaf_value(S, K, eta, lam, L2, bagging=1, kind="gh"):
    if kind == "mae":
        return np.array([eta / bagging * S[k] / max(EPS, S[2 * K] + lam * S[2 * K] + L2) for k in range(K)])
    if kind in ("cred_var", "cred_std"):
        return np.array([eta / bagging * S[k] / (S[2 * K] + L2) for k in range(K)])
    return np.array([-eta / bagging * S[k] / max(EPS, S[K + k] + lam * S[2 * K] + L2) for k in range(K)])


def first_output_value(kind, L, K, w, eta, lam, L2):
    """Leaf value of output 1 for every candidate side (monotone constraints compare the two sides' values)."""
    if kind == "mae":
        return eta * L[:, 0] / np.maximum(EPS, w + lam * w + L2)
    if kind in ("cred_var", "cred_std"):
        return eta * L[:, 0] / (w + L2)
    return -eta * L[:, 0] / np.maximum(EPS, L[:, K] + lam * w + L2)


def gains_matrix(h, S, js, feattypes, mono, K, lam, L2, min_weight, eta, kind="gh"):
    """Returns gains[jpos, bin] (-inf where not a candidate), for features js (1-based)."""
    nbins = h.shape[1]
    out = np.full((len(js), nbins), -np.inf)
    gp = parent_gain(kind, S, K, lam, L2)
    for jp, j in enumerate(js):
        hj = h[j - 1]
        if feattypes[j - 1]:
            L = np.cumsum(hj, axis=0)[: nbins - 1]
        else:
            L = hj.copy()
        wl = L[:, 2 * K]
        wr = S[2 * K] - wl
        ok = (wl > min_weight) & (wr > min_weight)
        with np.errstate(divide="ignore", invalid="ignore"):
            g = side_terms(kind, S, L, K, wl, wr, lam, L2) - gp
            if mono[j - 1] != 0:
                pl = first_output_value(kind, L, K, wl, eta, lam, L2)
                pr = first_output_value(kind, S[None, :] - L, K, wr, eta, lam, L2)
                ok &= (pl > pr) if mono[j - 1] == -1 else (pl < pr)
        out[jp, : L.shape[0]] = np.where(ok, g, -np.inf)
    return out


def grow(x_bin_FN, grad, rows, js, K, nbins, max_depth, eta=0.1, lam=0.0, L2=1.0, gamma=0.0, min_weight=1.0,
         feattypes=None, mono=None, oblivious=False, kind="gh", alphas=None, clamp_denom=True):
    """kind "quantile": gains as mae on the first gradient rows; a leaf's value of output k is eta times numpy's
    linear-interpolation quantile (level alphas[k]) of the leaf's rows' residuals, row K + k of grad, over
    1 + lam + L2 / w (floored at eps when clamp_denom)."""
    F, N = x_bin_FN.shape
    feattypes = np.ones(F, bool) if feattypes is None else np.asarray(feattypes, bool)
    mono = np.zeros(F, int) if mono is None else np.asarray(mono, int)
    nn = 2 ** max_depth - 1
    T = dict(feat=np.zeros(nn, np.int64), cond_bin=np.zeros(nn, np.uint8), w=np.zeros(nn, np.float32),
             gain=np.zeros(nn, np.float32), pred=np.zeros((nn, K), np.float32), split=np.zeros(nn, np.uint8))
    label = np.zeros(N, np.int64)
    label[rows] = 1

    def leaf_of(n):
        if kind != "quantile":
            return leaf_value(sums[n], K, eta, lam, L2, kind=kind)
        r = np.flatnonzero(label == n)
        d = 1.0 + lam + L2 / sums[n][2 * K]
        if clamp_denom:
            d = max(EPS, d)
        return np.array([eta * np.quantile(grad[r, K + k].astype(np.float64), alphas[k], method="linear") / d for k in range(K)])

    sums = {1: grad[rows].astype(np.float64).sum(axis=0)}
    hists = {}
    active = [1]
    for depth in range(1, max_depth + 1):
        if not active:
            break
        if depth == max_depth:
            for n in active:
                T["w"][n - 1] = sums[n][2 * K]
                T["pred"][n - 1] = leaf_of(n)
            break
        G = {}
        for n in active:
            r = np.flatnonzero(label == n)
            hists[n] = dense_hist(x_bin_FN, grad, r, nbins)
            T["w"][n - 1] = sums[n][2 * K]
            G[n] = gains_matrix(hists[n], sums[n], js, feattypes, mono, K, lam, L2, min_weight, eta, kind=kind)
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
                T["pred"][n - 1] = leaf_of(n)
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
