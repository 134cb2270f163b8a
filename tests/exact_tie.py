"""Exact comparison of two split candidates of one node, from the device's integer histogram.

The device accumulates fixed-point integers, so the decoded histogram of a node holds exact dyadic rationals and the
split gain of a candidate (src/split.jl:1, :108-117: sum over outputs of g^2 / max(eps, h + lambda w + L2) / 2 for the
left and the right side) can be evaluated in rational arithmetic.  Two candidates whose rational gains are EQUAL tie in
real arithmetic: the device resolves such a tie by position (lowest bin, then earliest feature), the reference by
Float64 rounding noise.  That is the only structural difference from the Float64 reference a test may accept; any other
is a parity failure."""
from fractions import Fraction

import numpy as np

EPS64 = Fraction(float(np.finfo(np.float64).eps))


def _side_gain(s, K, lam, L2):
    w = s[2 * K]
    tot = Fraction(0)
    for k in range(K):
        d = s[K + k] + lam * w + L2
        if d < EPS64:
            d = EPS64
        tot += s[k] * s[k] / d / 2
    return tot


def exact_split_gain(hist_nf, b, numeric, K, lam, L2):
    """hist_nf: (nbins, 2K+1) Float64 decoded integer histogram of one node and one feature; b: 1-based bin of the
    candidate; numeric: `<=` split, else `==` (src/fit-utils.jl:472-486).  Returns the split gain (parent's gain not
    subtracted: it is common to all candidates of a node) as a Fraction."""
    lam, L2 = Fraction(float(lam)), Fraction(float(L2))
    nb, nk = hist_nf.shape
    rows = [[Fraction(float(v)) for v in hist_nf[i]] for i in range(nb)]
    tot = [sum(rows[i][k] for i in range(nb)) for k in range(nk)]
    sel = range(0, b) if numeric else range(b - 1, b)
    left = [sum(rows[i][k] for i in sel) for k in range(nk)]
    right = [tot[k] - left[k] for k in range(nk)]
    return _side_gain(left, K, lam, L2) + _side_gain(right, K, lam, L2)


def first_difference(t_a, t_b):
    """1-based id of the first node (heap order) where the two trees choose differently, or 0."""
    d = np.flatnonzero((t_a.feat != t_b.feat) | (t_a.cond_bin != t_b.cond_bin) | (t_a.split != t_b.split))
    return int(d[0]) + 1 if d.size else 0


def is_exact_tie(H, t_gpu, t_ref, feattypes, K, lam, L2, oblivious=False):
    """H: the device's decoded histogram [node, feature, bin, k] (evt_get_hist).  At the first node where the trees
    differ, are the two chosen candidates equal in real arithmetic?  Returns (tie, text) where text names the node, both
    candidates and their gains.  A tree whose levels share one split (oblivious) compares the level's summed gains."""
    n0 = first_difference(t_gpu, t_ref)
    if n0 == 0:
        return True, "no difference"
    if not (t_gpu.split[n0 - 1] and t_ref.split[n0 - 1]):
        return False, "node %d: split on one side only (gpu %d, reference %d)" % (n0, t_gpu.split[n0 - 1], t_ref.split[n0 - 1])
    ca = (int(t_gpu.feat[n0 - 1]), int(t_gpu.cond_bin[n0 - 1]))
    cb = (int(t_ref.feat[n0 - 1]), int(t_ref.cond_bin[n0 - 1]))
    if oblivious:
        lvl0 = 1 << (n0.bit_length() - 1)
        nodes = [n for n in range(lvl0, 2 * lvl0) if t_gpu.w[n - 1] > 0]
    else:
        nodes = [n0]

    def total(c):
        f, b = c
        num = feattypes is None or bool(feattypes[f - 1])
        return sum(exact_split_gain(H[n - 1][f - 1], b, num, K, lam, L2) for n in nodes)

    ga, gb = total(ca), total(cb)
    text = "node %d: gpu (feat %d, bin %d) gain %.17g, reference (feat %d, bin %d) gain %.17g, exact difference %.3g" % (
        n0, ca[0], ca[1], float(ga), cb[0], cb[1], float(gb), float(ga - gb))
    return ga == gb, text
