"""Writes tests/golden/trees.json: small seeded inputs and the trees the CPU oracle (reference
arithmetic, mode 0) grows on them.

The reference holds no golden vectors for this path and cannot be run here (it is Julia; no Julia
toolchain is available), so these fixtures are generated from the oracle after it has been pinned
by tests/test_oracle_pins.py.  They freeze its behaviour: the oracle must keep reproducing them, and
the HIP path is checked against the same numbers.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as orc  # noqa: E402

CASES = [
    dict(name="mse_binary", loss="mse", N=256, F=4, B=8, D=3, tree_type="binary", weights=False, pk={}),
    dict(name="mse_weighted_lambda", loss="mse", N=300, F=5, B=8, D=4, tree_type="binary", weights=True, pk=dict(lambda_=0.5, gamma=0.01)),
    dict(name="logloss_binary", loss="logloss", N=256, F=4, B=16, D=3, tree_type="binary", weights=False, pk=dict(eta=0.05)),
    dict(name="gaussian_binary", loss="gaussian_mle", N=320, F=4, B=8, D=3, tree_type="binary", weights=False, pk=dict(min_weight=8.0)),
    dict(name="gaussian_oblivious", loss="gaussian_mle", N=320, F=4, B=8, D=3, tree_type="oblivious", weights=False, pk=dict(min_weight=8.0)),
    dict(name="mse_oblivious", loss="mse", N=256, F=4, B=8, D=4, tree_type="oblivious", weights=False, pk={}),
]


def build_case(c, seed):
    rng = np.random.default_rng(seed)
    N, F, B = c["N"], c["F"], c["B"]
    K = 2 if c["loss"] == "gaussian_mle" else 1
    x_bin = rng.integers(1, B + 1, size=(F, N), dtype=np.uint8)
    y = (rng.random(N) + 0.6 * (x_bin[0] / B) + 0.3 * (x_bin[F - 1] > B // 2)).astype(np.float32)
    if c["loss"] == "logloss":
        y = (y > np.median(y)).astype(np.float32)
    w = (rng.integers(1, 5, N) / 2).astype(np.float32) if c["weights"] else np.ones(N, np.float32)
    pred = np.round(rng.standard_normal((N, K)) * 0.25, 3).astype(np.float32)
    mask = rng.integers(0, 256, N, dtype=np.uint8)
    cond = 204  # round(255 * 0.8)
    rows = orc.subsample(mask, cond)
    js = np.array(sorted(rng.choice(F, F - 1, replace=False) + 1), np.uint32)
    p = orc.make_params(c["loss"], nbins=B, max_depth=c["D"], tree_type=c["tree_type"], **c["pk"])
    grad = np.zeros((N, 2 * K + 1), np.float32)
    grad[:, 2 * K] = w
    orc.update_grads(p, pred, y, grad)
    o = orc.Oracle(p, x_bin)
    t, nidx = o.grow_tree(grad, rows, js, mode=0)
    pred_after = pred.copy()
    o.predict_tree(t, pred_after)
    o.close()
    return dict(
        name=c["name"], loss=c["loss"], tree_type=c["tree_type"], N=N, F=F, B=B, D=c["D"], K=K, params=c["pk"], cond=cond,
        x_bin=x_bin.tolist(), y=y.tolist(), w=w.tolist(), weighted=c["weights"], pred=pred.tolist(), mask=mask.tolist(), js=js.tolist(),
        expect=dict(grad=[[float(v) for v in r] for r in grad], feat=t.feat.tolist(), cond_bin=t.cond_bin.tolist(), split=t.split.tolist(),
                    gain=[float(v) for v in t.gain], w=[float(v) for v in t.w], pred=[[float(v) for v in r] for r in t.pred],
                    nidx=nidx.tolist(), pred_after=[[float(v) for v in r] for r in pred_after]))


def main():
    out = [build_case(c, 1000 + i) for i, c in enumerate(CASES)]
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "trees.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
