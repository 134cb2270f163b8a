"""The oracle must keep reproducing the committed golden fixtures (tests/golden/trees.json)."""
import numpy as np
import pytest

from golden_util import load_cases
from oracle import oracle as orc

CASES = load_cases()


@pytest.mark.parametrize("c", CASES, ids=[c["name"] for c in CASES])
def test_oracle_reproduces_golden(c):
    e = c["expect"]
    p = orc.make_params(c["loss"], nbins=c["B"], max_depth=c["D"], tree_type=c["tree_type"], **c["params"])
    K = c["K"]
    grad = np.zeros((c["N"], 2 * K + 1), np.float32)
    grad[:, 2 * K] = c["w"]
    orc.update_grads(p, c["pred"], c["y"], grad)
    np.testing.assert_allclose(grad, e["grad"], rtol=2e-6, atol=1e-7)  # libm may differ by an ulp across hosts
    rows = orc.subsample(c["mask"], c["cond"])
    o = orc.Oracle(p, c["x_bin"])
    t, nidx = o.grow_tree(e["grad"], rows, c["js"], mode=0)  # grown from the fixture's gradients
    assert np.array_equal(t.feat, e["feat"]) and np.array_equal(t.cond_bin, e["cond_bin"]) and np.array_equal(t.split, e["split"])
    assert np.array_equal(t.gain, e["gain"]) and np.array_equal(t.w, e["w"]) and np.array_equal(t.pred, e["pred"])
    assert np.array_equal(nidx, e["nidx"])
    pr = c["pred"].copy()
    o.predict_tree(t, pr)
    assert np.array_equal(pr, e["pred_after"])
    assert t.split.sum() >= 2
    o.close()
