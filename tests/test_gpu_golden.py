"""HIP path against the committed golden fixtures (tests/golden/trees.json), through the C ABI."""
import numpy as np
import pytest

from golden_util import load_cases

pytestmark = pytest.mark.gpu
CASES = load_cases()


@pytest.mark.parametrize("c", CASES, ids=[c["name"] for c in CASES])
def test_gpu_reproduces_golden(evt, c):
    e = c["expect"]
    K = c["K"]
    h = evt.Handle(c["N"], c["F"], c["B"], K, c["D"], c["loss"], c["tree_type"])
    h.set_xbin(c["x_bin"])
    # the fixtures start from a per-row prediction: passed as offset on a zero bias
    h.set_target(c["y"], c["w"] if c["weighted"] else None, np.zeros(K, np.float32), offset=c["pred"])
    assert np.array_equal(h.get_pred(), c["pred"])
    h.update_grads()
    np.testing.assert_allclose(h.get_grads(), e["grad"], rtol=1e-5, atol=1e-7)
    h.set_grads(e["grad"])  # identical gradients -> structure must be identical
    pk = dict(c["params"])
    gp = evt.make_params(**pk)
    h.set_option("record_nidx", 1)
    t = h.grow_tree(c["js"], gp, mask=c["mask"], cond=c["cond"])
    assert np.array_equal(t.feat, e["feat"]) and np.array_equal(t.cond_bin, e["cond_bin"]) and np.array_equal(t.split, e["split"])
    np.testing.assert_allclose(t.gain, e["gain"], rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(t.pred, e["pred"], rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(t.w, e["w"], rtol=1e-5)
    assert np.array_equal(h.get_nidx(), e["nidx"])
    np.testing.assert_allclose(h.get_pred(), e["pred_after"], rtol=1e-5, atol=1e-7)
    h.close()
