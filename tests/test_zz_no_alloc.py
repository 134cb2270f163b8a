"""evt_predict_static - the entry point that allocates nothing - against evt_predict, bit for bit, through the C ABI:
two calls in a row on the same GPU (they share one static work area), the second on a smaller input; then the
size limit and the on-device model check."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as orc
from test_gpu_parity import _random_tree

pytestmark = pytest.mark.gpu


def _model_arrays(trees, K):
    off = np.zeros(len(trees) + 1, np.int64)
    off[1:] = np.cumsum([t.feat.shape[0] for t in trees])
    feat = np.ascontiguousarray(np.concatenate([t.feat for t in trees]), np.int64)
    cb = np.ascontiguousarray(np.concatenate([t.cond_bin for t in trees]), np.uint8)
    sp = np.ascontiguousarray(np.concatenate([t.split for t in trees]), np.uint8)
    pr = np.ascontiguousarray(np.concatenate([t.pred.reshape(-1, K) for t in trees]), np.float32)
    return off, feat, cb, pr, sp


def _static_call(evt, torch, x_bin, ft, loss, K, trees, apply_link, total_override=None):
    """Uploads everything with torch (device memory is the caller's business), calls the entry point on torch's current
    stream and returns (rc, out, status) after a synchronize."""
    L = evt._lib.load()
    F, N = x_bin.shape
    off, feat, cb, pr, sp = _model_arrays(trees, K)
    dev = torch.device("cuda:0")
    d = [torch.from_numpy(a).to(dev) for a in (x_bin, off, feat, cb, pr, sp)]
    d_ft = None if ft is None else torch.from_numpy(ft).to(dev)
    out = torch.full((N, K), float("nan"), dtype=torch.float32, device=dev)
    status = torch.full((1,), 77, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream().cuda_stream
    total = int(off[-1]) if total_override is None else total_override
    rc = L.evt_predict_static(C.c_void_p(stream), N, F, C.c_void_p(d[0].data_ptr()), C.c_void_p(d_ft.data_ptr()) if d_ft is not None else None,
                              evt._lib.LOSS_IDS[loss], K, len(trees), total, C.c_void_p(d[1].data_ptr()), C.c_void_p(d[2].data_ptr()),
                              C.c_void_p(d[3].data_ptr()), C.c_void_p(d[4].data_ptr()), C.c_void_p(d[5].data_ptr()), 1 if apply_link else 0,
                              C.c_void_p(out.data_ptr()), C.c_void_p(status.data_ptr()))
    torch.cuda.synchronize()
    return rc, out.cpu().numpy(), int(status.cpu()[0])


def test_predict_static_equals_predict(evt):
    torch = pytest.importorskip("torch")
    assert torch.cuda.is_available()
    rng = np.random.default_rng(5)
    # first call: the larger input (many outputs, categorical features, trees of several sizes); second: a smaller one
    cases = [(50_000, 40, 64, [9, 3, 11, 1, 9, 7], 6, "mlogloss", True), (3_001, 7, 16, [4, 1, 5], 1, "logloss", False)]
    for N, F, B, depths, K, loss, cat in cases:
        print("case", N, F, B, depths, K, loss, flush=True)
        x_bin = rng.integers(1, B + 1, size=(F, N), dtype=np.uint8)
        ft = (rng.random(F) > 0.2).astype(np.uint8) if cat else None
        trees = [_random_tree(rng, dd, F, B, K) for dd in depths]
        for link in (False, True):
            want = evt._lib.predict_model(x_bin, ft, loss, K, trees, apply_link=link)
            rc, got, status = _static_call(evt, torch, x_bin, ft, loss, K, trees, link)
            assert rc == 0 and status == 0
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        # and against the oracle's walk (raw sums)
        ref = np.zeros((N, K), np.float32)
        ftv = np.ones(F, np.uint8) if ft is None else ft
        for t in trees:
            orc.predict_tree(orc.LOSS_IDS[loss], K, x_bin, ftv, t, ref)
        rc, got, status = _static_call(evt, torch, x_bin, ft, loss, K, trees, False)
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_predict_static_limits_and_model_check(evt):
    torch = pytest.importorskip("torch")
    L = evt._lib.load()
    rng = np.random.default_rng(6)
    N, F, B, K = 2000, 5, 8, 1
    x_bin = rng.integers(1, B + 1, size=(F, N), dtype=np.uint8)
    trees = [_random_tree(rng, 4, F, B, K) for _ in range(3)]
    # a model larger than the static work area is refused on the host, before anything is queued
    rc, out, status = _static_call(evt, torch, x_bin, None, "mse", K, trees, False, total_override=(1 << 20) + 1)
    assert rc == evt._lib.EVT_ERR_ARG and b"static work area" in L.evt_last_error()
    assert status == 77 and np.isnan(out).all()
    # host memory is refused
    rc = L.evt_predict_static(None, N, F, evt._lib.ptr(x_bin), None, 0, K, 1, 15, None, None, None, None, None, 0, None, None)
    assert rc == evt._lib.EVT_ERR_ARG
    # a split node whose children lie outside its tree: found on the device, nothing is written, status says so
    bad = [_random_tree(rng, 4, F, B, K) for _ in range(3)]
    bad[1].split[10] = 1  # node 11 of 15: children 22, 23 do not exist
    bad[1].feat[10] = 1
    rc, out, status = _static_call(evt, torch, x_bin, None, "mse", K, bad, False)
    assert rc == 0 and status == evt._lib.EVT_ERR_ARG and np.isnan(out).all()
    # offsets that do not end at total_nodes
    rc, out, status = _static_call(evt, torch, x_bin, None, "mse", K, trees, False, total_override=46)
    assert rc == 0 and status == evt._lib.EVT_ERR_ARG and np.isnan(out).all()
    # the work area is clean again for the next, valid call
    rc, out, status = _static_call(evt, torch, x_bin, None, "mse", K, trees, False)
    assert rc == 0 and status == 0
    assert np.array_equal(out, evt._lib.predict_model(x_bin, None, "mse", K, trees, apply_link=False))


def test_predict_static_recorded_into_a_graph(evt):
    """The call recorded into a HIP graph (after one ordinary call on the device, which looks the work area up) and
    replayed three times with eager work, other models through the same work area and synchronisations in between:
    every replay equals evt_predict bit for bit.  The recorded call carries EVT_STATIC_TRUSTED (no pointer queries)."""
    torch = pytest.importorskip("torch")
    L = evt._lib.load()
    rng = np.random.default_rng(8)
    N, F, B, K, loss = 20_000, 12, 32, 2, "gaussian_mle"
    x_bin = rng.integers(1, B + 1, size=(F, N), dtype=np.uint8)
    trees = [_random_tree(rng, dd, F, B, K) for dd in (6, 2, 8, 5)]
    want = evt._lib.predict_model(x_bin, None, loss, K, trees, apply_link=True)
    rc, got, status = _static_call(evt, torch, x_bin, None, loss, K, trees, True)  # the ordinary first call
    assert rc == 0 and status == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32))
    off, feat, cb, pr, sp = _model_arrays(trees, K)
    dev = torch.device("cuda:0")
    d = [torch.from_numpy(a).to(dev) for a in (x_bin, off, feat, cb, pr, sp)]
    out = torch.zeros((N, K), dtype=torch.float32, device=dev)
    status_t = torch.full((1,), 77, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        stream = torch.cuda.current_stream().cuda_stream
        rc = L.evt_predict_static(C.c_void_p(stream), N, F, C.c_void_p(d[0].data_ptr()), None, evt._lib.LOSS_IDS[loss], K, len(trees), int(off[-1]),
                                  C.c_void_p(d[1].data_ptr()), C.c_void_p(d[2].data_ptr()), C.c_void_p(d[3].data_ptr()), C.c_void_p(d[4].data_ptr()),
                                  C.c_void_p(d[5].data_ptr()), 1 | 2, C.c_void_p(out.data_ptr()), C.c_void_p(status_t.data_ptr()))
    assert rc == 0
    other = [_random_tree(rng, 4, F, B, K) for _ in range(2)]
    for rep in range(3):
        out.fill_(float("nan"))
        status_t.fill_(77)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert int(status_t.cpu()[0]) == 0
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32)), rep
        # eager work through the same work area between the replays: another model, then a synchronize
        rc2, got2, st2 = _static_call(evt, torch, x_bin, None, loss, K, other, False)
        assert rc2 == 0 and st2 == 0
        assert np.array_equal(got2, evt._lib.predict_model(x_bin, None, loss, K, other, apply_link=False))
