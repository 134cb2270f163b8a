"""CPU-side checks of the C ABI: the library loads and exports every symbol the header declares;
no compute entry point is called here."""
import os
import re


def test_library_exports_every_declared_symbol(evt):
    L = evt._lib.load()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    hdr = open(os.path.join(root, "include", "evotrees_hip.h")).read()
    declared = sorted(set(re.findall(r"\b(evt_[a-z0-9_]+)\s*\(", hdr)))
    assert declared, "no declarations found"
    for name in declared:
        assert hasattr(L, name), "missing export " + name
    assert sorted(evt._lib.EXPORTS) == declared


def test_argument_errors_need_no_gpu(evt):
    import ctypes as C
    L = evt._lib.load()
    assert L.evt_device_count(None) == evt._lib.EVT_ERR_ARG
    h = C.c_void_p(None)
    assert L.evt_create(10, 3, 300, 1, 3, 0, 0, C.byref(h)) == evt._lib.EVT_ERR_ARG  # nbins > 255
    assert b"nbins" in L.evt_last_error()
    assert L.evt_create(10, 3, 8, 1, 3, 0, 0, None) == evt._lib.EVT_ERR_ARG
    assert L.evt_set_xbin(None, None) == evt._lib.EVT_ERR_ARG
    assert L.evt_destroy(None) == 0


def test_host_config_checks(evt):
    import pytest
    with pytest.raises(ValueError):
        evt.EvoTreeRegressor(nbins=256)
    with pytest.raises(ValueError):
        evt.EvoTreeRegressor(nbins=1)
    with pytest.raises(ValueError):
        evt.EvoTreeRegressor(rowsample=0.0)
    with pytest.raises(ValueError):
        evt.EvoTreeRegressor(tree_type="other")
    with pytest.raises(ValueError):
        evt.EvoTreeRegressor(loss="gaussian_mle")
    with pytest.raises(ValueError):
        evt.init(evt.EvoTreeRegressor(device="cpu"), [[1.0]], [1.0])
    assert evt.EvoTreeMLE().min_weight == 8.0 and evt.EvoTreeRegressor().min_weight == 1.0
    assert evt.EvoTreeRegressor(**{"lambda": 0.5}).lambda_ == 0.5
