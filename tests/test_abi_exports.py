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


def test_splitmix_mask_known_answers(evt):
    # SplitMix64's published outputs: seed 0 (the reference C source's first three) and seed 1234567 (first five)
    import numpy as np
    got = evt.splitmix_mask(0, 24).view("<u8")
    assert [int(v) for v in got] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    got = evt.splitmix_mask(1234567, 40).view("<u8")
    assert [int(v) for v in got] == [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431,
                                     16408922859458223821]
    # little end first, and a length that is not a multiple of eight cuts the last word short
    m = evt.splitmix_mask(0, 13)
    assert m.dtype == np.uint8 and m.shape == (13,)
    assert list(m[:8]) == [0xAF, 0xCD, 0x1D, 0x7B, 0x39, 0xA8, 0x20, 0xE2] and list(m[8:]) == [0xF4, 0x65, 0xB9, 0xA1, 0x6A]
