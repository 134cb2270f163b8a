"""ctypes binding of libevotrees_hip.so (the C ABI declared in include/evotrees_hip.h).

The library is mandatory: there is no CPU fallback.  Loading fails loudly when the shared
object has not been built, and every compute entry point fails when no MI355X is visible.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libevotrees_hip.so")

EVT_OK, EVT_ERR_ARG, EVT_ERR_HIP, EVT_ERR_STATE, EVT_ERR_EMPTY, EVT_ERR_NOMEM, EVT_ERR_INTERNAL = 0, -1, -2, -3, -4, -5, -6
LOSS_IDS = {"mse": 0, "logloss": 1, "gaussian_mle": 2, "poisson": 3, "gamma": 4, "tweedie": 5, "mlogloss": 6, "logistic_mle": 7, "mae": 8,
            "cred_var": 9, "cred_std": 10, "quantile": 11, "multiquantile": 12}
METRIC_IDS = {"mse": 0, "rmse": 1, "mae": 2, "logloss": 3, "gaussian_mle": 4, "poisson": 5, "gamma": 6, "tweedie": 7, "mlogloss": 8, "logistic_mle": 9, "quantile": 10, "multiquantile": 11}
TREE_TYPES = {"binary": 0, "oblivious": 1}
KERNEL_CLASSES = ["grad", "hist", "scan", "partition", "predict", "other"]

# every symbol include/evotrees_hip.h declares
EXPORTS = [
    "evt_last_error", "evt_device_count", "evt_create", "evt_destroy", "evt_set_xbin", "evt_binarize_f64",
    "evt_set_target", "evt_set_feature_meta", "evt_set_alphas", "evt_update_grads", "evt_set_grads", "evt_grow_tree",
    "evt_grow_tree_begin", "evt_grow_tree_end", "evt_stage_mask", "evt_grow_tree_begin_staged", "evt_draw_mask",
    "evt_tree_open", "evt_hist_build", "evt_split_scan", "evt_update_nodes_idx", "evt_tree_close", "evt_peek_tree",
    "evt_predict_tree", "evt_get_xbin", "evt_get_pred", "evt_get_grads", "evt_get_nidx", "evt_get_hist", "evt_get_quant",
    "evt_predict", "evt_predict_f64", "evt_predict_leaf_idx", "evt_eval_metric", "evt_set_profiling", "evt_get_profile", "evt_reset_profile",
    "evt_set_option", "evt_synchronize", "evt_copy_bandwidth", "evt_read_bandwidth", "evt_predict_static",
    "evt_lds_atomic_rate", "evt_global_atomic_rate",
]


class EvtError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("libevotrees_hip error %d: %s" % (code, msg))
        self.code = code


class EvtParams(C.Structure):
    _fields_ = [("eta", C.c_double), ("L2", C.c_double), ("lambda_", C.c_double), ("gamma", C.c_double),
                ("min_weight", C.c_double), ("bagging_size", C.c_int32), ("update_pred", C.c_int32)]


class EvtTreeOut(C.Structure):
    _fields_ = [("feat", C.c_void_p), ("cond_bin", C.c_void_p), ("w", C.c_void_p), ("gain", C.c_void_p),
                ("pred", C.c_void_p), ("split", C.c_void_p)]


_lib = None


def load():
    """Loads the shared library (once).  Raises if it is missing: build it with
    `python evotrees.jl_amd/build.py` (or `__graft_entry__.build()`)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("libevotrees_hip.so is not built (%s missing); run evotrees.jl_amd/build.py" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    vp, i64, i32 = C.c_void_p, C.c_int64, C.c_int32
    L.evt_last_error.restype = C.c_char_p
    L.evt_last_error.argtypes = []
    sigs = {
        "evt_device_count": [vp],
        "evt_create": [i64, i32, i32, i32, i32, i32, i32, vp],
        "evt_destroy": [vp],
        "evt_set_xbin": [vp, vp],
        "evt_binarize_f64": [vp, vp, vp, vp],
        "evt_set_target": [vp, vp, vp, vp, vp],
        "evt_set_feature_meta": [vp, vp, vp],
        "evt_set_alphas": [vp, vp, i32],
        "evt_update_grads": [vp],
        "evt_set_grads": [vp, vp],
        "evt_grow_tree": [vp, vp, C.c_uint8, vp, i32, C.POINTER(EvtParams), C.POINTER(EvtTreeOut)],
        "evt_grow_tree_begin": [vp, vp, C.c_uint8, vp, i32, C.POINTER(EvtParams)],
        "evt_grow_tree_end": [vp, C.POINTER(EvtTreeOut)],
        "evt_stage_mask": [vp, vp],
        "evt_draw_mask": [vp, C.c_uint64],
        "evt_grow_tree_begin_staged": [vp, C.c_uint8, vp, i32, C.POINTER(EvtParams)],
        "evt_tree_open": [vp, vp, C.c_uint8, vp, i32, C.POINTER(EvtParams)],
        "evt_hist_build": [vp, i32],
        "evt_split_scan": [vp, i32],
        "evt_update_nodes_idx": [vp, i32],
        "evt_tree_close": [vp],
        "evt_peek_tree": [vp, C.POINTER(EvtTreeOut)],
        "evt_predict_tree": [vp, i32, vp, vp, vp, vp],
        "evt_get_xbin": [vp, vp],
        "evt_get_pred": [vp, vp],
        "evt_get_grads": [vp, vp],
        "evt_get_nidx": [vp, vp],
        "evt_get_hist": [vp, vp],
        "evt_get_quant": [vp, vp, vp],
        "evt_predict": [i64, i32, vp, vp, i32, i32, i32, vp, vp, vp, vp, vp, i32, vp],
        "evt_predict_leaf_idx": [i64, i32, vp, vp, i32, vp, vp, vp, vp, vp],
        "evt_predict_f64": [i64, i32, vp, vp, vp, vp, i32, i32, i32, vp, vp, vp, vp, vp, i32, vp],
        "evt_eval_metric": [vp, i32, vp],
        "evt_set_profiling": [vp, i32],
        "evt_get_profile": [vp, vp, vp, vp],
        "evt_reset_profile": [vp],
        "evt_set_option": [vp, C.c_char_p, i64],
        "evt_synchronize": [vp],
        "evt_copy_bandwidth": [i64, i32, vp],
        "evt_read_bandwidth": [i64, i32, vp],
        "evt_lds_atomic_rate": [i32, i32, i32, vp, vp],
        "evt_global_atomic_rate": [i32, i32, i32, vp],
        "evt_predict_static": [vp, i64, i32, vp, vp, i32, i32, i32, i64, vp, vp, vp, vp, vp, i32, vp, vp],
    }
    for name, args in sigs.items():
        f = getattr(L, name)
        f.argtypes = args
        f.restype = C.c_int
    _lib = L
    return L


def check(rc):
    if rc != EVT_OK:
        raise EvtError(rc, load().evt_last_error().decode("utf-8", "replace"))


def ptr(a):
    if a is None:
        return None
    return a.ctypes.data_as(C.c_void_p)


def device_count():
    n = C.c_int32(0)
    check(load().evt_device_count(C.byref(n)))
    return n.value


def copy_bandwidth(nbytes=1 << 30, iters=10):
    out = C.c_double(0.0)
    check(load().evt_copy_bandwidth(nbytes, iters, C.byref(out)))
    return out.value


def lds_atomic_rate(pattern=0, lanes16=16, iters=200):
    """(lane-atomics per second, wavefront instructions per second) of 64-bit LDS atomics, device wide."""
    a, b = C.c_double(0.0), C.c_double(0.0)
    check(load().evt_lds_atomic_rate(pattern, lanes16, iters, C.byref(a), C.byref(b)))
    return a.value, b.value


def global_atomic_rate(words=12800, blocks=256, reps=4):
    """64-bit global atomics per second when `blocks` blocks each add `words` consecutive words of one slice."""
    a = C.c_double(0.0)
    check(load().evt_global_atomic_rate(words, blocks, reps, C.byref(a)))
    return a.value


def read_bandwidth(nbytes=1 << 30, iters=10):
    out = C.c_double(0.0)
    check(load().evt_read_bandwidth(nbytes, iters, C.byref(out)))
    return out.value


class TreeArrays:
    """Host arrays in the layout of Tree{L,K} (src/structs.jl:77-106)."""

    def __init__(self, K, nnodes):
        self.feat = np.zeros(nnodes, np.int64)
        self.cond_bin = np.zeros(nnodes, np.uint8)
        self.w = np.zeros(nnodes, np.float32)
        self.gain = np.zeros(nnodes, np.float32)
        self.pred = np.zeros((nnodes, K), np.float32)  # memory order of Julia's K x nnodes matrix
        self.split = np.zeros(nnodes, np.uint8)

    def as_out(self):
        return EvtTreeOut(ptr(self.feat), ptr(self.cond_bin), ptr(self.w), ptr(self.gain), ptr(self.pred), ptr(self.split))


class Handle:
    """One training cache on the device (the reference's CacheGPU)."""

    def __init__(self, nobs, nfeats, nbins, K, max_depth, loss, tree_type="binary"):
        self._h = C.c_void_p(None)
        self.N, self.F, self.B, self.K, self.D = int(nobs), int(nfeats), int(nbins), int(K), int(max_depth)
        self.NK = 2 * self.K + 1
        self.nnodes = (1 << self.D) - 1
        self.loss = loss
        check(load().evt_create(self.N, self.F, self.B, self.K, self.D, LOSS_IDS[loss], TREE_TYPES[tree_type], C.byref(self._h)))

    def close(self):
        if self._h:
            load().evt_destroy(self._h)
            self._h = C.c_void_p(None)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_xbin(self, x_bin_FN):
        """x_bin_FN: (F, N) C-order uint8 == Julia's N x F column-major matrix."""
        assert x_bin_FN.dtype == np.uint8 and x_bin_FN.flags.c_contiguous and x_bin_FN.shape == (self.F, self.N)
        check(load().evt_set_xbin(self._h, ptr(x_bin_FN)))

    def binarize(self, x_FN, edges):
        """x_FN: (F, N) C-order float64; edges: list of F ascending float64 arrays."""
        assert x_FN.dtype == np.float64 and x_FN.flags.c_contiguous and x_FN.shape == (self.F, self.N)
        off = np.zeros(self.F + 1, np.int32)
        off[1:] = np.cumsum([len(e) for e in edges])
        flat = np.ascontiguousarray(np.concatenate([np.asarray(e, np.float64) for e in edges]))
        check(load().evt_binarize_f64(self._h, ptr(x_FN), ptr(flat), ptr(off)))

    def set_target(self, y, w, mu, offset=None):
        y = np.ascontiguousarray(y, np.float32)
        w = None if w is None else np.ascontiguousarray(w, np.float32)
        mu = np.ascontiguousarray(mu, np.float32)
        offset = None if offset is None else np.ascontiguousarray(offset, np.float32)
        # one value per row and target: (N,) for one target, (N, T) C-order (Julia's T x N) for several
        T = 1 if self.loss in ("mlogloss", "multiquantile") else (self.K // 2 if self.loss in ("gaussian_mle", "logistic_mle") else self.K)
        assert (y.shape == (self.N,) and T == 1) or y.shape == (self.N, T)
        assert mu.shape == (self.K,)
        check(load().evt_set_target(self._h, ptr(y), ptr(w), ptr(mu), ptr(offset)))

    def set_feature_meta(self, feattypes=None, monotone=None):
        ft = None if feattypes is None else np.ascontiguousarray(feattypes, np.uint8)
        mo = None if monotone is None else np.ascontiguousarray(monotone, np.int32)
        check(load().evt_set_feature_meta(self._h, ptr(ft), ptr(mo)))

    def update_grads(self):
        check(load().evt_update_grads(self._h))

    def set_grads(self, grad):
        grad = np.ascontiguousarray(grad, np.float32)
        assert grad.shape == (self.N, self.NK)
        check(load().evt_set_grads(self._h, ptr(grad)))

    def grow_tree(self, js, params, mask=None, cond=255, want_tree=True):
        js = np.ascontiguousarray(js, np.uint32)
        if mask is not None:
            mask = np.ascontiguousarray(mask, np.uint8)
            assert mask.shape == (self.N,)
        t = TreeArrays(self.K, self.nnodes) if want_tree else None
        out = t.as_out() if want_tree else None
        check(load().evt_grow_tree(self._h, ptr(mask), int(cond), ptr(js), js.shape[0], C.byref(params),
                                   C.byref(out) if want_tree else None))
        return t

    def grow_tree_begin(self, js, params, mask=None, cond=255):
        """Queues one tree and returns while the device grows it; grow_tree_end collects it (the older one when two
        are in flight).  While ONE tree is in flight the next round may be queued behind it (update_grads, draw_mask /
        stage_mask, grow_tree_begin[_staged]); calls that read or rewrite the handle's state wait for grow_tree_end."""
        js = np.ascontiguousarray(js, np.uint32)
        if mask is not None:
            mask = np.ascontiguousarray(mask, np.uint8)
            assert mask.shape == (self.N,)
        check(load().evt_grow_tree_begin(self._h, ptr(mask), int(cond), ptr(js), js.shape[0], C.byref(params)))

    def stage_mask(self, mask):
        """Uploads the next tree's row mask while the tree begun with grow_tree_begin is still growing."""
        mask = np.ascontiguousarray(mask, np.uint8)
        assert mask.shape == (self.N,)
        check(load().evt_stage_mask(self._h, ptr(mask)))

    def draw_mask(self, seed):
        """The next tree's row mask drawn on the device: SplitMix64 started at `seed`, 8 mask bytes per output (see
        splitmix_mask for the same bytes on the host).  Takes the place of stage_mask."""
        check(load().evt_draw_mask(self._h, int(seed) & 0xFFFFFFFFFFFFFFFF))

    def grow_tree_begin_staged(self, js, params, cond):
        """grow_tree_begin with the mask last given to stage_mask."""
        js = np.ascontiguousarray(js, np.uint32)
        check(load().evt_grow_tree_begin_staged(self._h, int(cond), ptr(js), js.shape[0], C.byref(params)))

    def grow_tree_end(self, want_tree=True):
        t = TreeArrays(self.K, self.nnodes) if want_tree else None
        out = t.as_out() if want_tree else None
        check(load().evt_grow_tree_end(self._h, C.byref(out) if want_tree else None))
        return t

    # one tree, one kernel stage at a time (update_hist!, the split search, update_nodes_idx! per level)
    def tree_open(self, js, params, mask=None, cond=255):
        js = np.ascontiguousarray(js, np.uint32)
        if mask is not None:
            mask = np.ascontiguousarray(mask, np.uint8)
            assert mask.shape == (self.N,)
        check(load().evt_tree_open(self._h, ptr(mask), int(cond), ptr(js), js.shape[0], C.byref(params)))

    def hist_build(self, level):
        check(load().evt_hist_build(self._h, int(level)))

    def split_scan(self, level):
        check(load().evt_split_scan(self._h, int(level)))

    def update_nodes_idx(self, level):
        check(load().evt_update_nodes_idx(self._h, int(level)))

    def tree_close(self):
        check(load().evt_tree_close(self._h))

    def peek_tree(self):
        t = TreeArrays(self.K, self.nnodes)
        out = t.as_out()
        check(load().evt_peek_tree(self._h, C.byref(out)))
        return t

    def predict_tree(self, tree):
        check(load().evt_predict_tree(self._h, tree.feat.shape[0], ptr(tree.feat), ptr(tree.cond_bin), ptr(tree.pred), ptr(tree.split)))

    def set_alphas(self, alphas):
        """Levels of the quantile losses and metrics: one value (quantile) or one per output (multiquantile)."""
        a = np.ascontiguousarray(np.atleast_1d(alphas), np.float64)
        check(load().evt_set_alphas(self._h, ptr(a), a.shape[0]))

    def eval_metric(self, metric):
        """Metric of the handle's prediction against its target and weights (the eval CallBack's feval)."""
        v = C.c_double(0.0)
        check(load().evt_eval_metric(self._h, METRIC_IDS[metric], C.byref(v)))
        return v.value

    def get_xbin(self):
        out = np.empty((self.F, self.N), np.uint8)
        check(load().evt_get_xbin(self._h, ptr(out)))
        return out

    def get_pred(self):
        out = np.empty((self.N, self.K), np.float32)
        check(load().evt_get_pred(self._h, ptr(out)))
        return out

    def get_grads(self):
        out = np.empty((self.N, self.NK), np.float32)
        check(load().evt_get_grads(self._h, ptr(out)))
        return out

    def get_nidx(self):
        out = np.empty(self.N, np.uint32)
        check(load().evt_get_nidx(self._h, ptr(out)))
        return out

    def get_hist(self):
        """[node, feature, bin, k] Float64 view of the reference's h∇[k, bin, feature, node]."""
        out = np.empty((self.nnodes, self.F, self.B, self.NK), np.float64)
        check(load().evt_get_hist(self._h, ptr(out)))
        return out

    def get_quant(self):
        qb = np.zeros(self.NK, np.int32)
        qe = np.zeros(self.NK, np.int32)
        check(load().evt_get_quant(self._h, ptr(qb), ptr(qe)))
        return qb, qe

    def set_profiling(self, on):
        """on: False/True, or a list of kernel class names to time (e.g. ["hist"])."""
        if isinstance(on, (list, tuple)):
            mask = 0
            for name in on:
                mask |= 1 << KERNEL_CLASSES.index(name)
            if mask == 1:
                mask |= 1 << 30  # keep the value distinct from the "every class" code 1
            check(load().evt_set_profiling(self._h, mask))
        else:
            check(load().evt_set_profiling(self._h, 1 if on else 0))

    def reset_profile(self):
        check(load().evt_reset_profile(self._h))

    def get_profile(self):
        n = len(KERNEL_CLASSES)
        la = np.zeros(n, np.int64)
        ms = np.zeros(n, np.float64)
        un = np.zeros(n, np.int64)
        check(load().evt_get_profile(self._h, ptr(la), ptr(ms), ptr(un)))
        return {k: {"launches": int(la[i]), "ms": float(ms[i]), "units": int(un[i])} for i, k in enumerate(KERNEL_CLASSES)}

    def set_option(self, name, value):
        check(load().evt_set_option(self._h, name.encode(), int(value)))

    def synchronize(self):
        check(load().evt_synchronize(self._h))


def splitmix_mask(seed, N):
    """The bytes Handle.draw_mask(seed) writes on the device, computed on the host: output w (from 0) of SplitMix64
    started at `seed` holds mask bytes 8w .. 8w+7, little end first."""
    M = (1 << 64) - 1
    with np.errstate(over="ignore"):
        w = np.arange(1, (int(N) + 7) // 8 + 1, dtype=np.uint64)
        z = np.uint64(int(seed) & M) + w * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z ^= z >> np.uint64(31)
    return z.astype("<u8").view(np.uint8)[:int(N)]


def make_params(eta=0.1, L2=1.0, lambda_=0.0, gamma=0.0, min_weight=1.0, bagging_size=1, update_pred=True):
    return EvtParams(eta, L2, lambda_, gamma, min_weight, bagging_size, 1 if update_pred else 0)


def predict_model(x_bin_FN, feattypes, loss, K, trees, apply_link=True):
    """trees: list of objects with feat/cond_bin/pred/split arrays.  Returns (N, K) float32."""
    F, N = x_bin_FN.shape
    off = np.zeros(len(trees) + 1, np.int64)
    off[1:] = np.cumsum([t.feat.shape[0] for t in trees])
    feat = np.ascontiguousarray(np.concatenate([t.feat for t in trees]), np.int64)
    cb = np.ascontiguousarray(np.concatenate([t.cond_bin for t in trees]), np.uint8)
    sp = np.ascontiguousarray(np.concatenate([t.split for t in trees]), np.uint8)
    pr = np.ascontiguousarray(np.concatenate([t.pred.reshape(-1, K) for t in trees]), np.float32)
    ft = None if feattypes is None else np.ascontiguousarray(feattypes, np.uint8)
    out = np.empty((N, K), np.float32)
    check(load().evt_predict(N, F, ptr(x_bin_FN), ptr(ft), LOSS_IDS[loss], K, len(trees), ptr(off), ptr(feat), ptr(cb), ptr(pr),
                             ptr(sp), 1 if apply_link else 0, ptr(out)))
    return out


def predict_model_f64(x_FN, edges, feattypes, loss, K, trees, apply_link=True):
    """As predict_model, from raw features: x_FN (F, N) C-order float64, edges a list of F ascending arrays."""
    assert x_FN.dtype == np.float64 and x_FN.flags.c_contiguous
    F, N = x_FN.shape
    eoff = np.zeros(F + 1, np.int32)
    eoff[1:] = np.cumsum([len(e) for e in edges])
    eflat = np.ascontiguousarray(np.concatenate([np.asarray(e, np.float64) for e in edges]))
    off = np.zeros(len(trees) + 1, np.int64)
    off[1:] = np.cumsum([t.feat.shape[0] for t in trees])
    feat = np.ascontiguousarray(np.concatenate([t.feat for t in trees]), np.int64)
    cb = np.ascontiguousarray(np.concatenate([t.cond_bin for t in trees]), np.uint8)
    sp = np.ascontiguousarray(np.concatenate([t.split for t in trees]), np.uint8)
    pr = np.ascontiguousarray(np.concatenate([t.pred.reshape(-1, K) for t in trees]), np.float32)
    ft = None if feattypes is None else np.ascontiguousarray(feattypes, np.uint8)
    out = np.empty((N, K), np.float32)
    check(load().evt_predict_f64(N, F, ptr(x_FN), ptr(eflat), ptr(eoff), ptr(ft), LOSS_IDS[loss], K, len(trees), ptr(off), ptr(feat),
                                 ptr(cb), ptr(pr), ptr(sp), 1 if apply_link else 0, ptr(out)))
    return out


def predict_leaf_idx(x_bin_FN, feattypes, trees):
    F, N = x_bin_FN.shape
    off = np.zeros(len(trees) + 1, np.int64)
    off[1:] = np.cumsum([t.feat.shape[0] for t in trees])
    feat = np.ascontiguousarray(np.concatenate([t.feat for t in trees]), np.int64)
    cb = np.ascontiguousarray(np.concatenate([t.cond_bin for t in trees]), np.uint8)
    sp = np.ascontiguousarray(np.concatenate([t.split for t in trees]), np.uint8)
    ft = None if feattypes is None else np.ascontiguousarray(feattypes, np.uint8)
    out = np.empty((len(trees), N), np.uint32)  # Julia: N x ntrees column-major
    check(load().evt_predict_leaf_idx(N, F, ptr(x_bin_FN), ptr(ft), len(trees), ptr(off), ptr(feat), ptr(cb), ptr(sp), ptr(out)))
    return out.T
