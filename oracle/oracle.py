"""ctypes wrapper around libevo_oracle.so (the CPU oracle).

TEST INFRASTRUCTURE ONLY: imported by tests, the smoke check and the benchmark's
cpu_baseline leg.  The product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libevo_oracle.so")

LOSS_IDS = {"mse": 0, "logloss": 1, "gaussian_mle": 2, "poisson": 3, "gamma": 4, "tweedie": 5, "mlogloss": 6, "logistic_mle": 7, "mae": 8,
            "cred_var": 9, "cred_std": 10, "quantile": 11, "multiquantile": 12}
METRIC_IDS = {"mse": 0, "rmse": 1, "mae": 2, "logloss": 3, "gaussian_mle": 4, "poisson": 5, "gamma": 6, "tweedie": 7, "mlogloss": 8, "logistic_mle": 9, "quantile": 10, "multiquantile": 11}
TREE_TYPES = {"binary": 0, "oblivious": 1}


class OrcParams(C.Structure):
    _fields_ = [
        ("loss", C.c_int32),
        ("K", C.c_int32),
        ("nbins", C.c_int32),
        ("max_depth", C.c_int32),
        ("tree_type", C.c_int32),
        ("bagging_size", C.c_int32),
        ("eta", C.c_double),
        ("L2", C.c_double),
        ("lambda_", C.c_double),
        ("gamma", C.c_double),
        ("min_weight", C.c_double),
        ("n_alphas", C.c_int32),
        ("alphas", C.c_double * 16),
    ]


def build(force=False):
    """Compile the oracle with gcc (only needs evo_oracle.c)."""
    src = os.path.join(_HERE, "evo_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libevo_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        vp, i64, i32 = C.c_void_p, C.c_int64, C.c_int32
        L.orc_update_grads.argtypes = [C.POINTER(OrcParams), i64, vp, vp, vp]
        L.orc_update_grads.restype = None
        L.orc_binarize.argtypes = [i64, vp, vp, i32, vp]
        L.orc_binarize.restype = None
        L.orc_subsample.argtypes = [i64, vp, C.c_uint8, vp]
        L.orc_subsample.restype = i64
        L.orc_create.argtypes = [C.POINTER(OrcParams), i64, i32, vp, vp, vp, C.c_int]
        L.orc_create.restype = vp
        L.orc_destroy.argtypes = [vp]
        L.orc_destroy.restype = None
        L.orc_num_threads.argtypes = [vp]
        L.orc_num_threads.restype = C.c_int
        L.orc_hist_ptr.argtypes = [vp]
        L.orc_hist_ptr.restype = C.POINTER(C.c_double)
        L.orc_histq_ptr.argtypes = [vp]
        L.orc_histq_ptr.restype = C.POINTER(C.c_int64)
        L.orc_node_sums.argtypes = [vp]
        L.orc_node_sums.restype = C.POINTER(C.c_double)
        L.orc_set_quant.argtypes = [vp, vp, vp]
        L.orc_set_quant.restype = None
        L.orc_get_quant.argtypes = [vp, vp, vp]
        L.orc_get_quant.restype = None
        L.orc_grow_tree.argtypes = [vp, vp, vp, i64, vp, i32, C.c_int, vp, vp, vp, vp, vp, vp, vp]
        L.orc_grow_tree.restype = C.c_int
        L.orc_predict_tree.argtypes = [i32, i32, i64, vp, vp, vp, vp, vp, vp, vp]
        L.orc_predict_tree.restype = None
        L.orc_predict_leaf_idx.argtypes = [i64, vp, vp, vp, vp, vp, vp]
        L.orc_predict_leaf_idx.restype = None
        L.orc_apply_link.argtypes = [i32, i32, i64, vp]
        L.orc_apply_link.restype = None
        L.orc_eval_metric.argtypes = [i32, i32, i64, vp, vp, vp]
        L.orc_eval_metric.restype = C.c_double
        L.orc_eval_metric_quantile.argtypes = [i32, i32, i64, vp, vp, vp, vp]
        L.orc_eval_metric_quantile.restype = C.c_double
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def make_params(loss="mse", nbins=64, max_depth=6, tree_type="binary", bagging_size=1, eta=0.1, L2=1.0,
                lambda_=0.0, gamma=0.0, min_weight=1.0, K=None, alpha=0.5, alphas=None):
    """alpha: the quantile loss's level (every output); alphas: the multiquantile loss's levels, one output each."""
    if loss == "multiquantile":
        al = [float(a) for a in alphas]
        K = len(al)
    else:
        al = [float(alpha)]
    if K is None:
        K = 2 if loss in ("gaussian_mle", "logistic_mle") else 1
    arr = (C.c_double * 16)(*(al + [0.0] * (16 - len(al))))
    return OrcParams(LOSS_IDS[loss], K, nbins, max_depth, TREE_TYPES[tree_type], bagging_size, eta, L2, lambda_,
                     gamma, min_weight, len(al), arr)


class Tree:
    """Host mirror of Tree{L,K} (src/structs.jl:77-106)."""

    def __init__(self, K, nnodes):
        self.feat = np.zeros(nnodes, np.int64)
        self.cond_bin = np.zeros(nnodes, np.uint8)
        self.w = np.zeros(nnodes, np.float32)
        self.gain = np.zeros(nnodes, np.float32)
        self.pred = np.zeros((nnodes, K), np.float32)  # memory order = K fastest (Julia K x nnodes)
        self.split = np.zeros(nnodes, np.uint8)


def update_grads(params, pred, y, grad):
    """pred: (N, K) f32 C-order (== Julia K x N), y: (N,) f32, grad: (N, 2K+1) f32 in/out."""
    N = grad.shape[0]
    assert pred.dtype == np.float32 and y.dtype == np.float32 and grad.dtype == np.float32
    assert pred.flags.c_contiguous and grad.flags.c_contiguous
    lib().orc_update_grads(C.byref(params), N, _p(pred), _p(y), _p(grad))


def binarize(x, edges):
    """x: (N,) f64 one feature column; edges: (nedges,) f64 ascending -> (N,) u8 in 1..nedges+1."""
    x = np.ascontiguousarray(x, np.float64)
    edges = np.ascontiguousarray(edges, np.float64)
    out = np.empty(x.shape[0], np.uint8)
    lib().orc_binarize(x.shape[0], _p(x), _p(edges), edges.shape[0], _p(out))
    return out


def subsample(mask, cond):
    mask = np.ascontiguousarray(mask, np.uint8)
    out = np.empty(mask.shape[0], np.uint32)
    n = lib().orc_subsample(mask.shape[0], _p(mask), int(cond), _p(out))
    return out[:n].copy()


class Oracle:
    """Holds x_bin (column-major N x F, passed as an (F, N) C-order uint8 array) and work buffers."""

    def __init__(self, params, x_bin_FN, feattypes=None, monotone=None, with_fixed=True):
        assert x_bin_FN.dtype == np.uint8 and x_bin_FN.flags.c_contiguous
        self.params = params
        self.F, self.N = x_bin_FN.shape
        self.K = params.K
        self.NK = 2 * params.K + 1
        self.nnodes = (1 << params.max_depth) - 1
        self.x_bin = x_bin_FN
        self.feattypes = np.ones(self.F, np.uint8) if feattypes is None else np.ascontiguousarray(feattypes, np.uint8)
        self.monotone = np.zeros(self.F, np.int32) if monotone is None else np.ascontiguousarray(monotone, np.int32)
        self._h = lib().orc_create(C.byref(params), self.N, self.F, _p(x_bin_FN), _p(self.feattypes),
                                   _p(self.monotone), 1 if with_fixed else 0)
        self.with_fixed = with_fixed

    def close(self):
        if self._h:
            lib().orc_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    @property
    def nthreads(self):
        return lib().orc_num_threads(self._h)

    def set_quant(self, grad, qbits):
        qbits = np.ascontiguousarray(qbits, np.int32)
        lib().orc_set_quant(self._h, _p(grad), _p(qbits))

    def get_quant(self):
        qb = np.zeros(self.NK, np.int32)
        qe = np.zeros(self.NK, np.int32)
        lib().orc_get_quant(self._h, _p(qb), _p(qe))
        return qb, qe

    def grow_tree(self, grad, is_rows, js, mode=0, want_nidx=True):
        """grad (N, NK) f32; is_rows ascending 0-based uint32; js ascending 1-based uint32."""
        is_rows = np.ascontiguousarray(is_rows, np.uint32)
        js = np.ascontiguousarray(js, np.uint32)
        t = Tree(self.K, self.nnodes)
        nidx = np.zeros(self.N, np.uint32) if want_nidx else None
        rc = lib().orc_grow_tree(self._h, _p(grad), _p(is_rows), is_rows.shape[0], _p(js), js.shape[0], mode,
                                 _p(t.feat), _p(t.cond_bin), _p(t.w), _p(t.gain), _p(t.pred), _p(t.split), _p(nidx))
        if rc != 0:
            raise RuntimeError("orc_grow_tree failed (fixed mode needs with_fixed=True)")
        return t, nidx

    def hist(self, fixed=False):
        """Histogram of the last grown tree as an array indexed [node, feature, bin, k] (node 0 = root)."""
        shape = (self.nnodes, self.F, self.params.nbins, self.NK)
        n = int(np.prod(shape))
        if fixed:
            return np.ctypeslib.as_array(lib().orc_histq_ptr(self._h), shape=(n,)).reshape(shape)
        return np.ctypeslib.as_array(lib().orc_hist_ptr(self._h), shape=(n,)).reshape(shape)

    def node_sums(self):
        """(nnodes+2, NK) doubles; row n = sums of 1-based node n."""
        n = (self.nnodes + 2) * self.NK
        return np.ctypeslib.as_array(lib().orc_node_sums(self._h), shape=(n,)).reshape(self.nnodes + 2, self.NK)

    def predict_tree(self, tree, pred):
        """pred (N, K) f32 in/out."""
        lib().orc_predict_tree(self.params.loss, self.K, self.N, _p(self.x_bin), _p(self.feattypes), _p(tree.feat),
                               _p(tree.cond_bin), _p(tree.pred), _p(tree.split), _p(pred))


def predict_tree(loss_id, K, x_bin_FN, feattypes, tree, pred):
    F, N = x_bin_FN.shape
    lib().orc_predict_tree(loss_id, K, N, _p(x_bin_FN), _p(feattypes), _p(tree.feat), _p(tree.cond_bin),
                           _p(tree.pred), _p(tree.split), _p(pred))


def predict_leaf_idx(x_bin_FN, feattypes, tree):
    F, N = x_bin_FN.shape
    out = np.zeros(N, np.uint32)
    lib().orc_predict_leaf_idx(N, _p(x_bin_FN), _p(feattypes), _p(tree.feat), _p(tree.cond_bin), _p(tree.split), _p(out))
    return out


def apply_link(loss_id, K, pred):
    lib().orc_apply_link(loss_id, K, pred.shape[0], _p(pred))


def eval_metric(metric, K, pred, y, w=None, alphas=None):
    """pred (N, K) f32 raw (link not applied), y (N,) f32, w (N,) f32 or None."""
    w = None if w is None else np.ascontiguousarray(w, np.float32)
    if metric in ("quantile", "multiquantile"):
        al = np.ascontiguousarray(alphas, np.float32).reshape(-1)
        return lib().orc_eval_metric_quantile(METRIC_IDS[metric], K, pred.shape[0], _p(pred), _p(y), _p(w), _p(al))
    return lib().orc_eval_metric(METRIC_IDS[metric], K, pred.shape[0], _p(pred), _p(y), _p(w))
