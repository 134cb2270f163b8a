"""Host side of the MI355X tree-building backend, mirroring EvoTrees.jl's interface for the
hot path: learner configs (src/learners.jl), `fit(config; x_train, y_train, ...)`
(src/fit.jl:388-437), the model functor `m(x; ntree_limit, device)` (src/structs.jl:135-138),
`predict` (src/predict.jl:93-96) and `predict_leaf_idx` (src/predict.jl:173-185).

Everything data parallel runs in libevotrees_hip.so through the C ABI; this module only keeps
what the reference keeps on the host: argument checks, quantile edges, the bias, the random
row mask / column sample, and the list of trees.  There is no CPU compute path: `device` must be
a GPU device name and the shared library must be present.

Julia is not available where this package is developed, so the host side is Python; the random
streams are numpy's (PCG64), not Julia's Xoshiro, hence models are not stream-identical to a
Julia run with the same seed — the trees are identical for identical masks/column samples.
"""
import numpy as np

from . import _lib
from ._lib import EvtError, Handle, TreeArrays, make_params  # noqa: F401

__all__ = ["EvoTreeRegressor", "EvoTreeMLE", "EvoTree", "Tree", "fit", "predict", "predict_leaf_idx", "init", "grow_evotree",
           "get_edges", "check_args", "EvtError"]

_GPU_DEVICES = ("gpu", "rocm", "amd", "hip")
_LOSS_K = {"mse": 1, "logloss": 1, "gaussian_mle": 2}


def _device_check(device):
    name = str(device).lstrip(":")
    if name not in _GPU_DEVICES:
        raise ValueError("this backend only runs on the GPU: device must be one of %s, got %r" % (_GPU_DEVICES, device))


def check_args(args):
    """check_args, src/learners.jl:522-552."""
    def rng(name, lo, hi, integer=False):
        v = args[name]
        if integer and int(v) != v:
            raise ValueError("%s must be an integer" % name)
        if not (lo <= v <= hi):
            raise ValueError("%s must be in [%s, %s], got %s" % (name, lo, hi, v))
    rng("nrounds", 0, 2 ** 62, True)
    rng("max_depth", 1, 16, True)
    rng("nbins", 2, 255, True)
    for n in ("lambda_", "gamma", "min_weight", "L2"):
        rng(n, 0.0, float("inf"))
    eps = np.finfo(np.float64).eps
    rng("rowsample", eps, 1.0)
    rng("colsample", eps, 1.0)
    rng("eta", 0.0, float("inf"))
    if args["tree_type"] not in ("binary", "oblivious"):
        raise ValueError("Invalid input for `tree_type` parameter: `%s`. Must be of one of `binary` or `oblivious`" % args["tree_type"])
    if args["bagging_size"] < 1:
        raise ValueError("bagging_size must be >= 1")


class _Learner:
    _losses = ()
    _defaults = dict(loss="mse", nrounds=100, bagging_size=1, L2=1.0, lambda_=0.0, gamma=0.0, eta=0.1, max_depth=6, min_weight=1.0,
                     rowsample=1.0, colsample=1.0, nbins=64, monotone_constraints=None, tree_type="binary", seed=123, device="gpu")

    def __init__(self, **kwargs):
        if "lambda" in kwargs:
            kwargs["lambda_"] = kwargs.pop("lambda")
        args = dict(self._defaults)
        unknown = set(kwargs) - set(args)
        if unknown:
            raise TypeError("unsupported arguments: %s" % sorted(unknown))
        args.update(kwargs)
        args["loss"] = str(args["loss"]).lstrip(":")
        args["tree_type"] = str(args["tree_type"]).lstrip(":")
        if args["loss"] not in self._losses:
            raise ValueError("Invalid loss. Must be one of: %s" % (list(self._losses),))
        args["monotone_constraints"] = dict(args["monotone_constraints"] or {})
        check_args(args)
        self.__dict__.update(args)


class EvoTreeRegressor(_Learner):
    """EvoTreeRegressor (src/learners.jl:1-119), losses mse and logloss."""
    _losses = ("mse", "logloss")


class EvoTreeMLE(_Learner):
    """EvoTreeMLE (src/learners.jl:300-400), loss gaussian_mle; min_weight defaults to 8."""
    _losses = ("gaussian_mle",)
    _defaults = dict(_Learner._defaults, loss="gaussian_mle", min_weight=8.0)


class Tree(TreeArrays):
    """Tree{L,K} (src/structs.jl:77-106)."""

    @staticmethod
    def bias(mu):
        t = Tree(len(mu), 1)
        t.pred[0, :] = mu
        return t


class EvoTree:
    """EvoTree{L,K} (src/structs.jl:129-138): trees[0] is the bias tree."""

    def __init__(self, loss, K, trees, info):
        self.loss_type, self.K, self.trees, self.info = loss, K, trees, info

    def __call__(self, data, ntree_limit=None, device="gpu"):
        return predict(self, data, ntree_limit=ntree_limit, device=device)


def get_edges(x, nbins, rng):
    """get_edges, src/fit-utils.jl:7-24: type-7 quantiles at (1..nbins-1)/nbins of <= 1000*nbins sampled rows."""
    N, F = x.shape
    nobs = min(N, 1000 * nbins)
    idx = np.sort(rng.choice(N, nobs, replace=False)) if nobs < N else np.arange(N)
    q = np.arange(1, nbins) / nbins
    edges = []
    for j in range(F):
        col = np.asarray(x[idx, j], np.float64)
        e = np.quantile(col, q)  # numpy's default is the linear (type 7) rule Statistics.quantile uses
        if e.shape[0] == 1:
            e = np.array([col.min()])
        edges.append(np.ascontiguousarray(e))
    featbins = np.array([len(e) + 1 for e in edges], np.uint8)
    feattypes = np.ones(F, np.uint8)
    return edges, featbins, feattypes


def _logit(p):
    return np.log(p / (1 - p))


def _invsoftplus(x):
    return x + np.log(-np.expm1(-x))


def _init_target(loss, y):
    """_init_target, src/init.jl:10-146 (in-scope branches)."""
    y = np.asarray(y)
    if y.ndim != 1:
        raise ValueError("only vector targets are supported by this backend")
    y32 = y.astype(np.float32)
    if loss == "logloss":
        if y32.min() < 0 or y32.max() > 1:
            raise AssertionError("logloss targets must be in [0, 1]")
        mu = np.array([_logit(np.float32(y32.mean(dtype=np.float32)))], np.float32)
    elif loss == "gaussian_mle":
        m = np.float32(y32.mean(dtype=np.float32))
        s = np.float32(y32.std(ddof=1, dtype=np.float32))
        mu = np.array([m, _invsoftplus(s)], np.float32)
    else:
        mu = np.array([y32.mean(dtype=np.float32)], np.float32)
    return _LOSS_K[loss], y32, mu.astype(np.float32)


class Cache:
    """What CacheBaseGPU holds on the host side: the device handle plus RNG and sampling sizes."""

    def __init__(self, handle, rng, nfs, params, N, F):
        self.handle, self.rng, self.nfs, self.params, self.N, self.F = handle, rng, nfs, params, N, F


def init(config, x_train, y_train, w_train=None, offset_train=None, feature_names=None, device=None):
    """init / init_core for the GPU device (src/init.jl:316-339; ext/EvoTreesKernelAbstractionsExt/init.jl:1-151)."""
    _device_check(config.device if device is None else device)
    x = np.asarray(x_train)
    if x.ndim != 2:
        raise ValueError("x_train must be a matrix")
    N, F = x.shape
    feature_names = ["feat_%d" % (j + 1) for j in range(F)] if feature_names is None else [str(f) for f in feature_names]
    if len(feature_names) != F:
        raise AssertionError("length(feature_names) must equal size(x_train, 2)")
    rng = np.random.default_rng(config.seed)
    edges, featbins, feattypes = get_edges(x, config.nbins, rng)
    K, y32, mu = _init_target(config.loss, y_train)
    if y32.shape[0] != N:
        raise AssertionError("target length must equal the number of rows")
    w = None
    if w_train is not None:
        w = np.asarray(w_train, np.float32)
        if w.shape != (N,) or not (w.min() > 0):
            raise AssertionError("weights must be positive and match the number of rows")
    offset = None
    if offset_train is not None:
        offset = np.array(offset_train, np.float32).reshape(N, K)
        if config.loss == "logloss":
            offset = _logit(offset)
        elif config.loss == "gaussian_mle":
            offset[:, 1] = _invsoftplus(offset[:, 1])
        mu = np.zeros_like(mu)  # neutral bias when an offset is given (src/init.jl:164)
    h = Handle(N, F, config.nbins, K, config.max_depth, config.loss, config.tree_type)
    x_FN = np.ascontiguousarray(x.T, np.float64)
    h.binarize(x_FN, edges)
    mono = np.zeros(F, np.int32)
    for k, v in config.monotone_constraints.items():
        mono[int(k) - 1] = int(v)
    h.set_feature_meta(feattypes, mono)
    h.set_target(y32, w, mu, offset)
    info = dict(nrounds=0, feature_names=feature_names, target_levels=None, target_isordered=False, edges=edges, featbins=featbins,
                feattypes=feattypes)
    m = EvoTree(config.loss, K, [Tree.bias(mu)], info)
    nfs = int(np.ceil(config.colsample * F))
    params = make_params(config.eta, config.L2, config.lambda_, config.gamma, config.min_weight, config.bagging_size, True)
    return m, Cache(h, rng, nfs, params, N, F)


def grow_evotree(m, cache, config):
    """grow_evotree!, src/fit.jl:6-42 (device twin ext/.../fit.jl:1-21): gradients, then bagging_size trees."""
    h = cache.handle
    h.update_grads()
    cond = int(np.rint(255 * config.rowsample))  # round(UInt8, 255*rowsample), src/subsample.jl:9
    for _ in range(config.bagging_size):
        # all rows pass `mask <= 255`, so the draw is skipped when nothing can be dropped
        mask = None if cond >= 255 else cache.rng.integers(0, 256, cache.N, dtype=np.uint8)
        if cache.nfs >= cache.F:
            js = np.arange(1, cache.F + 1, dtype=np.uint32)
        else:
            js = (np.sort(cache.rng.choice(cache.F, cache.nfs, replace=False)) + 1).astype(np.uint32)
        t = Tree(m.K, h.nnodes)
        out = t.as_out()
        try:
            _lib.check(_lib.load().evt_grow_tree(h._h, _lib.ptr(mask), cond, _lib.ptr(js), js.shape[0], cache.params, out))
        except EvtError as e:
            if e.code == _lib.EVT_ERR_EMPTY:
                raise RuntimeError("no subsample observation - choose larger rowsample") from e
            raise
        m.trees.append(t)
    m.info["nrounds"] += 1


def fit(config, x_train=None, y_train=None, w_train=None, offset_train=None, feature_names=None, device=None, verbosity=1,
        return_cache=False):
    """fit(params; x_train, y_train, ...), src/fit.jl:388-437 (no eval set: the callback is outside this backend)."""
    if x_train is None or y_train is None:
        raise TypeError("x_train and y_train are required")
    m, cache = init(config, x_train, y_train, w_train=w_train, offset_train=offset_train, feature_names=feature_names, device=device)
    try:
        for _ in range(config.nrounds):
            grow_evotree(m, cache, config)
    finally:
        if not return_cache:
            cache.handle.close()  # post_fit_gc slot, src/fit.jl:340
    m.info["logger"] = None
    return (m, cache) if return_cache else m


def binarize(x, edges):
    """binarize, src/fit-utils.jl:66-72 — host version used for inference inputs (searchsortedfirst)."""
    x = np.asarray(x)
    F = x.shape[1]
    out = np.empty((F, x.shape[0]), np.uint8)
    for j in range(F):
        out[j] = np.searchsorted(edges[j], x[:, j], side="left") + 1
    return out


def predict(m, data, ntree_limit=None, device="gpu"):
    """_predict, ext/.../predict.jl:115-135: binarize, walk the first ntree_limit trees, apply the link."""
    _device_check(device)
    ntrees = len(m.trees)
    ntree_limit = ntrees if ntree_limit is None else ntree_limit
    if ntree_limit > ntrees:
        raise RuntimeError("ntree_limit is larger than number of trees %d." % ntrees)
    x_bin = binarize(data, m.info["edges"])
    p = _lib.predict_model(x_bin, m.info["feattypes"], m.loss_type, m.K, m.trees[:ntree_limit], apply_link=True)
    return p[:, 0].copy() if m.K == 1 else p


def predict_leaf_idx(m, data, ntree_limit=None, device="gpu"):
    """predict_leaf_idx, src/predict.jl:173-185 -> (nobs, ntree_limit) uint32."""
    _device_check(device)
    ntrees = len(m.trees)
    ntree_limit = ntrees if ntree_limit is None else ntree_limit
    if ntree_limit > ntrees:
        raise RuntimeError("ntree_limit is larger than number of trees %d." % ntrees)
    x_bin = binarize(data, m.info["edges"])
    return _lib.predict_leaf_idx(x_bin, m.info["feattypes"], m.trees[:ntree_limit])
