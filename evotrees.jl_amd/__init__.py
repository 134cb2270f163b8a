"""Host side of the MI355X tree-building backend, mirroring EvoTrees.jl's interface for the
hot path: learner configs (src/learners.jl), `fit(config; x_train, y_train, ...)`
(src/fit.jl:388-437), the model functor `m(x; ntree_limit, device)` (src/structs.jl:135-138),
`predict` (src/predict.jl:93-96) and `predict_leaf_idx` (src/predict.jl:173-185).

Everything data parallel runs in libevotrees_hip.so through the C ABI; this module only keeps
what the reference keeps on the host: argument checks, quantile edges, the bias, the random
column sample, the seed of each tree's row mask (the mask bytes themselves are drawn on the
device from it), and the list of trees.  There is no CPU compute path: `device` must be
a GPU device name and the shared library must be present.

Julia is not available where this package is developed, so the host side is Python; the random
streams are numpy's (PCG64), not Julia's Xoshiro, hence models are not stream-identical to a
Julia run with the same seed — the trees are identical for identical masks/column samples.
"""
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np

from . import _lib
from ._lib import EvtError, Handle, TreeArrays, make_params, splitmix_mask  # noqa: F401

__all__ = ["EvoTreeRegressor", "EvoTreeCount", "EvoTreeClassifier", "EvoTreeMLE", "EvoTree", "Tree", "fit", "predict", "predict_leaf_idx", "init",
           "grow_evotree", "update", "okay_to_continue", "get_edges", "get_edges_table", "binarize_table", "check_args", "CallBack", "init_logger", "update_logger", "EvtError"]

_GPU_DEVICES = ("gpu", "rocm", "amd", "hip")
_EXP_LINK = ("poisson", "gamma", "tweedie")
# is_maximise, src/metrics.jl:195-207
_MAXIMISE = {"mse": False, "rmse": False, "mae": False, "logloss": False, "poisson": False, "gamma": False, "tweedie": False,
             "gaussian_mle": True, "logistic_mle": True, "mlogloss": False, "quantile": False, "multiquantile": False}


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
    rng("early_stopping_rounds", 1, float("inf"))
    rng("early_stopping_tolerance", 0.0, float("inf"))
    if "alpha" in args:
        rng("alpha", 0.0, 1.0)
    if args.get("loss") == "multiquantile":  # check_alphas, src/learners.jl:504-515
        al = [float(a) for a in (args.get("alphas") or [])]
        if not al or any(not (0.0 < a < 1.0) for a in al) or any(b <= a for a, b in zip(al, al[1:])):
            raise ValueError("Invalid value for parameter `alphas`: %s. `alphas` must be a non-empty, strictly increasing vector with "
                             "values in (0, 1)." % (args.get("alphas"),))


class _Learner:
    _losses = ()
    _metrics = ()
    _defaults = dict(loss="mse", metric=None, early_stopping_rounds=2 ** 62, early_stopping_tolerance=0.0, nrounds=100, bagging_size=1, L2=1.0, lambda_=0.0, gamma=0.0, eta=0.1, max_depth=6, min_weight=1.0,
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
        if args["metric"] is None:  # the loss itself; mae for the credibility losses (src/learners.jl:76-81)
            args["metric"] = "mae" if args["loss"] in ("cred_var", "cred_std") else args["loss"]
        else:
            args["metric"] = str(args["metric"]).lstrip(":")
        if args["metric"] not in self._metrics:
            raise ValueError("Invalid metric. Must be one of: %s" % (list(self._metrics),))
        args["monotone_constraints"] = dict(args["monotone_constraints"] or {})
        check_args(args)
        self.__dict__.update(args)


class EvoTreeRegressor(_Learner):
    """EvoTreeRegressor (src/learners.jl:1-119); losses mse, logloss, poisson, gamma, tweedie, mae, quantile (level `alpha`),
    multiquantile (levels `alphas`, one output each), cred_var, cred_std."""
    _losses = ("mse", "logloss", "poisson", "gamma", "tweedie", "mae", "quantile", "multiquantile", "cred_var", "cred_std")
    _metrics = ("mse", "rmse", "mae", "logloss", "poisson", "gamma", "tweedie", "quantile", "multiquantile")
    _defaults = dict(_Learner._defaults, alpha=0.5, alphas=(0.1, 0.5, 0.9))


class EvoTreeCount(_Learner):
    """EvoTreeCount (src/learners.jl:121-205): poisson loss and metric."""
    _losses = ("poisson",)
    _metrics = ("poisson",)
    _defaults = dict(_Learner._defaults, loss="poisson")


class EvoTreeClassifier(_Learner):
    """EvoTreeClassifier (src/learners.jl:207-290): multi-class log loss over the levels of the target."""
    _losses = ("mlogloss",)
    _metrics = ("mlogloss",)
    _defaults = dict(_Learner._defaults, loss="mlogloss")


class EvoTreeMLE(_Learner):
    """EvoTreeMLE (src/learners.jl:300-400), losses gaussian_mle and logistic_mle; min_weight defaults to 8."""
    _losses = ("gaussian_mle", "logistic_mle")
    _metrics = ("gaussian_mle", "logistic_mle")
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


def _per_feature(fn, F):
    """[fn(0), ..., fn(F - 1)], on a few threads when there are enough features (numpy's sorts release the GIL)."""
    workers = min(16, os.cpu_count() or 1, F)
    if workers < 2 or F < 8:
        return [fn(j) for j in range(F)]
    with ThreadPoolExecutor(workers) as ex:
        return list(ex.map(fn, range(F)))


def get_edges(x, nbins, rng):
    """get_edges, src/fit-utils.jl:7-24: type-7 quantiles at (1..nbins-1)/nbins of <= 1000*nbins sampled rows."""
    N, F = x.shape
    nobs = min(N, 1000 * nbins)
    idx = np.sort(rng.choice(N, nobs, replace=False)) if nobs < N else np.arange(N)
    q = np.arange(1, nbins) / nbins

    def one(j):
        col = np.asarray(x[idx, j], np.float64)
        e = np.quantile(col, q)  # numpy's default is the linear (type 7) rule Statistics.quantile uses
        if e.shape[0] == 1:
            e = np.array([col.min()])
        return np.ascontiguousarray(e)

    edges = _per_feature(one, F)  # `@threads for j`, src/fit-utils.jl:15: the features are independent
    featbins = np.array([len(e) + 1 for e in edges], np.uint8)
    feattypes = np.ones(F, np.uint8)
    return edges, featbins, feattypes


def _logit(p):
    return np.log(p / (1 - p))


def _invsoftplus(x):
    return x + np.log(-np.expm1(-x))


def _levelcode(y, levels):
    """1-based position of every element of y in `levels` (eval_levelcode, src/callback.jl:11-19)."""
    levels = np.asarray(levels)
    order = np.argsort(levels, kind="stable")
    pos = np.searchsorted(levels[order], y)
    pos = np.clip(pos, 0, len(levels) - 1)
    found = levels[order][pos] == y
    if not found.all():
        raise RuntimeError("`y_eval` contains levels absent from `y_train`: %s. Training levels are %s."
                           % (sorted(set(np.asarray(y)[~found].tolist())), levels.tolist()))
    return (order[pos] + 1).astype(np.float32)


def _target_rows(y):
    """A vector target is one row; a matrix target holds one row per target (T x nobs, as the reference takes it)."""
    y = np.asarray(y)
    if y.ndim == 1:
        return y[None, :]
    if y.ndim != 2:
        raise ValueError("the target must be a vector or a targets x observations matrix")
    return y


def _init_target(loss, y, alphas=None):
    """_init_target, src/init.jl:10-146 (in-scope branches).  Returns K, y (Float32; (N,) for one target, (N, T) for a
    T x N matrix target), mu, target levels."""
    y = np.asarray(y)
    if loss == "mlogloss":  # src/init.jl:43-67: levels = sort(unique(y)), level codes, mu = log(proportions) - max
        if y.ndim != 1:  # src/init.jl:11-16
            raise RuntimeError("Multi-target (matrix target) is supported for gradient-regression losses (mse, logloss, poisson, "
                               "gamma, tweedie) and gaussian_mle. Got loss mlogloss.")
        if y.dtype.kind == "f":
            raise RuntimeError("Invalid target eltype: %s" % y.dtype)
        levels = np.unique(y)
        K = len(levels)
        if K < 2:
            raise RuntimeError("Classification requires a target with at least 2 levels, got %d: %s. "
                               "A single-class problem is not meaningful." % (K, levels.tolist()))
        codes = _levelcode(y, levels)
        prop = np.bincount(codes.astype(np.int64) - 1, minlength=K) / float(len(y))
        mu = np.log(prop).astype(np.float32)
        mu = mu - mu.max()
        return K, codes, mu.astype(np.float32), levels
    if loss == "multiquantile":  # src/init.jl:101-105: one target, an output per level, each starting at its quantile of y
        if y.ndim != 1:
            raise RuntimeError("Multi-target (matrix target) is not supported for loss multiquantile: its outputs are the levels.")
        y32 = y.astype(np.float32)
        mu = np.quantile(y32.astype(np.float64), [float(a) for a in alphas], method="linear").astype(np.float32)
        return mu.shape[0], y32, mu, None
    rows = _target_rows(y).astype(np.float32)  # T x N
    if loss == "logloss" and (rows.min() < 0 or rows.max() > 1):
        raise AssertionError("logloss targets must be in [0, 1]")
    mu = []
    for yt in rows:  # one bias per target (two for gaussian_mle), src/init.jl:24-31, :33-41, :68-83, :137-150
        m = np.float32(yt.mean(dtype=np.float32))
        if loss == "logloss":
            mu.append(_logit(m))
        elif loss == "gaussian_mle":
            mu += [m, _invsoftplus(np.float32(yt.std(ddof=1, dtype=np.float32)))]
        elif loss == "logistic_mle":  # src/init.jl:84-100: scale = std * sqrt(3) / pi, evaluated in Float64
            mu += [m, _invsoftplus(np.float64(np.float32(yt.std(ddof=1, dtype=np.float32))) * np.sqrt(3.0) / np.pi)]
        elif loss in _EXP_LINK:
            mu.append(np.log(m))
        else:
            mu.append(m)
    mu = np.array(mu, np.float32)
    y32 = rows[0] if y.ndim == 1 else np.ascontiguousarray(rows.T)
    return mu.shape[0], y32, mu, None


def _link_offset(loss, offset, N, K):
    """Offsets are given on the response scale and moved to the linear one (src/init.jl:30, :43, :69; src/callback.jl:76-80)."""
    offset = np.array(offset, np.float32).reshape(N, K)
    if loss == "logloss":
        offset = _logit(offset)
    elif loss in _EXP_LINK or loss == "mlogloss":
        offset = np.log(offset)
    elif loss in ("gaussian_mle", "logistic_mle"):
        offset[:, 1::2] = _invsoftplus(offset[:, 1::2])  # every scale column (unconstrain_mle_scale!)
    return offset.astype(np.float32)


def _is_table(data):
    """Tables.istable: a pandas DataFrame or a dict of equally long columns."""
    if isinstance(data, dict):
        return True
    return hasattr(data, "columns") and hasattr(data, "dtypes")


def _column(data, name):
    """Tables.getcolumn as a numpy array or a pandas Categorical."""
    col = data[name]
    if hasattr(col, "dtype") and str(col.dtype) == "category":
        return col.array if hasattr(col, "array") else col
    return np.asarray(col)


def _is_categorical(col):
    return hasattr(col, "categories") and hasattr(col, "codes")


def _table_names(data):
    return [str(c) for c in (data.keys() if isinstance(data, dict) else data.columns)]


def get_edges_table(data, feature_names, nbins, rng):
    """get_edges for Tables input, src/fit-utils.jl:26-63: a Bool column is a two-level categorical feature, a
    categorical column is split on its levels (`==`, or `<=` when its levels are ordered), a Real column on the unique
    quantiles of the sampled rows."""
    nrow = len(_column(data, feature_names[0]))
    nobs = min(nrow, 1000 * nbins)
    idx = np.sort(rng.choice(nrow, nobs, replace=False)) if nobs < nrow else np.arange(nrow)
    q = np.arange(1, nbins) / nbins
    edges, featbins, feattypes = [], [], []
    for name in feature_names:
        col = _column(data, name)
        if _is_categorical(col):
            e = list(col.categories)
            nb, ft = len(e), bool(col.ordered)
            if nb > nbins:
                raise RuntimeError("Max categorical levels is limited to `nbins` (%d). Feature %s has %d levels. Consider using larger "
                                   "`nbins`, up to 255." % (nbins, name, nb))
        elif col.dtype == np.bool_:
            e, nb, ft = [False, True], 2, False
        elif col.dtype.kind in "iuf":
            sub = np.asarray(col[idx], np.float64)
            e = np.unique(np.quantile(sub, q))
            if e.shape[0] == 1:
                e = np.array([sub.min()])
            e = np.ascontiguousarray(e)
            nb, ft = len(e) + 1, True
        else:
            raise RuntimeError("Invalid feature eltype: %s is %s" % (name, col.dtype))
        edges.append(e)
        featbins.append(nb)
        feattypes.append(1 if ft else 0)
    return edges, np.array(featbins, np.uint8), np.array(feattypes, np.uint8)


def binarize_table(data, feature_names, edges):
    """binarize for Tables input, src/fit-utils.jl:74-92 -> (F, N) uint8 (the memory order of Julia's N x F matrix)."""
    nrow = len(_column(data, feature_names[0]))
    out = np.empty((len(feature_names), nrow), np.uint8)
    for j, name in enumerate(feature_names):
        col = _column(data, name)
        if _is_categorical(col):
            if list(col.categories) != list(edges[j]):  # levelcode refers to the training levels
                col = col.set_categories(list(edges[j]))
            codes = np.asarray(col.codes)
            if (codes < 0).any():
                raise RuntimeError("feature %s holds missing values or levels the model was not trained on" % name)
            out[j] = codes + 1
        elif col.dtype == np.bool_:
            out[j] = col.astype(np.uint8) + 1
        elif col.dtype.kind in "iuf":
            out[j] = binarize(np.asarray(col, np.float64)[:, None], [edges[j]])[0]
        else:
            raise RuntimeError("Invalid feature eltype: %s is %s" % (name, col.dtype))
    return out


def _table_features(data, target_names, weight_name, offset_name, feature_names):
    """Feature columns of a table: the names given, or every Real / categorical column that is not the target, the
    weight or the offset (src/init.jl:253-282)."""
    names = _table_names(data)
    if feature_names is None:
        skip = set(target_names) | {weight_name, offset_name}
        out = []
        for n in names:
            col = _column(data, n)
            if n not in skip and (_is_categorical(col) or col.dtype == np.bool_ or col.dtype.kind in "iuf"):
                out.append(n)
        return out
    out = [feature_names] if isinstance(feature_names, str) else [str(f) for f in feature_names]
    for n in out:
        if n not in names:
            raise AssertionError("feature %s is not a column of the table" % n)
    return out


def _table_target(data, target_name):
    names = [str(t) for t in target_name] if isinstance(target_name, (list, tuple)) else [str(target_name)]
    if len(names) == 1:
        return names, np.asarray(data[names[0]])
    return names, np.stack([np.asarray(data[t]) for t in names])  # targets x observations


class Cache:
    """What CacheBaseGPU holds on the host side: the device handle plus RNG and sampling sizes."""

    def __init__(self, handle, rng, nfs, params, N, F, config=None):
        self.handle, self.rng, self.nfs, self.params, self.N, self.F, self.config = handle, rng, nfs, params, N, F, config
        self.pending = []  # trees queued on the device and not yet collected, oldest first (at most two)


def init(config, x_train, y_train=None, w_train=None, offset_train=None, feature_names=None, device=None, target_name=None, weight_name=None,
         offset_name=None):
    """init / init_core for the GPU device (src/init.jl:236-339; ext/EvoTreesKernelAbstractionsExt/init.jl:1-151).  x_train is a
    matrix (with y_train, w_train, offset_train) or a table (with target_name, weight_name, offset_name)."""
    _device_check(config.device if device is None else device)
    rng = np.random.default_rng(config.seed)
    table = _is_table(x_train)
    if table:
        if target_name is None:
            raise TypeError("target_name is required for a table")
        target_names, y_train = _table_target(x_train, target_name)
        feature_names = _table_features(x_train, target_names, weight_name, offset_name, feature_names)
        w_train = None if weight_name is None else np.asarray(x_train[str(weight_name)])
        offset_train = None if offset_name is None else np.asarray(x_train[str(offset_name)])
        F = len(feature_names)
        N = len(_column(x_train, feature_names[0]))
        edges, featbins, feattypes = get_edges_table(x_train, feature_names, config.nbins, rng)
    else:
        x = np.asarray(x_train)
        if x.ndim != 2:
            raise ValueError("x_train must be a matrix")
        N, F = x.shape
        feature_names = ["feat_%d" % (j + 1) for j in range(F)] if feature_names is None else [str(f) for f in feature_names]
        if len(feature_names) != F:
            raise AssertionError("length(feature_names) must equal size(x_train, 2)")
        edges, featbins, feattypes = get_edges(x, config.nbins, rng)
    K, y32, mu, target_levels = _init_target(config.loss, y_train, getattr(config, "alphas", None))
    if y32.shape[0] != N:
        raise AssertionError("target length must equal the number of rows")
    w = None
    if w_train is not None:
        w = np.asarray(w_train, np.float32)
        if w.shape != (N,) or not (w.min() > 0):
            raise AssertionError("weights must be positive and match the number of rows")
    offset = None
    if offset_train is not None:
        offset = _link_offset(config.loss, offset_train, N, K)
        mu = np.zeros_like(mu)  # neutral bias when an offset is given (src/init.jl:164)
    h = Handle(N, F, config.nbins, K, config.max_depth, config.loss, config.tree_type)
    if table:  # Bool and categorical columns have no edges to search: binned on the host as the reference does
        h.set_xbin(binarize_table(x_train, feature_names, edges))
    else:
        # the library takes the reference's memory order (column-major, a Julia matrix as it lies): free for a Fortran-ordered
        # numpy array, a transposing host copy for a C-ordered one
        h.binarize(np.ascontiguousarray(x.T, np.float64), edges)
    mono = np.zeros(F, np.int32)
    for k, v in config.monotone_constraints.items():
        mono[int(k) - 1] = int(v)
    h.set_feature_meta(feattypes, mono)
    _set_levels(h, config)
    h.set_target(y32, w, mu, offset)
    info = dict(nrounds=0, feature_names=feature_names, target_levels=target_levels, target_isordered=False, edges=edges, featbins=featbins,
                feattypes=feattypes)
    m = EvoTree(config.loss, K, [Tree.bias(mu)], info)
    nfs = int(np.ceil(config.colsample * F))
    params = make_params(config.eta, config.L2, config.lambda_, config.gamma, config.min_weight, config.bagging_size, True)
    if config.bagging_size == 1:
        h.set_option("grads_ahead", 1)  # the next round's gradient update runs while the host collects the tree
    return m, Cache(h, rng, nfs, params, N, F, config)


def _begin_tree(cache, config, first_of_round):
    """Queues one tree on the device (the round's gradient update first): the generator's draws of the tree in the
    reference's order (mask, then columns; src/fit.jl:13-20), then evt_grow_tree_begin.  All rows pass `mask <= 255`, so
    nothing is drawn for the mask when nothing can be dropped."""
    h = cache.handle
    if first_of_round:
        h.update_grads()
    cond = int(np.rint(255 * config.rowsample))  # round(UInt8, 255*rowsample), src/subsample.jl:9
    seed = int(cache.rng.integers(0, 1 << 64, dtype=np.uint64)) if cond < 255 else None
    if cache.nfs >= cache.F:
        js = np.arange(1, cache.F + 1, dtype=np.uint32)
    else:
        js = (np.sort(cache.rng.choice(cache.F, cache.nfs, replace=False)) + 1).astype(np.uint32)
    if seed is not None:
        h.draw_mask(seed)
        _lib.check(_lib.load().evt_grow_tree_begin_staged(h._h, cond, _lib.ptr(js), js.shape[0], cache.params))
    else:
        _lib.check(_lib.load().evt_grow_tree_begin(h._h, None, cond, _lib.ptr(js), js.shape[0], cache.params))
    cache.pending.append(Tree(h.K, h.nnodes))


def grow_evotree(m, cache, config, more=False):
    """grow_evotree!, src/fit.jl:6-42 (device twin ext/.../fit.jl:1-21): gradients, then bagging_size trees.

    The row mask of a tree (rand!(rng, mask), src/subsample.jl:7) is drawn on the device from ONE 64-bit draw of the
    fit's generator per tree (Handle.draw_mask: SplitMix64 keyed by that draw; splitmix_mask gives the same bytes on the
    host): numpy needs 4 ns per 8 mask bytes, which at a million rows is already longer than the device takes to grow
    the tree.  The bytes are compared with round(UInt8, 255 * rowsample) exactly as an uploaded mask is.

    The device runs one tree ahead of the host: a tree is queued before the one before it is collected (the library
    takes two trees in flight), so the device does not wait while the host copies a tree out and prepares the next
    call.  Within a round that is always possible; `more=True` says that another round follows and that nothing is read
    from the handle before it, so the next round's first tree is queued as well before this round's last is collected
    (the next call finds it in cache.pending).  Draws, trees and predictions are those of strictly alternating calls."""
    h = cache.handle
    n = config.bagging_size
    for b in range(n):
        if not cache.pending:
            _begin_tree(cache, config, b == 0)
        if b + 1 < n:
            _begin_tree(cache, config, False)
        elif more:
            _begin_tree(cache, config, True)
        t = cache.pending.pop(0)
        try:
            _lib.check(_lib.load().evt_grow_tree_end(h._h, t.as_out()))
        except EvtError as e:
            if e.code == _lib.EVT_ERR_EMPTY:
                raise RuntimeError("no subsample observation - choose larger rowsample") from e
            raise
        m.trees.append(t)
    m.info["nrounds"] += 1


def _set_levels(h, config):
    """params.alpha / params.alphas of the quantile losses and metrics (src/callback.jl:62-66)."""
    if config.loss == "multiquantile":
        h.set_alphas([float(a) for a in config.alphas])
    elif hasattr(config, "alpha"):
        h.set_alphas([float(config.alpha)])


class CallBack:
    """CallBack (src/callback.jl:21-135) on the device: a second handle holds the binned eval rows, their
    running prediction, target and weights; each call adds one tree and evaluates the metric there."""

    def __init__(self, config, m, x_eval, y_eval=None, w_eval=None, offset_eval=None, target_name=None, weight_name=None, offset_name=None):
        table = _is_table(x_eval)
        if table:  # the Tables form, src/callback.jl:31-80
            _, y_eval = _table_target(x_eval, target_name)
            w_eval = None if weight_name is None else np.asarray(x_eval[str(weight_name)])
            offset_eval = None if offset_name is None else np.asarray(x_eval[str(offset_name)])
            x_bin = binarize_table(x_eval, m.info["feature_names"], m.info["edges"])
            F, N = x_bin.shape
        else:
            x = np.asarray(x_eval)
            N, F = x.shape
        self.metric = config.metric
        self.maximise = _MAXIMISE[config.metric]
        if m.loss_type == "mlogloss":
            y32 = _levelcode(np.asarray(y_eval), m.info["target_levels"])
        else:
            ye = np.asarray(y_eval).astype(np.float32)
            y32 = ye if ye.ndim == 1 else np.ascontiguousarray(ye.T)  # a matrix target is targets x observations
        if y32.shape[0] != N:
            raise AssertionError("y_eval length must equal the number of eval rows")
        w = None if w_eval is None else np.asarray(w_eval, np.float32)
        offset = None if offset_eval is None else _link_offset(m.loss_type, offset_eval, N, m.K)
        h = Handle(N, F, config.nbins, m.K, 1, m.loss_type, "binary")
        try:
            if table:
                h.set_xbin(x_bin)
            else:
                h.binarize(np.ascontiguousarray(x.T, np.float64), m.info["edges"])
            h.set_feature_meta(m.info["feattypes"], None)
            _set_levels(h, config)
            h.set_target(y32, w, np.zeros(m.K, np.float32), offset)  # p = zeros (+ offset'), src/callback.jl:104, :82
        except Exception:
            h.close()
            raise
        self.handle = h

    def __call__(self, logger, it, tree):
        self.handle.predict_tree(tree)
        update_logger(logger, it, self.handle.eval_metric(self.metric))

    def close(self):
        self.handle.close()


def init_logger(metric, maximise, early_stopping_rounds, early_stopping_tolerance=0.0):
    """init_logger, src/callback.jl:137-151."""
    return dict(name=str(metric), maximise=maximise, early_stopping_rounds=early_stopping_rounds,
                early_stopping_tolerance=early_stopping_tolerance, nrounds=0, iter=[], metrics=[], iter_since_best=0, best_iter=0,
                best_metric=0.0)


def update_logger(logger, it, metric):
    """update_logger!, src/callback.jl:153-171."""
    logger["nrounds"] = it
    logger["iter"].append(it)
    logger["metrics"].append(metric)
    if it == 0:
        logger["best_metric"] = metric
        return
    tol = logger["early_stopping_tolerance"]
    improved = metric > logger["best_metric"] + tol if logger["maximise"] else metric < logger["best_metric"] - tol
    if improved:
        logger["best_metric"] = metric
        logger["best_iter"] = it
        logger["iter_since_best"] = 0
    else:
        logger["iter_since_best"] += logger["iter"][-1] - logger["iter"][-2]


def fit(config, dtrain=None, x_train=None, y_train=None, w_train=None, offset_train=None, x_eval=None, y_eval=None, w_eval=None, offset_eval=None,
        feature_names=None, print_every_n=9999, device=None, verbosity=1, return_cache=False, target_name=None, weight_name=None,
        offset_name=None, deval=None):
    """fit(params; x_train, y_train, ..., x_eval, y_eval, ...), src/fit.jl:388-437, and the Tables form
    fit(params, dtrain; target_name, feature_names, weight_name, offset_name, deval), src/fit.jl:302-345."""
    if dtrain is not None:
        if not _is_table(dtrain):
            raise AssertionError("fit(params, dtrain) only accepts Tables compatible input for `dtrain` (a DataFrame or a dict of columns)")
        m, cache = init(config, dtrain, feature_names=feature_names, device=device, target_name=target_name, weight_name=weight_name,
                        offset_name=offset_name)
        m.info["target_names"] = [str(t) for t in target_name] if isinstance(target_name, (list, tuple)) else [str(target_name)]
        x_eval, y_eval = None, None
    else:
        if x_train is None or y_train is None:
            raise TypeError("x_train and y_train are required")
        m, cache = init(config, x_train, y_train, w_train=w_train, offset_train=offset_train, feature_names=feature_names, device=device)
    logger, cb = None, None
    try:
        if dtrain is not None and deval is not None:
            cb = CallBack(config, m, deval, target_name=target_name, weight_name=weight_name, offset_name=offset_name)
            logger = init_logger(config.metric, cb.maximise, config.early_stopping_rounds, config.early_stopping_tolerance)
            cb(logger, 0, m.trees[-1])
            if verbosity > 0:
                print("initialization: %s = %.6g" % (config.metric, logger["metrics"][-1]))
        elif x_eval is not None and y_eval is not None:
            cb = CallBack(config, m, x_eval, y_eval, w_eval=w_eval, offset_eval=offset_eval)
            logger = init_logger(config.metric, cb.maximise, config.early_stopping_rounds, config.early_stopping_tolerance)
            cb(logger, 0, m.trees[-1])
            if verbosity > 0:
                print("initialization: %s = %.6g" % (config.metric, logger["metrics"][-1]))
        elif x_eval is not None or y_eval is not None:
            import warnings
            warnings.warn("To track eval metric in logger, both `x_eval` and `y_eval` must be provided.")
        for i in range(1, config.nrounds + 1):
            # without an eval set nothing is read between two rounds: the device may start the next one early
            grow_evotree(m, cache, config, more=(logger is None and i < config.nrounds))
            if logger is not None:
                cb(logger, i, m.trees[-1])  # as the reference: only the round's last tree reaches the eval prediction
                if i % print_every_n == 0 and verbosity > 0:
                    print("iter %d: %s = %.6g" % (i, config.metric, logger["metrics"][-1]))
                if logger["iter_since_best"] >= logger["early_stopping_rounds"]:
                    break
    finally:
        if cb is not None:
            cb.close()
        if not return_cache:
            cache.handle.close()  # post_fit_gc slot, src/fit.jl:340
    m.info["logger"] = logger
    return (m, cache) if return_cache else m


def okay_to_continue(config, m, cache):
    """okay_to_continue, src/MLJ.jl:30-33: only nrounds may differ, and it may not shrink below what is grown."""
    a, b = dict(config.__dict__), dict(cache.config.__dict__)
    a.pop("nrounds")
    b.pop("nrounds")
    return a == b and config.nrounds >= m.info["nrounds"]


def update(config, m, cache, x_train=None, y_train=None, w_train=None):
    """MMI.update, src/MLJ.jl:38-57: warm restart on the handle the first fit kept (`fit(..., return_cache=True)`);
    any change other than a larger nrounds refits from scratch."""
    if okay_to_continue(config, m, cache):
        while m.info["nrounds"] < config.nrounds:
            grow_evotree(m, cache, config, more=m.info["nrounds"] + 1 < config.nrounds)
        cache.config = config
        return m, cache
    cache.handle.close()
    return fit(config, x_train=x_train, y_train=y_train, w_train=w_train, return_cache=True)


def binarize(x, edges):
    """binarize, src/fit-utils.jl:66-72 — host version used for inference inputs (searchsortedfirst)."""
    x = np.asarray(x)
    F = x.shape[1]
    out = np.empty((F, x.shape[0]), np.uint8)
    for j in range(F):
        e = np.asarray(edges[j], np.float64)
        col = np.asarray(x[:, j], np.float64)
        idx = np.searchsorted(e, col, side="left")  # numpy orders NaN last, as isless does
        # isless also puts -0.0 before 0.0: a +0.0 value passes the -0.0 edges that `<` treats as equal
        pz = (col == 0) & ~np.signbit(col)
        if pz.any() and (e == 0).any():
            idx[pz] = np.searchsorted(e, 0.0, side="left") + int(((e == 0) & np.signbit(e)).sum())
        out[j] = idx + 1
    return out


def predict(m, data, ntree_limit=None, device="gpu"):
    """_predict, ext/.../predict.jl:115-135: binarize, walk the first ntree_limit trees, apply the link."""
    _device_check(device)
    ntrees = len(m.trees)
    ntree_limit = ntrees if ntree_limit is None else ntree_limit
    if ntree_limit > ntrees:
        raise RuntimeError("ntree_limit is larger than number of trees %d." % ntrees)
    if _is_table(data):  # Bool / categorical columns: binned on the host (src/fit-utils.jl:74-92), walked on the device
        x_bin = binarize_table(data, m.info["feature_names"], m.info["edges"])
        p = _lib.predict_model(x_bin, m.info["feattypes"], m.loss_type, m.K, m.trees[:ntree_limit], apply_link=True)
        return p[:, 0].copy() if m.K == 1 else p
    x_FN = np.ascontiguousarray(np.asarray(data).T, np.float64)
    p = _lib.predict_model_f64(x_FN, m.info["edges"], m.info["feattypes"], m.loss_type, m.K, m.trees[:ntree_limit], apply_link=True)
    return p[:, 0].copy() if m.K == 1 else p


def predict_leaf_idx(m, data, ntree_limit=None, device="gpu"):
    """predict_leaf_idx, src/predict.jl:173-185 -> (nobs, ntree_limit) uint32."""
    _device_check(device)
    ntrees = len(m.trees)
    ntree_limit = ntrees if ntree_limit is None else ntree_limit
    if ntree_limit > ntrees:
        raise RuntimeError("ntree_limit is larger than number of trees %d." % ntrees)
    x_bin = binarize_table(data, m.info["feature_names"], m.info["edges"]) if _is_table(data) else binarize(data, m.info["edges"])
    return _lib.predict_leaf_idx(x_bin, m.info["feattypes"], m.trees[:ntree_limit])
