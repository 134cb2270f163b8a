# EvoTreesHIP — the reference-side binding of libevotrees_hip.so.
#
# Loading this module next to EvoTrees.jl routes the device path of `fit` / `EvoTree` inference to the MI355X
# library: it owns, for the device types it claims, every generic function the reference's device seam consists of
# (ext/EvoTreesKernelAbstractionsExt.jl:17-27 and the files it includes), holds ONE opaque handle where the
# reference's CacheBaseGPU holds ~45 device arrays (ext/EvoTreesKernelAbstractionsExt/structs.jl:14-67), and forwards
# to the C ABI of include/evotrees_hip.h through `ccall`.  Host-side logic that must stay bit-compatible with the CPU
# path is NOT restated: `get_edges`, `binarize` (Tables input), `_init_target`, the Xoshiro mask and column-sample
# streams are the reference's own functions, called from here.
#
# Which `device=` reaches this module (src/structs.jl:8-15 maps the symbol to a device type):
#   :rocm, :amd -> EvoTrees.ROCmDevice : always claimed.
#   :gpu, :cuda -> EvoTrees.CUDADevice : claimed too unless ENV["EVOTREES_HIP_CLAIM_GPU"] == "0" when the module is
#                  loaded, so that `EvoTreeRegressor(device=:gpu)` / `m(x; device=:gpu)` work as written on an AMD box.
#                  (With CUDA.jl loaded, EvoTreesCUDAExt's `device_array_type(::Type{<:CUDADevice})` is the more
#                  specific method and wins: set the variable to "0" there and use :rocm for this library.)
# The methods below are declared on `Type{<:HIPDevice}`, which is strictly more specific than the
# `Type{<:EvoTrees.GPU}` the KernelAbstractions extension declares, so both can be loaded without ambiguity.
#
# This file has never been executed: no Julia toolchain exists where the library is built and tested.  The Python
# package next to the library (`evotrees.jl_amd/__init__.py`, `_lib.py`) is the executed twin of the same call sequence.
module EvoTreesHIP

using EvoTrees
using EvoTrees: EvoTree, Tree, EvoTypes
using EvoTrees.Random: rand!, Xoshiro
using EvoTrees.Tables

const LIB = get(ENV, "EVOTREES_HIP_LIB", joinpath(@__DIR__, "..", "evotrees.jl_amd", "libevotrees_hip.so"))

const CLAIM_GPU = get(ENV, "EVOTREES_HIP_CLAIM_GPU", "1") != "0"
const HIPDevice = CLAIM_GPU ? Union{EvoTrees.ROCmDevice,EvoTrees.CUDADevice} : EvoTrees.ROCmDevice

# ---------------------------------------------------------------------------------------------------------------
# C structs of include/evotrees_hip.h
struct EvtParams            # evt_params
    eta::Cdouble
    L2::Cdouble
    lambda::Cdouble
    gamma::Cdouble
    min_weight::Cdouble
    bagging_size::Cint
    update_pred::Cint
end
struct EvtTreeOut           # evt_tree_out: pointers into the arrays of a Tree{L,K} (src/structs.jl:77-84)
    feat::Ptr{Int64}
    cond_bin::Ptr{UInt8}
    w::Ptr{Float32}
    gain::Ptr{Float32}
    pred::Ptr{Float32}
    split::Ptr{Bool}
end

lasterr() = unsafe_string(ccall((:evt_last_error, LIB), Cstring, ()))
# the reference throws ErrorException (e.g. "no subsample observation", src/subsample.jl:36)
check(rc::Integer) = rc == 0 ? nothing : error(lasterr())

const LOSS_ID = Dict{Any,Cint}(
    EvoTrees.MSE => 0, EvoTrees.LogLoss => 1, EvoTrees.GaussianMLE => 2, EvoTrees.Poisson => 3,
    EvoTrees.Gamma => 4, EvoTrees.Tweedie => 5, EvoTrees.MLogLoss => 6, EvoTrees.LogisticMLE => 7,
    EvoTrees.MAE => 8, EvoTrees.CredVar => 9, EvoTrees.CredStd => 10, EvoTrees.Quantile => 11, EvoTrees.MultiQuantile => 12)
const METRIC_ID = Dict{Symbol,Cint}(
    :mse => 0, :rmse => 1, :mae => 2, :logloss => 3, :gaussian_mle => 4, :poisson => 5, :gamma => 6,
    :tweedie => 7, :mlogloss => 8, :logistic_mle => 9, :quantile => 10, :multiquantile => 11)
loss_id(::Type{L}) where {L} = haskey(LOSS_ID, L) ? LOSS_ID[L] : error("loss $L is not supported by libevotrees_hip (mse, logloss, poisson, gamma, tweedie, mlogloss, gaussian_mle, logistic_mle, mae, cred_var, cred_std, quantile, multiquantile)")

# ---------------------------------------------------------------------------------------------------------------
# device_array_type / device_ones: `init` calls both before `init_core` (src/init.jl:331-333, :283-285).  Host arrays
# cross the C ABI, so the "device array" of this backend is a plain Array: w and offset arrive as Vector{Float32} /
# Matrix{Float32}.  (The reference's twins: ext/EvoTreesAMDGPUExt.jl:7-8, ext/EvoTreesKernelAbstractionsExt.jl:20-21.)
EvoTrees.device_array_type(::Type{<:HIPDevice}) = Array
EvoTrees.device_ones(::Type{<:HIPDevice}, ::Type{T}, n::Int) where {T} = ones(T, n)
# gpu_backend (src/structs.jl:17) is only consulted by the KernelAbstractions kernels: not needed here.
# post_fit_gc (src/fit.jl:266, :340): the handle is freed by its finalizer; a full collection runs it.
EvoTrees.post_fit_gc(::Type{<:HIPDevice}) = GC.gc(true)

# ---------------------------------------------------------------------------------------------------------------
# The training cache: one handle.  <: CacheGPU so that `grow_evotree!(m, cache, params)` dispatches here
# (ext/EvoTreesKernelAbstractionsExt/fit.jl:1 is declared on ::EvoTrees.CacheGPU; ::CacheHIP is more specific).
mutable struct CacheHIP <: EvoTrees.CacheGPU
    h::Ptr{Cvoid}
    rng::Xoshiro
    mask::Vector{UInt8}
    js::Vector{UInt32}
    nfeats::Int
    K::Int
end

function destroy!(c::CacheHIP)
    if c.h != C_NULL
        ccall((:evt_destroy, LIB), Cint, (Ptr{Cvoid},), c.h)
        c.h = C_NULL
    end
    return nothing
end

# What the library does not take (evt_create, include/evotrees_hip.h): the reference has no such limits
# (src/learners.jl:525-527, src/init.jl:43-67), so a fit beyond them is sent back to the CPU path by name.
const MAX_OUTPUTS, MAX_DEPTH, MAX_FEATS = 16, 16, 65534
function check_limits(nfeats, K, max_depth)
    K <= MAX_OUTPUTS || error("libevotrees_hip takes at most $MAX_OUTPUTS outputs (this model has $K): fit it with device=:cpu")
    max_depth <= MAX_DEPTH || error("libevotrees_hip takes max_depth <= $MAX_DEPTH (got $max_depth): fit it with device=:cpu")
    nfeats <= MAX_FEATS || error("libevotrees_hip takes at most $MAX_FEATS features (got $nfeats): fit it with device=:cpu")
    return nothing
end

function create_handle(nobs, nfeats, nbins, K, max_depth, L, tree_type)
    check_limits(nfeats, K, max_depth)
    h = Ref{Ptr{Cvoid}}(C_NULL)
    check(ccall((:evt_create, LIB), Cint, (Int64, Cint, Cint, Cint, Cint, Cint, Cint, Ptr{Ptr{Cvoid}}),
        nobs, nfeats, nbins, K, max_depth, loss_id(L), tree_type == :oblivious ? 1 : 0, h))
    return h[]
end

# x_bin for a handle: a Float64 matrix is binned on the device (binarize, src/fit-utils.jl:66-72); anything else
# (Tables input with Bool / categorical columns, other element types) goes through the reference's own host
# `binarize` (src/fit-utils.jl:74-92) and is uploaded as UInt8.
function upload_features!(h::Ptr{Cvoid}, data, feature_names, edges)
    if data isa AbstractMatrix{Float64} && all(e -> e isa AbstractVector{Float64}, edges)
        x = data isa Matrix{Float64} ? data : Matrix{Float64}(data)   # column-major, as the ABI expects
        eflat = reduce(vcat, edges)
        eoff = Int32[0; cumsum(length.(edges))]
        GC.@preserve x eflat eoff check(ccall((:evt_binarize_f64, LIB), Cint,
            (Ptr{Cvoid}, Ptr{Float64}, Ptr{Float64}, Ptr{Int32}), h, x, eflat, eoff))
    else
        x_bin = EvoTrees.binarize(data; feature_names, edges)          # Matrix{UInt8}, nobs x nfeats
        GC.@preserve x_bin check(ccall((:evt_set_xbin, LIB), Cint, (Ptr{Cvoid}, Ptr{UInt8}), h, x_bin))
    end
    return nothing
end

# y as the ABI takes it: Float32, one value per row (the UInt32 level codes of mlogloss included) or the reference's
# targets x nobs matrix (src/init.jl:11-16); w == ones -> NULL (the row count then stands for the weight); offset is
# nobs x K on the host (src/init.jl:168-174 adds offset'), K x nobs across the ABI.
# params.alpha (every output of the quantile loss; also the level of the :quantile metric) or params.alphas (one output
# each, multiquantile): src/loss.jl:144-171, src/callback.jl:62-66
function upload_levels!(h::Ptr{Cvoid}, params, ::Type{L}) where {L}
    a = L == EvoTrees.MultiQuantile ? Vector{Float64}(params.alphas) :
        (hasproperty(params, :alpha) ? Float64[params.alpha] : Float64[])
    isempty(a) && return nothing
    GC.@preserve a check(ccall((:evt_set_alphas, LIB), Cint, (Ptr{Cvoid}, Ptr{Float64}, Cint), h, a, length(a)))
    return nothing
end

function upload_target!(h::Ptr{Cvoid}, y, w::AbstractVector, μ::AbstractVector, offset)
    yf = y isa Array{Float32} ? y : Array{Float32}(y)
    wf = w isa Vector{Float32} ? w : Vector{Float32}(w)
    μf = Vector{Float32}(μ)
    off_t = isnothing(offset) ? nothing : Matrix{Float32}(permutedims(reshape(Float32.(offset), size(offset, 1), :)))
    unit_w = all(==(1.0f0), wf)
    GC.@preserve yf wf μf off_t begin
        wptr = unit_w ? Ptr{Float32}(C_NULL) : pointer(wf)
        optr = isnothing(off_t) ? Ptr{Float32}(C_NULL) : pointer(off_t)
        check(ccall((:evt_set_target, LIB), Cint, (Ptr{Cvoid}, Ptr{Float32}, Ptr{Float32}, Ptr{Float32}, Ptr{Float32}),
            h, yf, wptr, μf, optr))
    end
    return nothing
end

# ---------------------------------------------------------------------------------------------------------------
# init_core(params, ::Type{<:GPU}, data, feature_names, y_train, w, offset)
#   reference: ext/EvoTreesKernelAbstractionsExt/init.jl:1-151 (CPU twin src/init.jl:148-262).
# Called by both `init` methods (matrix: src/init.jl:318-340, Tables: src/init.jl:264-297), i.e. by
# `fit(params; x_train, y_train, ...)` and `fit(params, dtrain; target_name, ...)` (src/fit.jl:302-345, :392-440).
function EvoTrees.init_core(params::EvoTypes, ::Type{<:HIPDevice}, data, feature_names, y_train, w, offset)
    rng = Xoshiro(params.seed)
    edges, featbins, feattypes = EvoTrees.get_edges(data; feature_names, nbins=params.nbins, rng)
    T = Float32
    L = EvoTrees._loss2type_dict[params.loss]
    K, y, μ, target_levels, target_isordered = EvoTrees._init_target(L, y_train, params, offset, T)
    μ = T.(μ)
    !isnothing(offset) && (μ .= 0)
    nobs = Tables.istable(data) ? length(Tables.getcolumn(data, 1)) : size(data, 1)
    nfeats = length(feature_names)
    @assert (size(y, ndims(y)) == length(w) && minimum(w) > 0)

    h = create_handle(nobs, nfeats, params.nbins, K, params.max_depth, L, params.tree_type)
    n_sampled_feats = max(1, ceil(Int, params.colsample * nfeats))
    cache = CacheHIP(h, rng, zeros(UInt8, nobs), zeros(UInt32, n_sampled_feats), nfeats, K)
    finalizer(destroy!, cache)

    upload_features!(h, data, feature_names, edges)
    monotone = zeros(Int32, nfeats)
    hasproperty(params, :monotone_constraints) && for (k, v) in params.monotone_constraints
        monotone[k] = v
    end
    ft = Vector{UInt8}(feattypes)
    GC.@preserve ft monotone check(ccall((:evt_set_feature_meta, LIB), Cint, (Ptr{Cvoid}, Ptr{UInt8}, Ptr{Int32}), h, ft, monotone))
    upload_levels!(h, params, L)
    upload_target!(h, y, w, μ, offset)
    # one tree per round: the next round's gradients are computed while the host stores the tree
    params.bagging_size == 1 && check(ccall((:evt_set_option, LIB), Cint, (Ptr{Cvoid}, Cstring, Int64), h, "grads_ahead", 1))

    info = Dict{Symbol,Any}(
        :nrounds => 0,
        :feature_names => feature_names,
        :target_levels => target_levels,
        :target_isordered => target_isordered,
        :edges => edges,
        :featbins => featbins,
        :feattypes => feattypes,
    )
    m = EvoTree{L,K}(L, K, [Tree{L,K}(μ)], info)
    return m, cache
end

# ---------------------------------------------------------------------------------------------------------------
# grow_evotree!(m, cache::CacheGPU, params)     reference: ext/EvoTreesKernelAbstractionsExt/fit.jl:1-21
# update_grads! (ext/.../loss.jl:183-191), subsample (ext/.../subsample.jl:2-8: the mask is drawn HERE, on the host
# stream, also when rowsample == 1, as src/fit.jl:13-16 does; threshold and compaction run on the device), the level
# loop of grow_tree! / grow_otree! (ext/.../fit.jl:132-342) with update_hist! / subtract_hist! / the split kernels /
# update_nodes_idx! (ext/.../fit-utils.jl), and predict! on the cache (ext/.../predict.jl:60-75) are all inside
# evt_update_grads + evt_grow_tree.
function EvoTrees.grow_evotree!(m::EvoTree{L,K}, cache::CacheHIP, params::EvoTypes) where {L,K}
    check(ccall((:evt_update_grads, LIB), Cint, (Ptr{Cvoid},), cache.h))
    p = Ref(EvtParams(params.eta, params.L2, params.lambda, params.gamma, params.min_weight, params.bagging_size, 1))
    cond = round(UInt8, 255 * params.rowsample)
    for _ in 1:params.bagging_size
        rand!(cache.rng, cache.mask)                                               # src/subsample.jl:7
        EvoTrees.sample!(cache.rng, UInt32(1):UInt32(cache.nfeats), cache.js, replace=false, ordered=true)   # src/fit.jl:16
        tree = Tree{L,K}(params.max_depth)
        feat, cond_bin, tw, gain, pred, split = tree.feat, tree.cond_bin, tree.w, tree.gain, tree.pred, tree.split
        mask, js = cache.mask, cache.js
        GC.@preserve feat cond_bin tw gain pred split mask js begin
            out = Ref(EvtTreeOut(pointer(feat), pointer(cond_bin), pointer(tw), pointer(gain), pointer(pred), Ptr{Bool}(pointer(split))))
            check(ccall((:evt_grow_tree, LIB), Cint,
                (Ptr{Cvoid}, Ptr{UInt8}, UInt8, Ptr{UInt32}, Cint, Ref{EvtParams}, Ref{EvtTreeOut}),
                cache.h, cond == 0xff ? Ptr{UInt8}(C_NULL) : pointer(mask), cond, js, length(js), p, out))
        end
        push!(m.trees, tree)            # predict!(cache.pred, tree, ...) was done by the library (update_pred = 1)
    end
    m.info[:nrounds] += 1
    return nothing
end

# ---------------------------------------------------------------------------------------------------------------
# The model as the ABI takes it: the trees' arrays concatenated (tree t owns [off[t], off[t+1]) ).
function flatten_trees(trees::AbstractVector{<:Tree})
    off = Int64[0; cumsum(length.(getfield.(trees, :feat)))]
    feat = reduce(vcat, getfield.(trees, :feat))
    cond_bin = reduce(vcat, getfield.(trees, :cond_bin))
    split = Vector{UInt8}(reduce(vcat, getfield.(trees, :split)))
    pred = reduce(hcat, getfield.(trees, :pred))          # K x total nodes
    return off, feat, cond_bin, split, pred
end

# _predict(m, data, ::Type{<:GPU}; ntree_limit)   reference: ext/EvoTreesKernelAbstractionsExt/predict.jl:115-135
# reached from `m(x; device=:gpu)` (src/structs.jl:135-138) and MMI.predict.  binarize + every tree + the link.
function EvoTrees._predict(m::EvoTree{L,K}, data, ::Type{<:HIPDevice}; ntree_limit=length(m.trees)) where {L,K}
    Tables.istable(data) ? data = Tables.columntable(data) : nothing
    ntrees = length(m.trees)
    ntree_limit > ntrees && error("ntree_limit is larger than number of trees $ntrees.")
    off, feat, cond_bin, split, pred = flatten_trees(view(m.trees, 1:ntree_limit))
    ft = Vector{UInt8}(m.info[:feattypes])
    edges = m.info[:edges]
    if data isa AbstractMatrix{Float64} && all(e -> e isa AbstractVector{Float64}, edges)
        x = data isa Matrix{Float64} ? data : Matrix{Float64}(data)
        nobs, nfeats = size(x)
        eflat = reduce(vcat, edges)
        eoff = Int32[0; cumsum(length.(edges))]
        out = Matrix{Float32}(undef, K, nobs)
        GC.@preserve x eflat eoff ft off feat cond_bin pred split out check(ccall((:evt_predict_f64, LIB), Cint,
            (Int64, Cint, Ptr{Float64}, Ptr{Float64}, Ptr{Int32}, Ptr{UInt8}, Cint, Cint, Cint, Ptr{Int64}, Ptr{Int64}, Ptr{UInt8},
                Ptr{Float32}, Ptr{UInt8}, Cint, Ptr{Float32}),
            nobs, nfeats, x, eflat, eoff, ft, loss_id(L), K, ntree_limit, off, feat, cond_bin, pred, split, 1, out))
    else
        x_bin = EvoTrees.binarize(data; feature_names=m.info[:feature_names], edges)
        nobs, nfeats = size(x_bin)
        out = Matrix{Float32}(undef, K, nobs)
        GC.@preserve x_bin ft off feat cond_bin pred split out check(ccall((:evt_predict, LIB), Cint,
            (Int64, Cint, Ptr{UInt8}, Ptr{UInt8}, Cint, Cint, Cint, Ptr{Int64}, Ptr{Int64}, Ptr{UInt8}, Ptr{Float32}, Ptr{UInt8}, Cint,
                Ptr{Float32}),
            nobs, nfeats, x_bin, ft, loss_id(L), K, ntree_limit, off, feat, cond_bin, pred, split, 1, out))
    end
    return K == 1 ? vec(Array(out')) : Array(out')
end

# _predict_leaf_indices(m, data, ::Type{<:GPU}; ntree_limit)   reference: ext/.../predict.jl:138-155 (+ :96-113)
function EvoTrees._predict_leaf_indices(m::EvoTree, data, ::Type{<:HIPDevice}; ntree_limit=length(m.trees))
    Tables.istable(data) ? data = Tables.columntable(data) : nothing
    ntrees = length(m.trees)
    ntree_limit > ntrees && error("ntree_limit is larger than number of trees $ntrees.")
    x_bin = EvoTrees.binarize(data; feature_names=m.info[:feature_names], edges=m.info[:edges])
    nobs, nfeats = size(x_bin)
    off, feat, cond_bin, split, _ = flatten_trees(view(m.trees, 1:ntree_limit))
    ft = Vector{UInt8}(m.info[:feattypes])
    leaves = Matrix{UInt32}(undef, nobs, ntree_limit)
    GC.@preserve x_bin ft off feat cond_bin split leaves check(ccall((:evt_predict_leaf_idx, LIB), Cint,
        (Int64, Cint, Ptr{UInt8}, Ptr{UInt8}, Cint, Ptr{Int64}, Ptr{Int64}, Ptr{UInt8}, Ptr{UInt8}, Ptr{UInt32}),
        nobs, nfeats, x_bin, ft, ntree_limit, off, feat, cond_bin, split, leaves))
    return Matrix{Int}(leaves)
end

# ---------------------------------------------------------------------------------------------------------------
# CallBack (src/callback.jl:21-128): a second handle holds the eval rows, their target, weights and running
# prediction; each round the new tree is added (predict!, ext/.../predict.jl:60-75) and the metric
# (src/metrics.jl, device twins ext/.../metrics.jl:7-24) is reduced on the device.
struct CallBackHIP
    feval::Function       # kept for `is_maximise(cb.feval)` in fit (src/fit.jl:323, :413)
    cache::CacheHIP
    metric::Cint
end

function eval_offset(::Type{L}, offset) where {L}
    isnothing(offset) && return nothing
    T = Float32
    off = T.(offset)
    L == EvoTrees.LogLoss && (off .= EvoTrees.logit.(off))
    L in [EvoTrees.Poisson, EvoTrees.Gamma, EvoTrees.Tweedie] && (off .= log.(off))
    L == EvoTrees.MLogLoss && (off .= log.(off))
    L in [EvoTrees.GaussianMLE, EvoTrees.LogisticMLE] && EvoTrees.unconstrain_mle_scale!(off)
    return off
end

function callback_core(params, m::EvoTree{L,K}, data, y_eval, w_eval, offset_eval) where {L,K}
    haskey(METRIC_ID, params.metric) || error("metric $(params.metric) is not supported by libevotrees_hip")
    nobs = Tables.istable(data) ? length(Tables.getcolumn(data, 1)) : size(data, 1)
    nfeats = length(m.info[:feature_names])
    h = create_handle(nobs, nfeats, params.nbins, K, 1, L, :binary)
    cache = CacheHIP(h, Xoshiro(0), UInt8[], UInt32[], nfeats, K)
    finalizer(destroy!, cache)
    upload_features!(h, data, m.info[:feature_names], m.info[:edges])
    ft = Vector{UInt8}(m.info[:feattypes])
    GC.@preserve ft check(ccall((:evt_set_feature_meta, LIB), Cint, (Ptr{Cvoid}, Ptr{UInt8}, Ptr{Int32}), h, ft, Ptr{Int32}(C_NULL)))
    y = L == EvoTrees.MLogLoss ? Float32.(EvoTrees.eval_levelcode(y_eval, m.info[:target_levels])) : Float32.(y_eval)
    w = isnothing(w_eval) ? ones(Float32, nobs) : Vector{Float32}(w_eval)
    upload_levels!(h, params, L)
    upload_target!(h, y, w, zeros(Float32, K), eval_offset(L, offset_eval))      # p = 0 (+ offset'), src/callback.jl:38,75
    return CallBackHIP(EvoTrees.metric_dict[params.metric], cache, METRIC_ID[params.metric])
end

# matrix form, src/callback.jl:82-121
function EvoTrees.CallBack(params::EvoTypes, m::EvoTree{L,K}, x_eval::AbstractMatrix, y_eval, ::Type{<:HIPDevice};
    w_eval=nothing, offset_eval=nothing) where {L,K}
    return callback_core(params, m, x_eval, y_eval, w_eval, offset_eval)
end

# Tables form, src/callback.jl:31-80
function EvoTrees.CallBack(params::EvoTypes, m::EvoTree{L,K}, deval, ::Type{<:HIPDevice};
    target_name, weight_name=nothing, offset_name=nothing) where {L,K}
    _target_names = target_name isa AbstractVector ? Symbol.(target_name) : [Symbol(target_name)]
    y_eval = length(_target_names) == 1 ?
             Tables.getcolumn(deval, _target_names[1]) :
             permutedims(reduce(hcat, [Tables.getcolumn(deval, t) for t in _target_names]))
    w_eval = isnothing(weight_name) ? nothing : Tables.getcolumn(deval, Symbol(weight_name))
    offset_eval = isnothing(offset_name) ? nothing : Tables.getcolumn(deval, Symbol(offset_name))
    return callback_core(params, m, deval, y_eval, w_eval, offset_eval)
end

function (cb::CallBackHIP)(logger, iter, tree)
    feat, cond_bin, pred, split = tree.feat, tree.cond_bin, tree.pred, tree.split
    GC.@preserve feat cond_bin pred split check(ccall((:evt_predict_tree, LIB), Cint,
        (Ptr{Cvoid}, Cint, Ptr{Int64}, Ptr{UInt8}, Ptr{Float32}, Ptr{Bool}),
        cb.cache.h, length(feat), feat, cond_bin, pred, split))
    v = Ref{Cdouble}(0.0)
    check(ccall((:evt_eval_metric, LIB), Cint, (Ptr{Cvoid}, Cint, Ptr{Cdouble}), cb.cache.h, cb.metric, v))
    EvoTrees.update_logger!(logger, iter, v[])
    return nothing
end

# ---------------------------------------------------------------------------------------------------------------
# Optional, for a host that overlaps its own work with the device (same trees, bit for bit):
#   evt_grow_tree_begin / evt_grow_tree_end        the call in two halves: draw the next mask in between
#   evt_stage_mask / evt_grow_tree_begin_staged    the next mask's upload on a stream of its own
#   evt_tree_open / evt_hist_build / evt_split_scan / evt_update_nodes_idx / evt_tree_close
#                                                  the reference's per-level device calls one at a time
#                                                  (update_hist!, the split search, update_nodes_idx!), with
#                                                  evt_get_hist / evt_get_nidx / evt_peek_tree readable in between
grow_tree_begin(cache::CacheHIP, mask, cond::UInt8, js::Vector{UInt32}, p::Ref{EvtParams}) =
    GC.@preserve mask js check(ccall((:evt_grow_tree_begin, LIB), Cint, (Ptr{Cvoid}, Ptr{UInt8}, UInt8, Ptr{UInt32}, Cint, Ref{EvtParams}),
        cache.h, isnothing(mask) ? Ptr{UInt8}(C_NULL) : pointer(mask), cond, js, length(js), p))
grow_tree_end(cache::CacheHIP, out::Ref{EvtTreeOut}) =
    check(ccall((:evt_grow_tree_end, LIB), Cint, (Ptr{Cvoid}, Ref{EvtTreeOut}), cache.h, out))
stage_mask(cache::CacheHIP, mask::Vector{UInt8}) =
    GC.@preserve mask check(ccall((:evt_stage_mask, LIB), Cint, (Ptr{Cvoid}, Ptr{UInt8}), cache.h, mask))
grow_tree_begin_staged(cache::CacheHIP, cond::UInt8, js::Vector{UInt32}, p::Ref{EvtParams}) =
    GC.@preserve js check(ccall((:evt_grow_tree_begin_staged, LIB), Cint, (Ptr{Cvoid}, UInt8, Ptr{UInt32}, Cint, Ref{EvtParams}),
        cache.h, cond, js, length(js), p))

end # module
