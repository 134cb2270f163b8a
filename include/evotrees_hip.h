/*
 * libevotrees_hip.so — C ABI of the MI355X (gfx950) tree-building backend.
 *
 * This is the drop-in boundary for the data-parallel hot path of EvoTrees.jl
 * (gradients -> histogram -> split search -> row partition -> predict).  Host code in
 * any language (Julia `ccall`, Python ctypes, C) owns the model (`EvoTree`, `Tree`) and the
 * random streams; the library owns one opaque training cache per handle, which replaces the
 * reference's device cache (ext/EvoTreesKernelAbstractionsExt/structs.jl:14-67).
 *
 * Conventions
 *  - Every function returns 0 on success and a negative evt_status on failure; the message
 *    is available from evt_last_error() (thread local).  No C++ exception crosses the ABI.
 *  - Host arrays are owned by the caller; the library copies in/out before it returns and
 *    never keeps a host pointer.  Input pointers may be host or device memory.
 *  - Matrices use the reference's Julia memory order: x_bin is nobs x nfeats column-major
 *    (x_bin[i + nobs*j]); pred is K x nobs and grad is (2K+1) x nobs with the first index
 *    fastest.
 *  - Feature ids and bins cross the boundary 1-based exactly as stored in Tree
 *    (src/structs.jl:77-84): feat 0 / cond_bin 0 mean "no split".
 *  - A handle is bound to the device that was current when it was created and to one HIP
 *    stream.  Calls on one handle must not overlap; different handles may be used from
 *    different threads.
 *  - The library installs no signal handlers and never calls back into the caller's runtime.
 *    The calls that take a whole matrix from host memory (evt_binarize_f64, evt_predict_f64,
 *    and evt_set_xbin / evt_predict from 64 MB up) copy it into pinned memory with up to six
 *    worker threads of their own, which only copy memory and are joined before the call
 *    returns; no other call starts a thread.
 */
#ifndef EVOTREES_HIP_H
#define EVOTREES_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct evt_ctx *evt_handle;

typedef enum {
    EVT_OK = 0,
    EVT_ERR_ARG = -1,   /* invalid argument (null pointer, range, unsupported size)        */
    EVT_ERR_HIP = -2,   /* a HIP runtime call or kernel launch failed                      */
    EVT_ERR_STATE = -3, /* call order violated (e.g. grow before x_bin / target were set)  */
    EVT_ERR_EMPTY = -4, /* "no subsample observation" (src/subsample.jl:36)                */
    EVT_ERR_NOMEM = -5,   /* a host or device allocation failed                             */
    EVT_ERR_INTERNAL = -6 /* any other failure inside the library (e.g. a worker thread could not start) */
} evt_status;

/* loss ids: the losses of src/loss.jl:20-34 */
enum {
    EVT_LOSS_MSE = 0,
    EVT_LOSS_LOGLOSS = 1,
    EVT_LOSS_GAUSSIAN_MLE = 2,
    EVT_LOSS_POISSON = 3,
    EVT_LOSS_GAMMA = 4,
    EVT_LOSS_TWEEDIE = 5,
    EVT_LOSS_MLOGLOSS = 6, /* K classes, y holds the 1-based class (level code) as a Float32 */
    EVT_LOSS_LOGISTIC_MLE = 7, /* the other two-parameter MLE loss (src/loss.jl:205-217): outputs and clamps as gaussian_mle */
    EVT_LOSS_MAE = 8,      /* rows [(y - p) w, 0, w] (src/loss.jl:78, :130-142); gain = shift of the children's mean residual
                              (src/split.jl:2, :68, :119-130); leaf = eta * sum(g) / (w + lambda w + L2) (src/predict.jl:250-258) */
    EVT_LOSS_CRED_VAR = 9, /* credibility losses: rows [d w, d^2 w, w], d = y - p (src/loss.jl:80-83, :173-185); gain terms */
    EVT_LOSS_CRED_STD = 10, /* Z |m1| / (1 + L2 / w), Z the ratio of variances / of standard deviations (src/loss.jl:275-290,
                              src/split.jl:3-4, :70-78, :132-141); leaf = eta * sum(g) / (w + L2) (src/predict.jl:211-217) */
    EVT_LOSS_QUANTILE = 11, /* one level alpha for every output; rows [(alpha or alpha - 1) w, y - p, w] (src/loss.jl:85-91,
                              :144-156); gains as mae; a leaf's value is eta * quantile(residuals of its rows, alpha) /
                              max(eps, 1 + lambda + L2 / w) (src/predict.jl:265-272) - computed on the device by sorting
                              (node, residual) pairs once the tree is complete.  Levels: evt_set_alphas */
    EVT_LOSS_MULTIQUANTILE = 12 /* K levels on ONE target (y has one column): output k follows alphas[k] (src/loss.jl:158-171,
                              src/predict.jl:275-281) */
};
/* evaluation metrics, metric_dict of src/metrics.jl:209-224 (in-scope subset) */
enum {
    EVT_METRIC_MSE = 0,
    EVT_METRIC_RMSE = 1,
    EVT_METRIC_MAE = 2,
    EVT_METRIC_LOGLOSS = 3,
    EVT_METRIC_GAUSSIAN_MLE = 4,
    EVT_METRIC_POISSON = 5,
    EVT_METRIC_GAMMA = 6,
    EVT_METRIC_TWEEDIE = 7,
    EVT_METRIC_MLOGLOSS = 8,
    EVT_METRIC_LOGISTIC_MLE = 9,
    EVT_METRIC_QUANTILE = 10,     /* pinball loss at the handle's alpha, averaged over the outputs (src/metrics.jl:4-6, :83-84) */
    EVT_METRIC_MULTIQUANTILE = 11 /* pinball loss of output k at alphas[k] against the one target (src/metrics.jl:117-134) */
};
/* params.tree_type, src/learners.jl:45 */
enum { EVT_TREE_BINARY = 0, EVT_TREE_OBLIVIOUS = 1 };

/* Per-tree hyper-parameters read by the kernels (fields of EvoTreeRegressor & co,
 * src/learners.jl:1-23). */
typedef struct {
    double eta;
    double L2;
    double lambda;
    double gamma;
    double min_weight;
    int32_t bagging_size;
    int32_t update_pred; /* 1: also apply predict!(cache.pred, tree, ...) as grow_evotree! does
                            (src/fit.jl:36-37); 0: only grow */
} evt_params;

/* Host arrays with the layout of Tree{L,K} (src/structs.jl:77-106), each of length
 * 2^max_depth - 1 (pred: K * that).  Zero-filled by the library before it writes. */
typedef struct {
    int64_t *feat;     /* Vector{Int}: 1-based feature id, 0 = none                        */
    uint8_t *cond_bin; /* Vector{UInt8}                                                    */
    float *w;          /* Vector{Float32}: sum of weights reaching the node                */
    float *gain;       /* Vector{Float32}                                                  */
    float *pred;       /* Matrix{Float32} K x nnodes                                       */
    uint8_t *split;    /* Vector{Bool}                                                     */
} evt_tree_out;

/* Message of the last failure on the calling thread ("" if none). */
const char *evt_last_error(void);

/* Number of visible HIP devices; fails (EVT_ERR_HIP) when the runtime finds none. */
int evt_device_count(int32_t *count);

/* ---- training cache ------------------------------------------------------------------
 * Replaces init_core(params, ::Type{<:GPU}, ...) device allocation
 * (ext/EvoTreesKernelAbstractionsExt/init.jl:1-151): sizes every device buffer.
 * nbins in [2,255] (src/learners.jl:527); nfeats in [1,65534] (a record of the observation-major copy may be any width;
 * the one shape without a wide-record histogram kernel - more than 1024 features with accumulator channels x nbins above
 * 512 - is refused when its first tree is grown); max_depth in [1,16] (the histogram buffer holds 2^max_depth - 1 node
 * slices).  The reference bounds neither (src/learners.jl:525-527).  K is the number of outputs (size(pred, 1) in the reference, at most 16):
 * the number of targets for mse / logloss / poisson / gamma / tweedie / mae / quantile / cred_var / cred_std (1, or more with
 * a matrix target, src/init.jl:11-16, :104-150), twice the number of targets for gaussian_mle and logistic_mle
 * (src/init.jl:68-100), the number of classes (2..16) for mlogloss, the number of levels for multiquantile (src/init.jl:101-103). */
int evt_create(int64_t nobs, int32_t nfeats, int32_t nbins, int32_t K, int32_t max_depth, int32_t loss,
               int32_t tree_type, evt_handle *out);
/* Frees all device memory; the slot post_fit_gc has in the reference (src/fit.jl:340). */
int evt_destroy(evt_handle h);

/* Upload of the binned matrix: `_to_device(x_bin)` in ext/.../init.jl:4-6.  Values must be in
 * 1..nbins (src/fit-utils.jl:66-72); anything else is rejected.  Also derives the
 * observation-major copy the histogram kernel streams (the CPU path's x_bin_T, src/init.jl:155). */
int evt_set_xbin(evt_handle h, const uint8_t *x_bin_colmajor);

/* Device binarize: searchsortedfirst(edges[j], x[i,j]) for every cell (src/fit-utils.jl:66-72),
 * written straight into the cache's x_bin.  x is nobs x nfeats column-major Float64; edges are
 * concatenated per feature, edge_off has nfeats+1 entries.  A matrix in host memory goes up in
 * 32 MB pieces through pinned buffers, each binned behind its copy (8 bytes per value over the bus:
 * 0.16 s for 10M x 100 where a plain copy from pageable memory takes 0.30 s). */
int evt_binarize_f64(evt_handle h, const double *x_colmajor, const double *edges, const int32_t *edge_off);

/* Target, weights and initial prediction: y Float32[nobs] (for mlogloss the 1-based level code of each row,
 * as _init_target builds it, src/init.jl:43-67) or, with T > 1 targets, the reference's T x nobs column-major matrix
 * (the T values of a row side by side; _target(y, k, i), src/loss.jl:49-50); w Float32[nobs] or NULL for ones
 * (device_ones, src/init.jl:300); pred[:, i] = mu (+ offset[:, i] if offset != NULL), offset is
 * K x nobs (src/init.jl:168-174).  Writes the weight row of the gradient matrix. */
int evt_set_target(evt_handle h, const float *y, const float *w, const float *mu, const float *offset);

/* feattypes[j] != 0: numeric (<=), 0: categorical (==); monotone[j] in {-1,0,1}
 * (cache.feattypes / cache.monotone_constraints, src/init.jl:183-187).  NULL = all numeric / none.
 * A constraint is refused (EVT_ERR_ARG) for mlogloss, the quantile losses and for more than one target: the reference
 * has no pred_scalar for the former two, and for the latter its pred_scalar (src/predict.jl:205-208, :235-238) reads the
 * statistics at the one-target positions. */
int evt_set_feature_meta(evt_handle h, const uint8_t *feattypes, const int32_t *monotone);

/* Levels of the quantile losses and metrics: params.alpha (n = 1: the quantile loss, every output) or params.alphas
 * (n = K: the multiquantile loss, one output each; strictly increasing, src/learners.jl:504-515), each in [0, 1]
 * (src/learners.jl:539).  A handle starts with alpha = 0.5, the reference's default (src/learners.jl:44).  The gradients
 * use the Float64 values (src/loss.jl:85-91), the metrics T(alpha) (src/callback.jl:62-66). */
int evt_set_alphas(evt_handle h, const double *alphas, int32_t n);

/* update_grads!(cache.∇, cache.pred, cache.y, L, params): src/loss.jl:100-111, :219-236;
 * device twin ext/.../loss.jl:183-191. */
int evt_update_grads(evt_handle h);

/* Overwrites the gradient matrix ((2K+1) x nobs Float32, weight row included) — used to feed
 * identical gradients to the library and to a CPU run.  The weight row must agree with evt_set_target:
 * all ones when that call got w == NULL (the row count then stands for the weight everywhere). */
int evt_set_grads(evt_handle h, const float *grad);

/*
 * One tree: subsample (src/subsample.jl:6-38 / ext/.../subsample.jl:2-8) + grow_tree! or
 * grow_otree! (src/fit.jl:45-263; device twin ext/.../fit.jl:132-342) + optionally predict!
 * on the cache (src/fit.jl:37).
 *  mask : UInt8[nobs] drawn by the host RNG, rows with mask[i] <= cond are kept; NULL keeps all.
 *  js   : sampled feature ids, 1-based, ascending, n_js of them (src/fit.jl:16).
 * Returns EVT_ERR_EMPTY when no row is kept.
 * When every row is kept and params->update_pred is set, the tree's leaf values may still be pending on
 * return: the library has recorded each row's leaf and adds the values in the next pass over the rows
 * (evt_update_grads does it on the way; evt_get_pred, evt_eval_metric, evt_predict_tree and the next
 * evt_grow_tree apply them first).  Every call sees the same predictions, bit for bit, as if predict! had
 * run inside this call.
 */
int evt_grow_tree(evt_handle h, const uint8_t *mask, uint8_t cond, const uint32_t *js, int32_t n_js,
                  const evt_params *params, evt_tree_out *tree);
/* The same call in two halves, for a host that overlaps its own work of the next round (drawing the next row
 * mask, src/subsample.jl:7; the reference's host does this between kernels of the device path,
 * ext/.../subsample.jl:2-8) with the device growing this round's tree.  begin reads mask and js before it
 * returns and queues all device work; end waits for it and fills the tree arrays (EVT_ERR_EMPTY when no row was
 * kept).  evt_grow_tree is begin followed by end.
 * TWO trees may be in flight: the next tree's begin (either form), the evt_update_grads and evt_draw_mask that go with
 * it and evt_set_profiling only queue work behind what is already queued, so they may be called while ONE tree waits
 * to be collected; end then collects the older tree.  A host whose next round does not depend on this round's tree
 * arrays (src/fit.jl:6-42 reads nothing back) thereby keeps the device busy while it collects a tree and prepares
 * the next call.  With two trees in flight only evt_grow_tree_end, evt_synchronize and evt_destroy are accepted; every
 * call not named here returns EVT_ERR_STATE while any tree is in flight.  The results are, bit for bit, those of
 * begin / end strictly in turn. */
int evt_grow_tree_begin(evt_handle h, const uint8_t *mask, uint8_t cond, const uint32_t *js, int32_t n_js,
                        const evt_params *params);
int evt_grow_tree_end(evt_handle h, evt_tree_out *tree);
/* The upload of the next tree's mask (nobs bytes over PCIe, src/subsample.jl:7-9 / ext/.../subsample.jl:2-8) taken off
 * the critical path: evt_stage_mask may be called while a tree begun with evt_grow_tree_begin is in flight; it copies
 * the mask on a stream of its own into a second device buffer and returns when the copy is done (the caller's buffer
 * is free again; the tree in flight keeps running; with TWO trees in flight it returns EVT_ERR_STATE, since the older
 * tree may still read the buffer the copy goes to).  evt_grow_tree_begin_staged is evt_grow_tree_begin with the mask
 * staged last; EVT_ERR_STATE when none has been staged since the last tree.  Same trees, bit for bit. */
int evt_stage_mask(evt_handle h, const uint8_t *mask);
int evt_grow_tree_begin_staged(evt_handle h, uint8_t cond, const uint32_t *js, int32_t n_js,
                               const evt_params *params);
/* The staged mask drawn by the device instead of uploaded, for a caller that does not need the byte stream of its own
 * generator (rand!(rng, mask), src/subsample.jl:7) but only a reproducible one: the caller draws ONE 64-bit seed per
 * tree from its generator and the mask's 8-byte word w becomes output w of SplitMix64 started at that seed
 * (z = seed + (w + 1) * 0x9E3779B97F4A7C15; z = (z ^ z >> 30) * 0xBF58476D1CE4E5B9; z = (z ^ z >> 27) *
 * 0x94D049BB133111EB; z ^= z >> 31), little end first: byte i of the mask is bits 8 * (i % 8) and up of word i / 8.
 * A row is kept when its byte <= cond, as with an uploaded mask, so P[keep] = (cond + 1) / 256 all the same.  The call
 * only takes note of the seed (it may come while a tree is in flight); the evt_grow_tree_begin_staged that follows draws
 * the bytes in its subsampling pass, on the device, with no host work per row.  A later evt_stage_mask replaces the seed.
 * The trees equal, bit for bit, those grown from the same bytes uploaded. */
int evt_draw_mask(evt_handle h, uint64_t seed);

/*
 * The same tree, one kernel stage at a time: the stages are the reference's own per-level calls, so each can be
 * checked (or timed) against its counterpart on its own.
 *   evt_tree_open        subsample + root set-up, as evt_grow_tree_begin up to the first level (src/fit.jl:59-66)
 *   evt_hist_build       update_hist! for the level's build nodes, i.e. the smaller child of every pair
 *                        (src/fit-utils.jl:345-394; device twin ext/.../fit-utils.jl:148-226)
 *   evt_split_scan       subtract_hist! for the larger children, then _scan_node!/get_best_split (update_gains! and
 *                        the level's common choice for oblivious trees), _child_sums! and the leaf values of the
 *                        nodes that end here (src/fit-utils.jl:321-332, :403-486; src/fit.jl:85-121, :190-217;
 *                        src/predict.jl:198-234)
 *   evt_update_nodes_idx split_set! / update_nodes_idx!: rows of split nodes move to the children, stably
 *                        (src/fit-utils.jl:93-132; ext/.../fit-utils.jl:9-31)
 *   evt_tree_close       the rest of evt_grow_tree_begin (predict! on rows outside the sample, the tree's way back);
 *                        evt_grow_tree_end then collects the tree
 * Levels run 1 .. max(1, max_depth - 1), each as hist_build, split_scan, update_nodes_idx in this order with the level
 * passed along; a call out of order returns EVT_ERR_STATE and says which call the tree expects.  Between the
 * stages evt_get_hist, evt_get_nidx (the node every sampled row has reached so far, read off the row lists the
 * partition wrote), evt_peek_tree and evt_synchronize are allowed; every other call returns EVT_ERR_STATE
 * until evt_tree_close.  A stage that fails closes the tree.  The stages queue exactly the kernels evt_grow_tree_begin
 * queues: the finished tree is the same, bit for bit.
 */
int evt_tree_open(evt_handle h, const uint8_t *mask, uint8_t cond, const uint32_t *js, int32_t n_js,
                  const evt_params *params);
int evt_hist_build(evt_handle h, int32_t level);
int evt_split_scan(evt_handle h, int32_t level);
int evt_update_nodes_idx(evt_handle h, int32_t level);
int evt_tree_close(evt_handle h);
/* The tree arrays as they stand on the device (nodes of levels not yet searched are zero). */
int evt_peek_tree(evt_handle h, evt_tree_out *tree);

/* predict!(cache.pred, tree, cache.x_bin, feattypes): src/predict.jl:1-46; ext/.../predict.jl:60-75.
 * Adds one host tree (arrays of length nnodes_tree) to the cache's prediction. */
int evt_predict_tree(evt_handle h, int32_t nnodes_tree, const int64_t *feat, const uint8_t *cond_bin,
                     const float *pred, const uint8_t *split);

/* The eval CallBack's metric (src/callback.jl:130-135 -> src/metrics.jl:30-48, :100-116) on the
 * handle's own state: sum_i(Float32(w[i] * sum_k value(pred[k, i], y[k, i]) / K)) / sum_i(w[i]), both sums in
 * Float64; rmse = sqrt(mse).  A handle created on the eval rows (evt_create + evt_set_xbin /
 * evt_binarize_f64 + evt_set_target with the eval y, w, offset and mu = 0) plays the CallBack: each
 * new tree is added with evt_predict_tree, then this call returns the metric.  The sum order is
 * fixed, so the result is bit-reproducible. */
int evt_eval_metric(evt_handle h, int32_t metric, double *value_out);

/* ---- read-back of cache state (parity tests, callbacks) ------------------------------ */
/* The cache's binned matrix (nobs x nfeats column-major), e.g. after evt_binarize_f64. */
int evt_get_xbin(evt_handle h, uint8_t *x_bin_out);
int evt_get_pred(evt_handle h, float *pred_out /* K x nobs */);
int evt_get_grads(evt_handle h, float *grad_out /* (2K+1) x nobs */);
/* Node each sampled row ended in for the last tree (update_nodes_idx!, ext/.../fit-utils.jl:9-31),
 * 1-based node id; 0 for rows outside the sample. */
int evt_get_nidx(evt_handle h, uint32_t *nidx_out /* nobs */);
/* Histogram of the last tree in the reference layout h∇[k, bin, feat, node] Float64
 * ((2K+1) x nbins x nfeats x (2^max_depth-1), src/init.jl:204); only slices of nodes that were
 * scanned (or, inside a tree grown in stages, built from rows at the current level) and features in js are
 * defined, the rest is zero.  The second gradient row has no accumulator for one-output mse, mae and quantile: it is
 * exported as derived (mse: twice the weight), as zero (mae, where the row is zero) or as zero in place of the sum of
 * residuals (quantile: the reference accumulates it and reads it nowhere). */
int evt_get_hist(evt_handle h, double *hist_out);
/* Fixed-point parameters of the last update: gradient row k is accumulated as
 * rint(v * 2^(qbits[k]-qexp[k])) in int64. */
int evt_get_quant(evt_handle h, int32_t *qbits /* 2K+1 */, int32_t *qexp /* 2K+1 */);

/* ---- inference: _predict(m, data, ::Type{<:GPU}) (ext/.../predict.jl:115-135) ----------
 * x_bin: nobs x nfeats column-major; trees concatenated: tree t owns entries
 * [tree_off[t], tree_off[t+1]) of feat / cond_bin / split and K times that of pred.
 * out: K x nobs raw sums, link applied when apply_link != 0 (src/predict.jl:105-116).
 * The transposition to nobs x K (src/predict.jl:134) is left to the host.
 * x_bin and out may be host or device pointers (device memory is used in place); feattypes and the tree arrays are host
 * arrays.  Models whose trees are full heaps (2^depth - 1 entries, as the reference stores them) of depth
 * <= 13 and fewer than 1024 features are walked from LDS (any K up to 16); others from global memory, with
 * identical results. */
int evt_predict(int64_t nobs, int32_t nfeats, const uint8_t *x_bin_colmajor, const uint8_t *feattypes,
                int32_t loss, int32_t K, int32_t ntrees, const int64_t *tree_off, const int64_t *feat,
                const uint8_t *cond_bin, const float *pred, const uint8_t *split, int32_t apply_link,
                float *out);
/* The same from raw features: binarize(data; edges) (src/fit-utils.jl:66-72, searchsortedfirst per
 * column) on the device, in row chunks, followed by the traversal above — the whole of
 * _predict(m, data, ::Type{<:GPU}).  x is nobs x nfeats column-major Float64; edges / edge_off as in
 * evt_binarize_f64 (at most 254 edges per feature). */
int evt_predict_f64(int64_t nobs, int32_t nfeats, const double *x_colmajor, const double *edges,
                    const int32_t *edge_off, const uint8_t *feattypes, int32_t loss, int32_t K, int32_t ntrees,
                    const int64_t *tree_off, const int64_t *feat, const uint8_t *cond_bin, const float *pred,
                    const uint8_t *split, int32_t apply_link, float *out);
/* predict_leaf_idx (src/predict.jl:138-185): out is nobs x ntrees column-major UInt32. */
int evt_predict_leaf_idx(int64_t nobs, int32_t nfeats, const uint8_t *x_bin_colmajor, const uint8_t *feattypes,
                         int32_t ntrees, const int64_t *tree_off, const int64_t *feat, const uint8_t *cond_bin,
                         const uint8_t *split, uint32_t *out);

/* No counterpart in the reference: evt_predict for callers that cannot allocate - code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  Every pointer is device memory: x_bin (nobs x nfeats column-major),
 * the model in the reference's arrays, concatenated as for evt_predict (tree_off has ntrees + 1 entries and ends at
 * total_nodes), feattypes (or NULL: all numeric), out (K x nobs).  Three kernels are queued on `stream` (a hipStream_t;
 * NULL = the default stream) and the call returns without waiting: it allocates nothing, copies nothing and
 * synchronises nothing.  The packed node words evt_predict allocates per call live in a file-scope device array of
 * EVT_STATIC_MAX_NODES words (4 MiB + a 256-byte header, held by each GPU the call has run on until the process ends);
 * a model with more nodes is refused with EVT_ERR_ARG.  The model is checked on the device by the rules evt_predict
 * applies on the host; a model that breaks them leaves `out` unwritten and EVT_ERR_ARG in *status (a device int32,
 * EVT_OK otherwise; may be NULL).  Results equal evt_predict's, bit for bit.  The device that is current on the calling
 * thread must be the one the pointers live on.  All calls on one GPU share the one array: calls that overlap on a GPU
 * (two streams, two threads) race, and a call must have finished before the next one is queued on another stream.
 * The first call on a device looks the array's address up (hipGetSymbolAddress, which may load the code object) and sets
 * kernel attributes: make it an ordinary call, outside any stream capture.  Every call queries the memory type of its
 * nine pointers unless EVT_STATIC_TRUSTED is added to apply_link (0 or 1): a caller that vouches for device pointers -
 * a serving loop, a call recorded into a HIP graph - skips the queries.  A captured call replays the three kernels on
 * the same array: the rule about overlapping calls holds for replays too. */
#define EVT_STATIC_MAX_NODES (1 << 20)
#define EVT_STATIC_TRUSTED 2
int evt_predict_static(void *stream, int64_t nobs, int32_t nfeats, const uint8_t *x_bin_dev, const uint8_t *feattypes_dev,
                       int32_t loss, int32_t K, int32_t ntrees, int64_t total_nodes, const int64_t *tree_off_dev,
                       const int64_t *feat_dev, const uint8_t *cond_bin_dev, const float *pred_dev, const uint8_t *split_dev,
                       int32_t apply_link, float *out_dev, int32_t *status_dev);

/* ---- measurement ---------------------------------------------------------------------
 * Kernel classes timed with HIP events on the handle's stream when profiling is on. */
enum {
    EVT_K_GRAD = 0,
    EVT_K_HIST = 1,
    EVT_K_SCAN = 2,
    EVT_K_PARTITION = 3,
    EVT_K_PREDICT = 4,
    EVT_K_OTHER = 5,
    EVT_K_COUNT = 6
};
/* on = 0: off; 1: every class; any other value: bit mask (1 << EVT_K_*) of the classes to time. */
int evt_set_profiling(evt_handle h, int32_t on);
/* Accumulated since the last reset: per class number of launches, milliseconds, and units
 * (GRAD/PREDICT: rows; HIST: rows built; SCAN: nodes scanned; PARTITION: rows moved). */
int evt_get_profile(evt_handle h, int64_t *launches, double *ms, int64_t *units);
int evt_reset_profile(evt_handle h);
/* Options: "hist_blocks", "hist_threads", "hist_min_rows", "hist_seg_cost", "hist_variant" (launch shape,
 * work split and kernel variant of the histogram builder, for sweeps; results do not depend on them);
 * "bit_planes" (1, default: before the first tree the library derives one bit plane per
 * (feature, bin threshold) from x_bin - F * (nbins - 1) * nobs / 8 bytes, taken only when that is at most 16 GiB and a third of the free
 * memory - and the row partition reads its decisions there; 0: it gathers bin bytes; same trees, bit for bit);
 * "record_nidx" (1: the partition also records every sampled row's final node while the tree grows;
 * 0, default: evt_get_nidx derives it afterwards by walking the finished tree); "defer_pred" (1, default:
 * leaf values of a tree grown on every row are added in row order by the next pass over the rows;
 * 0: they are added while the tree's last level is partitioned; results do not depend on it); "grads_ahead"
 * (1: a tree grown with update_pred queues the next evt_update_grads behind itself, so the device computes it
 * while the host collects the tree, and that next call returns at once; meant for bagging_size 1 - with more
 * trees per round only the last one's work is used; 0, default; results do not depend on it); "scan_fused"
 * (1, default: with at most 16 sampled features one kernel searches and finishes a node's split, 0: two kernels)
 * and "hist_in_scatter" (1, default: with at most 16 features and a quarter of a million rows the levels below
 * the root get their histograms from the partition's scatter pass, one kernel less per level; 0: a histogram
 * kernel per level) - same trees and histograms, bit for bit, either way. */
int evt_set_option(evt_handle h, const char *name, int64_t value);
/* Blocks until all work queued on the handle's stream is done. */
int evt_synchronize(evt_handle h);
/* Plain device copy of nbytes (read + write) timed with HIP events: the box's streaming
 * ceiling that roofline figures are quoted beside. */
int evt_copy_bandwidth(int64_t nbytes, int32_t iters, double *gbps_out);
/* Same for a read-only stream of nbytes (no write traffic). */
int evt_read_bandwidth(int64_t nbytes, int32_t iters, double *gbps_out);
/* Rate of 64-bit LDS atomics as the histogram kernel issues them (256 blocks of 1024 threads, one 64 KB LDS array each):
 * pattern 0 = the kernel's layout for 128-byte records (the 16 lanes the LDS serves per pass fall on 16 different bank
 * pairs, random bins), pattern 1 = random words; lanes16 of every 16 lanes issue (the 100-feature record of the headline
 * workload uses 13).  Outputs: lane-atomics per second and wavefront instructions per second, device wide.  No
 * counterpart in the reference (its histogram kernel adds into global memory, ext/.../fit-utils.jl:57-174): the ceiling
 * the kernel's row rate is quoted beside. */
int evt_lds_atomic_rate(int32_t pattern, int32_t lanes16, int32_t iters, double *lane_atomics_per_s, double *wave_instr_per_s);
/* Rate of 64-bit global atomics as the histogram kernel's flush issues them: `blocks` blocks each add `words` consecutive
 * words of one slice `reps` times.  Output: atomics per second, device wide. */
int evt_global_atomic_rate(int32_t words, int32_t blocks, int32_t reps, double *atomics_per_s);

#ifdef __cplusplus
}
#endif
#endif /* EVOTREES_HIP_H */
