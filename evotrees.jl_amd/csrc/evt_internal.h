// Internal declarations shared by the HIP translation units of libevotrees_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include <exception>
#include <new>
#include <string>
#include <vector>

#include "../../include/evotrees_hip.h"

// ---- node status on device ------------------------------------------------------------
#define ST_INACTIVE 0
#define ST_BUILD 1    // active at its level, histogram built from rows
#define ST_SUBTRACT 2 // active at its level, histogram = parent - sibling
#define ST_SPLIT 3    // scanned, split found
#define ST_LEAF 4     // scanned (or last level), leaf

#define EVT_CHUNK 2048        // rows per partition chunk (8 per thread of a 256-thread block)
#define EVT_CHUNK_WORDS 32    // 64-bit ballot words per chunk
#define EVT_MAX_NK 5  // gradient rows of the one- and two-output losses (register arrays of the specialised kernels)
#define EVT_MAX_NA 5
#define EVT_MAX_K 16     // classes of the multi-class loss
// the running maxima of the gradient rows are kept in EVT_ABSMAX_STRIPES copies, one 160-byte stripe each, and a block
// raises the copy of stripe blockIdx % EVT_ABSMAX_STRIPES: same-address atomics queue up one behind the other
#define EVT_ABSMAX_STRIPES 32
#define EVT_MC_MAX_NK 40 // >= 2 * EVT_MAX_K + 1: sizes of the per-row quantisation tables and of the generic kernels' arrays
#define EVT_HIST_GROUP 4 // accumulator channels one histogram launch handles; more channels take several launches
#define EVT_METRIC_BLOCKS 1024 // partial sums of the evaluation metric
#define EVT_MAX_DEPTH 16
#define EVT_MAX_FEATS 65534 // a feature's slot in the column sample is a 16-bit word, 0xFFFF = not sampled
#define EVT_PACK_QBITS 30     // fixed-point bits of the gradient channel that shares a word with the row count
#define EVT_PACK_CNT_BITS 16
// rows one LDS histogram may take between two flushes: the packed row counter has EVT_PACK_CNT_BITS bits, and
// 65535 * 2^EVT_PACK_QBITS < 2^46 leaves the gradient sum inside its 48 signed bits
#define EVT_HIST_MAX_ROWS_PER_BLOCK 65535

// Level table header slots (int64 each)
#define LH_N_ACT 0
#define LH_N_CHUNKS 1
#define LH_N_BUILD 2
#define LH_TOTAL_BUILD 3 // build rows of the level + hist_seg_cost per build node
#define LH_SIZE 8

struct LevelTab {
    int64_t *hdr;      // [LH_SIZE]
    int32_t *act_node; // active nodes in node (= position) order
    int64_t *cprefix;  // exclusive prefix of chunk counts over active nodes, n_act+1 entries
    int32_t *bnode;    // build nodes
    int64_t *bstart;   // their segment starts
    int64_t *bprefix;  // exclusive prefix of their lengths, n_build+1 entries
    uint4 *cdesc;      // per chunk of the level: {node, first position, end of the node's segment, first chunk of the node}
};

struct TreeDev {
    int32_t *feat;    // 1-based, 0 none
    uint8_t *cond_bin;
    float *w;
    float *gain;
    float *pred;      // K x nnodes
    uint8_t *split;
    uint32_t *packed; // feat | cond_bin << 16 | split << 24, for traversal
};

struct ProfRec {
    int cls;
    int level;
    int64_t seq; // tree the launch belongs to (evt_ctx::tree_seq when it was queued)
    hipEvent_t e0, e1;
};

struct evt_ctx {
    int device;
    hipStream_t stream;
    int64_t N;
    int32_t F, B, K, NK, D, loss, tree_type;
    int32_t T;         // target columns of y: K for the gradient-regression losses, K / 2 for gaussian_mle, 1 for mlogloss (the class) and multiquantile
    bool mc;           // more outputs than the specialised kernels take: run-time channel count (multi-class, several targets)
    int32_t nnodes;    // 2^D - 1
    int32_t maxlvl;    // 2^(D-1)
    int32_t RS;        // bytes per observation-major record
    int32_t LPR;       // 16-byte lanes per record
    // A record is made of pieces of PBL bytes (the unit one lane of the conflict-free histogram kernel loads) of which the
    // first PU hold features: feature f sits at byte (f / PU) * PBL + f % PU, the other bytes are padding (bin 1).  PU < PBL
    // spreads the features evenly over all the lanes a row has, so that a row costs PU LDS atomic instructions where
    // a densely packed record costs PBL of them with its last lanes idle.  PBL == PU == 1: densely packed (byte f = feature f).
    int32_t PBL, PU;
    bool unit_w;       // weights are all one (w == NULL at set_target)
    int32_t NA;        // LDS accumulator channels per bin
    int32_t NAg;       // global histogram channels per bin
    int32_t chan_k[EVT_MC_MAX_NK]; // gradient row of accumulator channel a
    bool have_xbin, have_target, have_grads;

    // data
    uint8_t *xcm;   // F x N bytes (column-major N x F)
    uint8_t *xrm;   // N records of RS bytes
    // Threshold bit planes: plane (f, b), b = 1..B-1, holds one bit per row, x_bin[row, f] <= b, 32 rows per word.
    // The partition's decision for a numeric split is one bit of one plane; a node's rows, ascending and 2^depth apart,
    // find theirs 8 times closer together than their bin bytes (1024 rows per 128-byte line instead of 128).
    // Built before the first tree when F * (B - 1) * N / 8 bytes fit the budget (HBM capacity traded for bandwidth).
    uint32_t *planes;
    int64_t plane_words; // words per plane: ceil(N / 32), rounded up to a multiple of 32
    bool planes_ready;   // the planes hold the current x_bin
    int use_planes;      // option "bit_planes": 0 never, 1 when they fit the budget (default)
    float *y;
    float *pred;    // K x N
    float *grad;    // NK x N
    unsigned long long *gq; // NA planes of N packed fixed-point words
    uint32_t *is_a, *is_b;
    uint32_t *is_id;   // [N] 0..N-1, written once: the root's row list when every row is in the tree
    uint32_t *nidx;
    uint8_t *mask;
    // the next tree's row mask, uploaded on a stream of its own while the current tree grows (evt_stage_mask)
    uint8_t *mask_next;
    hipStream_t copy_stream;
    bool mask_next_valid;
    bool mask_seed_valid;   // the next staged tree draws its mask on the device from mask_seed (evt_draw_mask) instead of using mask_next
    unsigned long long mask_seed;
    unsigned long long *flagw;
    int32_t *chunk_nleft;
    int64_t *chunk_lpre;
    int64_t max_chunks;
    long long *hist; // [node][jp][ag][bin]
    int64_t *seg_start, *seg_len;
    int32_t *status;
    long long *node_sum; // [node][NAg]
    TreeDev tree;
    uint8_t *tree_blob; // one allocation behind tree.{feat,w,gain,pred,cond_bin,split} and stats
    size_t blob_feat, blob_w, blob_gain, blob_pred, blob_stats, blob_bin, blob_split, blob_bytes;
    LevelTab lvl[2];
    uint32_t *js;      // [F]
    uint16_t *jsmap;   // [RS] slot of the feature at byte p of a record, 0xFFFF = not sampled / padding
    uint8_t *feattypes;
    int32_t *mono;
    uint32_t *absmax;  // [2][EVT_ABSMAX_STRIPES][EVT_MC_MAX_NK] float bits: two sets, raised by alternate gradient passes
    int absmax_cur;    // the set the next gradient pass raises
    // quantile losses: levels (Float64 for the gradients, Float32 for the metrics) and the sort buffers of the leaf pass
    double h_alphas[EVT_MAX_K];
    int32_t n_alphas;
    double *alphas;        // [EVT_MAX_K]
    float *alphas_f;       // [EVT_MAX_K]
    unsigned long long *qkeys_a, *qkeys_b; // [N] (node, residual) keys, unsorted / sorted
    void *qtemp;
    size_t qtemp_bytes;
    int32_t *qexp;     // [EVT_MC_MAX_NK]; points into qexp_buf: the tables of the gradients quantised last
    int32_t *qbits;    // [EVT_MC_MAX_NK]
    double *qscale;    // [2 * EVT_MC_MAX_NK]: decode scale per global channel, then encode multiplier per gradient row
    // The fixed-point tables exist twice: a gradient update writes the set the last grown tree does NOT use, so that the
    // tree's histogram can still be decoded (evt_get_hist, evt_get_quant) after the next round's gradients were
    // quantised behind it.  q_cur: set of the gradients quantised last; q_tree: set the last tree was grown on.
    int32_t *qexp_buf[2];
    double *qscale_buf[2];
    int q_cur, q_tree;
    double *metric_partial; // [2 * EVT_METRIC_BLOCKS + 1] evaluation-metric partial sums, result last
    int64_t *stats;    // [D+1] rows built per level
    int32_t *errflag;  // device-side validation flag
    double *ogains;    // oblivious: [maxlvl][F][B]
    void *sbest;       // split search: best candidate per (node of the level, feature group), 64 B each

    // host staging (pinned): two slots of h_stage_bytes each, so that a second tree can be queued before the first one
    // has been collected.  h_stage / h_stage_dev point at the slot of the tree queued last.
    uint8_t *h_stage;
    uint8_t *h_stage_base, *h_stage_dev_base;
    // evt_predict_tree: device copies of the tree handed in (packed nodes, leaf values) and the pinned buffer they are
    // uploaded through; kept between calls and grown on demand
    uint32_t *pt_nodes;
    float *pt_pred;
    uint8_t *pt_stage, *pt_stage_dev;
    size_t pt_cap; // nodes
    bool pt_busy;  // an upload from pt_stage has been queued since the stream was last drained here
    uint8_t *h_stage_dev; // the same pinned buffer as the device addresses it: the finished tree is written there by a kernel
    size_t h_stage_bytes;
    int32_t h_qbits[EVT_MC_MAX_NK];
    int32_t n_js_last;
    bool js_staged; // the column sample sits in the pinned staging slot and has not reached the device copies yet (k_tree_begin takes it along)
    std::vector<uint32_t> js_last;
    std::vector<uint8_t> h_feattypes; // host copy: trees handed in from outside are packed with it
    bool last_all_rows;

    // tunables
    int hist_blocks, hist_threads, hist_min_rows, hist_seg_cost;
    int hist_variant;  // 0 auto, 1 generic 16-byte-piece kernel, 2 conflict-free 8-byte-piece kernel where it applies
    int scan_fused;    // option: the split search of a node with at most 16 sampled features runs in one kernel
    int hist_in_scatter; // option: with 16-byte records and few chunks the partition's scatter pass builds the next level's histograms
    bool record_nidx;  // leaf finalisation also writes the node id of every sampled row
    bool nidx_valid;   // nidx holds the last tree's node ids
    bool defer_pred;   // a tree grown on every row records leaf ids and leaves the addition to the next row-order pass
    bool write_nidx;   // the tree being grown records the node id of every row it places
    bool grads_ahead;    // option: a tree with update_pred queues the next gradient update behind itself
    bool grads_ready;    // the gradients of the predictions as they stand were computed ahead: evt_update_grads has nothing to do
    hipEvent_t tree_evs[2]; // per slot, recorded behind the tree's transfer to the host: evt_grow_tree_end waits for this, not for the stream
    int tree_in_flight;     // trees queued by evt_grow_tree_begin that evt_grow_tree_end has not collected (0..2)
    int slot_w, slot_r;     // staging slot of the next tree queued / of the oldest tree not yet collected
    int64_t tree_seq;       // trees opened so far; slot_seq: the tree each slot holds
    int64_t slot_seq[2];
    // a tree grown one kernel stage at a time (evt_tree_open ... evt_tree_close); evt_grow_tree_begin drives the same stages
    struct {
        int phase; // 0 no tree open, 1 histogram next, 2 split search next, 3 partition next, 4 levels done
        int level;
        bool all_rows, defer, fuse_pred;
        bool hist_fused; // levels below the root get their histograms from the scatter pass of the level above
        bool blob_sent;  // the finished tree's transfer to the host rode along with the tree's last kernel
        uint32_t *is_cur, *is_next; // row-id lists of the current level and of the one below
        evt_params p;
    } step;
    bool pend_pred;    // pred lacks the leaf values tree.pred[nidx[i] - 1] of the last tree (the device Tree arrays keep them until the next tree starts, and what is pending is applied before that)
    uint8_t last_cond;

    // profiling
    int profiling;     // bit mask of kernel classes timed with events
    bool prof_open;
    hipEvent_t launch_e0, launch_e1; // events the next histogram launch carries itself (nullptr: none)
    std::vector<ProfRec> recs;
    std::vector<hipEvent_t> free_events;
    int64_t prof_launches[EVT_K_COUNT];
    double prof_ms[EVT_K_COUNT];
    int64_t prof_units[EVT_K_COUNT];
};

// A set-up step that has to run once per device (hipFuncSetAttribute applies to the current device), from whichever
// thread gets there first.  The step itself is idempotent, so two threads that both find it pending may both run it;
// the flag is an atomic bit per device.
struct EvtDevOnce {
    std::atomic<uint64_t> done{0};
    static int current() {
        int d = -1;
        if (hipGetDevice(&d) != hipSuccess) d = -1;
        return d;
    }
    bool pending(int device) const { return device < 0 || device >= 64 || !((done.load(std::memory_order_acquire) >> device) & 1ull); }
    void mark(int device) {
        if (device >= 0 && device < 64) done.fetch_or(1ull << device, std::memory_order_release);
    }
};

// ---- error plumbing ---------------------------------------------------------------------
void evt_set_error(const char *fmt, ...);
#define HIPCHK(call)                                                                       \
    do {                                                                                   \
        hipError_t _e = (call);                                                            \
        if (_e != hipSuccess) {                                                            \
            evt_set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(_e), __FILE__, __LINE__); \
            return EVT_ERR_HIP;                                                            \
        }                                                                                  \
    } while (0)
// No C++ exception crosses the C ABI: every entry point that returns a status runs inside this guard.
template <typename F>
static int guarded(F &&f) {
    try {
        return f();
    } catch (const std::bad_alloc &) {
        evt_set_error("out of host memory");
        return EVT_ERR_NOMEM;
    } catch (const std::exception &e) {
        evt_set_error("internal error: %s", e.what());
        return EVT_ERR_INTERNAL;
    } catch (...) {
        evt_set_error("internal error");
        return EVT_ERR_INTERNAL;
    }
}
#define ARGCHK(cond, msg)                \
    do {                                 \
        if (!(cond)) {                   \
            evt_set_error("%s", msg);    \
            return EVT_ERR_ARG;          \
        }                                \
    } while (0)

// predict!'s update of one row's K outputs with a leaf's values (src/predict.jl:1-62): plain sum (mse and the exp-link
// losses), clamp to [-15, 15] (logloss), floor -15 on the scale outputs (gaussian_mle), shift by the row maximum and
// floor -15 (mlogloss).  pr may point to registers or memory.
// A split node in one 32-bit word: feature id (1-based) | cond_bin << 16 | split << 24 | numeric << 25.  Leaves are 0.
// the two-parameter MLE losses: outputs come in (location, raw scale) pairs
#define EVT_IS_MLE2P(loss) ((loss) == EVT_LOSS_GAUSSIAN_MLE || (loss) == EVT_LOSS_LOGISTIC_MLE)
#define EVT_IS_CRED(loss) ((loss) == EVT_LOSS_CRED_VAR || (loss) == EVT_LOSS_CRED_STD)
#define EVT_IS_QUANTILE(loss) ((loss) == EVT_LOSS_QUANTILE || (loss) == EVT_LOSS_MULTIQUANTILE)
// losses whose gain is the weighted shift of the children's mean first-row value (Union{MAE,Quantile}, src/split.jl:68, :119)
#define EVT_IS_SHIFT(loss) ((loss) == EVT_LOSS_MAE || EVT_IS_QUANTILE(loss))
#define EVT_LOSS_LAST EVT_LOSS_MULTIQUANTILE
// One-target mse, mae and quantile need no accumulator for their second gradient row (mse: h = 2w; mae: h = 0; quantile:
// the raw residual, read per row when the leaves are valued; no gain reads it): their histograms hold the channels {g, w} only.
#define EVT_TWO_CHAN(loss, K) (((loss) == EVT_LOSS_MSE || EVT_IS_SHIFT(loss)) && (K) == 1)
#define EVT_NODE_SPLIT (1u << 24)
#define EVT_NODE_NUMERIC (1u << 25)
#ifdef __HIPCC__
__host__ __device__ __forceinline__ uint32_t evt_pack_node(int feat, int cond_bin, bool numeric) {
    return (uint32_t)feat | ((uint32_t)cond_bin << 16) | EVT_NODE_SPLIT | (numeric ? EVT_NODE_NUMERIC : 0u);
}
// The fixed-point word of channel a for one row.  The channel that shares its word with the row count holds 30 bits:
// it is staged as a 32-bit word (half the plane to gather from) and widened here to (q << 16) + 1.
template <bool PACK>
__device__ __forceinline__ unsigned long long evt_load_gq(const unsigned long long *__restrict__ gq, int64_t N, int a, uint32_t id) {
    if (PACK && a == 0) {
        const long long q = (long long)reinterpret_cast<const int32_t *>(gq)[id];
        return ((unsigned long long)q << EVT_PACK_CNT_BITS) + 1ull;
    }
    return gq[(size_t)a * N + id];
}

// Chunk descriptors of a level, for the partition kernels that run after the split search: chunk c of the level is
// chunk c - c0 of node n, whose segment ends at `end`: {n, first position, end, c0}.  One wavefront per active node
// writes the descriptors of that node's chunks, cprefix[i] .. cprefix[i + 1] (two dependent trips to memory, then
// stores); `w` of `nw` wavefronts share the level's nodes.
__device__ __forceinline__ void evt_fill_chunk_descriptors(const int64_t *__restrict__ hdr, const int32_t *__restrict__ act_node,
                                                           const int64_t *__restrict__ cprefix, const int64_t *__restrict__ seg_start,
                                                           const int64_t *__restrict__ seg_len, uint4 *cdesc, int w, int nw) {
    const int lane = threadIdx.x & 63;
    const int n_act = (int)hdr[LH_N_ACT];
    for (int i = w; i < n_act; i += nw) {
        const int n = act_node[i];
        const int64_t c0 = cprefix[i], c1 = cprefix[i + 1];
        const int64_t seg = seg_start[n], len = seg_len[n];
        for (int64_t c = c0 + lane; c < c1; c += 64)
            cdesc[c] = make_uint4((uint32_t)n, (uint32_t)(seg + (c - c0) * EVT_CHUNK), (uint32_t)(seg + len), (uint32_t)c0);
    }
}

__device__ __forceinline__ void evt_add_leaf(float *pr, const float *lp, int K, int loss) {
    if (loss == EVT_LOSS_LOGLOSS) {
        for (int k = 0; k < K; k++) pr[k] = fminf(fmaxf(pr[k] + lp[k], -15.0f), 15.0f);
    } else if (loss == EVT_LOSS_GAUSSIAN_MLE || loss == EVT_LOSS_LOGISTIC_MLE) {
        for (int t = 0; t < K / 2; t++) {
            pr[2 * t] += lp[2 * t];
            pr[2 * t + 1] = fmaxf(-15.0f, pr[2 * t + 1] + lp[2 * t + 1]);
        }
    } else if (loss == EVT_LOSS_MLOGLOSS) {
        float m = -INFINITY;
        for (int k = 0; k < K; k++) {
            pr[k] += lp[k];
            m = fmaxf(m, pr[k]);
        }
        for (int k = 0; k < K; k++) pr[k] = fmaxf(-15.0f, pr[k] - m);
    } else {
        for (int k = 0; k < K; k++) pr[k] += lp[k];
    }
}
#endif

// ---- kernel launchers (each only enqueues on c->stream) -----------------------------------
// grad
int launch_grads(evt_ctx *c);
int launch_quantize(evt_ctx *c);
int launch_apply_pending(evt_ctx *c);
int launch_set_weight_row(evt_ctx *c, const float *w_dev);
int launch_validate_classes(evt_ctx *c);
int launch_init_pred(evt_ctx *c, const float *mu_dev, const float *offset_dev);
// data layout
int launch_transpose_validate(evt_ctx *c);
int launch_binarize(evt_ctx *c, const double *x_dev, const double *edges_dev, const int32_t *edge_off_dev);
int launch_build_planes(evt_ctx *c);
int launch_binarize_cols(hipStream_t s, const double *x_dev, const double *edges_dev, const int32_t *edge_off_dev, uint8_t *xcm, int64_t n,
                         int F, int64_t ldx, int64_t ldo);
int launch_eval_metric(evt_ctx *c, int metric, double *partial);
// tree
int launch_tree_begin(evt_ctx *c);
int launch_iota(evt_ctx *c, uint32_t *dst, int64_t n);
int launch_compact_mask(evt_ctx *c, uint8_t cond, bool draw, unsigned long long seed);
int quantile_leaf_buffers(evt_ctx *c);
int launch_quantile_leaves(evt_ctx *c, const evt_params *p);
int launch_hist_build(evt_ctx *c, int level, const uint32_t *is_cur);
int launch_scan(evt_ctx *c, int level, const evt_params *p, bool leaf_level);
bool scan_folds_leaves(const evt_ctx *c);
int launch_obliv_select(evt_ctx *c, int level, const evt_params *p);
int launch_part_count(evt_ctx *c, int level, const uint32_t *is_cur);
int launch_part_scatter(evt_ctx *c, int level, const uint32_t *is_cur, uint32_t *is_next, bool fuse_pred);
bool scatter_can_build_hist(const evt_ctx *c, int nfs);
int launch_final_fused(evt_ctx *c, int level, const uint32_t *is_cur, bool fuse_pred, bool send_blob);
int launch_nidx_from_segments(evt_ctx *c, int level, const uint32_t *is_cur);
int launch_copy_to_host(evt_ctx *c, const void *src_dev, void *dst_host_dev, size_t nbytes);
int launch_copy_words(evt_ctx *c, const void *src, void *dst, size_t nbytes);
int launch_fill_u32(evt_ctx *c, uint32_t *dst, uint32_t v, int64_t n);
int launch_fill_bytes(evt_ctx *c, void *dst, int64_t nbytes);
// predict
int launch_predict_tree_cache(evt_ctx *c, bool send_blob);
int launch_hist_export(evt_ctx *c, double *out_dev);
int launch_nidx_from_tree(evt_ctx *c, bool use_mask, uint8_t cond);

// profiling helpers
void prof_begin(evt_ctx *c, int cls, int level);
void prof_begin_launch(evt_ctx *c, int cls, int level);
void prof_end(evt_ctx *c);
