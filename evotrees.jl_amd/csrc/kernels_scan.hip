// Split search: subtract_hist! + _scan_node!/get_best_split + _child_sums! + leaf values
// (src/fit-utils.jl:321-332, :403-486; src/split.jl:1, :58-66, :108-117; src/predict.jl:198-234).
//
// One block per node of the level; each wave takes sampled features round-robin; lanes are bins.
// The left sums of all bins of one (node, feature) come from one wavefront inclusive prefix scan
// of the int64 histogram (DPP row shifts + row broadcasts), the candidate gains are evaluated in
// Float64 with the reference's expression order, and the best candidate is found with a
// cross-lane arg-max whose ties go to the lowest bin, then the earliest feature of js — the
// reference's "first maximum wins" (strict '>' at src/fit-utils.jl:447).
#include "evt_internal.h"
#include <float.h>

#define NO_BIN 0x7fffffff

struct ScanBest {
    double gain;
    int jp, bin;
};
// The candidate as the one- and two-output kernels hand it over: with the feature (1-based id, negative when categorical)
// and the fixed-point totals left of the split, so that the pass that decides needs neither the feature tables nor the
// histogram again.
struct ScanBestQ {
    double gain;
    int jp, bin;
    int feat, pad;
    long long qL[EVT_MAX_NA];
};
static_assert(sizeof(ScanBestQ) == 64, "one candidate per 64-byte line");

struct ScanArgs {
    ScanBest *sbest; // ScanBestQ entries for k_scan / k_scan_fin (same buffer)
    long long *hist;
    int64_t node_stride;
    const uint32_t *js;
    const uint8_t *feattypes;
    const int32_t *mono;
    int32_t *status;
    long long *node_sum;
    const double *qscale;
    TreeDev tree;
    double *ogains;
    double eta, lambda, L2, gamma, min_weight;
    int bagging;
    int nfs, B, F, K, NK, NAg, loss, level, leaf_level, oblivious, zero_children;
    int fold_leaves; // the level's children are leaves: their weight and values are written along with the split (no pass of their own)
    // the level's chunk descriptors, written here when no histogram kernel runs at this level (cdesc == nullptr: not here)
    const int64_t *hdr;
    const int32_t *act_node;
    const int64_t *cprefix;
    const int64_t *seg_start;
    const int64_t *seg_len;
    uint4 *cdesc;
};

// ---- wavefront primitives -----------------------------------------------------------------
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ long long dpp_move_i64(long long x) {
    int lo = (int)(x & 0xffffffffll), hi = (int)(x >> 32);
    lo = __builtin_amdgcn_update_dpp(0, lo, CTRL, ROW_MASK, 0xf, false);
    hi = __builtin_amdgcn_update_dpp(0, hi, CTRL, ROW_MASK, 0xf, false);
    return ((long long)hi << 32) | (unsigned int)lo;
}

// Inclusive prefix sum over the 64 lanes of a wavefront.
// row_shr:1,2,4,8 scan each row of 16 lanes; row_bcast:15 then row_bcast:31 carry row totals forward.
__device__ __forceinline__ long long wave_incl_scan_i64(long long x) {
    x += dpp_move_i64<0x111, 0xf>(x); // row_shr:1
    x += dpp_move_i64<0x112, 0xf>(x); // row_shr:2
    x += dpp_move_i64<0x114, 0xf>(x); // row_shr:4
    x += dpp_move_i64<0x118, 0xf>(x); // row_shr:8
    x += dpp_move_i64<0x142, 0xa>(x); // row_bcast:15 into rows 1 and 3
    x += dpp_move_i64<0x143, 0xc>(x); // row_bcast:31 into rows 2 and 3
    return x;
}

__device__ __forceinline__ long long wave_sum_i64(long long x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        int lo = __shfl_xor((int)(x & 0xffffffffll), o), hi = __shfl_xor((int)(x >> 32), o);
        x += ((long long)hi << 32) | (unsigned int)lo;
    }
    return x;
}

// Arg-max over the 64 lanes of a wavefront: highest gain, of equal gains the lowest bin; every lane gets the result.
// Same data movement as the prefix scan above (row shifts, then row broadcasts; a lane without a source combines with
// the identity), so the reduction ends in lane 63 - VALU moves only, where a butterfly of cross-lane shuffles goes
// through the LDS crossbar eighteen times, each a dependent round trip.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ void argmax_step(double &g, int &b) {
    const long long gb = __double_as_longlong(g);
    const int olo = __builtin_amdgcn_update_dpp(0, (int)(gb & 0xffffffffll), CTRL, ROW_MASK, 0xf, false);
    const int ohi = __builtin_amdgcn_update_dpp((int)0xFFF00000, (int)(gb >> 32), CTRL, ROW_MASK, 0xf, false); // -inf
    const int ob = __builtin_amdgcn_update_dpp(NO_BIN, b, CTRL, ROW_MASK, 0xf, false);
    const double og = __longlong_as_double(((long long)ohi << 32) | (unsigned int)olo);
    if (og > g || (og == g && ob < b)) { g = og; b = ob; }
}
__device__ __forceinline__ void wave_argmax(double &g, int &b) {
    argmax_step<0x111, 0xf>(g, b); // row_shr:1
    argmax_step<0x112, 0xf>(g, b); // row_shr:2
    argmax_step<0x114, 0xf>(g, b); // row_shr:4
    argmax_step<0x118, 0xf>(g, b); // row_shr:8
    argmax_step<0x142, 0xa>(g, b); // row_bcast:15 into rows 1 and 3
    argmax_step<0x143, 0xc>(g, b); // row_bcast:31 into rows 2 and 3
    const long long gb = __double_as_longlong(g);
    const int lo = __builtin_amdgcn_readlane((int)(gb & 0xffffffffll), 63), hi = __builtin_amdgcn_readlane((int)(gb >> 32), 63);
    g = __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
    b = __builtin_amdgcn_readlane(b, 63);
}


// ---- Float64 gain algebra, expression order as in the reference ------------------------------
__device__ __forceinline__ double term_gh(double g, double h, double w, double lambda, double L2) {
    double d = h + lambda * w + L2;
    if (!(d > DBL_EPSILON)) d = DBL_EPSILON;
    return g * g / d / 2.0;
}

// fixed-point channel sums -> the 2K+1 Float64 statistics [g.., h.., w]
__device__ __forceinline__ void decode_vals(const long long *q, const double *sc, int loss, int NK, double *out) {
    if (EVT_TWO_CHAN(loss, (NK - 1) / 2)) { // one-target mse / mae: channels {g, w}; h = 2w (mse), 0 (mae)
        double w = (double)q[1] * sc[1];
        out[0] = (double)q[0] * sc[0];
        out[1] = (loss == EVT_LOSS_MSE) ? 2.0 * w : 0.0;
        out[2] = w;
    } else {
        for (int k = 0; k < NK; k++) out[k] = (double)q[k] * sc[k];
    }
}

// _term_cred with _cred_Z (src/split.jl:3-4, src/loss.jl:275-290): Z |m1| / (1 + L2 / w), Z = VHM / (VHM + EVPV) for
// cred_var and the same ratio of square roots for cred_std, VHM = (m1 / w)^2, EVPV = max(eps, m2 / w - VHM)
__device__ __forceinline__ double term_cred(int loss, double m1, double m2, double w, double L2) {
    const double mean = m1 / w;
    const double VHM = mean * mean;
    double EVPV = m2 / w - VHM;
    if (!(EVPV > DBL_EPSILON)) EVPV = DBL_EPSILON;
    const double Z = (loss == EVT_LOSS_CRED_VAR) ? VHM / (VHM + EVPV) : sqrt(VHM) / (sqrt(VHM) + sqrt(EVPV));
    return Z * fabs(m1) / (1.0 + L2 / w);
}

// One output's term of node_gain (src/split.jl:58-78): zero for mae.
__device__ __forceinline__ double node_gain_k(int loss, double g, double h, double w, double lambda, double L2) {
    if (EVT_IS_SHIFT(loss)) return 0.0;
    if (EVT_IS_CRED(loss)) return term_cred(loss, g, h, w, L2);
    return term_gh(g, h, w, lambda, L2);
}

// One output's term of split_gain (src/split.jl:108-141): left + right.  (Sg, Sh, w_p) are the node's totals.  mae:
// _term_shift (src/split.jl:2), |g / w - mu_p| w / d on either side with d = max(eps, 1 + lambda + L2 / w).
__device__ __forceinline__ double split_gain_k(int loss, double Sg, double Sh, double w_p, double g_l, double h_l, double w_l, double w_r,
                                               double lambda, double L2) {
    if (EVT_IS_SHIFT(loss)) {
        double d_l = 1.0 + lambda + L2 / w_l, d_r = 1.0 + lambda + L2 / w_r;
        if (!(d_l > DBL_EPSILON)) d_l = DBL_EPSILON;
        if (!(d_r > DBL_EPSILON)) d_r = DBL_EPSILON;
        const double mu_p = Sg / w_p;
        return fabs(g_l / w_l - mu_p) * w_l / d_l + fabs((Sg - g_l) / w_r - mu_p) * w_r / d_r;
    }
    if (EVT_IS_CRED(loss)) return term_cred(loss, g_l, h_l, w_l, L2) + term_cred(loss, Sg - g_l, Sh - h_l, w_r, L2);
    return term_gh(g_l, h_l, w_l, lambda, L2) + term_gh(Sg - g_l, Sh - h_l, w_r, lambda, L2);
}

// pred_leaf_cpu! / pred_scalar (src/predict.jl:198-262) for output k
__device__ __forceinline__ double leaf_value(int loss, const double *S, int k, int K, double eta, int bagging, double lambda, double L2) {
    if (EVT_IS_QUANTILE(loss)) return 0.0; // valued from the leaf's rows once the tree is complete (launch_quantile_leaves)
    if (EVT_IS_CRED(loss)) return eta / (double)bagging * S[k] / (S[2 * K] + L2);
    if (loss == EVT_LOSS_MAE) {
        double d = S[2 * K] + lambda * S[2 * K] + L2;
        if (!(d > DBL_EPSILON)) d = DBL_EPSILON;
        return eta / (double)bagging * S[k] / d;
    }
    double d = S[K + k] + lambda * S[2 * K] + L2;
    if (!(d > DBL_EPSILON)) d = DBL_EPSILON;
    return -eta / (double)bagging * S[k] / d;
}

// shared prologue: node totals -> Float64 statistics.  Root totals are the bin sums of its first
// sampled feature (exact in integers: every feature's bins sum to the same total); other nodes carry
// the totals their parent's split gave them.
template <int NAG>
__device__ __forceinline__ void node_totals(const ScanArgs &A, int n, const long long *hn, bool writer, long long *s_Sq, double *s_S,
                                            double *s_sc) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid < NAG) s_sc[tid] = A.qscale[tid];
    if (A.level == 1) {
        if (wave == 0) {
            for (int ag = 0; ag < NAG; ag++) {
                long long s = 0;
                for (int b = lane; b < A.B; b += 64) s += hn[(int64_t)ag * A.B + b];
                s = wave_sum_i64(s);
                if (lane == 0) {
                    s_Sq[ag] = s;
                    if (writer) A.node_sum[(int64_t)n * NAG + ag] = s;
                }
            }
        }
    } else if (tid < NAG) {
        s_Sq[tid] = A.node_sum[(int64_t)n * NAG + tid];
    }
    __syncthreads();
    if (tid == 0) {
        double v[EVT_MAX_NK];
        long long q[NAG];
        for (int ag = 0; ag < NAG; ag++) q[ag] = s_Sq[ag];
        decode_vals(q, s_sc, A.loss, A.NK, v);
        for (int k = 0; k < A.NK; k++) s_S[k] = v[k];
    }
    __syncthreads();
}

// The decision for one node (get_best_split's threshold, src/fit-utils.jl:444-450; the Tree arrays, src/fit.jl:96-103;
// a node without a split becomes a leaf, src/predict.jl:198-262): thread 0 holds the node's best candidate (bg, bj, bb)
// and its feature (1-based id, type); S: the node's statistics (in shared memory).  Leaves {found, bj, bb} in s_dec.
__device__ __forceinline__ void scan_decide(const ScanArgs &A, int n, const double *S, int *s_dec, double bg, int bj, int bb, int feat, bool numeric) {
    const int K = A.K;
    const int found = (bb != NO_BIN && bg > A.gamma) ? 1 : 0;
    s_dec[0] = found; s_dec[1] = bj; s_dec[2] = bb;
    if (found) {
        A.tree.feat[n - 1] = feat;
        A.tree.cond_bin[n - 1] = (uint8_t)bb;
        A.tree.gain[n - 1] = (float)bg;
        A.tree.split[n - 1] = 1;
        A.tree.packed[n - 1] = evt_pack_node(feat, bb, numeric);
        A.status[n] = ST_SPLIT;
    } else {
        for (int k = 0; k < K; k++) A.tree.pred[(int64_t)K * (n - 1) + k] = (float)leaf_value(A.loss, S, k, K, A.eta, A.bagging, A.lambda, A.L2);
        A.status[n] = ST_LEAF;
    }
}

// Totals of the two children from the left child's (qL; right = parent - left, exact in integers; _child_sums!,
// src/fit-utils.jl:472-486), by one lane.  With fold_leaves the children are leaves of the last level: their weight, values
// and state are written here too - what the leaf-level pass would compute from node_sum (same integers, same expressions).
template <int NAG>
__device__ __forceinline__ void write_children(const ScanArgs &A, int n, const long long *qL, const long long *s_Sq, const double *s_sc) {
    const int NK = A.NK, K = A.K;
#pragma unroll
    for (int child = 0; child < 2; child++) {
        const int cn = 2 * n + child;
        long long qc[NAG];
#pragma unroll
        for (int ag = 0; ag < NAG; ag++) {
            qc[ag] = child ? s_Sq[ag] - qL[ag] : qL[ag];
            A.node_sum[(int64_t)cn * NAG + ag] = qc[ag];
        }
        if (A.fold_leaves) {
            double v[EVT_MAX_NK];
            decode_vals(qc, s_sc, A.loss, NK, v);
            A.tree.w[cn - 1] = (float)v[NK - 1];
            for (int k = 0; k < K; k++) A.tree.pred[(int64_t)K * (cn - 1) + k] = (float)leaf_value(A.loss, v, k, K, A.eta, A.bagging, A.lambda, A.L2);
            A.status[cn] = ST_LEAF;
        }
    }
}

// the children's histogram slices start from zero (the build child accumulates into its own)
template <int NAG>
__device__ __forceinline__ void zero_children_slices(const ScanArgs &A, int n) {
    long long *hc = A.hist + (int64_t)(2 * n - 1) * A.node_stride;
    const int64_t used = (int64_t)A.nfs * NAG * A.B;
    for (int64_t i = threadIdx.x; i < used; i += blockDim.x) {
        hc[i] = 0;
        hc[A.node_stride + i] = 0;
    }
}

// Pass 1: grid (nodes of the level, feature groups); one wave per (node, sampled feature).
// Writes the group's best candidate to sbest[node][group] (or the gain matrix for oblivious trees)
// and, for subtract nodes, materialises h[n] = h[parent] - h[sibling].
// FUSED: one block of 16 waves per node covers every sampled feature (at most 16) and finishes the node itself
// (scan_finish): one launch per level instead of two where a level is a chain of small kernels.
template <int NAG, int BPL, bool FUSED>
__global__ __launch_bounds__(FUSED ? 1024 : 256) void k_scan(ScanArgs A) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int n = (1 << (A.level - 1)) + blockIdx.x; // 1-based node id
    if constexpr (FUSED) {
        // the partition's chunk descriptors of this level, when the level's histograms came from the scatter pass above
        // and no histogram kernel wrote them: the highest wavefronts take them (idle unless 16 features are sampled)
        if (A.cdesc)
            evt_fill_chunk_descriptors(A.hdr, A.act_node, A.cprefix, A.seg_start, A.seg_len, A.cdesc,
                                       (int)blockIdx.x * nwaves + (nwaves - 1 - wave), (int)gridDim.x * nwaves);
    }
    // The block's time is a chain of round trips to memory, so requests go out in as few dependent steps as the data
    // allows: node state and feature id first; then, in one batch of unconditional loads, the histogram slices, the
    // feature's type and constraint, the node totals and the decode scales.
    const int jp = blockIdx.y * nwaves + wave;
    const bool have = jp < A.nfs; // wave-uniform; a wave past the last feature loads the last one's data and drops it
    const int jpc = have ? jp : A.nfs - 1;
    int f = (int)A.js[jpc] - 1;
    const int st = A.status[n];
    asm volatile("" : "+v"(f)); // the feature id is requested ahead of the branch on the node state, not behind it
    if (st != ST_BUILD && st != ST_SUBTRACT) return;
    const bool is_sub = (st == ST_SUBTRACT);
    // the channel layout fixes the outputs: two-output MLE losses have five channels, every other shape here one output
    constexpr int K = (NAG == 5) ? 2 : 1, NK = 2 * K + 1;
    const int B = A.B;
    // BPL = bins per lane = ceil(nbins / 64), a template parameter so that nbins <= 64 keeps one bin per lane in registers
    long long *hn = A.hist + (int64_t)(n - 1) * A.node_stride;
    const long long *hp = A.hist + (int64_t)((n >> 1) - 1) * A.node_stride;
    const long long *hs = A.hist + (int64_t)((n ^ 1) - 1) * A.node_stride;

    __shared__ long long s_Sq[EVT_MAX_NA];
    __shared__ double s_S[EVT_MAX_NK];
    __shared__ double s_sc[EVT_MAX_NA];
    __shared__ double s_wg[16];
    __shared__ int s_wjp[16], s_wbin[16];
    __shared__ int s_wfeat[16]; // feature of each wave (1-based id, negative when categorical)
    __shared__ long long s_wq[FUSED ? 1 : 4][NAG]; // two-pass search: left totals of each wave's best candidate
    __shared__ int s_dec[3];

    long long pre[NAG][BPL];
    long long vb[NAG][BPL];
    long long excl[NAG];
    const int64_t o0 = (int64_t)jpc * NAG * B;
    if (is_sub) {
#pragma unroll
        for (int ag = 0; ag < NAG; ag++) {
#pragma unroll
            for (int t = 0; t < BPL; t++) {
                const int b = lane * BPL + t;
                const int64_t o = o0 + (int64_t)ag * B + (b < B ? b : B - 1);
                pre[ag][t] = hp[o];
                vb[ag][t] = hs[o];
            }
        }
    } else {
#pragma unroll
        for (int ag = 0; ag < NAG; ag++) {
#pragma unroll
            for (int t = 0; t < BPL; t++) {
                const int b = lane * BPL + t;
                pre[ag][t] = hn[o0 + (int64_t)ag * B + (b < B ? b : B - 1)];
                vb[ag][t] = 0;
            }
        }
    }
    const bool numeric = A.feattypes[f] != 0;
    const int constraint = A.mono[f];
    // node totals and decode scales: the same few words for every thread of the block (scalar loads), so that below the
    // root no thread waits at a barrier for another to decode them
    long long nsq[NAG];
    double sc[NAG];
#pragma unroll
    for (int ag = 0; ag < NAG; ag++) {
        sc[ag] = A.qscale[ag];
        nsq[ag] = A.node_sum[(int64_t)n * NAG + ag]; // not yet written at level 1, and not used there
    }

#pragma unroll
    for (int ag = 0; ag < NAG; ag++) {
#pragma unroll
        for (int t = 0; t < BPL; t++) {
            const int b = lane * BPL + t;
            const long long v = (have && b < B) ? pre[ag][t] - vb[ag][t] : 0;
            if (is_sub && have && b < B) hn[o0 + (int64_t)ag * B + b] = v; // subtract_hist!: h[n] = h[parent] - h[sibling]
            pre[ag][t] = v;
        }
    }

    // node totals -> Float64 statistics
    double S[NK];
    if (A.level == 1) { // the root's totals are the bin sums of its first sampled feature
        node_totals<NAG>(A, n, hn, blockIdx.y == 0, s_Sq, s_S, s_sc);
        for (int k = 0; k < NK; k++) S[k] = s_S[k];
#pragma unroll
        for (int ag = 0; ag < NAG; ag++) sc[ag] = s_sc[ag];
    } else {
        decode_vals(nsq, sc, A.loss, NK, S);
        if (FUSED && tid == 0) { // the block's last step reads them from shared memory, behind the barriers below
#pragma unroll
            for (int ag = 0; ag < NAG; ag++) {
                s_sc[ag] = sc[ag];
                s_Sq[ag] = nsq[ag];
            }
            for (int k = 0; k < NK; k++) s_S[k] = S[k];
        }
    }

    double gain_p = 0.0;
    for (int k = 0; k < K; k++) gain_p += node_gain_k(A.loss, S[k], S[K + k], S[2 * K], A.lambda, A.L2);
    const double w_p = S[NK - 1];

    double wbest = -INFINITY;
    int wjp = NO_BIN, wbin = NO_BIN;
    long long wq[NAG];
#pragma unroll
    for (int ag = 0; ag < NAG; ag++) wq[ag] = 0;
    const int nodeidx = blockIdx.x;

    if (have) {
        const int bmax = numeric ? B - 1 : B;
        // inclusive prefix over the bins: within the lane, then across the wavefront
#pragma unroll
        for (int ag = 0; ag < NAG; ag++) {
            long long run = 0;
#pragma unroll
            for (int t = 0; t < BPL; t++) {
                run += pre[ag][t];
                pre[ag][t] = run;
            }
            const long long incl = wave_incl_scan_i64(run);
            excl[ag] = incl - run;
#pragma unroll
            for (int t = 0; t < BPL; t++) pre[ag][t] += excl[ag];
        }
        double lg = -INFINITY;
        int lb = NO_BIN;
        long long lq[NAG]; // fixed-point totals left of this lane's best candidate
#pragma unroll
        for (int ag = 0; ag < NAG; ag++) lq[ag] = 0;
#pragma unroll
        for (int t = 0; t < BPL; t++) {
            const int b = lane * BPL + t;
            if (b < B) {
                double gain = 0.0;
                bool ok = false;
                long long q[NAG];
#pragma unroll
                for (int ag = 0; ag < NAG; ag++) q[ag] = 0;
                if (b + 1 <= bmax) {
#pragma unroll
                    for (int ag = 0; ag < NAG; ag++) {
                        const long long prev = (t == 0) ? excl[ag] : pre[ag][t > 0 ? t - 1 : 0];
                        q[ag] = numeric ? pre[ag][t] : (pre[ag][t] - prev); // _acc_left!: accumulate vs single bin
                    }
                    double SL[NK];
                    decode_vals(q, sc, A.loss, NK, SL);
                    const double w_l = SL[NK - 1];
                    const double w_r = w_p - w_l;
                    if (w_l > A.min_weight && w_r > A.min_weight) {
                        ok = true;
                        if (constraint != 0) {
                            double SR[NK];
                            for (int k = 0; k < NK; k++) SR[k] = S[k] - SL[k];
                            const double predL = leaf_value(A.loss, SL, 0, K, A.eta, A.bagging, A.lambda, A.L2);
                            const double predR = leaf_value(A.loss, SR, 0, K, A.eta, A.bagging, A.lambda, A.L2);
                            ok = (constraint == -1 && predL > predR) || (constraint == 1 && predL < predR);
                        }
                        if (ok) {
                            double sg = 0.0;
                            for (int k = 0; k < K; k++) {
                                sg += split_gain_k(A.loss, S[k], S[K + k], w_p, SL[k], SL[K + k], w_l, w_r, A.lambda, A.L2);
                            }
                            gain = sg - gain_p;
                        }
                    }
                }
                if (A.oblivious) {
                    A.ogains[((int64_t)nodeidx * A.nfs + jp) * B + b] = ok ? gain : 0.0; // update_gains!
                } else if (ok && gain > lg) {
                    lg = gain;
                    lb = b + 1;
#pragma unroll
                    for (int ag = 0; ag < NAG; ag++) lq[ag] = q[ag];
                }
            }
        }
        if (!A.oblivious) {
            wave_argmax(lg, lb);
            if (lg > wbest) { wbest = lg; wjp = jp; wbin = lb; }
            if constexpr (!FUSED) {
                // the lane that holds the winning bin hands its left totals to the whole wave
                const int owner = (lb != NO_BIN) ? (lb - 1) / BPL : 0;
#pragma unroll
                for (int ag = 0; ag < NAG; ag++) {
                    const int lo = __shfl((int)(lq[ag] & 0xffffffffll), owner), hi = __shfl((int)(lq[ag] >> 32), owner);
                    wq[ag] = ((long long)hi << 32) | (unsigned int)lo;
                }
            }
        }
    }
    if (A.oblivious) return; // decision is taken for the whole level by k_obliv_select

    if (lane == 0) {
        s_wg[wave] = wbest; s_wjp[wave] = wjp; s_wbin[wave] = wbin;
        s_wfeat[wave] = numeric ? f + 1 : -(f + 1);
        if constexpr (!FUSED) {
#pragma unroll
            for (int ag = 0; ag < NAG; ag++) s_wq[wave][ag] = wq[ag];
        }
    }
    __syncthreads();
    double bg = -INFINITY;
    int bj = NO_BIN, bb = NO_BIN, bw = 0;
    if (tid == 0) {
        for (int w = 0; w < nwaves; w++) {
            if (s_wg[w] > bg || (s_wg[w] == bg && s_wjp[w] < bj)) { bg = s_wg[w]; bj = s_wjp[w]; bb = s_wbin[w]; bw = w; }
        }
    }
    if constexpr (FUSED) {
        // the node is finished here: wave jp scanned sampled feature jp, so the winner's left totals are still in the
        // registers of the lane that holds the winning bin - no second read of the histogram
        if (tid == 0) {
            A.tree.w[n - 1] = (float)S[NK - 1];
            const int wf = (bb != NO_BIN) ? s_wfeat[bj] : 1;
            scan_decide(A, n, s_S, s_dec, bg, bj, bb, wf < 0 ? -wf : wf, wf > 0);
        }
        __syncthreads();
        if (!s_dec[0]) return;
        if (have && jp == s_dec[1]) {
            const int b0 = s_dec[2] - 1; // 0-based winning bin: lane b0 / BPL, position b0 % BPL
            long long qL[NAG];
#pragma unroll
            for (int ag = 0; ag < NAG; ag++) {
                long long v = 0;
#pragma unroll
                for (int t = 0; t < BPL; t++) {
                    const long long prev = (t == 0) ? excl[ag] : pre[ag][t > 0 ? t - 1 : 0];
                    const long long q = numeric ? pre[ag][t] : (pre[ag][t] - prev);
                    if (t == b0 % BPL) v = q;
                }
                qL[ag] = v;
            }
            if (lane == b0 / BPL) write_children<NAG>(A, n, qL, s_Sq, s_sc);
        }
        if (A.zero_children) zero_children_slices<NAG>(A, n);
    } else if (tid == 0) {
        ScanBestQ r;
        r.gain = bg; r.jp = bj; r.bin = bb;
        r.feat = s_wfeat[bw]; r.pad = 0;
#pragma unroll
        for (int ag = 0; ag < EVT_MAX_NA; ag++) r.qL[ag] = (ag < NAG) ? s_wq[bw][ag < NAG ? ag : 0] : 0;
        reinterpret_cast<ScanBestQ *>(A.sbest)[(int64_t)nodeidx * gridDim.y + blockIdx.y] = r;
    }
}

// Pass 2: one block per node.  Leaf level: leaf value only.  Otherwise: arg-max over the feature
// groups (first maximum: highest gain, then earliest feature, whose bin is already the lowest),
// split iff gain > gamma; writes the Tree arrays, the children's totals (_child_sums!: left = bins
// 1..bin of the parent histogram, or that bin alone for categorical features; right = parent - left,
// exact in integers) and zeroes the children's histogram slices.
template <int NAG>
__global__ __launch_bounds__(256) void k_scan_fin(ScanArgs A, int ngroups) {
    const int tid = threadIdx.x;
    const int n = (1 << (A.level - 1)) + blockIdx.x;
    if (blockIdx.y > 0) {
        // Blocks beyond the first of a node only clear the children's histogram slices (the build child accumulates
        // into its own; a level with few nodes would otherwise leave 200 KB per node to one block).  They do not wait
        // for the decision: the slices of a node that turns out a leaf are never read.  The node's state may already
        // read SPLIT or LEAF here (the first block sets it), anything but INACTIVE means the level reached it.
        if (A.status[n] == ST_INACTIVE) return;
        long long *hc = A.hist + (int64_t)(2 * n - 1) * A.node_stride;
        const int64_t used = (int64_t)A.nfs * NAG * A.B;
        const int64_t zb = gridDim.y - 1, per = (used + zb - 1) / zb;
        const int64_t i0 = (int64_t)(blockIdx.y - 1) * per, i1 = i0 + per < used ? i0 + per : used;
        for (int64_t i = i0 + tid; i < i1; i += blockDim.x) {
            hc[i] = 0;
            hc[A.node_stride + i] = 0;
        }
        return;
    }
    // Everything the block needs is requested in one batch of unconditional loads, ahead of the branch on the node's
    // state: the state itself, the node's totals and decode scales, and this thread's candidate (group tid, clamped).
    const int tq = tid < NAG ? tid : 0;
    double qs = A.qscale[tq];
    long long nsq = A.node_sum[(int64_t)n * NAG + tq]; // not yet written at level 1, and not used there
    union CandWords {
        ScanBestQ q;
        uint4 v[4];
    };
    CandWords cw;
    {
        const uint4 *cp = reinterpret_cast<const uint4 *>(reinterpret_cast<const ScanBestQ *>(A.sbest) + (int64_t)blockIdx.x * ngroups + (tid < ngroups ? tid : 0));
#pragma unroll
        for (int k = 0; k < 4; k++) cw.v[k] = cp[k];
    }
    // nodes of the last level are the children of the split nodes above them (the root when max_depth == 1)
    int st = A.leaf_level ? (n > 1 ? A.status[n >> 1] : ST_SPLIT) : A.status[n];
    asm volatile("" : "+v"(st), "+v"(qs), "+v"(nsq));
#pragma unroll
    for (int k = 0; k < 4; k++) asm volatile("" : "+v"(cw.v[k].x), "+v"(cw.v[k].y), "+v"(cw.v[k].z), "+v"(cw.v[k].w));
    if (A.leaf_level) {
        if (st != ST_SPLIT) return;
    } else {
        if (st != ST_BUILD && st != ST_SUBTRACT) return;
    }
    const int NK = A.NK, K = A.K;
    long long *hn = A.hist + (int64_t)(n - 1) * A.node_stride;

    __shared__ long long s_Sq[EVT_MAX_NA];
    __shared__ double s_S[EVT_MAX_NK];
    __shared__ double s_sc[EVT_MAX_NA];
    __shared__ double s_g[256];
    __shared__ int s_j[256], s_b[256];
    __shared__ int s_dec[3];

    if (A.level == 1) {
        node_totals<NAG>(A, n, hn, true, s_Sq, s_S, s_sc);
    } else {
        if (tid < NAG) {
            s_sc[tid] = qs;
            s_Sq[tid] = nsq;
        }
        __syncthreads();
        if (tid == 0) {
            double v[EVT_MAX_NK];
            long long q[NAG];
            for (int ag = 0; ag < NAG; ag++) q[ag] = s_Sq[ag];
            decode_vals(q, s_sc, A.loss, NK, v);
            for (int k = 0; k < NK; k++) s_S[k] = v[k];
        }
        __syncthreads();
    }
    double S[EVT_MAX_NK];
    for (int k = 0; k < NK; k++) S[k] = s_S[k];
    if (tid == 0) A.tree.w[n - 1] = (float)S[NK - 1];

    if (A.leaf_level) {
        if (tid < K) A.tree.pred[(int64_t)K * (n - 1) + tid] = (float)leaf_value(A.loss, S, tid, K, A.eta, A.bagging, A.lambda, A.L2);
        if (tid == 0) A.status[n] = ST_LEAF;
        return;
    }
    // a thread takes the groups tid, tid + 256, ... (more than 1024 sampled features): ascending feature positions, so
    // only a strictly larger gain replaces an earlier one.  It keeps the whole candidate: the thread whose candidate wins
    // decides the node and writes the children's totals from its own registers - no feature table, no histogram read.
    ScanBestQ mine = cw.q;
    if (tid >= ngroups) {
        mine.gain = -INFINITY; mine.jp = NO_BIN; mine.bin = NO_BIN;
    }
    const ScanBestQ *cand = reinterpret_cast<const ScanBestQ *>(A.sbest) + (int64_t)blockIdx.x * ngroups;
    for (int g = tid + 256; g < ngroups; g += 256) {
        const ScanBestQ r = cand[g];
        if (r.gain > mine.gain) mine = r;
    }
    s_g[tid] = mine.gain; s_j[tid] = mine.jp; s_b[tid] = mine.bin;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if (tid < o) {
            if (s_g[tid + o] > s_g[tid] || (s_g[tid + o] == s_g[tid] && s_j[tid + o] < s_j[tid])) {
                s_g[tid] = s_g[tid + o]; s_j[tid] = s_j[tid + o]; s_b[tid] = s_b[tid + o];
            }
        }
        __syncthreads();
    }
    const double bg = s_g[0];
    const int bj = s_j[0], bb = s_b[0];
    // every sampled feature belongs to one group and every group to one thread: exactly one thread holds the winner;
    // without any candidate the first thread turns the node into a leaf
    const bool found = (bb != NO_BIN && bg > A.gamma);
    const bool owner = found ? (mine.jp == bj && mine.bin != NO_BIN) : (tid == 0);
    if (owner) {
        const int feat = found ? (mine.feat < 0 ? -mine.feat : mine.feat) : 1;
        scan_decide(A, n, s_S, s_dec, bg, bj, bb, feat, found ? mine.feat > 0 : true);
        if (found) {
            long long qL[NAG];
#pragma unroll
            for (int ag = 0; ag < NAG; ag++) qL[ag] = mine.qL[ag];
            write_children<NAG>(A, n, qL, s_Sq, s_sc);
        }
    }
    if (!found) return;
    // with one block per node this block clears the children's slices, otherwise the node's other blocks have
    if (A.zero_children && gridDim.y == 1) zero_children_slices<NAG>(A, n);
}

// Oblivious trees (grow_otree!, src/fit.jl:190-257): per-level decision from the sum of the
// nodes' gain matrices, masked where any node's gain is not positive; first maximum in
// (feature position, bin) order; all nodes of the level split on it iff it exceeds gamma.
struct OblivArgs {
    long long *hist;
    int64_t node_stride;
    const uint32_t *js;
    const uint8_t *feattypes;
    int32_t *status;
    long long *node_sum;
    const double *qscale;
    TreeDev tree;
    const double *ogains;
    const int64_t *hdr;
    const int32_t *act_node;
    double eta, lambda, L2, gamma;
    int bagging, nfs, B, K, NK, NAg, loss, level, zero_children;
};

__global__ __launch_bounds__(1024) void k_obliv_select(OblivArgs A) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int n_act = (int)A.hdr[LH_N_ACT];
    if (n_act <= 0) return;
    const int B = A.B, K = A.K, NK = A.NK, NAG = A.NAg;
    const int first = 1 << (A.level - 1);
    __shared__ double s_g[1024];
    __shared__ int s_i[1024];
    __shared__ int s_dec[3];
    __shared__ double s_gain;
    __shared__ double s_sc[EVT_MC_MAX_NK];
    if (tid < NAG) s_sc[tid] = A.qscale[tid];
    // level matrix and its first maximum
    double bg = -INFINITY;
    int bi = NO_BIN;
    const int cells = A.nfs * B;
    for (int c = tid; c < cells; c += blockDim.x) {
        double acc = 0.0;
        bool allpos = true;
        for (int i = 0; i < n_act; i++) {
            const int n = A.act_node[i];
            const double g = A.ogains[(int64_t)(n - first) * cells + c];
            acc += g;
            if (n > 1) allpos = allpos && (g > 0.0);
        }
        const double v = allpos ? acc : 0.0;
        if (v > bg) { bg = v; bi = c; } // c ascending per thread: first maximum kept
    }
    s_g[tid] = bg;
    s_i[tid] = bi;
    __syncthreads();
    for (int o = blockDim.x >> 1; o > 0; o >>= 1) {
        if (tid < o) {
            if (s_g[tid + o] > s_g[tid] || (s_g[tid + o] == s_g[tid] && s_i[tid + o] < s_i[tid])) {
                s_g[tid] = s_g[tid + o];
                s_i[tid] = s_i[tid + o];
            }
        }
        __syncthreads();
    }
    if (tid == 0) {
        const int found = (s_i[0] != NO_BIN && s_g[0] > A.gamma) ? 1 : 0;
        s_dec[0] = found;
        s_dec[1] = found ? s_i[0] / B : 0;
        s_dec[2] = found ? (s_i[0] % B) + 1 : 0;
        s_gain = s_g[0];
    }
    __syncthreads();
    const int found = s_dec[0], bj = s_dec[1], bb = s_dec[2];
    const double bgain = s_gain;
    for (int i = wave; i < n_act; i += nwaves) {
        const int n = A.act_node[i];
        long long Sq[EVT_MC_MAX_NK];
        double S[EVT_MC_MAX_NK];
        for (int ag = 0; ag < NAG; ag++) Sq[ag] = A.node_sum[(int64_t)n * NAG + ag];
        decode_vals(Sq, s_sc, A.loss, NK, S);
        if (lane == 0) A.tree.w[n - 1] = (float)S[NK - 1];
        if (!found) {
            if (lane < K) A.tree.pred[(int64_t)K * (n - 1) + lane] = (float)leaf_value(A.loss, S, lane, K, A.eta, A.bagging, A.lambda, A.L2);
            if (lane == 0) A.status[n] = ST_LEAF;
            continue;
        }
        const int feat = (int)A.js[bj];
        const bool numeric = A.feattypes[feat - 1] != 0;
        const long long *hn = A.hist + (int64_t)(n - 1) * A.node_stride;
        for (int ag = 0; ag < NAG; ag++) {
            const int64_t o = ((int64_t)bj * NAG + ag) * B;
            long long s = 0;
            for (int b = lane; b < B; b += 64) {
                const bool in = numeric ? (b + 1 <= bb) : (b + 1 == bb);
                if (in) s += hn[o + b];
            }
            s = wave_sum_i64(s);
            if (lane == 0) {
                A.node_sum[(int64_t)(2 * n) * NAG + ag] = s;
                A.node_sum[(int64_t)(2 * n + 1) * NAG + ag] = Sq[ag] - s;
            }
        }
        if (lane == 0) {
            A.tree.feat[n - 1] = feat;
            A.tree.cond_bin[n - 1] = (uint8_t)bb;
            A.tree.gain[n - 1] = (float)bgain;
            A.tree.split[n - 1] = 1;
            A.tree.packed[n - 1] = evt_pack_node(feat, bb, A.feattypes[feat - 1] != 0);
            A.status[n] = ST_SPLIT;
        }
        if (!A.zero_children) continue;
        long long *hc = A.hist + (int64_t)(2 * n - 1) * A.node_stride;
        const int64_t used = (int64_t)A.nfs * NAG * B;
        for (int64_t t = lane; t < used; t += 64) {
            hc[t] = 0;
            hc[A.node_stride + t] = 0;
        }
    }
}

// ---- any number of outputs (multi-class log loss) ------------------------------------------------
// Same search as k_scan / k_scan_fin with the channel count a run-time value: the node statistics live in shared
// memory and the candidate gain is accumulated output by output, gain += term(left_k) + term(right_k) in the
// reference's order (split_gain, src/split.jl:108-117), from one prefix scan per channel.
__device__ __forceinline__ void node_totals_mc(const ScanArgs &A, int n, const long long *hn, bool writer, long long *s_Sq, double *s_S,
                                               double *s_sc) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int NAG = A.NAg;
    if (tid < NAG) s_sc[tid] = A.qscale[tid];
    if (A.level == 1) {
        for (int ag = wave; ag < NAG; ag += (blockDim.x >> 6)) {
            long long s = 0;
            for (int b = lane; b < A.B; b += 64) s += hn[(int64_t)ag * A.B + b];
            s = wave_sum_i64(s);
            if (lane == 0) {
                s_Sq[ag] = s;
                if (writer) A.node_sum[(int64_t)n * NAG + ag] = s;
            }
        }
    } else if (tid < NAG) {
        s_Sq[tid] = A.node_sum[(int64_t)n * NAG + tid];
    }
    __syncthreads();
    if (tid < NAG) s_S[tid] = (double)s_Sq[tid] * s_sc[tid];
    __syncthreads();
}

// left-side sums of one channel for this lane's BPL bins (numeric: inclusive prefix; categorical: the bin alone);
// subtract nodes materialise h[n] = h[parent] - h[sibling] on the way
template <int BPL>
__device__ __forceinline__ void left_sums(const ScanArgs &A, long long *hn, const long long *hp, const long long *hs, int64_t o, bool is_sub,
                                          bool numeric, int lane, long long *left) {
    long long val[BPL];
    long long run = 0;
#pragma unroll
    for (int t = 0; t < BPL; t++) {
        const int b = lane * BPL + t;
        long long v = 0;
        if (b < A.B) {
            if (is_sub) {
                v = hp[o + b] - hs[o + b];
                hn[o + b] = v;
            } else {
                v = hn[o + b];
            }
        }
        val[t] = v;
        run += v;
        left[t] = run;
    }
    const long long excl = wave_incl_scan_i64(run) - run;
#pragma unroll
    for (int t = 0; t < BPL; t++) left[t] = numeric ? left[t] + excl : val[t];
}

template <int BPL>
__global__ __launch_bounds__(256) void k_scan_mc(ScanArgs A) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int n = (1 << (A.level - 1)) + blockIdx.x;
    const int st = A.status[n];
    if (st != ST_BUILD && st != ST_SUBTRACT) return;
    const bool is_sub = (st == ST_SUBTRACT);
    const int B = A.B, NK = A.NK, K = A.K, NAG = A.NAg;
    long long *hn = A.hist + (int64_t)(n - 1) * A.node_stride;
    const long long *hp = A.hist + (int64_t)((n >> 1) - 1) * A.node_stride;
    const long long *hs = A.hist + (int64_t)((n ^ 1) - 1) * A.node_stride;

    __shared__ long long s_Sq[EVT_MC_MAX_NK];
    __shared__ double s_S[EVT_MC_MAX_NK];
    __shared__ double s_sc[EVT_MC_MAX_NK];
    __shared__ double s_wg[4];
    __shared__ int s_wjp[4], s_wbin[4];

    node_totals_mc(A, n, hn, blockIdx.y == 0, s_Sq, s_S, s_sc);
    double gain_p = 0.0;
    for (int k = 0; k < K; k++) gain_p += node_gain_k(A.loss, s_S[k], s_S[K + k], s_S[2 * K], A.lambda, A.L2);
    const double w_p = s_S[NK - 1];

    double wbest = -INFINITY;
    int wjp = NO_BIN, wbin = NO_BIN;
    const int nodeidx = blockIdx.x;
    const int jp = blockIdx.y * nwaves + wave;
    if (jp < A.nfs) {
        const int f = (int)A.js[jp] - 1;
        const bool numeric = A.feattypes[f] != 0;
        const int bmax = numeric ? B - 1 : B;
        long long lq[BPL];
        double w_l[BPL], w_r[BPL], sg[BPL];
        bool ok[BPL];
        left_sums<BPL>(A, hn, hp, hs, ((int64_t)jp * NAG + (NAG - 1)) * B, is_sub, numeric, lane, lq);
#pragma unroll
        for (int t = 0; t < BPL; t++) {
            const int b = lane * BPL + t;
            w_l[t] = (double)lq[t] * s_sc[NAG - 1];
            w_r[t] = w_p - w_l[t];
            ok[t] = (b < B) && (b + 1 <= bmax) && (w_l[t] > A.min_weight) && (w_r[t] > A.min_weight);
            sg[t] = 0.0;
        }
        for (int k = 0; k < K; k++) {
            long long gq[BPL], hq[BPL];
            left_sums<BPL>(A, hn, hp, hs, ((int64_t)jp * NAG + k) * B, is_sub, numeric, lane, gq);
            left_sums<BPL>(A, hn, hp, hs, ((int64_t)jp * NAG + K + k) * B, is_sub, numeric, lane, hq);
            const double Sg = s_S[k], Sh = s_S[K + k];
#pragma unroll
            for (int t = 0; t < BPL; t++) {
                const double g_l = (double)gq[t] * s_sc[k], h_l = (double)hq[t] * s_sc[K + k];
                sg[t] += split_gain_k(A.loss, Sg, Sh, w_p, g_l, h_l, w_l[t], w_r[t], A.lambda, A.L2);
            }
        }
        double lg = -INFINITY;
        int lb = NO_BIN;
#pragma unroll
        for (int t = 0; t < BPL; t++) {
            const int b = lane * BPL + t;
            if (b < B) {
                const double gain = sg[t] - gain_p;
                if (A.oblivious) {
                    A.ogains[((int64_t)nodeidx * A.nfs + jp) * B + b] = ok[t] ? gain : 0.0;
                } else if (ok[t] && gain > lg) {
                    lg = gain;
                    lb = b + 1;
                }
            }
        }
        if (!A.oblivious) {
            wave_argmax(lg, lb);
            if (lg > wbest) { wbest = lg; wjp = jp; wbin = lb; }
        }
    }
    if (A.oblivious) return;
    if (lane == 0) { s_wg[wave] = wbest; s_wjp[wave] = wjp; s_wbin[wave] = wbin; }
    __syncthreads();
    if (tid == 0) {
        double bg = -INFINITY;
        int bj = NO_BIN, bb = NO_BIN;
        for (int w = 0; w < nwaves; w++) {
            if (s_wg[w] > bg || (s_wg[w] == bg && s_wjp[w] < bj)) { bg = s_wg[w]; bj = s_wjp[w]; bb = s_wbin[w]; }
        }
        ScanBest r;
        r.gain = bg; r.jp = bj; r.bin = bb;
        A.sbest[(int64_t)nodeidx * gridDim.y + blockIdx.y] = r;
    }
}

__global__ __launch_bounds__(256) void k_scan_fin_mc(ScanArgs A, int ngroups) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = (1 << (A.level - 1)) + blockIdx.x;
    if (A.leaf_level) {
        if (n > 1 && A.status[n >> 1] != ST_SPLIT) return;
    } else {
        const int st = A.status[n];
        if (st != ST_BUILD && st != ST_SUBTRACT) return;
    }
    const int B = A.B, NK = A.NK, K = A.K, NAG = A.NAg;
    long long *hn = A.hist + (int64_t)(n - 1) * A.node_stride;
    __shared__ long long s_Sq[EVT_MC_MAX_NK];
    __shared__ double s_S[EVT_MC_MAX_NK];
    __shared__ double s_sc[EVT_MC_MAX_NK];
    __shared__ double s_g[256];
    __shared__ int s_j[256], s_b[256];
    __shared__ int s_dec[3];
    node_totals_mc(A, n, hn, true, s_Sq, s_S, s_sc);
    if (tid == 0) A.tree.w[n - 1] = (float)s_S[NK - 1];
    if (A.leaf_level) {
        if (tid < K) A.tree.pred[(int64_t)K * (n - 1) + tid] = (float)leaf_value(A.loss, s_S, tid, K, A.eta, A.bagging, A.lambda, A.L2);
        if (tid == 0) A.status[n] = ST_LEAF;
        return;
    }
    double bg = -INFINITY;
    int bj = NO_BIN, bb = NO_BIN;
    // a thread takes the groups tid, tid + 256, ... (more than 1024 sampled features): ascending feature positions, so
    // only a strictly larger gain replaces an earlier one
    for (int g = tid; g < ngroups; g += 256) {
        const ScanBest r = A.sbest[(int64_t)blockIdx.x * ngroups + g];
        if (r.gain > bg) { bg = r.gain; bj = r.jp; bb = r.bin; }
    }
    s_g[tid] = bg; s_j[tid] = bj; s_b[tid] = bb;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if (tid < o) {
            if (s_g[tid + o] > s_g[tid] || (s_g[tid + o] == s_g[tid] && s_j[tid + o] < s_j[tid])) {
                s_g[tid] = s_g[tid + o]; s_j[tid] = s_j[tid + o]; s_b[tid] = s_b[tid + o];
            }
        }
        __syncthreads();
    }
    if (tid == 0) {
        bg = s_g[0]; bj = s_j[0]; bb = s_b[0];
        const int found = (bb != NO_BIN && bg > A.gamma) ? 1 : 0;
        s_dec[0] = found; s_dec[1] = bj; s_dec[2] = bb;
        if (found) {
            const int feat = (int)A.js[bj];
            A.tree.feat[n - 1] = feat;
            A.tree.cond_bin[n - 1] = (uint8_t)bb;
            A.tree.gain[n - 1] = (float)bg;
            A.tree.split[n - 1] = 1;
            A.tree.packed[n - 1] = evt_pack_node(feat, bb, A.feattypes[feat - 1] != 0);
            A.status[n] = ST_SPLIT;
        } else {
            A.status[n] = ST_LEAF;
        }
    }
    __syncthreads();
    if (!s_dec[0]) {
        if (tid < K) A.tree.pred[(int64_t)K * (n - 1) + tid] = (float)leaf_value(A.loss, s_S, tid, K, A.eta, A.bagging, A.lambda, A.L2);
        return;
    }
    bj = s_dec[1]; bb = s_dec[2];
    {
        const int f = (int)A.js[bj] - 1;
        const bool numeric = A.feattypes[f] != 0;
        for (int ag = wave; ag < NAG; ag += (blockDim.x >> 6)) {
            const int64_t o = ((int64_t)bj * NAG + ag) * B;
            long long s = 0;
            for (int b = lane; b < B; b += 64) {
                const bool in = numeric ? (b + 1 <= bb) : (b + 1 == bb);
                if (in) s += hn[o + b];
            }
            s = wave_sum_i64(s);
            if (lane == 0) {
                A.node_sum[(int64_t)(2 * n) * NAG + ag] = s;
                A.node_sum[(int64_t)(2 * n + 1) * NAG + ag] = s_Sq[ag] - s;
            }
        }
    }
    if (!A.zero_children) return;
    long long *hc = A.hist + (int64_t)(2 * n - 1) * A.node_stride;
    const int64_t used = (int64_t)A.nfs * NAG * B;
    for (int64_t i = tid; i < used; i += blockDim.x) {
        hc[i] = 0;
        hc[A.node_stride + i] = 0;
    }
}

// The pass over the last split level also writes its children's leaf values (binary trees with the fixed channel layouts).
bool scan_folds_leaves(const evt_ctx *c) { return !c->mc && c->tree_type != EVT_TREE_OBLIVIOUS && c->D > 1; }

int launch_scan(evt_ctx *c, int level, const evt_params *p, bool leaf_level) {
    ScanArgs A;
    A.sbest = reinterpret_cast<ScanBest *>(c->sbest);
    A.hist = c->hist;
    A.node_stride = (int64_t)c->F * c->NAg * c->B;
    A.js = c->js;
    A.feattypes = c->feattypes;
    A.mono = c->mono;
    A.status = c->status;
    A.node_sum = c->node_sum;
    A.qscale = c->qscale;
    A.tree = c->tree;
    A.ogains = c->ogains;
    A.eta = p->eta; A.lambda = p->lambda; A.L2 = p->L2; A.gamma = p->gamma; A.min_weight = p->min_weight;
    A.bagging = p->bagging_size;
    A.nfs = c->n_js_last; A.B = c->B; A.F = c->F; A.K = c->K; A.NK = c->NK; A.NAg = c->NAg; A.loss = c->loss;
    A.level = level;
    A.leaf_level = leaf_level ? 1 : 0;
    A.oblivious = (c->tree_type == EVT_TREE_OBLIVIOUS) ? 1 : 0;
    A.zero_children = (level + 1 < c->D) ? 1 : 0; // children at the last level never get a histogram
    A.fold_leaves = (!leaf_level && scan_folds_leaves(c) && level + 1 == c->D) ? 1 : 0;
    A.cdesc = nullptr;
    if (c->step.hist_fused && level > 1 && !leaf_level) {
        const LevelTab &L = c->lvl[level & 1];
        A.hdr = L.hdr;
        A.act_node = L.act_node;
        A.cprefix = L.cprefix;
        A.seg_start = c->seg_start;
        A.seg_len = c->seg_len;
        A.cdesc = L.cdesc;
    }
    const unsigned nodes = 1u << (level - 1);
    const int ngroups = (A.nfs + 3) / 4; // 4 waves per block, one sampled feature each
    dim3 grid(nodes, (unsigned)ngroups);
    const int bpl = (c->B + 63) / 64;
    // extra blocks per node that only clear the children's histogram slices, while a level has few nodes
    unsigned zero_blocks = 0;
    if (!leaf_level && A.zero_children && !A.oblivious && nodes < 64) zero_blocks = 64 / nodes < 16 ? 64 / nodes : 16;
    if (c->mc) { // any number of outputs: multi-class, several targets
        if (!leaf_level) {
            if (bpl == 1) hipLaunchKernelGGL((k_scan_mc<1>), grid, dim3(256), 0, c->stream, A);
            else if (bpl == 2) hipLaunchKernelGGL((k_scan_mc<2>), grid, dim3(256), 0, c->stream, A);
            else hipLaunchKernelGGL((k_scan_mc<4>), grid, dim3(256), 0, c->stream, A);
        }
        if (!A.oblivious || leaf_level) hipLaunchKernelGGL(k_scan_fin_mc, dim3(nodes), dim3(256), 0, c->stream, A, ngroups);
        HIPCHK(hipGetLastError());
        return EVT_OK;
    }
    // few sampled features: one block of 16 waves scans a node's features and finishes the node, no second launch
    const bool fused = !leaf_level && !A.oblivious && A.nfs <= 16 && c->scan_fused;
#define SCASE(NAG_)                                                                                     \
    case NAG_:                                                                                          \
        if (fused) {                                                                                    \
            if (bpl == 1) hipLaunchKernelGGL((k_scan<NAG_, 1, true>), dim3(nodes), dim3(1024), 0, c->stream, A);      \
            else if (bpl == 2) hipLaunchKernelGGL((k_scan<NAG_, 2, true>), dim3(nodes), dim3(1024), 0, c->stream, A); \
            else hipLaunchKernelGGL((k_scan<NAG_, 4, true>), dim3(nodes), dim3(1024), 0, c->stream, A);               \
            break;                                                                                      \
        }                                                                                               \
        if (!leaf_level) {                                                                              \
            if (bpl == 1) hipLaunchKernelGGL((k_scan<NAG_, 1, false>), grid, dim3(256), 0, c->stream, A);      \
            else if (bpl == 2) hipLaunchKernelGGL((k_scan<NAG_, 2, false>), grid, dim3(256), 0, c->stream, A); \
            else hipLaunchKernelGGL((k_scan<NAG_, 4, false>), grid, dim3(256), 0, c->stream, A);               \
        }                                                                                               \
        if (!A.oblivious || leaf_level) hipLaunchKernelGGL(k_scan_fin<NAG_>, dim3(nodes, 1 + zero_blocks), dim3(256), 0, c->stream, A, ngroups); \
        break;
    switch (c->NAg) {
        SCASE(2)
        SCASE(3)
        SCASE(5)
    default: evt_set_error("unsupported global channel count %d", c->NAg); return EVT_ERR_ARG;
    }
#undef SCASE
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

int launch_obliv_select(evt_ctx *c, int level, const evt_params *p) {
    const LevelTab &L = c->lvl[level & 1];
    OblivArgs A;
    A.hist = c->hist;
    A.node_stride = (int64_t)c->F * c->NAg * c->B;
    A.js = c->js;
    A.feattypes = c->feattypes;
    A.status = c->status;
    A.node_sum = c->node_sum;
    A.qscale = c->qscale;
    A.tree = c->tree;
    A.ogains = c->ogains;
    A.hdr = L.hdr;
    A.act_node = L.act_node;
    A.eta = p->eta; A.lambda = p->lambda; A.L2 = p->L2; A.gamma = p->gamma;
    A.bagging = p->bagging_size;
    A.nfs = c->n_js_last; A.B = c->B; A.K = c->K; A.NK = c->NK; A.NAg = c->NAg; A.loss = c->loss; A.level = level;
    A.zero_children = (level + 1 < c->D) ? 1 : 0;
    hipLaunchKernelGGL(k_obliv_select, dim3(1), dim3(1024), 0, c->stream, A);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}
