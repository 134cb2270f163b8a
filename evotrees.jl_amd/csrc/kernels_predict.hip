// Tree traversal: predict! (src/predict.jl:1-46), predict_leaf_idx! (:138-154), _predict (:118-136).
//
// A node is packed in one 32-bit word (feat | cond_bin << 16 | split << 24) so that each visited
// node costs one cached 4-byte load.  Rows are independent; per row the walk reads one bin byte
// per level from the column-major x_bin (neighbouring rows share 64-byte sectors of a column).
#include "evt_internal.h"

__device__ __forceinline__ int walk_packed(const uint32_t *__restrict__ nodes, const uint8_t *__restrict__ xcm, int64_t N, int64_t i,
                                           const uint8_t *__restrict__ feattypes) {
    int nid = 1;
    uint32_t nd = nodes[0];
    while (nd >> 24) {
        const int feat = (int)(nd & 0xFFFFu);
        const uint32_t cb = (nd >> 16) & 0xFFu;
        const uint32_t xb = xcm[(size_t)(feat - 1) * N + i];
        const bool cond = feattypes[feat - 1] ? (xb <= cb) : (xb == cb);
        nid = (nid << 1) + (cond ? 0 : 1);
        nd = nodes[nid - 1];
    }
    return nid;
}

// one tree added to pred (K x N), all rows
__global__ __launch_bounds__(256) void k_predict_tree(const uint32_t *__restrict__ nodes, const float *__restrict__ leaf_pred,
                                                     const uint8_t *__restrict__ xcm, const uint8_t *__restrict__ feattypes, int64_t N,
                                                     int K, int loss, float *pred) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    const int nid = walk_packed(nodes, xcm, N, i, feattypes);
    evt_add_leaf(pred + (size_t)K * i, leaf_pred + (size_t)K * (nid - 1), K, loss);
}

// node each sampled row of the last tree ended in (0 outside the sample): the walk reproduces the
// partition's decisions row by row (update_nodes_idx!, ext/EvoTreesKernelAbstractionsExt/fit-utils.jl:9-31)
__global__ __launch_bounds__(256) void k_nidx_from_tree(const uint32_t *__restrict__ nodes, const uint8_t *__restrict__ xcm,
                                                       const uint8_t *__restrict__ feattypes, int64_t N, const uint8_t *__restrict__ mask,
                                                       uint32_t cond, uint32_t *out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    uint32_t r = 0;
    if (!mask || mask[i] <= cond) r = (uint32_t)walk_packed(nodes, xcm, N, i, feattypes);
    out[i] = r;
}

int launch_nidx_from_tree(evt_ctx *c, bool use_mask, uint8_t cond) {
    hipLaunchKernelGGL(k_nidx_from_tree, dim3((unsigned)((c->N + 255) / 256)), dim3(256), 0, c->stream, c->tree.packed, c->xcm, c->feattypes,
                       c->N, use_mask ? c->mask : nullptr, (uint32_t)cond, c->nidx);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

int launch_predict_tree_cache(evt_ctx *c) {
    hipLaunchKernelGGL(k_predict_tree, dim3((unsigned)((c->N + 255) / 256)), dim3(256), 0, c->stream, c->tree.packed, c->tree.pred, c->xcm,
                       c->feattypes, c->N, c->K, c->loss, c->pred);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

int launch_predict_tree_nodes(evt_ctx *c, const uint32_t *nodes_dev, const float *leaf_pred_dev) {
    hipLaunchKernelGGL(k_predict_tree, dim3((unsigned)((c->N + 255) / 256)), dim3(256), 0, c->stream, nodes_dev, leaf_pred_dev, c->xcm,
                       c->feattypes, c->N, c->K, c->loss, c->pred);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// whole model: trees concatenated, tree t owns nodes [off[t], off[t+1]); the running prediction
// stays in registers and is written once.  The per-tree clamps are applied after every tree, as
// predict! does.
template <int KMAX>
__global__ __launch_bounds__(256) void k_predict_model(const uint32_t *__restrict__ nodes, const float *__restrict__ leaf_pred,
                                                      const int64_t *__restrict__ off, int ntrees, const uint8_t *__restrict__ xcm,
                                                      const uint8_t *__restrict__ feattypes, int64_t N, int K, int loss, int apply_link,
                                                      float *out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    float acc[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; k++) acc[k] = 0.0f;
    for (int t = 0; t < ntrees; t++) {
        const int64_t o = off[t];
        const int nid = walk_packed(nodes + o, xcm, N, i, feattypes);
        const float *lp = leaf_pred + (size_t)K * (o + nid - 1);
        if (KMAX <= 4) {
            evt_add_leaf(acc, lp, K, loss);
        } else { // many outputs: constant trip counts keep the running prediction in registers
            float m = -INFINITY;
#pragma unroll
            for (int k = 0; k < KMAX; k++) {
                if (k < K) {
                    acc[k] += lp[k];
                    m = fmaxf(m, acc[k]);
                }
            }
            if (loss == EVT_LOSS_MLOGLOSS) {
#pragma unroll
                for (int k = 0; k < KMAX; k++) acc[k] = fmaxf(-15.0f, acc[k] - m);
            }
        }
    }
    if (apply_link) { // apply_prediction_link!, src/predict.jl:105-116
        if (loss == EVT_LOSS_LOGLOSS) {
            for (int k = 0; k < K; k++) acc[k] = 1.0f / (1.0f + expf(-acc[k]));
        } else if (loss == EVT_LOSS_GAUSSIAN_MLE) {
            for (int k = 1; k < K; k += 2) acc[k] = fmaxf(acc[k], 0.0f) + log1pf(expf(-fabsf(acc[k])));
        } else if (loss == EVT_LOSS_MLOGLOSS) { // softmax!, src/predict.jl:187-195
            float isum = 0.0f;
#pragma unroll
            for (int k = 0; k < KMAX; k++) {
                if (k < K) {
                    acc[k] = expf(acc[k]);
                    isum += acc[k];
                }
            }
#pragma unroll
            for (int k = 0; k < KMAX; k++) acc[k] /= isum;
        } else if (loss >= EVT_LOSS_POISSON) {
            for (int k = 0; k < K; k++) acc[k] = expf(acc[k]);
        }
    }
#pragma unroll
    for (int k = 0; k < KMAX; k++)
        if (k < K) out[(size_t)K * i + k] = acc[k];
}

__global__ __launch_bounds__(256) void k_leaf_idx_model(const uint32_t *__restrict__ nodes, const int64_t *__restrict__ off, int ntrees,
                                                       const uint8_t *__restrict__ xcm, const uint8_t *__restrict__ feattypes, int64_t N,
                                                       uint32_t *out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    for (int t = 0; t < ntrees; t++) out[(size_t)t * N + i] = (uint32_t)walk_packed(nodes + off[t], xcm, N, i, feattypes);
}

int launch_predict_model(hipStream_t s, const uint32_t *nodes, const float *leaf_pred, const int64_t *off, int ntrees, const uint8_t *xcm,
                         const uint8_t *feattypes, int64_t N, int K, int loss, int apply_link, float *out) {
    if (K <= 4)
        hipLaunchKernelGGL(k_predict_model<4>, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, s, nodes, leaf_pred, off, ntrees, xcm, feattypes, N,
                           K, loss, apply_link, out);
    else
        hipLaunchKernelGGL(k_predict_model<EVT_MAX_K>, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, s, nodes, leaf_pred, off, ntrees, xcm,
                           feattypes, N, K, loss, apply_link, out);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

int launch_leaf_idx_model(hipStream_t s, const uint32_t *nodes, const int64_t *off, int ntrees, const uint8_t *xcm, const uint8_t *feattypes,
                          int64_t N, uint32_t *out) {
    hipLaunchKernelGGL(k_leaf_idx_model, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, s, nodes, off, ntrees, xcm, feattypes, N, out);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}
