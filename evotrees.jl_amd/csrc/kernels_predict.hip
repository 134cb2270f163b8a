// Tree traversal: predict! (src/predict.jl:1-46), predict_leaf_idx! (:138-154), _predict (:118-136).
//
// A node is packed in one 32-bit word (feat | cond_bin << 16 | split << 24 | numeric << 25) so that each
// visited node costs one 4-byte load and nothing else has to be looked up.  Rows are independent; per row the
// walk reads one bin byte per level, from the column-major x_bin (neighbouring rows share 64-byte sectors of
// a column) or, in the whole-model kernel, from a copy of the block's rows in LDS.
#include "evt_internal.h"
#include <algorithm>

__device__ __forceinline__ int walk_packed(const uint32_t *__restrict__ nodes, const uint8_t *__restrict__ xcm, int64_t N, int64_t i) {
    int nid = 1;
    uint32_t nd = nodes[0];
    while (nd & EVT_NODE_SPLIT) {
        const int feat = (int)(nd & 0xFFFFu);
        const uint32_t cb = (nd >> 16) & 0xFFu;
        const uint32_t xb = xcm[(size_t)(feat - 1) * N + i];
        const bool cond = (nd & EVT_NODE_NUMERIC) ? (xb <= cb) : (xb == cb);
        nid = (nid << 1) + (cond ? 0 : 1);
        nd = nodes[nid - 1];
    }
    return nid;
}

// one tree added to pred (K x N), all rows.  copy_blocks extra blocks at the end of the grid carry copy_n 16-byte words
// from copy_src to copy_dst: the finished tree's way back to the host's pinned buffer, when this is the tree's last kernel.
// A row's walk is a chain of dependent loads (node word, bin byte, node word, ...), so the kernel is paced by latency, not by
// the bytes it moves: the first n_lds node words (the upper levels of the heap, all of it for depths up to 13) are copied to
// LDS, where a lookup costs a fraction of a trip to the caches, and a thread walks R rows side by side - R bin bytes are
// requested before the first is used.  Rows of a thread are 256 apart: the threads of a wavefront read neighbouring bytes.
template <int R>
__global__ __launch_bounds__(256) void k_predict_tree(const uint32_t *__restrict__ nodes, int n_lds, const float *__restrict__ leaf_pred,
                                                     const uint8_t *__restrict__ xcm, int64_t N, int K, int loss, float *pred,
                                                     const uint4 *__restrict__ copy_src, uint4 *__restrict__ copy_dst, int64_t copy_n,
                                                     int copy_blocks) {
    extern __shared__ uint32_t s_nodes[];
    const int64_t G = (int64_t)gridDim.x - copy_blocks;
    if ((int64_t)blockIdx.x >= G) {
        for (int64_t k = ((int64_t)blockIdx.x - G) * 256 + threadIdx.x; k < copy_n; k += (int64_t)copy_blocks * 256) copy_dst[k] = copy_src[k];
        return;
    }
    for (int k = threadIdx.x; k < n_lds; k += 256) s_nodes[k] = nodes[k];
    __syncthreads();
    const int64_t i0 = (int64_t)blockIdx.x * (256 * R) + threadIdx.x;
    int nid[R];
    uint32_t nd[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        nid[r] = 1;
        nd[r] = (i0 + 256 * r < N) ? s_nodes[0] : 0u; // a row past the end walks nothing
    }
    for (;;) {
        uint32_t xb[R];
        bool any = false;
#pragma unroll
        for (int r = 0; r < R; r++) {
            xb[r] = 0;
            if (nd[r] & EVT_NODE_SPLIT) {
                xb[r] = xcm[(size_t)((nd[r] & 0xFFFFu) - 1) * N + (i0 + 256 * r)];
                any = true;
            }
        }
        if (!any) break;
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (nd[r] & EVT_NODE_SPLIT) {
                const uint32_t cb = (nd[r] >> 16) & 0xFFu;
                const bool cond = (nd[r] & EVT_NODE_NUMERIC) ? (xb[r] <= cb) : (xb[r] == cb);
                nid[r] = (nid[r] << 1) + (cond ? 0 : 1);
                nd[r] = (nid[r] - 1 < n_lds) ? s_nodes[nid[r] - 1] : nodes[nid[r] - 1];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int64_t i = i0 + 256 * r;
        if (i < N) evt_add_leaf(pred + (size_t)K * i, leaf_pred + (size_t)K * (nid[r] - 1), K, loss);
    }
}

// rows per thread: four once the rows fill the device several times over, one for small inputs (more blocks)
static int launch_predict_tree_any(evt_ctx *c, const uint32_t *nodes, int nnodes, const float *leaf_pred, const uint4 *copy_src, uint4 *copy_dst,
                                   int64_t copy_n, int copy_blocks) {
    const int n_lds = nnodes < 8192 ? nnodes : 8192;
    const size_t lds = (size_t)n_lds * sizeof(uint32_t);
    if (c->N >= ((int64_t)1 << 21)) {
        hipLaunchKernelGGL(k_predict_tree<4>, dim3((unsigned)((c->N + 1023) / 1024) + (unsigned)copy_blocks), dim3(256), lds, c->stream, nodes, n_lds,
                           leaf_pred, c->xcm, c->N, c->K, c->loss, c->pred, copy_src, copy_dst, copy_n, copy_blocks);
    } else {
        hipLaunchKernelGGL(k_predict_tree<1>, dim3((unsigned)((c->N + 255) / 256) + (unsigned)copy_blocks), dim3(256), lds, c->stream, nodes, n_lds,
                           leaf_pred, c->xcm, c->N, c->K, c->loss, c->pred, copy_src, copy_dst, copy_n, copy_blocks);
    }
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// node each sampled row of the last tree ended in (0 outside the sample): the walk reproduces the
// partition's decisions row by row (update_nodes_idx!, ext/EvoTreesKernelAbstractionsExt/fit-utils.jl:9-31)
__global__ __launch_bounds__(256) void k_nidx_from_tree(const uint32_t *__restrict__ nodes, const uint8_t *__restrict__ xcm, int64_t N,
                                                       const uint8_t *__restrict__ mask, uint32_t cond, uint32_t *out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    uint32_t r = 0;
    if (!mask || mask[i] <= cond) r = (uint32_t)walk_packed(nodes, xcm, N, i);
    out[i] = r;
}

int launch_nidx_from_tree(evt_ctx *c, bool use_mask, uint8_t cond) {
    hipLaunchKernelGGL(k_nidx_from_tree, dim3((unsigned)((c->N + 255) / 256)), dim3(256), 0, c->stream, c->tree.packed, c->xcm, c->N,
                       use_mask ? c->mask : nullptr, (uint32_t)cond, c->nidx);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

int launch_predict_tree_cache(evt_ctx *c, bool send_blob) {
    const int64_t copy_n = send_blob ? (int64_t)(c->blob_bytes / 16) : 0;
    const int copy_blocks = (int)std::min<int64_t>(64, (copy_n + 255) / 256);
    const int r = launch_predict_tree_any(c, c->tree.packed, c->nnodes, c->tree.pred, reinterpret_cast<const uint4 *>(c->tree_blob),
                                          reinterpret_cast<uint4 *>(c->h_stage_dev), copy_n, copy_blocks);
    if (r != EVT_OK) return r;
    if (send_blob) c->step.blob_sent = true;
    return EVT_OK;
}

int launch_predict_tree_nodes(evt_ctx *c, const uint32_t *nodes_dev, int nnodes, const float *leaf_pred_dev) {
    return launch_predict_tree_any(c, nodes_dev, nnodes, leaf_pred_dev, static_cast<const uint4 *>(nullptr), static_cast<uint4 *>(nullptr), (int64_t)0, 0);
}

// apply_prediction_link!, src/predict.jl:105-116 (softmax!: :187-195)
template <int KMAX>
__device__ __forceinline__ void apply_link(float *acc, int K, int loss) {
    if (loss == EVT_LOSS_LOGLOSS) {
        for (int k = 0; k < K; k++) acc[k] = 1.0f / (1.0f + expf(-acc[k]));
    } else if (EVT_IS_MLE2P(loss)) {
        for (int k = 1; k < K; k += 2) acc[k] = fmaxf(acc[k], 0.0f) + log1pf(expf(-fabsf(acc[k])));
    } else if (loss == EVT_LOSS_MLOGLOSS) {
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
    } else if (loss >= EVT_LOSS_POISSON && loss <= EVT_LOSS_TWEEDIE) {
        for (int k = 0; k < K; k++) acc[k] = expf(acc[k]);
    }
}

// acc += leaf values of one tree, with the per-tree clamps of predict! (src/predict.jl:1-84)
template <int KMAX>
__device__ __forceinline__ void add_tree(float *acc, const float *lp, int K, int loss) {
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
        } else if (loss == EVT_LOSS_LOGLOSS) { // several targets: each clamped to [-15, 15]
#pragma unroll
            for (int k = 0; k < KMAX; k++) acc[k] = fminf(fmaxf(acc[k], -15.0f), 15.0f);
        } else if (EVT_IS_MLE2P(loss)) { // (location, raw scale) pairs: the scale outputs are floored at -15
#pragma unroll
            for (int k = 1; k < KMAX; k += 2) acc[k] = fmaxf(-15.0f, acc[k]);
        }
    }
}

// whole model: trees concatenated, tree t owns nodes [off[t], off[t+1]); the running prediction
// stays in registers and is written once.  The per-tree clamps are applied after every tree, as
// predict! does.  This variant gathers bin bytes from global memory: any tree size, any feature count.
template <int KMAX>
__global__ __launch_bounds__(256) void k_predict_model(const uint32_t *__restrict__ nodes, const float *__restrict__ leaf_pred,
                                                      const int64_t *__restrict__ off, int ntrees, const uint8_t *__restrict__ xcm, int64_t N,
                                                      int K, int loss, int link, float *out, const int32_t *__restrict__ skip_flag) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    if (skip_flag && *skip_flag) return; // the model was packed on the device and found invalid: nothing is walked
    float acc[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; k++) acc[k] = 0.0f;
    for (int t = 0; t < ntrees; t++) {
        const int64_t o = off[t];
        const int nid = walk_packed(nodes + o, xcm, N, i);
        add_tree<KMAX>(acc, leaf_pred + (size_t)K * (o + nid - 1), K, loss);
    }
    if (link) apply_link<KMAX>(acc, K, loss);
#pragma unroll
    for (int k = 0; k < KMAX; k++)
        if (k < K) out[(size_t)K * i + k] = acc[k];
}

// Whole model with the walk entirely in LDS, over trees the host has completed: every leaf above a tree's last
// level is replaced by a chain of nodes that always go left down to that level and carry its value there, so every
// row walks exactly depth - 1 levels of every tree.  No lane leaves the loop early, nothing is tested but the bin,
// and the leaf is found by position.  (Leaf indices of the original tree are what evt_predict_leaf_idx is for.)
//
// A block copies its RB rows into LDS once - the only pass over x_bin - laid out so that row r of a wavefront owns
// LDS bank r: word k of the row (features 4k .. 4k+3) sits at word (wave * S4 + k) * 64 + lane, so the 64 lanes read
// their bin bytes without bank conflicts whatever features their nodes test.  A tree's internal nodes sit in LDS too,
// double buffered (the next tree's words are requested before the walk and stored after it): a level costs two LDS
// reads and no trip to memory.  A node word is byte offset of the feature inside the row's words | cond_bin << 16 |
// numeric << 25.  The leaf values of a tree are requested after its walk and added after the next tree's, in order.
template <bool ALLNUM>
__device__ __forceinline__ uint32_t step_node(uint32_t nid, uint32_t nd, uint32_t xb) {
    const uint32_t cb = (nd >> 16) & 0xFFu;
    if (ALLNUM) return __builtin_amdgcn_alignbit(nid, cb - xb, 31); // (nid << 1) | (bin > cond_bin)
    const bool right = (nd & EVT_NODE_NUMERIC) ? (xb > cb) : (xb != cb);
    return 2 * nid + (right ? 1u : 0u);
}

struct ModelTree {
    int32_t node_off; // first internal node in the node array
    int32_t leaf_off; // first last-level value (K floats each) in the value array
    int32_t levels;   // depth - 1: levels walked
    int32_t n_int;    // internal nodes: 2^levels - 1
};

// NT trees are walked side by side (NT independent chains of LDS reads per lane hide each other's latency); groups of
// NT trees are double buffered.  PRE = words of the next group each thread carries across the walk (>= NT * max_int / RB).
template <int KMAX, int RB, int NT, int PRE, bool ALLNUM>
__global__ __launch_bounds__(RB) void k_predict_model_lds(const uint32_t *__restrict__ cnodes, const float *__restrict__ cleaf,
                                                         const ModelTree *__restrict__ meta, int ntrees, const uint8_t *__restrict__ xcm,
                                                         int64_t N, int F, int S4, int max_int, int K, int loss, int link, float *out) {
    extern __shared__ uint32_t smem[];
    uint32_t *T = smem;                                                        // [2][NT][max_int]
    uint8_t *R = reinterpret_cast<uint8_t *>(smem + 2 * (size_t)NT * max_int); // [RB / 64][S4][64] words
    const int tid = threadIdx.x;
    const int64_t i = (int64_t)blockIdx.x * RB + tid;
    const bool live = i < N;
    const int64_t ic = live ? i : N - 1;
    uint8_t *Rw = R + ((size_t)(tid >> 6) * S4 * 64 + (tid & 63)) * 4; // byte f of this row: Rw[(f >> 2) * 256 + (f & 3)]
    // a column at a time (RB consecutive bytes per request), 16 columns requested before the first is stored: the copy
    // costs F / 16 trips to memory, not F
    for (int f0 = 0; f0 < F; f0 += 16) {
        uint8_t v[16];
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const int f = f0 + j < F ? f0 + j : F - 1;
            v[j] = xcm[(size_t)f * N + ic];
        }
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const int f = f0 + j;
            if (f < F) Rw[(f >> 2) * 256 + (f & 3)] = v[j];
        }
    }
    const int ngroups = (ntrees + NT - 1) / NT;
    const int gw = NT * max_int; // words of one group's buffer
    // The host padded every tree to max_int words and the tree list to a whole number of groups (with trees of no
    // levels), so group g's LDS image is the plain run cnodes[g * gw, (g + 1) * gw) and meta has ngroups * NT entries.
    for (int w = tid; w < gw; w += RB) T[w] = cnodes[w];
    __syncthreads();
    float acc[KMAX], lpv[NT][KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; k++) {
        acc[k] = 0.0f;
#pragma unroll
        for (int j = 0; j < NT; j++) lpv[j][k] = 0.0f;
    }
    int nprev = 0; // trees whose values wait in lpv
    for (int g = 0; g < ngroups; g++) {
        const uint32_t *Tc = T + (size_t)(g & 1) * gw;
        uint32_t *Tn = T + (size_t)((g + 1) & 1) * gw;
        ModelTree m[NT];
#pragma unroll
        for (int j = 0; j < NT; j++) m[j] = meta[g * NT + j];
        // the next group's words: requested now, stored after the walk
        uint32_t pre[PRE];
        if (g + 1 < ngroups) {
            const uint32_t *src = cnodes + (size_t)(g + 1) * gw;
#pragma unroll
            for (int q = 0; q < PRE; q++) {
                const int w = q * RB + tid;
                pre[q] = src[w < gw ? w : 0];
            }
        }
        // heap index of the node reached (1-based; children of n are 2n and 2n + 1): the sign of cond_bin - bin is the
        // step to the right, shifted in with one v_alignbit when every feature is numeric
        uint32_t nid[NT];
#pragma unroll
        for (int j = 0; j < NT; j++) nid[j] = 1;
        bool same = true;
#pragma unroll
        for (int j = 1; j < NT; j++) same = same && (m[j].levels == m[0].levels);
        if (same) { // the usual case: NT chains advance level by level together
            for (int l = 0; l < m[0].levels; l++) {
                uint32_t nd[NT], xb[NT];
#pragma unroll
                for (int j = 0; j < NT; j++) nd[j] = Tc[j * max_int + nid[j] - 1];
#pragma unroll
                for (int j = 0; j < NT; j++) xb[j] = Rw[nd[j] & 0xFFFFu];
#pragma unroll
                for (int j = 0; j < NT; j++) nid[j] = step_node<ALLNUM>(nid[j], nd[j], xb[j]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < NT; j++) {
                for (int l = 0; l < m[j].levels; l++) {
                    const uint32_t nd = Tc[j * max_int + nid[j] - 1];
                    const uint32_t xb = Rw[nd & 0xFFFFu];
                    nid[j] = step_node<ALLNUM>(nid[j], nd, xb);
                }
            }
        }
        uint32_t pos[NT]; // position in the last level
#pragma unroll
        for (int j = 0; j < NT; j++) pos[j] = nid[j] - (1u << m[j].levels);
        // the previous group's values go in (tree order), then this group's are requested
#pragma unroll
        for (int j = 0; j < NT; j++)
            if (j < nprev) add_tree<KMAX>(acc, lpv[j], K, loss);
        nprev = ntrees - g * NT < NT ? ntrees - g * NT : NT;
#pragma unroll
        for (int j = 0; j < NT; j++) {
            const float *lp = cleaf + (size_t)K * (m[j].leaf_off + pos[j]);
            if (KMAX > 4 && (K & 3) == 0) { // rows of 4 values: 16-byte loads (the value array starts on an allocation boundary)
#pragma unroll
                for (int k = 0; k < KMAX; k += 4) {
                    if (k < K) {
                        const float4 v = *reinterpret_cast<const float4 *>(lp + k);
                        lpv[j][k] = v.x; lpv[j][k + 1] = v.y; lpv[j][k + 2] = v.z; lpv[j][k + 3] = v.w;
                    }
                }
            } else {
#pragma unroll
                for (int k = 0; k < KMAX; k++)
                    if (k < K) lpv[j][k] = lp[k];
            }
        }
        if (g + 1 < ngroups) {
#pragma unroll
            for (int q = 0; q < PRE; q++) {
                const int w = q * RB + tid;
                if (w < gw) Tn[w] = pre[q];
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < NT; j++)
        if (j < nprev) add_tree<KMAX>(acc, lpv[j], K, loss);
    if (link) apply_link<KMAX>(acc, K, loss);
    if (live) {
#pragma unroll
        for (int k = 0; k < KMAX; k++)
            if (k < K) out[(size_t)K * i + k] = acc[k];
    }
}

__global__ __launch_bounds__(256) void k_leaf_idx_model(const uint32_t *__restrict__ nodes, const int64_t *__restrict__ off, int ntrees,
                                                       const uint8_t *__restrict__ xcm, int64_t N, uint32_t *out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    for (int t = 0; t < ntrees; t++) out[(size_t)t * N + i] = (uint32_t)walk_packed(nodes + off[t], xcm, N, i);
}

template <int KMAX, int RB, int NT, int PRE, bool ALLNUM>
static int launch_model_lds(hipStream_t s, const uint32_t *cnodes, const float *cleaf, const void *meta, int ntrees, const uint8_t *xcm, int64_t N,
                            int F, int max_int, int K, int loss, int apply_link, float *out) {
    static EvtDevOnce once;
    const int dev = EvtDevOnce::current();
    if (once.pending(dev)) {
        HIPCHK(hipFuncSetAttribute(reinterpret_cast<const void *>(k_predict_model_lds<KMAX, RB, NT, PRE, ALLNUM>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        once.mark(dev);
    }
    const int S4 = (F + 3) >> 2;
    const size_t lds = (size_t)RB * S4 * 4 + 8 * (size_t)NT * max_int;
    hipLaunchKernelGGL((k_predict_model_lds<KMAX, RB, NT, PRE, ALLNUM>), dim3((unsigned)((N + RB - 1) / RB)), dim3(RB), lds, s, cnodes, cleaf,
                       static_cast<const ModelTree *>(meta), ntrees, xcm, N, F, S4, max_int, K, loss, apply_link, out);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// Launch shape of the LDS kernel for this model: 1 = 1024 rows per block, 4 trees side by side (one block per CU);
// 2 = 512 rows, 2 trees (two blocks per CU); 3 = 512 rows, 1 tree; 4 = 256 rows, 1 tree; 0 = does not apply.
// A row's running prediction and the leaf values of the trees walked side by side live in registers: up to 4 outputs
// take any shape, 5 - 8 outputs at most two trees side by side, 9 - 16 outputs one tree at a time.
int predict_lds_shape(int F, int max_int, int K, int hint) {
    if (K > EVT_MAX_K || F >= 1024 || max_int < 0) return 0;
    const size_t S = 4 * (size_t)((F + 3) >> 2), mi = (size_t)(max_int > 0 ? max_int : 1);
    const int first = K <= 4 ? 1 : (K <= 8 ? 2 : 3);
    const bool fits[5] = {false, 4 * mi <= 8 * 1024 && 1024 * S + 32 * mi <= 150 * 1024, 2 * mi <= 8 * 512 && 512 * S + 16 * mi <= 80 * 1024,
                          mi <= 8 * 512 && 512 * S + 8 * mi <= 80 * 1024, mi <= 16 * 256 && 256 * S + 8 * mi <= 80 * 1024};
    if (hint >= first && hint <= 4 && fits[hint]) return hint; // a sweep's choice, when the shape allows it
    for (int sh = first; sh <= 4; sh++)
        if (fits[sh]) return sh;
    return 0;
}

// Completed trees (see k_predict_model_lds): cnodes / cleaf / meta as the host prepared them.
int launch_predict_model_lds(hipStream_t s, const uint32_t *cnodes, const float *cleaf, const void *meta, int ntrees, const uint8_t *xcm, int64_t N,
                             int F, int max_int, int K, int loss, int apply_link, int all_numeric, int shape, float *out) {
    const int mi = max_int > 0 ? max_int : 1;
    shape = predict_lds_shape(F, max_int, K, shape);
#define EVT_PM(KM_, RB_, NT_, PRE_)                                                                                                          \
    return all_numeric ? launch_model_lds<KM_, RB_, NT_, PRE_, true>(s, cnodes, cleaf, meta, ntrees, xcm, N, F, mi, K, loss, apply_link, out) \
                       : launch_model_lds<KM_, RB_, NT_, PRE_, false>(s, cnodes, cleaf, meta, ntrees, xcm, N, F, mi, K, loss, apply_link, out)
    if (K <= 4) {
        if (shape == 1) { EVT_PM(4, 1024, 4, 8); }
        if (shape == 2) { EVT_PM(4, 512, 2, 8); }
        if (shape == 3) { EVT_PM(4, 512, 1, 8); }
        if (shape == 4) { EVT_PM(4, 256, 1, 16); }
    } else if (K <= 8) {
        if (shape == 2) { EVT_PM(8, 512, 2, 8); }
        if (shape == 3) { EVT_PM(8, 512, 1, 8); }
        if (shape == 4) { EVT_PM(8, 256, 1, 16); }
    } else {
        if (shape == 3) { EVT_PM(16, 512, 1, 8); }
        if (shape == 4) { EVT_PM(16, 256, 1, 16); }
    }
#undef EVT_PM
    evt_set_error("internal: model shape does not fit the LDS predict kernel");
    return EVT_ERR_ARG;
}

int launch_predict_model(hipStream_t s, const uint32_t *nodes, const float *leaf_pred, const int64_t *off, int ntrees, const uint8_t *xcm, int64_t N,
                         int K, int loss, int apply_link, float *out, const int32_t *skip_flag) {
    if (K <= 4)
        hipLaunchKernelGGL(k_predict_model<4>, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, s, nodes, leaf_pred, off, ntrees, xcm, N, K, loss,
                           apply_link, out, skip_flag);
    else
        hipLaunchKernelGGL(k_predict_model<EVT_MAX_K>, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, s, nodes, leaf_pred, off, ntrees, xcm, N, K,
                           loss, apply_link, out, skip_flag);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

int launch_leaf_idx_model(hipStream_t s, const uint32_t *nodes, const int64_t *off, int ntrees, const uint8_t *xcm, int64_t N, uint32_t *out) {
    hipLaunchKernelGGL(k_leaf_idx_model, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, s, nodes, off, ntrees, xcm, N, out);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}
