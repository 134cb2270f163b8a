// Gradient kernels: fused per-loss gradient + hessian rows, |max| reduction, fixed-point staging.
//
// Streaming work, HBM bound: per row the kernel reads pred (4K B), y (4 B) and the weight
// (4 B, last row of the gradient matrix) and writes 8K B.
//
// A tree grown on every row leaves its leaf values pending: growing recorded the leaf of each row and
// the addition to the prediction (predict!, src/predict.jl:1-46) happens here, in row order, as the
// first thing the next gradient pass does (4 B of node id read and 4K B written more per row) - or in
// k_apply_leaf when something else needs the predictions first.
#include "evt_internal.h"
#include <algorithm>

__device__ __forceinline__ float wave_max_f32(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

__device__ __forceinline__ float dev_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float dev_softplus(float x) { return fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x))); }

// mle2p_grad_hess, src/loss.jl:194-217: GaussianMLE (LOSS 2) and LogisticMLE (LOSS 7); raw is the unconstrained scale.
template <int LOSS>
__device__ __forceinline__ void mle2p_grad_hess(float loc, float raw, float y, float &g_loc, float &g_scale, float &h_loc, float &h_scale) {
    const float scale = dev_softplus(raw);
    const float dscale = dev_sigmoid(raw);
    const float ds = dscale / scale;
    if (LOSS == 2) {
        const float resid = loc - y;
        const float s2 = scale * scale;
        g_loc = resid / s2;
        g_scale = (1.0f - (resid * resid) / s2) * dscale / scale;
        h_loc = 1.0f / s2;
        h_scale = 2.0f * (ds * ds);
    } else {
        const float z = (y - loc) / scale;
        const float th = tanhf(z / 2.0f);
        g_loc = -th / scale;
        g_scale = (1.0f - z * th) * dscale / scale;
        h_loc = 1.0f / (3.0f * (scale * scale));
        h_scale = (3.14159274f * 3.14159274f + 3.0f) / 9.0f * (ds * ds); // oftype(scale, pi)^2
    }
}

// Raises the running maximum of gradient row k.  Same-address atomics from thousands of blocks queue up one behind the
// other (about 20 ns each - 40 us for the 2048 blocks of a gradient pass), so the maximum is kept in
// EVT_ABSMAX_STRIPES copies on different cache lines, a block raises the copy its index selects, and the one reader
// (the quantisation pass, k_quantize) takes the largest.  The value only grows while a pass runs: a block whose own maximum is already
// covered by what a device-scope load shows skips the atomic.
__device__ __forceinline__ void absmax_raise(uint32_t *absmax, int k, float m) {
    if (!(m > 0.0f)) return;
    uint32_t *p = absmax + (blockIdx.x % EVT_ABSMAX_STRIPES) * EVT_MC_MAX_NK + k;
    const uint32_t u = __float_as_uint(m);
    if (__hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < u) atomicMax(p, u);
}

// LOSS: 0 mse (src/loss.jl:52), 1 logloss (:54-57), 2 gaussian_mle (:194-203), 3 poisson (:59-62),
// 4 gamma (:64-67), 5 tweedie with rho = 1.5 (:69-76), 8 mae (:78), 9 cred_var / cred_std (:80-83).
// grad rows: [g_1..g_K, h_1..h_K, w]; every written value is multiplied by w (src/loss.jl:104-108, :223-233).
template <int LOSS>
__global__ __launch_bounds__(256) void k_grads(float *__restrict__ pred, const float *__restrict__ y, float *__restrict__ grad, int64_t N,
                                              uint32_t *absmax, const uint32_t *__restrict__ pend_nidx,
                                              const float *__restrict__ pend_leaf, int unit_w) {
    constexpr int K = (LOSS == 2 || LOSS == 7) ? 2 : 1;
    constexpr int NK = 2 * K + 1;
    float mx[2 * K];
#pragma unroll
    for (int k = 0; k < 2 * K; k++) mx[k] = 0.0f;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < N; i += (int64_t)gridDim.x * 256) {
        float out[2 * K];
        float *g = grad + (size_t)NK * i;
        const float w = unit_w ? 1.0f : g[NK - 1]; // unit weights: the weight row (all ones) is not read
        if (pend_nidx) evt_add_leaf(pred + (size_t)K * i, pend_leaf + (size_t)K * (pend_nidx[i] - 1), K, LOSS);
        if (LOSS == 0) {
            const float gg = 2.0f * (pred[i] - y[i]);
            out[0] = gg * w;
            out[1] = 2.0f * w;
        } else if (LOSS == 1) {
            const float s = dev_sigmoid(pred[i]);
            out[0] = (s - y[i]) * w;
            out[1] = (s * (1.0f - s)) * w;
        } else if (LOSS == 3) {
            const float e = expf(pred[i]);
            out[0] = (e - y[i]) * w;
            out[1] = e * w;
        } else if (LOSS == 4) {
            const float e = expf(pred[i]);
            out[0] = (2.0f * (1.0f - y[i] / e)) * w;
            out[1] = (2.0f * y[i] / e) * w;
        } else if (LOSS == 5) {
            const float e = expf(pred[i]);
            const float a = powf(e, 0.5f), b = powf(e, -0.5f);
            out[0] = (2.0f * (a - y[i] * b)) * w;
            out[1] = (2.0f * (0.5f * a - (-0.5f) * y[i] * b)) * w;
        } else if (LOSS == 8) { // mae (src/loss.jl:78): the residual, no second-order row
            out[0] = (y[i] - pred[i]) * w;
            out[1] = 0.0f * w;
        } else if (LOSS == 9) { // credibility losses (src/loss.jl:80-83): residual and its square
            const float d = y[i] - pred[i];
            out[0] = d * w;
            out[1] = (d * d) * w;
        } else {
            float g1, g2, h1, h2;
            mle2p_grad_hess<LOSS>(pred[2 * i], pred[2 * i + 1], y[i], g1, g2, h1, h2);
            out[0] = g1 * w;
            out[1] = g2 * w;
            out[2] = h1 * w;
            out[3] = h2 * w;
        }
#pragma unroll
        for (int k = 0; k < 2 * K; k++) {
            g[k] = out[k];
            mx[k] = fmaxf(mx[k], fabsf(out[k]));
        }
    }
    // per gradient row max |v| -> exponent bound of the fixed-point histogram.
    // One atomic per block and row: contended same-address atomics serialise in L2.
    __shared__ float s_m[4][2 * K];
#pragma unroll
    for (int k = 0; k < 2 * K; k++) {
        const float m = wave_max_f32(mx[k]);
        if ((threadIdx.x & 63) == 0) s_m[threadIdx.x >> 6][k] = m;
    }
    __syncthreads();
    if (threadIdx.x < 2 * K) {
        const int k = threadIdx.x;
        const float m = fmaxf(fmaxf(s_m[0][k], s_m[1][k]), fmaxf(s_m[2][k], s_m[3][k]));
        absmax_raise(absmax, k, m);
    }
}

// Several targets at once (y is T x N, one column per row of data; src/loss.jl:49-50, :100-111, :219-236): the same
// per-target expressions as k_grads with K = T outputs (2T for gaussian_mle, whose rows are
// [g_loc_1, g_scale_1, g_loc_2, ..., h_loc_1, h_scale_1, ..., w]).
template <int LOSS>
__device__ __forceinline__ void grad_hess_one(float pk, float yk, float &g, float &h) {
    if (LOSS == 0) {
        g = 2.0f * (pk - yk);
        h = 2.0f;
    } else if (LOSS == 1) {
        const float s = dev_sigmoid(pk);
        g = s - yk;
        h = s * (1.0f - s);
    } else if (LOSS == 3) {
        const float e = expf(pk);
        g = e - yk;
        h = e;
    } else if (LOSS == 4) {
        const float e = expf(pk);
        g = 2.0f * (1.0f - yk / e);
        h = 2.0f * yk / e;
    } else if (LOSS == 8) {
        g = yk - pk;
        h = 0.0f;
    } else if (LOSS == 9) {
        const float d = yk - pk;
        g = d;
        h = d * d;
    } else {
        const float e = expf(pk);
        const float a = powf(e, 0.5f), b = powf(e, -0.5f);
        g = 2.0f * (a - yk * b);
        h = 2.0f * (0.5f * a - (-0.5f) * yk * b);
    }
}

template <int LOSS>
__global__ __launch_bounds__(256) void k_grads_mt(float *__restrict__ pred, const float *__restrict__ y, float *__restrict__ grad, int64_t N,
                                                 int K, uint32_t *absmax, const uint32_t *__restrict__ pend_nidx,
                                                 const float *__restrict__ pend_leaf, int unit_w) {
    const int NK = 2 * K + 1;
    constexpr bool MLE2P = (LOSS == 2 || LOSS == 7);
    const int T = MLE2P ? K / 2 : K; // target columns
    __shared__ float s_m[4];
    float mx[2 * EVT_MAX_K];
#pragma unroll
    for (int k = 0; k < 2 * EVT_MAX_K; k++) mx[k] = 0.0f;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < N; i += (int64_t)gridDim.x * 256) {
        float *pr = pred + (size_t)K * i;
        float *g = grad + (size_t)NK * i;
        const float *yi = y + (size_t)T * i;
        const float w = unit_w ? 1.0f : g[NK - 1];
        if (pend_nidx) evt_add_leaf(pr, pend_leaf + (size_t)K * (pend_nidx[i] - 1), K, LOSS);
#pragma unroll
        for (int k = 0; k < EVT_MAX_K; k++) {
            if (k < K) {
                float gg, hh;
                if (MLE2P) {
                    // output k of pair t = k / 2: even = location, odd = raw scale
                    const int t = k >> 1;
                    float g1, g2, h1, h2;
                    mle2p_grad_hess<MLE2P ? LOSS : 2>(pr[2 * t], pr[2 * t + 1], yi[t], g1, g2, h1, h2);
                    gg = (((k & 1) == 0) ? g1 : g2) * w;
                    hh = (((k & 1) == 0) ? h1 : h2) * w;
                } else {
                    float g1, h1;
                    grad_hess_one<MLE2P ? 0 : LOSS>(pr[k], yi[k], g1, h1);
                    gg = g1 * w;
                    hh = h1 * w;
                }
                g[k] = gg;
                g[K + k] = hh;
                mx[k] = fmaxf(mx[k], fabsf(gg));
                mx[EVT_MAX_K + k] = fmaxf(mx[EVT_MAX_K + k], fabsf(hh));
            }
        }
    }
#pragma unroll
    for (int k = 0; k < 2 * EVT_MAX_K; k++) {
        const int kk = k < EVT_MAX_K ? k : k - EVT_MAX_K;
        if (kk < K) { // uniform
            const float m = wave_max_f32(mx[k]);
            __syncthreads();
            if ((threadIdx.x & 63) == 0) s_m[threadIdx.x >> 6] = m;
            __syncthreads();
            if (threadIdx.x == 0) {
                const float mm = fmaxf(fmaxf(s_m[0], s_m[1]), fmaxf(s_m[2], s_m[3]));
                const int row = k < EVT_MAX_K ? k : K + kk;
                absmax_raise(absmax, row, mm);
            }
        }
    }
}

// Multi-class log loss (src/loss.jl:93-98, :113-128): prob_k = exp(p_k) / sum_j exp(p_j); g_k = (prob_k - [y == k]) w,
// h_k = prob_k (1 - prob_k) w; y holds the 1-based class.  The row maxima are reduced one gradient row at a time.
__global__ __launch_bounds__(256) void k_grads_mlogloss(float *__restrict__ pred, const float *__restrict__ y, float *__restrict__ grad,
                                                       int64_t N, int K, uint32_t *absmax, const uint32_t *__restrict__ pend_nidx,
                                                       const float *__restrict__ pend_leaf, int unit_w) {
    const int NK = 2 * K + 1;
    __shared__ float s_m[4];
    float mx[2 * EVT_MAX_K];
#pragma unroll
    for (int k = 0; k < 2 * EVT_MAX_K; k++) mx[k] = 0.0f;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < N; i += (int64_t)gridDim.x * 256) {
        float *pr = pred + (size_t)K * i;
        float *g = grad + (size_t)NK * i;
        const float w = unit_w ? 1.0f : g[NK - 1]; // unit weights: the weight row (all ones) is not read
        const int cls = (int)y[i];
        if (pend_nidx) evt_add_leaf(pr, pend_leaf + (size_t)K * (pend_nidx[i] - 1), K, EVT_LOSS_MLOGLOSS);
        float e[EVT_MAX_K];
        float isum = 0.0f;
#pragma unroll
        for (int k = 0; k < EVT_MAX_K; k++) {
            if (k < K) {
                e[k] = expf(pr[k]);
                isum += e[k];
            }
        }
#pragma unroll
        for (int k = 0; k < EVT_MAX_K; k++) {
            if (k < K) {
                const float prob = e[k] / isum;
                const float gg = ((cls == k + 1) ? prob - 1.0f : prob) * w;
                const float hh = (prob * (1.0f - prob)) * w;
                g[k] = gg;
                g[K + k] = hh;
                mx[k] = fmaxf(mx[k], fabsf(gg));
                mx[EVT_MAX_K + k] = fmaxf(mx[EVT_MAX_K + k], fabsf(hh));
            }
        }
    }
#pragma unroll
    for (int k = 0; k < 2 * EVT_MAX_K; k++) {
        const int kk = k < EVT_MAX_K ? k : k - EVT_MAX_K;
        if (kk < K) { // uniform
            const float m = wave_max_f32(mx[k]);
            __syncthreads();
            if ((threadIdx.x & 63) == 0) s_m[threadIdx.x >> 6] = m;
            __syncthreads();
            if (threadIdx.x == 0) {
                const float mm = fmaxf(fmaxf(s_m[0], s_m[1]), fmaxf(s_m[2], s_m[3]));
                absmax_raise(absmax, k < EVT_MAX_K ? kk : K + kk, mm);
            }
        }
    }
}

// The quantile losses (src/loss.jl:85-91, :144-171): row k = (alpha or alpha - 1, a Float64) * w, row K + k = the raw
// residual (not weighted: the leaf pass takes its quantile).  multi: one target column and a level per output
// (multiquantile); otherwise one level and a target column per output (quantile).
__global__ __launch_bounds__(256) void k_grads_quantile(float *__restrict__ pred, const float *__restrict__ y, float *__restrict__ grad, int64_t N,
                                                       int K, int multi, const double *__restrict__ alphas, uint32_t *absmax,
                                                       const uint32_t *__restrict__ pend_nidx, const float *__restrict__ pend_leaf, int unit_w) {
    const int NK = 2 * K + 1;
    const int T = multi ? 1 : K;
    __shared__ float s_m[4];
    float mx[2 * EVT_MAX_K];
#pragma unroll
    for (int k = 0; k < 2 * EVT_MAX_K; k++) mx[k] = 0.0f;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < N; i += (int64_t)gridDim.x * 256) {
        float *pr = pred + (size_t)K * i;
        float *g = grad + (size_t)NK * i;
        const float *yi = y + (size_t)T * i;
        const float w = unit_w ? 1.0f : g[NK - 1];
        if (pend_nidx) evt_add_leaf(pr, pend_leaf + (size_t)K * (pend_nidx[i] - 1), K, EVT_LOSS_QUANTILE);
#pragma unroll
        for (int k = 0; k < EVT_MAX_K; k++) {
            if (k < K) {
                const double alpha = multi ? alphas[k] : alphas[0];
                const float diff = (multi ? yi[0] : yi[k]) - pr[k];
                const float gg = (float)((diff > 0.0f ? alpha : alpha - 1.0) * (double)w);
                g[k] = gg;
                g[K + k] = diff;
                mx[k] = fmaxf(mx[k], fabsf(gg));
                mx[EVT_MAX_K + k] = fmaxf(mx[EVT_MAX_K + k], fabsf(diff));
            }
        }
    }
#pragma unroll
    for (int k = 0; k < 2 * EVT_MAX_K; k++) {
        const int kk = k < EVT_MAX_K ? k : k - EVT_MAX_K;
        if (kk < K) { // uniform
            const float m = wave_max_f32(mx[k]);
            __syncthreads();
            if ((threadIdx.x & 63) == 0) s_m[threadIdx.x >> 6] = m;
            __syncthreads();
            if (threadIdx.x == 0) {
                const float mm = fmaxf(fmaxf(s_m[0], s_m[1]), fmaxf(s_m[2], s_m[3]));
                absmax_raise(absmax, k < EVT_MAX_K ? kk : K + kk, mm);
            }
        }
    }
}

// max |v| of every gradient row of an existing gradient matrix (injected gradients, weight row)
__global__ __launch_bounds__(256) void k_absmax(const float *__restrict__ grad, int64_t N, int NK, int k0, int k1, uint32_t *absmax) {
    // one gradient row at a time: any number of rows without per-thread arrays
    for (int k = k0; k < k1; k++) {
        float m = 0.0f;
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < N; i += (int64_t)gridDim.x * 256)
            m = fmaxf(m, fabsf(grad[(size_t)NK * i + k]));
        const float v = wave_max_f32(m);
        if ((threadIdx.x & 63) == 0) absmax_raise(absmax, k, v);
    }
}

// Quantisation tables of a gradient pass and the fixed-point words the histogram kernel adds, in one kernel.
// qexp[k] = ilogb(max |row k|) + 1 (0 for an all-zero row); qmul[k] = 2^(qbits - qexp) encodes, qscale decodes.  Every block
// derives the multipliers from the striped maxima itself (a few dozen cached loads: no kernel of its own in front of this one);
// block 0 also writes the tables for the readers that follow (split search, read-back).  The maxima live in two sets: a
// gradient pass raises one, this kernel reads it and clears the other - which nobody uses at that moment - for the next pass,
// so no pass starts from maxima an earlier one left behind.  The weight row (last) is written once and keeps its maximum.
// Plane a of gq holds, per row, q = rint(v * 2^(qbits - qexp)) of gradient row chan_k[a]; with unit weights plane 0 also carries
// the row count in its low 16 bits ((q << 16) + 1) so that one 64-bit LDS add serves both.
// Channel a reads gradient row a, except for mse whose channels are {g, w} = rows {0, 2}.
__global__ __launch_bounds__(256) void k_quantize(const float *__restrict__ grad, unsigned long long *__restrict__ gq, int64_t N,
                                                 int NK, int NA, int mse, int pack, const uint32_t *__restrict__ absmax, uint32_t *absmax_next,
                                                 const int32_t *__restrict__ qbits, int32_t *qexp, double *qmul, double *qscale_g, int NAg,
                                                 int loss, int unit_w) {
    __shared__ double s_qmul[EVT_MC_MAX_NK];
    __shared__ int s_qexp[EVT_MC_MAX_NK], s_qbits[EVT_MC_MAX_NK];
    const int t = threadIdx.x;
    if (t < NK) {
        uint32_t mu = 0u;
        for (int st = 0; st < EVT_ABSMAX_STRIPES; st++) {
            const uint32_t v = absmax[st * EVT_MC_MAX_NK + t]; // non-negative floats order as their bit patterns
            mu = v > mu ? v : mu;
        }
        const float m = __uint_as_float(mu);
        int e = 0;
        if (m > 0.0f) {
            e = ilogbf(m) + 1;
            if (e > 128) e = 128;
            if (e < -140) e = -140;
        }
        const int qb = qbits[t];
        s_qexp[t] = e;
        s_qbits[t] = qb;
        s_qmul[t] = scalbn(1.0, qb - e);
    }
    __syncthreads();
    if (blockIdx.x == 0) {
        if (t < NK) {
            qexp[t] = s_qexp[t];
            qmul[t] = s_qmul[t];
            if (t < NK - 1)
                for (int st = 0; st < EVT_ABSMAX_STRIPES; st++) absmax_next[st * EVT_MC_MAX_NK + t] = 0u;
        }
        if (t < NAg) {
            // global channel ag -> gradient row: mse {g, w}; otherwise identity; last channel is w (or the row count)
            const int kk = EVT_TWO_CHAN(loss, (NK - 1) / 2) ? (t == 0 ? 0 : 2) : t; // one-target mse / mae: channels {g, w}
            if (t == NAg - 1 && unit_w) qscale_g[t] = 1.0;
            else qscale_g[t] = scalbn(1.0, s_qexp[kk] - s_qbits[kk]);
        }
    }
    // a block takes many rows (grid-stride), so that the prologue above is paid a couple of thousand times, not once per 256 rows
    for (int64_t i = (int64_t)blockIdx.x * 256 + t; i < N; i += (int64_t)gridDim.x * 256) {
        const float *g = grad + (size_t)NK * i;
        for (int a = 0; a < NA; a++) {
            const int k = (mse && a == 1) ? 2 : a;
            long long q = __double2ll_rn((double)g[k] * s_qmul[k]);
            if (a == 0 && pack) { // 30 bits: staged as a 32-bit word, widened to (q << 16) + 1 (the row count) by the histogram kernel
                reinterpret_cast<int32_t *>(gq)[i] = (int32_t)q;
                continue;
            }
            gq[(size_t)a * N + i] = (unsigned long long)q;
        }
    }
}

// the set of striped maxima the next gradient pass raises (and the quantisation behind it reads)
static uint32_t *absmax_set(evt_ctx *c, int which) { return c->absmax + (size_t)which * EVT_ABSMAX_STRIPES * EVT_MC_MAX_NK; }

int launch_grads(evt_ctx *c) {
    // the maxima of the rows this kernel writes start from zero (cleared at creation and by the quantisation pass before last)
    uint32_t *const am = absmax_set(c, c->absmax_cur);
    int64_t nb = (c->N + 255) / 256;
    if (nb > 2048) nb = 2048;
    dim3 grid((unsigned)nb);
    const uint32_t *pn = c->pend_pred ? c->nidx : nullptr; // the last tree's leaf values are added on the way
    c->pend_pred = false;
    if (EVT_IS_QUANTILE(c->loss)) {
        hipLaunchKernelGGL(k_grads_quantile, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, c->K, c->loss == EVT_LOSS_MULTIQUANTILE ? 1 : 0,
                           c->alphas, am, pn, c->tree.pred, c->unit_w ? 1 : 0);
        HIPCHK(hipGetLastError());
        return EVT_OK;
    }
    const bool multi_target = c->loss != EVT_LOSS_MLOGLOSS && c->K > (EVT_IS_MLE2P(c->loss) ? 2 : 1);
    if (multi_target) {
#define MT(L_) hipLaunchKernelGGL(k_grads_mt<L_>, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, c->K, am, pn, c->tree.pred, c->unit_w ? 1 : 0)
        switch (c->loss) {
        case EVT_LOSS_MSE: MT(0); break;
        case EVT_LOSS_LOGLOSS: MT(1); break;
        case EVT_LOSS_GAUSSIAN_MLE: MT(2); break;
        case EVT_LOSS_POISSON: MT(3); break;
        case EVT_LOSS_GAMMA: MT(4); break;
        case EVT_LOSS_LOGISTIC_MLE: MT(7); break;
        case EVT_LOSS_MAE: MT(8); break;
        case EVT_LOSS_CRED_VAR:
        case EVT_LOSS_CRED_STD: MT(9); break;
        default: MT(5); break;
        }
#undef MT
        HIPCHK(hipGetLastError());
        return EVT_OK;
    }
    if (c->loss == EVT_LOSS_MSE)
        hipLaunchKernelGGL(k_grads<0>, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, am, pn, c->tree.pred, c->unit_w ? 1 : 0);
    else if (c->loss == EVT_LOSS_LOGLOSS)
        hipLaunchKernelGGL(k_grads<1>, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, am, pn, c->tree.pred, c->unit_w ? 1 : 0);
    else if (c->loss == EVT_LOSS_LOGISTIC_MLE)
        hipLaunchKernelGGL(k_grads<7>, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, am, pn, c->tree.pred, c->unit_w ? 1 : 0);
    else if (c->loss == EVT_LOSS_GAUSSIAN_MLE)
        hipLaunchKernelGGL(k_grads<2>, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, am, pn, c->tree.pred, c->unit_w ? 1 : 0);
    else if (c->loss == EVT_LOSS_POISSON)
        hipLaunchKernelGGL(k_grads<3>, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, am, pn, c->tree.pred, c->unit_w ? 1 : 0);
    else if (c->loss == EVT_LOSS_GAMMA)
        hipLaunchKernelGGL(k_grads<4>, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, am, pn, c->tree.pred, c->unit_w ? 1 : 0);
    else if (c->loss == EVT_LOSS_MAE)
        hipLaunchKernelGGL(k_grads<8>, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, am, pn, c->tree.pred, c->unit_w ? 1 : 0);
    else if (EVT_IS_CRED(c->loss))
        hipLaunchKernelGGL(k_grads<9>, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, am, pn, c->tree.pred, c->unit_w ? 1 : 0);
    else if (c->loss == EVT_LOSS_MLOGLOSS)
        hipLaunchKernelGGL(k_grads_mlogloss, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, c->K, am, pn, c->tree.pred, c->unit_w ? 1 : 0);
    else
        hipLaunchKernelGGL(k_grads<5>, grid, dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, am, pn, c->tree.pred, c->unit_w ? 1 : 0);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// Adds the pending leaf values of the last tree to the predictions, row by row.
__global__ __launch_bounds__(256) void k_apply_leaf(float *__restrict__ pred, const uint32_t *__restrict__ nidx,
                                                   const float *__restrict__ leaf, int64_t N, int K, int loss) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < N; i += (int64_t)gridDim.x * 256)
        evt_add_leaf(pred + (size_t)K * i, leaf + (size_t)K * (nidx[i] - 1), K, loss);
}

int launch_apply_pending(evt_ctx *c) {
    if (!c->pend_pred) return EVT_OK;
    int64_t nb = (c->N + 255) / 256;
    if (nb > 4096) nb = 4096;
    hipLaunchKernelGGL(k_apply_leaf, dim3((unsigned)nb), dim3(256), 0, c->stream, c->pred, c->nidx, c->tree.pred, c->N, c->K, c->loss);
    HIPCHK(hipGetLastError());
    c->pend_pred = false;
    return EVT_OK;
}

// Unit weights: the row count stands for the weight in every histogram, so a gradient matrix handed in from outside
// must carry ones in its weight row.  Flags the first kind of violation it sees.
__global__ __launch_bounds__(256) void k_check_unit_weight(const float *__restrict__ grad, int64_t N, int NK, int32_t *errflag) {
    bool bad = false;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < N; i += (int64_t)gridDim.x * 256) bad |= grad[(size_t)NK * i + NK - 1] != 1.0f;
    if (__ballot(bad) != 0ull && (threadIdx.x & 63) == 0) *errflag = 1;
}
int launch_check_unit_weight(evt_ctx *c) {
    int64_t nb = (c->N + 255) / 256;
    if (nb > 4096) nb = 4096;
    hipLaunchKernelGGL(k_check_unit_weight, dim3((unsigned)nb), dim3(256), 0, c->stream, c->grad, c->N, c->NK, c->errflag);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

__global__ void k_absmax_clear(uint32_t *absmax, int k0, int k1) {
    const int n = k1 - k0;
    for (int i = threadIdx.x; i < n * EVT_ABSMAX_STRIPES; i += blockDim.x) absmax[(i / n) * EVT_MC_MAX_NK + k0 + i % n] = 0u;
}

// absmax over rows [k0, k1) of the current gradient matrix, into the set the next quantisation reads; the weight row's
// maximum (row NK - 1) is kept in both sets, since no gradient pass renews it
int launch_absmax_rows(evt_ctx *c, int k0, int k1) {
    int64_t nb = (c->N + 255) / 256;
    if (nb > 2048) nb = 2048;
    for (int pass = 0; pass < 2; pass++) {
        uint32_t *am = absmax_set(c, pass == 0 ? c->absmax_cur : c->absmax_cur ^ 1);
        const int a0 = pass == 0 ? k0 : std::max(k0, c->NK - 1);
        if (a0 >= k1) continue;
        hipLaunchKernelGGL(k_absmax_clear, dim3(1), dim3(256), 0, c->stream, am, a0, k1);
        HIPCHK(hipGetLastError());
        hipLaunchKernelGGL(k_absmax, dim3((unsigned)nb), dim3(256), 0, c->stream, c->grad, c->N, c->NK, a0, k1, am);
        HIPCHK(hipGetLastError());
    }
    return EVT_OK;
}

int launch_quantize(evt_ctx *c) {
    // write the set of tables the last grown tree does not use: its histogram stays decodable
    c->q_cur = c->q_tree ^ 1;
    c->qexp = c->qexp_buf[c->q_cur];
    c->qscale = c->qscale_buf[c->q_cur];
    double *qmul = c->qscale + EVT_MC_MAX_NK; // decode scales per global channel first, then encode multipliers per gradient row
    hipLaunchKernelGGL(k_quantize, dim3((unsigned)std::min<int64_t>(4096, (c->N + 255) / 256)), dim3(256), 0, c->stream, c->grad, c->gq, c->N, c->NK, c->NA,
                       EVT_TWO_CHAN(c->loss, c->K) ? 1 : 0, c->unit_w ? 1 : 0, absmax_set(c, c->absmax_cur), absmax_set(c, c->absmax_cur ^ 1),
                       c->qbits, c->qexp, qmul, c->qscale, c->NAg, c->loss, c->unit_w ? 1 : 0);
    HIPCHK(hipGetLastError());
    c->absmax_cur ^= 1; // the next gradient pass raises the set this kernel cleared
    return EVT_OK;
}

// ---- evaluation metric ------------------------------------------------------------------------
// Per row value of src/metrics.jl:1-28 (:88-91 for gaussian_mle) in Float32, weighted as eval[i] = w * v / K
// (:43, :111), accumulated in Float64.  Two stages with a fixed shape (EVT_METRIC_BLOCKS partial sums, then one
// block) keep the summation order, hence the result, independent of scheduling.
__device__ __forceinline__ float metric_value_one(int metric, float pk, float yk);
// T: target columns of y (K, or 1 when every output is measured against the one target: _target(y::AbstractVector, k, i) = y[i],
// src/loss.jl:49).  alphas: the levels of the quantile metrics as Float32 (src/callback.jl:62-66).
__device__ __forceinline__ float metric_value(int metric, int K, int T, const float *__restrict__ pred, const float *__restrict__ y, int64_t i,
                                              const float *__restrict__ alphas) {
    if (metric == EVT_METRIC_QUANTILE || metric == EVT_METRIC_MULTIQUANTILE) { // src/metrics.jl:4-6, :83-84, :117-134
        float acc = 0.0f;
        for (int k = 0; k < K; k++) {
            const float pk = pred[(size_t)K * i + k], yk = y[(size_t)T * i + (T == 1 ? 0 : k)];
            const float alpha = (metric == EVT_METRIC_MULTIQUANTILE) ? alphas[k] : alphas[0];
            acc += alpha * fmaxf(yk - pk, 0.0f) + (1.0f - alpha) * fmaxf(pk - yk, 0.0f);
        }
        return acc;
    }
    if (metric == EVT_METRIC_MLOGLOSS) { // src/metrics.jl:59-77
        float isum = 0.0f;
        for (int k = 0; k < K; k++) isum += expf(pred[(size_t)K * i + k]);
        return logf(isum) - pred[(size_t)K * i + (int)y[i] - 1];
    }
    if (metric == EVT_METRIC_GAUSSIAN_MLE || metric == EVT_METRIC_LOGISTIC_MLE) { // src/metrics.jl:84-114: summed over the targets
        const int T = K / 2;
        float acc = 0.0f;
        for (int t = 0; t < T; t++) {
            const float loc = pred[(size_t)K * i + 2 * t], scale = dev_softplus(pred[(size_t)K * i + 2 * t + 1]);
            if (metric == EVT_METRIC_GAUSSIAN_MLE) {
                const float d = y[(size_t)T * i + t] - loc;
                acc += -(logf(scale) + (d * d) / (2.0f * (scale * scale)));
            } else {
                const float az = fabsf((y[(size_t)T * i + t] - loc) / scale);
                acc += -logf(scale) - az - 2.0f * log1pf(expf(-az));
            }
        }
        return acc;
    }
    float acc = 0.0f; // src/metrics.jl:39-43: the per-target values are added in Float32, starting from zero
    for (int k = 0; k < K; k++) acc += metric_value_one(metric, pred[(size_t)K * i + k], y[(size_t)T * i + (T == 1 ? 0 : k)]);
    return acc;
}

__device__ __forceinline__ float metric_value_one(int metric, float pk, float yk) {
    switch (metric) {
    case EVT_METRIC_MSE:
    case EVT_METRIC_RMSE: return (pk - yk) * (pk - yk);
    case EVT_METRIC_MAE: return fabsf(pk - yk);
    case EVT_METRIC_LOGLOSS: {
        const float s = dev_sigmoid(pk);
        return -yk * logf(s) + (yk - 1.0f) * logf(1.0f - s);
    }
    case EVT_METRIC_POISSON: {
        const float e = expf(pk);
        return 2.0f * (yk * logf(yk / e + 7.105427357601002e-15f) + e - yk); // eps(Float32(1e-7)) = 2^-47
    }
    case EVT_METRIC_GAMMA: {
        const float e = expf(pk);
        return 2.0f * (logf(e / yk) + yk / e - 1.0f);
    }
    default: {
        const float e = expf(pk);
        return 2.0f * (powf(yk, 0.5f) / (-0.5f) / 0.5f - yk * powf(e, -0.5f) / (-0.5f) + powf(e, 0.5f) / 0.5f);
    }
    }
}

__device__ __forceinline__ double block_sum_f64(double v, double *s_red) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (s_red[0] + s_red[1]) + (s_red[2] + s_red[3]);
}

__global__ __launch_bounds__(256) void k_metric_partial(const float *__restrict__ pred, const float *__restrict__ y,
                                                       const float *__restrict__ grad, int64_t N, int NK, int K, int T, int metric, float kdiv,
                                                       const float *__restrict__ alphas, double *__restrict__ partial) {
    __shared__ double s_red[4];
    double num = 0.0, den = 0.0;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < N; i += (int64_t)gridDim.x * 256) {
        const float w = grad[(size_t)NK * i + NK - 1];
        const float ev = w * metric_value(metric, K, T, pred, y, i, alphas) / kdiv;
        num += (double)ev;
        den += (double)w;
    }
    num = block_sum_f64(num, s_red);
    den = block_sum_f64(den, s_red);
    if (threadIdx.x == 0) {
        partial[2 * blockIdx.x] = num;
        partial[2 * blockIdx.x + 1] = den;
    }
}

__global__ __launch_bounds__(256) void k_metric_final(const double *__restrict__ partial, int nblocks, int metric, double *out) {
    __shared__ double s_red[4];
    double num = 0.0, den = 0.0;
    for (int b = threadIdx.x; b < nblocks; b += 256) {
        num += partial[2 * b];
        den += partial[2 * b + 1];
    }
    num = block_sum_f64(num, s_red);
    den = block_sum_f64(den, s_red);
    if (threadIdx.x == 0) {
        const double r = num / den;
        out[0] = (metric == EVT_METRIC_RMSE) ? sqrt(r) : r;
    }
}

// partial: 2 * EVT_METRIC_BLOCKS + 1 doubles; the metric lands in the last one
int launch_eval_metric(evt_ctx *c, int metric, double *partial) {
    int64_t nb = (c->N + 255) / 256;
    if (nb > EVT_METRIC_BLOCKS) nb = EVT_METRIC_BLOCKS;
    const float kdiv = (metric == EVT_METRIC_MLOGLOSS) ? 1.0f : (float)((metric == EVT_METRIC_GAUSSIAN_MLE || metric == EVT_METRIC_LOGISTIC_MLE) ? c->K / 2 : c->K);
    // y has K columns for the losses whose outputs each have a target; the multi-class, two-parameter and multiquantile
    // metrics index their own layouts
    const int T = (c->loss == EVT_LOSS_MULTIQUANTILE) ? 1 : c->K;
    hipLaunchKernelGGL(k_metric_partial, dim3((unsigned)nb), dim3(256), 0, c->stream, c->pred, c->y, c->grad, c->N, c->NK, c->K, T, metric, kdiv,
                       c->alphas_f, partial);
    HIPCHK(hipGetLastError());
    hipLaunchKernelGGL(k_metric_final, dim3(1), dim3(256), 0, c->stream, partial, (int)nb, metric, partial + 2 * EVT_METRIC_BLOCKS);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}
