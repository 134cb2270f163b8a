/*
 * CPU oracle for the EvoTrees.jl tree-building hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the algorithm of the
 * reference's CPU path so that the HIP library can be checked against it on identical
 * inputs.  It is never linked into, loaded by or called from the product library;
 * only tests, the smoke check and the benchmark's cpu_baseline leg use it.
 *
 * Every function names the reference file:line it follows (paths relative to the
 * EvoTrees.jl source tree).
 *
 * Two accumulation modes are provided for the histogram / node sums:
 *   mode 0  "f64"   : the reference arithmetic.  Float32 gradients are added, in row
 *                     order, into Float64 bins (src/fit-utils.jl:367-394, src/init.jl:204).
 *   mode 1  "fixed" : the same algorithm with every gradient first rounded to a
 *                     fixed-point integer q = rint(g * 2^(qbits-e)) (e = exponent bound of
 *                     the row of the gradient matrix) and all sums done in int64.  Sums are then
 *                     exact and order independent, which is what lets a parallel
 *                     device implementation be compared bit for bit.  It specifies
 *                     the arithmetic of the device's deterministic histogram mode.
 *
 * Parity status: pinned by tests/test_oracle_pins.py (brute-force dense histograms,
 * brute-force split search over all (feature, bin) pairs, closed-form gain for unit weights,
 * closed-form / finite-difference gradients, independent tree walk, stable
 * partition property, leaf-value closed form, tie and min_weight strictness cases; matrix
 * targets by reduction to the one-target gradients and metrics, bit for bit, and by the brute-force
 * search on multi-output gradients; binarize by numpy's searchsorted and hand-worked answers
 * for NaN, signed zeros and infinities under Julia's isless).
 * Not pinned (needs a Julia run; stays host-side by design): exact quantile edges
 * from StatsBase.sample + Statistics.quantile, the Xoshiro row-mask / column-sample
 * streams, and Julia's pairwise Float32 mean/std for the bias.  -> "parity unpinned"
 * for those three host-side inputs; the oracle and the device library both receive
 * their outputs as inputs.
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_LOGISTIC_MLE 7
#define ORC_IS_MLE2P(l) ((l) == ORC_GAUSSIAN_MLE || (l) == ORC_LOGISTIC_MLE)
#define ORC_MSE 0
#define ORC_LOGLOSS 1
#define ORC_GAUSSIAN_MLE 2
#define ORC_POISSON 3
#define ORC_GAMMA 4
#define ORC_TWEEDIE 5
#define ORC_MLOGLOSS 6
#define ORC_MAE 8
#define ORC_CRED_VAR 9
#define ORC_CRED_STD 10
#define ORC_IS_CRED(l) ((l) == ORC_CRED_VAR || (l) == ORC_CRED_STD)
#define ORC_QUANTILE 11
#define ORC_MULTIQUANTILE 12
#define ORC_IS_QUANTILE(l) ((l) == ORC_QUANTILE || (l) == ORC_MULTIQUANTILE)
#define ORC_IS_SHIFT(l) ((l) == ORC_MAE || ORC_IS_QUANTILE(l)) /* gains of Union{MAE,Quantile}, src/split.jl:68, :119 */
#define ORC_MAX_NK 40 /* 2K+1 with up to 16 classes, rounded up */

typedef struct {
    int32_t loss;         /* ORC_MSE / ORC_LOGLOSS / ORC_GAUSSIAN_MLE                      */
    int32_t K;            /* outputs per row (1, or 2 for gaussian_mle)                    */
    int32_t nbins;        /* params.nbins: second dim of the histogram (src/init.jl:203)   */
    int32_t max_depth;    /* tree arrays have 2^max_depth - 1 entries                      */
    int32_t tree_type;    /* 0 binary (grow_tree!), 1 oblivious (grow_otree!)              */
    int32_t bagging_size; /* divides the leaf value (src/predict.jl:202)                   */
    double eta, L2, lambda, gamma, min_weight;
    int32_t n_alphas;     /* 1: params.alpha (quantile); K: params.alphas (multiquantile)  */
    double alphas[16];
} orc_params;

typedef struct {
    orc_params p;
    int64_t N;
    int32_t F;
    int32_t NK;     /* 2K+1 */
    int32_t nnodes; /* 2^max_depth - 1 */
    uint8_t *x_bin;   /* N x F column-major, values 1..nbins (src/fit-utils.jl:66-72)      */
    uint8_t *x_bin_T; /* F x N: row i's features contiguous (src/init.jl:155)              */
    uint8_t *feattypes; /* 1 numeric (<=), 0 categorical (==)                              */
    int32_t *mono;      /* monotone constraint per feature (-1, 0, 1)                      */
    double *h;          /* NK x B x F x nnodes, k fastest (src/init.jl:204)                */
    int64_t *hq;        /* same shape, fixed-point mode                                    */
    double *gains;      /* B x F x nnodes (TrainNode.gains, oblivious trees only)          */
    uint32_t *is, *left, *right; /* row-id work buffers (0-based ids), src/init.jl:178-180 */
    int64_t *seg_off, *seg_len;  /* per node view into `is`                                */
    double *sum;   /* NK per node : TrainNode.∑                                            */
    int64_t *sumq; /* NK per node, fixed mode                                              */
    int32_t qbits[ORC_MAX_NK];
    int32_t qexp[ORC_MAX_NK];
    int nthreads;
} orc_cache;

/* ------------------------------------------------------------------------------------ */
/* scalar helpers: src/loss.jl:249-260                                                   */
static inline float orc_sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }
static inline float orc_softplusf(float x) {
    float ax = fabsf(x);
    return fmaxf(x, 0.0f) + log1pf(expf(-ax));
}

/*
 * update_grads!  — src/loss.jl:100-111 (GradientRegression: mse :52, logloss :54-57) and
 * src/loss.jl:219-236 with mle2p_grad_hess(GaussianMLE) :194-203.
 * grad is (2K+1) x N Float32, k fastest; row 2K+1 holds the weight and is only read.
 * pred is K x N.  y has one value per row and target (T x N: T = K targets, K / 2 for gaussian_mle; the class for mlogloss).
 */
void orc_update_grads(const orc_params *p, int64_t N, const float *pred, const float *y, float *grad) {
    const int K = p->K, NK = 2 * K + 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < N; i++) {
        float w = grad[(int64_t)NK * i + NK - 1];
        float *g = grad + (int64_t)NK * i;
        if (p->loss == ORC_MLOGLOSS) { /* src/loss.jl:93-98, :113-128; y holds the 1-based class */
            const float *pr = pred + (int64_t)K * i;
            float isum = 0.0f;
            for (int k = 0; k < K; k++) isum += expf(pr[k]);
            for (int k = 0; k < K; k++) {
                float prob = expf(pr[k]) / isum;
                float gg = ((int)y[i] == k + 1) ? prob - 1.0f : prob;
                g[k] = gg * w;
                g[K + k] = (prob * (1.0f - prob)) * w;
            }
            continue;
        }
        if (ORC_IS_MLE2P(p->loss)) { /* K = 2 x targets; rows [g_loc_1, g_scale_1, g_loc_2, ..., h_loc_1, h_scale_1, ..., w] */
            const int Y = K / 2;
            for (int t = 0; t < Y; t++) {
                int gb = 2 * t, hb = 2 * Y + 2 * t; /* src/loss.jl:224-225 */
                float loc = pred[(int64_t)K * i + 2 * t], raw = pred[(int64_t)K * i + 2 * t + 1];
                float scale = orc_softplusf(raw);
                float dscale = orc_sigmoidf(raw);
                float ds = dscale / scale;
                float g_loc, g_scale, h_loc, h_scale;
                if (p->loss == ORC_GAUSSIAN_MLE) { /* src/loss.jl:194-203 */
                    float resid = loc - y[(int64_t)Y * i + t];
                    float s2 = scale * scale;
                    g_loc = resid / s2;
                    g_scale = (1.0f - (resid * resid) / s2) * dscale / scale;
                    h_loc = 1.0f / s2;
                    h_scale = 2.0f * (ds * ds);
                } else { /* Logistic(loc, scale), src/loss.jl:205-217 */
                    float z = (y[(int64_t)Y * i + t] - loc) / scale;
                    float th = tanhf(z / 2.0f);
                    const float pi32 = 3.14159274f;
                    g_loc = -th / scale;
                    g_scale = (1.0f - z * th) * dscale / scale;
                    h_loc = 1.0f / (3.0f * (scale * scale));
                    h_scale = (pi32 * pi32 + 3.0f) / 9.0f * (ds * ds);
                }
                g[gb] = g_loc * w;
                g[gb + 1] = g_scale * w;
                g[hb] = h_loc * w;
                g[hb + 1] = h_scale * w;
            }
            continue;
        }
        for (int k = 0; k < K; k++) { /* one column of y per target: _target(y, k, i), src/loss.jl:49-50 */
            float pk = pred[(int64_t)K * i + k], yk = y[(int64_t)K * i + k];
            float gg, hh;
            if (p->loss == ORC_MSE) {
                gg = 2.0f * (pk - yk);
                hh = 2.0f;
            } else if (p->loss == ORC_LOGLOSS) {
                float s = orc_sigmoidf(pk);
                gg = s - yk;
                hh = s * (1.0f - s);
            } else if (p->loss == ORC_POISSON) { /* src/loss.jl:59-62 */
                float e = expf(pk);
                gg = e - yk;
                hh = e;
            } else if (p->loss == ORC_GAMMA) { /* src/loss.jl:64-67 */
                float e = expf(pk);
                gg = 2.0f * (1.0f - yk / e);
                hh = 2.0f * yk / e;
            } else if (ORC_IS_QUANTILE(p->loss)) {
                /* quantile_grad_diff, src/loss.jl:85-91; update_grads! :144-156 (quantile: one alpha, a target column per
                 * output) and :158-171 (multiquantile: one target, an alpha per output).  The first row is alpha or
                 * alpha - 1 (Float64) times the weight, the second the raw residual, NOT weighted. */
                const int mq = (p->loss == ORC_MULTIQUANTILE);
                const double alpha = mq ? p->alphas[k] : p->alphas[0];
                if (mq) yk = y[i];
                const float diff = yk - pk;
                g[k] = (float)((diff > 0.0f ? alpha : alpha - 1.0) * (double)w);
                g[K + k] = diff;
                continue;
            } else if (p->loss == ORC_MAE) { /* mae_grad_hess, src/loss.jl:78 (update_grads! :130-142) */
                gg = yk - pk;
                hh = 0.0f;
            } else if (ORC_IS_CRED(p->loss)) { /* cred_grad_hess, src/loss.jl:80-83 (update_grads! :173-185) */
                float d = yk - pk;
                gg = d;
                hh = d * d;
            } else { /* tweedie, src/loss.jl:69-76, rho = 1.5 */
                float e = expf(pk);
                float a = powf(e, 0.5f), b = powf(e, -0.5f);
                gg = 2.0f * (a - yk * b);
                hh = 2.0f * (0.5f * a - (-0.5f) * yk * b);
            }
            g[k] = gg * w;
            g[K + k] = hh * w;
        }
    }
}

/* Julia's isless on Float64, the order searchsortedfirst uses by default: IEEE `<`, except that NaN sorts after
 * everything (Inf included) and -0.0 before 0.0. */
static inline int jl_isless(double a, double b) {
    if (isnan(a)) return 0;
    if (isnan(b)) return 1;
    if (a == 0.0 && b == 0.0) return signbit(a) && !signbit(b);
    return a < b;
}

/* binarize — src/fit-utils.jl:66-72: searchsortedfirst(edges, x) = 1 + #(edges isless x); a NaN lands in the last bin. */
void orc_binarize(int64_t N, const double *x, const double *edges, int32_t nedges, uint8_t *out) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < N; i++) {
        double v = x[i];
        int lo = 0, hi = nedges; /* first index with edges[idx] >= v */
        while (lo < hi) {
            int mid = (lo + hi) >> 1;
            if (jl_isless(edges[mid], v)) lo = mid + 1; else hi = mid;
        }
        out[i] = (uint8_t)(lo + 1);
    }
}

/* subsample — src/subsample.jl:6-38: keep mask[i] <= cond, ascending; returns count. */
int64_t orc_subsample(int64_t N, const uint8_t *mask, uint8_t cond, uint32_t *is_out) {
    int64_t c = 0;
    for (int64_t i = 0; i < N; i++)
        if (mask[i] <= cond) is_out[c++] = (uint32_t)i;
    return c;
}

/* ------------------------------------------------------------------------------------ */
orc_cache *orc_create(const orc_params *p, int64_t N, int32_t F, const uint8_t *x_bin_colmajor,
                      const uint8_t *feattypes, const int32_t *mono, int with_fixed) {
    orc_cache *c = (orc_cache *)calloc(1, sizeof(orc_cache));
    c->p = *p;
    c->N = N;
    c->F = F;
    c->NK = 2 * p->K + 1;
    c->nnodes = (1 << p->max_depth) - 1;
    c->x_bin = (uint8_t *)malloc((size_t)N * F);
    memcpy(c->x_bin, x_bin_colmajor, (size_t)N * F);
    c->x_bin_T = (uint8_t *)malloc((size_t)N * F);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < N; i++)
        for (int j = 0; j < F; j++) c->x_bin_T[(size_t)i * F + j] = x_bin_colmajor[(size_t)j * N + i];
    c->feattypes = (uint8_t *)malloc(F);
    c->mono = (int32_t *)calloc(F, sizeof(int32_t));
    for (int j = 0; j < F; j++) {
        c->feattypes[j] = feattypes ? feattypes[j] : 1;
        c->mono[j] = mono ? mono[j] : 0;
    }
    size_t hsz = (size_t)c->NK * p->nbins * F * c->nnodes;
    c->h = (double *)calloc(hsz, sizeof(double));
    c->hq = with_fixed ? (int64_t *)calloc(hsz, sizeof(int64_t)) : NULL;
    c->gains = p->tree_type == 1 ? (double *)calloc((size_t)p->nbins * F * c->nnodes, sizeof(double)) : NULL;
    c->is = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)N);
    c->left = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)N);
    c->right = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)N);
    c->seg_off = (int64_t *)calloc(c->nnodes + 2, sizeof(int64_t));
    c->seg_len = (int64_t *)calloc(c->nnodes + 2, sizeof(int64_t));
    c->sum = (double *)calloc((size_t)(c->nnodes + 2) * c->NK, sizeof(double));
    c->sumq = (int64_t *)calloc((size_t)(c->nnodes + 2) * c->NK, sizeof(int64_t));
#ifdef _OPENMP
    c->nthreads = omp_get_max_threads();
#else
    c->nthreads = 1;
#endif
    return c;
}

void orc_destroy(orc_cache *c) {
    if (!c) return;
    free(c->x_bin); free(c->x_bin_T); free(c->feattypes); free(c->mono);
    free(c->h); free(c->hq); free(c->gains);
    free(c->is); free(c->left); free(c->right);
    free(c->seg_off); free(c->seg_len); free(c->sum); free(c->sumq);
    free(c);
}

int orc_num_threads(const orc_cache *c) { return c->nthreads; }
double *orc_hist_ptr(orc_cache *c) { return c->h; }
int64_t *orc_histq_ptr(orc_cache *c) { return c->hq; }

/* histogram index helper: h[k, bin, j, n] with k fastest (all 0-based here; node n is 1-based id - 1) */
static inline size_t hidx(const orc_cache *c, int k, int b, int j, int n) {
    return (size_t)k + (size_t)c->NK * ((size_t)b + (size_t)c->p.nbins * ((size_t)j + (size_t)c->F * (size_t)n));
}

/* Fixed-point rule shared with the device library: value v of gradient row k is
 * represented by q = llrint((double)v * 2^(qbits[k] - qexp[k])) (round to nearest even),
 * where 2^qexp[k] strictly bounds |v| over ALL N rows of that gradient row
 * (qexp = ilogb(max|v|) + 1, or 0 when the row is all zero).  decode(q) = q * 2^(qexp - qbits). */
static inline int64_t orc_quant(float v, int qb, int qe) { return llrint(ldexp((double)v, qb - qe)); }
static inline double orc_decode(int64_t q, int qb, int qe) { return ldexp((double)q, qe - qb); }

/* Computes qexp for each gradient row over all N rows; qbits are supplied by the caller. */
void orc_set_quant(orc_cache *c, const float *grad, const int32_t *qbits) {
    const int NK = c->NK;
    for (int k = 0; k < NK; k++) {
        float m = 0.0f;
        for (int64_t i = 0; i < c->N; i++) {
            float a = fabsf(grad[(int64_t)NK * i + k]);
            if (a > m) m = a;
        }
        c->qbits[k] = qbits[k];
        c->qexp[k] = (m > 0.0f) ? (ilogbf(m) + 1) : 0;
    }
}
void orc_get_quant(const orc_cache *c, int32_t *qbits, int32_t *qexp) {
    for (int k = 0; k < c->NK; k++) { qbits[k] = c->qbits[k]; qexp[k] = c->qexp[k]; }
}

/*
 * update_hist! + _hist!  — src/fit-utils.jl:345-394.  For each build node and each
 * sampled feature j: zero h[:, :, j, n] then add the node's rows in list order, reading
 * bins from the observation-major copy.  Threads over (node x feature tile) exactly as
 * the reference; within a (node, feature) the row order is sequential, so the Float64
 * result does not depend on the thread count.
 */
static void orc_update_hist(orc_cache *c, const int *build_nodes, int n_build, const float *grad,
                            const uint32_t *js, int nj, int mode) {
    if (n_build == 0) return;
    const int NK = c->NK, B = c->p.nbins, F = c->F;
    int nthr = c->nthreads;
    int per = (nthr + n_build - 1) / n_build;
    if (per < 1) per = 1;
    int tile = (nj + per - 1) / per;
    int ntiles = (nj + tile - 1) / tile;
#pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < n_build * ntiles; t++) {
        int ni = t / ntiles, ti = t % ntiles;
        int n = build_nodes[ni]; /* 1-based node id */
        int j0 = ti * tile, j1 = (ti + 1) * tile < nj ? (ti + 1) * tile : nj;
        for (int jj = j0; jj < j1; jj++) {
            int j = (int)js[jj] - 1;
            if (mode == 0) memset(c->h + hidx(c, 0, 0, j, n - 1), 0, sizeof(double) * NK * B);
            else memset(c->hq + hidx(c, 0, 0, j, n - 1), 0, sizeof(int64_t) * NK * B);
        }
        const uint32_t *rows = c->is + c->seg_off[n];
        int64_t len = c->seg_len[n];
        for (int64_t idx = 0; idx < len; idx++) {
            int64_t i = rows[idx];
            const float *g = grad + (int64_t)NK * i;
            const uint8_t *xb = c->x_bin_T + (size_t)i * F;
            if (mode == 0) {
                for (int jj = j0; jj < j1; jj++) {
                    int j = (int)js[jj] - 1;
                    int bin = xb[j] - 1;
                    double *hh = c->h + hidx(c, 0, bin, j, n - 1);
                    for (int k = 0; k < NK; k++) hh[k] += (double)g[k];
                }
            } else {
                int64_t q[ORC_MAX_NK];
                for (int k = 0; k < NK; k++) q[k] = orc_quant(g[k], c->qbits[k], c->qexp[k]);
                for (int jj = j0; jj < j1; jj++) {
                    int j = (int)js[jj] - 1;
                    int bin = xb[j] - 1;
                    int64_t *hh = c->hq + hidx(c, 0, bin, j, n - 1);
                    for (int k = 0; k < NK; k++) hh[k] += q[k];
                }
            }
        }
    }
}

/* subtract_hist! — src/fit-utils.jl:321-332: h[:, :, j, n] = h[:, :, j, n>>1] - h[:, :, j, n^1]. */
static void orc_subtract_hist(orc_cache *c, const int *nodes, int nn, const uint32_t *js, int nj, int mode) {
    const int NK = c->NK, B = c->p.nbins;
#pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < nn; t++) {
        int n = nodes[t], np = n >> 1, ns = n ^ 1;
        for (int jj = 0; jj < nj; jj++) {
            int j = (int)js[jj] - 1;
            size_t o = hidx(c, 0, 0, j, n - 1), op = hidx(c, 0, 0, j, np - 1), os = hidx(c, 0, 0, j, ns - 1);
            if (mode == 0) for (int i = 0; i < NK * B; i++) c->h[o + i] = c->h[op + i] - c->h[os + i];
            else for (int i = 0; i < NK * B; i++) c->hq[o + i] = c->hq[op + i] - c->hq[os + i];
        }
    }
}

/* _term_gh — src/split.jl:1 */
static inline double term_gh(double g, double h, double w, double lambda, double L2, double eps) {
    double d = h + lambda * w + L2;
    if (!(d > eps)) d = eps; /* max(eps, d) */
    return g * g / d / 2.0;
}

/* _term_shift — src/split.jl:2 */
static inline double term_shift(double g, double w, double mu_p, double d) { return fabs(g / w - mu_p) * w / d; }

/* _cred_Z — src/loss.jl:275-290: VHM = (m1 / w)^2, EVPV = max(eps, m2 / w - VHM); the ratio of variances (cred_var) or of
 * standard deviations (cred_std).  _term_cred — src/split.jl:3-4. */
static inline double term_cred(int loss, double m1, double m2, double w, double L2, double eps) {
    double mean = m1 / w;
    double VHM = mean * mean;
    double EVPV = m2 / w - VHM;
    if (!(EVPV > eps)) EVPV = eps;
    double Z = (loss == ORC_CRED_VAR) ? VHM / (VHM + EVPV) : sqrt(VHM) / (sqrt(VHM) + sqrt(EVPV));
    return Z * fabs(m1) / (1.0 + L2 / w);
}

/* node_gain — src/split.jl:58-66 (gradient losses), :68 (mae: zero), :70-78 (credibility losses) */
static double node_gain(int loss, const double *S, int K, double lambda, double L2, double eps) {
    double w = S[2 * K], gain = 0.0;
    if (ORC_IS_SHIFT(loss)) return 0.0;
    if (ORC_IS_CRED(loss)) {
        for (int k = 0; k < K; k++) gain += term_cred(loss, S[k], S[K + k], w, L2, eps);
        return gain;
    }
    for (int k = 0; k < K; k++) gain += term_gh(S[k], S[K + k], w, lambda, L2, eps);
    return gain;
}

/* split_gain — src/split.jl:108-117 (gradient losses), :119-130 (mae), :132-141 (credibility losses) */
static double split_gain(int loss, const double *S, const double *SL, int K, double w_l, double w_r, double lambda, double L2, double eps) {
    double gain = 0.0;
    if (ORC_IS_SHIFT(loss)) {
        double w_p = S[2 * K];
        double d_l = 1.0 + lambda + L2 / w_l, d_r = 1.0 + lambda + L2 / w_r;
        if (!(d_l > eps)) d_l = eps;
        if (!(d_r > eps)) d_r = eps;
        for (int k = 0; k < K; k++) {
            double mu_p = S[k] / w_p;
            gain += term_shift(SL[k], w_l, mu_p, d_l) + term_shift(S[k] - SL[k], w_r, mu_p, d_r);
        }
        return gain;
    }
    if (ORC_IS_CRED(loss)) {
        for (int k = 0; k < K; k++) {
            double m1l = SL[k], m2l = SL[K + k];
            gain += term_cred(loss, m1l, m2l, w_l, L2, eps) + term_cred(loss, S[k] - m1l, S[K + k] - m2l, w_r, L2, eps);
        }
        return gain;
    }
    for (int k = 0; k < K; k++) {
        double g_l = SL[k], h_l = SL[K + k];
        gain += term_gh(g_l, h_l, w_l, lambda, L2, eps) + term_gh(S[k] - g_l, S[K + k] - h_l, w_r, lambda, L2, eps);
    }
    return gain;
}

/* pred_scalar — src/predict.jl:205-208 (GradientRegression), :235-238 (MLE2P), :219-221 (credibility), :259-262 (mae) */
static double pred_scalar(const double *S, const orc_params *p) {
    int K = p->K;
    if (ORC_IS_CRED(p->loss)) return p->eta / (double)p->bagging_size * S[0] / (S[2 * K] + p->L2);
    if (p->loss == ORC_MAE) {
        double d = S[2 * K] + p->lambda * S[2 * K] + p->L2;
        if (!(d > DBL_EPSILON)) d = DBL_EPSILON;
        return p->eta / (double)p->bagging_size * S[0] / d;
    }
    double d = S[K] + p->lambda * S[2 * K] + p->L2;
    if (!(d > DBL_EPSILON)) d = DBL_EPSILON;
    return -p->eta / (double)p->bagging_size * S[0] / d;
}

/* pred_leaf_cpu! — src/predict.jl:198-204 (GradientRegression), :224-234 (MLE2P; for one
 * target the index pairs are (1,3),(2,4), i.e. (k, K+k) as well), :211-217 (credibility), :250-258 (mae).
 * Stored as Float32. */
static void pred_leaf(float *tree_pred, int n, const double *S, const orc_params *p) {
    int K = p->K;
    for (int k = 0; k < K; k++) {
        double v;
        if (ORC_IS_CRED(p->loss)) {
            v = p->eta / (double)p->bagging_size * S[k] / (S[2 * K] + p->L2);
        } else if (p->loss == ORC_MAE) {
            double d = S[2 * K] + p->lambda * S[2 * K] + p->L2;
            if (!(d > DBL_EPSILON)) d = DBL_EPSILON;
            v = p->eta / (double)p->bagging_size * S[k] / d;
        } else {
            double d = S[K + k] + p->lambda * S[2 * K] + p->L2;
            if (!(d > DBL_EPSILON)) d = DBL_EPSILON;
            v = -p->eta / (double)p->bagging_size * S[k] / d;
        }
        tree_pred[(size_t)K * (n - 1) + k] = (float)v;
    }
}

/* Statistics.quantile(v, p) with its defaults alpha = beta = 1 (the stdlib the reference calls; Hyndman & Fan's
 * definition 7, numpy's "linear"): on the sorted values, aleph = fma(n, p, 1 - p), j = clamp(trunc(aleph), 1, n - 1),
 * gamma = clamp(aleph - j, 0, 1), result v[j] + gamma * (v[j+1] - v[j]) with the difference taken in the values' own
 * Float32 and the rest in Float64.  v is sorted here (ascending). */
static int cmp_f32(const void *a, const void *b) {
    float x = *(const float *)a, y = *(const float *)b;
    return (x > y) - (x < y);
}
static double jl_quantile(float *v, int64_t n, double p) {
    qsort(v, (size_t)n, sizeof(float), cmp_f32);
    double aleph = fma((double)n, p, 1.0 - p);
    int64_t j = (int64_t)aleph;
    if (j > n - 1) j = n - 1; /* clamp(x, lo, hi) = ifelse(x > hi, hi, ifelse(x < lo, lo, x)) */
    else if (j < 1) j = 1;
    double gamma = aleph - (double)j;
    if (gamma > 1.0) gamma = 1.0;
    else if (gamma < 0.0) gamma = 0.0;
    float a, b;
    if (n == 1) { a = v[0]; b = v[0]; }
    else { a = v[j - 1]; b = v[j]; }
    if (isfinite(a) && isfinite(b)) return (double)a + gamma * (double)(b - a);
    return (1.0 - gamma) * (double)a + gamma * (double)b;
}

/* pred_leaf_cpu! of the quantile losses — src/predict.jl:265-272 (quantile: max(eps, denom)) and :275-281
 * (multiquantile): eta / bagging * quantile(residuals of the leaf's rows, alpha) / (1 + lambda + L2 / w).  rows: the
 * node's row ids; the residual of output k is row K + k of the gradient matrix. */
static void pred_leaf_quantile(float *tree_pred, int n, const double *S, const orc_params *p, const float *grad, const uint32_t *rows, int64_t nrows) {
    const int K = p->K, NK = 2 * K + 1;
    float *v = (float *)malloc(sizeof(float) * (size_t)(nrows > 0 ? nrows : 1));
    double denom = 1.0 + p->lambda + p->L2 / S[2 * K];
    if (p->loss == ORC_QUANTILE && !(denom > DBL_EPSILON)) denom = DBL_EPSILON;
    for (int k = 0; k < K; k++) {
        for (int64_t t = 0; t < nrows; t++) v[t] = grad[(int64_t)NK * rows[t] + K + k];
        const double alpha = (p->loss == ORC_MULTIQUANTILE) ? p->alphas[k] : p->alphas[0];
        const double q = nrows > 0 ? jl_quantile(v, nrows, alpha) : 0.0;
        tree_pred[(size_t)K * (n - 1) + k] = (float)(p->eta / (double)p->bagging_size * q / denom);
    }
    free(v);
}

typedef void (*scan_sink)(void *ctx, double gain, int j, int bin);

/*
 * _scan_node! — src/fit-utils.jl:403-436.  Walks features in js order and bins ascending;
 * numeric features scan bins 1..B-1, categorical 1..B (:414); eligibility is strict on both
 * sides (:419); monotone check :420-429; candidate value split_gain - gain_p (:430).
 * j and bin are reported 1-based.
 */
static void scan_node(orc_cache *c, int n, const uint32_t *js, int nj, int mode, scan_sink sink, void *ctx) {
    const orc_params *p = &c->p;
    const int NK = c->NK, K = p->K, B = p->nbins;
    const double eps = DBL_EPSILON;
    const double *S = c->sum + (size_t)n * NK;
    double SL[ORC_MAX_NK], SR[ORC_MAX_NK];
    int64_t SLq[ORC_MAX_NK];
    double gain_p = node_gain(p->loss, S, K, p->lambda, p->L2, eps);
    double w_p = S[NK - 1];
    for (int jj = 0; jj < nj; jj++) {
        int j = (int)js[jj] - 1;
        int constraint = c->mono[j];
        int is_numeric = c->feattypes[j];
        for (int k = 0; k < NK; k++) { SL[k] = 0.0; SLq[k] = 0; }
        int b_max = is_numeric ? B - 1 : B;
        for (int bin = 0; bin < b_max; bin++) {
            /* _acc_left! — src/split.jl:16-27 */
            if (mode == 0) {
                const double *hh = c->h + hidx(c, 0, bin, j, n - 1);
                for (int k = 0; k < NK; k++) SL[k] = is_numeric ? SL[k] + hh[k] : hh[k];
            } else {
                const int64_t *hh = c->hq + hidx(c, 0, bin, j, n - 1);
                for (int k = 0; k < NK; k++) {
                    SLq[k] = is_numeric ? SLq[k] + hh[k] : hh[k];
                    SL[k] = orc_decode(SLq[k], c->qbits[k], c->qexp[k]);
                }
            }
            double w_l = SL[NK - 1];
            double w_r = w_p - w_l;
            if (w_l > p->min_weight && w_r > p->min_weight) {
                int ok = 1;
                if (constraint != 0) {
                    for (int k = 0; k < NK; k++) SR[k] = S[k] - SL[k];
                    double predL = pred_scalar(SL, p), predR = pred_scalar(SR, p);
                    ok = (constraint == -1 && predL > predR) || (constraint == 1 && predL < predR);
                }
                if (ok) sink(ctx, split_gain(p->loss, S, SL, K, w_l, w_r, p->lambda, p->L2, eps) - gain_p, j + 1, bin + 1);
            }
        }
    }
}

typedef struct { double gain; int feat, bin; } best_t;
/* get_best_split — src/fit-utils.jl:444-450: strict '>' keeps the first maximum, start at gamma. */
static void best_sink(void *ctx, double gain, int j, int bin) {
    best_t *b = (best_t *)ctx;
    if (gain > b->gain) { b->gain = gain; b->feat = j; b->bin = bin; }
}
typedef struct { double *gains; int B; } gains_ctx;
/* update_gains! — src/fit-utils.jl:457-463 */
static void gains_sink(void *ctx, double gain, int j, int bin) {
    gains_ctx *g = (gains_ctx *)ctx;
    g->gains[(size_t)(bin - 1) + (size_t)g->B * (j - 1)] = gain;
}

/*
 * split_set! — src/fit-utils.jl:93-132 (single :277-312, threaded :217-275; both produce
 * the same stable partition).  Reads the node's view, writes lefts then rights at
 * is[offset ...].  Returns the number of lefts.
 */
static int64_t split_set(orc_cache *c, int64_t view_off, int64_t len, int feat, int cond_bin, int is_numeric, int64_t offset) {
    const uint8_t *col = c->x_bin + (size_t)(feat - 1) * c->N;
    int64_t nl = 0, nr = 0;
    for (int64_t t = 0; t < len; t++) {
        uint32_t i = c->is[view_off + t];
        int cond = is_numeric ? (col[i] <= cond_bin) : (col[i] == cond_bin);
        if (cond) c->left[nl++] = i; else c->right[nr++] = i;
    }
    memcpy(c->is + offset, c->left, sizeof(uint32_t) * nl);
    memcpy(c->is + offset + nl, c->right, sizeof(uint32_t) * nr);
    return nl;
}

/* _child_sums! — src/fit-utils.jl:472-486 and right = parent - left, src/fit.jl:120-121 */
static void child_sums(orc_cache *c, int n, int feat, int bin, int is_numeric, int mode) {
    const int NK = c->NK;
    double *SLd = c->sum + (size_t)(2 * n) * NK, *SRd = c->sum + (size_t)(2 * n + 1) * NK;
    const double *S = c->sum + (size_t)n * NK;
    if (mode == 0) {
        for (int k = 0; k < NK; k++) SLd[k] = 0.0;
        if (is_numeric) {
            for (int b = 0; b < bin; b++) {
                const double *hh = c->h + hidx(c, 0, b, feat - 1, n - 1);
                for (int k = 0; k < NK; k++) SLd[k] += hh[k];
            }
        } else {
            const double *hh = c->h + hidx(c, 0, bin - 1, feat - 1, n - 1);
            for (int k = 0; k < NK; k++) SLd[k] = hh[k];
        }
        for (int k = 0; k < NK; k++) SRd[k] = S[k] - SLd[k];
    } else {
        int64_t *SLq = c->sumq + (size_t)(2 * n) * NK, *SRq = c->sumq + (size_t)(2 * n + 1) * NK;
        const int64_t *Sq = c->sumq + (size_t)n * NK;
        for (int k = 0; k < NK; k++) SLq[k] = 0;
        if (is_numeric) {
            for (int b = 0; b < bin; b++) {
                const int64_t *hh = c->hq + hidx(c, 0, b, feat - 1, n - 1);
                for (int k = 0; k < NK; k++) SLq[k] += hh[k];
            }
        } else {
            const int64_t *hh = c->hq + hidx(c, 0, bin - 1, feat - 1, n - 1);
            for (int k = 0; k < NK; k++) SLq[k] = hh[k];
        }
        for (int k = 0; k < NK; k++) {
            SRq[k] = Sq[k] - SLq[k];
            SLd[k] = orc_decode(SLq[k], c->qbits[k], c->qexp[k]);
            SRd[k] = orc_decode(SRq[k], c->qbits[k], c->qexp[k]);
        }
    }
}

static int cmp_int(const void *a, const void *b) { return *(const int *)a - *(const int *)b; }

/*
 * grow_tree! (src/fit.jl:45-143) and grow_otree! (src/fit.jl:147-263).
 *
 * Inputs: grad (2K+1) x N Float32; is_in: n_is sampled row ids, ascending, 0-based;
 * js: n_js sampled feature ids, ascending, 1-based.
 * Outputs (all length nnodes = 2^max_depth-1, zero-initialised here like Tree{L,K}(depth),
 * src/structs.jl:97-106): feat (Int64, 1-based, 0 = none), cond_bin, w, gain, pred (K x nnodes),
 * split.  nidx_out (optional, length N): for each sampled row the 1-based id of the node it
 * ends in; 0 for rows not in the sample.
 * mode: 0 = Float64 reference arithmetic, 1 = fixed-point (orc_set_quant must have been called).
 */
int orc_grow_tree(orc_cache *c, const float *grad, const uint32_t *is_in, int64_t n_is, const uint32_t *js, int32_t n_js,
                  int mode, int64_t *t_feat, uint8_t *t_cond_bin, float *t_w, float *t_gain, float *t_pred, uint8_t *t_split,
                  uint32_t *nidx_out) {
    const orc_params *p = &c->p;
    const int NK = c->NK, K = p->K, B = p->nbins, nnodes = c->nnodes;
    if (mode == 1 && !c->hq) return -1;
    memset(t_feat, 0, sizeof(int64_t) * nnodes);
    memset(t_cond_bin, 0, nnodes);
    memset(t_w, 0, sizeof(float) * nnodes);
    memset(t_gain, 0, sizeof(float) * nnodes);
    memset(t_pred, 0, sizeof(float) * (size_t)K * nnodes);
    memset(t_split, 0, nnodes);
    if (nidx_out) memset(nidx_out, 0, sizeof(uint32_t) * (size_t)c->N);

    memcpy(c->is, is_in, sizeof(uint32_t) * (size_t)n_is);
    c->seg_off[1] = 0;
    c->seg_len[1] = n_is;

    /* root sums: src/fit.jl:66 (Float64 accumulation in list order) */
    {
        double *S = c->sum + (size_t)1 * NK;
        int64_t *Sq = c->sumq + (size_t)1 * NK;
        for (int k = 0; k < NK; k++) { S[k] = 0.0; Sq[k] = 0; }
        for (int64_t t = 0; t < n_is; t++) {
            const float *g = grad + (int64_t)NK * is_in[t];
            if (mode == 0) for (int k = 0; k < NK; k++) S[k] += (double)g[k];
            else for (int k = 0; k < NK; k++) Sq[k] += orc_quant(g[k], c->qbits[k], c->qexp[k]);
        }
        if (mode == 1) for (int k = 0; k < NK; k++) S[k] = orc_decode(Sq[k], c->qbits[k], c->qexp[k]);
    }

    int *n_current = (int *)malloc(sizeof(int) * (nnodes + 1));
    int *n_next = (int *)malloc(sizeof(int) * (nnodes + 1));
    int *tmp = (int *)malloc(sizeof(int) * (nnodes + 1));
    int ncur = 1, depth = 1;
    n_current[0] = 1;

    while (ncur > 0 && depth <= p->max_depth) {
        int64_t offset = 0;
        int nnext = 0;
        if (depth == p->max_depth) {
            for (int t = 0; t < ncur; t++) {
                int n = n_current[t];
                const double *S = c->sum + (size_t)n * NK;
                t_w[n - 1] = (float)S[NK - 1];
                if (ORC_IS_QUANTILE(p->loss)) pred_leaf_quantile(t_pred, n, S, p, grad, c->is + c->seg_off[n], c->seg_len[n]);
                else pred_leaf(t_pred, n, S, p);
                if (nidx_out) for (int64_t q = 0; q < c->seg_len[n]; q++) nidx_out[c->is[c->seg_off[n] + q]] = (uint32_t)n;
            }
        } else {
            /* build = odd positions, subtract = even positions (src/fit.jl:85-87) */
            int nb = 0, ns = 0;
            for (int t = 0; t < ncur; t += 2) tmp[nb++] = n_current[t];
            orc_update_hist(c, tmp, nb, grad, js, n_js, mode);
            for (int t = 1; t < ncur; t += 2) tmp[ns++] = n_current[t];
            orc_subtract_hist(c, tmp, ns, js, n_js, mode);
            qsort(n_current, ncur, sizeof(int), cmp_int);

            if (p->tree_type == 0) {
#pragma omp parallel for schedule(dynamic, 1)
                for (int t = 0; t < ncur; t++) {
                    int n = n_current[t];
                    t_w[n - 1] = (float)c->sum[(size_t)n * NK + NK - 1];
                    best_t best = {p->gamma, 0, 0};
                    scan_node(c, n, js, n_js, mode, best_sink, &best);
                    if (best.bin != 0) {
                        t_gain[n - 1] = (float)best.gain;
                        t_cond_bin[n - 1] = (uint8_t)best.bin;
                        t_feat[n - 1] = best.feat;
                        t_split[n - 1] = 1;
                    }
                }
            } else {
                /* src/fit.jl:190-257 */
#pragma omp parallel for schedule(dynamic, 1)
                for (int t = 0; t < ncur; t++) {
                    int n = n_current[t];
                    t_w[n - 1] = (float)c->sum[(size_t)n * NK + NK - 1];
                    double *gn = c->gains + (size_t)B * c->F * (n - 1);
                    for (int jj = 0; jj < n_js; jj++) memset(gn + (size_t)B * (js[jj] - 1), 0, sizeof(double) * B);
                    gains_ctx gc = {gn, B};
                    scan_node(c, n, js, n_js, mode, gains_sink, &gc);
                }
                double *g1 = c->gains; /* node 1 doubles as the level accumulator */
                if (depth > 1) for (int jj = 0; jj < n_js; jj++) memset(g1 + (size_t)B * (js[jj] - 1), 0, sizeof(double) * B);
                for (int t = 0; t < ncur; t++) {
                    int n = n_current[t];
                    if (n > 1) {
                        const double *gn = c->gains + (size_t)B * c->F * (n - 1);
                        for (int jj = 0; jj < n_js; jj++) {
                            size_t o = (size_t)B * (js[jj] - 1);
                            for (int b = 0; b < B; b++) g1[o + b] += gn[o + b];
                        }
                    }
                }
                for (int t = 0; t < ncur; t++) {
                    int n = n_current[t];
                    if (n > 1) {
                        const double *gn = c->gains + (size_t)B * c->F * (n - 1);
                        for (int jj = 0; jj < n_js; jj++) {
                            size_t o = (size_t)B * (js[jj] - 1);
                            for (int b = 0; b < B; b++) g1[o + b] *= (gn[o + b] > 0.0) ? 1.0 : 0.0;
                        }
                    }
                }
                /* findmax over view(gains, :, js): first maximum, bin fastest then js position */
                double best_gain = -INFINITY;
                int best_bin = 0, best_feat = 0;
                for (int jj = 0; jj < n_js; jj++) {
                    size_t o = (size_t)B * (js[jj] - 1);
                    for (int b = 0; b < B; b++) {
                        double v = g1[o + b];
                        /* Julia's findmax orders -0.0 below 0.0 (isless) */
                        int greater = (v > best_gain) || (v == best_gain && signbit(best_gain) && !signbit(v));
                        if (best_bin == 0 || greater) { best_gain = v; best_bin = b + 1; best_feat = (int)js[jj]; }
                    }
                }
                if (best_gain > p->gamma) {
                    for (int t = 0; t < ncur; t++) {
                        int n = n_current[t];
                        t_gain[n - 1] = (float)best_gain;
                        t_cond_bin[n - 1] = (uint8_t)best_bin;
                        t_feat[n - 1] = best_feat;
                        t_split[n - 1] = 1;
                    }
                }
            }

            for (int t = 0; t < ncur; t++) {
                int n = n_current[t];
                if (t_split[n - 1]) {
                    int feat = (int)t_feat[n - 1], bin = t_cond_bin[n - 1];
                    int is_num = c->feattypes[feat - 1];
                    int64_t len = c->seg_len[n];
                    int64_t nl = split_set(c, c->seg_off[n], len, feat, bin, is_num, offset);
                    c->seg_off[2 * n] = offset;
                    c->seg_len[2 * n] = nl;
                    c->seg_off[2 * n + 1] = offset + nl;
                    c->seg_len[2 * n + 1] = len - nl;
                    offset += len;
                    child_sums(c, n, feat, bin, is_num, mode);
                    if (len - nl >= nl) { n_next[nnext++] = 2 * n; n_next[nnext++] = 2 * n + 1; }
                    else { n_next[nnext++] = 2 * n + 1; n_next[nnext++] = 2 * n; }
                } else {
                    if (ORC_IS_QUANTILE(p->loss)) pred_leaf_quantile(t_pred, n, c->sum + (size_t)n * NK, p, grad, c->is + c->seg_off[n], c->seg_len[n]);
                    else pred_leaf(t_pred, n, c->sum + (size_t)n * NK, p);
                    /* rows of a finished node: record before later splits overwrite the buffer */
                    if (nidx_out) for (int64_t q = 0; q < c->seg_len[n]; q++) nidx_out[c->is[c->seg_off[n] + q]] = (uint32_t)n;
                }
            }
        }
        memcpy(n_current, n_next, sizeof(int) * nnext);
        ncur = nnext;
        depth++;
    }
    free(n_current); free(n_next); free(tmp);
    return 0;
}

/* node sums of the last grown tree (NK doubles per node, node ids 1..nnodes; index 0 unused) */
const double *orc_node_sums(const orc_cache *c) { return c->sum; }

/* leaf walk — src/predict.jl:3-8 (same rule in test/predict-leaf-idx.jl:34-49) */
static inline int walk(const uint8_t *x_bin, int64_t N, int64_t i, const uint8_t *feattypes, const int64_t *t_feat,
                       const uint8_t *t_cond_bin, const uint8_t *t_split) {
    int nid = 1;
    while (t_split[nid - 1]) {
        int feat = (int)t_feat[nid - 1];
        uint8_t xb = x_bin[(size_t)(feat - 1) * N + i];
        int cond = feattypes[feat - 1] ? (xb <= t_cond_bin[nid - 1]) : (xb == t_cond_bin[nid - 1]);
        nid = (nid << 1) + !cond;
    }
    return nid;
}

/* predict! — src/predict.jl:1-14 (GradientRegression), :16-29 (LogLoss clamp), :31-46 (MLE2P) */
void orc_predict_tree(int32_t loss, int32_t K, int64_t N, const uint8_t *x_bin, const uint8_t *feattypes, const int64_t *t_feat,
                      const uint8_t *t_cond_bin, const float *t_pred, const uint8_t *t_split, float *pred) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < N; i++) {
        int nid = walk(x_bin, N, i, feattypes, t_feat, t_cond_bin, t_split);
        const float *lp = t_pred + (size_t)K * (nid - 1);
        float *pr = pred + (size_t)K * i;
        if (loss == ORC_MLOGLOSS) { /* src/predict.jl:48-62: add, then shift by the row maximum, floor at -15 */
            float m = -INFINITY;
            for (int k = 0; k < K; k++) { pr[k] += lp[k]; if (pr[k] > m) m = pr[k]; }
            for (int k = 0; k < K; k++) { float v = pr[k] - m; pr[k] = v > -15.0f ? v : -15.0f; }
        } else if (loss == ORC_MSE || (loss >= ORC_POISSON && loss != ORC_LOGISTIC_MLE)) { /* generic method, src/predict.jl:68-81, for mae and the credibility losses */
            for (int k = 0; k < K; k++) pr[k] += lp[k];
        } else if (loss == ORC_LOGLOSS) {
            for (int k = 0; k < K; k++) {
                float v = pr[k] + lp[k];
                pr[k] = v < -15.0f ? -15.0f : (v > 15.0f ? 15.0f : v);
            }
        } else {
            for (int t = 0; t < K / 2; t++) {
                pr[2 * t] += lp[2 * t];
                float v = pr[2 * t + 1] + lp[2 * t + 1];
                pr[2 * t + 1] = v > -15.0f ? v : -15.0f;
            }
        }
    }
}

/* predict_leaf_idx! — src/predict.jl:138-154 */
void orc_predict_leaf_idx(int64_t N, const uint8_t *x_bin, const uint8_t *feattypes, const int64_t *t_feat, const uint8_t *t_cond_bin,
                          const uint8_t *t_split, uint32_t *leaf_idx) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < N; i++) leaf_idx[i] = (uint32_t)walk(x_bin, N, i, feattypes, t_feat, t_cond_bin, t_split);
}

/* apply_prediction_link! — src/predict.jl:105-116 (in place on K x N) */
void orc_apply_link(int32_t loss, int32_t K, int64_t N, float *pred) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < N; i++) {
        if (loss == ORC_LOGLOSS) {
            for (int k = 0; k < K; k++) pred[(size_t)K * i + k] = orc_sigmoidf(pred[(size_t)K * i + k]);
        } else if (ORC_IS_MLE2P(loss)) {
            for (int k = 1; k < K; k += 2) pred[(size_t)K * i + k] = orc_softplusf(pred[(size_t)K * i + k]);
        } else if (loss == ORC_MLOGLOSS) { /* softmax!, src/predict.jl:187-195 */
            float isum = 0.0f;
            for (int k = 0; k < K; k++) { pred[(size_t)K * i + k] = expf(pred[(size_t)K * i + k]); isum += pred[(size_t)K * i + k]; }
            for (int k = 0; k < K; k++) pred[(size_t)K * i + k] /= isum;
        } else if (loss >= ORC_POISSON && loss <= ORC_TWEEDIE) {
            for (int k = 0; k < K; k++) pred[(size_t)K * i + k] = expf(pred[(size_t)K * i + k]);
        }
    }
}

/*
 * Evaluation metrics — src/metrics.jl:1-48 (_eval_metric: eval[i] = w[i] * value / K in Float32, result
 * sum(Float64, eval) / sum(Float64, w)) and :88-112 (gaussian_mle: mean log-likelihood).
 * metric: 0 mse, 1 rmse, 2 mae, 3 logloss, 4 gaussian_mle, 5 poisson, 6 gamma, 7 tweedie, 9 logistic_mle, 8 mlogloss (:59-77,
 * eval[i] = w[i] * (log(sum_k exp(p[k,i])) - p[y[i], i]), not divided by K).
 */
/* quantile / multiquantile metrics — src/metrics.jl:4-6 (the pinball loss of one output in Float32, alpha given as
 * T(params.alpha), src/callback.jl:62-66), :83-84 (quantile: averaged over the K outputs like every other metric, one
 * target column each) and :117-134 (multiquantile: one target, alphas[k] for output k).  metric: 10 quantile, 11 multiquantile. */
double orc_eval_metric_quantile(int32_t metric, int32_t K, int64_t N, const float *pred, const float *y, const float *w, const float *alphas) {
    double num = 0.0, den = 0.0;
    for (int64_t i = 0; i < N; i++) {
        float wi = w ? w[i] : 1.0f, acc = 0.0f;
        for (int k = 0; k < K; k++) {
            float pk = pred[(size_t)K * i + k], yk = (metric == 11) ? y[i] : y[(size_t)K * i + k];
            float alpha = (metric == 11) ? alphas[k] : alphas[0];
            float up = yk - pk, dn = pk - yk;
            acc += alpha * (up > 0.0f ? up : 0.0f) + (1.0f - alpha) * (dn > 0.0f ? dn : 0.0f);
        }
        float ev = wi * acc / (float)K;
        num += (double)ev;
        den += (double)wi;
    }
    return num / den;
}

double orc_eval_metric(int32_t metric, int32_t K, int64_t N, const float *pred, const float *y, const float *w) {
    double num = 0.0, den = 0.0;
    for (int64_t i = 0; i < N; i++) {
        float wi = w ? w[i] : 1.0f;
        float v;
        if (metric == 8) {
            float isum = 0.0f;
            for (int k = 0; k < K; k++) isum += expf(pred[(size_t)K * i + k]);
            num += (double)(wi * (logf(isum) - pred[(size_t)K * i + (int)y[i] - 1]));
            den += (double)wi;
            continue;
        }
        v = 0.0f; /* acc = zero(T); acc += value per target, src/metrics.jl:39-43, :105-110 */
        if (metric == 4 || metric == 9) {
            const int Y = K / 2;
            for (int t = 0; t < Y; t++) {
                float loc = pred[(size_t)K * i + 2 * t], scale = orc_softplusf(pred[(size_t)K * i + 2 * t + 1]);
                if (metric == 4) {
                    float d = y[(size_t)Y * i + t] - loc;
                    v += -(logf(scale) + (d * d) / (2.0f * (scale * scale)));
                } else { /* logistic_mle, src/metrics.jl:92-97 */
                    float az = fabsf((y[(size_t)Y * i + t] - loc) / scale);
                    v += -logf(scale) - az - 2.0f * log1pf(expf(-az));
                }
            }
        } else {
            for (int k = 0; k < K; k++) {
                float pk = pred[(size_t)K * i + k], yk = y[(size_t)K * i + k], u;
                if (metric == 0 || metric == 1) u = (pk - yk) * (pk - yk);
                else if (metric == 2) u = fabsf(pk - yk);
                else if (metric == 3) { float s = orc_sigmoidf(pk); u = -yk * logf(s) + (yk - 1.0f) * logf(1.0f - s); }
                else if (metric == 5) { float e = expf(pk); const float eps = 7.105427357601002e-15f; /* eps(Float32(1e-7)) = 2^-47 */
                                        u = 2.0f * (yk * logf(yk / e + eps) + e - yk); }
                else if (metric == 6) { float e = expf(pk); u = 2.0f * (logf(e / yk) + yk / e - 1.0f); }
                else { float e = expf(pk); u = 2.0f * (powf(yk, 0.5f) / (-0.5f) / 0.5f - yk * powf(e, -0.5f) / (-0.5f) + powf(e, 0.5f) / 0.5f); }
                v += u;
            }
        }
        float ev = wi * v / (float)((metric == 4 || metric == 9) ? K / 2 : K);
        num += (double)ev;
        den += (double)wi;
    }
    double r = num / den;
    return metric == 1 ? sqrt(r) : r;
}
