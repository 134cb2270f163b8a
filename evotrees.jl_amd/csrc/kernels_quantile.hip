// Leaf values of the quantile losses (pred_leaf_cpu!, src/predict.jl:265-281; called per leaf with the leaf's rows,
// src/fit.jl:77, :131, :178, :251): eta / bagging * quantile(residuals of the leaf's rows, alpha) / (1 + lambda + L2 / w).
// The reference walks each leaf's row list on the host (its device path copies the gradients and node ids back for it,
// ext/EvoTreesKernelAbstractionsExt/fit.jl:304-330).  Here, once the tree is complete and every row in the sample
// carries the id of its leaf: one 64-bit key per row, (leaf id, residual in an order-preserving code); one radix sort;
// every leaf then finds its run of keys by binary search and interpolates between two of them.
//
// quantile(v, p) is Statistics.quantile with its defaults (Hyndman & Fan's definition 7): on the sorted values,
// aleph = fma(n, p, 1 - p), j = clamp(trunc(aleph), 1, n - 1), gamma = clamp(aleph - j, 0, 1), v[j] + gamma * (v[j+1] - v[j])
// with the difference in the values' Float32 and the rest in Float64.
#include "evt_internal.h"
#include <float.h>
#include <hipcub/hipcub.hpp>

// Float32 -> unsigned code with the same order (negative values: all bits flipped; others: the sign bit set)
__device__ __forceinline__ uint32_t order_code(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float order_decode(uint32_t c) {
    return __uint_as_float((c & 0x80000000u) ? (c & 0x7FFFFFFFu) : ~c);
}

// rows outside the tree's sample carry node 0 and sort ahead of every leaf
__global__ __launch_bounds__(256) void k_quantile_keys(const uint32_t *__restrict__ nidx, const float *__restrict__ grad, int64_t N, int NK, int row,
                                                      unsigned long long *__restrict__ keys) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < N; i += (int64_t)gridDim.x * 256)
        keys[i] = ((unsigned long long)nidx[i] << 32) | order_code(grad[(size_t)NK * i + row]);
}

__device__ __forceinline__ int64_t first_not_below(const unsigned long long *__restrict__ a, int64_t n, unsigned long long key) {
    int64_t lo = 0, hi = n;
    while (lo < hi) {
        const int64_t mid = lo + ((hi - lo) >> 1);
        if (a[mid] < key) lo = mid + 1;
        else hi = mid;
    }
    return lo;
}

// one thread per node; only leaves are valued.  k: the output whose residuals were sorted.
__global__ __launch_bounds__(256) void k_leaf_quantile(const unsigned long long *__restrict__ sorted, int64_t N, const int32_t *__restrict__ status,
                                                      const long long *__restrict__ node_sum, const double *__restrict__ qscale, int NAg, int nnodes,
                                                      int K, int k, int multi, const double *__restrict__ alphas, double eta, int bagging,
                                                      double lambda, double L2, float *__restrict__ tree_pred) {
    const int n = blockIdx.x * 256 + threadIdx.x + 1; // 1-based node id
    if (n > nnodes || status[n] != ST_LEAF) return;
    const int64_t lo = first_not_below(sorted, N, (unsigned long long)n << 32);
    const int64_t hi = first_not_below(sorted, N, (unsigned long long)(n + 1) << 32);
    const int64_t cnt = hi - lo;
    double q = 0.0;
    if (cnt > 0) {
        const double p = multi ? alphas[k] : alphas[0];
        const double aleph = fma((double)cnt, p, 1.0 - p);
        int64_t j = (int64_t)aleph;
        if (j > cnt - 1) j = cnt - 1; // clamp(x, lo, hi): the upper bound is tested first
        else if (j < 1) j = 1;
        double gamma = aleph - (double)j;
        if (gamma > 1.0) gamma = 1.0;
        else if (gamma < 0.0) gamma = 0.0;
        float a, b;
        if (cnt == 1) {
            a = b = order_decode((uint32_t)sorted[lo]);
        } else {
            a = order_decode((uint32_t)sorted[lo + j - 1]);
            b = order_decode((uint32_t)sorted[lo + j]);
        }
        if (isfinite(a) && isfinite(b)) q = (double)a + gamma * (double)(b - a);
        else q = (1.0 - gamma) * (double)a + gamma * (double)b;
    }
    const double w = (double)node_sum[(int64_t)n * NAg + NAg - 1] * qscale[NAg - 1];
    double denom = 1.0 + lambda + L2 / w;
    if (!multi && !(denom > DBL_EPSILON)) denom = DBL_EPSILON; // max(eps, denom): the quantile loss only (src/predict.jl:270)
    tree_pred[(int64_t)K * (n - 1) + k] = (float)(eta / (double)bagging * q / denom);
}

static int sort_bits(const evt_ctx *c) { return 32 + c->D + 1; } // node ids are below 2^D

// the two key arrays and the sort's work area, allocated when the first tree of a quantile loss is opened
int quantile_leaf_buffers(evt_ctx *c) {
    if (c->qkeys_a) return EVT_OK;
    if (c->N > (int64_t)0x7FFFFFFF) {
        evt_set_error("the quantile losses take at most 2^31 - 1 rows");
        return EVT_ERR_ARG;
    }
    size_t bytes = 0;
    hipError_t e = hipcub::DeviceRadixSort::SortKeys(nullptr, bytes, (const unsigned long long *)nullptr, (unsigned long long *)nullptr, (int)c->N, 0,
                                                     sort_bits(c), c->stream);
    if (e != hipSuccess) {
        evt_set_error("radix sort set-up failed: %s", hipGetErrorString(e));
        return EVT_ERR_HIP;
    }
    if (bytes < 256) bytes = 256;
    void *a = nullptr, *b = nullptr, *t = nullptr;
    if (hipMalloc(&a, sizeof(unsigned long long) * (size_t)c->N) != hipSuccess || hipMalloc(&b, sizeof(unsigned long long) * (size_t)c->N) != hipSuccess ||
        hipMalloc(&t, bytes) != hipSuccess) {
        (void)hipGetLastError();
        if (a) (void)hipFree(a);
        if (b) (void)hipFree(b);
        if (t) (void)hipFree(t);
        evt_set_error("out of device memory for the quantile losses' sort buffers (%zu bytes)", 2 * sizeof(unsigned long long) * (size_t)c->N + bytes);
        return EVT_ERR_NOMEM;
    }
    c->qkeys_a = static_cast<unsigned long long *>(a);
    c->qkeys_b = static_cast<unsigned long long *>(b);
    c->qtemp = t;
    c->qtemp_bytes = bytes;
    return EVT_OK;
}

int launch_quantile_leaves(evt_ctx *c, const evt_params *p) {
    int64_t nb = (c->N + 255) / 256;
    if (nb > 8192) nb = 8192;
    const int multi = (c->loss == EVT_LOSS_MULTIQUANTILE) ? 1 : 0;
    for (int k = 0; k < c->K; k++) {
        hipLaunchKernelGGL(k_quantile_keys, dim3((unsigned)nb), dim3(256), 0, c->stream, c->nidx, c->grad, c->N, c->NK, c->K + k, c->qkeys_a);
        HIPCHK(hipGetLastError());
        size_t bytes = c->qtemp_bytes;
        HIPCHK(hipcub::DeviceRadixSort::SortKeys(c->qtemp, bytes, (const unsigned long long *)c->qkeys_a, c->qkeys_b, (int)c->N, 0, sort_bits(c), c->stream));
        hipLaunchKernelGGL(k_leaf_quantile, dim3((unsigned)((c->nnodes + 255) / 256)), dim3(256), 0, c->stream, c->qkeys_b, c->N, c->status, c->node_sum,
                           c->qscale, c->NAg, c->nnodes, c->K, k, multi, c->alphas, p->eta, p->bagging_size, p->lambda, p->L2, c->tree.pred);
        HIPCHK(hipGetLastError());
    }
    return EVT_OK;
}
