// Data-layout kernels: observation-major copy of x_bin, device binarize, small fills.
#include "evt_internal.h"

// One thread = one observation x one 16-feature group.  Reads are coalesced along rows of each
// column; the 16 bytes are written as one 128-bit store into the observation-major record.
// Bins outside 1..B raise the device error flag (the histogram kernels index LDS with them).
// Padding bytes of a record are set to 1, so that a kernel may index with them unchecked.
// Byte p of a record holds feature (p / PBL) * PU + p % PBL when p % PBL < PU, padding otherwise (evt_ctx::PBL).
__global__ __launch_bounds__(256) void k_transpose_validate(const uint8_t *__restrict__ xcm, uint8_t *__restrict__ xrm,
                                                           int64_t N, int F, int B, int RS, int PBL, int PU, int32_t *errflag) {
    int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int grp = blockIdx.y;
    if (row >= N) return;
    uint32_t w[4] = {0, 0, 0, 0};
    bool bad = false;
#pragma unroll
    for (int t = 0; t < 16; t++) {
        const int p = grp * 16 + t;
        const int f = (p / PBL) * PU + p % PBL;
        uint32_t b = 1; // padding reads as bin 1: always a valid histogram index
        if (p % PBL < PU && f < F) {
            b = xcm[(size_t)f * N + row];
            bad |= (b == 0 || b > (uint32_t)B);
        }
        w[t >> 2] |= b << (8 * (t & 3));
    }
    if (bad) atomicOr(errflag, 1);
    uint4 v = make_uint4(w[0], w[1], w[2], w[3]);
    *reinterpret_cast<uint4 *>(xrm + (size_t)row * RS + grp * 16) = v;
}

int launch_transpose_validate(evt_ctx *c) {
    dim3 grid((unsigned)((c->N + 255) / 256), (unsigned)(c->RS / 16));
    hipLaunchKernelGGL(k_transpose_validate, grid, dim3(256), 0, c->stream, c->xcm, c->xrm, c->N, c->F, c->B, c->RS, c->PBL, c->PU, c->errflag);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// Threshold bit planes of x_bin: word w of plane (f, b) holds, for rows 32 w .. 32 w + 31, the bit x_bin[row, f] <= b.
// One thread reads its 32 bins once and writes one word of each of the feature's B - 1 planes (consecutive threads,
// consecutive words).  Rows past the end read as bin 255: their bits are 0 in every plane.
__global__ __launch_bounds__(256) void k_build_planes(const uint8_t *__restrict__ xcm, uint32_t *__restrict__ planes, int64_t N, int B,
                                                     int64_t W) {
    const int64_t w = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int f = blockIdx.y;
    if (w >= W) return;
    const uint8_t *col = xcm + (size_t)f * N;
    uint32_t v[32];
#pragma unroll
    for (int k = 0; k < 32; k++) {
        const int64_t row = 32 * w + k;
        v[k] = row < N ? (uint32_t)col[row] : 255u;
    }
    uint32_t *out = planes + ((size_t)f * (B - 1)) * W + w;
    for (int b = 1; b < B; b++) {
        uint32_t word = 0;
#pragma unroll
        for (int k = 0; k < 32; k++) word |= (v[k] <= (uint32_t)b ? 1u : 0u) << k;
        out[(size_t)(b - 1) * W] = word;
    }
}

int launch_build_planes(evt_ctx *c) {
    dim3 grid((unsigned)((c->plane_words + 255) / 256), (unsigned)c->F);
    hipLaunchKernelGGL(k_build_planes, grid, dim3(256), 0, c->stream, c->xcm, c->planes, c->N, c->B, c->plane_words);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// Julia's isless on Float64 (the default order of searchsortedfirst): IEEE `<`, except that NaN sorts after everything and
// -0.0 before 0.0.
__device__ __forceinline__ bool jl_isless(double a, double b) {
    if (a != a) return false;
    if (b != b) return true;
    if (a == 0.0 && b == 0.0) return (__double_as_longlong(a) < 0) && (__double_as_longlong(b) >= 0);
    return a < b;
}

// searchsortedfirst(edges_j, x) = 1 + number of edges that are isless than x (src/fit-utils.jl:69); a NaN lands in the last bin.
__global__ __launch_bounds__(256) void k_binarize(const double *__restrict__ x, const double *__restrict__ edges,
                                                 const int32_t *__restrict__ edge_off, uint8_t *__restrict__ xcm, int64_t N,
                                                 int64_t ldx, int64_t ldo) {
    int j = blockIdx.y;
    int e0 = edge_off[j], ne = edge_off[j + 1] - e0;
    extern __shared__ double s_edges[];
    for (int t = threadIdx.x; t < ne; t += 256) s_edges[t] = edges[e0 + t];
    __syncthreads();
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < N; i += (int64_t)gridDim.x * 256) {
        double v = x[(size_t)j * ldx + i];
        int lo = 0, hi = ne;
        while (lo < hi) {
            int mid = (lo + hi) >> 1;
            if (jl_isless(s_edges[mid], v)) lo = mid + 1; else hi = mid;
        }
        xcm[(size_t)j * ldo + i] = (uint8_t)(lo + 1);
    }
}

// n rows of F columns: column j is read at x_dev + j * ldx and written at xcm + j * ldo
int launch_binarize_cols(hipStream_t s, const double *x_dev, const double *edges_dev, const int32_t *edge_off_dev, uint8_t *xcm, int64_t n,
                         int F, int64_t ldx, int64_t ldo) {
    int64_t nb = (n + 255) / 256;
    if (nb > 4096) nb = 4096;
    dim3 grid((unsigned)nb, (unsigned)F);
    hipLaunchKernelGGL(k_binarize, grid, dim3(256), 256 * sizeof(double), s, x_dev, edges_dev, edge_off_dev, xcm, n, ldx, ldo);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}
int launch_binarize(evt_ctx *c, const double *x_dev, const double *edges_dev, const int32_t *edge_off_dev) {
    return launch_binarize_cols(c->stream, x_dev, edges_dev, edge_off_dev, c->xcm, c->N, c->F, c->N, c->N);
}

__global__ __launch_bounds__(256) void k_iota(uint32_t *dst, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) dst[i] = (uint32_t)i;
}
int launch_iota(evt_ctx *c, uint32_t *dst, int64_t n) {
    int64_t nb = (n + 255) / 256;
    if (nb > 8192) nb = 8192;
    if (nb < 1) nb = 1;
    hipLaunchKernelGGL(k_iota, dim3((unsigned)nb), dim3(256), 0, c->stream, dst, n);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// Small device -> pinned host copies by a kernel (16-byte words; nbytes is a multiple of 16).  A stream-ordered
// hipMemcpyAsync goes through the copy engine, and handing the stream over to it and back stalls the kernels queued
// behind it for tens of microseconds; a kernel's stores over the bus do not.
__global__ __launch_bounds__(256) void k_copy_to_host(const uint4 *__restrict__ src, uint4 *__restrict__ dst, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) dst[i] = src[i];
}
int launch_copy_to_host(evt_ctx *c, const void *src_dev, void *dst_host_dev, size_t nbytes) {
    const int64_t n = (int64_t)(nbytes / 16);
    if (n <= 0) return EVT_OK;
    int64_t nb = (n + 255) / 256;
    if (nb > 64) nb = 64;
    hipLaunchKernelGGL(k_copy_to_host, dim3((unsigned)nb), dim3(256), 0, c->stream, static_cast<const uint4 *>(src_dev),
                       static_cast<uint4 *>(dst_host_dev), n);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// the same for small pinned host -> device uploads, in 4-byte words
__global__ __launch_bounds__(256) void k_copy_words(const uint32_t *__restrict__ src, uint32_t *__restrict__ dst, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) dst[i] = src[i];
}
int launch_copy_words(evt_ctx *c, const void *src, void *dst, size_t nbytes) {
    const int64_t n = (int64_t)(nbytes / 4);
    if (n <= 0) return EVT_OK;
    int64_t nb = (n + 255) / 256;
    if (nb > 64) nb = 64;
    hipLaunchKernelGGL(k_copy_words, dim3((unsigned)nb), dim3(256), 0, c->stream, static_cast<const uint32_t *>(src), static_cast<uint32_t *>(dst), n);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

__global__ __launch_bounds__(256) void k_fill_u32(uint32_t *dst, uint32_t v, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) dst[i] = v;
}
int launch_fill_u32(evt_ctx *c, uint32_t *dst, uint32_t v, int64_t n) {
    if (n <= 0) return EVT_OK;
    int64_t nb = (n + 255) / 256;
    if (nb > 8192) nb = 8192;
    hipLaunchKernelGGL(k_fill_u32, dim3((unsigned)nb), dim3(256), 0, c->stream, dst, v, n);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}
// zero-fill of a byte range whose size is a multiple of 4
int launch_fill_bytes(evt_ctx *c, void *dst, int64_t nbytes) { return launch_fill_u32(c, (uint32_t *)dst, 0u, nbytes / 4); }

// grad[NK-1, i] = w[i] (or 1): the weight row is written once (src/init.jl:173-174).
__global__ __launch_bounds__(256) void k_set_weight_row(float *grad, const float *w, int64_t N, int NK) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    float *g = grad + (size_t)NK * i;
    for (int k = 0; k < NK - 1; k++) g[k] = 0.0f;
    g[NK - 1] = w ? w[i] : 1.0f;
}
int launch_set_weight_row(evt_ctx *c, const float *w_dev) {
    hipLaunchKernelGGL(k_set_weight_row, dim3((unsigned)((c->N + 255) / 256)), dim3(256), 0, c->stream, c->grad, w_dev, c->N, c->NK);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// pred[:, i] = mu (+ offset[:, i])  (src/init.jl:168-170)
__global__ __launch_bounds__(256) void k_init_pred(float *pred, const float *mu, const float *offset, int64_t N, int K) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    for (int k = 0; k < K; k++) {
        float v = mu[k];
        if (offset) v += offset[(size_t)K * i + k];
        pred[(size_t)K * i + k] = v;
    }
}
int launch_init_pred(evt_ctx *c, const float *mu_dev, const float *offset_dev) {
    hipLaunchKernelGGL(k_init_pred, dim3((unsigned)((c->N + 255) / 256)), dim3(256), 0, c->stream, c->pred, mu_dev, offset_dev, c->N, c->K);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// Multi-class targets are level codes 1..K stored as Float32; the gradient and metric kernels index with them.
__global__ __launch_bounds__(256) void k_validate_classes(const float *__restrict__ y, int64_t N, int K, int32_t *errflag) {
    bool bad = false;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < N; i += (int64_t)gridDim.x * 256) {
        const float v = y[i];
        bad |= !(v >= 1.0f && v <= (float)K && v == floorf(v));
    }
    if (bad) atomicOr(errflag, 1);
}
int launch_validate_classes(evt_ctx *c) {
    int64_t nb = (c->N + 255) / 256;
    if (nb > 2048) nb = 2048;
    hipLaunchKernelGGL(k_validate_classes, dim3((unsigned)nb), dim3(256), 0, c->stream, c->y, c->N, c->K, c->errflag);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}
