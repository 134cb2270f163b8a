// Measurement aids: the rates the histogram kernel's two atomic paths are bounded by on this device.  They run no
// part of a fit; bench.py prints them beside the kernel's own figures.
//
//  * evt_lds_atomic_rate: 64-bit LDS atomics (ds_add_u64) as the histogram kernel issues them - 256 blocks of 1024
//    threads, one LDS array of 8192 words per block, 16 adds per lane and loop trip.
//  * evt_global_atomic_rate: 64-bit global atomics as the kernel's flush issues them - every block adds `words`
//    consecutive words of one slice, 8 consecutive words per 8 lanes.
#include "evt_internal.h"

// pattern 0: word = (t * 64 + bin) * 16 + lane % 16 - the kernel's layout for 128-byte records: the 16 lanes the LDS
//            serves per pass fall on 16 different bank pairs whatever their bins are;
// pattern 1: any of the 8192 words (random bank pairs).
// Lanes with lane % 16 >= lanes16 issue nothing (the kernel's 100-feature record leaves 3 lanes of 16 idle).
__global__ __launch_bounds__(1024) void k_probe_lds_atomics(const uint32_t *__restrict__ bins, int pattern, int lanes16, int iters,
                                                            unsigned long long *out) {
    __shared__ unsigned long long H[8192];
    const int tid = threadIdx.x, lane = tid & 63;
    for (int i = tid; i < 8192; i += blockDim.x) H[i] = 0ull;
    uint32_t b[16];
#pragma unroll
    for (int t = 0; t < 16; t++) b[t] = bins[((size_t)blockIdx.x * blockDim.x + tid) * 16 + t];
    __syncthreads();
    const bool on = (lane & 15) < lanes16;
    const unsigned long long v = ((unsigned long long)(tid + 1) << 16) + 1ull;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const uint32_t r = b[t] + (uint32_t)it * 7u;
            const uint32_t w = pattern == 0 ? ((((uint32_t)(t & 7) * 64u + (r & 63u)) * 16u + (uint32_t)(lane & 15)) & 8191u) : (r & 8191u);
            if (on) atomicAdd(&H[w], v);
        }
    }
    __syncthreads();
    if (tid == 0) out[blockIdx.x] = H[0] + H[8191];
}

extern "C" int evt_lds_atomic_rate(int32_t pattern, int32_t lanes16, int32_t iters, double *lane_atomics_per_s, double *wave_instr_per_s) {
    return guarded([&]() -> int {
    ARGCHK(lane_atomics_per_s && wave_instr_per_s, "output pointers must not be NULL");
    ARGCHK((pattern == 0 || pattern == 1) && lanes16 >= 1 && lanes16 <= 16 && iters >= 1 && iters <= 100000, "invalid arguments");
    int ndev = 0;
    int r = evt_device_count(&ndev);
    if (r != EVT_OK) return r;
    const int blocks = 256, threads = 1024;
    const size_t n = (size_t)blocks * threads * 16;
    std::vector<uint32_t> h(n);
    uint64_t s = 0x9E3779B97F4A7C15ull;
    for (size_t i = 0; i < n; i++) { // xorshift64*: any stream of bins does
        s ^= s >> 12; s ^= s << 25; s ^= s >> 27;
        h[i] = (uint32_t)((s * 0x2545F4914F6CDD1Dull) >> 40);
    }
    uint32_t *d = nullptr;
    unsigned long long *out = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    float ms = 0.0f;
    hipError_t e = hipMalloc((void **)&d, n * 4);
    if (e == hipSuccess) e = hipMalloc((void **)&out, blocks * 8);
    if (e == hipSuccess) e = hipMemcpy(d, h.data(), n * 4, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(k_probe_lds_atomics, dim3(blocks), dim3(threads), 0, 0, d, pattern, lanes16, iters, out); // warm-up
        e = hipEventRecord(e0, 0);
        hipLaunchKernelGGL(k_probe_lds_atomics, dim3(blocks), dim3(threads), 0, 0, d, pattern, lanes16, iters, out);
        if (e == hipSuccess) e = hipEventRecord(e1, 0);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (d) (void)hipFree(d);
    if (out) (void)hipFree(out);
    if (e != hipSuccess) {
        evt_set_error("LDS atomic probe failed: %s", hipGetErrorString(e));
        return EVT_ERR_HIP;
    }
    const double instr = (double)blocks * (threads / 64) * 16.0 * iters;
    *wave_instr_per_s = instr / ((double)ms * 1e-3);
    *lane_atomics_per_s = instr * 4.0 * lanes16 / ((double)ms * 1e-3);
    return EVT_OK;
    });
}

// every block adds `words` consecutive words of the slice `reps` times, starting at a word that depends on the block
// (as the histogram kernel's flush rotates its start): a wavefront instruction covers 64 consecutive words
__global__ __launch_bounds__(1024) void k_probe_global_atomics(unsigned long long *slice, int words, int reps) {
    const int tid = threadIdx.x;
    const int rot = (int)(((int64_t)blockIdx.x * 1031) % (words >> 6)) << 6;
    for (int r = 0; r < reps; r++) {
        for (int k = tid; k < words; k += blockDim.x) {
            int idx = k + rot;
            if (idx >= words) idx -= words;
            atomicAdd(&slice[idx], (unsigned long long)(idx + r + 1));
        }
    }
}

extern "C" int evt_global_atomic_rate(int32_t words, int32_t blocks, int32_t reps, double *atomics_per_s) {
    return guarded([&]() -> int {
    ARGCHK(atomics_per_s != nullptr, "output pointer must not be NULL");
    ARGCHK(words >= 64 && words <= (1 << 24) && (words & 63) == 0 && blocks >= 1 && blocks <= 65535 && reps >= 1 && reps <= 1000,
           "invalid arguments");
    int ndev = 0;
    int r = evt_device_count(&ndev);
    if (r != EVT_OK) return r;
    unsigned long long *slice = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    float ms = 0.0f;
    hipError_t e = hipMalloc((void **)&slice, (size_t)words * 8);
    if (e == hipSuccess) e = hipMemset(slice, 0, (size_t)words * 8);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(k_probe_global_atomics, dim3(blocks), dim3(1024), 0, 0, slice, words, 1); // warm-up
        e = hipEventRecord(e0, 0);
        hipLaunchKernelGGL(k_probe_global_atomics, dim3(blocks), dim3(1024), 0, 0, slice, words, reps);
        if (e == hipSuccess) e = hipEventRecord(e1, 0);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (slice) (void)hipFree(slice);
    if (e != hipSuccess) {
        evt_set_error("global atomic probe failed: %s", hipGetErrorString(e));
        return EVT_ERR_HIP;
    }
    *atomics_per_s = (double)words * blocks * reps / ((double)ms * 1e-3);
    return EVT_OK;
    });
}
