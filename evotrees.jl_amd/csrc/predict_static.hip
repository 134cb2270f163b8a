// evt_predict_static: whole-model inference for callers that cannot allocate.
//
// evt_predict copies the model to the device and packs it into one 32-bit word per node in memory it allocates for the
// call.  Here the model already lives on the device in the reference's own arrays (Tree{L,K}, src/structs.jl:77-106,
// concatenated), a kernel packs it, and the packed words - the only memory the call needs beyond its inputs and its
// output - sit in a file-scope device array.  Nothing is allocated, copied or waited for: three kernels are queued on
// the caller's stream.
#include "evt_internal.h"

#include <mutex>

// header (256 bytes: word 0 = "model invalid" flag of the call in flight) + the packed node words
#define EVT_STATIC_HEADER_BYTES 256
static __device__ __align__(256) unsigned char scratch[EVT_STATIC_HEADER_BYTES + 4ull * EVT_STATIC_MAX_NODES];

// Each GPU holds its own copy of the array at its own address: looked up once per device, with that device current.
static std::mutex g_static_mu;
static unsigned char *g_static_ptr[64] = {nullptr};

static int static_scratch(unsigned char **out) {
    int dev = -1;
    HIPCHK(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) {
        evt_set_error("evt_predict_static: device %d out of range", dev);
        return EVT_ERR_ARG;
    }
    std::lock_guard<std::mutex> lock(g_static_mu);
    if (!g_static_ptr[dev]) {
        unsigned char *p = nullptr;
        const hipError_t e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            evt_set_error("hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
            return EVT_ERR_HIP;
        }
        g_static_ptr[dev] = p;
    }
    *out = g_static_ptr[dev];
    return EVT_OK;
}

// Start of a call: the flag of the previous call on this GPU is cleared by a kernel (a memset node must not be recorded
// into a captured graph), and the caller's status word starts at "ok".
__global__ void k_static_begin(int32_t *flag, int32_t *status) {
    *flag = 0;
    if (status) *status = EVT_OK;
}

// One block per tree (grid stride): checks the tree's place in the concatenated arrays and packs its nodes as the
// traversal reads them (feature | cond_bin << 16 | split << 24 | numeric << 25, leaves 0).  The same rules as the host
// packing of evt_predict: offsets start at 0, ascend strictly and end at total; a split node has both children inside
// its tree's arrays and a feature id in 1..nfeats.  Any violation raises the flag: the traversal then walks nothing.
__global__ __launch_bounds__(256) void k_static_pack(const int64_t *__restrict__ off, int ntrees, int64_t total, const int64_t *__restrict__ feat,
                                                    const uint8_t *__restrict__ cond_bin, const uint8_t *__restrict__ split,
                                                    const uint8_t *__restrict__ feattypes, int F, uint32_t *__restrict__ nodes, int32_t *flag,
                                                    int32_t *status) {
    for (int t = blockIdx.x; t < ntrees; t += gridDim.x) {
        const int64_t o = off[t], e = off[t + 1];
        const bool ok = o >= 0 && e > o && e <= total && (t > 0 || o == 0) && (t < ntrees - 1 || e == total);
        bool bad = !ok;
        if (ok) {
            const int64_t nn = e - o;
            for (int64_t n = 1 + threadIdx.x; n <= nn; n += 256) {
                uint32_t w = 0u;
                if (split[o + n - 1]) {
                    const int64_t f = feat[o + n - 1];
                    if (2 * n + 1 > nn || f < 1 || f > F) bad = true;
                    else w = evt_pack_node((int)f, cond_bin[o + n - 1], feattypes == nullptr || feattypes[f - 1] != 0);
                }
                nodes[o + n - 1] = w;
            }
        }
        if (bad) {
            *flag = 1;
            if (status) *status = EVT_ERR_ARG;
        }
    }
}

int launch_predict_model(hipStream_t s, const uint32_t *nodes, const float *leaf_pred, const int64_t *off, int ntrees, const uint8_t *xcm, int64_t N,
                         int K, int loss, int apply_link, float *out, const int32_t *skip_flag);

static bool device_visible(const void *p) {
    hipPointerAttribute_t attr;
    const bool ok = p && hipPointerGetAttributes(&attr, p) == hipSuccess && attr.devicePointer != nullptr &&
                    (attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeHost || attr.type == hipMemoryTypeManaged);
    (void)hipGetLastError();
    return ok;
}

extern "C" int evt_predict_static(void *stream, int64_t nobs, int32_t nfeats, const uint8_t *x_bin_dev, const uint8_t *feattypes_dev, int32_t loss,
                                  int32_t K, int32_t ntrees, int64_t total_nodes, const int64_t *tree_off_dev, const int64_t *feat_dev,
                                  const uint8_t *cond_bin_dev, const float *pred_dev, const uint8_t *split_dev, int32_t apply_link,
                                  float *out_dev, int32_t *status_dev) {
    ARGCHK(nobs >= 1 && nfeats >= 1 && nfeats <= 65535 && ntrees >= 1, "nobs, nfeats (<= 65535), ntrees must be >= 1");
    ARGCHK(K >= 1 && K <= EVT_MAX_K && loss >= 0 && loss <= EVT_LOSS_LAST, "invalid loss or K");
    ARGCHK(total_nodes >= ntrees, "total_nodes is smaller than the number of trees");
    if (total_nodes > (int64_t)EVT_STATIC_MAX_NODES) {
        evt_set_error("evt_predict_static: the model has %lld nodes, the static work area holds %lld (use evt_predict)", (long long)total_nodes,
                      (long long)EVT_STATIC_MAX_NODES);
        return EVT_ERR_ARG;
    }
    ARGCHK((apply_link & ~(1 | EVT_STATIC_TRUSTED)) == 0, "apply_link takes 0 or 1, plus EVT_STATIC_TRUSTED");
    const bool trusted = (apply_link & EVT_STATIC_TRUSTED) != 0;
    apply_link &= 1;
    ARGCHK(x_bin_dev && tree_off_dev && feat_dev && cond_bin_dev && pred_dev && split_dev && out_dev, "x_bin, the tree arrays and out must not be NULL");
    if (!trusted) { // nine pointer queries: a caller that vouches for its pointers (a serving loop, a capture) skips them
        ARGCHK(device_visible(x_bin_dev) && device_visible(tree_off_dev) && device_visible(feat_dev) && device_visible(cond_bin_dev) &&
                   device_visible(pred_dev) && device_visible(split_dev) && device_visible(out_dev),
               "evt_predict_static takes device memory only (x_bin, the tree arrays, out)");
        ARGCHK((!feattypes_dev || device_visible(feattypes_dev)) && (!status_dev || device_visible(status_dev)),
               "feattypes and status must be device memory (or NULL)");
    }
    unsigned char *ws = nullptr;
    const int r = static_scratch(&ws);
    if (r != EVT_OK) return r;
    int32_t *flag = reinterpret_cast<int32_t *>(ws);
    uint32_t *nodes = reinterpret_cast<uint32_t *>(ws + EVT_STATIC_HEADER_BYTES);
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(k_static_begin, dim3(1), dim3(1), 0, s, flag, status_dev);
    HIPCHK(hipGetLastError());
    hipLaunchKernelGGL(k_static_pack, dim3((unsigned)(ntrees < 1024 ? ntrees : 1024)), dim3(256), 0, s, tree_off_dev, ntrees, total_nodes, feat_dev,
                       cond_bin_dev, split_dev, feattypes_dev, nfeats, nodes, flag, status_dev);
    HIPCHK(hipGetLastError());
    return launch_predict_model(s, nodes, pred_dev, tree_off_dev, ntrees, x_bin_dev, nobs, K, loss, apply_link, out_dev, flag);
}
