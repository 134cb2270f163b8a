// Row partitioning and level bookkeeping, all device resident.
//
// split_set! (src/fit-utils.jl:93-312) is a stable partition of each split node's row-id segment;
// update_nodes_idx_kernel! (ext/EvoTreesKernelAbstractionsExt/fit-utils.jl:9-31) is the same
// decision written per row.  Here every node owns a contiguous segment [seg_start, seg_start+seg_len)
// of the row-id list; a split rewrites the segment in place order (lefts first, both sides keeping
// ascending row ids) into the other list buffer, so children are again contiguous segments.
// Segments are cut into chunks of EVT_CHUNK rows that never cross a node boundary:
//   count   : one block per chunk evaluates x_bin[row, feat] <= cond_bin, keeps the ballots,
//             counts lefts;
//   next    : one block scans the chunk counts, sets the children's segments, picks which child
//             is built (fewer rows; tie -> left, src/fit.jl:123-129) and writes the next level's
//             tables (active nodes, chunk prefix, build list); it is the last block of the scatter
//             kernel, except that inputs with thousands of chunks scan the counts in a kernel of
//             its own before the scatter;
//   scatter : one block per chunk moves row ids to their stable destination; chunks of nodes that
//             became leaves record the node id per row (and add the leaf value to the prediction).
// No host round trip is needed between levels.
#include "evt_internal.h"
#include <algorithm>

// largest i in [0, n) with pre[i] <= v   (pre ascending, pre[0] <= v): the number of such entries, less one.  Every
// wavefront counts them for itself, 64 entries per step, all loads independent: one trip to memory where a binary
// search makes log2(n) dependent ones - these blocks are short, so their chain of dependent loads is their run time.
__device__ __forceinline__ int find_owner(const int64_t *__restrict__ pre, int n, int64_t v) {
    const int lane = threadIdx.x & 63;
    int cnt = 0;
    for (int k0 = 0; k0 < n; k0 += 64) {
        const int k = k0 + lane;
        const bool hit = (k < n) && (pre[k < n ? k : 0] <= v);
        cnt += __popcll(__ballot(hit));
    }
    return cnt - 1;
}

struct PartArgs {
    const int64_t *hdr;
    const uint4 *cdesc; // per chunk: {node, first position, end of the node's segment, first chunk of the node}
    const int32_t *act_node;
    const int64_t *cprefix;
    const int32_t *status;
    const int64_t *seg_start;
    const int64_t *seg_len;
    const uint32_t *t_packed; // split nodes as one word: feature | cond_bin << 16 | split << 24 | numeric << 25
    const uint8_t *xcm;
    int64_t N;
    const uint32_t *is_cur;
    uint32_t *is_next;
    unsigned long long *flagw;
    int32_t *chunk_nleft;
    const int64_t *chunk_lpre;
    // leaf finalisation
    uint32_t *nidx;
    float *pred;
    const float *t_pred;
    int K, loss, fuse_pred, write_nidx;
    int stream_hint; // the binned matrix does not fit the last-level cache
    int fold;        // scatter: the level's bookkeeping block rides along and the blocks add up chunk counts themselves
    // threshold bit planes (nullptr: none): numeric splits read one bit of plane (feature, cond_bin) per row
    const uint32_t *planes;
    int64_t plane_words;
    int B;
    // scatter pass that also builds the next level's histograms (16-byte records)
    const uint8_t *xrm;
    const unsigned long long *gq;
    const uint16_t *jsmap;
    long long *hist;
    int64_t node_stride;
    int F, nfs, NAg;
    // last pass of a tree: the finished tree's arrays go to the host's pinned buffer in copy_blocks extra blocks
    const uint4 *copy_src;
    uint4 *copy_dst;
    int64_t copy_n;
    int copy_blocks;
};

// The word of the decision source that holds row `rid`: its bin byte, or - for a numeric split with bit planes - the
// plane word whose bit (rid & 31) says x_bin[rid, f] <= cond_bin.
template <bool NT>
__device__ __forceinline__ uint32_t load_decision(const uint8_t *__restrict__ col, const uint32_t *__restrict__ plane, uint32_t rid) {
    if (plane) {
        const uint32_t *p = plane + (rid >> 5);
        return NT ? __builtin_nontemporal_load(p) : *p;
    }
    const uint8_t *p = col + rid;
    return (uint32_t)(NT ? __builtin_nontemporal_load(p) : *p);
}
__device__ __forceinline__ bool decide_left(uint32_t v, bool use_plane, uint32_t rid, bool numeric, uint32_t cb) {
    if (use_plane) return (v >> (rid & 31u)) & 1u;
    return numeric ? (v <= cb) : (v == cb);
}

// NT: the streaming hint on the gathered bin bytes (a template parameter: a run-time branch between two otherwise
// identical loads is merged by the compiler, which drops the hint)
template <bool NT>
__global__ __launch_bounds__(256) void k_part_count(PartArgs A) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // the first descriptor is requested together with the level's chunk count (the grid never exceeds the table)
    uint4 cd = A.cdesc[blockIdx.x];
    const int64_t n_chunks = A.hdr[LH_N_CHUNKS];
    __shared__ int s_cnt[4];
    for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x, cd = A.cdesc[c < n_chunks ? c : 0]) {
        // the chunk's descriptor names its node and its positions: the row ids are requested together with the node's
        // state, one trip to memory after the descriptor
        const int n = (int)cd.x;
        const int64_t p0 = cd.y, pend = cd.z;
        constexpr int NI = EVT_CHUNK / 256;
        uint32_t rid[NI], xbv[NI];
#pragma unroll
        for (int it = 0; it < NI; it++) {
            const int64_t p = p0 + it * 256 + tid;
            rid[it] = A.is_cur[p < pend ? p : pend - 1];
        }
        // the node's split word is requested together with its state (and the row ids), not one trip later behind the
        // branch on the state: a node without a split holds 0 there, which is not used
        const int st = A.status[n];
        uint32_t nd = A.t_packed[n - 1];
        asm volatile("" : "+v"(nd));
        if (st != ST_SPLIT) {
            if (tid == 0) A.chunk_nleft[c] = 0;
            continue;
        }
        const int f = (int)(nd & 0xFFFFu) - 1;
        const uint32_t cb = (nd >> 16) & 0xFFu;
        const bool numeric = (nd & EVT_NODE_NUMERIC) != 0;
        const uint8_t *col = A.xcm + (size_t)f * A.N;
        const uint32_t *plane = (A.planes && numeric && cb >= 1u && cb < (uint32_t)A.B) ? A.planes + ((size_t)f * (A.B - 1) + (cb - 1)) * A.plane_words : nullptr;
        int cnt = 0;
        // a binned matrix larger than the last-level cache is gathered with the streaming hint: each byte's line would
        // displace data that is read again (row lists, gradient words) and is rarely hit a second time itself
#pragma unroll
        for (int it = 0; it < NI; it++) xbv[it] = load_decision<NT>(col, plane, rid[it]);
#pragma unroll
        for (int it = 0; it < NI; it++) {
            const int64_t p = p0 + it * 256 + tid;
            const bool flag = (p < pend) && decide_left(xbv[it], plane != nullptr, rid[it], numeric, cb);
            const unsigned long long bal = __ballot(flag);
            if (lane == 0) A.flagw[c * EVT_CHUNK_WORDS + it * 4 + wave] = bal;
            cnt += __popcll(bal);
        }
        if (lane == 0) s_cnt[wave] = cnt;
        __syncthreads();
        if (tid == 0) A.chunk_nleft[c] = s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3];
        __syncthreads();
    }
}

// ---- single-block scans -----------------------------------------------------------------------
// Exclusive prefix over the threads of the block (up to 1024); returns the prefix, *total gets the sum.
__device__ long long block_excl_scan(long long v, long long *total, long long *s_tmp /* [17] */) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    long long x = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        int lo = __shfl_up((int)(x & 0xffffffffll), o), hi = __shfl_up((int)(x >> 32), o);
        long long y = ((long long)hi << 32) | (unsigned int)lo;
        if (lane >= o) x += y;
    }
    __syncthreads(); // s_tmp may still be read from a previous call
    if (lane == 63) s_tmp[wave] = x;
    __syncthreads();
    if (tid == 0) {
        long long run = 0;
        const int nw = blockDim.x >> 6;
        for (int w = 0; w < nw; w++) { long long t = s_tmp[w]; s_tmp[w] = run; run += t; }
        s_tmp[16] = run;
    }
    __syncthreads();
    *total = s_tmp[16];
    return s_tmp[wave] + x - v;
}

struct NextArgs {
    const int64_t *hdr;
    const int32_t *act_node;
    const int64_t *cprefix;
    int32_t *status;
    int64_t *seg_start;
    int64_t *seg_len;
    const int32_t *chunk_nleft;
    int64_t *chunk_lpre;
    // next level
    int64_t *n_hdr;
    int32_t *n_act_node;
    int64_t *n_cprefix;
    int32_t *n_bnode;
    int64_t *n_bstart;
    int64_t *n_bprefix;
    int64_t *n_stats; // rows the next level builds (the level's slot of the per-tree counts; the histogram kernel writes the same figure when it runs)
    int64_t seg_cost; // cost units added per build node in the histogram kernel's span space
};

// Two exclusive prefixes in one pass (same shape as block_excl_scan); s_tmp holds 34 values.
__device__ void block_excl_scan2(long long va, long long vb, long long *pa, long long *pb, long long *ta, long long *tb, long long *s_tmp) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    long long xa = va, xb = vb;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int al = __shfl_up((int)(xa & 0xffffffffll), o), ah = __shfl_up((int)(xa >> 32), o);
        const int bl = __shfl_up((int)(xb & 0xffffffffll), o), bh = __shfl_up((int)(xb >> 32), o);
        if (lane >= o) {
            xa += ((long long)ah << 32) | (unsigned int)al;
            xb += ((long long)bh << 32) | (unsigned int)bl;
        }
    }
    __syncthreads(); // s_tmp may still be read from a previous call
    if (lane == 63) {
        s_tmp[wave] = xa;
        s_tmp[17 + wave] = xb;
    }
    __syncthreads();
    if (tid < 2) {
        long long *t = s_tmp + 17 * tid;
        long long run = 0;
        const int nw = blockDim.x >> 6;
        for (int w = 0; w < nw; w++) { long long x = t[w]; t[w] = run; run += x; }
        t[16] = run;
    }
    __syncthreads();
    *ta = s_tmp[16];
    *tb = s_tmp[33];
    *pa = s_tmp[wave] + xa - va;
    *pb = s_tmp[17 + wave] + xb - vb;
}

// One block turns the chunk counts of a level into the next level's tables (children's segments, which child is
// built, active nodes, chunk prefix, build list), in two halves: the scan of the chunk counts (A) and the tables (B).  It
// rides along as the last block of the scatter kernel, whose other blocks need nothing from it: they add up the chunk
// counts of their own node themselves - or, with thousands of chunks per level, read the counts scanned by half A in a
// kernel of its own just before, while half B runs beside them.  Loads that do not depend on each other are issued
// together (fixed-trip loops over clamped indices instead of data-dependent ones).
// A: exclusive scan of the chunks' left counts (chunk_lpre[c] = lefts in the chunks before c, chunk_lpre[n_chunks] = all)
__device__ void chunk_scan_block(const NextArgs &A, long long *s_tmp /* [34] */) {
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int64_t n_chunks = A.hdr[LH_N_CHUNKS];
    long long total;
    {
        constexpr int SP = 8;
        const int64_t span = (n_chunks + nthr - 1) / nthr;
        const int64_t c0 = (int64_t)tid * span, c1 = (c0 + span < n_chunks) ? c0 + span : n_chunks;
        if (span <= SP) {
            int v[SP];
#pragma unroll
            for (int k = 0; k < SP; k++) {
                const int64_t c = c0 + k;
                const int x = A.chunk_nleft[c < c1 ? c : 0];
                v[k] = c < c1 ? x : 0;
            }
            long long s = 0;
#pragma unroll
            for (int k = 0; k < SP; k++) s += v[k];
            long long pre = block_excl_scan(s, &total, s_tmp);
#pragma unroll
            for (int k = 0; k < SP; k++) {
                if (c0 + k < c1) A.chunk_lpre[c0 + k] = pre;
                pre += v[k];
            }
        } else {
            long long s = 0;
            for (int64_t c = c0; c < c1; c++) s += A.chunk_nleft[c];
            long long pre = block_excl_scan(s, &total, s_tmp);
            for (int64_t c = c0; c < c1; c++) { A.chunk_lpre[c] = pre; pre += A.chunk_nleft[c]; }
        }
        if (tid == 0) A.chunk_lpre[n_chunks] = total;
    }
}

// B: children segments + three scans over the active nodes (children count, chunks, build rows) -> the next level's tables
__device__ void level_tables_block(const NextArgs &A, long long *s_tmp /* [34] */) {
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int n_act = (int)A.hdr[LH_N_ACT];
    const int span = (n_act + nthr - 1) / nthr;
    const int i0 = tid * span, i1 = (i0 + span < n_act) ? i0 + span : n_act;
    long long s_pos = 0, s_chunks = 0, s_brows = 0;
    for (int i = i0; i < i1; i++) {
        const int n = A.act_node[i];
        const int64_t cp0 = A.cprefix[i], cp1 = A.cprefix[i + 1];
        const int st = A.status[n];
        const int64_t len = A.seg_len[n], start = A.seg_start[n];
        const int64_t nl = A.chunk_lpre[cp1] - A.chunk_lpre[cp0];
        if (st != ST_SPLIT) continue;
        const int64_t nr = len - nl;
        A.seg_start[2 * n] = start;
        A.seg_len[2 * n] = nl;
        A.seg_start[2 * n + 1] = start + nl;
        A.seg_len[2 * n + 1] = nr;
        const bool build_left = nr >= nl; // the smaller child is built, tie -> left (src/fit.jl:123-129)
        A.status[2 * n] = build_left ? ST_BUILD : ST_SUBTRACT;
        A.status[2 * n + 1] = build_left ? ST_SUBTRACT : ST_BUILD;
        s_pos += 1;
        s_chunks += (nl + EVT_CHUNK - 1) / EVT_CHUNK + (nr + EVT_CHUNK - 1) / EVT_CHUNK;
        s_brows += (build_left ? nl : nr) + A.seg_cost;
    }
    // children count (low 24 bits) and chunk count share one scan; the build rows take the other
    long long t_pc, t_brows, p_pc, p_brows;
    block_excl_scan2((s_chunks << 24) | s_pos, s_brows, &p_pc, &p_brows, &t_pc, &t_brows, s_tmp);
    long long p_pos = p_pc & 0xFFFFFF, p_chunks = p_pc >> 24;
    const long long t_pos = t_pc & 0xFFFFFF, t_chunks = t_pc >> 24;
    for (int i = i0; i < i1; i++) {
        const int n = A.act_node[i];
        if (A.status[n] != ST_SPLIT) continue;
        const int64_t nl = A.seg_len[2 * n], nr = A.seg_len[2 * n + 1];
        const int64_t start = A.seg_start[2 * n];
        const bool build_left = nr >= nl;
        A.n_act_node[2 * p_pos] = 2 * n;
        A.n_act_node[2 * p_pos + 1] = 2 * n + 1;
        A.n_cprefix[2 * p_pos] = p_chunks;
        A.n_cprefix[2 * p_pos + 1] = p_chunks + (nl + EVT_CHUNK - 1) / EVT_CHUNK;
        A.n_bnode[p_pos] = build_left ? 2 * n : 2 * n + 1;
        A.n_bstart[p_pos] = build_left ? start : start + nl;
        A.n_bprefix[p_pos] = p_brows;
        p_pos += 1;
        p_chunks += (nl + EVT_CHUNK - 1) / EVT_CHUNK + (nr + EVT_CHUNK - 1) / EVT_CHUNK;
        p_brows += (build_left ? nl : nr) + A.seg_cost;
    }
    if (tid == 0) {
        A.n_cprefix[2 * t_pos] = t_chunks;
        A.n_bprefix[t_pos] = t_brows;
        A.n_hdr[LH_N_ACT] = 2 * t_pos;
        A.n_hdr[LH_N_CHUNKS] = t_chunks;
        A.n_hdr[LH_N_BUILD] = t_pos;
        A.n_hdr[LH_TOTAL_BUILD] = t_brows;
        if (A.n_stats) *A.n_stats = t_brows - t_pos * A.seg_cost;
    }
}

// both halves by one block: the form that rides along in the scatter kernel for inputs of up to a thousand chunks per level
__device__ void level_next_block(const NextArgs &A, long long *s_tmp /* [34] */) {
    chunk_scan_block(A, s_tmp);
    __syncthreads();
    level_tables_block(A, s_tmp);
}

// Inputs with thousands of chunks per level: the scan of the chunk counts is a kernel of its own (one block of 1024 threads)
// between the count and the scatter pass - every scatter block adding up its node's chunk counts would cost more than this
// launch - and only the next level's tables, which no scatter block reads, ride along in the scatter kernel.
__global__ __launch_bounds__(1024) void k_chunk_scan(NextArgs A) {
    __shared__ long long s_tmp[34];
    chunk_scan_block(A, s_tmp);
}

// HNA > 0: the pass also builds the next level's histograms (update_hist!, src/fit-utils.jl:345-394) for inputs whose
// levels are chains of short kernels: 16-byte records (at most 16 features, one lane per row) and few chunks.  A block
// knows its node's left and right sizes, hence which child is built (the smaller, tie -> left, src/fit.jl:123-129); the rows
// of its chunk that go there are added into an LDS histogram of HNA channels (PACK: gradient and row count share channel
// 0's word) and the chunk's partial histogram is added to the child's zero-initialised slice with global atomics.  No
// histogram kernel runs below the root then.
template <int HNA, bool PACK>
__global__ __launch_bounds__(256) void k_part_scatter(PartArgs A, NextArgs NX) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    __shared__ long long s_tmp[34];
    extern __shared__ unsigned long long s_H[]; // HNA > 0: [HNA][sampled features][bins]
    // fold 1: the level's bookkeeping rides along whole and the blocks add up their node's chunk counts themselves;
    // fold 2: the chunk counts were scanned by k_chunk_scan, only the next level's tables ride along
    const bool fold = A.fold == 1;
    if (blockIdx.x == gridDim.x - 1) { // the level's bookkeeping, beside the blocks that move the rows
        if (fold) level_next_block(NX, s_tmp);
        else level_tables_block(NX, s_tmp);
        return;
    }
    // the 16 features of a record -> LDS word of their first bin (bins are 1-based); vmask bit t: feature t is sampled
    int off[16];
    unsigned vmask = 0;
    const int plane = (HNA > 0) ? A.nfs * A.B : 0;
    if constexpr (HNA > 0) {
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int sl = (t < A.F) ? (int)A.jsmap[t] : 0xFFFF;
            const bool ok = sl != 0xFFFF;
            off[t] = ok ? sl * A.B - 1 : 0;
            vmask |= ok ? (1u << t) : 0u;
        }
        for (int i = tid; i < HNA * plane; i += 256) s_H[i] = 0ull;
    }
    const int64_t G = gridDim.x - 1;
    uint4 cd = A.cdesc[blockIdx.x];
    const int64_t n_chunks = A.hdr[LH_N_CHUNKS];
    __shared__ unsigned long long s_w[EVT_CHUNK_WORDS];
    __shared__ int s_pre[EVT_CHUNK_WORDS];
    for (int64_t c = blockIdx.x; c < n_chunks; c += G, cd = A.cdesc[c < n_chunks ? c : 0]) {
        const int n = (int)cd.x;
        const int64_t p0 = cd.y, pend = cd.z, c0 = cd.w;
        const int64_t cl = c - c0;
        const int64_t seg = p0 - cl * EVT_CHUNK;
        // everything the chunk needs is requested at once, behind the descriptor: node state, the count pass's ballots
        // and prefixes, the left child's size and the row ids (positions past the end read the segment's last row)
        const int st = A.status[n];
        const unsigned long long fw = A.flagw[c * EVT_CHUNK_WORDS + (tid & (EVT_CHUNK_WORDS - 1))];
        // lefts of this node before this chunk, and in all of the node: the block adds up the node's chunk counts itself
        // (a node's chunks are few, or the sums are spread over the 256 threads)
        const int64_t c1 = c0 + (pend - seg + EVT_CHUNK - 1) / EVT_CHUNK;
        long long sum_before = 0, sum_node = 0;
        if (fold) {
            for (int64_t k = c0 + tid; k < c1; k += 256) {
                const int v = A.chunk_nleft[k];
                sum_node += v;
                sum_before += (k < c) ? v : 0;
            }
        } else { // the chunk counts were scanned before this kernel (the children's sizes are being written beside it)
            const long long l0 = A.chunk_lpre[c0];
            sum_before = A.chunk_lpre[c] - l0;
            sum_node = A.chunk_lpre[c1] - l0;
        }
        constexpr int NI = EVT_CHUNK / 256;
        uint32_t rid[NI];
#pragma unroll
        for (int it = 0; it < NI; it++) {
            const int64_t p = p0 + it * 256 + tid;
            rid[it] = A.is_cur[p < pend ? p : pend - 1];
        }
        // HNA > 0: the record and the gradient words of every row are requested along with everything else, before it is
        // known which child is built and which rows go there (16 + 4..8 bytes per row, off the block's chain of dependent loads)
        uint4 rec[HNA > 0 ? NI : 1];
        unsigned long long gw[HNA > 0 ? NI : 1][HNA > 0 ? HNA : 1];
        if constexpr (HNA > 0) {
#pragma unroll
            for (int it = 0; it < NI; it++) {
                rec[it] = *reinterpret_cast<const uint4 *>(A.xrm + (size_t)rid[it] * 16);
#pragma unroll
                for (int a = 0; a < HNA; a++) gw[it][a] = evt_load_gq<PACK>(A.gq, A.N, a, rid[it]);
            }
        }
        if (st == ST_SPLIT) {
            if (fold) {
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) {
                    sum_before += __shfl_xor(sum_before, o);
                    sum_node += __shfl_xor(sum_node, o);
                }
                if (lane == 0) { s_tmp[wave] = sum_before; s_tmp[4 + wave] = sum_node; }
            }
            if (tid < EVT_CHUNK_WORDS) s_w[tid] = fw;
            __syncthreads();
            if (tid == 0) {
                int run = 0;
                for (int t = 0; t < EVT_CHUNK_WORDS; t++) { s_pre[t] = run; run += __popcll(s_w[t]); }
            }
            __syncthreads();
            const int64_t lbase = fold ? s_tmp[0] + s_tmp[1] + s_tmp[2] + s_tmp[3] : sum_before; // lefts of this node before this chunk
            const int64_t nl_node = fold ? s_tmp[4] + s_tmp[5] + s_tmp[6] + s_tmp[7] : sum_node;
            const int64_t dstL = seg + lbase;
            const int64_t dstR = seg + nl_node + (cl * EVT_CHUNK - lbase);
            unsigned onmask = 0; // rows of this thread that go to the built child
            bool build_left = false;
            if constexpr (HNA > 0) {
                build_left = (pend - seg) - nl_node >= nl_node;
#pragma unroll
                for (int it = 0; it < NI; it++) {
                    const int64_t p = p0 + it * 256 + tid;
                    const bool flag = (s_w[it * 4 + wave] >> lane) & 1ull;
                    if (p < pend && flag == build_left) onmask |= 1u << it;
                }
            }
#pragma unroll
            for (int it = 0; it < NI; it++) {
                const int64_t p = p0 + it * 256 + tid;
                if (p < pend) {
                    const int wi = it * 4 + wave;
                    const unsigned long long word = s_w[wi];
                    const int lrank = s_pre[wi] + __popcll(word & ((1ull << lane) - 1ull));
                    const bool flag = (word >> lane) & 1ull;
                    const int within = it * 256 + tid;
                    const int64_t d = flag ? (dstL + lrank) : (dstR + (within - lrank));
                    A.is_next[d] = rid[it];
                }
            }
            if constexpr (HNA > 0) {
#pragma unroll
                for (int it = 0; it < NI; it++) {
                    if (onmask & (1u << it)) {
                        const uint32_t wds[4] = {rec[it].x, rec[it].y, rec[it].z, rec[it].w};
#pragma unroll
                        for (int t = 0; t < 16; t++) {
                            if (vmask & (1u << t)) {
                                const int idx = off[t] + (int)((wds[t >> 2] >> (8 * (t & 3))) & 0xFFu);
#pragma unroll
                                for (int a = 0; a < HNA; a++) atomicAdd(&s_H[a * plane + idx], gw[it][a]);
                            }
                        }
                    }
                }
                __syncthreads();
                // the chunk's partial histogram joins the built child's slice hist[node][slot][channel][bin]; chunks start
                // at different words so that concurrent flushes of one node do not queue on the same addresses
                unsigned long long *hn = reinterpret_cast<unsigned long long *>(A.hist) + (int64_t)(2 * n + (build_left ? 0 : 1) - 1) * A.node_stride;
                const int nwords = HNA * plane;
                const int rot = (int)((c * 1021) % nwords);
                for (int k = tid; k < nwords; k += 256) {
                    int idx = k + rot;
                    if (idx >= nwords) idx -= nwords;
                    const unsigned long long w = s_H[idx];
                    if (w != 0ull) {
                        s_H[idx] = 0ull;
                        const int a = idx / plane;
                        const int rem = idx - a * plane;
                        const int sl = rem / A.B;
                        const int bin = rem - sl * A.B;
                        unsigned long long *base = hn + ((int64_t)sl * A.NAg) * A.B + bin;
                        if (PACK && a == 0) {
                            const long long gsum = (long long)w >> EVT_PACK_CNT_BITS;
                            const unsigned long long cnt = w & ((1ull << EVT_PACK_CNT_BITS) - 1ull);
                            if (gsum != 0) atomicAdd(base, (unsigned long long)gsum);
                            atomicAdd(base + (int64_t)(A.NAg - 1) * A.B, cnt);
                        } else {
                            atomicAdd(base + (int64_t)a * A.B, w);
                        }
                    }
                }
            }
            __syncthreads();
        } else if (st == ST_LEAF && (A.write_nidx || A.fuse_pred)) {
            // rows of a node that stops here: record the node id; add the leaf value
            // (predict!, src/predict.jl:1-46: plain add / clamp(-15,15) / floor -15 on scale rows)
            const int K = A.K;
#pragma unroll
            for (int it = 0; it < EVT_CHUNK / 256; it++) {
                const int64_t p = p0 + it * 256 + tid;
                if (p < pend) {
                    const uint32_t row = rid[it];
                    if (A.write_nidx) A.nidx[row] = (uint32_t)n;
                    if (A.fuse_pred) {
                        float *pr = A.pred + (size_t)K * row;
                        const float *lp = A.t_pred + (size_t)K * (n - 1);
                        evt_add_leaf(pr, lp, K, A.loss);
                    }
                }
            }
        }
    }
}

// Last pass of a tree: rows of the deepest split level go straight to their leaf.  For a node that split,
// the child is decided from x_bin[row, feat] exactly as the partition would (left iff <= cond_bin, or ==
// for a categorical feature) but the row list is not rewritten: nothing reads it afterwards.  Each row
// gets its leaf's value added to the prediction (predict!, src/predict.jl:1-46) and, on request, its
// node id recorded.
template <bool NT>
__global__ __launch_bounds__(256) void k_final_fused(PartArgs A) {
    const int tid = threadIdx.x;
    const int64_t G = (int64_t)gridDim.x - A.copy_blocks;
    if ((int64_t)blockIdx.x >= G) {
        // the tree's arrays are complete (this is the tree's last kernel and writes none of them): their way back to the
        // host rides along instead of taking a launch of its own
        for (int64_t i = ((int64_t)blockIdx.x - G) * 256 + tid; i < A.copy_n; i += (int64_t)A.copy_blocks * 256) A.copy_dst[i] = A.copy_src[i];
        return;
    }
    uint4 cd = A.cdesc[blockIdx.x];
    const int64_t n_chunks = A.hdr[LH_N_CHUNKS];
    const int K = A.K;
    for (int64_t c = blockIdx.x; c < n_chunks; c += G, cd = A.cdesc[c < n_chunks ? c : 0]) {
        const int n = (int)cd.x;
        const int64_t p0 = cd.y, pend = cd.z;
        constexpr int NI = EVT_CHUNK / 256;
        uint32_t rid[NI], xbv[NI];
        float prv[NI];
#pragma unroll
        for (int it = 0; it < NI; it++) {
            const int64_t p = p0 + it * 256 + tid;
            rid[it] = A.is_cur[p < pend ? p : pend - 1];
        }
        const int st = A.status[n];
        uint32_t nd = A.t_packed[n - 1]; // requested with the state, not behind the branch on it
        asm volatile("" : "+v"(nd));
        if (st != ST_SPLIT && st != ST_LEAF) continue;
        const bool is_split = (st == ST_SPLIT);
        int f = 0;
        uint32_t cb = 0;
        bool numeric = true;
        if (is_split) {
            f = (int)(nd & 0xFFFFu) - 1;
            cb = (nd >> 16) & 0xFFu;
            numeric = (nd & EVT_NODE_NUMERIC) != 0;
        }
        const uint8_t *col = A.xcm + (size_t)f * A.N;
        const uint32_t *plane = (A.planes && is_split && numeric && cb >= 1u && cb < (uint32_t)A.B) ? A.planes + ((size_t)f * (A.B - 1) + (cb - 1)) * A.plane_words : nullptr;
        // every request of the chunk goes out before the first result is used: row ids (above), then bin bytes or plane
        // words, then (one output) the predictions; positions past the end read the segment's last row and are not written
#pragma unroll
        for (int it = 0; it < NI; it++) xbv[it] = is_split ? load_decision<NT>(col, plane, rid[it]) : 0u;
        const bool fast1 = A.fuse_pred && K == 1;
        if (fast1) {
#pragma unroll
            for (int it = 0; it < NI; it++) prv[it] = A.pred[rid[it]];
        }
#pragma unroll
        for (int it = 0; it < NI; it++) {
            const int64_t p = p0 + it * 256 + tid;
            if (p < pend) {
                const uint32_t row = rid[it];
                int leaf = n;
                if (is_split) {
                    const bool left = decide_left(xbv[it], plane != nullptr, row, numeric, cb);
                    leaf = 2 * n + (left ? 0 : 1);
                }
                if (A.write_nidx) A.nidx[row] = (uint32_t)leaf;
                if (fast1) {
                    const float s = prv[it] + A.t_pred[leaf - 1];
                    A.pred[row] = (A.loss == EVT_LOSS_LOGLOSS) ? fminf(fmaxf(s, -15.0f), 15.0f) : s;
                    continue;
                }
                if (A.fuse_pred) {
                    float *pr = A.pred + (size_t)K * row;
                    const float *lp = A.t_pred + (size_t)K * (leaf - 1);
                    evt_add_leaf(pr, lp, K, A.loss);
                }
            }
        }
    }
}

// Start of a tree: zero the Tree arrays (Tree{L,K}(depth), src/structs.jl:97-106) and node states,
// make the root the only active (build) node over rows [0, n_is), zero its histogram slice.
struct BeginArgs {
    TreeDev tree;
    int32_t *status;
    int64_t *seg_start;
    int64_t *seg_len;
    int64_t *hdr;
    int32_t *act_node;
    int64_t *cprefix;
    int32_t *bnode;
    int64_t *bstart;
    int64_t *bprefix;
    long long *hist;
    int64_t *stats;
    int64_t n_is;
    const int64_t *n_is_dev; // non-null: the number of sampled rows is the total the mask compaction left on the device
    int64_t seg_cost;
    int64_t root_words;
    int nnodes, K, D;
    // the tree's column sample and its inverse map, from the pinned staging buffer to the device copies (0 words: unchanged)
    const uint32_t *js_src, *map_src;
    uint32_t *js_dst, *map_dst;
    int js_words, map_words;
};

// One block prepares a tree: empty Tree arrays, node states, the root's histogram slice, the first level's tables, the
// column sample.  A kernel of its own for a tree on every row; with a row sample it is the last block of the kernel that
// compacts the sampled rows (k_mask_scatter), which hands it the number of rows kept.
__device__ void tree_begin_block(BeginArgs A) {
    const int tid = threadIdx.x, nthr = blockDim.x;
    for (int n = tid; n < A.nnodes; n += nthr) {
        A.tree.feat[n] = 0;
        A.tree.cond_bin[n] = 0;
        A.tree.w[n] = 0.0f;
        A.tree.gain[n] = 0.0f;
        A.tree.split[n] = 0;
        A.tree.packed[n] = 0u;
        for (int k = 0; k < A.K; k++) A.tree.pred[(int64_t)A.K * n + k] = 0.0f;
    }
    for (int n = tid; n < A.nnodes + 2; n += nthr) A.status[n] = ST_INACTIVE;
    for (int64_t i = tid; i < A.root_words; i += nthr) A.hist[i] = 0;
    for (int d = tid; d <= A.D; d += nthr) A.stats[d] = 0;
    for (int i = tid; i < A.js_words; i += nthr) A.js_dst[i] = A.js_src[i];
    for (int i = tid; i < A.map_words; i += nthr) A.map_dst[i] = A.map_src[i];
    __syncthreads();
    if (tid == 0) {
        if (A.n_is_dev) A.n_is = *A.n_is_dev;
        A.stats[0] = A.n_is; // read back with the tree: the host learns how many rows the mask kept
        A.status[1] = ST_BUILD;
        A.seg_start[1] = 0;
        A.seg_len[1] = A.n_is;
        A.hdr[LH_N_ACT] = 1;
        A.hdr[LH_N_CHUNKS] = (A.n_is + EVT_CHUNK - 1) / EVT_CHUNK;
        A.hdr[LH_N_BUILD] = 1;
        A.hdr[LH_TOTAL_BUILD] = A.n_is + A.seg_cost;
        A.act_node[0] = 1;
        A.cprefix[0] = 0;
        A.cprefix[1] = (A.n_is + EVT_CHUNK - 1) / EVT_CHUNK;
        A.bnode[0] = 1;
        A.bstart[0] = 0;
        A.bprefix[0] = 0;
        A.bprefix[1] = A.n_is + A.seg_cost;
    }
}

__global__ __launch_bounds__(1024) void k_tree_begin(BeginArgs A) { tree_begin_block(A); }

// ---- row subsampling: is = rows with mask <= cond, ascending (src/subsample.jl:6-38) -----------
__device__ __forceinline__ int wave_sum_i32(int v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// A thread takes 8 consecutive mask bytes (one load); the 8 flags of 8 neighbouring threads make one 64-row flag word.
// DRAW: the bytes are not read but drawn here and written to `mask` on the way: the mask's 8-byte word w is output w of
// SplitMix64 (Steele, Lea, Flood 2014: a Weyl sequence with increment 0x9E3779B97F4A7C15 passed through two
// multiply-xorshift rounds) started at state `seed`, stored little end first - byte i of the mask is bits 8*(i%8).. of output
// i/8.  Stands in for rand!(rng, mask) of src/subsample.jl:7 when the caller accepts a counter-based stream keyed by one 64-bit
// draw of its own generator per tree.
template <bool DRAW>
__global__ __launch_bounds__(256) void k_mask_count(uint8_t *mask, uint8_t cond, int64_t N, int64_t n_chunks,
                                                   unsigned long long *flagw, int32_t *chunk_nleft, unsigned long long seed) {
    static_assert(EVT_CHUNK == 2048 && EVT_CHUNK_WORDS == 32, "a chunk is 256 threads x 8 bytes");
    const int tid = threadIdx.x;
    __shared__ unsigned long long s_w[EVT_CHUNK_WORDS];
    uint8_t *s_b = reinterpret_cast<uint8_t *>(s_w);
    for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
        const int64_t p0 = c * EVT_CHUNK + (int64_t)tid * 8;
        unsigned long long v = ~0ull; // bytes past the end read as 255
        if (DRAW) {
            unsigned long long z = seed + (unsigned long long)((p0 >> 3) + 1) * 0x9E3779B97F4A7C15ull;
            z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
            z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
            z ^= z >> 31;
            v = z;
            if (p0 + 8 <= N) {
                *reinterpret_cast<unsigned long long *>(mask + p0) = z;
            } else {
                for (int j = 0; p0 + j < N; j++) mask[p0 + j] = (uint8_t)(z >> (8 * j));
            }
        } else if (p0 + 8 <= N) {
            v = *reinterpret_cast<const unsigned long long *>(mask + p0);
        } else {
            for (int j = 0; j < 8; j++)
                if (p0 + j < N) v = (v & ~(0xFFull << (8 * j))) | ((unsigned long long)mask[p0 + j] << (8 * j));
        }
        unsigned flags = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const bool keep = (p0 + j < N) && ((uint8_t)(v >> (8 * j)) <= cond);
            flags |= keep ? (1u << j) : 0u;
        }
        s_b[tid] = (uint8_t)flags; // little end first: byte t of the chunk's flag words covers rows 8t .. 8t+7
        __syncthreads();
        if (tid < 64) {
            const unsigned long long w = tid < EVT_CHUNK_WORDS ? s_w[tid] : 0ull;
            if (tid < EVT_CHUNK_WORDS) flagw[c * EVT_CHUNK_WORDS + tid] = w;
            int cnt = __popcll(w);
            cnt = wave_sum_i32(cnt);
            if (tid == 0) chunk_nleft[c] = cnt;
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(1024) void k_mask_scan(const int32_t *chunk_nleft, int64_t *chunk_lpre, int64_t n_chunks) {
    __shared__ long long s_tmp[17];
    const int tid = threadIdx.x;
    const int64_t span = (n_chunks + 1023) / 1024;
    const int64_t c0 = (int64_t)tid * span, c1 = (c0 + span < n_chunks) ? c0 + span : n_chunks;
    long long s = 0, total;
    for (int64_t c = c0; c < c1; c++) s += chunk_nleft[c];
    long long pre = block_excl_scan(s, &total, s_tmp);
    for (int64_t c = c0; c < c1; c++) { chunk_lpre[c] = pre; pre += chunk_nleft[c]; }
    if (tid == 0) chunk_lpre[n_chunks] = total;
}

// SELF: no k_mask_scan has run - every block adds up the counts of the chunks before its own (a few hundred values:
// cheaper than the launch).
// The last block of the grid prepares the tree that is grown on the sample (tree_begin_block), with the number of rows kept.
template <bool SELF>
__global__ __launch_bounds__(256) void k_mask_scatter(int64_t N, int64_t n_chunks, const unsigned long long *flagw,
                                                     const int32_t *chunk_nleft, int64_t *chunk_lpre, uint32_t *is_out, BeginArgs B) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    __shared__ unsigned long long s_w[EVT_CHUNK_WORDS];
    __shared__ int s_pre[EVT_CHUNK_WORDS];
    __shared__ int s_sum[4];
    const int64_t G = (int64_t)gridDim.x - 1;
    if ((int64_t)blockIdx.x == G) {
        int64_t kept;
        if (SELF) { // no scan has run: the chunk counts (a thousand at most) are added up here
            int part = 0;
            for (int64_t k = tid; k < n_chunks; k += 256) part += chunk_nleft[k];
            part = wave_sum_i32(part);
            if (lane == 0) s_sum[wave] = part;
            __syncthreads();
            kept = (int64_t)s_sum[0] + s_sum[1] + s_sum[2] + s_sum[3];
        } else {
            kept = chunk_lpre[n_chunks];
        }
        B.n_is = kept;
        B.n_is_dev = nullptr;
        tree_begin_block(B);
        return;
    }
    for (int64_t c = blockIdx.x; c < n_chunks; c += G) {
        if (tid < EVT_CHUNK_WORDS) s_w[tid] = flagw[c * EVT_CHUNK_WORDS + tid];
        int64_t base;
        if (SELF) {
            int part = 0;
            for (int64_t k = tid; k < c; k += 256) part += chunk_nleft[k];
            part = wave_sum_i32(part);
            if (lane == 0) s_sum[wave] = part;
        }
        __syncthreads();
        if (tid == 0) {
            int run = 0;
            for (int t = 0; t < EVT_CHUNK_WORDS; t++) { s_pre[t] = run; run += __popcll(s_w[t]); }
        }
        if (SELF) {
            base = (int64_t)s_sum[0] + s_sum[1] + s_sum[2] + s_sum[3];
        } else {
            base = chunk_lpre[c];
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < EVT_CHUNK / 256; it++) {
            const int64_t p = c * EVT_CHUNK + it * 256 + tid;
            const int wi = it * 4 + wave;
            const unsigned long long word = s_w[wi];
            if ((word >> lane) & 1ull) is_out[base + s_pre[wi] + __popcll(word & ((1ull << lane) - 1ull))] = (uint32_t)p;
        }
        __syncthreads();
    }
}

static unsigned grid_for_chunks(int64_t max_chunks) {
    int64_t g = max_chunks;
    if (g > 4096) g = 4096;
    if (g < 1) g = 1;
    return (unsigned)g;
}

static void fill_begin_args(evt_ctx *c, bool all_rows, BeginArgs &A) {
    const LevelTab &L = c->lvl[1];
    A.tree = c->tree;
    A.status = c->status;
    A.seg_start = c->seg_start;
    A.seg_len = c->seg_len;
    A.hdr = L.hdr;
    A.act_node = L.act_node;
    A.cprefix = L.cprefix;
    A.bnode = L.bnode;
    A.bstart = L.bstart;
    A.bprefix = L.bprefix;
    A.hist = c->hist;
    A.stats = c->stats;
    A.n_is = c->N;
    A.n_is_dev = all_rows ? nullptr : c->chunk_lpre + (c->N + EVT_CHUNK - 1) / EVT_CHUNK;
    A.seg_cost = c->hist_seg_cost;
    A.root_words = (int64_t)c->n_js_last * c->NAg * c->B;
    A.nnodes = c->nnodes;
    A.K = c->K;
    A.D = c->D;
    A.js_words = A.map_words = 0;
    A.js_src = A.map_src = nullptr;
    A.js_dst = A.map_dst = nullptr;
    if (c->js_staged) { // read from the pinned buffer by the kernel (no trip through the copy engine, no launch of its own)
        const size_t o_js = c->blob_bytes, o_map = c->blob_bytes + (size_t)c->F * 4;
        A.js_src = reinterpret_cast<const uint32_t *>(c->h_stage_dev + o_js);
        A.js_dst = c->js;
        A.js_words = c->n_js_last;
        A.map_src = reinterpret_cast<const uint32_t *>(c->h_stage_dev + o_map);
        A.map_dst = reinterpret_cast<uint32_t *>(c->jsmap);
        A.map_words = c->RS / 2;
    }
}

// a tree on every row: the set-up block as a kernel of its own
int launch_tree_begin(evt_ctx *c) {
    BeginArgs A;
    fill_begin_args(c, true, A);
    hipLaunchKernelGGL(k_tree_begin, dim3(1), dim3(1024), 0, c->stream, A);
    HIPCHK(hipGetLastError());
    c->js_staged = false;
    return EVT_OK;
}

// Subsampling of a tree and its set-up.  draw: the mask's bytes are drawn from `seed` by the count pass (and written to
// c->mask) instead of read.  The tree's set-up block rides in the scatter pass.
int launch_compact_mask(evt_ctx *c, uint8_t cond, bool draw, unsigned long long seed) {
    const int64_t n_chunks = (c->N + EVT_CHUNK - 1) / EVT_CHUNK;
    unsigned g = grid_for_chunks(n_chunks);
    if (draw) hipLaunchKernelGGL(k_mask_count<true>, dim3(g), dim3(256), 0, c->stream, c->mask, cond, c->N, n_chunks, c->flagw, c->chunk_nleft, seed);
    else hipLaunchKernelGGL(k_mask_count<false>, dim3(g), dim3(256), 0, c->stream, c->mask, cond, c->N, n_chunks, c->flagw, c->chunk_nleft, 0ull);
    HIPCHK(hipGetLastError());
    BeginArgs B;
    fill_begin_args(c, false, B);
    if (n_chunks <= 1024) { // the scatter's blocks add up the counts before their chunk themselves
        hipLaunchKernelGGL(k_mask_scatter<true>, dim3(g + 1), dim3(256), 0, c->stream, c->N, n_chunks, c->flagw, c->chunk_nleft, c->chunk_lpre, c->is_a, B);
    } else {
        hipLaunchKernelGGL(k_mask_scan, dim3(1), dim3(1024), 0, c->stream, c->chunk_nleft, c->chunk_lpre, n_chunks);
        HIPCHK(hipGetLastError());
        hipLaunchKernelGGL(k_mask_scatter<false>, dim3(g + 1), dim3(256), 0, c->stream, c->N, n_chunks, c->flagw, c->chunk_nleft, c->chunk_lpre, c->is_a, B);
    }
    HIPCHK(hipGetLastError());
    c->js_staged = false;
    return EVT_OK;
}

static void fill_part_args(evt_ctx *c, int level, const uint32_t *is_cur, uint32_t *is_next, bool fuse_pred, PartArgs &A) {
    const LevelTab &L = c->lvl[level & 1];
    A.hdr = L.hdr;
    A.cdesc = L.cdesc;
    A.act_node = L.act_node;
    A.cprefix = L.cprefix;
    A.status = c->status;
    A.seg_start = c->seg_start;
    A.seg_len = c->seg_len;
    A.t_packed = c->tree.packed;
    A.xcm = c->xcm;
    A.N = c->N;
    A.is_cur = is_cur;
    A.is_next = is_next;
    A.flagw = c->flagw;
    A.chunk_nleft = c->chunk_nleft;
    A.chunk_lpre = c->chunk_lpre;
    A.nidx = c->nidx;
    A.pred = c->pred;
    A.t_pred = c->tree.pred;
    A.K = c->K;
    A.loss = c->loss; // selects the leaf-add rule
    A.fuse_pred = fuse_pred ? 1 : 0;
    A.write_nidx = c->write_nidx ? 1 : 0;
    A.stream_hint = ((size_t)c->N * c->F > ((size_t)256 << 20)) ? 1 : 0;
    A.fold = 0;
    A.planes = c->planes_ready ? c->planes : nullptr;
    A.plane_words = c->plane_words;
    A.B = c->B;
    A.xrm = nullptr;
    A.gq = nullptr;
    A.jsmap = nullptr;
    A.hist = nullptr;
    A.node_stride = 0;
    A.F = A.nfs = A.NAg = 0;
    A.copy_src = nullptr;
    A.copy_dst = nullptr;
    A.copy_n = 0;
    A.copy_blocks = 0;
}

int launch_part_count(evt_ctx *c, int level, const uint32_t *is_cur) {
    PartArgs A;
    fill_part_args(c, level, is_cur, nullptr, false, A);
    if (A.stream_hint) hipLaunchKernelGGL(k_part_count<true>, dim3(grid_for_chunks(c->max_chunks)), dim3(256), 0, c->stream, A);
    else hipLaunchKernelGGL(k_part_count<false>, dim3(grid_for_chunks(c->max_chunks)), dim3(256), 0, c->stream, A);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

static void fill_next_args(evt_ctx *c, int level, NextArgs &A) {
    const LevelTab &L = c->lvl[level & 1];
    const LevelTab &Nx = c->lvl[(level + 1) & 1];
    A.hdr = L.hdr;
    A.act_node = L.act_node;
    A.cprefix = L.cprefix;
    A.status = c->status;
    A.seg_start = c->seg_start;
    A.seg_len = c->seg_len;
    A.chunk_nleft = c->chunk_nleft;
    A.chunk_lpre = c->chunk_lpre;
    A.n_hdr = Nx.hdr;
    A.n_act_node = Nx.act_node;
    A.n_cprefix = Nx.cprefix;
    A.n_bnode = Nx.bnode;
    A.n_bstart = Nx.bstart;
    A.n_bprefix = Nx.bprefix;
    A.n_stats = (level + 1 <= c->D) ? c->stats + level + 1 : nullptr;
    A.seg_cost = c->hist_seg_cost;
}

// Moves the rows of the level's split nodes to their children and, in one extra block, writes the next level's tables.
int launch_part_scatter(evt_ctx *c, int level, const uint32_t *is_cur, uint32_t *is_next, bool fuse_pred) {
    PartArgs A;
    fill_part_args(c, level, is_cur, is_next, fuse_pred, A);
    NextArgs NX;
    fill_next_args(c, level, NX);
    // up to a thousand chunks per level the bookkeeping rides along in the scatter kernel (one launch less per level)
    A.fold = c->max_chunks <= 1024 + c->maxlvl ? 1 : 2;
    if (A.fold == 2) {
        hipLaunchKernelGGL(k_chunk_scan, dim3(1), dim3(1024), 0, c->stream, NX);
        HIPCHK(hipGetLastError());
    }
    const dim3 grid(grid_for_chunks(c->max_chunks) + 1);
    if (c->step.hist_fused) {
        // the next level's histograms are built here: no histogram kernel runs at that level
        A.xrm = c->xrm;
        A.gq = c->gq;
        A.jsmap = c->jsmap;
        A.hist = c->hist;
        A.node_stride = (int64_t)c->F * c->NAg * c->B;
        A.F = c->F;
        A.nfs = c->n_js_last;
        A.NAg = c->NAg;
        const size_t lds = (size_t)c->NA * c->n_js_last * c->B * 8;
        if (A.fold != 1 || !scatter_can_build_hist(c, c->n_js_last)) {
            evt_set_error("internal: scatter pass cannot build histograms for this shape");
            return EVT_ERR_STATE;
        }
#define PSCASE(NA_)                                                                                                        \
    case NA_:                                                                                                              \
        if (c->unit_w) hipLaunchKernelGGL((k_part_scatter<NA_, true>), grid, dim3(256), lds, c->stream, A, NX);          \
        else hipLaunchKernelGGL((k_part_scatter<NA_, false>), grid, dim3(256), lds, c->stream, A, NX);                   \
        break;
        switch (c->NA) {
            PSCASE(1)
            PSCASE(2)
            PSCASE(3)
            PSCASE(4)
            PSCASE(5)
        default: evt_set_error("unsupported channel count %d", c->NA); return EVT_ERR_ARG;
        }
#undef PSCASE
    } else {
        hipLaunchKernelGGL((k_part_scatter<0, false>), grid, dim3(256), 0, c->stream, A, NX);
    }
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// The scatter pass can build the next level's histograms: 16-byte records, one launch's worth of channels in at most
// 32 KB of LDS, a split search that writes the chunk descriptors the histogram kernel otherwise leaves behind (one block
// per node: k_scan's fused form) and at most 128 chunks per level (a quarter of a million rows), where a level is a chain of
// kernels of a few microseconds each and one of them less is worth more than the histogram kernel's better use of the
// machine: at 100k rows x 10 features the pass takes 12 us against 5 + 10 us for the two kernels, at 1M rows 22 against 6 + 12.
bool scatter_can_build_hist(const evt_ctx *c, int nfs) {
    return c->hist_in_scatter && c->RS == 16 && !c->mc && c->tree_type != EVT_TREE_OBLIVIOUS && c->scan_fused && nfs <= 16 &&
           c->NA <= EVT_MAX_NA && c->max_chunks <= 128 + c->maxlvl && (size_t)c->NA * nfs * c->B * 8 <= 32 * 1024;
}

int launch_final_fused(evt_ctx *c, int level, const uint32_t *is_cur, bool fuse_pred, bool send_blob) {
    if (!fuse_pred && !c->write_nidx) return EVT_OK;
    PartArgs A;
    fill_part_args(c, level, is_cur, nullptr, fuse_pred, A);
    if (send_blob) {
        A.copy_src = reinterpret_cast<const uint4 *>(c->tree_blob);
        A.copy_dst = reinterpret_cast<uint4 *>(c->h_stage_dev);
        A.copy_n = (int64_t)(c->blob_bytes / 16);
        A.copy_blocks = (int)std::min<int64_t>(64, (A.copy_n + 255) / 256);
        c->step.blob_sent = true;
    }
    const dim3 grid(grid_for_chunks(c->max_chunks) + (unsigned)A.copy_blocks);
    if (A.stream_hint) hipLaunchKernelGGL(k_final_fused<true>, grid, dim3(256), 0, c->stream, A);
    else hipLaunchKernelGGL(k_final_fused<false>, grid, dim3(256), 0, c->stream, A);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

// Node of every row that is still on its way down, read off the row lists: node n of the level owns
// is[seg_start[n] .. +seg_len[n]).  Read-back for a tree grown in stages (rows that reached a leaf above this level
// had their node recorded when they got there).
__global__ __launch_bounds__(256) void k_nidx_from_segments(const uint32_t *__restrict__ is, const int64_t *__restrict__ seg_start,
                                                           const int64_t *__restrict__ seg_len, const int32_t *__restrict__ status,
                                                           int first_node, uint32_t *__restrict__ nidx) {
    const int n = first_node + blockIdx.x;
    if (status[n] == ST_INACTIVE) return;
    const int64_t start = seg_start[n], len = seg_len[n];
    for (int64_t i = (int64_t)blockIdx.y * 256 + threadIdx.x; i < len; i += (int64_t)gridDim.y * 256) nidx[is[start + i]] = (uint32_t)n;
}

int launch_nidx_from_segments(evt_ctx *c, int level, const uint32_t *is_cur) {
    const int first = 1 << (level - 1), count = first; // nodes first .. 2 * first - 1
    hipLaunchKernelGGL(k_nidx_from_segments, dim3((unsigned)count, 64), dim3(256), 0, c->stream, is_cur, c->seg_start, c->seg_len, c->status,
                       first, c->nidx);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

