// Histogram builder: the dominant kernel of tree growth (update_hist! / _hist!,
// src/fit-utils.jl:345-394; device twin ext/EvoTreesKernelAbstractionsExt/fit-utils.jl:57-174).
//
// Layout and mapping (gfx950, wave64):
//  * Rows are read from the observation-major copy of x_bin: one record of RS bytes per row,
//    fetched as 128-bit loads, LPR = RS/16 lanes per record, 64/LPR rows per wave instruction.
//    A node's rows are a contiguous, ascending segment of the row-id list, so consecutive lanes
//    touch consecutive (root: adjacent) records.
//  * Each lane owns 16 fixed features for the whole kernel; lanes of one record therefore add into
//    different feature planes of the LDS histogram and same-address collisions inside a wave
//    instruction can only come from the few rows that share the instruction.
//  * Accumulators are 64-bit fixed-point integers in LDS (ds_add_u64), one word per
//    (channel, sampled feature, bin).  Integer sums are exact and order independent, so the
//    result is bit-identical from run to run and across launch shapes.  With unit weights the
//    first gradient channel and the row count share one word (count in the low 16 bits), which
//    makes mse with unit weights a single LDS atomic per (row, feature).
//  * A block walks a contiguous span of the level's build rows (all build nodes concatenated)
//    and flushes its LDS histogram to the node's global histogram with 64-bit atomics whenever
//    the node changes, so the number of flushes is (#blocks + #build nodes) per level.
//
// Algorithmic HBM bytes per built row: RS-or-F bin bytes + 8*NA staged gradient bytes + 4 row-id bytes.
#include "evt_internal.h"
#include <hip/hip_ext.h>

struct HistArgs {
    const uint8_t *xrm;
    const unsigned long long *gq;
    const uint32_t *is;
    const int64_t *hdr;
    const int32_t *bnode;
    const int64_t *bstart;
    const int64_t *bprefix;
    const uint16_t *jsmap;
    long long *hist;
    int64_t *stats;
    int64_t N;
    int64_t node_stride;
    int RS, LPR, RPW, F, nfs, B, NAg, level;
    int NSL; // conflict-free kernel: lanes per row, the power of two >= 16 that covers a column tile's pieces
    int TW;  // conflict-free kernel: bytes of a record one block column (blockIdx.y) takes - a column tile
    int slots_per_tile;
    int min_rows;
    int seg_cost;
    int a0; // first global channel of this launch (channels beyond EVT_HIST_GROUP take further launches)
    // level bookkeeping that rides along with the first launch of a level: the partition kernels' chunk descriptors
    const int32_t *act_node;
    const int64_t *cprefix;
    const int64_t *seg_start;
    const int64_t *seg_len;
    uint4 *cdesc;
};

// First node of a block's span: the largest i with bprefix[i] <= start.  bprefix ascends from 0, so that is the number
// of entries <= start, less one.  Every wavefront counts them for itself, 64 entries per load instruction and eight
// load instructions in flight (clamped indices, no branch between them): one trip to memory for up to 512 build nodes
// where a binary search makes log2(n_build) dependent ones.
__device__ __forceinline__ int first_node_of_span(const int64_t *__restrict__ bprefix, int n_build, int64_t start) {
    const int lane = threadIdx.x & 63;
    int cnt = 0;
    for (int k0 = 0; k0 < n_build; k0 += 512) {
        int64_t v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int k = k0 + j * 64 + lane;
            v[j] = bprefix[k < n_build ? k : n_build - 1];
        }
#pragma unroll
        for (int j = 0; j < 8; j++) cnt += (k0 + j * 64 + lane < n_build && v[j] <= start) ? 1 : 0;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cnt += __shfl_xor(cnt, o);
    return cnt - 1;
}

// Chunk descriptors of the level (evt_fill_chunk_descriptors): they ride along with the first launch of a level, spread
// over the wavefronts of its first block column; the work hides behind the histogram kernel's own set-up.
__device__ __forceinline__ void fill_chunk_descriptors(const HistArgs &A) {
    if (blockIdx.y != 0 || A.a0 != 0) return;
    const int wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    evt_fill_chunk_descriptors(A.hdr, A.act_node, A.cprefix, A.seg_start, A.seg_len, A.cdesc, (int)blockIdx.x * nwaves + wave,
                               (int)gridDim.x * nwaves);
}

template <int NA, bool PACK>
__global__ __launch_bounds__(1024) void k_hist_build(HistArgs A) {
    extern __shared__ unsigned long long H[]; // [NA][tile slots][B]
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int lane = tid & 63, wave = tid >> 6, nwaves = nthr >> 6;
    const int n_build = (int)A.hdr[LH_N_BUILD];
    const int64_t total = A.hdr[LH_TOTAL_BUILD];
    fill_chunk_descriptors(A);
    if (n_build <= 0 || total <= 0) return;
    if (blockIdx.x == 0 && blockIdx.y == 0 && tid == 0 && A.a0 == 0) A.stats[A.level] = total - (int64_t)n_build * A.seg_cost;

    const int step = nwaves * A.RPW; // rows per block iteration
    // rows per block: an even share, but never so few that the flush of a whole LDS histogram
    // (and the chain of same-address global atomics it joins) outweighs the rows it covers
    int64_t T = (total + gridDim.x - 1) / gridDim.x;
    if (T < A.min_rows) T = A.min_rows;
    T = ((T + 2 * step - 1) / (2 * step)) * (2 * step);
    int64_t start = (int64_t)blockIdx.x * T;
    if (start >= total) return;
    int64_t end = start + T < total ? start + T : total;

    const int slot0 = blockIdx.y * A.slots_per_tile;
    int nslots = A.nfs - slot0;
    if (nslots > A.slots_per_tile) nslots = A.slots_per_tile;
    const int plane = nslots * A.B;

    for (int i = tid; i < NA * plane; i += nthr) H[i] = 0ull;

    // the 16 features this lane owns -> LDS word offset of their first bin (vmask bit t: in this tile)
    const int sub = lane % A.LPR, rloc = lane / A.LPR;
    int off[16];
    unsigned vmask = 0;
#pragma unroll
    for (int t = 0; t < 16; t++) {
        int s = (int)A.jsmap[sub * 16 + t]; // by record byte: 0xFFFF for padding and for features outside the sample
        s = (s == 0xFFFF) ? -1 : s - slot0;
        const bool ok = (s >= 0 && s < nslots);
        off[t] = ok ? s * A.B - 1 : 0; // bins are 1-based
        vmask |= ok ? (1u << t) : 0u;
    }
    const bool lane_on = (rloc < A.RPW) && vmask != 0;
    __syncthreads();

    int i = first_node_of_span(A.bprefix, n_build, start);
    const int64_t blk_start = start, blk_end = end;

    while (start < end) {
        // spans are cut in a cost space where node i occupies [bprefix[i], bprefix[i+1]): its rows first,
        // then seg_cost units standing for the fixed cost of one flush, so that a span holding many tiny
        // nodes carries proportionally fewer rows
        const int64_t nbeg = A.bprefix[i];
        const int64_t nxt = A.bprefix[i + 1];
        const int64_t nrows_end = nxt - A.seg_cost;
        const int64_t cend = end < nxt ? end : nxt;
        const int64_t nend_all = cend < nrows_end ? cend : nrows_end;
        if (start >= nend_all) { // only this node's padding lies in the span
            start = cend;
            i++;
            continue;
        }
        // the packed row counter holds 16 bits: a longer run of one node is flushed in several parts
        const int64_t nend = (PACK && nend_all - start > EVT_HIST_MAX_ROWS_PER_BLOCK) ? start + EVT_HIST_MAX_ROWS_PER_BLOCK : nend_all;
        const int64_t seg = A.bstart[i] - nbeg; // position in the row list = seg + p
        // software pipeline over U row groups per wave: the row ids of iteration k+2 and the records of
        // iteration k+1 are in flight while the LDS atomics of iteration k are issued
        {
            constexpr int U = 2;
            constexpr uint32_t INV = 0xFFFFFFFFu;
            const int64_t itstride = (int64_t)U * step;
            uint32_t rc[U], rn[U];
            uint4 vc[U], vn[U];
            unsigned long long gc[U][NA], gn[U][NA];
            int64_t b0 = start + (int64_t)wave * A.RPW;
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int64_t p = b0 + (int64_t)u * step + rloc;
                rc[u] = (lane_on && p < nend) ? A.is[seg + p] : INV;
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                vc[u] = make_uint4(0, 0, 0, 0);
                if (rc[u] != INV) {
                    vc[u] = *reinterpret_cast<const uint4 *>(A.xrm + (size_t)rc[u] * A.RS + sub * 16);
#pragma unroll
                    for (int a = 0; a < NA; a++) gc[u][a] = evt_load_gq<PACK>(A.gq, A.N, a, rc[u]);
                }
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int64_t p = b0 + itstride + (int64_t)u * step + rloc;
                rn[u] = (lane_on && p < nend) ? A.is[seg + p] : INV;
            }
            for (; b0 < nend; b0 += itstride) {
#pragma unroll
                for (int u = 0; u < U; u++) {
                    vn[u] = make_uint4(0, 0, 0, 0);
                    if (rn[u] != INV) {
                        vn[u] = *reinterpret_cast<const uint4 *>(A.xrm + (size_t)rn[u] * A.RS + sub * 16);
#pragma unroll
                        for (int a = 0; a < NA; a++) gn[u][a] = evt_load_gq<PACK>(A.gq, A.N, a, rn[u]);
                    }
                }
                uint32_t rnn[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const int64_t p = b0 + 2 * itstride + (int64_t)u * step + rloc;
                    rnn[u] = (lane_on && p < nend) ? A.is[seg + p] : INV;
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    if (rc[u] != INV) {
                        const uint32_t wds[4] = {vc[u].x, vc[u].y, vc[u].z, vc[u].w};
#pragma unroll
                        for (int t = 0; t < 16; t++) {
                            if (vmask & (1u << t)) {
                                const int idx = off[t] + (int)((wds[t >> 2] >> (8 * (t & 3))) & 0xFFu);
#pragma unroll
                                for (int a = 0; a < NA; a++) atomicAdd(&H[a * plane + idx], gc[u][a]);
                            }
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    rc[u] = rn[u];
                    vc[u] = vn[u];
#pragma unroll
                    for (int a = 0; a < NA; a++) gc[u][a] = gn[u][a];
                    rn[u] = rnn[u];
                }
            }
        }
        __syncthreads();
        // flush this node's partial histogram: hist[node][slot][ag][bin].  A node whose rows all lie in
        // this block's span has a single writer: plain stores into its zero-initialised slice; a node
        // shared with other blocks is accumulated with 64-bit global atomics.
        const bool sole = (nbeg >= blk_start) && (nrows_end <= blk_end) && !(PACK && nrows_end - nbeg > EVT_HIST_MAX_ROWS_PER_BLOCK);
        long long *hn = A.hist + (int64_t)(A.bnode[i] - 1) * A.node_stride;
        // blocks start at different words so that concurrent flushes of one node do not queue on the
        // same addresses
        const int nwords = NA * plane;
        const int rot = (int)(((int64_t)blockIdx.x * 1021) % nwords);
        for (int k = tid; k < nwords; k += nthr) {
            int idx = k + rot;
            if (idx >= nwords) idx -= nwords;
            const unsigned long long w = H[idx];
            if (w != 0ull) {
                H[idx] = 0ull;
                const int a = idx / plane;
                const int rem = idx - a * plane;
                const int s = rem / A.B;
                const int bin = rem - s * A.B;
                unsigned long long *base = reinterpret_cast<unsigned long long *>(hn) + ((int64_t)(slot0 + s) * A.NAg) * A.B + bin;
                if (PACK && a == 0) {
                    const long long gsum = (long long)w >> EVT_PACK_CNT_BITS;
                    const unsigned long long cnt = w & ((1ull << EVT_PACK_CNT_BITS) - 1ull);
                    if (sole) {
                        base[0] = (unsigned long long)gsum;
                        base[(int64_t)(A.NAg - 1) * A.B] = cnt;
                    } else {
                        if (gsum != 0) atomicAdd(base, (unsigned long long)gsum);
                        atomicAdd(base + (int64_t)(A.NAg - 1) * A.B, cnt);
                    }
                } else if (sole) {
                    base[(int64_t)(A.a0 + a) * A.B] = w;
                } else {
                    atomicAdd(base + (int64_t)(A.a0 + a) * A.B, w);
                }
            }
        }
        __syncthreads();
        if (nend < nend_all) {
            start = nend; // same node again
        } else {
            start = cend;
            i++;
        }
    }
}

// Bank-conflict-free variant for records of 32 / 64 / 128 / 256 / 512 bytes.
//
// A record is read in pieces of PB bytes, one lane each, NS = RS/PB lanes per row with PB chosen so that NS is a
// multiple of 16 (8-byte pieces from 128-byte records up, 4-byte pieces for 64-byte records, 2-byte pieces for
// 32-byte ones): every group of 16 consecutive lanes - the unit the LDS serves per cycle for 64-bit operations -
// holds 16 different pieces `sub` of ONE row.  The first PU bytes of a piece hold features (evt_ctx::PU; PU == PB for a
// densely packed record); a row costs PU LDS atomic instructions.  The LDS histogram is laid out as word(a, t, bin, sub)
// = ((a*PU + t)*B + bin)*NS + sub for byte t of piece sub, i.e. `sub` selects the bank pair, so the 16 lanes of a
// group always fall on 16 different bank pairs whatever their bins are.  Rows that share a wave instruction sit in
// different groups and cannot collide inside one LDS pass either.  (Two 64-byte records per 16-lane group, 8 lanes of
// 8-byte pieces each, collide whenever their bins' words share a bank half: cfg5's histograms took 0.64 ms per round
// that way and take 0.41 ms with 4-byte pieces.)
// FULL: a lane adds all PB bytes of its piece without testing which features are sampled.  A record's padding reads as
// bin 1 and features outside the sample have LDS words of their own, so the extra adds land in words the flush clears
// and never writes out; the per-feature test (FULL = false) only pays when most features are left out.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_row_bcast(uint32_t x) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xF, 0xF, false);
}
// value held by lane u of this lane's DPP row: the fetcher of row group u
template <int u>
__device__ __forceinline__ uint32_t grp_bcast(uint32_t x) {
    return dpp_row_bcast<0x150 + u>(x);
}

// A record piece of PB bytes in the low bytes of a register pair.
// NT: the streaming hint.  A record is read once per level; when the record array is larger than the last-level cache the
// hint keeps it from displacing the gradient words, which neighbouring rows of other nodes will gather again.  A smaller
// array is better left to the caches: it is still there at the next level.
template <int PB, bool NT>
__device__ __forceinline__ uint2 load_piece(const uint8_t *p) {
    if constexpr (PB == 8) {
        if constexpr (NT) {
            const unsigned long long v = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long *>(p));
            return make_uint2((uint32_t)v, (uint32_t)(v >> 32));
        } else {
            return *reinterpret_cast<const uint2 *>(p);
        }
    } else if constexpr (PB == 4) {
        const uint32_t *q = reinterpret_cast<const uint32_t *>(p);
        return make_uint2(NT ? __builtin_nontemporal_load(q) : *q, 0u);
    } else {
        const uint16_t *q = reinterpret_cast<const uint16_t *>(p);
        return make_uint2((uint32_t)(NT ? __builtin_nontemporal_load(q) : *q), 0u);
    }
}
template <bool NT>
__device__ __forceinline__ uint32_t load_id(const uint32_t *p) {
    return NT ? __builtin_nontemporal_load(p) : *p;
}

template <int NA, bool PACK, int U, bool FULL, int PB, int PU, bool NT>
__global__ __launch_bounds__(1024) void k_hist_build16(HistArgs A) {
    extern __shared__ unsigned long long H[]; // [NA][PU][B][NS]
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int lane = tid & 63, wave = tid >> 6, nwaves = nthr >> 6;
    const int n_build = (int)A.hdr[LH_N_BUILD];
    const int64_t total = A.hdr[LH_TOTAL_BUILD];
    fill_chunk_descriptors(A);
    if (n_build <= 0 || total <= 0) return;
    if (blockIdx.x == 0 && tid == 0 && A.a0 == 0) A.stats[A.level] = total - (int64_t)n_build * A.seg_cost;

    static_assert(PB == 8 || PB == 4 || PB == 2, "a piece is 8, 4 or 2 bytes");
    static_assert(PU >= 1 && PU <= PB, "features per piece");
    const int NS = A.NSL;         // lanes per row: one per piece of the record, idle ones beyond its last piece
    const int RPW = 64 / NS;      // rows per wave instruction
    const int step = nwaves * RPW;
    int64_t T = (total + gridDim.x - 1) / gridDim.x;
    if (T < A.min_rows) T = A.min_rows;
    T = ((T + U * step - 1) / (U * step)) * (U * step);
    int64_t start = (int64_t)blockIdx.x * T;
    if (start >= total) return;
    int64_t end = start + T < total ? start + T : total;

    const int B = A.B;
    const int plane = PU * B * NS; // words per channel
    for (int i = tid; i < NA * plane; i += nthr) H[i] = 0ull;

    const int sub = lane % NS, rloc = lane / NS;
    // column tile: block column y takes bytes [y * TW, (y + 1) * TW) of every record and keeps their histograms only -
    // a record too wide for one LDS histogram is covered by several block columns, each reading its own bytes
    const int tb = (int)blockIdx.y * A.TW;
    const int subl = (tb + sub * PB < A.RS) ? sub : 0; // an idle lane loads the tile's first piece and adds nothing (no feature: vmask 0)
    // byte offset of (t, bin 0) for this lane; bins are 1-based so bin*NS*8 is added on top
    // (32-bit unsigned arithmetic throughout: one 24-bit multiply-add per LDS address)
    uint32_t coff[PU];
    unsigned vmask = 0;
    {
        // the slots of this lane's PB features in one load (jsmap has an entry for every byte of the record, 0xFFFF for
        // the padding and for features outside the sample)
        const int f0 = tb + sub * PB;
        uint32_t mw[4] = {0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu};
        if (f0 < A.RS) {
            if constexpr (PB == 8) {
                const uint4 q = *reinterpret_cast<const uint4 *>(A.jsmap + f0);
                mw[0] = q.x; mw[1] = q.y; mw[2] = q.z; mw[3] = q.w;
            } else if constexpr (PB == 4) {
                const uint2 q = *reinterpret_cast<const uint2 *>(A.jsmap + f0);
                mw[0] = q.x; mw[1] = q.y;
            } else {
                mw[0] = *reinterpret_cast<const uint32_t *>(A.jsmap + f0);
            }
        }
#pragma unroll
        for (int t = 0; t < PU; t++) {
            const bool ok = ((mw[t >> 1] >> (16 * (t & 1))) & 0xFFFFu) != 0xFFFFu;
            coff[t] = (uint32_t)(((t * B - 1) * NS + sub) * 8);
            vmask |= ok ? (1u << t) : 0u;
        }
    }
    const uint32_t binmul = (uint32_t)NS * 8u;
    const bool lane_on = vmask != 0;
    __syncthreads();

    int i = first_node_of_span(A.bprefix, n_build, start);
    const int64_t blk_start = start, blk_end = end;
    char *Hb = reinterpret_cast<char *>(H);

    while (start < end) {
        // spans are cut in a cost space where node i occupies [bprefix[i], bprefix[i+1]): its rows first,
        // then seg_cost units standing for the fixed cost of one flush, so that a span holding many tiny
        // nodes carries proportionally fewer rows
        const int64_t nbeg = A.bprefix[i];
        const int64_t nxt = A.bprefix[i + 1];
        int64_t bst = A.bstart[i];
        asm volatile("" : "+v"(bst)); // requested with the two above, not behind the branch below
        const int64_t nrows_end = nxt - A.seg_cost;
        const int64_t cend = end < nxt ? end : nxt;
        const int64_t nend_all = cend < nrows_end ? cend : nrows_end;
        if (start >= nend_all) { // only this node's padding lies in the span
            start = cend;
            i++;
            continue;
        }
        // the packed row counter holds 16 bits: a longer run of one node is flushed in several parts
        const int64_t nend = (PACK && nend_all - start > EVT_HIST_MAX_ROWS_PER_BLOCK) ? start + EVT_HIST_MAX_ROWS_PER_BLOCK : nend_all;
        const int64_t seg = bst - nbeg;
        // A wave takes SR = U * RPW consecutive positions of the run per iteration (U row groups of RPW rows).
        // Row ids and gradient words are fetched one position per lane (one load instruction per SR rows instead of
        // one per group): the number of load instructions in flight, not their bytes, is what a CU runs out of
        // first.  Lane L holds position (L % 16) * RPW + rloc, i.e. lane u of every 16-lane DPP row holds what
        // group u of that row's record needs, and a row broadcast (v_mov_dpp row_newbcast:u) hands it over.
        // Rolling software pipeline: group u's atomics are issued as soon as its record (requested one iteration
        // ago) is there, and the same registers are then reloaded with the group's record of the next iteration.
        // Loads are unconditional (positions past the end are clamped to the run's last row, their groups are
        // masked at the atomics) and the prologue issues its loads in the loop's order, so that the compiler's count
        // of outstanding loads is exact and no wait drains the queue.
        {
            const int SR = U * RPW; // positions per wave iteration (<= 64)
            const int64_t itstride = (int64_t)nwaves * SR;
            const uint32_t *isp = A.is + seg;
            // a record's address: row id times record size as one 32 x 32 -> 64 bit multiply-add, plus the piece's byte offset
            const uint32_t rs32 = (uint32_t)A.RS, pofs = (uint32_t)(tb + subl * PB);
            const int64_t lastp = nend - 1;          // >= start
            int64_t pw = start + (int64_t)wave * SR; // first position of this wave's iteration
            // lane j of a DPP row fetches for row group j the row its DPP row belongs to (a record wider than a DPP row is
            // fetched for by every DPP row it covers)
            const int myu = lane & 15;
            const int mypos = myu * RPW + rloc; // position (within the iteration) this lane fetches
            const bool fetcher = myu < U;
            uint32_t idc, idn;
            unsigned long long gc[NA], gn[NA];
            uint2 v[U];
            {
                const int64_t p = pw + mypos;
                idc = load_id<NT>(isp + ((fetcher && p < nend) ? p : lastp));
            }
#pragma unroll
            for (int a = 0; a < NA; a++) gc[a] = evt_load_gq<PACK>(A.gq, A.N, a, idc);
            {
                const int64_t p = pw + itstride + mypos;
                idn = load_id<NT>(isp + ((fetcher && p < nend) ? p : lastp));
            }
            __builtin_amdgcn_sched_barrier(0);
#define EVT_H16_PRO(u_)                                                                                               \
    if constexpr ((u_) < U) {                                                                                         \
        const uint32_t row = grp_bcast<(u_) < U ? (u_) : 0>(idc);                                               \
        v[(u_) < U ? (u_) : 0] = load_piece<PB, NT>(A.xrm + ((size_t)row * rs32 + pofs));                   \
        __builtin_amdgcn_sched_barrier(0);                                                                            \
    }
            EVT_H16_PRO(0) EVT_H16_PRO(1) EVT_H16_PRO(2) EVT_H16_PRO(3) EVT_H16_PRO(4) EVT_H16_PRO(5) EVT_H16_PRO(6) EVT_H16_PRO(7)
            EVT_H16_PRO(8) EVT_H16_PRO(9) EVT_H16_PRO(10) EVT_H16_PRO(11) EVT_H16_PRO(12) EVT_H16_PRO(13) EVT_H16_PRO(14) EVT_H16_PRO(15)
#undef EVT_H16_PRO
            for (; pw < nend; pw += itstride) {
                // positions of this lane's rows left in the run, as a 32-bit number: group u is inside while u * RPW < rem
                const int64_t rem64 = nend - pw - rloc;
                const int rem = rem64 > 0x7fffffff ? 0x7fffffff : (int)rem64;
                // next iteration's gradient words and the row ids of the one after: ahead of the records in issue order
#pragma unroll
                for (int a = 0; a < NA; a++) gn[a] = evt_load_gq<PACK>(A.gq, A.N, a, idn);
                uint32_t idnn;
                {
                    const int64_t p = pw + 2 * itstride + mypos;
                    idnn = load_id<NT>(isp + ((fetcher && p < nend) ? p : lastp));
                }
                __builtin_amdgcn_sched_barrier(0);
#define EVT_H16_STEP(u_)                                                                                              \
    if constexpr ((u_) < U) {                                                                                         \
        constexpr int ui = (u_) < U ? (u_) : 0;                                                                       \
        {                                                                                                             \
            unsigned long long gg[NA];                                                                                \
            _Pragma("unroll") for (int a = 0; a < NA; a++) {                                                          \
                const uint32_t glo = grp_bcast<ui>((uint32_t)gc[a]);                                            \
                const uint32_t ghi = grp_bcast<ui>((uint32_t)(gc[a] >> 32));                                    \
                gg[a] = ((unsigned long long)ghi << 32) | glo;                                                         \
            }                                                                                                         \
            if (lane_on && ((u_) * RPW < rem)) {                                                                       \
                const uint32_t wds[2] = {v[ui].x, v[ui].y};                                                            \
                _Pragma("unroll") for (int t = 0; t < PU; t++) {                                                       \
                    if (FULL || (vmask & (1u << t))) {                                                                \
                        const uint32_t bo = __umul24((wds[t >> 2] >> (8 * (t & 3))) & 0xFFu, binmul) + coff[t];       \
                        _Pragma("unroll") for (int a = 0; a < NA; a++)                                                 \
                            atomicAdd(reinterpret_cast<unsigned long long *>(Hb + bo + (uint32_t)(a * plane * 8)), gg[a]); \
                    }                                                                                                 \
                }                                                                                                     \
            }                                                                                                         \
        }                                                                                                             \
        const uint32_t row = grp_bcast<ui>(idn);                                                                \
        v[ui] = load_piece<PB, NT>(A.xrm + ((size_t)row * rs32 + pofs));                                  \
        __builtin_amdgcn_sched_barrier(0);                                                                            \
    }
                EVT_H16_STEP(0) EVT_H16_STEP(1) EVT_H16_STEP(2) EVT_H16_STEP(3) EVT_H16_STEP(4) EVT_H16_STEP(5) EVT_H16_STEP(6) EVT_H16_STEP(7)
                EVT_H16_STEP(8) EVT_H16_STEP(9) EVT_H16_STEP(10) EVT_H16_STEP(11) EVT_H16_STEP(12) EVT_H16_STEP(13) EVT_H16_STEP(14) EVT_H16_STEP(15)
#undef EVT_H16_STEP
#pragma unroll
                for (int a = 0; a < NA; a++) gc[a] = gn[a];
                idc = idn;
                idn = idnn;
            }
        }
        __syncthreads();
        // flush: a wave covers 8 consecutive bins of 8 pieces `sub` (or of all NS pieces and 8 / NS bin chunks) of one
        // (channel, t): global accesses are whole 64-byte runs of one feature's bins, LDS reads spread over the bank
        // pairs.  Blocks start at different items so that concurrent flushes of one node do not queue on the same addresses.
        const bool sole = (nbeg >= blk_start) && (nrows_end <= blk_end) && !(PACK && nrows_end - nbeg > EVT_HIST_MAX_ROWS_PER_BLOCK);
        long long *hn = A.hist + (int64_t)(A.bnode[i] - 1) * A.node_stride;
        const int nchunks = (B + 7) >> 3;
        const int nitems = NA * PU * nchunks * NS * 8; // (channel, t, bin chunk, piece, bin in chunk), the last fastest
        const int rot = (int)(((int64_t)blockIdx.x * 1031) % (nitems >> 6)) << 6;
        // FU items per thread at a time: their LDS words (and, when features are sampled, their slots) are all
        // requested before the first is used, so a flush costs one LDS and one memory round trip, not FU of each
        constexpr int FU = 8;
        const bool all_feats = A.nfs == A.F; // slot of feature f is f itself
        const int piece0 = tb / PB;          // first piece of this column tile
        const bool pow2 = (nchunks & (nchunks - 1)) == 0; // decode with shifts
        const int ns_sh = __ffs(NS) - 1, nc_sh = __ffs(nchunks) - 1;
        for (int k0 = tid; k0 < nitems; k0 += FU * nthr) {
            unsigned long long wv[FU];
            unsigned long long *hwv[FU];
            int av[FU], bv[FU], slotv[FU];
#pragma unroll
            for (int j = 0; j < FU; j++) {
                int k = k0 + j * nthr;
                wv[j] = 0ull;
                hwv[j] = H;
                av[j] = 0; bv[j] = 0; slotv[j] = 0xFFFF;
                if (k < nitems) {
                    k += rot;
                    if (k >= nitems) k -= nitems;
                    const int bl = k & 7;
                    int rest = k >> 3;
                    const int sidx = rest & (NS - 1);
                    rest >>= ns_sh;
                    int chunk;
                    if (pow2) {
                        chunk = rest & (nchunks - 1);
                        rest >>= nc_sh;
                    } else {
                        chunk = rest % nchunks;
                        rest /= nchunks;
                    }
                    const int t = rest % PU;
                    const int a = rest / PU;
                    const int b = chunk * 8 + bl;
                    const int f = (piece0 + sidx) * PU + t; // the feature at byte t of the piece
                    if (b < B) {
                        hwv[j] = &H[(size_t)a * plane + ((size_t)t * B + b) * NS + sidx];
                        wv[j] = *hwv[j];
                        av[j] = a; bv[j] = b;
                        if (f < A.F) slotv[j] = all_feats ? f : (int)A.jsmap[tb + sidx * PB + t]; // a padding byte's word has no slot
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < FU; j++) {
                const unsigned long long w = wv[j];
                if (w == 0ull) continue;
                *hwv[j] = 0ull;
                const int slot = slotv[j], a = av[j], b = bv[j];
                if (slot == 0xFFFF) continue;
                unsigned long long *base = reinterpret_cast<unsigned long long *>(hn) + ((int64_t)slot * A.NAg) * B + b;
                if (PACK && a == 0) {
                    const long long gsum = (long long)w >> EVT_PACK_CNT_BITS;
                    const unsigned long long cnt = w & ((1ull << EVT_PACK_CNT_BITS) - 1ull);
                    if (sole) {
                        base[0] = (unsigned long long)gsum;
                        base[(int64_t)(A.NAg - 1) * B] = cnt;
                    } else {
                        if (gsum != 0) atomicAdd(base, (unsigned long long)gsum);
                        atomicAdd(base + (int64_t)(A.NAg - 1) * B, cnt);
                    }
                } else if (sole) {
                    base[(int64_t)(A.a0 + a) * B] = w;
                } else {
                    atomicAdd(base + (int64_t)(A.a0 + a) * B, w);
                }
            }
        }
        __syncthreads();
        if (nend < nend_all) {
            start = nend; // same node again
        } else {
            start = cend;
            i++;
        }
    }
}

template <int NA, bool PACK, int U, int PB, int PU, bool NT>
static int launch_hist16_q(evt_ctx *c, const HistArgs &A, dim3 grid, int threads, size_t lds) {
    // unpredicated atomics for every feature of the record pay off unless most features are left out: the words of
    // features outside the sample are simply not flushed
    const bool full = 2 * c->n_js_last >= c->F;
    if (lds > 64 * 1024) { // one block per CU may take most of its 160 KB
        static EvtDevOnce once;
        if (once.pending(c->device)) {
            HIPCHK(hipFuncSetAttribute(reinterpret_cast<const void *>(k_hist_build16<NA, PACK, U, true, PB, PU, NT>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            HIPCHK(hipFuncSetAttribute(reinterpret_cast<const void *>(k_hist_build16<NA, PACK, U, false, PB, PU, NT>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            once.mark(c->device);
        }
    }
    // c->launch_e0 / launch_e1 (when profiling): the kernel's own dispatch records them
    if (full)
        hipExtLaunchKernelGGL((k_hist_build16<NA, PACK, U, true, PB, PU, NT>), grid, dim3(threads), (uint32_t)lds, c->stream, c->launch_e0, c->launch_e1, 0, A);
    else
        hipExtLaunchKernelGGL((k_hist_build16<NA, PACK, U, false, PB, PU, NT>), grid, dim3(threads), (uint32_t)lds, c->stream, c->launch_e0, c->launch_e1, 0, A);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

template <int NA, bool PACK>
static int launch_hist16_t(evt_ctx *c, const HistArgs &A, dim3 grid, int threads, size_t lds) {
    // row groups (records) in flight per wave: as many as a DPP row can address, fewer when registers run out
    constexpr int U = (NA <= 2) ? 16 : 8;
    // records larger in total than the last-level cache (256 MB) are streamed past it
    const bool nt = (size_t)c->N * c->RS > ((size_t)256 << 20);
    // (piece bytes, features per piece): a densely packed record has PU == PB, record_layout() picks the others
    const int pb = A.TW >= 128 ? 8 : (A.TW == 64 ? 4 : 2);
    const int pu = c->PU < c->PBL ? c->PU : pb;
#define H16Q(PB_, PU_)                                                                                                     \
    if (pb == PB_ && pu == PU_)                                                                                            \
        return nt ? launch_hist16_q<NA, PACK, U, PB_, PU_, true>(c, A, grid, threads, lds) : launch_hist16_q<NA, PACK, U, PB_, PU_, false>(c, A, grid, threads, lds);
    H16Q(8, 8) H16Q(8, 7) H16Q(8, 6) H16Q(8, 5) H16Q(4, 4) H16Q(4, 3) H16Q(2, 2)
#undef H16Q
    evt_set_error("no histogram kernel for pieces of %d bytes holding %d features", pb, pu);
    return EVT_ERR_INTERNAL;
}

template <int NA, bool PACK>
static int launch_hist_t(evt_ctx *c, const HistArgs &A, dim3 grid, int threads, size_t lds) {
    static EvtDevOnce once;
    if (lds > 64 * 1024 && once.pending(c->device)) {
        HIPCHK(hipFuncSetAttribute(reinterpret_cast<const void *>(k_hist_build<NA, PACK>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        once.mark(c->device);
    }
    hipExtLaunchKernelGGL((k_hist_build<NA, PACK>), grid, dim3(threads), (uint32_t)lds, c->stream, c->launch_e0, c->launch_e1, 0, A);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}

int launch_hist_build(evt_ctx *c, int level, const uint32_t *is_cur) {
    const LevelTab &L = c->lvl[level & 1];
    const int nfs = c->n_js_last;
    HistArgs A;
    A.xrm = c->xrm;
    A.gq = c->gq;
    A.is = is_cur;
    A.hdr = L.hdr;
    A.bnode = L.bnode;
    A.bstart = L.bstart;
    A.bprefix = L.bprefix;
    A.act_node = L.act_node;
    A.cprefix = L.cprefix;
    A.seg_start = c->seg_start;
    A.seg_len = c->seg_len;
    A.cdesc = L.cdesc;
    A.jsmap = c->jsmap;
    A.hist = c->hist;
    A.stats = c->stats;
    A.N = c->N;
    A.node_stride = (int64_t)c->F * c->NAg * c->B;
    A.RS = c->RS;
    A.LPR = c->LPR;
    A.RPW = 64 / c->LPR;
    A.F = c->F;
    A.nfs = nfs;
    A.B = c->B;
    A.NAg = c->NAg;
    A.level = level;
    A.min_rows = c->hist_min_rows;
    A.seg_cost = c->hist_seg_cost;
    const int threads = c->hist_threads;
    const int64_t blocks = c->hist_blocks;
    // accumulator channels are taken EVT_HIST_GROUP at a time (one launch each; the one- and two-output losses need
    // a single launch); the packed row counter rides on channel 0, i.e. in the first group only
    // timing events: one launch carries them itself; several launches (channel groups) are bracketed by event records
    const bool one_launch = c->NA <= EVT_MAX_NA;
    hipEvent_t ev0 = c->launch_e0, ev1 = c->launch_e1;
    if (!one_launch) {
        c->launch_e0 = c->launch_e1 = nullptr;
        if (ev0) (void)hipEventRecord(ev0, c->stream);
    }
    for (int a0 = 0; a0 < c->NA; a0 += (c->NA <= EVT_MAX_NA ? EVT_MAX_NA : EVT_HIST_GROUP)) {
        const int na = (c->NA <= EVT_MAX_NA) ? c->NA : (c->NA - a0 < EVT_HIST_GROUP ? c->NA - a0 : EVT_HIST_GROUP);
        A.a0 = a0;
        A.gq = c->gq + (size_t)a0 * c->N;
        const bool pack = c->unit_w && a0 == 0;
        // feature tiling so that one block's LDS histogram stays within budget
        const size_t budget = 64 * 1024;
        const size_t per_slot = (size_t)na * c->B * 8;
        int slots_per_tile = (int)(budget / per_slot);
        if (slots_per_tile < 1) slots_per_tile = 1;
        if (slots_per_tile > nfs) slots_per_tile = nfs;
        const int ntiles = (nfs + slots_per_tile - 1) / slots_per_tile;
        slots_per_tile = (nfs + ntiles - 1) / ntiles;
        A.slots_per_tile = slots_per_tile;
        const size_t lds = per_slot * slots_per_tile;
        dim3 grid((unsigned)blocks, (unsigned)ntiles);
        // conflict-free variant: a block column takes a tile of TW bytes of every record - the whole record when its LDS
        // histogram fits, else the widest power of two that does (down to 32 bytes) - with 16, 32 or 64 lanes per row;
        // lanes past the record's last piece idle.  (16-byte records as 1-byte pieces were measured: no faster than the
        // generic kernel.)
        int tw = 32;
        while (tw < c->RS && tw < 512) tw <<= 1;
        const bool spread = c->PU < c->PBL; // features spread over all pieces: one tile takes the whole record (record_layout)
        while (!spread && tw > 32 && (size_t)na * c->B * tw * 8 > 128 * 1024) tw >>= 1;
        const int pb16 = tw >= 128 ? 8 : (tw == 64 ? 4 : 2);
        A.TW = tw;
        A.NSL = tw / pb16;
        const int ntiles16 = (c->RS + tw - 1) / tw;
        const size_t lds16 = (size_t)na * c->B * A.NSL * (spread ? c->PU : pb16) * 8; // channels x bins x feature bytes of a tile, words
        const bool can16 = c->RS >= 32 && lds16 <= 128 * 1024 && (!spread || (pb16 == c->PBL && ntiles16 == 1));
        const bool use16 = (c->hist_variant == 1) ? false : can16;
        if (!use16 && c->LPR > 64) { // the generic kernel reads a record with one wavefront instruction: 64 lanes of 16 bytes
            evt_set_error("%d accumulator channels x %d bins need the generic histogram kernel, which takes at most 1024 features", na, c->B);
            return EVT_ERR_ARG;
        }
        int r = EVT_ERR_ARG;
        if (use16) {
            // several block columns share the launch's blocks: the same number of LDS histograms is flushed per node
            int64_t bx = blocks / ntiles16;
            if (bx < 64) bx = blocks < 64 ? blocks : 64;
            dim3 grid16((unsigned)bx, (unsigned)ntiles16);
#define H16CASE(NA_) \
    case NA_: r = pack ? launch_hist16_t<NA_, true>(c, A, grid16, threads, lds16) : launch_hist16_t<NA_, false>(c, A, grid16, threads, lds16); break;
            switch (na) {
                H16CASE(1)
                H16CASE(2)
                H16CASE(3)
                H16CASE(4)
                H16CASE(5)
            }
#undef H16CASE
        } else {
#define HCASE(NA_) \
    case NA_: r = pack ? launch_hist_t<NA_, true>(c, A, grid, threads, lds) : launch_hist_t<NA_, false>(c, A, grid, threads, lds); break;
            switch (na) {
                HCASE(1)
                HCASE(2)
                HCASE(3)
                HCASE(4)
                HCASE(5)
            }
#undef HCASE
        }
        if (r != EVT_OK) {
            if (r == EVT_ERR_ARG) evt_set_error("unsupported channel count %d", na);
            return r;
        }
    }
    if (!one_launch && ev1) (void)hipEventRecord(ev1, c->stream);
    return EVT_OK;
}

// Reference-layout export for parity checks: out[k, bin, feat, node] Float64 (src/init.jl:204).
__global__ __launch_bounds__(256) void k_hist_export(const long long *__restrict__ hist, const uint32_t *__restrict__ js, int nfs, int F,
                                                    int B, int NK, int NAg, int loss, const double *__restrict__ qscale,
                                                    const int32_t *__restrict__ status, int nnodes, int last_level_first, double *out) {
    int node = blockIdx.x; // 0-based
    if (node + 1 >= last_level_first) return; // nodes of the last level never get a histogram
    int st = status[node + 1];
    if (st != ST_SPLIT && st != ST_LEAF && st != ST_BUILD) return; // ST_BUILD: built from rows, not yet searched (a tree grown in stages)
    const long long *hn = hist + (int64_t)node * F * NAg * B;
    for (int idx = threadIdx.x; idx < nfs * B; idx += 256) {
        int jp = idx / B, b = idx - jp * B;
        int f = (int)js[jp] - 1;
        double ch[EVT_MC_MAX_NK];
        for (int ag = 0; ag < NAg; ag++) ch[ag] = (double)hn[((int64_t)jp * NAg + ag) * B + b] * qscale[ag];
        double *o = out + (((int64_t)node * F + f) * B + b) * NK;
        if (EVT_TWO_CHAN(loss, (NK - 1) / 2)) { // channels {g, w}: h = 2w (mse) or 0 (mae)
            o[0] = ch[0];
            o[1] = (loss == EVT_LOSS_MSE) ? 2.0 * ch[1] : 0.0;
            o[2] = ch[1];
        } else {
            for (int k = 0; k < NK; k++) o[k] = ch[k];
        }
    }
}

int launch_hist_export(evt_ctx *c, double *out_dev) {
    hipLaunchKernelGGL(k_hist_export, dim3((unsigned)c->nnodes), dim3(256), 0, c->stream, c->hist, c->js, c->n_js_last, c->F, c->B, c->NK,
                       c->NAg, c->loss, c->qscale_buf[c->q_tree], c->status, c->nnodes, 1 << (c->D - 1), out_dev);
    HIPCHK(hipGetLastError());
    return EVT_OK;
}
