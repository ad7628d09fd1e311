// Centroid update of the LBG loop (src/utils.rs:83-102) as a deterministic ordered sum.
//
// The reference gathers the members of every cluster in row order and calls mean_vector
// (src/vector.rs:282-318).  Order of the f32 additions, per cluster:
//   1..1024 members ("small"): one sequential sum in row order from 0.0 — the reference's own,
//       deterministic order.  The rows of the small clusters are grouped by code with a STABLE
//       counting sort (per-part histograms -> exclusive scans -> ballot-ranked scatter of row
//       ids) and every cluster's list is walked by one lane per component.
//   more than 1024 ("large"): the reference switches to a Rayon reduce whose tree depends on
//       work stealing and cannot be reproduced even by itself.  Here the order is fixed as:
//       the rows are cut into parts of 4096 consecutive rows; inside a part the cluster's
//       members are added in row order from 0.0; the per-part sums are added in part order
//       from 0.0.  For 32-byte sub-vectors this is one streaming pass over the rows
//       (k_lbg_stream8) with the accumulators in LDS; other shapes take per-part leaves
//       through the gather path.
// No floating-point atomics anywhere; integer LDS atomics only for the histograms.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "assign_mfma.hpp"

namespace vq {

constexpr int kPartRows = 4096;      // rows per part (histogram block and summation part)
constexpr int kScanSeg = 32;         // parts per scan segment
constexpr int kMaxK = 256;           // codes are uint8
constexpr int kSeqMax = 1024;        // PARALLEL_THRESHOLD, src/vector.rs:16

struct LbgState {
    // per column block s
    int *changed;          // m
    int *done;             // m
    int *iters;            // m
    int *used;             // m   re-seed entries consumed so far
    int *ubase;            // m   value of used[s] at the start of the current update
    int *nleaves;          // m
    int *nsmall;           // m   clusters with 1..1024 members
    int *err;              // 1   set to 1 when a re-seed stream runs out
    // per (s, j)
    uint32_t *count;       // m*256
    uint32_t *start;       // m*256 first position of cluster j in perm[s]
    uint32_t *leaf_start;  // m*256
    uint32_t *empty_rank;  // m*256 rank of an empty cluster among the empty clusters of s
    // bulk
    uint32_t *hist;        // m*nparts*256 (histogram, then exclusive prefix over parts)
    uint32_t *seg;         // m*nseg*256 (per-segment sums, then exclusive prefix over segments)
    uint32_t *perm;        // m*n  row ids grouped by code, row order inside a group
    uint2 *leaf_desc;      // m*leaf_cap  [lo, hi) positions in perm[s]
    float *leaf_sum;       // m*leaf_cap*sd
    float *part_sum;       // m*nparts*256*8 per-part sums of the streaming kernel, or null
    uint8_t *codes;        // m*n  (column-block major)
    int nparts;
    int nseg;
    int leaf_cap;
    int stream;            // 1: the large clusters are summed by k_lbg_stream8 / k_lbg_combine8
};

// The short kernels of the gather path run beside the streaming kernel, whose waves keep the
// vector ALU busy: their waves are given the higher issue priority, or they would wait for it.
__device__ __forceinline__ void side_chain_priority() { __builtin_amdgcn_s_setprio(3); }

static __global__ void k_lbg_init(LbgState st, int m) {
    int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s < m) {
        st.changed[s] = 0;
        st.done[s] = 0;
        st.iters[s] = 0;
        st.used[s] = 0;
        st.ubase[s] = 0;
        st.nleaves[s] = 0;
        st.nsmall[s] = 0;
    }
    if (s == 0) st.err[0] = 0;
}

// codebook[s][j][t] = x[idx[s][j]][s*sd + t]     (src/utils.rs:54)
static __global__ void k_gather_rows(const float *__restrict__ x, int64_t ld, int m, int k, int sd,
                              const uint32_t *__restrict__ idx, float *__restrict__ cb) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t total = (int64_t)m * k * sd;
    if (i >= total) return;
    int t = (int)(i % sd);
    int64_t sj = i / sd;
    int s = (int)(sj / k);
    cb[i] = x[(int64_t)idx[sj] * ld + (int64_t)s * sd + t];
}

// The same from a residual whose update is still pending (one column block):
// codebook[j][t] = x[idx[j]][t] - pend_cb[pend_codes[idx[j]]][t], the row as the update will leave it.
static __global__ void k_gather_rows_pend(const float *__restrict__ x, int64_t ld, int k, int sd,
                                          const uint32_t *__restrict__ idx, float *__restrict__ cb,
                                          const float *__restrict__ pend_cb, const uint8_t *__restrict__ pend_codes) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)k * sd) return;
    const int t = (int)(i % sd);
    const uint32_t row = idx[i / sd];
    cb[i] = x[(int64_t)row * ld + t] - pend_cb[(size_t)pend_codes[row] * sd + t];
}

// One wave per (part, column block): histogram of the codes of kPartRows rows.
static __global__ void __launch_bounds__(64) k_lbg_hist(LbgState st, int64_t n) {
    side_chain_priority();
    const int s = blockIdx.y, b = blockIdx.x;
    if (st.done[s]) return;
    __shared__ uint32_t cnt[kMaxK];
    for (int j = threadIdx.x; j < kMaxK; j += 64) cnt[j] = 0;
    __syncthreads();
    const uint8_t *codes = st.codes + (size_t)s * n;
    int64_t lo = (int64_t)b * kPartRows;
    int64_t hi = lo + kPartRows < n ? lo + kPartRows : n;
    if (hi - lo == kPartRows && ((uintptr_t)(codes + lo) & 15) == 0) {
        // a full part: every lane takes 64 consecutive codes with four loads in flight together
        // (a histogram does not care which lane counts which row)
        const uint4 *cp = reinterpret_cast<const uint4 *>(codes + lo) + threadIdx.x * 4;
        uint4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = cp[u];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int sh = 0; sh < 32; sh += 8) atomicAdd(&cnt[(w[q] >> sh) & 255u], 1u);
        }
    } else {
        for (int64_t i = lo + threadIdx.x; i < hi; i += 64) atomicAdd(&cnt[codes[i]], 1u);
    }
    __syncthreads();
    uint32_t *h = st.hist + ((size_t)s * st.nparts + b) * kMaxK;
    for (int j = threadIdx.x; j < kMaxK; j += 64) h[j] = cnt[j];
}

// Scan step 1: per (column block, segment of kScanSeg parts) sum of the histograms.
static __global__ void __launch_bounds__(256) k_lbg_scan_seg(LbgState st) {
    side_chain_priority();
    const int s = blockIdx.y, g = blockIdx.x, j = threadIdx.x;
    if (st.done[s]) return;
    const int b0 = g * kScanSeg, b1 = (b0 + kScanSeg < st.nparts) ? b0 + kScanSeg : st.nparts;
    const uint32_t *h = st.hist + ((size_t)s * st.nparts + b0) * kMaxK + j;
    uint32_t sum = 0;
    uint32_t v[kScanSeg];  // all loads of the segment in flight together
#pragma unroll
    for (int u = 0; u < kScanSeg; ++u) v[u] = h[(size_t)(b0 + u < b1 ? u : b1 - 1 - b0) * kMaxK];
#pragma unroll
    for (int u = 0; u < kScanSeg; ++u) sum += (b0 + u < b1) ? v[u] : 0u;
    st.seg[((size_t)s * st.nseg + g) * kMaxK + j] = sum;
}

// Scan step 2 ("plan"): one workgroup of 256 threads per column block; thread j owns cluster j.
// Segment sums -> exclusive prefixes; per cluster: count, first position in perm, first leaf,
// rank among the empty clusters; per column block: number of leaves and of small clusters, and
// the re-seed cursor advanced by the number of empty clusters.
// Leaves: a small cluster (1..1024 members) is one leaf over its whole member list; a large
// cluster has one leaf per part, unless the streaming kernel sums the large clusters.
static __global__ void __launch_bounds__(256) k_lbg_plan(LbgState st, int k) {
    side_chain_priority();
    const int s = blockIdx.x, j = threadIdx.x;
    if (st.done[s]) return;
    __shared__ uint32_t sh_cnt[4], sh_leaf[4], sh_empty[4], sh_small[4];  // totals of the four waves
    uint32_t run = 0;
    uint32_t *h = st.seg + (size_t)s * st.nseg * kMaxK + j;
    for (int g0 = 0; g0 < st.nseg; g0 += 8) {
        uint32_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = (g0 + u < st.nseg) ? h[(size_t)(g0 + u) * kMaxK] : 0u;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (g0 + u < st.nseg) h[(size_t)(g0 + u) * kMaxK] = run;
            run += v[u];
        }
    }
    const bool live = j < k;
    const uint32_t cnt = live ? run : 0;
    const bool small = cnt > 0 && cnt <= (uint32_t)kSeqMax;
    const bool big = cnt > (uint32_t)kSeqMax;
    const uint32_t nl = small ? 1u : ((big && !st.stream) ? (uint32_t)st.nparts : 0u);
    const uint32_t emp = (live && cnt == 0) ? 1u : 0u;
    // exclusive prefixes over j: inside a wave by shuffles, the three waves before by their totals
    // (a serial walk per thread is 4 x 255 dependent LDS reads for the last one: 10 us on this chain)
    uint32_t ic = cnt, il = nl, ie = emp, is = small ? 1u : 0u;  // inclusive inside the wave
    const int lane = j & 63, wv = j >> 6;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t oc = __shfl_up(ic, off), ol = __shfl_up(il, off), oe = __shfl_up(ie, off), os = __shfl_up(is, off);
        if (lane >= off) {
            ic += oc;
            il += ol;
            ie += oe;
            is += os;
        }
    }
    if (lane == 63) {
        sh_cnt[wv] = ic;
        sh_leaf[wv] = il;
        sh_empty[wv] = ie;
        sh_small[wv] = is;
    }
    __syncthreads();
    uint32_t pc = ic - cnt, pl = il - nl, pe = ie - emp, ps = is - (small ? 1u : 0u);
    for (int u = 0; u < wv; ++u) {
        pc += sh_cnt[u];
        pl += sh_leaf[u];
        pe += sh_empty[u];
        ps += sh_small[u];
    }
    const size_t sj = (size_t)s * kMaxK + j;
    st.count[sj] = cnt;
    st.start[sj] = pc;
    st.leaf_start[sj] = pl;
    st.empty_rank[sj] = pe;
    if (small) st.leaf_desc[(size_t)s * st.leaf_cap + pl] = make_uint2(pc, pc + cnt);
    if (j == kMaxK - 1) {
        st.nleaves[s] = (int)(pl + nl);
        st.nsmall[s] = (int)(ps + (small ? 1u : 0u));
        int u = st.used[s];
        st.ubase[s] = u;
        st.used[s] = u + (int)(pe + emp);
    }
}

// Scan step 3: per (column block, segment): histograms -> exclusive prefixes over parts (offset
// of part b inside cluster j), in place; emits the per-part leaves of the large clusters when
// they are summed by the gather path.
static __global__ void __launch_bounds__(256) k_lbg_scan_blocks(LbgState st) {
    side_chain_priority();
    const int s = blockIdx.y, g = blockIdx.x, j = threadIdx.x;
    if (st.done[s]) return;
    const int b0 = g * kScanSeg, b1 = (b0 + kScanSeg < st.nparts) ? b0 + kScanSeg : st.nparts;
    uint32_t *h = st.hist + ((size_t)s * st.nparts + b0) * kMaxK + j;
    uint32_t run = st.seg[((size_t)s * st.nseg + g) * kMaxK + j];
    const size_t sj = (size_t)s * kMaxK + j;
    const bool leaves = !st.stream && st.count[sj] > (uint32_t)kSeqMax;
    const uint32_t first = st.start[sj];
    uint2 *desc = st.leaf_desc + (size_t)s * st.leaf_cap + st.leaf_start[sj] + b0;
    // the segment's entries in one memory round trip (unconditional loads, clamped to the last part)
    uint32_t v[kScanSeg];
#pragma unroll
    for (int u = 0; u < kScanSeg; ++u) v[u] = h[(size_t)(b0 + u < b1 ? u : b1 - 1 - b0) * kMaxK];
#pragma unroll
    for (int u = 0; u < kScanSeg; ++u) {
        if (b0 + u < b1) {
            h[(size_t)u * kMaxK] = run;
            if (leaves) desc[u] = make_uint2(first + run, first + run + v[u]);
            run += v[u];
        }
    }
}

// One wave per (part, column block): stable ranked scatter of row ids into perm[s].  When the
// streaming kernel sums the large clusters only the rows of small clusters are listed.
static __global__ void __launch_bounds__(64) k_lbg_scatter(LbgState st, int64_t n) {
    side_chain_priority();
    const int s = blockIdx.y, b = blockIdx.x;
    if (st.done[s]) return;
    if (st.stream && st.nsmall[s] == 0) return;
    __shared__ uint32_t base[kMaxK];
    __shared__ uint8_t listed[kMaxK];
    // codes are staged a quarter of the part at a time (16 per lane, the next quarter's load in
    // flight meanwhile): the workgroup keeps 2.3 KB of LDS and fits beside the streaming kernel
    constexpr int kStage = kPartRows / 4;
    __shared__ __attribute__((aligned(16))) uint8_t pcodes[kStage];
    const uint32_t *h = st.hist + ((size_t)s * st.nparts + b) * kMaxK;
    const uint32_t *start = st.start + (size_t)s * kMaxK;
    const uint32_t *count = st.count + (size_t)s * kMaxK;
    for (int j = threadIdx.x; j < kMaxK; j += 64) {
        base[j] = start[j] + h[j];
        listed[j] = (!st.stream || count[j] <= (uint32_t)kSeqMax) ? 1 : 0;
    }
    const uint8_t *codes = st.codes + (size_t)s * n;
    uint32_t *perm = st.perm + (size_t)s * n;
    const int lane = threadIdx.x;
    const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    int64_t lo = (int64_t)b * kPartRows;
    int64_t hi = lo + kPartRows < n ? lo + kPartRows : n;
    const bool vec = ((uintptr_t)(codes + lo) & 15) == 0;
    auto fetch = [&](int64_t q0) {  // codes of rows q0 + 16 lane .. + 15; rows from hi on read as 0, never used
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        const int64_t r0 = q0 + 16 * lane;
        if (vec && r0 + 16 <= hi) {
            v = *reinterpret_cast<const uint4 *>(codes + r0);
        } else {
            uint32_t w[4] = {0u, 0u, 0u, 0u};
            for (int u = 0; u < 16; ++u)
                if (r0 + u < hi) w[u >> 2] |= (uint32_t)codes[r0 + u] << (8 * (u & 3));
            v = make_uint4(w[0], w[1], w[2], w[3]);
        }
        return v;
    };
    uint4 ahead = fetch(lo);
    for (int64_t q0 = lo; q0 < hi; q0 += kStage) {
        __syncthreads();  // the previous quarter has been consumed (and base / listed are written)
        reinterpret_cast<uint4 *>(pcodes)[lane] = ahead;
        if (q0 + kStage < hi) ahead = fetch(q0 + kStage);
        __syncthreads();
        const int64_t qhi = q0 + kStage < hi ? q0 + kStage : hi;
        for (int64_t i0 = q0; i0 < qhi; i0 += 64) {
            int64_t i = i0 + lane;
            bool valid = i < hi;
            uint32_t c = valid ? pcodes[i - q0] : 0u;
            valid = valid && listed[c];
            uint64_t mask = __ballot(valid);
            if (mask == 0) continue;  // uniform
            if (__popcll(mask) <= 4) {
                // few listed rows (the small clusters beside the streaming kernel): one lane at a time,
                // in lane = row order; LDS operations of one wave are performed in program order
                for (uint64_t mm = mask; mm; mm &= mm - 1) {
                    if (lane == __ffsll((unsigned long long)mm) - 1) {
                        const uint32_t pos = base[c];
                        base[c] = pos + 1;
                        perm[pos] = (uint32_t)i;
                    }
                    __builtin_amdgcn_wave_barrier();
                }
                continue;
            }
    #pragma unroll
            for (int bit = 0; bit < 8; ++bit) {
                bool set = (c >> bit) & 1u;
                uint64_t bal = __ballot(set);
                mask &= set ? bal : ~bal;
            }
            // lanes with equal code and valid: mask (invalid lanes have a stale mask, unused)
            uint32_t rank = (uint32_t)__popcll(mask & lt);
            uint32_t tot = (uint32_t)__popcll(mask);
            uint32_t pos = 0;
            if (valid) pos = base[c] + rank;
            __builtin_amdgcn_wave_barrier();  // one wave, LDS in program order: reads above, updates below
            if (valid && rank == 0) base[c] += tot;
            __builtin_amdgcn_wave_barrier();
            if (valid) perm[pos] = (uint32_t)i;
        }
    }
}

// The same scatter by a workgroup of four waves per (part, column block): wave w ranks the rows
// [1024 w, 1024 w + 1024) of the part.  A first sweep counts the listed codes of each quarter, so
// that a wave's first position inside cluster j is the part's position plus the members in the
// quarters before its own; the order of the rows inside a cluster stays the row order.  One wave
// per part is a chain of 64 dependent LDS round trips per part (and a handful of waves on the whole
// GPU when there is one column block).
static __global__ void __launch_bounds__(256) k_lbg_scatter_wg(LbgState st, int64_t n) {
    side_chain_priority();
    const int s = blockIdx.y, b = blockIdx.x;
    if (st.done[s]) return;
    if (st.stream && st.nsmall[s] == 0) return;
    constexpr int kQuarter = kPartRows / 4;
    __shared__ uint32_t cntq[4][kMaxK];
    __shared__ uint32_t base[4][kMaxK];
    __shared__ uint8_t listed[kMaxK];
    __shared__ __attribute__((aligned(16))) uint8_t pcodes[kPartRows];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const uint8_t *codes = st.codes + (size_t)s * n;
    uint32_t *perm = st.perm + (size_t)s * n;
    const int64_t lo = (int64_t)b * kPartRows;
    const int64_t hi = lo + kPartRows < n ? lo + kPartRows : n;
    const int rows = (int)(hi - lo);
    for (int j = threadIdx.x; j < 4 * kMaxK; j += 256) (&cntq[0][0])[j] = 0u;
    listed[threadIdx.x] = (!st.stream || st.count[(size_t)s * kMaxK + threadIdx.x] <= (uint32_t)kSeqMax) ? 1 : 0;
    // the part's codes into LDS, 16 per thread
    {
        const int64_t r0 = lo + 16 * (int64_t)threadIdx.x;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (((uintptr_t)(codes + lo) & 15) == 0 && r0 + 16 <= hi) {
            v = *reinterpret_cast<const uint4 *>(codes + r0);
        } else {
            uint32_t q[4] = {0u, 0u, 0u, 0u};
            for (int u = 0; u < 16; ++u)
                if (r0 + u < hi) q[u >> 2] |= (uint32_t)codes[r0 + u] << (8 * (u & 3));
            v = make_uint4(q[0], q[1], q[2], q[3]);
        }
        reinterpret_cast<uint4 *>(pcodes)[threadIdx.x] = v;
    }
    __syncthreads();
    const int q0 = w * kQuarter, q1 = q0 + kQuarter < rows ? q0 + kQuarter : rows;
    for (int i = q0 + lane; i < q1; i += 64) {
        const uint32_t c = pcodes[i];
        if (listed[c]) atomicAdd(&cntq[w][c], 1u);
    }
    __syncthreads();
    {
        const uint32_t *h = st.hist + ((size_t)s * st.nparts + b) * kMaxK;
        const uint32_t *start = st.start + (size_t)s * kMaxK;
        const int j = threadIdx.x;  // kMaxK == 256 threads
        uint32_t run = start[j] + h[j];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            base[q][j] = run;
            run += cntq[q][j];
        }
    }
    __syncthreads();
    uint32_t *mybase = base[w];
    const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    for (int i0 = q0; i0 < q1; i0 += 64) {
        const int i = i0 + lane;
        bool valid = i < q1;
        const uint32_t c = valid ? pcodes[i] : 0u;
        valid = valid && listed[c];
        uint64_t mask = __ballot(valid);
        if (mask == 0) continue;  // uniform
#pragma unroll
        for (int bit = 0; bit < 8; ++bit) {
            const bool set = (c >> bit) & 1u;
            const uint64_t bal = __ballot(set);
            mask &= set ? bal : ~bal;
        }
        // lanes with equal code and valid: mask (invalid lanes have a stale mask, unused)
        const uint32_t rank = (uint32_t)__popcll(mask & lt);
        const uint32_t tot = (uint32_t)__popcll(mask);
        uint32_t pos = 0;
        if (valid) pos = mybase[c] + rank;
        __builtin_amdgcn_wave_barrier();  // one wave per table, LDS in program order: reads above, updates below
        if (valid && rank == 0) mybase[c] += tot;
        __builtin_amdgcn_wave_barrier();
        if (valid) perm[pos] = (uint32_t)(lo + i);
    }
}

// One lane per (leaf, component): sequential sum of the leaf's members in list order.
static __global__ void __launch_bounds__(256) k_lbg_leafsum(LbgState st, const float *__restrict__ x,
                                                     int64_t n, int64_t ld, int sd) {
    const int s = blockIdx.y;
    if (st.done[s]) return;
    int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t leaf = gid / sd;
    int t = (int)(gid % sd);
    if (leaf >= st.nleaves[s]) return;
    uint2 d = st.leaf_desc[(size_t)s * st.leaf_cap + leaf];
    const uint32_t *__restrict__ perm = st.perm + (size_t)s * n;
    const float *__restrict__ xc = x + (int64_t)s * sd + t;
    float acc = 0.0f;
    // Batches of 16 members: the loads of a batch are independent (issued unconditionally, a batch
    // past the end of the list repeats its last row and is not added), the adds stay in list order;
    // the row ids of the next batch are fetched while the current rows are in flight.
    constexpr int B = 16;
    uint32_t rn[B];
    const uint32_t lastp = d.y - 1;  // leaves are never empty
#pragma unroll
    for (int u = 0; u < B; ++u) rn[u] = perm[d.x + u < d.y ? d.x + u : lastp];
    for (uint32_t p = d.x; p < d.y; p += B) {
        float v[B];
#pragma unroll
        for (int u = 0; u < B; ++u) v[u] = xc[(int64_t)rn[u] * ld];
#pragma unroll
        for (int u = 0; u < B; ++u) rn[u] = perm[p + B + u < d.y ? p + B + u : lastp];
        const uint32_t cnt = d.y - p;  // the same in every lane of the leaf
#pragma unroll
        for (int u = 0; u < B; ++u)
            if ((uint32_t)u < cnt) acc = acc + v[u];
    }
    st.leaf_sum[((size_t)s * st.leaf_cap + leaf) * sd + t] = acc;
}

// Narrow column blocks (sub_dim a power of two up to 32): one wave per leaf.  A lane-per-component
// walk as above leaves most of the wave idle and pays one memory round trip per 32 members; here
// the 64 lanes fetch up to 2048 / sub_dim members at a time into LDS (row ids first, then the
// sub-vectors, all loads of a chunk in flight together), and lanes 0..sub_dim-1 add them in list
// order.
constexpr int kLeafStage = 2048;  // floats staged per wave

static __global__ void __launch_bounds__(256) k_lbg_leafsum_wave(LbgState st, const float *__restrict__ x,
                                                                 int64_t n, int64_t ld, int sd, int sd_shift) {
    const int s = blockIdx.y;
    if (st.done[s]) return;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int64_t leaf = (int64_t)blockIdx.x * 4 + w;
    if (leaf >= st.nleaves[s]) return;  // uniform per wave; the waves never synchronise
    __shared__ float stage_all[4][kLeafStage];
    float *stage = stage_all[w];
    const uint2 d = st.leaf_desc[(size_t)s * st.leaf_cap + leaf];
    const uint32_t *__restrict__ perm = st.perm + (size_t)s * n;
    const float *__restrict__ xs = x + (int64_t)s * sd;
    const uint32_t chunk = (uint32_t)(kLeafStage >> sd_shift);  // members per chunk
    constexpr int E = kLeafStage / 64;                          // elements per lane and chunk
    float acc = 0.0f;
    for (uint32_t p = d.x; p < d.y; p += chunk) {
        const uint32_t cm = (d.y - p < chunk) ? d.y - p : chunk;
        const uint32_t tot = cm << sd_shift;
        uint32_t row[E];
        float v[E];
#pragma unroll
        for (int i = 0; i < E; ++i) {
            const uint32_t e = (uint32_t)lane + 64u * i;
            row[i] = (e < tot) ? perm[p + (e >> sd_shift)] : 0u;
        }
#pragma unroll
        for (int i = 0; i < E; ++i) {
            const uint32_t e = (uint32_t)lane + 64u * i;
            v[i] = (e < tot) ? xs[(int64_t)row[i] * ld + (e & (uint32_t)(sd - 1))] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < E; ++i) stage[lane + 64 * i] = v[i];
        __builtin_amdgcn_wave_barrier();
        if (lane < sd) {
            uint32_t mbr = 0;
            for (; mbr + 8 <= cm; mbr += 8) {
                float t[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) t[u] = stage[((mbr + u) << sd_shift) + lane];
#pragma unroll
                for (int u = 0; u < 8; ++u) acc = acc + t[u];
            }
            for (; mbr < cm; ++mbr) acc = acc + stage[(mbr << sd_shift) + lane];
        }
        __builtin_amdgcn_wave_barrier();
    }
    if (lane < sd) st.leaf_sum[((size_t)s * st.leaf_cap + leaf) * sd + lane] = acc;
}

// Few, long leaves (the small clusters beside the streaming kernel: up to 1024 members each): one
// workgroup per leaf.  All 256 threads fetch the members of a chunk (row ids, then 16-byte pieces
// of the sub-vectors, every load of the chunk in flight together) and store them transposed in
// LDS; lanes 0..sub_dim-1 of wave 0 then add them in list order, four members per LDS read.  The
// chain of dependent adds is the only serial part left.
constexpr int kLeafWgFloats = 8192;  // floats staged per chunk

static __global__ void __launch_bounds__(256) k_lbg_leafsum_wg(LbgState st, const float *__restrict__ x, int64_t n,
                                                               int64_t ld, int sd, int sd_shift) {
    side_chain_priority();
    const int s = blockIdx.y;
    if (st.done[s]) return;
    const int64_t leaf = blockIdx.x;
    if (leaf >= st.nleaves[s]) return;  // uniform per workgroup
    __shared__ float stage[kLeafWgFloats + 4 * 32];
    const int tid = threadIdx.x;
    const uint2 d = st.leaf_desc[(size_t)s * st.leaf_cap + leaf];
    const uint32_t *__restrict__ perm = st.perm + (size_t)s * n;
    const float *__restrict__ xs = x + (int64_t)s * sd;
    const uint32_t chunk = (uint32_t)(kLeafWgFloats >> sd_shift);  // members per chunk, a multiple of 4
    const uint32_t stride = chunk + 4;                             // floats per component row in LDS
    const int pshift = sd_shift - 2;                               // 16-byte pieces per member: 1 << pshift
    constexpr int E = kLeafWgFloats / 4 / 256;                     // pieces per thread and chunk
    float acc = 0.0f;
    for (uint32_t p = d.x; p < d.y; p += chunk) {
        const uint32_t cm = (d.y - p < chunk) ? d.y - p : chunk;
        const uint32_t tot = cm << pshift;
        uint32_t row[E];
        float4 v[E];
#pragma unroll
        for (int i = 0; i < E; ++i) {
            const uint32_t e = (uint32_t)tid + 256u * i;
            row[i] = (e < tot) ? perm[p + (e >> pshift)] : 0u;
        }
#pragma unroll
        for (int i = 0; i < E; ++i) {
            const uint32_t e = (uint32_t)tid + 256u * i;
            const uint32_t piece = e & ((1u << pshift) - 1u);
            v[i] = (e < tot) ? *reinterpret_cast<const float4 *>(xs + (int64_t)row[i] * ld + 4 * piece)
                             : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        __syncthreads();  // the previous chunk has been added
#pragma unroll
        for (int i = 0; i < E; ++i) {
            const uint32_t e = (uint32_t)tid + 256u * i;
            if (e < tot) {
                const uint32_t mbr = e >> pshift, t0 = 4 * (e & ((1u << pshift) - 1u));
                stage[(t0 + 0) * stride + mbr] = v[i].x;
                stage[(t0 + 1) * stride + mbr] = v[i].y;
                stage[(t0 + 2) * stride + mbr] = v[i].z;
                stage[(t0 + 3) * stride + mbr] = v[i].w;
            }
        }
        __syncthreads();
        if (tid < sd) {
            const float *mine = stage + (size_t)tid * stride;
            uint32_t mbr = 0;
            for (; mbr + 16 <= cm; mbr += 16) {
                float4 q[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) q[u] = *reinterpret_cast<const float4 *>(mine + mbr + 4 * u);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    acc = acc + q[u].x;
                    acc = acc + q[u].y;
                    acc = acc + q[u].z;
                    acc = acc + q[u].w;
                }
            }
            for (; mbr < cm; ++mbr) acc = acc + mine[mbr];
        }
    }
    if (tid < sd) st.leaf_sum[((size_t)s * st.leaf_cap + leaf) * sd + tid] = acc;
}

// One lane per (cluster, component): the mean of a small cluster, the sequential fold over the
// per-part leaves of a large one (gather path), or the re-seed row of an empty cluster
// (src/vector.rs:315-316, src/utils.rs:98-101).
static __global__ void __launch_bounds__(256) k_lbg_finalize(LbgState st, const float *__restrict__ x,
                                                      int64_t ld, int k, int sd,
                                                      const uint32_t *__restrict__ reseed,
                                                      int n_reseed, float *__restrict__ cb) {
    const int s = blockIdx.y;
    if (st.done[s]) return;
    int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int j = (int)(gid / sd);
    int t = (int)(gid % sd);
    if (j >= k) return;
    const size_t sj = (size_t)s * kMaxK + j;
    uint32_t cnt = st.count[sj];
    float *out = cb + ((size_t)s * k + j) * sd + t;
    if (cnt == 0) {
        int pos = st.ubase[s] + (int)st.empty_rank[sj];
        if (pos >= n_reseed) {
            st.err[0] = 1;
            return;
        }
        uint32_t r = reseed[(size_t)s * n_reseed + pos];
        *out = x[(int64_t)r * ld + (int64_t)s * sd + t];
        return;
    }
    const float *ls = st.leaf_sum + ((size_t)s * st.leaf_cap + st.leaf_start[sj]) * sd + t;
    float sum;
    if (cnt <= (uint32_t)kSeqMax) {
        sum = ls[0];
    } else {
        if (st.stream) return;  // k_lbg_combine8 writes the large clusters
        // the per-part sums in part order; 64 loads in flight (the kernel's time is memory round
        // trips; with 245 parts of a million rows the 64 MB of leaf sums then come in at the HBM rate),
        // the adds one chain
        sum = 0.0f;
        constexpr int B = 64;
        const int np = st.nparts;
        for (int p = 0; p < np; p += B) {
            float v[B];
#pragma unroll
            for (int u = 0; u < B; ++u) v[u] = ls[(size_t)(p + u < np ? p + u : np - 1) * sd];
#pragma unroll
            for (int u = 0; u < B; ++u)
                if (p + u < np) sum = sum + v[u];
        }
    }
    *out = sum / __uint2float_rn(cnt);
}

// ---- streaming sums of the large clusters (sub_dim 8, 4 column blocks per 128-byte line) ------
// One workgroup per (part, group of 4 column blocks); wave w of the group owns column block
// 4g + w, so the four waves together consume whole 128-byte lines of the rows.  A wave walks
// its part 64 rows at a time; a lane holds the 32-byte sub-vector of its row.  The rows of a
// chunk are ranked inside their cluster with wave ballots and added to the cluster's
// accumulator in LDS in rank order (round r: the lanes of rank r, all on different clusters) —
// so every cluster receives its rows of this part in row order, one at a time, starting from
// 0.0.  Emits the per-part sums (k_lbg_hist counts the members, on another stream at the same
// time); no floating-point atomics.  The four waves meet at a workgroup barrier before every
// chunk (the barrier waits for nothing else: the prefetches stay in flight): each of them reads
// a different 32-byte quarter of the same lines, and waves that drift apart by the length of
// their prefetch queues find those lines gone from the compute unit's cache.
static __global__ void __launch_bounds__(256) k_lbg_stream8(LbgState st, const float *__restrict__ x, int64_t n,
                                                            int64_t ld) {
    const int g = blockIdx.y, b = blockIdx.x;
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int s = 4 * g + w;
    __shared__ float4 acc_lo[4][kMaxK], acc_hi[4][kMaxK];  // components 0-3 and 4-7 of every cluster
    if (st.done[4 * g] && st.done[4 * g + 1] && st.done[4 * g + 2] && st.done[4 * g + 3]) return;
    float4 *alo = acc_lo[w], *ahi = acc_hi[w];
    for (int i = lane; i < kMaxK; i += 64) {
        alo[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        ahi[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __builtin_amdgcn_wave_barrier();
    const int64_t lo = (int64_t)b * kPartRows;
    const int64_t hi = lo + kPartRows < n ? lo + kPartRows : n;
    constexpr int PF = 3;
    const int rows = (int)(hi - lo);
    const int nchunks = (rows + 63) / 64, rows_last = rows - 64 * (nchunks - 1);
    const int nsteps = (nchunks + PF - 1) / PF * PF;  // chunk steps of the loop below, one barrier each
    if (st.done[s]) {  // this wave's column block has stopped: it only keeps the others' barriers company
        for (int c = 0; c < nsteps; ++c) __builtin_amdgcn_s_barrier();
        return;
    }
    // The sub-vectors and codes of the next PF chunks are kept in flight: one chunk's arithmetic
    // is far shorter than a memory round trip.  The loads are unconditional and in chunk order (a
    // load under a branch, or out of order, makes the compiler wait for every load in flight at
    // the first use): a lane without a row in the part's last chunk reads that chunk's first row,
    // the fetches past the last chunk read that chunk again, and both are dropped.
    float4 b0[PF], b1[PF];
    uint8_t bc[PF];  // (bytes until they are used: widened where they are loaded, they would be waited for there)
    // Lanes 2p and 2p+1 fetch the two 16-byte halves of row p of the chunk (b0) and of row 32 + p
    // (b1): one load instruction touches each 64-byte piece of a line once instead of twice.  The
    // neighbours then swap a half, so that lane 2p owns row p and lane 2p + 1 owns row 32 + p.
    const int pr = lane >> 1, hf = lane & 1;
    const int ridx = hf ? 32 + pr : pr;  // this lane's row of a chunk
    // addresses: a scalar base per chunk plus 32-bit lane offsets (a part spans 4096 rows: the
    // host keeps the leading dimension below 2^20 floats)
    const char *xbase = reinterpret_cast<const char *>(x + lo * ld + (int64_t)s * 8);
    const uint8_t *cbase = st.codes + (size_t)s * n + lo;
    const uint32_t hoff = 16u * (uint32_t)hf;
    const uint32_t f0 = 4u * (uint32_t)pr * (uint32_t)ld + hoff, f1 = f0 + 128u * (uint32_t)ld;
    const uint32_t l0 = pr < rows_last ? f0 : hoff, l1 = 32 + pr < rows_last ? f1 : hoff;
    const uint32_t lc = ridx < rows_last ? (uint32_t)ridx : 0u;
    const int64_t chunkb = 256 * ld;  // bytes of 64 rows
    auto fetch = [&](int chunk, float4 &d0, float4 &d1, uint8_t &dc) {
        const int cc = chunk < nchunks ? chunk : nchunks - 1;  // uniform
        const bool last = cc == nchunks - 1;
        const char *xb = xbase + cc * chunkb;
        const uint8_t *cb = cbase + 64 * cc;
        d0 = *reinterpret_cast<const float4 *>(xb + (uint64_t)(last ? l0 : f0));
        d1 = *reinterpret_cast<const float4 *>(xb + (uint64_t)(last ? l1 : f1));
        dc = cb[last ? lc : (uint32_t)ridx];
    };
#pragma unroll
    for (int u = 0; u < PF; ++u) {
        fetch(u, b0[u], b1[u], bc[u]);
        __builtin_amdgcn_sched_barrier(0);
    }
    // lanes whose row comes before this lane's row
    const unsigned long long even = 0x5555555555555555ull, below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    const unsigned long long ltm = hf ? (even | (~even & below)) : (even & below);
    const uint32_t lt_lo = (uint32_t)ltm, lt_hi = (uint32_t)(ltm >> 32);
    for (int base = 0; base < nsteps; base += PF) {
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            // (a chunk past the part's end has no pending lane and falls through: an exit from here,
            // which the compiler routes past the loop's head, would make it wait there for every
            // load in flight)
            __builtin_amdgcn_s_barrier();  // step base + u of nsteps
            const bool pending = 64 * (base + u) + ridx < rows;
            const float4 fa = b0[u], fb = b1[u];
            uint32_t c = pending ? (uint32_t)bc[u] : 0u;
            // swap: the even lane sends its half of row 32 + p, the odd lane its half of row p
            const float4 snd = hf ? fa : fb;
            float4 rcv;
            rcv.x = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(snd.x), 0xB1, 0xF, 0xF, true));
            rcv.y = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(snd.y), 0xB1, 0xF, 0xF, true));
            rcv.z = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(snd.z), 0xB1, 0xF, 0xF, true));
            rcv.w = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(snd.w), 0xB1, 0xF, 0xF, true));
            float4 v0 = hf ? rcv : fa;  // components 0-3 of this lane's row
            float4 v1 = hf ? fb : rcv;  // components 4-7
            // the slot's registers are free from here on (the empty statement pins the selects
            // above it): its next loads go out now
            asm volatile("" : "+v"(v0.x), "+v"(v0.y), "+v"(v0.z), "+v"(v0.w), "+v"(v1.x), "+v"(v1.y), "+v"(v1.z),
                         "+v"(v1.w), "+v"(c));
            fetch(base + u + PF, b0[u], b1[u], bc[u]);
            __builtin_amdgcn_sched_barrier(0);
            // Lanes of the same cluster, found with one wave ballot per code bit: a lane differs
            // from lane j when some bit of its code differs from j's bit in the ballot.
            const unsigned long long vb = __ballot(pending);
            uint32_t bad_lo = ~(uint32_t)vb, bad_hi = ~(uint32_t)(vb >> 32);
#pragma unroll
            for (int bit = 0; bit < 8; bit += 2) {
                const int sp0 = (int)(c << (31 - bit)) >> 31, sp1 = (int)(c << (30 - bit)) >> 31;  // 0 or -1
                const unsigned long long bal0 = __ballot(sp0 != 0), bal1 = __ballot(sp1 != 0);
                bad_lo = bad_lo | ((uint32_t)bal0 ^ (uint32_t)sp0) | ((uint32_t)bal1 ^ (uint32_t)sp1);
                bad_hi = bad_hi | ((uint32_t)(bal0 >> 32) ^ (uint32_t)sp0) | ((uint32_t)(bal1 >> 32) ^ (uint32_t)sp1);
            }
            const uint32_t same_lo = ~bad_lo, same_hi = ~bad_hi;
            const uint32_t rank =
                pending ? (uint32_t)(__popc(same_lo & lt_lo) + __popc(same_hi & lt_hi)) : 0xFFFFFFFFu;
            // Round r: the lanes of rank r (all on different clusters) add their rows.  LDS
            // operations of one wave are performed in program order, so the next round sees these
            // writes; the wave barrier only pins the compiler's schedule (a fence or s_barrier
            // here would also wait for the row prefetches in flight).
            for (uint32_t r = 0; __any(rank != 0xFFFFFFFFu && rank >= r); ++r) {
                if (rank == r) {
                    float4 a0 = alo[c], a1 = ahi[c];
                    a0.x = a0.x + v0.x;
                    a0.y = a0.y + v0.y;
                    a0.z = a0.z + v0.z;
                    a0.w = a0.w + v0.w;
                    a1.x = a1.x + v1.x;
                    a1.y = a1.y + v1.y;
                    a1.z = a1.z + v1.z;
                    a1.w = a1.w + v1.w;
                    alo[c] = a0;
                    ahi[c] = a1;
                }
                __builtin_amdgcn_wave_barrier();
            }
        }
    }
    __builtin_amdgcn_wave_barrier();
    float4 *ps = reinterpret_cast<float4 *>(st.part_sum) + ((size_t)s * st.nparts + b) * kMaxK * 2;
    for (int i = lane; i < kMaxK * 2; i += 64) ps[i] = (i & 1) ? ahi[i >> 1] : alo[i >> 1];
}

// One lane per (cluster, component): sequential fold of the per-part sums of a large cluster.
static __global__ void __launch_bounds__(256) k_lbg_combine8(LbgState st, int k, float *__restrict__ cb) {
    const int s = blockIdx.y;
    if (st.done[s]) return;
    const int gid = blockIdx.x * 256 + threadIdx.x;
    const int j = gid / 8, t = gid % 8;
    if (j >= k) return;
    const uint32_t cnt = st.count[(size_t)s * kMaxK + j];
    if (cnt <= (uint32_t)kSeqMax) return;
    const float *ps = st.part_sum + ((size_t)s * st.nparts * kMaxK + j) * 8 + t;
    // the kernel is a handful of waves: its time is memory round trips, so 32 loads are in flight
    // at a time (unconditional, clamped to the last part); the adds stay one chain in part order
    float sum = 0.0f;
    constexpr int B = 32;
    const int np = st.nparts;
    for (int p = 0; p < np; p += B) {
        float v[B];
#pragma unroll
        for (int u = 0; u < B; ++u) v[u] = ps[(size_t)(p + u < np ? p + u : np - 1) * kMaxK * 8];
#pragma unroll
        for (int u = 0; u < B; ++u)
            if (p + u < np) sum = sum + v[u];
    }
    cb[((size_t)s * k + j) * 8 + t] = sum / __uint2float_rn(cnt);
}

// The same fold for every cluster, sum only (big_sum[s][j][t]): it needs nothing from the gather
// path, so it can follow the streaming kernel at once; k_lbg_finalize_prep8 picks the large
// clusters' sums and divides.
static __global__ void __launch_bounds__(256) k_lbg_fold8(LbgState st, int k, float *__restrict__ big_sum) {
    const int s = blockIdx.y;
    if (st.done[s]) return;
    const int gid = blockIdx.x * 256 + threadIdx.x;
    const int j = gid / 8, t = gid % 8;
    if (j >= k) return;
    const float *ps = st.part_sum + ((size_t)s * st.nparts * kMaxK + j) * 8 + t;
    float sum = 0.0f;
    constexpr int B = 128;  // two memory round trips for the 245 parts of a million rows
    const int np = st.nparts;
    for (int p = 0; p < np; p += B) {
        float v[B];
#pragma unroll
        for (int u = 0; u < B; ++u) v[u] = ps[(size_t)(p + u < np ? p + u : np - 1) * kMaxK * 8];
#pragma unroll
        for (int u = 0; u < B; ++u)
            if (p + u < np) sum = sum + v[u];
    }
    big_sum[((size_t)s * kMaxK + j) * 8 + t] = sum;
}

// Loop control of src/utils.rs:57,104-106, one thread per column block.
static __global__ void k_lbg_advance(LbgState st, int m) {
    int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= m || st.done[s]) return;
    st.iters[s] += 1;
    if (!st.changed[s]) st.done[s] = 1;
    st.changed[s] = 0;
}

// The end of an update and the start of the next assignment pass, one workgroup per column block
// (8-float blocks, streaming path, matrix-core assignment).  Thread j makes centroid j — the mean
// of a small cluster from its leaf or of a large one from k_lbg_fold8's sum, the re-seed row of
// an empty cluster (src/vector.rs:315-316, src/utils.rs:98-101) — thread 0 does the loop
// control of src/utils.rs:57,104-106, and all of them the tables of k_assign_mfma_bf from the
// centroids they hold.  Needs x 16-byte aligned, ld % 4 == 0 (as the streaming kernel does).
static __global__ void __launch_bounds__(256) k_lbg_finalize_prep8(
    LbgState st, const float *__restrict__ x, int64_t ld, int k, const uint32_t *__restrict__ reseed, int n_reseed,
    float *__restrict__ cb, const float *__restrict__ big_sum, int nb, u32x4 *__restrict__ atab,
    float *__restrict__ maxc2, float *__restrict__ mu, uint32_t *__restrict__ stat) {
    const int s = blockIdx.x, j = threadIdx.x;
    if (s == 0 && j < kStatSlots) stat[j * kStatStride] = 0u;
    if (st.done[s]) return;  // the same in the whole workgroup; a finished block is skipped by the assignment
    float c[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (j < k) {
        const size_t sj = (size_t)s * kMaxK + j;
        const uint32_t cnt = st.count[sj];
        float4 *out = reinterpret_cast<float4 *>(cb + ((size_t)s * k + j) * 8);
        float4 lo4, hi4;
        bool write = true;
        if (cnt == 0) {
            const int pos = st.ubase[s] + (int)st.empty_rank[sj];
            if (pos >= n_reseed) {
                st.err[0] = 1;
                lo4 = out[0];  // the centroid stays
                hi4 = out[1];
                write = false;
            } else {
                const float4 *row =
                    reinterpret_cast<const float4 *>(x + (int64_t)reseed[(size_t)s * n_reseed + pos] * ld + (int64_t)s * 8);
                lo4 = row[0];
                hi4 = row[1];
            }
        } else {
            const float4 *ls = reinterpret_cast<const float4 *>(
                cnt <= (uint32_t)kSeqMax ? st.leaf_sum + ((size_t)s * st.leaf_cap + st.leaf_start[sj]) * 8
                                         : big_sum + ((size_t)s * kMaxK + j) * 8);
            const float d = __uint2float_rn(cnt);
            const float4 a = ls[0], b = ls[1];
            lo4 = make_float4(a.x / d, a.y / d, a.z / d, a.w / d);
            hi4 = make_float4(b.x / d, b.y / d, b.z / d, b.w / d);
        }
        if (write) {
            out[0] = lo4;
            out[1] = hi4;
        }
        c[0] = lo4.x, c[1] = lo4.y, c[2] = lo4.z, c[3] = lo4.w;
        c[4] = hi4.x, c[5] = hi4.y, c[6] = hi4.z, c[7] = hi4.w;
    }
    __syncthreads();  // every thread has read done[s]
    if (j == 0) {
        st.iters[s] += 1;
        if (!st.changed[s]) st.done[s] = 1;
        st.changed[s] = 0;
    }
    mfma_bf_prep_block(c, s, j, k, nb, atab, maxc2, mu);
}

}  // namespace vq
