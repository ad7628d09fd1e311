// Centroid update of the LBG loop (src/utils.rs:83-102) as a deterministic segmented sum.
//
// The reference gathers the members of every cluster in row order and calls mean_vector
// (src/vector.rs:282-318): a sequential f32 sum in row order for at most 1024 members.  To
// reproduce that order bit for bit the rows are first grouped by code with a STABLE counting
// sort (per-row-block histograms -> exclusive scan -> ranked scatter), then every cluster is
// summed by walking its member list in order, one lane per (leaf, component).  Clusters above
// 1024 members are split at the midpoint of the member list to the uniform depth
// d = min{d : count <= 1024 << d}; leaves are summed sequentially and combined left + right.
// No floating-point atomics anywhere; integer LDS atomics only for the histograms.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vq {

constexpr int kRowBlock = 2048;      // rows per histogram block
constexpr int kMaxK = 256;           // codes are uint8
constexpr int kLeafMax = 1024;       // PARALLEL_THRESHOLD, src/vector.rs:16

struct LbgState {
    // per column block s
    int *changed;          // m
    int *done;             // m
    int *iters;            // m
    int *used;             // m   re-seed entries consumed so far
    int *ubase;            // m   value of used[s] at the start of the current update
    int *nleaves;          // m
    int *err;              // 1   set to 1 when a re-seed stream runs out
    // per (s, j)
    uint32_t *count;       // m*256
    uint32_t *start;       // m*256 first position of cluster j in perm[s]
    uint32_t *leaf_start;  // m*256
    uint32_t *depth;       // m*256
    uint32_t *empty_rank;  // m*256 rank of an empty cluster among the empty clusters of s
    // bulk
    uint32_t *hist;        // m*nblk*256 (histogram, then exclusive prefix over blocks)
    uint32_t *perm;        // m*n  row ids grouped by code, row order inside a group
    uint2 *leaf_desc;      // m*leaf_cap  [lo, hi) positions in perm[s]
    float *leaf_sum;       // m*leaf_cap*sd
    uint8_t *codes;        // m*n  (column-block major)
    int nblk;
    int leaf_cap;
};

static __global__ void k_lbg_init(LbgState st, int m) {
    int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s < m) {
        st.changed[s] = 0;
        st.done[s] = 0;
        st.iters[s] = 0;
        st.used[s] = 0;
        st.ubase[s] = 0;
        st.nleaves[s] = 0;
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

// One wave per (row block, column block): histogram of the codes of kRowBlock rows.
static __global__ void __launch_bounds__(64) k_lbg_hist(LbgState st, int64_t n) {
    const int s = blockIdx.y, b = blockIdx.x;
    if (st.done[s]) return;
    __shared__ uint32_t cnt[kMaxK];
    for (int j = threadIdx.x; j < kMaxK; j += 64) cnt[j] = 0;
    __syncthreads();
    const uint8_t *codes = st.codes + (size_t)s * n;
    int64_t lo = (int64_t)b * kRowBlock;
    int64_t hi = lo + kRowBlock < n ? lo + kRowBlock : n;
    for (int64_t i = lo + threadIdx.x; i < hi; i += 64) atomicAdd(&cnt[codes[i]], 1u);
    __syncthreads();
    uint32_t *h = st.hist + ((size_t)s * st.nblk + b) * kMaxK;
    for (int j = threadIdx.x; j < kMaxK; j += 64) h[j] = cnt[j];
}

__device__ __forceinline__ uint32_t tree_depth(uint32_t count) {
    uint32_t d = 0;
    while ((uint64_t)count > ((uint64_t)kLeafMax << d)) ++d;
    return d;
}

// One workgroup of 256 threads per column block; thread j owns cluster j.
// Turns the histograms into exclusive prefixes over row blocks, derives cluster offsets,
// tree depths, leaf descriptors, the rank of every empty cluster, and advances the re-seed
// cursor by the number of empty clusters.
static __global__ void __launch_bounds__(256) k_lbg_scan(LbgState st, int k) {
    const int s = blockIdx.x, j = threadIdx.x;
    if (st.done[s]) return;
    __shared__ uint32_t sh_cnt[kMaxK], sh_leaf[kMaxK], sh_empty[kMaxK];
    uint32_t run = 0;
    uint32_t *h = st.hist + (size_t)s * st.nblk * kMaxK + j;
    for (int b = 0; b < st.nblk; ++b) {
        uint32_t v = h[(size_t)b * kMaxK];
        h[(size_t)b * kMaxK] = run;
        run += v;
    }
    const bool live = j < k;
    uint32_t cnt = live ? run : 0;
    uint32_t dep = tree_depth(cnt);
    uint32_t nl = (live && cnt > 0) ? (1u << dep) : 0u;
    uint32_t emp = (live && cnt == 0) ? 1u : 0u;
    sh_cnt[j] = cnt;
    sh_leaf[j] = nl;
    sh_empty[j] = emp;
    __syncthreads();
    // exclusive prefixes over j (k <= 256: a serial walk per thread is cheap and simple)
    uint32_t pc = 0, pl = 0, pe = 0;
    for (int i = 0; i < j; ++i) {
        pc += sh_cnt[i];
        pl += sh_leaf[i];
        pe += sh_empty[i];
    }
    const size_t sj = (size_t)s * kMaxK + j;
    st.count[sj] = cnt;
    st.start[sj] = pc;
    st.leaf_start[sj] = pl;
    st.depth[sj] = dep;
    st.empty_rank[sj] = pe;
    if (j == kMaxK - 1) {
        st.nleaves[s] = (int)(pl + nl);
        int u = st.used[s];
        st.ubase[s] = u;
        st.used[s] = u + (int)(pe + emp);
    }
    // leaf descriptors: leaf l of a depth-d tree is reached by taking bit (d-1-i) of l at level i
    uint2 *desc = st.leaf_desc + (size_t)s * st.leaf_cap + pl;
    for (uint32_t l = 0; l < nl; ++l) {
        uint32_t lo = 0, hi = cnt;
        for (int bit = (int)dep - 1; bit >= 0; --bit) {
            uint32_t mid = lo + (hi - lo) / 2;
            if ((l >> bit) & 1u)
                lo = mid;
            else
                hi = mid;
        }
        desc[l] = make_uint2(pc + lo, pc + hi);
    }
}

// One wave per (row block, column block): stable ranked scatter of row ids into perm[s].
static __global__ void __launch_bounds__(64) k_lbg_scatter(LbgState st, int64_t n) {
    const int s = blockIdx.y, b = blockIdx.x;
    if (st.done[s]) return;
    __shared__ uint32_t base[kMaxK];
    const uint32_t *h = st.hist + ((size_t)s * st.nblk + b) * kMaxK;
    const uint32_t *start = st.start + (size_t)s * kMaxK;
    for (int j = threadIdx.x; j < kMaxK; j += 64) base[j] = start[j] + h[j];
    __syncthreads();
    const uint8_t *codes = st.codes + (size_t)s * n;
    uint32_t *perm = st.perm + (size_t)s * n;
    const int lane = threadIdx.x;
    const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    int64_t lo = (int64_t)b * kRowBlock;
    int64_t hi = lo + kRowBlock < n ? lo + kRowBlock : n;
    for (int64_t i0 = lo; i0 < hi; i0 += 64) {
        int64_t i = i0 + lane;
        bool valid = i < hi;
        uint32_t c = valid ? codes[i] : 0u;
        uint64_t mask = __ballot(valid);
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
        __syncthreads();  // single wave: orders the reads above before the updates below
        if (valid && rank == 0) base[c] += tot;
        __syncthreads();
        if (valid) perm[pos] = (uint32_t)i;
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
    uint32_t p = d.x;
    for (; p + 8 <= d.y; p += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = xc[(int64_t)perm[p + u] * ld];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc = acc + v[u];
    }
    for (; p < d.y; ++p) acc = acc + xc[(int64_t)perm[p] * ld];
    st.leaf_sum[((size_t)s * st.leaf_cap + leaf) * sd + t] = acc;
}

// One lane per (cluster, component): combine leaves left + right, divide by the count
// (src/vector.rs:315-316), or copy the re-seed row for an empty cluster (src/utils.rs:98-101).
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
    uint32_t nl = 1u << st.depth[sj];
    float *ls = st.leaf_sum + ((size_t)s * st.leaf_cap + st.leaf_start[sj]) * sd + t;
    for (uint32_t h = 1; h < nl; h <<= 1)
        for (uint32_t i = 0; i < nl; i += 2 * h) ls[(size_t)i * sd] = ls[(size_t)i * sd] + ls[(size_t)(i + h) * sd];
    float nf = __uint2float_rn(cnt);
    *out = ls[0] / nf;
}

// Loop control of src/utils.rs:57,104-106, one thread per column block.
static __global__ void k_lbg_advance(LbgState st, int m) {
    int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= m || st.done[s]) return;
    st.iters[s] += 1;
    if (!st.changed[s]) st.done[s] = 1;
    st.changed[s] = 0;
}

}  // namespace vq
