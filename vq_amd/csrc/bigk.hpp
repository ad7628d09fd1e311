// Codebooks of more than 256 centroids (16-bit codes).
//
// Assignment: the codebook of every column block is cut into chunks of 256 consecutive centroids.
// Each chunk goes through the 8-bit assignment kernels unchanged, which leave the chunk's own
// winner (the lowest index of the smallest distance inside the chunk, src/utils.rs:62-70); a merge
// kernel then evaluates that winner's distance in the reference's operation order and keeps it
// when it is strictly below the running minimum of the earlier chunks.  Chunks are visited in
// ascending order, so the survivor is the lowest index of the overall minimum, as one loop over
// all k centroids gives.
//
// LBG update (src/utils.rs:76-102): the (column block, code, row) triples are sorted as 64-bit
// keys, which lists every cluster's members in row order; clusters of up to 1024 members are
// summed sequentially from 0.0 (src/vector.rs:306-313), larger ones in parts of 4096 row indices
// (members of a part in row order from 0.0, the part sums in part order from 0.0), empty ones take
// the next entry of the re-seed stream (src/utils.rs:98-101).
//
// This translation unit must be compiled with -ffp-contract=off.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "assign_exact.hpp"

namespace vq {

constexpr int kChunk = 256;          // centroids per chunk: what an 8-bit code can name
constexpr int kBigSeqMax = 1024;     // PARALLEL_THRESHOLD, src/vector.rs:16
constexpr int kBigPartRows = 4096;   // rows per part of the fixed summation order above it

// chunk[s][j][t] = cb[s][base + j][t], j < kc
static __global__ void k_chunk_tables(const float *__restrict__ cb, int m, int k, int sd, int base, int kc,
                                      float *__restrict__ chunk) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t per = (int64_t)kc * sd;
    if (i >= per * m) return;
    const int s = (int)(i / per);
    const int64_t r = i % per;
    chunk[i] = cb[((size_t)s * k + base) * sd + r];
}

// Distance of one row's sub-vector to one centroid in the reference's operation order
// (src/distances.rs:129-152; the squared form of src/vector.rs:214-220 for the LBG).
template <int METRIC>
__device__ __forceinline__ float pair_distance(const float *__restrict__ x, const float *__restrict__ c, int sd) {
    if constexpr (METRIC == M_SQ || METRIC == M_EUCLID) {
        float acc = 0.0f;
        for (int t = 0; t < sd; ++t) {
            const float d = x[t] - c[t];
            const float p = d * d;
            acc = acc + p;
        }
        return METRIC == M_EUCLID ? sqrtf(acc) : acc;
    } else if constexpr (METRIC == M_L1) {
        float acc = 0.0f;
        for (int t = 0; t < sd; ++t) {
            const float d = x[t] - c[t];
            acc = acc + fabsf(d);
        }
        return acc;
    } else {
        float dot = 0.0f, sa = 0.0f, sb = 0.0f;
        for (int t = 0; t < sd; ++t) {
            const float p = x[t] * c[t];
            dot = dot + p;
            const float pa = x[t] * x[t];
            sa = sa + pa;
            const float pb = c[t] * c[t];
            sb = sb + pb;
        }
        const float na = sqrtf(sa), nb = sqrtf(sb);
        const float den = na * nb;
        const float q = dot / den;
        const float d = 1.0f - q;
        return (na == 0.0f || nb == 0.0f) ? 1.0f : d;
    }
}

// One thread per (row, column block): folds the winner of chunk `base / 256` into the running
// minimum.  win8: the chunk's codes, n x m; best_d, out: n x m.
// A chunk whose own first distance is NaN reports local index 0 whatever follows (nothing is
// below NaN), while the loop over all k centroids would carry the earlier chunks' minimum into
// it: such a pair walks the chunk again with the running minimum, one centroid at a time.
// win_d: the winners' distances where the assignment kernel has written them (the same arithmetic),
// else null and the distance is computed here.
template <int METRIC>
__global__ void __launch_bounds__(256) k_chunk_merge(const float *__restrict__ x, int64_t n, int64_t ld, int m,
                                                     int sd, int kc, const float *__restrict__ chunk,
                                                     const uint8_t *__restrict__ win8,
                                                     const float *__restrict__ win_d, int base,
                                                     float *__restrict__ best_d, uint16_t *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n * m) return;
    const int64_t row = i / m;
    const int s = (int)(i % m);
    const float *xr = x + row * ld + (int64_t)s * sd;
    const float *cs = chunk + (size_t)s * kc * sd;
    const int w = win8[i];
    const float d = win_d ? win_d[i] : pair_distance<METRIC>(xr, cs + (size_t)w * sd, sd);
    if (base == 0) {
        best_d[i] = d;
        out[i] = (uint16_t)w;
        return;
    }
    float bd = best_d[i];
    if (d != d) {
        int bi = -1;
        for (int j = 0; j < kc; ++j) {
            const float dj = pair_distance<METRIC>(xr, cs + (size_t)j * sd, sd);
            if (dj < bd) {
                bd = dj;
                bi = j;
            }
        }
        if (bi >= 0) {
            best_d[i] = bd;
            out[i] = (uint16_t)(base + bi);
        }
        return;
    }
    if (d < bd) {
        best_d[i] = d;
        out[i] = (uint16_t)(base + w);
    }
}

// ------------------------------------------------------------------------------ LBG, k > 256
struct BigLbg {
    int *changed, *done, *iters, *used, *ubase, *nbig, *err;  // per column block; err: one int
    uint16_t *codes;        // [m][n] current assignment
    uint32_t *count;        // [m][k]
    uint32_t *start;        // [m][k] first position of the cluster in its block's sorted rows
    uint32_t *empty_rank;   // [m][k] rank among the block's empty clusters
    uint32_t *big_list;     // [m][big_cap] clusters above 1024 members
    int big_cap;
};

static __global__ void k_big_init(BigLbg st, int m) {
    const int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s < m) {
        st.changed[s] = 0;
        st.done[s] = 0;
        st.iters[s] = 0;
        st.used[s] = 0;
        st.ubase[s] = 0;
        st.nbig[s] = 0;
    }
    if (s == 0) st.err[0] = 0;
}

// New codes (n x m, from the merge) into the assignment ([m][n]); src/utils.rs:66-72.  Also the
// sort key of the pair: the row in bits 0-31, the code in the code_bits above them, the column
// block above that.  The keys are written block by block in row order, so a stable sort on the
// bits from 32 up lists every cluster's members in row order.
static __global__ void __launch_bounds__(256) k_big_commit(BigLbg st, const uint16_t *__restrict__ fresh, int64_t n,
                                                           int m, int code_bits, uint64_t *__restrict__ keys) {
    const int s = blockIdx.y;
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= n) return;
    uint16_t *cur = st.codes + (size_t)s * n + row;
    uint16_t c = *cur;
    if (!st.done[s]) {
        const uint16_t f = fresh[row * m + s];
        if (f != c) {
            *cur = f;
            c = f;
            mark_changed(st.changed + s);
        }
    }
    keys[(size_t)s * n + row] = ((uint64_t)s << (32 + code_bits)) | ((uint64_t)c << 32) | (uint64_t)row;
}

// Sorted keys -> first position and size of every cluster that has members.
static __global__ void __launch_bounds__(256) k_big_bounds(BigLbg st, const uint64_t *__restrict__ sorted, int64_t n,
                                                           int m, int k, int code_bits) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n * m) return;
    const uint32_t sc = (uint32_t)(sorted[i] >> 32);  // (block << code_bits) | code
    const int s = (int)(sc >> code_bits), j = (int)(sc & ((1u << code_bits) - 1u));
    const int64_t in_block = i - (int64_t)s * n;
    const bool first = i == 0 || (uint32_t)(sorted[i - 1] >> 32) != sc;
    const bool last = i + 1 == n * m || (uint32_t)(sorted[i + 1] >> 32) != sc;
    const size_t sj = (size_t)s * k + j;
    if (first) st.start[sj] = (uint32_t)in_block;
    // first and last of a cluster may sit in different threads: the size is last + 1 - first,
    // put together from two integer additions (exact in any order)
    if (first) atomicAdd(st.count + sj, (uint32_t)(0u - (uint32_t)in_block));
    if (last) atomicAdd(st.count + sj, (uint32_t)in_block + 1u);
}

// One workgroup per column block: rank of every empty cluster among the empty ones, the list of
// the clusters above 1024 members, the re-seed cursor advanced by the number of empty clusters.
static __global__ void __launch_bounds__(256) k_big_plan(BigLbg st, int k) {
    const int s = blockIdx.x, tid = threadIdx.x;
    if (st.done[s]) return;
    __shared__ uint32_t sh_e[256], sh_b[256];
    const int span = (k + 255) / 256;
    const int j0 = tid * span, j1 = min(j0 + span, k);
    uint32_t ne = 0, nb = 0;
    for (int j = j0; j < j1; ++j) {
        const uint32_t c = st.count[(size_t)s * k + j];
        ne += c == 0;
        nb += c > (uint32_t)kBigSeqMax;
    }
    sh_e[tid] = ne;
    sh_b[tid] = nb;
    __syncthreads();
    uint32_t pe = 0, pb = 0;
    for (int i = 0; i < tid; ++i) {
        pe += sh_e[i];
        pb += sh_b[i];
    }
    for (int j = j0; j < j1; ++j) {
        const uint32_t c = st.count[(size_t)s * k + j];
        if (c == 0) st.empty_rank[(size_t)s * k + j] = pe++;
        if (c > (uint32_t)kBigSeqMax) st.big_list[(size_t)s * st.big_cap + pb++] = (uint32_t)j;
    }
    if (tid == 255) {
        st.nbig[s] = (int)pb;
        const int u = st.used[s];
        st.ubase[s] = u;
        st.used[s] = u + (int)pe;
    }
}

// One thread per (cluster, component): mean of a cluster of up to 1024 members, re-seed row of
// an empty one.
static __global__ void __launch_bounds__(256) k_big_small_means(BigLbg st, const uint64_t *__restrict__ sorted,
                                                                const float *__restrict__ x, int64_t n, int64_t ld,
                                                                int k, int sd, const uint32_t *__restrict__ reseed,
                                                                int n_reseed, float *__restrict__ cb) {
    const int s = blockIdx.y;
    if (st.done[s]) return;
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int j = (int)(gid / sd), t = (int)(gid % sd);
    if (j >= k) return;
    const size_t sj = (size_t)s * k + j;
    const uint32_t cnt = st.count[sj];
    float *out = cb + sj * sd + t;
    const float *col = x + (int64_t)s * sd + t;
    if (cnt == 0) {
        const int pos = st.ubase[s] + (int)st.empty_rank[sj];
        if (pos >= n_reseed) {
            st.err[0] = 1;
            return;
        }
        *out = col[(int64_t)reseed[(size_t)s * n_reseed + pos] * ld];
        return;
    }
    if (cnt > (uint32_t)kBigSeqMax) return;
    const uint64_t *mem = sorted + (size_t)s * n + st.start[sj];
    float sum = 0.0f;
    constexpr int B = 8;  // loads in flight; the additions stay one chain
    for (uint32_t p = 0; p < cnt; p += B) {
        float v[B];
#pragma unroll
        for (int u = 0; u < B; ++u) v[u] = col[(int64_t)(uint32_t)mem[p + u < cnt ? p + u : cnt - 1] * ld];
#pragma unroll
        for (int u = 0; u < B; ++u)
            if (p + u < cnt) sum = sum + v[u];
    }
    *out = sum / __uint2float_rn(cnt);
}

// One workgroup per cluster above 1024 members.  Thread (p, l): part q0 + p of a round, component
// t0 + l; the part sums of a round meet in LDS and thread (0, l) adds them in part order.
// A part without members adds +0.0 to a sum that is never -0.0, which changes nothing.
static __global__ void __launch_bounds__(256) k_big_large_means(BigLbg st, const uint64_t *__restrict__ sorted,
                                                                const float *__restrict__ x, int64_t n, int64_t ld,
                                                                int k, int sd, float *__restrict__ cb) {
    const int s = blockIdx.y;
    if (st.done[s] || (int)blockIdx.x >= st.nbig[s]) return;  // uniform over the workgroup
    const int j = (int)st.big_list[(size_t)s * st.big_cap + blockIdx.x];
    const size_t sj = (size_t)s * k + j;
    const uint32_t cnt = st.count[sj];
    const uint64_t *mem = sorted + (size_t)s * n + st.start[sj];
    const int L = sd < 256 ? sd : 256, P = 256 / L;
    const int p = threadIdx.x / L, l = threadIdx.x % L;
    const int nparts = (int)((n + kBigPartRows - 1) / kBigPartRows);
    __shared__ float sh[256];
    auto lower = [&](uint32_t row) {  // first member position whose row is >= row
        uint32_t lo = 0, hi = cnt;
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if ((uint32_t)mem[mid] < row) lo = mid + 1; else hi = mid;
        }
        return lo;
    };
    for (int t0 = 0; t0 < sd; t0 += L) {
        const int t = t0 + l;
        const bool live = p < P && t < sd;
        const float *col = x + (int64_t)s * sd + (live ? t : 0);
        float acc = 0.0f;
        for (int q0 = 0; q0 < nparts; q0 += P) {
            const int q = q0 + p;
            float part = 0.0f;
            if (live && q < nparts) {
                const uint32_t lo = lower((uint32_t)q * kBigPartRows);
                const uint64_t end_row = (uint64_t)(q + 1) * kBigPartRows;
                const uint32_t hi = end_row >= (uint64_t)n ? cnt : lower((uint32_t)end_row);
                constexpr int B = 8;
                for (uint32_t i = lo; i < hi; i += B) {
                    float v[B];
#pragma unroll
                    for (int u = 0; u < B; ++u) v[u] = col[(int64_t)(uint32_t)mem[i + u < hi ? i + u : hi - 1] * ld];
#pragma unroll
                    for (int u = 0; u < B; ++u)
                        if (i + u < hi) part = part + v[u];
                }
            }
            if (p < P) sh[p * L + l] = part;
            __syncthreads();
            if (p == 0 && t < sd) {
                const int np = nparts - q0 < P ? nparts - q0 : P;
                for (int pp = 0; pp < np; ++pp) acc = acc + sh[pp * L + l];
            }
            __syncthreads();
        }
        if (p == 0 && t < sd) cb[sj * sd + t] = acc / __uint2float_rn(cnt);
    }
}

// Loop control of src/utils.rs:57,104-106.
static __global__ void k_big_advance(BigLbg st, int m) {
    const int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= m || st.done[s]) return;
    st.iters[s] += 1;
    if (!st.changed[s]) st.done[s] = 1;
    st.changed[s] = 0;
}

// 8-bit codes widened (k <= 256 through the 16-bit entry points).
static __global__ void k_widen_codes(const uint8_t *__restrict__ in, int64_t count, uint16_t *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) out[i] = in[i];
}

}  // namespace vq
