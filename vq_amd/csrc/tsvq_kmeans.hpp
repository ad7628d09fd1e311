// TSVQ built with 2-means splits: lbg_quantize (src/utils.rs:32-109) with k = 2 on the rows of every
// node of a tree level at once.  NOT the reference's split (src/tsvq.rs:87-123 takes the median of
// the maximum-variance coordinate); an explicit, non-default mode.
//
// A level's splitting nodes are segments [lo, hi) of `perm`, the list of row ids that keeps the rows
// of a node contiguous and in original row order.  Position p - lo inside a segment is the row's
// number in the node's own data array, which is what the LBG's rules refer to:
//   initial centroids  rows number i0 = d[0] % c and i1 = d[1] % (c - 1), plus one if i1 >= i0, where
//                      d are the node's draws and c its row count (utils.rs:54: k distinct rows)
//   assignment         squared L2, sequential f32 sums, strict '<' (utils.rs:59-73)
//   update             mean of the members in row order (src/vector.rs:306-313) for clusters of at most
//                      1024 members; above, the node's array is cut into parts of 4096 rows, a part's
//                      members are added in row order from 0.0 and the part sums in part order from 0.0
//                      (the order this library fixes for mean_vector's unordered reduce)
//   empty cluster      the i-th one met takes row number d[2 + i] % c (utils.rs:98-101)
//   early stop         when no assignment changed, after the update (utils.rs:104-106)
// A row goes left when the first of the two final centroids is its nearest.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tsvq.hpp"

namespace vq {

constexpr int kKmPart = 4096;     // rows per part of a node's array
constexpr int kKmSeqMax = 1024;   // PARALLEL_THRESHOLD, src/vector.rs:16

struct KmState {
    const uint32_t *perm;    // row ids, node-contiguous
    const uint2 *range;      // [ns] segment [lo, hi) of every splitting node
    const uint32_t *draws;   // [ns][per_node]
    int per_node;
    int ns;
    float *cen;              // [ns][2][dim]
    uint8_t *codes;          // [n] assignment per position
    uint32_t *part_first;    // [ns + 1] first part of every segment (parts numbered over the level)
    float *part_sum;         // [parts][2][dim]
    uint32_t *part_cnt;      // [parts][2]
    int *changed, *done, *used, *iters, *err;  // [ns] each (err: one flag)
};

// squared distance in the reference's order: d = x - c, p = d * d, acc = acc + p (src/vector.rs:214-220)
__device__ __forceinline__ float km_d2(const float *__restrict__ xr, const float *__restrict__ c, int dim) {
    float acc = 0.0f;
    if ((dim & 3) == 0 && ((reinterpret_cast<uintptr_t>(xr) | reinterpret_cast<uintptr_t>(c)) & 15) == 0) {
        for (int t = 0; t < dim; t += 4) {
            const float4 a = *reinterpret_cast<const float4 *>(xr + t), b = *reinterpret_cast<const float4 *>(c + t);
            float d0 = a.x - b.x, d1 = a.y - b.y, d2 = a.z - b.z, d3 = a.w - b.w;
            float p0 = d0 * d0, p1 = d1 * d1, p2 = d2 * d2, p3 = d3 * d3;
            acc = acc + p0;
            acc = acc + p1;
            acc = acc + p2;
            acc = acc + p3;
        }
    } else {
        for (int t = 0; t < dim; ++t) {
            float d = xr[t] - c[t];
            float p = d * d;
            acc = acc + p;
        }
    }
    return acc;
}

// One workgroup per splitting node: the two initial centroids, zeroed state.
static __global__ void __launch_bounds__(256) k_km_init(KmState st, const float *__restrict__ x, int64_t ld, int dim) {
    const int g = blockIdx.x;
    const uint2 r = st.range[g];
    const uint32_t c = r.y - r.x;
    const uint32_t *d = st.draws + (size_t)g * st.per_node;
    uint32_t i0 = d[0] % c, i1 = d[1] % (c - 1);  // c >= 2: a node of one row does not split
    if (i1 >= i0) i1 += 1;
    const float *x0 = x + (int64_t)st.perm[r.x + i0] * ld, *x1 = x + (int64_t)st.perm[r.x + i1] * ld;
    for (int t = threadIdx.x; t < dim; t += 256) {
        st.cen[((size_t)g * 2 + 0) * dim + t] = x0[t];
        st.cen[((size_t)g * 2 + 1) * dim + t] = x1[t];
    }
    if (threadIdx.x == 0) {
        st.changed[g] = 0;
        st.done[g] = 0;
        st.used[g] = 0;
        st.iters[g] = 0;
    }
}

// One thread per position: the nearer of its node's two centroids.  LBG: nodes that have stopped are
// skipped and a changed assignment raises the node's flag; otherwise every splitting node's rows are
// assigned and flags[p] = 1 for the rows that go left (0 outside the splitting nodes).
template <bool LBG>
static __global__ void __launch_bounds__(256) k_km_assign(KmState st, int64_t n, const float *__restrict__ x,
                                                          int64_t ld, int dim, uint32_t *__restrict__ flags) {
    const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= n) return;
    const int g = find_segment(st.range, st.ns, (uint32_t)p);
    if (g < 0) {
        if (!LBG) flags[p] = 0u;
        return;
    }
    if (LBG && st.done[g]) return;
    const float *xr = x + (int64_t)st.perm[p] * ld;
    const float *c0 = st.cen + (size_t)g * 2 * dim;
    const float d0 = km_d2(xr, c0, dim), d1 = km_d2(xr, c0 + dim, dim);
    const uint8_t code = d1 < d0 ? 1 : 0;  // strict '<': ties and NaN stay with the first
    if (LBG) {
        if (st.codes[p] != code) {
            st.codes[p] = code;
            if (st.changed[g] == 0) st.changed[g] = 1;
        }
    } else {
        flags[p] = code == 0 ? 1u : 0u;
    }
}

// The same with the row in registers (DIM a multiple of 4 up to 128, 16-byte aligned rows): a lane
// fetches its row once, all loads in flight together, and the two centroids come from LDS when the
// workgroup's 256 positions lie in one node (the usual case: every lane reads the same address).
template <bool LBG, int DIM>
static __global__ void __launch_bounds__(256) k_km_assign_reg(KmState st, int64_t n, const float *__restrict__ x,
                                                              int64_t ld, uint32_t *__restrict__ flags) {
    __shared__ __attribute__((aligned(16))) float lds_c[2 * DIM];
    const int64_t p0 = (int64_t)blockIdx.x * 256, p = p0 + threadIdx.x;
    const int64_t plast = p0 + 255 < n ? p0 + 255 : n - 1;
    const int gfirst = find_segment(st.range, st.ns, (uint32_t)p0), glast = find_segment(st.range, st.ns, (uint32_t)plast);
    const bool one = gfirst >= 0 && gfirst == glast;  // the same in the whole workgroup
    if (one) {
        if (LBG && st.done[gfirst]) return;
        for (int t = threadIdx.x; t < 2 * DIM; t += 256) lds_c[t] = st.cen[(size_t)gfirst * 2 * DIM + t];
        __syncthreads();
    }
    if (p >= n) return;
    const int g = one ? gfirst : find_segment(st.range, st.ns, (uint32_t)p);
    if (g < 0) {
        if (!LBG) flags[p] = 0u;
        return;
    }
    if (LBG && st.done[g]) return;
    float xr[DIM];
    {
        const float4 *xp = reinterpret_cast<const float4 *>(x + (int64_t)st.perm[p] * ld);
#pragma unroll
        for (int q = 0; q < DIM / 4; ++q) {
            const float4 v = xp[q];
            xr[4 * q] = v.x;
            xr[4 * q + 1] = v.y;
            xr[4 * q + 2] = v.z;
            xr[4 * q + 3] = v.w;
        }
    }
    float d0 = 0.0f, d1 = 0.0f;
    if (one) {
#pragma unroll
        for (int q = 0; q < DIM / 4; ++q) {
            const float4 a = *reinterpret_cast<const float4 *>(lds_c + 4 * q);
            const float4 b = *reinterpret_cast<const float4 *>(lds_c + DIM + 4 * q);
            const float ca[4] = {a.x, a.y, a.z, a.w}, cb[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const float e0 = xr[4 * q + u] - ca[u], e1 = xr[4 * q + u] - cb[u];
                const float s0 = e0 * e0, s1 = e1 * e1;
                d0 = d0 + s0;
                d1 = d1 + s1;
            }
        }
    } else {
        const float *c0 = st.cen + (size_t)g * 2 * DIM;
        for (int t = 0; t < DIM; ++t) {
            const float e0 = xr[t] - c0[t], e1 = xr[t] - c0[DIM + t];
            const float s0 = e0 * e0, s1 = e1 * e1;
            d0 = d0 + s0;
            d1 = d1 + s1;
        }
    }
    const uint8_t code = d1 < d0 ? 1 : 0;
    if (LBG) {
        if (st.codes[p] != code) {
            st.codes[p] = code;
            if (st.changed[g] == 0) st.changed[g] = 1;
        }
    } else {
        flags[p] = code == 0 ? 1u : 0u;
    }
}

// Assignment and part sums of one LBG iteration in one pass over the rows (DIM a multiple of 32 up to
// 128, 16-byte aligned rows).  One workgroup of 512 threads per part, which walks the part in tiles of
// 128 positions through two LDS buffers.  Waves 0-3 bring a tile in with coalesced loads (a row is read
// by DIM / 4 neighbouring lanes; the next tile's loads in flight meanwhile), lay it out in LDS with a row stride of
// DIM + 4 floats (which both access patterns below read without bank conflicts) and find the code of
// every row against the node's two centroids, in the operation order of k_km_assign_reg.  Waves
// 4-7 work one tile behind: thread (component c, cluster j) adds the tile's rows of its cluster to its
// sum in row order.  A row of the other cluster is added as +0.0 (its bits under an all-zero mask): the
// sum starts at +0.0 and a sum of floats is -0.0 only if every term is, so that addition changes
// nothing, and the sums are the part sums of k_km_partsum, bit for bit.
// Dynamic LDS: km_assign_sum_lds(DIM) bytes.
constexpr int kKmTile = 128;
constexpr size_t km_assign_sum_lds(int dim) { return (size_t)2 * kKmTile * (dim + 4) * sizeof(float); }

template <int DIM>
static __global__ void __launch_bounds__(512) k_km_assign_sum(KmState st, const float *__restrict__ x, int64_t ld) {
    constexpr int TR = kKmTile;
    constexpr int STRIDE = DIM + 4;
    constexpr int D4 = DIM / 4;             // float4 per row
    constexpr int RPS = 256 / D4;           // rows per sweep of the 256 loading threads (the first RPS * D4 of them load)
    constexpr int K = (TR + RPS - 1) / RPS; // sweeps per tile
    static_assert(DIM % 32 == 0 && DIM <= 128, "row shape");
    extern __shared__ __attribute__((aligned(16))) float tile[];  // [2][TR][STRIDE]
    __shared__ __attribute__((aligned(16))) float lds_c[2 * DIM];
    __shared__ __attribute__((aligned(16))) uint32_t lds_sel[2][2][TR];  // [buffer][cluster][row]: all ones where the row is the cluster's
    __shared__ uint32_t lds_cnt[2];
    __shared__ uint32_t lds_perm[kKmPart];  // the part's row ids
    __shared__ uint8_t lds_old[kKmPart];    // and the codes they come with
    const uint32_t part = blockIdx.x;
    int lo = 0, hi = st.ns - 1;
    while (lo < hi) {  // the segment this part belongs to: part_first is ascending
        const int mid = (lo + hi + 1) >> 1;
        if (st.part_first[mid] <= part)
            lo = mid;
        else
            hi = mid - 1;
    }
    const int g = lo;
    if (st.done[g]) return;  // the same in the whole workgroup
    // (the same in every lane: told to the compiler, so that the loops below are scalar loops)
    const uint32_t rx = __builtin_amdgcn_readfirstlane(st.range[g].x), ry = __builtin_amdgcn_readfirstlane(st.range[g].y);
    const uint32_t pf = __builtin_amdgcn_readfirstlane(st.part_first[g]);
    const uint32_t p0 = rx + (part - pf) * (uint32_t)kKmPart;
    const uint32_t p1 = p0 + kKmPart < ry ? p0 + kKmPart : ry;
    const uint32_t np = p1 - p0;  // positions in this part
    const int ntiles = (int)((np + TR - 1) / TR);
    const int tid = threadIdx.x, lt = tid & 255;
    const bool producer = tid < 256;
    const int lrow = lt / D4, lcol = lt % D4;  // a loading thread's place in a sweep
    const bool loader = producer && lt < RPS * D4;
    for (uint32_t q = tid; q < np; q += 512) {
        lds_perm[q] = st.perm[p0 + q];
        lds_old[q] = st.codes[p0 + q];
    }
    for (int t = tid; t < 2 * DIM; t += 512) lds_c[t] = st.cen[(size_t)g * 2 * DIM + t];
    if (tid < 2) lds_cnt[tid] = 0u;
    __syncthreads();
    // The loads of a tile are unconditional (a row past the tile's end reads the tile's last row instead,
    // and its value never reaches a sum): loads under a branch would make every wait a wait for all of them.
    // (The loaded values are assigned component by component: as a copy of the 16-byte struct from global
    // memory the staging array stays in scratch memory.)
    float4 stage[K];
    auto fetch = [&](int t, float4(&stg)[K]) {
        const uint32_t base = (uint32_t)t * TR;
        const uint32_t rows = np - base < (uint32_t)TR ? np - base : (uint32_t)TR;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint32_t row = (uint32_t)(k * RPS + lrow);
            const float4 v = reinterpret_cast<const float4 *>(x + (int64_t)lds_perm[base + (row < rows ? row : rows - 1u)] * ld)[lcol];
            stg[k] = make_float4(v.x, v.y, v.z, v.w);
        }
    };
    if (producer) fetch(0, stage);
    const int c = lt % DIM, j = lt / DIM;  // a summing thread's chain (lt < 2 * DIM)
    const bool summer = !producer && lt < 2 * DIM;
    float acc = 0.0f;
    uint32_t n0 = 0, n1 = 0;
    bool any_changed = false;
    // rows [64 * half, 64 * half + 64) of the tile in buffer b into the chains
    auto sum_half = [&](int b, int half) {
        const float *tb = tile + (size_t)b * TR * STRIDE + (size_t)(64 * half) * STRIDE + c;
        const uint4 *sel = reinterpret_cast<const uint4 *>(&lds_sel[b][j][64 * half]);
#pragma unroll 4
        for (int r4 = 0; r4 < 16; ++r4) {
            const uint4 m = sel[r4];
            const float v0 = tb[(4 * r4 + 0) * STRIDE], v1 = tb[(4 * r4 + 1) * STRIDE];
            const float v2 = tb[(4 * r4 + 2) * STRIDE], v3 = tb[(4 * r4 + 3) * STRIDE];
            acc = acc + __uint_as_float(__float_as_uint(v0) & m.x);
            acc = acc + __uint_as_float(__float_as_uint(v1) & m.y);
            acc = acc + __uint_as_float(__float_as_uint(v2) & m.z);
            acc = acc + __uint_as_float(__float_as_uint(v3) & m.w);
        }
    };
    auto step = [&](int i, float4(&stg)[K]) {
        const int b = i & 1;
        // first half: tile i into LDS, tile i + 1 on its way | rows 0..63 of tile i - 1 into the sums
        if (producer) {
            if (i < ntiles) {
                float *tb = tile + (size_t)b * TR * STRIDE;
#pragma unroll
                for (int k = 0; k < K; ++k)
                    if (loader && k * RPS + lrow < TR)
                        *reinterpret_cast<float4 *>(tb + (k * RPS + lrow) * STRIDE + 4 * lcol) = stg[k];
                fetch(i + 1 < ntiles ? i + 1 : i, stg);  // (unconditional: the last tile is asked for twice)
            }
        } else if (summer && i >= 1) {
            sum_half(b ^ 1, 0);
        }
        lds_only_barrier();  // (not __syncthreads: the loads of the next tile stay in flight)
        // second half: codes of tile i | rows 64..127 of tile i - 1
        if (producer) {
            if (i < ntiles) {
                // lanes l and l + 32 of a wave take one row: the distance to the first centroid in the
                // lower lane, to the second in the upper one (each a chain of its own, as in the reference)
                const int prow = ((lt >> 6) << 5) | (lt & 31), which = (lt >> 5) & 1;
                const uint32_t q = (uint32_t)i * TR + prow;
                const float *xr = tile + (size_t)b * TR * STRIDE + prow * STRIDE;
                const float *cp = lds_c + which * DIM;
                float d = 0.0f;
#pragma unroll 8
                for (int qq = 0; qq < D4; ++qq) {
                    const float4 v = *reinterpret_cast<const float4 *>(xr + 4 * qq);
                    const float4 a = *reinterpret_cast<const float4 *>(cp + 4 * qq);
                    const float xv[4] = {v.x, v.y, v.z, v.w}, ca[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const float e = xv[u] - ca[u];
                        const float sq = e * e;
                        d = d + sq;
                    }
                }
                const float other = __shfl_xor(d, 32);
                if (which == 0) {
                    uint32_t is0 = 0u, is1 = 0u;  // neither cluster: a position past the part's end
                    if (q < np) {
                        const uint8_t code = other < d ? 1 : 0;  // strict '<': ties and NaN stay with the first
                        if (lds_old[q] != code) {
                            st.codes[p0 + q] = code;
                            any_changed = true;
                        }
                        is1 = code ? 0xffffffffu : 0u;
                        is0 = ~is1;
                        n1 += code;
                        n0 += 1u - code;
                    }
                    lds_sel[b][0][prow] = is0;
                    lds_sel[b][1][prow] = is1;
                }
            }
        } else if (summer && i >= 1) {
            sum_half(b ^ 1, 1);
        }
        lds_only_barrier();
    };
    for (int i = 0; i <= ntiles; ++i) step(i, stage);
    if (any_changed && st.changed[g] == 0) st.changed[g] = 1;
    if (n0) atomicAdd(&lds_cnt[0], n0);
    if (n1) atomicAdd(&lds_cnt[1], n1);
    __syncthreads();
    if (summer) st.part_sum[((size_t)part * 2 + j) * DIM + c] = acc;
    if (tid < 2) st.part_cnt[(size_t)part * 2 + tid] = lds_cnt[tid];
}

// One workgroup per part (4096 consecutive rows of a node's array): thread t owns components t, t +
// blockDim, ... and adds the part's rows to the sum of their cluster in row order, from 0.0; thread 0
// counts.  blockDim: 64, 128 or 256 (the smallest that covers dim, so that short rows leave no idle waves).
static __global__ void __launch_bounds__(256) k_km_partsum(KmState st, const float *__restrict__ x, int64_t ld,
                                                           int dim) {
    const uint32_t part = blockIdx.x;
    // the segment this part belongs to: part_first is ascending
    int lo = 0, hi = st.ns - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (st.part_first[mid] <= part)
            lo = mid;
        else
            hi = mid - 1;
    }
    const int g = lo;
    if (st.done[g]) return;
    const uint2 r = st.range[g];
    const uint32_t p0 = r.x + (part - st.part_first[g]) * (uint32_t)kKmPart;
    const uint32_t p1 = p0 + kKmPart < r.y ? p0 + kKmPart : r.y;
    uint32_t n0 = 0, n1 = 0;
    const int nthr = (int)blockDim.x;
    for (int t0 = 0; t0 < dim; t0 += nthr) {
        const int t = t0 + threadIdx.x;
        const bool on = t < dim;
        const float *xc = x + (on ? t : 0);
        float a0 = 0.0f, a1 = 0.0f;
        // Batches of 16 rows: the row ids and codes of batch b + 2 and the rows of batch b + 1 are in
        // flight while batch b is added (loads unconditional, clamped to the part's last row); the
        // adds keep their order.
        constexpr int B = 16;
        const uint32_t last = p1 - 1;
        uint32_t idn[B], idf[B];
        uint8_t cdn[B], cdf[B], cdc[B];
        float vn[B];
#pragma unroll
        for (int u = 0; u < B; ++u) {
            const uint32_t q = p0 + u <= last ? p0 + u : last;
            idn[u] = st.perm[q];
            cdn[u] = st.codes[q];
        }
#pragma unroll
        for (int u = 0; u < B; ++u) {
            const uint32_t q = p0 + B + u <= last ? p0 + B + u : last;
            idf[u] = st.perm[q];
            cdf[u] = st.codes[q];
        }
#pragma unroll
        for (int u = 0; u < B; ++u) vn[u] = xc[(int64_t)idn[u] * ld];
        for (uint32_t p = p0; p < p1; p += B) {
            float v[B];
#pragma unroll
            for (int u = 0; u < B; ++u) {
                v[u] = vn[u];
                cdc[u] = cdn[u];
            }
#pragma unroll
            for (int u = 0; u < B; ++u) {
                idn[u] = idf[u];
                cdn[u] = cdf[u];
                vn[u] = xc[(int64_t)idn[u] * ld];
            }
#pragma unroll
            for (int u = 0; u < B; ++u) {
                const uint32_t q = p + 2 * B + u <= last ? p + 2 * B + u : last;
                idf[u] = st.perm[q];
                cdf[u] = st.codes[q];
            }
#pragma unroll
            for (int u = 0; u < B; ++u)
                if (p + u < p1) {
                    if (cdc[u]) {
                        a1 = a1 + v[u];
                        n1 += t0 == 0;
                    } else {
                        a0 = a0 + v[u];
                        n0 += t0 == 0;
                    }
                }
        }
        if (on) {
            st.part_sum[((size_t)part * 2 + 0) * dim + t] = a0;
            st.part_sum[((size_t)part * 2 + 1) * dim + t] = a1;
        }
    }
    if (threadIdx.x == 0) {
        st.part_cnt[(size_t)part * 2 + 0] = n0;
        st.part_cnt[(size_t)part * 2 + 1] = n1;
    }
}

// One workgroup per splitting node: the new centroids (utils.rs:95-102) and the loop control (104-106).
static __global__ void __launch_bounds__(256) k_km_update(KmState st, const float *__restrict__ x, int64_t ld,
                                                          int dim) {
    const int g = blockIdx.x;
    if (st.done[g]) return;  // the same in the whole workgroup: written only at the end, behind a barrier
    const uint2 r = st.range[g];
    const uint32_t c = r.y - r.x;
    const uint32_t f = st.part_first[g], nparts = st.part_first[g + 1] - f;
    __shared__ uint32_t cnt[2];
    __shared__ uint32_t list[kKmSeqMax];
    __shared__ uint32_t nlist;
    if (threadIdx.x < 2) {
        uint32_t s = 0;
        for (uint32_t q = 0; q < nparts; ++q) s += st.part_cnt[(size_t)(f + q) * 2 + threadIdx.x];
        cnt[threadIdx.x] = s;
    }
    __syncthreads();
    int used = st.used[g];
    for (int j = 0; j < 2; ++j) {
        const uint32_t m = cnt[j];
        float *out = st.cen + ((size_t)g * 2 + j) * dim;
        if (m == 0) {
            // the next draw of the node's stream (the same in every thread)
            if (2 + used >= st.per_node) {
                if (threadIdx.x == 0) st.err[0] = 1;
            } else {
                const uint32_t row = st.perm[r.x + st.draws[(size_t)g * st.per_node + 2 + used] % c];
                for (int t = threadIdx.x; t < dim; t += 256) out[t] = x[(int64_t)row * ld + t];
            }
            ++used;
        } else if (m <= (uint32_t)kKmSeqMax && nparts > 1) {
            // a small cluster in a node of several parts: its members, in row order, as ONE chain
            // (their part sums would associate differently).  The workgroup lists them part by part.
            __syncthreads();
            if (threadIdx.x == 0) nlist = 0;
            __syncthreads();
            for (uint32_t q = 0; q < nparts; ++q) {
                if (st.part_cnt[(size_t)(f + q) * 2 + j] == 0) continue;  // uniform
                const uint32_t p0 = r.x + q * (uint32_t)kKmPart, p1 = p0 + kKmPart < r.y ? p0 + kKmPart : r.y;
                for (uint32_t base = p0; base < p1; base += 256) {
                    const uint32_t p = base + threadIdx.x;
                    const bool mine = p < p1 && st.codes[p] == (uint8_t)j;
                    // stable compaction of the 256 positions: ballots per wave, wave totals through LDS
                    const unsigned long long bal = __ballot(mine);
                    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
                    __shared__ uint32_t wtot[4];
                    if (lane == 0) wtot[w] = (uint32_t)__popcll(bal);
                    __syncthreads();
                    uint32_t before = nlist;
                    for (int u = 0; u < w; ++u) before += wtot[u];
                    if (mine) list[before + (uint32_t)__popcll(bal & ((1ull << lane) - 1ull))] = st.perm[p];
                    __syncthreads();
                    if (threadIdx.x == 0) nlist += wtot[0] + wtot[1] + wtot[2] + wtot[3];
                    __syncthreads();
                }
            }
            const float dv = __uint2float_rn(m);
            for (int t = threadIdx.x; t < dim; t += 256) {
                float acc = 0.0f;
                for (uint32_t i = 0; i < m; ++i) acc = acc + x[(int64_t)list[i] * ld + t];
                out[t] = acc / dv;
            }
        } else {
            // part sums in part order from 0.0 (one part: 0.0 + sum is the sum itself)
            const float dv = __uint2float_rn(m);
            for (int t = threadIdx.x; t < dim; t += 256) {
                float acc = 0.0f;
                const float *ps = st.part_sum + ((size_t)f * 2 + j) * dim + t;
                const size_t pstride = (size_t)2 * dim;
                uint32_t q = 0;
                for (; q + 8 <= nparts; q += 8) {  // eight loads in flight, added in part order
                    float v[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) v[u] = ps[(size_t)(q + u) * pstride];
#pragma unroll
                    for (int u = 0; u < 8; ++u) acc = acc + v[u];
                }
                for (; q < nparts; ++q) acc = acc + ps[(size_t)q * pstride];
                out[t] = (m <= (uint32_t)kKmSeqMax) ? st.part_sum[((size_t)f * 2 + j) * dim + t] / dv : acc / dv;
            }
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        st.used[g] = used;
        st.iters[g] += 1;
        if (!st.changed[g]) st.done[g] = 1;
        st.changed[g] = 0;
    }
}

}  // namespace vq
