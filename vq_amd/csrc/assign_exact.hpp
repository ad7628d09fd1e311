// Exact nearest-centroid assignment on the vector ALU.
//
// Every distance is evaluated in the reference's own operation order (sequential f32
// accumulation from 0.0, separately rounded multiply and add, strict '<' so the lowest index
// wins: src/utils.rs:62-70, src/vector.rs:197-201,259-264, src/distances.rs:129-152), so the
// codes are bit-identical to the CPU path by construction.  This translation unit must be
// compiled with -ffp-contract=off.
//
// Mapping: one lane = one row.  The lane keeps its sub-vectors in registers; the centroid
// operand is identical for all lanes of a wave and is read from LDS as a broadcast.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vq {

enum { M_SQ = 0, M_EUCLID = 1, M_COS = 2, M_L1 = 3 };

struct AssignArgs {
    const float *x;       // n x ld
    int64_t n;
    int64_t ld;
    int m;                // column blocks
    int k;                // centroids per block
    const float *cb;      // m*k*sd
    const float *cnorm;   // m*k centroid L2 norms (cosine only)
    uint8_t *codes;       // LBG mode: [m][n] in place (old -> new); encode mode: [n][m]
    int *changed;         // LBG mode: changed[s] set to 1 when any code of block s differs
    const int *done;      // LBG mode: blocks with done[s] != 0 are skipped
    float *dist = nullptr;  // encode mode, k_assign_mfma_bf only: [n][m] distance of the chosen centroid, or null
    // A residual update that the pass applies before it scores the rows (single wide column block,
    // k_assign_mfma_wide_bf only): x[i] = src[i] - pend_cb[pend_codes[i]], where src is the rows
    // themselves (an update in place) or, pend_src != null, other rows of stride pend_src_ld that
    // stay as they are.  pend_cb null: the rows are read as they are.
    const float *pend_cb = nullptr;
    const uint8_t *pend_codes = nullptr;
    const float *pend_src = nullptr;
    int64_t pend_src_ld = 0;
};

// Called by the lanes of a wave that changed a code.  Every store to one address is serialised
// in its L2 channel and a million rows may change in a pass, so one lane of the wave stores, and
// only when it still reads 0 (a stale 0 from the vector cache costs a store, nothing else).
__device__ __forceinline__ void mark_changed(int *flag) {
    const unsigned long long active = __ballot(1);
    if ((int)__lane_id() == __ffsll(active) - 1 && *flag == 0) *flag = 1;
}

// sqrt(sum of squares) of every centroid, sequential order (map_sum, src/distances.rs:66-69,144)
static __global__ void k_centroid_norms(const float *__restrict__ cb, int64_t total, int sd,
                                 float *__restrict__ out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const float *c = cb + i * sd;
    float acc = 0.0f;
    for (int t = 0; t < sd; ++t) {
        float p = c[t] * c[t];
        acc = acc + p;
    }
    out[i] = sqrtf(acc);
}

template <int SD>
__device__ __forceinline__ float d_sq(const float (&x)[SD], const float (&c)[SD]) {
    float d0 = x[0] - c[0];
    float acc = d0 * d0;  // 0.0 + p == p for p >= +0
#pragma unroll
    for (int t = 1; t < SD; ++t) {
        float d = x[t] - c[t];
        float p = d * d;
        acc = acc + p;
    }
    return acc;
}

template <int SD>
__device__ __forceinline__ float d_l1(const float (&x)[SD], const float (&c)[SD]) {
    float acc = fabsf(x[0] - c[0]);
#pragma unroll
    for (int t = 1; t < SD; ++t) {
        float d = x[t] - c[t];
        acc = acc + fabsf(d);
    }
    return acc;
}

template <int SD>
__device__ __forceinline__ float d_dot(const float (&x)[SD], const float (&c)[SD]) {
    float acc = 0.0f;
#pragma unroll
    for (int t = 0; t < SD; ++t) {
        float p = x[t] * c[t];
        acc = acc + p;
    }
    return acc;
}

template <int SD>
__device__ __forceinline__ void lds_centroid(const float *lds, int j, float (&c)[SD]) {
    if constexpr (SD % 4 == 0) {
        const float4 *p = reinterpret_cast<const float4 *>(lds + j * SD);
#pragma unroll
        for (int q = 0; q < SD / 4; ++q) {
            float4 v = p[q];
            c[4 * q + 0] = v.x;
            c[4 * q + 1] = v.y;
            c[4 * q + 2] = v.z;
            c[4 * q + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int t = 0; t < SD; ++t) c[t] = lds[j * SD + t];
    }
}

// Argmin of one row's sub-vector against the k centroids held in LDS.
template <int SD, int METRIC>
__device__ __forceinline__ int argmin_lds(const float (&x)[SD], const float *lds, const float *cn,
                                          int k) {
    float c[SD];
    int best = 0;
    if constexpr (METRIC == M_SQ || METRIC == M_EUCLID) {
        lds_centroid<SD>(lds, 0, c);
        float bd = d_sq<SD>(x, c);
        float pd = __builtin_inff();  // squared distance of the previous running minimum
#pragma unroll 4
        for (int j = 1; j < k; ++j) {
            lds_centroid<SD>(lds, j, c);
            float d = d_sq<SD>(x, c);
            bool u = d < bd;
            if constexpr (METRIC == M_EUCLID) pd = u ? bd : pd;
            bd = u ? d : bd;
            best = u ? j : best;
        }
        if constexpr (METRIC == M_EUCLID) {
            // The reference compares sqrt(d2) (src/distances.rs:134-140).  sqrt is monotone, so
            // its running minimum is the first element of the strictly decreasing chain of d2
            // minima whose root equals the root of the smallest d2.  Only when the previous
            // chain element shares that root can the answer be an earlier index: rescan.
            float s = sqrtf(bd);
            if (sqrtf(pd) == s) {
                for (int j = 0; j < best; ++j) {
                    lds_centroid<SD>(lds, j, c);
                    if (sqrtf(d_sq<SD>(x, c)) == s) {
                        best = j;
                        break;
                    }
                }
            }
        }
    } else if constexpr (METRIC == M_L1) {
        lds_centroid<SD>(lds, 0, c);
        float bd = d_l1<SD>(x, c);
#pragma unroll 4
        for (int j = 1; j < k; ++j) {
            lds_centroid<SD>(lds, j, c);
            float d = d_l1<SD>(x, c);
            bool u = d < bd;
            bd = u ? d : bd;
            best = u ? j : best;
        }
    } else {  // cosine, src/distances.rs:141-151
        float sa = 0.0f;
#pragma unroll
        for (int t = 0; t < SD; ++t) {
            float p = x[t] * x[t];
            sa = sa + p;
        }
        float na = sqrtf(sa);
        float bd = 0.0f;
        for (int j = 0; j < k; ++j) {
            lds_centroid<SD>(lds, j, c);
            float dot = d_dot<SD>(x, c);
            float nb = cn[j];
            float den = na * nb;
            float q = dot / den;
            float d = 1.0f - q;
            d = (na == 0.0f || nb == 0.0f) ? 1.0f : d;
            bool u = (j == 0) || (d < bd);
            bd = u ? d : bd;
            best = u ? j : best;
        }
    }
    return best;
}

// One lane = one row, G consecutive column blocks per lane (G*SD floats in registers, G
// codebooks in LDS).  blockIdx.x = tile * (m/G) + block group.
template <int SD, int G, int METRIC, bool LBG>
__global__ void __launch_bounds__(256) k_assign_static(AssignArgs a) {
    extern __shared__ float lds[];
    const int groups = a.m / G;
    const int sg = blockIdx.x % groups;
    const int64_t tile = blockIdx.x / groups;
    const int s0 = sg * G;
    const int k = a.k;
    float *lds_cn = lds + (size_t)G * k * SD;

    bool any = true;
    if constexpr (LBG) {
        any = false;
#pragma unroll
        for (int g = 0; g < G; ++g) any |= (a.done[s0 + g] == 0);
        if (!any) return;  // uniform over the workgroup
    }
    // codebooks of blocks s0..s0+G-1 are contiguous: G*k*SD floats
    {
        const float *src = a.cb + (size_t)s0 * k * SD;
        const int total = G * k * SD;
        for (int i = threadIdx.x; i < total; i += 256) lds[i] = src[i];
        if constexpr (METRIC == M_COS) {
            const float *cn = a.cnorm + (size_t)s0 * k;
            for (int i = threadIdx.x; i < G * k; i += 256) lds_cn[i] = cn[i];
        }
    }
    __syncthreads();

    const int64_t row = tile * 256 + threadIdx.x;
    if (row >= a.n) return;

    float x[G][SD];
    {
        const float *xr = a.x + row * a.ld + (int64_t)s0 * SD;
        if constexpr ((G * SD) % 4 == 0) {
            if ((a.ld % 4 == 0) && ((reinterpret_cast<uintptr_t>(a.x) & 15) == 0)) {
                const float4 *p = reinterpret_cast<const float4 *>(xr);
                float *xf = &x[0][0];
#pragma unroll
                for (int q = 0; q < G * SD / 4; ++q) {
                    float4 v = p[q];
                    xf[4 * q + 0] = v.x;
                    xf[4 * q + 1] = v.y;
                    xf[4 * q + 2] = v.z;
                    xf[4 * q + 3] = v.w;
                }
            } else {
#pragma unroll
                for (int g = 0; g < G; ++g)
#pragma unroll
                    for (int t = 0; t < SD; ++t) x[g][t] = xr[g * SD + t];
            }
        } else {
#pragma unroll
            for (int g = 0; g < G; ++g)
#pragma unroll
                for (int t = 0; t < SD; ++t) x[g][t] = xr[g * SD + t];
        }
    }

    uint32_t packed = 0;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int s = s0 + g;
        if constexpr (LBG) {
            if (a.done[s]) continue;  // uniform
        }
        int best = argmin_lds<SD, METRIC>(x[g], lds + (size_t)g * k * SD, lds_cn + g * k, k);
        if constexpr (LBG) {
            uint8_t *p = a.codes + (size_t)s * a.n + row;
            if (*p != (uint8_t)best) {
                *p = (uint8_t)best;
                mark_changed(a.changed + s);
            }
        } else {
            if constexpr (G == 4)
                packed |= (uint32_t)best << (8 * g);
            else
                a.codes[row * a.m + s] = (uint8_t)best;
        }
    }
    if constexpr (!LBG && G == 4) {
        // m % 4 == 0 here, so the 4 codes of this lane are one aligned 32-bit word
        *reinterpret_cast<uint32_t *>(a.codes + row * a.m + s0) = packed;
    }
}

// Fallback for any sub_dim: one lane = one row, one column block per blockIdx.y, sub-vector
// re-read from memory for every group of 4 centroids; centroids read through wave-uniform
// addresses.  Same operation order as above.
template <int METRIC, bool LBG>
__global__ void __launch_bounds__(256) k_assign_dyn(AssignArgs a, int sd) {
    const int s = blockIdx.y;
    if constexpr (LBG) {
        if (a.done[s]) return;
    }
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= a.n) return;
    const int k = a.k;
    const float *__restrict__ xr = a.x + row * a.ld + (int64_t)s * sd;
    const float *__restrict__ cb = a.cb + (size_t)s * k * sd;
    const float *__restrict__ cn = a.cnorm ? a.cnorm + (size_t)s * k : nullptr;
    int best = 0;
    float bd = 0.0f, pd = __builtin_inff();
    float na = 0.0f;
    if constexpr (METRIC == M_COS) {
        float sa = 0.0f;
        for (int t = 0; t < sd; ++t) {
            float p = xr[t] * xr[t];
            sa = sa + p;
        }
        na = sqrtf(sa);
    }
    for (int j0 = 0; j0 < k; j0 += 4) {
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        const int jn = (k - j0 < 4) ? (k - j0) : 4;
        for (int t = 0; t < sd; ++t) {
            float xv = xr[t];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (u < jn) {
                    float cv = cb[(size_t)(j0 + u) * sd + t];
                    if constexpr (METRIC == M_COS) {
                        float p = xv * cv;
                        acc[u] = acc[u] + p;
                    } else if constexpr (METRIC == M_L1) {
                        float d = xv - cv;
                        acc[u] = acc[u] + fabsf(d);
                    } else {
                        float d = xv - cv;
                        float p = d * d;
                        acc[u] = acc[u] + p;
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (u < jn) {
                float d = acc[u];
                if constexpr (METRIC == M_COS) {
                    float nb = cn[j0 + u];
                    float den = na * nb;
                    float q = d / den;
                    d = 1.0f - q;
                    d = (na == 0.0f || nb == 0.0f) ? 1.0f : d;
                }
                bool upd = (j0 + u == 0) || (d < bd);
                if constexpr (METRIC == M_EUCLID) pd = (upd && (j0 + u) != 0) ? bd : pd;
                bd = upd ? d : bd;
                best = upd ? (j0 + u) : best;
            }
        }
    }
    if constexpr (METRIC == M_EUCLID) {
        float sr = sqrtf(bd);
        if (sqrtf(pd) == sr) {
            for (int j = 0; j < best; ++j) {
                float acc = 0.0f;
                for (int t = 0; t < sd; ++t) {
                    float d = xr[t] - cb[(size_t)j * sd + t];
                    float p = d * d;
                    acc = acc + p;
                }
                if (sqrtf(acc) == sr) {
                    best = j;
                    break;
                }
            }
        }
    }
    if constexpr (LBG) {
        uint8_t *p = a.codes + (size_t)s * a.n + row;
        if (*p != (uint8_t)best) {
            *p = (uint8_t)best;
            mark_changed(a.changed + s);
        }
    } else {
        a.codes[row * a.m + s] = (uint8_t)best;
    }
}

}  // namespace vq

// ---------------------------------------------------------------------------------------------
// Exact assignment for wide column blocks: one lane = up to 4 centroids, one wave = 8 rows.
// The wave keeps its 8 rows in LDS (read back as broadcasts) and every lane walks the codebook
// rows of its centroids, so each (row, centroid) distance is still one sequential f32 chain in
// the reference's order.  The argmin over centroids is a lexicographic (distance, index) minimum,
// which is exactly "strict '<', lowest index wins"; a NaN never wins unless it sits at index 0.
// Rows come either from a contiguous range (LISTED = false, grid.y = column block) or from the
// list of undecided pairs left by the matrix-core pass (LISTED = true).
namespace vq {

constexpr int kWideRows = 8;

template <int METRIC>
__device__ __forceinline__ void wide_step(float &acc, float xv, float cv) {
    if constexpr (METRIC == M_COS) {
        float p = xv * cv;
        acc = acc + p;
    } else if constexpr (METRIC == M_L1) {
        float d = xv - cv;
        acc = acc + fabsf(d);
    } else {
        float d = xv - cv;
        float p = d * d;
        acc = acc + p;
    }
}

// Distances of the wave's rows (in lds_x, row stride sd) to the centroids of block s, then the
// reference argmin per row.  rows[i] < 0 marks an unused slot.  Lane 0 returns the codes.
template <int METRIC, bool VEC, int NR>
__device__ __forceinline__ void wide_argmin(const AssignArgs &a, int sd, int s, const float *lds_x, int lane,
                                            int (&best_out)[NR]) {
    const int k = a.k;
    const float *__restrict__ cb = a.cb + (size_t)s * k * sd;
    float acc[4][NR];
    float sa[NR];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int i = 0; i < NR; ++i) acc[q][i] = 0.0f;
#pragma unroll
    for (int i = 0; i < NR; ++i) sa[i] = 0.0f;
    const float *cq[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        int j = lane + 64 * q;
        cq[q] = cb + (size_t)(j < k ? j : 0) * sd;
    }
    int t = 0;
    if constexpr (VEC) {
        // (one row per wave is a latency-bound walk over the centroids: more loads in flight)
        constexpr int kAhead = NR == 1 ? 4 : 1;
#pragma unroll kAhead
        for (; t + 4 <= sd; t += 4) {
            float4 cv[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) cv[q] = *reinterpret_cast<const float4 *>(cq[q] + t);
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const float4 xv = *reinterpret_cast<const float4 *>(lds_x + i * sd + t);
                if constexpr (METRIC == M_COS) {
                    float p;
                    p = xv.x * xv.x; sa[i] = sa[i] + p;
                    p = xv.y * xv.y; sa[i] = sa[i] + p;
                    p = xv.z * xv.z; sa[i] = sa[i] + p;
                    p = xv.w * xv.w; sa[i] = sa[i] + p;
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    wide_step<METRIC>(acc[q][i], xv.x, cv[q].x);
                    wide_step<METRIC>(acc[q][i], xv.y, cv[q].y);
                    wide_step<METRIC>(acc[q][i], xv.z, cv[q].z);
                    wide_step<METRIC>(acc[q][i], xv.w, cv[q].w);
                }
            }
        }
    }
    for (; t < sd; ++t) {
        float cv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) cv[q] = cq[q][t];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const float xv = lds_x[i * sd + t];
            if constexpr (METRIC == M_COS) {
                float p = xv * xv;
                sa[i] = sa[i] + p;
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) wide_step<METRIC>(acc[q][i], xv, cv[q]);
        }
    }
    const float inf = __builtin_inff();
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        float bd = inf, d0 = 0.0f;
        int bi = 0x7fffffff;
        float dq[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int j = lane + 64 * q;
            float d = acc[q][i];
            if constexpr (METRIC == M_COS) {
                const float na = sqrtf(sa[i]);
                const float nb = (j < k) ? a.cnorm[(size_t)s * k + j] : 1.0f;
                const float den = na * nb;
                const float qq = d / den;
                d = 1.0f - qq;
                d = (na == 0.0f || nb == 0.0f) ? 1.0f : d;
            }
            if (q == 0) d0 = d;  // lane 0 holds the distance of centroid 0
            const bool nan = !(d == d);
            d = (j < k && !nan) ? d : inf;
            dq[q] = d;
            if (j < k && d < bd) {  // ascending j inside the lane: strict '<' keeps the first
                bd = d;
                bi = j;
            }
        }
        if (bi == 0x7fffffff) bi = lane;  // all +inf in this lane: lowest index of the lane
        if (lane >= k) bi = 0x7fffffff;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float od = __shfl_xor(bd, off);
            const int oi = __shfl_xor(bi, off);
            const bool take = (od < bd) || (od == bd && oi < bi);
            bd = take ? od : bd;
            bi = take ? oi : bi;
        }
        if constexpr (METRIC == M_EUCLID) {
            // first index whose root equals the root of the smallest squared distance
            const float sr = sqrtf(bd);
            int fi = 0x7fffffff;
#pragma unroll
            for (int q = 3; q >= 0; --q) {
                const int j = lane + 64 * q;
                if (j < k && sqrtf(dq[q]) == sr) fi = j;
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const int oi = __shfl_xor(fi, off);
                fi = oi < fi ? oi : fi;
            }
            bi = fi;
        }
        const float d0b = __shfl(d0, 0);
        if (!(d0b == d0b)) bi = 0;  // NaN at index 0 is never displaced
        best_out[i] = bi;
    }
}

// The wave's share of the groups of NR rows (or listed pairs).
template <int METRIC, bool LBG, bool LISTED, bool VEC, int NR>
__device__ __forceinline__ void wide_exact_groups(const AssignArgs &a, int sd, const uint32_t *__restrict__ list,
                                                  int64_t total, float *lds_x, int lane, int wave, unsigned block,
                                                  unsigned nblocks) {
    const int64_t groups = (total + NR - 1) / NR;
    for (int64_t grp = (int64_t)block * 4 + wave; grp < groups; grp += (int64_t)nblocks * 4) {
        int64_t rows[NR];
        int ss[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int64_t e = grp * NR + i;
            rows[i] = -1;
            ss[i] = LISTED ? -1 : (int)blockIdx.y;
            if (e < total) {
                if constexpr (LISTED) {
                    const uint32_t v = list[e];
                    rows[i] = v / (uint32_t)a.m;
                    ss[i] = (int)(v % (uint32_t)a.m);
                } else {
                    rows[i] = e;
                }
            }
        }
        // sub-groups of slots that share the column block (always one group when not LISTED)
        bool pending[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) pending[i] = rows[i] >= 0;
        for (;;) {
            int s = -1;
#pragma unroll
            for (int i = NR - 1; i >= 0; --i)
                if (pending[i]) s = ss[i];
            if (s < 0) break;
            // stage the rows of this sub-group (unused slots repeat a valid row)
            int64_t fill = -1;
#pragma unroll
            for (int i = 0; i < NR; ++i)
                if (pending[i] && ss[i] == s && fill < 0) fill = rows[i];
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const int64_t rr = (pending[i] && ss[i] == s) ? rows[i] : fill;
                const float *xr = a.x + rr * a.ld + (int64_t)s * sd;
                for (int t = lane; t < sd; t += 64) lds_x[i * sd + t] = xr[t];
            }
            __builtin_amdgcn_wave_barrier();
            int best[NR];
            wide_argmin<METRIC, VEC, NR>(a, sd, s, lds_x, lane, best);
            __builtin_amdgcn_wave_barrier();
            if (lane == 0) {
#pragma unroll
                for (int i = 0; i < NR; ++i) {
                    if (pending[i] && ss[i] == s) {
                        if constexpr (LBG) {
                            uint8_t *p = a.codes + (size_t)s * a.n + rows[i];
                            if (*p != (uint8_t)best[i]) {
                                *p = (uint8_t)best[i];
                                mark_changed(a.changed + s);
                            }
                        } else {
                            a.codes[rows[i] * a.m + s] = (uint8_t)best[i];
                        }
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < NR; ++i)
                if (ss[i] == s) pending[i] = false;
        }
    }
}

// One listed pair by a whole workgroup: thread j walks centroid j (k <= 256) over the sub-vector in
// the reference's order.  The centroids come through LDS 32 dimensions at a time: a wave fetches
// the slice of its 64 centroids as whole 128-byte segments (eight lanes per centroid) and each lane
// then reads its own centroid's 32 floats from a row of 33 (no bank conflicts); the next slice is
// in flight meanwhile.  Thread j reading its centroid straight from memory touched 64 different
// lines per load instruction: 37 us for a handful of pairs.  Squared L2 and Euclidean only;
// sd % 4 == 0 and 16-byte aligned centroids.  lds: the row (sd floats), 16 floats of reduction
// space, then 256 x 33 floats of centroid slices.
constexpr int kPairWgLdsFloats = 16 + 256 * 33;  // beside the row
template <int METRIC, bool LBG>
__device__ __forceinline__ void wide_exact_pair_wg(const AssignArgs &a, int sd, uint32_t entry, float *lds) {
    static_assert(METRIC == M_SQ || METRIC == M_EUCLID, "squared L2 / Euclidean");
    const int j = threadIdx.x, lane = j & 63, wave = j >> 6, k = a.k;
    const int64_t row = entry / (uint32_t)a.m;
    const int s = (int)(entry % (uint32_t)a.m);
    const float *xr = a.x + row * a.ld + (int64_t)s * sd;
    for (int t = j; t < sd; t += 256) lds[t] = xr[t];
    __syncthreads();
    float *slice = lds + sd + 16 + wave * 64 * 33;  // this wave's 64 centroids x 33
    const float *cbs = a.cb + (size_t)s * k * sd;
    const int sub = lane >> 3, piece = lane & 7;     // centroid within a group of 8, float4 within the slice
    const int nsl = (sd + 31) / 32;
    float4 pre[8];
    auto fetch = [&](int sl) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int c = 64 * wave + 8 * i + sub;
            const int d = 32 * sl + 4 * piece;
            pre[i] = *reinterpret_cast<const float4 *>(cbs + (size_t)(c < k ? c : 0) * sd + (d < sd ? d : 0));
        }
    };
    fetch(0);
    float acc = 0.0f;
    for (int sl = 0; sl < nsl; ++sl) {
        __builtin_amdgcn_wave_barrier();  // the lanes have read the previous slice
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float *dst = slice + (8 * i + sub) * 33 + 4 * piece;
            dst[0] = pre[i].x;
            dst[1] = pre[i].y;
            dst[2] = pre[i].z;
            dst[3] = pre[i].w;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        fetch(sl + 1 < nsl ? sl + 1 : sl);
        const float *mine = slice + lane * 33;
        const int nd = sd - 32 * sl < 32 ? sd - 32 * sl : 32;
        if (nd == 32) {
#pragma unroll
            for (int t = 0; t < 32; ++t) wide_step<METRIC>(acc, lds[32 * sl + t], mine[t]);
        } else {
            for (int t = 0; t < nd; ++t) wide_step<METRIC>(acc, lds[32 * sl + t], mine[t]);
        }
    }
    const float inf = __builtin_inff();
    const float d = (j < k && acc == acc) ? acc : inf;  // a NaN distance never wins
    float *red_d = lds + sd;
    int *red_i = reinterpret_cast<int *>(lds + sd + 4);
    int *red_f = reinterpret_cast<int *>(lds + sd + 8);
    float bd = d;
    int bi = j < k ? j : 0x7fffffff;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float od = __shfl_xor(bd, off);
        const int oi = __shfl_xor(bi, off);
        const bool take = (od < bd) || (od == bd && oi < bi);
        bd = take ? od : bd;
        bi = take ? oi : bi;
    }
    if (lane == 0) {
        red_d[wave] = bd;
        red_i[wave] = bi;
    }
    if (j == 0) lds[sd + 12] = acc;  // centroid 0's distance as computed
    __syncthreads();
    bd = red_d[0];
    bi = red_i[0];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
        const float od = red_d[w];
        const int oi = red_i[w];
        const bool take = (od < bd) || (od == bd && oi < bi);
        bd = take ? od : bd;
        bi = take ? oi : bi;
    }
    if constexpr (METRIC == M_EUCLID) {
        // the reference compares the roots: first index whose root equals the smallest root
        const float sr = sqrtf(bd);
        int fi = (j < k && sqrtf(d) == sr) ? j : 0x7fffffff;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const int oi = __shfl_xor(fi, off);
            fi = oi < fi ? oi : fi;
        }
        if (lane == 0) red_f[wave] = fi;
        __syncthreads();
        bi = red_f[0];
#pragma unroll
        for (int w = 1; w < 4; ++w) bi = red_f[w] < bi ? red_f[w] : bi;
    }
    const float d0 = lds[sd + 12];
    if (!(d0 == d0)) bi = 0;  // NaN at index 0 is never displaced
    if (j == 0) {
        if constexpr (LBG) {
            uint8_t *p = a.codes + (size_t)s * a.n + row;
            if (*p != (uint8_t)bi) {
                *p = (uint8_t)bi;
                mark_changed(a.changed + s);
            }
        } else {
            a.codes[row * a.m + s] = (uint8_t)bi;
        }
    }
}

// Listed rows of a single column block (m == 1) eight at a time by a whole workgroup: the scheme of
// wide_exact_pair_wg with eight rows in LDS, so that the codebook is read once per eight rows (a
// wave that takes a listed row on its own reads every centroid for that row alone: 256 KB per row
// at k = 256, D = 256, which is what bounds a list of a few thousand rows).  Thread j keeps eight
// distances to centroid j, each a sequential chain over the sub-vector in the reference's order.
// lds: 8 rows (8 * sd floats), 8 x 16 floats of reduction space, 256 x 33 floats of centroid slices.
constexpr int kRowsWg = 8;
constexpr int kRowsWgLdsFloats = kRowsWg * 16 + 256 * 33;  // beside the rows
template <int METRIC, bool LBG>
__device__ __forceinline__ void wide_exact_rows_wg(const AssignArgs &a, int sd, const uint32_t *__restrict__ list,
                                                   int64_t total, unsigned block, unsigned nblocks, float *lds) {
    static_assert(METRIC == M_SQ || METRIC == M_EUCLID, "squared L2 / Euclidean");
    constexpr int NR = kRowsWg;
    const int j = threadIdx.x, lane = j & 63, wave = j >> 6, k = a.k;
    float *red = lds + NR * sd;                      // [NR][16]
    float *slice = red + NR * 16 + wave * 64 * 33;   // this wave's 64 centroids x 33
    const float *cbs = a.cb;
    const int sub = lane >> 3, piece = lane & 7;     // centroid within a group of 8, float4 within the slice
    const int nsl = (sd + 31) / 32;
    const float inf = __builtin_inff();
    for (int64_t grp = block; grp * NR < total; grp += nblocks) {
        int64_t rows[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int64_t e = grp * NR + i;
            rows[i] = list[e < total ? e : total - 1];  // (m == 1: an entry is a row; the tail repeats the last one)
        }
#pragma unroll
        for (int i = 0; i < NR; ++i)
            for (int t = j; t < sd; t += 256) lds[i * sd + t] = a.x[rows[i] * a.ld + t];
        __syncthreads();
        float4 pre[8];
        auto fetch = [&](int sl) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int c = 64 * wave + 8 * i + sub;
                const int d = 32 * sl + 4 * piece;
                const float4 v = *reinterpret_cast<const float4 *>(cbs + (size_t)(c < k ? c : 0) * sd + (d < sd ? d : 0));
                pre[i] = make_float4(v.x, v.y, v.z, v.w);
            }
        };
        fetch(0);
        float acc[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) acc[i] = 0.0f;
        for (int sl = 0; sl < nsl; ++sl) {
            __builtin_amdgcn_wave_barrier();  // the lanes have read the previous slice
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float *dst = slice + (8 * i + sub) * 33 + 4 * piece;
                dst[0] = pre[i].x;
                dst[1] = pre[i].y;
                dst[2] = pre[i].z;
                dst[3] = pre[i].w;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            fetch(sl + 1 < nsl ? sl + 1 : sl);
            const float *mine = slice + lane * 33;
            const int nd = sd - 32 * sl < 32 ? sd - 32 * sl : 32;
            if (nd == 32) {
#pragma unroll
                for (int t4 = 0; t4 < 8; ++t4) {
                    const float c0 = mine[4 * t4], c1 = mine[4 * t4 + 1], c2 = mine[4 * t4 + 2], c3 = mine[4 * t4 + 3];
#pragma unroll
                    for (int i = 0; i < NR; ++i) {
                        const float4 xv = *reinterpret_cast<const float4 *>(lds + i * sd + 32 * sl + 4 * t4);
                        wide_step<METRIC>(acc[i], xv.x, c0);
                        wide_step<METRIC>(acc[i], xv.y, c1);
                        wide_step<METRIC>(acc[i], xv.z, c2);
                        wide_step<METRIC>(acc[i], xv.w, c3);
                    }
                }
            } else {
                for (int t = 0; t < nd; ++t) {
                    const float cv = mine[t];
#pragma unroll
                    for (int i = 0; i < NR; ++i) wide_step<METRIC>(acc[i], lds[i * sd + 32 * sl + t], cv);
                }
            }
        }
        // per row: the smallest (distance, index), the reference's strict '<' scan
        float dd[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            dd[i] = (j < k && acc[i] == acc[i]) ? acc[i] : inf;  // a NaN distance never wins
            float bd = dd[i];
            int bi = j < k ? j : 0x7fffffff;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const float od = __shfl_xor(bd, off);
                const int oi = __shfl_xor(bi, off);
                const bool take = (od < bd) || (od == bd && oi < bi);
                bd = take ? od : bd;
                bi = take ? oi : bi;
            }
            if (lane == 0) {
                red[i * 16 + wave] = bd;
                reinterpret_cast<int *>(red)[i * 16 + 4 + wave] = bi;
            }
            if (j == 0) red[i * 16 + 12] = acc[i];  // centroid 0's distance as computed
        }
        __syncthreads();
        int best[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            float bd = red[i * 16];
            int bi = reinterpret_cast<int *>(red)[i * 16 + 4];
#pragma unroll
            for (int w = 1; w < 4; ++w) {
                const float od = red[i * 16 + w];
                const int oi = reinterpret_cast<int *>(red)[i * 16 + 4 + w];
                const bool take = (od < bd) || (od == bd && oi < bi);
                bd = take ? od : bd;
                bi = take ? oi : bi;
            }
            best[i] = bi;
            if constexpr (METRIC == M_EUCLID) {
                // the reference compares the roots: first index whose root equals the smallest root
                const float sr = sqrtf(bd);
                int fi = (j < k && sqrtf(dd[i]) == sr) ? j : 0x7fffffff;
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) {
                    const int oi = __shfl_xor(fi, off);
                    fi = oi < fi ? oi : fi;
                }
                if (lane == 0) reinterpret_cast<int *>(red)[i * 16 + 8 + wave] = fi;
            }
        }
        if constexpr (METRIC == M_EUCLID) {
            __syncthreads();
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const int *rf = reinterpret_cast<const int *>(red) + i * 16 + 8;
                int bi = rf[0];
#pragma unroll
                for (int w = 1; w < 4; ++w) bi = rf[w] < bi ? rf[w] : bi;
                best[i] = bi;
            }
        }
        if (j < NR) {
            // thread i writes row i's code
            int bi = 0;
            int64_t row = 0;
#pragma unroll
            for (int i = 0; i < NR; ++i)
                if (i == j) {
                    bi = best[i];
                    row = rows[i];
                }
            const float d0 = red[j * 16 + 12];
            if (!(d0 == d0)) bi = 0;  // NaN at index 0 is never displaced
            if (grp * NR + j < total) {
                if constexpr (LBG) {
                    uint8_t *p = a.codes + row;
                    if (*p != (uint8_t)bi) {
                        *p = (uint8_t)bi;
                        mark_changed(a.changed);
                    }
                } else {
                    a.codes[row] = (uint8_t)bi;
                }
            }
        }
        __syncthreads();  // the rows and the reduction space are written again by the next group
    }
}

// Exact decision between two candidate centroids per listed (row, column block) pair — the
// pairs the matrix-core pass narrowed down to its two best scores.  Lanes 2i and 2i + 1 take
// candidates c1 and c2 of entry i: each accumulates its distance in the reference's order
// (sequential over the sub-vector), then the smaller (distance, index) wins, which is the
// reference's strict '<' scan restricted to the only two centroids that can win it.  Euclidean
// compares the roots, as the reference does.  Requires sd % 4 == 0 and 16-byte aligned rows
// and centroids.
// Workgroup `block` of `nblocks` that share the list.
template <int METRIC, bool LBG>
__device__ __forceinline__ void wide_pair_blocks(const AssignArgs &a, int sd, const uint2 *__restrict__ pairs,
                                                 uint32_t total, unsigned block, unsigned nblocks) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float inf = __builtin_inff();
    for (uint64_t base = ((uint64_t)block * 4 + wave) * 32; base < total; base += (uint64_t)nblocks * 4 * 32) {
        const uint64_t e = base + (lane >> 1);
        const bool active = e < total;
        const uint2 ent = pairs[active ? e : base];
        const int64_t row = ent.x / (uint32_t)a.m;
        const int s = (int)(ent.x % (uint32_t)a.m);
        const int j = (int)((ent.y >> (8 * (lane & 1))) & 0xFFu);
        const float4 *xp = reinterpret_cast<const float4 *>(a.x + row * a.ld + (int64_t)s * sd);
        const float4 *cp = reinterpret_cast<const float4 *>(a.cb + ((size_t)s * a.k + j) * sd);
        float acc = 0.0f;
#pragma unroll 4
        for (int t = 0; t < sd / 4; ++t) {
            const float4 xv = xp[t], cv = cp[t];
            wide_step<METRIC>(acc, xv.x, cv.x);
            wide_step<METRIC>(acc, xv.y, cv.y);
            wide_step<METRIC>(acc, xv.z, cv.z);
            wide_step<METRIC>(acc, xv.w, cv.w);
        }
        float d = acc;
        if constexpr (METRIC == M_EUCLID) d = sqrtf(d);
        d = (d == d) ? d : inf;
        const float od = __shfl_xor(d, 1);
        const int oj = __shfl_xor(j, 1);
        const int best = (od < d || (od == d && oj < j)) ? oj : j;
        if (active && (lane & 1) == 0) {
            if constexpr (LBG) {
                uint8_t *p = a.codes + (size_t)s * a.n + row;
                if (*p != (uint8_t)best) {
                    *p = (uint8_t)best;
                    mark_changed(a.changed + s);
                }
            } else {
                a.codes[row * a.m + s] = (uint8_t)best;
            }
        }
    }
}

template <int METRIC, bool LBG, bool LISTED, bool VEC>
__global__ void __launch_bounds__(256) k_assign_wide_exact(AssignArgs a, int sd, const uint32_t *__restrict__ list,
                                                           const uint32_t *__restrict__ list_count,
                                                           const uint2 *__restrict__ pairs,
                                                           const uint32_t *__restrict__ pair_count,
                                                           unsigned exact_blocks) {
    extern __shared__ float lds_wide[];  // 4 waves x 8 rows x sd
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // The first gridDim.x - exact_blocks workgroups take the list of pairs with two candidates: the two
    // follow-ups of the matrix-core pass are independent and run side by side in one launch (the
    // pairs first: workgroups start in index order, and behind a long list of rows they would wait).
    unsigned block = blockIdx.x;
    if constexpr (LISTED && (METRIC == M_SQ || METRIC == M_EUCLID)) {
        const unsigned pair_blocks = gridDim.x - exact_blocks;
        if (block < pair_blocks) {
            wide_pair_blocks<METRIC, LBG>(a, sd, pairs, *pair_count, block, pair_blocks);
            return;
        }
        block -= pair_blocks;
    }
    float *lds_x = lds_wide + (size_t)wave * kWideRows * sd;
    const int64_t total = LISTED ? (int64_t)*list_count : a.n;
    if constexpr (LBG && !LISTED) {
        if (a.done[blockIdx.y]) return;
    }
    if constexpr (LISTED && VEC && (METRIC == M_SQ || METRIC == M_EUCLID)) {
        // a handful of pairs: one per workgroup, one centroid per thread
        if (a.k <= 256 && total <= (a.m == 1 ? 1024 : (int64_t)exact_blocks)) {
            if ((int64_t)block < total) wide_exact_pair_wg<METRIC, LBG>(a, sd, list[block], lds_wide);
            return;
        }
        // rows of a single column block: eight per workgroup, the codebook read once per eight
        if (a.k <= 256 && a.m == 1) {
            wide_exact_rows_wg<METRIC, LBG>(a, sd, list, total, block, exact_blocks, lds_wide);
            return;
        }
    }
    if constexpr (LISTED) {
        // a short list: one pair per wave, so that the pass is as long as one pair's scan, not eight
        if (total <= (int64_t)exact_blocks * 4) {
            wide_exact_groups<METRIC, LBG, LISTED, VEC, 1>(a, sd, list, total, lds_x, lane, wave, block, exact_blocks);
            return;
        }
    }
    wide_exact_groups<METRIC, LBG, LISTED, VEC, kWideRows>(a, sd, list, total, lds_x, lane, wave, block, exact_blocks);
}

}  // namespace vq
