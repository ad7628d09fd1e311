// Nearest-centroid assignment for squared-L2 / Euclidean on the matrix cores, exact by re-check.
//
// Pass 1 (k_assign_mfma): for a tile of 32 rows and one column block, the scores
//     s[j] = ||c_j||^2 + ||x||^2 - 2 x.c_j
// of 32 centroids at a time come from v_mfma_f32_32x32x2_f32 (fp32 in, fp32 accumulate; the
// accumulator starts at ||c_j||^2 + ||x||^2, the products carry -2 c_j).  The running smallest and
// second-smallest score of every row are kept with the centroid index packed into the 8 low
// mantissa bits (one v_and_or, one v_med3, one v_min per score).
// The matrix form rounds differently from the reference's sequential (x-c)^2 sum, so a row is
// only decided here when its two best scores are further apart than a bound on every error
// involved (matrix accumulation, the packed bits, the reference's own rounding):
//     gap > 2^-14 |second| + 2^-16 (||x||^2 + max_j ||c_j||^2)
// Then the smallest exact distance is provably the same centroid.  Every other (row, block)
// pair — exact ties, near ties, sqrt collisions under Euclidean, non-finite values — is appended
// to a list and decided by pass 2.
// Pass 2 (k_assign_recheck): the reference-order argmin of assign_exact.hpp on the listed pairs.
// The result is therefore bit-identical to the all-VALU path for every input.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "assign_exact.hpp"

namespace vq {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// Score of the padding centroids that fill the last block of 32; a row whose best score is not
// well below it is sent to the exact pass.
constexpr float kPadScore = 1e30f;

struct MfmaTables {
    const float *atab;     // [m][nb][64][SD/2]  -2*c in MFMA A-operand order
    const float *c2perm;   // [m][nb][2][16]     ||c||^2 in accumulator order (kPadScore for padding)
    const float *maxc2;    // [m]
    uint32_t *list;        // flagged pairs: row*m + s
    uint32_t *list_count;  // 1
    int nb;                // ceil(k/32)
};

// Builds the tables from the codebooks.  One thread per (s, padded centroid).
template <int SD>
__global__ void __launch_bounds__(256) k_mfma_prep(const float *__restrict__ cb, int m, int k, int nb,
                                                   float *__restrict__ atab, float *__restrict__ c2perm,
                                                   float *__restrict__ maxc2, uint32_t *__restrict__ list_count) {
    constexpr int HS = SD / 2;
    const int s = blockIdx.x;
    __shared__ float sh_max[256];
    float mx = 0.0f;
    for (int j = threadIdx.x; j < nb * 32; j += 256) {
        const int b = j / 32, i = j % 32;
        float c2 = kPadScore;  // padding centroids: finite, so that index bits can be packed in
        float c[SD];
        if (j < k) {
            c2 = 0.0f;
#pragma unroll
            for (int t = 0; t < SD; ++t) {
                c[t] = cb[((size_t)s * k + j) * SD + t];
                c2 = __builtin_fmaf(c[t], c[t], c2);
            }
            mx = fmaxf(mx, c2);
            if (!(c2 == c2)) mx = c2;  // a NaN poisons the bound on purpose
        } else {
#pragma unroll
            for (int t = 0; t < SD; ++t) c[t] = 0.0f;
        }
        // A operand: lane = i + 32*h holds dims [h*HS, (h+1)*HS)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int t = 0; t < HS; ++t)
                atab[(((size_t)s * nb + b) * 64 + i + 32 * h) * HS + t] = -2.0f * c[h * HS + t];
        // accumulator order: lane half h, register v <-> centroid 8*(v/4) + 4*h + v%4
        const int hh = (i / 4) % 2, v = (i / 8) * 4 + i % 4;
        c2perm[(((size_t)s * nb + b) * 2 + hh) * 16 + v] = c2;
    }
    sh_max[threadIdx.x] = mx;
    __syncthreads();
    if (threadIdx.x == 0) {
        float r = 0.0f;
        for (int i = 0; i < 256; ++i) {
            float v = sh_max[i];
            r = (v == v) ? fmaxf(r, v) : v;
            if (!(r == r)) break;
        }
        maxc2[s] = r;
        if (s == 0) *list_count = 0;
    }
}

// Scores are compared through their bit patterns as signed integers: for non-negative floats
// that is the float order, a slightly negative score (cancellation) still sorts below every
// positive one, and integer min / med3 need no NaN canonicalisation.  Two negative scores sort
// in reverse, which only happens inside the error bound, i.e. for pairs that are re-checked.
__device__ __forceinline__ int imin(int a, int b) { return a < b ? a : b; }
__device__ __forceinline__ int imax(int a, int b) { return a > b ? a : b; }
__device__ __forceinline__ int imed3(int a, int b, int c) {
    return imax(imin(a, b), imin(imax(a, b), c));
}

// One wave = TILES tiles of 32 rows, all column blocks.  256 threads = 4 waves.
// The sub-vectors of SG consecutive column blocks are loaded together, so that with SG * SD * 4
// = 128 bytes every line of the rows is fetched once.
template <int SD, bool LBG, int TILES, int SG>
__global__ void __launch_bounds__(256) k_assign_mfma(AssignArgs a, MfmaTables tb) {
    constexpr int HS = SD / 2;     // floats per lane of a sub-vector
    extern __shared__ float lds_c2[];  // [m][nb][2][16]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int nb = tb.nb, m = a.m;
    for (int i = threadIdx.x; i < m * nb * 32; i += 256) lds_c2[i] = tb.c2perm[i];
    __syncthreads();
    const int64_t row_base = ((int64_t)blockIdx.x * 4 + wave) * (32 * TILES);
    if (row_base >= a.n) return;

    // index bits of the 16 accumulator registers of this lane half
    uint32_t cvh[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) cvh[v] = (uint32_t)(8 * (v / 4) + 4 * h + v % 4);

    // encode mode: the codes of a row are collected in registers and stored once per row
    constexpr int MAXW = 4;  // up to 16 column blocks packed
    const bool packed_out = !LBG && (m % 4 == 0) && (m <= 4 * MAXW);
    uint32_t cw[TILES][MAXW];
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int w = 0; w < MAXW; ++w) cw[t][w] = 0u;

    for (int s0 = 0; s0 < m; s0 += SG) {
      float xall[TILES][SG][HS];
#pragma unroll
      for (int t = 0; t < TILES; ++t) {
          const int64_t row = row_base + 32 * t + r;
          if (row < a.n) {
              const float *xr = a.x + row * a.ld + (int64_t)s0 * SD + h * HS;
#pragma unroll
              for (int q = 0; q < SG; ++q)
#pragma unroll
                  for (int u = 0; u < HS; ++u) xall[t][q][u] = xr[q * SD + u];
          } else {
#pragma unroll
              for (int q = 0; q < SG; ++q)
#pragma unroll
                  for (int u = 0; u < HS; ++u) xall[t][q][u] = 0.0f;
          }
      }
#pragma unroll
      for (int q = 0; q < SG; ++q) {
        const int s = s0 + q;
        if constexpr (LBG) {
            if (a.done[s]) continue;
        }
        float xb[TILES][HS], x2[TILES];
        int m1[TILES], m2[TILES];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            float p = 0.0f;
#pragma unroll
            for (int u = 0; u < HS; ++u) {
                xb[t][u] = xall[t][q][u];
                p = __builtin_fmaf(xb[t][u], xb[t][u], p);
            }
            x2[t] = p + __shfl_xor(p, 32);
            m1[t] = 0x7f800000;  // +inf
            m2[t] = 0x7f800000;
        }
        const float *ap = tb.atab + ((size_t)s * nb * 64 + lane) * HS;
        const float *cp = lds_c2 + ((size_t)s * nb * 2 + h) * 16;
        for (int b = 0; b < nb; ++b) {
            float av[HS], c2v[16];
#pragma unroll
            for (int u = 0; u < HS; ++u) av[u] = ap[(size_t)b * 64 * HS + u];
#pragma unroll
            for (int v = 0; v < 16; ++v) c2v[v] = cp[b * 32 + v];
            uint32_t idxb[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) idxb[v] = cvh[v] | ((uint32_t)b << 5);
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                floatx16 acc;
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[v] = c2v[v] + x2[t];
#pragma unroll
                for (int u = 0; u < HS; ++u)
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u], xb[t][u], acc, 0, 0, 0);
                // running smallest / second smallest with the centroid index in the low 8 bits
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    int key = (int)((__float_as_uint(acc[v]) & 0xFFFFFF00u) | idxb[v]);
                    m2[t] = imed3(m1[t], m2[t], key);
                    m1[t] = imin(m1[t], key);
                }
            }
        }
        const float mc2 = tb.maxc2[s];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            // the partner lane (other half) saw the other 16 centroids of every block
            int o1 = __shfl_xor(m1[t], 32), o2 = __shfl_xor(m2[t], 32);
            const float s1 = __int_as_float(imin(m1[t], o1));
            const float s2 = __int_as_float(imin(imax(m1[t], o1), imin(m2[t], o2)));
            const int64_t row = row_base + 32 * t + r;
            if (h == 0 && row < a.n) {
                float bound = x2[t] + mc2;
                float margin = 6.103515625e-05f * fabsf(s2) + 1.52587890625e-05f * bound;
                bool sure = (s2 - s1) > margin;  // false for NaN / inf-inf
                sure = sure && (bound < 1e29f) && (s1 < 1e29f);
                if (sure) {
                    uint8_t code = (uint8_t)(__float_as_uint(s1) & 0xFFu);
                    if constexpr (LBG) {
                        uint8_t *p = a.codes + (size_t)s * a.n + row;
                        if (*p != code) {
                            *p = code;
                            a.changed[s] = 1;
                        }
                    } else if (packed_out) {
#pragma unroll
                        for (int w = 0; w < MAXW; ++w)
                            if (w == (s >> 2)) cw[t][w] |= (uint32_t)code << (8 * (s & 3));
                    } else {
                        a.codes[row * m + s] = code;
                    }
                } else {
                    uint32_t pos = atomicAdd(tb.list_count, 1u);
                    tb.list[pos] = (uint32_t)(row * m + s);
                }
            }
        }
    }
    }  // column-block group
    if constexpr (!LBG) {
        if (packed_out && h == 0) {
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                const int64_t row = row_base + 32 * t + r;
                if (row < a.n) {
                    uint32_t *dst = reinterpret_cast<uint32_t *>(a.codes + row * m);
#pragma unroll
                    for (int w = 0; w < MAXW; ++w)
                        if (w < m / 4) dst[w] = cw[t][w];
                }
            }
        }
    }
}

// Pass 2: exact reference-order argmin for the listed (row, block) pairs.  One lane per pair.
template <int SD, int METRIC, bool LBG>
__global__ void __launch_bounds__(256) k_assign_recheck(AssignArgs a, const uint32_t *__restrict__ list,
                                                        const uint32_t *__restrict__ list_count) {
    const uint32_t count = *list_count;
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < count; i += gridDim.x * 256) {
        const uint32_t e = list[i];
        const int64_t row = e / (uint32_t)a.m;
        const int s = (int)(e % (uint32_t)a.m);
        float x[SD], c[SD];
        const float *xr = a.x + row * a.ld + (int64_t)s * SD;
#pragma unroll
        for (int t = 0; t < SD; ++t) x[t] = xr[t];
        const float *cb = a.cb + (size_t)s * a.k * SD;
        int best = 0;
#pragma unroll
        for (int t = 0; t < SD; ++t) c[t] = cb[t];
        float bd = d_sq<SD>(x, c), pd = __builtin_inff();
        for (int j = 1; j < a.k; ++j) {
#pragma unroll
            for (int t = 0; t < SD; ++t) c[t] = cb[(size_t)j * SD + t];
            float d = d_sq<SD>(x, c);
            bool u = d < bd;
            if constexpr (METRIC == M_EUCLID) pd = u ? bd : pd;
            bd = u ? d : bd;
            best = u ? j : best;
        }
        if constexpr (METRIC == M_EUCLID) {
            float sr = sqrtf(bd);
            if (sqrtf(pd) == sr) {
                for (int j = 0; j < best; ++j) {
#pragma unroll
                    for (int t = 0; t < SD; ++t) c[t] = cb[(size_t)j * SD + t];
                    if (sqrtf(d_sq<SD>(x, c)) == sr) {
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
                a.changed[s] = 1;
            }
        } else {
            a.codes[row * a.m + s] = (uint8_t)best;
        }
    }
}

}  // namespace vq

// =============================================================================================
// Wide column blocks (sub_dim a multiple of 8, up to the full dimension: RVQ stages).
// Same two-pass scheme; the contraction over sub_dim is a loop over chunks of 8 dimensions with
// the scores of all 8 blocks of 32 centroids kept in accumulators (128 registers per lane), the
// -2c operand of a chunk staged once per workgroup in LDS and shared by its 4 waves.
namespace vq {

struct MfmaWideTables {
    const float *atab;     // [m][sd/8][nb][64][4]  -2*c in MFMA A-operand order, chunk-major
    const float *c2perm;   // [m][nb][2][16]
    const float *maxc2;    // [m]
    uint32_t *list;
    uint32_t *list_count;
    int nb;
    int sd;
    float kappa;           // error-bound coefficient on (||x||^2 + max ||c||^2)
};

static __global__ void __launch_bounds__(256) k_mfma_wide_prep(const float *__restrict__ cb, int m, int k, int nb,
                                                               int sd, float *__restrict__ atab,
                                                               float *__restrict__ c2perm,
                                                               float *__restrict__ maxc2,
                                                               uint32_t *__restrict__ list_count) {
    const int s = blockIdx.x;
    const int nkc = sd / 8;
    __shared__ float sh_max[256];
    float mx = 0.0f;
    for (int j = threadIdx.x; j < nb * 32; j += 256) {
        const int b = j / 32, i = j % 32;
        const float *c = cb + ((size_t)s * k + j) * sd;
        float c2 = kPadScore;
        if (j < k) {
            c2 = 0.0f;
            for (int t = 0; t < sd; ++t) c2 = __builtin_fmaf(c[t], c[t], c2);
            mx = fmaxf(mx, c2);
            if (!(c2 == c2)) mx = c2;
        }
        for (int kc = 0; kc < nkc; ++kc)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    atab[((((size_t)s * nkc + kc) * nb + b) * 64 + i + 32 * h) * 4 + u] =
                        (j < k) ? -2.0f * c[kc * 8 + 4 * h + u] : 0.0f;
        const int hh = (i / 4) % 2, v = (i / 8) * 4 + i % 4;
        c2perm[(((size_t)s * nb + b) * 2 + hh) * 16 + v] = c2;
    }
    sh_max[threadIdx.x] = mx;
    __syncthreads();
    if (threadIdx.x == 0) {
        float r = 0.0f;
        for (int i = 0; i < 256; ++i) {
            float v = sh_max[i];
            r = (v == v) ? fmaxf(r, v) : v;
            if (!(r == r)) break;
        }
        maxc2[s] = r;
        if (s == 0) *list_count = 0;
    }
}

// grid (ceil(n/128), m); 256 threads = 4 waves, one tile of 32 rows per wave.
template <bool LBG>
__global__ void __launch_bounds__(256) k_assign_mfma_wide(AssignArgs a, MfmaWideTables tb) {
    constexpr int NBMAX = 8;
    __shared__ float4 lds_a[2][NBMAX * 64];
    __shared__ float lds_c2[NBMAX * 32];
    const int s = blockIdx.y;
    if constexpr (LBG) {
        if (a.done[s]) return;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int nb = tb.nb, sd = tb.sd, nkc = sd / 8;
    const int64_t row = ((int64_t)blockIdx.x * 4 + wave) * 32 + r;
    const bool valid = row < a.n;
    const float4 *ag = reinterpret_cast<const float4 *>(tb.atab) + (size_t)s * nkc * nb * 64;
    const int chunk4 = nb * 64;  // float4 per chunk
    for (int i = threadIdx.x; i < nb * 32; i += 256) lds_c2[i] = tb.c2perm[(size_t)s * nb * 32 + i];
    for (int i = threadIdx.x; i < chunk4; i += 256) lds_a[0][i] = ag[i];
    __syncthreads();

    floatx16 acc[NBMAX];
#pragma unroll
    for (int b = 0; b < NBMAX; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[b][v] = 0.0f;
    const float *xr = a.x + (valid ? row : 0) * a.ld + (int64_t)s * sd + 4 * h;
    float p = 0.0f;
    for (int kc = 0; kc < nkc; ++kc) {
        const int cur = kc & 1;
        // fetch the next chunk of the -2c operand while this one is used
        float4 pre[2];
        const bool more = kc + 1 < nkc;
        if (more) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                int i = threadIdx.x + 256 * q;
                if (i < chunk4) pre[q] = ag[(size_t)(kc + 1) * chunk4 + i];
            }
        }
        float4 xv = make_float4(0.f, 0.f, 0.f, 0.f);
        if (valid) xv = *reinterpret_cast<const float4 *>(xr + kc * 8);
        p = __builtin_fmaf(xv.x, xv.x, p);
        p = __builtin_fmaf(xv.y, xv.y, p);
        p = __builtin_fmaf(xv.z, xv.z, p);
        p = __builtin_fmaf(xv.w, xv.w, p);
#pragma unroll
        for (int b = 0; b < NBMAX; ++b) {
            if (b < nb) {
                const float4 av = lds_a[cur][b * 64 + lane];
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.x, xv.x, acc[b], 0, 0, 0);
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.y, xv.y, acc[b], 0, 0, 0);
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.z, xv.z, acc[b], 0, 0, 0);
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.w, xv.w, acc[b], 0, 0, 0);
            }
        }
        if (more) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                int i = threadIdx.x + 256 * q;
                if (i < chunk4) lds_a[cur ^ 1][i] = pre[q];
            }
        }
        __syncthreads();
    }
    const float x2 = p + __shfl_xor(p, 32);
    int m1 = 0x7f800000, m2 = 0x7f800000;
#pragma unroll
    for (int b = 0; b < NBMAX; ++b) {
        if (b < nb) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float sc = acc[b][v] + (lds_c2[(b * 2 + h) * 16 + v] + x2);
                const uint32_t idx = (uint32_t)(32 * b + 8 * (v / 4) + 4 * h + v % 4);
                const int key = (int)((__float_as_uint(sc) & 0xFFFFFF00u) | idx);
                m2 = imed3(m1, m2, key);
                m1 = imin(m1, key);
            }
        }
    }
    const int o1 = __shfl_xor(m1, 32), o2 = __shfl_xor(m2, 32);
    const float s1 = __int_as_float(imin(m1, o1));
    const float s2 = __int_as_float(imin(imax(m1, o1), imin(m2, o2)));
    if (h == 0 && valid) {
        const float bound = x2 + tb.maxc2[s];
        const float margin = 6.103515625e-05f * fabsf(s2) + tb.kappa * bound;
        bool sure = (s2 - s1) > margin;
        sure = sure && (bound < 1e29f) && (s1 < 1e29f);
        if (sure) {
            const uint8_t code = (uint8_t)(__float_as_uint(s1) & 0xFFu);
            if constexpr (LBG) {
                uint8_t *pc = a.codes + (size_t)s * a.n + row;
                if (*pc != code) {
                    *pc = code;
                    a.changed[s] = 1;
                }
            } else {
                a.codes[row * a.m + s] = code;
            }
        } else {
            const uint32_t pos = atomicAdd(tb.list_count, 1u);
            tb.list[pos] = (uint32_t)(row * a.m + s);
        }
    }
}

// Pass 2 for any sub_dim: exact reference-order argmin for the listed pairs, one lane per pair.
template <int METRIC, bool LBG>
__global__ void __launch_bounds__(256) k_assign_recheck_dyn(AssignArgs a, int sd, const uint32_t *__restrict__ list,
                                                            const uint32_t *__restrict__ list_count) {
    const uint32_t count = *list_count;
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < count; i += gridDim.x * 256) {
        const uint32_t e = list[i];
        const int64_t row = e / (uint32_t)a.m;
        const int s = (int)(e % (uint32_t)a.m);
        const float *__restrict__ xr = a.x + row * a.ld + (int64_t)s * sd;
        const float *__restrict__ cb = a.cb + (size_t)s * a.k * sd;
        int best = 0;
        float bd = 0.0f, pd = __builtin_inff();
        for (int j = 0; j < a.k; ++j) {
            float acc = 0.0f;
            for (int t = 0; t < sd; ++t) {
                float d = xr[t] - cb[(size_t)j * sd + t];
                float q = d * d;
                acc = acc + q;
            }
            bool u = (j == 0) || (acc < bd);
            if constexpr (METRIC == M_EUCLID) pd = (u && j != 0) ? bd : pd;
            bd = u ? acc : bd;
            best = u ? j : best;
        }
        if constexpr (METRIC == M_EUCLID) {
            float sr = sqrtf(bd);
            if (sqrtf(pd) == sr) {
                for (int j = 0; j < best; ++j) {
                    float acc = 0.0f;
                    for (int t = 0; t < sd; ++t) {
                        float d = xr[t] - cb[(size_t)j * sd + t];
                        float q = d * d;
                        acc = acc + q;
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
                a.changed[s] = 1;
            }
        } else {
            a.codes[row * a.m + s] = (uint8_t)best;
        }
    }
}

}  // namespace vq
