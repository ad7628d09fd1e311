// Nearest-centroid assignment for squared-L2 / Euclidean on the matrix cores, exact by re-check.
//
// The scores  s[j] = ||c_j||^2 + ||x||^2 - 2 x.c_j  of 32 rows against 32 centroids at a time come
// out of the matrix cores.  The matrix form rounds differently from the reference's sequential
// (x-c)^2 sum, so a row is only decided from the scores when its best candidates are further
// apart than a bound on every error involved (operand splitting, matrix accumulation, the index
// bits packed into the 8 low mantissa bits, the reference's own rounding).  Then the smallest
// exact distance provably lies where the scores say.  Every other (row, block) pair — exact ties,
// near ties, sqrt collisions under Euclidean, non-finite values — is decided by the
// reference-order argmin, so the result is bit-identical to the all-VALU path for every input.
// The 8-float kernel keeps the two smallest keys over runs of four consecutive centroids (the
// run's smallest score, tagged with the run's first index) and picks inside the best run by exact
// distances; the wide kernel keeps the three smallest scores, one tag per score.
//
// 8-float column blocks (k_assign_mfma_bf): bf16 matrix cores with split operands; the undecided
// rows are resolved inside the same wave.  Wider blocks (k_assign_mfma_wide_bf): the same split
// per chunk of 8 dimensions; the undecided pairs are listed for the exact kernel of assign_exact.hpp.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "assign_exact.hpp"

namespace vq {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// Score of the padding centroids that fill the last block of 32; a row whose best score is not
// well below it is decided by the exact path.
constexpr float kPadScore = 1e30f;

// Scores are compared through their bit patterns as signed integers: for non-negative floats
// that is the float order, a slightly negative score (cancellation) still sorts below every
// positive one, and integer min / med3 need no NaN canonicalisation.  Two negative scores sort
// in reverse, which only happens inside the error bound, i.e. for pairs that are re-checked.
__device__ __forceinline__ int imin(int a, int b) { return a < b ? a : b; }
__device__ __forceinline__ int imax(int a, int b) { return a > b ? a : b; }
__device__ __forceinline__ int imed3(int a, int b, int c) {
    return imax(imin(a, b), imin(imax(a, b), c));
}
// v_min3_i32 by name: the compiler otherwise splits the chain of smallest keys into pairs of v_min_i32.
__device__ __forceinline__ int imin3(int a, int b, int c) {
    int r;
    asm("v_min3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// (score bits & keep) | tag as one v_and_or_b32 with the tag in a scalar register: keep must be a
// vector register the compiler cannot see through (with a literal mask it emits a v_and with the
// literal and a v_or with the scalar operand, twice the issue time).  Left to the compiler rather
// than written as inline assembly so that it inserts the wait states between a matrix
// instruction and the first read of its result.
__device__ __forceinline__ uint32_t opaque_vgpr(uint32_t value) {
    uint32_t r;
    asm volatile("v_mov_b32 %0, %1" : "=v"(r) : "s"(value));
    return r;
}
__device__ __forceinline__ int pack_tag(float score, uint32_t keep, uint32_t tag) {
    return (int)((__float_as_uint(score) & keep) | tag);
}

// The values of lanes l and l ^ 32 in one vector instruction (v_permlane32_swap: the upper half of
// the first operand and the lower half of the second change places).  Lanes below 32 get
// (own, partner), the others (partner, own): for symmetric uses only.
__device__ __forceinline__ void swap_halves(int v, int &a, int &b) {
    const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    a = (int)r[0];
    b = (int)r[1];
}

// v_med3_i32 / v_max3_i32 by name, for the same reason.  Not for operands that a matrix instruction
// has just written: the compiler does not count wait states for inline assembly.
__device__ __forceinline__ int imed3a(int a, int b, int c) {
    int r;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ int imax3a(int a, int b, int c) {
    int r;
    asm("v_max3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Four new keys into the running three smallest (m1 <= m2 <= m3): 10 operations.  The smallest
// comes out of two min3 steps; the second is the smallest of m2 and the two medians; the third
// is the smallest of everything else that can still be third: the median of those three, the
// two maxima, and m3.
__device__ __forceinline__ void top3_push4(int &m1, int &m2, int &m3, int k0, int k1, int k2, int k3) {
    const int ta = imed3a(m1, k0, k1), xa = imax3a(m1, k0, k1), a1 = imin3(m1, k0, k1);
    const int tb = imed3a(a1, k2, k3), xb = imax3a(a1, k2, k3);
    m1 = imin3(a1, k2, k3);
    const int md = imed3a(m2, ta, tb);
    m2 = imin3(m2, ta, tb);
    m3 = imin(imin3(m3, xa, xb), md);
}

// Four new keys into the running (smallest, second smallest): 5 operations.
// second smallest of {m1, m2, x, y} with m1 <= m2 is min(m2, med3(m1, x, y)).
__device__ __forceinline__ void top2_push4(int &m1, int &m2, int k0, int k1, int k2, int k3) {
    const int ta = imed3(m1, k0, k1);
    const int a1 = imin3(m1, k0, k1);
    const int tb = imed3(a1, k2, k3);
    m1 = imin3(a1, k2, k3);
    m2 = imin3(m2, ta, tb);
}

// ---------------------------------------------------------------------------------------------
// 8-float column blocks on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16, 4x the fp32 rate).
//
// Every fp32 operand is split into two bf16 numbers, v = vh + vl + e with |e| <= 2^-16 |v|
// (round-to-nearest-even twice).  With a = -2c, the lanes of half h = lane / 32 own dimensions
// [4h, 4h + 4) of the block and the 8 contraction slots of that half hold
//     instruction 1:  ah . xh  (4 slots)   ah . xl  (4 slots)
//     instruction 2:  al . xh  (4 slots)   1 . (the half's share of ||x||^2, one slot; an empty
//                                               slot; ||c||^2 in three bf16 parts over the two halves)
// so a lane loads and splits only its own 16 bytes of the row and both halves do the same work:
// the result is the score ||c||^2 + ||x||^2 - 2 x.c + delta with an error of at most
// 3 * 2^-16 * sum|a_t||x_t| <= 3 * 2^-16 (||x||^2 + ||c||^2) from the dropped terms (a ex, x ea,
// al xl) plus at most 2^-17.9 (||x||^2 + ||c||^2) from the fp32 accumulation of the 2 x 15
// addends.  delta: the share of ||x||^2 rides as ONE bf16 number rounded up, 0 <= delta <
// 2^-7 ||x||^2; the product 1 . share is exact and the same addend in every score of the row, so
// delta cancels in the difference of two scores (it lengthens the partial sums, and with them the
// accumulation bound, by under 1 %), and rounding up keeps scores of near-zero distances from
// turning negative.  Two candidates compared: below 2^-13.2 (||x||^2 + max ||c||^2); the test
// uses 2^-13, plus 2^-14 |second| for the packed bits and the reference's own rounding.  bf16
// keeps the fp32 exponent range, so no scaling is needed; non-finite values fail the test.
// x and c here are the row and the centroid minus the block's centre mu (rounded to fp32): the
// rounding of the two differences moves a squared distance by at most 2^-22 (||x||^2 + ||c||^2),
// far inside the slack between 2^-13.2 and 2^-13, and the bound itself shrinks with the norms.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kStatSlots = 64;    // counters of undecided pairs, one 128-byte line apart
constexpr int kStatStride = 32;

struct MfmaBfTables {
    const u32x4 *atab;     // [m][nb][2][64]  A operands of the two instructions, lane order
    const float *maxc2;    // [m]  largest ||c - mu||^2 of the column block (NaN if any is NaN)
    const float *mu;       // [m][8]  the block's centre: mean of its centroids
    uint32_t *stat;        // [kStatSlots * kStatStride]  pairs decided by the exact path (measurement)
    int nb;                // blocks of 32 centroids, padded to an even number
};

// float -> bf16 bits, round to nearest even (NaN stays NaN).
__host__ __device__ __forceinline__ uint32_t bf16_rne_bits(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __uint_as_float(b << 16); }

// two floats -> packed bf16 pair (lo = first), round to nearest even
__device__ __forceinline__ uint32_t bf16_pack2(float a, float b) {
    floatx2 f = {a, b};
    bf16x2 h = __builtin_convertvector(f, bf16x2);
    return __builtin_bit_cast(uint32_t, h);
}

// Tables for k_assign_mfma_bf.  One workgroup per column block s, one thread per padded centroid
// (k <= 256).  Rows and centroids are scored relative to mu[s] = mean of the block's centroids
// (distances do not change under a common shift, the bound on the score error, which is
// proportional to ||x - mu||^2 + ||c - mu||^2, does); maxc2[s] = largest ||c - mu||^2 of the
// block (NaN if any is NaN).  mfma_bf_prep_block is the work of one workgroup, given centroid j
// of the block in thread j's registers (zeros from k on); k_mfma_bf_prep reads the centroids from
// the codebook, the LBG loop's last update kernel has just computed them.
__device__ __forceinline__ void mfma_bf_prep_block(float (&c)[8], int s, int j, int k, int nb,
                                                   u32x4 *__restrict__ atab, float *__restrict__ maxc2,
                                                   float *__restrict__ mu) {
    __shared__ float sh_max[4];
    __shared__ float sh_mu[4][8];
    // centre: sum of c / 256 (no overflow for k <= 256), then * 256 / k
    float centre[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        float v = c[t] * 0.00390625f;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
        if ((j & 63) == 0) sh_mu[j >> 6][t] = v;
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        centre[t] = (((sh_mu[0][t] + sh_mu[1][t]) + sh_mu[2][t]) + sh_mu[3][t]) * (256.0f / (float)k);
        if (j == 0) mu[s * 8 + t] = centre[t];
    }
    float mx = 0.0f;
    if (j < nb * 32) {
        const int b = j / 32, i = j % 32;
        float c2 = kPadScore;  // padding centroids: finite, so that index bits can be packed in
        if (j < k) {
            c2 = 0.0f;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                c[t] -= centre[t];
                c2 = __builtin_fmaf(c[t], c[t], c2);
            }
            mx = c2;
        }
        uint32_t hb[8], lb[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const float a = -2.0f * c[t];
            hb[t] = bf16_rne_bits(a);
            lb[t] = bf16_rne_bits(a - bf16_bits_to_float(hb[t]));
        }
        // ||c - mu||^2 rides in the spare slots of the second instruction as three bf16 parts
        // (exact: 3 x 8 bits), against ones in the row operand
        const uint32_t c2a = bf16_rne_bits(c2);
        const float c2r = c2 - bf16_bits_to_float(c2a);
        const uint32_t c2b = bf16_rne_bits(c2r);
        const uint32_t c2c = bf16_rne_bits(c2r - bf16_bits_to_float(c2b));
        // lane i + 32 h: instruction 1 {ah[4h..4h+3], ah[4h..4h+3]}, instruction 2
        // {al[4h..4h+3], 1, 1, c2 parts: (1st, 2nd) in the lower half, (3rd, 0) in the upper}
        u32x4 *dst = atab + ((size_t)s * nb + b) * 128;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t ah0 = hb[4 * h] | (hb[4 * h + 1] << 16), ah1 = hb[4 * h + 2] | (hb[4 * h + 3] << 16);
            const uint32_t al0 = lb[4 * h] | (lb[4 * h + 1] << 16), al1 = lb[4 * h + 2] | (lb[4 * h + 3] << 16);
            dst[32 * h + i] = u32x4{ah0, ah1, ah0, ah1};
            dst[64 + 32 * h + i] = u32x4{al0, al1, 0x3f803f80u, h == 0 ? (c2a | (c2b << 16)) : c2c};
        }
    }
    // largest ||c||^2; a NaN poisons the bound on purpose
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_xor(mx, off);
        mx = (mx == mx && o == o) ? fmaxf(mx, o) : __builtin_nanf("");
    }
    if ((j & 63) == 0) sh_max[j >> 6] = mx;
    __syncthreads();
    if (j == 0) {
        float r = sh_max[0];
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            const float o = sh_max[w];
            r = (r == r && o == o) ? fmaxf(r, o) : __builtin_nanf("");
        }
        maxc2[s] = r;
    }
}

static __global__ void __launch_bounds__(256) k_mfma_bf_prep(const float *__restrict__ cb, int m, int k, int nb,
                                                             u32x4 *__restrict__ atab, float *__restrict__ maxc2,
                                                             float *__restrict__ mu, uint32_t *__restrict__ stat) {
    const int s = blockIdx.x, j = threadIdx.x;
    if (s == 0 && j < kStatSlots) stat[j * kStatStride] = 0u;
    float c[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) c[t] = (j < k) ? cb[((size_t)s * k + j) * 8 + t] : 0.0f;
    mfma_bf_prep_block(c, s, j, k, nb, atab, maxc2, mu);
}

// ---- the exact path of k_assign_mfma_bf ---------------------------------------------------------
// Undecided rows of one (tile of 32 rows, column block) are decided by the whole wave in the
// reference's order (src/utils.rs:63-70, src/pq.rs:166-174): lane l owns centroids l, l + 64,
// l + 128, l + 192 (read from the wave's copy in LDS), computes their distances to the row in sequential f32 order, keeps the first smallest
// (strict '<' over ascending indices), and the smallest (distance, index) pair over the lanes wins.
// A NaN distance is never chosen unless it is centroid 0's, which is never replaced.  Euclidean
// compares the roots, as the reference does.  No LDS and, per batch of up to eight rows, one
// memory round trip: lane L fetches float L % 8 of the batch's row L / 8, and the row's floats
// reach every lane as scalars (v_readlane).
template <int CTRL> __device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}
// (d, i) <- the lexicographically smaller of (d, i) and (od, oi); d holds non-negative float bits
__device__ __forceinline__ void lexmin(uint32_t &d, uint32_t &i, uint32_t od, uint32_t oi) {
    const bool take = od < d || (od == d && oi < i);
    d = take ? od : d;
    i = take ? oi : i;
}

// cl: the column block's centroids in LDS (k x 8 floats, this wave's copy).
// todo: ballot of the lanes (below 32) whose row is undecided; xblk = first row of the tile.
// Returns the codes of those rows in their lanes, and their distances in dist (other lanes keep
// `code` and `dist`).
template <int METRIC>
__device__ __forceinline__ int exact_rows8(unsigned long long todo, int code, float &dist, const float *cl,
                                           const float *__restrict__ xblk, int64_t ld, int k, int lane) {
    const float inf = __builtin_inff();
    while (todo) {
        int src[8];
        int cnt = 0;
        int mine = __builtin_amdgcn_readfirstlane(__ffsll(todo) - 1);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            src[i] = todo ? __builtin_amdgcn_readfirstlane(__ffsll(todo) - 1) : src[0];
            if (todo) ++cnt;
            todo &= todo - 1;
            if ((lane >> 3) == i) mine = src[i];
        }
        const float val = xblk[(int64_t)mine * ld + (lane & 7)];
        for (int i = 0; i < cnt; ++i) {
            float xs[8];
#pragma unroll
            for (int d = 0; d < 8; ++d)
                xs[d] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(val), 8 * i + d));
            float bd = inf, dfirst = 0.0f;
            uint32_t bi = 0x7fffffffu;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int j = lane + 64 * q;
                const float4 *cp = reinterpret_cast<const float4 *>(cl + (j < k ? j : 0) * 8);
                const float4 c0 = cp[0], c1 = cp[1];
                const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
                float d = d_sq<8>(xs, c);
                if constexpr (METRIC == M_EUCLID) d = sqrtf(d);
                if (q == 0) dfirst = d;
                d = (d == d) ? d : inf;
                if (j < k && (d < bd || bi == 0x7fffffffu)) {
                    bd = d;
                    bi = (uint32_t)j;
                }
            }
            uint32_t kd = __float_as_uint(bd), ki = bi;
            lexmin(kd, ki, dpp_u32<0xB1>(kd), dpp_u32<0xB1>(ki));
            lexmin(kd, ki, dpp_u32<0x4E>(kd), dpp_u32<0x4E>(ki));
            lexmin(kd, ki, dpp_u32<0x141>(kd), dpp_u32<0x141>(ki));
            lexmin(kd, ki, dpp_u32<0x140>(kd), dpp_u32<0x140>(ki));
            uint32_t rd = (uint32_t)__builtin_amdgcn_readlane((int)kd, 0), ri = (uint32_t)__builtin_amdgcn_readlane((int)ki, 0);
#pragma unroll
            for (int row = 1; row < 4; ++row)
                lexmin(rd, ri, (uint32_t)__builtin_amdgcn_readlane((int)kd, 16 * row),
                       (uint32_t)__builtin_amdgcn_readlane((int)ki, 16 * row));
            const float d0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(dfirst), 0));
            const int best = (d0 == d0) ? (int)ri : 0;
            int who = src[0];
#pragma unroll
            for (int u = 1; u < 8; ++u) who = (i == u) ? src[u] : who;
            if (lane == who) {
                code = best;
                dist = (d0 == d0) ? __uint_as_float(rd) : d0;  // the chosen centroid's distance as computed
            }
        }
    }
    return code;
}

// One wave = one column block of 8 floats against a run of tiles of 32 rows.  The wave keeps the
// A operands of all the block's centroids in registers (8 blocks of 32 centroids x 2 instructions
// x 4 registers) and a copy of the block's centroids in LDS, and streams the rows past them: the
// inner loop reads no memory.  A lane's 16 scores of a tile are four runs of four consecutive
// centroids; the smallest score of a run, tagged with the run's first index, is the run's key, and
// the smallest and second-smallest key of the row are kept (two minima and one v_and_or per run,
// five v_min3 / v_med3 per four runs: 17 vector instructions for 16 scores).  When the two best
// keys are further apart than the error bound, every centroid outside the best run is provably
// further from the row than the run's best one, and the reference's choice is the first smallest
// exact distance among the run's four centroids, which the two lane halves compute from the LDS
// copy, two centroids each.  Otherwise the row goes through the reference-order argmin.
// SG = 4: the four waves of a workgroup take the four column blocks of one 128-byte line of the
// same rows.  SG = 1 (m not a multiple of 4): the four waves take consecutive runs of one block.
// FULL: 8 blocks of 32 centroids (k above 224), scored without a branch between them.
template <int METRIC, bool LBG, int SG, bool FULL>
__global__ void __launch_bounds__(256, 3) k_assign_mfma_bf(AssignArgs a, MfmaBfTables tb, int run_tiles, int64_t nruns,
                                                            int64_t run_stride) {
    constexpr int SD = 8;
    __shared__ __attribute__((aligned(16))) float lds_cb[4][256 * SD];
    // the wave's number through readfirstlane: what follows from it (column block, first row, base
    // addresses) is then uniform for the compiler and lives in scalar registers
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int r = lane & 31, h = lane >> 5;
    const int nb = FULL ? 8 : tb.nb, m = a.m, k = a.k;
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2: workgroups id, id + 8,
    // id + 16, ... (the same XCD, dispatched close together) take the column-block groups of one
    // run of rows, so that the code bytes of a row are merged in one L2 before they are written back.
    const int ngroups = m / SG;
    const unsigned per_chunk = 8u * (unsigned)ngroups;
    const unsigned chunk_id = blockIdx.x / per_chunk, rem = blockIdx.x % per_chunk;
    const int g = (int)(rem / 8u);
    const int64_t run_first = (int64_t)chunk_id * 8 + (rem % 8u);
    const int s = SG == 4 ? g * 4 + wave : g;
    if (run_first >= nruns) return;
    if constexpr (LBG) {
        if (__builtin_amdgcn_readfirstlane(a.done[s]) != 0) return;  // the block has converged
    }

    // the block's centroids: this wave's copy in LDS (no other wave reads it: no barrier)
    float *cl = lds_cb[wave];
    {
        const float4 *src = reinterpret_cast<const float4 *>(a.cb + (size_t)s * k * SD);
        float4 *dst = reinterpret_cast<float4 *>(cl);
        const int nv = 2 * k;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int i = lane + 64 * c;
            const float4 v = src[i < nv ? i : 0];
            if (i < nv) dst[i] = v;
        }
    }
    // the A operands of every block of 32 centroids
    u32x4 A1[8], A2[8];
    {
        const u32x4 *ap = tb.atab + (size_t)s * nb * 128 + lane;
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const int bc = b < nb ? b : 0;
            A1[b] = ap[(size_t)bc * 128];
            A2[b] = ap[(size_t)bc * 128 + 64];
        }
    }
    float muh[4];  // the centre's dimensions [4h, 4h + 4)
#pragma unroll
    for (int u = 0; u < 4; ++u) muh[u] = tb.mu[(size_t)s * 8 + 4 * h + u];
    const float mc2 = tb.maxc2[s];
    const uint32_t keep = opaque_vgpr(0xFFFFFF00u);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    uint32_t n_exact = 0;
    bool chg = false;
    // The workgroup walks over its runs of rows (run_first, run_first + run_stride, ...) with the
    // operands it has loaded: the grid is a few workgroups per compute unit, not one per run.
    for (int64_t run_id = run_first; run_id < nruns; run_id += run_stride) {
    const int64_t tile0 = SG == 4 ? run_id * run_tiles : (run_id * 4 + wave) * run_tiles;
    const int64_t row0 = tile0 * 32;
    if (row0 >= a.n) break;  // SG == 1: the last run may end before this wave's share
    const int64_t left = (a.n - row0 + 31) / 32;
    const int ntiles = (int)(left < run_tiles ? left : run_tiles);
    // rows two tiles ahead.  Addresses are a scalar base (the run's first row) plus a 32-bit lane
    // offset that moves on by 32 rows per tile (the host keeps the run's extent below 2^31 bytes).
    const float *xrun = a.x + row0 * a.ld + (int64_t)s * SD;          // uniform
    const uint8_t *crun = a.codes + (size_t)s * a.n + row0;           // uniform (LBG: [m][n] codes)
    const int64_t lane_rows = a.n - (row0 + r);                       // rows from this lane's first to the end
    const int64_t lane_left = lane_rows > 0 ? (lane_rows + 31) / 32 : 0;
    // tiles of this run in which the lane has a row; the fetches past the run's end read the run's
    // first row (the next run belongs to a workgroup on another XCD: its rows would be fetched into two L2s)
    const int lane_tiles = (int)(lane_left < run_tiles ? lane_left : run_tiles);
    const uint32_t xstep = 128u * (uint32_t)a.ld;                                          // bytes per tile
    uint32_t xoff = 4u * ((uint32_t)r * (uint32_t)a.ld + 4u * (uint32_t)h), coff = (uint32_t)r;  // of the lane's row in tile 0
    // rows may start at any float (any leading dimension): a 16-byte load that only claims 4-byte alignment
    typedef float rowpiece __attribute__((ext_vector_type(4), aligned(4)));
    auto fetch_x = [&](int t) {
        const char *p = reinterpret_cast<const char *>(xrun) + (t < lane_tiles ? xoff : 16u * (uint32_t)h);
        const rowpiece v = *reinterpret_cast<const rowpiece *>(p);
        return make_float4(v[0], v[1], v[2], v[3]);
    };
    auto fetch_c = [&](int t) { return crun[t < lane_tiles ? coff : 0u]; };
    float4 xa = fetch_x(0);
    uint8_t oa = 0, ob = 0;
    if constexpr (LBG) oa = fetch_c(0);
    xoff += xstep;
    coff += 32;
    float4 xb = fetch_x(1);
    if constexpr (LBG) ob = fetch_c(1);
    for (int t = 0; t < ntiles; ++t) {
        const float4 xc = xa;
        const uint8_t old = oa;
        xa = xb;
        oa = ob;
        xoff += xstep;
        coff += 32;
        xb = fetch_x(t + 2);
        if constexpr (LBG) ob = fetch_c(t + 2);
        const float xraw[4] = {xc.x, xc.y, xc.z, xc.w};
        u32x4 b1, b2;
        float x2;
        {
            float xv[4];  // relative to the block's centre
#pragma unroll
            for (int u = 0; u < 4; ++u) xv[u] = xraw[u] - muh[u];
            float p = 0.0f;
#pragma unroll
            for (int u = 0; u < 4; ++u) p = __builtin_fmaf(xv[u], xv[u], p);
            const uint32_t h01 = bf16_pack2(xv[0], xv[1]), h23 = bf16_pack2(xv[2], xv[3]);
            const uint32_t l01 = bf16_pack2(xv[0] - __uint_as_float(h01 << 16), xv[1] - __uint_as_float(h01 & 0xffff0000u));
            const uint32_t l23 = bf16_pack2(xv[2] - __uint_as_float(h23 << 16), xv[3] - __uint_as_float(h23 & 0xffff0000u));
            // this half's share of ||x||^2 as one bf16 number rounded up (p >= 0; the same in every score
            // of the row, so its rounding cancels in their differences, and rounding up keeps the
            // scores from turning negative), then ones for the parts of ||c||^2
            const uint32_t p0 = (__float_as_uint(p) + 0xFFFFu) >> 16;
            b1 = u32x4{h01, h23, l01, l23};
            b2 = u32x4{h01, h23, p0, 0x3f803f80u};
            int pa, pb;
            swap_halves(__float_as_int(p), pa, pb);
            x2 = __int_as_float(pa) + __int_as_float(pb);  // lower half's share + upper half's, in both
        }
        int m1 = 0x7f800000, m2 = 0x7f800000;  // +inf
        // One block of 32 centroids.  The tag leaves out the lane half (bit 2), so it is the same in
        // every lane and lives in scalar registers.
        // The scores of block b + 1 are made while block b's go through the selection: a matrix
        // instruction holds back the vector instructions of OTHER waves of its SIMD for as long as it
        // runs, but independent vector instructions of its own wave issue in its shadow, so every
        // matrix instruction is followed by half a block's selection from the same wave.
#define VQ_MFMA_1(b, acc)                                                                                       \
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, A1[b]),                            \
                                                  __builtin_bit_cast(bf16x8, b1), zero, 0, 0, 0);
#define VQ_MFMA_2(b, acc)                                                                                       \
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, A2[b]),                            \
                                                  __builtin_bit_cast(bf16x8, b2), acc, 0, 0, 0);
#define VQ_RUN_KEY(b, acc, p)                                                                                   \
    {                                                                                                           \
        const int gmin = imin(imin(imin(__float_as_int(acc[4 * p]), __float_as_int(acc[4 * p + 1])),            \
                                   __float_as_int(acc[4 * p + 2])),                                             \
                              __float_as_int(acc[4 * p + 3]));                                                  \
        key[p] = (int)(((uint32_t)gmin & keep) | (uint32_t)(32 * (b) + 8 * p));                                 \
    }
        // selection of block b (scores in cur) with the matrix instructions of block nb (into nxt) in between
#define VQ_SCORE_BLOCK(b, cur, nb, nxt, more)                                                                   \
    {                                                                                                           \
        int key[4];                                                                                             \
        if (more) { VQ_MFMA_1(nb, nxt) }                                                                        \
        __builtin_amdgcn_sched_barrier(0);                                                                      \
        VQ_RUN_KEY(b, cur, 0) VQ_RUN_KEY(b, cur, 1)                                                             \
        __builtin_amdgcn_sched_barrier(0);                                                                      \
        if (more) { VQ_MFMA_2(nb, nxt) }                                                                        \
        __builtin_amdgcn_sched_barrier(0);                                                                      \
        VQ_RUN_KEY(b, cur, 2) VQ_RUN_KEY(b, cur, 3)                                                             \
        top2_push4(m1, m2, key[0], key[1], key[2], key[3]);                                                     \
        __builtin_amdgcn_sched_barrier(0);                                                                      \
    }
        const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        floatx16 accA, accB;
        VQ_MFMA_1(0, accA)
        VQ_MFMA_2(0, accA)
        if constexpr (FULL) {
            VQ_SCORE_BLOCK(0, accA, 1, accB, true) VQ_SCORE_BLOCK(1, accB, 2, accA, true)
            VQ_SCORE_BLOCK(2, accA, 3, accB, true) VQ_SCORE_BLOCK(3, accB, 4, accA, true)
            VQ_SCORE_BLOCK(4, accA, 5, accB, true) VQ_SCORE_BLOCK(5, accB, 6, accA, true)
            VQ_SCORE_BLOCK(6, accA, 7, accB, true) VQ_SCORE_BLOCK(7, accB, 0, accA, false)
        } else {
            VQ_SCORE_BLOCK(0, accA, 1, accB, true)
            if (nb > 2) {
                VQ_SCORE_BLOCK(1, accB, 2, accA, true) VQ_SCORE_BLOCK(2, accA, 3, accB, true)
                if (nb > 4) {
                    VQ_SCORE_BLOCK(3, accB, 4, accA, true) VQ_SCORE_BLOCK(4, accA, 5, accB, true)
                    if (nb > 6) {
                        VQ_SCORE_BLOCK(5, accB, 6, accA, true) VQ_SCORE_BLOCK(6, accA, 7, accB, true)
                        VQ_SCORE_BLOCK(7, accB, 0, accA, false)
                    } else {
                        VQ_SCORE_BLOCK(5, accB, 0, accA, false)
                    }
                } else {
                    VQ_SCORE_BLOCK(3, accB, 0, accA, false)
                }
            } else {
                VQ_SCORE_BLOCK(1, accB, 0, accA, false)
            }
        }
#undef VQ_MFMA_1
#undef VQ_MFMA_2
#undef VQ_RUN_KEY
#undef VQ_SCORE_BLOCK
        // the partner lane (other half) saw the other 16 centroids of every block
        m1 |= 4 * h;  // bit 2 of the centroid index: the lane half
        m2 |= 4 * h;
        int f1, g1, f2, g2;
        swap_halves(m1, f1, g1);
        swap_halves(m2, f2, g2);
        const float s1 = __int_as_float(imin(f1, g1));
        const float s2 = __int_as_float(imin(imax(f1, g1), imin(f2, g2)));
        const bool mine = h == 0 && t < lane_tiles;  // the lane's row of this tile exists
        const float bound = x2 + mc2;
        const float margin = 6.103515625e-05f * fabsf(s2) + 1.220703125e-04f * bound;
        bool sure = (s2 - s1) > margin;  // false for NaN / inf-inf
        // below 1e-31 the bf16 parts of ||c - mu||^2 may be subnormal, which the matrix cores may
        // flush: up to 3 * 2^-126 lost, more than the margin allows for at such a bound
        sure = sure && (bound < 1e29f) && (bound > 1e-31f) && (s1 < 1e29f);
        const int first = (int)(__float_as_uint(s1) & 0xFFu);  // first centroid of the best run
        const unsigned long long todo = __ballot(mine && !sure);
        int code;
        float dist;  // of the chosen centroid, as the reference computes it
        {
            // the best run's four centroids, two per lane half, in the reference's order
            const int j0 = first + 2 * h;
            const int ja = j0 < k ? j0 : k - 1, jb = j0 + 1 < k ? j0 + 1 : k - 1;
            const float4 *pa = reinterpret_cast<const float4 *>(cl + ja * SD);
            const float4 *pb = reinterpret_cast<const float4 *>(cl + jb * SD);
            const float4 ca0 = pa[0], ca1 = pa[1], cb0 = pb[0], cb1 = pb[1];
            float xs[8];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                int lo, hi;
                swap_halves(__float_as_int(xraw[u]), lo, hi);
                xs[u] = __int_as_float(lo);
                xs[4 + u] = __int_as_float(hi);
            }
            const float ca[8] = {ca0.x, ca0.y, ca0.z, ca0.w, ca1.x, ca1.y, ca1.z, ca1.w};
            const float cc[8] = {cb0.x, cb0.y, cb0.z, cb0.w, cb1.x, cb1.y, cb1.z, cb1.w};
            float da = d_sq<8>(xs, ca), db = d_sq<8>(xs, cc);
            if constexpr (METRIC == M_EUCLID) {
                da = sqrtf(da);
                db = sqrtf(db);
            }
            const bool second = (j0 + 1 < k) && (db < da);  // strict: the first of equals
            uint32_t kd = __float_as_uint(second ? db : da);
            const uint32_t ki = (uint32_t)(second ? j0 + 1 : j0);
            kd = j0 < k ? kd : 0x7f800000u;  // a padding centroid
            int dlo, dhi, ilo, ihi;
            swap_halves((int)kd, dlo, dhi);
            swap_halves((int)ki, ilo, ihi);
            code = (uint32_t)dhi < (uint32_t)dlo ? ihi : ilo;  // the lower half holds the lower indices
            dist = __uint_as_float((uint32_t)dhi < (uint32_t)dlo ? (uint32_t)dhi : (uint32_t)dlo);
        }
        if (todo) {  // the same in every lane: the reference-order argmin of the undecided rows
            n_exact += (uint32_t)__popcll(todo);
            code = exact_rows8<METRIC>(todo, code, dist, cl, a.x + (row0 + 32 * (int64_t)t) * a.ld + (int64_t)s * SD, a.ld,
                                           k, lane);
        }
        if (mine) {
            const uint32_t rr = 32u * (uint32_t)t + (uint32_t)r;  // row within the run
            if constexpr (LBG) {
                if (old != (uint8_t)code) {
                    a.codes[(size_t)s * a.n + row0 + rr] = (uint8_t)code;
                    chg = true;
                }
            } else {
                const size_t out0 = (size_t)row0 * m + s;  // uniform
                a.codes[out0 + rr * (uint32_t)m] = (uint8_t)code;
                if (a.dist) a.dist[out0 + rr * (uint32_t)m] = dist;  // for the caller that merges chunks of a larger codebook
            }
        }
    }
    }  // runs
    if constexpr (LBG) {
        // changed[s]: one lane per wave, once per wave, and only where the flag still reads 0 (every
        // store to one address is serialised in its L2 channel; a stale 0 from the vector cache
        // costs a store, nothing else).
        if (__any(chg) && lane == 0 && a.changed[s] == 0) a.changed[s] = 1;
    }
    if (lane == 0 && n_exact)
        atomicAdd(tb.stat + ((run_first * 4 + wave) & (kStatSlots - 1)) * kStatStride, n_exact);
}

}  // namespace vq

// =============================================================================================
// Wide column blocks (sub_dim a multiple of 8, up to the full dimension: RVQ stages).
namespace vq {

// ---------------------------------------------------------------------------------------------
// Wide column blocks on the bf16 matrix cores: the operand split of k_assign_mfma_bf applied to
// 16 dimensions at a time.  With the high and low bf16 parts of the centroid operand (ah, al) and
// of the row operand (xh, xl), a tile of 32 rows x 32 centroids takes three instructions per 16
// dimensions, ah.xh + al.xh + ah.xl, each with all 16 contraction slots in use (each lane half
// owns 8 of the 16 dimensions).  An earlier shape worked on 8 dimensions with two instructions,
// {ah, al}.{xh, xh} and {ah, al}.{xl, 0}: a quarter of the slots multiplied zeros.
// A workgroup = 128 rows; a wave takes one tile of 32 rows against every tile of 32 centroids: 8
// accumulator tiles (128 registers) that start at ||c - mu||^2.  The centroid operands of a tile
// are the 16 bytes of ah and the 16 bytes of al as they lie in LDS, and the row is split once per
// 16 dimensions for 3 NB matrix instructions, so no operand is assembled in registers (vector
// and matrix instructions take turns on a SIMD).  ||x - mu||^2 is summed on the vector ALU and
// added to the scores before the selection.  The A operands of 16 dimensions (16 KB for 256
// centroids) are staged in LDS once per workgroup, double-buffered; the next A operands are
// fetched one stage ahead, the row two.
// Error of a score: 3 * 2^-16 (split, as above) + (34 * sd/8 + 16) * 2^-24 (fp32 accumulation, an
// upper bound: at most 17 additions per instruction, 1.5 instructions per 8 dimensions, and the
// final sum) + 2^-22 (rounding of x - mu and c - mu), per unit of ||x - mu||^2 + ||c - mu||^2;
// twice that for two candidates.
constexpr int kWideCentreMax = 2048;  // widest column block whose centre is staged in LDS

struct MfmaWideBfTables {
    const u32x4 *atab;     // [m][ceil(sd/16)][nb][2][64]  ah, then al, of the lane's eight dimensions
    const float *c2perm;   // [m][nb][2][16]
    const float *blockmax; // [m][nb]  largest ||c - mu||^2 per block of 32 centroids (NaN if any is NaN)
    const float *mu;       // [m][sd]  centre of every column block: mean of its centroids
    const int *shifted;    // [m]  0: the centre is not used
    uint32_t *list;        // undecided pairs (row * m + s) for the exact kernel over all centroids
    uint32_t *list_count;  // [0] entries of list, [1] entries of pairs
    uint2 *pairs;          // undecided pairs with only two candidates: {row * m + s, c1 | c2 << 8}
    int nb;
    int sd;
    float kappa;           // error-bound coefficient on (||x||^2 + max ||c||^2)
};

// One workgroup per (column block s, block b of 32 centroids): thread (i, g) = (tid % 32, tid / 32)
// writes the chunks kc = g, g + 8, ... of centroid 32 b + i and sums their share of ||c||^2; the
// eight shares are added in g order.  blockmax[s][b] = largest ||c||^2 of the block (NaN stays).
// mu[s][t] = mean over the k <= 256 centroids of column block s (sum of c / 256, then * 256 / k:
// no overflow).  Rows and centroids are scored relative to it, as in k_mfma_bf_prep, when that
// shrinks the norms the error bound is proportional to: k_mfma_wide_bf_prep sets shifted[s] = 0
// and ignores the centre if ||mu||^2 is no more than a quarter of the mean ||c||^2 (or the block
// is wider than kWideCentreMax), and the assignment kernel then skips the subtraction.  Grid (m, ceil(sd / 32)); thread (i, g) =
// (tid % 32, tid / 32) adds the centroids g, g + 8, ... of dimension 32 y + i; norms[s][y] =
// this slice's share of {||mu||^2, mean ||c||^2}.
static __global__ void __launch_bounds__(256) k_block_centres(const float *__restrict__ cb, int k, int sd,
                                                              float *__restrict__ mu, float2 *__restrict__ norms) {
    const int s = blockIdx.x, y = blockIdx.y;
    const int i = threadIdx.x & 31, g = threadIdx.x >> 5;
    const int t = 32 * y + i;
    __shared__ float part[2][8][32];
    float acc = 0.0f, sq = 0.0f;
    if (t < sd) {
        const float *c = cb + (size_t)s * k * sd + t;
        float v[32];  // k <= 256: all of the thread's loads are in flight together
#pragma unroll
        for (int u = 0; u < 32; ++u) {
            const int j = g + 8 * u;
            v[u] = c[(size_t)(j < k ? j : 0) * sd];
        }
#pragma unroll
        for (int u = 0; u < 32; ++u) {
            const float w = (g + 8 * u < k) ? v[u] * 0.00390625f : 0.0f;
            acc += w;
            sq = __builtin_fmaf(w, w, sq);
        }
    }
    part[0][g][i] = acc;
    part[1][g][i] = sq;
    __syncthreads();
    if (g == 0) {
        float a = 0.0f, q = 0.0f;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            a += part[0][u][i];
            q += part[1][u][i];
        }
        const float ctr = a * (256.0f / (float)k);
        if (t < sd) mu[(size_t)s * sd + t] = ctr;
        float mm = (t < sd) ? ctr * ctr : 0.0f, cc = q * (65536.0f / (float)k);
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) {
            mm += __shfl_xor(mm, off);
            cc += __shfl_xor(cc, off);
        }
        if (i == 0) norms[(size_t)s * gridDim.y + y] = make_float2(mm, cc);
    }
}

static __global__ void __launch_bounds__(256) k_mfma_wide_bf_prep(const float *__restrict__ cb,
                                                                  const float *__restrict__ mu,
                                                                  const float2 *__restrict__ norms,
                                                                  int *__restrict__ shifted, int m, int k, int nb,
                                                                  int sd, u32x4 *__restrict__ atab,
                                                                  float *__restrict__ c2perm,
                                                                  float *__restrict__ blockmax,
                                                                  uint32_t *__restrict__ list_count) {
    const int s = blockIdx.x, b = blockIdx.y;
    const int i = threadIdx.x & 31, g = threadIdx.x >> 5;
    const int j = b * 32 + i;
    const int npair = (sd + 15) / 16;
    __shared__ float part[8][32];
    // the same decision in every workgroup of the column block (same values, same order)
    float mm = 0.0f, cc = 0.0f;
    for (int y = 0; y < (sd + 31) / 32; ++y) {
        const float2 v = norms[(size_t)s * ((sd + 31) / 32) + y];
        mm += v.x;
        cc += v.y;
    }
    const bool on = mm > 0.25f * cc && mm < 1e30f && sd <= kWideCentreMax;  // false for NaN
    if (b == 0 && threadIdx.x == 0) shifted[s] = on ? 1 : 0;
    const float *c = cb + ((size_t)s * k + (j < k ? j : 0)) * sd;
    float p = 0.0f;
    for (int pr = g; pr < npair; pr += 8) {
        // lane i + 32 h holds the dimensions 16 pr + 8 h .. + 7 (zeros past the block's width): 16
        // bytes of high parts, then, 64 entries on, 16 bytes of low parts, each the operand of a
        // matrix instruction as it lies in LDS
        u32x4 *dst = atab + (((size_t)s * npair + pr) * nb + b) * 128;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int d0 = 16 * pr + 8 * h;
            const bool in = d0 < sd;  // sd is a multiple of 8
            const int dc = in ? d0 : 0;
            const float4 v0 = *reinterpret_cast<const float4 *>(c + dc);
            const float4 v1 = *reinterpret_cast<const float4 *>(c + dc + 4);
            float4 u0 = make_float4(0.f, 0.f, 0.f, 0.f), u1 = u0;
            if (on) {
                u0 = *reinterpret_cast<const float4 *>(mu + (size_t)s * sd + dc);
                u1 = *reinterpret_cast<const float4 *>(mu + (size_t)s * sd + dc + 4);
            }
            float cv[8] = {v0.x - u0.x, v0.y - u0.y, v0.z - u0.z, v0.w - u0.w,
                           v1.x - u1.x, v1.y - u1.y, v1.z - u1.z, v1.w - u1.w};
            uint32_t hw[4], lw[4];  // packed pairs of the high and low parts
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                uint32_t hb[2], lb[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float x = in ? cv[2 * w + e] : 0.0f;
                    p = __builtin_fmaf(x, x, p);
                    const float a = (j < k) ? -2.0f * x : 0.0f;
                    hb[e] = bf16_rne_bits(a);
                    lb[e] = bf16_rne_bits(a - bf16_bits_to_float(hb[e]));
                }
                hw[w] = hb[0] | (hb[1] << 16);
                lw[w] = lb[0] | (lb[1] << 16);
            }
            dst[32 * h + i] = u32x4{hw[0], hw[1], hw[2], hw[3]};
            dst[64 + 32 * h + i] = u32x4{lw[0], lw[1], lw[2], lw[3]};
        }
    }
    part[g][i] = p;
    __syncthreads();
    if (g == 0) {
        float c2 = 0.0f;
#pragma unroll
        for (int q = 0; q < 8; ++q) c2 = c2 + part[q][i];
        float mx = c2;
        if (j >= k) {
            c2 = kPadScore;
            mx = 0.0f;
        }
        const int hh = (i / 4) % 2, v = (i / 8) * 4 + i % 4;
        c2perm[(((size_t)s * nb + b) * 2 + hh) * 16 + v] = c2;
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) {
            const float o = __shfl_xor(mx, off);
            mx = (mx == mx && o == o) ? fmaxf(mx, o) : __builtin_nanf("");
        }
        if (i == 0) blockmax[(size_t)s * nb + b] = mx;
        if (s == 0 && b == 0 && i < 2) list_count[i] = 0;
    }
}

// LDS writes of this wave done, then the workgroup barrier; vector-memory loads stay in flight
// (__syncthreads would wait for the prefetches as well).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// grid (ceil(n/128), m); 256 threads = 4 waves, one tile of 32 rows each against every centroid.
// NB = tiles of 32 centroids (tb.nb), a template parameter so that the chains of matrix
// instructions are straight-line code.
// PEND (one column block): the rows are a residual whose update by the previous stage's codebook is
// still pending, x[i] -= pend_cb[pend_codes[i]] (src/rvq.rs:124-129 in a fit, 200-202 in an encode).
// A workgroup first updates its own 128 rows — whole rows per wave instruction, one f32 subtraction
// per element, as the separate pass would; in place, or from the rows of a.pend_src into a.x — and
// then scores them as any other rows, which it now reads from the cache levels it has just written
// through.  No other workgroup reads or writes these rows.
template <bool LBG, int NB, bool PEND = false>
__global__ void __launch_bounds__(256, 2) k_assign_mfma_wide_bf(AssignArgs a, MfmaWideBfTables tb) {
    constexpr int NBMAX = 8;
    __shared__ u32x4 lds_a[2][NBMAX * 128];  // 2 stages x 16 dimensions x 256 centroids x {high, low}: 2 x 16 KB
    __shared__ float lds_c2[NBMAX * 32];
    __shared__ float lds_mu[kWideCentreMax];
    __shared__ uint32_t wg_list[128];
    __shared__ uint2 wg_pairs[128];
    __shared__ uint32_t wg_count, wg_base, wg_pcount, wg_pbase;
    const int s = blockIdx.y;
    if constexpr (LBG) {
        if (a.done[s]) return;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    constexpr int nb = NB;
    const int sd = tb.sd, npair = (sd + 15) / 16;
    const u32x4 *ag = tb.atab + (size_t)s * npair * nb * 128;
    const int pair16 = nb * 128;  // 16-byte pieces per 16 dimensions
    for (int i = threadIdx.x; i < nb * 32; i += 256) lds_c2[i] = tb.c2perm[(size_t)s * nb * 32 + i];
    for (int i = threadIdx.x; i < pair16; i += 256) lds_a[0][i] = ag[i];
    if (threadIdx.x == 0) {
        wg_count = 0;
        wg_pcount = 0;
    }
    if (tb.shifted[s] != 0)
        for (int i = threadIdx.x; i < sd; i += 256) lds_mu[i] = tb.mu[(size_t)s * sd + i];
    if constexpr (PEND) {
        const int64_t row0 = (int64_t)blockIdx.x * 128;
        const int nrows = a.n - row0 < 128 ? (int)(a.n - row0) : 128;
        float *xw = const_cast<float *>(a.x) + row0 * a.ld;
        const float *xr = a.pend_src ? a.pend_src + row0 * a.pend_src_ld : xw;
        const int64_t xr_ld = a.pend_src ? a.pend_src_ld : a.ld;
        const uint8_t *pc = a.pend_codes + row0;
        const int per_row = sd / 4, total = nrows * per_row;  // 16-byte pieces
        constexpr int B = 8;  // pieces of a thread in flight together
        for (int i0 = threadIdx.x; i0 < total; i0 += 256 * B) {
            float4 v[B], c[B];
#pragma unroll
            for (int u = 0; u < B; ++u) {
                const int i = i0 + 256 * u < total ? i0 + 256 * u : i0;
                const int rr = i / per_row, cc = i - rr * per_row;
                v[u] = *reinterpret_cast<const float4 *>(xr + (int64_t)rr * xr_ld + 4 * cc);
                c[u] = *reinterpret_cast<const float4 *>(a.pend_cb + (size_t)pc[rr] * sd + 4 * cc);
            }
#pragma unroll
            for (int u = 0; u < B; ++u) {
                const int i = i0 + 256 * u;
                if (i < total) {
                    const int rr = i / per_row, cc = i - rr * per_row;
                    *reinterpret_cast<float4 *>(xw + (int64_t)rr * a.ld + 4 * cc) =
                        make_float4(v[u].x - c[u].x, v[u].y - c[u].y, v[u].z - c[u].z, v[u].w - c[u].w);
                }
            }
        }
    }
    __syncthreads();  // (PEND: the updated rows are visible to every wave of the workgroup)

    const int64_t row = (int64_t)blockIdx.x * 128 + wave * 32 + r;
    const bool valid = row < a.n;
    // the workgroup's first row is a scalar base, the lane's row a 32-bit byte offset from it (the
    // host keeps 128 rows below 2^31 bytes); a row past the end reads the workgroup's first row
    const char *xwg = reinterpret_cast<const char *>(a.x + (int64_t)blockIdx.x * 128 * a.ld + (int64_t)s * sd);
    const uint32_t xlane = valid ? 4u * (uint32_t)(wave * 32 + r) * (uint32_t)a.ld : 0u;
    auto row_piece = [&](int d) { return *reinterpret_cast<const float4 *>(xwg + (xlane + 4u * (uint32_t)d)); };
    const bool shifted = tb.shifted[s] != 0;  // uniform
    // the accumulators start at ||c - mu||^2; ||x - mu||^2, the same in every score of a row, is
    // summed on the side and added before the selection
    floatx16 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[b][v] = lds_c2[(b * 2 + h) * 16 + v];
    // Loads are unconditional (a row past the end reads row 0 and is never stored; pieces past
    // the block's width are clamped and zeroed): loads under a branch make the compiler wait for
    // every outstanding load at each use instead of counting them.
    // This half's 8 of the 16 dimensions of a stage: 16 pr + 8 h .. + 7.
    auto piece = [&](int pr) { return 16 * pr + 8 * h < sd ? 16 * pr + 8 * h : 0; };
    float4 xn0 = row_piece(piece(0));  // the next piece of the row
    float4 xn1 = row_piece(piece(0) + 4);
    const int second = npair > 1 ? 1 : 0;
    float4 xf0 = row_piece(piece(second));  // and the one after it
    float4 xf1 = row_piece(piece(second) + 4);
    float x2 = 0.0f;
    // The row operands of a stage: this half's 8 dimensions relative to the centre, their share of
    // ||x - mu||^2, and their high and low bf16 parts.
    auto split = [&](int st, const float4 &p0, const float4 &p1, u32x4 &bh, u32x4 &bl) {
        float xv[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
        if (shifted) {
            const float4 m0 = *reinterpret_cast<const float4 *>(lds_mu + piece(st));
            const float4 m1 = *reinterpret_cast<const float4 *>(lds_mu + piece(st) + 4);
            xv[0] -= m0.x;
            xv[1] -= m0.y;
            xv[2] -= m0.z;
            xv[3] -= m0.w;
            xv[4] -= m1.x;
            xv[5] -= m1.y;
            xv[6] -= m1.z;
            xv[7] -= m1.w;
        }
        if (st == npair - 1 && (sd & 8) != 0) {  // uniform: a width that is an odd multiple of 8 ends in the lower half
            if (h != 0) {
#pragma unroll
                for (int u = 0; u < 8; ++u) xv[u] = 0.0f;
            }
        }
        uint32_t hp[4], lp[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            x2 = __builtin_fmaf(xv[2 * u], xv[2 * u], x2);
            x2 = __builtin_fmaf(xv[2 * u + 1], xv[2 * u + 1], x2);
            hp[u] = bf16_pack2(xv[2 * u], xv[2 * u + 1]);
            lp[u] = bf16_pack2(xv[2 * u] - __uint_as_float(hp[u] << 16), xv[2 * u + 1] - __uint_as_float(hp[u] & 0xffff0000u));
        }
        bh = u32x4{hp[0], hp[1], hp[2], hp[3]};
        bl = u32x4{lp[0], lp[1], lp[2], lp[3]};
    };
    // A stage is 16 dimensions: with the high and low parts of the centroid operand (ah, al) and of
    // the row operand (xh, xl), three matrix instructions per tile of 32 centroids,
    //   ah . xh + al . xh + ah . xl,
    // every contraction slot of each in use; one barrier per 3 NB matrix instructions of a wave.
    // The row operands of stage st + 1 are made while the matrix instructions of stage st run: a
    // matrix instruction holds back the vector instructions of the other waves of its SIMD, but
    // independent vector instructions of its own wave issue in its shadow.
    const int total16 = npair * pair16;
    u32x4 bh, bl;
    split(0, xn0, xn1, bh, bl);
    xn0 = xf0;
    xn1 = xf1;
    {
        const int nx = 2 < npair ? 2 : npair - 1;
        xf0 = row_piece(piece(nx));
        xf1 = row_piece(piece(nx) + 4);
    }
    for (int st = 0; st < npair; ++st) {
        const int cur = st & 1;
        const bool more = st + 1 < npair;
        // the A operands of the next stage: into registers now, into LDS at the end of this stage
        u32x4 pre[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t i = (uint32_t)((st + 1) * pair16) + threadIdx.x + 256u * (uint32_t)q;
            const uint32_t ic = i < (uint32_t)total16 ? i : (uint32_t)total16 - 1u;
            pre[q] = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const char *>(ag) + 16u * ic);
        }
        // The stage's centroid operands are read from LDS four tiles (one group) at a time.
        constexpr int NG = (NB + 3) / 4;  // groups of four centroid tiles
        u32x4 nbh = bh, nbl = bl;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            u32x4 ah[4], al[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int b = 4 * g + c < nb ? 4 * g + c : nb - 1;  // past the last block: read it, not multiplied
                ah[c] = lds_a[cur][b * 128 + lane];
                al[c] = lds_a[cur][b * 128 + 64 + lane];
            }
            // the three dependent instructions of a tile are three others apart
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (4 * g + c < nb)
                    acc[4 * g + c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8, ah[c]), __builtin_bit_cast(bf16x8, bh), acc[4 * g + c], 0, 0, 0);
            if (g == 0 && more) {
                // next stage's row operands, behind the first matrix instructions of this stage
                split(st + 1, xn0, xn1, nbh, nbl);
                const int nx = st + 3 < npair ? st + 3 : npair - 1;
                xn0 = xf0;
                xn1 = xf1;
                xf0 = row_piece(piece(nx));
                xf1 = row_piece(piece(nx) + 4);
            }
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (4 * g + c < nb)
                    acc[4 * g + c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8, al[c]), __builtin_bit_cast(bf16x8, bh), acc[4 * g + c], 0, 0, 0);
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (4 * g + c < nb)
                    acc[4 * g + c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8, ah[c]), __builtin_bit_cast(bf16x8, bl), acc[4 * g + c], 0, 0, 0);
        }
        bh = nbh;
        bl = nbl;
        if (more) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int i = threadIdx.x + 256 * q;
                if (i < pair16) lds_a[cur ^ 1][i] = pre[q];
            }
        }
        lds_barrier();
    }
    x2 += __shfl_xor(x2, 32);  // both halves' shares of ||x - mu||^2
    // the three smallest scores of the row, the index in the low 8 bits (one v_and_or per score; the
    // tag leaves out the lane half, bit 2, so it is the same in every lane: a scalar operand)
    int m1 = 0x7f800000, m2 = 0x7f800000, m3 = 0x7f800000;
    const uint32_t keep = opaque_vgpr(0xFFFFFF00u);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
        for (int v = 0; v < 16; v += 4) {
            int key[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                key[u] = pack_tag(acc[b][v + u] + x2, keep, (uint32_t)(32 * b + 8 * (v / 4) + u));
            top3_push4(m1, m2, m3, key[0], key[1], key[2], key[3]);
        }
    }
    {
        m1 |= 4 * h;
        m2 |= 4 * h;
        const int o1 = __shfl_xor(m1, 32), o2 = __shfl_xor(m2, 32), o3 = __shfl_xor(m3, 32);
        top3_push4(m1, m2, m3, o1, o2, o3, 0x7f800000);
    }
    const uint32_t i1 = (uint32_t)m1 & 0xFFu, i2 = (uint32_t)m2 & 0xFFu;
    if (h == 0) {
        float mc2 = 0.0f;  // largest ||c||^2 of the column block; a NaN stays
        for (int b = 0; b < nb; ++b) {
            const float o = tb.blockmax[(size_t)s * nb + b];
            mc2 = (mc2 == mc2 && o == o) ? fmaxf(mc2, o) : __builtin_nanf("");
        }
        const float s1 = __int_as_float(m1), s2 = __int_as_float(m2), s3 = __int_as_float(m3);
        if (valid) {
            const float bound = x2 + mc2;
            const bool finite = (bound < 1e29f) && (s1 < 1e29f);  // false for NaN
            const float slack = tb.kappa * bound;
            // the smallest exact distance is the best-scored centroid's when the second score is
            // further away than the error bound ...
            const bool sure = finite && (s2 - s1) > 6.103515625e-05f * fabsf(s2) + slack;
            // ... and one of the two best-scored centroids' when the third score is
            const bool two = finite && (s2 < 1e29f) && (s3 - s1) > 6.103515625e-05f * fabsf(s3) + slack;
            if (sure) {
                const uint8_t code = (uint8_t)i1;
                if constexpr (LBG) {
                    uint8_t *pc = a.codes + (size_t)s * a.n + row;
                    if (*pc != code) {
                        *pc = code;
                        mark_changed(a.changed + s);
                    }
                } else {
                    a.codes[row * a.m + s] = code;
                }
            } else if (two) {
                wg_pairs[atomicAdd(&wg_pcount, 1u)] = make_uint2((uint32_t)(row * a.m + s), i1 | (i2 << 8));
            } else {
                wg_list[atomicAdd(&wg_count, 1u)] = (uint32_t)(row * a.m + s);
            }
        }
    }
    __syncthreads();
    const uint32_t cnt = wg_count, pcnt = wg_pcount;
    if (cnt == 0 && pcnt == 0) return;
    if (threadIdx.x == 0) {
        if (cnt) wg_base = atomicAdd(tb.list_count, cnt);
        if (pcnt) wg_pbase = atomicAdd(tb.list_count + 1, pcnt);
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < cnt; i += 256) tb.list[wg_base + i] = wg_list[i];
    for (uint32_t i = threadIdx.x; i < pcnt; i += 256) tb.pairs[wg_pbase + i] = wg_pairs[i];
}

}  // namespace vq
