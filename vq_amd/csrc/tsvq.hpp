// Tree-structured VQ: node statistics for the build (src/tsvq.rs:71-148) and the descent
// encode (src/tsvq.rs:162-181).
//
// Build, one tree level at a time.  `perm` lists row ids so that the rows of every node of the
// level are contiguous and in original row order (the reference's partition is stable).
//   mean      mean_vector over the node's rows: sequential up to 1024 rows, the fixed midpoint
//             tree above (same order as the LBG update)
//   variance  per dimension, sum over the node's rows IN ROW ORDER of (x - mean)^2, f32
//             (Iterator::sum is sequential, src/tsvq.rs:88-99) — one lane per (node, dimension)
//   median    of the split column by a segmented sort (host picks the middle values)
//   partition stable, by `x[split] <= median`
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vq {

// One lane per (leaf, component): sequential sum over perm[lo, hi).
static __global__ void __launch_bounds__(256) k_seg_leafsum(const uint32_t *__restrict__ perm,
                                                     const uint2 *__restrict__ desc, int64_t nleaves,
                                                     const float *__restrict__ x, int64_t ld, int sd,
                                                     float *__restrict__ leaf_sum) {
    int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t leaf = gid / sd;
    int t = (int)(gid % sd);
    if (leaf >= nleaves) return;
    uint2 d = desc[leaf];
    const float *__restrict__ xc = x + t;
    float acc = 0.0f;
    // a leaf has up to 1024 rows and the lane adds them one after the other: 32 loads are in
    // flight per memory round trip (unconditional, clamped to the leaf's last row), the adds keep
    // their order
    uint32_t p = d.x;
    if (d.y > d.x) {
        const uint32_t last = d.y - 1;
        for (; p < d.y; p += 32) {
            uint32_t id[32];
            float v[32];
#pragma unroll
            for (int u = 0; u < 32; ++u) id[u] = perm[p + u <= last ? p + u : last];
#pragma unroll
            for (int u = 0; u < 32; ++u) v[u] = xc[(int64_t)id[u] * ld];
#pragma unroll
            for (int u = 0; u < 32; ++u)
                if (p + u <= last) acc = acc + v[u];
        }
    }
    leaf_sum[leaf * sd + t] = acc;
}

// One lane per (segment, component): combine 2^depth leaves left + right, divide by the count.
// seg_info[g] = {first leaf, depth, count, unused}
static __global__ void __launch_bounds__(256) k_seg_mean(float *__restrict__ leaf_sum,
                                                  const uint4 *__restrict__ seg_info, int nseg, int sd,
                                                  float *__restrict__ out, int64_t out_first) {
    int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int g = (int)(gid / sd);
    int t = (int)(gid % sd);
    if (g >= nseg) return;
    uint4 info = seg_info[g];
    uint32_t nl = 1u << info.y;
    float *ls = leaf_sum + (size_t)info.x * sd + t;
    // the pairs of one level of the tree are independent: eight of them per memory round trip
    // (clamped to the level's last pair); a lane only reads what it wrote itself
    for (uint32_t h = 1; h < nl; h <<= 1) {
        const uint32_t npairs = nl / (2 * h);
        for (uint32_t q0 = 0; q0 < npairs; q0 += 8) {
            float a[8], b[8];
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u) {
                const uint32_t qi = q0 + u < npairs ? q0 + u : npairs - 1;
                a[u] = ls[(size_t)(2 * h * qi) * sd];
                b[u] = ls[(size_t)(2 * h * qi + h) * sd];
            }
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u)
                if (q0 + u < npairs) ls[(size_t)(2 * h * (q0 + u)) * sd] = a[u] + b[u];
        }
    }
    out[(out_first + g) * sd + t] = ls[0] / __uint2float_rn(info.z);
}

// The same tree for the levels near the root, where a segment has hundreds of leaves and there are
// few segments: one workgroup per (segment, 8 components), the leaf sums in LDS, the pairs of a tree
// level side by side — the same additions as k_seg_mean, which walks them in one thread.
constexpr int kMeanWgLeaves = 1024;
static __global__ void __launch_bounds__(256) k_seg_mean_wg(const float *__restrict__ leaf_sum,
                                                            const uint4 *__restrict__ seg_info, int sd,
                                                            float *__restrict__ out, int64_t out_first) {
    __shared__ float tree[kMeanWgLeaves][8];
    const int g = blockIdx.x, t = threadIdx.x & 7, q = threadIdx.x >> 3;
    const int c = blockIdx.y * 8 + t;
    const uint4 info = seg_info[g];
    const uint32_t nl = 1u << info.y;  // <= kMeanWgLeaves (the host checks)
    const float *ls = leaf_sum + (size_t)info.x * sd + (c < sd ? c : 0);
    for (uint32_t leaf = q; leaf < nl; leaf += 32) tree[leaf][t] = ls[(size_t)leaf * sd];
    __syncthreads();
    for (uint32_t h = 1; h < nl; h <<= 1) {
        const uint32_t npairs = nl / (2 * h);
        for (uint32_t qi = q; qi < npairs; qi += 32) tree[2 * h * qi][t] = tree[2 * h * qi][t] + tree[2 * h * qi + h][t];
        __syncthreads();
    }
    if (q == 0 && c < sd) out[(out_first + g) * sd + c] = tree[0][t] / __uint2float_rn(info.z);
}

// One lane per (segment, dimension): sequential sum of squared deviations in row order.
// seg_range[g] = {lo, hi} positions in perm; mean of segment g at means[(first + g) * dim].
static __global__ void __launch_bounds__(64) k_seg_variance(const uint32_t *__restrict__ perm,
                                                     const uint2 *__restrict__ seg_range, int nseg,
                                                     const float *__restrict__ means, int64_t first,
                                                     const float *__restrict__ x, int64_t ld, int dim,
                                                     float *__restrict__ var) {
    int64_t gid = (int64_t)blockIdx.x * 64 + threadIdx.x;
    int g = (int)(gid / dim);
    int t = (int)(gid % dim);
    if (g >= nseg) return;
    uint2 r = seg_range[g];
    const float mu = means[(first + g) * dim + t];
    const float *__restrict__ xc = x + t;
    float acc = 0.0f;
    uint32_t p = r.x;
    for (; p + 16 <= r.y; p += 16) {
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) v[u] = xc[(int64_t)perm[p + u] * ld];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            float d = v[u] - mu;
            float q = d * d;
            acc = acc + q;
        }
    }
    for (; p < r.y; ++p) {
        float d = xc[(int64_t)perm[p] * ld] - mu;
        float q = d * d;
        acc = acc + q;
    }
    var[(size_t)g * dim + t] = acc;
}

// ---- per-dimension sums of squared deviations in two steps (dim a multiple of 8) --------------
// Step 1, on the whole GPU: sq = (x - mean)^2, the same two roundings as in the chain, stored so
// that 32 consecutive positions of a column sit side by side:
//   sq32[(lo_g + 32 g) * dim + ((p - lo_g) / 32) * 32 * dim + (c / 8) * 256 + (c % 8) * 32 + (p - lo_g) % 32]
// (every segment starts on its own group of 32 positions: n + 32 nseg rows of room).
// Grid (blocks of 64 positions, segments); one lane per (group of 32 positions, column).
constexpr int kChainGroup = 32;  // positions per group

// Index of a segment's first group in the per-group tables (group sums, binade guesses, maps):
// segment g's squares start at row range.x + 32 g of sq32, and the groups of different segments
// never share an index.
__device__ __forceinline__ size_t seg_group0(const uint2 range, int g) {
    return ((size_t)range.x + 32u * (size_t)g) / 32u;
}

static __global__ void __launch_bounds__(256) k_seg_sqdev32(const uint32_t *__restrict__ perm,
                                                            const uint2 *__restrict__ seg_range,
                                                            const float *__restrict__ means, int64_t first,
                                                            const float *__restrict__ x, int64_t ld, int dim,
                                                            float *__restrict__ sq32, float *__restrict__ gsum) {
    // sq32 == nullptr: only the group sums are wanted (the squares are made again where they are used)
    const int g = blockIdx.y;
    const uint2 range = seg_range[g];
    const uint32_t count = range.y - range.x;
    const uint32_t P0 = blockIdx.x * 2u;  // first group of this block
    if (P0 * 32u >= count) return;
    const uint32_t nP = (count + 31u) / 32u;
    const uint32_t groups = nP - P0 < 2u ? nP - P0 : 2u;
    const float *mrow = means + (first + g) * dim;
    float *out = sq32 + ((size_t)range.x + 32u * (size_t)g) * dim;
    const uint32_t *pm = perm + range.x;
    for (uint32_t e = threadIdx.x; e < groups * (uint32_t)dim; e += 256) {
        const uint32_t P = P0 + e / (uint32_t)dim, c = e % (uint32_t)dim;
        const float m = mrow[c];
        float4 *o = reinterpret_cast<float4 *>(out + (size_t)P * 32 * dim + (c / 8u) * 256u + (c % 8u) * 32u);
        float gs = 0.0f;  // the group's sum, any order: only used to guess the running sum's binade
#pragma unroll
        for (int h = 0; h < 2; ++h) {  // sixteen loads in flight at a time
            float q[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t p = 32u * P + 16u * h + r;  // past the end: the last row again, never added
                const float d = x[(int64_t)pm[p < count ? p : count - 1] * ld + c] - m;
                q[r] = d * d;
                gs += p < count ? q[r] : 0.0f;
            }
            if (sq32)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[4 * h + r] = make_float4(q[4 * r], q[4 * r + 1], q[4 * r + 2], q[4 * r + 3]);
        }
        if (gsum) gsum[(seg_group0(range, g) + P) * dim + c] = gs;
    }
}

// Step 2: the sequential sums.  Grid (segments, dim / 32); a wave owns 8 columns, eight
// neighbouring lanes own one column: lane 8 cc + j loads positions 4j .. 4j+3 of column cc of a
// group — one 16-byte load per lane moves 32 positions of 8 columns, 1 KB contiguous per wave —
// and the first lane of the eight adds the 32 values in position order, its neighbours' values
// fetched by DPP row-shift moves.  A lane keeps kChainRing loads in flight: 768
// positions per wave cover a memory round trip of 3 us at 3-4 ns per position with a ring of 96
// registers; one 16-byte load per 4 positions of a lane's own column could keep 240 in flight at
// most (the counter of outstanding loads holds 63) and measured 12 ns per position.
constexpr int kChainRing = 24;

template <int J>
__device__ __forceinline__ float lane_ahead(float v) {  // the value of the lane J places up in its row of 16
    static_assert(J >= 1 && J <= 15, "row shift");
    float r = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x100 + J, 0xF, 0xF, true));
    // The move stays a move (the compiler would fold it into the add as a DPP operand): an add
    // with a DPP operand has a longer latency than a plain one, and the adds are one dependent
    // chain, while the moves are independent and issue in its shadow (measured: 11 -> 8.6 cycles
    // per position).
    asm volatile("" : "+v"(r));
    return r;
}

static __global__ void __launch_bounds__(256) k_seg_chain32(const float *__restrict__ sq32,
                                                           const uint2 *__restrict__ seg_range, int dim,
                                                           float *__restrict__ var) {
    const int g = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cb = blockIdx.y * 4 + wave;  // block of 8 columns
    if (cb * 8 >= dim) return;
    const uint2 range = seg_range[g];
    const uint32_t count = range.y - range.x;
    float acc = 0.0f;
    if (count > 0) {
        const uint32_t nP = (count + 31u) / 32u, last = nP - 1u;
        const size_t stride = (size_t)8 * dim;  // float4 per group of 32 positions
        const float4 *q = reinterpret_cast<const float4 *>(sq32 + ((size_t)range.x + 32u * (size_t)g) * dim) +
                          (size_t)cb * 64 + lane;
        // rem: positions of this group inside the segment (the same in every lane)
        auto add4 = [&](float a, float b, float c, float d, int rem, int at) {
            if (rem > at) acc = acc + a;
            if (rem > at + 1) acc = acc + b;
            if (rem > at + 2) acc = acc + c;
            if (rem > at + 3) acc = acc + d;
        };
        auto add32 = [&](const float4 &v, int rem) {
            add4(v.x, v.y, v.z, v.w, rem, 0);
            add4(lane_ahead<1>(v.x), lane_ahead<1>(v.y), lane_ahead<1>(v.z), lane_ahead<1>(v.w), rem, 4);
            add4(lane_ahead<2>(v.x), lane_ahead<2>(v.y), lane_ahead<2>(v.z), lane_ahead<2>(v.w), rem, 8);
            add4(lane_ahead<3>(v.x), lane_ahead<3>(v.y), lane_ahead<3>(v.z), lane_ahead<3>(v.w), rem, 12);
            add4(lane_ahead<4>(v.x), lane_ahead<4>(v.y), lane_ahead<4>(v.z), lane_ahead<4>(v.w), rem, 16);
            add4(lane_ahead<5>(v.x), lane_ahead<5>(v.y), lane_ahead<5>(v.z), lane_ahead<5>(v.w), rem, 20);
            add4(lane_ahead<6>(v.x), lane_ahead<6>(v.y), lane_ahead<6>(v.z), lane_ahead<6>(v.w), rem, 24);
            add4(lane_ahead<7>(v.x), lane_ahead<7>(v.y), lane_ahead<7>(v.z), lane_ahead<7>(v.w), rem, 28);
        };
        float4 buf[kChainRing];
#pragma unroll
        for (int k = 0; k < kChainRing; ++k) {
            buf[k] = q[(size_t)((uint32_t)k < last ? (uint32_t)k : last) * stride];
            // the first loads are issued in slot order, as the loop issues them: the loop's waits count
            // the loads issued after a slot's, and one order on both ways into the loop keeps them exact
            asm volatile("" ::: "memory");
        }
        const uint32_t full = count / 32u;  // groups with all their positions
        uint32_t P = 0;
        for (; P + kChainRing <= full; P += kChainRing) {
#pragma unroll
            for (int k = 0; k < kChainRing; ++k) {
                // (added first, refilled after: the slot's register is free when its load is issued,
                // so no copy of the ring is carried around the loop)
                add32(buf[k], 32);
                const uint32_t nx = P + kChainRing + k;
                buf[k] = q[(size_t)(nx < last ? nx : last) * stride];
            }
        }
#pragma unroll
        for (int k = 0; k < kChainRing; ++k) {
            const int rem = (int)count - 32 * (int)(P + k);
            if (rem > 0) add32(buf[k], rem);
        }
    }
    if ((lane & 7) == 0) var[(size_t)g * dim + cb * 8 + (lane >> 3)] = acc;
}

// ---- the same sequential sums without the long chain -------------------------------------------
// A sequential f32 sum of non-negative terms is, while the running sum S stays inside one binade
// [2^e, 2^(e+1)], an integer accumulation: with u = 2^(e-23) and S = s u, fl(S + t) = (s + r) u where
// r is t / u rounded to an integer, to nearest, a tie to the value that makes s + r even.  So a
// group of 32 terms acts on s as s -> s + inc[parity of s], two integers per group that depend on e
// only, and the maps of consecutive groups compose.  Three steps on top of k_seg_sqdev32 (which
// also emits every group's approximate sum):
//   k_seg_chain_guess    per column, a prefix over the group sums in f64 gives the binade the running
//                        sum will be in at each group (two candidates near a boundary)
//   k_seg_chain_maps     per (group, column), on the whole GPU: inc[0], inc[1] for the guessed binade(s)
//   k_seg_chain_compose  per column, one wave: 64 groups at a time, the maps composed by a scan over
//                        the lanes; it checks every assumption (S is in the guessed binade at the
//                        group's start and does not leave it) and adds a group's 32 terms one by one
//                        where one fails — the groups in which S crosses a binade, the first groups,
//                        non-finite values.  The result is the sequential sum, bit for bit.
// The value of the lane K places down in its row of 16 lanes (DPP row shift), `fill` where that lane
// is outside the row: scans over the wave take four of these steps and three broadcasts of a row's
// last lane instead of six permutes through LDS.
template <int K>
__device__ __forceinline__ uint32_t row_shr(uint32_t v, uint32_t fill) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)fill, (int)v, 0x110 + K, 0xF, 0xF, false);
}
template <int K>
__device__ __forceinline__ double row_shr_f64(double v) {  // 0.0 where the lane is outside the row
    const unsigned long long b = (unsigned long long)__double_as_longlong(v);
    const uint32_t lo = row_shr<K>((uint32_t)b, 0u), hi = row_shr<K>((uint32_t)(b >> 32), 0u);
    return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}
__device__ __forceinline__ double lane_f64(double v, int src) {  // src: a constant lane
    const unsigned long long b = (unsigned long long)__double_as_longlong(v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, src);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), src);
    return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

constexpr uint32_t kMapInvalid = 0xFFFFFFFFu;
// guess code: exponent field of the lower candidate | two candidates | all terms zero | usable
constexpr uint16_t kGuessOk = 0x8000u, kGuessTwo = 0x0100u, kGuessZero = 0x0200u;

// Long columns are cut into blocks of kGuessBlock groups that are guessed side by side: the f64 sum
// of every block first (grid (segments, dim / 4, blocks); 4 waves, one column each), then a block's
// prefix starts from the sum of the blocks before it.
constexpr uint32_t kGuessBlock = 1024;
static __global__ void __launch_bounds__(256) k_seg_chain_bsum(const float *__restrict__ gsum,
                                                              const uint2 *__restrict__ seg_range, int dim,
                                                              double *__restrict__ bsum) {
    const int g = blockIdx.x, lane = threadIdx.x & 63, c = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (c >= dim) return;
    const uint2 range = seg_range[g];
    const uint32_t count = range.y - range.x, nP = (count + 31u) / 32u;
    const uint32_t P0 = blockIdx.z * kGuessBlock;
    if (P0 >= nP) return;
    const size_t g0 = seg_group0(range, g);
    float vin[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) {
        const uint32_t P = P0 + 64 * k + lane;
        vin[k] = gsum[(g0 + (P < nP ? P : nP - 1)) * dim + c];
    }
    double acc = 0.0;
#pragma unroll
    for (int k = 0; k < 16; ++k) acc += (P0 + 64 * k + lane < nP) ? (double)vin[k] : 0.0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (lane == 0) bsum[((size_t)g * gridDim.z + blockIdx.z) * dim + c] = acc;
}

// grid (segments, dim / 4, blocks); 256 threads = 4 waves, one column each.  bsum == nullptr: one
// block per column, whatever its length.
static __global__ void __launch_bounds__(256) k_seg_chain_guess(const float *__restrict__ gsum,
                                                               const uint2 *__restrict__ seg_range, int dim,
                                                               const double *__restrict__ bsum,
                                                               uint16_t *__restrict__ guess) {
    const int g = blockIdx.x, lane = threadIdx.x & 63, c = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (c >= dim) return;
    const uint2 range = seg_range[g];
    const uint32_t count = range.y - range.x, nP_all = (count + 31u) / 32u;
    const size_t g0 = seg_group0(range, g);
    double carry = 0.0;
    uint32_t P_first = 0, nP = nP_all;
    if (bsum) {
        P_first = blockIdx.z * kGuessBlock;
        if (P_first >= nP_all) return;
        nP = nP_all - P_first < kGuessBlock ? nP_all : P_first + kGuessBlock;
        for (uint32_t b = lane; b < blockIdx.z; b += 64) carry += bsum[((size_t)g * gridDim.z + b) * dim + c];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) carry += __shfl_xor(carry, off);
    }
    constexpr int R = 16;  // batches of 64 groups per round of loads (one memory round trip per round)
    for (uint32_t P0 = P_first; P0 < nP; P0 += 64 * R) {
        float vin[R];
#pragma unroll
        for (int k = 0; k < R; ++k) {
            const uint32_t P = P0 + 64 * k + lane;
            vin[k] = gsum[(g0 + (P < nP ? P : nP - 1)) * dim + c];
        }
#pragma unroll
        for (int k = 0; k < R; ++k) {
            const uint32_t P = P0 + 64 * k + lane;
            const double v = P < nP ? (double)vin[k] : 0.0;
            // inclusive prefix over the lanes: inside the rows of 16, then row by row
            double inc = v;
            inc += row_shr_f64<1>(inc);
            inc += row_shr_f64<2>(inc);
            inc += row_shr_f64<4>(inc);
            inc += row_shr_f64<8>(inc);
            {
                const double r0 = lane_f64(inc, 15);
                if ((lane >> 4) == 1) inc += r0;
                const double r1 = lane_f64(inc, 31);
                if ((lane >> 4) == 2) inc += r1;
                const double r2 = lane_f64(inc, 47);
                if ((lane >> 4) == 3) inc += r2;
            }
            const double before = carry + (inc - v), after = carry + inc;
            carry = lane_f64(after, 63);
            if (P < nP) {
                // the sequential f32 sum is within 2^-9 of the f64 one by a wide margin
                const float lo = (float)(before * (1.0 - 0.001953125)), hi = (float)(after * (1.0 + 0.001953125));
                const uint32_t elo = __float_as_uint(lo) >> 23, ehi = __float_as_uint(hi) >> 23;  // both >= +0
                uint16_t code = 0;
                if (v == 0.0)  // non-negative terms with a zero sum: every one is +0 and leaves any S as it is
                    code = (uint16_t)(kGuessOk | kGuessZero);
                else if (before > 0.0 && elo >= 30u && ehi <= 250u && ehi - elo <= 1u)
                    code = (uint16_t)(kGuessOk | (ehi != elo ? kGuessTwo : 0u) | elo);
                guess[(g0 + P) * dim + c] = code;
            }
        }
    }
}

// inc[0], inc[1] of one group for a running sum in the binade of exponent field e (30 <= e <= 250).
// A term over the unit, y = t / u = t * 2^(150 - e), is exact (a scaling by a power of two; a product
// that underflows stays below 1/2 and counts as zero either way), so its integer part, and whether
// the rest is above or exactly one half, come from a floor and a subtraction, both exact below 2^24.
__device__ __forceinline__ void chain_group_map(const float (&t)[32], int valid, uint32_t e, uint32_t &inc0,
                                                uint32_t &inc1) {
    const float inv_u = __uint_as_float((277u - e) << 23);  // 2^(150 - e)
    // s0, s1: the running sum's integer for an even and for an odd start, less the (even) start
    // itself: their lowest bits are the parities the tie rule asks for
    uint32_t s0 = 0, s1 = 1;
    bool bad = false;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        if (i < valid) {
            const float y = t[i] * inv_u;
            // a negative term, a NaN, an infinity, or a term of a higher binade than the sum's
            bad = bad || !(y >= 0.0f) || !(y < 16777216.0f);
            const float f = floorf(y);
            const float rest = y - f;
            const uint32_t q = (uint32_t)f;
            const uint32_t tie = rest == 0.5f ? 1u : 0u;
            const uint32_t step = q + (rest > 0.5f ? 1u : 0u);
            // a tie goes up when that makes the sum even: when sum + q is odd
            s0 += step + (tie & (s0 + q));
            s1 += step + (tie & (s1 + q));
        }
    }
    inc0 = bad ? kMapInvalid : s0;
    inc1 = bad ? kMapInvalid : s1 - 1u;
}

// Grid (blocks of 64 positions, segments), as k_seg_sqdev32: one thread per (group, column).
static __global__ void __launch_bounds__(256) k_seg_chain_maps(const uint32_t *__restrict__ perm,
                                                              const uint2 *__restrict__ seg_range,
                                                              const float *__restrict__ means, int64_t first,
                                                              const float *__restrict__ x, int64_t ld, int dim,
                                                              const uint16_t *__restrict__ guess,
                                                              uint4 *__restrict__ maps) {
    const int g = blockIdx.y;
    const uint2 range = seg_range[g];
    const uint32_t count = range.y - range.x;
    const uint32_t P0 = blockIdx.x * 2u;
    if (P0 * 32u >= count) return;
    const uint32_t nP = (count + 31u) / 32u;
    const uint32_t groups = nP - P0 < 2u ? nP - P0 : 2u;
    const float *mrow = means + (first + g) * dim;
    const uint32_t *pm = perm + range.x;
    const size_t g0 = seg_group0(range, g);
    for (uint32_t e = threadIdx.x; e < groups * (uint32_t)dim; e += 256) {
        const uint32_t P = P0 + e / (uint32_t)dim, c = e % (uint32_t)dim;
        const uint16_t code = guess[(g0 + P) * dim + c];
        uint4 out = make_uint4(kMapInvalid, kMapInvalid, kMapInvalid, kMapInvalid);
        if (code & kGuessZero) {
            out = make_uint4(0u, 0u, 0u, 0u);
        } else if (code & kGuessOk) {
            // the squares again, with the same two roundings (past the end: the last row, not counted)
            const float m = mrow[c];
            float t[32];
#pragma unroll
            for (int r = 0; r < 32; ++r) {
                const uint32_t p = 32u * P + r;
                const float d = x[(int64_t)pm[p < count ? p : count - 1] * ld + c] - m;
                t[r] = d * d;
            }
            const int valid = (int)(count - 32u * P < 32u ? count - 32u * P : 32u);
            const uint32_t elo = code & 255u;
            chain_group_map(t, valid, elo, out.x, out.y);
            if (code & kGuessTwo) chain_group_map(t, valid, elo + 1u, out.z, out.w);
        }
        maps[(g0 + P) * dim + c] = out;
    }
}

// The map of the lanes' groups composed over the wave: on return lane p holds the map of the groups
// of lanes first .. p (lanes outside [first, last) supply the identity), as increments for an even
// and for an odd start, saturated at 2^25.
__device__ __forceinline__ void chain_scan_maps(uint32_t &a0, uint32_t &a1, int lane) {
    const uint32_t cap = 1u << 25;
    // left, then this lane's map: c_p = l_p + a_[(p + l_p) mod 2]; (0, 0) is the identity, which is what a
    // lane outside the row supplies
    auto after_left = [&](uint32_t l0, uint32_t l1) {
        const uint32_t n0 = l0 + ((l0 & 1u) ? a1 : a0);        // start even: after l0 the parity is l0 & 1
        const uint32_t n1 = l1 + (((l1 + 1u) & 1u) ? a1 : a0);  // start odd
        a0 = n0 < cap ? n0 : cap;
        a1 = n1 < cap ? n1 : cap;
    };
    after_left(row_shr<1>(a0, 0u), row_shr<1>(a1, 0u));
    after_left(row_shr<2>(a0, 0u), row_shr<2>(a1, 0u));
    after_left(row_shr<4>(a0, 0u), row_shr<4>(a1, 0u));
    after_left(row_shr<8>(a0, 0u), row_shr<8>(a1, 0u));
    uint32_t t0 = (uint32_t)__builtin_amdgcn_readlane((int)a0, 15), t1 = (uint32_t)__builtin_amdgcn_readlane((int)a1, 15);
    if ((lane >> 4) == 1) after_left(t0, t1);
    t0 = (uint32_t)__builtin_amdgcn_readlane((int)a0, 31), t1 = (uint32_t)__builtin_amdgcn_readlane((int)a1, 31);
    if ((lane >> 4) == 2) after_left(t0, t1);
    t0 = (uint32_t)__builtin_amdgcn_readlane((int)a0, 47), t1 = (uint32_t)__builtin_amdgcn_readlane((int)a1, 47);
    if ((lane >> 4) == 3) after_left(t0, t1);
}

// Runs of kRunGroups consecutive groups of a long column get their maps composed ahead of the walk
// (k_seg_chain_runs): a run is "clean" when every group has one guessed binade, the same in all of
// them (groups of zeros fit any), and a usable map.  The walk then passes a clean run in one step
// when S is in that binade at the run's start and does not leave it by the run's end — S never
// decreases, so it is in the binade at every group in between and each group's map applies, which is
// all the group-by-group walk checks.  Any other run is walked group by group as before.
constexpr uint32_t kRunGroups = 256;
constexpr uint32_t kRunClean = 0x80000000u, kRunAnyBinade = 0x40000000u;

// Index of a segment's first run in the per-run table (runs of different segments never share one).
__device__ __forceinline__ size_t seg_run0(const uint2 range, int g) {
    return seg_group0(range, g) / kRunGroups + (size_t)g;
}

// grid (segments, dim / 4, ceil(groups / 1024)); 256 threads = 4 waves, one column each; a wave
// composes four runs (16 batches of 64 groups, one round of loads).
static __global__ void __launch_bounds__(256) k_seg_chain_runs(const uint2 *__restrict__ seg_range, int dim,
                                                              const uint16_t *__restrict__ guess,
                                                              const uint4 *__restrict__ maps,
                                                              uint4 *__restrict__ runs) {
    const int g = blockIdx.x, lane = threadIdx.x & 63, c = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (c >= dim) return;
    const uint2 range = seg_range[g];
    const uint32_t count = range.y - range.x, nP = (count + 31u) / 32u;
    const uint32_t P0 = blockIdx.z * (4u * kRunGroups);
    if (P0 >= nP) return;
    const size_t g0 = seg_group0(range, g), r0 = seg_run0(range, g);
    constexpr int R = 16;
    uint16_t codeR[R];
    uint4 mpR[R];
#pragma unroll
    for (int k = 0; k < R; ++k) {
        const uint32_t idx = P0 + 64u * k + lane;
        const size_t at = (g0 + (idx < nP ? idx : nP - 1u)) * dim + c;
        codeR[k] = guess[at];
        mpR[k] = maps[at];
    }
    const uint32_t cap = 1u << 25;
#pragma unroll
    for (int run = 0; run < 4; ++run) {
        const uint32_t Pr = P0 + run * kRunGroups;
        if (Pr >= nP) break;  // uniform
        uint32_t c0 = 0, c1 = 0, e = 0;
        bool clean = true, any_binade = true;
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4) {
            const int k = 4 * run + k4;
            const uint32_t base = Pr + 64u * k4;
            const uint32_t left = base >= nP ? 0u : (nP - base < 64u ? nP - base : 64u);
            if (left == 0u) break;  // uniform
            const uint16_t code = codeR[k];
            const uint4 mp = mpR[k];
            const bool mine = (uint32_t)lane < left;
            const bool zero = (code & kGuessZero) != 0;
            const uint32_t elo = code & 255u;
            const bool usable = (code & kGuessOk) &&
                                (zero || (!(code & kGuessTwo) && mp.x != kMapInvalid && elo >= 30u && elo <= 250u));
            if (__ballot(mine && !usable)) clean = false;
            const unsigned long long binade = __ballot(mine && !zero);
            if (binade) {
                const uint32_t ef = (uint32_t)__builtin_amdgcn_readlane((int)elo, __ffsll((long long)binade) - 1);
                if (any_binade) e = ef;
                any_binade = false;
                if (__ballot(mine && !zero && elo != e)) clean = false;
            }
            uint32_t a0 = (mine && !zero) ? (mp.x < cap ? mp.x : cap) : 0u;
            uint32_t a1 = (mine && !zero) ? (mp.y < cap ? mp.y : cap) : 0u;
            chain_scan_maps(a0, a1, lane);
            const uint32_t b0 = (uint32_t)__builtin_amdgcn_readlane((int)a0, 63), b1 = (uint32_t)__builtin_amdgcn_readlane((int)a1, 63);
            // the run so far, then this batch
            const uint32_t n0 = c0 + ((c0 & 1u) ? b1 : b0), n1 = c1 + (((c1 + 1u) & 1u) ? b1 : b0);
            c0 = n0 < cap ? n0 : cap;
            c1 = n1 < cap ? n1 : cap;
        }
        if (lane == 0)
            runs[(r0 + Pr / kRunGroups) * dim + c] =
                make_uint4(c0, c1, (clean ? kRunClean : 0u) | (any_binade ? kRunAnyBinade : 0u) | e, 0u);
    }
}

// One batch of up to 64 groups (lane = group base + lane) added to S, which is the same value in every
// lane: runs of usable groups through their composed maps, any other group term by term.
__device__ __forceinline__ void chain_batch(float &S, uint32_t base, uint32_t left, uint16_t code, uint4 mp,
                                            const uint32_t *__restrict__ pm, uint32_t count,
                                            const float *__restrict__ x, int64_t ld, int c, float mean_c, int lane) {
    const uint32_t elo = code & 255u;
    const bool zero = (code & kGuessZero) != 0;
    uint32_t start = 0;  // groups of the batch already added
    while (start < left) {
        // S is +0, positive, +inf or a NaN; with the sign bit of a NaN eS is above every guess
        const uint32_t Sb = __float_as_uint(S), eS = Sb >> 23;
        const uint32_t s = (Sb & 0x7fffffu) | 0x800000u;  // S / u for a normal S
        const bool is_lo = elo == eS, is_hi = (code & kGuessTwo) && elo + 1u == eS;
        uint32_t a0 = is_lo ? mp.x : mp.z, a1 = is_lo ? mp.y : mp.w;
        // a group of zeros keeps any finite S; another group needs S in the binade of its map
        const bool mine = (uint32_t)lane >= start && (uint32_t)lane < left;
        const bool ok = (code & kGuessOk) &&
                        (zero ? eS < 255u : (eS >= 30u && eS <= 250u && (is_lo || is_hi) && a0 != kMapInvalid));
        if (zero) a0 = a1 = 0u;
        // the run of usable groups that starts at `start`
        const unsigned long long stop = __ballot(mine && !ok) | (left < 64u ? ~0ull << left : 0ull);
        const uint32_t end = stop ? (uint32_t)__ffsll((long long)stop) - 1u : 64u;
        bool advanced = false;
        if (end > start) {
            const uint32_t cap = 1u << 25;
            const bool part = (uint32_t)lane >= start && (uint32_t)lane < end;
            a0 = part ? (a0 < cap ? a0 : cap) : 0u;
            a1 = part ? (a1 < cap ? a1 : cap) : 0u;
            // inclusive scan: the map of groups start .. lane, as increments for a start parity
            chain_scan_maps(a0, a1, lane);
            const uint32_t send = s + ((s & 1u) ? a1 : a0);
            const bool fits = part && send <= (1u << 24);
            const int nv = __popcll(__ballot(fits));  // fits is monotone: the sums never decrease
            if (nv > 0) {
                const uint32_t take = (uint32_t)__builtin_amdgcn_readlane((int)send, __builtin_amdgcn_readfirstlane((int)start + nv - 1));
                // (a subnormal or zero S only passes groups of zeros: take == s and S stays)
                S = __uint_as_float(take == (1u << 24) ? (eS + 1u) << 23 : (eS << 23) | (take - (1u << 23)));
                start += (uint32_t)nv;
                advanced = true;
            }
        }
        if (!advanced) {
            // the group's terms one by one (positions past the end add +0.0, which changes nothing)
            const uint32_t P = base + start;
            float t = 0.0f;
            if (lane < 32 && P * 32u + (uint32_t)lane < count) {
                const float d = x[(int64_t)pm[P * 32u + lane] * ld + c] - mean_c;
                t = d * d;
            }
#pragma unroll
            for (int i = 0; i < 32; ++i) S = S + __shfl(t, i);
            start += 1u;
        }
    }
}

// grid (segments, dim / 4); 256 threads = 4 waves, one column each.  runs == nullptr: every group is
// walked (short columns); else the table of k_seg_chain_runs.
static __global__ void __launch_bounds__(256) k_seg_chain_compose(const uint32_t *__restrict__ perm,
                                                                 const uint2 *__restrict__ seg_range,
                                                                 const float *__restrict__ means, int64_t first,
                                                                 const float *__restrict__ x, int64_t ld, int dim,
                                                                 const uint16_t *__restrict__ guess,
                                                                 const uint4 *__restrict__ maps,
                                                                 const uint4 *__restrict__ runs,
                                                                 float *__restrict__ var) {
    const int g = blockIdx.x, lane = threadIdx.x & 63, c = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (c >= dim) return;
    const uint2 range = seg_range[g];
    const uint32_t count = range.y - range.x, nP = (count + 31u) / 32u;
    const size_t g0 = seg_group0(range, g);
    const float mean_c = means[(first + g) * dim + c];
    const uint32_t *pm = perm + range.x;
    float S = 0.0f;  // the same value in every lane
    if (runs) {
        const size_t r0 = seg_run0(range, g);
        const uint32_t nR = (nP + kRunGroups - 1u) / kRunGroups;
        for (uint32_t rb = 0; rb < nR; rb += 64) {
            const uint32_t ri = rb + lane;
            const uint4 rm = runs[(r0 + (ri < nR ? ri : nR - 1u)) * dim + c];  // lane = run rb + lane
            const uint32_t here = nR - rb < 64u ? nR - rb : 64u;
            for (uint32_t j = 0; j < here; ++j) {
                const uint32_t c0 = (uint32_t)__builtin_amdgcn_readlane((int)rm.x, (int)j);
                const uint32_t c1 = (uint32_t)__builtin_amdgcn_readlane((int)rm.y, (int)j);
                const uint32_t meta = (uint32_t)__builtin_amdgcn_readlane((int)rm.z, (int)j);
                const uint32_t Sb = __float_as_uint(S), eS = Sb >> 23;
                const uint32_t s = (Sb & 0x7fffffu) | 0x800000u;
                const uint32_t send = s + ((s & 1u) ? c1 : c0);
                const bool binade_ok = (meta & kRunAnyBinade) ? eS < 255u : (eS == (meta & 255u) && eS >= 30u && eS <= 250u);
                if ((meta & kRunClean) && binade_ok && send <= (1u << 24)) {
                    // (a run of zeros: send == s and S stays, whatever finite value it has)
                    if (!(meta & kRunAnyBinade))
                        S = __uint_as_float(send == (1u << 24) ? (eS + 1u) << 23 : (eS << 23) | (send - (1u << 23)));
                    continue;
                }
                // group by group: the run's four batches
                const uint32_t Pr = (rb + j) * kRunGroups;
                uint16_t codeR[4];
                uint4 mpR[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t idx = Pr + 64u * k + lane;
                    const size_t at = (g0 + (idx < nP ? idx : nP - 1u)) * dim + c;
                    codeR[k] = guess[at];
                    mpR[k] = maps[at];
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t base = Pr + 64u * k;
                    const uint32_t left = base >= nP ? 0u : (nP - base < 64u ? nP - base : 64u);
                    chain_batch(S, base, left, codeR[k], mpR[k], pm, count, x, ld, c, mean_c, lane);
                }
            }
        }
        if (lane == 0) var[(size_t)g * dim + c] = S;
        return;
    }
    // Batches of 64 groups at fixed positions (lane = group 64 b + lane), R batches per round of
    // loads: one memory round trip per round instead of one per batch.
    constexpr int R = 16;
    const uint32_t nB = (nP + 63u) / 64u;
    for (uint32_t b0 = 0; b0 < nB; b0 += R) {
        uint16_t codeR[R];
        uint4 mpR[R];
#pragma unroll
        for (int k = 0; k < R; ++k) {
            const uint32_t idx = (b0 + k) * 64u + lane;
            const size_t at = (g0 + (idx < nP ? idx : nP - 1u)) * dim + c;
            codeR[k] = guess[at];
            mpR[k] = maps[at];
        }
#pragma unroll
        for (int k = 0; k < R; ++k) {
            const uint32_t base = (b0 + k) * 64u;  // first group of the batch
            // groups in the batch (none past the end: the loop inside does not run; uniform)
            const uint32_t left = base >= nP ? 0u : (nP - base < 64u ? nP - base : 64u);
            chain_batch(S, base, left, codeR[k], mpR[k], pm, count, x, ld, c, mean_c, lane);
        }
    }
    if (lane == 0) var[(size_t)g * dim + c] = S;
}

// The same sums with everything but the adds taken off the chain of dependent adds.  One workgroup
// of 1024 threads per segment: all threads fetch rows (16-byte pieces, whole rows contiguous)
// eight chunks ahead into registers, turn them into squared deviations (v - mean)^2 — the same
// two roundings as in the chain — and hand those over through two LDS tiles; threads 0..dim-1
// add the squares of the current tile in row order, one add per row.  A chunk is 8192 / dim rows;
// about 512 rows (256 KB at dim = 128) are in flight per workgroup, which is what one chain of adds
// consumes per memory round trip.  The barrier waits for LDS only, so the loads in flight are not
// drained.
constexpr int kVarStage = 8192;  // floats per LDS tile
constexpr int kVarAhead = 8;     // chunks in flight

__device__ __forceinline__ void lds_only_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// acc + the squares of one component over the rows of one LDS tile, in row order.  DIM > 0: the row
// stride as a constant, so that the reads pair up with constant offsets and the next sixteen
// values are on their way while sixteen are added; DIM = 0: any stride.
template <int DIM>
__device__ __forceinline__ float seg_variance_chunk(const float *t, int rows, int dim, float acc) {
    const int stride = DIM > 0 ? DIM : dim;
    int r = 0;
    if (rows >= 16) {
        float v[16];
#pragma unroll
        for (int q = 0; q < 16; ++q) v[q] = t[q * stride];
        for (; r + 32 <= rows; r += 16) {
            float w[16];
#pragma unroll
            for (int q = 0; q < 16; ++q) w[q] = t[(r + 16 + q) * stride];
#pragma unroll
            for (int q = 0; q < 16; ++q) acc = acc + v[q];
#pragma unroll
            for (int q = 0; q < 16; ++q) v[q] = w[q];
        }
#pragma unroll
        for (int q = 0; q < 16; ++q) acc = acc + v[q];
        r += 16;
    }
    for (; r < rows; ++r) acc = acc + t[r * stride];
    return acc;
}

template <int DIM>
static __global__ void __launch_bounds__(1024) k_seg_variance_wg(const uint32_t *__restrict__ perm,
                                                                const uint2 *__restrict__ seg_range,
                                                                const float *__restrict__ means, int64_t first,
                                                                const float *__restrict__ x, int64_t ld, int dim,
                                                                float *__restrict__ var) {
    __shared__ float4 tile[2][kVarStage / 4];
    const int g = blockIdx.x, tid = threadIdx.x;
    const uint2 range = seg_range[g];
    const uint32_t count = range.y - range.x;
    const int ppr = dim / 4;                  // 16-byte pieces per row
    const int R = kVarStage / dim;            // rows per chunk
    const int pieces = R * ppr;               // pieces per chunk (<= 2048)
    const int nch = (int)((count + R - 1) / R);
    // this thread's two pieces of every chunk
    int rr[2], pc[2];
    bool has[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int e = tid + 1024 * j;
        has[j] = e < pieces;
        rr[j] = has[j] ? e / ppr : 0;
        pc[j] = has[j] ? e % ppr : 0;
    }
    if (count == 0) {  // uniform
        if (tid < dim) var[(size_t)g * dim + tid] = 0.0f;
        return;
    }
    const uint32_t *pm = perm + range.x;
    // Loads are unconditional (positions clamped into the segment; surplus rows are fetched and
    // never read): loads under a branch would make the compiler wait for every outstanding load
    // at each use instead of counting them.  The rings are plain arrays with constant indices.
    // (Eight named slots instead of an array: an array of this size is left in scratch memory.)
    const float *xp0 = x + 4 * pc[0], *xp1 = x + 4 * pc[1];
    // the means of this thread's columns
    const float *mrow = means + (first + g) * dim;
    const float4 mu0 = *reinterpret_cast<const float4 *>(mrow + 4 * pc[0]);
    const float4 mu1 = *reinterpret_cast<const float4 *>(mrow + 4 * pc[1]);
    auto sq_dev = [](float4 v, float4 m) {
        float4 d, p;
        d.x = v.x - m.x;
        d.y = v.y - m.y;
        d.z = v.z - m.z;
        d.w = v.w - m.w;
        p.x = d.x * d.x;
        p.y = d.y * d.y;
        p.z = d.z * d.z;
        p.w = d.w * d.w;
        return p;
    };
#define VAR_DECL(S) uint32_t ida_##S, idb_##S; float4 xa_##S, xb_##S;
    VAR_DECL(0) VAR_DECL(1) VAR_DECL(2) VAR_DECL(3) VAR_DECL(4) VAR_DECL(5) VAR_DECL(6) VAR_DECL(7)
#define VAR_IDS(S, chunk)                                                     \
    {                                                                         \
        const uint32_t m0 = (uint32_t)(chunk) * R + rr[0], m1 = (uint32_t)(chunk) * R + rr[1]; \
        ida_##S = pm[m0 < count ? m0 : count - 1];                            \
        idb_##S = pm[m1 < count ? m1 : count - 1];                            \
    }
#define VAR_ROWS(S)                                                           \
    {                                                                         \
        xa_##S = *reinterpret_cast<const float4 *>(xp0 + (int64_t)ida_##S * ld); \
        xb_##S = *reinterpret_cast<const float4 *>(xp1 + (int64_t)idb_##S * ld); \
    }
#define VAR_STORE(buf, S)                                                     \
    {                                                                         \
        if (has[0]) tile[buf][rr[0] * ppr + pc[0]] = sq_dev(xa_##S, mu0);     \
        if (has[1]) tile[buf][rr[1] * ppr + pc[1]] = sq_dev(xb_##S, mu1);     \
    }
    // prologue: ids of chunks 0..15, rows of chunks 0..7, chunk 0 in LDS
    VAR_IDS(0, 0) VAR_IDS(1, 1) VAR_IDS(2, 2) VAR_IDS(3, 3) VAR_IDS(4, 4) VAR_IDS(5, 5) VAR_IDS(6, 6) VAR_IDS(7, 7)
#define VAR_PRO(S) VAR_ROWS(S) VAR_IDS(S, S + kVarAhead)
    VAR_PRO(0) VAR_PRO(1) VAR_PRO(2) VAR_PRO(3) VAR_PRO(4) VAR_PRO(5) VAR_PRO(6) VAR_PRO(7)
    VAR_STORE(0, 0)
    lds_only_barrier();
    float acc = 0.0f;
    // One step: rows of chunk i + 8 into the slot chunk i has left, ids of chunk i + 16 behind
    // them; chunk i + 1 (fetched seven steps ago) into the other tile; chunk i added.  Chunks past
    // the end run empty, so every thread reaches every barrier.
#define VAR_STEP(S, SN)                                                       \
    {                                                                         \
        const int i = base + S;                                               \
        VAR_ROWS(S)                                                           \
        VAR_IDS(S, i + 2 * kVarAhead)                                         \
        VAR_STORE((i + 1) & 1, SN)                                            \
        if (tid < dim && i < nch) {                                           \
            const float *t = reinterpret_cast<const float *>(tile[i & 1]) + tid; \
            const int rows = (int)(((uint32_t)(i + 1) * R <= count) ? R : count - (uint32_t)i * R); \
            acc = seg_variance_chunk<DIM>(t, rows, dim, acc);                 \
        }                                                                     \
        lds_only_barrier();                                                   \
    }
    for (int base = 0; base < nch; base += kVarAhead) {
        VAR_STEP(0, 1) VAR_STEP(1, 2) VAR_STEP(2, 3) VAR_STEP(3, 4)
        VAR_STEP(4, 5) VAR_STEP(5, 6) VAR_STEP(6, 7) VAR_STEP(7, 0)
    }
#undef VAR_DECL
#undef VAR_PRO
#undef VAR_STEP
#undef VAR_IDS
#undef VAR_ROWS
#undef VAR_STORE
    if (tid < dim) var[(size_t)g * dim + tid] = acc;
}

__device__ __forceinline__ int find_segment(const uint2 *__restrict__ seg_range, int nseg, uint32_t p) {
    // segments are sorted by position and disjoint; returns -1 when p lies in none
    int lo = 0, hi = nseg - 1;
    while (lo <= hi) {
        int mid = (lo + hi) >> 1;
        uint2 r = seg_range[mid];
        if (p < r.x)
            hi = mid - 1;
        else if (p >= r.y)
            lo = mid + 1;
        else
            return mid;
    }
    return -1;
}

// vals[p] = x[perm[p]][split_dim[segment of p]]; positions outside every segment get +inf
static __global__ void __launch_bounds__(256) k_seg_gather_col(const uint32_t *__restrict__ perm, int64_t n,
                                                        const uint2 *__restrict__ seg_range, int nseg,
                                                        const int *__restrict__ split_dim,
                                                        const float *__restrict__ x, int64_t ld,
                                                        float *__restrict__ vals) {
    int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= n) return;
    int g = find_segment(seg_range, nseg, (uint32_t)p);
    vals[p] = g < 0 ? __builtin_inff() : x[(int64_t)perm[p] * ld + split_dim[g]];
}

// flags[p] = 1 when the row at position p goes left (value <= median of its segment)
static __global__ void __launch_bounds__(256) k_seg_flags(const float *__restrict__ vals, int64_t n,
                                                   const uint2 *__restrict__ seg_range, int nseg,
                                                   const float *__restrict__ median,
                                                   uint32_t *__restrict__ flags) {
    int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= n) return;
    int g = find_segment(seg_range, nseg, (uint32_t)p);
    flags[p] = (g >= 0 && vals[p] <= median[g]) ? 1u : 0u;
}

// Stable partition inside every segment using the exclusive scan of flags.
// nleft[g] = number of rows going left.
static __global__ void __launch_bounds__(256) k_seg_partition(const uint32_t *__restrict__ perm_in, int64_t n,
                                                       const uint2 *__restrict__ seg_range, int nseg,
                                                       const uint32_t *__restrict__ flags,
                                                       const uint32_t *__restrict__ scan,
                                                       uint32_t *__restrict__ perm_out,
                                                       uint32_t *__restrict__ nleft) {
    int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= n) return;
    int g = find_segment(seg_range, nseg, (uint32_t)p);
    if (g < 0) {
        perm_out[p] = perm_in[p];
        return;
    }
    uint2 r = seg_range[g];
    uint32_t before = scan[p] - scan[r.x];                       // left rows before p in the segment
    uint32_t total_left = scan[r.y - 1] + flags[r.y - 1] - scan[r.x];
    uint32_t dst = flags[p] ? r.x + before : r.x + total_left + ((uint32_t)p - r.x - before);
    perm_out[dst] = perm_in[p];
    if ((uint32_t)p == r.x) nleft[g] = total_left;
}

static __global__ void __launch_bounds__(256) k_iota_u32(uint32_t *__restrict__ p, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = (uint32_t)i;
}

// ---- middle values by radix select ---------------------------------------------------------
// The reference sorts the split column and takes values[c/2] (and values[c/2 - 1] for an even
// count, src/tsvq.rs:108-117); only those two order statistics are needed.  Floats are mapped to
// unsigned keys of the same order; four passes of 8 bits narrow each target down: a pass counts,
// per segment and target, the keys that share the target's known high bits by their next byte
// (LDS histograms per workgroup, flushed with integer atomics), then one thread per (segment,
// target) picks the byte whose bin holds the target's rank.
struct SegSelect {
    uint32_t prefix;  // known high bits of the key (low bits zero)
    uint32_t rank;    // rank of the target among the keys that share the prefix
};

__device__ __forceinline__ uint32_t float_order_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float float_from_order_key(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// One workgroup per 4096 positions; pass = 0..3 looks at key bits [31 - 8 pass, 24 - 8 pass].
static __global__ void __launch_bounds__(256) k_seg_select_hist(const float *__restrict__ vals, int64_t n,
                                                                const uint2 *__restrict__ seg_range, int nseg,
                                                                const SegSelect *__restrict__ sel, int pass,
                                                                uint32_t *__restrict__ hist) {
    __shared__ uint32_t lh[512];
    const int64_t lo = (int64_t)blockIdx.x * 4096;
    const int64_t hi = lo + 4096 < n ? lo + 4096 : n;
    const int shift = 24 - 8 * pass;
    const uint32_t high_mask = pass == 0 ? 0u : (0xFFFFFFFFu << (shift + 8));
    // segments are sorted by position and disjoint: walk the ones that overlap this chunk
    int g = 0;
    {
        int a = 0, b = nseg;  // first segment whose end is beyond lo
        while (a < b) {
            const int mid = (a + b) >> 1;
            if (seg_range[mid].y <= (uint32_t)lo) a = mid + 1; else b = mid;
        }
        g = a;
    }
    for (; g < nseg; ++g) {
        const uint2 r = seg_range[g];
        if ((int64_t)r.x >= hi) break;
        const int64_t from = (int64_t)r.x > lo ? (int64_t)r.x : lo, to = (int64_t)r.y < hi ? (int64_t)r.y : hi;
        const uint32_t p0 = sel[2 * g].prefix, p1 = sel[2 * g + 1].prefix;
        __syncthreads();
        lh[threadIdx.x] = 0u;
        lh[256 + threadIdx.x] = 0u;
        __syncthreads();
        for (int64_t p = from + threadIdx.x; p < to; p += 256) {
            const uint32_t key = float_order_key(vals[p]);
            const uint32_t byte = (key >> shift) & 255u;
            if ((key & high_mask) == p0) atomicAdd(&lh[byte], 1u);
            if ((key & high_mask) == p1) atomicAdd(&lh[256 + byte], 1u);
        }
        __syncthreads();
        uint32_t *gh = hist + (size_t)g * 512;
        if (lh[threadIdx.x]) atomicAdd(&gh[threadIdx.x], lh[threadIdx.x]);
        if (lh[256 + threadIdx.x]) atomicAdd(&gh[256 + threadIdx.x], lh[256 + threadIdx.x]);
    }
}

// One wave per (segment, target): the byte whose bin holds the rank; clears the bins.  A lane
// takes four bins, a scan over the lanes finds the one whose bins hold the rank.
static __global__ void __launch_bounds__(64) k_seg_select_pick(uint32_t *__restrict__ hist,
                                                               SegSelect *__restrict__ sel, int nseg, int pass) {
    const int i = blockIdx.x, lane = threadIdx.x;
    if (i >= 2 * nseg) return;
    uint4 *h = reinterpret_cast<uint4 *>(hist + (size_t)i * 256);
    const uint4 c = h[lane];
    h[lane] = make_uint4(0u, 0u, 0u, 0u);
    const SegSelect s = sel[i];
    const uint32_t tot = c.x + c.y + c.z + c.w;
    uint32_t inc = tot;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t v = __shfl_up(inc, off);
        if (lane >= off) inc += v;
    }
    const uint32_t exc = inc - tot;
    const bool mine = s.rank >= exc && s.rank < inc;
    const int shift = 24 - 8 * pass;
    if (mine) {
        uint32_t r = s.rank - exc, byte = 4u * (uint32_t)lane;
        if (r >= c.x) {
            r -= c.x;
            ++byte;
            if (r >= c.y) {
                r -= c.y;
                ++byte;
                if (r >= c.z) {
                    r -= c.z;
                    ++byte;
                }
            }
        }
        sel[i] = SegSelect{s.prefix | (byte << shift), r};
    }
    // a rank beyond the counted keys (never for a rank inside its segment): the last byte
    const uint32_t all = __shfl(inc, 63);
    if (lane == 0 && s.rank >= all) sel[i] = SegSelect{s.prefix | (255u << shift), s.rank - all};
}

// The split dimension of every segment: argmax of its per-dimension sums with the LAST maximal
// element winning (Iterator::max_by, src/tsvq.rs:102-106); one thread per segment.
// The same launch starts the radix select of the middle values: bins cleared, ranks of the two
// targets of every segment (the lower and the upper middle).  Grid over nseg * 512 bins.
static __global__ void k_seg_argmax_last(const float *__restrict__ var, int nseg, int dim, int *__restrict__ sdim,
                                         const uint2 *__restrict__ seg_range, SegSelect *__restrict__ sel,
                                         uint32_t *__restrict__ hist) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < nseg * 512) hist[i] = 0u;
    if (i >= nseg) return;
    {
        const uint2 r = seg_range[i];
        const uint32_t c = r.y - r.x;
        sel[2 * i] = SegSelect{0u, (c % 2 == 0) ? c / 2 - 1 : c / 2};
        sel[2 * i + 1] = SegSelect{0u, c / 2};
    }
    const float *v = var + (size_t)i * dim;
    int best = 0;
    float vb = v[0];
    for (int t0 = 1; t0 < dim; t0 += 16) {
        float w[16];  // sixteen loads in flight
#pragma unroll
        for (int u = 0; u < 16; ++u) w[u] = v[t0 + u < dim ? t0 + u : dim - 1];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            if (t0 + u < dim && !(w[u] < vb)) {
                best = t0 + u;
                vb = w[u];
            }
        }
    }
    sdim[i] = best;
}

// The median of every segment from its two middle values (src/tsvq.rs:112-117): their f32 sum
// divided by two for an even count, the middle value otherwise.
static __global__ void k_seg_median(const SegSelect *__restrict__ sel, const uint2 *__restrict__ seg_range, int nseg,
                                    float *__restrict__ median) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nseg) return;
    const uint32_t cnt = seg_range[i].y - seg_range[i].x;
    // the selected keys back as floats
    const float a = float_from_order_key(sel[2 * i].prefix), b = float_from_order_key(sel[2 * i + 1].prefix);
    const float sum = a + b;
    median[i] = (cnt % 2u == 0u) ? sum / 2.0f : a;
}

// out[i][t] = means[idx[i]][t]: the means of the nodes that split, side by side
static __global__ void __launch_bounds__(256) k_gather_means(const float *__restrict__ means,
                                                             const int *__restrict__ idx, int ns, int dim,
                                                             float *__restrict__ out) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= (int64_t)ns * dim) return;
    out[e] = means[(size_t)idx[e / dim] * dim + e % dim];
}

// ---- descent -------------------------------------------------------------------------------
template <int METRIC>
__device__ __forceinline__ float tsvq_dist(const float *__restrict__ xr, const float *__restrict__ c,
                                           int dim, float na, float nb) {
    float acc = 0.0f;
    if constexpr (METRIC == M_COS) {
        for (int t = 0; t < dim; ++t) {
            float p = xr[t] * c[t];
            acc = acc + p;
        }
        float den = na * nb;
        float q = acc / den;
        float d = 1.0f - q;
        return (na == 0.0f || nb == 0.0f) ? 1.0f : d;
    } else if constexpr (METRIC == M_L1) {
        for (int t = 0; t < dim; ++t) {
            float d = xr[t] - c[t];
            acc = acc + fabsf(d);
        }
        return acc;
    } else {
        for (int t = 0; t < dim; ++t) {
            float d = xr[t] - c[t];
            float p = d * d;
            acc = acc + p;
        }
        return METRIC == M_EUCLID ? sqrtf(acc) : acc;
    }
}

// One lane = one row; walks from the root, `<=` goes left (src/tsvq.rs:171), single children are
// followed unconditionally (177-178).  Both distances of a level are accumulated together.
template <int METRIC>
__global__ void __launch_bounds__(256) k_tsvq_descend(const float *__restrict__ x, int64_t n, int64_t ld,
                                                      int dim, const float *__restrict__ cen,
                                                      const float *__restrict__ cnorm,
                                                      const int *__restrict__ left,
                                                      const int *__restrict__ right,
                                                      int *__restrict__ leaf) {
    int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= n) return;
    const float *__restrict__ xr = x + row * ld;
    float na = 0.0f;
    if constexpr (METRIC == M_COS) {
        float sa = 0.0f;
        for (int t = 0; t < dim; ++t) {
            float p = xr[t] * xr[t];
            sa = sa + p;
        }
        na = sqrtf(sa);
    }
    int node = 0;
    for (;;) {
        int l = left[node], r = right[node];
        if (l >= 0 && r >= 0) {
            const float *__restrict__ cl = cen + (size_t)l * dim;
            const float *__restrict__ cr = cen + (size_t)r * dim;
            float al = 0.0f, ar = 0.0f;
            for (int t = 0; t < dim; ++t) {
                float xv = xr[t];
                if constexpr (METRIC == M_COS) {
                    float pl = xv * cl[t], pr = xv * cr[t];
                    al = al + pl;
                    ar = ar + pr;
                } else if constexpr (METRIC == M_L1) {
                    float dl = xv - cl[t], dr = xv - cr[t];
                    al = al + fabsf(dl);
                    ar = ar + fabsf(dr);
                } else {
                    float dl = xv - cl[t], dr = xv - cr[t];
                    float pl = dl * dl, pr = dr * dr;
                    al = al + pl;
                    ar = ar + pr;
                }
            }
            float dl, dr;
            if constexpr (METRIC == M_COS) {
                float nl = cnorm[l], nr = cnorm[r];
                float ql = al / (na * nl), qr = ar / (na * nr);
                dl = (na == 0.0f || nl == 0.0f) ? 1.0f : 1.0f - ql;
                dr = (na == 0.0f || nr == 0.0f) ? 1.0f : 1.0f - qr;
            } else if constexpr (METRIC == M_EUCLID) {
                dl = sqrtf(al);
                dr = sqrtf(ar);
            } else {
                dl = al;
                dr = ar;
            }
            node = (dl <= dr) ? l : r;
        } else if (l >= 0) {
            node = l;
        } else if (r >= 0) {
            node = r;
        } else {
            break;
        }
    }
    leaf[row] = node;
}

// The same walk with the row held in registers (DIM a multiple of 32 up to 128).  One wave = 64
// rows, eight waves per workgroup: the rows are read with whole-line loads through a small padded LDS tile, so every byte of
// the input is fetched once; the two child centroids of a lane's node are read 64 bytes at a
// time, the next piece in flight while the current one is accumulated.  The sums stay one
// sequential chain per (row, child), as in the reference.
template <int METRIC>
__device__ __forceinline__ void tsvq_step(float &al, float &ar, float xv, float cl, float cr) {
    if constexpr (METRIC == M_COS) {
        float pl = xv * cl, pr = xv * cr;
        al = al + pl;
        ar = ar + pr;
    } else if constexpr (METRIC == M_L1) {
        float dl = xv - cl, dr = xv - cr;
        al = al + fabsf(dl);
        ar = ar + fabsf(dr);
    } else {
        float dl = xv - cl, dr = xv - cr;
        float pl = dl * dl, pr = dr * dr;
        al = al + pl;
        ar = ar + pr;
    }
}

// The centroids of the first kTopNodes nodes (the upper levels of a tree numbered level by level)
// are staged in LDS: down there the lanes of a wave sit on a handful of nodes, and per-lane
// global reads of a few distinct lines cost the address unit as much as fully scattered ones.  Row
// stride DIM + 4: the 16-byte reads of up to 8 nodes at the same offset fall into different banks.
constexpr int kTopNodes = 255;  // levels 0-7 of a complete tree

template <int METRIC, int DIM>
__global__ void __launch_bounds__(512) k_tsvq_descend_reg(const float *__restrict__ x, int64_t n, int64_t ld,
                                                         const float *__restrict__ cen,
                                                         const float *__restrict__ cnorm,
                                                         const int *__restrict__ left,
                                                         const int *__restrict__ right, int n_nodes,
                                                         int *__restrict__ leaf) {
    constexpr int TS = DIM + 4;
    // The centroids of the first nodes are staged once per workgroup; the workgroup then walks over
    // batches of 8 x 64 rows (grid: one workgroup per compute unit), every lane fetching its own
    // row with 16-byte loads, all of them in flight together.
    constexpr int kTopFloats = kTopNodes * TS;
    __shared__ float lds[kTopFloats];
    __shared__ int lds_child[2 * kTopNodes];  // children of the staged nodes: the walk's dependent reads stay in LDS
    const int lane = threadIdx.x & 63;
    float *top = lds;
    const int ntop = n_nodes < kTopNodes ? n_nodes : kTopNodes;
    __shared__ float lds_cn[kTopNodes];  // their norms (cosine)
    for (int e = threadIdx.x; e < ntop; e += 512) {
        lds_child[2 * e] = left[e];
        lds_child[2 * e + 1] = right[e];
        if constexpr (METRIC == M_COS) lds_cn[e] = cnorm[e];
    }
    for (int e = threadIdx.x; e < ntop * (DIM / 4); e += 512) {
        const int nd = e / (DIM / 4), pc = e % (DIM / 4);
        *reinterpret_cast<float4 *>(&top[nd * TS + pc * 4]) =
            *reinterpret_cast<const float4 *>(cen + (size_t)nd * DIM + pc * 4);
    }
    __syncthreads();
    const int64_t nbatch = (n + 63) / 64;
    for (int64_t batch = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 6); batch < nbatch; batch += (int64_t)gridDim.x * 8) {
    const int64_t row0 = batch * 64;  // one wave = 64 rows
    float xr[DIM];
    {
        const int64_t row = row0 + lane < n ? row0 + lane : n - 1;  // past the end: the last row, not stored
        const float4 *xp = reinterpret_cast<const float4 *>(x + row * ld);
#pragma unroll
        for (int q = 0; q < DIM / 4; ++q) {
            const float4 v = xp[q];
            xr[q * 4 + 0] = v.x;
            xr[q * 4 + 1] = v.y;
            xr[q * 4 + 2] = v.z;
            xr[q * 4 + 3] = v.w;
        }
    }
    float na = 0.0f;
    if constexpr (METRIC == M_COS) {
        float sa = 0.0f;
#pragma unroll
        for (int t = 0; t < DIM; ++t) {
            float p = xr[t] * xr[t];
            sa = sa + p;
        }
        na = sqrtf(sa);
    }
    int node = 0;
    bool active = row0 + lane < n;
    while (__any(active)) {
        int l = -1, r = -1;
        if (active) {
            if (node < ntop) {
                l = lds_child[2 * node];
                r = lds_child[2 * node + 1];
            } else {
                l = left[node];
                r = right[node];
            }
        }
        const bool both = l >= 0 && r >= 0;
        // every lane that compares two children finds them in LDS: the whole wave reads there
        if (!__any(both && (l >= ntop || r >= ntop))) {
            if (both) {
                const float *pl = &top[l * TS], *pr = &top[r * TS];
                float al = 0.0f, ar = 0.0f;
#pragma unroll
                for (int q = 0; q < DIM / 4; ++q) {
                    const float4 a = *reinterpret_cast<const float4 *>(pl + q * 4);
                    const float4 b = *reinterpret_cast<const float4 *>(pr + q * 4);
                    tsvq_step<METRIC>(al, ar, xr[q * 4 + 0], a.x, b.x);
                    tsvq_step<METRIC>(al, ar, xr[q * 4 + 1], a.y, b.y);
                    tsvq_step<METRIC>(al, ar, xr[q * 4 + 2], a.z, b.z);
                    tsvq_step<METRIC>(al, ar, xr[q * 4 + 3], a.w, b.w);
                }
                float dl, dr;
                if constexpr (METRIC == M_COS) {
                    float nl = lds_cn[l], nr = lds_cn[r];
                    float ql = al / (na * nl), qr = ar / (na * nr);
                    dl = (na == 0.0f || nl == 0.0f) ? 1.0f : 1.0f - ql;
                    dr = (na == 0.0f || nr == 0.0f) ? 1.0f : 1.0f - qr;
                } else if constexpr (METRIC == M_EUCLID) {
                    dl = sqrtf(al);
                    dr = sqrtf(ar);
                } else {
                    dl = al;
                    dr = ar;
                }
                node = (dl <= dr) ? l : r;
            } else if (l >= 0) {
                node = l;
            } else if (r >= 0) {
                node = r;
            } else {
                active = false;
            }
            continue;
        }
        if (both) {
            const float4 *pl = reinterpret_cast<const float4 *>(cen + (size_t)l * DIM);
            const float4 *pr = reinterpret_cast<const float4 *>(cen + (size_t)r * DIM);
            float al = 0.0f, ar = 0.0f;
            float4 bl[2][4], br[2][4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                bl[0][q] = pl[q];
                br[0][q] = pr[q];
            }
#pragma unroll
            for (int c = 0; c < DIM / 16; ++c) {
                if (c + 1 < DIM / 16) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        bl[(c + 1) & 1][q] = pl[(c + 1) * 4 + q];
                        br[(c + 1) & 1][q] = pr[(c + 1) * 4 + q];
                    }
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 a = bl[c & 1][q], b = br[c & 1][q];
                    tsvq_step<METRIC>(al, ar, xr[c * 16 + q * 4 + 0], a.x, b.x);
                    tsvq_step<METRIC>(al, ar, xr[c * 16 + q * 4 + 1], a.y, b.y);
                    tsvq_step<METRIC>(al, ar, xr[c * 16 + q * 4 + 2], a.z, b.z);
                    tsvq_step<METRIC>(al, ar, xr[c * 16 + q * 4 + 3], a.w, b.w);
                }
            }
            float dl, dr;
            if constexpr (METRIC == M_COS) {
                float nl = cnorm[l], nr = cnorm[r];
                float ql = al / (na * nl), qr = ar / (na * nr);
                dl = (na == 0.0f || nl == 0.0f) ? 1.0f : 1.0f - ql;
                dr = (na == 0.0f || nr == 0.0f) ? 1.0f : 1.0f - qr;
            } else if constexpr (METRIC == M_EUCLID) {
                dl = sqrtf(al);
                dr = sqrtf(ar);
            } else {
                dl = al;
                dr = ar;
            }
            node = (dl <= dr) ? l : r;
        } else if (l >= 0) {
            node = l;
        } else if (r >= 0) {
            node = r;
        } else {
            active = false;
        }
    }
    if (row0 + lane < n) leaf[row0 + lane] = node;
    }  // batches
}

// ---- descent decided by one inner product per node, exact where that cannot decide ---------------
// Cosine: the reference goes left iff dl <= dr with dl = 1 - (x.cl) / (|x| |cl|) (src/tsvq.rs:167-171,
// src/distances.rs:141-151), which in exact arithmetic is the sign of x.w, w = cl / |cl| - cr / |cr|.
// Squared Euclidean and Euclidean: the sign of x.w + b, w = 2 (cl - cr), b = |cr|^2 - |cl|^2.  So a
// node costs one vector of the table below instead of two centroids, and one chain of fused
// multiply-adds instead of two of rounded products.  The rounded sums of the reference can only
// differ from that sign when the value is small, and how small is bounded (u = 2^-24, D <= 128):
//   cosine   each of dl, dr is within 133.2 u of its exact value (129 u for the sequential sum of D
//            rounded products, relative to |x| |c|; 2 u for the product of the norms and the division;
//            2 u for 1 - q), the computed x.w within 260.1 u |x| of the exact one (4 u |x| from the
//            rounding of w, 256 u |x| from the sum): |x.w| > 600 u na decides, na the computed |x|.
//   L2       each of the sums within 131 u of its exact value, relatively; the roots of two sums that
//            differ by more than 6 u, relatively, differ after rounding; the computed x.w + b within
//            131 u S of the exact one, S = 4 |x|^2 + 2 (|cl|^2 + |cr|^2) >= both sums together:
//            |x.w + b| > 300 u (4 x2 + s) decides, x2 the computed |x|^2, s rounded up.
// Everything else — near ties, norms outside [1e-15, 1e15] (zero norms have their own rule in the
// reference, huge ones overflow), non-finite values (they fail the comparison) — is decided for that
// lane by the two sums in the reference's order, read from global memory.  Manhattan has no such form
// and keeps the two-centroid kernel.
constexpr float kDescendCosMargin = 600.0f * 5.9604644775390625e-08f;
constexpr float kDescendL2Margin = 300.0f * 5.9604644775390625e-08f;

// Tables for the nodes below kTopNodes, one wave per node: w[node][DIM], and per node
//   cosine: sc[node] = kDescendCosMargin, or +inf when a child's norm is outside [1e-15, 1e15]
//   L2:     sc[2 node] = b, sc[2 node + 1] = kDescendL2Margin * s (+inf when s is not in [1e-30, 1e30])
// Nodes without two children get zeros and +inf (they are never consulted).
template <bool COS>
static __global__ void __launch_bounds__(64) k_tsvq_wtable(const float *__restrict__ cen,
                                                           const float *__restrict__ cnorm,
                                                           const int *__restrict__ left,
                                                           const int *__restrict__ right, int dim,
                                                           float *__restrict__ w, float *__restrict__ sc) {
    const int node = blockIdx.x, lane = threadIdx.x;
    const int l = left[node], r = right[node];
    const bool both = l >= 0 && r >= 0;
    const float inf = __builtin_inff();
    if (!both) {
        for (int t = lane; t < dim; t += 64) w[(size_t)node * dim + t] = 0.0f;
        if (lane == 0) {
            if (COS) {
                sc[node] = inf;
            } else {
                sc[2 * node] = 0.0f;
                sc[2 * node + 1] = inf;
            }
        }
        return;
    }
    const float *cl = cen + (size_t)l * dim, *cr = cen + (size_t)r * dim;
    if constexpr (COS) {
        const float nl = cnorm[l], nr = cnorm[r];
        for (int t = lane; t < dim; t += 64) {
            const float a = cl[t] / nl, b = cr[t] / nr;
            w[(size_t)node * dim + t] = a - b;
        }
        const bool ok = nl >= 1e-15f && nl <= 1e15f && nr >= 1e-15f && nr <= 1e15f;
        if (lane == 0) sc[node] = ok ? kDescendCosMargin : inf;
    } else {
        double sl = 0.0, sr = 0.0;
        for (int t = lane; t < dim; t += 64) {
            const float a = cl[t], b = cr[t];
            w[(size_t)node * dim + t] = 2.0f * (a - b);
            sl += (double)a * (double)a;
            sr += (double)b * (double)b;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            sl += __shfl_xor(sl, off);
            sr += __shfl_xor(sr, off);
        }
        if (lane == 0) {
            const double s = 2.0 * (sl + sr);
            const bool ok = s >= 1e-30 && s <= 1e30;  // false for NaN
            sc[2 * node] = (float)(sr - sl);
            sc[2 * node + 1] = ok ? (float)(s * 1.000001) * kDescendL2Margin : inf;
        }
    }
}

// The walk of k_tsvq_descend_reg with the decision above: the table of the first kTopNodes nodes
// in LDS (same layout and stride), the row in registers.  METRIC: M_SQ, M_EUCLID or M_COS.
template <int METRIC, int DIM>
__global__ void __launch_bounds__(512) k_tsvq_descend_w(const float *__restrict__ x, int64_t n, int64_t ld,
                                                       const float *__restrict__ cen,
                                                       const float *__restrict__ cnorm,
                                                       const int *__restrict__ left,
                                                       const int *__restrict__ right, int n_nodes,
                                                       const float *__restrict__ wtab,
                                                       const float *__restrict__ sctab, int *__restrict__ leaf) {
    constexpr int TS = DIM + 4;
    constexpr bool COS = METRIC == M_COS;
    __shared__ float top[kTopNodes * TS];
    __shared__ int lds_child[2 * kTopNodes];
    __shared__ float lds_sc[2 * kTopNodes];
    const int lane = threadIdx.x & 63;
    const int ntop = n_nodes < kTopNodes ? n_nodes : kTopNodes;
    for (int e = threadIdx.x; e < ntop; e += 512) {
        lds_child[2 * e] = left[e];
        lds_child[2 * e + 1] = right[e];
        if constexpr (COS) {
            lds_sc[e] = sctab[e];
        } else {
            lds_sc[2 * e] = sctab[2 * e];
            lds_sc[2 * e + 1] = sctab[2 * e + 1];
        }
    }
    for (int e = threadIdx.x; e < ntop * (DIM / 4); e += 512) {
        const int nd = e / (DIM / 4), pc = e % (DIM / 4);
        *reinterpret_cast<float4 *>(&top[nd * TS + pc * 4]) =
            *reinterpret_cast<const float4 *>(wtab + (size_t)nd * DIM + pc * 4);
    }
    __syncthreads();
    const int64_t nbatch = (n + 63) / 64;
    for (int64_t batch = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 6); batch < nbatch; batch += (int64_t)gridDim.x * 8) {
        const int64_t row0 = batch * 64;  // one wave = 64 rows
        float xr[DIM];
        {
            const int64_t row = row0 + lane < n ? row0 + lane : n - 1;  // past the end: the last row, not stored
            const float4 *xp = reinterpret_cast<const float4 *>(x + row * ld);
#pragma unroll
            for (int q = 0; q < DIM / 4; ++q) {
                const float4 v = xp[q];
                xr[q * 4 + 0] = v.x;
                xr[q * 4 + 1] = v.y;
                xr[q * 4 + 2] = v.z;
                xr[q * 4 + 3] = v.w;
            }
        }
        // |x|^2 in the reference's order (the exact step's cosine needs it so; the margins take it as it is)
        float sa = 0.0f;
#pragma unroll
        for (int t = 0; t < DIM; ++t) {
            float p = xr[t] * xr[t];
            sa = sa + p;
        }
        const float na = sqrtf(sa);
        // the row's own share of the margin; a row whose norm is out of range (or not finite) never
        // passes the test: +inf
        const float inf = __builtin_inff();
        float mrow;
        if constexpr (COS)
            mrow = (na >= 1e-15f && na <= 1e15f) ? na : inf;
        else
            mrow = (sa <= 1e30f) ? 4.0f * kDescendL2Margin * sa : inf;  // false for NaN
        int node = 0;
        bool active = row0 + lane < n;
        while (__any(active)) {
            int l = -1, r = -1;
            if (active) {
                if (node < ntop) {
                    l = lds_child[2 * node];
                    r = lds_child[2 * node + 1];
                } else {
                    l = left[node];
                    r = right[node];
                }
            }
            const bool both = l >= 0 && r >= 0;
            bool undecided = both;
            if (both && node < ntop) {
                const float *pw = &top[node * TS];
                float f0 = 0.0f, f1 = 0.0f, f2 = 0.0f, f3 = 0.0f;
#pragma unroll
                for (int q = 0; q < DIM / 4; ++q) {
                    const float4 a = *reinterpret_cast<const float4 *>(pw + q * 4);
                    f0 = __builtin_fmaf(xr[q * 4 + 0], a.x, f0);
                    f1 = __builtin_fmaf(xr[q * 4 + 1], a.y, f1);
                    f2 = __builtin_fmaf(xr[q * 4 + 2], a.z, f2);
                    f3 = __builtin_fmaf(xr[q * 4 + 3], a.w, f3);
                }
                float f = (f0 + f1) + (f2 + f3);
                float theta;
                if constexpr (COS) {
                    theta = lds_sc[node] * mrow;
                } else {
                    f += lds_sc[2 * node];
                    theta = lds_sc[2 * node + 1] + mrow;
                }
                // (inf * 0 and inf - inf give NaN, which fails both tests)
                if (f > theta) {
                    node = l;
                    undecided = false;
                } else if (f < -theta) {
                    node = r;
                    undecided = false;
                }
            } else if (!both) {
                if (l >= 0)
                    node = l;
                else if (r >= 0)
                    node = r;
                else
                    active = false;
            }
            if (__any(undecided)) {
                if (undecided) {
                    // the two sums in the reference's order (src/tsvq.rs:167-171), from global memory
                    const float4 *pl = reinterpret_cast<const float4 *>(cen + (size_t)l * DIM);
                    const float4 *pr = reinterpret_cast<const float4 *>(cen + (size_t)r * DIM);
                    float al = 0.0f, ar = 0.0f;
#pragma unroll
                    for (int q = 0; q < DIM / 4; ++q) {
                        const float4 a = pl[q], b = pr[q];
                        tsvq_step<METRIC>(al, ar, xr[q * 4 + 0], a.x, b.x);
                        tsvq_step<METRIC>(al, ar, xr[q * 4 + 1], a.y, b.y);
                        tsvq_step<METRIC>(al, ar, xr[q * 4 + 2], a.z, b.z);
                        tsvq_step<METRIC>(al, ar, xr[q * 4 + 3], a.w, b.w);
                    }
                    float dl, dr;
                    if constexpr (COS) {
                        float nl = cnorm[l], nr = cnorm[r];
                        float ql = al / (na * nl), qr = ar / (na * nr);
                        dl = (na == 0.0f || nl == 0.0f) ? 1.0f : 1.0f - ql;
                        dr = (na == 0.0f || nr == 0.0f) ? 1.0f : 1.0f - qr;
                    } else if constexpr (METRIC == M_EUCLID) {
                        dl = sqrtf(al);
                        dr = sqrtf(ar);
                    } else {
                        dl = al;
                        dr = ar;
                    }
                    node = (dl <= dr) ? l : r;
                }
            }
        }
        if (row0 + lane < n) leaf[row0 + lane] = node;
    }  // batches
}

// out[i][t] = f16(centroid[leaf[i]][t])   (src/tsvq.rs:242-248)
static __global__ void __launch_bounds__(256) k_tsvq_decode_f16(const int *__restrict__ leaf, int64_t n, int dim,
                                                         const float *__restrict__ cen,
                                                         uint16_t *__restrict__ out) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n * dim) return;
    int64_t row = i / dim;
    int t = (int)(i % dim);
    out[i] = __half_as_ushort(__float2half_rn(cen[(size_t)leaf[row] * dim + t]));
}

// Four consecutive components per thread (dim a multiple of 4, 16-byte aligned centroids and output).
static __global__ void __launch_bounds__(256) k_tsvq_decode4_f16(const int *__restrict__ leaf, int64_t n, int dim,
                                                          const float *__restrict__ cen,
                                                          uint2 *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int dim4 = dim / 4;
    if (i >= n * dim4) return;
    const int64_t row = i / dim4;
    const int t = (int)(i % dim4) * 4;
    const float4 v = *reinterpret_cast<const float4 *>(cen + (size_t)leaf[row] * dim + t);
    uint2 o;
    o.x = (uint32_t)__half_as_ushort(__float2half_rn(v.x)) | ((uint32_t)__half_as_ushort(__float2half_rn(v.y)) << 16);
    o.y = (uint32_t)__half_as_ushort(__float2half_rn(v.z)) | ((uint32_t)__half_as_ushort(__float2half_rn(v.w)) << 16);
    out[i] = o;
}

}  // namespace vq
