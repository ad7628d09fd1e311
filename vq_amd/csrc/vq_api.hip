// libvqhip — host side of the C ABI declared in include/vq_hip.h.
// Compile with: hipcc --offload-arch=gfx950 -O3 -ffp-contract=off
//               -Xclang -target-feature -Xclang -packed-fp32-ops
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hip_fp16.h>

#include <algorithm>
#include <cstdarg>
#include <type_traits>
#include <cstdio>
#include <cstring>
#include <string>
#include <atomic>
#include <mutex>
#include <thread>
#include <vector>

#include "ctx.hpp"
#include "assign_exact.hpp"
#include "assign_mfma.hpp"

#ifndef VQ_MFMA_RUN
#define VQ_MFMA_RUN 8    // tiles of 32 rows per wave in the matrix-core assignment (a power of two)
#endif
#ifndef VQ_MFMA_WGS
#define VQ_MFMA_WGS 3072 // workgroups of the matrix-core assignment: four rounds of three per compute unit
#endif
#include "lbg_update.hpp"
#include "calibrate.hpp"

namespace vqh {
std::string &create_error() {
    thread_local std::string e;
    return e;
}
}  // namespace vqh

using namespace vqh;

namespace {

// ---- the scratch of vq_assign_noalloc --------------------------------------------------------
// One array per GPU, held from the moment the library is loaded on that GPU until the process
// ends.  Host code never uses the array's name as an address: vq_ctx_create asks the runtime for
// the device address once per context (hipGetSymbolAddress, with the context's device current)
// and everything else goes through that pointer.
constexpr size_t kNoAllocTabBytes = 1u << 20;       // A operands: 64 bytes per (column block, padded centroid)
constexpr int kNoAllocMaxCells = 16384;             // column blocks x centroids (padded to 64) the tables hold
constexpr int kNoAllocMaxM = 1024;
constexpr size_t kNoAllocAuxOff = kNoAllocTabBytes;                                   // maxc2 [m], mu [m][8]
constexpr size_t kNoAllocStatOff = kNoAllocAuxOff + 9 * sizeof(float) * kNoAllocMaxM + 256;  // counters
constexpr size_t kNoAllocNormOff = kNoAllocStatOff + sizeof(uint32_t) * vq::kStatSlots * vq::kStatStride;
constexpr size_t kNoAllocBytes = kNoAllocNormOff + sizeof(float) * kNoAllocMaxCells;  // centroid norms (cosine)
static_assert(kNoAllocStatOff % 256 == 0 && kNoAllocNormOff % 256 == 0, "scratch areas stay 256-byte aligned");
static __device__ __align__(256) unsigned char scratch[kNoAllocBytes];
// The context whose calls used a GPU's array last (null: none yet).  Another context may take the
// array over once everything on that context's stream has finished; until then its calls are
// refused, because their kernels would overwrite tables that kernels in flight still read.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
vq_ctx *g_scratch_owner[kMaxDevices];

// ---- assignment dispatch -------------------------------------------------------------------

template <int METRIC, bool LBG>
int32_t launch_wide_exact(vq_ctx *ctx, const vq::AssignArgs &a, int sd, const uint32_t *list,
                          const uint32_t *count, const uint2 *pairs = nullptr, const uint32_t *pair_count = nullptr);

template <int SD, int G, int METRIC, bool LBG>
int32_t launch_static(vq_ctx *ctx, const vq::AssignArgs &a) {
    size_t lds = (size_t)G * a.k * SD * sizeof(float);
    if (METRIC == vq::M_COS) lds += (size_t)G * a.k * sizeof(float);
    auto kern = vq::k_assign_static<SD, G, METRIC, LBG>;
    if (lds > 48 * 1024)
        VQ_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    int64_t tiles = (a.n + 255) / 256;
    int64_t blocks = tiles * (a.m / G);
    if (blocks > 0x7fffffffLL) return fail(ctx, VQ_ERR_UNSUPPORTED, "grid too large");
    {
        ProfSpan sp(ctx, VQ_PROF_ASSIGN_KERNEL);
        hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), lds, ctx->stream, a);
    }
    VQ_HIP(ctx, hipGetLastError());
    return VQ_OK;
}

template <int SD, int METRIC, bool LBG>
int32_t launch_static_g(vq_ctx *ctx, const vq::AssignArgs &a) {
    // G column blocks per lane: as many as keep the lane's floats within 32 registers and the
    // codebooks within 64 KB of LDS.
    size_t per = (size_t)a.k * SD * sizeof(float) + (METRIC == vq::M_COS ? a.k * sizeof(float) : 0);
    if constexpr (SD * 4 <= 32) {
        if (a.m % 4 == 0 && 4 * per <= 64 * 1024) return launch_static<SD, 4, METRIC, LBG>(ctx, a);
    }
    if constexpr (SD * 2 <= 32) {
        if (a.m % 2 == 0 && 2 * per <= 64 * 1024) return launch_static<SD, 2, METRIC, LBG>(ctx, a);
    }
    return launch_static<SD, 1, METRIC, LBG>(ctx, a);
}

template <int METRIC, bool LBG>
int32_t launch_assign_m(vq_ctx *ctx, const vq::AssignArgs &a, int sd) {
    size_t per = (size_t)a.k * sd * sizeof(float) + a.k * sizeof(float);
    if (per <= 64 * 1024) {
        switch (sd) {
        case 1: return launch_static_g<1, METRIC, LBG>(ctx, a);
        case 2: return launch_static_g<2, METRIC, LBG>(ctx, a);
        case 3: return launch_static_g<3, METRIC, LBG>(ctx, a);
        case 4: return launch_static_g<4, METRIC, LBG>(ctx, a);
        case 5: return launch_static_g<5, METRIC, LBG>(ctx, a);
        case 6: return launch_static_g<6, METRIC, LBG>(ctx, a);
        case 8: return launch_static_g<8, METRIC, LBG>(ctx, a);
        case 12: return launch_static_g<12, METRIC, LBG>(ctx, a);
        case 16: return launch_static_g<16, METRIC, LBG>(ctx, a);
        case 32: return launch_static_g<32, METRIC, LBG>(ctx, a);
        default: break;
        }
    }
    if (a.m > 65535) return fail(ctx, VQ_ERR_UNSUPPORTED, "m too large for the generic kernel");
    if (sd >= 24) {
        ProfSpan sp(ctx, VQ_PROF_ASSIGN_KERNEL);
        return launch_wide_exact<METRIC, LBG>(ctx, a, sd, nullptr, nullptr);
    }
    hipLaunchKernelGGL((vq::k_assign_dyn<METRIC, LBG>), dim3(cdiv(a.n, 256), (unsigned)a.m),
                       dim3(256), 0, ctx->stream, a, sd);
    VQ_HIP(ctx, hipGetLastError());
    return VQ_OK;
}

// 8-float column blocks: bf16-split scores on the matrix cores, undecided rows resolved in the
// same kernel by the reference-order argmin (assign_mfma.hpp).
// Where the tables of k_assign_mfma_bf live in the workspace.
struct MfmaTabPtrs {
    vq::u32x4 *atab;
    float *maxc2, *mu;
    uint32_t *stat;
    int nb;
};
int32_t mfma_tab_ptrs(vq_ctx *ctx, int m, int k, MfmaTabPtrs &t) {
    t.nb = 2 * ((k + 63) / 64);  // blocks of 32 centroids, an even number (the kernel scores them in pairs)
    // A operands: 2 x 64 lanes x 16 bytes per (s, block of 32 centroids)
    const size_t n_atab = (size_t)m * t.nb * 512;
    if (ctx->no_alloc) {  // the fixed scratch array; vq_assign_noalloc has checked that the shape fits
        t.atab = (vq::u32x4 *)ctx->static_scratch;
        t.maxc2 = (float *)(ctx->static_scratch + kNoAllocAuxOff);
        t.mu = t.maxc2 + m;
        t.stat = (uint32_t *)(ctx->static_scratch + kNoAllocStatOff);
        return VQ_OK;
    }
    VQ_TRY(ensure(ctx, ctx->mfma_tab, sizeof(float) * (n_atab + 9 * (size_t)m) + 64));
    VQ_TRY(ensure(ctx, ctx->mfma_stat, sizeof(uint32_t) * vq::kStatSlots * vq::kStatStride));
    float *atab = (float *)ctx->mfma_tab.p;
    t.atab = (vq::u32x4 *)atab;
    t.maxc2 = atab + n_atab;
    t.mu = t.maxc2 + m;
    t.stat = (uint32_t *)ctx->mfma_stat.p;
    return VQ_OK;
}

// tables_ready: the caller's last kernel has already written the tables of these centroids.
// Events ride on the kernel's own dispatch (hipExtLaunchKernelGGL) instead of being recorded
// around it: a record is a packet of its own on the queue and delays the next kernel by several
// microseconds.  With timing on, the kernel's start and stop events are a span of the kernel
// class; started / done (if asked for) receive events that mark the kernel's start and end —
// done is what another stream waits for — or stay null when the launch carries none.
template <int METRIC, bool LBG>
int32_t launch_mfma(vq_ctx *ctx, const vq::AssignArgs &a, bool tables_ready, hipEvent_t *started = nullptr,
                    hipEvent_t *done = nullptr) {
    MfmaTabPtrs t;
    VQ_TRY(mfma_tab_ptrs(ctx, a.m, a.k, t));
    const int nb = t.nb;
    if (!tables_ready)
        hipLaunchKernelGGL(vq::k_mfma_bf_prep, dim3(a.m), dim3(256), 0, ctx->stream, a.cb, a.m, a.k, nb, t.atab,
                           t.maxc2, t.mu, t.stat);
    vq::MfmaBfTables tb{(const vq::u32x4 *)t.atab, t.maxc2, t.mu, t.stat, nb};
    // a workgroup = 4 column blocks of 8 floats (one 128-byte line per row) against one run of row
    // tiles, or, where m is not a multiple of 4, one column block against four runs
    const bool grouped = a.m % 4 == 0, full = nb == 8;
    const void *kern =
        grouped ? (full ? (const void *)vq::k_assign_mfma_bf<METRIC, LBG, 4, true> : (const void *)vq::k_assign_mfma_bf<METRIC, LBG, 4, false>)
                : (full ? (const void *)vq::k_assign_mfma_bf<METRIC, LBG, 1, true> : (const void *)vq::k_assign_mfma_bf<METRIC, LBG, 1, false>);
    // A wave loads the operands of its column block once (16 KB + 8 KB) and amortises them over
    // its run: 8 tiles of 32 rows where that still leaves several rounds of workgroups per compute unit.
    const int64_t tiles = cdiv(a.n, 32);
    const int64_t groups = grouped ? a.m / 4 : a.m;
    int run_tiles = VQ_MFMA_RUN;
    while (run_tiles > 1 && cdiv(tiles, (grouped ? 1 : 4) * run_tiles) * groups < 8192) run_tiles >>= 1;
    int64_t runs = cdiv(tiles, (grouped ? 1 : 4) * (int64_t)run_tiles);
    // a workgroup walks over several runs with the operands it has loaded once; the grid is a few
    // rounds of the three workgroups a compute unit holds (768: the slowest workgroup sets the
    // time; one workgroup per run: the operands are loaded 15,000 times), a multiple of 8 per group
    int64_t run_stride = std::max<int64_t>(8, (VQ_MFMA_WGS / groups) / 8 * 8);
    run_stride = std::min<int64_t>(run_stride, cdiv(runs, 8) * 8);
    const int64_t blocks = run_stride * groups;
    if (blocks >= (1LL << 31)) return fail(ctx, VQ_ERR_UNSUPPORTED, "n * m too large for one launch");
    hipEvent_t ev_a = nullptr, ev_b = nullptr;
    if (ctx->prof_on) {
        ev_a = prof_event(ctx);
        ev_b = prof_event(ctx);
        ctx->prof_open.push_back({VQ_PROF_ASSIGN_KERNEL, ev_a, ev_b, true, true});
    } else if (done) {
        ev_b = ctx->ev_fork;
    }
    vq::AssignArgs aa = a;
    void *args[] = {&aa, &tb, &run_tiles, &runs, &run_stride};
    if (ev_a || ev_b)
        VQ_HIP(ctx, hipExtLaunchKernel(kern, dim3((unsigned)blocks), dim3(256), args, 0, ctx->stream, ev_a, ev_b, 0u));
    else
        VQ_HIP(ctx, hipLaunchKernel(kern, dim3((unsigned)blocks), dim3(256), args, 0, ctx->stream));
    VQ_HIP(ctx, hipGetLastError());
    if (started) *started = ev_a;
    if (done) *done = ev_b;
    ctx->recheck_src = ctx->no_alloc ? 3 : 1;
    return VQ_OK;
}

// Exact assignment for wide column blocks, on a row range (list == nullptr) or on the list of
// undecided pairs of the matrix-core pass.
template <int METRIC, bool LBG>
int32_t launch_wide_exact(vq_ctx *ctx, const vq::AssignArgs &a, int sd, const uint32_t *list,
                          const uint32_t *count, const uint2 *pairs, const uint32_t *pair_count) {
    const bool vec = sd % 4 == 0 && (reinterpret_cast<uintptr_t>(a.cb) & 15) == 0;
    const bool listed = list != nullptr;
    size_t lds = sizeof(float) * 4 * vq::kWideRows * (size_t)sd;
    // a handful of listed pairs: one per workgroup, the row and slices of every centroid in LDS
    if (listed) lds = std::max(lds, sizeof(float) * ((size_t)sd + vq::kPairWgLdsFloats));
    // ... or eight rows of a single column block per workgroup
    if (listed && a.m == 1) lds = std::max(lds, sizeof(float) * ((size_t)vq::kRowsWg * sd + vq::kRowsWgLdsFloats));
    if (lds > 160 * 1024) return fail(ctx, VQ_ERR_UNSUPPORTED, "sub_dim %d too large", sd);
    auto pick = [&](auto L, auto V) {
        constexpr bool LISTED = decltype(L)::value, VEC = decltype(V)::value;
        return reinterpret_cast<const void *>(vq::k_assign_wide_exact<METRIC, LBG, LISTED, VEC>);
    };
    const void *kern = listed ? (vec ? pick(std::true_type{}, std::true_type{}) : pick(std::true_type{}, std::false_type{}))
                              : (vec ? pick(std::false_type{}, std::true_type{}) : pick(std::false_type{}, std::false_type{}));
    if (lds > 48 * 1024)
        VQ_HIP(ctx, hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    const int64_t groups = (a.n + vq::kWideRows - 1) / vq::kWideRows;
    dim3 grid(listed ? 2048u : (unsigned)std::min<int64_t>((groups + 3) / 4, 1 << 20), listed ? 1u : (unsigned)a.m);
    unsigned exact_blocks = grid.x;
    if (pairs) grid.x += 1024u;  // the workgroups of the two-candidate list (they come first in the grid)
    vq::AssignArgs aa = a;
    int sdv = sd;
    void *args[] = {&aa, &sdv, (void *)&list, (void *)&count, (void *)&pairs, (void *)&pair_count, &exact_blocks};
    VQ_HIP(ctx, hipLaunchKernel(kern, grid, dim3(256), args, lds, ctx->stream));
    return VQ_OK;
}

// Wide column blocks (sub_dim a multiple of 8 above 8): chunked contraction on the bf16 matrix
// cores with split operands, undecided pairs listed for the exact kernel.
template <int METRIC, bool LBG>
int32_t launch_mfma_wide(vq_ctx *ctx, const vq::AssignArgs &a, int sd) {
    const int nb = (a.k + 31) / 32, nkc = sd / 8, nsl = (sd + 31) / 32;
    // A operands: 2 x 64 lanes x 16 bytes per (s, 16 dimensions, block of 32 centroids)
    const size_t n_atab = (size_t)a.m * ((sd + 15) / 16) * nb * 128 * 4, n_c2 = (size_t)a.m * nb * 32;  // floats
    VQ_TRY(ensure(ctx, ctx->mfma_tab, sizeof(float) * (n_atab + n_c2 + (size_t)a.m * nb + (size_t)a.m * sd + a.m + 2 * (size_t)a.m * nsl + 8) + 64));
    // header (two counts), the list for the all-centroid check, the list for the two-candidate check
    const size_t n_pairs = (size_t)a.n * a.m;
    VQ_TRY(ensure(ctx, ctx->mfma_list, sizeof(uint32_t) * (4 + ((n_pairs + 1) & ~(size_t)1) + 2 * n_pairs)));
    float *atab = (float *)ctx->mfma_tab.p;
    float *c2perm = atab + n_atab;
    float *maxc2 = c2perm + n_c2;  // per block of 32 centroids
    float *mu = maxc2 + (((size_t)a.m * nb + 3) & ~(size_t)3);  // 16-byte aligned: read as float4
    uint32_t *count = (uint32_t *)ctx->mfma_list.p;
    uint32_t *list = count + 4;
    uint2 *pairs = (uint2 *)(list + ((n_pairs + 1) & ~(size_t)1));  // 8-byte aligned
    float2 *norms = (float2 *)(mu + (size_t)a.m * sd);  // sd is a multiple of 8: 8-byte aligned
    int *shifted = (int *)(norms + (size_t)a.m * nsl);
    hipLaunchKernelGGL(vq::k_block_centres, dim3(a.m, nsl), dim3(256), 0, ctx->stream, a.cb, a.k, sd, mu, norms);
    hipLaunchKernelGGL(vq::k_mfma_wide_bf_prep, dim3(a.m, nb), dim3(256), 0, ctx->stream, a.cb, mu, norms, shifted,
                       a.m, a.k, nb, sd,
                       (vq::u32x4 *)atab, c2perm, maxc2, count);
    // two candidates, each: operand split 3 * 2^-16, fp32 accumulation (34 per 8 dimensions + 16)
    // * 2^-24 (an upper bound), rounding of the differences from the centre 2^-22
    const float kappa = 2.0f * (3.0f * 1.52587890625e-05f + (34.0f * nkc + 16.0f + 4.0f) * 5.9604644775390625e-08f);
    vq::MfmaWideBfTables tb{(const vq::u32x4 *)atab, c2perm, maxc2, mu, shifted, list, count, pairs, nb, sd, kappa};
    {
        ProfSpan sp(ctx, VQ_PROF_ASSIGN_KERNEL);
#define WIDE(NB)                                                                                             \
    if (a.pend_cb)                                                                                           \
        hipLaunchKernelGGL((vq::k_assign_mfma_wide_bf<LBG, NB, true>), dim3(cdiv(a.n, 128), (unsigned)a.m),    \
                           dim3(256), 0, ctx->stream, a, tb);                                                \
    else                                                                                                     \
        hipLaunchKernelGGL((vq::k_assign_mfma_wide_bf<LBG, NB>), dim3(cdiv(a.n, 128), (unsigned)a.m), dim3(256), 0, \
                           ctx->stream, a, tb)
        switch (nb) {
        case 1: WIDE(1); break;
        case 2: WIDE(2); break;
        case 3: WIDE(3); break;
        case 4: WIDE(4); break;
        case 5: WIDE(5); break;
        case 6: WIDE(6); break;
        case 7: WIDE(7); break;
        default: WIDE(8); break;
        }
#undef WIDE
    }
    VQ_HIP(ctx, hipGetLastError());
    ctx->recheck_src = 2;
    // undecided pairs with two candidates and the few that need every centroid, in one launch
    return launch_wide_exact<METRIC, LBG>(ctx, a, sd, list, count, (const uint2 *)pairs,
                                          (const uint32_t *)(count + 1));
}

template <int METRIC, bool LBG>
bool mfma_wide_applicable(const vq_ctx *ctx, const vq::AssignArgs &a, int sd) {
    if (ctx->assign_path == 1 || ctx->no_alloc) return false;  // its lists grow with n: not for a fixed scratch
    if (METRIC != vq::M_SQ && METRIC != vq::M_EUCLID) return false;
    if (sd < 16 || sd % 8 != 0 || a.k > 256 || a.m > 65535) return false;
    // float4 row and centroid loads; the rows of a workgroup and the operand table within 32-bit byte offsets
    if (a.ld % 4 != 0 || ((reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.cb)) & 15) != 0)
        return false;
    if (a.ld > (1 << 20) || sd > (1 << 16)) return false;
    return (int64_t)a.n * a.m < (1LL << 32);
}

template <int METRIC, bool LBG>
bool mfma_applicable(const vq_ctx *ctx, const vq::AssignArgs &a, int sd) {
    if (ctx->assign_path == 1) return false;
    if (METRIC != vq::M_SQ && METRIC != vq::M_EUCLID) return false;
    if (sd != 8 || (reinterpret_cast<uintptr_t>(a.cb) & 15) != 0) return false;  // float4 centroid loads
    // the kernel addresses the rows of a wave's run (at most 288 of them) with 32-bit offsets
    if (a.ld > (1 << 20) || a.m > (1 << 16)) return false;
    return a.k <= 256;
}

template <bool LBG>
int32_t launch_assign(vq_ctx *ctx, int metric, const vq::AssignArgs &a, int sd, bool tables_ready = false,
                      hipEvent_t *started = nullptr, hipEvent_t *done = nullptr) {
    if (started) *started = nullptr;
    if (done) *done = nullptr;
    if (metric == VQ_SQEUCLIDEAN && mfma_applicable<vq::M_SQ, LBG>(ctx, a, sd))
        return launch_mfma<vq::M_SQ, LBG>(ctx, a, tables_ready, started, done);
    if (metric == VQ_EUCLIDEAN && mfma_applicable<vq::M_EUCLID, LBG>(ctx, a, sd))
        return launch_mfma<vq::M_EUCLID, LBG>(ctx, a, tables_ready, started, done);
    if (metric == VQ_SQEUCLIDEAN && mfma_wide_applicable<vq::M_SQ, LBG>(ctx, a, sd))
        return launch_mfma_wide<vq::M_SQ, LBG>(ctx, a, sd);
    if (metric == VQ_EUCLIDEAN && mfma_wide_applicable<vq::M_EUCLID, LBG>(ctx, a, sd))
        return launch_mfma_wide<vq::M_EUCLID, LBG>(ctx, a, sd);
    switch (metric) {
    case VQ_SQEUCLIDEAN: return launch_assign_m<vq::M_SQ, LBG>(ctx, a, sd);
    case VQ_EUCLIDEAN: return launch_assign_m<vq::M_EUCLID, LBG>(ctx, a, sd);
    case VQ_COSINE: return launch_assign_m<vq::M_COS, LBG>(ctx, a, sd);
    case VQ_MANHATTAN: return launch_assign_m<vq::M_L1, LBG>(ctx, a, sd);
    default: return fail(ctx, VQ_ERR_UNSUPPORTED, "metric %d has no kernel", metric);
    }
}

template <typename CodeT>
__global__ void k_decode_f16(const CodeT *__restrict__ codes, int64_t n, int m, int sd, int k,
                             const float *__restrict__ cb, uint16_t *__restrict__ out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t dim = (int64_t)m * sd;
    if (i >= n * dim) return;
    int64_t row = i / dim;
    int c = (int)(i % dim);
    int s = c / sd, t = c % sd;
    float v = cb[((size_t)s * k + codes[row * m + s]) * sd + t];
    out[i] = __half_as_ushort(__float2half_rn(v));
}

// Four consecutive components per thread (sub_dim a multiple of 4, 16-byte aligned codebooks and
// output rows): one 16-byte load of the centroid, one 8- or 16-byte store.  F16: binary16 bit
// patterns (round to nearest even), else f32.
template <bool F16, typename CodeT>
__global__ void __launch_bounds__(256) k_decode_vec4(const CodeT *__restrict__ codes, int64_t n, int m, int sd,
                                                     int k, const float *__restrict__ cb, void *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // group of four components
    const int64_t dim4 = (int64_t)m * sd / 4;
    if (i >= n * dim4) return;
    const int64_t row = i / dim4;
    const int c = (int)(i % dim4) * 4;
    const int s = c / sd, t = c % sd;
    const float4 v = *reinterpret_cast<const float4 *>(cb + ((size_t)s * k + codes[row * m + s]) * sd + t);
    if constexpr (F16) {
        uint2 o;
        o.x = (uint32_t)__half_as_ushort(__float2half_rn(v.x)) | ((uint32_t)__half_as_ushort(__float2half_rn(v.y)) << 16);
        o.y = (uint32_t)__half_as_ushort(__float2half_rn(v.z)) | ((uint32_t)__half_as_ushort(__float2half_rn(v.w)) << 16);
        reinterpret_cast<uint2 *>(out)[i] = o;
    } else {
        reinterpret_cast<float4 *>(out)[i] = v;
    }
}

// The same gather with the whole codebook table resident in LDS (up to 128 KB, one workgroup of
// 1024 threads per compute unit walking over the output): a thread makes one 16-byte piece of the
// output per step — eight f16 values (F16; sub_dim a multiple of 8) or four f32 values (sub_dim a
// multiple of 4) — so a wave's stores are 1 KB of consecutive bytes, its code reads consecutive
// bytes, and the centroid comes from LDS instead of a scattered read of the 128 KB table through
// the vector cache.  Four pieces per thread are in flight.
template <bool F16, typename CodeT>
__global__ void __launch_bounds__(1024) k_decode_resident(const CodeT *__restrict__ codes, int64_t n, int m, int sd,
                                                          int k, const float *__restrict__ cb,
                                                          vq::u32x4 *__restrict__ out) {
    extern __shared__ __attribute__((aligned(16))) vq::u32x4 tab[];  // [m * k][pieces of a centroid]
    const int pieces = F16 ? sd / 8 : sd / 4;                        // 16-byte output pieces per centroid
    const int entries = m * k * pieces;
    for (int e = threadIdx.x; e < entries; e += 1024) {
        if constexpr (F16) {
            const float4 a = reinterpret_cast<const float4 *>(cb)[2 * (size_t)e];
            const float4 b = reinterpret_cast<const float4 *>(cb)[2 * (size_t)e + 1];
            auto two = [](float lo, float hi) {
                return (uint32_t)__half_as_ushort(__float2half_rn(lo)) | ((uint32_t)__half_as_ushort(__float2half_rn(hi)) << 16);
            };
            tab[e] = vq::u32x4{two(a.x, a.y), two(a.z, a.w), two(b.x, b.y), two(b.z, b.w)};
        } else {
            tab[e] = reinterpret_cast<const vq::u32x4 *>(cb)[e];
        }
    }
    __syncthreads();
    const int64_t total = n * m * pieces;
    const int64_t stride = (int64_t)gridDim.x * 1024;
    const int per_row = m * pieces;
    constexpr int U = F16 ? 4 : 8;  // pieces in flight per thread
    for (int64_t i0 = (int64_t)blockIdx.x * 1024 + threadIdx.x; i0 < total; i0 += U * stride) {
        uint32_t code[U];
        int64_t idx[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            idx[u] = i0 + u * stride;
            const int64_t ic = idx[u] < total ? idx[u] : i0;
            code[u] = codes[ic / pieces];  // codes are n x m row-major: piece ic belongs to (row, block) ic / pieces
        }
        vq::u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t ic = idx[u] < total ? idx[u] : i0;
            const int within = (int)(ic % per_row);  // (block, piece) of the row
            const int s = within / pieces, pc = within % pieces;
            v[u] = tab[(s * k + (int)code[u]) * pieces + pc];
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (idx[u] < total) out[idx[u]] = v[u];
    }
}

template <typename CodeT>
__global__ void k_decode_f32(const CodeT *__restrict__ codes, int64_t n, int m, int sd, int k,
                             const float *__restrict__ cb, float *__restrict__ out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t dim = (int64_t)m * sd;
    if (i >= n * dim) return;
    int64_t row = i / dim;
    int c = (int)(i % dim);
    int s = c / sd, t = c % sd;
    out[i] = cb[((size_t)s * k + codes[row * m + s]) * sd + t];
}

__global__ void __launch_bounds__(256) k_copy_f32(const float4 *__restrict__ src,
                                                  float4 *__restrict__ dst, int64_t n4,
                                                  const float *__restrict__ src_tail,
                                                  float *__restrict__ dst_tail, int tail) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * 256;
    for (; i < n4; i += stride) dst[i] = src[i];
    if (blockIdx.x == 0 && (int)threadIdx.x < tail) dst_tail[threadIdx.x] = src_tail[threadIdx.x];
}

// LDS-resident decode where the table fits and the output is large enough to pay for staging it.
template <bool F16, typename CodeT>
int32_t launch_decode_resident(vq_ctx *ctx, const CodeT *d_codes, int64_t n, int m, int sd, int k,
                               const float *d_codebooks, void *d_out, bool *done) {
    *done = false;
    const size_t lds = (size_t)m * k * sd * (F16 ? 2 : 4);
    if (sd % (F16 ? 8 : 4) != 0 || lds > 128 * 1024 || n * m < (1 << 16)) return VQ_OK;
    if ((reinterpret_cast<uintptr_t>(d_codebooks) | reinterpret_cast<uintptr_t>(d_out)) & 15) return VQ_OK;
    auto kern = k_decode_resident<F16, CodeT>;
    // the kernel's LDS limit and the number of compute units: asked for once per context and kernel
    const int slot = (F16 ? 2 : 0) + (sizeof(CodeT) == 2 ? 1 : 0);
    if ((size_t)ctx->decode_lds_set[slot] < lds) {
        VQ_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
        ctx->decode_lds_set[slot] = 128 * 1024;
    }
    if (ctx->compute_units == 0) {
        int cus = 0;
        VQ_HIP(ctx, hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, ctx->device));
        ctx->compute_units = cus > 0 ? cus : 1;
    }
    const int64_t pieces = (int64_t)n * m * (F16 ? sd / 8 : sd / 4);
    const unsigned per_cu = lds <= 64 * 1024 ? 2u : 1u;
    const unsigned wgs = (unsigned)std::min<int64_t>((int64_t)ctx->compute_units * per_cu, cdiv(pieces, 4096));
    hipLaunchKernelGGL(kern, dim3(wgs), dim3(1024), lds, ctx->stream, d_codes, n, m, sd, k, d_codebooks,
                       (vq::u32x4 *)d_out);
    VQ_HIP(ctx, hipGetLastError());
    *done = true;
    return VQ_OK;
}

// Decode of 8- or 16-bit codes to binary16 bit patterns (F16) or f32.
template <bool F16, typename CodeT>
int32_t decode_codes(vq_ctx *ctx, const CodeT *d_codes, int64_t n, int32_t m, int32_t sd, int32_t k, int32_t k_max,
                     const float *d_codebooks, void *d_out) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (n == 0) return VQ_OK;
    if (!d_codes || !d_codebooks || !d_out || n < 0 || m <= 0 || sd <= 0 || k <= 0 || k > k_max)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter");
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    bool done = false;
    VQ_TRY((launch_decode_resident<F16, CodeT>(ctx, d_codes, n, m, sd, k, d_codebooks, d_out, &done)));
    if (done) return VQ_OK;
    if (sd % 4 == 0 && ((reinterpret_cast<uintptr_t>(d_codebooks) | reinterpret_cast<uintptr_t>(d_out)) & 15) == 0)
        hipLaunchKernelGGL((k_decode_vec4<F16, CodeT>), dim3(cdiv(n * m * sd / 4, 256)), dim3(256), 0, ctx->stream,
                           d_codes, n, m, sd, k, d_codebooks, d_out);
    else if constexpr (F16)
        hipLaunchKernelGGL(k_decode_f16<CodeT>, dim3(cdiv(n * m * sd, 256)), dim3(256), 0, ctx->stream, d_codes, n, m,
                           sd, k, d_codebooks, (uint16_t *)d_out);
    else
        hipLaunchKernelGGL(k_decode_f32<CodeT>, dim3(cdiv(n * m * sd, 256)), dim3(256), 0, ctx->stream, d_codes, n, m,
                           sd, k, d_codebooks, (float *)d_out);
    VQ_HIP(ctx, hipGetLastError());
    return VQ_OK;
}

}  // namespace

namespace vqh {
int32_t check_common(vq_ctx *ctx, const void *x, int64_t n, int64_t ld, int32_t m, int32_t sd,
                     int32_t k, int32_t k_max) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (n == 0) return fail(ctx, VQ_ERR_EMPTY_INPUT, "Empty input: at least one vector is required.");
    if (!x || n < 0 || m <= 0 || sd <= 0)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: null pointer or non-positive size");
    if (ld < (int64_t)m * sd)
        return fail(ctx, VQ_ERR_DIM_MISMATCH, "Dimension mismatch: expected %lld, got %lld",
                    (long long)m * sd, (long long)ld);
    if (k <= 0) return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: k must be greater than 0");
    if (k > k_max)
        return fail(ctx, VQ_ERR_UNSUPPORTED,
                    k_max <= vq::kMaxK ? "k = %d: the codes of this entry point are uint8, k must be <= 256"
                                       : "k = %d: codes are at most 16 bits wide, k must be <= 65536", k);
    if (n >= (1LL << 32)) return fail(ctx, VQ_ERR_UNSUPPORTED, "n must be below 2^32");
    return VQ_OK;
}


bool assign_pending_fusable(const vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t sd,
                            int32_t k, const float *d_codebook) {
    vq::AssignArgs a;
    a.x = d_x;
    a.n = n;
    a.ld = ld;
    a.m = 1;
    a.k = k;
    a.cb = d_codebook;
    if (k < 1 || sd % 4 != 0) return false;
    return (metric == VQ_SQEUCLIDEAN && mfma_wide_applicable<vq::M_SQ, false>(ctx, a, sd)) ||
           (metric == VQ_EUCLIDEAN && mfma_wide_applicable<vq::M_EUCLID, false>(ctx, a, sd));
}

int32_t assign_codes(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t m,
                  int32_t sd, int32_t k, const float *d_codebooks, uint8_t *d_codes, float *d_dist,
                  bool *dist_written, const PendingUpdate *pend) {
    if (dist_written) *dist_written = false;
    VQ_TRY(check_common(ctx, d_x, n, ld, m, sd, k));
    if (!d_codebooks || !d_codes) return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: null pointer");
    if (reinterpret_cast<uintptr_t>(d_codes) & 3)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: d_codes must be 4-byte aligned");
    if (m > 65535) return fail(ctx, VQ_ERR_UNSUPPORTED, "m must be at most 65535");
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    vq::AssignArgs a;
    a.x = d_x;
    a.n = n;
    a.ld = ld;
    a.m = m;
    a.k = k;
    a.cb = d_codebooks;
    a.cnorm = nullptr;
    a.codes = d_codes;
    a.changed = nullptr;
    a.done = nullptr;
    if (pend) {
        if (m != 1 || !assign_pending_fusable(ctx, metric, d_x, n, ld, sd, k, d_codebooks) || !pend->cb ||
            !pend->codes || (reinterpret_cast<uintptr_t>(pend->cb) & 15) != 0 ||
            (pend->src && (pend->src_ld % 4 != 0 || (reinterpret_cast<uintptr_t>(pend->src) & 15) != 0)))
            return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: no pass that takes a pending update");
        a.pend_cb = pend->cb;
        a.pend_codes = pend->codes;
        a.pend_src = pend->src;
        a.pend_src_ld = pend->src_ld;
    }
    if (metric == VQ_COSINE) {
        float *cnorm = (float *)(ctx->static_scratch + kNoAllocNormOff);
        if (!ctx->no_alloc) {
            VQ_TRY(ensure(ctx, ctx->cnorm, sizeof(float) * (size_t)m * k));
            cnorm = (float *)ctx->cnorm.p;
        }
        hipLaunchKernelGGL(vq::k_centroid_norms, dim3(cdiv((int64_t)m * k, 256)), dim3(256), 0,
                           ctx->stream, d_codebooks, (int64_t)m * k, sd, cnorm);
        a.cnorm = cnorm;
    }
    // the 8-float matrix-core kernel has the chosen centroid's exact distance at hand
    if (d_dist && dist_written &&
        ((metric == VQ_SQEUCLIDEAN && mfma_applicable<vq::M_SQ, false>(ctx, a, sd)) ||
         (metric == VQ_EUCLIDEAN && mfma_applicable<vq::M_EUCLID, false>(ctx, a, sd)))) {
        a.dist = d_dist;
        *dist_written = true;
    }
    ProfSpan sp(ctx, VQ_PROF_ENCODE);
    return launch_assign<false>(ctx, metric, a, sd);
}

}  // namespace vqh

// =============================================================================================
extern "C" {

int32_t vq_ctx_create(int32_t device, vq_ctx **out) {
    if (!out) return fail(nullptr, VQ_ERR_INVALID_ARG, "out is null");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0)
        return fail(nullptr, VQ_ERR_HIP, "no HIP device available (%s)",
                    e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    if (device < 0 || device >= count)
        return fail(nullptr, VQ_ERR_INVALID_ARG, "device %d out of range [0,%d)", device, count);
    vq_ctx *ctx = new vq_ctx;
    ctx->device = device;
    if ((e = hipSetDevice(device)) != hipSuccess ||
        (e = hipStreamCreate(&ctx->stream)) != hipSuccess ||
        (e = hipEventCreate(&ctx->ev0)) != hipSuccess ||
        (e = hipEventCreate(&ctx->ev1)) != hipSuccess ||
        (e = hipStreamCreate(&ctx->side)) != hipSuccess ||
        (e = hipEventCreate(&ctx->ev_fork)) != hipSuccess ||  // rides on a kernel dispatch as its stop event
        (e = hipEventCreateWithFlags(&ctx->ev_join, hipEventDisableTiming | hipEventReleaseToDevice)) != hipSuccess) {
        int32_t rc = fail(nullptr, VQ_ERR_HIP, "context set-up failed: %s", hipGetErrorString(e));
        delete ctx;
        return rc;
    }
    // this GPU's copy of the scratch array (every GPU holds its own, at its own address)
    void *sp = nullptr;
    if ((e = hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch))) != hipSuccess || !sp) {
        int32_t rc = fail(nullptr, VQ_ERR_HIP, "address of the scratch array: %s", hipGetErrorString(e));
        vq_ctx_destroy(ctx);
        return rc;
    }
    ctx->static_scratch = (unsigned char *)sp;
    *out = ctx;
    return VQ_OK;
}

int32_t vq_ctx_destroy(vq_ctx *ctx) {
    if (!ctx) return VQ_OK;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->side) (void)hipStreamSynchronize(ctx->side);
    DevBuf *bufs[] = {&ctx->flags, &ctx->tables, &ctx->hist, &ctx->perm, &ctx->leaf_desc,
                      &ctx->leaf_sum, &ctx->codes, &ctx->idx, &ctx->reseed, &ctx->cnorm,
                      &ctx->seg, &ctx->part_sum, &ctx->mfma_tab, &ctx->mfma_list, &ctx->mfma_stat, &ctx->tsvq_sq, &ctx->tsvq_split, &ctx->tsvq_level, &ctx->tsvq_means, &ctx->tsvq_scan, &ctx->tsvq_km, &ctx->tsvq_bsum, &ctx->tsvq_segmaps, &ctx->tsvq_gsum, &ctx->tsvq_guess, &ctx->tsvq_maps, &ctx->tmp_a, &ctx->tmp_b, &ctx->tmp_c, &ctx->tmp_d, &ctx->tmp_e, &ctx->tmp_f,
                      &ctx->big_chunk, &ctx->big_win, &ctx->big_wind, &ctx->big_best, &ctx->big_fresh, &ctx->big_codes, &ctx->big_keys,
                      &ctx->big_sorted, &ctx->big_sort_tmp, &ctx->big_tables, &ctx->big_flags};
    for (DevBuf *b : bufs)
        if (b->p) (void)hipFree(b->p);
    if (ctx->tsvq_pin) (void)hipHostFree(ctx->tsvq_pin);
    for (int i = 0; i < vq_ctx::kStageBuffers; ++i) {
        if (ctx->h2d_stage[i]) (void)hipHostFree(ctx->h2d_stage[i]);
        if (ctx->h2d_event[i]) (void)hipEventDestroy(ctx->h2d_event[i]);
    }
    prof_collect(ctx);
    if (ctx->device >= 0 && ctx->device < kMaxDevices) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (g_scratch_owner[ctx->device] == ctx) g_scratch_owner[ctx->device] = nullptr;
    }
    for (hipEvent_t e : ctx->prof_pool) (void)hipEventDestroy(e);
    (void)hipEventDestroy(ctx->ev0);
    (void)hipEventDestroy(ctx->ev1);
    if (ctx->ev_fork) (void)hipEventDestroy(ctx->ev_fork);
    if (ctx->ev_join) (void)hipEventDestroy(ctx->ev_join);
    if (ctx->side) (void)hipStreamDestroy(ctx->side);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return VQ_OK;
}

const char *vq_last_error(const vq_ctx *ctx) { return ctx ? ctx->err.c_str() : vqh::create_error().c_str(); }

int32_t vq_ctx_sync(vq_ctx *ctx) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return VQ_OK;
}

void *vq_ctx_stream(vq_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int32_t vq_malloc(vq_ctx *ctx, size_t bytes, void **d_ptr) {
    if (!ctx || !d_ptr) return VQ_ERR_INVALID_ARG;
    *d_ptr = nullptr;
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    VQ_HIP(ctx, hipMalloc(d_ptr, bytes ? bytes : 1));
    return VQ_OK;
}

int32_t vq_free(vq_ctx *ctx, void *d_ptr) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (!d_ptr) return VQ_OK;
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    VQ_HIP(ctx, hipFree(d_ptr));
    return VQ_OK;
}

int32_t vq_host_alloc(vq_ctx *ctx, size_t bytes, void **h_ptr) {
    if (!ctx || !h_ptr) return VQ_ERR_INVALID_ARG;
    *h_ptr = nullptr;
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    VQ_HIP(ctx, hipHostMalloc(h_ptr, bytes ? bytes : 1, hipHostMallocDefault));
    return VQ_OK;
}

int32_t vq_host_free(vq_ctx *ctx, void *h_ptr) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (!h_ptr) return VQ_OK;
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    VQ_HIP(ctx, hipHostFree(h_ptr));
    return VQ_OK;
}

// A large upload from pageable memory: host threads stage it chunk by chunk into page-locked buffers
// while the copy engine uploads the chunk before, instead of the runtime's single-threaded staging.
static int32_t h2d_staged(vq_ctx *ctx, char *d_dst, const char *h_src, size_t bytes) {
    constexpr size_t kChunk = 16u << 20;
    constexpr int NB = vq_ctx::kStageBuffers;
    for (int i = 0; i < NB; ++i) {
        if (!ctx->h2d_stage[i]) VQ_HIP(ctx, hipHostMalloc(&ctx->h2d_stage[i], kChunk, hipHostMallocDefault));
        if (!ctx->h2d_event[i]) VQ_HIP(ctx, hipEventCreateWithFlags(&ctx->h2d_event[i], hipEventDisableTiming));
    }
    const size_t nchunks = (bytes + kChunk - 1) / kChunk;
    const unsigned hw = std::thread::hardware_concurrency();
    const int T = (int)std::min<unsigned>(8u, std::max<unsigned>(1u, hw / 2));
    std::atomic<size_t> stageable{(size_t)NB};  // chunks below this index may be staged: their buffer is free
    std::vector<std::atomic<int>> staged(nchunks);
    for (auto &a : staged) a.store(0, std::memory_order_relaxed);
    auto work = [&](int t) {
        for (size_t c = 0; c < nchunks; ++c) {
            while (c >= stageable.load(std::memory_order_acquire)) std::this_thread::yield();
            const size_t len = std::min(kChunk, bytes - c * kChunk);
            const size_t per = ((len + T - 1) / T + 63) & ~(size_t)63;
            const size_t lo = std::min(len, per * (size_t)t), hi = std::min(len, lo + per);
            if (hi > lo) memcpy((char *)ctx->h2d_stage[c % NB] + lo, h_src + c * kChunk + lo, hi - lo);
            staged[c].fetch_add(1, std::memory_order_release);
        }
    };
    // (the staging buffers may still be the source of an earlier call's uploads that failed half way)
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    std::vector<std::thread> pool;
    std::thread first;
    try {
        for (int t = 1; t < T; ++t) pool.emplace_back(work, t);
        first = std::thread(work, 0);
    } catch (const std::exception &) {
        // no threads to be had: let the ones that started run through, then one plain copy
        stageable.store(nchunks + (size_t)NB, std::memory_order_release);
        for (auto &th : pool) th.join();
        VQ_HIP(ctx, hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, ctx->stream));
        VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
        return VQ_OK;
    }
    hipError_t err = hipSuccess;
    for (size_t c = 0; c < nchunks; ++c) {
        while (staged[c].load(std::memory_order_acquire) < T) std::this_thread::yield();
        const size_t len = std::min(kChunk, bytes - c * kChunk);
        if (err == hipSuccess)
            err = hipMemcpyAsync(d_dst + c * kChunk, ctx->h2d_stage[c % NB], len, hipMemcpyHostToDevice, ctx->stream);
        if (err == hipSuccess) err = hipEventRecord(ctx->h2d_event[c % NB], ctx->stream);
        // chunk c + 1 takes the buffer of chunk c + 1 - NB: wait for that upload (on an error the
        // workers are let through to the end, nothing more is uploaded)
        if (c + 1 >= (size_t)NB && err == hipSuccess) err = hipEventSynchronize(ctx->h2d_event[(c + 1) % NB]);
        stageable.store(c + 2 > (size_t)NB ? c + 2 : (size_t)NB, std::memory_order_release);
    }
    first.join();
    for (auto &th : pool) th.join();
    if (err != hipSuccess) (void)hipStreamSynchronize(ctx->stream);  // uploads already enqueued read the staging buffers
    VQ_HIP(ctx, err);
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return VQ_OK;
}

int32_t vq_h2d(vq_ctx *ctx, void *d_dst, const void *h_src, size_t bytes) {
    if (!ctx || (bytes && (!d_dst || !h_src))) return VQ_ERR_INVALID_ARG;
    if (bytes >= (64u << 20)) {
        hipPointerAttribute_t attr;
        const bool locked = hipPointerGetAttributes(&attr, h_src) == hipSuccess && attr.type == hipMemoryTypeHost;
        (void)hipGetLastError();  // an unregistered host pointer is reported as an error: that is the pageable case
        if (!locked) return h2d_staged(ctx, (char *)d_dst, (const char *)h_src, bytes);
    }
    VQ_HIP(ctx, hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, ctx->stream));
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return VQ_OK;
}

// The other direction: the copy engine fills page-locked chunks, host threads copy the chunk before
// out to the pageable destination.
static int32_t d2h_staged(vq_ctx *ctx, char *h_dst, const char *d_src, size_t bytes) {
    constexpr size_t kChunk = 16u << 20;
    constexpr int NB = vq_ctx::kStageBuffers;
    for (int i = 0; i < NB; ++i) {
        if (!ctx->h2d_stage[i]) VQ_HIP(ctx, hipHostMalloc(&ctx->h2d_stage[i], kChunk, hipHostMallocDefault));
        if (!ctx->h2d_event[i]) VQ_HIP(ctx, hipEventCreateWithFlags(&ctx->h2d_event[i], hipEventDisableTiming));
    }
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));  // the staging buffers are idle
    const size_t nchunks = (bytes + kChunk - 1) / kChunk;
    const unsigned hw = std::thread::hardware_concurrency();
    const int T = (int)std::min<unsigned>(8u, std::max<unsigned>(1u, hw / 2));
    std::atomic<size_t> arrived{0};  // chunks below this index are in their staging buffer
    std::vector<std::atomic<int>> copied(nchunks);
    for (auto &a : copied) a.store(0, std::memory_order_relaxed);
    auto work = [&](int t) {
        for (size_t c = 0; c < nchunks; ++c) {
            while (c >= arrived.load(std::memory_order_acquire)) std::this_thread::yield();
            const size_t len = std::min(kChunk, bytes - c * kChunk);
            const size_t per = ((len + T - 1) / T + 63) & ~(size_t)63;
            const size_t lo = std::min(len, per * (size_t)t), hi = std::min(len, lo + per);
            if (hi > lo) memcpy(h_dst + c * kChunk + lo, (const char *)ctx->h2d_stage[c % NB] + lo, hi - lo);
            copied[c].fetch_add(1, std::memory_order_release);
        }
    };
    std::vector<std::thread> pool;
    try {
        for (int t = 0; t < T; ++t) pool.emplace_back(work, t);
    } catch (const std::exception &) {
        // no threads to be had: the ones that started copy nothing that is not there yet (nothing
        // has arrived), so they are let through and one plain copy does the work
        arrived.store(nchunks, std::memory_order_release);
        for (auto &th : pool) th.join();
        VQ_HIP(ctx, hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, ctx->stream));
        VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
        return VQ_OK;
    }
    hipError_t err = hipSuccess;
    size_t issued = 0;
    auto issue = [&]() {  // the download of chunk `issued` into its buffer
        const size_t len = std::min(kChunk, bytes - issued * kChunk);
        if (err == hipSuccess)
            err = hipMemcpyAsync(ctx->h2d_stage[issued % NB], d_src + issued * kChunk, len, hipMemcpyDeviceToHost, ctx->stream);
        if (err == hipSuccess) err = hipEventRecord(ctx->h2d_event[issued % NB], ctx->stream);
        ++issued;
    };
    while (issued < nchunks && issued < (size_t)NB) issue();
    for (size_t c = 0; c < nchunks; ++c) {
        if (err == hipSuccess) err = hipEventSynchronize(ctx->h2d_event[c % NB]);
        arrived.store(c + 1, std::memory_order_release);  // (on an error the workers run through: the call fails)
        if (issued < nchunks) {  // chunk c + NB takes this buffer once the threads have emptied it
            while (copied[c].load(std::memory_order_acquire) < T) std::this_thread::yield();
            issue();
        }
    }
    for (auto &th : pool) th.join();
    if (err != hipSuccess) (void)hipStreamSynchronize(ctx->stream);  // downloads already enqueued write the staging buffers
    VQ_HIP(ctx, err);
    return VQ_OK;
}

int32_t vq_d2h(vq_ctx *ctx, void *h_dst, const void *d_src, size_t bytes) {
    if (!ctx || (bytes && (!h_dst || !d_src))) return VQ_ERR_INVALID_ARG;
    if (bytes >= (64u << 20)) {
        hipPointerAttribute_t attr;
        const bool locked = hipPointerGetAttributes(&attr, h_dst) == hipSuccess && attr.type == hipMemoryTypeHost;
        (void)hipGetLastError();
        if (!locked) return d2h_staged(ctx, (char *)h_dst, (const char *)d_src, bytes);
    }
    VQ_HIP(ctx, hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return VQ_OK;
}

int32_t vq_timer_start(vq_ctx *ctx) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    VQ_HIP(ctx, hipEventRecord(ctx->ev0, ctx->stream));
    return VQ_OK;
}

int32_t vq_timer_stop(vq_ctx *ctx, float *h_ms) {
    if (!ctx || !h_ms) return VQ_ERR_INVALID_ARG;
    VQ_HIP(ctx, hipEventRecord(ctx->ev1, ctx->stream));
    VQ_HIP(ctx, hipEventSynchronize(ctx->ev1));
    VQ_HIP(ctx, hipEventElapsedTime(h_ms, ctx->ev0, ctx->ev1));
    return VQ_OK;
}

int32_t vq_calibrate(vq_ctx *ctx, int32_t what, double *h_rate) {
    if (!ctx || !h_rate) return VQ_ERR_INVALID_ARG;
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    hipStream_t st = ctx->stream;
    float ms = 0.f;
    if (what == VQ_CALIB_HBM_COPY) {
        // 512 MB read + 512 MB written by the plain copy kernel, best of five
        const int64_t count = 128LL * 1000 * 1000;
        VQ_TRY(ensure(ctx, ctx->tmp_a, sizeof(float) * count));
        VQ_TRY(ensure(ctx, ctx->tmp_b, sizeof(float) * count));
        VQ_HIP(ctx, hipMemsetAsync(ctx->tmp_a.p, 0, sizeof(float) * count, st));
        float best = 1e30f;
        for (int rep = 0; rep < 6; ++rep) {
            VQ_HIP(ctx, hipEventRecord(ctx->ev0, st));
            VQ_TRY(vq_copy_f32(ctx, (float *)ctx->tmp_b.p, (const float *)ctx->tmp_a.p, count));
            VQ_HIP(ctx, hipEventRecord(ctx->ev1, st));
            VQ_HIP(ctx, hipEventSynchronize(ctx->ev1));
            VQ_HIP(ctx, hipEventElapsedTime(&ms, ctx->ev0, ctx->ev1));
            if (rep > 0 && ms < best) best = ms;
        }
        *h_rate = 2.0 * sizeof(float) * (double)count / (best * 1e-3) / 1e9;  // GB/s, read + write
        return VQ_OK;
    }
    if (what < VQ_CALIB_VALU_FMA || what > VQ_CALIB_VALU_ADD)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: calibration kind %d", what);
    hipDeviceProp_t prop;
    VQ_HIP(ctx, hipGetDeviceProperties(&prop, ctx->device));
    const int iters = 2048;
    const unsigned blocks = (unsigned)prop.multiProcessorCount * 8u;  // 8 waves on every SIMD
    VQ_TRY(ensure(ctx, ctx->tmp_a, 256));
    float best = 1e30f;
    for (int rep = 0; rep < 4; ++rep) {
        VQ_HIP(ctx, hipEventRecord(ctx->ev0, st));
        uint32_t *sink = (uint32_t *)ctx->tmp_a.p;
        switch (what) {
        case VQ_CALIB_VALU_FMA: hipLaunchKernelGGL(vq::k_calib_valu<0>, dim3(blocks), dim3(256), 0, st, iters, 1u, sink); break;
        case VQ_CALIB_VALU_MIN3: hipLaunchKernelGGL(vq::k_calib_valu<1>, dim3(blocks), dim3(256), 0, st, iters, 1u, sink); break;
        case VQ_CALIB_VALU_MED3: hipLaunchKernelGGL(vq::k_calib_valu<2>, dim3(blocks), dim3(256), 0, st, iters, 1u, sink); break;
        case VQ_CALIB_VALU_AND_OR: hipLaunchKernelGGL(vq::k_calib_valu<3>, dim3(blocks), dim3(256), 0, st, iters, 1u, sink); break;
        default: hipLaunchKernelGGL(vq::k_calib_valu<4>, dim3(blocks), dim3(256), 0, st, iters, 1u, sink); break;
        }
        VQ_HIP(ctx, hipGetLastError());
        VQ_HIP(ctx, hipEventRecord(ctx->ev1, st));
        VQ_HIP(ctx, hipEventSynchronize(ctx->ev1));
        VQ_HIP(ctx, hipEventElapsedTime(&ms, ctx->ev0, ctx->ev1));
        if (rep > 0 && ms < best) best = ms;
    }
    // wave64 instructions per second over the whole GPU
    const double instr = (double)blocks * 4.0 * iters * vq::kCalibChains * vq::kCalibUnroll;
    *h_rate = instr / (best * 1e-3);
    return VQ_OK;
}

int32_t vq_calibrate_overlap(vq_ctx *ctx, int32_t mode, double *h_ms, uint32_t *h_waves) {
    if (!ctx || !h_ms || mode < 0 || mode > 2)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: overlap calibration mode %d", mode);
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    hipStream_t st = ctx->stream;
    hipDeviceProp_t prop;
    VQ_HIP(ctx, hipGetDeviceProperties(&prop, ctx->device));
    const unsigned waves_per_cu = 32u;  // 8 on every SIMD
    VQ_TRY(ensure(ctx, ctx->tmp_a, 256));
    uint32_t *sink = (uint32_t *)ctx->tmp_a.p, *where = sink + 8;
    const int n_mfma = 4096;
    const int vpm = mode == 0 ? 8 : mode == 1 ? 7 : 3;  // vector instructions per matrix instruction
    const int n_valu = n_mfma * vpm;
    for (int which = 0; which < 3; ++which) {
        const int nm = which == 1 ? 0 : n_mfma, nv = which == 0 ? 0 : n_valu;
        float best = 1e30f, ms = 0.f;
        for (int rep = 0; rep < 4; ++rep) {
            VQ_HIP(ctx, hipMemsetAsync(where, 0, 8 * sizeof(uint32_t), st));
            VQ_HIP(ctx, hipEventRecord(ctx->ev0, st));
            if (mode == 0)
                hipLaunchKernelGGL((vq::k_calib_overlap<0, 8>), dim3((unsigned)prop.multiProcessorCount * waves_per_cu / 8u),
                                   dim3(512), 0, st, nm, nv, 1u, sink, where);
            else if (mode == 1)
                hipLaunchKernelGGL((vq::k_calib_overlap<1, 7>), dim3((unsigned)prop.multiProcessorCount * waves_per_cu / 4u),
                                   dim3(256), 0, st, nm, nv, 1u, sink, where);
            else
                hipLaunchKernelGGL((vq::k_calib_overlap<1, 3>), dim3((unsigned)prop.multiProcessorCount * waves_per_cu / 4u),
                                   dim3(256), 0, st, nm, nv, 1u, sink, where);
            VQ_HIP(ctx, hipGetLastError());
            VQ_HIP(ctx, hipEventRecord(ctx->ev1, st));
            VQ_HIP(ctx, hipEventSynchronize(ctx->ev1));
            VQ_HIP(ctx, hipEventElapsedTime(&ms, ctx->ev0, ctx->ev1));
            if (rep > 0 && ms < best) best = ms;
        }
        h_ms[which] = best;
    }
    if (h_waves) {
        if (mode == 0) {
            VQ_HIP(ctx, hipMemcpyAsync(h_waves, where, 8 * sizeof(uint32_t), hipMemcpyDeviceToHost, st));
            VQ_HIP(ctx, hipStreamSynchronize(st));
        } else {
            for (int i = 0; i < 8; ++i) h_waves[i] = 0u;
        }
    }
    return VQ_OK;
}

int32_t vq_ctx_set_tsvq_variance_path(vq_ctx *ctx, int32_t path) {
    if (!ctx || (path != 0 && path != 1)) return VQ_ERR_INVALID_ARG;
    ctx->tsvq_var_path = path;
    return VQ_OK;
}

int32_t vq_ctx_set_assign_path(vq_ctx *ctx, int32_t path) {
    if (!ctx || (path != 0 && path != 1)) return VQ_ERR_INVALID_ARG;
    ctx->assign_path = path;
    return VQ_OK;
}

int32_t vq_ctx_last_recheck_count(vq_ctx *ctx, uint32_t *h_count) {
    if (!ctx || !h_count) return VQ_ERR_INVALID_ARG;
    uint32_t all = 0, two = 0;
    const int32_t rc = vq_ctx_last_recheck_split(ctx, &all, &two);
    *h_count = all + two;
    return rc;
}

int32_t vq_ctx_last_recheck_split(vq_ctx *ctx, uint32_t *h_count, uint32_t *h_two) {
    if (!ctx || !h_count || !h_two) return VQ_ERR_INVALID_ARG;
    *h_count = 0;
    *h_two = 0;
    if (ctx->recheck_src == 1 || ctx->recheck_src == 3) {
        uint32_t h[vq::kStatSlots * vq::kStatStride];
        const void *src = ctx->recheck_src == 1 ? ctx->mfma_stat.p : ctx->static_scratch + kNoAllocStatOff;
        VQ_HIP(ctx, hipMemcpyAsync(h, src, sizeof(h), hipMemcpyDeviceToHost, ctx->stream));
        VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
        for (int i = 0; i < vq::kStatSlots; ++i) *h_count += h[i * vq::kStatStride];
    } else if (ctx->recheck_src == 2) {
        uint32_t h[2];  // all-centroid checks, two-candidate checks
        VQ_HIP(ctx, hipMemcpyAsync(h, ctx->mfma_list.p, sizeof(h), hipMemcpyDeviceToHost, ctx->stream));
        VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
        *h_count = h[0];
        *h_two = h[1];
    }
    return VQ_OK;
}

int32_t vq_prof_enable(vq_ctx *ctx, int32_t on) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    prof_collect(ctx);
    ctx->prof_on = on != 0;
    for (int i = 0; i < VQ_PROF_CLASSES; ++i) {
        ctx->prof_ms[i] = 0;
        ctx->prof_launches[i] = 0;
    }
    return VQ_OK;
}

int32_t vq_prof_read(vq_ctx *ctx, int32_t cls, double *h_total_ms, int64_t *h_spans) {
    if (!ctx || cls < 0 || cls >= VQ_PROF_CLASSES || !h_total_ms || !h_spans)
        return VQ_ERR_INVALID_ARG;
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    prof_collect(ctx);
    *h_total_ms = ctx->prof_ms[cls];
    *h_spans = ctx->prof_launches[cls];
    return VQ_OK;
}

int32_t vq_copy_f32(vq_ctx *ctx, float *d_dst, const float *d_src, int64_t count) {
    if (!ctx || count < 0 || (count && (!d_dst || !d_src))) return VQ_ERR_INVALID_ARG;
    if ((reinterpret_cast<uintptr_t>(d_dst) | reinterpret_cast<uintptr_t>(d_src)) & 15)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: buffers must be 16-byte aligned");
    if (count == 0) return VQ_OK;
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    int64_t n4 = count / 4;
    int tail = (int)(count % 4);
    unsigned blocks = (unsigned)std::min<int64_t>(std::max<int64_t>((n4 + 255) / 256, 1), 256 * 32);
    hipLaunchKernelGGL(k_copy_f32, dim3(blocks), dim3(256), 0, ctx->stream, (const float4 *)d_src,
                       (float4 *)d_dst, n4, d_src + n4 * 4, d_dst + n4 * 4, tail);
    VQ_HIP(ctx, hipGetLastError());
    return VQ_OK;
}

// pend_cb / pend_codes: a residual update x[i] -= pend_cb[pend_codes[i]] that the fit applies to the
// rows in place as its first assignment pass reads them (the caller has checked that this shape's
// first pass is the kernel that can: lbg_pending_fusable).
static int32_t lbg_fit_impl(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t m, int32_t sd,
                            int32_t k, int32_t max_iters, const uint32_t *h_init_idx,
                            const uint32_t *h_reseed_stream, int32_t n_reseed, float *d_codebooks,
                            int32_t *h_iters_run, int32_t *h_reseeds_used, const float *pend_cb,
                            const uint8_t *pend_codes) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (k == 0) return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: k must be greater than 0");
    VQ_TRY(check_common(ctx, d_x, n, ld, m, sd, k, 65536));
    if (n < k)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: Not enough data points for k clusters");
    if (m > 65535) return fail(ctx, VQ_ERR_UNSUPPORTED, "m must be at most 65535");
    if (!h_init_idx || !d_codebooks || max_iters < 0 || n_reseed < 0 || (n_reseed && !h_reseed_stream))
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: null pointer or negative size");
    for (int64_t i = 0; i < (int64_t)m * k; ++i)
        if (h_init_idx[i] >= (uint64_t)n)
            return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: init index %u out of range", h_init_idx[i]);
    for (int64_t i = 0; i < (int64_t)m * n_reseed; ++i)
        if (h_reseed_stream[i] >= (uint64_t)n)
            return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: reseed index %u out of range", h_reseed_stream[i]);
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    if (k > vq::kMaxK)
        return vqh::lbg_fit_big(ctx, d_x, n, ld, m, sd, k, max_iters, h_init_idx, h_reseed_stream, n_reseed,
                                d_codebooks, h_iters_run, h_reseeds_used);
    hipStream_t st = ctx->stream;

    const int nparts = (int)((n + vq::kPartRows - 1) / vq::kPartRows);
    const int nseg = (nparts + vq::kScanSeg - 1) / vq::kScanSeg;
    // streaming sums of the large clusters: 32-byte sub-vectors, 4 per 128-byte line, aligned rows
    const bool stream = sd == 8 && m % 4 == 0 && ld % 4 == 0 && ld <= (1 << 20) &&
                        (reinterpret_cast<uintptr_t>(d_x) & 15) == 0;  // (32-bit lane offsets inside a chunk)
    const int64_t leaf_cap64 = stream ? (int64_t)k : (int64_t)k * nparts;
    if (leaf_cap64 * sd > (1LL << 31)) return fail(ctx, VQ_ERR_UNSUPPORTED, "n * k * sub_dim too large");
    const int leaf_cap = (int)leaf_cap64;
    VQ_TRY(ensure(ctx, ctx->flags, sizeof(int) * (7 * (size_t)m + 1)));
    VQ_TRY(ensure(ctx, ctx->tables, sizeof(uint32_t) * 4 * (size_t)m * vq::kMaxK));
    VQ_TRY(ensure(ctx, ctx->hist, sizeof(uint32_t) * (size_t)m * nparts * vq::kMaxK));
    VQ_TRY(ensure(ctx, ctx->seg, sizeof(uint32_t) * (size_t)m * nseg * vq::kMaxK));
    VQ_TRY(ensure(ctx, ctx->perm, sizeof(uint32_t) * (size_t)m * n));
    // per-part sums of the streaming kernel, then one folded sum per cluster
    if (stream) VQ_TRY(ensure(ctx, ctx->part_sum, sizeof(float) * (size_t)m * (nparts + 1) * vq::kMaxK * 8));
    VQ_TRY(ensure(ctx, ctx->leaf_desc, sizeof(uint2) * (size_t)m * leaf_cap));
    VQ_TRY(ensure(ctx, ctx->leaf_sum, sizeof(float) * (size_t)m * leaf_cap * sd));
    VQ_TRY(ensure(ctx, ctx->codes, (size_t)m * n));
    VQ_TRY(ensure(ctx, ctx->idx, sizeof(uint32_t) * (size_t)m * k));
    VQ_TRY(ensure(ctx, ctx->reseed, sizeof(uint32_t) * ((size_t)m * n_reseed + 1)));

    vq::LbgState S;
    int *f = (int *)ctx->flags.p;
    S.changed = f;
    S.done = f + m;
    S.iters = f + 2 * m;
    S.used = f + 3 * m;
    S.ubase = f + 4 * m;
    S.nleaves = f + 5 * m;
    S.nsmall = f + 6 * m;
    S.err = f + 7 * m;
    uint32_t *tb = (uint32_t *)ctx->tables.p;
    const size_t mk = (size_t)m * vq::kMaxK;
    S.count = tb;
    S.start = tb + mk;
    S.leaf_start = tb + 2 * mk;
    S.empty_rank = tb + 3 * mk;
    S.hist = (uint32_t *)ctx->hist.p;
    S.seg = (uint32_t *)ctx->seg.p;
    S.perm = (uint32_t *)ctx->perm.p;
    S.leaf_desc = (uint2 *)ctx->leaf_desc.p;
    S.leaf_sum = (float *)ctx->leaf_sum.p;
    S.part_sum = stream ? (float *)ctx->part_sum.p : nullptr;
    S.codes = (uint8_t *)ctx->codes.p;
    S.nparts = nparts;
    S.nseg = nseg;
    S.leaf_cap = leaf_cap;
    S.stream = stream ? 1 : 0;

    VQ_HIP(ctx, hipMemcpyAsync(ctx->idx.p, h_init_idx, sizeof(uint32_t) * (size_t)m * k,
                               hipMemcpyHostToDevice, st));
    if (n_reseed)
        VQ_HIP(ctx, hipMemcpyAsync(ctx->reseed.p, h_reseed_stream,
                                   sizeof(uint32_t) * (size_t)m * n_reseed, hipMemcpyHostToDevice, st));
    VQ_HIP(ctx, hipMemsetAsync(S.codes, 0, (size_t)m * n, st));  // assignments = vec![0; n], utils.rs:55
    hipLaunchKernelGGL(vq::k_lbg_init, dim3(cdiv(m, 64)), dim3(64), 0, st, S, m);
    if (pend_cb)
        hipLaunchKernelGGL(vq::k_gather_rows_pend, dim3(cdiv((int64_t)k * sd, 256)), dim3(256), 0, st, d_x, ld, k, sd,
                           (const uint32_t *)ctx->idx.p, d_codebooks, pend_cb, pend_codes);
    else
        hipLaunchKernelGGL(vq::k_gather_rows, dim3(cdiv((int64_t)m * k * sd, 256)), dim3(256), 0, st, d_x,
                           ld, m, k, sd, (const uint32_t *)ctx->idx.p, d_codebooks);
    VQ_HIP(ctx, hipGetLastError());

    vq::AssignArgs a;
    a.x = d_x;
    a.n = n;
    a.ld = ld;
    a.m = m;
    a.k = k;
    a.cb = d_codebooks;
    a.cnorm = nullptr;
    a.codes = S.codes;
    a.changed = S.changed;
    a.done = S.done;

    // With the streaming sums and the matrix-core assignment, one kernel ends the update: the new
    // centroids, the loop control and the tables of the next assignment pass.
    const bool fused_tail = stream && mfma_applicable<vq::M_SQ, true>(ctx, a, sd);
    MfmaTabPtrs tabs{};
    if (fused_tail) VQ_TRY(mfma_tab_ptrs(ctx, m, k, tabs));
    // Timing classes of the loop: where the assignment kernel carries its own events (started,
    // done) the assignment span is the kernel's and an update span runs from one kernel's end to
    // the next one's start, so nothing is recorded between the kernels of an iteration.
    hipEvent_t prev_done = nullptr;
    for (int it = 0; it < max_iters; ++it) {
        hipEvent_t started = nullptr, done = nullptr;
        a.pend_cb = it == 0 ? pend_cb : nullptr;  // the first pass leaves the rows updated
        a.pend_codes = it == 0 ? pend_codes : nullptr;
        {
            ProfSpan sp(ctx, fused_tail ? -1 : VQ_PROF_LBG_ASSIGN);
            VQ_TRY(launch_assign<true>(ctx, VQ_SQEUCLIDEAN, a, sd, fused_tail && it > 0, &started, &done));
        }
        if (ctx->prof_on && started && done) {
            ctx->prof_open.push_back({VQ_PROF_LBG_ASSIGN, started, done, false, false});
            if (prev_done) ctx->prof_open.push_back({VQ_PROF_LBG_UPDATE, prev_done, started, false, false});
        }
        prev_done = done;
        ProfSpan sp(ctx, fused_tail ? -1 : VQ_PROF_LBG_UPDATE);
        int shift = 0;
        while ((1 << shift) < sd) ++shift;
        const bool leaf_wg = stream && sd >= 4 && sd <= 32 && (1 << shift) == sd && ld % 4 == 0 &&
                             (reinterpret_cast<uintptr_t>(d_x) & 15) == 0;
        // The gather path of the small clusters needs only the new codes: with the streaming sums
        // it runs on the second stream beside them (a chain of short, latency-bound kernels next to
        // one long pass over the rows), and the two meet again before the large clusters' fold.
        hipStream_t gs = stream ? ctx->side : st;
        if (stream) {
            if (!done) {  // the assignment kernel carried no event
                VQ_HIP(ctx, hipEventRecord(ctx->ev_fork, st));
                done = ctx->ev_fork;
            }
            VQ_HIP(ctx, hipStreamWaitEvent(gs, done, 0));
            hipLaunchKernelGGL(vq::k_lbg_stream8, dim3(nparts, m / 4), dim3(256), 0, st, S, d_x, n, ld);
        }
        hipLaunchKernelGGL(vq::k_lbg_hist, dim3(nparts, m), dim3(64), 0, gs, S, n);
        hipLaunchKernelGGL(vq::k_lbg_scan_seg, dim3(nseg, m), dim3(256), 0, gs, S);
        hipLaunchKernelGGL(vq::k_lbg_plan, dim3(m), dim3(256), 0, gs, S, k);
        hipLaunchKernelGGL(vq::k_lbg_scan_blocks, dim3(nseg, m), dim3(256), 0, gs, S);
        if (stream)  // beside the streaming kernel: one wave per part (four waves per part take its resources: 40 us, and 15 us more for the streaming kernel)
            hipLaunchKernelGGL(vq::k_lbg_scatter, dim3(nparts, m), dim3(64), 0, gs, S, n);
        else  // every row is listed: four waves per part
            hipLaunchKernelGGL(vq::k_lbg_scatter_wg, dim3(nparts, m), dim3(256), 0, gs, S, n);
        if (leaf_wg) {
            // leaves are the few clusters of up to 1024 members beside the streaming kernel
            hipLaunchKernelGGL(vq::k_lbg_leafsum_wg, dim3(leaf_cap, m), dim3(256), 0, gs, S, d_x, n, ld, sd,
                               shift);
        } else if (sd <= 32 && (1 << shift) == sd) {
            hipLaunchKernelGGL(vq::k_lbg_leafsum_wave, dim3(cdiv(leaf_cap, 4), m), dim3(256), 0, gs, S, d_x, n,
                               ld, sd, shift);
        } else {
            hipLaunchKernelGGL(vq::k_lbg_leafsum, dim3(cdiv((int64_t)leaf_cap * sd, 256), m), dim3(256), 0, gs,
                               S, d_x, n, ld, sd);
        }
        float *big_sum = stream ? S.part_sum + (size_t)m * nparts * vq::kMaxK * 8 : nullptr;
        if (fused_tail)  // needs the streaming kernel only: in flight while the gather path ends
            hipLaunchKernelGGL(vq::k_lbg_fold8, dim3(cdiv((int64_t)k * 8, 256), m), dim3(256), 0, st, S, k, big_sum);
        if (stream) {
            VQ_HIP(ctx, hipEventRecord(ctx->ev_join, gs));
            VQ_HIP(ctx, hipStreamWaitEvent(st, ctx->ev_join, 0));
            if (!fused_tail)
                hipLaunchKernelGGL(vq::k_lbg_combine8, dim3(cdiv((int64_t)k * 8, 256), m), dim3(256), 0, st, S, k,
                                   d_codebooks);
        }
        if (fused_tail) {
            hipLaunchKernelGGL(vq::k_lbg_finalize_prep8, dim3(m), dim3(256), 0, st, S, d_x, ld, k,
                               (const uint32_t *)ctx->reseed.p, n_reseed, d_codebooks, (const float *)big_sum,
                               tabs.nb, tabs.atab, tabs.maxc2, tabs.mu, tabs.stat);
        } else {
            hipLaunchKernelGGL(vq::k_lbg_finalize, dim3(cdiv((int64_t)k * sd, 256), m), dim3(256), 0, st, S,
                               d_x, ld, k, sd, (const uint32_t *)ctx->reseed.p, n_reseed, d_codebooks);
            hipLaunchKernelGGL(vq::k_lbg_advance, dim3(cdiv(m, 64)), dim3(64), 0, st, S, m);
        }
        VQ_HIP(ctx, hipGetLastError());
    }
    if (ctx->prof_on && fused_tail && prev_done) {  // the last update: up to an event recorded here
        hipEvent_t end = prof_event(ctx);
        VQ_HIP(ctx, hipEventRecord(end, st));
        ctx->prof_open.push_back({VQ_PROF_LBG_UPDATE, prev_done, end, false, true});
    }
    std::vector<int> host(7 * (size_t)m + 1);
    VQ_HIP(ctx, hipMemcpyAsync(host.data(), f, sizeof(int) * host.size(), hipMemcpyDeviceToHost, st));
    VQ_HIP(ctx, hipStreamSynchronize(st));
    prof_collect(ctx);
    if (h_iters_run) memcpy(h_iters_run, host.data() + 2 * m, sizeof(int) * m);
    if (h_reseeds_used) memcpy(h_reseeds_used, host.data() + 3 * m, sizeof(int) * m);
    if (host[7 * (size_t)m])
        return fail(ctx, VQ_ERR_RESEED_EXHAUSTED,
                    "re-seed stream exhausted: pass n_reseed = k*max_iters");
    return VQ_OK;
}

int32_t vq_lbg_fit(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t m, int32_t sd,
                   int32_t k, int32_t max_iters, const uint32_t *h_init_idx,
                   const uint32_t *h_reseed_stream, int32_t n_reseed, float *d_codebooks,
                   int32_t *h_iters_run, int32_t *h_reseeds_used) {
    return lbg_fit_impl(ctx, d_x, n, ld, m, sd, k, max_iters, h_init_idx, h_reseed_stream, n_reseed, d_codebooks,
                        h_iters_run, h_reseeds_used, nullptr, nullptr);
}

int32_t vq_lbg_fit_residual(vq_ctx *ctx, float *d_res, int64_t n, int64_t ld, int32_t dim, int32_t k,
                            int32_t max_iters, const uint32_t *h_init_idx, const uint32_t *h_reseed_stream,
                            int32_t n_reseed, float *d_codebook, const float *d_prev_codebook, int32_t k_prev,
                            const uint8_t *d_prev_codes, int32_t *h_iters_run, int32_t *h_reseeds_used) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (!d_prev_codebook || !d_prev_codes || k_prev <= 0 || k_prev > 256)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: the previous stage's codebook and codes");
    // The first assignment pass can apply the update as it reads the rows when it is the matrix-core
    // pass over one wide column block and there is a first pass; the arguments the fused path does
    // not check itself are checked by the two calls of the other path.
    vq::AssignArgs a;
    a.x = d_res;
    a.n = n;
    a.ld = ld;
    a.m = 1;
    a.k = k;
    a.cb = d_codebook;
    const bool fusable = d_res && d_codebook && n >= k && k >= 1 && k <= vq::kMaxK && dim >= 16 && ld >= dim &&
                         max_iters >= 1 && (reinterpret_cast<uintptr_t>(d_prev_codebook) & 15) == 0 &&
                         mfma_wide_applicable<vq::M_SQ, true>(ctx, a, dim) &&
                         !mfma_applicable<vq::M_SQ, true>(ctx, a, dim);
    if (!fusable) {
        VQ_TRY(vq_residual_sub(ctx, d_res, n, ld, dim, k_prev, d_prev_codebook, d_prev_codes));
        return lbg_fit_impl(ctx, d_res, n, ld, 1, dim, k, max_iters, h_init_idx, h_reseed_stream, n_reseed,
                            d_codebook, h_iters_run, h_reseeds_used, nullptr, nullptr);
    }
    return lbg_fit_impl(ctx, d_res, n, ld, 1, dim, k, max_iters, h_init_idx, h_reseed_stream, n_reseed, d_codebook,
                        h_iters_run, h_reseeds_used, d_prev_codebook, d_prev_codes);
}

int32_t vq_assign(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t m,
                  int32_t sd, int32_t k, const float *d_codebooks, uint8_t *d_codes) {
    return vqh::assign_codes(ctx, metric, d_x, n, ld, m, sd, k, d_codebooks, d_codes);
}

int32_t vq_assign_noalloc(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t m,
                          int32_t sd, int32_t k, const float *d_codebooks, uint8_t *d_codes) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    // Which shapes touch the fixed scratch: the matrix-core kernel of 8-float column blocks (its
    // tables and counters) and the cosine kernels (the centroid norms).  Only they are bound by its
    // size, and only they need the GPU's one array for themselves.
    const bool uses_scratch =
        metric == VQ_COSINE ||
        ((metric == VQ_SQEUCLIDEAN || metric == VQ_EUCLIDEAN) && sd == 8 && ctx->assign_path == 0);
    if (uses_scratch && m > 0 && k > 0 && k <= vq::kMaxK) {
        // the tables of the call must fit: column blocks x centroids padded to 64
        const int64_t cells = (int64_t)m * 64 * ((k + 63) / 64);
        if (m > kNoAllocMaxM || cells > kNoAllocMaxCells)
            return fail(ctx, VQ_ERR_UNSUPPORTED,
                        "vq_assign_noalloc: m * k (k padded to 64) = %lld exceeds the fixed scratch of %d "
                        "(use vq_assign, which may allocate)", (long long)cells, kNoAllocMaxCells);
        if (ctx->device < 0 || ctx->device >= kMaxDevices)
            return fail(ctx, VQ_ERR_UNSUPPORTED, "vq_assign_noalloc: device %d", ctx->device);
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        vq_ctx *owner = g_scratch_owner[ctx->device];
        if (owner && owner != ctx) {
            const hipError_t busy = hipStreamQuery(owner->stream);
            (void)hipGetLastError();
            if (busy != hipSuccess)
                return fail(ctx, VQ_ERR_UNSUPPORTED,
                            "vq_assign_noalloc: the fixed scratch of GPU %d is in use by another context whose "
                            "stream has not finished (calls that use it must not overlap on one GPU)", ctx->device);
        }
        g_scratch_owner[ctx->device] = ctx;
    }
    // no timing spans (their events are created on demand) and no workspace growth inside the call
    const bool prof = ctx->prof_on;
    ctx->prof_on = false;
    ctx->no_alloc = true;
    const int32_t rc = vqh::assign_codes(ctx, metric, d_x, n, ld, m, sd, k, d_codebooks, d_codes);
    ctx->no_alloc = false;
    ctx->prof_on = prof;
    return rc;
}

int32_t vq_decode_f16(vq_ctx *ctx, const uint8_t *d_codes, int64_t n, int32_t m, int32_t sd, int32_t k,
                      const float *d_codebooks, uint16_t *d_out) {
    return decode_codes<true>(ctx, d_codes, n, m, sd, k, vq::kMaxK, d_codebooks, (void *)d_out);
}

int32_t vq_decode_f32(vq_ctx *ctx, const uint8_t *d_codes, int64_t n, int32_t m, int32_t sd, int32_t k,
                      const float *d_codebooks, float *d_out) {
    return decode_codes<false>(ctx, d_codes, n, m, sd, k, vq::kMaxK, d_codebooks, (void *)d_out);
}

int32_t vq_decode_f16_u16(vq_ctx *ctx, const uint16_t *d_codes, int64_t n, int32_t m, int32_t sd, int32_t k,
                          const float *d_codebooks, uint16_t *d_out) {
    return decode_codes<true>(ctx, d_codes, n, m, sd, k, 65536, d_codebooks, (void *)d_out);
}

int32_t vq_decode_f32_u16(vq_ctx *ctx, const uint16_t *d_codes, int64_t n, int32_t m, int32_t sd, int32_t k,
                          const float *d_codebooks, float *d_out) {
    return decode_codes<false>(ctx, d_codes, n, m, sd, k, 65536, d_codebooks, (void *)d_out);
}

}  // extern "C"
