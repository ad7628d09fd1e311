// Shared host-side state of libvqhip: the context, error reporting, the grow-only device
// workspace and the per-kernel-class event timing.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "../../include/vq_hip.h"

struct DevBuf {
    void *p = nullptr;
    size_t cap = 0;
};

struct vq_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    // second stream of the LBG update: the small clusters' gather path runs beside the streaming sums
    hipStream_t side = nullptr;
    hipEvent_t ev_fork = nullptr, ev_join = nullptr;
    std::string err;
    // grow-only device workspace
    DevBuf flags, tables, hist, seg, part_sum, perm, leaf_desc, leaf_sum, codes, idx, reseed, cnorm;
    DevBuf tsvq_sq;              // TSVQ build: squared deviations of a level
    DevBuf tsvq_split;           // TSVQ build: the small per-level tables of the nodes being split
    DevBuf tsvq_level;           // TSVQ build: the level's uploaded tables and the leaf sums of its node means
    DevBuf tsvq_means;           // TSVQ build: the means of all nodes, read back once at the end
    DevBuf tsvq_scan;            // TSVQ build: workspace of the partition's prefix scan
    DevBuf tsvq_km;              // TSVQ build with 2-means splits: centroids, part sums, flags, draws of a level
    void *tsvq_pin = nullptr;    // TSVQ build: page-locked staging of a level's tables and decisions
    size_t tsvq_pin_cap = 0;
    // vq_h2d from pageable memory: page-locked staging buffers and the events of their uploads
    static constexpr int kStageBuffers = 3;
    void *h2d_stage[kStageBuffers] = {nullptr, nullptr, nullptr};
    hipEvent_t h2d_event[kStageBuffers] = {nullptr, nullptr, nullptr};
    DevBuf tsvq_gsum, tsvq_guess, tsvq_maps;  // per group of 32 squares: sum, binade guess, integer maps
    DevBuf tsvq_bsum, tsvq_segmaps;           // per block of groups: f64 sum; per run of groups: composed map
    int tsvq_var_path = 0;       // 0 = composed integer maps, 1 = one chain of adds per column
    DevBuf mfma_tab, mfma_list, mfma_stat;  // tables, re-check list and counters of the matrix-core assignment
    int recheck_src = 0;         // where the last pass counted its undecided pairs: 1 mfma_stat, 2 mfma_list, 3 the fixed scratch
    int assign_path = 0;         // 0 = matrix cores where a kernel exists, 1 = vector ALU only
    int compute_units = 0;       // of the context's GPU (0: not asked for yet)
    int decode_lds_set[4] = {0, 0, 0, 0};  // dynamic-LDS limit already granted to the four resident decode kernels
    int tsvq_descend_path = 0;   // 0 = one inner product per node where it decides (cosine, L2), 1 = two distances per node always
    int procrustes_path = 0;     // 0 = Newton-Schulz polar factor first, SVD when it does not converge; 1 = SVD only
    // vq_assign_noalloc: the device address of this GPU's file-scope scratch array, and whether a
    // call that must not allocate is running (then `ensure` refuses to grow the workspace)
    unsigned char *static_scratch = nullptr;
    bool no_alloc = false;
    DevBuf tmp_a, tmp_b, tmp_c, tmp_d, tmp_e, tmp_f;  // scratch of the RVQ / OPQ / TSVQ entry points
    // codebooks above 256 centroids: chunk tables, chunk winners, running minimum, merged codes,
    // the LBG's assignment, sort keys in and out, the sort's workspace, per-cluster tables, flags
    DevBuf big_chunk, big_win, big_wind, big_best, big_fresh, big_codes, big_keys, big_sorted, big_sort_tmp, big_tables,
        big_flags;
    // optional per-kernel-class timing (HIP events on the stream)
    bool prof_on = false;
    std::vector<hipEvent_t> prof_pool;
    struct Span {
        int cls;
        hipEvent_t a, b;
        bool own_a = true, own_b = true;  // false: the event belongs to another span (returned to the pool once)
    };
    std::vector<Span> prof_open;
    double prof_ms[VQ_PROF_CLASSES] = {0};
    int64_t prof_launches[VQ_PROF_CLASSES] = {0};
};

namespace vqh {

std::string &create_error();

inline int32_t fail(vq_ctx *ctx, int32_t code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (ctx)
        ctx->err = buf;
    else
        create_error() = buf;
    return code;
}

#define VQ_HIP(ctx, call)                                                                          \
    do {                                                                                           \
        hipError_t e__ = (call);                                                                   \
        if (e__ != hipSuccess) {                                                                   \
            (void)hipGetLastError(); /* the runtime keeps the error until it is read: a later   */ \
                                     /* check of a good launch would report this one again      */ \
            return vqh::fail(ctx, e__ == hipErrorOutOfMemory ? VQ_ERR_OOM : VQ_ERR_HIP,            \
                             "%s: %s (%s:%d)", #call, hipGetErrorString(e__), __FILE__, __LINE__); \
        }                                                                                          \
    } while (0)

#define VQ_TRY(expr)                    \
    do {                                \
        int32_t rc__ = (expr);          \
        if (rc__ != VQ_OK) return rc__; \
    } while (0)

inline int32_t ensure(vq_ctx *ctx, DevBuf &b, size_t bytes) {
    if (bytes <= b.cap) return VQ_OK;
    if (ctx->no_alloc)
        return fail(ctx, VQ_ERR_UNSUPPORTED, "this shape needs a workspace allocation, which this entry point may not make");
    if (b.p) {
        VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
        VQ_HIP(ctx, hipFree(b.p));
        b.p = nullptr;
        b.cap = 0;
    }
    size_t want = bytes + bytes / 8 + 256;
    VQ_HIP(ctx, hipMalloc(&b.p, want));
    b.cap = want;
    return VQ_OK;
}

inline unsigned cdiv(int64_t a, int64_t b) { return (unsigned)((a + b - 1) / b); }

inline hipEvent_t prof_event(vq_ctx *ctx) {
    if (!ctx->prof_pool.empty()) {
        hipEvent_t e = ctx->prof_pool.back();
        ctx->prof_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    (void)hipEventCreate(&e);
    return e;
}

struct ProfSpan {
    vq_ctx *ctx;
    int cls;
    hipEvent_t a = nullptr;
    ProfSpan(vq_ctx *c, int k) : ctx(c), cls(k) {  // k < 0: no span
        if (ctx->prof_on && k >= 0) {
            a = prof_event(ctx);
            (void)hipEventRecord(a, ctx->stream);
        }
    }
    ~ProfSpan() {
        if (a) {
            hipEvent_t b = prof_event(ctx);
            (void)hipEventRecord(b, ctx->stream);
            ctx->prof_open.push_back({cls, a, b, true, true});
        }
    }
};

// Resolves the recorded spans; the stream must have been synchronised.
inline void prof_collect(vq_ctx *ctx) {
    for (auto &sp : ctx->prof_open) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, sp.a, sp.b) == hipSuccess) {
            ctx->prof_ms[sp.cls] += ms;
            ctx->prof_launches[sp.cls] += 1;
        }
    }
    for (auto &sp : ctx->prof_open) {
        if (sp.own_a) ctx->prof_pool.push_back(sp.a);
        if (sp.own_b) ctx->prof_pool.push_back(sp.b);
    }
    ctx->prof_open.clear();
}

// Argument checks shared by the entry points that take a row matrix and codebooks.
// k_max: 256 where the codes are bytes, 65536 where they are 16 bits wide.
int32_t check_common(vq_ctx *ctx, const void *x, int64_t n, int64_t ld, int32_t m, int32_t sd, int32_t k,
                     int32_t k_max = 256);

// Launchers defined in vq_api.hip, used by the RVQ / OPQ entry points.
// d_dist (optional, n x m floats): receives the chosen centroids' distances where the kernel that runs
// computes them anyway; *dist_written says whether it did.
// pend (optional; one column block, and only where assign_pending_fusable says so): a residual
// update that the pass applies to the rows before it scores them, d_x[i] = src[i] - cb[codes[i]]
// with src = the rows of d_x themselves (src null: d_x is updated in place) or other rows of stride
// src_ld that stay as they are.
struct PendingUpdate {
    const float *cb;
    const uint8_t *codes;
    const float *src;
    int64_t src_ld;
};
int32_t assign_codes(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t m,
                     int32_t sd, int32_t k, const float *d_codebooks, uint8_t *d_codes, float *d_dist = nullptr,
                     bool *dist_written = nullptr, const PendingUpdate *pend = nullptr);
// Whether the assignment of these rows (one column block of sd floats) runs on the pass that can
// take a pending update along.
bool assign_pending_fusable(const vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t sd,
                            int32_t k, const float *d_codebook);

// Defined in vq_api_bigk.hip: the same for any k up to 65536 with 16-bit codes, and the LBG above
// 256 centroids (arguments as vq_lbg_fit, already validated).
int32_t assign_codes_u16(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t m,
                         int32_t sd, int32_t k, const float *d_codebooks, uint16_t *d_codes);
int32_t lbg_fit_big(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t m, int32_t sd, int32_t k,
                    int32_t max_iters, const uint32_t *h_init_idx, const uint32_t *h_reseed_stream,
                    int32_t n_reseed, float *d_codebooks, int32_t *h_iters_run, int32_t *h_reseeds_used);

}  // namespace vqh
