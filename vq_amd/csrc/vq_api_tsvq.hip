// libvqhip — tree-structured VQ entry points: build (TSVQNode::fit, src/tsvq.rs:71-148) and
// descent encode (src/tsvq.rs:162-181,231-249).
#include <cstring>

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <rocprim/rocprim.hpp>

#include <algorithm>
#include <vector>

#include "ctx.hpp"
#include "assign_exact.hpp"
#include "tsvq.hpp"
#include "tsvq_kmeans.hpp"

using namespace vqh;

// Nodes are numbered breadth-first: the root is 0; children are appended level by level, left
// before right.  left/right hold -1 for "no child".
struct vq_tree {
    int device = 0;
    int32_t n_nodes = 0;
    int32_t dim = 0;
    std::vector<float> h_centroids;
    std::vector<int32_t> h_left, h_right, h_split_dim;
    std::vector<float> h_split_val;
    std::vector<int64_t> h_count;
    void *d_block = nullptr;  // one allocation: centroids, their norms, left and right children
    float *d_centroids = nullptr, *d_cnorm = nullptr;
    int32_t *d_left = nullptr, *d_right = nullptr;
    // per node below vq::kTopNodes: the vector and the scalars that decide a descent step by one
    // inner product (cosine; squared Euclidean and Euclidean)
    float *d_wcos = nullptr, *d_sccos = nullptr, *d_wl2 = nullptr, *d_scl2 = nullptr;
};

namespace {

constexpr int kLeafMaxRows = 1024;  // PARALLEL_THRESHOLD, src/vector.rs:16

int tree_depth(uint64_t count) {
    int d = 0;
    while (count > ((uint64_t)kLeafMaxRows << d)) ++d;
    return d;
}

struct Seg {
    int32_t node;
    uint32_t lo, hi;
    uint64_t heap = 1;  // position in the complete binary tree: root 1, children 2 h and 2 h + 1
};

// The 2-means split (vq_tsvq_build_kmeans): LBG iterations per node and the nodes' draws.
struct KmOpts {
    int32_t lbg_iters;
    const uint32_t *h_draws;
    int32_t per_node;
};

// d_means: the centroids where they already are on the device (the build's node means), else they
// go up from the host copy.
int32_t tree_to_device(vq_ctx *ctx, vq_tree *t, const float *d_means = nullptr) {
    size_t nn = (size_t)t->n_nodes, dim = (size_t)t->dim;
    auto pad = [](size_t z) { return (z + 255) & ~(size_t)255; };
    const size_t cen_b = pad(sizeof(float) * nn * dim), idx_b = pad(sizeof(int32_t) * nn);
    const size_t ntop = std::min<size_t>(nn, (size_t)vq::kTopNodes);
    const size_t w_b = pad(sizeof(float) * ntop * dim), sc_b = pad(sizeof(float) * 2 * ntop);
    VQ_HIP(ctx, hipMalloc(&t->d_block, cen_b + 3 * idx_b + 2 * w_b + 2 * sc_b));
    char *base = (char *)t->d_block;
    t->d_centroids = (float *)base;
    t->d_cnorm = (float *)(base + cen_b);
    t->d_left = (int32_t *)(base + cen_b + idx_b);
    t->d_right = (int32_t *)(base + cen_b + 2 * idx_b);
    t->d_wcos = (float *)(base + cen_b + 3 * idx_b);
    t->d_wl2 = (float *)(base + cen_b + 3 * idx_b + w_b);
    t->d_sccos = (float *)(base + cen_b + 3 * idx_b + 2 * w_b);
    t->d_scl2 = (float *)(base + cen_b + 3 * idx_b + 2 * w_b + sc_b);
    hipStream_t st = ctx->stream;
    if (d_means)
        VQ_HIP(ctx, hipMemcpyAsync(t->d_centroids, d_means, sizeof(float) * nn * dim, hipMemcpyDeviceToDevice, st));
    else
        VQ_HIP(ctx, hipMemcpyAsync(t->d_centroids, t->h_centroids.data(), sizeof(float) * nn * dim,
                                   hipMemcpyHostToDevice, st));
    VQ_HIP(ctx, hipMemcpyAsync(t->d_left, t->h_left.data(), sizeof(int32_t) * nn, hipMemcpyHostToDevice, st));
    VQ_HIP(ctx, hipMemcpyAsync(t->d_right, t->h_right.data(), sizeof(int32_t) * nn, hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL(vq::k_centroid_norms, dim3(cdiv((int64_t)nn, 256)), dim3(256), 0, st, t->d_centroids,
                       (int64_t)nn, (int)dim, t->d_cnorm);
    hipLaunchKernelGGL(vq::k_tsvq_wtable<true>, dim3((unsigned)ntop), dim3(64), 0, st, t->d_centroids, t->d_cnorm,
                       t->d_left, t->d_right, (int)dim, t->d_wcos, t->d_sccos);
    hipLaunchKernelGGL(vq::k_tsvq_wtable<false>, dim3((unsigned)ntop), dim3(64), 0, st, t->d_centroids, t->d_cnorm,
                       t->d_left, t->d_right, (int)dim, t->d_wl2, t->d_scl2);
    VQ_HIP(ctx, hipGetLastError());
    VQ_HIP(ctx, hipStreamSynchronize(st));
    return VQ_OK;
}

void tree_release(vq_tree *t) {
    if (!t) return;
    (void)hipFree(t->d_block);
    delete t;
}

}  // namespace

extern "C" {

static int32_t tsvq_build_impl(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t dim, int32_t max_depth,
                               const KmOpts *km, vq_tree **out);

int32_t vq_tsvq_build(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t dim, int32_t max_depth,
                      vq_tree **out) {
    return tsvq_build_impl(ctx, d_x, n, ld, dim, max_depth, nullptr, out);
}

int32_t vq_tsvq_build_kmeans(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t dim, int32_t max_depth,
                             int32_t lbg_iters, const uint32_t *h_draws, int32_t draws_per_node, vq_tree **out) {
    if (!ctx || !out) return VQ_ERR_INVALID_ARG;
    *out = nullptr;
    if (max_depth > 20) return fail(ctx, VQ_ERR_UNSUPPORTED, "2-means tree: max_depth %d above 20", max_depth);
    if (lbg_iters < 0 || draws_per_node < 2 + lbg_iters || (max_depth > 0 && !h_draws))
        return fail(ctx, VQ_ERR_INVALID_ARG,
                    "Invalid parameter: a node needs 2 + lbg_iters draws (two initial rows, one re-seed per iteration)");
    KmOpts km{lbg_iters, h_draws, draws_per_node};
    return tsvq_build_impl(ctx, d_x, n, ld, dim, max_depth, &km, out);
}

static int32_t tsvq_build_impl(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t dim, int32_t max_depth,
                               const KmOpts *km, vq_tree **out) {
    if (!ctx || !out) return VQ_ERR_INVALID_ARG;
    *out = nullptr;
    if (n == 0) return fail(ctx, VQ_ERR_EMPTY_INPUT, "Empty input: at least one vector is required.");
    if (!d_x || n < 0 || dim <= 0 || ld < dim || max_depth < 0) return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter");
    if (n >= (1LL << 31)) return fail(ctx, VQ_ERR_UNSUPPORTED, "n must be below 2^31");
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    hipStream_t st = ctx->stream;

    // workspace: two row-id lists, column values, flags, scan
    VQ_TRY(ensure(ctx, ctx->tmp_a, sizeof(uint32_t) * (size_t)n));
    VQ_TRY(ensure(ctx, ctx->tmp_b, sizeof(uint32_t) * (size_t)n));
    VQ_TRY(ensure(ctx, ctx->tmp_c, sizeof(float) * (size_t)n));
    VQ_TRY(ensure(ctx, ctx->tmp_d, sizeof(float) * (size_t)n));
    VQ_TRY(ensure(ctx, ctx->tmp_e, sizeof(uint32_t) * (size_t)n));
    VQ_TRY(ensure(ctx, ctx->tmp_f, sizeof(uint32_t) * (size_t)n));
    // two-step variance (squares on the whole GPU, then the chains): dim a multiple of 8, and room
    // for a level's squares with every node starting on its own group of 32 positions
    constexpr int kChainSegs = 2048;  // levels with more nodes than this take the other kernels
    const bool var_chain = dim % 8 == 0;
    // per group of 32 squares (composed-maps path): approximate sum, binade guess, integer maps;
    // the chain path keeps the squares themselves
    const bool var_maps = var_chain && ctx->tsvq_var_path == 0;
    if (var_chain && !var_maps)
        VQ_TRY(ensure(ctx, ctx->tsvq_sq, sizeof(float) * ((size_t)n + vq::kChainGroup * (size_t)kChainSegs) * dim));
    float *d_sq = (float *)ctx->tsvq_sq.p;
    if (var_maps) {
        const size_t ngroups = ((size_t)n + vq::kChainGroup * (size_t)kChainSegs) / vq::kChainGroup + 2;
        VQ_TRY(ensure(ctx, ctx->tsvq_gsum, sizeof(float) * ngroups * dim));
        VQ_TRY(ensure(ctx, ctx->tsvq_guess, sizeof(uint16_t) * ngroups * dim));
        VQ_TRY(ensure(ctx, ctx->tsvq_maps, sizeof(uint4) * ngroups * dim));
    }
    uint32_t *perm = (uint32_t *)ctx->tmp_a.p, *perm2 = (uint32_t *)ctx->tmp_b.p;
    float *vals = (float *)ctx->tmp_c.p;
    uint32_t *flags = (uint32_t *)ctx->tmp_e.p, *scan = (uint32_t *)ctx->tmp_f.p;
    hipLaunchKernelGGL(vq::k_iota_u32, dim3(cdiv(n, 256)), dim3(256), 0, st, perm, n);

    vq_tree *T = new vq_tree;
    T->device = ctx->device;
    T->dim = dim;
    std::vector<Seg> level{{0, 0u, (uint32_t)n, 1}};
    T->h_left.push_back(-1);
    T->h_right.push_back(-1);
    T->h_split_dim.push_back(-1);
    T->h_split_val.push_back(0.f);
    T->h_count.push_back(n);
    int depth_left = max_depth;

    // small per-level device tables, re-allocated per level (a level has at most 2^level nodes)
    auto cleanup_fail = [&](int32_t rc) {
        tree_release(T);
        return rc;
    };
    int32_t rc = VQ_OK;
    int km_err = 0;  // 2-means: a node ran out of re-seed draws
    struct LevelMeans {
        void *d;
        int32_t first_node;
        int nseg;
    };
    std::vector<LevelMeans> level_means;  // device means of every level, read back after the last one
    std::vector<uint2> desc;
    std::vector<uint4> info;
    std::vector<uint32_t> km_draws, km_first;  // 2-means: the splitting nodes' draws and first parts
    // The means of all nodes in one workspace buffer when the deepest possible tree stays small (nodes
    // are numbered level by level, so a level's means are one run of it); else an allocation per level.
    const uint64_t max_nodes = std::min<uint64_t>(2 * (uint64_t)n - 1, (2ull << std::min(max_depth, 40)) - 1);
    const bool means_arena = max_nodes * (uint64_t)dim * sizeof(float) <= (256ull << 20);
    if (means_arena) VQ_TRY(ensure(ctx, ctx->tsvq_means, sizeof(float) * (size_t)max_nodes * dim));
    auto free_means = [&]() {
        if (!means_arena)
            for (auto &lm : level_means) (void)hipFree(lm.d);
        level_means.clear();
    };
    // A level's small tables go up in ONE copy from page-locked memory and its decisions come back in
    // one: the host waits for the GPU once per level, so the staging area is free again by then.
    auto pinned = [&](size_t bytes) -> int32_t {
        if (bytes <= ctx->tsvq_pin_cap) return VQ_OK;
        if (ctx->tsvq_pin) (void)hipHostFree(ctx->tsvq_pin);
        ctx->tsvq_pin = nullptr;
        ctx->tsvq_pin_cap = 0;
        const size_t want = bytes + bytes / 2 + 4096;
        VQ_HIP(ctx, hipHostMalloc(&ctx->tsvq_pin, want, hipHostMallocDefault));
        ctx->tsvq_pin_cap = want;
        return VQ_OK;
    };
    auto pad = [](size_t z) { return (z + 255) & ~(size_t)255; };

    while (!level.empty()) {
        const int nseg = (int)level.size();
        // ---- means of every node of the level ------------------------------------------------
        desc.clear();  // (both outlive the level: their uploads are enqueued, not waited for)
        info.assign(nseg, make_uint4(0u, 0u, 0u, 0u));
        for (int g = 0; g < nseg; ++g) {
            uint32_t cnt = level[g].hi - level[g].lo;
            int dep = tree_depth(cnt);
            info[g] = make_uint4((uint32_t)desc.size(), (uint32_t)dep, cnt, 0u);
            for (uint32_t l = 0; l < (1u << dep); ++l) {
                uint32_t lo = 0, hi = cnt;
                for (int bit = dep - 1; bit >= 0; --bit) {
                    uint32_t mid = lo + (hi - lo) / 2;
                    if ((l >> bit) & 1u)
                        lo = mid;
                    else
                        hi = mid;
                }
                desc.push_back(make_uint2(level[g].lo + lo, level[g].lo + hi));
            }
        }
        const size_t nleaves = desc.size();
        // ---- which nodes split (src/tsvq.rs:78): their sizes decide, nothing waits for the GPU ----
        std::vector<int> split;  // indices into level
        if (depth_left > 0)
            for (int g = 0; g < nseg; ++g)
                if (level[g].hi - level[g].lo > 1) split.push_back(g);
        const int ns = (int)split.size();
        std::vector<uint2> range(ns);
        for (int i = 0; i < ns; ++i) range[i] = make_uint2(level[split[i]].lo, level[split[i]].hi);
        // The level's tables live in a grow-only arena of the context; its node means stay on the
        // device until the end of the build, when all means are read back at once.
        void *d_desc = nullptr, *d_info = nullptr, *d_range = nullptr, *d_split = nullptr, *d_lsum = nullptr,
             *d_means = nullptr;
#define LV_HIP(call)                                                                              \
    do {                                                                                          \
        hipError_t e__ = (call);                                                                  \
        if (e__ != hipSuccess) {                                                                  \
            (void)hipGetLastError();                                                              \
            free_means();                                                                         \
            return cleanup_fail(fail(ctx, e__ == hipErrorOutOfMemory ? VQ_ERR_OOM : VQ_ERR_HIP,   \
                                     "%s: %s (%s:%d)", #call, hipGetErrorString(e__), __FILE__,   \
                                     __LINE__));                                                  \
        }                                                                                         \
    } while (0)
        // uploaded tables first (one contiguous run: descriptors, node info, ranges, split indices)
        const size_t up_sizes[4] = {sizeof(uint2) * nleaves, sizeof(uint4) * (size_t)nseg, sizeof(uint2) * (size_t)ns,
                                    sizeof(int) * (size_t)ns};
        const void *up_src[4] = {desc.data(), info.data(), range.data(), split.data()};
        size_t up_bytes = 0;
        for (size_t z : up_sizes) up_bytes += pad(z);
        const size_t down_bytes = 3 * sizeof(uint32_t) * (size_t)ns;
        {
            void **ptrs[5] = {&d_desc, &d_info, &d_range, &d_split, &d_lsum};
            const size_t total = up_bytes + pad(sizeof(float) * nleaves * dim);
            int32_t rc = ensure(ctx, ctx->tsvq_level, total);
            if (rc == VQ_OK) rc = pinned(up_bytes + pad(down_bytes));
            if (rc != VQ_OK) {
                free_means();
                return cleanup_fail(rc);
            }
            char *at = (char *)ctx->tsvq_level.p, *h = (char *)ctx->tsvq_pin;
            for (int z = 0; z < 4; ++z) {
                *ptrs[z] = at;
                if (up_sizes[z]) memcpy(h, up_src[z], up_sizes[z]);
                at += pad(up_sizes[z]);
                h += pad(up_sizes[z]);
            }
            d_lsum = at;
        }
        const int32_t first_node = level[0].node;
        if (means_arena)
            d_means = (float *)ctx->tsvq_means.p + (size_t)first_node * dim;
        else
            LV_HIP(hipMalloc(&d_means, sizeof(float) * (size_t)nseg * dim));
        level_means.push_back({d_means, first_node, nseg});
        LV_HIP(hipMemcpyAsync(ctx->tsvq_level.p, ctx->tsvq_pin, up_bytes, hipMemcpyHostToDevice, st));
        hipLaunchKernelGGL(vq::k_seg_leafsum, dim3(cdiv((int64_t)nleaves * dim, 256)), dim3(256), 0, st, perm,
                           (const uint2 *)d_desc, (int64_t)nleaves, d_x, ld, dim, (float *)d_lsum);
        int max_dep = 0;
        for (int g = 0; g < nseg; ++g) max_dep = std::max(max_dep, (int)info[g].y);
        if (max_dep >= 5 && (1 << max_dep) <= vq::kMeanWgLeaves && nseg <= 64)  // few segments of many leaves
            hipLaunchKernelGGL(vq::k_seg_mean_wg, dim3((unsigned)nseg, cdiv(dim, 8)), dim3(256), 0, st,
                               (const float *)d_lsum, (const uint4 *)d_info, dim, (float *)d_means, (int64_t)0);
        else
            hipLaunchKernelGGL(vq::k_seg_mean, dim3(cdiv((int64_t)nseg * dim, 256)), dim3(256), 0, st,
                               (float *)d_lsum, (const uint4 *)d_info, nseg, dim, (float *)d_means, (int64_t)0);
        LV_HIP(hipGetLastError());

        if (split.empty()) break;
        // the level's small tables: one grow-only arena of the context instead of nine allocations;
        // split dimension, median and left count of every node side by side, so that one copy returns them
        void *d_smeans = nullptr, *d_var = nullptr, *d_down = nullptr, *d_sel = nullptr,
             *d_hist = nullptr;
#define SP_HIP(call)                                                                              \
    do {                                                                                          \
        hipError_t e__ = (call);                                                                  \
        if (e__ != hipSuccess) {                                                                  \
            (void)hipGetLastError();                                                              \
            free_means();                                                                         \
            return cleanup_fail(fail(ctx, e__ == hipErrorOutOfMemory ? VQ_ERR_OOM : VQ_ERR_HIP,   \
                                     "%s: %s (%s:%d)", #call, hipGetErrorString(e__), __FILE__,   \
                                     __LINE__));                                                  \
        }                                                                                         \
    } while (0)
        {
            const size_t cap = (size_t)std::max(ns, 1024);  // sized once for the usual depths
            const size_t sizes[5] = {sizeof(float) * cap * dim, sizeof(float) * cap * dim, 3 * sizeof(uint32_t) * cap,
                                     sizeof(vq::SegSelect) * 2 * cap, sizeof(uint32_t) * 512 * cap};
            void **ptrs[5] = {&d_smeans, &d_var, &d_down, &d_sel, &d_hist};
            size_t total = 0;
            for (size_t z : sizes) total += (z + 255) & ~(size_t)255;
            const int32_t rc = ensure(ctx, ctx->tsvq_split, total);
            if (rc != VQ_OK) {
                free_means();
                return cleanup_fail(rc);
            }
            char *at = (char *)ctx->tsvq_split.p;
            for (int z = 0; z < 5; ++z) {
                *ptrs[z] = at;
                at += (sizes[z] + 255) & ~(size_t)255;
            }
        }
        int *d_sdim = (int *)d_down;
        float *d_median = (float *)d_down + ns;
        uint32_t *d_nleft = (uint32_t *)d_down + 2 * (size_t)ns;
        if (km) {
            // ---- 2-means split: lbg_quantize with k = 2 on every splitting node's rows ----------
            km_first.assign((size_t)ns + 1, 0u);
            for (int i = 0; i < ns; ++i)
                km_first[i + 1] = km_first[i] + (uint32_t)cdiv((int64_t)(range[i].y - range[i].x), vq::kKmPart);
            const uint32_t parts = km_first[ns];
            km_draws.resize((size_t)ns * km->per_node);
            for (int i = 0; i < ns; ++i)
                memcpy(km_draws.data() + (size_t)i * km->per_node,
                       km->h_draws + (size_t)(level[split[i]].heap - 1) * km->per_node, sizeof(uint32_t) * km->per_node);
            auto pad4 = [](size_t z) { return (z + 255) & ~(size_t)255; };
            const size_t sz[6] = {sizeof(float) * 2 * (size_t)ns * dim, sizeof(uint32_t) * ((size_t)ns + 1),
                                  sizeof(float) * 2 * (size_t)parts * dim, sizeof(uint32_t) * 2 * (size_t)parts,
                                  sizeof(int) * (4 * (size_t)ns + 1), sizeof(uint32_t) * (size_t)ns * km->per_node};
            size_t total = 0;
            for (size_t z : sz) total += pad4(z);
            {
                const int32_t rc = ensure(ctx, ctx->tsvq_km, total);
                if (rc != VQ_OK) {
                    free_means();
                    return cleanup_fail(rc);
                }
            }
            char *at = (char *)ctx->tsvq_km.p;
            vq::KmState S{};
            S.perm = perm;
            S.range = (const uint2 *)d_range;
            S.per_node = km->per_node;
            S.ns = ns;
            S.cen = (float *)at;
            at += pad4(sz[0]);
            S.part_first = (uint32_t *)at;
            at += pad4(sz[1]);
            S.part_sum = (float *)at;
            at += pad4(sz[2]);
            S.part_cnt = (uint32_t *)at;
            at += pad4(sz[3]);
            int *fl = (int *)at;
            at += pad4(sz[4]);
            S.changed = fl;
            S.done = fl + ns;
            S.used = fl + 2 * (size_t)ns;
            S.iters = fl + 3 * (size_t)ns;
            S.err = fl + 4 * (size_t)ns;
            uint32_t *d_draws = (uint32_t *)at;
            S.draws = d_draws;
            S.codes = (uint8_t *)vals;  // the split column's buffer is not used in this mode
            SP_HIP(hipMemcpyAsync(S.part_first, km_first.data(), sz[1], hipMemcpyHostToDevice, st));
            SP_HIP(hipMemcpyAsync(d_draws, km_draws.data(), sz[5], hipMemcpyHostToDevice, st));
            SP_HIP(hipMemsetAsync(S.codes, 0, (size_t)n, st));  // assignments = vec![0; n], utils.rs:55
            SP_HIP(hipMemsetAsync(S.err, 0, sizeof(int), st));
            hipLaunchKernelGGL(vq::k_km_init, dim3(ns), dim3(256), 0, st, S, d_x, ld, dim);
            const bool reg = dim % 32 == 0 && dim <= 128 && ld % 4 == 0 && (reinterpret_cast<uintptr_t>(d_x) & 15) == 0;
            auto assign = [&](bool lbg, uint32_t *fl_out) {
                const dim3 grid(cdiv(n, 256)), block(256);
#define KM_REG(D)                                                                                          \
    if (lbg)                                                                                               \
        hipLaunchKernelGGL((vq::k_km_assign_reg<true, D>), grid, block, 0, st, S, n, d_x, ld, fl_out);     \
    else                                                                                                   \
        hipLaunchKernelGGL((vq::k_km_assign_reg<false, D>), grid, block, 0, st, S, n, d_x, ld, fl_out)
                if (reg) {
                    switch (dim) {
                    case 32: KM_REG(32); break;
                    case 64: KM_REG(64); break;
                    case 96: KM_REG(96); break;
                    default: KM_REG(128); break;
                    }
                } else if (lbg) {
                    hipLaunchKernelGGL(vq::k_km_assign<true>, grid, block, 0, st, S, n, d_x, ld, dim, fl_out);
                } else {
                    hipLaunchKernelGGL(vq::k_km_assign<false>, grid, block, 0, st, S, n, d_x, ld, dim, fl_out);
                }
#undef KM_REG
            };
            const unsigned sum_threads = dim <= 64 ? 64u : dim <= 128 ? 128u : 256u;
            // the fused kernel where a workgroup may hold its two tiles in LDS, else the two kernels apart
            const void *fused = nullptr;
            if (reg) {
                int optin = 0;
                SP_HIP(hipDeviceGetAttribute(&optin, hipDeviceAttributeSharedMemPerBlockOptin, ctx->device));
                const size_t lds = vq::km_assign_sum_lds(dim);
                if (lds + 24 * 1024 <= (size_t)optin) {  // (+ the kernel's static LDS: the part's row ids, masks, centroids)
                    switch (dim) {
                    case 32: fused = reinterpret_cast<const void *>(vq::k_km_assign_sum<32>); break;
                    case 64: fused = reinterpret_cast<const void *>(vq::k_km_assign_sum<64>); break;
                    case 96: fused = reinterpret_cast<const void *>(vq::k_km_assign_sum<96>); break;
                    default: fused = reinterpret_cast<const void *>(vq::k_km_assign_sum<128>); break;
                    }
                    if (lds > 48 * 1024)
                        SP_HIP(hipFuncSetAttribute(fused, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
                }
            }
            for (int it = 0; it < km->lbg_iters; ++it) {
                if (fused) {  // assignment and part sums in one pass over the rows
                    const size_t lds = vq::km_assign_sum_lds(dim);
                    switch (dim) {
                    case 32: hipLaunchKernelGGL(vq::k_km_assign_sum<32>, dim3(parts), dim3(512), lds, st, S, d_x, ld); break;
                    case 64: hipLaunchKernelGGL(vq::k_km_assign_sum<64>, dim3(parts), dim3(512), lds, st, S, d_x, ld); break;
                    case 96: hipLaunchKernelGGL(vq::k_km_assign_sum<96>, dim3(parts), dim3(512), lds, st, S, d_x, ld); break;
                    default: hipLaunchKernelGGL(vq::k_km_assign_sum<128>, dim3(parts), dim3(512), lds, st, S, d_x, ld); break;
                    }
                } else {
                    assign(true, nullptr);
                    hipLaunchKernelGGL(vq::k_km_partsum, dim3(parts), dim3(sum_threads), 0, st, S, d_x, ld, dim);
                }
                hipLaunchKernelGGL(vq::k_km_update, dim3(ns), dim3(256), 0, st, S, d_x, ld, dim);
            }
            // rows whose nearest of the two final centroids is the first go left
            assign(false, flags);
            SP_HIP(hipGetLastError());
            SP_HIP(hipMemcpyAsync(&km_err, S.err, sizeof(int), hipMemcpyDeviceToHost, st));
        } else {
        // the means of the splitting nodes, compacted on the device
        hipLaunchKernelGGL(vq::k_gather_means, dim3(cdiv((int64_t)ns * dim, 256)), dim3(256), 0, st,
                           (const float *)d_means, (const int *)d_split, ns, dim, (float *)d_smeans);
        // per-dimension sums of squared deviations (src/tsvq.rs:88-99)
        if (var_chain && ns <= kChainSegs) {
            uint32_t longest = 0;
            for (int i = 0; i < ns; ++i) longest = std::max(longest, range[i].y - range[i].x);
            hipLaunchKernelGGL(vq::k_seg_sqdev32, dim3((unsigned)cdiv((int64_t)longest, 64), (unsigned)ns), dim3(256),
                               0, st, perm, (const uint2 *)d_range, (const float *)d_smeans, (int64_t)0, d_x, ld, dim,
                               var_maps ? (float *)nullptr : d_sq, var_maps ? (float *)ctx->tsvq_gsum.p : (float *)nullptr);
            if (var_maps) {
                // columns above kGuessBlock groups: the blocks' sums first, then all blocks side by side
                // (both pay from about 4096 groups per column on: 22 us for the block sums, 48 us for the runs)
                const unsigned nblk_all = cdiv(cdiv((int64_t)longest, 32), vq::kGuessBlock);
                const unsigned nblk = nblk_all > 4 ? nblk_all : 1u;
                double *d_bsum = nullptr;
                if (nblk > 1) {
                    const int32_t rc = ensure(ctx, ctx->tsvq_bsum, sizeof(double) * (size_t)ns * nblk * dim);
                    if (rc != VQ_OK) {
                        free_means();
                        return cleanup_fail(rc);
                    }
                    d_bsum = (double *)ctx->tsvq_bsum.p;
                    hipLaunchKernelGGL(vq::k_seg_chain_bsum, dim3((unsigned)ns, (unsigned)cdiv(dim, 4), nblk), dim3(256), 0,
                                       st, (const float *)ctx->tsvq_gsum.p, (const uint2 *)d_range, dim, d_bsum);
                }
                hipLaunchKernelGGL(vq::k_seg_chain_guess, dim3((unsigned)ns, (unsigned)cdiv(dim, 4), nblk), dim3(256), 0,
                                   st, (const float *)ctx->tsvq_gsum.p, (const uint2 *)d_range, dim,
                                   (const double *)d_bsum, (uint16_t *)ctx->tsvq_guess.p);
                hipLaunchKernelGGL(vq::k_seg_chain_maps, dim3((unsigned)cdiv((int64_t)longest, 64), (unsigned)ns),
                                   dim3(256), 0, st, perm, (const uint2 *)d_range, (const float *)d_smeans, (int64_t)0,
                                   d_x, ld, dim, (const uint16_t *)ctx->tsvq_guess.p, (uint4 *)ctx->tsvq_maps.p);
                // long columns: the maps of runs of 256 groups composed ahead, so that the walk passes a
                // clean run in one step
                uint4 *d_runs = nullptr;
                if (nblk > 1) {
                    const size_t nruns = ((size_t)n + vq::kChainGroup * (size_t)kChainSegs) / (32 * vq::kRunGroups) + ns + 2;
                    const int32_t rc = ensure(ctx, ctx->tsvq_segmaps, sizeof(uint4) * nruns * dim);
                    if (rc != VQ_OK) {
                        free_means();
                        return cleanup_fail(rc);
                    }
                    d_runs = (uint4 *)ctx->tsvq_segmaps.p;
                    hipLaunchKernelGGL(vq::k_seg_chain_runs,
                                       dim3((unsigned)ns, (unsigned)cdiv(dim, 4), cdiv(cdiv((int64_t)longest, 32), 4 * vq::kRunGroups)),
                                       dim3(256), 0, st, (const uint2 *)d_range, dim, (const uint16_t *)ctx->tsvq_guess.p,
                                       (const uint4 *)ctx->tsvq_maps.p, d_runs);
                }
                hipLaunchKernelGGL(vq::k_seg_chain_compose, dim3((unsigned)ns, (unsigned)cdiv(dim, 4)), dim3(256), 0,
                                   st, perm, (const uint2 *)d_range, (const float *)d_smeans, (int64_t)0, d_x, ld, dim,
                                   (const uint16_t *)ctx->tsvq_guess.p, (const uint4 *)ctx->tsvq_maps.p,
                                   (const uint4 *)d_runs, (float *)d_var);
            } else {
                hipLaunchKernelGGL(vq::k_seg_chain32, dim3((unsigned)ns, (unsigned)cdiv(dim, 32)), dim3(256), 0, st,
                                   (const float *)d_sq, (const uint2 *)d_range, dim, (float *)d_var);
            }
        } else if (dim % 4 == 0 && dim <= 1024 && ld % 4 == 0 && (reinterpret_cast<uintptr_t>(d_x) & 15) == 0) {
#define VARIANCE_WG(D)                                                                                     \
    hipLaunchKernelGGL((vq::k_seg_variance_wg<D>), dim3(ns), dim3(1024), 0, st, perm, (const uint2 *)d_range, \
                       (const float *)d_smeans, (int64_t)0, d_x, ld, dim, (float *)d_var)
            switch (dim) {  // the common row lengths get constant LDS strides
            case 32: VARIANCE_WG(32); break;
            case 64: VARIANCE_WG(64); break;
            case 128: VARIANCE_WG(128); break;
            case 256: VARIANCE_WG(256); break;
            default: VARIANCE_WG(0); break;
            }
#undef VARIANCE_WG
        } else
            hipLaunchKernelGGL(vq::k_seg_variance, dim3(cdiv((int64_t)ns * dim, 64)), dim3(64), 0, st, perm,
                               (const uint2 *)d_range, ns, (const float *)d_smeans, (int64_t)0, d_x, ld, dim,
                               (float *)d_var);
        SP_HIP(hipGetLastError());
        // split dimension on the device (src/tsvq.rs:102-106); read back with the left counts below
        hipLaunchKernelGGL(vq::k_seg_argmax_last, dim3(cdiv((int64_t)ns * 512, 256)), dim3(256), 0, st,
                           (const float *)d_var, ns, dim, (int *)d_sdim, (const uint2 *)d_range, (vq::SegSelect *)d_sel,
                           (uint32_t *)d_hist);
        // split column, middle values by radix select (src/tsvq.rs:109-117)
        hipLaunchKernelGGL(vq::k_seg_gather_col, dim3(cdiv(n, 256)), dim3(256), 0, st, perm, n,
                           (const uint2 *)d_range, ns, (const int *)d_sdim, d_x, ld, vals);
        for (int pass = 0; pass < 4; ++pass) {
            hipLaunchKernelGGL(vq::k_seg_select_hist, dim3(cdiv(n, 4096)), dim3(256), 0, st, (const float *)vals, n,
                               (const uint2 *)d_range, ns, (const vq::SegSelect *)d_sel, pass, (uint32_t *)d_hist);
            hipLaunchKernelGGL(vq::k_seg_select_pick, dim3(2 * ns), dim3(64), 0, st, (uint32_t *)d_hist,
                               (vq::SegSelect *)d_sel, ns, pass);
        }
        SP_HIP(hipGetLastError());
        hipLaunchKernelGGL(vq::k_seg_median, dim3(cdiv(ns, 64)), dim3(64), 0, st, (const vq::SegSelect *)d_sel,
                           (const uint2 *)d_range, ns, (float *)d_median);
        // stable partition by `<= median` (src/tsvq.rs:120-123)
        hipLaunchKernelGGL(vq::k_seg_flags, dim3(cdiv(n, 256)), dim3(256), 0, st, vals, n, (const uint2 *)d_range,
                           ns, (const float *)d_median, flags);
        }  // median split
        size_t need = 0;
        SP_HIP(rocprim::exclusive_scan(nullptr, need, flags, scan, 0u, (size_t)n, rocprim::plus<uint32_t>(), st));
        {
            const int32_t rc = ensure(ctx, ctx->tsvq_scan, need);
            if (rc != VQ_OK) {
                free_means();
                return cleanup_fail(rc);
            }
        }
        SP_HIP(rocprim::exclusive_scan(ctx->tsvq_scan.p, need, flags, scan, 0u, (size_t)n, rocprim::plus<uint32_t>(), st));
        hipLaunchKernelGGL(vq::k_seg_partition, dim3(cdiv(n, 256)), dim3(256), 0, st, perm, n,
                           (const uint2 *)d_range, ns, flags, scan, perm2, (uint32_t *)d_nleft);
        SP_HIP(hipGetLastError());
        char *h_down = (char *)ctx->tsvq_pin + up_bytes;
        SP_HIP(hipMemcpyAsync(h_down, d_down, down_bytes, hipMemcpyDeviceToHost, st));
        SP_HIP(hipStreamSynchronize(st));
        const int *sdim = (const int *)h_down;
        const float *median = (const float *)h_down + ns;
        const uint32_t *nleft = (const uint32_t *)h_down + 2 * (size_t)ns;
        std::swap(perm, perm2);
        if (km && km_err) {
            free_means();
            return cleanup_fail(fail(ctx, VQ_ERR_RESEED_EXHAUSTED, "2-means tree: a node met more empty clusters than it has draws"));
        }

        // ---- children (src/tsvq.rs:126-141) ---------------------------------------------------
        std::vector<Seg> next;
        for (int i = 0; i < ns; ++i) {
            const Seg &sg = level[split[i]];
            uint32_t cnt = sg.hi - sg.lo, nl = nleft[i], nr = cnt - nl;
            T->h_split_dim[sg.node] = km ? -1 : sdim[i];
            T->h_split_val[sg.node] = km ? 0.f : median[i];
            const uint64_t heap = sg.heap;
            auto add_child = [&](uint32_t lo, uint32_t hi, uint64_t child_heap) {
                int32_t id = (int32_t)T->h_left.size();
                T->h_left.push_back(-1);
                T->h_right.push_back(-1);
                T->h_split_dim.push_back(-1);
                T->h_split_val.push_back(0.f);
                T->h_count.push_back((int64_t)hi - lo);
                next.push_back({id, lo, hi, child_heap});
                return id;
            };
            if (nl > 0 && nl < cnt) T->h_left[sg.node] = add_child(sg.lo, sg.lo + nl, 2 * heap);
            if (nr > 0 && nr < cnt) T->h_right[sg.node] = add_child(sg.lo + nl, sg.hi, 2 * heap + 1);
        }
        level.swap(next);
        --depth_left;
    }
    T->n_nodes = (int32_t)T->h_left.size();
    T->h_centroids.resize((size_t)T->n_nodes * dim);
    if (means_arena)
        LV_HIP(hipMemcpyAsync(T->h_centroids.data(), ctx->tsvq_means.p, sizeof(float) * (size_t)T->n_nodes * dim,
                              hipMemcpyDeviceToHost, st));
    else
        for (auto &lm : level_means)
            LV_HIP(hipMemcpyAsync(T->h_centroids.data() + (size_t)lm.first_node * dim, lm.d,
                                  sizeof(float) * (size_t)lm.nseg * dim, hipMemcpyDeviceToHost, st));
    LV_HIP(hipStreamSynchronize(st));
#undef LV_HIP
#undef SP_HIP
    rc = tree_to_device(ctx, T, means_arena ? (const float *)ctx->tsvq_means.p : nullptr);
    free_means();
    if (rc != VQ_OK) return cleanup_fail(rc);
    *out = T;
    return VQ_OK;
}

int32_t vq_tree_create(vq_ctx *ctx, int32_t n_nodes, int32_t dim, const float *h_centroids,
                       const int32_t *h_left, const int32_t *h_right, vq_tree **out) {
    if (!ctx || !out) return VQ_ERR_INVALID_ARG;
    *out = nullptr;
    if (n_nodes <= 0 || dim <= 0 || !h_centroids || !h_left || !h_right)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter");
    for (int i = 0; i < n_nodes; ++i)
        if (h_left[i] < -1 || h_left[i] >= n_nodes || h_right[i] < -1 || h_right[i] >= n_nodes ||
            (h_left[i] >= 0 && h_left[i] <= i) || (h_right[i] >= 0 && h_right[i] <= i))
            return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: child index of node %d (children must have larger indices)", i);
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    vq_tree *T = new vq_tree;
    T->device = ctx->device;
    T->n_nodes = n_nodes;
    T->dim = dim;
    T->h_centroids.assign(h_centroids, h_centroids + (size_t)n_nodes * dim);
    T->h_left.assign(h_left, h_left + n_nodes);
    T->h_right.assign(h_right, h_right + n_nodes);
    T->h_split_dim.assign(n_nodes, -1);
    T->h_split_val.assign(n_nodes, 0.f);
    T->h_count.assign(n_nodes, 0);
    int32_t rc = tree_to_device(ctx, T);
    if (rc != VQ_OK) {
        tree_release(T);
        return rc;
    }
    *out = T;
    return VQ_OK;
}

int32_t vq_tree_free(vq_ctx *ctx, vq_tree *tree) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (!tree) return VQ_OK;
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    tree_release(tree);
    return VQ_OK;
}

int32_t vq_tree_info(const vq_tree *tree, int32_t *n_nodes, int32_t *dim) {
    if (!tree) return VQ_ERR_INVALID_ARG;
    if (n_nodes) *n_nodes = tree->n_nodes;
    if (dim) *dim = tree->dim;
    return VQ_OK;
}

int32_t vq_tree_download(const vq_tree *tree, float *h_centroids, int32_t *h_left, int32_t *h_right,
                         int32_t *h_split_dim, float *h_split_val, int64_t *h_count) {
    if (!tree) return VQ_ERR_INVALID_ARG;
    size_t nn = (size_t)tree->n_nodes;
    if (h_centroids) std::copy(tree->h_centroids.begin(), tree->h_centroids.end(), h_centroids);
    if (h_left) std::copy_n(tree->h_left.begin(), nn, h_left);
    if (h_right) std::copy_n(tree->h_right.begin(), nn, h_right);
    if (h_split_dim) std::copy_n(tree->h_split_dim.begin(), nn, h_split_dim);
    if (h_split_val) std::copy_n(tree->h_split_val.begin(), nn, h_split_val);
    if (h_count) std::copy_n(tree->h_count.begin(), nn, h_count);
    return VQ_OK;
}

int32_t vq_ctx_set_tsvq_descend_path(vq_ctx *ctx, int32_t path) {
    if (!ctx || (path != 0 && path != 1)) return VQ_ERR_INVALID_ARG;
    ctx->tsvq_descend_path = path;
    return VQ_OK;
}

int32_t vq_tsvq_descend(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld,
                        const vq_tree *tree, int32_t *d_leaf) {
    if (!ctx || !tree) return VQ_ERR_INVALID_ARG;
    if (n == 0) return VQ_OK;
    if (!d_x || !d_leaf || n < 0) return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter");
    if (ld < tree->dim)
        return fail(ctx, VQ_ERR_DIM_MISMATCH, "Dimension mismatch: expected %d, got %lld", tree->dim, (long long)ld);
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    // rows in registers: dim a multiple of 32 up to 128, 16-byte aligned rows
    if (tree->dim % 32 == 0 && tree->dim <= 128 && ld % 4 == 0 && (reinterpret_cast<uintptr_t>(d_x) & 15) == 0) {
        // one workgroup per compute unit (the staged centroids fill its LDS), walking over the rows
        int cus = 0;
        VQ_HIP(ctx, hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, ctx->device));
        dim3 g(std::min<unsigned>(cdiv(n, 512), (unsigned)std::max(cus, 1))), b(512);
        // cosine and (squared) Euclidean: a step decided by one inner product with the node's vector,
        // the two sums of the reference only where that cannot decide
        if (ctx->tsvq_descend_path == 0 && metric != VQ_MANHATTAN && metric >= VQ_SQEUCLIDEAN && metric <= VQ_COSINE) {
            const bool cosine = metric == VQ_COSINE;
            const float *wt = cosine ? tree->d_wcos : tree->d_wl2, *sc = cosine ? tree->d_sccos : tree->d_scl2;
#define DESC_W(M, D)                                                                                   \
    hipLaunchKernelGGL((vq::k_tsvq_descend_w<M, D>), g, b, 0, ctx->stream, d_x, n, ld, tree->d_centroids, \
                       tree->d_cnorm, tree->d_left, tree->d_right, (int)tree->h_left.size(), wt, sc, d_leaf)
#define DESC_WDIM(M)                                                                                   \
    switch (tree->dim) {                                                                               \
    case 32: DESC_W(M, 32); break;                                                                     \
    case 64: DESC_W(M, 64); break;                                                                     \
    case 96: DESC_W(M, 96); break;                                                                     \
    default: DESC_W(M, 128); break;                                                                    \
    }
            switch (metric) {
            case VQ_SQEUCLIDEAN: DESC_WDIM(vq::M_SQ); break;
            case VQ_EUCLIDEAN: DESC_WDIM(vq::M_EUCLID); break;
            default: DESC_WDIM(vq::M_COS); break;
            }
#undef DESC_WDIM
#undef DESC_W
            VQ_HIP(ctx, hipGetLastError());
            return VQ_OK;
        }
#define DESC_REG(M, D)                                                                                \
    hipLaunchKernelGGL((vq::k_tsvq_descend_reg<M, D>), g, b, 0, ctx->stream, d_x, n, ld,              \
                       tree->d_centroids, tree->d_cnorm, tree->d_left, tree->d_right, (int)tree->h_left.size(),    \
                       d_leaf)
#define DESC_DIM(M)                                                                                   \
    switch (tree->dim) {                                                                              \
    case 32: DESC_REG(M, 32); break;                                                                  \
    case 64: DESC_REG(M, 64); break;                                                                  \
    case 96: DESC_REG(M, 96); break;                                                                  \
    default: DESC_REG(M, 128); break;                                                                 \
    }
        switch (metric) {
        case VQ_SQEUCLIDEAN: DESC_DIM(vq::M_SQ); break;
        case VQ_EUCLIDEAN: DESC_DIM(vq::M_EUCLID); break;
        case VQ_COSINE: DESC_DIM(vq::M_COS); break;
        case VQ_MANHATTAN: DESC_DIM(vq::M_L1); break;
        default: return fail(ctx, VQ_ERR_UNSUPPORTED, "metric %d has no kernel", metric);
        }
#undef DESC_DIM
#undef DESC_REG
        VQ_HIP(ctx, hipGetLastError());
        return VQ_OK;
    }
    dim3 grid(cdiv(n, 256)), block(256);
#define DESC(M)                                                                                       \
    hipLaunchKernelGGL((vq::k_tsvq_descend<M>), grid, block, 0, ctx->stream, d_x, n, ld, tree->dim,   \
                       tree->d_centroids, tree->d_cnorm, tree->d_left, tree->d_right, d_leaf)
    switch (metric) {
    case VQ_SQEUCLIDEAN: DESC(vq::M_SQ); break;
    case VQ_EUCLIDEAN: DESC(vq::M_EUCLID); break;
    case VQ_COSINE: DESC(vq::M_COS); break;
    case VQ_MANHATTAN: DESC(vq::M_L1); break;
    default: return fail(ctx, VQ_ERR_UNSUPPORTED, "metric %d has no kernel", metric);
    }
#undef DESC
    VQ_HIP(ctx, hipGetLastError());
    return VQ_OK;
}

int32_t vq_tsvq_decode_f16(vq_ctx *ctx, const vq_tree *tree, const int32_t *d_leaf, int64_t n, uint16_t *d_out) {
    if (!ctx || !tree) return VQ_ERR_INVALID_ARG;
    if (n == 0) return VQ_OK;
    if (!d_leaf || !d_out || n < 0) return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter");
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    if (tree->dim % 4 == 0 &&
        ((reinterpret_cast<uintptr_t>(tree->d_centroids) | reinterpret_cast<uintptr_t>(d_out)) & 15) == 0)
        hipLaunchKernelGGL(vq::k_tsvq_decode4_f16, dim3(cdiv(n * (tree->dim / 4), 256)), dim3(256), 0, ctx->stream,
                           d_leaf, n, tree->dim, tree->d_centroids, reinterpret_cast<uint2 *>(d_out));
    else
        hipLaunchKernelGGL(vq::k_tsvq_decode_f16, dim3(cdiv(n * tree->dim, 256)), dim3(256), 0, ctx->stream, d_leaf,
                           n, tree->dim, tree->d_centroids, d_out);
    VQ_HIP(ctx, hipGetLastError());
    return VQ_OK;
}

}  // extern "C"
