// libvqhip — codebooks of more than 256 centroids: 16-bit codes (declared in include/vq_hip.h).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>
#include <vector>

#include <rocprim/device/device_radix_sort.hpp>

#include "ctx.hpp"
#include "lbg_update.hpp"
#include "bigk.hpp"

using namespace vqh;

namespace {

template <int METRIC>
void launch_merge(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int m, int sd, int kc, const float *chunk,
                  const uint8_t *win, const float *win_d, int base, float *best, uint16_t *out) {
    hipLaunchKernelGGL(vq::k_chunk_merge<METRIC>, dim3(cdiv(n * m, 256)), dim3(256), 0, ctx->stream, d_x, n, ld, m, sd,
                       kc, chunk, win, win_d, base, best, out);
}

}  // namespace

namespace vqh {

int32_t assign_codes_u16(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t m,
                         int32_t sd, int32_t k, const float *d_codebooks, uint16_t *d_codes) {
    VQ_TRY(check_common(ctx, d_x, n, ld, m, sd, k, 65536));
    if (!d_codebooks || !d_codes) return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: null pointer");
    if (reinterpret_cast<uintptr_t>(d_codes) & 1)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter: d_codes must be 2-byte aligned");
    if (m > 65535) return fail(ctx, VQ_ERR_UNSUPPORTED, "m must be at most 65535");
    if (metric < VQ_SQEUCLIDEAN || metric > VQ_MANHATTAN)
        return fail(ctx, VQ_ERR_UNSUPPORTED, "metric %d has no kernel", metric);
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    const size_t pairs = (size_t)n * m;
    VQ_TRY(ensure(ctx, ctx->big_win, (pairs + 3) & ~(size_t)3));
    uint8_t *win = (uint8_t *)ctx->big_win.p;
    if (k <= vq::kChunk) {  // one chunk: its winner is the answer
        VQ_TRY(assign_codes(ctx, metric, d_x, n, ld, m, sd, k, d_codebooks, win));
        hipLaunchKernelGGL(vq::k_widen_codes, dim3(cdiv((int64_t)pairs, 256)), dim3(256), 0, ctx->stream,
                           (const uint8_t *)win, (int64_t)pairs, d_codes);
        VQ_HIP(ctx, hipGetLastError());
        return VQ_OK;
    }
    VQ_TRY(ensure(ctx, ctx->big_chunk, sizeof(float) * (size_t)m * vq::kChunk * sd));
    VQ_TRY(ensure(ctx, ctx->big_best, sizeof(float) * pairs));
    VQ_TRY(ensure(ctx, ctx->big_wind, sizeof(float) * pairs));
    float *chunk = (float *)ctx->big_chunk.p;
    float *best = (float *)ctx->big_best.p;
    float *wind = (float *)ctx->big_wind.p;
    for (int base = 0; base < k; base += vq::kChunk) {
        const int kc = std::min(vq::kChunk, k - base);
        hipLaunchKernelGGL(vq::k_chunk_tables, dim3(cdiv((int64_t)m * kc * sd, 256)), dim3(256), 0, ctx->stream,
                           d_codebooks, m, k, sd, base, kc, chunk);
        VQ_HIP(ctx, hipGetLastError());
        // the winners' distances come with the codes where the assignment kernel computes them anyway
        bool have_d = false;
        VQ_TRY(assign_codes(ctx, metric, d_x, n, ld, m, sd, kc, chunk, win, wind, &have_d));
        const float *wd = have_d ? wind : nullptr;
        switch (metric) {
        case VQ_SQEUCLIDEAN: launch_merge<vq::M_SQ>(ctx, d_x, n, ld, m, sd, kc, chunk, win, wd, base, best, d_codes); break;
        case VQ_EUCLIDEAN: launch_merge<vq::M_EUCLID>(ctx, d_x, n, ld, m, sd, kc, chunk, win, wd, base, best, d_codes); break;
        case VQ_COSINE: launch_merge<vq::M_COS>(ctx, d_x, n, ld, m, sd, kc, chunk, win, wd, base, best, d_codes); break;
        default: launch_merge<vq::M_L1>(ctx, d_x, n, ld, m, sd, kc, chunk, win, wd, base, best, d_codes); break;
        }
        VQ_HIP(ctx, hipGetLastError());
    }
    return VQ_OK;
}

int32_t lbg_fit_big(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t m, int32_t sd, int32_t k,
                    int32_t max_iters, const uint32_t *h_init_idx, const uint32_t *h_reseed_stream,
                    int32_t n_reseed, float *d_codebooks, int32_t *h_iters_run, int32_t *h_reseeds_used) {
    hipStream_t st = ctx->stream;
    const size_t pairs = (size_t)n * m;
    if (pairs >= (1ULL << 32)) return fail(ctx, VQ_ERR_UNSUPPORTED, "n * m must be below 2^32 when k is above 256");
    const int big_cap = (int)std::min<int64_t>(k, n / (vq::kBigSeqMax + 1) + 1);
    const size_t mk = (size_t)m * k;
    VQ_TRY(ensure(ctx, ctx->big_flags, sizeof(int) * (6 * (size_t)m + 1)));
    VQ_TRY(ensure(ctx, ctx->big_tables, sizeof(uint32_t) * (3 * mk + (size_t)m * big_cap)));
    VQ_TRY(ensure(ctx, ctx->big_codes, sizeof(uint16_t) * pairs));
    VQ_TRY(ensure(ctx, ctx->big_fresh, sizeof(uint16_t) * pairs));
    VQ_TRY(ensure(ctx, ctx->big_keys, sizeof(uint64_t) * pairs));
    VQ_TRY(ensure(ctx, ctx->big_sorted, sizeof(uint64_t) * pairs));
    VQ_TRY(ensure(ctx, ctx->idx, sizeof(uint32_t) * mk));
    VQ_TRY(ensure(ctx, ctx->reseed, sizeof(uint32_t) * ((size_t)m * n_reseed + 1)));
    // keys: row in bits 0-31, code in the next code_bits, column block above; they are written block by
    // block in row order, so the sort covers the bits from 32 up only (a radix sort is stable)
    int code_bits = 1;
    while ((1 << code_bits) < k) ++code_bits;
    unsigned end_bit = 32u + (unsigned)code_bits;
    while (end_bit < 64 && ((uint64_t)(m - 1) >> (end_bit - 32u - (unsigned)code_bits)) != 0) ++end_bit;
    uint64_t *keys = (uint64_t *)ctx->big_keys.p, *sorted = (uint64_t *)ctx->big_sorted.p;
    size_t sort_bytes = 0;
    VQ_HIP(ctx, rocprim::radix_sort_keys(nullptr, sort_bytes, keys, sorted, pairs, 32u, end_bit, st));
    VQ_TRY(ensure(ctx, ctx->big_sort_tmp, sort_bytes));

    vq::BigLbg S;
    int *f = (int *)ctx->big_flags.p;
    S.changed = f;
    S.done = f + m;
    S.iters = f + 2 * m;
    S.used = f + 3 * m;
    S.ubase = f + 4 * m;
    S.nbig = f + 5 * m;
    S.err = f + 6 * m;
    uint32_t *tb = (uint32_t *)ctx->big_tables.p;
    S.count = tb;
    S.start = tb + mk;
    S.empty_rank = tb + 2 * mk;
    S.big_list = tb + 3 * mk;
    S.big_cap = big_cap;
    S.codes = (uint16_t *)ctx->big_codes.p;
    uint16_t *fresh = (uint16_t *)ctx->big_fresh.p;

    VQ_HIP(ctx, hipMemcpyAsync(ctx->idx.p, h_init_idx, sizeof(uint32_t) * mk, hipMemcpyHostToDevice, st));
    if (n_reseed)
        VQ_HIP(ctx, hipMemcpyAsync(ctx->reseed.p, h_reseed_stream, sizeof(uint32_t) * (size_t)m * n_reseed,
                                   hipMemcpyHostToDevice, st));
    VQ_HIP(ctx, hipMemsetAsync(S.codes, 0, sizeof(uint16_t) * pairs, st));  // assignments = vec![0; n], utils.rs:55
    hipLaunchKernelGGL(vq::k_big_init, dim3(cdiv(m, 64)), dim3(64), 0, st, S, m);
    hipLaunchKernelGGL(vq::k_gather_rows, dim3(cdiv((int64_t)mk * sd, 256)), dim3(256), 0, st, d_x, ld, m, k, sd,
                       (const uint32_t *)ctx->idx.p, d_codebooks);
    VQ_HIP(ctx, hipGetLastError());

    std::vector<int> host(6 * (size_t)m + 1);
    for (int it = 0; it < max_iters; ++it) {
        {
            ProfSpan sp(ctx, VQ_PROF_LBG_ASSIGN);
            VQ_TRY(assign_codes_u16(ctx, VQ_SQEUCLIDEAN, d_x, n, ld, m, sd, k, d_codebooks, fresh));
        }
        ProfSpan sp(ctx, VQ_PROF_LBG_UPDATE);
        hipLaunchKernelGGL(vq::k_big_commit, dim3(cdiv(n, 256), m), dim3(256), 0, st, S, (const uint16_t *)fresh, n, m,
                           code_bits, keys);
        VQ_HIP(ctx, hipGetLastError());
        VQ_HIP(ctx, rocprim::radix_sort_keys(ctx->big_sort_tmp.p, sort_bytes, keys, sorted, pairs, 32u, end_bit, st));
        VQ_HIP(ctx, hipMemsetAsync(S.count, 0, sizeof(uint32_t) * mk, st));
        hipLaunchKernelGGL(vq::k_big_bounds, dim3(cdiv((int64_t)pairs, 256)), dim3(256), 0, st, S,
                           (const uint64_t *)sorted, n, m, k, code_bits);
        hipLaunchKernelGGL(vq::k_big_plan, dim3(m), dim3(256), 0, st, S, k);
        hipLaunchKernelGGL(vq::k_big_small_means, dim3(cdiv((int64_t)k * sd, 256), m), dim3(256), 0, st, S,
                           (const uint64_t *)sorted, d_x, n, ld, k, sd, (const uint32_t *)ctx->reseed.p, n_reseed,
                           d_codebooks);
        hipLaunchKernelGGL(vq::k_big_large_means, dim3(big_cap, m), dim3(256), 0, st, S, (const uint64_t *)sorted, d_x,
                           n, ld, k, sd, d_codebooks);
        hipLaunchKernelGGL(vq::k_big_advance, dim3(cdiv(m, 64)), dim3(64), 0, st, S, m);
        VQ_HIP(ctx, hipGetLastError());
        // every column block converged (src/utils.rs:104-106): the remaining passes would change nothing
        VQ_HIP(ctx, hipMemcpyAsync(host.data(), f, sizeof(int) * host.size(), hipMemcpyDeviceToHost, st));
        VQ_HIP(ctx, hipStreamSynchronize(st));
        bool all_done = true;
        for (int s = 0; s < m; ++s) all_done = all_done && host[(size_t)m + s] != 0;
        if (all_done || host[6 * (size_t)m]) break;
    }
    if (max_iters == 0) {
        VQ_HIP(ctx, hipMemcpyAsync(host.data(), f, sizeof(int) * host.size(), hipMemcpyDeviceToHost, st));
        VQ_HIP(ctx, hipStreamSynchronize(st));
    }
    prof_collect(ctx);
    if (h_iters_run) memcpy(h_iters_run, host.data() + 2 * (size_t)m, sizeof(int) * m);
    if (h_reseeds_used) memcpy(h_reseeds_used, host.data() + 3 * (size_t)m, sizeof(int) * m);
    if (host[6 * (size_t)m])
        return fail(ctx, VQ_ERR_RESEED_EXHAUSTED, "re-seed stream exhausted: pass n_reseed = k*max_iters");
    return VQ_OK;
}

}  // namespace vqh

extern "C" {

int32_t vq_assign_u16(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t m, int32_t sd,
                      int32_t k, const float *d_codebooks, uint16_t *d_codes) {
    return vqh::assign_codes_u16(ctx, metric, d_x, n, ld, m, sd, k, d_codebooks, d_codes);
}

}  // extern "C"
