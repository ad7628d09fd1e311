// libvqhip — entry points around the assignment for ResidualQuantizer and
// OptimizedProductQuantizer (declared in include/vq_hip.h).
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

#include "ctx.hpp"
#include "rvq_opq.hpp"
#include "procrustes_host.hpp"
#include "polar.hpp"

using namespace vqh;

namespace {

template <typename CodeT>
int32_t residual_sub(vq_ctx *ctx, float *d_res, int64_t n, int64_t ld, int32_t dim, int32_t k, int32_t k_max,
                     const float *d_codebook, const CodeT *d_codes) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (n == 0) return VQ_OK;
    if (!d_res || !d_codebook || !d_codes || n < 0 || dim <= 0 || ld < dim || k <= 0 || k > k_max)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter");
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    if (dim % 4 == 0 && ld % 4 == 0 &&
        ((reinterpret_cast<uintptr_t>(d_res) | reinterpret_cast<uintptr_t>(d_codebook)) & 15) == 0)
        hipLaunchKernelGGL(vq::k_residual_sub4<CodeT>, dim3(cdiv(n * (dim / 4), 1024)), dim3(256), 0, ctx->stream,
                           d_res, n, ld, dim / 4, d_codebook, d_codes, (const uint8_t *)nullptr, (CodeT *)nullptr, 0, 0,
                           (uint8_t *)nullptr, (const float *)d_res, ld);
    else
        hipLaunchKernelGGL(vq::k_residual_sub<CodeT>, dim3(cdiv(n * dim, 256)), dim3(256), 0, ctx->stream, d_res, n,
                           ld, dim, d_codebook, d_codes, 1);
    VQ_HIP(ctx, hipGetLastError());
    return VQ_OK;
}

inline int32_t assign_any(vq_ctx *ctx, int32_t metric, const float *x, int64_t n, int64_t ld, int32_t dim,
                          int32_t k, const float *cb, uint8_t *codes) {
    return assign_codes(ctx, metric, x, n, ld, 1, dim, k, cb, codes);
}
inline int32_t assign_any(vq_ctx *ctx, int32_t metric, const float *x, int64_t n, int64_t ld, int32_t dim,
                          int32_t k, const float *cb, uint16_t *codes) {
    return assign_codes_u16(ctx, metric, x, n, ld, 1, dim, k, cb, codes);
}

template <typename CodeT>
int32_t rvq_encode(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t dim, int32_t stages,
                   int32_t k, int32_t k_max, const float *d_codebooks, float epsilon, CodeT *d_codes,
                   uint8_t *d_stages_used, uint16_t *d_recon_f16) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (n == 0) return VQ_OK;
    if (!d_x || !d_codebooks || !d_codes || n < 0 || dim <= 0 || ld < dim || stages < 0 || k <= 0 || k > k_max ||
        stages > 255)
        return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter");
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    hipStream_t st = ctx->stream;
    const bool vec4 = dim % 4 == 0 && (reinterpret_cast<uintptr_t>(d_codebooks) & 15) == 0;
    // The first stage reads the caller's rows where they lie and writes the first residual; the last
    // stage leaves the residual alone.  One stage then needs no residual buffer at all.
    const bool direct = vec4 && ld % 4 == 0 && (reinterpret_cast<uintptr_t>(d_x) & 15) == 0;
    const bool need_res = stages > 1 || (stages == 1 && !direct);
    if (need_res) VQ_TRY(ensure(ctx, ctx->tmp_c, sizeof(float) * (size_t)n * dim));   // residual
    const size_t codes_bytes = ((size_t)n * sizeof(CodeT) + 3) & ~(size_t)3;
    VQ_TRY(ensure(ctx, ctx->tmp_e, 2 * codes_bytes + 2 * (size_t)n + 16));  // stage codes (two), active, used
    VQ_TRY(ensure(ctx, ctx->tmp_a, sizeof(float) * (size_t)n));         // row norms
    float *norms = (float *)ctx->tmp_a.p;
    float *res = (float *)ctx->tmp_c.p;
    CodeT *stage_codes[2] = {(CodeT *)ctx->tmp_e.p, (CodeT *)((uint8_t *)ctx->tmp_e.p + codes_bytes)};
    uint8_t *active = (uint8_t *)ctx->tmp_e.p + 2 * codes_bytes;
    uint8_t *used = active + n;
    // With no norm test between the stages (epsilon <= 0: every row uses every stage) the update of
    // the residual by a stage's centroids waits for the next stage's assignment, where that pass can
    // take it along: one pass over the rows per stage instead of two.
    bool defer = false;
    if constexpr (sizeof(CodeT) == 1)
        defer = !(epsilon > 0.0f) && stages > 1 && k >= 2 && vec4 &&
                assign_pending_fusable(ctx, metric, res, n, dim, dim, k, d_codebooks);
    if (need_res && !direct)
        VQ_HIP(ctx, hipMemcpy2DAsync(res, sizeof(float) * dim, d_x, sizeof(float) * ld, sizeof(float) * dim,
                                     (size_t)n, hipMemcpyDeviceToDevice, st));
    hipLaunchKernelGGL(vq::k_fill<uint8_t>, dim3(cdiv(n, 256)), dim3(256), 0, st, active, n, (uint8_t)1);
    hipLaunchKernelGGL(vq::k_fill<uint8_t>, dim3(cdiv(n, 256)), dim3(256), 0, st, used, n, (uint8_t)0);
    const float *pend_cb = nullptr;  // the stage whose update of the residual is still to come
    const CodeT *pend_codes = nullptr;
    bool pend_from_x = false;        // ... and reads the caller's rows
    for (int s = 0; s < stages; ++s) {
        const float *cb = d_codebooks + (size_t)s * k * dim;
        CodeT *cur = stage_codes[s & 1];
        const bool from_x = direct && s == 0;
        const float *rows = from_x ? d_x : res;
        const int64_t rows_ld = from_x ? ld : (int64_t)dim;
        if (k < 2) {  // src/rvq.rs:186-187
            hipLaunchKernelGGL(vq::k_fill<CodeT>, dim3(cdiv(n, 256)), dim3(256), 0, st, cur, n, (CodeT)0);
        } else if (pend_cb) {
            if constexpr (sizeof(CodeT) == 1) {
                const PendingUpdate pu{pend_cb, pend_codes, pend_from_x ? d_x : nullptr, pend_from_x ? ld : 0};
                VQ_TRY(assign_codes(ctx, metric, res, n, dim, 1, dim, k, cb, cur, nullptr, nullptr, &pu));
            }
            pend_cb = nullptr;
        } else {
            VQ_TRY(assign_any(ctx, metric, rows, n, rows_ld, dim, k, cb, cur));
        }
        if (s == stages - 1 || defer) {
            hipLaunchKernelGGL(vq::k_rvq_stage_record<CodeT>, dim3(cdiv(n, 256)), dim3(256), 0, st, n,
                               (const CodeT *)cur, (const uint8_t *)active, d_codes, stages, s, used);
            if (s == stages - 1) break;
            pend_cb = cb;
            pend_codes = cur;
            pend_from_x = from_x;
            continue;
        }
        if (vec4)
            hipLaunchKernelGGL(vq::k_residual_sub4<CodeT>, dim3(cdiv(n * (dim / 4), 1024)), dim3(256), 0, st, res, n,
                               (int64_t)dim, dim / 4, cb, (const CodeT *)cur, (const uint8_t *)active, d_codes,
                               stages, s, used, rows, rows_ld);
        else
            hipLaunchKernelGGL(vq::k_rvq_stage_apply<CodeT>, dim3(cdiv(n * dim, 256)), dim3(256), 0, st, res, n, dim,
                               cb, (const CodeT *)cur, d_codes, stages, s, (const uint8_t *)active, used);
        if (epsilon > 0.0f) {  // a norm is never below a non-positive threshold
            hipLaunchKernelGGL(vq::k_row_norms, dim3(cdiv(n, 64)), dim3(64), 0, st, res, n, (int64_t)dim, dim,
                               norms);
            hipLaunchKernelGGL(vq::k_rvq_stage_stop, dim3(cdiv(n, 256)), dim3(256), 0, st, norms, n, epsilon,
                               active);
        }
    }
    if (d_stages_used)
        VQ_HIP(ctx, hipMemcpyAsync(d_stages_used, used, (size_t)n, hipMemcpyDeviceToDevice, st));
    if (d_recon_f16) {
        if (vec4 && (reinterpret_cast<uintptr_t>(d_recon_f16) & 7) == 0)
            hipLaunchKernelGGL(vq::k_rvq_recon4_f16<CodeT>, dim3(cdiv(n * (dim / 4), 1024)), dim3(256), 0, st, n,
                               dim / 4, k, d_codebooks, (const CodeT *)d_codes, stages, (const uint8_t *)used,
                               d_recon_f16);
        else
            hipLaunchKernelGGL(vq::k_rvq_recon_f16<CodeT>, dim3(cdiv(n * dim, 256)), dim3(256), 0, st, n, dim, k,
                               d_codebooks, (const CodeT *)d_codes, stages, (const uint8_t *)used, d_recon_f16);
    }
    VQ_HIP(ctx, hipGetLastError());
    return VQ_OK;
}

}  // namespace

namespace {

// R = the orthogonal polar factor of A^T by Newton-Schulz steps (polar.hpp).  *done = false when the
// iteration has not converged within its step limit (the caller then takes the SVD).
int32_t polar_newton_schulz(vq_ctx *ctx, const double *h_A, int dim, double *h_R, bool *done) {
    *done = false;
    if (dim > vq::kPolarMaxDim) return VQ_OK;
    const int P = (dim + 15) / 16 * 16;
    const size_t total = (size_t)P * P;
    // |A|_1 and |A|_inf: largest column and row sums of |a|
    std::vector<double> colsum((size_t)dim, 0.0);
    double norm_inf = 0.0;
    for (int i = 0; i < dim; ++i) {
        double r = 0.0;
        for (int j = 0; j < dim; ++j) {
            const double v = std::fabs(h_A[(size_t)i * dim + j]);
            r += v;
            colsum[j] += v;
        }
        norm_inf = std::max(norm_inf, r);
    }
    double norm_1 = 0.0;
    for (double c : colsum) norm_1 = std::max(norm_1, c);
    double fro = 0.0;
    for (size_t e = 0; e < (size_t)dim * dim; ++e) fro += h_A[e] * h_A[e];
    // two upper bounds of the largest singular value; the smaller one
    const double scale = std::min(std::sqrt(fro), std::sqrt(norm_1) * std::sqrt(norm_inf));
    if (!(scale > 0.0) || !std::isfinite(scale)) return VQ_OK;  // zero or non-finite: the SVD path decides
    std::vector<double> x0(total, 0.0);  // A^T / scale, zero-padded to P x P
    const double inv = 1.0 / scale;
    for (int i = 0; i < dim; ++i)
        for (int j = 0; j < dim; ++j) x0[(size_t)j * P + i] = h_A[(size_t)i * dim + j] * inv;
    VQ_TRY(ensure(ctx, ctx->tmp_a, sizeof(double) * total));
    VQ_TRY(ensure(ctx, ctx->tmp_b, sizeof(double) * total));
    VQ_TRY(ensure(ctx, ctx->tmp_f, 1024));
    double *X[2] = {(double *)ctx->tmp_a.p, (double *)ctx->tmp_b.p};
    unsigned long long *errs = (unsigned long long *)ctx->tmp_f.p;  // kPolarMaxSteps of them, then the flags
    int *fin = (int *)(errs + vq::kPolarMaxSteps);
    static_assert(sizeof(unsigned long long) * vq::kPolarMaxSteps + sizeof(int) * (vq::kPolarMaxSteps + 2) <= 1024,
                  "step tables");
    hipStream_t st = ctx->stream;
    VQ_HIP(ctx, hipMemsetAsync(ctx->tmp_f.p, 0, 1024, st));
    VQ_HIP(ctx, hipMemcpyAsync(X[0], x0.data(), sizeof(double) * total, hipMemcpyHostToDevice, st));
    const unsigned strips = (unsigned)(P / 16), waves = strips < 8u ? strips : 8u;
    const size_t lds = sizeof(double) * 16 * (size_t)P;
    if (lds > 48 * 1024)
        VQ_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(vq::k_polar_step<0>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    unsigned long long h_errs[vq::kPolarMaxSteps];
    int s = 0, last = -1;
    double low = 1e-3;  // assumed lower bound of the singular values after the first (plain) step
    while (s < vq::kPolarMaxSteps && last < 0) {
        const int upto = std::min(vq::kPolarMaxSteps, s == 0 ? 16 : s + 6);
        for (; s < upto; ++s) {
            double rho = 1.0;
            if (s > 0 && low < 0.9) {
                rho = std::sqrt(3.0 / (1.0 + low + low * low));
                low = rho * low * (3.0 - rho * rho * low * low) * 0.5;
            }
            if (P == 128)
                hipLaunchKernelGGL(vq::k_polar_step<8>, dim3(strips), dim3(64 * waves), lds, st,
                                   (const double *)X[s & 1], P, dim, s, rho, errs, fin, X[(s + 1) & 1]);
            else
                hipLaunchKernelGGL(vq::k_polar_step<0>, dim3(strips), dim3(64 * waves), lds, st,
                                   (const double *)X[s & 1], P, dim, s, rho, errs, fin, X[(s + 1) & 1]);
        }
        VQ_HIP(ctx, hipGetLastError());
        VQ_HIP(ctx, hipMemcpyAsync(h_errs, errs, sizeof(unsigned long long) * s, hipMemcpyDeviceToHost, st));
        VQ_HIP(ctx, hipStreamSynchronize(st));
        for (int t = 0; t < s && last < 0; ++t) {
            double e;
            std::memcpy(&e, &h_errs[t], sizeof e);
            if (e < vq::kPolarLastStepErr) last = t;
        }
    }
    if (last < 0) return VQ_OK;
    std::vector<double> r(total);
    VQ_HIP(ctx, hipMemcpyAsync(r.data(), X[(last + 1) & 1], sizeof(double) * total, hipMemcpyDeviceToHost, st));
    VQ_HIP(ctx, hipStreamSynchronize(st));
    for (int i = 0; i < dim; ++i)
        for (int j = 0; j < dim; ++j) h_R[(size_t)i * dim + j] = r[(size_t)i * P + j];
    *done = true;
    return VQ_OK;
}

}  // namespace

extern "C" {

int32_t vq_residual_sub(vq_ctx *ctx, float *d_res, int64_t n, int64_t ld, int32_t dim, int32_t k,
                        const float *d_codebook, const uint8_t *d_codes) {
    return residual_sub<uint8_t>(ctx, d_res, n, ld, dim, k, 256, d_codebook, d_codes);
}

int32_t vq_residual_sub_u16(vq_ctx *ctx, float *d_res, int64_t n, int64_t ld, int32_t dim, int32_t k,
                            const float *d_codebook, const uint16_t *d_codes) {
    return residual_sub<uint16_t>(ctx, d_res, n, ld, dim, k, 65536, d_codebook, d_codes);
}

int32_t vq_rvq_encode(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t dim,
                      int32_t stages, int32_t k, const float *d_codebooks, float epsilon, uint8_t *d_codes,
                      uint8_t *d_stages_used, uint16_t *d_recon_f16) {
    return rvq_encode<uint8_t>(ctx, metric, d_x, n, ld, dim, stages, k, 256, d_codebooks, epsilon, d_codes,
                               d_stages_used, d_recon_f16);
}

int32_t vq_rvq_encode_u16(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t dim,
                          int32_t stages, int32_t k, const float *d_codebooks, float epsilon, uint16_t *d_codes,
                          uint8_t *d_stages_used, uint16_t *d_recon_f16) {
    return rvq_encode<uint16_t>(ctx, metric, d_x, n, ld, dim, stages, k, 65536, d_codebooks, epsilon, d_codes,
                                d_stages_used, d_recon_f16);
}

int32_t vq_mean_l2norm(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t dim, float *h_out) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (n == 0) return fail(ctx, VQ_ERR_EMPTY_INPUT, "Empty input: at least one vector is required.");
    if (!d_x || !h_out || n < 0 || dim <= 0 || ld < dim) return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter");
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    const int64_t per_block = 4096;
    const int blocks = (int)cdiv(n, per_block);
    VQ_TRY(ensure(ctx, ctx->tmp_a, sizeof(float) * (size_t)n));
    VQ_TRY(ensure(ctx, ctx->tmp_b, sizeof(double) * ((size_t)blocks + 1)));
    float *norms = (float *)ctx->tmp_a.p;
    double *part = (double *)ctx->tmp_b.p;
    hipLaunchKernelGGL(vq::k_row_norms, dim3(cdiv(n, 64)), dim3(64), 0, ctx->stream, d_x, n, ld, dim, norms);
    hipLaunchKernelGGL(vq::k_sum_f64, dim3(blocks), dim3(256), 0, ctx->stream, norms,
                       (const double *)nullptr, n, per_block, part);
    hipLaunchKernelGGL(vq::k_sum_f64, dim3(1), dim3(256), 0, ctx->stream, (const float *)nullptr, part,
                       (int64_t)blocks, (int64_t)blocks, part + blocks);
    VQ_HIP(ctx, hipGetLastError());
    double total = 0.0;
    VQ_HIP(ctx, hipMemcpyAsync(&total, part + blocks, sizeof(double), hipMemcpyDeviceToHost, ctx->stream));
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    *h_out = (float)total / (float)n;  // src/rvq.rs:137-138
    return VQ_OK;
}

int32_t vq_rotate(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t dim, const float *d_R,
                  float *d_y) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (n == 0) return VQ_OK;
    if (!d_x || !d_R || !d_y || n < 0 || dim <= 0 || ld < dim) return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter");
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    // matrix-core kernel: dim a multiple of 32 up to 256, rows and output 16-byte aligned
    if (dim % 32 == 0 && dim <= 256 && ld % 4 == 0 &&
        ((reinterpret_cast<uintptr_t>(d_x) | reinterpret_cast<uintptr_t>(d_y)) & 15) == 0) {
        // operand table: 32 bytes per (output dimension, 4 input dimensions)
        VQ_TRY(ensure(ctx, ctx->tmp_f, 8 * (size_t)dim * dim));
        vq::rot_u32x4 *rtab = (vq::rot_u32x4 *)ctx->tmp_f.p;
        hipLaunchKernelGGL(vq::k_rotate_prep, dim3(cdiv((int64_t)dim * dim / 4, 256)), dim3(256), 0, ctx->stream,
                           d_R, dim, rtab);
        // dim <= 128: the table (dim / 32 x 32 KB) stays in LDS, one workgroup per compute unit
#define ROTATE_RESIDENT(NB, TILES)                                                                              \
    do {                                                                                                        \
        const size_t lds = (size_t)NB * 32 * 1024;                                                              \
        auto kern = vq::k_rotate_mfma_resident<NB, TILES>;                                                      \
        VQ_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                                   \
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                 \
        hipDeviceProp_t prop;                                                                                   \
        VQ_HIP(ctx, hipGetDeviceProperties(&prop, ctx->device));                                                \
        const int64_t groups = cdiv(n, 32 * TILES);                                                             \
        const unsigned wgs = (unsigned)std::min<int64_t>(prop.multiProcessorCount, cdiv(groups, 8));            \
        hipLaunchKernelGGL(kern, dim3(wgs), dim3(512), lds, ctx->stream, d_x, n, ld,                            \
                           (const vq::rot_u32x4 *)rtab, d_y);                                                   \
    } while (0)
#define ROTATE(NB, TILES)                                                                                    \
    hipLaunchKernelGGL((vq::k_rotate_mfma<NB, TILES>), dim3(cdiv(n, 128 * TILES)), dim3(256), 0, ctx->stream, \
                       d_x, n, ld, (const vq::rot_u32x4 *)rtab, d_y)
        switch (dim / 32) {
        case 1: ROTATE_RESIDENT(1, 2); break;
        case 2: ROTATE_RESIDENT(2, 2); break;
        case 3: ROTATE_RESIDENT(3, 2); break;
        case 4: ROTATE_RESIDENT(4, 2); break;
        case 5: ROTATE(5, 1); break;
        case 6: ROTATE(6, 1); break;
        case 7: ROTATE(7, 1); break;
        default: ROTATE(8, 1); break;
        }
#undef ROTATE
#undef ROTATE_RESIDENT
        VQ_HIP(ctx, hipGetLastError());
        return VQ_OK;
    }
    size_t lds = sizeof(float) * 64 * ((size_t)dim + 1);
    if (lds > 160 * 1024) return fail(ctx, VQ_ERR_UNSUPPORTED, "rotation: dim %d too large", dim);
    if (lds > 48 * 1024)
        VQ_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(vq::k_rotate_generic),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(vq::k_rotate_generic, dim3(cdiv(n, 64)), dim3(256), lds, ctx->stream, d_x, n, ld,
                       dim, d_R, d_y);
    VQ_HIP(ctx, hipGetLastError());
    return VQ_OK;
}

int32_t vq_cross_cov(vq_ctx *ctx, const float *d_y, const float *d_x, int64_t n, int32_t dim, double *h_A) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (n == 0) return fail(ctx, VQ_ERR_EMPTY_INPUT, "Empty input: at least one vector is required.");
    if (!d_y || !d_x || !h_A || n < 0 || dim <= 0) return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter");
    if (dim > 4096) return fail(ctx, VQ_ERR_UNSUPPORTED, "cross-covariance: dim %d > 4096", dim);
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    // chunks of 2048 rows up to dim 128; longer chunks for larger matrices, so that the partial
    // sums (one dim x dim matrix per chunk) stay at about 64 B per row
    const int64_t scale = ((int64_t)dim + 127) / 128;
    const int64_t rows_per_chunk = 2048 * scale * scale;
    const int chunks = (int)cdiv(n, rows_per_chunk);
    const int total = dim * dim;
    VQ_TRY(ensure(ctx, ctx->tmp_a, sizeof(double) * (size_t)chunks * total));
    VQ_TRY(ensure(ctx, ctx->tmp_b, sizeof(double) * (size_t)total));
    VQ_TRY(ensure(ctx, ctx->tmp_c, sizeof(double) * (size_t)total * ((chunks + 31) / 32)));
    if (dim % 16 == 0) {
        const int nt_all = dim / 16, full = dim / 128, rest = nt_all % 8;
        double *part = (double *)ctx->tmp_a.p;
#define CROSSCOV(NT, B0, Z)                                                                                 \
    hipLaunchKernelGGL((vq::k_crosscov_mfma<NT>), dim3(chunks, (nt_all + 7) / 8, Z), dim3(256), 0, ctx->stream, \
                       d_y, d_x, n, dim, B0, rows_per_chunk, part)
        if (full) CROSSCOV(8, 0, full);
        switch (rest) {
        case 1: CROSSCOV(1, 128 * full, 1); break;
        case 2: CROSSCOV(2, 128 * full, 1); break;
        case 3: CROSSCOV(3, 128 * full, 1); break;
        case 4: CROSSCOV(4, 128 * full, 1); break;
        case 5: CROSSCOV(5, 128 * full, 1); break;
        case 6: CROSSCOV(6, 128 * full, 1); break;
        case 7: CROSSCOV(7, 128 * full, 1); break;
        default: break;
        }
#undef CROSSCOV
    } else {
        const int tiles = (dim + 127) / 128;
        hipLaunchKernelGGL(vq::k_crosscov_partial, dim3(chunks, tiles * tiles), dim3(256), 0, ctx->stream, d_y, d_x,
                           n, dim, rows_per_chunk, (double *)ctx->tmp_a.p);
    }
    // chunk sums in groups of 32 chunks, then the groups
    const int per_group = 32, groups = (chunks + per_group - 1) / per_group;
    hipLaunchKernelGGL(vq::k_crosscov_reduce, dim3(cdiv(total, 256), groups), dim3(256), 0, ctx->stream,
                       (const double *)ctx->tmp_a.p, chunks, per_group, total, (double *)ctx->tmp_c.p);
    hipLaunchKernelGGL(vq::k_crosscov_reduce, dim3(cdiv(total, 256), 1), dim3(256), 0, ctx->stream,
                       (const double *)ctx->tmp_c.p, groups, groups, total, (double *)ctx->tmp_b.p);
    VQ_HIP(ctx, hipGetLastError());
    VQ_HIP(ctx, hipMemcpyAsync(h_A, ctx->tmp_b.p, sizeof(double) * total, hipMemcpyDeviceToHost, ctx->stream));
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return VQ_OK;
}

int32_t vq_ctx_set_procrustes_path(vq_ctx *ctx, int32_t path) {
    if (!ctx || (path != 0 && path != 1)) return VQ_ERR_INVALID_ARG;
    ctx->procrustes_path = path;
    return VQ_OK;
}

int32_t vq_procrustes_rotation(vq_ctx *ctx, const double *h_A, int32_t dim, double *h_R) {
    if (!ctx) return VQ_ERR_INVALID_ARG;
    if (!h_A || !h_R || dim < 1) return fail(ctx, VQ_ERR_INVALID_ARG, "Invalid parameter");
    if (dim > 4096) return fail(ctx, VQ_ERR_UNSUPPORTED, "rotation update: dim %d above 4096", dim);
    const size_t total = (size_t)dim * dim;
    // First the polar factor by Newton-Schulz steps on the f64 matrix cores (any dim up to 512); a
    // matrix that does not converge there — singular, badly conditioned, non-finite — takes the
    // one-sided Jacobi SVD: on the device for even dim up to 128, else the same routine on the host
    // (the reference runs its SVD on the host as well, src/opq.rs:180).
    if (dim > vq::kPolarMaxDim && (dim > vq::kJacobiMax || dim % 2 != 0)) {
        vqh::procrustes_host(h_A, (size_t)dim, h_R);
        return VQ_OK;
    }
    VQ_HIP(ctx, hipSetDevice(ctx->device));
    if (ctx->procrustes_path == 0) {
        bool done = false;
        VQ_TRY(polar_newton_schulz(ctx, h_A, dim, h_R, &done));
        if (done) return VQ_OK;
    }
    if (dim > vq::kJacobiMax || dim % 2 != 0) {
        vqh::procrustes_host(h_A, (size_t)dim, h_R);
        return VQ_OK;
    }
    const int half = dim / 2;
    VQ_TRY(ensure(ctx, ctx->tmp_a, sizeof(double) * total));
    VQ_TRY(ensure(ctx, ctx->tmp_b, sizeof(double) * total));
    VQ_TRY(ensure(ctx, ctx->tmp_c, sizeof(double) * (total + dim)));
    VQ_TRY(ensure(ctx, ctx->tmp_d, sizeof(double) * total));
    VQ_TRY(ensure(ctx, ctx->tmp_e, sizeof(double2) * (size_t)vq::kJacobiSweeps * (dim - 1) * half));
    VQ_TRY(ensure(ctx, ctx->tmp_f, 256));
    double *d_A = (double *)ctx->tmp_a.p, *d_vt = (double *)ctx->tmp_b.p, *d_uhat = (double *)ctx->tmp_c.p;
    double *d_sv = d_uhat + total;
    double *d_out = (double *)ctx->tmp_d.p;
    double2 *d_rot = (double2 *)ctx->tmp_e.p;
    int *d_rounds = (int *)ctx->tmp_f.p;
    VQ_HIP(ctx, hipMemcpyAsync(d_A, h_A, sizeof(double) * total, hipMemcpyHostToDevice, ctx->stream));
    constexpr int kLanes = 8;
    const size_t lds = sizeof(double) * (size_t)dim * vq::kJacobiStride;
    VQ_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(vq::k_jacobi_sweeps<kLanes>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(vq::k_jacobi_sweeps<kLanes>, dim3(1), dim3(64 * kLanes), lds, ctx->stream, (const double *)d_A,
                       dim, d_rot, d_rounds, d_uhat, d_sv);
    hipLaunchKernelGGL(vq::k_jacobi_accumulate, dim3(dim), dim3(64), 0, ctx->stream, (const double2 *)d_rot,
                       (const int *)d_rounds, dim, d_vt);
    hipLaunchKernelGGL(vq::k_jacobi_product, dim3((unsigned)cdiv(total, 256)), dim3(256), 0, ctx->stream,
                       (const double *)d_vt, (const double *)d_uhat, dim, d_out);
    VQ_HIP(ctx, hipGetLastError());
    std::vector<double> sv((size_t)dim);
    VQ_HIP(ctx, hipMemcpyAsync(h_R, d_out, sizeof(double) * total, hipMemcpyDeviceToHost, ctx->stream));
    VQ_HIP(ctx, hipMemcpyAsync(sv.data(), d_sv, sizeof(double) * dim, hipMemcpyDeviceToHost, ctx->stream));
    VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
    // A singular A leaves directions of U open (their columns came back as zero or as rounding
    // noise): complete them on the host and form the product again.  Rare; a full-rank A ends here.
    double top = 0.0;
    for (double v : sv) top = std::max(top, v);
    bool open = false;
    for (double v : sv) open = open || !(top > 0.0 && v > vqh::kNullRel * top);
    if (open) {
        std::vector<double> Ut(total), Vt(total);
        VQ_HIP(ctx, hipMemcpyAsync(Ut.data(), d_uhat, sizeof(double) * total, hipMemcpyDeviceToHost, ctx->stream));
        VQ_HIP(ctx, hipMemcpyAsync(Vt.data(), d_vt, sizeof(double) * total, hipMemcpyDeviceToHost, ctx->stream));
        VQ_HIP(ctx, hipStreamSynchronize(ctx->stream));
        vqh::complete_null_columns(Ut, Vt, sv, (size_t)dim);
        vqh::product_v_ut(Vt, Ut, (size_t)dim, h_R);
    }
    return VQ_OK;
}

}  // extern "C"
