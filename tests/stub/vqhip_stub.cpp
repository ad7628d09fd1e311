// A stand-in for libvqhip on machines without a GPU, for ONE purpose: running the host mirror
// (vq_amd/host/vq.hpp, vq_host_c.cpp) under the address and undefined-behaviour sanitizers.  Test
// infrastructure only: nothing in the package loads it.  "Device" memory is host memory of exactly
// the size asked for, so a buffer the host mirror sizes wrongly is an out-of-bounds access the
// sanitizer reports; every entry point reads all of its inputs and writes all of its outputs, with
// values that are simple functions of the inputs (not the library's results).
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/vq_hip.h"

struct vq_ctx {
    std::string err;
    long live = 0;  // allocations not yet freed
};
struct vq_tree {
    int32_t n_nodes = 0, dim = 0;
    std::vector<float> cen;
    std::vector<int32_t> left, right;
};

namespace {
uint32_t checksum = 0;  // keeps the reads of the inputs alive
template <class T> void touch(const T *p, size_t count) {
    const unsigned char *b = reinterpret_cast<const unsigned char *>(p);
    for (size_t i = 0; i < count * sizeof(T); ++i) checksum = checksum * 31u + b[i];
}
int32_t bad(vq_ctx *c, int32_t code, const char *msg) {
    if (c) c->err = msg;
    return code;
}
}  // namespace

extern "C" {

int32_t vq_ctx_create(int32_t, vq_ctx **out) {
    *out = new vq_ctx();
    return VQ_OK;
}
int32_t vq_ctx_destroy(vq_ctx *c) {
    if (c && c->live != 0) std::abort();  // the host mirror leaked or double-freed device memory
    delete c;
    return VQ_OK;
}
const char *vq_last_error(const vq_ctx *c) { return c ? c->err.c_str() : ""; }
int32_t vq_ctx_sync(vq_ctx *) { return VQ_OK; }
int32_t vq_malloc(vq_ctx *c, size_t bytes, void **p) {
    *p = std::malloc(bytes ? bytes : 1);
    if (!*p) return bad(c, VQ_ERR_OOM, "out of memory");
    std::memset(*p, 0xA5, bytes);
    ++c->live;
    return VQ_OK;
}
int32_t vq_free(vq_ctx *c, void *p) {
    if (p) {
        std::free(p);
        --c->live;
    }
    return VQ_OK;
}
int32_t vq_h2d(vq_ctx *, void *d, const void *h, size_t bytes) {
    std::memcpy(d, h, bytes);
    return VQ_OK;
}
int32_t vq_d2h(vq_ctx *, void *h, const void *d, size_t bytes) {
    std::memcpy(h, d, bytes);
    return VQ_OK;
}
int32_t vq_copy_f32(vq_ctx *, float *d, const float *s, int64_t count) {
    std::memmove(d, s, sizeof(float) * (size_t)count);
    return VQ_OK;
}

int32_t vq_lbg_fit(vq_ctx *c, const float *x, int64_t n, int64_t ld, int32_t m, int32_t sd, int32_t k, int32_t iters,
                   const uint32_t *init, const uint32_t *reseed, int32_t n_reseed, float *cb, int32_t *iters_run,
                   int32_t *used) {
    if (k <= 0 || n < k) return bad(c, VQ_ERR_INVALID_ARG, "Invalid parameter: k");
    touch(reseed, (size_t)m * (size_t)(n_reseed > 0 ? n_reseed : 0));
    for (int s = 0; s < m; ++s)
        for (int j = 0; j < k; ++j) {
            const uint32_t row = init[(size_t)s * k + j];
            if ((int64_t)row >= n) return bad(c, VQ_ERR_INVALID_ARG, "Invalid parameter: initial row out of range");
            for (int t = 0; t < sd; ++t) cb[((size_t)s * k + j) * sd + t] = x[(size_t)row * ld + (size_t)s * sd + t];
        }
    touch(x, (size_t)(n - 1) * ld + (size_t)m * sd);
    for (int s = 0; s < m; ++s) {
        if (iters_run) iters_run[s] = iters;
        if (used) used[s] = 0;
    }
    return VQ_OK;
}

static int32_t assign_any(const float *x, int64_t n, int64_t ld, int32_t m, int32_t sd, int32_t k, const float *cb,
                          void *codes, int width) {
    touch(cb, (size_t)m * k * sd);
    if (n > 0) touch(x, (size_t)(n - 1) * ld + (size_t)m * sd);
    for (int64_t i = 0; i < n * m; ++i) {
        const uint32_t v = (uint32_t)(i % k);
        if (width == 1)
            ((uint8_t *)codes)[i] = (uint8_t)v;
        else
            ((uint16_t *)codes)[i] = (uint16_t)v;
    }
    return VQ_OK;
}
int32_t vq_assign(vq_ctx *, int32_t, const float *x, int64_t n, int64_t ld, int32_t m, int32_t sd, int32_t k,
                  const float *cb, uint8_t *codes) {
    return assign_any(x, n, ld, m, sd, k, cb, codes, 1);
}
int32_t vq_assign_u16(vq_ctx *, int32_t, const float *x, int64_t n, int64_t ld, int32_t m, int32_t sd, int32_t k,
                      const float *cb, uint16_t *codes) {
    return assign_any(x, n, ld, m, sd, k, cb, codes, 2);
}

}  // extern "C"
template <class CodeT, class OutT>
static int32_t decode_any(const CodeT *codes, int64_t n, int32_t m, int32_t sd, int32_t k, const float *cb, OutT *out) {
    for (int64_t i = 0; i < n; ++i)
        for (int s = 0; s < m; ++s) {
            const size_t j = codes[i * m + s];
            if ((int)j >= k) std::abort();
            for (int t = 0; t < sd; ++t) out[((size_t)i * m + s) * sd + t] = (OutT)cb[((size_t)s * k + j) * sd + t];
        }
    return VQ_OK;
}
extern "C" {
int32_t vq_decode_f16(vq_ctx *, const uint8_t *codes, int64_t n, int32_t m, int32_t sd, int32_t k, const float *cb,
                      uint16_t *out) {
    return decode_any(codes, n, m, sd, k, cb, out);
}
int32_t vq_decode_f32(vq_ctx *, const uint8_t *codes, int64_t n, int32_t m, int32_t sd, int32_t k, const float *cb,
                      float *out) {
    return decode_any(codes, n, m, sd, k, cb, out);
}
int32_t vq_decode_f16_u16(vq_ctx *, const uint16_t *codes, int64_t n, int32_t m, int32_t sd, int32_t k, const float *cb,
                          uint16_t *out) {
    return decode_any(codes, n, m, sd, k, cb, out);
}
int32_t vq_decode_f32_u16(vq_ctx *, const uint16_t *codes, int64_t n, int32_t m, int32_t sd, int32_t k, const float *cb,
                          float *out) {
    return decode_any(codes, n, m, sd, k, cb, out);
}

}  // extern "C"
template <class CodeT>
static int32_t residual_any(float *res, int64_t n, int64_t ld, int32_t dim, int32_t k, const float *cb, const CodeT *codes) {
    for (int64_t i = 0; i < n; ++i) {
        if ((int)codes[i] >= k) std::abort();
        for (int t = 0; t < dim; ++t) res[i * ld + t] -= cb[(size_t)codes[i] * dim + t];
    }
    return VQ_OK;
}
extern "C" {
int32_t vq_residual_sub(vq_ctx *, float *res, int64_t n, int64_t ld, int32_t dim, int32_t k, const float *cb,
                        const uint8_t *codes) {
    return residual_any(res, n, ld, dim, k, cb, codes);
}
int32_t vq_residual_sub_u16(vq_ctx *, float *res, int64_t n, int64_t ld, int32_t dim, int32_t k, const float *cb,
                            const uint16_t *codes) {
    return residual_any(res, n, ld, dim, k, cb, codes);
}
int32_t vq_lbg_fit_residual(vq_ctx *c, float *res, int64_t n, int64_t ld, int32_t dim, int32_t k, int32_t iters,
                            const uint32_t *init, const uint32_t *reseed, int32_t n_reseed, float *cb,
                            const float *prev_cb, int32_t k_prev, const uint8_t *prev_codes, int32_t *iters_run,
                            int32_t *used) {
    const int32_t rc = vq_residual_sub(c, res, n, ld, dim, k_prev, prev_cb, prev_codes);
    if (rc != VQ_OK) return rc;
    return vq_lbg_fit(c, res, n, ld, 1, dim, k, iters, init, reseed, n_reseed, cb, iters_run, used);
}
int32_t vq_mean_l2norm(vq_ctx *, const float *x, int64_t n, int64_t ld, int32_t dim, float *out) {
    double s = 0;
    for (int64_t i = 0; i < n; ++i) {
        double q = 0;
        for (int t = 0; t < dim; ++t) q += (double)x[i * ld + t] * x[i * ld + t];
        s += std::sqrt(q);
    }
    *out = (float)(s / (double)n);
    return VQ_OK;
}
}  // extern "C"
template <class CodeT>
static int32_t rvq_any(const float *x, int64_t n, int64_t ld, int32_t dim, int32_t stages, int32_t k, const float *cb,
                       CodeT *codes, uint8_t *used, uint16_t *recon) {
    touch(cb, (size_t)stages * k * dim);
    if (n > 0) touch(x, (size_t)(n - 1) * ld + dim);
    for (int64_t i = 0; i < n * stages; ++i) codes[i] = (CodeT)(i % k);
    if (used)
        for (int64_t i = 0; i < n; ++i) used[i] = (uint8_t)stages;
    if (recon)
        for (int64_t i = 0; i < n * dim; ++i) recon[i] = 0x3c00;
    return VQ_OK;
}
extern "C" {
int32_t vq_rvq_encode(vq_ctx *, int32_t, const float *x, int64_t n, int64_t ld, int32_t dim, int32_t stages, int32_t k,
                      const float *cb, float, uint8_t *codes, uint8_t *used, uint16_t *recon) {
    return rvq_any(x, n, ld, dim, stages, k, cb, codes, used, recon);
}
int32_t vq_rvq_encode_u16(vq_ctx *, int32_t, const float *x, int64_t n, int64_t ld, int32_t dim, int32_t stages,
                          int32_t k, const float *cb, float, uint16_t *codes, uint8_t *used, uint16_t *recon) {
    return rvq_any(x, n, ld, dim, stages, k, cb, codes, used, recon);
}

int32_t vq_rotate(vq_ctx *, const float *x, int64_t n, int64_t ld, int32_t dim, const float *R, float *y) {
    touch(R, (size_t)dim * dim);
    for (int64_t i = 0; i < n; ++i)
        for (int t = 0; t < dim; ++t) y[i * dim + t] = x[i * ld + t];
    return VQ_OK;
}
int32_t vq_cross_cov(vq_ctx *, const float *y, const float *x, int64_t n, int32_t dim, double *A) {
    touch(y, (size_t)n * dim);
    touch(x, (size_t)n * dim);
    for (int a = 0; a < dim; ++a)
        for (int b = 0; b < dim; ++b) A[(size_t)a * dim + b] = a == b ? 1.0 : 0.0;
    return VQ_OK;
}
int32_t vq_procrustes_rotation(vq_ctx *, const double *A, int32_t dim, double *R) {
    touch(A, (size_t)dim * dim);
    for (int a = 0; a < dim; ++a)
        for (int b = 0; b < dim; ++b) R[(size_t)a * dim + b] = a == b ? 1.0 : 0.0;
    return VQ_OK;
}

// a tree of depth min(max_depth, 1): the mean of all rows, and two children equal to the first and last row
int32_t vq_tsvq_build(vq_ctx *, const float *x, int64_t n, int64_t ld, int32_t dim, int32_t max_depth, vq_tree **out) {
    vq_tree *t = new vq_tree();
    const bool split = max_depth > 0 && n > 1;
    t->n_nodes = split ? 3 : 1;
    t->dim = dim;
    t->cen.assign((size_t)t->n_nodes * dim, 0.f);
    for (int64_t i = 0; i < n; ++i)
        for (int d = 0; d < dim; ++d) t->cen[d] += x[i * ld + d] / (float)n;
    t->left.assign(t->n_nodes, -1);
    t->right.assign(t->n_nodes, -1);
    if (split) {
        t->left[0] = 1;
        t->right[0] = 2;
        for (int d = 0; d < dim; ++d) {
            t->cen[dim + d] = x[d];
            t->cen[2 * dim + d] = x[(n - 1) * ld + d];
        }
    }
    *out = t;
    return VQ_OK;
}
int32_t vq_tsvq_build_kmeans(vq_ctx *c, const float *x, int64_t n, int64_t ld, int32_t dim, int32_t max_depth,
                             int32_t lbg_iters, const uint32_t *draws, int32_t per_node, vq_tree **out) {
    if (per_node < 2 + lbg_iters) return bad(c, VQ_ERR_INVALID_ARG, "Invalid parameter: draws");
    if (max_depth > 0) touch(draws, (((size_t)1 << max_depth) - 1) * (size_t)per_node);
    return vq_tsvq_build(c, x, n, ld, dim, max_depth, out);
}
int32_t vq_tree_free(vq_ctx *, vq_tree *t) {
    delete t;
    return VQ_OK;
}
int32_t vq_tree_info(const vq_tree *t, int32_t *nn, int32_t *dim) {
    if (nn) *nn = t->n_nodes;
    if (dim) *dim = t->dim;
    return VQ_OK;
}
int32_t vq_tree_download(const vq_tree *t, float *cen, int32_t *left, int32_t *right, int32_t *sdim, float *sval,
                         int64_t *cnt) {
    const size_t nn = (size_t)t->n_nodes;
    if (cen) std::memcpy(cen, t->cen.data(), sizeof(float) * nn * t->dim);
    if (left) std::memcpy(left, t->left.data(), sizeof(int32_t) * nn);
    if (right) std::memcpy(right, t->right.data(), sizeof(int32_t) * nn);
    for (size_t i = 0; i < nn; ++i) {
        if (sdim) sdim[i] = -1;
        if (sval) sval[i] = 0.f;
        if (cnt) cnt[i] = 0;
    }
    return VQ_OK;
}
int32_t vq_tsvq_descend(vq_ctx *, int32_t, const float *x, int64_t n, int64_t ld, const vq_tree *t, int32_t *leaf) {
    if (n > 0) touch(x, (size_t)(n - 1) * ld + t->dim);
    for (int64_t i = 0; i < n; ++i) leaf[i] = t->n_nodes == 1 ? 0 : 1 + (int32_t)(i & 1);
    return VQ_OK;
}
int32_t vq_tsvq_decode_f16(vq_ctx *, const vq_tree *t, const int32_t *leaf, int64_t n, uint16_t *out) {
    for (int64_t i = 0; i < n; ++i) {
        if (leaf[i] < 0 || leaf[i] >= t->n_nodes) std::abort();
        for (int d = 0; d < t->dim; ++d) out[i * t->dim + d] = (uint16_t)(leaf[i] + d);
    }
    return VQ_OK;
}

}  // extern "C"
