/*
 * vq_oracle.c — CPU restatement of the codebook hot path of the `vq` crate.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the GPU library is
 * compared against; nothing in the shipped library links, loads or calls it.
 *
 * Every function follows the floating-point OPERATION ORDER of the reference
 * (Rust, f32, no FMA contraction, no reassociation).  Build with
 *     gcc -O2 -ffp-contract=off -fno-fast-math -fPIC -shared
 * so that `acc + a*b` stays two roundings, as in Rust.
 *
 * Reference citations are relative to the reference crate root.
 *
 * Randomness: the reference draws initial centroids with
 * `choose_multiple(&mut StdRng, k)` and empty-cluster re-seeds with
 * `choose(&mut rng)` (src/utils.rs:52-54,100).  The `rand` crate is not part of
 * the reference tree, so the index streams enter here as explicit arrays:
 *   init_idx[k]       rows copied as the initial centroids
 *   reseed_stream[R]  the successive `choose` draws; the i-th empty cluster met
 *                     (iteration-major, cluster index ascending) takes entry i.
 * PARITY UNPINNED: the mapping seed -> index stream (rand 0.9 StdRng).
 *
 * Summation order of `mean_vector` (src/vector.rs:282-318):
 *   <= 1024 members: sequential from 0.0 in row order — the reference's exact,
 *                    deterministic order;
 *   >  1024 members: the reference uses a Rayon reduce whose tree depends on
 *                    work stealing (not reproducible even by the reference).
 *                    The oracle fixes ONE order per call site:
 *      - inside lbg_quantize (vqo_mean_rows_parts): the rows are cut into parts
 *        of 4096 consecutive row indices; the cluster's members inside a part are
 *        added in row order from 0.0, and the per-part sums are added in part
 *        order from 0.0.  (Chosen because it is a single streaming pass on the
 *        GPU; it is a fixed order, not a tree Rayon would build.)
 *      - for a TSVQ node (vqo_mean_rows): the member list is split at its
 *        midpoint, recursively, to the uniform depth
 *        d = min{d : count <= 1024 * 2^d}; leaves are summed sequentially from
 *        0.0, siblings are added left + right (a tree Rayon can produce).
 * PARITY UNPINNED (by construction of the reference): the order above 1024.
 *
 * Other places where the reference's own order is not fixed and the oracle
 * picks the sequential order: Rayon `sum` of residual norms (src/rvq.rs:131-138),
 * nalgebra gemm/gemv/SVD rounding (src/opq.rs:179-190).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define VQO_PARALLEL_THRESHOLD 1024 /* src/vector.rs:16 */

enum { VQO_SQEUCLIDEAN = 0, VQO_EUCLIDEAN = 1, VQO_COSINE = 2, VQO_MANHATTAN = 3 };

/* ---------------------------------------------------------------- L1 prims */

/* Vector::dot, sequential branch (src/vector.rs:197-201): fold(0, acc + a*b). */
float vqo_dot(const float *a, const float *b, int64_t n) {
    float acc = 0.0f;
    for (int64_t t = 0; t < n; ++t) {
        float p = a[t] * b[t];
        acc = acc + p;
    }
    return acc;
}

/* Vector::distance2 (src/vector.rs:214-220): diff = a - b (247-266), then
 * diff.dot(diff). */
float vqo_distance2(const float *a, const float *b, int64_t n) {
    float acc = 0.0f;
    for (int64_t t = 0; t < n; ++t) {
        float d = a[t] - b[t];
        float p = d * d;
        acc = acc + p;
    }
    return acc;
}

/* Distance::compute (src/distances.rs:115-172), sequential branch of
 * zip_map_sum / map_sum (26-31, 66-69). Returns NaN for an unknown metric. */
float vqo_distance(int metric, const float *a, const float *b, int64_t n) {
    switch (metric) {
    case VQO_SQEUCLIDEAN: { /* 130-133 */
        float acc = 0.0f;
        for (int64_t t = 0; t < n; ++t) {
            float d = a[t] - b[t];
            float p = d * d;
            acc = acc + p;
        }
        return acc;
    }
    case VQO_EUCLIDEAN: { /* 134-140 */
        float acc = 0.0f;
        for (int64_t t = 0; t < n; ++t) {
            float d = a[t] - b[t];
            float p = d * d;
            acc = acc + p;
        }
        return sqrtf(acc);
    }
    case VQO_COSINE: { /* 141-151 */
        float dot = 0.0f, sa = 0.0f, sb = 0.0f;
        for (int64_t t = 0; t < n; ++t) {
            float p = a[t] * b[t];
            dot = dot + p;
        }
        for (int64_t t = 0; t < n; ++t) {
            float p = a[t] * a[t];
            sa = sa + p;
        }
        for (int64_t t = 0; t < n; ++t) {
            float p = b[t] * b[t];
            sb = sb + p;
        }
        float na = sqrtf(sa), nb = sqrtf(sb);
        if (na == 0.0f || nb == 0.0f) return 1.0f;
        float den = na * nb;
        float q = dot / den;
        return 1.0f - q;
    }
    case VQO_MANHATTAN: { /* 152 */
        float acc = 0.0f;
        for (int64_t t = 0; t < n; ++t) {
            float d = a[t] - b[t];
            acc = acc + fabsf(d);
        }
        return acc;
    }
    default:
        return NAN;
    }
}

/* half::f16::from_f32: IEEE binary32 -> binary16, round to nearest even,
 * overflow to +-inf, subnormals kept, NaN stays NaN (quiet bit forced).
 * Call sites src/pq.rs:179, src/opq.rs:260, src/rvq.rs:212, src/tsvq.rs:246. */
uint16_t vqo_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 0xffu) { /* inf / nan */
        if (man == 0) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | 0x7c00u | 0x0200u | (man >> 13));
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u); /* overflow */
    if (e <= 0) {                                     /* subnormal or zero */
        if (e < -10) return (uint16_t)sign;           /* below half of min subnormal */
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);          /* 14..24 */
        uint32_t h = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1u))) h += 1;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h += 1; /* may carry into exp / inf */
    return (uint16_t)(sign | h);
}

float vqo_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t x;
    if (exp == 0) {
        if (man == 0) {
            x = sign;
        } else {
            int e = -1;
            do {
                man <<= 1;
                ++e;
            } while (!(man & 0x400u));
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 0x1f) {
        x = sign | 0x7f800000u | (man << 13);
    } else {
        x = sign | ((exp - 15 + 127) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* Sequential leaf of mean_vector (src/vector.rs:306-313): sum starts at 0.0 and
 * adds members in list order, component-wise. */
static void sum_seq(const float *x, int64_t ld, int64_t off, int64_t d, const uint32_t *rows,
                    int64_t lo, int64_t hi, float *out) {
    for (int64_t t = 0; t < d; ++t) out[t] = 0.0f;
    for (int64_t p = lo; p < hi; ++p) {
        const float *v = x + (int64_t)rows[p] * ld + off;
        for (int64_t t = 0; t < d; ++t) out[t] = out[t] + v[t];
    }
}

static void sum_tree(const float *x, int64_t ld, int64_t off, int64_t d, const uint32_t *rows,
                     int64_t lo, int64_t hi, int depth, float *out, float *tmp) {
    if (depth == 0) {
        sum_seq(x, ld, off, d, rows, lo, hi, out);
        return;
    }
    int64_t mid = lo + (hi - lo) / 2;
    float *right = tmp; /* tmp holds depth*d floats */
    sum_tree(x, ld, off, d, rows, lo, mid, depth - 1, out, tmp + d);
    sum_tree(x, ld, off, d, rows, mid, hi, depth - 1, right, tmp + d);
    for (int64_t t = 0; t < d; ++t) out[t] = out[t] + right[t];
}

/* Depth of the canonical midpoint tree for `count` members (see file header). */
int vqo_tree_depth(int64_t count) {
    int depth = 0;
    while (count > ((int64_t)VQO_PARALLEL_THRESHOLD << depth)) ++depth;
    return depth;
}

/* mean_vector (src/vector.rs:282-318) over the rows x[rows[p]*ld + off .. +d),
 * p in [0,count), count >= 1.  Divides by (count as f64) as f32 (315-316). */
void vqo_mean_rows(const float *x, int64_t ld, int64_t off, int64_t d, const uint32_t *rows,
                   int64_t count, float *out) {
    int depth = vqo_tree_depth(count);
    float *tmp = (float *)malloc(sizeof(float) * (size_t)d * (size_t)(depth + 1));
    sum_tree(x, ld, off, d, rows, 0, count, depth, out, tmp);
    free(tmp);
    float n = (float)(double)count;
    for (int64_t t = 0; t < d; ++t) out[t] = out[t] / n;
}

#define VQO_PART_ROWS 4096

/* mean_vector as used inside lbg_quantize: rows[] ascending row indices of the
 * cluster's members.  See the file header for the order above 1024 members. */
void vqo_mean_rows_parts(const float *x, int64_t ld, int64_t off, int64_t d, const uint32_t *rows,
                         int64_t count, int64_t n_rows, float *out) {
    if (count <= VQO_PARALLEL_THRESHOLD) {
        sum_seq(x, ld, off, d, rows, 0, count, out);
    } else {
        float *part = (float *)malloc(sizeof(float) * (size_t)d);
        for (int64_t t = 0; t < d; ++t) out[t] = 0.0f;
        int64_t p = 0;
        int64_t nparts = (n_rows + VQO_PART_ROWS - 1) / VQO_PART_ROWS;
        for (int64_t q = 0; q < nparts; ++q) {
            int64_t lo = p;
            while (p < count && (int64_t)rows[p] < (q + 1) * VQO_PART_ROWS) ++p;
            sum_seq(x, ld, off, d, rows, lo, p, part); /* 0.0 for a part without members */
            for (int64_t t = 0; t < d; ++t) out[t] = out[t] + part[t];
        }
        free(part);
    }
    float n = (float)(double)count;
    for (int64_t t = 0; t < d; ++t) out[t] = out[t] / n;
}

/* ------------------------------------------------------------ L2: the LBG  */

/* Nearest centroid under squared L2 with strict '<' (src/utils.rs:62-71). */
static uint32_t argmin_d2(const float *v, const float *c, int64_t k, int64_t d) {
    uint32_t best = 0;
    float best_dist = vqo_distance2(v, c, d);
    for (int64_t j = 1; j < k; ++j) {
        float dist = vqo_distance2(v, c + j * d, d);
        if (dist < best_dist) {
            best = (uint32_t)j;
            best_dist = dist;
        }
    }
    return best;
}

/* Nearest centroid under `metric` with strict '<' — the inline loops at
 * src/pq.rs:166-174, src/opq.rs:155-163,250-258, src/rvq.rs:116-124,189-197. */
static uint32_t argmin_metric(int metric, const float *v, const float *c, int64_t k, int64_t d) {
    uint32_t best = 0;
    float best_dist = vqo_distance(metric, v, c, d);
    for (int64_t j = 1; j < k; ++j) {
        float dist = vqo_distance(metric, v, c + j * d, d);
        if (dist < best_dist) {
            best_dist = dist;
            best = (uint32_t)j;
        }
    }
    return best;
}

/* lbg_quantize (src/utils.rs:32-109) on the column block [off, off+d) of the
 * row-major n x ld matrix x.
 *   centroids  out, k*d
 *   assign     optional out (n), the assignments of the last iteration run
 *   iters_run  optional out, number of loop bodies executed
 *   reseeds_used optional out
 * Returns 0, or -1 (k == 0), -2 (n < k), -3 (reseed stream exhausted). */
int vqo_lbg(const float *x, int64_t n, int64_t ld, int64_t off, int64_t d, int64_t k,
            int64_t max_iters, const uint32_t *init_idx, const uint32_t *reseed_stream,
            int64_t n_reseed, float *centroids, uint32_t *assign_out, int32_t *iters_run,
            int32_t *reseeds_used) {
    if (k == 0) return -1; /* utils.rs:39-44 */
    if (n < k) return -2;  /* utils.rs:45-50 */
    for (int64_t j = 0; j < k; ++j) /* utils.rs:54 */
        memcpy(centroids + j * d, x + (int64_t)init_idx[j] * ld + off, sizeof(float) * (size_t)d);
    uint32_t *assign = (uint32_t *)calloc((size_t)n, sizeof(uint32_t)); /* utils.rs:55 */
    uint32_t *next = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)n);
    uint32_t *members = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)n);
    int64_t *start = (int64_t *)malloc(sizeof(int64_t) * (size_t)(k + 1));
    int64_t *fill = (int64_t *)malloc(sizeof(int64_t) * (size_t)k);
    int64_t used = 0;
    int32_t it = 0;
    int rc = 0;
    for (; it < max_iters;) {
        /* assignment, utils.rs:59-73 */
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < n; ++i) next[i] = argmin_d2(x + i * ld + off, centroids, k, d);
        /* changed, utils.rs:76-80 */
        int changed = 0;
        for (int64_t i = 0; i < n; ++i)
            if (next[i] != assign[i]) {
                changed = 1;
                break;
            }
        memcpy(assign, next, sizeof(uint32_t) * (size_t)n);
        /* gather members in row order, utils.rs:83-92 (stable counting sort) */
        for (int64_t j = 0; j <= k; ++j) start[j] = 0;
        for (int64_t i = 0; i < n; ++i) start[assign[i] + 1]++;
        for (int64_t j = 0; j < k; ++j) start[j + 1] += start[j];
        for (int64_t j = 0; j < k; ++j) fill[j] = start[j];
        for (int64_t i = 0; i < n; ++i) members[fill[assign[i]]++] = (uint32_t)i;
        /* update / re-seed, utils.rs:95-102 */
        for (int64_t j = 0; j < k; ++j) {
            int64_t cnt = start[j + 1] - start[j];
            if (cnt > 0) {
                vqo_mean_rows_parts(x, ld, off, d, members + start[j], cnt, n, centroids + j * d);
            } else {
                if (used >= n_reseed) {
                    rc = -3;
                    goto done;
                }
                uint32_t r = reseed_stream[used++];
                memcpy(centroids + j * d, x + (int64_t)r * ld + off, sizeof(float) * (size_t)d);
            }
        }
        ++it;
        if (!changed) break; /* utils.rs:104-106 */
    }
done:
    if (assign_out) memcpy(assign_out, assign, sizeof(uint32_t) * (size_t)n);
    if (iters_run) *iters_run = it;
    if (reseeds_used) *reseeds_used = (int32_t)used;
    free(assign);
    free(next);
    free(members);
    free(start);
    free(fill);
    return rc;
}

/* --------------------------------------------------------- L3: PQ (pq.rs)  */

/* ProductQuantizer::fit (src/pq.rs:79-129): m independent LBG problems on the
 * contiguous column blocks of width dim/m; subspace i uses its own index
 * streams (the reference seeds subspace i with seed + i, pq.rs:119).
 *   init_idx       m*k
 *   reseed_stream  m*n_reseed
 *   codebooks      out, m*k*sub_dim
 * Returns 0 or -10 (n == 0), -11 (dim < m), -12 (dim % m != 0), or vqo_lbg's code. */
int vqo_pq_fit(const float *x, int64_t n, int64_t dim, int64_t m, int64_t k, int64_t max_iters,
               const uint32_t *init_idx, const uint32_t *reseed_stream, int64_t n_reseed,
               float *codebooks, int32_t *iters_run, int32_t *reseeds_used) {
    if (n == 0) return -10;      /* pq.rs:87-89 */
    if (dim < m) return -11;     /* pq.rs:91-96 */
    if (dim % m != 0) return -12; /* pq.rs:97-102 */
    int64_t sd = dim / m;
    for (int64_t i = 0; i < m; ++i) {
        int rc = vqo_lbg(x, n, dim, i * sd, sd, k, max_iters, init_idx + i * k,
                         reseed_stream + i * n_reseed, n_reseed, codebooks + i * k * sd, NULL,
                         iters_run ? iters_run + i : NULL, reseeds_used ? reseeds_used + i : NULL);
        if (rc) return rc;
    }
    return 0;
}

/* The argmin of ProductQuantizer::quantize (src/pq.rs:159-174) for every row:
 * codes[i*m + s] = first index of the minimum of metric(x_i[s-block], c_{s,j}). */
void vqo_pq_encode(int metric, const float *x, int64_t n, int64_t ld, int64_t m, int64_t sd,
                   int64_t k, const float *codebooks, uint32_t *codes) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i)
        for (int64_t s = 0; s < m; ++s)
            codes[i * m + s] =
                argmin_metric(metric, x + i * ld + s * sd, codebooks + s * k * sd, k, sd);
}

/* The output of ProductQuantizer::quantize (src/pq.rs:176-186): chosen
 * centroids converted to f16, concatenated. out is n x (m*sd) f16 bit patterns. */
void vqo_pq_decode_f16(const uint32_t *codes, int64_t n, int64_t m, int64_t sd, int64_t k,
                       const float *codebooks, uint16_t *out) {
    for (int64_t i = 0; i < n; ++i)
        for (int64_t s = 0; s < m; ++s) {
            const float *c = codebooks + (s * k + codes[i * m + s]) * sd;
            for (int64_t t = 0; t < sd; ++t) out[i * m * sd + s * sd + t] = vqo_f32_to_f16(c[t]);
        }
}

/* ------------------------------------------------------- L3: RVQ (rvq.rs)  */

/* ResidualQuantizer::fit (src/rvq.rs:87-154).
 *   init_idx       stages*k, reseed_stream stages*n_reseed (stage s seeds with seed+s, rvq.rs:107)
 *   codebooks      out, stages*k*dim
 *   residuals      out (optional, n*dim): the residuals after the last stage run
 *   avg_norms      out (optional, stages)
 * Returns the number of stages actually produced (rvq.rs:145) or a negative code. */
int vqo_rvq_fit(int metric, const float *x, int64_t n, int64_t dim, int64_t stages, int64_t k,
                int64_t max_iters, float epsilon, const uint32_t *init_idx,
                const uint32_t *reseed_stream, int64_t n_reseed, float *codebooks,
                float *residuals_out, float *avg_norms) {
    if (n == 0) return -10; /* rvq.rs:96-98 */
    float *res = (float *)malloc(sizeof(float) * (size_t)(n * dim));
    memcpy(res, x, sizeof(float) * (size_t)(n * dim)); /* rvq.rs:103 */
    int produced = 0;
    for (int64_t st = 0; st < stages; ++st) {
        float *cb = codebooks + st * k * dim;
        int rc = vqo_lbg(res, n, dim, 0, dim, k, max_iters, init_idx + st * k,
                         reseed_stream + st * n_reseed, n_reseed, cb, NULL, NULL, NULL);
        if (rc) {
            free(res);
            return rc;
        }
        ++produced;
        /* residual update, rvq.rs:111-128 */
        for (int64_t i = 0; i < n; ++i) {
            float *r = res + i * dim;
            uint32_t best = (k < 2) ? 0 : argmin_metric(metric, r, cb, k, dim);
            const float *c = cb + (int64_t)best * dim;
            for (int64_t t = 0; t < dim; ++t) r[t] = r[t] - c[t];
        }
        /* average residual norm, rvq.rs:131-138 (sequential order chosen) */
        float total = 0.0f;
        for (int64_t i = 0; i < n; ++i) {
            const float *r = res + i * dim;
            float ns = 0.0f;
            for (int64_t t = 0; t < dim; ++t) {
                float p = r[t] * r[t];
                ns = ns + p;
            }
            total = total + sqrtf(ns);
        }
        float avg = total / (float)n;
        if (avg_norms) avg_norms[st] = avg;
        if (avg < epsilon) break; /* rvq.rs:139-141 */
    }
    if (residuals_out) memcpy(residuals_out, res, sizeof(float) * (size_t)(n * dim));
    free(res);
    return produced;
}

/* ResidualQuantizer::quantize (src/rvq.rs:171-215) for every row.
 *   codes   out n*stages (entries of stages not reached are 0xFFFFFFFF)
 *   recon   out n*dim f16 bit patterns (f16 of the f32 sum of chosen codewords) */
void vqo_rvq_quantize(int metric, const float *x, int64_t n, int64_t dim, int64_t stages,
                      int64_t k, float epsilon, const float *codebooks, uint32_t *codes,
                      uint16_t *recon) {
    float *r = (float *)malloc(sizeof(float) * (size_t)dim);
    float *sum = (float *)malloc(sizeof(float) * (size_t)dim);
    for (int64_t i = 0; i < n; ++i) {
        memcpy(r, x + i * dim, sizeof(float) * (size_t)dim);
        for (int64_t t = 0; t < dim; ++t) sum[t] = 0.0f;
        for (int64_t st = 0; st < stages; ++st)
            if (codes) codes[i * stages + st] = 0xFFFFFFFFu;
        for (int64_t st = 0; st < stages; ++st) {
            const float *cb = codebooks + st * k * dim;
            uint32_t best = (k < 2) ? 0 : argmin_metric(metric, r, cb, k, dim);
            if (codes) codes[i * stages + st] = best;
            const float *c = cb + (int64_t)best * dim;
            for (int64_t t = 0; t < dim; ++t) sum[t] = sum[t] + c[t]; /* rvq.rs:201 */
            for (int64_t t = 0; t < dim; ++t) r[t] = r[t] - c[t];     /* rvq.rs:202 */
            float ns = 0.0f;
            for (int64_t t = 0; t < dim; ++t) {
                float p = r[t] * r[t];
                ns = ns + p;
            }
            if (sqrtf(ns) < epsilon) break; /* rvq.rs:204-207 */
        }
        if (recon)
            for (int64_t t = 0; t < dim; ++t) recon[i * dim + t] = vqo_f32_to_f16(sum[t]);
    }
    free(r);
    free(sum);
}

/* ------------------------------------------------------ L3: TSVQ (tsvq.rs) */

/* Flat node table: node i has centroid[i*dim..], left[i], right[i] (-1 = none).
 * Node 0 is the root; nodes are numbered in pre-order (node, left subtree,
 * right subtree). */
typedef struct {
    const float *x;
    int64_t dim;
    float *centroids;
    int32_t *left, *right;
    int32_t *split_dim; /* optional: -1 for leaves */
    float *split_val;   /* optional: median */
    int64_t *node_count; /* optional */
    int64_t max_nodes, n_nodes;
    int overflow;
} tsvq_build_t;

static int cmp_f32(const void *a, const void *b) {
    float fa = *(const float *)a, fb = *(const float *)b;
    return (fa > fb) - (fa < fb);
}

/* TSVQNode::fit (src/tsvq.rs:71-148). rows: this node's rows, in original order. */
static int32_t tsvq_fit_node(tsvq_build_t *B, const uint32_t *rows, int64_t cnt, int64_t depth) {
    if (B->n_nodes >= B->max_nodes) {
        B->overflow = 1;
        return -1;
    }
    int32_t me = (int32_t)B->n_nodes++;
    int64_t dim = B->dim;
    float *cen = B->centroids + (int64_t)me * dim;
    vqo_mean_rows(B->x, dim, 0, dim, rows, cnt, cen); /* tsvq.rs:76 */
    B->left[me] = -1;
    B->right[me] = -1;
    if (B->split_dim) B->split_dim[me] = -1;
    if (B->split_val) B->split_val[me] = 0.0f;
    if (B->node_count) B->node_count[me] = cnt;
    if (depth == 0 || cnt <= 1) return me; /* tsvq.rs:78-84 */
    /* per-dimension sum of squared deviations, sequential over rows (88-99) */
    int64_t sdim = 0;
    float best = 0.0f;
    for (int64_t t = 0; t < dim; ++t) {
        float acc = 0.0f;
        for (int64_t p = 0; p < cnt; ++p) {
            float diff = B->x[(int64_t)rows[p] * dim + t] - cen[t];
            float sq = diff * diff;
            acc = acc + sq;
        }
        /* Iterator::max_by returns the LAST maximal element (102-106) */
        if (t == 0 || !(acc < best)) {
            best = acc;
            sdim = t;
        }
    }
    /* median of the chosen column by full sort (109-117) */
    float *vals = (float *)malloc(sizeof(float) * (size_t)cnt);
    for (int64_t p = 0; p < cnt; ++p) vals[p] = B->x[(int64_t)rows[p] * dim + sdim];
    qsort(vals, (size_t)cnt, sizeof(float), cmp_f32);
    float median;
    if (cnt % 2 == 0) {
        float s = vals[cnt / 2 - 1] + vals[cnt / 2];
        median = s / 2.0f;
    } else {
        median = vals[cnt / 2];
    }
    free(vals);
    if (B->split_dim) B->split_dim[me] = (int32_t)sdim;
    if (B->split_val) B->split_val[me] = median;
    /* stable partition by `<= median` (120-123) */
    uint32_t *l = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)cnt);
    uint32_t *r = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)cnt);
    int64_t nl = 0, nr = 0;
    for (int64_t p = 0; p < cnt; ++p) {
        if (B->x[(int64_t)rows[p] * dim + sdim] <= median)
            l[nl++] = rows[p];
        else
            r[nr++] = rows[p];
    }
    /* a child exists only if non-empty and strictly smaller (128, 135) */
    if (nl > 0 && nl < cnt) B->left[me] = tsvq_fit_node(B, l, nl, depth - 1);
    if (nr > 0 && nr < cnt) B->right[me] = tsvq_fit_node(B, r, nr, depth - 1);
    free(l);
    free(r);
    return me;
}

/* TSVQ::new (src/tsvq.rs:209-215). Returns the number of nodes, -10 for empty
 * input, -20 if max_nodes is too small. */
int64_t vqo_tsvq_fit(const float *x, int64_t n, int64_t dim, int64_t max_depth, int64_t max_nodes,
                     float *centroids, int32_t *left, int32_t *right, int32_t *split_dim,
                     float *split_val, int64_t *node_count) {
    if (n == 0) return -10;
    tsvq_build_t B = {x, dim, centroids, left, right, split_dim, split_val, node_count,
                      max_nodes, 0, 0};
    uint32_t *rows = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)n);
    for (int64_t i = 0; i < n; ++i) rows[i] = (uint32_t)i;
    tsvq_fit_node(&B, rows, n, max_depth);
    free(rows);
    if (B.overflow) return -20;
    return B.n_nodes;
}

/* ---- TSVQ with 2-means splits (NOT the reference's behaviour) ------------------
 * The reference splits a node at the median of its maximum-variance coordinate
 * (src/tsvq.rs:87-123, vqo_tsvq_fit above).  This variant keeps everything else of
 * TSVQNode::fit (node centroid = mean_vector of its rows, 76; leaf at depth 0 or with
 * <= 1 row, 78; a child only if non-empty and strictly smaller, 128,135) and replaces
 * the split by lbg_quantize (src/utils.rs:32-109, vqo_lbg above) with k = 2 on the
 * node's rows, taken in row order: a row goes left when the first of the two returned
 * centroids is its nearest (squared L2, strict '<': ties to the first).
 * Randomness crosses as draws: node at heap position h (root 1, children 2h, 2h+1)
 * owns draws[(h-1)*per_node ..]; with c rows, the initial rows are the node's rows
 * number i0 = d[0] % c and i1 = d[1] % (c-1), plus one if i1 >= i0 (distinct), and the
 * i-th empty cluster takes row number d[2+i] % c.  Built from parts that are pinned
 * (vqo_lbg, vqo_mean_rows); the composition has no counterpart to compare with. */
typedef struct {
    tsvq_build_t b;
    int64_t lbg_iters;
    const uint32_t *draws;
    int64_t per_node;
    int64_t max_heap;
} tsvq_km_t;

static int32_t tsvq_km_node(tsvq_km_t *K, const uint32_t *rows, int64_t cnt, int64_t depth, int64_t heap) {
    tsvq_build_t *B = &K->b;
    if (B->n_nodes >= B->max_nodes) {
        B->overflow = 1;
        return -1;
    }
    int32_t me = (int32_t)B->n_nodes++;
    int64_t dim = B->dim;
    float *cen = B->centroids + (int64_t)me * dim;
    vqo_mean_rows(B->x, dim, 0, dim, rows, cnt, cen);
    B->left[me] = -1;
    B->right[me] = -1;
    if (B->node_count) B->node_count[me] = cnt;
    if (depth == 0 || cnt <= 1) return me;
    const uint32_t *d = K->draws + (heap - 1) * K->per_node;
    float *xn = (float *)malloc(sizeof(float) * (size_t)cnt * (size_t)dim);
    for (int64_t p = 0; p < cnt; ++p)
        memcpy(xn + p * dim, B->x + (int64_t)rows[p] * dim, sizeof(float) * (size_t)dim);
    uint32_t init[2];
    init[0] = (uint32_t)(d[0] % (uint64_t)cnt);
    init[1] = (uint32_t)(d[1] % (uint64_t)(cnt - 1));
    if (init[1] >= init[0]) init[1] += 1;
    int64_t nres = K->per_node - 2;
    uint32_t *reseed = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)(nres > 0 ? nres : 1));
    for (int64_t i = 0; i < nres; ++i) reseed[i] = (uint32_t)(d[2 + i] % (uint64_t)cnt);
    float *c2 = (float *)malloc(sizeof(float) * 2 * (size_t)dim);
    int rc = vqo_lbg(xn, cnt, dim, 0, dim, 2, K->lbg_iters, init, reseed, nres, c2, NULL, NULL, NULL);
    uint32_t *l = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)cnt);
    uint32_t *r = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)cnt);
    int64_t nl = 0, nr = 0;
    for (int64_t p = 0; p < cnt; ++p) {
        if (argmin_d2(xn + p * dim, c2, 2, dim) == 0)
            l[nl++] = rows[p];
        else
            r[nr++] = rows[p];
    }
    free(xn);
    free(reseed);
    free(c2);
    if (rc != 0) B->overflow = 2; /* re-seed draws exhausted */
    if (nl > 0 && nl < cnt) B->left[me] = tsvq_km_node(K, l, nl, depth - 1, 2 * heap);
    if (nr > 0 && nr < cnt) B->right[me] = tsvq_km_node(K, r, nr, depth - 1, 2 * heap + 1);
    free(l);
    free(r);
    return me;
}

/* Returns the number of nodes, -10 for empty input, -20 if max_nodes is too small,
 * -21 if per_node < 2 + lbg_iters (a node can meet one empty cluster per iteration),
 * -22 if the re-seed draws ran out.  draws: (2^max_depth - 1) * per_node values. */
int64_t vqo_tsvq_fit_kmeans(const float *x, int64_t n, int64_t dim, int64_t max_depth, int64_t lbg_iters,
                            const uint32_t *draws, int64_t per_node, int64_t max_nodes, float *centroids,
                            int32_t *left, int32_t *right, int64_t *node_count) {
    if (n == 0) return -10;
    if (per_node < 2 + lbg_iters) return -21;
    tsvq_km_t K = {{x, dim, centroids, left, right, NULL, NULL, node_count, max_nodes, 0, 0},
                   lbg_iters, draws, per_node, 0};
    uint32_t *rows = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)n);
    for (int64_t i = 0; i < n; ++i) rows[i] = (uint32_t)i;
    tsvq_km_node(&K, rows, n, max_depth, 1);
    free(rows);
    if (K.b.overflow == 1) return -20;
    if (K.b.overflow == 2) return -22;
    return K.b.n_nodes;
}

/* TSVQNode::quantize_with_distance (src/tsvq.rs:162-181) for every row:
 * leaf[i] = node index of the leaf reached. */
void vqo_tsvq_descend(int metric, const float *x, int64_t n, int64_t dim, const float *centroids,
                      const int32_t *left, const int32_t *right, int32_t *leaf) {
    for (int64_t i = 0; i < n; ++i) {
        const float *v = x + i * dim;
        int32_t node = 0;
        for (;;) {
            int32_t l = left[node], r = right[node];
            if (l >= 0 && r >= 0) {
                float dl = vqo_distance(metric, v, centroids + (int64_t)l * dim, dim);
                float dr = vqo_distance(metric, v, centroids + (int64_t)r * dim, dim);
                node = (dl <= dr) ? l : r; /* tsvq.rs:171 */
            } else if (l >= 0) {
                node = l;
            } else if (r >= 0) {
                node = r;
            } else {
                break;
            }
        }
        leaf[i] = node;
    }
}

/* ------------------------------------------------------- L3: OPQ (opq.rs)  */

/* y = R x for every row (src/opq.rs:186-194, 232-234): y_i = sum_j R[i][j] x_j,
 * accumulated in ascending j.  R is row-major dim x dim.  PARITY UNPINNED:
 * nalgebra's gemv accumulation order. */
void vqo_rotate(const float *x, int64_t n, int64_t dim, const float *R, float *y) {
    for (int64_t i = 0; i < n; ++i)
        for (int64_t a = 0; a < dim; ++a) {
            float acc = 0.0f;
            for (int64_t b = 0; b < dim; ++b) {
                float p = R[a * dim + b] * x[i * dim + b];
                acc = acc + p;
            }
            y[i * dim + a] = acc;
        }
}

/* Cyclic one-sided Jacobi SVD in f64 of the row-major dim x dim matrix A,
 * then the orthogonal Procrustes solution R = V U^T (src/opq.rs:180-183).
 * R is the transpose of the polar factor of A and does not depend on the SVD's
 * sign / ordering conventions when A is non-singular. */
void vqo_procrustes(const double *A, int64_t dim, double *R) {
    int64_t n = dim;
    double *U = (double *)malloc(sizeof(double) * (size_t)(n * n)); /* columns become U*S */
    double *V = (double *)malloc(sizeof(double) * (size_t)(n * n));
    memcpy(U, A, sizeof(double) * (size_t)(n * n));
    for (int64_t i = 0; i < n; ++i)
        for (int64_t j = 0; j < n; ++j) V[i * n + j] = (i == j) ? 1.0 : 0.0;
    for (int sweep = 0; sweep < 60; ++sweep) {
        double off = 0.0;
        for (int64_t p = 0; p < n - 1; ++p)
            for (int64_t q = p + 1; q < n; ++q) {
                double alpha = 0, beta = 0, gamma = 0;
                for (int64_t i = 0; i < n; ++i) {
                    double up = U[i * n + p], uq = U[i * n + q];
                    alpha += up * up;
                    beta += uq * uq;
                    gamma += up * uq;
                }
                if (gamma == 0.0) continue;
                double lim = fabs(gamma) / sqrt(alpha * beta + 1e-300);
                if (lim > off) off = lim;
                double zeta = (beta - alpha) / (2.0 * gamma);
                double t = (zeta >= 0 ? 1.0 : -1.0) / (fabs(zeta) + sqrt(1.0 + zeta * zeta));
                double c = 1.0 / sqrt(1.0 + t * t), s = c * t;
                for (int64_t i = 0; i < n; ++i) {
                    double up = U[i * n + p], uq = U[i * n + q];
                    U[i * n + p] = c * up - s * uq;
                    U[i * n + q] = s * up + c * uq;
                    double vp = V[i * n + p], vq = V[i * n + q];
                    V[i * n + p] = c * vp - s * vq;
                    V[i * n + q] = s * vp + c * vq;
                }
            }
        if (off < 1e-15) break;
    }
    /* normalise the columns of U (divide by singular values) */
    double *sv = (double *)malloc(sizeof(double) * (size_t)n);
    double top = 0.0;
    for (int64_t j = 0; j < n; ++j) {
        double s = 0;
        for (int64_t i = 0; i < n; ++i) s += U[i * n + j] * U[i * n + j];
        s = sqrt(s);
        sv[j] = s;
        if (s > top) top = s;
        if (s > 0)
            for (int64_t i = 0; i < n; ++i) U[i * n + j] /= s;
    }
    /* A singular A does not determine the columns of U that belong to its zero singular values
     * (an SVD library returns some orthonormal completion; nalgebra gives U = V = I for A = 0).
     * Complete them, in ascending order: the matching column of V with the fixed columns
     * projected out if more than half of it is left, else the unit vector of which the most is
     * left.  U is then orthogonal and so is R. */
    char *fixed = (char *)malloc((size_t)n);
    double *w = (double *)malloc(sizeof(double) * (size_t)n);
    double *best = (double *)malloc(sizeof(double) * (size_t)n);
    for (int64_t j = 0; j < n; ++j) fixed[j] = top > 0.0 && sv[j] > 1e-12 * top;
    for (int64_t j = 0; j < n; ++j) {
        if (fixed[j]) continue;
        double nrm = -1.0;
        for (int64_t cand = -1; cand < n; ++cand) { /* -1: column j of V; then e_0 ... e_{n-1} */
            for (int64_t i = 0; i < n; ++i) w[i] = cand < 0 ? V[i * n + j] : (i == cand ? 1.0 : 0.0);
            for (int round = 0; round < 2; ++round)
                for (int64_t l = 0; l < n; ++l) {
                    if (!fixed[l]) continue;
                    double d = 0.0;
                    for (int64_t i = 0; i < n; ++i) d += U[i * n + l] * w[i];
                    for (int64_t i = 0; i < n; ++i) w[i] -= d * U[i * n + l];
                }
            double r = 0.0;
            for (int64_t i = 0; i < n; ++i) r += w[i] * w[i];
            r = sqrt(r);
            if (cand < 0) {
                if (r > 0.5) {
                    nrm = r;
                    memcpy(best, w, sizeof(double) * (size_t)n);
                    break;
                }
            } else if (r > nrm) {
                nrm = r;
                memcpy(best, w, sizeof(double) * (size_t)n);
            }
        }
        for (int64_t i = 0; i < n; ++i) U[i * n + j] = best[i] / nrm;
        fixed[j] = 1;
    }
    free(sv);
    free(fixed);
    free(w);
    free(best);
    /* R = V U^T */
    for (int64_t i = 0; i < n; ++i)
        for (int64_t j = 0; j < n; ++j) {
            double acc = 0;
            for (int64_t l = 0; l < n; ++l) acc += V[i * n + l] * U[j * n + l];
            R[i * n + j] = acc;
        }
    free(U);
    free(V);
}

/* OptimizedProductQuantizer::fit (src/opq.rs:90-205).
 *   rotation   out, row-major dim x dim (R_T)
 *   codebooks  out, m*k*sd, trained on data rotated by R_{T-1} (the reference's
 *              order of operations: codebooks 127-142, then rotation 183)
 * The same index streams are used in every outer iteration (the reference
 * re-creates StdRng(seed+i) inside each lbg_quantize call, opq.rs:140).
 * A = Y X^T is accumulated in f64 here (the reference: f32 nalgebra gemm,
 * PARITY UNPINNED); the result is rounded to f32. */
int vqo_opq_fit(int metric, const float *x, int64_t n, int64_t dim, int64_t m, int64_t k,
                int64_t max_iters, int64_t opq_iters, const uint32_t *init_idx,
                const uint32_t *reseed_stream, int64_t n_reseed, float *rotation,
                float *codebooks) {
    if (n == 0) return -10;
    if (dim < m) return -11;
    if (dim % m != 0) return -12;
    int64_t sd = dim / m;
    float *rot = (float *)malloc(sizeof(float) * (size_t)(n * dim));
    float *rec = (float *)malloc(sizeof(float) * (size_t)(n * dim));
    uint32_t *codes = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)(n * m));
    double *A = (double *)malloc(sizeof(double) * (size_t)(dim * dim));
    double *Rd = (double *)malloc(sizeof(double) * (size_t)(dim * dim));
    memcpy(rot, x, sizeof(float) * (size_t)(n * dim)); /* opq.rs:121 */
    for (int64_t a = 0; a < dim; ++a)
        for (int64_t b = 0; b < dim; ++b) rotation[a * dim + b] = (a == b) ? 1.0f : 0.0f;
    int rc = 0;
    for (int64_t it = 0; it < opq_iters; ++it) {
        rc = vqo_pq_fit(rot, n, dim, m, k, max_iters, init_idx, reseed_stream, n_reseed,
                        codebooks, NULL, NULL);
        if (rc) break;
        vqo_pq_encode(metric, rot, n, dim, m, sd, k, codebooks, codes); /* 146-168 */
        for (int64_t i = 0; i < n; ++i)
            for (int64_t s = 0; s < m; ++s)
                memcpy(rec + i * dim + s * sd, codebooks + (s * k + codes[i * m + s]) * sd,
                       sizeof(float) * (size_t)sd);
        /* A = Y X^T with X, Y as dim x n column-major (172-179): A[a][b] = sum_i y_i[a] x_i[b] */
        for (int64_t a = 0; a < dim * dim; ++a) A[a] = 0.0;
        for (int64_t i = 0; i < n; ++i)
            for (int64_t a = 0; a < dim; ++a) {
                double ya = rec[i * dim + a];
                for (int64_t b = 0; b < dim; ++b) A[a * dim + b] += ya * (double)rot[i * dim + b];
            }
        for (int64_t a = 0; a < dim * dim; ++a) A[a] = (double)(float)A[a];
        vqo_procrustes(A, dim, Rd); /* 180-183 */
        for (int64_t a = 0; a < dim * dim; ++a) rotation[a] = (float)Rd[a];
        vqo_rotate(x, n, dim, rotation, rot); /* 186-194 */
    }
    free(rot);
    free(rec);
    free(codes);
    free(A);
    free(Rd);
    return rc;
}

/* OptimizedProductQuantizer::quantize argmin (src/opq.rs:232-258) for every row. */
void vqo_opq_encode(int metric, const float *x, int64_t n, int64_t dim, int64_t m, int64_t k,
                    const float *rotation, const float *codebooks, uint32_t *codes) {
    float *y = (float *)malloc(sizeof(float) * (size_t)(n * dim));
    vqo_rotate(x, n, dim, rotation, y);
    vqo_pq_encode(metric, y, n, dim, m, dim / m, k, codebooks, codes);
    free(y);
}

/* Reconstruction MSE of the eval harness (src/bin/utils.rs:50-67): sum of squared
 * element differences over n*dim; accumulated in f64 here. recon is f16 bits. */
double vqo_mse_f16(const float *x, const uint16_t *recon, int64_t n, int64_t dim) {
    double acc = 0.0;
    for (int64_t i = 0; i < n * dim; ++i) {
        double d = (double)x[i] - (double)vqo_f16_to_f32(recon[i]);
        acc += d * d;
    }
    return acc / (double)(n * dim);
}

/* ------------------------------------------------- timing helper for bench */

#ifdef _OPENMP
#include <omp.h>
#endif
/* Threads used by the row-parallel loops (assignment and encode are independent
 * per row, so the thread count does not change any result). */
int vqo_set_threads(int t) {
#ifdef _OPENMP
    if (t > 0) omp_set_num_threads(t);
    return omp_get_max_threads();
#else
    (void)t;
    return 1;
#endif
}

/* One full PQ fit + encode, single-threaded, used as the CPU baseline. */
int vqo_pq_fit_encode(int metric, const float *x, int64_t n, int64_t dim, int64_t m, int64_t k,
                      int64_t max_iters, const uint32_t *init_idx, const uint32_t *reseed_stream,
                      int64_t n_reseed, float *codebooks, uint32_t *codes) {
    int rc = vqo_pq_fit(x, n, dim, m, k, max_iters, init_idx, reseed_stream, n_reseed, codebooks,
                        NULL, NULL);
    if (rc) return rc;
    vqo_pq_encode(metric, x, n, dim, m, dim / m, k, codebooks, codes);
    return 0;
}
