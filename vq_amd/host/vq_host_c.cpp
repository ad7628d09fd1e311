// Flat C entry points over the C++ host classes of vq.hpp, so that the Python tests can drive
// the same objects a C++ (or Rust) application would.  Exceptions become status codes; the
// message of the last one is kept per thread.
#include <cstdint>
#include <cstring>
#include <memory>
#include <string>

#include "vq.hpp"

namespace {
thread_local std::string g_err;

struct Obj {
    int kind = 0;  // 1 pq, 2 opq, 3 rvq, 4 tsvq
    std::unique_ptr<vq::ProductQuantizer> pq;
    std::unique_ptr<vq::OptimizedProductQuantizer> opq;
    std::unique_ptr<vq::ResidualQuantizer> rvq;
    std::unique_ptr<vq::TSVQ> tsvq;
    int64_t dim = 0;
};

// The caller's rows are one contiguous array already: a view, no per-row vectors.  (The conversion
// from the reference's `&[Vector<f32>]` shape is exercised by vqh_quantize, which goes through
// `quantize(&Vector<f32>)`.)
vq::Rows rows_of(const float *x, int64_t n, int64_t dim) { return vq::Rows::view(x, (size_t)n, (size_t)dim); }

vq::IndexStreams streams_of(const uint32_t *init, size_t n_init, const uint32_t *reseed, size_t problems,
                            int32_t n_reseed) {
    vq::IndexStreams s;
    s.init.assign(init, init + n_init);
    s.n_reseed = n_reseed;
    if (n_reseed > 0) s.reseed.assign(reseed, reseed + problems * (size_t)n_reseed);
    return s;
}

template <class F>
int guarded(F &&f) {
    try {
        f();
        return 0;
    } catch (const vq::VqError &e) {
        g_err = e.what();
        return e.code ? e.code : -1;
    } catch (const std::exception &e) {
        g_err = e.what();
        return -100;
    }
}

void flatten(const std::vector<uint16_t> &q, uint16_t *out) {
    if (!q.empty()) std::memcpy(out, q.data(), q.size() * sizeof(uint16_t));
}
}  // namespace

extern "C" {

const char *vqh_last_error() { return g_err.c_str(); }

int vqh_lbg_quantize(const float *x, int64_t n, int64_t dim, int64_t k, int64_t max_iters, uint64_t seed,
                     const uint32_t *init, const uint32_t *reseed, int32_t n_reseed, float *out) {
    return guarded([&] {
        auto rows = rows_of(x, n, dim);
        vq::IndexStreams st;
        if (init) st = streams_of(init, (size_t)k, reseed, 1, n_reseed);
        auto c = vq::lbg_quantize(rows, (size_t)k, (size_t)max_iters, seed, init ? &st : nullptr);
        for (size_t j = 0; j < c.size(); ++j) std::memcpy(out + j * dim, c[j].data.data(), sizeof(float) * dim);
    });
}

int vqh_pq_fit(const float *x, int64_t n, int64_t dim, int64_t m, int64_t k, int64_t max_iters, int distance,
               double p, uint64_t seed, const uint32_t *init, const uint32_t *reseed, int32_t n_reseed,
               void **out) {
    return guarded([&] {
        auto rows = rows_of(x, n, dim);
        vq::IndexStreams st;
        if (init) st = streams_of(init, (size_t)(m * k), reseed, (size_t)m, n_reseed);
        auto o = std::make_unique<Obj>();
        o->kind = 1;
        o->dim = dim;
        o->pq = std::make_unique<vq::ProductQuantizer>(vq::ProductQuantizer::fit(
            rows, (size_t)m, (size_t)k, (size_t)max_iters, vq::Distance((vq::Distance::Kind)distance, p), seed,
            init ? &st : nullptr));
        *out = o.release();
    });
}

int vqh_opq_fit(const float *x, int64_t n, int64_t dim, int64_t m, int64_t k, int64_t max_iters,
                int64_t opq_iters, int distance, double p, uint64_t seed, const uint32_t *init,
                const uint32_t *reseed, int32_t n_reseed, void **out) {
    return guarded([&] {
        auto rows = rows_of(x, n, dim);
        vq::IndexStreams st;
        if (init) st = streams_of(init, (size_t)(m * k), reseed, (size_t)m, n_reseed);
        auto o = std::make_unique<Obj>();
        o->kind = 2;
        o->dim = dim;
        o->opq = std::make_unique<vq::OptimizedProductQuantizer>(vq::OptimizedProductQuantizer::fit(
            rows, (size_t)m, (size_t)k, (size_t)max_iters, (size_t)opq_iters,
            vq::Distance((vq::Distance::Kind)distance, p), seed, init ? &st : nullptr));
        *out = o.release();
    });
}

int vqh_rvq_fit(const float *x, int64_t n, int64_t dim, int64_t stages, int64_t k, int64_t max_iters,
                float epsilon, int distance, double p, uint64_t seed, const uint32_t *init,
                const uint32_t *reseed, int32_t n_reseed, void **out) {
    return guarded([&] {
        auto rows = rows_of(x, n, dim);
        vq::IndexStreams st;
        if (init) st = streams_of(init, (size_t)(stages * k), reseed, (size_t)stages, n_reseed);
        auto o = std::make_unique<Obj>();
        o->kind = 3;
        o->dim = dim;
        o->rvq = std::make_unique<vq::ResidualQuantizer>(vq::ResidualQuantizer::fit(
            rows, (size_t)stages, (size_t)k, (size_t)max_iters, epsilon,
            vq::Distance((vq::Distance::Kind)distance, p), seed, init ? &st : nullptr));
        *out = o.release();
    });
}

int vqh_tsvq_new(const float *x, int64_t n, int64_t dim, int64_t max_depth, int distance, double p, void **out) {
    return guarded([&] {
        auto rows = rows_of(x, n, dim);
        auto o = std::make_unique<Obj>();
        o->kind = 4;
        o->dim = dim;
        o->tsvq = std::make_unique<vq::TSVQ>(
            vq::TSVQ::create(rows, (size_t)max_depth, vq::Distance((vq::Distance::Kind)distance, p)));
        *out = o.release();
    });
}

// the tree with 2-means splits (not in the crate); draws: nullable, (2^max_depth - 1) * (2 + lbg_iters) values
int vqh_tsvq_new_kmeans(const float *x, int64_t n, int64_t dim, int64_t max_depth, int64_t lbg_iters, int distance,
                        double p, uint64_t seed, const uint32_t *draws, void **out) {
    return guarded([&] {
        auto rows = rows_of(x, n, dim);
        std::vector<uint32_t> d;
        if (draws && max_depth <= 20)
            d.assign(draws, draws + (((size_t)1 << max_depth) - 1) * (size_t)(2 + lbg_iters));
        auto o = std::make_unique<Obj>();
        o->kind = 4;
        o->dim = dim;
        o->tsvq = std::make_unique<vq::TSVQ>(vq::TSVQ::create_kmeans(
            rows, (size_t)max_depth, (size_t)lbg_iters, vq::Distance((vq::Distance::Kind)distance, p), seed,
            draws ? &d : nullptr));
        *out = o.release();
    });
}

// quantize(&Vector<f32>) of whichever quantizer obj holds; len is the vector's own length
// *out_len (nullable) receives the length of the returned vector
int vqh_quantize(void *obj, const float *v, int64_t len, uint16_t *out, int64_t *out_len) {
    return guarded([&] {
        Obj *o = (Obj *)obj;
        vq::Vector<float> vec(std::vector<float>(v, v + len));
        vq::Vector<vq::f16> q;
        switch (o->kind) {
        case 1: q = o->pq->quantize(vec); break;
        case 2: q = o->opq->quantize(vec); break;
        case 3: q = o->rvq->quantize(vec); break;
        default: q = o->tsvq->quantize(vec); break;
        }
        for (size_t t = 0; t < q.len(); ++t) out[t] = q.data[t].bits;
        if (out_len) *out_len = (int64_t)q.len();
    });
}

int vqh_quantize_batch(void *obj, const float *x, int64_t n, int64_t dim, uint16_t *out) {
    return guarded([&] {
        Obj *o = (Obj *)obj;
        auto rows = rows_of(x, n, dim);
        switch (o->kind) {
        case 1: flatten(o->pq->quantize_batch_flat(rows), out); break;
        case 2: flatten(o->opq->quantize_batch_flat(rows), out); break;
        case 3: flatten(o->rvq->quantize_batch_flat(rows), out); break;
        default: flatten(o->tsvq->quantize_batch_flat(rows), out); break;
        }
    });
}

// The same through the reference's own shape, one heap-allocated Vector<f32> per row
// (`&[Vector<f32>]` -> Vec<Vector<f16>>); row `short_row` (if >= 0) is cut to `short_len` floats.
int vqh_quantize_batch_vectors(void *obj, const float *x, int64_t n, int64_t dim, int64_t short_row,
                               int64_t short_len, uint16_t *out) {
    return guarded([&] {
        Obj *o = (Obj *)obj;
        std::vector<vq::Vector<float>> rows((size_t)n);
        for (int64_t i = 0; i < n; ++i)
            rows[(size_t)i].data.assign(x + i * dim, x + i * dim + (i == short_row ? short_len : dim));
        std::vector<vq::Vector<vq::f16>> q;
        switch (o->kind) {
        case 1: q = o->pq->quantize_batch(rows); break;
        case 2: q = o->opq->quantize_batch(rows); break;
        case 3: q = o->rvq->quantize_batch(rows); break;
        default: q = o->tsvq->quantize_batch(rows); break;
        }
        size_t at = 0;
        for (const auto &v : q)
            for (const auto &h : v.data) out[at++] = h.bits;
    });
}

// codes: PQ / OPQ n*m bytes, RVQ n*stages bytes
int vqh_encode(void *obj, const float *x, int64_t n, int64_t dim, uint8_t *codes) {
    return guarded([&] {
        Obj *o = (Obj *)obj;
        auto rows = rows_of(x, n, dim);
        std::vector<uint8_t> c;
        switch (o->kind) {
        case 1: c = o->pq->encode(rows); break;
        case 2: c = o->opq->encode(rows); break;
        case 3: o->rvq->quantize_batch_flat(rows, &c); break;
        default: throw vq::VqError::InvalidParameter("TSVQ has leaves, not codes");
        }
        std::memcpy(codes, c.data(), c.size());
    });
}

// the same 16 bits wide: any k up to 65536
int vqh_encode16(void *obj, const float *x, int64_t n, int64_t dim, uint16_t *codes) {
    return guarded([&] {
        Obj *o = (Obj *)obj;
        auto rows = rows_of(x, n, dim);
        std::vector<uint16_t> c;
        switch (o->kind) {
        case 1: c = o->pq->encode16(rows); break;
        case 2: c = o->opq->encode16(rows); break;
        case 3: o->rvq->quantize_batch_flat(rows, nullptr, &c); break;
        default: throw vq::VqError::InvalidParameter("TSVQ has leaves, not codes");
        }
        std::memcpy(codes, c.data(), c.size() * sizeof(uint16_t));
    });
}

int vqh_leaves(void *obj, const float *x, int64_t n, int64_t dim, int32_t *leaves) {
    return guarded([&] {
        Obj *o = (Obj *)obj;
        if (o->kind != 4) throw vq::VqError::InvalidParameter("not a TSVQ");
        std::vector<int32_t> l;
        o->tsvq->quantize_batch_flat(rows_of(x, n, dim), &l);
        std::memcpy(leaves, l.data(), l.size() * sizeof(int32_t));
    });
}

// info[0..6] = kind, m, k, sub_dim, dim, stages, n_nodes
int vqh_info(void *obj, int64_t *info) {
    return guarded([&] {
        Obj *o = (Obj *)obj;
        for (int i = 0; i < 7; ++i) info[i] = 0;
        info[0] = o->kind;
        info[4] = o->dim;
        if (o->kind == 1) {
            info[1] = (int64_t)o->pq->m();
            info[2] = (int64_t)o->pq->k();
            info[3] = (int64_t)o->pq->sub_dim();
        } else if (o->kind == 2) {
            info[1] = (int64_t)o->opq->m();
            info[2] = o->opq->trained() ? (int64_t)o->opq->k() : 0;  // no codebooks after opq_iters == 0
            info[3] = (int64_t)o->opq->sub_dim();
        } else if (o->kind == 3) {
            info[5] = (int64_t)o->rvq->stages();
        } else if (o->kind == 4) {
            info[6] = o->tsvq->n_nodes();
        }
    });
}

int vqh_codebooks(void *obj, float *out) {
    return guarded([&] {
        Obj *o = (Obj *)obj;
        std::vector<float> c;
        switch (o->kind) {
        case 1: c = o->pq->codebooks(); break;
        case 2: c = o->opq->codebooks(); break;
        case 3: c = o->rvq->codebooks(); break;
        default: throw vq::VqError::InvalidParameter("TSVQ has a tree, not codebooks");
        }
        std::memcpy(out, c.data(), c.size() * sizeof(float));
    });
}

int vqh_rotation(void *obj, float *out) {
    return guarded([&] {
        Obj *o = (Obj *)obj;
        if (o->kind != 2) throw vq::VqError::InvalidParameter("not an OPQ");
        std::memcpy(out, o->opq->rotation().data(), o->opq->rotation().size() * sizeof(float));
    });
}

// TSVQ node table, breadth-first numbering
int vqh_tree(void *obj, float *centroids, int32_t *left, int32_t *right) {
    return guarded([&] {
        Obj *o = (Obj *)obj;
        if (o->kind != 4) throw vq::VqError::InvalidParameter("not a TSVQ");
        vq_tree_download(o->tsvq->tree(), centroids, left, right, nullptr, nullptr, nullptr);
    });
}

void vqh_free(void *obj) { delete (Obj *)obj; }

}  // extern "C"
