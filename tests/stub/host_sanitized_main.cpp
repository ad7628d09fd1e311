// The host mirror (vq.hpp and the flat C entry points of vq_host_c.cpp) driven on the CPU against
// the stand-in library of vqhip_stub.cpp, for a build with -fsanitize=address,undefined: packing of
// per-row vectors, validation and its messages, the index streams, the four quantizers' call
// sequences and buffer sizes, the C flattening.  Values are the stand-in's, only shapes, messages
// and memory behaviour are checked.  Prints "host mirror: ok" and returns 0.
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "../../vq_amd/host/vq_host_c.cpp"

static int failures = 0;
#define CHECK(cond)                                                         \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, #cond); \
            ++failures;                                                     \
        }                                                                   \
    } while (0)

template <class F>
static std::string message_of(F &&f) {
    try {
        f();
    } catch (const vq::VqError &e) {
        return e.what();
    }
    return "";
}

static std::vector<vq::Vector<float>> make_rows(size_t n, size_t dim, unsigned seed) {
    std::vector<vq::Vector<float>> rows(n);
    unsigned s = seed * 2654435761u + 1u;
    for (auto &r : rows) {
        r.data.resize(dim);
        for (auto &v : r.data) {
            s = s * 1664525u + 1013904223u;
            v = (float)(s >> 8) / 16777216.0f - 0.5f;
        }
    }
    return rows;
}

int main() {
    using namespace vq;
    const size_t n = 300, dim = 12;
    auto rows = make_rows(n, dim, 1);
    std::vector<float> flat;
    for (auto &r : rows) flat.insert(flat.end(), r.data.begin(), r.data.end());

    // index streams: k distinct initial rows per problem, all below n; re-seed draws below n
    {
        IndexStreams st = IndexStreams::from_seed(42, 3, n, 16, 5);
        CHECK(st.init.size() == 3 * 16);
        for (size_t p = 0; p < 3; ++p)
            for (size_t a = 0; a < 16; ++a) {
                CHECK(st.init[p * 16 + a] < n);
                for (size_t b = 0; b < a; ++b) CHECK(st.init[p * 16 + a] != st.init[p * 16 + b]);
            }
        CHECK(st.reseed.size() == 3 * (size_t)st.n_reseed);
        for (uint32_t v : st.reseed) CHECK(v < n);
        IndexStreams tight = IndexStreams::from_seed(7, 1, 5, 5, 2);  // k = n: every row once
        std::vector<int> seen(5, 0);
        for (uint32_t v : tight.init) ++seen[v];
        for (int c : seen) CHECK(c == 1);
    }
    // lbg_quantize and its panics (src/utils.rs:39-50)
    CHECK(lbg_quantize(rows, 4, 3, 1).size() == 4);
    CHECK(message_of([&] { lbg_quantize(rows, 0, 3, 1); }) == "Invalid parameter: k must be greater than 0");
    CHECK(message_of([&] { lbg_quantize(make_rows(3, 4, 2), 5, 3, 1); }) ==
          "Invalid parameter: Not enough data points for k clusters");
    // ragged rows are reported as the reference's row-by-row check would
    {
        auto ragged = rows;
        ragged[5].data.resize(7);
        CHECK(message_of([&] { ProductQuantizer::fit(ragged, 3, 4, 2, Distance(Distance::Euclidean), 0); }) ==
              "Dimension mismatch: expected 12, got 7");
    }
    // ProductQuantizer: fit, quantize, batch, codes, panics (src/pq.rs:87-102, 147-156)
    {
        auto q = ProductQuantizer::fit(rows, 3, 4, 2, Distance(Distance::Euclidean), 0);
        CHECK(q.quantize(rows[0]).len() == dim);
        CHECK(q.quantize_batch(rows).size() == n);
        CHECK(q.encode(rows).size() == n * 3);
        CHECK(q.codebooks().size() == 3 * 4 * 4);
        CHECK(message_of([&] { q.quantize(Vector<float>(std::vector<float>(5, 0.f))); }) ==
              "Dimension mismatch: expected 12, got 5");
        CHECK(message_of([&] { ProductQuantizer::fit(std::vector<Vector<float>>{}, 3, 4, 2, Distance(Distance::Euclidean), 0); }) ==
              "Empty input: at least one vector is required.");
        CHECK(!message_of([&] { ProductQuantizer::fit(rows, 5, 4, 2, Distance(Distance::Euclidean), 0); }).empty());
        // a metric without a kernel is stored by fit (which never uses it, src/pq.rs:79-129) and refused by quantize
        auto cheb = ProductQuantizer::fit(rows, 3, 4, 2, Distance(Distance::Chebyshev), 0);
        CHECK(!message_of([&] { cheb.quantize(rows[0]); }).empty());
        auto wide = ProductQuantizer::fit(rows, 3, 280, 1, Distance(Distance::SquaredEuclidean), 0);  // 16-bit codes
        CHECK(wide.encode16(rows).size() == n * 3);
        CHECK(wide.quantize_batch(rows).size() == n);
    }
    // OptimizedProductQuantizer, with and without outer iterations (src/opq.rs:119-122)
    {
        auto q = OptimizedProductQuantizer::fit(rows, 3, 4, 2, 2, Distance(Distance::Euclidean), 0);
        CHECK(q.quantize(rows[1]).len() == dim);
        CHECK(q.quantize_batch(rows).size() == n);
        CHECK(q.rotation().size() == dim * dim);
        CHECK(q.encode(rows).size() == n * 3);
        auto none = OptimizedProductQuantizer::fit(rows, 3, 4, 2, 0, Distance(Distance::Euclidean), 0);
        CHECK(!none.trained());
        CHECK(none.quantize(rows[1]).len() == 0);
        CHECK(none.codebooks().empty());
    }
    // ResidualQuantizer, also with an epsilon stop and with k = 1 (src/rvq.rs:113-115, 139-141)
    {
        auto q = ResidualQuantizer::fit(rows, 3, 4, 2, 0.0f, Distance(Distance::Euclidean), 0);
        CHECK(q.quantize(rows[2]).len() == dim);
        CHECK(q.quantize_batch(rows).size() == n);
        auto early = ResidualQuantizer::fit(rows, 3, 4, 2, 1e9f, Distance(Distance::Euclidean), 0);
        CHECK(early.quantize_batch(rows).size() == n);
        auto one = ResidualQuantizer::fit(rows, 2, 1, 2, 0.0f, Distance(Distance::Manhattan), 0);
        CHECK(one.quantize(rows[0]).len() == dim);
    }
    // TSVQ
    {
        auto t = TSVQ::create(rows, 3, Distance(Distance::CosineDistance));
        CHECK(t.quantize(rows[3]).len() == dim);
        CHECK(t.quantize_batch(rows).size() == n);
        auto k = TSVQ::create_kmeans(rows, 3, 4, Distance(Distance::Euclidean), 11);
        CHECK(k.quantize_batch(rows).size() == n);
        std::vector<uint32_t> wrong(5, 0u);
        CHECK(!message_of([&] { TSVQ::create_kmeans(rows, 3, 4, Distance(Distance::Euclidean), 11, &wrong); }).empty());
    }
    // the flat C entry points, as the Python binding drives them
    {
        void *obj = nullptr;
        CHECK(vqh_pq_fit(flat.data(), (int64_t)n, (int64_t)dim, 3, 4, 2, 1, 0.0, 0, nullptr, nullptr, 0, &obj) == 0);
        std::vector<uint16_t> out(n * dim);
        int64_t got = 0;
        CHECK(vqh_quantize(obj, flat.data(), (int64_t)dim, out.data(), &got) == 0 && got == (int64_t)dim);
        CHECK(vqh_quantize_batch(obj, flat.data(), (int64_t)n, (int64_t)dim, out.data()) == 0);
        CHECK(vqh_quantize_batch_vectors(obj, flat.data(), (int64_t)n, (int64_t)dim, -1, 0, out.data()) == 0);
        CHECK(vqh_quantize_batch_vectors(obj, flat.data(), (int64_t)n, (int64_t)dim, 5, 7, out.data()) != 0);
        CHECK(std::string(vqh_last_error()) == "Dimension mismatch: expected 12, got 7");
        std::vector<uint8_t> codes(n * 3);
        CHECK(vqh_encode(obj, flat.data(), (int64_t)n, (int64_t)dim, codes.data()) == 0);
        int64_t info[7];
        CHECK(vqh_info(obj, info) == 0 && info[1] == 3 && info[2] == 4);
        std::vector<float> cb(3 * 4 * 4);
        CHECK(vqh_codebooks(obj, cb.data()) == 0);
        vqh_free(obj);
        CHECK(vqh_pq_fit(flat.data(), (int64_t)n, (int64_t)dim, 3, 0, 2, 1, 0.0, 0, nullptr, nullptr, 0, &obj) != 0);
        CHECK(std::string(vqh_last_error()) == "Invalid parameter: k must be greater than 0");
        void *tr = nullptr;
        CHECK(vqh_tsvq_new(flat.data(), (int64_t)n, (int64_t)dim, 2, 2, 0.0, &tr) == 0);
        std::vector<int32_t> leaves(n);
        CHECK(vqh_leaves(tr, flat.data(), (int64_t)n, (int64_t)dim, leaves.data()) == 0);
        vqh_free(tr);
    }
    if (failures) {
        std::fprintf(stderr, "host mirror: %d check(s) failed\n", failures);
        return 1;
    }
    std::printf("host mirror: ok\n");
    return 0;
}
