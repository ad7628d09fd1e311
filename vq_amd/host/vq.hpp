// vq.hpp — host-side mirror of the `vq` crate's public API for the codebook quantizers, written
// in C++ above the C ABI of libvqhip (include/vq_hip.h).  The reference is Rust; this image has
// no Rust toolchain, so this header plays the role the Rust host crate would: same type names,
// same argument order and meaning, same validation, and the reference's panic messages as
// exception texts.
//
//   Vector<T>                      src/vector.rs:149-173
//   Distance                       src/distances.rs:73-88 (kernels: the first four variants)
//   VqError                        src/exceptions.rs:9-25   (panics become C++ exceptions)
//   lbg_quantize                   src/utils.rs:32-109
//   ProductQuantizer               src/pq.rs:52-188
//   OptimizedProductQuantizer      src/opq.rs:57-265
//   ResidualQuantizer              src/rvq.rs:57-216
//   TSVQ                           src/tsvq.rs:189-250
//
// Beyond the reference API every quantizer offers batch calls (quantize_batch, encode): one
// vector at a time cannot feed a GPU.
//
// Randomness.  The reference seeds rand 0.9's StdRng (`seed + i` per sub-problem) and draws
// `choose_multiple` / `choose`.  That crate is not available here, so IndexStreams::from_seed
// is this host's OWN documented sampler (SplitMix64 + Floyd's algorithm): same contract
// (k distinct rows, uniform re-seed rows, deterministic in the seed), different numbers.
// A host that owns the real generator passes explicit IndexStreams instead.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <unordered_set>
#include <vector>

#include "../../include/vq_hip.h"

namespace vq {

// ---- errors (src/exceptions.rs) ----------------------------------------------------------------
struct VqError : std::runtime_error {
    int code;
    VqError(int c, const std::string &m) : std::runtime_error(m), code(c) {}
    static VqError DimensionMismatch(size_t expected, size_t found) {
        return VqError(VQ_ERR_DIM_MISMATCH, "Dimension mismatch: expected " + std::to_string(expected) +
                                                ", got " + std::to_string(found));
    }
    static VqError EmptyInput() {
        return VqError(VQ_ERR_EMPTY_INPUT, "Empty input: at least one vector is required.");
    }
    static VqError InvalidParameter(const std::string &s) {
        return VqError(VQ_ERR_INVALID_ARG, "Invalid parameter: " + s);
    }
    static VqError InvalidMetricParameter(const std::string &metric, const std::string &details) {
        return VqError(VQ_ERR_UNSUPPORTED, "Invalid metric parameter for " + metric + ": " + details);
    }
};

// ---- f16 and Vector (src/vector.rs) ------------------------------------------------------------
struct f16 {
    uint16_t bits = 0;
    float to_f32() const {
        uint32_t sign = ((uint32_t)bits & 0x8000u) << 16, exp = (bits >> 10) & 0x1fu, man = bits & 0x3ffu, x;
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
        std::memcpy(&f, &x, 4);
        return f;
    }
    bool operator==(const f16 &o) const { return bits == o.bits; }
};

template <class T>
struct Vector {
    std::vector<T> data;
    Vector() = default;
    explicit Vector(std::vector<T> d) : data(std::move(d)) {}
    size_t len() const { return data.size(); }
    bool is_empty() const { return data.empty(); }
    bool operator==(const Vector &o) const { return data == o.data; }
};

// ---- Distance (src/distances.rs:73-88) ------------------------------------------------------------
struct Distance {
    enum Kind { SquaredEuclidean, Euclidean, CosineDistance, Manhattan, Chebyshev, Minkowski, Hamming };
    Kind kind = SquaredEuclidean;
    double p = 0.0;
    Distance() = default;
    Distance(Kind k, double p_ = 0.0) : kind(k), p(p_) {}
    // The metric id of the C ABI; the three variants without a kernel are rejected.
    int32_t abi_metric() const {
        switch (kind) {
        case SquaredEuclidean: return VQ_SQEUCLIDEAN;
        case Euclidean: return VQ_EUCLIDEAN;
        case CosineDistance: return VQ_COSINE;
        case Manhattan: return VQ_MANHATTAN;
        case Chebyshev: throw VqError::InvalidMetricParameter("Chebyshev", "no device kernel");
        case Minkowski: throw VqError::InvalidMetricParameter("Minkowski", "no device kernel");
        default: throw VqError::InvalidMetricParameter("Hamming", "no device kernel");
        }
    }
};

// ---- index streams -----------------------------------------------------------------------------
struct IndexStreams {
    std::vector<uint32_t> init;    // problems * k
    std::vector<uint32_t> reseed;  // problems * n_reseed
    int32_t n_reseed = 0;

    static uint64_t splitmix(uint64_t &s) {
        uint64_t z = (s += 0x9e3779b97f4a7c15ull);
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        return z ^ (z >> 31);
    }
    static uint64_t below(uint64_t &s, uint64_t bound) {  // unbiased, by rejection
        uint64_t lim = UINT64_MAX - UINT64_MAX % bound;
        uint64_t r;
        do r = splitmix(s);
        while (r >= lim);
        return r % bound;
    }
    // Problem i is seeded with seed + i (src/pq.rs:119, src/opq.rs:140, src/rvq.rs:107): first k
    // distinct rows (Floyd's algorithm, insertion order), then k*max_iters re-seed draws.
    static IndexStreams from_seed(uint64_t seed, size_t problems, size_t n, size_t k, size_t max_iters) {
        IndexStreams st;
        st.n_reseed = (int32_t)(k * max_iters);
        st.init.resize(problems * k);
        st.reseed.resize(problems * (size_t)st.n_reseed);
        for (size_t i = 0; i < problems; ++i) {
            uint64_t s = seed + i;
            std::unordered_set<uint32_t> seen;
            size_t w = 0;
            for (size_t j = n - k; j < n; ++j) {
                uint32_t t = (uint32_t)below(s, j + 1);
                uint32_t pick = seen.insert(t).second ? t : (uint32_t)j;
                if (pick == (uint32_t)j) seen.insert(pick);
                st.init[i * k + w++] = pick;
            }
            for (int32_t r = 0; r < st.n_reseed; ++r)
                st.reseed[i * (size_t)st.n_reseed + r] = (uint32_t)below(s, n);
        }
        return st;
    }
};

// ---- device plumbing ---------------------------------------------------------------------------
class Device {
public:
    explicit Device(int index = 0) {
        if (vq_ctx_create(index, &ctx_) != VQ_OK) throw VqError(VQ_ERR_HIP, vq_last_error(nullptr));
    }
    ~Device() { vq_ctx_destroy(ctx_); }
    Device(const Device &) = delete;
    Device &operator=(const Device &) = delete;
    vq_ctx *ctx() const { return ctx_; }
    void check(int32_t rc) const {
        if (rc != VQ_OK) throw VqError(rc, vq_last_error(ctx_));
    }
    static std::shared_ptr<Device> shared() {
        static std::shared_ptr<Device> d = std::make_shared<Device>(0);
        return d;
    }

private:
    vq_ctx *ctx_ = nullptr;
};

template <class T>
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    DeviceBuffer(std::shared_ptr<Device> d, size_t count) : dev_(std::move(d)), count_(count) {
        void *p = nullptr;
        dev_->check(vq_malloc(dev_->ctx(), count * sizeof(T), &p));
        ptr_ = static_cast<T *>(p);
    }
    DeviceBuffer(DeviceBuffer &&o) noexcept { *this = std::move(o); }
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept {
        release();
        dev_ = std::move(o.dev_);
        ptr_ = o.ptr_;
        count_ = o.count_;
        o.ptr_ = nullptr;
        o.count_ = 0;
        return *this;
    }
    ~DeviceBuffer() { release(); }
    T *get() const { return ptr_; }
    size_t size() const { return count_; }
    void upload(const T *src, size_t count) { dev_->check(vq_h2d(dev_->ctx(), ptr_, src, count * sizeof(T))); }
    void download(T *dst, size_t count) const { dev_->check(vq_d2h(dev_->ctx(), dst, ptr_, count * sizeof(T))); }
    std::vector<T> to_host() const {
        std::vector<T> v(count_);
        if (count_) download(v.data(), count_);
        return v;
    }

private:
    void release() {
        if (ptr_ && dev_) vq_free(dev_->ctx(), ptr_);
        ptr_ = nullptr;
    }
    std::shared_ptr<Device> dev_;
    T *ptr_ = nullptr;
    size_t count_ = 0;
};

// Device codes of either width: bytes up to 256 centroids, 16 bits above (`k: usize` in the
// reference, src/utils.rs:32-37; the library's *_u16 entry points).
class DeviceCodes {
public:
    DeviceCodes() = default;
    DeviceCodes(std::shared_ptr<Device> dev, size_t count, size_t k) : wide_(k > 256) {
        if (wide_)
            b16_ = DeviceBuffer<uint16_t>(std::move(dev), count);
        else
            b8_ = DeviceBuffer<uint8_t>(std::move(dev), count);
    }
    bool wide() const { return wide_; }
    DeviceBuffer<uint8_t> &narrow() { return b8_; }
    uint8_t *p8() const { return b8_.get(); }
    uint16_t *p16() const { return b16_.get(); }
    std::vector<uint8_t> to_host8() const {
        if (wide_) throw VqError::InvalidParameter("codes above 256 centroids are 16 bits wide");
        return b8_.to_host();
    }
    std::vector<uint16_t> to_host16() const {
        if (wide_) return b16_.to_host();
        const std::vector<uint8_t> v = b8_.to_host();
        return std::vector<uint16_t>(v.begin(), v.end());
    }

private:
    bool wide_ = false;
    DeviceBuffer<uint8_t> b8_;
    DeviceBuffer<uint16_t> b16_;
};

inline int32_t abi_assign(vq_ctx *c, int32_t metric, const float *x, size_t n, size_t ld, size_t m, size_t sd,
                          size_t k, const float *cb, const DeviceCodes &codes) {
    return codes.wide() ? vq_assign_u16(c, metric, x, (int64_t)n, (int64_t)ld, (int32_t)m, (int32_t)sd, (int32_t)k,
                                        cb, codes.p16())
                        : vq_assign(c, metric, x, (int64_t)n, (int64_t)ld, (int32_t)m, (int32_t)sd, (int32_t)k, cb,
                                    codes.p8());
}
inline int32_t abi_decode_f16(vq_ctx *c, const DeviceCodes &codes, size_t n, size_t m, size_t sd, size_t k,
                              const float *cb, uint16_t *out) {
    return codes.wide() ? vq_decode_f16_u16(c, codes.p16(), (int64_t)n, (int32_t)m, (int32_t)sd, (int32_t)k, cb, out)
                        : vq_decode_f16(c, codes.p8(), (int64_t)n, (int32_t)m, (int32_t)sd, (int32_t)k, cb, out);
}
inline int32_t abi_decode_f32(vq_ctx *c, const DeviceCodes &codes, size_t n, size_t m, size_t sd, size_t k,
                              const float *cb, float *out) {
    return codes.wide() ? vq_decode_f32_u16(c, codes.p16(), (int64_t)n, (int32_t)m, (int32_t)sd, (int32_t)k, cb, out)
                        : vq_decode_f32(c, codes.p8(), (int64_t)n, (int32_t)m, (int32_t)sd, (int32_t)k, cb, out);
}

// `&[Vector<f32>]` as the device wants it: one row-major buffer.  The reference's shape — one
// heap allocation per vector (src/vector.rs:150-152) — converts implicitly: packed once, lengths
// checked.  Rows that are contiguous already (a matrix of another library, a memory-mapped file)
// are taken as a view, without a copy.
class Rows {
public:
    Rows(const std::vector<Vector<float>> &rows) : n_(rows.size()), dim_(rows.empty() ? 0 : rows[0].len()) {
        own_.resize(n_ * dim_);
        for (size_t i = 0; i < n_; ++i) {
            if (rows[i].len() != dim_) {  // reported by expect_dim, in the order a row-by-row check would
                ragged_ = true;
                ragged_len_ = rows[i].len();
                break;
            }
            std::memcpy(own_.data() + i * dim_, rows[i].data.data(), dim_ * sizeof(float));
        }
        p_ = own_.data();
    }
    static Rows view(const float *p, size_t n, size_t dim) {
        Rows r;
        r.p_ = p;
        r.n_ = n;
        r.dim_ = dim;
        return r;
    }
    bool empty() const { return n_ == 0; }
    size_t size() const { return n_; }
    size_t dim() const { return dim_; }  // length of the first row
    const float *data() const { return p_; }
    // every row has `dim` floats, or "Dimension mismatch" with the first length that differs
    void expect_dim(size_t dim) const {
        if (n_ == 0) return;
        if (dim_ != dim) throw VqError::DimensionMismatch(dim, dim_);
        if (ragged_) throw VqError::DimensionMismatch(dim, ragged_len_);
    }

private:
    Rows() = default;
    std::vector<float> own_;
    const float *p_ = nullptr;
    size_t n_ = 0, dim_ = 0, ragged_len_ = 0;
    bool ragged_ = false;
};

inline std::vector<Vector<f16>> unpack_f16(const std::vector<uint16_t> &flat, size_t n, size_t dim) {
    if (flat.empty()) return {};
    std::vector<Vector<f16>> out(n);
    for (size_t i = 0; i < n; ++i) {
        out[i].data.resize(dim);
        for (size_t t = 0; t < dim; ++t) out[i].data[t].bits = flat[i * dim + t];
    }
    return out;
}

// ---- lbg_quantize (src/utils.rs:32-109) --------------------------------------------------------
inline std::vector<Vector<float>> lbg_quantize(const Rows &data, size_t k,
                                               size_t max_iters, uint64_t seed,
                                               const IndexStreams *streams = nullptr,
                                               std::shared_ptr<Device> dev = Device::shared()) {
    size_t n = data.size();
    if (k == 0) throw VqError::InvalidParameter("k must be greater than 0");
    if (n < k) throw VqError::InvalidParameter("Not enough data points for k clusters");
    size_t dim = data.dim();
    data.expect_dim(dim);
    IndexStreams own;
    if (!streams) {
        own = IndexStreams::from_seed(seed, 1, n, k, max_iters);
        streams = &own;
    }
    DeviceBuffer<float> dx(dev, n * dim), dcb(dev, k * dim);
    dx.upload(data.data(), n * dim);
    dev->check(vq_lbg_fit(dev->ctx(), dx.get(), (int64_t)n, (int64_t)dim, 1, (int32_t)dim, (int32_t)k,
                          (int32_t)max_iters, streams->init.data(), streams->reseed.data(),
                          streams->n_reseed, dcb.get(), nullptr, nullptr));
    std::vector<float> cb = dcb.to_host();
    std::vector<Vector<float>> out(k);
    for (size_t j = 0; j < k; ++j) out[j].data.assign(cb.begin() + j * dim, cb.begin() + (j + 1) * dim);
    return out;
}

// ---- ProductQuantizer (src/pq.rs) ----------------------------------------------------------------
class ProductQuantizer {
public:
    // src/pq.rs:79-129
    static ProductQuantizer fit(const Rows &training_data, size_t m, size_t k,
                                size_t max_iters, Distance distance, uint64_t seed,
                                const IndexStreams *streams = nullptr,
                                std::shared_ptr<Device> dev = Device::shared()) {
        if (training_data.empty()) throw VqError::EmptyInput();
        size_t n = training_data.dim();
        if (n < m) throw VqError::InvalidParameter("Data dimension must be at least m");
        if (n % m != 0) throw VqError::InvalidParameter("Data dimension must be divisible by m");
        size_t rows = training_data.size();
        if (k == 0) throw VqError::InvalidParameter("k must be greater than 0");
        if (rows < k) throw VqError::InvalidParameter("Not enough data points for k clusters");
        ProductQuantizer pq;
        pq.dev_ = dev;
        pq.m_ = m;
        pq.k_ = k;
        pq.sub_dim_ = n / m;
        pq.distance_ = distance;
        training_data.expect_dim(n);
        const float *flat = training_data.data();
        IndexStreams own;
        if (!streams) {
            own = IndexStreams::from_seed(seed, m, rows, k, max_iters);
            streams = &own;
        }
        DeviceBuffer<float> dx(dev, rows * n);
        dx.upload(flat, dx.size());
        pq.codebooks_ = DeviceBuffer<float>(dev, m * k * pq.sub_dim_);
        dev->check(vq_lbg_fit(dev->ctx(), dx.get(), (int64_t)rows, (int64_t)n, (int32_t)m, (int32_t)pq.sub_dim_,
                              (int32_t)k, (int32_t)max_iters, streams->init.data(), streams->reseed.data(),
                              streams->n_reseed, pq.codebooks_.get(), nullptr, nullptr));
        return pq;
    }

    // src/pq.rs:146-187
    Vector<f16> quantize(const Vector<float> &vector) const {
        if (vector.len() != sub_dim_ * m_) throw VqError::DimensionMismatch(sub_dim_ * m_, vector.len());
        return quantize_batch(std::vector<Vector<float>>{vector})[0];
    }

    std::vector<Vector<f16>> quantize_batch(const Rows &vectors) const {
        return unpack_f16(quantize_batch_flat(vectors), vectors.size(), sub_dim_ * m_);
    }

    // the same reconstructions as one row-major n x dim array of f16 bit patterns
    std::vector<uint16_t> quantize_batch_flat(const Rows &vectors) const {
        size_t dim = sub_dim_ * m_, n = vectors.size();
        if (n == 0) return {};
        vectors.expect_dim(dim);
        const float *flat = vectors.data();
        DeviceBuffer<float> dx(dev_, n * dim);
        dx.upload(flat, dx.size());
        DeviceCodes dcodes(dev_, n * m_, k_);
        DeviceBuffer<uint16_t> dout(dev_, n * dim);
        dev_->check(abi_assign(dev_->ctx(), distance_.abi_metric(), dx.get(), n, dim, m_, sub_dim_, k_,
                               codebooks_.get(), dcodes));
        dev_->check(abi_decode_f16(dev_->ctx(), dcodes, n, m_, sub_dim_, k_, codebooks_.get(), dout.get()));
        return dout.to_host();
    }

    // The integer codes the reference keeps only as `best_index` (src/pq.rs:166-174): n x m bytes
    // (k <= 256), or 16 bits each for any k.
    std::vector<uint8_t> encode(const Rows &vectors) const { return encode_device(vectors).to_host8(); }
    std::vector<uint16_t> encode16(const Rows &vectors) const { return encode_device(vectors).to_host16(); }

    std::vector<float> codebooks() const { return codebooks_.to_host(); }  // m*k*sub_dim
    size_t m() const { return m_; }
    size_t k() const { return k_; }
    size_t sub_dim() const { return sub_dim_; }

private:
    DeviceCodes encode_device(const Rows &vectors) const {
        size_t dim = sub_dim_ * m_, n = vectors.size();
        if (n == 0) return DeviceCodes();
        vectors.expect_dim(dim);
        const float *flat = vectors.data();
        DeviceBuffer<float> dx(dev_, n * dim);
        dx.upload(flat, dx.size());
        DeviceCodes dcodes(dev_, n * m_, k_);
        dev_->check(abi_assign(dev_->ctx(), distance_.abi_metric(), dx.get(), n, dim, m_, sub_dim_, k_,
                               codebooks_.get(), dcodes));
        dev_->check(vq_ctx_sync(dev_->ctx()));
        return dcodes;
    }
    std::shared_ptr<Device> dev_;
    DeviceBuffer<float> codebooks_;
    size_t sub_dim_ = 0, m_ = 0, k_ = 0;
    Distance distance_;
};

// ---- OptimizedProductQuantizer (src/opq.rs) -----------------------------------------------------
class OptimizedProductQuantizer {
public:
    // src/opq.rs:90-205
    static OptimizedProductQuantizer fit(const Rows &training_data, size_t m, size_t k,
                                         size_t max_iters, size_t opq_iters, Distance distance, uint64_t seed,
                                         const IndexStreams *streams = nullptr,
                                         std::shared_ptr<Device> dev = Device::shared()) {
        if (training_data.empty()) throw VqError::EmptyInput();
        size_t dim = training_data.dim();
        if (dim < m) throw VqError::InvalidParameter("Dimension must be at least m");
        if (dim % m != 0) throw VqError::InvalidParameter("Dimension must be divisible by m");
        size_t n = training_data.size(), sd = dim / m;
        if (k == 0) throw VqError::InvalidParameter("k must be greater than 0");
        if (n < k) throw VqError::InvalidParameter("Not enough data points for k clusters");
        OptimizedProductQuantizer q;
        q.dev_ = dev;
        q.m_ = m;
        q.k_ = k;
        q.sub_dim_ = sd;
        q.dim_ = dim;
        q.distance_ = distance;
        const int32_t metric = distance.abi_metric();
        training_data.expect_dim(dim);
        const float *flat = training_data.data();
        IndexStreams own;
        if (!streams) {  // the same streams in every outer iteration (opq.rs:140 re-seeds seed + i)
            own = IndexStreams::from_seed(seed, m, n, k, max_iters);
            streams = &own;
        }
        vq_ctx *c = dev->ctx();
        DeviceBuffer<float> dx(dev, n * dim), drot(dev, n * dim), drec(dev, n * dim);
        DeviceCodes dcodes(dev, n * m, k);
        dx.upload(flat, dx.size());
        dev->check(vq_copy_f32(c, drot.get(), dx.get(), (int64_t)(n * dim)));  // opq.rs:121
        q.codebooks_ = DeviceBuffer<float>(dev, m * k * sd);
        q.rotation_.assign(dim * dim, 0.f);
        for (size_t i = 0; i < dim; ++i) q.rotation_[i * dim + i] = 1.f;  // opq.rs:119
        q.d_rotation_ = DeviceBuffer<float>(dev, dim * dim);
        std::vector<double> A(dim * dim), Rd;
        for (size_t it = 0; it < opq_iters; ++it) {
            dev->check(vq_lbg_fit(c, drot.get(), (int64_t)n, (int64_t)dim, (int32_t)m, (int32_t)sd, (int32_t)k,
                                  (int32_t)max_iters, streams->init.data(), streams->reseed.data(),
                                  streams->n_reseed, q.codebooks_.get(), nullptr, nullptr));  // 127-142
            dev->check(abi_assign(c, metric, drot.get(), n, dim, m, sd, k, q.codebooks_.get(), dcodes));  // 146-163
            dev->check(abi_decode_f32(c, dcodes, n, m, sd, k, q.codebooks_.get(), drec.get()));         // 164-167
            dev->check(vq_cross_cov(c, drec.get(), drot.get(), (int64_t)n, (int32_t)dim, A.data())); // 172-179
            for (double &v : A) v = (double)(float)v;  // the reference's A is a DMatrix<f32>
            // 180-183 (the library runs the SVD on the device while its kernel takes the size,
            // else on the host, and completes the directions a singular A leaves open)
            Rd.resize(dim * dim);
            dev->check(vq_procrustes_rotation(c, A.data(), (int32_t)dim, Rd.data()));
            for (size_t i = 0; i < dim * dim; ++i) q.rotation_[i] = (float)Rd[i];
            q.d_rotation_.upload(q.rotation_.data(), dim * dim);
            dev->check(vq_rotate(c, dx.get(), (int64_t)n, (int64_t)dim, (int32_t)dim, q.d_rotation_.get(),
                                 drot.get()));                                                    // 186-194
        }
        if (opq_iters == 0) {
            // no outer iteration: the reference keeps an identity rotation and NO codebooks
            // (src/opq.rs:122), so quantize returns an empty vector
            q.d_rotation_.upload(q.rotation_.data(), dim * dim);
            q.codebooks_ = DeviceBuffer<float>();
            q.trained_ = false;
        }
        return q;
    }

    // src/opq.rs:222-264
    Vector<f16> quantize(const Vector<float> &vector) const {
        if (vector.len() != dim_) throw VqError::DimensionMismatch(dim_, vector.len());
        if (!trained_) return Vector<f16>();  // the loop over no codebooks pushes nothing (opq.rs:244-263)
        return quantize_batch(std::vector<Vector<float>>{vector})[0];
    }

    std::vector<Vector<f16>> quantize_batch(const Rows &vectors) const {
        if (!trained_) {
            vectors.expect_dim(dim_);
            return std::vector<Vector<f16>>(vectors.size());
        }
        return unpack_f16(quantize_batch_flat(vectors), vectors.size(), dim_);
    }

    // n x dim f16 bit patterns; empty (n rows of length 0) when fit ran no outer iteration
    std::vector<uint16_t> quantize_batch_flat(const Rows &vectors) const {
        size_t n = vectors.size();
        if (n == 0) return {};
        if (!trained_) {
            vectors.expect_dim(dim_);
            return {};
        }
        DeviceCodes dcodes = encode_device(vectors);
        DeviceBuffer<uint16_t> dout(dev_, n * dim_);
        dev_->check(abi_decode_f16(dev_->ctx(), dcodes, n, m_, sub_dim_, k_, codebooks_.get(), dout.get()));
        return dout.to_host();
    }

    std::vector<uint8_t> encode(const Rows &vectors) const {
        if (vectors.empty() || !trained_) return {};
        return encode_device(vectors).to_host8();
    }
    std::vector<uint16_t> encode16(const Rows &vectors) const {  // any k
        if (vectors.empty() || !trained_) return {};
        return encode_device(vectors).to_host16();
    }

    std::vector<float> codebooks() const { return trained_ ? codebooks_.to_host() : std::vector<float>(); }
    const std::vector<float> &rotation() const { return rotation_; }  // row-major dim x dim
    bool trained() const { return trained_; }  // false: fit ran with opq_iters == 0
    size_t m() const { return m_; }
    size_t k() const { return k_; }
    size_t sub_dim() const { return sub_dim_; }

private:
    DeviceCodes encode_device(const Rows &vectors) const {
        size_t n = vectors.size();
        vectors.expect_dim(dim_);
        const float *flat = vectors.data();
        DeviceBuffer<float> dx(dev_, n * dim_), dy(dev_, n * dim_);
        dx.upload(flat, dx.size());
        DeviceCodes dcodes(dev_, n * m_, k_);
        vq_ctx *c = dev_->ctx();
        dev_->check(vq_rotate(c, dx.get(), (int64_t)n, (int64_t)dim_, (int32_t)dim_, d_rotation_.get(), dy.get()));
        dev_->check(abi_assign(c, distance_.abi_metric(), dy.get(), n, dim_, m_, sub_dim_, k_, codebooks_.get(),
                               dcodes));
        dev_->check(vq_ctx_sync(c));
        return dcodes;
    }
    std::shared_ptr<Device> dev_;
    DeviceBuffer<float> codebooks_, d_rotation_;
    std::vector<float> rotation_;
    bool trained_ = true;
    size_t sub_dim_ = 0, m_ = 0, k_ = 0, dim_ = 0;
    Distance distance_;
};

// ---- ResidualQuantizer (src/rvq.rs) --------------------------------------------------------------
class ResidualQuantizer {
public:
    // src/rvq.rs:87-154
    static ResidualQuantizer fit(const Rows &training_data, size_t stages, size_t k,
                                 size_t max_iters, float epsilon, Distance distance, uint64_t seed,
                                 const IndexStreams *streams = nullptr,
                                 std::shared_ptr<Device> dev = Device::shared()) {
        if (training_data.empty()) throw VqError::EmptyInput();
        size_t dim = training_data.dim(), n = training_data.size();
        if (stages > 0) {
            if (k == 0) throw VqError::InvalidParameter("k must be greater than 0");
            if (n < k) throw VqError::InvalidParameter("Not enough data points for k clusters");
        }
        ResidualQuantizer q;
        q.dev_ = dev;
        q.dim_ = dim;
        q.k_ = k;
        q.epsilon_ = epsilon;
        q.distance_ = distance;
        const int32_t metric = distance.abi_metric();
        training_data.expect_dim(dim);
        const float *flat = training_data.data();
        IndexStreams own;
        if (!streams) {
            own = IndexStreams::from_seed(seed, stages, n, k, max_iters);
            streams = &own;
        }
        vq_ctx *c = dev->ctx();
        DeviceBuffer<float> dx(dev, n * dim), dres(dev, n * dim);
        DeviceCodes dcodes(dev, n + 16, k);
        dx.upload(flat, dx.size());
        dev->check(vq_copy_f32(c, dres.get(), dx.get(), (int64_t)(n * dim)));  // rvq.rs:103
        q.codebooks_ = DeviceBuffer<float>(dev, std::max<size_t>(stages * k * dim, 1));
        std::vector<uint8_t> zeros(n, 0);
        size_t produced = 0;
        const float *pending_cb = nullptr;  // a residual update that rides on the next stage's fit
        for (size_t st = 0; st < stages; ++st) {
            float *cb = q.codebooks_.get() + st * k * dim;
            if (pending_cb)  // rvq.rs:127 of the stage before, then rvq.rs:107
                dev->check(vq_lbg_fit_residual(c, dres.get(), (int64_t)n, (int64_t)dim, (int32_t)dim, (int32_t)k,
                                               (int32_t)max_iters, streams->init.data() + st * k,
                                               streams->reseed.data() + st * (size_t)streams->n_reseed,
                                               streams->n_reseed, cb, pending_cb, (int32_t)k, dcodes.p8(), nullptr,
                                               nullptr));
            else
                dev->check(vq_lbg_fit(c, dres.get(), (int64_t)n, (int64_t)dim, 1, (int32_t)dim, (int32_t)k,
                                      (int32_t)max_iters, streams->init.data() + st * k,
                                      streams->reseed.data() + st * (size_t)streams->n_reseed, streams->n_reseed, cb,
                                      nullptr, nullptr));  // rvq.rs:107
            pending_cb = nullptr;
            ++produced;
            // The residuals are a local of the reference's fit (rvq.rs:103) and nothing follows the
            // last stage: its residual update and norm test (111-141) cannot be observed and are left out.
            if (st + 1 == stages) break;
            if (k < 2)  // rvq.rs:113-115
                dcodes.narrow().upload(zeros.data(), n);
            else
                dev->check(abi_assign(c, metric, dres.get(), n, dim, 1, dim, k, cb, dcodes));  // rvq.rs:116-125
            if (!dcodes.wide() && !(epsilon > 0.f)) {
                // nothing looks at the residual before the next stage trains on it: the update is
                // handed to that fit, whose first pass over the rows applies it
                pending_cb = cb;
                continue;
            }
            dev->check(dcodes.wide()
                           ? vq_residual_sub_u16(c, dres.get(), (int64_t)n, (int64_t)dim, (int32_t)dim, (int32_t)k, cb,
                                                 dcodes.p16())
                           : vq_residual_sub(c, dres.get(), (int64_t)n, (int64_t)dim, (int32_t)dim, (int32_t)k, cb,
                                             dcodes.p8()));  // rvq.rs:127
            if (epsilon > 0.f) {  // a mean norm is never below a non-positive (or NaN) threshold
                float avg = 0.f;
                dev->check(vq_mean_l2norm(c, dres.get(), (int64_t)n, (int64_t)dim, (int32_t)dim, &avg));  // 131-138
                if (avg < epsilon) break;  // rvq.rs:139-141
            }
        }
        q.stages_ = produced;  // rvq.rs:145
        return q;
    }

    // src/rvq.rs:171-215
    Vector<f16> quantize(const Vector<float> &vector) const {
        if (vector.len() != dim_) throw VqError::DimensionMismatch(dim_, vector.len());
        return quantize_batch(std::vector<Vector<float>>{vector})[0];
    }

    std::vector<Vector<f16>> quantize_batch(const Rows &vectors, std::vector<uint8_t> *codes = nullptr) const {
        return unpack_f16(quantize_batch_flat(vectors, codes), vectors.size(), dim_);
    }

    // codes: n x stages bytes (k <= 256 only); codes16: the same 16 bits wide, any k
    std::vector<uint16_t> quantize_batch_flat(const Rows &vectors, std::vector<uint8_t> *codes = nullptr,
                                              std::vector<uint16_t> *codes16 = nullptr) const {
        size_t n = vectors.size();
        if (n == 0) return {};
        vectors.expect_dim(dim_);
        const float *flat = vectors.data();
        DeviceBuffer<float> dx(dev_, n * dim_);
        dx.upload(flat, dx.size());
        DeviceCodes dcodes(dev_, std::max<size_t>(n * stages_, 1), k_);
        DeviceBuffer<uint16_t> dout(dev_, n * dim_);
        const int32_t k = (int32_t)std::max<size_t>(k_, 1);
        dev_->check(dcodes.wide()
                        ? vq_rvq_encode_u16(dev_->ctx(), distance_.abi_metric(), dx.get(), (int64_t)n, (int64_t)dim_,
                                            (int32_t)dim_, (int32_t)stages_, k, codebooks_.get(), epsilon_,
                                            dcodes.p16(), nullptr, dout.get())
                        : vq_rvq_encode(dev_->ctx(), distance_.abi_metric(), dx.get(), (int64_t)n, (int64_t)dim_,
                                        (int32_t)dim_, (int32_t)stages_, k, codebooks_.get(), epsilon_, dcodes.p8(),
                                        nullptr, dout.get()));
        if (codes) *codes = dcodes.to_host8();
        if (codes16) *codes16 = dcodes.to_host16();
        return dout.to_host();
    }

    size_t stages() const { return stages_; }
    std::vector<float> codebooks() const {  // stages*k*dim
        std::vector<float> all = codebooks_.to_host();
        all.resize(stages_ * k_ * dim_);
        return all;
    }

private:
    std::shared_ptr<Device> dev_;
    DeviceBuffer<float> codebooks_;
    size_t stages_ = 0, dim_ = 0, k_ = 0;
    float epsilon_ = 0.f;
    Distance distance_;
};

// ---- TSVQ (src/tsvq.rs) --------------------------------------------------------------------------
class TSVQ {
public:
    Distance distance;  // `pub distance`, src/tsvq.rs:193

    // TSVQ::new, src/tsvq.rs:209-215
    static TSVQ create(const Rows &training_data, size_t max_depth, Distance distance,
                       std::shared_ptr<Device> dev = Device::shared()) {
        if (training_data.empty()) throw VqError::EmptyInput();
        size_t dim = training_data.dim(), n = training_data.size();
        training_data.expect_dim(dim);
        const float *flat = training_data.data();
        TSVQ t;
        t.dev_ = dev;
        t.distance = distance;
        t.dim_ = dim;
        DeviceBuffer<float> dx(dev, n * dim);
        dx.upload(flat, dx.size());
        vq_tree *tree = nullptr;
        dev->check(vq_tsvq_build(dev->ctx(), dx.get(), (int64_t)n, (int64_t)dim, (int32_t)dim, (int32_t)max_depth,
                                 &tree));
        std::shared_ptr<Device> keep = dev;
        t.tree_ = std::shared_ptr<vq_tree>(tree, [keep](vq_tree *p) { vq_tree_free(keep->ctx(), p); });
        return t;
    }

    // NOT in the crate: the same tree with 2-means splits (lbg_quantize with k = 2 and lbg_iters
    // iterations on every node's rows) instead of the median split of src/tsvq.rs:87-123.  The node at
    // position h of the complete binary tree (root 1) draws from a generator seeded with seed + h:
    // two initial rows, one re-seed row per iteration; or the caller passes the draws themselves,
    // (2^max_depth - 1) x (2 + lbg_iters) values.
    static TSVQ create_kmeans(const Rows &training_data, size_t max_depth, size_t lbg_iters, Distance distance,
                              uint64_t seed, const std::vector<uint32_t> *draws = nullptr,
                              std::shared_ptr<Device> dev = Device::shared()) {
        if (training_data.empty()) throw VqError::EmptyInput();
        if (max_depth > 20) throw VqError::InvalidParameter("max_depth above 20 for a 2-means tree");
        size_t dim = training_data.dim(), n = training_data.size();
        training_data.expect_dim(dim);
        const size_t per_node = 2 + lbg_iters, positions = ((size_t)1 << max_depth) - 1;
        std::vector<uint32_t> own;
        if (!draws) {
            own.resize(positions * per_node);
            for (size_t h = 1; h <= positions; ++h) {
                uint64_t s = seed + h;
                for (size_t i = 0; i < per_node; ++i) own[(h - 1) * per_node + i] = (uint32_t)IndexStreams::splitmix(s);
            }
            draws = &own;
        } else if (draws->size() != positions * per_node) {
            throw VqError::InvalidParameter("a 2-means tree needs (2^max_depth - 1) * (2 + lbg_iters) draws");
        }
        TSVQ t;
        t.dev_ = dev;
        t.distance = distance;
        t.dim_ = dim;
        DeviceBuffer<float> dx(dev, n * dim);
        dx.upload(training_data.data(), dx.size());
        vq_tree *tree = nullptr;
        dev->check(vq_tsvq_build_kmeans(dev->ctx(), dx.get(), (int64_t)n, (int64_t)dim, (int32_t)dim, (int32_t)max_depth,
                                        (int32_t)lbg_iters, draws->data(), (int32_t)per_node, &tree));
        std::shared_ptr<Device> keep = dev;
        t.tree_ = std::shared_ptr<vq_tree>(tree, [keep](vq_tree *p) { vq_tree_free(keep->ctx(), p); });
        return t;
    }

    // src/tsvq.rs:231-249
    Vector<f16> quantize(const Vector<float> &vector) const {
        if (vector.len() != dim_) throw VqError::DimensionMismatch(dim_, vector.len());
        return quantize_batch(std::vector<Vector<float>>{vector})[0];
    }

    std::vector<Vector<f16>> quantize_batch(const Rows &vectors, std::vector<int32_t> *leaves = nullptr) const {
        return unpack_f16(quantize_batch_flat(vectors, leaves), vectors.size(), dim_);
    }

    std::vector<uint16_t> quantize_batch_flat(const Rows &vectors, std::vector<int32_t> *leaves = nullptr) const {
        size_t n = vectors.size();
        if (n == 0) return {};
        vectors.expect_dim(dim_);
        const float *flat = vectors.data();
        DeviceBuffer<float> dx(dev_, n * dim_);
        dx.upload(flat, dx.size());
        DeviceBuffer<int32_t> dleaf(dev_, n);
        DeviceBuffer<uint16_t> dout(dev_, n * dim_);
        dev_->check(vq_tsvq_descend(dev_->ctx(), distance.abi_metric(), dx.get(), (int64_t)n, (int64_t)dim_,
                                    tree_.get(), dleaf.get()));
        dev_->check(vq_tsvq_decode_f16(dev_->ctx(), tree_.get(), dleaf.get(), (int64_t)n, dout.get()));
        if (leaves) *leaves = dleaf.to_host();
        return dout.to_host();
    }

    int32_t n_nodes() const {
        int32_t nn = 0;
        vq_tree_info(tree_.get(), &nn, nullptr);
        return nn;
    }
    const vq_tree *tree() const { return tree_.get(); }

private:
    std::shared_ptr<Device> dev_;
    std::shared_ptr<vq_tree> tree_;
    size_t dim_ = 0;
};

}  // namespace vq
