// Host side of the OPQ rotation update R = V U^T for A = U S V^T (src/opq.rs:180-183): the
// one-sided Jacobi SVD in f64 for the sizes the device kernel does not take, and the completion
// of singular directions that A does not determine.  Plain C++, no HIP.
#pragma once
#include <cmath>
#include <cstddef>
#include <vector>

namespace vqh {

// A singular value this far below the largest one carries no direction (f64 Jacobi leaves columns
// of a rank-deficient matrix at rounding level, or exactly zero for an all-zero column of A).
constexpr double kNullRel = 1e-12;

// Ut[j*n + i] = U[i][j] (column j of U as a contiguous row), unit length where sv[j] is not null;
// Vt likewise, orthonormal.  Every null column j of U, in ascending j, becomes a unit vector
// orthogonal to all the columns fixed so far: the matching column of V if enough of it is left
// after the projection (an all-zero A then gives U = V, R = I, which is what an SVD library
// returns for it), else the unit vector e_i of which the most is left.  U ends up orthogonal,
// so R = V U^T is a rotation (or reflection) whatever the rank of A.
inline void complete_null_columns(std::vector<double> &Ut, const std::vector<double> &Vt,
                                  const std::vector<double> &sv, size_t n) {
    double top = 0.0;
    for (size_t j = 0; j < n; ++j) top = std::max(top, sv[j]);
    std::vector<char> fixed(n);
    bool any = false;
    for (size_t j = 0; j < n; ++j) {
        fixed[j] = top > 0.0 && sv[j] > kNullRel * top;
        any = any || !fixed[j];
    }
    if (!any) return;
    std::vector<double> w(n), best(n);
    auto residual = [&](std::vector<double> &v) {  // two rounds of Gram-Schmidt, then the norm left
        for (int round = 0; round < 2; ++round)
            for (size_t l = 0; l < n; ++l) {
                if (!fixed[l]) continue;
                double d = 0.0;
                for (size_t i = 0; i < n; ++i) d += Ut[l * n + i] * v[i];
                for (size_t i = 0; i < n; ++i) v[i] -= d * Ut[l * n + i];
            }
        double s = 0.0;
        for (size_t i = 0; i < n; ++i) s += v[i] * v[i];
        return std::sqrt(s);
    };
    for (size_t j = 0; j < n; ++j) {
        if (fixed[j]) continue;
        for (size_t i = 0; i < n; ++i) w[i] = Vt[j * n + i];
        double nrm = residual(w);
        if (!(nrm > 0.5)) {
            double bn = -1.0;
            for (size_t e = 0; e < n; ++e) {
                for (size_t i = 0; i < n; ++i) w[i] = i == e ? 1.0 : 0.0;
                const double r = residual(w);
                if (r > bn) {
                    bn = r;
                    best = w;
                }
            }
            w = best;
            nrm = bn;
        }
        for (size_t i = 0; i < n; ++i) Ut[j * n + i] = w[i] / nrm;
        fixed[j] = 1;
    }
}

// R[i][j] = sum_l V[i][l] U[j][l], l ascending
inline void product_v_ut(const std::vector<double> &Vt, const std::vector<double> &Ut, size_t n, double *R) {
    for (size_t i = 0; i < n * n; ++i) R[i] = 0.0;
    for (size_t l = 0; l < n; ++l)
        for (size_t i = 0; i < n; ++i) {
            const double v = Vt[l * n + i];
            for (size_t j = 0; j < n; ++j) R[i * n + j] += v * Ut[l * n + j];
        }
}

// Cyclic one-sided Jacobi on the columns of A (row-major n x n), any n >= 1.
inline void procrustes_host(const double *A, size_t n, double *R) {
    std::vector<double> Ut(n * n), Vt(n * n, 0.0), sv(n);
    for (size_t i = 0; i < n; ++i) {
        Vt[i * n + i] = 1.0;
        for (size_t j = 0; j < n; ++j) Ut[j * n + i] = A[i * n + j];
    }
    for (int sweep = 0; sweep < 60; ++sweep) {
        double off = 0.0;
        for (size_t p = 0; p + 1 < n; ++p)
            for (size_t q = p + 1; q < n; ++q) {
                double *up = &Ut[p * n], *uq = &Ut[q * n];
                double alpha = 0, beta = 0, gamma = 0;
                for (size_t i = 0; i < n; ++i) {
                    alpha += up[i] * up[i];
                    beta += uq[i] * uq[i];
                    gamma += up[i] * uq[i];
                }
                if (gamma == 0.0) continue;
                off = std::max(off, std::fabs(gamma) / std::sqrt(alpha * beta + 1e-300));
                const double zeta = (beta - alpha) / (2.0 * gamma);
                const double t = (zeta >= 0 ? 1.0 : -1.0) / (std::fabs(zeta) + std::sqrt(1.0 + zeta * zeta));
                const double c = 1.0 / std::sqrt(1.0 + t * t), s = c * t;
                double *vp = &Vt[p * n], *vq = &Vt[q * n];
                for (size_t i = 0; i < n; ++i) {
                    const double a = up[i], b = uq[i];
                    up[i] = c * a - s * b;
                    uq[i] = s * a + c * b;
                    const double d = vp[i], e = vq[i];
                    vp[i] = c * d - s * e;
                    vq[i] = s * d + c * e;
                }
            }
        if (off < 1e-15) break;
    }
    for (size_t j = 0; j < n; ++j) {
        double s = 0;
        for (size_t i = 0; i < n; ++i) s += Ut[j * n + i] * Ut[j * n + i];
        sv[j] = s = std::sqrt(s);
        if (s > 0)
            for (size_t i = 0; i < n; ++i) Ut[j * n + i] /= s;
    }
    complete_null_columns(Ut, Vt, sv, n);
    product_v_ut(Vt, Ut, n, R);
}

}  // namespace vqh
