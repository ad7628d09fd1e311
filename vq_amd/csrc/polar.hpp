// The rotation update of OPQ, R = V U^T for A = U S V^T (src/opq.rs:180-183), without an SVD: R is the
// orthogonal polar factor of A^T, and for a non-singular A that factor is unique, so any convergent
// method gives the same matrix as the SVD does.  Newton-Schulz iteration on X_0 = A^T / s,
//     X_{k+1} = X_k (3 I - X_k^T X_k) / 2,
// converges to it when every singular value of X_0 lies in (0, sqrt 3): s = min(|A|_F, sqrt(|A|_1
// |A|_inf)) >= |A|_2 puts them in (0, 1].  A singular value sigma grows by 1.5 per step while it is
// small and converges quadratically once it is near 1: about log_1.5(cond) + 6 steps.  Scaled steps
// shorten the first phase: with every singular value in [l, 1], X (1.5 rho I - 0.5 rho^3 X^T X) with
// rho = sqrt(3 / (1 + l + l^2)) maps both ends of that interval to the same new lower bound
// l' = rho l (3 - rho^2 l^2) / 2 and everything between them into [l', 1] — small values grow by up to
// 2.6 per step.  l starts from a guess (1e-3 after the first, plain step); the map is valid for every
// singular value in (0, 1] whatever l is, so a wrong guess costs steps, never correctness.  The host
// passes rho_s with each step: the sequence that follows from the guess, then 1 (plain steps, which
// converge quadratically to the exact factor).  A matrix whose first error is below 0.005 is within
// 0.64 of orthogonal in the 2-norm (128 x the largest entry bounds it), so every singular value is
// above 0.6 already: it takes plain steps only — a scaled step would first spread them out.  A step is ONE launch (what a step costs is mostly the launch): a workgroup
// owns a strip of 16 columns; its waves first make the strip of G = X^T X, one 16 x 16 tile each, in
// f64 on the matrix cores (v_mfma_f64_16x16x4_f64), leave M = 1.5 I - 0.5 G for the strip in LDS, meet,
// and then make their tiles of the strip of X M (the operands sit in L2; every operand of a tile is
// fetched before its first matrix instruction).  The first half also gives err_k = max |X_k^T X_k - I|;
// once it is below 1e-7 the update that follows squares it to rounding level and is the last one: the
// kernel of step s + 1 sees errs[s], returns at once and sets fin[s + 2], which the kernels after it
// read (the host has already enqueued them).  A matrix that has not
// converged within the step limit (singular or badly conditioned: cond above about 1e6) goes to the
// Jacobi SVD, which also completes the directions a singular A leaves open.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vq {

constexpr int kPolarMaxSteps = 56;
constexpr int kPolarMaxDim = 512;
constexpr double kPolarLastStepErr = 1e-7;
constexpr double kPolarPlainBelow = 0.005;  // no scaled steps at all when the first error is below this

typedef double polar_d4 __attribute__((ext_vector_type(4)));

// One 16 x 16 tile of a product over KS steps of four k: lane l supplies, per step,
// A[i = l % 16][k = 4 u + l / 16] and B[k = 4 u + l / 16][j = l % 16]; register v of lane l receives
// C[4 v + l / 16][l % 16].  Two chains of matrix instructions (even and odd steps), added at the end.
template <int KS> __device__ __forceinline__ polar_d4 polar_mfma(const double (&a)[KS], const double (&b)[KS]) {
    polar_d4 acc0 = {0.0, 0.0, 0.0, 0.0}, acc1 = {0.0, 0.0, 0.0, 0.0};
#pragma unroll
    for (int u = 0; u < KS; u += 2) {
        acc0 = __builtin_amdgcn_mfma_f64_16x16x4f64(a[u], b[u], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f64_16x16x4f64(a[u + 1], b[u + 1], acc1, 0, 0, 0);
    }
    return acc0 + acc1;
}

// The same for any P (a multiple of 16), 16 steps' operands in flight at a time.  pa / pb point at the
// lane's first operands; they move on by sa / sb doubles per step.
__device__ __forceinline__ polar_d4 polar_tile(const double *__restrict__ pa, size_t sa,
                                               const double *__restrict__ pb, size_t sb, int P) {
    polar_d4 acc = {0.0, 0.0, 0.0, 0.0};
    for (int k0 = 0; k0 < P; k0 += 64) {
        double a[16], b[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const bool in = k0 + 4 * u < P;
            const int kc = in ? k0 / 4 + u : P / 4 - 1;  // clamped: unconditional loads
            a[u] = pa[(size_t)kc * sa];
            b[u] = in ? pb[(size_t)kc * sb] : 0.0;
            a[u] = in ? a[u] : 0.0;
        }
        acc = acc + polar_mfma<16>(a, b);
    }
    return acc;
}

// Step s: Xout = Xin (1.5 r I - 0.5 r^3 Xin^T Xin) with r = rho when the error of step 0 was at
// least kPolarPlainBelow, else 1; errs[s] = max |Xin^T Xin - I| over the dim x dim block that holds
// data (NaN counts as infinite).  P x P matrices, row-major, zero beyond dim.  Grid: P / 16
// workgroups (column strips) of min(P / 16, 8) waves; dynamic LDS: P * 16 doubles.
// PT = P / 16 when that is at most 8 (every operand of a tile fetched at once, and the rows of Xin
// for the second half already on their way during the first), 0: any P.
template <int PT>
static __global__ void __launch_bounds__(512) k_polar_step(const double *__restrict__ Xin, int P, int dim, int s,
                                                           double rho, unsigned long long *__restrict__ errs,
                                                           int *__restrict__ fin, double *__restrict__ Xout) {
    extern __shared__ __attribute__((aligned(16))) double m_strip[];  // M[c][16 tj + jj] at [c * 16 + jj]
    const double prev = s > 0 ? __longlong_as_double((long long)errs[s - 1]) : 2.0;
    const bool dead = fin[s] != 0 || prev < kPolarLastStepErr;
    if (dead) {  // the same in every workgroup
        if (blockIdx.x == 0 && threadIdx.x == 0) fin[s + 1] = 1;
        return;
    }
    const double first = s > 0 ? __longlong_as_double((long long)errs[0]) : 0.0;
    const double r = first >= kPolarPlainBelow ? rho : 1.0;
    const double ca = 1.5 * r, cb = 0.5 * r * r * r;
    const int nt = P / 16, tj = blockIdx.x;
    const int lane = threadIdx.x & 63, kk = lane >> 4, jj = lane & 15;
    const int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
    double e = 0.0;
    auto emit = [&](const polar_d4 &acc, int ti) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int i = 16 * ti + 4 * v + kk, j = 16 * tj + jj;
            const double d = i == j ? 1.0 : 0.0, g = acc[v];
            m_strip[i * 16 + jj] = ca * d - cb * g;
            if (i < dim && j < dim) {
                const double dev = fabs(g - d);
                e = (dev <= e) ? e : (dev == dev ? dev : __builtin_inf());
            }
        }
    };
    if constexpr (PT > 0) {
        constexpr int KS = 4 * PT, PP = 16 * PT;
        const int ti = w;  // one tile per wave
        // G[i][j] = sum_r X[r][i] X[r][j]: both operands run down a column of X, four rows per step
        double a[KS], b[KS], a2[KS];
        const double *pa = Xin + (size_t)kk * PP + 16 * ti + jj, *pb = Xin + (size_t)kk * PP + 16 * tj + jj;
#pragma unroll
        for (int u = 0; u < KS; ++u) {
            a[u] = pa[(size_t)u * 4 * PP];
            b[u] = pb[(size_t)u * 4 * PP];
        }
        // the second half's rows of Xin: Xout[r][j] = sum_c Xin[r][c] M[c][j], A runs along a row
        const double *pr = Xin + (size_t)(16 * ti + jj) * PP + kk;
#pragma unroll
        for (int u = 0; u < KS; ++u) a2[u] = pr[4 * u];
        emit(polar_mfma<KS>(a, b), ti);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const double o = __shfl_xor(e, off);
            e = o > e ? o : e;
        }
        // non-negative doubles order like their bit patterns
        if (lane == 0) atomicMax(errs + s, (unsigned long long)__double_as_longlong(e));
        __syncthreads();
#pragma unroll
        for (int u = 0; u < KS; ++u) b[u] = m_strip[(4 * u + kk) * 16 + jj];
        const polar_d4 acc = polar_mfma<KS>(a2, b);
#pragma unroll
        for (int v = 0; v < 4; ++v) Xout[(size_t)(16 * ti + 4 * v + kk) * PP + 16 * tj + jj] = acc[v];
    } else {
        for (int ti = w; ti < nt; ti += nw)
            emit(polar_tile(Xin + (size_t)kk * P + 16 * ti + jj, 4 * (size_t)P, Xin + (size_t)kk * P + 16 * tj + jj,
                            4 * (size_t)P, P),
                 ti);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const double o = __shfl_xor(e, off);
            e = o > e ? o : e;
        }
        if (lane == 0) atomicMax(errs + s, (unsigned long long)__double_as_longlong(e));
        __syncthreads();
        for (int ti = w; ti < nt; ti += nw) {
            const polar_d4 acc = polar_tile(Xin + (size_t)(16 * ti + jj) * P + kk, 4, m_strip + kk * 16 + jj, 64, P);
#pragma unroll
            for (int v = 0; v < 4; ++v) Xout[(size_t)(16 * ti + 4 * v + kk) * P + 16 * tj + jj] = acc[v];
        }
    }
}

}  // namespace vq
