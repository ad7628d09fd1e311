// Kernels around the assignment for the residual and the optimized product quantizer:
// residual update and norms (src/rvq.rs:111-141,200-207), rotation y = R x
// (src/opq.rs:186-194,232-234) and the cross-covariance A = Y X^T (src/opq.rs:172-179).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vq {

// res[i] -= codebook[code[i]]   (src/rvq.rs:127).  One lane per element.
static __global__ void __launch_bounds__(256) k_residual_sub(float *__restrict__ res, int64_t n, int64_t ld,
                                                      int dim, const float *__restrict__ cb,
                                                      const uint8_t *__restrict__ codes,
                                                      int code_stride) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n * dim) return;
    int64_t row = i / dim;
    int t = (int)(i % dim);
    float *p = res + row * ld + t;
    *p = *p - cb[(size_t)codes[row * code_stride] * dim + t];
}

// The same, four components per lane (dim and ld multiples of 4, 16-byte aligned pointers); a
// workgroup covers 1024 consecutive float4 of the n x dim/4 grid.  active == nullptr: every row.
// codes_out / used (both or neither): RVQ encode bookkeeping of the stage, written by the lane
// that holds a row's first components (src/rvq.rs:196-202).
static __global__ void __launch_bounds__(256) k_residual_sub4(float *__restrict__ res, int64_t n, int64_t ld,
                                                       int dim4, const float *__restrict__ cb,
                                                       const uint8_t *__restrict__ codes,
                                                       const uint8_t *__restrict__ active,
                                                       uint8_t *__restrict__ codes_out, int stages, int stage,
                                                       uint8_t *__restrict__ used) {
    const int64_t first = (int64_t)blockIdx.x * 1024;
    const int64_t row0 = first / dim4;            // uniform
    const uint32_t rem0 = (uint32_t)(first % dim4);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const uint32_t local = rem0 + threadIdx.x + 256u * u;
        const int64_t row = row0 + local / (uint32_t)dim4;
        const uint32_t t4 = local % (uint32_t)dim4;
        if (row >= n) continue;
        const bool on = active ? active[row] != 0 : true;
        const uint32_t code = on ? codes[row] : 0u;
        if (codes_out && t4 == 0) {
            codes_out[row * stages + stage] = (uint8_t)code;
            if (on) used[row] = (uint8_t)(stage + 1);
        }
        if (!on) continue;
        float4 *p = reinterpret_cast<float4 *>(res + row * ld) + t4;
        const float4 c = reinterpret_cast<const float4 *>(cb + (size_t)code * dim4 * 4)[t4];
        float4 v = *p;
        v.x = v.x - c.x;
        v.y = v.y - c.y;
        v.z = v.z - c.z;
        v.w = v.w - c.w;
        *p = v;
    }
}

// norms[i] = sqrt(sum_t x[i][t]^2), sequential f32 order (src/rvq.rs:134-135).
// One wave = 64 rows.  The rows are read coalesced, 64 columns at a time, into a padded LDS tile;
// each lane then walks its own row of the tile, so the per-row sum stays one sequential chain.
static __global__ void __launch_bounds__(64) k_row_norms(const float *__restrict__ x, int64_t n, int64_t ld,
                                                   int dim, float *__restrict__ norms) {
    __shared__ float tile[64][65];
    const int lane = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.x * 64;
    const int64_t last = n - 1;
    float acc = 0.0f;
    for (int c0 = 0; c0 < dim; c0 += 64) {
        const int w = (dim - c0 < 64) ? (dim - c0) : 64;
        // Loads are unconditional (clamped to the last row and column, the surplus is never
        // summed) and issued sixteen at a time: under a branch each one would be waited for.
        const int col = c0 + (lane < w ? lane : w - 1);
        __syncthreads();
        for (int r0 = 0; r0 < 64; r0 += 16) {
            float v[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t row = row0 + r0 + r;
                v[r] = x[(row < n ? row : last) * ld + col];
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) tile[r0 + r][lane] = v[r];
        }
        __syncthreads();
        for (int t = 0; t < w; ++t) {
            float v = tile[lane][t];
            float q = v * v;
            acc = acc + q;
        }
    }
    if (row0 + lane < n) norms[row0 + lane] = sqrtf(acc);
}

// Fixed-shape two-level sum of n floats in f64: every workgroup sums a contiguous slice with a
// fixed intra-group tree; a second launch of one workgroup sums the partials the same way.
static __global__ void __launch_bounds__(256) k_sum_f64(const float *__restrict__ in_f32,
                                                 const double *__restrict__ in_f64, int64_t n,
                                                 int64_t per_block, double *__restrict__ out) {
    __shared__ double sh[256];
    int64_t lo = (int64_t)blockIdx.x * per_block;
    int64_t hi = lo + per_block < n ? lo + per_block : n;
    double acc = 0.0;
    for (int64_t i = lo + threadIdx.x; i < hi; i += 256) acc += in_f32 ? (double)in_f32[i] : in_f64[i];
    sh[threadIdx.x] = acc;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) sh[threadIdx.x] += sh[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[blockIdx.x] = sh[0];
}

// One stage of ResidualQuantizer::quantize for every row still active (src/rvq.rs:200-202), the
// residual's half: residual -= c; the stage's code and the number of stages used are recorded.
// The other half (sum += c) is replayed from the codes by k_rvq_recon_f16.  One lane per element.
static __global__ void __launch_bounds__(256) k_rvq_stage_apply(float *__restrict__ res, int64_t n, int dim,
                                                         const float *__restrict__ cb,
                                                         const uint8_t *__restrict__ stage_codes,
                                                         uint8_t *__restrict__ codes_out, int stages,
                                                         int stage, const uint8_t *__restrict__ active,
                                                         uint8_t *__restrict__ used) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n * dim) return;
    const int64_t row = i / dim;
    const int t = (int)(i % dim);
    const bool on = active[row] != 0;
    const int code = on ? stage_codes[row] : 0;
    if (t == 0) {
        codes_out[row * stages + stage] = (uint8_t)code;
        if (on) used[row] = (uint8_t)(stage + 1);
    }
    if (!on) return;
    res[i] = res[i] - cb[(size_t)code * dim + t];
}

// The reconstruction of ResidualQuantizer::quantize from the codes: sum = 0; for every stage the
// row used, in order, sum = sum + c (src/rvq.rs:183,201); then f16 (src/rvq.rs:212).  One lane
// per element; the codebooks (stages x k x dim) stay in L2.
static __global__ void __launch_bounds__(256) k_rvq_recon_f16(int64_t n, int dim, int k,
                                                       const float *__restrict__ codebooks,
                                                       const uint8_t *__restrict__ codes, int stages,
                                                       const uint8_t *__restrict__ used,
                                                       uint16_t *__restrict__ out) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n * dim) return;
    const int64_t row = i / dim;
    const int t = (int)(i % dim);
    const int nst = used[row];
    float sum = 0.0f;
    for (int st = 0; st < nst; ++st)
        sum = sum + codebooks[((size_t)st * k + codes[row * stages + st]) * dim + t];
    out[i] = __half_as_ushort(__float2half_rn(sum));
}

// The same, four components per lane (dim a multiple of 4, 16-byte aligned codebooks, 8-byte
// aligned output).
static __global__ void __launch_bounds__(256) k_rvq_recon4_f16(int64_t n, int dim4, int k,
                                                        const float *__restrict__ codebooks,
                                                        const uint8_t *__restrict__ codes, int stages,
                                                        const uint8_t *__restrict__ used,
                                                        uint16_t *__restrict__ out) {
    const int64_t first = (int64_t)blockIdx.x * 1024;
    const int64_t row0 = first / dim4;
    const uint32_t rem0 = (uint32_t)(first % dim4);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const uint32_t local = rem0 + threadIdx.x + 256u * u;
        const int64_t row = row0 + local / (uint32_t)dim4;
        const uint32_t t4 = local % (uint32_t)dim4;
        if (row >= n) continue;
        const int nst = used[row];
        float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int st = 0; st < nst; ++st) {
            const float4 c =
                reinterpret_cast<const float4 *>(codebooks + ((size_t)st * k + codes[row * stages + st]) * dim4 * 4)[t4];
            sum.x = sum.x + c.x;
            sum.y = sum.y + c.y;
            sum.z = sum.z + c.z;
            sum.w = sum.w + c.w;
        }
        uint2 h;
        h.x = (uint32_t)__half_as_ushort(__float2half_rn(sum.x)) | ((uint32_t)__half_as_ushort(__float2half_rn(sum.y)) << 16);
        h.y = (uint32_t)__half_as_ushort(__float2half_rn(sum.z)) | ((uint32_t)__half_as_ushort(__float2half_rn(sum.w)) << 16);
        reinterpret_cast<uint2 *>(out + row * (int64_t)dim4 * 4)[t4] = h;
    }
}

// The row stops when ||residual|| < epsilon (src/rvq.rs:204-207).
static __global__ void __launch_bounds__(256) k_rvq_stage_stop(const float *__restrict__ norms, int64_t n,
                                                        float epsilon, uint8_t *__restrict__ active) {
    int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row < n && active[row] && norms[row] < epsilon) active[row] = 0;
}

static __global__ void __launch_bounds__(256) k_fill_u8(uint8_t *__restrict__ p, int64_t count, uint8_t v) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) p[i] = v;
}

// ---- rotation ------------------------------------------------------------------------------
// y[i][a] = sum_b R[a][b] * x[i][b].  Generic dimension: one workgroup = 64 rows, x tile and
// (a slab of) R staged in LDS, fused multiply-add accumulation in ascending b.
static __global__ void __launch_bounds__(256) k_rotate_generic(const float *__restrict__ x, int64_t n,
                                                        int64_t ld, int dim,
                                                        const float *__restrict__ R,
                                                        float *__restrict__ y) {
    extern __shared__ float lds[];  // 64 * (dim + 1) floats of x
    const int stride = dim + 1;
    const int64_t row0 = (int64_t)blockIdx.x * 64;
    for (int i = threadIdx.x; i < 64 * dim; i += 256) {
        int r = i / dim, t = i % dim;
        int64_t row = row0 + r;
        lds[r * stride + t] = row < n ? x[row * ld + t] : 0.0f;
    }
    __syncthreads();
    // thread -> (row r = tid % 64, outputs a = tid / 64, +4, +8, ...)
    const int r = threadIdx.x % 64;
    const int64_t row = row0 + r;
    for (int a = threadIdx.x / 64; a < dim; a += 4) {
        const float *Ra = R + (size_t)a * dim;  // wave-uniform
        float acc = 0.0f;
        for (int b = 0; b < dim; ++b) acc = __builtin_fmaf(Ra[b], lds[r * stride + b], acc);
        if (row < n) y[row * dim + a] = acc;
    }
}

// ---- cross-covariance ----------------------------------------------------------------------
// part[c][a][b] = sum over the rows of chunk c of yr[i][a] * x[i][b], accumulated in f64 in row
// order; chunks are combined in chunk order by k_crosscov_reduce.  Generic dimension.
static __global__ void __launch_bounds__(256) k_crosscov_partial(const float *__restrict__ yr,
                                                          const float *__restrict__ x, int64_t n,
                                                          int dim, int64_t rows_per_chunk,
                                                          double *__restrict__ part) {
    extern __shared__ float lds[];  // 2 * 32 * dim floats
    float *ly = lds, *lx = lds + 32 * dim;
    const int64_t lo = (int64_t)blockIdx.x * rows_per_chunk;
    const int64_t hi = lo + rows_per_chunk < n ? lo + rows_per_chunk : n;
    const int total = dim * dim;
    // each thread owns outputs e = tid, tid+256, ... (at most 64 per thread: dim <= 128)
    double acc[64];
#pragma unroll
    for (int u = 0; u < 64; ++u) acc[u] = 0.0;
    for (int64_t r0 = lo; r0 < hi; r0 += 32) {
        int rows = (int)((hi - r0) < 32 ? (hi - r0) : 32);
        __syncthreads();
        for (int i = threadIdx.x; i < rows * dim; i += 256) {
            ly[i] = yr[r0 * dim + i];
            lx[i] = x[r0 * dim + i];
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < 64; ++u) {
            int e = threadIdx.x + u * 256;
            if (e < total) {
                int a = e / dim, b = e % dim;
                double s = acc[u];
                for (int r = 0; r < rows; ++r) s += (double)ly[r * dim + a] * (double)lx[r * dim + b];
                acc[u] = s;
            }
        }
    }
    double *out = part + (size_t)blockIdx.x * total;
#pragma unroll
    for (int u = 0; u < 64; ++u) {
        int e = threadIdx.x + u * 256;
        if (e < total) out[e] = acc[u];
    }
}

// The same partial sums on the f64 matrix cores (v_mfma_f64_16x16x4_f64) for dim = 16 * NT <= 128.
// One wave owns the 16 output rows [16 ti, 16 ti + 16) of a chunk and all NT column tiles; a
// contraction step takes 4 rows: lane l supplies y[row + l/16][16 ti + l%16] and, per column
// tile, x[row + l/16][16 tj + l%16], converted to f64 (the products are then exact).  The result
// register v of lane l is A[16 ti + 4 v + l/16][16 tj + l%16].  Fixed order: deterministic.
typedef double doublex4 __attribute__((ext_vector_type(4)));

template <int NT>
__global__ void __launch_bounds__(256) k_crosscov_mfma(const float *__restrict__ yr, const float *__restrict__ x,
                                                       int64_t n, int64_t rows_per_chunk,
                                                       double *__restrict__ part) {
    constexpr int DIM = 16 * NT;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int ti = blockIdx.y * 4 + w;
    if (ti >= NT) return;
    const int kk = lane >> 4, jj = lane & 15;
    const int64_t lo = (int64_t)blockIdx.x * rows_per_chunk;
    const int64_t hi = lo + rows_per_chunk < n ? lo + rows_per_chunk : n;
    doublex4 acc[NT];
#pragma unroll
    for (int tj = 0; tj < NT; ++tj) acc[tj] = doublex4{0.0, 0.0, 0.0, 0.0};
    const float *yp = yr + (lo + kk) * DIM + 16 * ti + jj;
    const float *xp = x + (lo + kk) * DIM + jj;
    float a = 0.0f, b[NT];
    bool valid = lo + kk < hi;
    a = valid ? *yp : 0.0f;
#pragma unroll
    for (int tj = 0; tj < NT; ++tj) b[tj] = valid ? xp[16 * tj] : 0.0f;
    for (int64_t r = lo; r < hi; r += 4) {
        const float ac = a;
        float bc[NT];
#pragma unroll
        for (int tj = 0; tj < NT; ++tj) bc[tj] = b[tj];
        yp += 4 * DIM;
        xp += 4 * DIM;
        valid = r + 4 + kk < hi;  // the next step's operands are fetched while this one is multiplied
        a = valid ? *yp : 0.0f;
#pragma unroll
        for (int tj = 0; tj < NT; ++tj) b[tj] = valid ? xp[16 * tj] : 0.0f;
#pragma unroll
        for (int tj = 0; tj < NT; ++tj)
            acc[tj] = __builtin_amdgcn_mfma_f64_16x16x4f64((double)ac, (double)bc[tj], acc[tj], 0, 0, 0);
    }
    double *out = part + (size_t)blockIdx.x * DIM * DIM;
#pragma unroll
    for (int tj = 0; tj < NT; ++tj)
#pragma unroll
        for (int v = 0; v < 4; ++v) out[(size_t)(16 * ti + 4 * v + kk) * DIM + 16 * tj + jj] = acc[tj][v];
}

static __global__ void __launch_bounds__(256) k_crosscov_reduce(const double *__restrict__ part, int chunks,
                                                         int total, double *__restrict__ out) {
    int e = blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    double s = 0.0;
    for (int c = 0; c < chunks; ++c) s += part[(size_t)c * total + e];
    out[e] = s;
}

}  // namespace vq

// ---- rotation on the matrix cores ------------------------------------------------------------
// y[i][a] = sum_b R[a][b] * x[i][b] for dim a multiple of 32, at most 256: D = R * X^T in tiles of
// 32 output dimensions x 32 rows with v_mfma_f32_32x32x2_f32 (fp32 in, fp32 accumulate).
namespace vq {

typedef float rot_floatx16 __attribute__((ext_vector_type(16)));

// rtab[kc][b][lane][u] = R[32 b + lane % 32][8 kc + 4 (lane / 32) + u]   (MFMA A-operand order)
static __global__ void __launch_bounds__(256) k_rotate_prep(const float *__restrict__ R, int dim,
                                                            float *__restrict__ rtab) {
    const int nb = dim / 32, nkc = dim / 8;
    const int total = nkc * nb * 64 * 4;
    for (int e = blockIdx.x * 256 + threadIdx.x; e < total; e += gridDim.x * 256) {
        const int u = e % 4, lane = (e / 4) % 64, b = (e / 256) % nb, kc = e / (256 * nb);
        rtab[e] = R[(size_t)(32 * b + lane % 32) * dim + 8 * kc + 4 * (lane / 32) + u];
    }
}

// grid ceil(n/128); 256 threads = 4 waves, one tile of 32 rows per wave.
static __global__ void __launch_bounds__(256) k_rotate_mfma(const float *__restrict__ x, int64_t n, int64_t ld,
                                                            int dim, const float *__restrict__ rtab,
                                                            float *__restrict__ y) {
    constexpr int NBMAX = 8;
    __shared__ float4 lds_a[2][NBMAX * 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int nb = dim / 32, nkc = dim / 8;
    const int64_t row = ((int64_t)blockIdx.x * 4 + wave) * 32 + r;
    const bool valid = row < n;
    const float4 *ag = reinterpret_cast<const float4 *>(rtab);
    const int chunk4 = nb * 64;
    for (int i = threadIdx.x; i < chunk4; i += 256) lds_a[0][i] = ag[i];
    __syncthreads();
    rot_floatx16 acc[NBMAX];
#pragma unroll
    for (int b = 0; b < NBMAX; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[b][v] = 0.0f;
    const float *xr = x + (valid ? row : 0) * ld + 4 * h;
    for (int kc = 0; kc < nkc; ++kc) {
        const int cur = kc & 1;
        float4 pre[2];
        const bool more = kc + 1 < nkc;
        if (more) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                int i = threadIdx.x + 256 * q;
                if (i < chunk4) pre[q] = ag[(size_t)(kc + 1) * chunk4 + i];
            }
        }
        float4 xv = make_float4(0.f, 0.f, 0.f, 0.f);
        if (valid) xv = *reinterpret_cast<const float4 *>(xr + kc * 8);
#pragma unroll
        for (int b = 0; b < NBMAX; ++b) {
            if (b < nb) {
                const float4 av = lds_a[cur][b * 64 + lane];
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.x, xv.x, acc[b], 0, 0, 0);
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.y, xv.y, acc[b], 0, 0, 0);
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.z, xv.z, acc[b], 0, 0, 0);
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.w, xv.w, acc[b], 0, 0, 0);
            }
        }
        if (more) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                int i = threadIdx.x + 256 * q;
                if (i < chunk4) lds_a[cur ^ 1][i] = pre[q];
            }
        }
        __syncthreads();
    }
    if (!valid) return;
    // register v of block b holds output dimension 32 b + 8 (v / 4) + 4 h + v % 4 of this lane's row
    float *yr = y + row * dim + 4 * h;
#pragma unroll
    for (int b = 0; b < NBMAX; ++b) {
        if (b < nb) {
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<float4 *>(yr + 32 * b + 8 * g) =
                    make_float4(acc[b][4 * g], acc[b][4 * g + 1], acc[b][4 * g + 2], acc[b][4 * g + 3]);
        }
    }
}

}  // namespace vq
