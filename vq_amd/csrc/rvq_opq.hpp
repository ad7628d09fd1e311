// Kernels around the assignment for the residual and the optimized product quantizer:
// residual update and norms (src/rvq.rs:111-141,200-207), rotation y = R x
// (src/opq.rs:186-194,232-234) and the cross-covariance A = Y X^T (src/opq.rs:172-179).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vq {

// res[i] -= codebook[code[i]]   (src/rvq.rs:127).  One lane per element.
template <typename CodeT>
static __global__ void __launch_bounds__(256) k_residual_sub(float *__restrict__ res, int64_t n, int64_t ld,
                                                      int dim, const float *__restrict__ cb,
                                                      const CodeT *__restrict__ codes,
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
// that holds a row's first components (src/rvq.rs:196-202).  The rows are read from src (row
// stride src_ld floats) and written to res: the same buffer for an update in place, or the
// caller's rows for the first stage of an encode, whose inactive rows do not occur.
template <typename CodeT>
static __global__ void __launch_bounds__(256) k_residual_sub4(float *res, int64_t n, int64_t ld, int dim4,
                                                       const float *__restrict__ cb,
                                                       const CodeT *__restrict__ codes,
                                                       const uint8_t *__restrict__ active,
                                                       CodeT *__restrict__ codes_out, int stages, int stage,
                                                       uint8_t *__restrict__ used, const float *src,
                                                       int64_t src_ld) {
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
            codes_out[row * stages + stage] = (CodeT)code;
            if (on) used[row] = (uint8_t)(stage + 1);
        }
        if (!on) continue;
        float4 *p = reinterpret_cast<float4 *>(res + row * ld) + t4;
        const float4 c = reinterpret_cast<const float4 *>(cb + (size_t)code * dim4 * 4)[t4];
        float4 v = reinterpret_cast<const float4 *>(src + row * src_ld)[t4];
        v.x = v.x - c.x;
        v.y = v.y - c.y;
        v.z = v.z - c.z;
        v.w = v.w - c.w;
        *p = v;
    }
}

// The bookkeeping of an encode's last stage alone: nothing reads the residual after it
// (src/rvq.rs:200-206: the norm test of the last stage only ends a loop that is over).
template <typename CodeT>
static __global__ void __launch_bounds__(256) k_rvq_stage_record(int64_t n, const CodeT *__restrict__ stage_codes,
                                                          const uint8_t *__restrict__ active,
                                                          CodeT *__restrict__ codes_out, int stages, int stage,
                                                          uint8_t *__restrict__ used) {
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= n) return;
    const bool on = active[row] != 0;
    codes_out[row * stages + stage] = on ? stage_codes[row] : (CodeT)0;
    if (on) used[row] = (uint8_t)(stage + 1);
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
template <typename CodeT>
static __global__ void __launch_bounds__(256) k_rvq_stage_apply(float *__restrict__ res, int64_t n, int dim,
                                                         const float *__restrict__ cb,
                                                         const CodeT *__restrict__ stage_codes,
                                                         CodeT *__restrict__ codes_out, int stages,
                                                         int stage, const uint8_t *__restrict__ active,
                                                         uint8_t *__restrict__ used) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n * dim) return;
    const int64_t row = i / dim;
    const int t = (int)(i % dim);
    const bool on = active[row] != 0;
    const int code = on ? stage_codes[row] : 0;
    if (t == 0) {
        codes_out[row * stages + stage] = (CodeT)code;
        if (on) used[row] = (uint8_t)(stage + 1);
    }
    if (!on) return;
    res[i] = res[i] - cb[(size_t)code * dim + t];
}

// The reconstruction of ResidualQuantizer::quantize from the codes: sum = 0; for every stage the
// row used, in order, sum = sum + c (src/rvq.rs:183,201); then f16 (src/rvq.rs:212).  One lane
// per element; the codebooks (stages x k x dim) stay in L2.
template <typename CodeT>
static __global__ void __launch_bounds__(256) k_rvq_recon_f16(int64_t n, int dim, int k,
                                                       const float *__restrict__ codebooks,
                                                       const CodeT *__restrict__ codes, int stages,
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
template <typename CodeT>
static __global__ void __launch_bounds__(256) k_rvq_recon4_f16(int64_t n, int dim4, int k,
                                                        const float *__restrict__ codebooks,
                                                        const CodeT *__restrict__ codes, int stages,
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

template <typename T>
static __global__ void __launch_bounds__(256) k_fill(T *__restrict__ p, int64_t count, T v) {
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
// order; chunks are combined in chunk order by k_crosscov_reduce.  Generic dimension: a workgroup
// takes one tile of up to 128 x 128 outputs of one chunk (grid.y walks the tiles row by row).
static __global__ void __launch_bounds__(256) k_crosscov_partial(const float *__restrict__ yr,
                                                          const float *__restrict__ x, int64_t n,
                                                          int dim, int64_t rows_per_chunk,
                                                          double *__restrict__ part) {
    __shared__ float ly[32 * 128], lx[32 * 128];
    const int tiles = (dim + 127) / 128;
    const int a0 = (int)(blockIdx.y / tiles) * 128, b0 = (int)(blockIdx.y % tiles) * 128;
    const int da = dim - a0 < 128 ? dim - a0 : 128, db = dim - b0 < 128 ? dim - b0 : 128;
    const int64_t lo = (int64_t)blockIdx.x * rows_per_chunk;
    const int64_t hi = lo + rows_per_chunk < n ? lo + rows_per_chunk : n;
    const int total = da * db;
    // each thread owns outputs e = tid, tid+256, ... of the tile (at most 64 per thread)
    double acc[64];
#pragma unroll
    for (int u = 0; u < 64; ++u) acc[u] = 0.0;
    for (int64_t r0 = lo; r0 < hi; r0 += 32) {
        int rows = (int)((hi - r0) < 32 ? (hi - r0) : 32);
        __syncthreads();
        for (int i = threadIdx.x; i < rows * da; i += 256) ly[i] = yr[(r0 + i / da) * dim + a0 + i % da];
        for (int i = threadIdx.x; i < rows * db; i += 256) lx[i] = x[(r0 + i / db) * dim + b0 + i % db];
        __syncthreads();
#pragma unroll
        for (int u = 0; u < 64; ++u) {
            int e = threadIdx.x + u * 256;
            if (e < total) {
                int a = e / db, b = e % db;
                double s = acc[u];
#pragma unroll 1
                for (int r = 0; r < rows; ++r) s += (double)ly[r * da + a] * (double)lx[r * db + b];
                acc[u] = s;
            }
        }
    }
    double *out = part + (size_t)blockIdx.x * dim * dim;
#pragma unroll
    for (int u = 0; u < 64; ++u) {
        int e = threadIdx.x + u * 256;
        if (e < total) out[(size_t)(a0 + e / db) * dim + b0 + e % db] = acc[u];
    }
}

// The same partial sums on the f64 matrix cores (v_mfma_f64_16x16x4_f64) for dim a multiple of 16:
// a launch covers the output columns [b0 + 128 z, b0 + 128 z + 16 NT) for z = blockIdx.z and every
// output row.
// One wave owns the 32 output rows [16 ti, 16 ti + 32) of a chunk and NT column tiles; a
// contraction step takes 4 rows: lane l supplies y[row + l/16][16 ti + l%16] and, per column
// tile, x[row + l/16][16 tj + l%16], converted to f64 (the products are then exact).  The result
// register v of lane l is A[16 ti + 4 v + l/16][16 tj + l%16].  Fixed order: deterministic.
typedef double doublex4 __attribute__((ext_vector_type(4)));

template <int NT>
__global__ void __launch_bounds__(256) k_crosscov_mfma(const float *__restrict__ yr, const float *__restrict__ x,
                                                       int64_t n, int DIM, int b0, int64_t rows_per_chunk,
                                                       double *__restrict__ part) {
    // a wave owns TWO tiles of 16 output rows (32 dimensions of y), so every operand of x it
    // fetches feeds two matrix instructions
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ti = 2 * (blockIdx.y * 4 + w), nti = DIM / 16;
    if (ti >= nti) return;
    const bool two = ti + 1 < nti;  // without a second tile acc1 repeats acc0 and is not stored
    b0 += 128 * blockIdx.z;
    const int kk = lane >> 4, jj = lane & 15;
    const int64_t lo = (int64_t)blockIdx.x * rows_per_chunk;
    const int64_t hi = lo + rows_per_chunk < n ? lo + rows_per_chunk : n;
    doublex4 acc0[NT], acc1[NT];
#pragma unroll
    for (int tj = 0; tj < NT; ++tj) {
        acc0[tj] = doublex4{0.0, 0.0, 0.0, 0.0};
        acc1[tj] = doublex4{0.0, 0.0, 0.0, 0.0};
    }
    // Addresses: a scalar base that moves on by four rows per step plus one fixed 32-bit lane
    // offset (and the column tile as the instruction's immediate), so the loop spends no vector
    // instruction on them; the vector ALU and the matrix cores take turns on a SIMD, and what the
    // loop still needs of the first is the conversions to f64.
    const int nsteps = (int)((hi - lo) / 4);  // steps in which every lane has a row
    const int tail = (int)((hi - lo) % 4);
    uint32_t lane_off = 4u * ((uint32_t)kk * (uint32_t)DIM + (uint32_t)jj);
    const int64_t stepb = 16 * (int64_t)DIM;
    const char *ybase = reinterpret_cast<const char *>(yr + lo * (int64_t)DIM + 16 * ti);
    const char *xbase = reinterpret_cast<const char *>(x + lo * (int64_t)DIM + b0);
    const int ysec = two ? 64 : 0;
    auto ldf = [](const char *base, uint32_t off, int imm) {
        return *reinterpret_cast<const float *>(base + (uint64_t)off + imm);
    };
    if (nsteps > 0) {
        // Operands are fetched kAhead steps ahead.  The loads are unconditional (a load under a
        // branch makes the compiler wait for every load in flight at its use): past the last
        // whole step they read that step again and the values are dropped.
        constexpr int kAhead = 4;
        float a0[kAhead], a1[kAhead], b[kAhead][NT];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int st = u < nsteps ? u : nsteps - 1;
            const char *yb = ybase + st * stepb, *xb = xbase + st * stepb;
            a0[u] = ldf(yb, lane_off, 0);
            a1[u] = ldf(yb + ysec, lane_off, 0);
#pragma unroll
            for (int tj = 0; tj < NT; ++tj) b[u][tj] = ldf(xb, lane_off, 64 * tj);
            // in step order: the loop waits for the oldest loads only
            __builtin_amdgcn_sched_barrier(0);
        }
        for (int i = 0; i < nsteps; i += kAhead) {
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                double ac0 = (double)a0[u], ac1 = (double)a1[u];
                double bc[NT];
#pragma unroll
                for (int tj = 0; tj < NT; ++tj) bc[tj] = (double)b[u][tj];
                // The conversions stay here (the empty statements pin them: a conversion moved
                // below the slot's next loads would need copies of the old values, and a wait for
                // them), so the slot's registers are free for those loads; and the lane offset
                // stays a 32-bit register beside a scalar base.
                asm volatile("" : "+v"(ac0), "+v"(ac1));
#pragma unroll
                for (int tj = 0; tj < NT; ++tj) asm volatile("" : "+v"(bc[tj]));
                asm volatile("" : "+v"(lane_off));
                const int nx = i + u + kAhead;  // the step this slot holds next
                const int st = nx < nsteps ? nx : nsteps - 1;
                const char *yb = ybase + st * stepb, *xb = xbase + st * stepb;
                a0[u] = ldf(yb, lane_off, 0);
                a1[u] = ldf(yb + ysec, lane_off, 0);
#pragma unroll
                for (int tj = 0; tj < NT; ++tj) b[u][tj] = ldf(xb, lane_off, 64 * tj);
                __builtin_amdgcn_sched_barrier(0);
                if (i + u < nsteps) {  // the same in every lane
#pragma unroll
                    for (int tj = 0; tj < NT; ++tj) {
                        acc0[tj] = __builtin_amdgcn_mfma_f64_16x16x4f64(ac0, bc[tj], acc0[tj], 0, 0, 0);
                        acc1[tj] = __builtin_amdgcn_mfma_f64_16x16x4f64(ac1, bc[tj], acc1[tj], 0, 0, 0);
                    }
                }
            }
        }
    }
    if (tail) {  // the chunk's last one to three rows: zeros in the lanes of the missing rows
        const bool ok = kk < tail;
        const char *yb = ybase + nsteps * stepb, *xb = xbase + nsteps * stepb;
        const uint32_t off = ok ? lane_off : 4u * (uint32_t)jj;
        const double ac0 = ok ? (double)ldf(yb, off, 0) : 0.0, ac1 = ok ? (double)ldf(yb + ysec, off, 0) : 0.0;
#pragma unroll
        for (int tj = 0; tj < NT; ++tj) {
            const double bc = ok ? (double)ldf(xb, off, 64 * tj) : 0.0;
            acc0[tj] = __builtin_amdgcn_mfma_f64_16x16x4f64(ac0, bc, acc0[tj], 0, 0, 0);
            acc1[tj] = __builtin_amdgcn_mfma_f64_16x16x4f64(ac1, bc, acc1[tj], 0, 0, 0);
        }
    }
    double *out = part + (size_t)blockIdx.x * DIM * DIM;
#pragma unroll
    for (int tj = 0; tj < NT; ++tj)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            out[(size_t)(16 * ti + 4 * v + kk) * DIM + b0 + 16 * tj + jj] = acc0[tj][v];
            if (two) out[(size_t)(16 * ti + 16 + 4 * v + kk) * DIM + b0 + 16 * tj + jj] = acc1[tj][v];
        }
}

// out[e] = sum over the chunks [g * per_group, (g + 1) * per_group) of part[c][e], c ascending, for
// group g = blockIdx.y: called once over the chunks (out = one sum per group) and once more over
// those sums, so the order of the additions is fixed (groups of chunks in chunk order, then the
// groups in group order) whatever the GPU does.  Sixteen loads in flight per thread.
static __global__ void __launch_bounds__(256) k_crosscov_reduce(const double *__restrict__ part, int chunks,
                                                         int per_group, int total, double *__restrict__ out) {
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    const int c0 = blockIdx.y * per_group, c1 = min(chunks, c0 + per_group);
    double s = 0.0;
    for (int c = c0; c < c1; c += 16) {
        double v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) v[u] = part[(size_t)min(c + u, c1 - 1) * total + e];
#pragma unroll
        for (int u = 0; u < 16; ++u)
            if (c + u < c1) s += v[u];
    }
    out[(size_t)blockIdx.y * total + e] = s;
}

}  // namespace vq

// ---- rotation on the matrix cores ------------------------------------------------------------
// y[i][a] = sum_b R[a][b] * x[i][b] for dim a multiple of 32, at most 256: D = R * X^T in tiles of
// 32 output dimensions x 32 rows on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16, 16x the rate
// of the fp32 instruction).  Every fp32 number is the exact sum of three bf16 numbers
// (v = h + m + l, round to nearest even three times: 3 x 8 significant bits), and the six
// products hh, hm, mh, mm, hl, lh are accumulated in fp32; the three left out (ml, lm, ll) are
// below 2^-23 of |R||x| each, so the result is as good as an fp32 fused-multiply-add chain, and a
// rotation by the identity returns the rows bit for bit.  With the matrix time at 0.08 ms for
// 1M x 128 the kernel is bound by the 1 GB it moves.
namespace vq {

typedef float rot_floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 rot_bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t rot_u32x4 __attribute__((ext_vector_type(4)));

// v -> (h, m, l) bf16 bit patterns, h + m + l == v
__device__ __forceinline__ void rot_split3(float v, uint32_t &h, uint32_t &m, uint32_t &l) {
    auto rne = [](float f) -> uint32_t {
        uint32_t u = __float_as_uint(f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
        u += 0x7fffu + ((u >> 16) & 1u);
        return u >> 16;
    };
    h = rne(v);
    const float r1 = v - __uint_as_float(h << 16);
    m = rne(r1);
    const float r2 = r1 - __uint_as_float(m << 16);
    l = rne(r2);
}

// two floats -> their (h, m, l) parts as packed bf16 pairs (low half = first), by the hardware's
// round-to-nearest-even conversion
typedef float rot_floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 rot_bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t rot_pack2(float a, float b) {
    rot_floatx2 f = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, rot_bf16x2));
}
__device__ __forceinline__ void rot_split3_pair(float a, float b, uint32_t &h, uint32_t &m, uint32_t &l) {
    h = rot_pack2(a, b);
    const float ra = a - __uint_as_float(h << 16), rb = b - __uint_as_float(h & 0xffff0000u);
    m = rot_pack2(ra, rb);
    l = rot_pack2(ra - __uint_as_float(m << 16), rb - __uint_as_float(m & 0xffff0000u));
}

// rtab[kc][b][e][lane] (16 bytes each), lane = 32 hh + o: the parts of R[32 b + o][8 kc + 4 hh + u],
// u = 0..3:  e = 0: {h01, h23, m01, m23}   e = 1: {h01, h23, l01, l23}
static __global__ void __launch_bounds__(256) k_rotate_prep(const float *__restrict__ R, int dim,
                                                            rot_u32x4 *__restrict__ rtab) {
    const int nb = dim / 32, nkc = dim / 8;
    const int total = nkc * nb * 64;
    for (int e = blockIdx.x * 256 + threadIdx.x; e < total; e += gridDim.x * 256) {
        const int lane = e % 64, b = (e / 64) % nb, kc = e / (64 * nb);
        const float *src = R + (size_t)(32 * b + lane % 32) * dim + 8 * kc + 4 * (lane / 32);
        uint32_t h[4], m[4], l[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) rot_split3(src[u], h[u], m[u], l[u]);
        const uint32_t h01 = h[0] | (h[1] << 16), h23 = h[2] | (h[3] << 16);
        rot_u32x4 *dst = rtab + ((size_t)kc * nb + b) * 128;
        dst[lane] = rot_u32x4{h01, h23, m[0] | (m[1] << 16), m[2] | (m[3] << 16)};
        dst[64 + lane] = rot_u32x4{h01, h23, l[0] | (l[1] << 16), l[2] | (l[3] << 16)};
    }
}

// grid ceil(n / (128 TILES)); 256 threads = 4 waves, TILES tiles of 32 rows per wave, NB = dim / 32.
// The operands of R for a chunk of 8 dimensions (NB x 2 KB) are staged in LDS by the workgroup,
// double-buffered behind a barrier that waits for LDS only; a lane's 16 bytes of a row and chunk
// are fetched kRotAhead chunks ahead and stay in flight across the barriers.
template <int NB, int TILES>
static __global__ void __launch_bounds__(256) k_rotate_mfma(const float *__restrict__ x, int64_t n, int64_t ld,
                                                            const rot_u32x4 *__restrict__ rtab,
                                                            float *__restrict__ y) {
    constexpr int DIM = 32 * NB, NKC = DIM / 8, CHUNK = NB * 128;  // u32x4 entries per chunk
    __shared__ rot_u32x4 lds_a[2][CHUNK];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    int64_t row[TILES];
    const float *xr[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        row[t] = (((int64_t)blockIdx.x * 4 + wave) * TILES + t) * 32 + r;
        xr[t] = x + (row[t] < n ? row[t] : 0) * ld + 4 * h;  // a row past the end reads row 0, never stored
    }
    for (int i = threadIdx.x; i < CHUNK; i += 256) lds_a[0][i] = rtab[i];
    __syncthreads();
    rot_floatx16 acc[TILES][NB];
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[t][b][v] = 0.0f;
    constexpr int kRotAhead = 4;  // NKC is a multiple of 4
    float4 xq[TILES][kRotAhead];
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int u = 0; u < kRotAhead; ++u) xq[t][u] = *reinterpret_cast<const float4 *>(xr[t] + u * 8);
    for (int kc0 = 0; kc0 < NKC; kc0 += kRotAhead) {
#pragma unroll
        for (int u = 0; u < kRotAhead; ++u) {
            const int kc = kc0 + u;
            const int cur = kc & 1;
            constexpr int PER = (CHUNK + 255) / 256;
            rot_u32x4 pre[PER];
            const bool more = kc + 1 < NKC;
            if (more) {
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    const int i = threadIdx.x + 256 * q;
                    if (i < CHUNK) pre[q] = rtab[(size_t)(kc + 1) * CHUNK + i];
                }
            }
            rot_u32x4 b1[TILES], b2[TILES], b3[TILES];
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                const float4 xv = xq[t][u];
                const int nx = kc + kRotAhead < NKC ? kc + kRotAhead : NKC - 1;
                xq[t][u] = *reinterpret_cast<const float4 *>(xr[t] + nx * 8);
                uint32_t h01, m01, l01, h23, m23, l23;
                rot_split3_pair(xv.x, xv.y, h01, m01, l01);
                rot_split3_pair(xv.z, xv.w, h23, m23, l23);
                b1[t] = rot_u32x4{h01, h23, h01, h23};
                b2[t] = rot_u32x4{m01, m23, m01, m23};
                b3[t] = rot_u32x4{l01, l23, h01, h23};
            }
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const rot_u32x4 a12 = lds_a[cur][b * 128 + lane];       // {Rh, Rm}
                const rot_u32x4 a3 = lds_a[cur][b * 128 + 64 + lane];   // {Rh, Rl}
#pragma unroll
                for (int t = 0; t < TILES; ++t) {
                    acc[t][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(rot_bf16x8, a12), __builtin_bit_cast(rot_bf16x8, b1[t]), acc[t][b], 0, 0, 0);
                    acc[t][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(rot_bf16x8, a12), __builtin_bit_cast(rot_bf16x8, b2[t]), acc[t][b], 0, 0, 0);
                    acc[t][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(rot_bf16x8, a3), __builtin_bit_cast(rot_bf16x8, b3[t]), acc[t][b], 0, 0, 0);
                }
            }
            if (more) {
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    const int i = threadIdx.x + 256 * q;
                    if (i < CHUNK) lds_a[cur ^ 1][i] = pre[q];
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        }
    }
    // register v of block b holds output dimension 32 b + 8 (v / 4) + 4 h + v % 4 of this lane's row
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        if (row[t] >= n) continue;
        float *yr = y + row[t] * DIM + 4 * h;
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<float4 *>(yr + 32 * b + 8 * g) =
                    make_float4(acc[t][b][4 * g], acc[t][b][4 * g + 1], acc[t][b][4 * g + 2], acc[t][b][4 * g + 3]);
    }
}

// The same product for dim <= 128 with the whole operand table of R resident in LDS (NB * 32 KB):
// one workgroup of 8 waves per compute unit stages it once and then walks over the row tiles, so
// the steady state has no barrier, and a wave's row fetches run kRotAhead chunks ahead straight
// across tile boundaries while the finished tile's 32 KB of output is still being written.
template <int NB, int TILES>
static __global__ void __launch_bounds__(512) k_rotate_mfma_resident(const float *__restrict__ x, int64_t n,
                                                                     int64_t ld, const rot_u32x4 *__restrict__ rtab,
                                                                     float *__restrict__ y) {
    constexpr int DIM = 32 * NB, NKC = DIM / 8, CHUNK = NB * 128;
    extern __shared__ __attribute__((aligned(16))) rot_u32x4 lds_r[];  // [NKC][NB][2][64]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    for (int i = threadIdx.x; i < NKC * CHUNK; i += 512) lds_r[i] = rtab[i];
    __syncthreads();
    const int64_t groups = (n + 32 * TILES - 1) / (32 * TILES);  // groups of TILES row tiles
    const int64_t stride = (int64_t)gridDim.x * 8;
    int64_t g = (int64_t)blockIdx.x * 8 + wave;
    if (g >= groups) return;
    auto row_ptr = [&](int64_t grp, int t) {
        const int64_t row = (grp * TILES + t) * 32 + r;
        return x + (row < n ? row : 0) * ld + 4 * h;  // a row past the end reads row 0, never stored
    };
    constexpr int kRotAhead = 4;  // NKC is a multiple of 4
    const float *xr[TILES];
    float4 xq[TILES][kRotAhead];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        xr[t] = row_ptr(g, t);
#pragma unroll
        for (int u = 0; u < kRotAhead; ++u) xq[t][u] = *reinterpret_cast<const float4 *>(xr[t] + u * 8);
    }
    for (; g < groups; g += stride) {
        const int64_t gn = g + stride < groups ? g + stride : g;  // the next group (or this one again: unused loads)
        const float *xn[TILES];
#pragma unroll
        for (int t = 0; t < TILES; ++t) xn[t] = row_ptr(gn, t);
        rot_floatx16 acc[TILES][NB];
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[t][b][v] = 0.0f;
#pragma unroll 1
        for (int kc0 = 0; kc0 < NKC; kc0 += kRotAhead) {
#pragma unroll
            for (int u = 0; u < kRotAhead; ++u) {
                const int kc = kc0 + u;
                rot_u32x4 b1[TILES], b2[TILES], b3[TILES];
#pragma unroll
                for (int t = 0; t < TILES; ++t) {
                    const float4 xv = xq[t][u];
                    const float *src = kc + kRotAhead < NKC ? xr[t] + (kc + kRotAhead) * 8 : xn[t] + (kc + kRotAhead - NKC) * 8;
                    xq[t][u] = *reinterpret_cast<const float4 *>(src);
                    uint32_t h01, m01, l01, h23, m23, l23;
                    rot_split3_pair(xv.x, xv.y, h01, m01, l01);
                    rot_split3_pair(xv.z, xv.w, h23, m23, l23);
                    b1[t] = rot_u32x4{h01, h23, h01, h23};
                    b2[t] = rot_u32x4{m01, m23, m01, m23};
                    b3[t] = rot_u32x4{l01, l23, h01, h23};
                }
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    const rot_u32x4 a12 = lds_r[(size_t)kc * CHUNK + b * 128 + lane];      // {Rh, Rm}
                    const rot_u32x4 a3 = lds_r[(size_t)kc * CHUNK + b * 128 + 64 + lane];  // {Rh, Rl}
#pragma unroll
                    for (int t = 0; t < TILES; ++t) {
                        acc[t][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(rot_bf16x8, a12), __builtin_bit_cast(rot_bf16x8, b1[t]), acc[t][b], 0, 0, 0);
                        acc[t][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(rot_bf16x8, a12), __builtin_bit_cast(rot_bf16x8, b2[t]), acc[t][b], 0, 0, 0);
                        acc[t][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            __builtin_bit_cast(rot_bf16x8, a3), __builtin_bit_cast(rot_bf16x8, b3[t]), acc[t][b], 0, 0, 0);
                    }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            const int64_t row = (g * TILES + t) * 32 + r;
            if (row < n) {
                float *yr = y + row * DIM + 4 * h;
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int gq = 0; gq < 4; ++gq)
                        *reinterpret_cast<float4 *>(yr + 32 * b + 8 * gq) = make_float4(
                            acc[t][b][4 * gq], acc[t][b][4 * gq + 1], acc[t][b][4 * gq + 2], acc[t][b][4 * gq + 3]);
            }
            xr[t] = xn[t];
        }
    }
}

}  // namespace vq

// ---- orthogonal Procrustes (src/opq.rs:180-183) -------------------------------------------------
// R = V U^T for A = U S V^T by a one-sided Jacobi SVD in f64.  The columns of A are made orthogonal
// by plane rotations; V is the product of those rotations.  The rotations depend on the columns of
// A only, never on V, so the work is split in three:
//   k_jacobi_sweeps      one workgroup, the columns of A as rows of ut in LDS (n <= 128, n even:
//                        133 KB).  A round rotates n / 2 disjoint pairs at once, sixteen lanes per
//                        pair (round-robin pairing: n - 1 rounds are a sweep over all pairs), and
//                        writes each rotation (c, s) to a list.  Sweeps stop when no pair is
//                        further from orthogonal than 1e-15, as in the host routine.
//   k_jacobi_accumulate  replays the list on V, one wave per row of V: lane g holds the two
//                        entries that pair g of the round rotates, and the entries move one lane
//                        along after every round as the pairing does, so nothing leaves registers.
//   k_jacobi_product     out = V U^T with the columns of U scaled to unit length.
// Pair g of round r is (a, b) = ((r + g) mod (n - 1), (r - g) mod (n - 1)), pair 0 is (r, n - 1);
// its rotation maps (a, b) to (c a - s b, s a + c b).
namespace vq {

constexpr int kJacobiMax = 128;
constexpr int kJacobiSweeps = 60;
constexpr int kJacobiStride = kJacobiMax + 16;  // rows one apart are half the LDS banks apart

// the value of the lane that a DPP control names (quad permutation, row mirror ...)
template <int CTRL> __device__ __forceinline__ double dpp_f64(double v) {
    const long long bits = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)bits, CTRL, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(bits >> 32), CTRL, 0xf, 0xf, false);
    return __longlong_as_double(((long long)hi << 32) | (unsigned)lo);
}
// sum over the LANES (4, 8 or 16) adjacent lanes of a pair, in every one of them
template <int LANES> __device__ __forceinline__ double pair_sum(double v) {
    v += dpp_f64<0xB1>(v);  // quad_perm [1,0,3,2]
    v += dpp_f64<0x4E>(v);  // quad_perm [2,3,0,1]
    if (LANES >= 8) v += dpp_f64<0x141>(v);   // row_half_mirror: the other quad of the eight
    if (LANES == 16) v += dpp_f64<0x128>(v);  // row_ror 8: the other eight of the sixteen
    return v;
}
// 1 / x and 1 / sqrt(x) to within a few ulp for positive normal x: the hardware's estimate and two
// Newton steps (the rotations need c^2 + s^2 = 1 to rounding, not correctly rounded quotients)
__device__ __forceinline__ double rcp_newton(double x) {
    double r = __builtin_amdgcn_rcp(x);
    r = fma(fma(-x, r, 1.0), r, r);
    return fma(fma(-x, r, 1.0), r, r);
}
__device__ __forceinline__ double rsq_newton(double x) {
    double y = __builtin_amdgcn_rsq(x);
    y = fma(fma(-x * y, y, 1.0), 0.5 * y, y);
    return fma(fma(-x * y, y, 1.0), 0.5 * y, y);
}

// LANES lanes per pair, 64 * LANES threads; a lane holds 128 / LANES entries of both rows.  Rows
// are kJacobiMax long whatever n is: the entries from n on are zero and stay zero.
template <int LANES>
static __global__ void __launch_bounds__(64 * LANES) k_jacobi_sweeps(const double *__restrict__ A, int n,
                                                                      double2 *__restrict__ rot,
                                                                      int *__restrict__ n_rounds,
                                                                      double *__restrict__ uhat,
                                                                      double *__restrict__ sv) {
    extern __shared__ __attribute__((aligned(16))) double ut[];  // n rows of stride kJacobiStride
    __shared__ int unfinished;
    constexpr int S = kJacobiStride, NT = 64 * LANES, PER = kJacobiMax / (2 * LANES);
    const int tid = threadIdx.x, pair = tid / LANES, sub = tid % LANES;
    for (int e = tid; e < n * kJacobiMax; e += NT) {
        const int j = e / kJacobiMax, i = e % kJacobiMax;
        ut[j * S + i] = i < n ? A[(size_t)i * n + j] : 0.0;  // row j of ut = column j of A
    }
    if (tid == 0) unfinished = 0;
    __syncthreads();
    const int half = n / 2;
    int round = 0;
    for (int sweep = 0; sweep < kJacobiSweeps; ++sweep) {
        for (int r = 0; r < n - 1; ++r, ++round) {
            if (pair < half) {
                const int p = (r + pair) % (n - 1);
                const int q = pair == 0 ? n - 1 : (r - pair + (n - 1)) % (n - 1);
                double2 *up = reinterpret_cast<double2 *>(ut + p * S) + sub;
                double2 *uq = reinterpret_cast<double2 *>(ut + q * S) + sub;
                double2 a[PER], b[PER];
#pragma unroll
                for (int j = 0; j < PER; ++j) {
                    a[j] = up[LANES * j];
                    b[j] = uq[LANES * j];
                }
                double alpha = 0.0, beta = 0.0, gamma = 0.0;
#pragma unroll
                for (int j = 0; j < PER; ++j) {
                    alpha = fma(a[j].x, a[j].x, alpha);
                    beta = fma(b[j].x, b[j].x, beta);
                    gamma = fma(a[j].x, b[j].x, gamma);
                    alpha = fma(a[j].y, a[j].y, alpha);
                    beta = fma(b[j].y, b[j].y, beta);
                    gamma = fma(a[j].y, b[j].y, gamma);
                }
                alpha = pair_sum<LANES>(alpha);
                beta = pair_sum<LANES>(beta);
                gamma = pair_sum<LANES>(gamma);
                // the pair counts as orthogonal below a cosine of 1e-16 and is left alone; a
                // cosine of 1e-15 or more asks for another sweep (the host routine's test)
                const double g2 = gamma * gamma, ab = alpha * beta;
                double c = 1.0, s = 0.0;
                if (g2 > 1e-32 * ab) {  // the same in the lanes of a pair
                    if (sub == 0 && g2 >= 1e-30 * ab) __atomic_store_n(&unfinished, 1, __ATOMIC_RELAXED);
                    // tan of the angle that makes the rows orthogonal: the smaller root of
                    // t^2 + 2 zeta t - 1 = 0, zeta = delta / gamma, written without the quotient
                    const double delta = 0.5 * (beta - alpha);
                    const double h2 = fma(delta, delta, g2);
                    const double hyp = h2 * rsq_newton(h2);
                    const double t = (delta >= 0.0 ? gamma : -gamma) * rcp_newton(fabs(delta) + hyp);
                    c = rsq_newton(fma(t, t, 1.0));
                    s = c * t;
#pragma unroll
                    for (int j = 0; j < PER; ++j) {
                        up[LANES * j] = make_double2(fma(c, a[j].x, -(s * b[j].x)), fma(c, a[j].y, -(s * b[j].y)));
                        uq[LANES * j] = make_double2(fma(s, a[j].x, c * b[j].x), fma(s, a[j].y, c * b[j].y));
                    }
                }
                if (sub == 0) rot[(size_t)round * half + pair] = make_double2(c, s);
            }
            __syncthreads();
        }
        const int more = __atomic_load_n(&unfinished, __ATOMIC_RELAXED);
        __syncthreads();
        if (tid == 0) unfinished = 0;
        __syncthreads();
        if (!more) break;  // the same in every thread
    }
    if (tid == 0) *n_rounds = round;
    // unit columns of U and their lengths, the singular values; a zero column stays zero (the
    // host completes the directions that A does not determine)
    for (int j = pair; j < n; j += 64) {
        double s = 0.0;
        for (int i = sub; i < n; i += LANES) s += ut[j * S + i] * ut[j * S + i];
        s = sqrt(pair_sum<LANES>(s));
        if (sub == 0) sv[j] = s;
        for (int i = sub; i < n; i += LANES) uhat[(size_t)j * n + i] = s > 0.0 ? ut[j * S + i] / s : ut[j * S + i];
    }
}

constexpr int kJacobiRing = 16;

// vt[l][i] = V[i][l]; grid = n workgroups of one wave, workgroup i makes row i of V
static __global__ void __launch_bounds__(64) k_jacobi_accumulate(const double2 *__restrict__ rot,
                                                                 const int *__restrict__ n_rounds, int n,
                                                                 double *__restrict__ vt) {
    const int i = blockIdx.x, g = threadIdx.x, half = n / 2;
    const int rounds = *n_rounds;
    const bool act = g < half;
    const int gl = act ? g : 0;  // idle lanes follow lane 0's addresses and keep nothing
    // seats of round 0: a = g, b = n - 1 - g (pair 0: n - 1)
    double xa = (act && g == i) ? 1.0 : 0.0;
    double xb = (act && (g == 0 ? n - 1 : n - 1 - g) == i) ? 1.0 : 0.0;
    const int from_up = min(g + 1, 63), from_down = max(g - 1, 0);
    double2 cs[kJacobiRing];
#pragma unroll
    for (int j = 0; j < kJacobiRing; ++j) {
        cs[j] = rot[(size_t)min(j, rounds - 1) * half + gl];
        asm volatile("" ::: "memory");
    }
    for (int t0 = 0; t0 < rounds; t0 += kJacobiRing) {
#pragma unroll
        for (int j = 0; j < kJacobiRing; ++j) {
            const double c = cs[j].x, s = cs[j].y;
            cs[j] = rot[(size_t)min(t0 + j + kJacobiRing, rounds - 1) * half + gl];
            if (t0 + j < rounds) {  // the same in every lane
                const double na = c * xa - s * xb, nb = s * xa + c * xb;
                // the pairing of the next round: a moves down a lane, b up; the ends cross over
                const double a_up = __shfl(na, from_up), b_down = __shfl(nb, from_down);
                const double a0 = __shfl(na, 0);
                xa = (g == half - 1 && half > 1) ? nb : (half > 1 ? a_up : na);  // n = 2: nothing moves
                xb = g == 0 ? nb : (g == 1 ? a0 : b_down);
            }
        }
    }
    if (act) {
        const int r = rounds % (n - 1);
        const int ia = (r + g) % (n - 1), ib = g == 0 ? n - 1 : (r - g + (n - 1)) % (n - 1);
        vt[(size_t)ia * n + i] = xa;
        vt[(size_t)ib * n + i] = xb;
    }
}

// out[i][j] = sum_l V[i][l] U[j][l], l ascending
static __global__ void __launch_bounds__(256) k_jacobi_product(const double *__restrict__ vt,
                                                               const double *__restrict__ uhat, int n,
                                                               double *__restrict__ out) {
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e >= n * n) return;
    const int i = e / n, j = e % n;
    double acc = 0.0;
    for (int l = 0; l < n; ++l) acc += vt[(size_t)l * n + i] * uhat[(size_t)l * n + j];
    out[e] = acc;
}

}  // namespace vq
