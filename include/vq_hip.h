/*
 * vq_hip.h — C ABI of libvqhip: the codebook hot path of the `vq` crate on MI355X (gfx950).
 *
 * The reference is a pure-Rust crate with no FFI layer; the seam this library fills is the
 * crate-private `utils::lbg_quantize` (src/utils.rs:32-109) and the inline nearest-centroid
 * loops of the four codebook quantizers.  A Rust `-sys` crate binds exactly these symbols
 * (plain pointers and sizes, no C++ or torch types).
 *
 * Conventions
 *   - every function returns an int32 status: 0 = VQ_OK, negative = error; the message of
 *     the last error of a context is returned by vq_last_error().
 *   - pointers named d_* are DEVICE pointers (from vq_malloc or any HIP allocation on the
 *     context's device); pointers named h_* are host pointers.
 *   - matrices are row-major f32, `ld` = row stride in elements; a "column block" s of width
 *     sub_dim covers columns [s*sub_dim, (s+1)*sub_dim).
 *   - codes are uint8 (k <= 256) or, in the entry points named *_u16, uint16 (k <= 65536: the
 *     reference's k is a usize, src/utils.rs:32-37, and its codes are usize indices); row-major
 *     n x m unless stated otherwise.
 *   - all work is enqueued on the context's stream; functions that return host values
 *     synchronise that stream before returning, the others are asynchronous.
 *   - one context = one stream; a context is not re-entrant, distinct contexts are independent.
 *     (vq_lbg_fit also runs part of its update on a second stream that the context owns; that
 *     work is joined back into the context's stream inside the call, so callers order their own
 *     work against the context's stream only.)
 *   - randomness never crosses the boundary as a seed: the host draws the index streams
 *     (initial rows, re-seed rows) with its own RNG and passes them as arrays.
 */
#ifndef VQ_HIP_H
#define VQ_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct vq_ctx vq_ctx;

enum vq_status {
    VQ_OK = 0,
    VQ_ERR_INVALID_ARG = -1,      /* VqError::InvalidParameter, src/exceptions.rs:19 */
    VQ_ERR_DIM_MISMATCH = -2,     /* VqError::DimensionMismatch, src/exceptions.rs:11 */
    VQ_ERR_EMPTY_INPUT = -3,      /* VqError::EmptyInput, src/exceptions.rs:15 */
    VQ_ERR_UNSUPPORTED = -4,      /* metric or size outside what the kernels cover */
    VQ_ERR_OOM = -5,
    VQ_ERR_HIP = -6,
    VQ_ERR_RESEED_EXHAUSTED = -7  /* more empty clusters met than re-seed indices supplied */
};

/* Distance variants with a kernel (src/distances.rs:73-88; Chebyshev, Minkowski and Hamming
 * stay on the host). */
enum vq_metric {
    VQ_SQEUCLIDEAN = 0, /* src/distances.rs:130-133 */
    VQ_EUCLIDEAN = 1,   /* src/distances.rs:134-140 */
    VQ_COSINE = 2,      /* src/distances.rs:141-151 */
    VQ_MANHATTAN = 3    /* src/distances.rs:152 */
};

/* ---- context and device memory ------------------------------------------------------- */

int32_t vq_ctx_create(int32_t device, vq_ctx **out);
int32_t vq_ctx_destroy(vq_ctx *ctx);
/* Message of the last failing call on ctx (ctx may be NULL: last failing vq_ctx_create). */
const char *vq_last_error(const vq_ctx *ctx);
int32_t vq_ctx_sync(vq_ctx *ctx);
/* The context's hipStream_t, as an opaque pointer. */
void *vq_ctx_stream(vq_ctx *ctx);

/* Which kernels decide the squared-L2 / Euclidean assignment where both exist:
 *   0 (default)  matrix-core scores (bf16 matrix instructions on operands split into two bf16
 *                parts, for 8-float column blocks and for wider ones whose width is a multiple
 *                of 8) with an exact re-check of every undecided (row, block) pair
 *   1            the all-vector-ALU kernel in the reference's operation order
 * Both give bit-identical codes; the switch exists for measurement and tests. */
int32_t vq_ctx_set_assign_path(vq_ctx *ctx, int32_t path);

/* How vq_tsvq_build sums a node's squared deviations per dimension in row order (src/tsvq.rs:88-99)
 * when dim is a multiple of 8:
 *   0 (default)  groups of 32 squares as integer maps on the running sum, composed by a scan, with
 *                the groups in which the sum changes binade added one by one
 *   1            one chain of dependent adds per column
 * Both give the reference's sequential f32 sums bit for bit; the switch exists for measurement and
 * tests.  No counterpart in the reference. */
int32_t vq_ctx_set_tsvq_variance_path(vq_ctx *ctx, int32_t path);

/* Measured peaks of this GPU, for pricing the kernels (measurement only; no counterpart in the
 * reference).  VQ_CALIB_HBM_COPY: GB/s of the plain copy kernel over 512 MB (bytes read + bytes
 * written per second).  VQ_CALIB_VALU_*: wave64 instructions of that kind per second over the
 * whole GPU with every SIMD kept full (v_fma_f32, v_min3_i32, v_med3_i32, v_and_or_b32, v_add_u32).
 * Synchronises. */
enum {
    VQ_CALIB_HBM_COPY = 0,
    VQ_CALIB_VALU_FMA = 1,
    VQ_CALIB_VALU_MIN3 = 2,
    VQ_CALIB_VALU_MED3 = 3,
    VQ_CALIB_VALU_AND_OR = 4,
    VQ_CALIB_VALU_ADD = 5
};
int32_t vq_calibrate(vq_ctx *ctx, int32_t what, double *h_rate);
/* Whether the matrix and the vector instructions of one SIMD run side by side or take turns
 * (measurement only; no counterpart in the reference).  Every SIMD holds 8 waves.
 *   mode 0  four waves of a SIMD issue chains of v_mfma_f32_32x32x16_bf16 (4096 each), the other four
 *           chains of v_min3_i32 (8 x 4096 each): the two kinds come from different waves
 *   mode 1  every wave issues both in one instruction stream, 7 independent v_min3_i32 after each
 *           matrix instruction;  mode 2: the same with 3
 * h_ms[0] = milliseconds of the matrix instructions alone, h_ms[1] of the vector instructions alone,
 * h_ms[2] of both together (same counts).  h_waves (nullable, 8 numbers; mode 0 only, else zeros):
 * how many waves of the last launch ran on SIMD 0..3 of their compute unit, first the matrix waves,
 * then the vector waves — equal numbers mean every SIMD held both kinds.  Synchronises. */
int32_t vq_calibrate_overlap(vq_ctx *ctx, int32_t mode, double *h_ms, uint32_t *h_waves);

/* Number of (row, block) pairs the most recent matrix-core assignment pass left to the exact
 * re-check (0 if that path has not run).  Synchronises.  Measurement only. */
int32_t vq_ctx_last_recheck_count(vq_ctx *ctx, uint32_t *h_count);
/* The same count split by how the pair was decided: by the reference-order scan over all
 * centroids, or (wide column blocks only) between the two best-scored candidates. */
int32_t vq_ctx_last_recheck_split(vq_ctx *ctx, uint32_t *h_all_centroids, uint32_t *h_two_candidates);

int32_t vq_malloc(vq_ctx *ctx, size_t bytes, void **d_ptr);
int32_t vq_free(vq_ctx *ctx, void *d_ptr);
/* Page-locked host memory for the packed rows and the returned codes: copies from and to it run at
 * the link's rate (a pageable buffer is staged through a bounce buffer by the runtime, about half
 * the rate).  The host packs `&[Vector<f32>]` (one heap allocation per row, src/vector.rs:150-152)
 * straight into such a buffer.  No counterpart in the reference. */
int32_t vq_host_alloc(vq_ctx *ctx, size_t bytes, void **h_ptr);
int32_t vq_host_free(vq_ctx *ctx, void *h_ptr);
/* Synchronous copies (they synchronise the context's stream). Replaces the per-vector heap
 * layout `&[Vector<f32>]` (src/vector.rs:150-152): the host packs rows into one buffer.
 * vq_h2d of 64 MiB or more from pageable memory is staged by the library: up to eight host threads
 * copy 16 MiB chunks into page-locked buffers of the context while the copy engine uploads the chunk
 * before (about 50 GB/s instead of 18-29 for one plain copy; a page-locked source goes up directly);
 * vq_d2h into pageable memory does the same in the other direction. */
int32_t vq_h2d(vq_ctx *ctx, void *d_dst, const void *h_src, size_t bytes);
int32_t vq_d2h(vq_ctx *ctx, void *h_dst, const void *d_src, size_t bytes);

/* Device-to-device copy of `count` floats by a plain streaming kernel (the initial
 * `rotated_data = training_data.to_vec()` of src/opq.rs:121 and `residuals = training_data.to_vec()`
 * of src/rvq.rs:103; also the known-size kernel the HBM counters are calibrated against).
 * Both pointers 16-byte aligned.  Asynchronous. */
int32_t vq_copy_f32(vq_ctx *ctx, float *d_dst, const float *d_src, int64_t count);

/* ---- timing (HIP events on the context's stream) --------------------------------------- */
int32_t vq_timer_start(vq_ctx *ctx);
/* Records the stop event, synchronises, returns elapsed milliseconds since vq_timer_start. */
int32_t vq_timer_stop(vq_ctx *ctx, float *h_ms);

/* Per-kernel-class timing with HIP events on the context's stream around the launches the
 * library makes (no counterpart in the reference; measurement only): recorded before and after
 * the launches of a class, or, for the matrix-core assignment kernel, carried by the kernel's own
 * dispatch as its start and stop events, which puts no extra packet on the queue.  Enabling
 * resets the accumulators.  vq_prof_read synchronises the stream and returns the summed event
 * time and the number of timed spans of one class. */
enum vq_prof_class {
    VQ_PROF_LBG_ASSIGN = 0, /* the assignment kernels of one LBG iteration (utils.rs:59-73) */
    VQ_PROF_LBG_UPDATE = 1, /* the update kernels of one LBG iteration (utils.rs:83-102): from the end of
                               its assignment kernel to the start of the next one */
    VQ_PROF_ENCODE = 2,     /* the kernels of one vq_assign call */
    VQ_PROF_ASSIGN_KERNEL = 3, /* the main assignment kernel alone (matrix-core pass or the
                                  vector-ALU kernel), in training and in vq_assign */
    VQ_PROF_CLASSES = 4
};
int32_t vq_prof_enable(vq_ctx *ctx, int32_t on);
int32_t vq_prof_read(vq_ctx *ctx, int32_t cls, double *h_total_ms, int64_t *h_spans);

/* ---- LBG training: replaces utils::lbg_quantize (src/utils.rs:32-109) ------------------ */

/* m independent LBG problems, one per column block of width sub_dim of d_x (n x ld).
 * m = 1, sub_dim = dim is the plain lbg_quantize call of src/rvq.rs:107; m > 1 is the batched
 * form of the per-subspace calls at src/pq.rs:106-121 and src/opq.rs:127-142.
 *
 *   h_init_idx       m*k  row indices copied as initial centroids (choose_multiple, utils.rs:54)
 *   h_reseed_stream  m*n_reseed  successive `choose` draws (utils.rs:100); the i-th empty
 *                    cluster met by problem s (iteration-major, cluster index ascending) takes
 *                    h_reseed_stream[s*n_reseed + i].  n_reseed = k*max_iters can never run out.
 *   d_codebooks      out, m*k*sub_dim
 *   h_iters_run      out (nullable), m: loop bodies executed per problem (early break, 104-106)
 *   h_reseeds_used   out (nullable), m
 * Assignment is squared-L2, sequential f32 accumulation, strict '<' (utils.rs:62-70); the mean
 * follows mean_vector's order (src/vector.rs:282-318) for clusters of at most 1024 rows (row order
 * from 0.0).  Above 1024 the reference's Rayon reduce has no fixed order; this library fixes one:
 * the rows are cut into parts of 4096 consecutive rows, a cluster's members inside a part are added
 * in row order from 0.0, and the part sums are added in part order from 0.0.
 * k up to 65536: above 256 the assignment runs chunk by chunk (see vq_assign_u16) and the update
 * lists the clusters' members with a sort of (column block, code, row) keys, same orders of
 * summation; that path needs n * m < 2^32.
 * Errors: k == 0 or n < k -> VQ_ERR_INVALID_ARG (utils.rs:39-50); k > 65536 -> VQ_ERR_UNSUPPORTED.
 * Synchronises the stream before returning. */
int32_t vq_lbg_fit(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t m,
                   int32_t sub_dim, int32_t k, int32_t max_iters, const uint32_t *h_init_idx,
                   const uint32_t *h_reseed_stream, int32_t n_reseed, float *d_codebooks,
                   int32_t *h_iters_run, int32_t *h_reseeds_used);

/* ---- nearest-centroid assignment / encode ---------------------------------------------- */

/* d_codes[i*m + s] = first index j minimising metric(x_i[block s], codebook[s][j]), strict '<'.
 * Replaces the inline loops at src/pq.rs:166-174, src/opq.rs:155-163,250-258,
 * src/rvq.rs:116-124,189-197 (m = 1 there).  Asynchronous. */
int32_t vq_assign(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t m,
                  int32_t sub_dim, int32_t k, const float *d_codebooks, uint8_t *d_codes);

/* vq_assign with 16-bit codes, for any k up to 65536 (`k: usize` at src/utils.rs:32-37 and
 * src/pq.rs:79-86; the reference's codes are usize indices).  Same rule, same metrics.  Above 256
 * centroids every column block's codebook is cut into chunks of 256 consecutive centroids; each
 * chunk goes through the kernels of vq_assign and its winner's distance, evaluated in the
 * reference's operation order, replaces the running minimum only when strictly below it, chunks
 * in ascending order — the lowest index of the overall minimum, as one loop over all k gives.
 * d_codes 2-byte aligned.  Asynchronous. */
int32_t vq_assign_u16(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t m,
                      int32_t sub_dim, int32_t k, const float *d_codebooks, uint16_t *d_codes);

/* vq_assign for callers that cannot allocate device memory (tight serving loops, harnesses that
 * forbid hipMalloc, code that must not call an allocator between two points).  No counterpart in the
 * reference.  Same arguments, same codes, bit for bit; the call makes no hipMalloc / hipFree and
 * never grows the context's workspace.  The tables of the matrix-core kernel (8-float column blocks
 * under squared-L2 / Euclidean) and the centroid norms (cosine) live in one fixed array of 1.2 MB of
 * device memory that the library holds on every GPU it runs on until the process ends.
 *   limit (for the shapes that use the array: cosine, and 8-float column blocks under squared-L2 /
 *          Euclidean on the default assignment path): m <= 1024 and m * (k rounded up to a multiple
 *          of 64) <= 16384 (e.g. m = 64, k = 256); beyond it VQ_ERR_UNSUPPORTED, and nothing is
 *          launched.  Other shapes (Manhattan, other widths) need no scratch and have no such limit.
 *   wider column blocks under squared-L2 / Euclidean take the vector-ALU kernel (the matrix-core
 *   kernel for them keeps lists that grow with n).
 * This is the one exception to "distinct contexts are independent": a GPU has ONE such array, and
 * calls that use it must not overlap in time on that GPU.  Calls of one context follow each other on
 * its stream.  A call from another context is accepted once everything on the stream of the context
 * that used the array last has finished, and returns VQ_ERR_UNSUPPORTED before (its kernels would
 * overwrite tables that kernels in flight still read).  A call leaves nothing the next one depends on.
 * The call has not been exercised under HIP graph capture (it sets a function attribute on its
 * first use of a kernel).  Asynchronous. */
int32_t vq_assign_noalloc(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t m,
                          int32_t sub_dim, int32_t k, const float *d_codebooks, uint8_t *d_codes);

/* d_out[i*(m*sub_dim) + s*sub_dim + t] = f16(codebook[s][code[i][s]][t]) — the value returned by
 * ProductQuantizer::quantize (src/pq.rs:176-186; f16::from_f32, round to nearest even).
 * d_out holds IEEE binary16 bit patterns.  Asynchronous. */
int32_t vq_decode_f16(vq_ctx *ctx, const uint8_t *d_codes, int64_t n, int32_t m, int32_t sub_dim,
                      int32_t k, const float *d_codebooks, uint16_t *d_out);

/* Same gather without the f16 conversion (the f32 reconstruction of src/opq.rs:146-168). */
int32_t vq_decode_f32(vq_ctx *ctx, const uint8_t *d_codes, int64_t n, int32_t m, int32_t sub_dim,
                      int32_t k, const float *d_codebooks, float *d_out);

/* The two decodes for the 16-bit codes of vq_assign_u16 (k <= 65536). */
int32_t vq_decode_f16_u16(vq_ctx *ctx, const uint16_t *d_codes, int64_t n, int32_t m, int32_t sub_dim,
                          int32_t k, const float *d_codebooks, uint16_t *d_out);
int32_t vq_decode_f32_u16(vq_ctx *ctx, const uint16_t *d_codes, int64_t n, int32_t m, int32_t sub_dim,
                          int32_t k, const float *d_codebooks, float *d_out);

/* ---- residual quantizer (src/rvq.rs) -------------------------------------------------------- */

/* d_res[i] -= d_codebook[d_codes[i]] for every row (the residual update of src/rvq.rs:127).
 * d_codes: n uint8 (the output of vq_assign with m = 1).  Asynchronous. */
int32_t vq_residual_sub(vq_ctx *ctx, float *d_res, int64_t n, int64_t ld, int32_t dim, int32_t k,
                        const float *d_codebook, const uint8_t *d_codes);
/* The same for the 16-bit codes of vq_assign_u16 (k <= 65536; `k: usize` at src/rvq.rs:87-95). */
int32_t vq_residual_sub_u16(vq_ctx *ctx, float *d_res, int64_t n, int64_t ld, int32_t dim, int32_t k,
                            const float *d_codebook, const uint16_t *d_codes);

/* The residual update of one stage and the training of the next in one call (src/rvq.rs:103-129 across
 * two turns of the stage loop): d_res[i] -= d_prev_codebook[d_prev_codes[i]] for every row, exactly as
 * vq_residual_sub does, then vq_lbg_fit with m = 1, sub_dim = dim on the updated rows, exactly as
 * vq_lbg_fit does (same arguments, same results bit for bit; on return d_res holds the updated
 * residual).  Where the fit's first assignment pass is the matrix-core pass over one wide column block
 * (dim a multiple of 8 from 16 on, k <= 256, 16-byte aligned rows and codebooks, max_iters >= 1) that
 * pass applies the update as it reads the rows and writes them back in place, which saves the
 * separate pass over the rows; otherwise the two steps run one after the other.  d_prev_codes: n uint8
 * codes below k_prev <= 256.  After an error d_res may or may not have been updated.  Synchronises
 * like vq_lbg_fit. */
int32_t vq_lbg_fit_residual(vq_ctx *ctx, float *d_res, int64_t n, int64_t ld, int32_t dim, int32_t k,
                            int32_t max_iters, const uint32_t *h_init_idx, const uint32_t *h_reseed_stream,
                            int32_t n_reseed, float *d_codebook, const float *d_prev_codebook, int32_t k_prev,
                            const uint8_t *d_prev_codes, int32_t *h_iters_run, int32_t *h_reseeds_used);

/* *h_out = (sum_i sqrt(sum_t x[i][t]^2)) / n — the early-stop statistic of src/rvq.rs:131-138.
 * Row norms follow the reference's sequential f32 order; the sum over rows (a Rayon sum of
 * unspecified order in the reference) is a fixed-shape f64 tree.  Synchronises. */
int32_t vq_mean_l2norm(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t dim, float *h_out);

/* ResidualQuantizer::quantize for every row (src/rvq.rs:171-215): stage by stage argmin under
 * `metric` (index 0 when k < 2), sum += c, residual -= c, the row stops when
 * ||residual|| < epsilon.
 *   d_codebooks    stages*k*dim
 *   d_codes        out, n*stages uint8 (0 for stages a row did not reach)
 *   d_stages_used  out (nullable), n uint8: stages applied to the row
 *   d_recon_f16    out (nullable), n*dim binary16 bit patterns of the f32 sum (rvq.rs:209-214)
 * stages <= 255 (the count of a row's stages is a byte).  Asynchronous. */
int32_t vq_rvq_encode(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t dim,
                      int32_t stages, int32_t k, const float *d_codebooks, float epsilon,
                      uint8_t *d_codes, uint8_t *d_stages_used, uint16_t *d_recon_f16);
/* The same with n*stages uint16 codes, k <= 65536 (`k: usize` at src/rvq.rs:87-95). */
int32_t vq_rvq_encode_u16(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld, int32_t dim,
                          int32_t stages, int32_t k, const float *d_codebooks, float epsilon,
                          uint16_t *d_codes, uint8_t *d_stages_used, uint16_t *d_recon_f16);

/* ---- optimized product quantizer (src/opq.rs) ---------------------------------------------- */

/* d_y[i] = R * d_x[i] for every row, R row-major dim x dim (src/opq.rs:186-194, 232-234).
 * d_y is n x dim, compact.  f32 fused multiply-add accumulation (the reference's nalgebra
 * rounding is implementation-defined).  Asynchronous. */
int32_t vq_rotate(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t dim, const float *d_R,
                  float *d_y);

/* h_A[a*dim + b] = sum_i d_y[i][a] * d_x[i][b], both n x dim compact — the matrix A = Y X^T of
 * src/opq.rs:172-179, accumulated in f64 in a fixed order (f64 matrix instructions when dim is a
 * multiple of 16).  dim <= 4096.  Synchronises. */
int32_t vq_cross_cov(vq_ctx *ctx, const float *d_y, const float *d_x, int64_t n, int32_t dim, double *h_A);

/* h_R = V U^T for h_A = U S V^T (both dim x dim, row-major, host memory): the rotation update of
 * src/opq.rs:180-183.  dim <= 4096, any parity.  V U^T is the orthogonal polar factor of A^T, unique
 * for a non-singular A, and is computed
 *   - for dim <= 512 by Newton-Schulz steps in f64 on the matrix cores; when they have not
 *     converged within their step limit (A singular, condition number above about 1e6, or
 *     non-finite), and for larger dim,
 *   - by a one-sided Jacobi SVD in f64: on the device for even dim <= 128, otherwise the same
 *     routine in host code of this library (the reference runs its SVD on the host as well);
 *     directions a singular A leaves open are completed to an orthonormal basis.
 * The result is a tolerance quantity (the reference's nalgebra SVD is not restated): both ways
 * agree to about 1e-10 for condition numbers up to 1e6.  Synchronises. */
int32_t vq_procrustes_rotation(vq_ctx *ctx, const double *h_A, int32_t dim, double *h_R);
/* 0 (default): as above; 1: the SVD only.  The switch exists for measurement and tests.  No
 * counterpart in the reference. */
int32_t vq_ctx_set_procrustes_path(vq_ctx *ctx, int32_t path);

/* ---- tree-structured VQ (src/tsvq.rs) ------------------------------------------------------ */

typedef struct vq_tree vq_tree;

/* TSVQ::new / TSVQNode::fit (src/tsvq.rs:71-148, 209-215): node mean, leaf test, per-dimension
 * sum of squared deviations in row order, last-maximum split dimension, exact median, stable
 * partition by `<= median`, children only when non-empty and strictly smaller.  Nodes are
 * numbered breadth-first (root 0, left before right).  Synchronises. */
int32_t vq_tsvq_build(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t dim,
                      int32_t max_depth, vq_tree **out);
/* The same tree built with 2-means splits instead of the median split — NOT the reference's
 * behaviour (src/tsvq.rs:87-123 splits at the median of the maximum-variance coordinate, which
 * vq_tsvq_build reproduces); an explicit mode for callers that want a k-means tree (2-means with a
 * number of LBG iterations per node).  Everything else of TSVQNode::fit stays: the node's centroid
 * is the mean of its rows (76), a node is a leaf at depth 0 or with at most one row (78), a child
 * exists only if non-empty and strictly smaller than its parent (128, 135).  The split is
 * lbg_quantize (src/utils.rs:32-109) with k = 2 on the node's rows in row order; a row goes left
 * when the first of the two returned centroids is its nearest (squared L2, strict '<').
 *   h_draws          (2^max_depth - 1) * draws_per_node values: the node at position h of the
 *                    complete binary tree (root 1, children 2h and 2h + 1) owns
 *                    h_draws[(h - 1) * draws_per_node ..].  With c rows in the node, its initial
 *                    centroids are its rows number d[0] % c and d[1] % (c - 1), plus one if that is
 *                    not below the first (k distinct rows, utils.rs:54), and the i-th empty
 *                    cluster it meets takes its row number d[2 + i] % c (utils.rs:100).
 *   draws_per_node   >= 2 + lbg_iters (one cluster can be empty per iteration)
 * max_depth <= 20.  Synchronises. */
int32_t vq_tsvq_build_kmeans(vq_ctx *ctx, const float *d_x, int64_t n, int64_t ld, int32_t dim,
                             int32_t max_depth, int32_t lbg_iters, const uint32_t *h_draws,
                             int32_t draws_per_node, vq_tree **out);
/* A tree from host arrays (children must have larger indices than their parent; -1 = none). */
int32_t vq_tree_create(vq_ctx *ctx, int32_t n_nodes, int32_t dim, const float *h_centroids,
                       const int32_t *h_left, const int32_t *h_right, vq_tree **out);
int32_t vq_tree_free(vq_ctx *ctx, vq_tree *tree);
int32_t vq_tree_info(const vq_tree *tree, int32_t *n_nodes, int32_t *dim);
/* Any output may be NULL.  h_split_dim is -1 and h_count 0 where unknown. */
int32_t vq_tree_download(const vq_tree *tree, float *h_centroids, int32_t *h_left, int32_t *h_right,
                         int32_t *h_split_dim, float *h_split_val, int64_t *h_count);

/* TSVQNode::quantize_with_distance for every row (src/tsvq.rs:162-181): d_leaf[i] = index of the
 * leaf reached; `<=` goes left, single children are followed.  Asynchronous. */
int32_t vq_tsvq_descend(vq_ctx *ctx, int32_t metric, const float *d_x, int64_t n, int64_t ld,
                        const vq_tree *tree, int32_t *d_leaf);
/* How vq_tsvq_descend decides a node under cosine, squared Euclidean and Euclidean distance when
 * the row fits in registers (dim a multiple of 32 up to 128):
 *   0 (default)  by the sign of one inner product with a vector of the node (the difference of the
 *                children's normalised centroids, or of the centroids with a norm term), whenever
 *                its value clears a proven bound on every rounding error of the reference's two
 *                sums; otherwise, for that row, by those two sums
 *   1            by the two sums always
 * Both give the reference's leaves bit for bit; the switch exists for measurement and tests.
 * Manhattan always takes the two sums.  No counterpart in the reference. */
int32_t vq_ctx_set_tsvq_descend_path(vq_ctx *ctx, int32_t path);
/* d_out[i] = f16(centroid of leaf d_leaf[i]) (src/tsvq.rs:241-248), n x dim.  Asynchronous. */
int32_t vq_tsvq_decode_f16(vq_ctx *ctx, const vq_tree *tree, const int32_t *d_leaf, int64_t n,
                           uint16_t *d_out);

#ifdef __cplusplus
}
#endif
#endif /* VQ_HIP_H */
