"""GPU parity for the residual quantizer and the optimized product quantizer pieces."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import data

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def ctx():
    import vq_amd
    c = vq_amd.Context(0)
    yield c
    c.close()


def gpu_rvq_fit(ctx, metric, x, stages, k, iters, eps, init, reseed):
    """ResidualQuantizer::fit (src/rvq.rs:87-154) composed from the C-ABI calls."""
    n, dim = x.shape
    dx = ctx.to_device(x)
    dres = ctx.empty((n, dim), F)
    ctx.copy_f32(dres, dx, n * dim)
    dcb = ctx.empty((stages, k, dim), F)
    dcodes = ctx.empty(n, np.uint8)
    norms = []
    produced = 0
    for st in range(stages):
        cb_ptr = dcb.ptr + st * k * dim * 4
        ctx.lbg_fit(dres, n, dim, 1, dim, k, iters, init[st], reseed[st], cb_ptr)
        produced += 1
        if k < 2:
            dcodes.upload(np.zeros(n, np.uint8))
        else:
            ctx.assign(metric, dres, n, dim, 1, dim, k, cb_ptr, dcodes)
        ctx.residual_sub(dres, n, dim, dim, k, cb_ptr, dcodes)
        norms.append(ctx.mean_l2norm(dres, n, dim, dim))
        if norms[-1] < eps:
            break
    return dcb.download()[:produced], dres.download(), np.array(norms, F), dcb


@pytest.mark.parametrize("n,dim,ld,k,k_prev,iters,kind", [
    (5000, 256, 256, 256, 256, 3, "normal"),   # the RVQ stage shape: the first pass applies the update
    (1000, 40, 40, 7, 5, 4, "normal"),         # an odd multiple of 8: the last stage's upper half is past the width
    (333, 16, 24, 3, 200, 2, "normal"),        # rows inside a wider buffer, n not a multiple of 128
    (4097, 128, 128, 64, 1, 3, "integers"),    # exact ties; a previous codebook of one centroid
    (700, 64, 64, 16, 9, 2, "nonfinite"),
    (900, 72, 72, 5, 4, 0, "normal"),          # no pass to ride on: the two steps one after the other
    (900, 12, 12, 5, 4, 3, "normal"),          # a width without the matrix-core pass: the same
    (600, 8, 8, 4, 3, 3, "normal"),            # the 8-float kernel: the same
])
def test_lbg_fit_residual_equals_the_two_steps(ctx, n, dim, ld, k, k_prev, iters, kind):
    """vq_lbg_fit_residual = vq_residual_sub, then vq_lbg_fit: same residual, codebook, iteration and
    re-seed counts, bit for bit, on the shapes where the first pass applies the update and on those
    where it cannot; and the oracle's residual update and fit on the same inputs."""
    rng = np.random.default_rng(n + dim + k)
    if kind == "integers":
        x = np.round(rng.standard_normal((n, ld)) * 2).astype(F)
        prev = np.round(rng.standard_normal((k_prev, dim)) * 2).astype(F)
    else:
        x = rng.standard_normal((n, ld)).astype(F)
        prev = rng.standard_normal((k_prev, dim)).astype(F)
    if kind == "nonfinite":
        x[::17, 3] = np.inf
        x[5::29, 11] = np.nan
        prev[2, 7] = -np.inf
    codes = rng.integers(0, k_prev, n).astype(np.uint8)
    init, reseed = data.index_streams(n, 1, k, max(iters, 1), seed=n)
    dprev, dcodes = ctx.to_device(prev), ctx.to_device(codes)
    # the two steps
    da = ctx.to_device(x)
    cba = ctx.empty((k, dim), F)
    ctx.residual_sub(da, n, ld, dim, k_prev, dprev, dcodes)
    it_a, used_a = ctx.lbg_fit(da, n, ld, 1, dim, k, iters, init[0], reseed[0], cba)
    # the one call
    db = ctx.to_device(x)
    cbb = ctx.empty((k, dim), F)
    it_b, used_b = ctx.lbg_fit_residual(db, n, ld, dim, k, iters, init[0], reseed[0], cbb, dprev, k_prev, dcodes)
    ra, rb = da.download(), db.download()
    assert np.array_equal(ra.view(np.uint32), rb.view(np.uint32))
    assert np.array_equal(cba.download().view(np.uint32), cbb.download().view(np.uint32))
    assert np.array_equal(it_a, it_b) and np.array_equal(used_a, used_b)
    # against the arithmetic itself: one f32 subtraction per element (src/rvq.rs:127), columns past dim untouched
    if kind != "nonfinite":  # (the bits of a NaN that a subtraction makes differ between CPU and GPU)
        want = x.copy()
        want[:, :dim] = x[:, :dim] - prev[codes]
        assert np.array_equal(rb.view(np.uint32), want.view(np.uint32))
        ref = O.pq_fit(np.ascontiguousarray(want[:, :dim]), 1, k, iters, init, reseed)
        assert np.array_equal(cbb.download().view(np.uint32), ref["codebooks"].reshape(k, dim).view(np.uint32))
    for b in (dprev, dcodes, da, db, cba, cbb):
        b.free()


def test_lbg_fit_residual_argument_errors(ctx):
    import vq_amd
    x = np.zeros((100, 16), F)
    d, cb, prev, codes = ctx.to_device(x), ctx.empty((4, 16), F), ctx.to_device(np.zeros((4, 16), F)), \
        ctx.to_device(np.zeros(100, np.uint8))
    init, reseed = data.index_streams(100, 1, 4, 2, seed=1)
    with pytest.raises(vq_amd.VqError):
        ctx.lbg_fit_residual(d, 100, 16, 16, 4, 2, init[0], reseed[0], cb, 0, 4, codes)  # no previous codebook
    with pytest.raises(vq_amd.VqError):
        ctx.lbg_fit_residual(d, 100, 16, 16, 4, 2, init[0], reseed[0], cb, prev, 300, codes)  # codes are 8-bit
    with pytest.raises(vq_amd.VqError):
        ctx.lbg_fit_residual(d, 3, 16, 16, 4, 2, init[0], reseed[0], cb, prev, 4, codes)  # fewer rows than clusters


@pytest.mark.parametrize("metric", [O.SQEUCLIDEAN, O.EUCLIDEAN, O.COSINE, O.MANHATTAN])
@pytest.mark.parametrize("n,dim,stages,k,iters", [(1000, 10, 2, 2, 50), (600, 32, 3, 16, 5),
                                                    (400, 256, 2, 8, 3), (3000, 6, 2, 2, 4)])
def test_rvq_fit_and_quantize_match_oracle(ctx, metric, n, dim, stages, k, iters):
    rng = np.random.default_rng(n + dim)
    x = rng.standard_normal((n, dim)).astype(F)
    init, reseed = data.index_streams(n, stages, k, iters, seed=3)
    want = O.rvq_fit(metric, x, stages, k, iters, 0.0, init, reseed)
    cb, res, norms, dcb = gpu_rvq_fit(ctx, metric, x, stages, k, iters, 0.0, init, reseed)
    assert want["stages"] == len(cb)
    assert np.array_equal(cb.view(np.uint32), want["codebooks"].view(np.uint32))
    assert np.array_equal(res.view(np.uint32), want["residuals"].view(np.uint32))
    # sum of row norms: Rayon order in the reference, so a tolerance (1e-5 relative)
    assert np.allclose(norms, want["avg_norms"], rtol=1e-5, atol=0)
    # quantize
    wcodes, wrec = O.rvq_quantize(metric, x, want["codebooks"], 0.0)
    dx = ctx.to_device(x)
    dcodes = ctx.empty((n, stages), np.uint8)
    dused = ctx.empty(n, np.uint8)
    drec = ctx.empty((n, dim), np.uint16)
    ctx.rvq_encode(metric, dx, n, dim, dim, stages, k, dcb, 0.0, dcodes, dused, drec)
    assert np.array_equal(dcodes.download(), wcodes.astype(np.uint8))
    assert np.all(dused.download() == stages)
    assert np.array_equal(drec.download(), wrec)


def test_rvq_quantize_epsilon_stops_rows_individually(ctx):
    rng = np.random.default_rng(8)
    n, dim, stages, k = 500, 8, 3, 4
    cb = rng.standard_normal((stages, k, dim)).astype(F)
    x = rng.standard_normal((n, dim)).astype(F)
    x[::5] = cb[0, 2]          # these rows hit a codeword exactly -> residual 0 after stage 1
    x[1::5] = cb[0, 1] + cb[1, 3]  # and these after stage 2 (if stage 1 picks codeword 1)
    eps = 1e-3
    wcodes, wrec = O.rvq_quantize(O.EUCLIDEAN, x, cb, eps)
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    dcodes = ctx.empty((n, stages), np.uint8)
    dused = ctx.empty(n, np.uint8)
    drec = ctx.empty((n, dim), np.uint16)
    ctx.rvq_encode(O.EUCLIDEAN, dx, n, dim, dim, stages, k, dcb, eps, dcodes, dused, drec)
    used = dused.download()
    reached = wcodes != 0xFFFFFFFF
    assert np.array_equal(used, reached.sum(1))
    assert used.min() == 1 and used.max() == stages
    got = dcodes.download()
    assert np.array_equal(got[reached], wcodes[reached].astype(np.uint8))
    assert np.all(got[~reached] == 0)
    assert np.array_equal(drec.download(), wrec)


@pytest.mark.parametrize("n,dim,ld,stages,k,eps,metric", [
    (3000, 256, 256, 1, 256, 0.0, O.EUCLIDEAN),    # one stage: no residual at all
    (3000, 256, 256, 4, 256, 0.0, O.EUCLIDEAN),    # the stage shape of the wide pass
    (1500, 64, 80, 3, 16, 0.0, O.SQEUCLIDEAN),     # rows inside a wider buffer, read where they lie
    (1500, 64, 70, 3, 16, 0.0, O.COSINE),          # a row stride that is no multiple of 4: copied first
    (1500, 64, 70, 3, 16, 0.0, O.SQEUCLIDEAN),     # ... and the updates ride on the next stage's pass, in place
    (2100, 40, 44, 5, 7, 0.0, O.EUCLIDEAN),        # five stages of an odd multiple of 8 floats
    (130, 16, 16, 2, 2, 0.0, O.SQEUCLIDEAN),
    (5000, 24, 24, 3, 256, float("nan"), O.EUCLIDEAN),  # a threshold that no norm is below
    (901, 30, 33, 2, 5, 0.0, O.MANHATTAN),         # a width that is no multiple of 4
    (901, 30, 33, 1, 5, 0.0, O.MANHATTAN),
    (2000, 32, 48, 4, 8, 4.5, O.EUCLIDEAN),        # rows stop at different stages
    (2000, 32, 32, 1, 8, 100.0, O.EUCLIDEAN),      # every row stops after the one stage
    (700, 16, 16, 3, 1, 0.0, O.EUCLIDEAN),         # one centroid per stage
    (1200, 128, 128, 2, 300, 0.0, O.EUCLIDEAN),    # 16-bit codes
    (1200, 128, 132, 1, 300, 0.0, O.SQEUCLIDEAN),
])
def test_rvq_encode_first_and_last_stage_paths(ctx, n, dim, ld, stages, k, eps, metric):
    """vq_rvq_encode against the oracle where the first stage reads the caller's rows in place (or cannot)
    and the last stage only records its codes; the caller's buffer stays as it was."""
    rng = np.random.default_rng(n + dim + ld + stages)
    buf = rng.standard_normal((n, ld)).astype(F)
    cb = (rng.standard_normal((stages, k, dim)) * np.array([1.0, 0.6, 0.4, 0.3, 0.2])[:stages, None, None]).astype(F)
    if eps > 0:  # rows at different distances from a first-stage centroid
        buf[:, :dim] = cb[0][rng.integers(0, k, n)] + buf[:, :dim] * rng.uniform(0.3, 1.5, (n, 1)).astype(F)
    x = np.ascontiguousarray(buf[:, :dim])
    wcodes, wrec = O.rvq_quantize(metric, x, cb, eps)
    dx, dcb = ctx.to_device(buf), ctx.to_device(cb)
    wide = k > 256
    dcodes = ctx.empty((n, stages), np.uint16 if wide else np.uint8)
    dused = ctx.empty(n, np.uint8)
    drec = ctx.empty((n, dim), np.uint16)
    (ctx.rvq_encode_u16 if wide else ctx.rvq_encode)(metric, dx, n, ld, dim, stages, k, dcb, eps, dcodes, dused, drec)
    used = dused.download()
    reached = wcodes != 0xFFFFFFFF
    assert np.array_equal(used, reached.sum(1))
    if eps == 4.5:
        assert used.min() < used.max()
    got = dcodes.download()
    assert np.array_equal(got[reached], wcodes[reached].astype(got.dtype))
    assert np.all(got[~reached] == 0)
    assert np.array_equal(drec.download(), wrec)
    assert np.array_equal(dx.download().view(np.uint32), buf.view(np.uint32))
    for b in (dx, dcb, dcodes, dused, drec):
        b.free()


def test_rvq_k1_and_early_training_stop(ctx):
    x = np.tile(np.array([[1, 2, 3, 4]], F), (20, 1))
    init = np.array([[0, 1], [0, 1], [0, 1]], np.uint32)
    reseed = np.zeros((3, 30), np.uint32)
    want = O.rvq_fit(O.SQEUCLIDEAN, x, 3, 2, 5, 0.01, init, reseed)
    cb, res, norms, _ = gpu_rvq_fit(ctx, O.SQEUCLIDEAN, x, 3, 2, 5, 0.01, init, reseed)
    assert len(cb) == want["stages"] == 1 and norms[0] == 0.0
    assert np.array_equal(cb, want["codebooks"])
    rng = np.random.default_rng(22)
    x = rng.standard_normal((30, 3)).astype(F)
    init1, reseed1 = np.array([[4], [5]], np.uint32), np.zeros((2, 3), np.uint32)
    want = O.rvq_fit(O.COSINE, x, 2, 1, 3, 0.0, init1, reseed1)
    cb, res, _, _ = gpu_rvq_fit(ctx, O.COSINE, x, 2, 1, 3, 0.0, init1, reseed1)
    assert np.array_equal(cb, want["codebooks"]) and np.array_equal(res, want["residuals"])


# ---- OPQ pieces -------------------------------------------------------------------------------
@pytest.mark.parametrize("n,dim", [(1000, 10), (4097, 128), (300, 64), (70, 33), (129, 256), (5000, 32), (2500, 96),
                                   (3001, 160), (1111, 224), (300001, 64)])
def test_rotate_matches_matrix_product(ctx, n, dim):
    rng = np.random.default_rng(dim)
    x = rng.standard_normal((n, dim)).astype(F)
    Q, _ = np.linalg.qr(rng.standard_normal((dim, dim)))
    R = Q.astype(F)
    dx, dR, dy = ctx.to_device(x), ctx.to_device(R), ctx.empty((n, dim), F)
    ctx.rotate(dx, n, dim, dim, dR, dy)
    y = dy.download()
    exact = x.astype(np.float64) @ R.astype(np.float64).T
    # f32 accumulation of dim products: tolerance 1e-5 relative to the row norm
    assert np.abs(y - exact).max() <= 1e-5 * np.abs(exact).max()
    assert np.abs(y - O.rotate(x, R)).max() <= 1e-5 * np.abs(exact).max()
    ctx.rotate(dx, n, dim, dim, ctx.to_device(np.eye(dim, dtype=F)), dy)
    assert np.array_equal(dy.download(), x)  # identity is exact (opq.rs:119-121)


@pytest.mark.parametrize("n,dim", [(1000, 10), (5000, 128), (2049, 32), (4099, 16), (2050, 80), (777, 20),
                                   (9000, 256), (5000, 144), (3000, 200), (2100, 135), (10000, 384)])
def test_cross_cov_matches_f64_product(ctx, n, dim):
    rng = np.random.default_rng(n)
    x = rng.standard_normal((n, dim)).astype(F)
    y = rng.standard_normal((n, dim)).astype(F)
    A = ctx.cross_cov(ctx.to_device(y), ctx.to_device(x), n, dim)
    exact = y.astype(np.float64).T @ x.astype(np.float64)
    assert np.allclose(A, exact, rtol=1e-12, atol=1e-10)
    # deterministic: the same call gives the same bits
    assert np.array_equal(A, ctx.cross_cov(ctx.to_device(y), ctx.to_device(x), n, dim))


@pytest.mark.parametrize("dim", [2, 4, 10, 16, 64, 128])
def test_procrustes_rotation_is_the_polar_factor(ctx, dim):
    """The device rotation update (src/opq.rs:180-183: R = V U^T of svd(A)) against what the
    mathematics fixes: R is orthogonal, R A is symmetric positive semi-definite with trace equal
    to the nuclear norm of A, an orthogonal A gives A^T; and against the oracle's host SVD."""
    rng = np.random.default_rng(dim)
    A = (rng.standard_normal((dim, dim)) @ np.diag(rng.uniform(0.1, 50.0, dim))
         @ rng.standard_normal((dim, dim))).astype(F).astype(np.float64)
    R = ctx.procrustes_rotation(A)
    assert np.allclose(R.T @ R, np.eye(dim), atol=1e-11)
    P = R @ A
    assert np.allclose(P, P.T, atol=1e-9 * np.abs(A).max())
    assert np.linalg.eigvalsh((P + P.T) / 2).min() > -1e-9 * np.abs(A).max()
    assert abs(np.trace(P) - np.linalg.svd(A, compute_uv=False).sum()) <= 1e-10 * np.abs(P).sum()
    assert np.allclose(R, O.procrustes(A), atol=1e-9)
    Q, _ = np.linalg.qr(rng.standard_normal((dim, dim)))
    assert np.allclose(ctx.procrustes_rotation(Q), Q.T, atol=1e-12)
    # a zero matrix determines no singular vector: the completion gives the identity (U = V = I,
    # as an SVD library returns), not a rank-deficient R
    assert np.array_equal(ctx.procrustes_rotation(np.zeros((dim, dim))), np.eye(dim))


@pytest.mark.parametrize("dim", [2, 5, 16, 40, 128, 130, 200])
@pytest.mark.parametrize("cond", [1.0, 50.0, 1e4, 1e6])
def test_procrustes_rotation_newton_schulz_and_svd_agree(ctx, dim, cond):
    """The two ways to R = V U^T (src/opq.rs:180-183) — Newton-Schulz steps to the polar factor of
    A^T on the f64 matrix cores (the default) and the one-sided Jacobi SVD — on matrices of a given
    condition number, against each other, against numpy's SVD and against the polar-factor
    properties.  The polar factor moves by about eps * cond under rounding, whichever way it is
    computed, so the tolerance follows cond."""
    rng = np.random.default_rng(1000 * dim + int(np.log10(cond)))
    U, _ = np.linalg.qr(rng.standard_normal((dim, dim)))
    V, _ = np.linalg.qr(rng.standard_normal((dim, dim)))
    sv = np.geomspace(1.0, 1.0 / cond, dim) * 37.0
    A = (U * sv) @ V.T
    tol = 1e-11 + 3e-15 * cond
    ctx.set_procrustes_path(1)
    R_svd = ctx.procrustes_rotation(A)
    ctx.set_procrustes_path(0)
    R = ctx.procrustes_rotation(A)
    u, _, vt = np.linalg.svd(A)
    assert np.abs(R - vt.T @ u.T).max() <= tol
    assert np.abs(R - R_svd).max() <= tol
    assert np.abs(R.T @ R - np.eye(dim)).max() <= 1e-11
    P = R @ A
    assert np.abs(P - P.T).max() <= 1e-9 * np.abs(A).max()
    assert np.array_equal(R, ctx.procrustes_rotation(A))  # deterministic


def test_procrustes_rotation_that_newton_schulz_cannot_take_falls_to_the_svd(ctx):
    """Singular, nearly singular (condition number 1e13) and non-finite matrices leave the
    Newton-Schulz steps without convergence; the SVD path answers, as it does when it is the only
    path."""
    rng = np.random.default_rng(5)
    dim = 64
    U, _ = np.linalg.qr(rng.standard_normal((dim, dim)))
    V, _ = np.linalg.qr(rng.standard_normal((dim, dim)))
    for sv in (np.geomspace(1.0, 1e-13, dim), np.r_[np.ones(dim - 3), np.zeros(3)]):
        A = (U * sv) @ V.T
        ctx.set_procrustes_path(1)
        want = ctx.procrustes_rotation(A)
        ctx.set_procrustes_path(0)
        got = ctx.procrustes_rotation(A)
        assert np.array_equal(got, want)
        assert np.abs(got.T @ got - np.eye(dim)).max() <= 1e-10


@pytest.mark.parametrize("dim,rank", [(4, 2), (16, 10), (64, 63), (128, 100), (7, 3), (130, 60)])
def test_procrustes_rotation_of_a_singular_matrix_is_orthogonal(ctx, dim, rank):
    """Directions that A leaves open (zero singular values; an all-zero column such as a padded
    dimension) are completed to an orthonormal basis: R stays orthogonal and optimal.  Even sizes
    up to 128 run the device SVD, the others the host routine inside the library."""
    rng = np.random.default_rng(dim + rank)
    A = rng.standard_normal((dim, rank)) @ rng.standard_normal((rank, dim))
    for M in (A, np.where(np.arange(dim) == dim - 1, 0.0, rng.standard_normal((dim, dim)))):
        R = ctx.procrustes_rotation(M)
        assert np.allclose(R.T @ R, np.eye(dim), atol=1e-10)
        P = R @ M
        assert np.allclose(P, P.T, atol=1e-8 * np.abs(M).max())
        assert abs(np.trace(P) - np.linalg.svd(M, compute_uv=False).sum()) <= 1e-9 * np.abs(P).sum()


@pytest.mark.parametrize("dim", [3, 9, 130, 200])
def test_procrustes_rotation_sizes_outside_the_device_kernel(ctx, dim):
    rng = np.random.default_rng(dim)
    A = rng.standard_normal((dim, dim))
    R = ctx.procrustes_rotation(A)
    assert np.allclose(R.T @ R, np.eye(dim), atol=1e-10)
    assert np.allclose(R, O.procrustes(A), atol=1e-9)


def test_opq_outer_iteration_stepwise(ctx):
    """One OPQ outer iteration (src/opq.rs:124-195) on the GPU, every step checked against the
    oracle on identical inputs; the rotation's rounding is the only tolerance."""
    rng = np.random.default_rng(43)
    n, dim, m, k, iters = 3000, 16, 4, 16, 6
    sd = dim // m
    x = (rng.standard_normal((n, dim)) @ rng.standard_normal((dim, dim))).astype(F)
    init, reseed = data.index_streams(n, m, k, iters, seed=5)
    dx = ctx.to_device(x)
    drot = ctx.empty((n, dim), F)
    ctx.copy_f32(drot, dx, n * dim)
    dcb = ctx.empty((m, k, sd), F)
    dcodes = ctx.empty((n, m), np.uint8)
    drec = ctx.empty((n, dim), F)
    R = np.eye(dim, dtype=F)
    for outer in range(2):
        rot = drot.download()
        ctx.lbg_fit(drot, n, dim, m, sd, k, iters, init, reseed, dcb)
        want_cb = O.pq_fit(rot, m, k, iters, init, reseed)["codebooks"]
        assert np.array_equal(dcb.download(), want_cb)
        ctx.assign(O.EUCLIDEAN, drot, n, dim, m, sd, k, dcb, dcodes)
        want_codes = O.pq_encode(O.EUCLIDEAN, rot, want_cb)
        assert np.array_equal(dcodes.download(), want_codes.astype(np.uint8))
        ctx.decode_f32(dcodes, n, m, sd, k, dcb, drec)
        rec = np.concatenate([want_cb[s][want_codes[:, s]] for s in range(m)], 1)
        assert np.array_equal(drec.download(), rec)
        A = ctx.cross_cov(drec, drot, n, dim)
        assert np.allclose(A, rec.astype(np.float64).T @ rot.astype(np.float64), rtol=1e-12, atol=1e-9)
        Rd = O.procrustes(A.astype(F).astype(np.float64))
        assert np.allclose(Rd.T @ Rd, np.eye(dim), atol=1e-10)
        R = Rd.astype(F)
        ctx.rotate(dx, n, dim, dim, ctx.to_device(R), drot)
        assert np.abs(drot.download() - O.rotate(x, R)).max() <= 1e-5 * np.abs(x).max() * np.sqrt(dim)
    # the quantizer that fit returns: codebooks of the last iteration, rotation R_T; encode
    dy = ctx.empty((n, dim), F)
    ctx.rotate(dx, n, dim, dim, ctx.to_device(R), dy)
    ctx.assign(O.EUCLIDEAN, dy, n, dim, m, sd, k, dcb, dcodes)
    want = O.pq_encode(O.EUCLIDEAN, dy.download(), dcb.download())
    assert np.array_equal(dcodes.download(), want.astype(np.uint8))
