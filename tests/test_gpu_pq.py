"""GPU parity: LBG training and PQ encode through the C ABI against the CPU oracle.
Integer outputs (codes) and trained centroids are compared bit for bit."""
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


def gpu_lbg(ctx, x, m, k, iters, init, reseed):
    n, dim = x.shape
    sd = dim // m
    dx = ctx.to_device(x)
    dcb = ctx.empty((m, k, sd), F)
    it, used = ctx.lbg_fit(dx, n, dim, m, sd, k, iters, init, reseed, dcb)
    return dcb.download(), it, used, dx, dcb


def gpu_encode(ctx, metric, dx, n, dim, m, k, dcb):
    dcodes = ctx.empty((n, m), np.uint8)
    ctx.assign(metric, dx, n, dim, m, dim // m, k, dcb, dcodes)
    return dcodes.download()


LBG_CASES = [
    # n, dim, m, k, iters, kind
    (1000, 10, 2, 2, 50, "wide"),      # the reference's own test shape (tests/test_pq.rs)
    (64, 8, 1, 4, 5, "normal"),
    (300, 16, 2, 16, 8, "normal"),
    (257, 8, 1, 256, 3, "normal"),     # k close to n -> empty clusters and re-seeds
    (5000, 32, 4, 64, 6, "uniform"),
    (700, 6, 3, 7, 10, "grid"),        # integer grid: exact distance ties, duplicate rows
    (100, 4, 1, 8, 10, "same"),        # all rows equal: everything in cluster 0, k-1 re-seeds
    (3000, 2, 1, 2, 6, "normal"),      # clusters above 1024 members -> midpoint tree
    (9000, 4, 2, 3, 5, "normal"),      # depth-2 trees
    (400, 7, 1, 5, 6, "normal"),       # sub_dim without a register kernel
    (400, 40, 2, 9, 4, "normal"),      # sub_dim 20
    (300, 256, 1, 16, 3, "normal"),    # full-dimension problem (RVQ stage shape)
    (2049, 3, 3, 1, 4, "normal"),      # k = 1, sub_dim 1
    (50, 8, 1, 4, 0, "normal"),        # max_iters = 0 -> initial rows
    (50000, 32, 4, 8, 4, "normal"),    # sub_dim 8: every cluster large -> streaming part sums
    (30000, 32, 4, 24, 4, "skewed"),   # sub_dim 8: small and large clusters side by side
    (70000, 16, 2, 3, 3, "same"),      # sub_dim 8: one huge cluster, empties re-seeded
    (13000, 24, 3, 5, 3, "normal"),    # sub_dim 8 but m % 4 != 0 -> per-part leaves, gather path
    (13000, 6, 1, 4, 3, "normal"),     # sub_dim 6, clusters above 1024 -> per-part leaves
    (300001, 32, 4, 256, 2, "normal"), # sub_dim 8: a workgroup of the assignment walks over several runs of rows
    (4200000, 2, 1, 5, 2, "normal"),   # 1026 parts of 4096 rows in 33 scan segments (the plan walks them eight at a time)
    (4200000, 8, 1, 3, 2, "uniform"),  # the same at sub_dim 8 without the streaming sums (m % 4 != 0)
]


@pytest.mark.parametrize("n,dim,m,k,iters,kind", LBG_CASES)
def test_lbg_fit_matches_oracle_bitwise(ctx, n, dim, m, k, iters, kind):
    rng = np.random.default_rng(n * 31 + dim)
    if kind == "normal":
        x = rng.standard_normal((n, dim)).astype(F)
    elif kind == "uniform":
        x = rng.random((n, dim), dtype=F)
    elif kind == "wide":
        x = rng.uniform(-1000, 1000, (n, dim)).astype(F)  # tests/utils.rs:9-10
    elif kind == "grid":
        x = np.round(rng.standard_normal((n, dim)) * 1.5).astype(F)
    elif kind == "skewed":  # a few tight far-away blobs with few rows + one broad mass
        x = rng.standard_normal((n, dim)).astype(F)
        for b in range(6):
            x[b * 150:(b + 1) * 150] = (20.0 * (b + 1) + 0.01 * rng.standard_normal((150, dim))).astype(F)
        x = x[rng.permutation(n)]
    else:
        x = np.tile(rng.standard_normal((1, dim)).astype(F), (n, 1))
    init, reseed = data.index_streams(n, m, k, iters, seed=n)
    want = O.pq_fit(x, m, k, iters, init, reseed)
    assert want["rc"] == 0
    got, it, used, _, _ = gpu_lbg(ctx, x, m, k, iters, init, reseed)
    assert np.array_equal(it, want["iters"])
    assert np.array_equal(used, want["reseeds"])
    assert np.array_equal(got.view(np.uint32), want["codebooks"].view(np.uint32))


def test_column_blocks_of_one_group_stop_at_different_iterations(ctx):
    """src/utils.rs:104-106 per column block: blocks 0 and 2 of a group of four hold constant rows and
    stop after their first pass, blocks 1 and 3 go on (the group's streaming sums are one workgroup)."""
    rng = np.random.default_rng(77)
    n, dim, m, k, iters = 40000, 64, 8, 5, 6
    x = rng.standard_normal((n, dim)).astype(F)
    for s in (0, 2, 4, 5, 6, 7):
        x[:, 8 * s:8 * s + 8] = x[0, 8 * s:8 * s + 8]
    init, reseed = data.index_streams(n, m, k, iters, seed=5)
    want = O.pq_fit(x, m, k, iters, init, reseed)
    assert want["rc"] == 0
    got, it, used, _, _ = gpu_lbg(ctx, x, m, k, iters, init, reseed)
    assert len(set(want["iters"][:4].tolist())) > 1 and want["iters"][4:].max() < iters
    assert np.array_equal(it, want["iters"])
    assert np.array_equal(used, want["reseeds"])
    assert np.array_equal(got.view(np.uint32), want["codebooks"].view(np.uint32))


@pytest.mark.parametrize("metric", [O.SQEUCLIDEAN, O.EUCLIDEAN, O.COSINE, O.MANHATTAN])
@pytest.mark.parametrize("n,dim,m,k,kind", [
    (1000, 128, 16, 256, "uniform"),
    (777, 10, 2, 2, "wide"),
    (500, 6, 3, 16, "grid"),
    (300, 21, 3, 11, "normal"),
    (200, 256, 1, 37, "normal"),
    (130, 64, 2, 256, "normal"),
    (65, 12, 1, 3, "zeros"),
])
def test_assign_matches_oracle_bitwise(ctx, metric, n, dim, m, k, kind):
    rng = np.random.default_rng(n + 7 * metric)
    if kind == "uniform":
        x = rng.random((n, dim), dtype=F)
        cb = rng.random((m, k, dim // m), dtype=F)
    elif kind == "wide":
        x = rng.uniform(-1000, 1000, (n, dim)).astype(F)
        cb = rng.uniform(-1000, 1000, (m, k, dim // m)).astype(F)
    elif kind == "grid":
        x = np.round(rng.standard_normal((n, dim)) * 2).astype(F)
        cb = np.round(rng.standard_normal((m, k, dim // m)) * 2).astype(F)
    elif kind == "zeros":  # zero-norm rows and centroids (cosine returns 1)
        x = rng.standard_normal((n, dim)).astype(F)
        x[::3] = 0
        cb = rng.standard_normal((m, k, dim // m)).astype(F)
        cb[:, 1] = 0
    else:
        x = rng.standard_normal((n, dim)).astype(F)
        cb = rng.standard_normal((m, k, dim // m)).astype(F)
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    got = gpu_encode(ctx, metric, dx, n, dim, m, k, dcb)
    want = O.pq_encode(metric, x, cb)
    assert np.array_equal(got, want.astype(np.uint8))


def test_euclidean_sqrt_collisions_on_gpu(ctx):
    # many candidates whose squared distances differ in the last bits: the sqrt of several of
    # them coincide and the earlier index must win (src/distances.rs:134-140 + strict '<').
    rng = np.random.default_rng(99)
    n, k = 4096, 256
    x = np.zeros((n, 2), F)
    x[:, 0] = rng.random(n, dtype=F) * F(1e-3)
    b = (0.5 + rng.random(k) * 2e-5).astype(F)
    cb = np.stack([np.ones(k, F), b], 1)[None]  # m = 1, k x 2
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    sq = gpu_encode(ctx, O.SQEUCLIDEAN, dx, n, 2, 1, k, dcb)
    eu = gpu_encode(ctx, O.EUCLIDEAN, dx, n, 2, 1, k, dcb)
    want_sq = O.pq_encode(O.SQEUCLIDEAN, x, cb).astype(np.uint8)
    want_eu = O.pq_encode(O.EUCLIDEAN, x, cb).astype(np.uint8)
    assert np.array_equal(sq, want_sq) and np.array_equal(eu, want_eu)
    assert np.count_nonzero(want_sq != want_eu) > 50  # the case is exercised


def test_config1_pq_fit_encode_decode(ctx):
    """PQ on 10,000 x 128 U[0,1) rows, seed 42, m=16, k=256, 10 iterations, Euclidean."""
    n, dim, m, k, iters = 10000, 128, 16, 256, 10
    x = data.uniform(n, dim, 42)
    init, reseed = data.index_streams(n, m, k, iters, seed=42)
    want = O.pq_fit_encode(O.EUCLIDEAN, x, m, k, iters, init, reseed, threads=8)
    got_cb, it, used, dx, dcb = gpu_lbg(ctx, x, m, k, iters, init, reseed)
    assert np.array_equal(got_cb.view(np.uint32), want["codebooks"].view(np.uint32))
    codes = gpu_encode(ctx, O.EUCLIDEAN, dx, n, dim, m, k, dcb)
    assert np.array_equal(codes, want["codes"].astype(np.uint8))
    drec = ctx.empty((n, dim), np.uint16)
    dcodes = ctx.to_device(codes)
    ctx.decode_f16(dcodes, n, m, dim // m, k, dcb, drec)
    rec = drec.download()
    assert np.array_equal(rec, O.pq_decode_f16(want["codes"], want["codebooks"]))
    mse = O.mse_f16(x, rec)
    assert abs(mse - 0.019639) < 4e-4  # notebooks/performance_analysis.ipynb:398,405


def test_errors_match_reference_panics(ctx):
    import vq_amd
    x = ctx.to_device(np.zeros((4, 8), F))
    cb = ctx.empty((1, 8, 8), F)
    with pytest.raises(vq_amd.VqError, match="k must be greater than 0") as e:
        ctx.lbg_fit(x, 4, 8, 1, 8, 0, 3, np.zeros(1, np.uint32), np.zeros(1, np.uint32), cb)
    assert e.value.code == -1
    with pytest.raises(vq_amd.VqError, match="Not enough data points for k clusters"):
        ctx.lbg_fit(x, 4, 8, 1, 8, 8, 3, np.zeros(8, np.uint32), np.zeros(8, np.uint32), cb)
    with pytest.raises(vq_amd.VqError, match="Empty input"):
        ctx.lbg_fit(x, 0, 8, 1, 8, 2, 3, np.zeros(2, np.uint32), np.zeros(2, np.uint32), cb)
    with pytest.raises(vq_amd.VqError, match="Dimension mismatch"):
        ctx.assign(0, x, 4, 8, 2, 8, 2, cb, ctx.empty((4, 2), np.uint8))


# ---- matrix-core assignment path vs vector-ALU path ---------------------------------------------
@pytest.mark.parametrize("metric", [O.SQEUCLIDEAN, O.EUCLIDEAN])
@pytest.mark.parametrize("n,m,k,kind", [
    (5000, 16, 256, "uniform"), (1000, 16, 256, "mixture"), (700, 4, 100, "normal"),
    (513, 1, 1, "normal"), (64, 2, 33, "grid"), (2000, 16, 256, "offset"), (300, 3, 7, "same"),
    (900, 16, 256, "nonfinite"),
    # enough rows for a workgroup to walk over several runs of rows, the last one partial
    (200001, 4, 256, "uniform"), (150001, 3, 200, "normal"),
])
def test_mfma_path_equals_oracle_and_valu_path(ctx, metric, n, m, k, kind):
    """sub_dim 8: the default path is the matrix-core pass + exact re-check.  It must give the
    oracle's codes bit for bit on ties, near ties, offsets that blow up the error bound,
    padding (k not a multiple of 32) and non-finite values."""
    rng = np.random.default_rng(n + k)
    dim = 8 * m
    if kind == "uniform":
        x, cb = rng.random((n, dim), dtype=F), rng.random((m, k, 8), dtype=F)
    elif kind == "mixture":
        x = data.gaussian_mixture(n, dim, 64, 0.05, seed=1)
        cb = x[rng.choice(n, k, replace=False)].reshape(k, m, 8).transpose(1, 0, 2).copy()
    elif kind == "grid":
        x = np.round(rng.standard_normal((n, dim))).astype(F)
        cb = np.round(rng.standard_normal((m, k, 8))).astype(F)
    elif kind == "offset":  # far from the origin: scored relative to the block's centre, so still few re-checks
        x = (1000 + rng.random((n, dim))).astype(F)
        cb = (1000 + rng.random((m, k, 8))).astype(F)
    elif kind == "same":
        x = np.tile(rng.standard_normal((1, dim)).astype(F), (n, 1))
        cb = np.tile(x[:1].reshape(m, 1, 8), (1, k, 1)).copy()
    elif kind == "nonfinite":
        x, cb = rng.random((n, dim), dtype=F), rng.random((m, k, 8), dtype=F)
        x[::7, 3] = np.inf
        x[1::11, 9] = np.nan
        x[2::13, 20] = 1e30
        cb[1, 5, 2] = np.nan
        cb[2, 0, :] = np.nan  # NaN at index 0 can never be displaced (strict '<')
        cb[3, 9, 1] = -np.inf
    else:
        x, cb = rng.standard_normal((n, dim)).astype(F), rng.standard_normal((m, k, 8)).astype(F)
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    with np.errstate(all="ignore"):
        want = O.pq_encode(metric, x, cb).astype(np.uint8)
    ctx.set_assign_path(0)
    got = gpu_encode(ctx, metric, dx, n, dim, m, k, dcb)
    frac = ctx.last_recheck_count() / float(n * m)
    ctx.set_assign_path(1)
    valu = gpu_encode(ctx, metric, dx, n, dim, m, k, dcb)
    ctx.set_assign_path(0)
    assert np.array_equal(valu, want)
    assert np.array_equal(got, want)
    if kind in ("normal", "uniform", "offset") and k > 1:
        assert frac < 0.05, frac  # the matrix-core pass decides almost every row itself


@pytest.mark.parametrize("metric", [O.SQEUCLIDEAN, O.EUCLIDEAN])
@pytest.mark.parametrize("n,m,k", [(3000, 4, 256), (1500, 3, 255), (800, 8, 6), (2100, 1, 37), (5000, 16, 254)])
def test_ties_and_near_ties_inside_a_run_of_four_centroids(ctx, metric, n, m, k):
    """The matrix-core pass keeps one key per run of four consecutive centroids and picks inside the
    best run by exact distances.  Duplicates and neighbours one ulp apart inside a run (in one lane
    half: 4j and 4j + 1; across the halves: 4j + 1 and 4j + 2), a codebook that ends inside a run,
    and rows that sit exactly on centroids: the oracle's first-smallest choice, and few rows that
    need the full reference-order scan."""
    rng = np.random.default_rng(100 * n + k)
    dim = 8 * m
    cb = rng.standard_normal((m, k, 8)).astype(F)
    for j in range(0, k - 3, 8):
        cb[:, j + 1] = cb[:, j]                                   # exact tie inside a lane half
        cb[:, j + 2] = np.nextafter(cb[:, j + 1], F(np.inf))      # one ulp away, across the halves
    if k % 4 >= 2:
        cb[:, k - 1] = cb[:, k - 2]                               # a tie in the last, partial run
    x = rng.standard_normal((n, dim)).astype(F)
    pick = rng.integers(0, k, n // 2)
    x[: n // 2] = cb[:, pick].transpose(1, 0, 2).reshape(n // 2, dim)   # rows on centroids
    x[: n // 4] += (rng.standard_normal((n // 4, dim)) * 1e-4).astype(F)
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    want = O.pq_encode(metric, x, cb).astype(np.uint8)
    ctx.set_assign_path(0)
    got = gpu_encode(ctx, metric, dx, n, dim, m, k, dcb)
    frac = ctx.last_recheck_count() / float(n * m)
    assert np.array_equal(got, want)
    assert frac < 0.05, frac


def test_lbg_fit_same_result_on_both_assignment_paths(ctx):
    n, dim, m, k, iters = 20000, 128, 16, 256, 5
    x = data.gaussian_mixture(n, dim, 256, 0.05, seed=1)
    init, reseed = data.index_streams(n, m, k, iters, seed=11)
    ctx.set_assign_path(1)
    a, it_a, used_a, _, _ = gpu_lbg(ctx, x, m, k, iters, init, reseed)
    ctx.set_assign_path(0)
    b, it_b, used_b, _, _ = gpu_lbg(ctx, x, m, k, iters, init, reseed)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(it_a, it_b) and np.array_equal(used_a, used_b)
    want = O.pq_fit(x, m, k, iters, init, reseed)
    assert np.array_equal(b.view(np.uint32), want["codebooks"].view(np.uint32))


@pytest.mark.parametrize("metric", [O.SQEUCLIDEAN, O.EUCLIDEAN])
@pytest.mark.parametrize("n,m,sd,k,kind", [
    (3000, 1, 256, 256, "normal"), (1000, 2, 64, 100, "uniform"), (513, 4, 16, 33, "grid"),
    (700, 1, 128, 256, "offset"), (300, 1, 24, 7, "same"), (640, 1, 256, 64, "nonfinite"),
    (257, 3, 32, 1, "normal"),
    # long lists of rows for the all-centroid check in a single column block (eight rows per workgroup)
    (5000, 1, 40, 100, "offset"), (20000, 1, 256, 256, "offset"), (3000, 1, 72, 256, "same"),
    (2500, 1, 136, 255, "nonfinite"),
])
def test_wide_mfma_path_equals_oracle_and_valu_path(ctx, metric, n, m, sd, k, kind):
    """sub_dim a multiple of 8 above 8 (RVQ stages use the full dimension): chunked matrix-core
    contraction + exact re-check must give the oracle's codes bit for bit."""
    rng = np.random.default_rng(n + k + sd)
    dim = sd * m
    if kind == "uniform":
        x, cb = rng.random((n, dim), dtype=F), rng.random((m, k, sd), dtype=F)
    elif kind == "grid":
        x = np.round(rng.standard_normal((n, dim))).astype(F)
        cb = np.round(rng.standard_normal((m, k, sd))).astype(F)
    elif kind == "offset":
        x = (100 + rng.random((n, dim))).astype(F)
        cb = (100 + rng.random((m, k, sd))).astype(F)
    elif kind == "same":
        x = np.tile(rng.standard_normal((1, dim)).astype(F), (n, 1))
        cb = np.tile(x[:1].reshape(m, 1, sd), (1, k, 1)).copy()
    elif kind == "nonfinite":
        x, cb = rng.random((n, dim), dtype=F), rng.random((m, k, sd), dtype=F)
        x[::7, 3] = np.inf
        x[1::11, 9] = np.nan
        x[2::13, 20] = 1e30
        cb[0, 5, 2] = np.nan
        cb[0, 9, 1] = -np.inf
    else:
        x, cb = rng.standard_normal((n, dim)).astype(F), rng.standard_normal((m, k, sd)).astype(F)
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    with np.errstate(all="ignore"):
        want = O.pq_encode(metric, x, cb).astype(np.uint8)
    ctx.set_assign_path(0)
    got = gpu_encode(ctx, metric, dx, n, dim, m, k, dcb)
    frac = ctx.last_recheck_count() / float(n * m)
    ctx.set_assign_path(1)
    valu = gpu_encode(ctx, metric, dx, n, dim, m, k, dcb)
    ctx.set_assign_path(0)
    assert np.array_equal(valu, want)
    assert np.array_equal(got, want)
    if kind in ("normal", "uniform", "offset") and k > 1:
        assert frac < 0.05, frac  # the matrix-core pass decides almost every row itself


@pytest.mark.parametrize("sd,m,k", [(8, 4, 64), (8, 16, 256), (32, 2, 100), (6, 3, 9)])
@pytest.mark.parametrize("pad,shift", [(0, 0), (1, 0), (3, 1), (4, 0), (6, 2)])
def test_rows_with_leading_dimension_and_offset(ctx, sd, m, k, pad, shift):
    """Rows inside a wider buffer (ld > dim) that starts `shift` floats into the allocation: the
    matrix-core kernels take 16-byte pieces of the rows where they can and must give the same
    codes and centroids when the rows are not 16-byte aligned."""
    n, dim = 3000, sd * m
    ld = dim + pad + shift
    rng = np.random.default_rng(sd * 100 + pad * 10 + shift)
    buf = rng.standard_normal((n, ld)).astype(F)
    x = np.ascontiguousarray(buf[:, shift:shift + dim])
    cb = np.ascontiguousarray(x[rng.choice(n, k, replace=False)].reshape(k, m, sd).transpose(1, 0, 2))
    dbuf, dcb = ctx.to_device(buf), ctx.to_device(cb)
    dcodes = ctx.empty((n, m), np.uint8)
    for metric in (O.SQEUCLIDEAN, O.EUCLIDEAN):
        want = O.pq_encode(metric, x, cb).astype(np.uint8)
        ctx.assign(metric, dbuf.ptr + 4 * shift, n, ld, m, sd, k, dcb, dcodes)
        assert np.array_equal(dcodes.download(), want)
    init, reseed = data.index_streams(n, m, k, 3, seed=pad + shift)
    w = O.pq_fit(x, m, k, 3, init, reseed)
    assert w["rc"] == 0
    dcb2 = ctx.empty((m, k, sd), F)
    it, _ = ctx.lbg_fit(dbuf.ptr + 4 * shift, n, ld, m, sd, k, 3, init, reseed, dcb2)
    assert np.array_equal(it, w["iters"])
    assert np.array_equal(dcb2.download().view(np.uint32), w["codebooks"].view(np.uint32))


def test_leading_dimension_beyond_the_kernels_32_bit_offsets(ctx):
    """A row stride above 2^20 floats: the matrix-core assignment and the streaming sums address a
    run of rows with 32-bit offsets and leave such input to the other kernels; codes and centroids
    are the oracle's all the same.  The rows sit in a device buffer that is mostly never written."""
    n, sd, m, k, ld = 130, 8, 4, 16, (1 << 20) + 8
    dim = sd * m
    rng = np.random.default_rng(5)
    x = rng.standard_normal((n, dim)).astype(F)
    from vq_amd import _ffi
    dbuf = ctx.empty((n, ld), F)
    for i in range(n):  # row i of the wide buffer
        row = np.ascontiguousarray(x[i])
        ctx._check(_ffi.lib().vq_h2d(ctx._h, dbuf.ptr + 4 * i * ld, row.ctypes.data, row.nbytes))
    cb = np.ascontiguousarray(x[rng.choice(n, k, replace=False)].reshape(k, m, sd).transpose(1, 0, 2))
    dcb = ctx.to_device(cb)
    dcodes = ctx.empty((n, m), np.uint8)
    for metric in (O.SQEUCLIDEAN, O.EUCLIDEAN):
        want = O.pq_encode(metric, x, cb).astype(np.uint8)
        ctx.assign(metric, dbuf, n, ld, m, sd, k, dcb, dcodes)
        assert np.array_equal(dcodes.download(), want)
    init, reseed = data.index_streams(n, m, k, 3, seed=11)
    w = O.pq_fit(x, m, k, 3, init, reseed)
    assert w["rc"] == 0
    dcb2 = ctx.empty((m, k, sd), F)
    it, _ = ctx.lbg_fit(dbuf, n, ld, m, sd, k, 3, init, reseed, dcb2)
    assert np.array_equal(it, w["iters"])
    assert np.array_equal(dcb2.download().view(np.uint32), w["codebooks"].view(np.uint32))


@pytest.mark.parametrize("path", [0, 1])
def test_timing_classes_count_every_pass(ctx, path):
    """The per-class timers (measurement only): a fit of `iters` passes yields `iters` spans of the
    assignment kernel, of the assignment class and of the update class, an encode one span more of
    the kernel and one of the encode class — on the matrix-core path, where the events ride on the
    kernel's dispatch, and on the vector path, where they are recorded around the launches — and
    timing leaves the results as they are."""
    import vq_amd
    n, dim, m, k, iters = 20000, 64, 8, 64, 4
    x = data.gaussian_mixture(n, dim, 4 * k, 0.05, seed=9)
    init, reseed = data.index_streams(n, m, k, iters, seed=9)
    ctx.set_assign_path(path)
    try:
        plain, _, _, dx, dcb = gpu_lbg(ctx, x, m, k, iters, init, reseed)
        ctx.prof_enable(True)
        for _ in range(2):  # twice: the events of the first fit are reused by the second
            timed, it, _, dx, dcb = gpu_lbg(ctx, x, m, k, iters, init, reseed)
        codes = gpu_encode(ctx, vq_amd.EUCLIDEAN, dx, n, dim, m, k, dcb)
        spans = {c: ctx.prof_read(c) for c in (vq_amd._ffi.PROF_LBG_ASSIGN, vq_amd._ffi.PROF_LBG_UPDATE,
                                              vq_amd._ffi.PROF_ENCODE, vq_amd._ffi.PROF_ASSIGN_KERNEL)}
    finally:
        ctx.prof_enable(False)
        ctx.set_assign_path(0)
    assert np.array_equal(plain.view(np.uint32), timed.view(np.uint32)) and int(it.max()) == iters
    assert spans[vq_amd._ffi.PROF_LBG_ASSIGN][1] == 2 * iters
    assert spans[vq_amd._ffi.PROF_LBG_UPDATE][1] == 2 * iters
    assert spans[vq_amd._ffi.PROF_ASSIGN_KERNEL][1] == 2 * iters + 1
    assert spans[vq_amd._ffi.PROF_ENCODE][1] == 1
    assert all(ms > 0.0 for ms, _ in spans.values())
    assert spans[vq_amd._ffi.PROF_ASSIGN_KERNEL][0] <= spans[vq_amd._ffi.PROF_LBG_ASSIGN][0] + spans[vq_amd._ffi.PROF_ENCODE][0] + 1e-3
    assert codes.shape == (n, m)


def test_calibration_reports_plausible_peaks(ctx):
    """vq_calibrate (measurement only): the plain copy kernel's rate lies between a tenth of and the
    whole published HBM peak (read + write), a vector instruction costs between 1 and 16 cycles of a
    2.4 GHz SIMD, and the three-input integer operations are not faster than a plain add."""
    copy = ctx.calibrate(0)
    assert 800.0 < copy < 8000.0, copy
    simds = 256 * 4
    rates = {kind: ctx.calibrate(kind) for kind in (1, 2, 3, 4, 5)}
    for kind, r in rates.items():
        cycles = 2.4e9 * simds / r
        assert 1.0 < cycles < 16.0, (kind, cycles)
    assert rates[2] <= 1.05 * rates[5] and rates[4] <= 1.05 * rates[5]
    with pytest.raises(Exception):
        ctx.calibrate(9)


def test_failures_forced_from_the_host_come_back_as_status_codes(ctx):
    """Error paths of the ABI, forced from the host (no kernel faults): an allocation no GPU can
    satisfy is VQ_ERR_OOM with the context still usable, and a re-seed stream that runs out is
    VQ_ERR_RESEED_EXHAUSTED (the reference draws from an endless RNG, src/utils.rs:100; the ABI
    takes a finite stream and must say when it was too short)."""
    import vq_amd
    with pytest.raises(vq_amd.VqError) as e:
        ctx.empty((1 << 46,), np.uint8)  # 64 TiB
    assert e.value.code == vq_amd._ffi.ERR_OOM
    # all rows equal: every row lands in cluster 0, clusters 1..3 are empty in the first update
    x = np.ones((64, 8), F)
    dx = ctx.to_device(x)
    dcb = ctx.empty((1, 4, 8), F)
    init = np.arange(4, dtype=np.uint32)[None]
    with pytest.raises(vq_amd.VqError) as e:
        ctx.lbg_fit(dx, 64, 8, 1, 8, 4, 3, init, np.zeros((1, 2), np.uint32), dcb)
    assert e.value.code == vq_amd._ffi.ERR_RESEED_EXHAUSTED
    with pytest.raises(vq_amd.VqError) as e:   # the generic update path (sub_dim 3) reports it too
        ctx.lbg_fit(ctx.to_device(np.ones((64, 3), F)), 64, 3, 1, 3, 4, 3, init, np.zeros((1, 1), np.uint32),
                    ctx.empty((1, 4, 3), F))
    assert e.value.code == vq_amd._ffi.ERR_RESEED_EXHAUSTED
    # the context survives both: the same fit with a stream that is long enough matches the oracle
    reseed = np.arange(12, dtype=np.uint32)[None] % 64
    ctx.lbg_fit(dx, 64, 8, 1, 8, 4, 3, init, reseed, dcb)
    want = O.lbg(x, 4, 3, init[0], reseed[0])
    assert np.array_equal(dcb.download()[0].view(np.uint32), want["centroids"].view(np.uint32))


@pytest.mark.parametrize("nbytes", [(64 << 20) - 4, 64 << 20, (64 << 20) + 4, (150 << 20) + 12345 * 4])
def test_large_upload_from_pageable_memory_is_exact(ctx, nbytes):
    """vq_h2d stages a pageable source of 64 MiB or more through page-locked chunks with several host
    threads: every byte must arrive, whatever the size relative to the chunks and the threads' slices."""
    n = nbytes // 4
    x = np.random.default_rng(nbytes % 997).integers(0, 2 ** 31, n, dtype=np.int64).astype(np.uint32).view(F)
    d = ctx.empty((n,), F)
    d.upload(x)
    assert np.array_equal(d.download().view(np.uint32), x.view(np.uint32))
    hx = ctx.host_empty((n,), F)   # page-locked source: one direct copy
    np.copyto(hx, x[::-1])
    d.upload(hx)
    assert np.array_equal(d.download().view(np.uint32), x[::-1].view(np.uint32))
    ctx.host_free(hx)
