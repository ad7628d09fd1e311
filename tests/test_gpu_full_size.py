"""GPU checks at the full sizes of the benchmark configurations (1,000,000 rows).

The oracle cannot train at these sizes in seconds, so every check is one that does not need it to:
an encode decides each row on its own, so a random sample of rows, encoded by the oracle with the
codebooks (or tree) that the GPU trained, must reproduce the GPU's codes bit for bit; one LBG
iteration and the tree build are cheap enough for the oracle on all rows and are compared bit for
bit; the rest are invariants of the algorithms (optimality of the chosen centroid, falling residual
norms, the residual chain, an orthogonal rotation, leaf counts) and equal bits on a second run."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import data
from tests.test_gpu_tsvq import assert_same_tree, bfs_order

pytestmark = pytest.mark.gpu
F = np.float32
N = 1_000_000


@pytest.fixture(scope="module")
def ctx():
    import vq_amd
    c = vq_amd.Context(0)
    yield c
    c.close()


def sample_rows(n, count, seed):
    """Random rows plus the first and the last one (the edges of the grid)."""
    idx = np.random.default_rng(seed).choice(n, count, replace=False)
    idx[0], idx[1] = 0, n - 1
    return np.sort(idx)


def test_pq_1m_x_128_fit_and_encode(ctx):
    """PQ at scale: 1,000,000 x 128 mixture rows (seed 1), m = 16, k = 256, 10 LBG iterations,
    Euclidean encode (src/pq.rs:79-129, 146-187)."""
    import vq_amd
    dim, m, k, iters, sd = 128, 16, 256, 10, 8
    x = data.gaussian_mixture(N, dim, 1024, 0.05, seed=1)
    init, reseed = data.index_streams(N, m, k, iters, seed=1)
    dx = ctx.to_device(x)
    dcb = ctx.empty((m, k, sd), F)
    dcodes = ctx.empty((N, m), np.uint8)

    # one LBG iteration on all rows: the oracle needs seconds; centroids bit for bit
    it, _ = ctx.lbg_fit(dx, N, dim, m, sd, k, 1, init, reseed, dcb)
    want = O.pq_fit(x, m, k, 1, init, reseed)
    assert np.array_equal(it, want["iters"])
    assert np.array_equal(dcb.download().view(np.uint32), want["codebooks"].view(np.uint32))

    # the full fit, twice: equal bits
    it, _ = ctx.lbg_fit(dx, N, dim, m, sd, k, iters, init, reseed, dcb)
    cb = dcb.download()
    ctx.assign(vq_amd.EUCLIDEAN, dx, N, dim, m, sd, k, dcb, dcodes)
    codes = dcodes.download()
    it2, _ = ctx.lbg_fit(dx, N, dim, m, sd, k, iters, init, reseed, dcb)
    ctx.assign(vq_amd.EUCLIDEAN, dx, N, dim, m, sd, k, dcb, dcodes)
    assert np.array_equal(it, it2) and int(it.max()) <= iters
    assert np.array_equal(cb.view(np.uint32), dcb.download().view(np.uint32))
    assert np.array_equal(codes, dcodes.download())
    assert np.isfinite(cb).all()

    # a sample of rows through the oracle's encode with the GPU's codebooks: bit for bit
    idx = sample_rows(N, 20000, 11)
    assert np.array_equal(codes[idx], O.pq_encode(O.EUCLIDEAN, x[idx], cb).astype(np.uint8))

    # the chosen centroid is a nearest one for every row of two column blocks (float64 distances,
    # slack for the f32 rounding of the sequential sums)
    for s in (0, m - 1):
        xs = x[:, s * sd:(s + 1) * sd].astype(np.float64)
        c = cb[s].astype(np.float64)
        d = (xs * xs).sum(1)[:, None] - 2.0 * xs @ c.T + (c * c).sum(1)[None, :]
        chosen = d[np.arange(N), codes[:, s]]
        assert (chosen <= d.min(1) + 1e-5 * (1.0 + np.abs(chosen))).all()


def test_rvq_1m_x_256_fit_and_encode(ctx):
    """RVQ: 1,000,000 x 256 mixture rows (seed 7), 8 stages of 256 centroids, 10 LBG iterations,
    epsilon 0 (src/rvq.rs:87-154, 171-215)."""
    import vq_amd
    dim, stages, k, iters = 256, 8, 256, 10
    x = data.gaussian_mixture(N, dim, 4096, 0.1, seed=7, centers="normal")
    init, reseed = data.index_streams(N, stages, k, iters, seed=7)
    dx = ctx.to_device(x)
    dres = ctx.empty((N, dim), F)
    dcb = ctx.empty((stages, k, dim), F)
    dcodes = ctx.empty(N, np.uint8)

    # one LBG iteration of the first stage on all rows against the oracle, bit for bit
    it, _ = ctx.lbg_fit(dx, N, dim, 1, dim, k, 1, init[0], reseed[0], dcb)
    want = O.lbg(x, k, 1, init[0], reseed[0])
    assert np.array_equal(dcb.download()[0].view(np.uint32), want["centroids"].view(np.uint32))

    ctx.copy_f32(dres, dx, N * dim)
    norms = [ctx.mean_l2norm(dres, N, dim, dim)]
    for st in range(stages):
        cbp = dcb.ptr + st * k * dim * 4
        ctx.lbg_fit(dres, N, dim, 1, dim, k, iters, init[st], reseed[st], cbp)
        ctx.assign(vq_amd.EUCLIDEAN, dres, N, dim, 1, dim, k, cbp, dcodes)
        ctx.residual_sub(dres, N, dim, dim, k, cbp, dcodes)
        norms.append(ctx.mean_l2norm(dres, N, dim, dim))
    cb = dcb.download()
    assert np.isfinite(cb).all()
    # every stage takes something off the mean residual norm (src/rvq.rs:131-141)
    assert all(b < a for a, b in zip(norms, norms[1:])), norms
    res = dres.download()
    want_norm = np.sqrt((res.astype(np.float64) ** 2).sum(1)).mean()
    assert abs(norms[-1] - want_norm) <= 1e-5 * want_norm

    dall = ctx.empty((N, stages), np.uint8)
    drec = ctx.empty((N, dim), np.uint16)
    ctx.rvq_encode(vq_amd.EUCLIDEAN, dx, N, dim, dim, stages, k, dcb, 0.0, dall, None, drec)
    codes, rec = dall.download(), drec.download()
    idx = sample_rows(N, 3000, 12)
    wc, wr = O.rvq_quantize(O.EUCLIDEAN, x[idx], cb, 0.0)
    assert np.array_equal(codes[idx], wc.astype(np.uint8))
    assert np.array_equal(rec[idx], wr)
    # the encode replays the fit's residual chain: what is left of a row is the fit's residual
    part = slice(0, 50000)
    left = x[part].copy()
    for st in range(stages):
        left = left - cb[st][codes[part, st]]
    assert np.array_equal(left.view(np.uint32), res[part].view(np.uint32))


def test_tsvq_1m_x_128_build_and_descent(ctx):
    """TSVQ: 1,000,000 unit rows of dimension 128 (seed 3), depth 8; cosine descent, then Manhattan
    on the same tree (src/tsvq.rs:71-148, 162-181)."""
    dim, depth = 128, 8
    x = data.unit_rows(N, dim, seed=3)
    dx = ctx.to_device(x)
    tree = ctx.tsvq_build(dx, N, dim, dim, depth)
    got = tree.download()
    otree = O.tsvq_fit(x, depth)  # the whole build on all rows: seconds
    want_tree, new_id = bfs_order(otree)
    assert_same_tree(got, want_tree)
    assert got["n_nodes"] == 511 and int(got["count"][0]) == N
    leaves = np.flatnonzero((got["left"] < 0) & (got["right"] < 0))
    assert int(got["count"][leaves].sum()) == N
    again = ctx.tsvq_build(dx, N, dim, dim, depth).download()
    assert_same_tree(again, got)

    dleaf = ctx.empty(N, np.int32)
    idx = sample_rows(N, 20000, 13)
    for metric in (O.COSINE, O.MANHATTAN):
        ctx.tsvq_descend(metric, dx, N, dim, tree, dleaf)
        leaf = dleaf.download()
        assert np.isin(leaf, leaves).all()
        want = np.array([new_id[v] for v in O.tsvq_descend(metric, x[idx], otree)], np.int32)
        assert np.array_equal(leaf[idx], want)


def test_opq_1m_x_128_fit(ctx):
    """OPQ: the 1,000,000 x 128 mixture rows, m = 16, k = 256, 5 outer x 10 LBG iterations,
    Euclidean, through the host classes (src/opq.rs:90-205, 222-264)."""
    import vq_amd
    from vq_amd import api
    dim, m, k, iters, outer, sd = 128, 16, 256, 10, 5, 8
    x = data.gaussian_mixture(N, dim, 1024, 0.05, seed=1)
    streams = data.index_streams(N, m, k, iters, seed=1)
    q = api.OptimizedProductQuantizer.fit(x, m, k, iters, outer, api.Distance.Euclidean, 0, streams=streams)
    R = q.rotation()
    cb = q.codebooks()
    assert np.isfinite(R).all() and np.isfinite(cb).all()
    R64 = R.astype(np.float64)
    assert np.abs(R64.T @ R64 - np.eye(dim)).max() < 1e-5
    # encode of a sample: the rotation is a matrix product (tolerance), the argmin that follows is
    # exact on the rows the GPU rotated
    idx = sample_rows(N, 20000, 14)
    xs = np.ascontiguousarray(x[idx])
    codes = q.encode(xs)
    dxs = ctx.to_device(xs)
    dy = ctx.empty((len(idx), dim), F)
    ctx.rotate(dxs, len(idx), dim, dim, ctx.to_device(R), dy)
    y = dy.download()
    y64 = xs.astype(np.float64) @ R64.T
    assert np.abs(y - y64).max() <= 1e-5 * np.abs(y64).max()
    assert np.array_equal(codes, O.pq_encode(O.EUCLIDEAN, y, cb).astype(np.uint8))
    # The rotation keeps lengths, so the error in the rotated frame is the error of the rows.  The
    # reference's last rotation is newer than its codebooks (src/opq.rs:127-194: the codebooks are
    # trained before the rotation is updated), so the error need not be below the plain product
    # quantizer's; it stays of its size and far below the spread of the rows.
    rec_opq = cb[np.arange(m)[None, :], codes].reshape(len(idx), dim).astype(np.float64)
    mse_opq = ((y64 - rec_opq) ** 2).sum(1).mean()
    p = api.ProductQuantizer.fit(x, m, k, iters, api.Distance.Euclidean, 0, streams=streams)
    pc = p.encode(xs)
    rec_pq = p.codebooks()[np.arange(m)[None, :], pc].reshape(len(idx), dim).astype(np.float64)
    mse_pq = ((xs.astype(np.float64) - rec_pq) ** 2).sum(1).mean()
    spread = ((xs.astype(np.float64) - xs.astype(np.float64).mean(0)) ** 2).sum(1).mean()
    assert mse_pq < 0.25 * spread and mse_opq < 1.5 * mse_pq, (mse_opq, mse_pq, spread)
