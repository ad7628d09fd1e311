"""GPU parity for codebooks above 256 centroids (16-bit codes): LBG training, encode and decode
through the C ABI against the CPU oracle, bit for bit, on both assignment paths (matrix cores
where a kernel exists / vector ALU only)."""
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
    c.set_assign_path(0)
    c.close()


def make_rows(rng, n, dim, kind):
    if kind == "uniform":
        return rng.random((n, dim), dtype=F)
    if kind == "grid":  # exact distance ties and duplicate rows
        return np.round(rng.standard_normal((n, dim)) * 3).astype(F)
    if kind == "blobs":  # a few heavy clusters (above 1024 members) beside many light ones
        x = rng.standard_normal((n, dim)).astype(F)
        x[: n // 2] = (0.001 * rng.standard_normal((n // 2, dim)) + 9.0).astype(F)
        return x[rng.permutation(n)]
    return rng.standard_normal((n, dim)).astype(F)


LBG_CASES = [
    # n, dim, m, k, iters, kind
    (2000, 16, 2, 257, 4, "normal"),     # one centroid beyond the 8-bit range
    (6000, 32, 4, 1000, 3, "normal"),
    (5000, 8, 1, 1024, 3, "uniform"),
    (1100, 8, 1, 1024, 3, "normal"),     # k close to n: empty clusters and re-seeds
    (9000, 24, 3, 300, 4, "blobs"),      # sub_dim 8, clusters above 1024 members
    (20000, 6, 2, 260, 3, "blobs"),      # sub_dim 3, parts of 4096 rows with and without members
    (3000, 6, 3, 400, 5, "grid"),
    (1500, 64, 1, 513, 2, "normal"),     # wide column block (RVQ stage shape)
    (700, 8, 1, 300, 0, "normal"),       # max_iters = 0 -> initial rows
]


@pytest.mark.parametrize("path", [0, 1])
@pytest.mark.parametrize("n,dim,m,k,iters,kind", LBG_CASES)
def test_lbg_fit_above_256_matches_oracle_bitwise(ctx, path, n, dim, m, k, iters, kind):
    rng = np.random.default_rng(n * 13 + k)
    x = make_rows(rng, n, dim, kind)
    init, reseed = data.index_streams(n, m, k, iters, seed=n + k)
    want = O.pq_fit(x, m, k, iters, init, reseed)
    assert want["rc"] == 0
    ctx.set_assign_path(path)
    sd = dim // m
    dx = ctx.to_device(x)
    dcb = ctx.empty((m, k, sd), F)
    it, used = ctx.lbg_fit(dx, n, dim, m, sd, k, iters, init, reseed, dcb)
    assert np.array_equal(it, want["iters"])
    assert np.array_equal(used, want["reseeds"])
    assert np.array_equal(dcb.download().view(np.uint32), want["codebooks"].view(np.uint32))


@pytest.mark.parametrize("path", [0, 1])
@pytest.mark.parametrize("metric", [O.SQEUCLIDEAN, O.EUCLIDEAN, O.COSINE, O.MANHATTAN])
@pytest.mark.parametrize("n,dim,m,k,kind", [
    (900, 32, 4, 257, "normal"),
    (1200, 128, 16, 1000, "uniform"),
    (800, 8, 1, 1024, "normal"),
    (500, 6, 3, 700, "grid"),
    (300, 64, 1, 600, "normal"),
    (400, 21, 3, 300, "normal"),
    (100, 16, 2, 40, "normal"),       # k <= 256 through the 16-bit entry point
    (260, 12, 1, 515, "zeros"),
])
def test_assign_u16_matches_oracle_bitwise(ctx, path, metric, n, dim, m, k, kind):
    rng = np.random.default_rng(n + 11 * metric + k)
    sd = dim // m
    if kind == "zeros":  # zero-norm rows and centroids (cosine returns 1)
        x = rng.standard_normal((n, dim)).astype(F)
        x[::3] = 0
        cb = rng.standard_normal((m, k, sd)).astype(F)
        cb[:, 1] = 0
        cb[:, 300] = 0
    elif kind == "grid":
        x = make_rows(rng, n, dim, kind)
        cb = np.round(rng.standard_normal((m, k, sd)) * 3).astype(F)
    else:
        x = make_rows(rng, n, dim, kind)
        cb = make_rows(rng, m * k, sd, kind).reshape(m, k, sd)
    ctx.set_assign_path(path)
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    dcodes = ctx.empty((n, m), np.uint16)
    ctx.assign_u16(metric, dx, n, dim, m, sd, k, dcb, dcodes)
    want = O.pq_encode(metric, x, cb)
    got = dcodes.download()
    assert np.array_equal(got, want.astype(np.uint16))
    # decode of the 16-bit codes: the centroids themselves, as f32 and as binary16
    d32 = ctx.empty((n, dim), F)
    ctx.decode_f32_u16(dcodes, n, m, sd, k, dcb, d32)
    ref = cb[np.arange(m)[None, :], want.astype(np.int64)].reshape(n, dim)
    assert np.array_equal(d32.download().view(np.uint32), ref.view(np.uint32))
    d16 = ctx.empty((n, dim), np.uint16)
    ctx.decode_f16_u16(dcodes, n, m, sd, k, dcb, d16)
    assert np.array_equal(d16.download(), ref.astype(np.float16).view(np.uint16))


def test_nan_distances_follow_the_single_loop(ctx):
    """A NaN at the head of a chunk: the loop over all centroids keeps its running minimum and
    goes on (nothing is below NaN, NaN is below nothing, src/utils.rs:62-70)."""
    rng = np.random.default_rng(5)
    n, sd, k = 300, 8, 700
    x = rng.standard_normal((n, sd)).astype(F)
    cb = rng.standard_normal((1, k, sd)).astype(F)
    cb[0, 256] = np.nan      # head of the second chunk
    cb[0, 513] = np.nan      # inside the third
    x[7] = np.nan            # every distance of the row is NaN: index 0
    ctx.set_assign_path(0)
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    dcodes = ctx.empty((n, 1), np.uint16)
    for metric in (O.SQEUCLIDEAN, O.EUCLIDEAN, O.COSINE, O.MANHATTAN):
        ctx.assign_u16(metric, dx, n, sd, 1, sd, k, dcb, dcodes)
        want = O.pq_encode(metric, x, cb)
        assert np.array_equal(dcodes.download(), want.astype(np.uint16)), metric


def test_k_limits(ctx):
    import vq_amd
    x = np.zeros((10, 8), F)
    dx = ctx.to_device(x)
    cb = ctx.empty((1, 8, 8), F)
    c8 = ctx.empty((10, 1), np.uint8)
    c16 = ctx.empty((10, 1), np.uint16)
    with pytest.raises(vq_amd.VqError) as e:
        ctx.assign(O.SQEUCLIDEAN, dx, 10, 8, 1, 8, 257, cb, c8)      # 8-bit codes stop at 256
    assert e.value.code == -4
    with pytest.raises(vq_amd.VqError) as e:
        ctx.assign_u16(O.SQEUCLIDEAN, dx, 10, 8, 1, 8, 65537, cb, c16)
    assert e.value.code == -4
    with pytest.raises(vq_amd.VqError) as e:
        ctx.lbg_fit(dx, 10, 8, 1, 8, 65537, 1, np.zeros(65537, np.uint32), np.zeros((1, 0), np.uint32), cb)
    assert e.value.code == -4
    with pytest.raises(vq_amd.VqError) as e:                          # n < k, src/utils.rs:45-50
        ctx.lbg_fit(dx, 10, 8, 1, 8, 300, 1, np.zeros(300, np.uint32), np.zeros((1, 0), np.uint32), cb)
    assert e.value.code == -1


# ---- the quantizer classes above 256 centroids ---------------------------------------------------
@pytest.fixture(scope="module")
def vq():
    from vq_amd import api
    return api


def test_pq_class_above_256_matches_oracle(vq):
    x = data.uniform(4000, 32, 11)
    m, k, iters = 4, 300, 4
    streams = data.index_streams(4000, m, k, iters, seed=2)
    pq = vq.ProductQuantizer.fit(x, m, k, iters, vq.Distance.Euclidean, 42, streams=streams)
    want = O.pq_fit_encode(O.EUCLIDEAN, x, m, k, iters, *streams)
    assert np.array_equal(pq.codebooks(), want["codebooks"])
    codes = pq.encode(x)
    assert codes.dtype == np.uint16 and np.array_equal(codes, want["codes"].astype(np.uint16))
    assert np.array_equal(pq.quantize_batch(x).view(np.uint16),
                          O.pq_decode_f16(want["codes"], want["codebooks"]))
    assert np.array_equal(pq.quantize(x[5]).view(np.uint16),
                          O.pq_decode_f16(want["codes"][5:6], want["codebooks"])[0])


def test_rvq_class_above_256_matches_oracle(vq):
    x = np.random.default_rng(8).standard_normal((2500, 24)).astype(F)
    stages, k, iters = 3, 260, 3
    streams = data.index_streams(2500, stages, k, iters, seed=3)
    for dist, metric in ((vq.Distance.Euclidean, O.EUCLIDEAN), (vq.Distance.Manhattan, O.MANHATTAN)):
        rvq = vq.ResidualQuantizer.fit(x, stages, k, iters, 0.0, dist, 1, streams=streams)
        want = O.rvq_fit(metric, x, stages, k, iters, 0.0, *streams)
        assert rvq.stages == want["stages"] == stages
        assert np.array_equal(rvq.codebooks(), want["codebooks"])
        wcodes, wrec = O.rvq_quantize(metric, x, want["codebooks"], 0.0)
        codes = rvq.encode(x)
        assert codes.dtype == np.uint16 and np.array_equal(codes, wcodes.astype(np.uint16))
        assert np.array_equal(rvq.quantize_batch(x).view(np.uint16), wrec)
    # rows that stop early (epsilon above some residual norms): unused stages keep code 0
    rvq = vq.ResidualQuantizer.fit(x, stages, k, iters, 0.0, vq.Distance.Euclidean, 1, streams=streams)
    want = O.rvq_fit(O.EUCLIDEAN, x, stages, k, iters, 0.0, *streams)
    eps = 1.6
    wcodes, wrec = O.rvq_quantize(O.EUCLIDEAN, x, want["codebooks"], eps)
    from vq_amd import Context
    c = Context(0)
    try:
        dx, dcb = c.to_device(x), c.to_device(want["codebooks"])
        dcodes = c.empty((2500, stages), np.uint16)
        drec = c.empty((2500, 24), np.uint16)
        c.rvq_encode_u16(O.EUCLIDEAN, dx, 2500, 24, 24, stages, k, dcb, eps, dcodes, None, drec)
        reached = wcodes != 0xFFFFFFFF  # the oracle marks the stages a row did not reach
        assert 0 < (~reached).sum() < reached.size
        assert np.array_equal(dcodes.download(), np.where(reached, wcodes, 0).astype(np.uint16))
        assert np.array_equal(drec.download(), wrec)
    finally:
        c.close()


def test_opq_class_above_256_first_iteration_matches_oracle(vq):
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((3000, 16)) @ rng.standard_normal((16, 16))).astype(F)
    m, k, iters = 2, 280, 3
    streams = data.index_streams(3000, m, k, iters, seed=5)
    got = vq.OptimizedProductQuantizer.fit(x, m, k, iters, 1, vq.Distance.Euclidean, 0, streams=streams)
    want = O.opq_fit(O.EUCLIDEAN, x, m, k, iters, 1, *streams)
    assert np.array_equal(got.codebooks(), want["codebooks"])
    assert np.allclose(got.rotation(), want["rotation"], atol=2e-6)
    codes = got.encode(x)
    assert codes.dtype == np.uint16 and codes.shape == (3000, m) and codes.max() < k
    # the codes are the argmin of the class's own rotation and codebooks
    y = (x.astype(np.float64) @ got.rotation().astype(np.float64).T)
    rec = np.concatenate([got.codebooks()[s][codes[:, s]] for s in range(m)], 1)
    assert np.array_equal(got.quantize_batch(x).view(np.uint16), rec.astype(np.float16).view(np.uint16))
    assert ((y - rec) ** 2).mean() < ((y - y.mean(0)) ** 2).mean()


# ---- seeded random shapes ------------------------------------------------------------------------
@pytest.mark.parametrize("seed", range(32))
def test_random_shapes_above_256(ctx, seed):
    """Encode under a random metric and two LBG iterations on a random shape with 257..1500
    centroids, against the oracle bit for bit."""
    rng = np.random.default_rng(9000 + seed)
    sd = int(rng.choice([1, 2, 3, 5, 8, 8, 8, 16, 24, 32]))
    m = int(rng.choice([1, 2, 3, 4, 8]))
    k = int(rng.integers(257, 1501))
    n = int(rng.integers(k, k + 4000))
    kind = ["normal", "grid", "uniform", "blobs", "offset", "dup"][seed % 6]
    dim = m * sd
    if kind == "offset":      # far from the origin: cancellation in the matrix-core scores
        x = (1000.0 + rng.standard_normal((n, dim))).astype(F)
    elif kind == "dup":       # duplicate rows -> duplicate centroids, exact ties
        base = rng.standard_normal((max(n // 7, 1), dim)).astype(F)
        x = base[rng.integers(0, base.shape[0], n)]
    else:
        x = make_rows(rng, n, dim, kind)
    metric = int(rng.integers(0, 4))
    ctx.set_assign_path(seed % 2)
    init, reseed = data.index_streams(n, m, k, 2, seed=seed)
    want = O.pq_fit(x, m, k, 2, init, reseed)
    assert want["rc"] == 0
    dx = ctx.to_device(x)
    dcb = ctx.empty((m, k, sd), F)
    it, used = ctx.lbg_fit(dx, n, dim, m, sd, k, 2, init, reseed, dcb)
    assert np.array_equal(it, want["iters"]) and np.array_equal(used, want["reseeds"])
    assert np.array_equal(dcb.download().view(np.uint32), want["codebooks"].view(np.uint32))
    dcodes = ctx.empty((n, m), np.uint16)
    ctx.assign_u16(metric, dx, n, dim, m, sd, k, dcb, dcodes)
    assert np.array_equal(dcodes.download(), O.pq_encode(metric, x, want["codebooks"]).astype(np.uint16))
