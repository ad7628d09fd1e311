"""GPU parity on seeded random shapes: the matrix-core assignment paths (8-float and wider column
blocks, encode and LBG mode) against the CPU oracle, bit for bit, over block widths, codebook sizes,
metrics and data kinds drawn at random: far offsets, duplicate centroids (exact ties between
candidates), tiny and huge magnitudes, non-finite values."""
import os

import numpy as np
import pytest

from oracle import oracle as O
from tests import data

pytestmark = pytest.mark.gpu
F = np.float32
# VQ_PARITY_CASES widens the sweep (the same draws, more seeds)
N_CASES = int(os.environ.get("VQ_PARITY_CASES", "72"))
KINDS = ["normal", "uniform", "grid", "offset", "mixture", "dupcb", "tiny", "huge", "nonfinite"]


@pytest.fixture(scope="module")
def ctx():
    import vq_amd
    c = vq_amd.Context(0)
    yield c
    c.close()


def draw(rng, case):
    sd = int(rng.choice([8, 8, 8, 16, 24, 32, 64, 128, 256]))
    m = int(rng.choice([1, 2, 3, 4, 8, 16])) if sd <= 32 else int(rng.choice([1, 2]))
    k = int(rng.choice([1, 2, 3, 5, 17, 31, 32, 33, 64, 100, 128, 200, 255, 256]))
    n = int(rng.integers(max(k, 1), 4000))
    dim = sd * m
    kind = KINDS[case % len(KINDS)]
    if kind == "normal":
        x, cb = rng.standard_normal((n, dim)).astype(F), rng.standard_normal((m, k, sd)).astype(F)
    elif kind == "uniform":
        x, cb = rng.random((n, dim), dtype=F), rng.random((m, k, sd), dtype=F)
    elif kind == "grid":
        x = np.round(rng.standard_normal((n, dim)) * 2).astype(F)
        cb = np.round(rng.standard_normal((m, k, sd)) * 2).astype(F)
    elif kind == "offset":
        off = float(rng.choice([10, 1000, -300, 1e5]))
        x, cb = (off + rng.random((n, dim))).astype(F), (off + rng.random((m, k, sd))).astype(F)
    elif kind == "mixture":
        x = data.gaussian_mixture(n, dim, 37, 0.05, seed=int(rng.integers(1 << 30)))
        cb = x[rng.choice(n, k, replace=n < k)].reshape(k, m, sd).transpose(1, 0, 2).copy()
    elif kind == "dupcb":
        x, cb = rng.standard_normal((n, dim)).astype(F), rng.standard_normal((m, k, sd)).astype(F)
        if k > 3:
            cb[:, k // 2] = cb[:, 1]
            cb[:, k - 1] = cb[:, 1]
            cb[:, 2] = cb[:, 0]
    elif kind == "tiny":
        x = (rng.standard_normal((n, dim)) * 1e-20).astype(F)
        cb = (rng.standard_normal((m, k, sd)) * 1e-20).astype(F)
    elif kind == "huge":
        x = (rng.standard_normal((n, dim)) * 1e15).astype(F)
        cb = (rng.standard_normal((m, k, sd)) * 1e15).astype(F)
    else:
        x, cb = rng.random((n, dim), dtype=F), rng.random((m, k, sd), dtype=F)
        x[rng.integers(0, n, 5), rng.integers(0, dim, 5)] = np.inf
        x[rng.integers(0, n, 5), rng.integers(0, dim, 5)] = np.nan
        cb[rng.integers(0, m), rng.integers(0, k), rng.integers(0, sd)] = np.nan
        if rng.random() < 0.5:
            cb[rng.integers(0, m), 0, :] = np.nan  # NaN at index 0 is never displaced
    return n, dim, m, k, sd, kind, x, cb


@pytest.mark.parametrize("case", range(N_CASES))
def test_random_shape_encode_and_fit(ctx, case):
    import vq_amd
    rng = np.random.default_rng(1000 + case)
    n, dim, m, k, sd, kind, x, cb = draw(rng, case)
    metric = vq_amd.EUCLIDEAN if case % 2 else vq_amd.SQEUCLIDEAN
    with np.errstate(all="ignore"):
        want = O.pq_encode(metric, x, cb).astype(np.uint8)
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    dcodes = ctx.empty((n, m), np.uint8)
    ctx.set_assign_path(0)
    ctx.assign(metric, dx, n, dim, m, sd, k, dcb, dcodes)
    assert np.array_equal(dcodes.download(), want), (n, dim, m, k, kind)
    if kind == "nonfinite" or n < k:
        return
    # two LBG iterations from random rows: LBG-mode assignment, update and re-seeding
    init, reseed = data.index_streams(n, m, k, 2, seed=case)
    with np.errstate(all="ignore"):
        w = O.pq_fit(x, m, k, 2, init, reseed)
    assert w["rc"] == 0
    dcb2 = ctx.empty((m, k, sd), F)
    it, used = ctx.lbg_fit(dx, n, dim, m, sd, k, 2, init, reseed, dcb2)
    assert np.array_equal(it, w["iters"])
    assert np.array_equal(dcb2.download().view(np.uint32), w["codebooks"].view(np.uint32)), (n, dim, m, k, kind)


@pytest.mark.parametrize("case", range(12))
def test_random_fit_over_many_parts(ctx, case):
    """Whole fits of 8-float blocks over up to 22 parts of 4096 rows: clusters on both sides of the
    1024-member switch of mean_vector (src/vector.rs:298-313), empty clusters and re-seeds
    (src/utils.rs:98-101), early stops; centroids, iteration and re-seed counts against the oracle,
    and a second run that must give the same bits (the update runs on two streams)."""
    rng = np.random.default_rng([case, 0x51])
    m = int(rng.choice([4, 8, 16, 3]))
    k = int(rng.choice([2, 8, 17, 64, 256]))
    n = int(rng.integers(max(k, 5000), 90000))
    iters = int(rng.integers(2, 6))
    dim = 8 * m
    kind = case % 4
    if kind == 0:
        x = rng.random((n, dim), dtype=F)
    elif kind == 1:  # fewer centres than clusters: empty clusters and re-seeds
        x = data.gaussian_mixture(n, dim, max(1, k // 4), 0.01, seed=case)
    elif kind == 2:
        x = data.gaussian_mixture(n, dim, 4 * k + 3, 0.05, seed=case)
    else:            # many identical rows: ties
        base = rng.random((max(2, k // 2), dim), dtype=F)
        x = base[rng.integers(0, base.shape[0], n)]
    init, reseed = data.index_streams(n, m, k, iters, seed=case)
    want = O.pq_fit(x, m, k, iters, init, reseed)
    dx = ctx.to_device(x)
    dcb = ctx.empty((m, k, 8), F)
    it, used = ctx.lbg_fit(dx, n, dim, m, 8, k, iters, init, reseed, dcb)
    got = dcb.download()
    assert np.array_equal(got.view(np.uint32), want["codebooks"].view(np.uint32))
    assert np.array_equal(it, want["iters"]) and np.array_equal(used, want["reseeds"])
    ctx.lbg_fit(dx, n, dim, m, 8, k, iters, init, reseed, dcb)
    assert np.array_equal(dcb.download().view(np.uint32), got.view(np.uint32))
