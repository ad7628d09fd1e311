"""GPU parity on seeded random shapes for the paths beside the matrix-core assignment: cosine and
Manhattan encode, the TSVQ build and its descent under the four metrics, and the residual
quantizer's encode — each against the CPU oracle, bit for bit.  Data kinds: normal, integer grid
(exact ties), far offset, zero rows and zero centroids (the cosine rule for zero norms,
src/distances.rs:141-151), many duplicate rows.  VQ_PARITY_CASES widens the sweep."""
import os

import numpy as np
import pytest

from oracle import oracle as O
from tests.test_gpu_tsvq import assert_same_tree, bfs_order

pytestmark = pytest.mark.gpu
F = np.float32
N_CASES = int(os.environ.get("VQ_PARITY_CASES", "40"))


@pytest.fixture(scope="module")
def ctx():
    import vq_amd
    c = vq_amd.Context(0)
    yield c
    c.close()


def gen(rng, n, dim, kind):
    if kind == 0:
        return rng.standard_normal((n, dim)).astype(F)
    if kind == 1:
        return np.round(rng.standard_normal((n, dim)) * 2).astype(F)
    if kind == 2:
        return (1000 + rng.random((n, dim))).astype(F)
    if kind == 3:
        x = rng.standard_normal((n, dim)).astype(F)
        x[rng.integers(0, n, max(1, n // 10))] = 0.0
        return x
    base = rng.random((max(2, n // 50), dim), dtype=F)
    return base[rng.integers(0, base.shape[0], n)]


@pytest.mark.parametrize("case", range(N_CASES))
def test_random_cosine_and_manhattan_encode(ctx, case):
    import vq_amd
    rng = np.random.default_rng([7000, case])
    kind = case % 5
    sd = int(rng.choice([1, 3, 4, 8, 10, 16, 32, 40, 128]))
    m = int(rng.choice([1, 2, 4, 8])) if sd <= 16 else 1
    k = int(rng.choice([1, 2, 7, 32, 100, 256]))
    n = int(rng.integers(1, 3000))
    x = gen(rng, n, sd * m, kind)
    cb = gen(rng, m * k, sd, kind).reshape(m, k, sd)
    if kind == 3 and k > 2:
        cb[:, 1] = 0.0
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    dcodes = ctx.empty((n, m), np.uint8)
    for metric in (vq_amd.COSINE, vq_amd.MANHATTAN):
        with np.errstate(all="ignore"):
            want = O.pq_encode(metric, x, cb).astype(np.uint8)
        ctx.assign(metric, dx, n, sd * m, m, sd, k, dcb, dcodes)
        assert np.array_equal(dcodes.download(), want), (metric, n, m, k, sd, kind)


@pytest.mark.parametrize("case", range(N_CASES))
def test_random_tsvq_build_and_descent(ctx, case):
    rng = np.random.default_rng([7001, case])
    kind = case % 5
    dim = int(rng.choice([1, 2, 5, 8, 16, 24, 33, 64, 128]))
    n = int(rng.integers(1, 6000))
    depth = int(rng.integers(0, 9))
    x = gen(rng, n, dim, kind)
    otree = O.tsvq_fit(x, depth)
    want_tree, new_id = bfs_order(otree)
    tree = ctx.tsvq_build(ctx.to_device(x), n, dim, dim, depth)
    assert_same_tree(tree.download(), want_tree)
    q = gen(rng, int(rng.integers(1, 3000)), dim, kind)
    dq = ctx.to_device(q)
    dleaf = ctx.empty(q.shape[0], np.int32)
    for metric in (O.SQEUCLIDEAN, O.EUCLIDEAN, O.COSINE, O.MANHATTAN):
        ctx.tsvq_descend(metric, dq, q.shape[0], dim, tree, dleaf)
        with np.errstate(all="ignore"):
            want = np.array([new_id[v] for v in O.tsvq_descend(metric, q, otree)], np.int32)
        assert np.array_equal(dleaf.download(), want), (metric, n, dim, depth, kind)


@pytest.mark.parametrize("case", range(N_CASES))
def test_random_rvq_encode(ctx, case):
    import vq_amd
    rng = np.random.default_rng([7002, case])
    kind = case % 5
    dim = int(rng.choice([4, 8, 10, 32, 64, 256]))
    stages = int(rng.integers(1, 5))
    k = int(rng.choice([1, 2, 16, 100, 256]))
    n = int(rng.integers(1, 2000))
    x = gen(rng, n, dim, kind)
    cb = (gen(rng, stages * k, dim, kind).reshape(stages, k, dim) * F(0.5)).astype(F)
    eps = float(rng.choice([0.0, 0.0, 0.5, 3.0]))
    ld = dim + int(rng.choice([0, 0, 1, 4, 8]))  # the rows inside a wider buffer, aligned or not
    buf = np.full((n, ld), 7.0, F)
    buf[:, :dim] = x
    dx, dcb = ctx.to_device(buf), ctx.to_device(cb)
    dall = ctx.empty((n, stages), np.uint8)
    drec = ctx.empty((n, dim), np.uint16)
    dused = ctx.empty(n, np.uint8)
    for metric in (vq_amd.SQEUCLIDEAN, vq_amd.EUCLIDEAN, vq_amd.COSINE, vq_amd.MANHATTAN):
        with np.errstate(all="ignore"):
            wc, wr = O.rvq_quantize(metric, x, cb, eps)
        ctx.rvq_encode(metric, dx, n, ld, dim, stages, k, dcb, eps, dall, dused, drec)
        reached = wc != 0xFFFFFFFF
        got = dall.download()
        assert np.array_equal(dused.download(), reached.sum(1)), (metric, n, dim, ld, stages, k, eps, kind)
        assert np.array_equal(got[reached], wc[reached].astype(np.uint8)), (metric, n, dim, ld, stages, k, eps, kind)
        assert np.all(got[~reached] == 0)
        assert np.array_equal(drec.download(), wr), (metric, n, dim, ld, stages, k, eps, kind)
    assert np.array_equal(dx.download().view(np.uint32), buf.view(np.uint32))  # the caller's rows stay as they were
