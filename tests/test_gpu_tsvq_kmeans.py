"""GPU: the TSVQ build with 2-means splits (vq_tsvq_build_kmeans) against the oracle through the C ABI.

This mode is NOT the reference's behaviour (src/tsvq.rs:87-123 splits at the median; that build is
tests/test_gpu_tsvq.py): it exists for the benchmark configuration that words the tree as "2-means with
10 LBG iterations per node".  The oracle is the pinned vqo_lbg applied per node (vqo_tsvq_fit_kmeans);
beyond it, closed forms: two separated blobs per node split into the blobs and their exact means."""
import numpy as np
import pytest

from oracle import oracle as O
from tests.test_gpu_tsvq import assert_same_tree, bfs_order

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def ctx():
    import vq_amd
    c = vq_amd.Context(0)
    yield c
    c.close()


def _draws(seed, depth, iters, extra=0):
    rng = np.random.default_rng(seed)
    return rng.integers(0, 2 ** 32, (max(2 ** depth - 1, 1), 2 + iters + extra), dtype=np.uint64).astype(np.uint32)


def _data(kind, n, dim, seed):
    rng = np.random.default_rng(seed)
    if kind == "normal":
        return rng.standard_normal((n, dim)).astype(F)
    if kind == "blobs":
        c = rng.standard_normal((8, dim)).astype(F) * 6
        return (c[rng.integers(0, 8, n)] + rng.standard_normal((n, dim)).astype(F) * 0.3).astype(F)
    if kind == "outliers":  # a few rows far away: a cluster of at most 1024 members in a node of several parts
        x = rng.standard_normal((n, dim)).astype(F)
        far = rng.choice(n, 300, replace=False)
        x[far] += 50.0
        return x
    if kind == "duplicates":  # many equal rows: equal initial centroids, empty clusters, ties
        base = np.round(rng.standard_normal((5, dim)) * 2).astype(F)
        return base[rng.integers(0, 5, n)]
    if kind == "integers":
        return np.round(rng.standard_normal((n, dim)) * 3).astype(F)
    raise ValueError(kind)


@pytest.mark.parametrize("kind,n,dim,depth,iters", [
    ("normal", 3000, 16, 4, 10), ("blobs", 20000, 128, 5, 10), ("normal", 9000, 8, 3, 3),
    ("blobs", 50000, 32, 2, 10), ("outliers", 20000, 16, 3, 10), ("outliers", 70000, 128, 2, 4),
    ("duplicates", 6000, 12, 4, 10), ("integers", 12000, 10, 5, 10), ("normal", 500, 7, 8, 10),
    ("normal", 4097, 24, 1, 10), ("blobs", 8192, 64, 3, 0), ("normal", 100, 5, 0, 10),
    ("normal", 2, 3, 4, 10), ("blobs", 150000, 128, 3, 10),
    # the row widths of the one-pass kernel (multiples of 32 up to 128) with parts that end inside a tile
    ("blobs", 30000, 64, 4, 10), ("normal", 25001, 96, 3, 10), ("outliers", 9000, 96, 5, 6),
    ("duplicates", 12345, 32, 6, 10), ("integers", 40000, 64, 2, 10)])
def test_kmeans_build_matches_oracle(ctx, kind, n, dim, depth, iters):
    x = _data(kind, n, dim, seed=n + dim)
    draws = _draws(depth * 1000 + iters, depth, iters)
    want, new_id = bfs_order(O.tsvq_fit_kmeans(x, depth, iters, draws))
    dx = ctx.to_device(x)
    tree = ctx.tsvq_build_kmeans(dx, n, dim, dim, depth, iters, draws)
    got = tree.download()
    assert got["n_nodes"] == want["n_nodes"]
    assert np.array_equal(got["left"], want["left"]) and np.array_equal(got["right"], want["right"])
    assert np.array_equal(got["count"], want["count"])
    assert np.array_equal(got["centroids"].view(np.uint32), want["centroids"].view(np.uint32))
    # the tree descends like any other
    dleaf = ctx.empty(n, np.int32)
    ctx.tsvq_descend(O.EUCLIDEAN, dx, n, dim, tree, dleaf)
    otree = O.tsvq_fit_kmeans(x, depth, iters, draws)
    wl = np.array([new_id[v] for v in O.tsvq_descend(O.EUCLIDEAN, x, otree)], np.int32)
    assert np.array_equal(dleaf.download(), wl)
    # a second build gives the same bits
    again = ctx.tsvq_build_kmeans(dx, n, dim, dim, depth, iters, draws).download()
    assert np.array_equal(again["centroids"].view(np.uint32), got["centroids"].view(np.uint32))


def test_kmeans_split_of_two_separated_blobs_is_the_blobs(ctx):
    """Closed form: two blobs far apart (whichever rows start the two centroids, one iteration
    separates them unless both start in one blob, two do then) split into the blobs; the children's
    centroids are the blobs' means in row order."""
    rng = np.random.default_rng(3)
    n, dim = 3000, 9
    lab = rng.integers(0, 2, n).astype(bool)
    x = (rng.standard_normal((n, dim)) * 0.05 + np.where(lab[:, None], 7.0, -7.0)).astype(F)
    draws = _draws(5, 1, 10)
    tree = ctx.tsvq_build_kmeans(ctx.to_device(x), n, dim, dim, 1, 10, draws).download()
    assert tree["n_nodes"] == 3
    sizes = sorted(tree["count"][1:].tolist())
    assert sizes == sorted([int(lab.sum()), int((~lab).sum())])
    for child in (1, 2):
        members = lab if tree["centroids"][child][0] > 0 else ~lab
        acc = np.zeros(dim, F)
        rows = x[members]
        if len(rows) <= 1024:
            for r in rows:
                acc = acc + r
            assert np.array_equal(tree["centroids"][child], acc / F(len(rows)))
        else:
            assert np.allclose(tree["centroids"][child], rows.astype(np.float64).mean(0), rtol=0, atol=1e-5)


def test_kmeans_build_rejects_too_few_draws(ctx):
    import vq_amd
    x = _data("normal", 100, 4, 1)
    dx = ctx.to_device(x)
    with pytest.raises(vq_amd.VqError) as e:
        ctx.tsvq_build_kmeans(dx, 100, 4, 4, 2, 10, _draws(1, 2, 3))
    assert e.value.code == vq_amd._ffi.ERR_INVALID_ARG
    with pytest.raises(vq_amd.VqError) as e:
        ctx.tsvq_build_kmeans(dx, 100, 4, 4, 21, 1, np.zeros((1, 3), np.uint32))
    assert e.value.code == vq_amd._ffi.ERR_UNSUPPORTED


def test_kmeans_tree_through_the_host_classes(ctx):
    """TSVQ.new_kmeans of the host mirror (not in the crate): with the draws given it is the oracle's
    tree; with a seed it is a valid tree whose quantize returns leaf centroids."""
    from vq_amd import api
    x = _data("blobs", 6000, 16, 9)
    draws = _draws(77, 4, 6)
    t = api.TSVQ.new_kmeans(x, 4, 6, api.Distance.Euclidean, 0, draws=draws)
    want, new_id = bfs_order(O.tsvq_fit_kmeans(x, 4, 6, draws))
    got = t.tree()
    assert np.array_equal(got["left"], want["left"]) and np.array_equal(got["right"], want["right"])
    assert np.array_equal(got["centroids"].view(np.uint32), want["centroids"].view(np.uint32))
    t2 = api.TSVQ.new_kmeans(x, 4, 6, api.Distance.Euclidean, 123)
    q = t2.quantize_batch(x[:100])
    cen16 = t2.tree()["centroids"].astype(np.float16)
    assert all(any(np.array_equal(row, c) for c in cen16) for row in q)
