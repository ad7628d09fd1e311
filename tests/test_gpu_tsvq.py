"""GPU parity for the tree-structured VQ: build (node statistics) and descent encode."""
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


def bfs_order(tree):
    """Renumber an oracle tree (pre-order ids) breadth-first, left before right."""
    order, frontier = [], [0]
    while frontier:
        nxt = []
        for v in frontier:
            order.append(v)
            for c in (tree["left"][v], tree["right"][v]):
                if c >= 0:
                    nxt.append(c)
        frontier = nxt
    new_id = {old: i for i, old in enumerate(order)}
    remap = lambda a: np.array([new_id[c] if c >= 0 else -1 for c in a[order]], np.int32)
    return dict(n_nodes=len(order), centroids=tree["centroids"][order], left=remap(tree["left"]),
                right=remap(tree["right"]), split_dim=tree["split_dim"][order],
                split_val=tree["split_val"][order], count=tree["count"][order]), new_id


def assert_same_tree(got, want):
    assert got["n_nodes"] == want["n_nodes"]
    assert np.array_equal(got["left"], want["left"]) and np.array_equal(got["right"], want["right"])
    assert np.array_equal(got["count"], want["count"])
    assert np.array_equal(got["split_dim"], want["split_dim"])
    internal = want["split_dim"] >= 0
    assert np.array_equal(got["split_val"][internal], want["split_val"][internal])
    assert np.array_equal(got["centroids"].view(np.uint32), want["centroids"].view(np.uint32))


@pytest.mark.parametrize("n,dim,depth,kind", [
    (1000, 10, 3, "wide"),     # tests/test_tsvq.rs:25-41
    (10, 5, 3, "same"),        # tests/test_tsvq.rs:11-22
    (5000, 16, 6, "normal"),
    (3001, 7, 10, "normal"),   # odd counts, deep
    (600, 4, 12, "grid"),      # duplicates: ties at the median, children that do not shrink
    (40, 3, 20, "normal"),     # deeper than log2(n): single-row leaves
    (20000, 8, 2, "normal"),   # nodes above 1024 rows -> midpoint-tree means
    (1, 4, 3, "normal"),
    (700, 6, 0, "normal"),     # max_depth 0: the root is a leaf
    (30000, 32, 9, "normal"),  # dim a multiple of 8: squares on the whole GPU, then the chains
    (12345, 128, 7, "normal"), # node sizes that are no multiples of 32
    (9000, 64, 13, "normal"),  # deep: levels with more than 2048 nodes take the lane-per-sum kernel
    (400000, 16, 2, "normal"), # columns above 4096 groups: block sums before the guesses, runs of composed maps
    (270001, 8, 4, "grid"),
    (5000, 24, 5, "grid"),     # dim 24, tied variances and medians
])
def test_build_matches_oracle(ctx, n, dim, depth, kind):
    rng = np.random.default_rng(n + depth)
    if kind == "normal":
        x = rng.standard_normal((n, dim)).astype(F)
    elif kind == "wide":
        x = rng.uniform(-1000, 1000, (n, dim)).astype(F)
    elif kind == "grid":
        x = np.round(rng.standard_normal((n, dim))).astype(F)
    else:
        x = np.tile(np.array([[1, 2, 3, 4, 5]], F)[:, :dim], (n, 1))
    want, _ = bfs_order(O.tsvq_fit(x, depth))
    tree = ctx.tsvq_build(ctx.to_device(x), n, dim, dim, depth)
    assert_same_tree(tree.download(), want)
    tree.free()


def test_equal_variances_take_the_last_dimension(ctx):
    x = np.array([[0, 0, 0], [2, 2, 2], [0, 2, 0], [2, 0, 2]], F)
    tree = ctx.tsvq_build(ctx.to_device(x), 4, 3, 3, 1)
    assert tree.download()["split_dim"][0] == 2


@pytest.mark.parametrize("metric", [O.SQEUCLIDEAN, O.EUCLIDEAN, O.COSINE, O.MANHATTAN])
@pytest.mark.parametrize("n,dim,depth", [(4000, 16, 6), (1000, 10, 3), (777, 128, 8), (1500, 32, 5),
                                         (1300, 64, 7), (900, 96, 4)])
def test_descent_matches_oracle(ctx, metric, n, dim, depth):
    rng = np.random.default_rng(n + metric)
    x = data.unit_rows(n, dim, seed=3) if dim == 128 else rng.standard_normal((n, dim)).astype(F)
    otree = O.tsvq_fit(x, depth)
    want_tree, new_id = bfs_order(otree)
    dx = ctx.to_device(x)
    tree = ctx.tsvq_build(dx, n, dim, dim, depth)
    q = np.concatenate([x, rng.standard_normal((500, dim)).astype(F), np.zeros((3, dim), F)])
    want = np.array([new_id[v] for v in O.tsvq_descend(metric, q, otree)], np.int32)
    dq = ctx.to_device(q)
    dleaf = ctx.empty(len(q), np.int32)
    ctx.tsvq_descend(metric, dq, len(q), dim, tree, dleaf)
    leaf = dleaf.download()
    assert np.array_equal(leaf, want)
    dout = ctx.empty((len(q), dim), np.uint16)
    ctx.tsvq_decode_f16(tree, dleaf, len(q), dout)
    assert np.array_equal(dout.download(),
                          want_tree["centroids"][want].astype(np.float16).view(np.uint16))


def test_descent_on_a_hand_made_tree_with_single_children_and_ties(ctx):
    # node 0 -> (1, 2); node 1 -> left only (3); node 2 -> right only (4); 3, 4 leaves
    cen = np.array([[0, 0], [-1, 0], [1, 0], [-1, 5], [1, 5]], F)
    left = np.array([1, 3, -1, -1, -1], np.int32)
    right = np.array([2, -1, 4, -1, -1], np.int32)
    tree = ctx.tree_create(cen, left, right)
    q = np.array([[-3, 0], [3, 0], [0, 7]], F)  # the last one is equidistant -> left (`<=`)
    dleaf = ctx.empty(3, np.int32)
    ctx.tsvq_descend(O.SQEUCLIDEAN, ctx.to_device(q), 3, 2, tree, dleaf)
    assert np.array_equal(dleaf.download(), [3, 4, 3])
    want = O.tsvq_descend(O.SQEUCLIDEAN, q, dict(centroids=cen, left=left, right=right))
    assert np.array_equal(dleaf.download(), want)


def test_config5_shape_unit_rows_cosine_then_manhattan(ctx):
    """Depth-8 tree on unit-normalised N(0,1) rows (seed 3), cosine descent, then Manhattan on the
    same tree; 20,000 rows here, the oracle needs seconds."""
    n, dim, depth = 20000, 128, 8
    x = data.unit_rows(n, dim, seed=3)
    otree = O.tsvq_fit(x, depth)
    want_tree, new_id = bfs_order(otree)
    dx = ctx.to_device(x)
    tree = ctx.tsvq_build(dx, n, dim, dim, depth)
    assert_same_tree(tree.download(), want_tree)
    dleaf = ctx.empty(n, np.int32)
    for metric in (O.COSINE, O.MANHATTAN):
        ctx.tsvq_descend(metric, dx, n, dim, tree, dleaf)
        want = np.array([new_id[v] for v in O.tsvq_descend(metric, x, otree)], np.int32)
        assert np.array_equal(dleaf.download(), want)


@pytest.mark.parametrize("kind", ["constant_columns", "all_zero", "tiny", "huge", "mixed", "integers", "wide_range"])
@pytest.mark.parametrize("n,dim,depth", [(70000, 8, 3), (20000, 128, 5), (33, 16, 2), (4097, 24, 4),
                                         (300000, 8, 3)])  # the last: columns long enough for blocks and runs
def test_variance_paths_agree_with_the_oracle_on_edge_data(ctx, kind, n, dim, depth):
    """The two ways of summing a node's squared deviations in row order (composed integer maps, one
    chain of adds per column) against the oracle's sequential sums, through the tree they decide:
    columns that never vary (every square is zero), values whose squares are subnormal or close to
    the largest float, integers (every rounding a tie or exact), magnitudes spread over many binades."""
    rng = np.random.default_rng([n, dim, len(kind)])
    if kind == "constant_columns":
        x = rng.standard_normal((n, dim)).astype(F)
        x[:, ::3] = F(1.25)
        x[:, 1] = 0.0
    elif kind == "all_zero":
        x = np.zeros((n, dim), F)
    elif kind == "tiny":
        x = (rng.standard_normal((n, dim)) * 1e-22).astype(F)
    elif kind == "huge":
        x = (rng.standard_normal((n, dim)) * 1e15).astype(F)
    elif kind == "mixed":
        x = (rng.standard_normal((n, dim)) * rng.choice([1e-6, 1.0, 1e4], (n, 1))).astype(F)
    elif kind == "integers":
        x = np.round(rng.standard_normal((n, dim)) * 3).astype(F)
    else:
        x = (rng.standard_normal((n, dim)) * np.exp2(rng.integers(-30, 30, (n, dim)))).astype(F)
    want_tree, _ = bfs_order(O.tsvq_fit(x, depth))
    dx = ctx.to_device(x)
    try:
        for path in (0, 1):
            ctx.set_tsvq_variance_path(path)
            assert_same_tree(ctx.tsvq_build(dx, n, dim, dim, depth).download(), want_tree)
    finally:
        ctx.set_tsvq_variance_path(0)


def _hand_tree(ctx, cen, depth):
    """A complete binary tree of the given depth over the rows of cen (breadth-first ids)."""
    nn = 2 ** (depth + 1) - 1
    assert len(cen) == nn
    left = np.array([2 * i + 1 if 2 * i + 2 < nn else -1 for i in range(nn)], np.int32)
    right = np.array([2 * i + 2 if 2 * i + 2 < nn else -1 for i in range(nn)], np.int32)
    return ctx.tree_create(cen, left, right), dict(centroids=cen, left=left, right=right)


@pytest.mark.parametrize("metric", [O.SQEUCLIDEAN, O.EUCLIDEAN, O.COSINE])
@pytest.mark.parametrize("dim", [32, 64, 128])
@pytest.mark.parametrize("kind", ["ties", "near_ties", "scales", "zero_norms", "non_finite", "far_offset",
                                  "equal_children"])
def test_descent_by_one_inner_product_agrees_with_the_two_distances(ctx, metric, dim, kind):
    """The default descent decides a node by the sign of one inner product when its value clears a
    bound on every rounding error of the reference's two sums, else by those sums.  Both paths
    against the oracle on data made to sit on the boundary: rows equidistant from both children
    (exactly, and to within a few units in the last place of the sums), magnitudes from 1e-20 to
    1e18 (outside the range the bound is proven for), zero rows and zero centroids (the cosine's own
    rule), NaN and infinities, children that only differ far from the origin, identical children."""
    rng = np.random.default_rng([dim, metric, len(kind)])
    depth = 4
    nn = 2 ** (depth + 1) - 1
    cen = rng.standard_normal((nn, dim)).astype(F)
    n = 3000
    q = rng.standard_normal((n, dim)).astype(F)
    if kind == "ties":
        cen = np.round(cen * 2).astype(F)
        q = np.round(q * 2).astype(F)
        # rows on the bisector of the root's children: the mean of the two plus a vector orthogonal to their difference
        d = (cen[1] - cen[2]).astype(np.float64)
        for i in range(0, n, 3):
            v = np.round(rng.standard_normal(dim) * 2)
            j = int(np.argmax(np.abs(d)))
            v[j] = 0.0
            q[i] = ((cen[1] + cen[2]) / 2 + v).astype(F)
    elif kind == "near_ties":
        mid = ((cen[1].astype(np.float64) + cen[2]) / 2)
        d = (cen[1] - cen[2]).astype(np.float64)
        for i in range(n):
            v = rng.standard_normal(dim)
            v -= d * (v @ d) / (d @ d)  # orthogonal to the difference: equidistant in exact arithmetic
            row = (mid + v + d * rng.uniform(-3e-7, 3e-7)).astype(F)
            q[i] = row if metric != O.COSINE else (v + rng.uniform(-3e-7, 3e-7) * (cen[1] / np.linalg.norm(cen[1])
                                                                            - cen[2] / np.linalg.norm(cen[2]))).astype(F)
    elif kind == "scales":
        q = (q * np.exp(rng.uniform(np.log(1e-20), np.log(1e18), (n, 1)))).astype(F)
        cen = (cen * np.exp(rng.uniform(np.log(1e-18), np.log(1e16), (nn, 1)))).astype(F)
    elif kind == "zero_norms":
        q[::5] = 0.0
        cen[[1, 4, 9, 20]] = 0.0
        q[1::7, : dim // 2] = 0.0
    elif kind == "non_finite":
        q[::11, 3] = np.nan
        q[5::13, 7] = np.inf
        q[6::17, 2] = -np.inf
        cen[6, 1] = np.nan
        cen[11, 0] = np.inf
    elif kind == "far_offset":
        cen = (1000.0 + cen * 1e-3).astype(F)
        q = (1000.0 + q * 1e-3).astype(F)
    else:
        cen[2] = cen[1]
        cen[8] = cen[7]
    tree, otree = _hand_tree(ctx, cen, depth)
    with np.errstate(all="ignore"):
        want = O.tsvq_descend(metric, q, otree)
    dq = ctx.to_device(q)
    dleaf = ctx.empty(n, np.int32)
    try:
        for path in (0, 1):
            ctx.set_tsvq_descend_path(path)
            ctx.tsvq_descend(metric, dq, n, dim, tree, dleaf)
            got = dleaf.download()
            assert np.array_equal(got, want), (path, int((got != want).sum()))
    finally:
        ctx.set_tsvq_descend_path(0)
