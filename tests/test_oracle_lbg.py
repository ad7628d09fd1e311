"""Pins the oracle's LBG / PQ / RVQ / TSVQ / OPQ restatements: the reference's own
value-level pins, closed forms, invariants and an independent numpy statement."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import np_ref

F = np.float32


def _streams(rng, n, k, iters, m=1):
    init = np.stack([rng.choice(n, k, replace=False) for _ in range(m)]).astype(np.uint32)
    reseed = rng.integers(0, n, (m, max(1, k * iters))).astype(np.uint32)
    return init, reseed


# --- the reference's own pins (src/utils.rs:111-161) ----------------------------
def test_single_point_k1_returns_the_point():  # utils.rs:148-153
    x = np.array([[1.0, 2.0]], F)
    r = O.lbg(x, 1, 10, [0], [0])
    assert r["rc"] == 0 and np.array_equal(r["centroids"], x)


def test_k_zero_and_too_few_points_are_errors():  # utils.rs:134-145
    x = np.array([[1.0, 2.0], [2.0, 3.0]], F)
    assert O.lbg(x, 0, 10, [], [0])["rc"] == -1
    assert O.lbg(x[:1], 2, 10, [0, 0], [0])["rc"] == -2


def test_basic_shapes():  # utils.rs:127-131,156-160
    x = np.array([[1, 2], [2, 3], [3, 4], [4, 5]], F)
    for iters in (10, 100):
        r = O.lbg(x, 2, iters, [0, 3], [0] * 8)
        assert r["centroids"].shape == (2, 2)
        # two groups on a line: {1,2} and {3,4} rows -> means
        assert np.array_equal(r["centroids"], np.array([[1.5, 2.5], [3.5, 4.5]], F))


# --- closed forms ------------------------------------------------------------------
def test_k1_is_the_mean_after_one_iteration():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((300, 4)).astype(F)
    r = O.lbg(x, 1, 10, [17], [0])
    # assignments start at 0 and stay 0 -> not changed -> exactly one iteration
    assert r["iters"] == 1
    assert np.array_equal(r["centroids"][0], np_ref.mean_seq(x))


def test_k_equals_n_distinct_rows_reconstruct_themselves():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((40, 5)).astype(F)
    perm = rng.permutation(40)
    r = O.lbg(x, 40, 10, perm, [0])
    assert np.array_equal(r["centroids"], x[perm])
    assert np.array_equal(r["assign"], np.argsort(perm))


def test_well_separated_clusters_give_exact_means():
    rng = np.random.default_rng(5)
    centers = np.array([[0, 0], [100, 0], [0, 100]], F)
    lab = rng.integers(0, 3, 600)
    x = (centers[lab] + rng.standard_normal((600, 2))).astype(F)
    first = [int(np.flatnonzero(lab == j)[0]) for j in range(3)]
    r = O.lbg(x, 3, 10, first, [0] * 30)
    for j in range(3):
        assert np.array_equal(r["centroids"][j], np_ref.mean_seq(x[lab == j]))
    assert np.array_equal(r["assign"], lab)
    assert r["iters"] == 2  # second pass changes nothing


def test_max_iters_zero_returns_initial_rows():
    x = np.arange(20, dtype=F).reshape(10, 2)
    r = O.lbg(x, 3, 0, [7, 2, 5], [0])
    assert np.array_equal(r["centroids"], x[[7, 2, 5]]) and r["iters"] == 0


def test_identical_rows_stop_after_one_iteration():
    # benches/utils.rs:14-21 style data: every row equal -> everything lands in cluster 0,
    # which equals the all-zero start -> not changed -> one update, then break.  The update
    # still re-seeds the k-1 empty clusters, in cluster order, from successive stream entries.
    x = np.tile(np.array([[1, 2, 3]], F), (50, 1))
    x[7] = [9, 9, 9]
    r = O.lbg(x, 4, 10, [0, 1, 2, 3], [7, 8, 9, 10, 11])
    assert r["iters"] == 1 and r["reseeds"] == 3
    assert np.array_equal(r["centroids"][1], x[7]) and np.array_equal(r["centroids"][2], x[8])
    assert np.array_equal(r["centroids"][0], np_ref.mean_seq(x))


def test_empty_clusters_take_stream_entries_in_order_every_iteration():
    x = np.tile(np.array([[1, 2, 3]], F), (50, 1))
    x[7] = [9, 9, 9]
    # c0 = [9,9,9]; c1..c3 = [1,2,3]: row 7 -> 0, all others -> 1 (first of the tied indices)
    r = O.lbg(x, 4, 10, [7, 0, 1, 2], [7, 8, 20, 7, 11])
    # iteration 1: changed; clusters 2, 3 empty -> stream[0], stream[1]
    # iteration 2: same assignments -> clusters 2, 3 empty again -> stream[2], stream[3]; break
    assert r["iters"] == 2 and r["reseeds"] == 4
    assert np.array_equal(r["centroids"][2], x[20]) and np.array_equal(r["centroids"][3], x[7])
    assert np.array_equal(r["assign"], np.where(np.arange(50) == 7, 0, 1))


def test_reseed_stream_exhaustion_is_reported():
    x = np.tile(np.array([[1, 2, 3]], F), (10, 1))
    assert O.lbg(x, 4, 10, [0, 1, 2, 3], [1])["rc"] == -3


# --- independent numpy statement on small inputs --------------------------------------
@pytest.mark.parametrize("n,d,k,iters,seed", [(64, 8, 4, 5, 0), (50, 3, 7, 10, 1),
                                               (200, 8, 16, 6, 2), (33, 1, 5, 10, 3),
                                               (3000, 2, 2, 4, 4), (9000, 2, 3, 3, 5)])
def test_lbg_matches_numpy_statement(n, d, k, iters, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, d)).astype(F)
    if seed == 1:
        x = np.round(x)  # many exact ties and duplicate rows -> exercises '<' and empties
    init, reseed = _streams(rng, n, k, iters)
    r = O.lbg(x, k, iters, init[0], reseed[0])
    cen, assign, it, used = np_ref.lbg(x, k, iters, init[0], reseed[0])
    assert r["rc"] == 0
    assert np.array_equal(r["centroids"], cen)
    assert np.array_equal(r["assign"], assign)
    assert (r["iters"], r["reseeds"]) == (it, used)


def test_invariants_means_and_monotone_distortion():
    rng = np.random.default_rng(9)
    x = rng.random((2000, 8)).astype(F)
    init, reseed = _streams(rng, 2000, 32, 12)
    prev = None
    for iters in range(1, 8):
        r = O.lbg(x, 32, iters, init[0], reseed[0])
        assert r["reseeds"] == 0
        for j in range(32):  # every centroid is the mean of its assigned rows
            assert np.array_equal(r["centroids"][j],
                                  np_ref.mean_parts(x, np.flatnonzero(r["assign"] == j)))
        d = np_ref.dist_matrix("sq", x, r["centroids"]).astype(np.float64).min(1).sum()
        if prev is not None:
            assert d <= prev * (1 + 1e-6)
        prev = d


# --- PQ ---------------------------------------------------------------------------------
def test_pq_subspaces_are_independent_column_blocks():
    rng = np.random.default_rng(11)
    x = rng.random((500, 12)).astype(F)
    init, reseed = _streams(rng, 500, 8, 5, m=3)
    r = O.pq_fit(x, 3, 8, 5, init, reseed)
    for s in range(3):
        sub = np.ascontiguousarray(x[:, 4 * s:4 * s + 4])
        cen, _, _, _ = np_ref.lbg(sub, 8, 5, init[s], reseed[s])
        assert np.array_equal(r["codebooks"][s], cen)
    x2 = x.copy()
    x2[:, 8:] = rng.random((500, 4)).astype(F)  # touching block 2 leaves blocks 0, 1 alone
    r2 = O.pq_fit(x2, 3, 8, 5, init, reseed)
    assert np.array_equal(r2["codebooks"][:2], r["codebooks"][:2])


def test_pq_validation_codes():  # src/pq.rs:87-102
    x = np.zeros((4, 6), F)
    i, r = np.zeros((4, 1), np.uint32), np.zeros((4, 1), np.uint32)
    assert O.lib().vqo_pq_fit(x, 0, 6, 2, 1, 1, i, r, 1, np.zeros(12, F), None, None) == -10
    assert O.lib().vqo_pq_fit(x, 4, 2, 4, 1, 1, i, r, 1, np.zeros(12, F), None, None) == -11
    assert O.lib().vqo_pq_fit(x, 4, 6, 4, 1, 1, i, r, 1, np.zeros(12, F), None, None) == -12


@pytest.mark.parametrize("metric,name", [(O.SQEUCLIDEAN, "sq"), (O.EUCLIDEAN, "euclid"),
                                        (O.COSINE, "cos"), (O.MANHATTAN, "l1")])
def test_pq_encode_matches_numpy_argmin(metric, name):
    rng = np.random.default_rng(12 + metric)
    x = np.round(rng.standard_normal((300, 6)) * 2).astype(F)  # integer grid -> exact ties
    cb = np.round(rng.standard_normal((3, 16, 2)) * 2).astype(F)
    codes = O.pq_encode(metric, x, cb)
    for s in range(3):
        want = np_ref.argmin_first(np_ref.dist_matrix(name, x[:, 2 * s:2 * s + 2], cb[s]))
        assert np.array_equal(codes[:, s], want)


def test_euclidean_sqrt_collision_keeps_earlier_index():
    # two different squared distances whose f32 square roots coincide: under Euclidean the
    # earlier index wins (strict '<' on the rooted values), under SquaredEuclidean the
    # smaller square wins.  Found by a 2-d search: c = (1, b), b swept finely.
    x = np.zeros((1, 2), F)
    bs = np.linspace(0.5, 0.5001, 20000).astype(F)
    d2 = np.array([O.distance2(x[0], np.array([1.0, b], F)) for b in bs], F)
    found = 0
    for i in range(len(bs) - 1):
        for j in range(i + 1, min(i + 40, len(bs))):
            if d2[j] > d2[i] and np.sqrt(d2[j]) == np.sqrt(d2[i]):
                cb = np.array([[[1.0, bs[j]], [1.0, bs[i]]]], F)  # index 0 is the farther one
                assert O.pq_encode(O.SQEUCLIDEAN, x, cb)[0, 0] == 1
                assert O.pq_encode(O.EUCLIDEAN, x, cb)[0, 0] == 0
                found += 1
                break
        if found >= 5:
            break
    assert found >= 5


def test_pq_decode_is_gather_plus_f16():
    rng = np.random.default_rng(13)
    cb = rng.standard_normal((2, 4, 3)).astype(F)
    codes = rng.integers(0, 4, (10, 2)).astype(np.uint32)
    out = O.pq_decode_f16(codes, cb)
    want = np.concatenate([cb[0][codes[:, 0]], cb[1][codes[:, 1]]], 1).astype(np.float16)
    assert np.array_equal(out, want.view(np.uint16))


def test_pq_uniform_10k_mse_matches_published_value():
    # notebooks/performance_analysis.ipynb:398,405: PQ 10k x 128, m=16, k=256, 10 iterations,
    # uniform [0,1) -> MSE 0.019639.  Different data seed and index stream, so statistical.
    rng = np.random.default_rng(42)
    x = rng.random((10000, 128), dtype=F)
    init, reseed = _streams(rng, 10000, 256, 10, m=16)
    r = O.pq_fit_encode(O.EUCLIDEAN, x, 16, 256, 10, init, reseed, threads=8)
    rec = O.pq_decode_f16(r["codes"], r["codebooks"])
    mse = O.mse_f16(x, rec)
    assert abs(mse - 0.019639) < 4e-4, mse


# --- RVQ --------------------------------------------------------------------------------
def test_rvq_residual_norms_decrease_and_quantize_replays_fit():
    rng = np.random.default_rng(21)
    x = rng.standard_normal((400, 6)).astype(F)
    init, reseed = _streams(rng, 400, 8, 6, m=3)
    r = O.rvq_fit(O.EUCLIDEAN, x, 3, 8, 6, 0.0, init, reseed)
    assert r["stages"] == 3
    assert np.all(np.diff(r["avg_norms"]) < 0)
    codes, recon = O.rvq_quantize(O.EUCLIDEAN, x, r["codebooks"], 0.0)
    # quantize on the training rows replays the fit's residual chain exactly
    res = x.copy()
    acc = np.zeros_like(x)
    for st in range(3):
        j = np_ref.argmin_first(np_ref.dist_matrix("euclid", res, r["codebooks"][st]))
        assert np.array_equal(j, codes[:, st])
        acc = acc + r["codebooks"][st][j]
        res = res - r["codebooks"][st][j]
    assert np.array_equal(res, r["residuals"])
    assert np.array_equal(recon, acc.astype(np.float16).view(np.uint16))


def test_rvq_epsilon_stops_early():
    x = np.tile(np.array([[1, 2, 3, 4]], F), (20, 1))
    init = np.array([[0, 1], [0, 1], [0, 1]], np.uint32)
    reseed = np.zeros((3, 30), np.uint32)
    r = O.rvq_fit(O.SQEUCLIDEAN, x, 3, 2, 5, 0.01, init, reseed)
    assert r["stages"] == 1 and r["avg_norms"][0] == 0.0  # residual is exactly zero
    codes, _ = O.rvq_quantize(O.SQEUCLIDEAN, x, r["codebooks"], 0.01)
    assert np.all(codes[:, 0] == 0)


def test_rvq_k1_takes_index_zero():  # src/rvq.rs:113-115
    rng = np.random.default_rng(22)
    x = rng.standard_normal((30, 3)).astype(F)
    r = O.rvq_fit(O.COSINE, x, 2, 1, 3, 0.0, np.array([[4], [5]], np.uint32),
                  np.zeros((2, 3), np.uint32))
    assert r["stages"] == 2
    assert np.array_equal(r["codebooks"][0][0], np_ref.mean_seq(x))


# --- TSVQ -------------------------------------------------------------------------------
def test_tsvq_identical_rows_is_a_single_leaf():  # tests/test_tsvq.rs:11-22
    x = np.tile(np.array([[1, 2, 3, 4, 5]], F), (10, 1))
    t = O.tsvq_fit(x, 3)
    # median == every value -> everything goes left -> child not strictly smaller -> leaf
    assert t["n_nodes"] == 1 and t["left"][0] == -1 and t["right"][0] == -1
    assert np.array_equal(t["centroids"][0], x[0])
    assert np.all(O.tsvq_descend(O.SQEUCLIDEAN, x, t) == 0)


def test_tsvq_structure_small():
    # column 1 has the larger spread; 4 rows -> median = mean of the two middle values
    x = np.array([[0, 0], [0, 10], [1, 20], [1, 30]], F)
    t = O.tsvq_fit(x, 1)
    assert t["n_nodes"] == 3 and t["split_dim"][0] == 1 and t["split_val"][0] == 15.0
    assert np.array_equal(t["centroids"][1], np.array([0, 5], F))
    assert np.array_equal(t["centroids"][2], np.array([1, 25], F))
    assert np.array_equal(O.tsvq_descend(O.SQEUCLIDEAN, x, t), [1, 1, 2, 2])


def test_tsvq_equal_variances_take_the_last_dimension():  # Iterator::max_by keeps the last max
    x = np.array([[0, 0, 0], [2, 2, 2], [0, 2, 0], [2, 0, 2]], F)
    t = O.tsvq_fit(x, 1)
    assert t["split_dim"][0] == 2


def test_tsvq_partition_sizes_and_leaf_means():
    rng = np.random.default_rng(31)
    x = rng.standard_normal((1000, 10)).astype(F)
    t = O.tsvq_fit(x, 3)
    assert t["n_nodes"] == 15
    assert t["count"][0] == 1000 and sorted(t["count"][[1, 8]]) == [500, 500]
    leaf = O.tsvq_descend(O.SQEUCLIDEAN, x, t)
    assert set(leaf) <= set(np.flatnonzero(t["left"] < 0))
    # ties in descent go left
    mid = ((t["centroids"][1] + t["centroids"][8]) / 2).astype(F)[None]
    dl = O.distance(O.SQEUCLIDEAN, mid[0], t["centroids"][1])
    dr = O.distance(O.SQEUCLIDEAN, mid[0], t["centroids"][8])
    first = O.tsvq_descend(O.SQEUCLIDEAN, mid, t)[0]
    assert (first < 8) == (dl <= dr)


# --- OPQ --------------------------------------------------------------------------------
def test_procrustes_is_the_polar_factor():
    rng = np.random.default_rng(41)
    A = rng.standard_normal((16, 16))
    R = O.procrustes(A)
    assert np.allclose(R @ R.T, np.eye(16), atol=1e-12)
    U, _, Vt = np.linalg.svd(A)
    assert np.allclose(R, Vt.T @ U.T, atol=1e-10)
    Q, _ = np.linalg.qr(rng.standard_normal((16, 16)))
    assert np.allclose(O.procrustes(Q), Q.T, atol=1e-12)  # orthogonal A -> R = A^T


@pytest.mark.parametrize("dim,rank", [(4, 0), (6, 3), (8, 7), (5, 1), (16, 10)])
def test_procrustes_of_a_singular_matrix_is_still_orthogonal(dim, rank):
    """A of rank < dim leaves directions of U open; whatever completion is chosen, R = V U^T must
    be orthogonal, R A symmetric positive semi-definite with trace = nuclear norm of A (that is
    what makes it a Procrustes solution), and A = 0 gives the identity, as an SVD library's
    U = V = I does."""
    rng = np.random.default_rng(dim * 31 + rank)
    A = (rng.standard_normal((dim, rank)) @ rng.standard_normal((rank, dim))) if rank else np.zeros((dim, dim))
    R = O.procrustes(A)
    assert np.allclose(R.T @ R, np.eye(dim), atol=1e-10)
    P = R @ A
    assert np.allclose(P, P.T, atol=1e-9 * max(1.0, np.abs(A).max()))
    assert abs(np.trace(P) - np.linalg.svd(A, compute_uv=False).sum()) <= 1e-9 * max(1.0, np.abs(P).sum())
    if rank == 0:
        assert np.array_equal(R, np.eye(dim))
    # an all-zero column (a padded dimension) must not cost the rotation its rank
    B = rng.standard_normal((dim, dim))
    B[:, dim - 1] = 0.0
    Rb = O.procrustes(B)
    assert np.allclose(Rb.T @ Rb, np.eye(dim), atol=1e-10)
    assert abs(np.trace(Rb @ B) - np.linalg.svd(B, compute_uv=False).sum()) <= 1e-9 * np.abs(B).sum()


def test_rotate_is_matrix_vector_product():
    rng = np.random.default_rng(42)
    x = rng.standard_normal((20, 8)).astype(F)
    R = rng.standard_normal((8, 8)).astype(F)
    y = O.rotate(x, R)
    assert np.allclose(y, x @ R.T, rtol=1e-5, atol=1e-5)
    assert np.array_equal(O.rotate(x, np.eye(8, dtype=F)), x)


def test_opq_rotation_is_orthogonal_and_quirk_is_kept():
    rng = np.random.default_rng(43)
    x = (rng.standard_normal((600, 8)) @ rng.standard_normal((8, 8))).astype(F)
    init, reseed = _streams(rng, 600, 8, 5, m=2)
    r1 = O.opq_fit(O.EUCLIDEAN, x, 2, 8, 5, 1, init, reseed)
    assert r1["rc"] == 0
    R = r1["rotation"].astype(np.float64)
    assert np.allclose(R.T @ R, np.eye(8), atol=1e-5)
    # with one outer iteration the codebooks were trained on UN-rotated data (opq.rs:127-142
    # run before the rotation update at 183)
    assert np.array_equal(r1["codebooks"], O.pq_fit(x, 2, 8, 5, init, reseed)["codebooks"])
    r2 = O.opq_fit(O.EUCLIDEAN, x, 2, 8, 5, 2, init, reseed)
    y1 = O.rotate(x, r1["rotation"])
    assert np.array_equal(r2["codebooks"], O.pq_fit(y1, 2, 8, 5, init, reseed)["codebooks"])
    codes = O.opq_encode(O.EUCLIDEAN, x, r2["rotation"], r2["codebooks"])
    assert np.array_equal(codes, O.pq_encode(O.EUCLIDEAN, O.rotate(x, r2["rotation"]),
                                             r2["codebooks"]))


def test_tsvq_kmeans_oracle_closed_forms():
    """vqo_tsvq_fit_kmeans (2-means splits, not the reference's median split) on inputs whose answer
    is known: two separated blobs split into the blobs, with exact means; identical rows cannot be
    split (every row ties with the first centroid: the right side is empty, the node stays a leaf);
    depth 0 is the mean of everything; the split only depends on the node's own draws."""
    rng = np.random.default_rng(0)
    n, dim = 400, 6
    lab = rng.integers(0, 2, n).astype(bool)
    x = (rng.standard_normal((n, dim)) * 0.1 + np.where(lab[:, None], 5.0, -5.0)).astype(np.float32)
    draws = rng.integers(0, 2 ** 32, (1, 12), dtype=np.uint64).astype(np.uint32)
    t = O.tsvq_fit_kmeans(x, 1, 10, draws)
    assert t["n_nodes"] == 3 and sorted(t["count"][1:].tolist()) == sorted([int(lab.sum()), int((~lab).sum())])
    for child in (1, 2):
        members = lab if t["centroids"][child][0] > 0 else ~lab
        acc = np.zeros(dim, np.float32)
        for r in x[members]:
            acc = acc + r
        assert np.array_equal(t["centroids"][child], acc / np.float32(members.sum()))
    same = np.tile(np.array([[1.5, -2.0, 3.0]], np.float32), (10, 1))
    t = O.tsvq_fit_kmeans(same, 3, 10, rng.integers(0, 2 ** 32, (7, 12), dtype=np.uint64).astype(np.uint32))
    assert t["n_nodes"] == 1 and np.array_equal(t["centroids"][0], same[0])
    t0 = O.tsvq_fit_kmeans(x, 0, 10, np.zeros((0, 12), np.uint32))
    assert t0["n_nodes"] == 1
    # draws of other nodes do not matter: the root's split is the same under different draws for the children
    d2 = rng.integers(0, 2 ** 32, (3, 12), dtype=np.uint64).astype(np.uint32)
    d3 = d2.copy()
    d3[1:] = rng.integers(0, 2 ** 32, (2, 12), dtype=np.uint64).astype(np.uint32)
    a, b = O.tsvq_fit_kmeans(x, 2, 10, d2), O.tsvq_fit_kmeans(x, 2, 10, d3)
    assert a["count"][1] == b["count"][1]
