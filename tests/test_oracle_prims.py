"""Pins the oracle's L1 primitives on the reference's own known-answer tests
(tests/test_distances.rs, tests/test_vector.rs), on IEEE facts and on an
independent numpy float32 statement."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import np_ref

F = np.float32


# --- known answers held by the reference's tests ------------------------------
def test_squared_euclidean_known_answer():  # tests/test_distances.rs:16-23
    assert O.distance(O.SQEUCLIDEAN, [1, 2, 3], [4, 6, 8]) == 50.0


def test_squared_euclidean_long():  # tests/test_distances.rs:26-34 (sequential order here)
    n = 1024 + 10
    a = np.arange(n, dtype=F)
    assert O.distance(O.SQEUCLIDEAN, a, a + 1) == float(n)


def test_euclidean_known_answer():  # tests/test_distances.rs:40-48
    assert abs(O.distance(O.EUCLIDEAN, [1, 2, 3], [4, 6, 8]) - np.sqrt(F(50.0))) < 1e-6


def test_cosine_known_answers():  # tests/test_distances.rs:66-79
    assert abs(O.distance(O.COSINE, [1, 0], [0, 1]) - 1.0) < 1e-6
    assert abs(O.distance(O.COSINE, [1, 1], [1, 1]) - 0.0) < 1e-6


def test_cosine_long_identical():  # tests/test_distances.rs:82-90
    a = np.ones(1034, F)
    assert abs(O.distance(O.COSINE, a, a)) < 1e-6


def test_cosine_zero_norm_rule():  # src/distances.rs:146-147
    assert O.distance(O.COSINE, [0, 0, 0], [1, 2, 3]) == 1.0
    assert O.distance(O.COSINE, [1, 2, 3], [0, 0, 0]) == 1.0


def test_manhattan_known_answers():  # tests/test_distances.rs:96-115
    assert O.distance(O.MANHATTAN, [1, 2, 3], [4, 6, 8]) == 12.0
    n = 1034
    a = np.arange(n, dtype=F)
    assert O.distance(O.MANHATTAN, a, a + 2) == 2.0 * n


def test_dot_and_distance2_known_answers():  # tests/test_vector.rs:37-44, 68-75
    assert O.dot([1, 2, 3], [4, 5, 6]) == 32.0
    assert O.distance2([1, 2, 3], [4, 5, 6]) == 27.0


def test_mean_vector_known_answers():  # tests/test_vector.rs:78-105
    x = np.array([[1, 2, 3], [4, 5, 6], [7, 8, 9]], F)
    assert np.array_equal(O.mean_rows(x, [0, 1, 2]), np.array([4, 5, 6], F))
    x = np.tile(np.arange(5, dtype=F), (1034, 1))
    assert np.array_equal(O.mean_rows(x, np.arange(1034)), np.arange(5, dtype=F))


# --- arithmetic order: a wrong order or a fused multiply-add fails these ------
def test_sum_order_is_left_to_right():
    # 1e8 + 3 + 3 + 3: left to right every +3 is absorbed (ulp(1e8) = 8); any
    # association that first adds the small terms gives 1e8 + 8.
    a = np.array([1e4, np.sqrt(3.0), np.sqrt(3.0), np.sqrt(3.0)], F)
    b = np.zeros(4, F)
    seq = F(0)
    for v in a:
        seq = F(seq + F(v * v))
    assert float(seq) == 1e8
    assert O.distance2(a, b) == 1e8
    assert O.distance2(a[::-1].copy(), b) != 1e8  # reversed order accumulates the small terms


def test_no_fma_contraction():
    # d*d rounded separately: choose d so that fma(d,d,acc) != acc + fl(d*d)
    rng = np.random.default_rng(5)
    hits = 0
    for _ in range(200):
        a = rng.standard_normal(8).astype(F)
        b = rng.standard_normal(8).astype(F)
        acc = F(0)
        fused = np.float64(0)
        for t in range(8):
            d = F(a[t] - b[t])
            acc = F(acc + F(d * d))
            fused = np.float64(F(np.float64(fused) + np.float64(d) * np.float64(d)))
        assert O.distance2(a, b) == float(acc)
        hits += float(fused) != float(acc)
    assert hits > 0  # the test data does distinguish fused from unfused


@pytest.mark.parametrize("metric,name", [(O.SQEUCLIDEAN, "sq"), (O.EUCLIDEAN, "euclid"),
                                        (O.COSINE, "cos"), (O.MANHATTAN, "l1")])
@pytest.mark.parametrize("d", [1, 3, 8, 37, 256])
def test_distance_matches_numpy_statement(metric, name, d):
    rng = np.random.default_rng(d * 7 + metric)
    X = rng.standard_normal((6, d)).astype(F)
    Cb = rng.standard_normal((5, d)).astype(F)
    ref = np_ref.dist_matrix(name, X, Cb)
    for i in range(6):
        for j in range(5):
            assert O.distance(metric, X[i], Cb[j]) == float(ref[i, j])


# --- f32 -> f16 ---------------------------------------------------------------
def test_f16_matches_ieee_rne():
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(4000).astype(F),
        (rng.standard_normal(2000) * 1e-6).astype(F),  # f16 subnormal range
        (rng.standard_normal(2000) * 1e5).astype(F),  # overflow range
        np.array([0.0, -0.0, 65504.0, 65520.0, 65519.99, 65536.0, 1e-8, 5.9604645e-8,
                  2.9802322e-8, 2.98023259e-8, 6.1035156e-5, 6.0975552e-5, np.inf, -np.inf,
                  1.0009765625, 1.00048828125, 1.00146484375], F),
    ])
    got = O.f32_to_f16_bits(vals)
    want = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    assert (O.f32_to_f16_bits(np.array([np.nan], F))[0] & 0x7c00) == 0x7c00
    assert (O.f32_to_f16_bits(np.array([np.nan], F))[0] & 0x03ff) != 0


def test_f16_halfway_ties_go_to_even():
    # 1 + 2^-11 is exactly halfway between 1.0 and 1+2^-10 -> rounds to even (1.0)
    assert O.f32_to_f16_bits(np.array([1.0 + 2.0 ** -11], F))[0] == 0x3c00
    # 1 + 3*2^-11 is halfway between 1+2^-10 (odd) and 1+2^-9 (even) -> up
    assert O.f32_to_f16_bits(np.array([1.0 + 3 * 2.0 ** -11], F))[0] == 0x3c02


# --- mean_vector order --------------------------------------------------------
def test_mean_sequential_branch_is_row_order():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((700, 6)) * 100).astype(F)
    rows = np.sort(rng.choice(700, 600, replace=False))
    assert np.array_equal(O.mean_rows(x, rows), np_ref.mean_seq(x[rows]))


@pytest.mark.parametrize("c", [1025, 2048, 2049, 3000, 4097, 9000])
def test_mean_tree_branch(c):
    rng = np.random.default_rng(c)
    x = (rng.standard_normal((c + 50, 3)) * 100).astype(F)
    rows = np.sort(rng.choice(c + 50, c, replace=False))
    got = O.mean_rows(x, rows)
    assert np.array_equal(got, np_ref.mean_tree(x[rows]))
    # and it is a tree, not the sequential sum (the data is chosen so they differ)
    assert not np.array_equal(got, np_ref.mean_seq(x[rows]))
    exact = x[rows].astype(np.float64).mean(0)
    assert np.allclose(got, exact, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("n,c", [(5000, 1025), (9000, 3000), (20000, 1500), (4096 * 3 + 5, 9000)])
def test_mean_parts_order_used_by_lbg(n, c):
    rng = np.random.default_rng(n + c)
    x = (rng.standard_normal((n, 3)) * 100).astype(F)
    rows = np.sort(rng.choice(n, c, replace=False))
    got = O.mean_rows_parts(x, rows)
    assert np.array_equal(got, np_ref.mean_parts(x, rows))
    if n > 4096:  # more than one part: differs from the plain sequential sum
        assert not np.array_equal(got, np_ref.mean_seq(x[rows]))
    assert np.allclose(got, x[rows].astype(np.float64).mean(0), rtol=1e-4, atol=1e-3)
    small = rows[:1024]  # at most 1024 members: the reference's sequential order
    assert np.array_equal(O.mean_rows_parts(x, small), np_ref.mean_seq(x[small]))


def test_tree_depth_rule():
    L = O.lib()
    assert L.vqo_tree_depth(1) == 0 and L.vqo_tree_depth(1024) == 0
    assert L.vqo_tree_depth(1025) == 1 and L.vqo_tree_depth(2048) == 1
    assert L.vqo_tree_depth(2049) == 2 and L.vqo_tree_depth(1 << 20) == 10
