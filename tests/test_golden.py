"""The oracle against the committed fixtures of tests/golden/ (made by tests/golden/make_golden.py
from the reference's own known answers, numpy's IEEE conversions and an independent numpy
statement; the oracle had no part in them)."""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
G = np.load(os.path.join(HERE, "golden.npz"))
F = np.float32
LBG_CASES = sorted({k.split("/")[1] for k in G.keys() if k.startswith("lbg/")})


def test_reference_known_answers():
    with open(os.path.join(HERE, "reference_known_answers.json")) as f:
        cases = json.load(f)
    assert len(cases) == 9
    for c in cases:
        got = O.distance(c["metric"], np.array(c["a"], F), np.array(c["b"], F))
        assert abs(got - c["expected"]) < c["tol"] * max(1.0, abs(c["expected"])), c["source"]


def test_f16_conversion_bit_for_bit():
    got = O.f32_to_f16_bits(G["f16_in_bits"].view(np.float32))
    assert np.array_equal(got, G["f16_out_bits"])


@pytest.mark.parametrize("name", LBG_CASES)
def test_lbg_cases_bit_for_bit(name):
    g = lambda key: G[f"lbg/{name}/{key}"]
    r = O.lbg(g("x"), int(g("k")), int(g("iters")), g("init"), g("reseed"))
    assert r["rc"] == 0
    assert np.array_equal(r["centroids"].view(np.uint32), g("centroids").view(np.uint32))
    assert r["iters"] == int(g("iters_run")) and r["reseeds"] == int(g("reseeds_used"))
    if int(g("iters")) > 0:
        assert np.array_equal(r["assign"].astype(np.uint8), g("codes"))


@pytest.mark.parametrize("metric,name", [(O.SQEUCLIDEAN, "sq"), (O.EUCLIDEAN, "euclid"), (O.COSINE, "cos"),
                                         (O.MANHATTAN, "l1")])
def test_encode_cases_bit_for_bit(metric, name):
    codes = O.pq_encode(metric, G["encode_x"], G["encode_cb"])
    assert np.array_equal(codes.astype(np.uint8), G["encode_" + name])


def test_sqrt_collision_case():
    x, cb = G["sqrt_collision_x"], G["sqrt_collision_cb"]
    assert np.array_equal(O.pq_encode(O.SQEUCLIDEAN, x, cb).astype(np.uint8), G["sqrt_collision_sq"])
    assert np.array_equal(O.pq_encode(O.EUCLIDEAN, x, cb).astype(np.uint8), G["sqrt_collision_euclid"])


def test_tsvq_build_and_descent():
    t = O.tsvq_fit(G["tsvq_x"], int(G["tsvq_depth"]))
    assert t["n_nodes"] == len(G["tsvq_left"])
    assert np.array_equal(t["left"], G["tsvq_left"]) and np.array_equal(t["right"], G["tsvq_right"])
    assert np.array_equal(t["centroids"].view(np.uint32), G["tsvq_centroids"].view(np.uint32))
    internal = G["tsvq_split_dim"] >= 0
    assert np.array_equal(t["split_dim"][internal], G["tsvq_split_dim"][internal])
    leaf = O.tsvq_descend(O.SQEUCLIDEAN, G["tsvq_queries"], t)
    assert np.array_equal(t["centroids"][leaf].view(np.uint32), G["tsvq_leaf_centroid_of_query"].view(np.uint32))
