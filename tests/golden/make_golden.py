#!/usr/bin/env python3
"""Writes the golden fixtures of this directory.

    python tests/golden/make_golden.py

Nothing here calls the oracle (oracle/) or the GPU library: the expected outputs come from
 (1) known answers written out in the reference's own tests (cited per entry),
 (2) numpy's IEEE conversions (float32 -> float16, round to nearest even),
 (3) tests/np_ref.py, a plain numpy float32 statement of the reference's loops, and a small
     median-split tree builder below (sequential float32 sums, valid for nodes of <= 1024 rows).
Both the oracle (CPU tests) and the HIP library (GPU tests) are compared with these files.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from tests import np_ref  # noqa: E402

F = np.float32
SQ, EUCLID, COS, L1 = 0, 1, 2, 3
NAME = {SQ: "sq", EUCLID: "euclid", COS: "cos", L1: "l1"}  # metric names of tests/np_ref.py


def reference_known_answers():
    """Values asserted by the reference's tests (file:line in 'source')."""
    n = 1024 + 10  # PARALLEL_THRESHOLD + 10, src/vector.rs:16
    ramp = [float(i) for i in range(n)]
    return [
        dict(source="tests/test_distances.rs:16-23", metric=SQ, a=[1, 2, 3], b=[4, 6, 8], expected=50.0, tol=1e-6),
        dict(source="tests/test_distances.rs:26-34", metric=SQ, a=ramp, b=[v + 1 for v in ramp], expected=float(n), tol=1e-6),
        dict(source="tests/test_distances.rs:40-48", metric=EUCLID, a=[1, 2, 3], b=[4, 6, 8], expected=float(np.sqrt(F(50))), tol=1e-6),
        dict(source="tests/test_distances.rs:51-60", metric=EUCLID, a=ramp, b=[v + 1 for v in ramp], expected=float(np.sqrt(F(n))), tol=1e-6),
        dict(source="tests/test_distances.rs:66-72", metric=COS, a=[1, 0], b=[0, 1], expected=1.0, tol=1e-6),
        dict(source="tests/test_distances.rs:74-78", metric=COS, a=[1, 1], b=[1, 1], expected=0.0, tol=1e-6),
        dict(source="tests/test_distances.rs:82-90", metric=COS, a=[1.0] * n, b=[1.0] * n, expected=0.0, tol=1e-6),
        dict(source="tests/test_distances.rs:96-103", metric=L1, a=[1, 2, 3], b=[4, 6, 8], expected=12.0, tol=1e-6),
        dict(source="tests/test_distances.rs:106-115", metric=L1, a=ramp, b=[v + 2 for v in ramp], expected=2.0 * n, tol=1e-6),
    ]


def f16_cases():
    """float32 bit patterns around every rounding boundary of binary16, and numpy's conversion."""
    rng = np.random.default_rng(16)
    bits = [0x00000000, 0x80000000, 0x7f800000, 0xff800000, 0x3f800000, 0x477fe000, 0x477ff000, 0x477fefff,
            0x47800000, 0x33000000, 0x33000001, 0x33800000, 0x387fc000, 0x387fe000, 0x38800000, 0x3f801000,
            0x3f803000, 0x3f802000, 0x3f801001, 0x3f800fff, 0x7f7fffff, 0x00000001, 0x00800000, 0xc77fe000]
    bits += [int(b) for b in rng.integers(0, 2 ** 32, 2000, dtype=np.uint64)]
    halves = [(0x3c00 + i) << 13 | 0x1000 for i in range(64)]  # exact halfway points above 1.0
    bits += [0x38000000 + h for h in halves]
    u = np.array(bits, dtype=np.uint32)
    f = u.view(np.float32)
    keep = ~np.isnan(f)  # NaN payloads are not part of the contract
    u = u[keep]
    with np.errstate(over="ignore"):
        h = u.view(np.float32).astype(np.float16).view(np.uint16)
    return u, h


def lbg_cases():
    rng = np.random.default_rng(7)
    cases = {}

    def add(name, x, k, iters, init, reseed):
        x = np.ascontiguousarray(x, F)
        init = np.asarray(init, np.uint32)
        reseed = np.asarray(reseed, np.uint32)
        cb, codes, it, used = np_ref.lbg(x, k, iters, init, reseed)
        cases[name] = dict(x=x, k=k, iters=iters, init=init, reseed=reseed, centroids=np.asarray(cb, F),
                           iters_run=int(it), reseeds_used=int(used), codes=np.asarray(codes, np.uint8))

    # ordinary run
    x = rng.standard_normal((300, 8))
    add("random_300x8_k16", x, 16, 6, rng.choice(300, 16, replace=False), rng.integers(0, 300, 16 * 6))
    # duplicates of one point among the initial rows: their clusters stay empty and are re-seeded
    # from the stream, iteration-major, cluster index ascending (src/utils.rs:98-101)
    x = rng.standard_normal((200, 4))
    x[10] = x[3]
    x[57] = x[3]
    add("empty_clusters_200x4_k8", x, 8, 5, [3, 10, 57, 100, 120, 140, 160, 180], rng.integers(0, 200, 40))
    # every row identical: all land in cluster 0 in the first pass, nothing changes from the all-zero
    # start, the loop stops after one update (src/utils.rs:76-80,104-106)
    x = np.tile(rng.standard_normal((1, 6)), (50, 1))
    add("identical_rows_50x6_k4", x, 4, 10, [0, 1, 2, 3], rng.integers(0, 50, 40))
    # integer grid: exact distance ties, the lowest index wins (strict '<', src/utils.rs:64)
    x = np.round(rng.standard_normal((400, 3)) * 2)
    add("ties_grid_400x3_k12", x, 12, 8, rng.choice(400, 12, replace=False), rng.integers(0, 400, 96))
    # max_iters = 0 returns the initial rows
    x = rng.standard_normal((40, 5))
    add("zero_iters_40x5_k7", x, 7, 0, rng.choice(40, 7, replace=False), [0])
    return cases


def encode_cases():
    rng = np.random.default_rng(11)
    out = {}
    x = rng.standard_normal((257, 24)).astype(F)
    cb = rng.standard_normal((3, 19, 8)).astype(F)  # m = 3 blocks of 8, k = 19
    cb[1, 7] = cb[1, 2]  # duplicate centroid: the earlier index must win
    x[5, 8:16] = 0.0     # zero-norm sub-vector: cosine distance is 1 to everything (src/distances.rs:146-147)
    cb[2, 4] = 0.0
    for metric, name in ((SQ, "sq"), (EUCLID, "euclid"), (COS, "cos"), (L1, "l1")):
        codes = np.stack([np_ref.argmin_first(np_ref.dist_matrix(NAME[metric], x[:, 8 * s:8 * s + 8], cb[s]))
                          for s in range(3)], axis=1)
        out["encode_" + name] = codes.astype(np.uint8)
    out["encode_x"] = x
    out["encode_cb"] = cb
    # Euclidean: two different squared distances whose float32 roots are equal; the earlier centroid wins
    # although the later one is strictly closer in squared distance (src/distances.rs:134-140)
    # found by a fine sweep of c = (1, b) against the origin
    q = np.zeros(2, F)
    bs = np.linspace(0.5, 0.5001, 20000).astype(F)
    d2 = np_ref.dist_matrix("sq", q[None, :], np.stack([np.ones_like(bs), bs], 1))[0]
    found = None
    for i in range(len(bs) - 1):
        for j in range(i + 1, min(i + 40, len(bs))):
            if d2[j] > d2[i] and np.sqrt(d2[j]) == np.sqrt(d2[i]):
                found = (q, np.array([[1.0, bs[j]], [1.0, bs[i]]], F))  # index 0 is the farther one
                break
        if found is not None:
            break
    assert found is not None
    out["sqrt_collision_x"] = found[0][None, :]
    out["sqrt_collision_cb"] = found[1][None, :, :]
    out["sqrt_collision_sq"] = np.array([[1]], np.uint8)
    out["sqrt_collision_euclid"] = np.array([[0]], np.uint8)
    return out


def tsvq_build(x, max_depth):
    """TSVQNode::fit (src/tsvq.rs:71-148) for nodes of at most 1024 rows, nodes in pre-order."""
    nodes = []

    def seq_sum(a):  # f32, left to right
        acc = F(0)
        for v in a:
            acc = F(acc + v)
        return acc

    def fit(rows, depth):
        me = len(nodes)
        cnt = F(float(len(rows)))
        centroid = np.array([F(seq_sum(x[rows, t]) / cnt) for t in range(x.shape[1])], F)
        nodes.append(dict(centroid=centroid, left=-1, right=-1, split_dim=-1, split_val=F(0), count=len(rows)))
        if depth == 0 or len(rows) <= 1:
            return me
        var = np.array([seq_sum((x[rows, t] - centroid[t]) * (x[rows, t] - centroid[t])) for t in range(x.shape[1])], F)
        sd = 0
        for t in range(1, x.shape[1]):  # max_by keeps the last maximal element
            if not (var[t] < var[sd]):
                sd = t
        vals = np.sort(x[rows, sd], kind="stable")
        n = len(vals)
        median = F(F(vals[n // 2 - 1] + vals[n // 2]) / F(2)) if n % 2 == 0 else vals[n // 2]
        left = [r for r in rows if x[r, sd] <= median]
        right = [r for r in rows if not (x[r, sd] <= median)]
        nodes[me]["split_dim"], nodes[me]["split_val"] = sd, median
        if left and len(left) < len(rows):
            nodes[me]["left"] = fit(left, depth - 1)
        if right and len(right) < len(rows):
            nodes[me]["right"] = fit(right, depth - 1)
        return me

    fit(list(range(len(x))), max_depth)
    return nodes


def tsvq_descend(nodes, q):
    """quantize_with_distance under squared L2 (src/tsvq.rs:162-181): '<=' goes left."""
    i = 0
    while True:
        l, r = nodes[i]["left"], nodes[i]["right"]
        if l >= 0 and r >= 0:
            dl = np_ref.dist_matrix("sq", q[None, :], nodes[l]["centroid"][None, :])[0, 0]
            dr = np_ref.dist_matrix("sq", q[None, :], nodes[r]["centroid"][None, :])[0, 0]
            i = l if dl <= dr else r
        elif l >= 0:
            i = l
        elif r >= 0:
            i = r
        else:
            return i


def tsvq_cases():
    rng = np.random.default_rng(5)
    x = np.round(rng.standard_normal((97, 4)) * 4).astype(F) / F(4)  # many equal values: ties at the median
    x[:, 3] = x[:, 1]  # equal variances in dimensions 1 and 3: the later one is taken
    nodes = tsvq_build(x, 4)
    q = np.concatenate([x, rng.standard_normal((40, 4)).astype(F)])
    leaf = np.array([tsvq_descend(nodes, v) for v in q], np.int32)
    return dict(
        tsvq_x=x, tsvq_depth=np.int32(4), tsvq_queries=q,
        tsvq_centroids=np.stack([n["centroid"] for n in nodes]),
        tsvq_left=np.array([n["left"] for n in nodes], np.int32),
        tsvq_right=np.array([n["right"] for n in nodes], np.int32),
        tsvq_split_dim=np.array([n["split_dim"] for n in nodes], np.int32),
        tsvq_split_val=np.array([n["split_val"] for n in nodes], F),
        tsvq_count=np.array([n["count"] for n in nodes], np.int64),
        tsvq_leaf_centroid_of_query=np.stack([nodes[i]["centroid"] for i in leaf]),
    )


def main():
    with open(os.path.join(HERE, "reference_known_answers.json"), "w") as f:
        json.dump(reference_known_answers(), f, indent=0)
    arrays = {}
    u, h = f16_cases()
    arrays["f16_in_bits"], arrays["f16_out_bits"] = u, h
    for name, c in lbg_cases().items():
        for key, val in c.items():
            arrays[f"lbg/{name}/{key}"] = np.asarray(val)
    arrays.update(encode_cases())
    arrays.update(tsvq_cases())
    np.savez_compressed(os.path.join(HERE, "golden.npz"), **arrays)
    print("wrote", len(arrays), "arrays")


if __name__ == "__main__":
    main()
