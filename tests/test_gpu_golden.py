"""The HIP library, through the C ABI, against the committed fixtures of tests/golden/."""
import os

import numpy as np
import pytest

import vq_amd

pytestmark = pytest.mark.gpu

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
G = np.load(os.path.join(HERE, "golden.npz"))
F = np.float32
LBG_CASES = sorted({k.split("/")[1] for k in G.keys() if k.startswith("lbg/")})


@pytest.fixture(scope="module")
def ctx():
    return vq_amd.Context(0)


@pytest.mark.parametrize("name", LBG_CASES)
def test_lbg_cases_bit_for_bit(ctx, name):
    g = lambda key: G[f"lbg/{name}/{key}"]
    x, k, iters = g("x"), int(g("k")), int(g("iters"))
    n, d = x.shape
    dcb = ctx.empty((1, k, d), F)
    reseed = g("reseed") if iters > 0 else np.zeros(0, np.uint32)
    it, used = ctx.lbg_fit(ctx.to_device(x), n, d, 1, d, k, iters, g("init"), reseed, dcb)
    assert np.array_equal(dcb.download()[0].view(np.uint32), g("centroids").view(np.uint32))
    assert int(it[0]) == int(g("iters_run")) and int(used[0]) == int(g("reseeds_used"))


@pytest.mark.parametrize("metric,name", [(vq_amd.SQEUCLIDEAN, "sq"), (vq_amd.EUCLIDEAN, "euclid"),
                                         (vq_amd.COSINE, "cos"), (vq_amd.MANHATTAN, "l1")])
@pytest.mark.parametrize("path", [0, 1])
def test_encode_cases_bit_for_bit(ctx, metric, name, path):
    x, cb = G["encode_x"], G["encode_cb"]
    n, dim = x.shape
    m, k, sd = cb.shape
    dcodes = ctx.empty((n, m), np.uint8)
    ctx.set_assign_path(path)
    try:
        ctx.assign(metric, ctx.to_device(x), n, dim, m, sd, k, ctx.to_device(cb), dcodes)
    finally:
        ctx.set_assign_path(0)
    assert np.array_equal(dcodes.download(), G["encode_" + name])


def test_sqrt_collision_case(ctx):
    x, cb = G["sqrt_collision_x"], G["sqrt_collision_cb"]
    for metric, want in ((vq_amd.SQEUCLIDEAN, "sqrt_collision_sq"), (vq_amd.EUCLIDEAN, "sqrt_collision_euclid")):
        dcodes = ctx.empty((1, 1), np.uint8)
        ctx.assign(metric, ctx.to_device(x), 1, 2, 1, 2, 2, ctx.to_device(cb), dcodes)
        assert np.array_equal(dcodes.download(), G[want])


def test_f16_of_decoded_centroids(ctx):
    # vq_decode_f16 converts centroid values: feed the fixture's float32 values through it as a codebook
    vals = G["f16_in_bits"].view(np.float32)
    k = 256
    pad = (-len(vals)) % k
    cb = np.concatenate([vals, np.zeros(pad, F)]).reshape(-1, k, 1)  # m column blocks of width 1
    m = cb.shape[0]
    codes = np.tile(np.arange(k, dtype=np.uint8)[:, None], (1, m))   # row j takes centroid j of every block
    out = ctx.empty((k, m), np.uint16)
    ctx.decode_f16(ctx.to_device(codes), k, m, 1, k, ctx.to_device(cb), out)
    got = out.download().T.reshape(-1)[:len(vals)]
    assert np.array_equal(got, G["f16_out_bits"])


def test_tsvq_build_and_descent(ctx):
    x, depth = G["tsvq_x"], int(G["tsvq_depth"])
    n, dim = x.shape
    tree = ctx.tsvq_build(ctx.to_device(x), n, dim, dim, depth)
    t = tree.download()
    assert tree.n_nodes == len(G["tsvq_left"])
    # node numbering differs (breadth-first here, pre-order in the fixture): compare as sets of nodes
    key = lambda cen, cnt: sorted((int(c), tuple(v.view(np.uint32).tolist())) for v, c in zip(cen, cnt))
    assert key(t["centroids"], t["count"]) == key(G["tsvq_centroids"], G["tsvq_count"])
    q = G["tsvq_queries"]
    dleaf = ctx.empty(len(q), np.int32)
    ctx.tsvq_descend(vq_amd.SQEUCLIDEAN, ctx.to_device(q), len(q), dim, tree, dleaf)
    leaf = dleaf.download()
    assert np.array_equal(t["centroids"][leaf].view(np.uint32), G["tsvq_leaf_centroid_of_query"].view(np.uint32))
