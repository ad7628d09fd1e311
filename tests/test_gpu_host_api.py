"""The reference's own tests, restated against the host classes that mirror its API
(tests/test_pq.rs, test_opq.rs, test_rvq.rs, test_tsvq.rs, src/utils.rs:111-161), plus parity
of the same calls with the CPU oracle when the index streams are passed explicitly."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import data
from tests.test_gpu_tsvq import bfs_order

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def vq():
    from vq_amd import api
    return api


def generate_test_data(n, dim):  # tests/utils.rs:16-25 (own generator: rand is not available)
    return np.random.default_rng(42).uniform(-1000.0, 1000.0, (n, dim)).astype(F)


# ---- src/utils.rs tests ------------------------------------------------------------------------
def test_lbg_quantize_basic_functionality(vq):
    d = np.array([[1, 2], [2, 3], [3, 4], [4, 5]], F)
    assert vq.lbg_quantize(d, 2, 10, 42).shape == (2, 2)
    assert vq.lbg_quantize(d, 2, 100, 42).shape == (2, 2)


def test_lbg_quantize_k_zero(vq):
    with pytest.raises(vq.VqError, match="k must be greater than 0"):
        vq.lbg_quantize(np.array([[1, 2], [2, 3]], F), 0, 10, 42)


def test_lbg_quantize_not_enough_data_points(vq):
    with pytest.raises(vq.VqError, match="Not enough data points for k clusters"):
        vq.lbg_quantize(np.array([[1, 2]], F), 2, 10, 42)


def test_lbg_quantize_single_data_point(vq):
    c = vq.lbg_quantize(np.array([[1, 2]], F), 1, 10, 42)
    assert np.array_equal(c, np.array([[1, 2]], F))


# ---- tests/test_pq.rs ----------------------------------------------------------------------------
def test_pq_on_random_vectors(vq):
    training = generate_test_data(1000, 10)
    pq = vq.ProductQuantizer.fit(training, 2, 2, 50, vq.Distance.SquaredEuclidean, 42)
    for v in training[:50]:
        q = pq.quantize(v)
        assert len(q) == len(v)
        assert np.isfinite(np.abs(v - q.astype(F)).sum())
    qb = pq.quantize_batch(training)
    assert qb.shape == training.shape and np.isfinite(np.abs(training - qb.astype(F)).sum())
    assert np.array_equal(qb[:50], np.stack([pq.quantize(v) for v in training[:50]]))


def test_pq_panics(vq):
    x = generate_test_data(20, 10)
    with pytest.raises(vq.VqError, match="Empty input"):
        vq.ProductQuantizer.fit(np.zeros((0, 10), F), 2, 2, 5, vq.Distance.Euclidean, 1)
    with pytest.raises(vq.VqError, match="Data dimension must be at least m"):
        vq.ProductQuantizer.fit(x, 11, 2, 5, vq.Distance.Euclidean, 1)
    with pytest.raises(vq.VqError, match="Data dimension must be divisible by m"):
        vq.ProductQuantizer.fit(x, 3, 2, 5, vq.Distance.Euclidean, 1)
    pq = vq.ProductQuantizer.fit(x, 2, 2, 5, vq.Distance.Euclidean, 1)
    with pytest.raises(vq.VqError, match="Dimension mismatch: expected 10, got 9"):
        pq.quantize(x[0, :9])
    with pytest.raises(vq.VqError, match="Invalid metric parameter for Chebyshev"):
        vq.ProductQuantizer.fit(x, 2, 2, 5, vq.Distance.Chebyshev, 1).quantize(x[0])


def test_pq_matches_oracle_with_explicit_streams(vq):
    x = data.uniform(3000, 32, 7)
    m, k, iters = 4, 64, 8
    streams = data.index_streams(3000, m, k, iters, seed=9)
    pq = vq.ProductQuantizer.fit(x, m, k, iters, vq.Distance.Euclidean, 42, streams=streams)
    want = O.pq_fit_encode(O.EUCLIDEAN, x, m, k, iters, *streams)
    assert np.array_equal(pq.codebooks(), want["codebooks"])
    assert np.array_equal(pq.encode(x), want["codes"].astype(np.uint8))
    assert np.array_equal(pq.quantize_batch(x).view(np.uint16),
                          O.pq_decode_f16(want["codes"], want["codebooks"]))
    # seeded fit without streams: deterministic in the seed, different seeds differ
    a = vq.ProductQuantizer.fit(x, m, k, iters, vq.Distance.Euclidean, 42).codebooks()
    b = vq.ProductQuantizer.fit(x, m, k, iters, vq.Distance.Euclidean, 42).codebooks()
    c = vq.ProductQuantizer.fit(x, m, k, iters, vq.Distance.Euclidean, 43).codebooks()
    assert np.array_equal(a, b) and not np.array_equal(a, c)


# ---- tests/test_opq.rs ---------------------------------------------------------------------------
def test_opq_on_random_vectors(vq):
    training = generate_test_data(1000, 10)
    opq = vq.OptimizedProductQuantizer.fit(training, 2, 2, 50, 5, vq.Distance.SquaredEuclidean, 42)
    qb = opq.quantize_batch(training)
    assert qb.shape == training.shape and np.isfinite(np.abs(training - qb.astype(F)).sum())
    q = opq.quantize(training[3])
    assert len(q) == 10 and np.array_equal(q, qb[3])
    R = opq.rotation().astype(np.float64)
    assert np.allclose(R.T @ R, np.eye(10), atol=1e-5)
    with pytest.raises(vq.VqError, match="Dimension must be divisible by m"):
        vq.OptimizedProductQuantizer.fit(training, 3, 2, 5, 2, vq.Distance.Euclidean, 1)


def test_opq_first_outer_iteration_matches_oracle(vq):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((2000, 16)) @ rng.standard_normal((16, 16))).astype(F)
    m, k, iters = 4, 16, 6
    streams = data.index_streams(2000, m, k, iters, seed=4)
    got = vq.OptimizedProductQuantizer.fit(x, m, k, iters, 1, vq.Distance.Euclidean, 0, streams=streams)
    want = O.opq_fit(O.EUCLIDEAN, x, m, k, iters, 1, *streams)
    # codebooks of the first outer iteration are trained on un-rotated data: bit-exact
    assert np.array_equal(got.codebooks(), want["codebooks"])
    # the rotation goes through a Jacobi SVD in both (device here, host there): equal to f32 rounding
    assert np.allclose(got.rotation(), want["rotation"], atol=2e-6)
    # three outer iterations: same reconstruction quality as the oracle's run (1e-3 relative)
    got3 = vq.OptimizedProductQuantizer.fit(x, m, k, iters, 3, vq.Distance.Euclidean, 0, streams=streams)
    want3 = O.opq_fit(O.EUCLIDEAN, x, m, k, iters, 3, *streams)

    def mse(R, cb, codes):
        y = x.astype(np.float64) @ R.astype(np.float64).T
        rec = np.concatenate([cb[s][codes[:, s]] for s in range(m)], 1)
        return ((y - rec) ** 2).mean()
    e_got = mse(got3.rotation(), got3.codebooks(), got3.encode(x))
    e_want = mse(want3["rotation"], want3["codebooks"],
                 O.opq_encode(O.EUCLIDEAN, x, want3["rotation"], want3["codebooks"]))
    assert abs(e_got - e_want) <= 0.02 * e_want


@pytest.mark.parametrize("dim,m", [(256, 16), (135, 3), (144, 2)])
def test_opq_fit_above_dim_128_matches_oracle(vq, dim, m):
    """The reference takes any dim divisible by m (src/opq.rs:103-115).  Above 128 the cross-
    covariance runs in 128-wide output blocks and the rotation update on the host inside the
    library; the first outer iteration is compared with the oracle as at dim 16."""
    rng = np.random.default_rng(dim)
    n, k, iters = 1500, 8, 4
    x = (rng.standard_normal((n, dim)) @ (np.eye(dim) + 0.3 * rng.standard_normal((dim, dim)))).astype(F)
    streams = data.index_streams(n, m, k, iters, seed=dim)
    got = vq.OptimizedProductQuantizer.fit(x, m, k, iters, 1, vq.Distance.Euclidean, 0, streams=streams)
    want = O.opq_fit(O.EUCLIDEAN, x, m, k, iters, 1, *streams)
    assert np.array_equal(got.codebooks(), want["codebooks"])
    R = got.rotation().astype(np.float64)
    assert np.allclose(R.T @ R, np.eye(dim), atol=1e-5)
    assert np.allclose(got.rotation(), want["rotation"], atol=5e-6)
    qb = got.quantize_batch(x[:100])
    assert qb.shape == (100, dim) and np.isfinite(qb.astype(F)).all()


def test_opq_with_no_outer_iteration_has_no_codebooks(vq):
    """opq_iters = 0: the reference returns an identity rotation and an empty codebook list, so
    quantize pushes nothing and returns an empty vector (src/opq.rs:119-122, 244-263)."""
    x = generate_test_data(100, 8)
    opq = vq.OptimizedProductQuantizer.fit(x, 2, 4, 5, 0, vq.Distance.Euclidean, 1)
    assert np.array_equal(opq.rotation(), np.eye(8, dtype=F))
    assert len(opq.quantize(x[0])) == 0
    assert opq.quantize_batch(x).shape == (100, 0)
    assert opq.k == 0
    with pytest.raises(vq.VqError, match="Dimension mismatch"):
        opq.quantize(x[0][:5])


# ---- tests/test_rvq.rs ---------------------------------------------------------------------------
def test_rvq_on_random_vectors(vq):
    training = generate_test_data(1000, 10)
    rvq = vq.ResidualQuantizer.fit(training, 2, 2, 50, 1e-6, vq.Distance.SquaredEuclidean, 42)
    qb = rvq.quantize_batch(training)
    assert qb.shape == training.shape and np.isfinite(np.abs(training - qb.astype(F)).sum())
    assert np.array_equal(rvq.quantize(training[0]), qb[0])


def test_rvq_matches_oracle_with_explicit_streams(vq):
    x = np.random.default_rng(3).standard_normal((1500, 24)).astype(F)
    stages, k, iters = 3, 16, 5
    streams = data.index_streams(1500, stages, k, iters, seed=6)
    rvq = vq.ResidualQuantizer.fit(x, stages, k, iters, 0.0, vq.Distance.Euclidean, 1, streams=streams)
    want = O.rvq_fit(O.EUCLIDEAN, x, stages, k, iters, 0.0, *streams)
    assert rvq.stages == want["stages"] == stages
    assert np.array_equal(rvq.codebooks(), want["codebooks"])
    wcodes, wrec = O.rvq_quantize(O.EUCLIDEAN, x, want["codebooks"], 0.0)
    assert np.array_equal(rvq.encode(x), wcodes.astype(np.uint8))
    assert np.array_equal(rvq.quantize_batch(x).view(np.uint16), wrec)


# ---- tests/test_tsvq.rs --------------------------------------------------------------------------
def test_tsvq_on_identical_vectors(vq):
    v = np.array([1.0, 2.0, 3.0, 4.0, 5.0], F)
    tsvq = vq.TSVQ.new(np.tile(v, (10, 1)), 3, vq.Distance.SquaredEuclidean)
    q = tsvq.quantize(v)
    assert len(q) == len(v) and np.all(np.abs(v - q.astype(F)) < 1e-6)


def test_tsvq_on_random_vectors(vq):
    training = generate_test_data(1000, 10)
    tsvq = vq.TSVQ.new(training, 3, vq.Distance.SquaredEuclidean)
    qb = tsvq.quantize_batch(training)
    assert qb.shape == training.shape and np.isfinite(np.abs(training - qb.astype(F)).sum())
    otree = O.tsvq_fit(training, 3)
    want_tree, new_id = bfs_order(otree)
    want = np.array([new_id[v] for v in O.tsvq_descend(O.SQEUCLIDEAN, training, otree)])
    assert np.array_equal(tsvq.leaves(training), want)
    assert np.array_equal(qb.view(np.uint16),
                          want_tree["centroids"][want].astype(np.float16).view(np.uint16))
    with pytest.raises(vq.VqError, match="Dimension mismatch: expected 10, got 4"):
        tsvq.quantize(training[0, :4])
    with pytest.raises(vq.VqError, match="Empty input"):
        vq.TSVQ.new(np.zeros((0, 10), F), 3, vq.Distance.Euclidean)


def test_rows_as_vectors_and_as_one_array_agree(vq):
    """`&[Vector<f32>]` (one heap vector per row, packed by the host layer) and a contiguous array
    (taken as a view) give the same reconstructions; a short row is a "Dimension mismatch" with the
    lengths the reference's row-by-row check would name."""
    x = generate_test_data(300, 12)
    pq = vq.ProductQuantizer.fit(x, 3, 8, 5, vq.Distance.Euclidean, 1)
    tsvq = vq.TSVQ.new(x, 3, vq.Distance.Manhattan)
    rvq = vq.ResidualQuantizer.fit(x, 2, 4, 5, 1e-6, vq.Distance.Euclidean, 1)
    opq = vq.OptimizedProductQuantizer.fit(x, 3, 8, 5, 2, vq.Distance.Euclidean, 1)
    for q in (pq, tsvq, rvq, opq):
        a = q.quantize_batch(x)
        b = q.quantize_batch_vectors(x)
        assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
        with pytest.raises(vq.VqError, match="Dimension mismatch: expected 12, got 7"):
            q.quantize_batch_vectors(x, short_row=5, short_len=7)
        with pytest.raises(vq.VqError, match="Dimension mismatch: expected 12, got 3"):
            q.quantize_batch_vectors(x, short_row=0, short_len=3)


def test_host_classes_under_ubsan():
    """This file's tests once more in a child process that loads the host mirror built with
    -fsanitize=undefined -fno-sanitize-recover (any finding aborts the child)."""
    import os
    import subprocess
    import sys
    if os.environ.get("VQ_HOST_LIB"):
        pytest.skip("already the sanitizer run")
    if not os.environ.get("VQ_SANITIZERS_ON_GPU"):
        pytest.skip("a sanitizer runtime inside a process that drives the GPU: only with VQ_SANITIZERS_ON_GPU=1 "
                    "(the host mirror runs under the sanitizers without a GPU in tests/test_host_sanitized.py)")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = os.path.join(root, "vq_amd", "libvqhost_ubsan.so")
    assert os.path.exists(lib), "build it with `python -m vq_amd.build`"
    env = dict(os.environ, VQ_HOST_LIB=lib, UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    res = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider", "-m", "gpu",
                          os.path.abspath(__file__)], cwd=root, env=env, capture_output=True, text=True,
                         timeout=600)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-3000:]
    assert "runtime error" not in res.stderr


def test_host_classes_under_asan():
    """The same once more against the host mirror built with -fsanitize=address,undefined (host
    code only: the kernels are not instrumented).  The sanitizer's runtime is preloaded into the
    child in front of whatever is preloaded already."""
    import os
    import subprocess
    import sys
    if os.environ.get("VQ_HOST_LIB"):
        pytest.skip("already the sanitizer run")
    if not os.environ.get("VQ_SANITIZERS_ON_GPU"):
        pytest.skip("a sanitizer runtime inside a process that drives the GPU: only with VQ_SANITIZERS_ON_GPU=1 "
                    "(the host mirror runs under the sanitizers without a GPU in tests/test_host_sanitized.py)")
    from tests.test_oracle_sanitized import asan_env
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = os.path.join(root, "vq_amd", "libvqhost_asan.so")
    assert os.path.exists(lib), "build it with `python -m vq_amd.build`"
    res = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider", "-m", "gpu",
                          os.path.abspath(__file__)], cwd=root, env=asan_env(VQ_HOST_LIB=lib),
                         capture_output=True, text=True, timeout=900)
    at = max(res.stderr.find("AddressSanitizer"), 0)
    assert res.returncode == 0, res.stdout[-1500:] + res.stderr[max(at - 200, 0):at + 4000]
    assert "AddressSanitizer" not in res.stderr and "runtime error" not in res.stderr
