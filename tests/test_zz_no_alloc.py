"""GPU: vq_assign_noalloc (fixed scratch, no device allocation) against vq_assign through the C ABI.

Codes must be bit-identical.  Every case makes two calls in a row on one context, the second
with a smaller input, so that whatever the first call left in the shared scratch array cannot leak
into the second; the oracle is the third witness on the smaller input."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def ctx():
    import vq_amd
    c = vq_amd.Context(0)
    yield c
    c.close()


def _case(seed, n, m, sd, k):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, m * sd)).astype(F)
    cb = rng.standard_normal((m, k, sd)).astype(F)
    return x, cb


def _both(ctx, metric, x, cb):
    n, dim = x.shape
    m, k, sd = cb.shape
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    want = ctx.empty((n, m), np.uint8)
    got = ctx.empty((n, m), np.uint8)
    ctx.assign(metric, dx, n, dim, m, sd, k, dcb, want)
    ctx.sync()
    ctx.assign_noalloc(metric, dx, n, dim, m, sd, k, dcb, got)
    ctx.sync()
    return want.download(), got.download()


# (first call, second call): n, m, sub_dim, k — the second is smaller in every size
PAIRS = [
    ((20000, 16, 8, 256), (3000, 4, 8, 100)),   # matrix-core tables in the scratch
    ((5000, 64, 8, 256), (777, 8, 8, 33)),      # the largest table the scratch holds
    ((4000, 2, 32, 64), (500, 1, 16, 7)),       # wide column blocks: vector-ALU kernel, no scratch
    ((3000, 4, 6, 50), (100, 2, 3, 5)),         # sub_dim without a matrix-core kernel
]


@pytest.mark.parametrize("metric", [0, 1, 2, 3])
@pytest.mark.parametrize("first,second", PAIRS)
def test_noalloc_matches_assign_twice_in_a_row(ctx, metric, first, second):
    x1, cb1 = _case(11, *first)
    want1, got1 = _both(ctx, metric, x1, cb1)
    assert np.array_equal(want1, got1)
    x2, cb2 = _case(12, *second)
    want2, got2 = _both(ctx, metric, x2, cb2)
    assert np.array_equal(want2, got2)
    ref = O.pq_encode(metric, x2, cb2)
    assert np.array_equal(got2, ref.astype(np.uint8))


def test_noalloc_back_to_back_without_sync(ctx):
    """Two enqueued calls on one stream, no synchronisation between them: the second call's table
    kernel must not overwrite tables the first call's kernel still reads (stream order)."""
    x1, cb1 = _case(21, 30000, 16, 8, 256)
    x2, cb2 = _case(22, 2000, 8, 8, 64)
    dx1, dcb1, dx2, dcb2 = (ctx.to_device(a) for a in (x1, cb1, x2, cb2))
    g1 = ctx.empty((30000, 16), np.uint8)
    g2 = ctx.empty((2000, 8), np.uint8)
    ctx.assign_noalloc(1, dx1, 30000, 128, 16, 8, 256, dcb1, g1)
    ctx.assign_noalloc(1, dx2, 2000, 64, 8, 8, 64, dcb2, g2)
    ctx.sync()
    w1 = ctx.empty((30000, 16), np.uint8)
    w2 = ctx.empty((2000, 8), np.uint8)
    ctx.assign(1, dx1, 30000, 128, 16, 8, 256, dcb1, w1)
    ctx.assign(1, dx2, 2000, 64, 8, 8, 64, dcb2, w2)
    assert np.array_equal(g1.download(), w1.download())
    assert np.array_equal(g2.download(), w2.download())


def test_noalloc_rejects_shapes_beyond_the_scratch(ctx):
    import vq_amd
    x, cb = _case(31, 256, 128, 8, 256)  # 128 x 256 = 32768 cells > 16384
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    out = ctx.empty((256, 128), np.uint8)
    with pytest.raises(vq_amd.VqError) as e:
        ctx.assign_noalloc(0, dx, 256, 1024, 128, 8, 256, dcb, out)
    assert e.value.code == vq_amd._ffi.ERR_UNSUPPORTED
    assert "scratch" in str(e.value)
    # the same shape through the allocating entry point works
    ctx.assign(0, dx, 256, 1024, 128, 8, 256, dcb, out)
    assert np.array_equal(out.download(), O.pq_encode(0, x, cb).astype(np.uint8))


def test_noalloc_on_a_fresh_context_first(ctx):
    """A context whose workspace has never been grown: the call must not need it."""
    import vq_amd
    c2 = vq_amd.Context(0)
    try:
        x, cb = _case(41, 4096, 16, 8, 256)
        dx, dcb = c2.to_device(x), c2.to_device(cb)
        got = c2.empty((4096, 16), np.uint8)
        c2.assign_noalloc(2, dx, 4096, 128, 16, 8, 256, dcb, got)   # cosine: norms in the scratch
        assert np.array_equal(got.download(), O.pq_encode(2, x, cb).astype(np.uint8))
        c2.assign_noalloc(0, dx, 4096, 128, 16, 8, 256, dcb, got)
        assert np.array_equal(got.download(), O.pq_encode(0, x, cb).astype(np.uint8))
        assert c2.last_recheck_count() >= 0
    finally:
        c2.close()


def test_noalloc_from_a_second_context_is_refused_while_the_first_is_running(ctx):
    """One scratch array per GPU: a call from another context while the stream of the context that
    used the array last is still busy is refused (VQ_ERR_UNSUPPORTED) instead of racing on the
    tables; once that stream has drained the other context may use the array."""
    import vq_amd
    n = 2_000_000
    x1, cb1 = _case(51, n, 16, 8, 256)
    x2, cb2 = _case(52, 3000, 8, 8, 64)
    dx1, dcb1 = ctx.to_device(x1), ctx.to_device(cb1)
    g1 = ctx.empty((n, 16), np.uint8)
    c2 = vq_amd.Context(0)
    try:
        dx2, dcb2 = c2.to_device(x2), c2.to_device(cb2)
        g2 = c2.empty((3000, 8), np.uint8)
        ctx.sync()
        for _ in range(4):  # about a millisecond of kernels on the first context's stream
            ctx.assign_noalloc(1, dx1, n, 128, 16, 8, 256, dcb1, g1)
        with pytest.raises(vq_amd.VqError) as e:
            c2.assign_noalloc(1, dx2, 3000, 64, 8, 8, 64, dcb2, g2)
        assert e.value.code == vq_amd._ffi.ERR_UNSUPPORTED and "another context" in str(e.value)
        # a shape that does not use the array is not concerned
        xm, cbm = _case(53, 500, 2, 5, 9)
        gm = c2.empty((500, 2), np.uint8)
        c2.assign_noalloc(3, c2.to_device(xm), 500, 10, 2, 5, 9, c2.to_device(cbm), gm)
        assert np.array_equal(gm.download(), O.pq_encode(3, xm, cbm).astype(np.uint8))
        ctx.sync()
        c2.assign_noalloc(1, dx2, 3000, 64, 8, 8, 64, dcb2, g2)
        assert np.array_equal(g2.download(), O.pq_encode(1, x2, cb2).astype(np.uint8))
        # and back: the first context again, after the second one's stream has drained
        c2.sync()
        ctx.assign_noalloc(1, dx1, n, 128, 16, 8, 256, dcb1, g1)
        w1 = ctx.empty((n, 16), np.uint8)
        ctx.assign(1, dx1, n, 128, 16, 8, 256, dcb1, w1)
        assert np.array_equal(g1.download(), w1.download())
    finally:
        c2.close()


def test_noalloc_limit_only_binds_the_shapes_that_use_the_scratch(ctx):
    """Manhattan, and squared-L2 on a width without a matrix-core kernel, keep nothing in the fixed
    array: a shape far beyond its size goes through."""
    x, cb = _case(61, 300, 128, 6, 256)   # 128 x 256 cells: twice what the array holds
    dx, dcb = ctx.to_device(x), ctx.to_device(cb)
    for metric in (0, 3):
        out = ctx.empty((300, 128), np.uint8)
        ctx.assign_noalloc(metric, dx, 300, 768, 128, 6, 256, dcb, out)
        assert np.array_equal(out.download(), O.pq_encode(metric, x, cb).astype(np.uint8))
