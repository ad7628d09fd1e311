"""ctypes loader for the CPU oracle (oracle/vq_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg as the checker / reported baseline.  The shipped
package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libvq_oracle.so")

SQEUCLIDEAN, EUCLIDEAN, COSINE, MANHATTAN = 0, 1, 2, 3


def build(force=False):
    """Compile the oracle with the flags that keep the reference's rounding.  VQ_ORACLE_LIB names
    another build of the same source to load instead (the sanitizer build of the tests)."""
    other = os.environ.get("VQ_ORACLE_LIB")
    if other:
        return other
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-B", "-C", _HERE, "libvq_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
_i64 = C.c_int64


def lib():
    global _lib
    if _lib is None:
        L = C.CDLL(build())
        L.vqo_dot.restype = C.c_float
        L.vqo_dot.argtypes = [_f32p, _f32p, _i64]
        L.vqo_distance2.restype = C.c_float
        L.vqo_distance2.argtypes = [_f32p, _f32p, _i64]
        L.vqo_distance.restype = C.c_float
        L.vqo_distance.argtypes = [C.c_int, _f32p, _f32p, _i64]
        L.vqo_f32_to_f16.restype = C.c_uint16
        L.vqo_f32_to_f16.argtypes = [C.c_float]
        L.vqo_f16_to_f32.restype = C.c_float
        L.vqo_f16_to_f32.argtypes = [C.c_uint16]
        L.vqo_tree_depth.restype = C.c_int
        L.vqo_tree_depth.argtypes = [_i64]
        L.vqo_mean_rows.restype = None
        L.vqo_mean_rows.argtypes = [_f32p, _i64, _i64, _i64, _u32p, _i64, _f32p]
        L.vqo_mean_rows_parts.restype = None
        L.vqo_mean_rows_parts.argtypes = [_f32p, _i64, _i64, _i64, _u32p, _i64, _i64, _f32p]
        L.vqo_lbg.restype = C.c_int
        L.vqo_lbg.argtypes = [_f32p, _i64, _i64, _i64, _i64, _i64, _i64, _u32p, _u32p, _i64,
                              _f32p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.vqo_pq_fit.restype = C.c_int
        L.vqo_pq_fit.argtypes = [_f32p, _i64, _i64, _i64, _i64, _i64, _u32p, _u32p, _i64, _f32p,
                                 C.c_void_p, C.c_void_p]
        L.vqo_pq_encode.restype = None
        L.vqo_pq_encode.argtypes = [C.c_int, _f32p, _i64, _i64, _i64, _i64, _i64, _f32p, _u32p]
        L.vqo_pq_decode_f16.restype = None
        L.vqo_pq_decode_f16.argtypes = [_u32p, _i64, _i64, _i64, _i64, _f32p, _u16p]
        L.vqo_rvq_fit.restype = C.c_int
        L.vqo_rvq_fit.argtypes = [C.c_int, _f32p, _i64, _i64, _i64, _i64, _i64, C.c_float, _u32p,
                                  _u32p, _i64, _f32p, C.c_void_p, C.c_void_p]
        L.vqo_rvq_quantize.restype = None
        L.vqo_rvq_quantize.argtypes = [C.c_int, _f32p, _i64, _i64, _i64, _i64, C.c_float, _f32p,
                                       _u32p, _u16p]
        L.vqo_tsvq_fit.restype = _i64
        L.vqo_tsvq_fit.argtypes = [_f32p, _i64, _i64, _i64, _i64, _f32p, _i32p, _i32p, _i32p,
                                   _f32p, C.c_void_p]
        L.vqo_tsvq_descend.restype = None
        L.vqo_tsvq_descend.argtypes = [C.c_int, _f32p, _i64, _i64, _f32p, _i32p, _i32p, _i32p]
        L.vqo_rotate.restype = None
        L.vqo_rotate.argtypes = [_f32p, _i64, _i64, _f32p, _f32p]
        L.vqo_procrustes.restype = None
        L.vqo_procrustes.argtypes = [np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS"),
                                     _i64,
                                     np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")]
        L.vqo_opq_fit.restype = C.c_int
        L.vqo_opq_fit.argtypes = [C.c_int, _f32p, _i64, _i64, _i64, _i64, _i64, _i64, _u32p,
                                  _u32p, _i64, _f32p, _f32p]
        L.vqo_opq_encode.restype = None
        L.vqo_opq_encode.argtypes = [C.c_int, _f32p, _i64, _i64, _i64, _i64, _f32p, _f32p, _u32p]
        L.vqo_mse_f16.restype = C.c_double
        L.vqo_mse_f16.argtypes = [_f32p, _u16p, _i64, _i64]
        L.vqo_pq_fit_encode.restype = C.c_int
        L.vqo_pq_fit_encode.argtypes = [C.c_int, _f32p, _i64, _i64, _i64, _i64, _i64, _u32p,
                                        _u32p, _i64, _f32p, _u32p]
        L.vqo_set_threads.restype = C.c_int
        L.vqo_set_threads.argtypes = [C.c_int]
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


def distance(metric, a, b):
    a, b = _f32(a), _f32(b)
    return float(lib().vqo_distance(metric, a, b, a.size))


def distance2(a, b):
    a, b = _f32(a), _f32(b)
    return float(lib().vqo_distance2(a, b, a.size))


def dot(a, b):
    a, b = _f32(a), _f32(b)
    return float(lib().vqo_dot(a, b, a.size))


def f32_to_f16_bits(a):
    a = _f32(a).ravel()
    L = lib()
    return np.array([L.vqo_f32_to_f16(float(v)) for v in a], dtype=np.uint16)


def mean_rows(x, rows, off=0, d=None):
    x = _f32(x)
    ld = x.shape[1]
    d = ld - off if d is None else d
    rows = _u32(rows)
    out = np.empty(d, np.float32)
    lib().vqo_mean_rows(x, ld, off, d, rows, rows.size, out)
    return out


def mean_rows_parts(x, rows, off=0, d=None):
    """mean_vector in the order lbg_quantize uses (parts of 4096 rows above 1024 members)."""
    x = _f32(x)
    ld = x.shape[1]
    d = ld - off if d is None else d
    rows = _u32(rows)
    out = np.empty(d, np.float32)
    lib().vqo_mean_rows_parts(x, ld, off, d, rows, rows.size, x.shape[0], out)
    return out


def lbg(x, k, max_iters, init_idx, reseed_stream, off=0, d=None):
    """lbg_quantize on columns [off, off+d) of x. Returns dict."""
    x = _f32(x)
    n, ld = x.shape
    d = ld - off if d is None else d
    init_idx, reseed_stream = _u32(init_idx), _u32(reseed_stream)
    cen = np.zeros((max(k, 1), d), np.float32)
    assign = np.zeros(n, np.uint32)
    it = C.c_int32(0)
    used = C.c_int32(0)
    rs = reseed_stream if reseed_stream.size else np.zeros(1, np.uint32)
    rc = lib().vqo_lbg(x, n, ld, off, d, k, max_iters, init_idx if init_idx.size else
                       np.zeros(1, np.uint32), rs, reseed_stream.size, cen,
                       assign.ctypes.data_as(C.c_void_p), C.addressof(it), C.addressof(used))
    return dict(rc=rc, centroids=cen[:k], assign=assign, iters=it.value, reseeds=used.value)


def pq_fit(x, m, k, max_iters, init_idx, reseed_stream):
    x = _f32(x)
    n, dim = x.shape
    init_idx = _u32(init_idx).reshape(m, k)
    reseed_stream = _u32(reseed_stream).reshape(m, -1)
    sd = dim // m
    cb = np.zeros((m, k, sd), np.float32)
    iters = np.zeros(m, np.int32)
    used = np.zeros(m, np.int32)
    rc = lib().vqo_pq_fit(x, n, dim, m, k, max_iters, init_idx, reseed_stream,
                          reseed_stream.shape[1], cb, iters.ctypes.data_as(C.c_void_p),
                          used.ctypes.data_as(C.c_void_p))
    return dict(rc=rc, codebooks=cb, iters=iters, reseeds=used)


def pq_encode(metric, x, codebooks):
    x = _f32(x)
    cb = _f32(codebooks)
    m, k, sd = cb.shape
    n = x.shape[0]
    codes = np.zeros((n, m), np.uint32)
    lib().vqo_pq_encode(metric, x, n, x.shape[1], m, sd, k, cb, codes)
    return codes


def pq_decode_f16(codes, codebooks):
    cb = _f32(codebooks)
    m, k, sd = cb.shape
    codes = _u32(codes)
    n = codes.shape[0]
    out = np.zeros((n, m * sd), np.uint16)
    lib().vqo_pq_decode_f16(codes, n, m, sd, k, cb, out)
    return out


def rvq_fit(metric, x, stages, k, max_iters, epsilon, init_idx, reseed_stream):
    x = _f32(x)
    n, dim = x.shape
    init_idx = _u32(init_idx).reshape(stages, k)
    reseed_stream = _u32(reseed_stream).reshape(stages, -1)
    cb = np.zeros((stages, k, dim), np.float32)
    res = np.zeros((n, dim), np.float32)
    norms = np.zeros(stages, np.float32)
    produced = lib().vqo_rvq_fit(metric, x, n, dim, stages, k, max_iters, epsilon, init_idx,
                                 reseed_stream, reseed_stream.shape[1], cb,
                                 res.ctypes.data_as(C.c_void_p), norms.ctypes.data_as(C.c_void_p))
    return dict(stages=produced, codebooks=cb[:max(produced, 0)], residuals=res,
                avg_norms=norms[:max(produced, 0)])


def rvq_quantize(metric, x, codebooks, epsilon):
    x = _f32(x)
    cb = _f32(codebooks)
    stages, k, dim = cb.shape
    n = x.shape[0]
    codes = np.zeros((n, stages), np.uint32)
    recon = np.zeros((n, dim), np.uint16)
    lib().vqo_rvq_quantize(metric, x, n, dim, stages, k, epsilon, cb, codes, recon)
    return codes, recon


def tsvq_fit(x, max_depth):
    x = _f32(x)
    n, dim = x.shape
    max_nodes = min(2 * n, 2 ** (max_depth + 1)) + 1
    cen = np.zeros((max_nodes, dim), np.float32)
    left = np.zeros(max_nodes, np.int32)
    right = np.zeros(max_nodes, np.int32)
    sdim = np.zeros(max_nodes, np.int32)
    sval = np.zeros(max_nodes, np.float32)
    cnt = np.zeros(max_nodes, np.int64)
    nn = lib().vqo_tsvq_fit(x, n, dim, max_depth, max_nodes, cen, left, right, sdim, sval,
                            cnt.ctypes.data_as(C.c_void_p))
    assert nn > 0, nn
    return dict(n_nodes=nn, centroids=cen[:nn], left=left[:nn], right=right[:nn],
                split_dim=sdim[:nn], split_val=sval[:nn], count=cnt[:nn])


def tsvq_fit_kmeans(x, max_depth, lbg_iters, draws):
    """TSVQ with 2-means splits (vqo_tsvq_fit_kmeans): draws is ((2**max_depth - 1), per_node) uint32."""
    x = _f32(x)
    n, dim = x.shape
    draws = _u32(draws).reshape(2 ** max_depth - 1 if max_depth > 0 else 0, -1) if max_depth > 0 \
        else np.zeros((0, 2 + lbg_iters), np.uint32)
    max_nodes = min(2 * n, 2 ** (max_depth + 1)) + 1
    cen = np.zeros((max_nodes, dim), np.float32)
    left = np.zeros(max_nodes, np.int32)
    right = np.zeros(max_nodes, np.int32)
    cnt = np.zeros(max_nodes, np.int64)
    fn = lib().vqo_tsvq_fit_kmeans
    fn.restype = C.c_int64
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_int64, C.c_int64,
                   C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    d = np.ascontiguousarray(draws if draws.size else np.zeros((1, 2 + lbg_iters), np.uint32))
    nn = fn(x.ctypes.data, n, dim, max_depth, lbg_iters, d.ctypes.data, d.shape[1], max_nodes, cen.ctypes.data,
            left.ctypes.data, right.ctypes.data, cnt.ctypes.data)
    assert nn > 0, nn
    return dict(n_nodes=nn, centroids=cen[:nn], left=left[:nn], right=right[:nn],
                split_dim=np.full(nn, -1, np.int32), split_val=np.zeros(nn, np.float32), count=cnt[:nn])


def tsvq_descend(metric, x, tree):
    x = _f32(x)
    n, dim = x.shape
    leaf = np.zeros(n, np.int32)
    lib().vqo_tsvq_descend(metric, x, n, dim, _f32(tree["centroids"]),
                           np.ascontiguousarray(tree["left"], np.int32),
                           np.ascontiguousarray(tree["right"], np.int32), leaf)
    return leaf


def rotate(x, R):
    x, R = _f32(x), _f32(R)
    y = np.empty_like(x)
    lib().vqo_rotate(x, x.shape[0], x.shape[1], R, y)
    return y


def procrustes(A):
    A = np.ascontiguousarray(A, np.float64)
    R = np.empty_like(A)
    lib().vqo_procrustes(A, A.shape[0], R)
    return R


def opq_fit(metric, x, m, k, max_iters, opq_iters, init_idx, reseed_stream):
    x = _f32(x)
    n, dim = x.shape
    init_idx = _u32(init_idx).reshape(m, k)
    reseed_stream = _u32(reseed_stream).reshape(m, -1)
    R = np.zeros((dim, dim), np.float32)
    cb = np.zeros((m, k, dim // m), np.float32)
    rc = lib().vqo_opq_fit(metric, x, n, dim, m, k, max_iters, opq_iters, init_idx,
                           reseed_stream, reseed_stream.shape[1], R, cb)
    return dict(rc=rc, rotation=R, codebooks=cb)


def opq_encode(metric, x, rotation, codebooks):
    x = _f32(x)
    cb = _f32(codebooks)
    m, k, sd = cb.shape
    codes = np.zeros((x.shape[0], m), np.uint32)
    lib().vqo_opq_encode(metric, x, x.shape[0], x.shape[1], m, k, _f32(rotation), cb, codes)
    return codes


def mse_f16(x, recon_bits):
    x = _f32(x)
    r = np.ascontiguousarray(recon_bits, np.uint16)
    return float(lib().vqo_mse_f16(x, r, x.shape[0], x.shape[1]))


def pq_fit_encode(metric, x, m, k, max_iters, init_idx, reseed_stream, threads=0):
    x = _f32(x)
    n, dim = x.shape
    init_idx = _u32(init_idx).reshape(m, k)
    reseed_stream = _u32(reseed_stream).reshape(m, -1)
    cb = np.zeros((m, k, dim // m), np.float32)
    codes = np.zeros((n, m), np.uint32)
    used = lib().vqo_set_threads(threads)
    rc = lib().vqo_pq_fit_encode(metric, x, n, dim, m, k, max_iters, init_idx, reseed_stream,
                                 reseed_stream.shape[1], cb, codes)
    return dict(rc=rc, codebooks=cb, codes=codes, threads=used)
