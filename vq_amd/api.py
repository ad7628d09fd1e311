"""Python view of the C++ host classes (vq_amd/host/vq.hpp) that mirror the reference's public
API: lbg_quantize, ProductQuantizer, OptimizedProductQuantizer, ResidualQuantizer, TSVQ, with the
reference's argument order and its panic messages as exception texts (VqError).

Quantized outputs are numpy float16 arrays (the reference's Vector<f16>)."""
import ctypes as C
import os

import numpy as np

from . import _ffi
from ._ffi import VqError

_HERE = os.path.dirname(os.path.abspath(__file__))
# VQ_HOST_LIB names another build of the host mirror to load (the sanitizer build of the tests)
HOST_LIB_PATH = os.environ.get("VQ_HOST_LIB") or os.path.join(_HERE, "libvqhost.so")

if not os.path.exists(HOST_LIB_PATH):
    raise ImportError(f"{HOST_LIB_PATH} is missing: build it with `python -m vq_amd.build`")
_h = C.CDLL(HOST_LIB_PATH)
_h.vqh_last_error.restype = C.c_char_p
_vp, _i64, _i32, _u64 = C.c_void_p, C.c_int64, C.c_int32, C.c_uint64


class Distance:
    """src/distances.rs:73-88.  The first four variants have kernels."""
    SquaredEuclidean, Euclidean, CosineDistance, Manhattan, Chebyshev, _Minkowski, Hamming = range(7)

    @staticmethod
    def Minkowski(p):
        return (Distance._Minkowski, float(p))


def _dist(d):
    return (d[0], d[1]) if isinstance(d, tuple) else (int(d), 0.0)


def _check(rc):
    if rc != 0:
        raise VqError(rc, (_h.vqh_last_error() or b"").decode())


def _rows(data):
    if len(data) == 0:
        return np.zeros((0, 0), np.float32)
    x = np.ascontiguousarray(data, dtype=np.float32)
    if x.ndim != 2:
        raise VqError(_ffi.ERR_DIM_MISMATCH, "Dimension mismatch: rows of different length")
    return x


def _streams(streams):
    if streams is None:
        return None, None, 0
    init, reseed = streams
    init = np.ascontiguousarray(init, np.uint32)
    reseed = np.ascontiguousarray(reseed, np.uint32)
    reseed = reseed.reshape(init.shape[0] if init.ndim > 1 else 1, -1)
    return init, reseed, reseed.shape[1]


def _p(a):
    return a.ctypes.data_as(_vp) if a is not None else None


def lbg_quantize(data, k, max_iters, seed, streams=None):
    """src/utils.rs:32-37.  Returns the k centroids as a (k, dim) float32 array."""
    x = _rows(data)
    n, dim = x.shape
    out = np.zeros((max(k, 0), dim), np.float32)
    init, reseed, nr = _streams(streams)
    _check(_h.vqh_lbg_quantize(_p(x), _i64(n), _i64(dim), _i64(k), _i64(max_iters), _u64(seed),
                               _p(init), _p(reseed), _i32(nr), _p(out)))
    return out


class _Quantizer:
    def __init__(self, handle):
        self._o = handle
        info = (C.c_int64 * 7)()
        _check(_h.vqh_info(_vp(handle), info))
        self.kind, self.m, self.k, self.sub_dim, self.dim, self.stages, self.n_nodes = list(info)

    def __del__(self):
        try:
            if self._o:
                _h.vqh_free(_vp(self._o))
                self._o = None
        except Exception:
            pass

    def quantize(self, vector):
        """quantize(&self, &Vector<f32>) -> Vector<f16>"""
        v = np.ascontiguousarray(vector, np.float32).reshape(-1)
        out = np.zeros(max(self.dim, v.size), np.uint16)
        got = _i64(0)
        _check(_h.vqh_quantize(_vp(self._o), _p(v), _i64(v.size), _p(out), C.byref(got)))
        return out[:got.value].view(np.float16)

    def quantize_batch(self, data):
        x = _rows(data)
        out = np.zeros(x.shape, np.uint16)
        _check(_h.vqh_quantize_batch(_vp(self._o), _p(x), _i64(x.shape[0]), _i64(x.shape[1]), _p(out)))
        return out.view(np.float16)

    def _encode(self, x, width):
        """n x width codes: bytes up to 256 centroids, uint16 above."""
        if self.k > 256:
            codes = np.zeros((x.shape[0], width), np.uint16)
            _check(_h.vqh_encode16(_vp(self._o), _p(x), _i64(x.shape[0]), _i64(x.shape[1]), _p(codes)))
        else:
            codes = np.zeros((x.shape[0], width), np.uint8)
            _check(_h.vqh_encode(_vp(self._o), _p(x), _i64(x.shape[0]), _i64(x.shape[1]), _p(codes)))
        return codes

    def quantize_batch_vectors(self, data, short_row=-1, short_len=0):
        """quantize_batch through the reference's shape, one heap-allocated vector per row; row
        `short_row` (if >= 0) is passed with only `short_len` floats."""
        x = _rows(data)
        out = np.zeros(x.shape, np.uint16)
        _check(_h.vqh_quantize_batch_vectors(_vp(self._o), _p(x), _i64(x.shape[0]), _i64(x.shape[1]),
                                             _i64(short_row), _i64(short_len), _p(out)))
        return out.view(np.float16)


class ProductQuantizer(_Quantizer):
    @classmethod
    def fit(cls, training_data, m, k, max_iters, distance, seed, streams=None):
        """src/pq.rs:79-86"""
        x = _rows(training_data)
        n, dim = x.shape
        init, reseed, nr = _streams(streams)
        kind, p = _dist(distance)
        h = _vp()
        _check(_h.vqh_pq_fit(_p(x), _i64(n), _i64(dim), _i64(m), _i64(k), _i64(max_iters), kind,
                             C.c_double(p), _u64(seed), _p(init), _p(reseed), _i32(nr), C.byref(h)))
        return cls(h.value)

    def encode(self, data):
        x = _rows(data)
        return self._encode(x, self.m)

    def codebooks(self):
        out = np.zeros((self.m, self.k, self.sub_dim), np.float32)
        _check(_h.vqh_codebooks(_vp(self._o), _p(out)))
        return out


class OptimizedProductQuantizer(_Quantizer):
    @classmethod
    def fit(cls, training_data, m, k, max_iters, opq_iters, distance, seed, streams=None):
        """src/opq.rs:90-98"""
        x = _rows(training_data)
        n, dim = x.shape
        init, reseed, nr = _streams(streams)
        kind, p = _dist(distance)
        h = _vp()
        _check(_h.vqh_opq_fit(_p(x), _i64(n), _i64(dim), _i64(m), _i64(k), _i64(max_iters),
                              _i64(opq_iters), kind, C.c_double(p), _u64(seed), _p(init), _p(reseed),
                              _i32(nr), C.byref(h)))
        return cls(h.value)  # m, k, sub_dim from vqh_info; k = 0 when opq_iters == 0 left no codebooks

    def quantize_batch(self, data):
        if self.k == 0:  # the reference returns an empty vector per row (src/opq.rs:122,244-263)
            x = _rows(data)
            _check(_h.vqh_quantize_batch(_vp(self._o), _p(x), _i64(x.shape[0]), _i64(x.shape[1]), None))
            return np.zeros((x.shape[0], 0), np.float16)
        return super().quantize_batch(data)

    def encode(self, data):
        x = _rows(data)
        return self._encode(x, self.m)

    def codebooks(self):
        out = np.zeros((self.m, self.k, self.sub_dim), np.float32)
        _check(_h.vqh_codebooks(_vp(self._o), _p(out)))
        return out

    def rotation(self):
        out = np.zeros((self.dim, self.dim), np.float32)
        _check(_h.vqh_rotation(_vp(self._o), _p(out)))
        return out


class ResidualQuantizer(_Quantizer):
    @classmethod
    def fit(cls, training_data, stages, k, max_iters, epsilon, distance, seed, streams=None):
        """src/rvq.rs:87-95"""
        x = _rows(training_data)
        n, dim = x.shape
        init, reseed, nr = _streams(streams)
        kind, p = _dist(distance)
        h = _vp()
        _check(_h.vqh_rvq_fit(_p(x), _i64(n), _i64(dim), _i64(stages), _i64(k), _i64(max_iters),
                              C.c_float(epsilon), kind, C.c_double(p), _u64(seed), _p(init), _p(reseed),
                              _i32(nr), C.byref(h)))
        q = cls(h.value)
        q.k = k
        return q

    def encode(self, data):
        x = _rows(data)
        return self._encode(x, self.stages)

    def codebooks(self):
        out = np.zeros((self.stages, self.k, self.dim), np.float32)
        _check(_h.vqh_codebooks(_vp(self._o), _p(out)))
        return out


class TSVQ(_Quantizer):
    @classmethod
    def new(cls, training_data, max_depth, distance):
        """src/tsvq.rs:209"""
        x = _rows(training_data)
        n, dim = x.shape
        kind, p = _dist(distance)
        h = _vp()
        _check(_h.vqh_tsvq_new(_p(x), _i64(n), _i64(dim), _i64(max_depth), kind, C.c_double(p), C.byref(h)))
        return cls(h.value)

    @classmethod
    def new_kmeans(cls, training_data, max_depth, lbg_iters, distance, seed, draws=None):
        """Not in the crate: the tree with 2-means splits (lbg_quantize with k = 2 per node) instead of
        the median split.  draws (optional): (2**max_depth - 1, 2 + lbg_iters) uint32."""
        x = _rows(training_data)
        n, dim = x.shape
        kind, p = _dist(distance)
        d = None if draws is None else np.ascontiguousarray(draws, np.uint32)
        h = _vp()
        _check(_h.vqh_tsvq_new_kmeans(_p(x), _i64(n), _i64(dim), _i64(max_depth), _i64(lbg_iters), kind, C.c_double(p),
                                      _u64(seed), _p(d), C.byref(h)))
        return cls(h.value)

    def leaves(self, data):
        x = _rows(data)
        out = np.zeros(x.shape[0], np.int32)
        _check(_h.vqh_leaves(_vp(self._o), _p(x), _i64(x.shape[0]), _i64(x.shape[1]), _p(out)))
        return out

    def tree(self):
        cen = np.zeros((self.n_nodes, self.dim), np.float32)
        left = np.zeros(self.n_nodes, np.int32)
        right = np.zeros(self.n_nodes, np.int32)
        _check(_h.vqh_tree(_vp(self._o), _p(cen), _p(left), _p(right)))
        return dict(centroids=cen, left=left, right=right)
