"""ctypes binding of libvqhip.so (the C ABI declared in include/vq_hip.h).

The library is the only compute path: if it is missing or fails to load, importing this
module raises — there is no CPU fallback.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libvqhip.so")

VQ_OK = 0
ERR_INVALID_ARG, ERR_DIM_MISMATCH, ERR_EMPTY_INPUT = -1, -2, -3
ERR_UNSUPPORTED, ERR_OOM, ERR_HIP, ERR_RESEED_EXHAUSTED = -4, -5, -6, -7

SQEUCLIDEAN, EUCLIDEAN, COSINE, MANHATTAN = 0, 1, 2, 3
PROF_LBG_ASSIGN, PROF_LBG_UPDATE, PROF_ENCODE, PROF_ASSIGN_KERNEL = 0, 1, 2, 3

# every symbol include/vq_hip.h declares: name -> (restype, argtypes)
_vp, _i32, _i64, _sz = C.c_void_p, C.c_int32, C.c_int64, C.c_size_t
SYMBOLS = {
    "vq_ctx_create": (_i32, [_i32, C.POINTER(_vp)]),
    "vq_ctx_destroy": (_i32, [_vp]),
    "vq_last_error": (C.c_char_p, [_vp]),
    "vq_ctx_sync": (_i32, [_vp]),
    "vq_ctx_stream": (_vp, [_vp]),
    "vq_ctx_set_assign_path": (_i32, [_vp, _i32]),
    "vq_ctx_set_tsvq_variance_path": (_i32, [_vp, _i32]),
    "vq_calibrate": (_i32, [_vp, _i32, C.POINTER(C.c_double)]),
    "vq_ctx_set_procrustes_path": (_i32, [_vp, _i32]),
    "vq_ctx_set_tsvq_descend_path": (_i32, [_vp, _i32]),
    "vq_calibrate_overlap": (_i32, [_vp, _i32, C.POINTER(C.c_double), C.POINTER(C.c_uint32)]),
    "vq_ctx_last_recheck_count": (_i32, [_vp, C.POINTER(C.c_uint32)]),
    "vq_ctx_last_recheck_split": (_i32, [_vp, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "vq_procrustes_rotation": (_i32, [_vp, _vp, _i32, _vp]),
    "vq_malloc": (_i32, [_vp, _sz, C.POINTER(_vp)]),
    "vq_free": (_i32, [_vp, _vp]),
    "vq_host_alloc": (_i32, [_vp, _sz, C.POINTER(_vp)]),
    "vq_host_free": (_i32, [_vp, _vp]),
    "vq_h2d": (_i32, [_vp, _vp, _vp, _sz]),
    "vq_d2h": (_i32, [_vp, _vp, _vp, _sz]),
    "vq_copy_f32": (_i32, [_vp, _vp, _vp, _i64]),
    "vq_timer_start": (_i32, [_vp]),
    "vq_timer_stop": (_i32, [_vp, C.POINTER(C.c_float)]),
    "vq_prof_enable": (_i32, [_vp, _i32]),
    "vq_prof_read": (_i32, [_vp, _i32, C.POINTER(C.c_double), C.POINTER(_i64)]),
    "vq_lbg_fit": (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _i32, _i32, _vp, _vp, _i32, _vp, _vp,
                          _vp]),
    "vq_lbg_fit_residual": (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _i32, _vp, _vp, _i32, _vp, _vp, _i32, _vp,
                                   _vp, _vp]),
    "vq_assign": (_i32, [_vp, _i32, _vp, _i64, _i64, _i32, _i32, _i32, _vp, _vp]),
    "vq_assign_noalloc": (_i32, [_vp, _i32, _vp, _i64, _i64, _i32, _i32, _i32, _vp, _vp]),
    "vq_assign_u16": (_i32, [_vp, _i32, _vp, _i64, _i64, _i32, _i32, _i32, _vp, _vp]),
    "vq_decode_f16": (_i32, [_vp, _vp, _i64, _i32, _i32, _i32, _vp, _vp]),
    "vq_decode_f32": (_i32, [_vp, _vp, _i64, _i32, _i32, _i32, _vp, _vp]),
    "vq_decode_f16_u16": (_i32, [_vp, _vp, _i64, _i32, _i32, _i32, _vp, _vp]),
    "vq_decode_f32_u16": (_i32, [_vp, _vp, _i64, _i32, _i32, _i32, _vp, _vp]),
    "vq_residual_sub": (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _vp, _vp]),
    "vq_residual_sub_u16": (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _vp, _vp]),
    "vq_rvq_encode_u16": (_i32, [_vp, _i32, _vp, _i64, _i64, _i32, _i32, _i32, _vp, C.c_float, _vp, _vp,
                                 _vp]),
    "vq_mean_l2norm": (_i32, [_vp, _vp, _i64, _i64, _i32, C.POINTER(C.c_float)]),
    "vq_rvq_encode": (_i32, [_vp, _i32, _vp, _i64, _i64, _i32, _i32, _i32, _vp, C.c_float, _vp, _vp,
                             _vp]),
    "vq_rotate": (_i32, [_vp, _vp, _i64, _i64, _i32, _vp, _vp]),
    "vq_cross_cov": (_i32, [_vp, _vp, _vp, _i64, _i32, _vp]),
    "vq_tsvq_build": (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, C.POINTER(_vp)]),
    "vq_tsvq_build_kmeans": (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _i32, _vp, _i32, C.POINTER(_vp)]),
    "vq_tree_create": (_i32, [_vp, _i32, _i32, _vp, _vp, _vp, C.POINTER(_vp)]),
    "vq_tree_free": (_i32, [_vp, _vp]),
    "vq_tree_info": (_i32, [_vp, C.POINTER(_i32), C.POINTER(_i32)]),
    "vq_tree_download": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "vq_tsvq_descend": (_i32, [_vp, _i32, _vp, _i64, _i64, _vp, _vp]),
    "vq_tsvq_decode_f16": (_i32, [_vp, _vp, _vp, _i64, _vp]),
}


class VqError(RuntimeError):
    """Raised for any non-zero status of the C ABI; .code holds the status."""

    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


def load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `python -m vq_amd.build` "
                          "(there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = load()


def lib():
    return _lib


class DeviceArray:
    """A typed device allocation owned by a Context."""

    def __init__(self, ctx, shape, dtype):
        self.ctx = ctx
        self.shape = tuple(int(s) for s in np.atleast_1d(shape))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        p = _vp()
        ctx._check(_lib.vq_malloc(ctx._h, self.nbytes, C.byref(p)))
        self.ptr = p.value

    def upload(self, host):
        host = np.ascontiguousarray(host, dtype=self.dtype)
        assert host.nbytes == self.nbytes, (host.shape, self.shape)
        self.ctx._check(_lib.vq_h2d(self.ctx._h, self.ptr, host.ctypes.data, self.nbytes))
        return self

    def download(self):
        out = np.empty(self.shape, self.dtype)
        self.ctx._check(_lib.vq_d2h(self.ctx._h, out.ctypes.data, self.ptr, self.nbytes))
        return out

    def free(self):
        if self.ptr:
            _lib.vq_free(self.ctx._h, self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Tree:
    """A TSVQ node table held by the library (breadth-first node numbering)."""

    def __init__(self, ctx, handle):
        self.ctx, self._h = ctx, handle
        nn, dim = _i32(0), _i32(0)
        ctx._check(_lib.vq_tree_info(handle, C.byref(nn), C.byref(dim)))
        self.n_nodes, self.dim = nn.value, dim.value

    def download(self):
        nn, dim = self.n_nodes, self.dim
        cen = np.empty((nn, dim), np.float32)
        left, right, sdim = (np.empty(nn, np.int32) for _ in range(3))
        sval = np.empty(nn, np.float32)
        cnt = np.empty(nn, np.int64)
        self.ctx._check(_lib.vq_tree_download(self._h, cen.ctypes.data, left.ctypes.data,
                                              right.ctypes.data, sdim.ctypes.data, sval.ctypes.data,
                                              cnt.ctypes.data))
        return dict(n_nodes=nn, centroids=cen, left=left, right=right, split_dim=sdim,
                    split_val=sval, count=cnt)

    def free(self):
        if self._h:
            _lib.vq_tree_free(self.ctx._h, self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Context:
    def __init__(self, device=0):
        h = _vp()
        rc = _lib.vq_ctx_create(device, C.byref(h))
        if rc != VQ_OK:
            raise VqError(rc, (_lib.vq_last_error(None) or b"").decode())
        self._h = h
        self._pinned = {}

    def close(self):
        if self._h:
            if self._pinned:
                # arrays handed out by host_empty() view this memory: after close() they dangle
                import warnings
                warnings.warn(f"Context.close(): {len(self._pinned)} page-locked array(s) from host_empty() were "
                              "not released with host_free(); their memory is freed now and the arrays "
                              "must not be used any more", ResourceWarning, stacklevel=2)
            for p in list(self._pinned.values()):
                _lib.vq_host_free(self._h, p)
            self._pinned.clear()
            _lib.vq_ctx_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc):
        if rc != VQ_OK:
            raise VqError(rc, (_lib.vq_last_error(self._h) or b"").decode())

    # -- memory ------------------------------------------------------------------------------
    def empty(self, shape, dtype):
        return DeviceArray(self, shape, dtype)

    def to_device(self, host, dtype=None):
        host = np.ascontiguousarray(host, dtype=dtype)
        return DeviceArray(self, host.shape, host.dtype).upload(host)

    def host_empty(self, shape, dtype):
        """A numpy array over page-locked host memory (vq_host_alloc).  The array does not own the
        memory: release it with host_free(array) once no view of it is in use, and before the
        context is closed — close() frees what is left (with a ResourceWarning), after which the
        array and every view of it point at freed memory."""
        dtype = np.dtype(dtype)
        shape = tuple(int(s) for s in np.atleast_1d(shape))
        nbytes = int(np.prod(shape)) * dtype.itemsize
        p = _vp()
        self._check(_lib.vq_host_alloc(self._h, nbytes, C.byref(p)))
        buf = (C.c_char * max(nbytes, 1)).from_address(p.value)
        arr = np.frombuffer(buf, dtype=dtype, count=int(np.prod(shape))).reshape(shape)
        self._pinned[arr.ctypes.data] = p.value
        return arr

    def host_free(self, arr):
        p = self._pinned.pop(arr.ctypes.data, None)
        if p:
            self._check(_lib.vq_host_free(self._h, p))

    def copy_f32(self, d_dst, d_src, count):
        self._check(_lib.vq_copy_f32(self._h, d_dst.ptr, d_src.ptr, count))

    def set_assign_path(self, path):
        """0 = matrix cores + exact re-check (default), 1 = vector ALU only."""
        self._check(_lib.vq_ctx_set_assign_path(self._h, path))

    def calibrate(self, what):
        """Measured peak: 0 copy GB/s (read + write); 1-5 wave64 instructions per second of
        v_fma_f32, v_min3_i32, v_med3_i32, v_and_or_b32, v_add_u32 over the whole GPU."""
        out = C.c_double(0)
        self._check(_lib.vq_calibrate(self._h, what, C.byref(out)))
        return out.value

    def calibrate_overlap(self, mode):
        """Milliseconds of (matrix instructions alone, vector instructions alone, both together) on
        every SIMD; mode 0: from different waves, 1 / 2: one stream with 7 / 3 vector instructions
        per matrix instruction.  Second value: waves per SIMD number (mode 0: four counts of the matrix
        waves, four of the vector waves)."""
        out = (C.c_double * 3)()
        waves = (C.c_uint32 * 8)()
        self._check(_lib.vq_calibrate_overlap(self._h, mode, out, waves))
        return tuple(out), tuple(waves)

    def set_tsvq_variance_path(self, path):
        """0: composed integer maps (default); 1: one chain of adds per column."""
        self._check(_lib.vq_ctx_set_tsvq_variance_path(self._h, path))

    def last_recheck_count(self):
        c = C.c_uint32(0)
        self._check(_lib.vq_ctx_last_recheck_count(self._h, C.byref(c)))
        return c.value

    def last_recheck_split(self):
        """(pairs decided over all centroids, pairs decided between two candidates)."""
        a, b = C.c_uint32(0), C.c_uint32(0)
        self._check(_lib.vq_ctx_last_recheck_split(self._h, C.byref(a), C.byref(b)))
        return a.value, b.value

    def sync(self):
        self._check(_lib.vq_ctx_sync(self._h))

    def timer_start(self):
        self._check(_lib.vq_timer_start(self._h))

    def timer_stop(self):
        ms = C.c_float(0)
        self._check(_lib.vq_timer_stop(self._h, C.byref(ms)))
        return ms.value

    def prof_enable(self, on=True):
        self._check(_lib.vq_prof_enable(self._h, 1 if on else 0))

    def prof_read(self, cls):
        """(total_ms, spans) of PROF_LBG_ASSIGN / PROF_LBG_UPDATE / PROF_ENCODE."""
        ms, cnt = C.c_double(0), _i64(0)
        self._check(_lib.vq_prof_read(self._h, cls, C.byref(ms), C.byref(cnt)))
        return ms.value, cnt.value

    # -- compute -----------------------------------------------------------------------------
    def lbg_fit(self, d_x, n, ld, m, sub_dim, k, max_iters, init_idx, reseed_stream, d_codebooks):
        init_idx = np.ascontiguousarray(init_idx, np.uint32).reshape(-1)
        reseed_stream = np.ascontiguousarray(reseed_stream, np.uint32).reshape(m, -1) \
            if np.size(reseed_stream) else np.zeros((m, 0), np.uint32)
        n_reseed = reseed_stream.shape[1]
        iters = np.zeros(m, np.int32)
        used = np.zeros(m, np.int32)
        self._check(_lib.vq_lbg_fit(self._h, _ptr(d_x), n, ld, m, sub_dim, k, max_iters,
                                    init_idx.ctypes.data, reseed_stream.ctypes.data if n_reseed
                                    else None, n_reseed, _ptr(d_codebooks), iters.ctypes.data,
                                    used.ctypes.data))
        return iters, used

    def lbg_fit_residual(self, d_res, n, ld, dim, k, max_iters, init_idx, reseed_stream, d_codebook,
                         d_prev_codebook, k_prev, d_prev_codes):
        """d_res[i] -= d_prev_codebook[d_prev_codes[i]], then lbg_fit (m = 1) on the updated rows."""
        init_idx = np.ascontiguousarray(init_idx, np.uint32).reshape(-1)
        reseed_stream = np.ascontiguousarray(reseed_stream, np.uint32).reshape(1, -1) \
            if np.size(reseed_stream) else np.zeros((1, 0), np.uint32)
        n_reseed = reseed_stream.shape[1]
        iters = np.zeros(1, np.int32)
        used = np.zeros(1, np.int32)
        self._check(_lib.vq_lbg_fit_residual(self._h, _ptr(d_res), n, ld, dim, k, max_iters,
                                             init_idx.ctypes.data, reseed_stream.ctypes.data if n_reseed
                                             else None, n_reseed, _ptr(d_codebook), _ptr(d_prev_codebook),
                                             k_prev, _ptr(d_prev_codes), iters.ctypes.data, used.ctypes.data))
        return iters, used

    def assign(self, metric, d_x, n, ld, m, sub_dim, k, d_codebooks, d_codes):
        self._check(_lib.vq_assign(self._h, metric, _ptr(d_x), n, ld, m, sub_dim, k,
                                   _ptr(d_codebooks), _ptr(d_codes)))

    def assign_noalloc(self, metric, d_x, n, ld, m, sub_dim, k, d_codebooks, d_codes):
        """vq_assign without any device allocation (fixed scratch; m * k padded <= 16384)."""
        self._check(_lib.vq_assign_noalloc(self._h, metric, _ptr(d_x), n, ld, m, sub_dim, k,
                                           _ptr(d_codebooks), _ptr(d_codes)))

    def assign_u16(self, metric, d_x, n, ld, m, sub_dim, k, d_codebooks, d_codes):
        """vq_assign with uint16 codes (k <= 65536)."""
        self._check(_lib.vq_assign_u16(self._h, metric, _ptr(d_x), n, ld, m, sub_dim, k,
                                       _ptr(d_codebooks), _ptr(d_codes)))

    def decode_f16_u16(self, d_codes, n, m, sub_dim, k, d_codebooks, d_out):
        self._check(_lib.vq_decode_f16_u16(self._h, d_codes.ptr, n, m, sub_dim, k, d_codebooks.ptr,
                                           d_out.ptr))

    def decode_f32_u16(self, d_codes, n, m, sub_dim, k, d_codebooks, d_out):
        self._check(_lib.vq_decode_f32_u16(self._h, d_codes.ptr, n, m, sub_dim, k, d_codebooks.ptr,
                                           d_out.ptr))

    def decode_f16(self, d_codes, n, m, sub_dim, k, d_codebooks, d_out):
        self._check(_lib.vq_decode_f16(self._h, d_codes.ptr, n, m, sub_dim, k, d_codebooks.ptr,
                                       d_out.ptr))

    def decode_f32(self, d_codes, n, m, sub_dim, k, d_codebooks, d_out):
        self._check(_lib.vq_decode_f32(self._h, d_codes.ptr, n, m, sub_dim, k, d_codebooks.ptr,
                                       d_out.ptr))

    # -- residual quantizer --------------------------------------------------------------------
    def residual_sub(self, d_res, n, ld, dim, k, d_codebook, d_codes):
        self._check(_lib.vq_residual_sub(self._h, d_res.ptr, n, ld, dim, k, _ptr(d_codebook),
                                         d_codes.ptr))

    def residual_sub_u16(self, d_res, n, ld, dim, k, d_codebook, d_codes):
        self._check(_lib.vq_residual_sub_u16(self._h, d_res.ptr, n, ld, dim, k, _ptr(d_codebook),
                                             d_codes.ptr))

    def mean_l2norm(self, d_x, n, ld, dim):
        out = C.c_float(0)
        self._check(_lib.vq_mean_l2norm(self._h, d_x.ptr, n, ld, dim, C.byref(out)))
        return out.value

    def rvq_encode(self, metric, d_x, n, ld, dim, stages, k, d_codebooks, epsilon, d_codes,
                   d_used=None, d_recon=None):
        self._check(_lib.vq_rvq_encode(self._h, metric, d_x.ptr, n, ld, dim, stages, k,
                                       d_codebooks.ptr, epsilon, d_codes.ptr,
                                       d_used.ptr if d_used else None,
                                       d_recon.ptr if d_recon else None))

    def rvq_encode_u16(self, metric, d_x, n, ld, dim, stages, k, d_codebooks, epsilon, d_codes,
                       d_used=None, d_recon=None):
        self._check(_lib.vq_rvq_encode_u16(self._h, metric, d_x.ptr, n, ld, dim, stages, k,
                                           d_codebooks.ptr, epsilon, d_codes.ptr,
                                           d_used.ptr if d_used else None,
                                           d_recon.ptr if d_recon else None))

    # -- optimized product quantizer -----------------------------------------------------------
    def rotate(self, d_x, n, ld, dim, d_R, d_y):
        self._check(_lib.vq_rotate(self._h, d_x.ptr, n, ld, dim, d_R.ptr, d_y.ptr))

    def cross_cov(self, d_y, d_x, n, dim):
        A = np.empty((dim, dim), np.float64)
        self._check(_lib.vq_cross_cov(self._h, d_y.ptr, d_x.ptr, n, dim, A.ctypes.data))
        return A

    def set_tsvq_descend_path(self, path):
        """0: one inner product per node where it decides (default); 1: two distances per node always."""
        self._check(_lib.vq_ctx_set_tsvq_descend_path(self._h, path))

    def set_procrustes_path(self, path):
        """0: Newton-Schulz polar factor first, the SVD when it does not converge (default); 1: SVD only."""
        self._check(_lib.vq_ctx_set_procrustes_path(self._h, path))

    def procrustes_rotation(self, A):
        A = np.ascontiguousarray(A, np.float64)
        R = np.empty_like(A)
        self._check(_lib.vq_procrustes_rotation(self._h, A.ctypes.data, A.shape[0], R.ctypes.data))
        return R

    # -- tree-structured VQ --------------------------------------------------------------------
    def tsvq_build(self, d_x, n, ld, dim, max_depth):
        h = _vp()
        self._check(_lib.vq_tsvq_build(self._h, d_x.ptr, n, ld, dim, max_depth, C.byref(h)))
        return Tree(self, h)

    def tsvq_build_kmeans(self, d_x, n, ld, dim, max_depth, lbg_iters, draws):
        """The tree with 2-means splits (not the reference's median split).  draws: uint32 array of
        shape (2**max_depth - 1, per_node), per_node >= 2 + lbg_iters."""
        draws = np.ascontiguousarray(draws, np.uint32)
        per_node = draws.shape[-1] if draws.ndim > 1 else int(draws.size)
        h = _vp()
        self._check(_lib.vq_tsvq_build_kmeans(self._h, d_x.ptr, n, ld, dim, max_depth, lbg_iters,
                                              draws.ctypes.data if draws.size else None, per_node, C.byref(h)))
        return Tree(self, h)

    def tree_create(self, centroids, left, right):
        cen = np.ascontiguousarray(centroids, np.float32)
        left = np.ascontiguousarray(left, np.int32)
        right = np.ascontiguousarray(right, np.int32)
        h = _vp()
        self._check(_lib.vq_tree_create(self._h, cen.shape[0], cen.shape[1], cen.ctypes.data,
                                        left.ctypes.data, right.ctypes.data, C.byref(h)))
        return Tree(self, h)

    def tsvq_descend(self, metric, d_x, n, ld, tree, d_leaf):
        self._check(_lib.vq_tsvq_descend(self._h, metric, d_x.ptr, n, ld, tree._h, d_leaf.ptr))

    def tsvq_decode_f16(self, tree, d_leaf, n, d_out):
        self._check(_lib.vq_tsvq_decode_f16(self._h, tree._h, d_leaf.ptr, n, d_out.ptr))


def _ptr(a):
    """Device address of a DeviceArray or a raw integer address."""
    return a.ptr if isinstance(a, DeviceArray) else a
