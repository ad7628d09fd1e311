"""vq_amd — MI355X-native codebook hot path of the `vq` crate (LBG training + encode).

Importing the package loads libvqhip.so; a missing library is an ImportError.
"""
from . import _ffi
from ._ffi import (COSINE, EUCLIDEAN, MANHATTAN, SQEUCLIDEAN, Context, DeviceArray, Tree,  # noqa: F401
                   VqError)
