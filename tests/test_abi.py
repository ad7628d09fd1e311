"""CPU-side checks of the C ABI: the library loads and exports every symbol the header
declares.  No compute call is made (there is no GPU here)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "vq_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vq_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_all_exported_and_bound():
    import ctypes
    from vq_amd import _ffi
    names = _declared()
    assert len(names) >= 10
    lib = ctypes.CDLL(_ffi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/vq_hip.h but not exported"
    assert set(names) == set(_ffi.SYMBOLS), set(names) ^ set(_ffi.SYMBOLS)


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present")
def test_context_creation_without_gpu_fails_loudly():
    import vq_amd
    with pytest.raises(vq_amd.VqError) as e:
        vq_amd.Context(0)
    assert e.value.code == vq_amd._ffi.ERR_HIP
