"""The C-ABI library loads and exports every symbol include/hchip.h declares, the ctypes
prototypes cover the same set, and creating a context without a GPU fails cleanly.
No compute calls."""
import ctypes
import os
import re

import pytest

from honeycrisp_amd import _lib
from honeycrisp_amd.backend import Backend, HIPBackend
from honeycrisp_amd.descriptors import BackendError

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "hchip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hc_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_families():
    syms = declared_symbols()
    for name in ("hc_init", "hc_malloc", "hc_memcpy_h2d", "hc_launch", "hc_matmul", "hc_binary_op",
                 "hc_elemwise", "hc_reduce", "hc_gather", "hc_axis_permutation", "hc_log_softmax"):
        assert name in syms


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, "libhchip.so does not export %s" % missing


def test_ctypes_prototypes_match_header():
    assert sorted(_lib.PROTOTYPES) == declared_symbols()


def test_struct_layout_matches_header():
    assert ctypes.sizeof(_lib.hc_strides) == 8 + 8 * 8 + 8 * 8
    assert _lib.hc_strides.shape.offset == 8 and _lib.hc_strides.strides.offset == 72


def test_bare_backend_is_the_poison_backend():
    """Every op of the base class raises notImplemented (Backend.swift:170-172 etc.)."""
    b = Backend()
    for call in (lambda: b.matmul(None, False, None, False, False, 1, 1, 1, None),
                 lambda: b.binaryOp(None, None, None, None),
                 lambda: b.gather(None, None, None), lambda: b.reduce(None, None, None, None)):
        with pytest.raises(BackendError) as e:
            call()
        assert e.value.kind == "notImplemented"


def test_init_without_gpu_fails_loudly():
    try:
        backend = HIPBackend()
    except BackendError as e:
        assert e.kind == "failedToLoadKernels"
        assert "HIP device" in str(e) or "gfx950" in str(e)
    else:
        info = backend.deviceInfo()
        assert info["arch"].startswith("gfx950")
