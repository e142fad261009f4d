"""The C-ABI library loads and exports every symbol include/am_hip.h declares; the host mirror
raises the reference's exception types for bad arguments — CPU only, no compute call is made."""
import ctypes
import os
import re

import numpy as np
import pytest

import arraymancer_amd as am
from arraymancer_amd import _lib, metadata as md
from arraymancer_amd.tensor_hip import HipTensor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "am_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(am_hip_\w+)\s*\(", text)))


def test_header_and_binding_agree():
    syms = declared_symbols()
    assert len(syms) >= 30
    assert sorted(_lib.SIGNATURES) == syms


def test_nim_and_cpp_host_layers_bind_every_declared_symbol():
    """nim/hip_abi.nim imports each entry point the header declares; the C++ host layer includes the header itself."""
    nim = open(os.path.join(ROOT, "nim", "hip_abi.nim")).read()
    for s in declared_symbols():
        assert re.search(rf"\bproc {s}\*\(", nim), f"{s} has no importc declaration in nim/hip_abi.nim"
    assert '#include "am_hip.h"' in open(os.path.join(ROOT, "include", "am_hip_tensor.hpp")).read()


def test_library_exports_every_declared_symbol():
    L = ctypes.CDLL(_lib.LIB_PATH)
    for s in declared_symbols():
        assert hasattr(L, s), s


def test_status_and_version_without_device():
    L = am.load_library()
    assert b"gfx950" in L.am_hip_version()
    n = ctypes.c_int(-1)
    assert L.am_hip_device_count(ctypes.byref(n)) == _lib.AM_OK and n.value >= 0


class _FakeStorage:
    ptr, nelems, itemsize = 0x1000, 1 << 20, 4


def _fake(shape, dtype=np.float32):
    return HipTensor(md.contiguous(shape), _FakeStorage(), dtype)


def test_host_side_checks_raise_like_the_reference():
    # matmul dimension mismatch -> IndexDefect in the reference (test_operators_blas.nim:110-117)
    c = _fake((2, 3))
    with pytest.raises(IndexError):
        am.matmul(c, c)
    # rank errors -> ValueError (operators_blas_l2l3.nim:100)
    with pytest.raises(ValueError):
        am.matmul(_fake((3,)), _fake((3, 2)))
    # element-wise shape mismatch -> ValueError (test_operators_blas_cuda.nim:156-158)
    with pytest.raises(ValueError):
        _fake((3, 3)) + _fake((2, 2))
    with pytest.raises(ValueError):
        am.bc_add(_fake((4, 2)), _fake((1, 3)))
    with pytest.raises(ValueError):
        _fake((4, 3)).bc_iadd(_fake((4, 1)).broadcast((4, 3))[:, :2])
    with pytest.raises(TypeError):
        am.map2("add", _fake((2, 2)), _fake((2, 2), np.float64))
    with pytest.raises(TypeError):
        am.empty((2, 2), np.float16)


def test_views_are_metadata_only():
    t = _fake((6, 4))
    v = t.transpose()[1:3]
    assert v.storage is t.storage and v.shape == (2, 6) and v.strides == (1, 4) and v.offset == 1
    assert t.broadcast((6, 4)).strides == (4, 1)
    assert _fake((1, 4)).broadcast((6, 4)).strides == (0, 1)
    assert v.data_ptr() == 0x1000 + 4
