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


_C2NIM = {"int": "cint", "int64_t": "int64", "int32_t": "int32", "uint8_t": "uint8", "float": "cfloat", "double": "cdouble",
          "size_t": "csize_t", "void*": "pointer", "char*": "cstring", "void**": "ptr pointer"}


def _c_type_as_nim(ctype: str) -> str:
    t = re.sub(r"\bconst\b", "", ctype).replace(" ", "")
    if t in _C2NIM:
        return _C2NIM[t]
    if t.endswith("*"):
        return "ptr " + _c_type_as_nim(t[:-1])
    raise AssertionError(f"no Nim spelling known for C type {ctype!r}")


def c_prototypes():
    """name -> (result type, [parameter types]) of every prototype in include/am_hip.h, spelled as Nim types."""
    text = open(os.path.join(ROOT, "include", "am_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#[^\n]*$", "", text, flags=re.M)                    # preprocessor lines
    text = text.replace('extern "C" {', "")
    out = {}
    for stmt in text.split(";"):
        m = re.match(r"^([\w\s\*]+?)\b(am_hip_\w+)\s*\(([^)]*)\)\s*$", stmt.strip(), flags=re.S)
        if not m:
            continue
        res, name, params = m.group(1).strip(), m.group(2), m.group(3).strip()
        types = []
        if params != "void":
            for prm in params.split(","):
                pm = re.match(r"^(.*?)(\w+)$", prm.strip(), flags=re.S)   # the type is everything before the parameter's name
                types.append(_c_type_as_nim(pm.group(1)))
        out[name] = (_c_type_as_nim(res), types)
    return out


def nim_prototypes():
    """name -> (result type, [parameter types]) of every importc proc in nim/hip_abi.nim."""
    text = open(os.path.join(ROOT, "nim", "hip_abi.nim")).read()
    text = re.sub(r"#[^\n]*", "", text)
    out = {}
    for m in re.finditer(r"proc (am_hip_\w+)\*\(([^)]*)\)\s*(?::\s*([\w ]+?))?\s*\{\.importc\.\}", text, flags=re.S):
        name, params, res = m.group(1), m.group(2), (m.group(3) or "void").strip()
        types, pending = [], 0
        for piece in re.split(r"[;,]", params):
            piece = piece.strip()
            if not piece:
                continue
            if ":" in piece:            # `a, b, c: T` declares three parameters of type T
                types.extend([" ".join(piece.split(":", 1)[1].split())] * (pending + 1))
                pending = 0
            else:
                pending += 1
        assert pending == 0, name
        out[name] = (res, types)
    return out


def test_nim_binding_matches_the_header_type_for_type():
    """Arity and the C type of every parameter and result of nim/hip_abi.nim against include/am_hip.h (the Nim
    file cannot be compiled here, so this is the check that a swapped or mistyped parameter fails)."""
    c, nim = c_prototypes(), nim_prototypes()
    assert sorted(c) == declared_symbols()
    assert sorted(nim) == sorted(c)
    for name, (res, types) in c.items():
        nres, ntypes = nim[name]
        assert len(ntypes) == len(types), f"{name}: {len(ntypes)} parameters in Nim, {len(types)} in C"
        for i, (a, b) in enumerate(zip(types, ntypes)):
            assert a == b, f"{name}: parameter {i} is {b} in Nim, {a} in C"
        assert nres == res, f"{name}: result {nres} in Nim, {res} in C"


def test_ctypes_binding_matches_the_header_arity():
    c = c_prototypes()
    for name, (res, args) in _lib.SIGNATURES.items():
        assert len(args) == len(c[name][1]), name
        for i, (ct, nt) in enumerate(zip(args, c[name][1])):
            is_ptr = nt.startswith("ptr ") or nt in ("pointer", "cstring")
            got_ptr = ct in (ctypes.c_void_p, ctypes.c_char_p) or hasattr(ct, "contents")
            assert is_ptr == got_ptr, f"{name}: parameter {i} is {nt} in C, {ct} in ctypes"
            if not is_ptr:
                want = {"cint": ctypes.c_int, "int64": ctypes.c_int64, "int32": ctypes.c_int32, "cfloat": ctypes.c_float,
                        "cdouble": ctypes.c_double, "csize_t": ctypes.c_size_t}[nt]
                assert ct is want, f"{name}: parameter {i} is {nt} in C, {ct} in ctypes"


def test_header_is_plain_c99(tmp_path):
    import subprocess
    src = tmp_path / "use_header.c"
    src.write_text('#include "am_hip.h"\nint main(void) { return am_hip_version() == 0; }\n')
    res = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), str(src)],
                         capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


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


def test_graph_handles_that_the_library_did_not_hand_out_are_refused():
    """am_hip_graph_launch / _destroy accept only a live graph of am_hip_graph_end: a stale, foreign or twice-destroyed
    pointer is answered with AM_E_ARG before anything reaches the runtime (no device needed to refuse it)."""
    L = am.load_library()
    bogus = ctypes.c_void_p(0x1234560)
    assert L.am_hip_graph_launch(bogus) == _lib.AM_E_ARG and "not a graph" in _lib.last_error()
    assert L.am_hip_graph_destroy(bogus) == _lib.AM_E_ARG and "not a graph" in _lib.last_error()
    assert L.am_hip_graph_destroy(None) == _lib.AM_OK          # NULL: nothing to destroy
    assert L.am_hip_graph_launch(None) == _lib.AM_E_ARG


def test_unsigned_tensors_take_the_signed_kernels_for_ring_operations_only():
    """uint32 / uint64 ride the int32 / int64 kernels for + - * and products (gemm.nim:275-307); what reads the sign
    is a TypeError before any device call."""
    for dt, twin in ((np.uint32, "i32"), (np.uint64, "i64")):
        t = _fake((2, 2), dt)
        assert t.ring_sfx == twin
        with pytest.raises(TypeError, match="sign"):
            t.sfx
        for refused in (lambda: am.bc_div(t, t), lambda: am.bc_mod(t, t), lambda: t / 2, lambda: am.bc_lt(t, t),
                        lambda: am.min(t), lambda: am.max(t, 0), lambda: am.mean(t), lambda: am.relu(t), lambda: am.sgn(t)):
            with pytest.raises(TypeError):
                refused()
    assert _fake((2, 2), np.int32).ring_sfx == "i32" and _fake((2, 2)).ring_sfx == "f32"
    with pytest.raises(TypeError):
        am.empty((2, 2), np.uint16)


def test_digit_plane_handles_that_the_library_did_not_hand_out_are_refused():
    L = am.load_library()
    bogus = ctypes.c_void_p(0x1234560)
    assert L.am_hip_digits_release(bogus) == _lib.AM_E_ARG and "not a handle" in _lib.last_error()
    assert L.am_hip_digits_release(None) == _lib.AM_OK
    z = ctypes.c_void_p(0x1000)
    rc = L.am_hip_gemm_prepared_i32(4, 4, 4, 1, z, 4, 1, bogus, z, 4, 1, None, 0, z, 4, 1)
    assert rc == _lib.AM_E_ARG and "not a live handle" in _lib.last_error()
