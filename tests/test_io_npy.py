""".npy I/O (src/arraymancer/io/io_npy.nim:64-183). The files under tests/golden/npy are the data
files of the reference's own test (tests/io/npy_files/*.npy, written there by NumPy); its
expectations are tests/io/test_numpy.nim:15-96. Host half (parser, writer bytes) here without a
GPU; the device round trips carry the gpu marker."""
import os

import numpy as np
import pytest

from arraymancer_amd import io_npy

NPY = os.path.join(os.path.dirname(__file__), "golden", "npy")
EXPECTED_1D = np.array([1, 2, 3, 4], dtype=np.int64)
EXPECTED_2D = np.array([[1, 2, 3, 4], [5, 6, 7, 8]], dtype=np.int64)
FILES = {
    "int.npy": (EXPECTED_1D, False), "int_2D_c.npy": (EXPECTED_2D, False), "int_2D_f.npy": (EXPECTED_2D, True),
    "f32LE.npy": (EXPECTED_1D, False), "f32LE_2D_c.npy": (EXPECTED_2D, False), "f32LE_2D_f.npy": (EXPECTED_2D, True),
    "u64BE.npy": (EXPECTED_1D, False), "u64BE_2D_c.npy": (EXPECTED_2D, False), "u64BE_2D_f.npy": (EXPECTED_2D, True),
}


@pytest.mark.parametrize("name", sorted(FILES))
def test_parser_on_reference_files(name):
    want, fortran = FILES[name]
    raw, shape, is_f = io_npy.parse_npy(os.path.join(NPY, name))
    assert shape == want.shape and is_f == fortran
    got = raw.astype(np.int64).reshape(shape, order="F" if is_f else "C")
    assert np.array_equal(got, want)
    # and NumPy's own loader agrees on what the file holds
    assert np.array_equal(np.load(os.path.join(NPY, name), allow_pickle=False).astype(np.int64), want)


@pytest.mark.parametrize("name", ["int.npy", "int_2D_c.npy", "int_2D_f.npy", "f32LE.npy", "f32LE_2D_c.npy", "f32LE_2D_f.npy"])
def test_writer_bytes_equal_reference_files(name):
    """test_numpy.nim:58-83: the bytes written for the expected tensors equal the NumPy-written files."""
    want, fortran = FILES[name]
    dt = np.float32 if name.startswith("f32") else np.int64
    host = np.ascontiguousarray(want.astype(dt))
    assert io_npy.npy_bytes(host, fortran) == open(os.path.join(NPY, name), "rb").read()


def test_big_endian_writer_bytes():
    for name in ("u64BE.npy", "u64BE_2D_c.npy", "u64BE_2D_f.npy"):
        want, fortran = FILES[name]
        host = np.ascontiguousarray(want.astype(">u8"))
        assert io_npy.npy_bytes(host, fortran) == open(os.path.join(NPY, name), "rb").read()


def test_header_padding_and_version_2(tmp_path):
    # data starts on a 16-byte boundary whatever the header length
    for shape in [(1,), (12345,), (3, 1, 7, 11, 2, 5)]:
        b = io_npy.npy_bytes(np.zeros(shape, np.float64), False)
        hl = int.from_bytes(b[8:10], "little")
        assert b[6:8] == b"\x01\x00" and (10 + hl) % 16 == 0 and b[10 + hl - 1:10 + hl] == b"\n"
        assert len(b) == 10 + hl + 8 * int(np.prod(shape))
    # a version 2.0 file (4-byte header length) is read back
    p = tmp_path / "v2.npy"
    header = "{'descr': '<i4', 'fortran_order': False, 'shape': (3,), }".ljust(53) + "\n"
    p.write_bytes(b"\x93NUMPY\x02\x00" + len(header).to_bytes(4, "little") + header.encode() + np.array([7, 8, 9], "<i4").tobytes())
    raw, shape, f = io_npy.parse_npy(str(p))
    assert shape == (3,) and not f and raw.tolist() == [7, 8, 9]


def test_parser_errors(tmp_path):
    with pytest.raises(IOError):
        io_npy.parse_npy(str(tmp_path / "missing.npy"))
    bad = tmp_path / "bad.npy"
    bad.write_bytes(b"not a numpy file at all")
    with pytest.raises(AssertionError):
        io_npy.parse_npy(str(bad))
    c = tmp_path / "complex.npy"
    np.save(c, np.zeros(3, np.complex64))
    with pytest.raises((ValueError, AssertionError)):
        io_npy.parse_npy(str(c))


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(FILES))
def test_read_npy_to_device(hip, name):
    want, fortran = FILES[name]
    for dt in (np.int64, np.int32, np.float32, np.float64):
        t = hip.read_npy(os.path.join(NPY, name), dt)
        assert t.dtype == np.dtype(dt) and t.shape == want.shape
        assert (t.is_F_contiguous() and not t.is_C_contiguous()) == (fortran and want.ndim > 1)
        assert np.array_equal(t.toCpu(), want.astype(dt))


@pytest.mark.gpu
def test_write_npy_from_device(hip, tmp_path):
    out = str(tmp_path / "out.npy")
    e2 = hip.toHip(EXPECTED_2D)
    hip.write_npy(hip.toHip(EXPECTED_1D), out)
    assert open(out, "rb").read() == open(os.path.join(NPY, "int.npy"), "rb").read()
    hip.write_npy(e2, out)
    assert open(out, "rb").read() == open(os.path.join(NPY, "int_2D_c.npy"), "rb").read()
    # column-major tensor -> fortran_order: True (asContiguous(colMajor, force = true) in the reference's test)
    f = hip.toHip(np.ascontiguousarray(EXPECTED_2D.T)).transpose()
    hip.write_npy(f, out)
    assert open(out, "rb").read() == open(os.path.join(NPY, "int_2D_f.npy"), "rb").read()
    hip.write_npy(hip.toHip(EXPECTED_2D.astype(np.float32)), out)
    assert open(out, "rb").read() == open(os.path.join(NPY, "f32LE_2D_c.npy"), "rb").read()
    # a strided view is made contiguous first; NumPy reads back the same values
    v = hip.toHip(np.arange(48, dtype=np.float64).reshape(6, 8))[1:5:2, ::3]
    hip.write_npy(v, out)
    assert np.array_equal(np.load(out, allow_pickle=False), np.arange(48, dtype=np.float64).reshape(6, 8)[1:5:2, ::3])
    # round trip through the device
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 7, 3)).astype(np.float32)
    hip.write_npy(hip.toHip(x), out)
    assert np.array_equal(hip.read_npy(out, np.float32).toCpu(), x)
