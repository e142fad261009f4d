"""NumPy .npy files <-> device tensors (src/arraymancer/io/io_npy.nim:64-183).

read_npy(path, dtype) parses the file on the host (format versions 1.0 and 2.0; element types
<f4 >f4 <f8 >f8 <i4 >i4 <i8 >i8 <u4 >u4 <u8 >u8, converted element by element to `dtype` the way
the reference's `x.readXxx.T` does; C or Fortran order, kept as the tensor's strides) and uploads
the buffer. write_npy(t, path) writes what the reference writes: a contiguous copy of the tensor
(C order, or Fortran order when the tensor is column-major), a version 1.0 header (2.0 when it
does not fit 16 bits) padded with spaces so that the data starts on a 16-byte boundary.

The file format itself is parsed and produced here from its specification; NumPy is used only as
the host array container.
"""
from __future__ import annotations

import os
import re
import struct

import numpy as np

from . import metadata as md
from . import tensor_hip as th

_MAGIC = b"\x93NUMPY"
_DESCR = {"<f4", ">f4", "<f8", ">f8", "<i4", ">i4", "<i8", ">i8", "<u4", ">u4", "<u8", ">u8"}
_HEADER = re.compile(r"\{'descr': '(.+?)', 'fortran_order': (.+?), 'shape': (.+?), \}")


def parse_npy(path: str):
    """Host half of read_npy: (raw elements as a flat NumPy array in file order and file type,
    shape, fortran_order)."""
    if not os.path.exists(path):
        raise IOError(f'.npy file "{path}" does not exist')
    with open(path, "rb") as f:
        if f.read(6) != _MAGIC:
            raise AssertionError("This file is not a Numpy file")
        major, minor = f.read(1)[0], f.read(1)[0]
        if (major, minor) not in ((1, 0), (2, 0)):
            raise AssertionError(f"Unsupported .npy format. Only 1.0 or 2.0 files can be loaded but the file {path} "
                                 f"is at version ({major}, {minor}).")
        header_len = struct.unpack("<H", f.read(2))[0] if major == 1 else struct.unpack("<I", f.read(4))[0]
        header = f.read(header_len).decode("latin-1")
        m = _HEADER.match(header)
        if m is None:
            raise AssertionError(f"Error while parsing .npy header {header}")
        descr, fortran, shape_txt = m.groups()
        if descr not in _DESCR:
            raise ValueError(f"Numpy type not supported: {descr} in file.")
        if fortran not in ("False", "True"):
            raise ValueError(f"Invalid token '{fortran}' in numpy description {header}")
        if not shape_txt.startswith("("):
            raise AssertionError(f"Invalid numpy shape {shape_txt}")
        shape = []
        for tok in shape_txt[1:].split(")")[0].replace(" ", "").split(","):
            if tok == "":
                continue
            if not tok.isdigit():
                raise ValueError(f"Invalid token '{tok[0]}' in numpy shape {shape_txt}")
            shape.append(int(tok))
        count = 1
        for s in shape:
            count *= s
        raw = np.frombuffer(f.read(count * int(descr[2])), dtype=np.dtype(descr), count=count)
    return raw, tuple(shape), fortran == "True"


def read_npy(path: str, dtype) -> "th.HipTensor":
    """read_npy[T](path): a device tensor of element type `dtype`; a Fortran-ordered file gives a
    column-major tensor (same values at the same indices)."""
    dtype = np.dtype(dtype)
    raw, shape, fortran = parse_npy(path)
    # element-wise conversion, like `stream.readFloat32LE.T`: float -> int truncates, u64 -> i64 wraps
    with np.errstate(invalid="ignore", over="ignore"):
        host = raw.astype(dtype.newbyteorder("="), casting="unsafe")
    if not fortran:
        return th.toHip(host.reshape(shape))
    # the file holds the elements in column-major sequence: upload them as they are and describe
    # them with column-major strides (initTensorMetadata(..., colMajor), io_npy.nim:107-110)
    flat = th.toHip(host)
    return th.HipTensor(md.contiguous(shape, "F"), flat.storage, flat.dtype)


def npy_bytes(host: np.ndarray, fortran_order: bool) -> bytes:
    """The exact bytes write_npy emits for a contiguous host array (C order, or Fortran order when
    fortran_order: `host` then holds the elements in column-major sequence)."""
    dt = host.dtype
    kind = {"u": "u", "i": "i", "f": "f"}.get(dt.kind)
    if kind is None:
        raise TypeError(f"write_npy supports integer, unsigned and float tensors, not {dt}")
    endian = "<" if (dt.byteorder == "<" or (dt.byteorder in "=|" and np.little_endian)) else ">"
    descr = f"{endian}{kind}{dt.itemsize}"
    shape = host.shape
    if len(shape) == 0:
        raise AssertionError("write_npy: rank-0 tensors are not supported")
    shape_txt = "(" + ", ".join(str(s) for s in shape) + ("," if len(shape) == 1 else "") + ")"
    header = f"{{'descr': '{descr}', 'fortran_order': {'True' if fortran_order else 'False'}, 'shape': {shape_txt}, }}"
    meta_len = 6 + 4 + len(header) + 1
    v1 = meta_len <= 0xFFFF
    if not v1:
        meta_len += 2
    header += " " * ((16 - (meta_len & 15)) & 15) + "\n"
    out = bytearray(_MAGIC)
    out += bytes((1, 0)) + struct.pack("<H", len(header)) if v1 else bytes((2, 0)) + struct.pack("<I", len(header))
    out += header.encode("latin-1")
    out += (host.T if fortran_order else host).tobytes(order="C")
    return bytes(out)


def write_npy(t: "th.HipTensor", path: str) -> None:
    """t.write_npy(path): `t.asContiguous` written in C order, or in Fortran order when the tensor
    is column-major (io_npy.nim:136-141)."""
    if t.rank == 0:
        raise AssertionError("write_npy: rank-0 tensors are not supported")
    fortran = t.rank > 1 and t.is_F_contiguous() and not t.is_C_contiguous()
    host = t.toCpu()                 # logical values; strided views are gathered on the device first
    with open(path, "wb") as f:
        f.write(npy_bytes(np.ascontiguousarray(host), fortran))
