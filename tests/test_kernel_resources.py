"""Register spills and scratch memory of the built kernels, read from the code objects that the in-tree build left
in arraymancer_amd/csrc/_obj (no GPU needed, nothing is compiled here).

A kernel that spills in its main loop loses far more than the spill count suggests (the headline GEMM kernel once
went from 0 to 280 spilled registers through a change elsewhere in its source and ran 5 % slower, with no test
failing), and a streaming kernel that indexes its argument arrays with a run-time index gets them moved to scratch
memory, whose loads then queue behind the stream's own. These are properties of the compiled code, so they are
checked on the compiled code."""
import glob
import os
import re
import shutil
import struct
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
OBJ = os.path.join(ROOT, "arraymancer_amd", "csrc", "_obj")
READELF = shutil.which("llvm-readelf") or "/opt/rocm/llvm/bin/llvm-readelf"

pytestmark = pytest.mark.skipif(not (os.path.isdir(OBJ) and glob.glob(os.path.join(OBJ, "*.o")) and os.path.exists(READELF)),
                                reason="no in-tree object files (run __graft_entry__.build()) or no llvm-readelf")


def _device_code_object(path):
    """The gfx950 member of the clang offload bundle inside a host object's .hip_fatbin section."""
    data = open(path, "rb").read()
    i = data.find(b"__CLANG_OFFLOAD_BUNDLE__")
    if i < 0:
        return None
    n = struct.unpack_from("<Q", data, i + 24)[0]
    off = i + 32
    for _ in range(n):
        o, size, triple_len = struct.unpack_from("<QQQ", data, off)
        off += 24
        triple = data[off:off + triple_len].decode()
        off += triple_len
        if "gfx950" in triple:
            return data[i + o:i + o + size]
    return None


def _kernels(path, tmp):
    """[(mangled name, vgprs, spilled vgprs, scratch bytes per lane)] of one object file."""
    co = _device_code_object(path)
    if not co:
        return []
    dev = os.path.join(tmp, os.path.basename(path) + ".co")
    with open(dev, "wb") as f:
        f.write(co)
    text = subprocess.run([READELF, "--notes", dev], capture_output=True, text=True, check=True).stdout
    out = []
    for block in re.split(r"\n\s+- \.agpr_count", text)[1:]:
        field = lambda k: re.search(r"\." + k + r":\s+(\S+)", block).group(1)
        out.append((field("name"), int(field("vgpr_count")), int(field("vgpr_spill_count")), int(field("private_segment_fixed_size"))))
    return out


@pytest.fixture(scope="module")
def built(tmp_path_factory):
    tmp = str(tmp_path_factory.mktemp("code_objects"))
    return {os.path.basename(p)[:-2]: _kernels(p, tmp) for p in sorted(glob.glob(os.path.join(OBJ, "*.o")))}


def test_every_translation_unit_was_read(built):
    for unit in ("gemm_f32", "gemm_f64", "gemm_i32", "gemm_i64", "elementwise_f32", "reduce", "gemv", "im2col", "diag"):
        assert built.get(unit), f"{unit}: no gfx950 kernels found in its object file"


@pytest.mark.parametrize("unit", ["elementwise_f32", "elementwise_f64", "elementwise_i32", "elementwise_i64", "reduce", "gemv",
                                  "im2col", "diag"])
def test_streaming_kernels_use_no_scratch(built, unit):
    bad = [(n, s, p) for n, _, s, p in built[unit] if s or p]
    assert not bad, f"{unit}: kernels with spilled registers or scratch memory: {bad[:5]}"


def test_headline_gemm_kernels_do_not_spill(built):
    # f32 256 x 256 tile (the 4096^3 kernel) with both operands moved in 16-byte vectors: loader kinds 0 / 1
    head = [k for k in built["gemm_f32"] if "gemm_mfmaIfNS0_4MfmaIfEELi256ELi256E" in k[0] and re.search(r"Li[01]ELi[01]EEEv", k[0])]
    assert len(head) == 4, [k[0] for k in head]
    assert all(k[2] == 0 and k[3] == 0 for k in head), head
    # the mid-size and small float32 tiles with vector loaders
    for tile in ("Li64ELi64ELi16E", "Li128ELi128ELi16E", "Li32ELi32ELi32E"):
        ks = [k for k in built["gemm_f32"] if "gemm_mfmaIf" in k[0] and tile in k[0] and re.search(r"Li[01]ELi[01]EEEv", k[0])]
        assert ks and all(k[2] == 0 for k in ks), (tile, ks)
    # the digit-sliced integer kernels
    digits = [k for k in built["gemm_i32"] + built["gemm_i64"] if "gemm_i8_digits" in k[0]]
    assert digits and all(k[2] == 0 and k[3] == 0 for k in digits), digits
    # the fused convolution's kernels (gathered B operand, loader kind 3)
    conv = [k for k in built["gemm_f32"] if re.search(r"Li0ELi3EEEv", k[0])]
    assert conv and all(k[2] == 0 for k in conv), conv
