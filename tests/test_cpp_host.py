"""The compiled (C++) host layer include/am_hip_tensor.hpp: builds against the C ABI on any
machine; on the GPU box its test program replays the reference's GPU-backend literals."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP_DIR = os.path.join(ROOT, "tests", "cpp")
BIN = os.path.join(CPP_DIR, "test_tensor_hip")


def test_cpp_host_layer_builds():
    res = subprocess.run(["make", "-C", CPP_DIR, "-B", "test_tensor_hip"], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-3000:]
    assert os.path.exists(BIN)


@pytest.mark.gpu
def test_cpp_host_layer_on_device(hip):
    if not os.path.exists(BIN):
        pytest.fail("tests/cpp/test_tensor_hip is not built (python -c 'import __graft_entry__ as g; g.build()')")
    res = subprocess.run([BIN, os.path.join(ROOT, "tests", "golden", "npy")], capture_output=True, text=True, timeout=120)
    print(res.stdout)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-1000:]
    assert " 0 failed" in res.stdout
