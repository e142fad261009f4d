"""The compiled (C++) host layer include/am_hip_tensor.hpp: builds against the C ABI on any
machine; on the GPU box its test program replays the reference's GPU-backend literals."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP_DIR = os.path.join(ROOT, "tests", "cpp")
BIN = os.path.join(CPP_DIR, "test_tensor_hip")


BIN_ASAN = os.path.join(CPP_DIR, "test_tensor_hip_asan")


def test_cpp_host_layer_builds():
    res = subprocess.run(["make", "-C", CPP_DIR, "-B", "test_tensor_hip", "test_tensor_hip_asan"], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-3000:]
    assert os.path.exists(BIN) and os.path.exists(BIN_ASAN)


@pytest.mark.gpu
def test_cpp_host_layer_on_device(hip):
    if not os.path.exists(BIN):
        pytest.fail("tests/cpp/test_tensor_hip is not built (python -c 'import __graft_entry__ as g; g.build()')")
    res = subprocess.run([BIN, os.path.join(ROOT, "tests", "golden", "npy")], capture_output=True, text=True, timeout=120)
    print(res.stdout)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-1000:]
    assert " 0 failed" in res.stdout


@pytest.mark.gpu
def test_cpp_host_layer_on_device_under_sanitizers(hip):
    """The same program with its host side (tensor ownership, views, printing, the test code) under
    AddressSanitizer + UndefinedBehaviorSanitizer. Leak detection is off: the HIP runtime keeps its own
    allocations until the process ends."""
    if not os.path.exists(BIN_ASAN):
        pytest.fail("tests/cpp/test_tensor_hip_asan is not built (python -c 'import __graft_entry__ as g; g.build()')")
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:protect_shadow_gap=0", UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    res = subprocess.run([BIN_ASAN, os.path.join(ROOT, "tests", "golden", "npy")], capture_output=True, text=True, timeout=180, env=env)
    print(res.stdout)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-3000:]
    assert " 0 failed" in res.stdout and "AddressSanitizer" not in res.stderr and "runtime error" not in res.stderr


def test_division_by_launch_constants_is_exact():
    """csrc/fastdiv.h (multiply-and-shift division used by the im2col / col2im kernels' index arithmetic), compiled
    for the host and compared with the machine's division over 4000+ divisors and the dividends where a wrong
    multiplier or shift would show."""
    res = subprocess.run(["make", "-C", CPP_DIR, "-B", "test_fastdiv"], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-3000:]
    res = subprocess.run([os.path.join(CPP_DIR, "test_fastdiv")], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0 and " 0 wrong" in res.stdout, res.stdout[-2000:] + res.stderr[-2000:]
