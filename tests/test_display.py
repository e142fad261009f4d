"""The tensor printer against the reference's own expected-output literals
(tests/tensor/test_display.nim, held in tests/golden/display_vectors.json). The printer formats a host
copy of the tensor, so the format itself is checked here without a device; the GPU test prints real
device tensors through the same code."""
import json
import os

import numpy as np
import pytest

from arraymancer_amd import display

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
with open(os.path.join(ROOT, "tests", "golden", "display_vectors.json")) as f:
    VEC = json.load(f)
DT = {"f64": np.float64, "i64": np.int64}


def build(inp):
    dt = DT[inp["dtype"]]
    if "values" in inp:
        a = np.array(inp["values"], dtype=dt)
    elif "arange" in inp:
        a = np.arange(*inp["arange"], dtype=dt)
    elif "linspace" in inp:
        a = np.linspace(*inp["linspace"]).astype(dt)
    else:
        n = inp["vandermonde"]
        a = np.array([[(i + 1) ** (j + 1) for j in range(n)] for i in range(n)], dtype=dt)
    return a.reshape(inp["shape"])


def compare_strings(got: str, want: str):
    """The reference's own comparison (test_display.nim:18-23): same number of lines, each equal after strip."""
    g, w = got.split("\n"), want.split("\n")
    assert len(g) == len(w), (got, want)
    for x, y in zip(g, w):
        assert x.strip() == y.strip(), (got, want)


@pytest.mark.parametrize("case", VEC["compare_strings"], ids=lambda c: c["source"][18:] + " " + c["call"]["specifier"])
def test_reference_display_literals(case):
    got = display.pretty_array(build(case["input"]), "Tensor", "Cpu", **case["call"])
    want = case["expect"]
    if want.startswith("\n"):          # literals that open with a line break: the reference's `$t` has none there
        want = want[1:]
    # a trailing line of the literal that only holds indentation is part of the literal, not of the output
    compare_strings(got.rstrip("\n"), want.rstrip(" \n"))


@pytest.mark.parametrize("case", VEC["exact"], ids=lambda c: c["source"][18:] + " " + c["call"]["specifier"])
def test_reference_format_string_literals(case):
    assert display.pretty_array(build(case["input"]), "Tensor", "Cpu", **case["call"]) == case["expect"]


def test_empty_bool_and_special_values():
    assert display.pretty_array(np.zeros((0, 3)), "HipTensor", "Hip") == \
        'HipTensor[system.float] of shape "[0, 3]" on backend "Hip"\n    [] (empty)'
    assert display.pretty_array(np.array([True, False]), "HipTensor", "Hip", specifier="<>") == "HipTensor[bool]<2>:[true, false]"
    assert display.pretty_array(np.array([np.nan, np.inf, -np.inf, -0.0], dtype=np.float32), "T", "Hip", specifier="[]") == "[nan, inf, -inf, -0]"
    with pytest.raises(ValueError):
        display.pretty_array(np.zeros(3), "T", "Hip", specifier="+<>06.2f")


# ---- the C++ host layer's printer (am::pretty_host), host-only program built under ASan + UBSan
import subprocess

CPP_DIR = os.path.join(ROOT, "tests", "cpp")
CPP_BIN = os.path.join(CPP_DIR, "test_display_host")


@pytest.fixture(scope="module")
def cpp_printer():
    res = subprocess.run(["make", "-C", CPP_DIR, "-B", "test_display_host"], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-3000:]
    return CPP_BIN


def _cpp_args(case):
    inp, call = case["input"], case["call"]
    if "values" in inp:
        gen = ["values"] + [repr(v) for v in inp["values"]]
    elif "arange" in inp:
        gen = ["arange"] + [str(v) for v in inp["arange"]]
    elif "linspace" in inp:
        gen = ["linspace"] + [str(v) for v in inp["linspace"]]
    else:
        gen = ["vandermonde", str(inp["vandermonde"])]
    return [inp["dtype"], *gen, "--", *[str(s) for s in inp["shape"]], "--", call["specifier"], str(call.get("precision", -1))]


def test_cpp_printer_matches_the_reference_literals(cpp_printer):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1", UBSAN_OPTIONS="halt_on_error=1")
    for case in VEC["compare_strings"] + VEC["exact"]:
        res = subprocess.run([cpp_printer, *_cpp_args(case)], capture_output=True, text=True, env=env)
        assert res.returncode == 0, (case["source"], res.stderr[-2000:])
        want = case["expect"]
        if case in VEC["exact"]:
            assert res.stdout == want, case["source"]
        else:
            compare_strings(res.stdout.rstrip("\n"), (want[1:] if want.startswith("\n") else want).rstrip(" \n"))
        # and the two host layers agree character for character
        assert res.stdout == display.pretty_array(build(case["input"]), "Tensor", "Cpu", **case["call"]), case["source"]
