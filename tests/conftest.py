import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

import zlib


def seed_of(*parts) -> int:
    """Deterministic 32-bit seed from a test's parameters (str hashes vary per process)."""
    return zlib.crc32(repr(parts).encode())


DTYPES = {"f32": np.float32, "f64": np.float64, "i32": np.int32, "i64": np.int64}


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def vectors():
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def oracle():
    import am_oracle
    am_oracle.lib()
    return am_oracle


@pytest.fixture(scope="session")
def hip():
    """The product package with its HIP library loaded and a device initialised."""
    import arraymancer_amd as am
    am.load_library()
    am.sync()   # raises HipError when no gfx950 device is usable
    return am


def np_apply_ops(arr: np.ndarray, ops):
    """Applies fixture view ops (transpose / inclusive slices in the reference's notation) to an ndarray."""
    for op in ops:
        if op[0] == "transpose":
            arr = arr.T
        elif op[0] == "slice":
            key = []
            for a, b, step in op[1]:
                stop = b + (1 if step > 0 else -1)
                key.append(slice(a, stop if stop >= 0 else None, step))
            arr = arr[tuple(key)]
        else:
            raise KeyError(op[0])
    return arr


def hip_apply_ops(t, ops):
    from arraymancer_amd import Step
    for op in ops:
        if op[0] == "transpose":
            t = t.transpose()
        elif op[0] == "slice":
            t = t.slice_(*[Step(a, b, s) for a, b, s in op[1]])
        else:
            raise KeyError(op[0])
    return t


PARENT_SHAPE = {
    "C": lambda m, n: (m, n), "F": lambda m, n: (n, m), "rowstep2": lambda m, n: (2 * m, n),
    "colstep2": lambda m, n: (m, 2 * n), "neg_rows": lambda m, n: (m, n), "neg_cols": lambda m, n: (m, n),
    "inner_block": lambda m, n: (m + 3, n + 5), "bcast_rows": lambda m, n: (1, n),
}


def view_of(parent: np.ndarray, kind: str, shape):
    """The [m, n] view of geometry `kind` over `parent` (which has PARENT_SHAPE[kind](m, n))."""
    m, n = shape
    return {
        "C": lambda p: p, "F": lambda p: p.T, "rowstep2": lambda p: p[::2], "colstep2": lambda p: p[:, ::2],
        "neg_rows": lambda p: p[::-1], "neg_cols": lambda p: p[:, ::-1],
        "inner_block": lambda p: p[2:2 + m, 1:1 + n], "bcast_rows": lambda p: np.broadcast_to(p, (m, n)),
    }[kind](parent)


def strided_view(rng, shape, dtype, kind):
    """A NumPy array of `shape` whose memory layout is `kind`; returns (view, parent)."""
    ps = PARENT_SHAPE[kind](*shape)
    if np.dtype(dtype).kind == "f":
        parent = rng.uniform(-1, 1, size=ps).astype(dtype)
    else:
        parent = rng.integers(-100, 101, size=ps).astype(dtype)
    return view_of(parent, kind, shape), parent


VIEW_KINDS = ["C", "F", "rowstep2", "colstep2", "neg_rows", "neg_cols", "inner_block", "bcast_rows"]
