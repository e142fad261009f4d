import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

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


def strided_view(rng, shape, dtype, kind):
    """A NumPy array of `shape` whose memory layout is `kind`; returns (view, parent)."""
    m, n = shape
    def fill(s):
        if np.dtype(dtype).kind == "f":
            return rng.uniform(-1, 1, size=s).astype(dtype)
        return rng.integers(-100, 101, size=s).astype(dtype)
    if kind == "C":
        p = fill((m, n)); return p, p
    if kind == "F":
        p = fill((n, m)); return p.T, p
    if kind == "rowstep2":
        p = fill((2 * m, n)); return p[::2], p
    if kind == "colstep2":
        p = fill((m, 2 * n)); return p[:, ::2], p
    if kind == "neg_rows":
        p = fill((m, n)); return p[::-1], p
    if kind == "neg_cols":
        p = fill((m, n)); return p[:, ::-1], p
    if kind == "inner_block":
        p = fill((m + 3, n + 5)); return p[2:2 + m, 1:1 + n], p
    if kind == "bcast_rows":
        p = fill((1, n)); return np.broadcast_to(p, (m, n)), p
    raise KeyError(kind)

VIEW_KINDS = ["C", "F", "rowstep2", "colstep2", "neg_rows", "neg_cols", "inner_block", "bcast_rows"]
