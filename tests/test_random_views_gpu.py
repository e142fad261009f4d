"""Seeded random shapes and views through the element-wise, reduction, softmax, matrix-vector and matrix-matrix entry
points against NumPy. The kernels behind these calls are picked by shape, stride and alignment (row, short-row, tiled,
generic forms; walks, lane groups, chunked rows; skinny, tiled and split products), so the cases are drawn to land on
every side of those decisions: extents around the vector width and the tile edges, tall / skinny / wide / square,
windows that keep and that break 16-byte alignment, steps, reversals, transposes and broadcasts."""
import numpy as np
import pytest

from conftest import DTYPES, seed_of

pytestmark = pytest.mark.gpu
ALL = ["f32", "f64", "i32", "i64"]
EXTENTS = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 255, 256, 260, 500, 512, 1000, 1024, 1031, 2048, 4100]


def say(*a):
    print(*a, flush=True)


def fill(rng, shape, dt):
    if np.dtype(dt).kind == "f":
        return rng.uniform(-2, 2, shape).astype(dt)
    return rng.integers(-50, 50, shape).astype(dt)


def random_2d(rng, budget=600_000):
    """(rows, cols) with rows * cols within the budget: a mix of square-ish, tall and wide."""
    kind = rng.integers(0, 4)
    if kind == 0:
        r, c = rng.choice(EXTENTS), rng.choice(EXTENTS)
    elif kind == 1:
        c = int(rng.choice([4, 8, 12, 16, 24, 64, 128, 10, 3])); r = int(rng.integers(1000, 40_000))
    elif kind == 2:
        r = int(rng.choice([1, 2, 5, 16, 64])); c = int(rng.integers(5_000, 120_000))
    else:
        r, c = int(rng.integers(1, 700)), int(rng.integers(1, 700))
    r, c = int(r), int(c)
    while r * c > budget:
        if r > c: r //= 2
        else: c //= 2
    return max(r, 1), max(c, 1)


def random_view(rng, arr, darr):
    """The same random view of a host array and of its device twin."""
    kind = rng.integers(0, 7)
    r, c = arr.shape
    if kind == 0 or r < 4 or c < 12:
        return arr, darr, "whole"
    if kind == 1:
        lo = int(rng.choice([4, 8])); key = (slice(None), slice(lo, c - int(rng.choice([0, 4]))))
        return arr[key], darr[key], f"aligned columns from {lo}"
    if kind == 2:
        lo = int(rng.choice([1, 3, 5])); key = (slice(int(rng.integers(0, 3)), None), slice(lo, None))
        return arr[key], darr[key], f"columns from {lo}"
    if kind == 3:
        key = (slice(None, None, 2), slice(None))
        return arr[key], darr[key], "every other row"
    if kind == 4:
        key = (slice(None), slice(None, None, 2))
        return arr[key], darr[key], "every other column"
    if kind == 5:
        key = (slice(None, None, -1), slice(None, None, -1))
        return arr[key], darr[key], "reversed"
    return arr.T, darr.transpose(), "transposed"


@pytest.mark.parametrize("sfx", ALL)
def test_random_elementwise(hip, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("random-ew", sfx))
    for case in range(60):
        r, c = random_2d(rng)
        A, B, C = fill(rng, (r, c), dt), fill(rng, (r, c), dt), fill(rng, (r, c), dt)
        dA, dB, dC = hip.toHip(A), hip.toHip(B), hip.toHip(C)
        a, da, what = random_view(rng, A, dA)
        # operands of the view's shape: another view with the same key is not available for every kind, so fresh ones
        b = fill(rng, a.shape, dt); db = hip.toHip(b)
        bt = np.ascontiguousarray(b.T); dbt = hip.toHip(bt).transpose()          # same values, unit stride on the other axis
        row, col = fill(rng, (1, a.shape[1]), dt), fill(rng, (a.shape[0], 1), dt)
        say("random element-wise", sfx, case, (r, c), what, a.shape)
        with np.errstate(over="ignore"):
            assert np.array_equal(hip.map2("add", da, db).toCpu(), a + b), (case, what, "add")
            assert np.array_equal(hip.map2("sub", da, dbt).toCpu(), a - b), (case, what, "sub transposed")
            assert np.array_equal(hip.bc_mul(da, hip.toHip(row)).toCpu(), a * row), (case, what, "row vector")
            assert np.array_equal(hip.bc_add(hip.toHip(col), da).toCpu(), col + a), (case, what, "column vector")
            assert np.array_equal(hip.scalar_op("mul", da, 3).toCpu(), a * dt(3)), (case, what, "scalar")
            assert np.array_equal(hip.unary("neg", da).toCpu(), -a), (case, what, "neg")
            assert np.array_equal(hip.map3("muladd", da, db, dbt).toCpu(), a * b + b), (case, what, "muladd")
        assert np.array_equal(hip.bc_lt(da, db).toCpu(), a < b), (case, what, "<")
        assert np.array_equal(hip.bc_ge(da, hip.toHip(col)).toCpu(), a >= col), (case, what, ">= column")
        assert np.array_equal(da.clone().toCpu(), a), (case, what, "clone")
        # in place on the view: nothing outside it changes
        expect = A.copy()
        with np.errstate(over="ignore"):
            _same_view(expect, a, A)[...] += b
        da += db
        assert np.array_equal(dA.toCpu(), expect), (case, what, "in place")


def _same_view(host_copy, view, parent):
    """The view of host_copy that corresponds to `view` of `parent` (same offset and strides)."""
    off = (view.__array_interface__["data"][0] - parent.__array_interface__["data"][0]) // parent.itemsize
    return np.lib.stride_tricks.as_strided(host_copy.reshape(-1)[off:], shape=view.shape, strides=view.strides)


@pytest.mark.parametrize("sfx", ALL)
def test_random_reductions(hip, oracle, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("random-red", sfx))
    tol = {"f32": 1e-5, "f64": 1e-13}.get(sfx)
    for case in range(50):
        r, c = random_2d(rng)
        A = fill(rng, (r, c), dt)
        dA = hip.toHip(A)
        a, da, what = random_view(rng, A, dA)
        say("random reductions", sfx, case, (r, c), what, a.shape)
        for ax in (0, 1):
            got = hip.sum(da, ax).toCpu()
            if tol is None:
                with np.errstate(over="ignore"):
                    assert np.array_equal(got, a.sum(ax, keepdims=True, dtype=dt)), (case, what, ax, "sum")
            else:
                ref = a.astype(np.longdouble).sum(ax, keepdims=True)
                scale = np.abs(a).astype(np.longdouble).sum(ax, keepdims=True) + np.finfo(dt).tiny
                assert np.all(np.abs(got - ref) <= tol * scale * max(1, np.log2(a.shape[ax] + 1))), (case, what, ax, "sum")
            assert np.array_equal(hip.max(da, ax).toCpu(), a.max(ax, keepdims=True)), (case, what, ax, "max")
            assert np.array_equal(hip.min(da, ax).toCpu(), a.min(ax, keepdims=True)), (case, what, ax, "min")
            gi, gv = hip.argmax_max(da, ax)
            wi, wv = oracle.argreduce("max", np.ascontiguousarray(a), ax)
            assert np.array_equal(gi.toCpu(), wi) and np.array_equal(gv.toCpu(), wv), (case, what, ax, "argmax")
        if tol is not None:
            got = hip.softmax(da).toCpu()
            al = a.astype(np.longdouble)
            e = np.exp(al - al.max(1, keepdims=True))
            exact = e / e.sum(1, keepdims=True)
            assert np.max(np.abs(got - exact) / exact) <= (1e-5 if sfx == "f32" else 1e-13), (case, what, "softmax")


@pytest.mark.parametrize("sfx", ALL)
def test_random_products(hip, oracle, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("random-prod", sfx))
    bar = {"f32": 1e-4, "f64": 1e-12}.get(sfx)
    for case in range(40):
        m, k = random_2d(rng, 300_000)
        n = int(rng.choice([1, 3, 8, 16, 33, 64, 100, 256, 500]))
        while k * n > 300_000:
            n = max(1, n // 2)
        A, B, x = fill(rng, (m, k), dt), fill(rng, (k, n), dt), fill(rng, (k,), dt)
        dA, dB, dx = hip.toHip(A), hip.toHip(B), hip.toHip(x)
        layouts = [("C", A, dA), ("F", A, hip.toHip(np.ascontiguousarray(A.T)).transpose())]
        for name, a, da in layouts:
            say("random products", sfx, case, (m, k, n), name)
            got_v = (da * dx).toCpu()
            got_m = (da * dB).toCpu()
            if bar is None:
                with np.errstate(over="ignore"):
                    assert np.array_equal(got_v, (a.astype(np.int64) @ x.astype(np.int64)).astype(dt)), (case, name, "gemv")
                    assert np.array_equal(got_m, (a.astype(np.int64) @ B.astype(np.int64)).astype(dt)), (case, name, "gemm")
            else:
                ref_v = a.astype(np.longdouble) @ x.astype(np.longdouble)
                ref_m = a.astype(np.float64) @ B.astype(np.float64)
                assert np.linalg.norm((got_v - ref_v).astype(np.float64)) <= bar * max(np.linalg.norm(ref_v.astype(np.float64)), 1e-30), (case, name, "gemv")
                assert oracle.rel_frobenius(got_m, ref_m.astype(dt)) <= bar, (case, name, "gemm")
