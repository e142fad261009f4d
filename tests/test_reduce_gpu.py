"""Reductions, row softmax and max pooling on the GPU through the C ABI: the reference's literal
vectors, oracle parity on strided views of every rank, chunked long axes, edge cases.

Bars: integers bit-exact (wrapping sums and products are order independent); float min / max
bit-exact; float sums along a non-unit-stride axis bit-exact (one lane folds the axis in the
reference's order); float sums that the device reassociates (unit-stride axis, whole tensor) within
1e-5 (f32) / 1e-13 (f64) of the serial fold relative to sum(|x|); softmax within 8e-6 / 4e-14
relative per element of the closed form; pooling identical values and indices."""
import numpy as np
import pytest

from conftest import DTYPES, seed_of

pytestmark = pytest.mark.gpu
ALL = ["f32", "f64", "i32", "i64"]
SUM_TOL = {"f32": 1e-5, "f64": 1e-13}
OPS = ["sum", "product", "min", "max"]


def say(*a):
    print(*a, flush=True)


def fill(rng, shape, dt, op="sum"):
    if np.dtype(dt).kind == "f":
        if op == "product":      # keep products finite and away from zero
            return rng.uniform(0.9, 1.1, size=shape).astype(dt) * rng.choice([-1, 1], size=shape).astype(dt)
        return rng.uniform(-1, 1, size=shape).astype(dt)
    info = np.iinfo(dt)
    return rng.integers(info.min, info.max, size=shape, endpoint=True).astype(dt)


def close(sfx, op, got, want, ref_abs):
    """got vs the serial fold `want`; ref_abs = fold of |x| (scale of the rounding error)."""
    if sfx in ("i32", "i64") or op in ("min", "max"):
        return np.array_equal(got, want)
    if op == "product":
        return np.allclose(got, want, rtol=1e-4 if sfx == "f32" else 1e-12)
    return np.all(np.abs(np.asarray(got, dtype=np.float64) - np.asarray(want, dtype=np.float64)) <= SUM_TOL[sfx] * np.asarray(ref_abs, dtype=np.float64))


@pytest.mark.parametrize("sfx", ALL)
def test_reference_aggregate_vectors(hip, vectors, sfx):
    g = vectors["aggregate"]
    dt = DTYPES[sfx]
    t = hip.toHip(np.array(g["t"], dtype=dt))
    assert hip.sum(t) == g["sum"]
    assert np.array_equal(hip.sum(t, axis=0).toCpu(), np.array(g["sum_axis0"], dtype=dt))
    assert np.array_equal(hip.sum(t, axis=1).toCpu(), np.array(g["sum_axis1"], dtype=dt))
    assert hip.product(t) == g["product_t"]
    a = hip.toHip(np.array(g["a"], dtype=dt))
    assert hip.product(a) == g["product_a"]
    assert np.array_equal(hip.product(a, 0).toCpu(), np.array(g["product_a_axis0"], dtype=dt))
    assert np.array_equal(hip.product(a, 1).toCpu(), np.array(g["product_a_axis1"], dtype=dt))
    v, b = hip.toHip(np.array(g["v"], dtype=dt)), hip.toHip(np.array(g["b"], dtype=dt))
    assert hip.min(v) == g["min_v"] and hip.max(v) == g["max_v"]
    for op in ("min", "max"):
        for ax in (0, 1):
            assert np.array_equal(getattr(hip, op)(b, ax).toCpu(), np.array(g[f"{op}_b_axis{ax}"], dtype=dt))
    if np.dtype(dt).kind == "f":
        assert hip.mean(t) == g["mean_float"]
        assert np.array_equal(hip.mean(t, 0).toCpu(), np.array(g["mean_axis0"], dtype=dt))
        assert np.array_equal(hip.mean(t, 1).toCpu(), np.array(g["mean_axis1"], dtype=dt))
    else:
        assert hip.mean(t) == 5                                    # 66 div 12
        assert hip.mean(hip.toHip(np.array([-7, 2, 1], dtype=dt))) == -1
        assert np.array_equal(hip.mean(hip.toHip(np.array([[-7, 5], [2, 2]], dtype=dt)), 0).toCpu(), np.array([[-2, 3]], dtype=dt))


def views(x):
    """(name, numpy view, function producing the same view of a HipTensor)."""
    out = [("C", x, lambda d: d)]
    if x.ndim >= 2:
        perm = tuple(range(x.ndim - 1, -1, -1))
        out.append(("reversed-axes", x.transpose(perm), lambda d: d.transpose() if d.rank == 2 else None))
    sl = tuple(slice(None, None, 2) if i % 2 == 0 else slice(1, None) for i in range(x.ndim))
    out.append(("stepped", x[sl], lambda d: d[sl]))
    neg = tuple(slice(None, None, -1) for _ in range(x.ndim))
    out.append(("negative", x[neg], lambda d: d[neg]))
    return out


SHAPES = [(1,), (63,), (64,), (1000,), (5, 7), (64, 64), (1, 300), (300, 1), (129, 257), (7, 5, 9), (3, 4, 5, 6), (2, 3, 2, 3, 2, 3)]


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("shape", SHAPES)
def test_reductions_vs_oracle(hip, oracle, sfx, shape):
    dt = DTYPES[sfx]
    for op in OPS:
        rng = np.random.default_rng(seed_of("reduce", sfx, shape, op))
        x = fill(rng, shape, dt, op)
        dx = hip.toHip(x)
        for name, v, mk in views(x):
            dv = mk(dx)
            if dv is None or v.size == 0:
                continue
            say("reduce", sfx, shape, op, name)
            assert dv.shape == v.shape
            absv = np.abs(v)
            assert close(sfx, op, getattr(hip, op)(dv), oracle.reduce_all(op, v), oracle.reduce_all("sum", absv) if op == "sum" else None), (op, name, "all")
            for ax in range(v.ndim):
                got = getattr(hip, op)(dv, ax).toCpu()
                want = oracle.reduce_axis(op, v, ax)
                assert got.shape == want.shape
                assert close(sfx, op, got, want, oracle.reduce_axis("sum", absv, ax) if op == "sum" else None), (op, name, ax)


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_sum_over_non_unit_stride_axis_is_the_serial_fold(hip, oracle, sfx):
    """Sum over the leading axis of a row-major tensor with enough outputs to fill the chip on their
    own (no chunking of the axis): one lane per output walks the axis in order, so the result equals
    the CPU's serial fold bit for bit. (With few outputs the axis is cut up and the sum is
    reassociated: covered with a tolerance by the other tests.)"""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("rowsum", sfx))
    for shape in [(64, 1_100_000), (20, 1100, 1000), (63, 1_048_576), (5, 3, 1_200_000)]:
        x = rng.uniform(-1, 1, shape).astype(dt)
        say("serial-order sum", sfx, shape)
        assert np.array_equal(hip.sum(hip.toHip(x), 0).toCpu(), oracle.reduce_axis("sum", x, 0))


@pytest.mark.parametrize("sfx", ALL)
def test_long_axes_are_chunked(hip, oracle, sfx):
    """Few outputs, long axis: the axis is cut into chunks folded by a second pass."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("chunked", sfx))
    for shape, ax in [((3, 1 << 20), 1), ((1 << 20, 3), 0), ((1, 3_000_001), 1), ((200_000, 17), 0), ((2, 70_000, 2), 1)]:
        x = fill(rng, shape, dt)
        dx = hip.toHip(x)
        for op in ("sum", "max"):
            say("chunked", sfx, shape, ax, op)
            got = getattr(hip, op)(dx, ax).toCpu()
            want = oracle.reduce_axis(op, x, ax)
            assert close(sfx, op, got, want, oracle.reduce_axis("sum", np.abs(x), ax))
            assert close(sfx, op, getattr(hip, op)(dx), oracle.reduce_all(op, x), oracle.reduce_all("sum", np.abs(x)))


@pytest.mark.parametrize("sfx", ALL)
def test_tall_skinny_reductions(hip, oracle, sfx):
    """Matrices with many rows and few columns, both ways: down the rows (the bias gradient of a dense layer: the
    workgroup-wide walk with a second pass over chunk partials, also on column windows of wider buffers) and along
    short rows (several rows per wavefront, row lengths that fill their lane group and that do not), on 2-D and 3-D
    tensors. Integers, min and max exactly; float sums and products against the serial fold with the usual bound."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("tall-skinny", sfx))
    cases = [((70_000, 64), 0, None), ((5_000, 512), 0, None), ((3_000, 128), 0, (slice(None), slice(16, 80))), ((600, 8), 0, None),
             ((70_000, 64), 1, None), ((300_000, 16), 1, None), ((100_000, 24), 1, None), ((5_000, 8, 32), 2, None),
             ((9_000, 128), 1, (slice(None), slice(8, 72))), ((4_100, 4), 1, None), ((5_000, 512), 1, None), ((4_200, 1000), 1, None),
             ((4_100, 264), 1, None), ((4_500, 520), 1, None)]
    for shape, ax, window in cases:
        for op in OPS:
            if op == "product" and sfx in ("f32", "f64") and shape[ax] > 3000:
                continue   # thousands of factors near 1 leave the normal range: nothing to compare
            x = fill(rng, shape, dt, op)
            dx = hip.toHip(x)
            v, dv = (x[window], dx[window]) if window else (x, dx)
            say("tall-skinny", sfx, shape, ax, op, "window" if window else "whole")
            got = getattr(hip, op)(dv, ax).toCpu()
            want = oracle.reduce_axis(op, v, ax)
            assert got.shape == want.shape
            if sfx in ("i32", "i64") or op in ("min", "max"):
                assert np.array_equal(got, want), (shape, ax, op)
            else:
                assert close(sfx, op, got, want, oracle.reduce_axis("sum", np.abs(v), ax) if op == "sum" else None), (shape, ax, op)
    if sfx in ("f32", "f64"):   # mean and variance ride the same kernels
        x = rng.uniform(-1, 1, (50_000, 32)).astype(dt)
        dx = hip.toHip(x)
        rtol = 2e-5 if sfx == "f32" else 1e-12
        for ax in (0, 1):
            assert np.allclose(hip.mean(dx, ax).toCpu(), x.astype(np.float64).mean(ax, keepdims=True), rtol=rtol, atol=rtol)
            assert np.allclose(hip.variance(dx, ax).toCpu(), oracle.variance(x, ax), rtol=rtol * 10)


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_variance_and_std(hip, oracle, vectors, sfx):
    """variance / std (aggregate.nim:115-158): the reference's own literals, then the oracle on
    larger tensors and views, along every axis and over all elements."""
    dt = DTYPES[sfx]
    g = vectors["aggregate_float"]
    tol = 1e-8 if sfx == "f64" else 2e-6
    a, b = hip.toHip(np.array(g["a"], dtype=dt)), hip.toHip(np.array(g["b"], dtype=dt))
    assert abs(hip.variance(a) - g["variance_a"]) < tol * 5 and abs(hip.std(a) - g["std_a"]) < tol * 5
    assert np.array_equal(hip.variance(b, 0).toCpu(), np.array(g["variance_b_axis0"], dtype=dt))
    for ax in (0, 1):
        assert np.abs(hip.variance(b, ax).toCpu() - np.array(g[f"variance_b_axis{ax}"])).sum() < tol * 50
        assert np.abs(hip.std(b, ax).toCpu() - np.array(g[f"std_b_axis{ax}"])).sum() < tol * 10
    rng = np.random.default_rng(seed_of("variance", sfx))
    rtol = 2e-5 if sfx == "f32" else 1e-12
    for shape in [(300, 70), (5, 2048), (4100, 3), (6, 50, 7)]:
        x = (rng.standard_normal(shape) * 3 + 1).astype(dt)
        dx = hip.toHip(x)
        say("variance", sfx, shape)
        assert np.isclose(hip.variance(dx), oracle.variance(x), rtol=rtol)
        assert np.isclose(hip.std(dx), oracle.std(x), rtol=rtol)
        for ax in range(len(shape)):
            got = hip.variance(dx, ax).toCpu()
            assert got.shape == oracle.variance(x, ax).shape
            assert np.allclose(got, oracle.variance(x, ax), rtol=rtol)
            assert np.allclose(hip.std(dx, ax).toCpu(), oracle.std(x, ax), rtol=rtol)
        if len(shape) == 2:
            assert np.allclose(hip.variance(dx.transpose(), 0).toCpu(), oracle.variance(x.T, 0), rtol=rtol)
    with pytest.raises(TypeError):
        hip.variance(hip.zeros((3, 3), np.int32))


@pytest.mark.parametrize("sfx", ALL)
def test_argmax_argmin(hip, oracle, vectors, sfx):
    """argmax_max / argmin_min (aggregate.nim:159-271): the reference's literals, then the oracle on
    tie-heavy and random data, along every axis, over views, through both kernels (one lane per
    output; one wavefront per output for long axes), bit-exact in positions and values."""
    dt = DTYPES[sfx]
    for case in vectors["argmax_argmin"]["cases"]:
        a = hip.toHip(np.array(case["a"], dtype=dt))
        for name in ("argmax", "argmin"):
            for ax, want in case[name].items():
                got = getattr(hip, name)(a, int(ax))
                assert got.dtype == np.int64 and np.array_equal(got.toCpu(), np.array(want)), (name, ax)
    rng = np.random.default_rng(seed_of("argmax", sfx))
    for shape in [(7, 33, 5), (300, 70), (5, 5000), (5000, 5), (64, 10), (3, 2, 4, 3, 2, 3), (1, 1), (2100, 1100)]:
        for ties in (True, False):
            x = rng.integers(-4, 5, shape).astype(dt) if ties else fill(rng, shape, dt)
            dx = hip.toHip(x)
            for name, v, mk in views(x):
                dv = mk(dx)
                if dv is None or v.size == 0:
                    continue
                for ax in range(v.ndim):
                    for op, fn in (("max", hip.argmax_max), ("min", hip.argmin_min)):
                        say("argreduce", sfx, shape, ties, name, ax, op)
                        gi, gv = fn(dv, ax)
                        wi, wv = oracle.argreduce(op, v, ax)
                        assert gi.shape == wi.shape and np.array_equal(gi.toCpu(), wi), (shape, name, ax, op)
                        assert np.array_equal(gv.toCpu(), wv), (shape, name, ax, op)
    with pytest.raises(IndexError):
        hip.argmax(hip.zeros((2, 2), dt), 2)
    assert hip.argmax(hip.empty((0, 3), dt), 0).shape == (0, 3)


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_argmax_nan_rules(hip, oracle, sfx):
    """A NaN in slice 0 stays, a NaN elsewhere is never taken — also when the axis is long enough for
    the wavefront kernel, whose lanes each see only every 64th element."""
    dt = DTYPES[sfx]
    nan = np.nan
    x = np.array([[nan, 1, 2], [1, nan, 3], [1, nan, 0], [nan, nan, nan], [2, 2, nan]], dtype=dt)
    for op, fn in (("max", hip.argmax_max), ("min", hip.argmin_min)):
        gi, gv = fn(hip.toHip(x), 1)
        wi, wv = oracle.argreduce(op, x, 1)
        assert np.array_equal(gi.toCpu(), wi) and np.array_equal(gv.toCpu(), wv, equal_nan=True)
    rng = np.random.default_rng(seed_of("argmax-nan", sfx))
    z = rng.standard_normal((2000, 1100)).astype(dt)     # many outputs, long axis: the walk is cut into chunks
    z[0, 0] = nan; z[1:, 1] = nan; z[::7, 2] = nan; z[:, 3] = nan; z[0, 4] = 99; z[63:70, 5] = nan; z[1000:, 6] = nan; z[:1000, 7] = nan
    z[0, 7] = -99
    for op, fn in (("max", hip.argmax_max), ("min", hip.argmin_min)):
        gi, gv = fn(hip.toHip(z), 0)
        wi, wv = oracle.argreduce(op, z, 0)
        assert np.array_equal(gi.toCpu(), wi) and np.array_equal(gv.toCpu(), wv, equal_nan=True), op
    y = rng.standard_normal((6, 1000)).astype(dt)
    y[0, 0] = nan; y[1, 500] = nan; y[2, ::3] = nan; y[3, 1:] = nan; y[4, :] = nan; y[5, 64] = nan; y[5, 0] = y[5].max()
    for v, dv in ((y, hip.toHip(y)), (y.T, hip.toHip(np.ascontiguousarray(y.T)))):
        ax = 1 if v is y else 0
        for op, fn in (("max", hip.argmax_max), ("min", hip.argmin_min)):
            gi, gv = fn(dv, ax)
            wi, wv = oracle.argreduce(op, v, ax)
            assert np.array_equal(gi.toCpu(), wi), (op, ax)
            assert np.array_equal(gv.toCpu(), wv, equal_nan=True), (op, ax)


@pytest.mark.parametrize("sfx", ALL)
def test_argmax_tall_skinny_and_long_rows(hip, oracle, sfx):
    """Positions and values of the first maximum / minimum on shapes away from square: many short rows (lane groups per
    row), a walk down many rows of few columns (workgroup-wide, chunks merged in axis order), few long rows (chunks of a
    row over several wavefronts); tie-heavy data, so that 'first' matters across lanes, row classes and chunks, and
    NaN in row 0, elsewhere, and everywhere for floats. Bit-exact against the serial walk."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("argmax-shapes", sfx))
    for shape, ax in [((70_000, 64), 1), ((9_000, 16), 1), ((5_000, 24), 1), ((4_100, 128), 1), ((70_000, 64), 0), ((3_000, 512), 0),
                      ((600, 8), 0), ((5, 300_000), 1), ((64, 20_000), 1), ((300_000, 5), 0)]:
        for ties in (True, False):
            x = rng.integers(-3, 4, shape).astype(dt) if ties else fill(rng, shape, dt)
            if sfx in ("f32", "f64"):
                other = 1 - ax
                idx = [slice(None), slice(None)]
                n_other = shape[other]
                def at(o, l):
                    k = [0, 0]; k[other] = o; k[ax] = l; return tuple(k)
                x[at(0, 0)] = np.nan                       # NaN in position 0: stays
                if n_other > 1: x[at(1, shape[ax] // 2)] = np.nan   # NaN elsewhere: never taken
                if n_other > 2:
                    k = [slice(None), slice(None)]; k[other] = 2; x[tuple(k)] = np.nan      # nothing but NaN
                if n_other > 3:
                    k = [slice(None), slice(None)]; k[other] = 3; k[ax] = slice(1, None); x[tuple(k)] = np.nan   # only position 0 is a number
            dx = hip.toHip(x)
            for op, fn in (("max", hip.argmax_max), ("min", hip.argmin_min)):
                say("argreduce shapes", sfx, shape, ax, ties, op)
                gi, gv = fn(dx, ax)
                wi, wv = oracle.argreduce(op, x, ax)
                assert gi.shape == wi.shape and np.array_equal(gi.toCpu(), wi), (shape, ax, ties, op)
                assert np.array_equal(gv.toCpu(), wv, equal_nan=True), (shape, ax, ties, op)


@pytest.mark.parametrize("sfx", ALL)
def test_column_walks_with_16_byte_lanes(hip, oracle, sfx):
    """Walks across a unit-stride dimension take 16 bytes of adjacent outputs per lane when extents,
    strides and base addresses allow it, and one output per lane otherwise; both fold every output
    front to back, so without chunking floats equal the serial fold bit for bit."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("colvec", sfx))
    cases = [((4096, 2048), 0, True), ((70, 4100), 0, False), ((70, 4098), 0, False), ((120, 6, 512), 0, False),
             ((300, 600, 8), 1, True), ((9, 2048, 4), 0, False)]
    for shape, ax, chunked in cases:
        lead = (slice(None),) * (len(shape) - 1)
        for op in OPS:
            x = fill(rng, shape, dt, op)
            dx = hip.toHip(x)
            for name, sl in (("whole", ()), ("every other slice", (slice(None, None, 2),)), ("columns from 4", lead + (slice(4, None),)),
                             ("columns from 1", lead + (slice(1, None),)), ("columns reversed", lead + (slice(None, None, -1),))):
                v, dv = x[sl], dx[sl] if sl else dx
                say("column walk", sfx, shape, ax, name, op)
                got = getattr(hip, op)(dv, ax).toCpu()
                want = oracle.reduce_axis(op, v, ax)
                if sfx in ("i32", "i64") or op in ("min", "max") or not chunked:
                    assert np.array_equal(got, want), (shape, ax, name, op)
                else:
                    assert close(sfx, op, got, want, oracle.reduce_axis("sum", np.abs(v), ax)), (shape, ax, name, op)


@pytest.mark.parametrize("sfx", ["f32", "i32"])
def test_full_size_sum_8192(hip, oracle, sfx):
    """8192 x 8192: column sums, row sums and the total, against the oracle; and the total as the
    sum of the column sums computed on the device (two different kernels agree)."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("sum8192", sfx))
    x = fill(rng, (8192, 8192), dt) if sfx == "i32" else rng.uniform(0, 1, (8192, 8192)).astype(dt)
    dx = hip.toHip(x)
    say("8192 col sums", sfx)
    cols = hip.sum(dx, 0)
    assert close(sfx, "sum", cols.toCpu(), oracle.reduce_axis("sum", x, 0), oracle.reduce_axis("sum", np.abs(x), 0))
    say("8192 row sums", sfx)
    rows = hip.sum(dx, 1)
    assert close(sfx, "sum", rows.toCpu(), oracle.reduce_axis("sum", x, 1), oracle.reduce_axis("sum", np.abs(x), 1))
    say("8192 total", sfx)
    total = hip.sum(dx)
    if sfx == "i32":
        assert total == hip.sum(cols) == hip.sum(rows) == oracle.reduce_all("sum", x)
    else:
        exact = float(np.sum(x, dtype=np.float64))
        for t in (total, hip.sum(cols), hip.sum(rows)):
            assert abs(float(t) - exact) <= 1e-5 * exact


def test_edge_cases(hip):
    e = hip.empty((0, 3), np.float32)
    assert hip.sum(e, 0).shape == (0, 3)                       # returnEmptyIfEmpty
    with pytest.raises(ValueError):
        hip.sum(e)                                             # nothing to start the fold from
    with pytest.raises(IndexError):
        hip.sum(hip.zeros((2, 2), np.float32), 2)
    z = hip.toHip(np.array([-0.0, -0.0, -0.0] * 50, dtype=np.float32))
    assert np.signbit(hip.sum(z)) and np.signbit(hip.sum(z.reshape(3, 50), 1).toCpu()).all()   # no +0 identity mixed in
    one = hip.toHip(np.array([[4.5]], dtype=np.float64))
    assert hip.sum(one) == 4.5 and hip.max(one, 0).toCpu()[0, 0] == 4.5
    inf = hip.toHip(np.array([1.0, np.inf, -3.0], dtype=np.float32))
    assert hip.max(inf) == np.inf and hip.min(inf) == -3.0


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_softmax_vs_oracle(hip, oracle, sfx):
    dt = DTYPES[sfx]
    tol = 2e-6 if sfx == "f32" else 1e-14
    rng = np.random.default_rng(seed_of("softmax-gpu", sfx))
    # (rows, cols): a wavefront, a workgroup or sixteen wavefronts per row by length; from 1024 rows on, several short
    # rows per wavefront (whole vectors per row) or a lane per row (any length up to 64)
    for shape in [(1, 1), (3, 5), (64, 10), (256, 1000), (7, 4096), (5, 4097), (3, 8192), (4, 12288), (3, 16384), (3, 50_000),
                  (1000, 3), (3, 65536), (2, 40_000), (2, 70_000), (5000, 64), (3000, 16), (2000, 24), (1030, 4), (1500, 128),
                  (20_000, 10), (1100, 63), (3, 300_000), (70, 131_072)]:
        x = (rng.standard_normal(shape) * 4).astype(dt)
        say("softmax", sfx, shape)
        want = oracle.softmax(x)
        got = hip.softmax(hip.toHip(x)).toCpu()
        # closed form in extended precision: the tight bar
        xl = x.astype(np.longdouble)
        e = np.exp(xl - xl.max(1, keepdims=True))
        exact = e / e.sum(1, keepdims=True)
        assert np.max(np.abs(got - exact) / exact) <= tol * 4, shape
        # the oracle sums the row serially in the tensor's precision: its own rounding error grows
        # with the row length, so the bar against it does too
        assert np.max(np.abs(got - want) / want) <= max(tol * 8, shape[1] * np.finfo(dt).eps), shape
        assert np.allclose(got.sum(1), 1, atol=1e-5 if sfx == "f32" else 1e-13)
        # transposed view in (strided path of the kernel), same values out up to the order of the row sum
        xt = hip.toHip(np.ascontiguousarray(x.T)).transpose()
        assert np.max(np.abs(hip.softmax(xt).toCpu() - exact) / exact) <= tol * 4, shape
    big = np.array([[1000, 1001, 999], [-1000, -1001, -999]], dtype=dt)
    assert np.allclose(hip.softmax(hip.toHip(big)).toCpu(), oracle.softmax(big), rtol=tol * 8)
    with pytest.raises(TypeError):
        hip.softmax(hip.zeros((2, 2), np.int32))


@pytest.mark.parametrize("sfx", ALL)
def test_maxpool_vs_oracle(hip, oracle, vectors, sfx):
    dt = DTYPES[sfx]
    g = vectors["maxpool"]
    x = np.array(g["input"], dtype=dt).reshape(g["input_shape"])
    x0 = x
    idx, pooled = hip.maxpool2d(hip.toHip(x), g["kernel"], g["padding"], g["stride"])
    assert np.array_equal(pooled.toCpu(), np.array(g["pooled"], dtype=dt).reshape(g["pooled_shape"]))
    assert np.array_equal(idx.toCpu(), np.array(g["max_indices"], dtype=np.int64))
    rng = np.random.default_rng(seed_of("maxpool-gpu", sfx))
    cases = [((2, 3, 7, 9), (2, 2), (0, 0), (2, 2)), ((4, 20, 24, 24), (2, 2), (0, 0), (2, 2)), ((3, 5, 13, 11), (3, 3), (1, 1), (1, 1)),
             ((2, 2, 9, 8), (3, 2), (1, 0), (2, 3)), ((1, 1, 5, 5), (2, 2), (2, 2), (1, 1)), ((64, 50, 8, 8), (2, 2), (0, 0), (2, 2)),
             # the small-window kernels: 3 x 3 with stride 2 and padding (four windows per element), stride 3 (one), padding
             # as wide as the reach; 2 x 2 with stride 1 (four), 3 (gaps between the windows) and odd widths (14 x 14 maps)
             ((3, 4, 16, 16), (3, 3), (1, 1), (2, 2)), ((2, 3, 15, 17), (3, 3), (1, 1), (2, 2)), ((2, 2, 10, 11), (3, 3), (0, 0), (3, 3)),
             ((1, 2, 6, 7), (3, 3), (2, 2), (1, 1)), ((2, 3, 9, 9), (2, 2), (0, 0), (1, 1)), ((2, 3, 11, 10), (2, 2), (1, 1), (3, 3)),
             ((8, 16, 14, 14), (2, 2), (0, 0), (2, 2)), ((2, 2, 7, 9), (3, 3), (1, 1), (2, 1)), ((1, 1, 4, 4), (4, 4), (0, 0), (4, 4))]
    for shape, kernel, pad, stride in cases:
        x = rng.integers(-5, 5, shape).astype(dt)        # ties are frequent: the first maximum must win
        say("maxpool", sfx, shape, kernel, pad, stride)
        want_idx, want = oracle.maxpool2d(x, kernel, pad, stride)
        idx, got = hip.maxpool2d(hip.toHip(x), kernel, pad, stride)
        assert np.array_equal(got.toCpu(), want) and np.array_equal(idx.toCpu(), want_idx)
        # backward: the serial scatter of the reference, overlapping windows included (last output wins)
        go = rng.integers(-99, 100, want.shape).astype(dt)
        want_grad = oracle.maxpool2d_backward(shape, want_idx, go)
        grad = hip.maxpool2d_backward(shape, idx, hip.toHip(go))
        assert grad.shape == tuple(shape) and np.array_equal(grad.toCpu(), want_grad), ("backward", shape, kernel, pad, stride)
        bare = hip.toHip(want_idx)                                          # indices that did not come from maxpool2d
        assert np.array_equal(hip.maxpool2d_backward(shape, bare, hip.toHip(go), kernel, pad, stride).toCpu(), want_grad)
        with pytest.raises(ValueError):
            hip.maxpool2d_backward(shape, bare, hip.toHip(go))
    gb = hip.maxpool2d_backward(g["input_shape"], *hip.maxpool2d(hip.toHip(x0), g["kernel"], g["padding"], g["stride"]))
    assert np.array_equal(gb.toCpu().reshape(4, 4), np.array(g["backward"]["grad_input"], dtype=dt))
    with pytest.raises(ValueError):
        hip.maxpool2d(hip.zeros((4, 4), dt), (2, 2))                       # rank
    with pytest.raises(ValueError):
        hip.maxpool2d(hip.zeros((2, 3, 4, 4), dt).transpose(), (2, 2))     # not C-contiguous (the reference asserts)


def test_reduce_all_of_a_view_with_millions_of_runs(hip, oracle):
    """Whole-tensor folds of a strided view whose per-run partials (one per row here: 4.5 M rows x 8 bytes = 36 MB)
    exceed what the library keeps in its workspace: the partials then come from the block cache."""
    rows = 4_500_000
    rng = np.random.default_rng(seed_of("reduce-many-runs"))
    parent = rng.integers(-3, 3, (rows, 4), endpoint=True).astype(np.int64)
    d = hip.toHip(parent)
    view, host = d[:, 1:3], parent[:, 1:3]                     # [4.5 M, 2] with row stride 4: 4.5 M runs of 2
    say("reduce_all, strided view with 4.5 M runs")
    assert hip.sum(view) == host.sum()
    assert hip.max(view) == host.max() and hip.min(view) == host.min()
    f = hip.toHip(parent.astype(np.float64))[::1, 0:3:2]       # columns 0 and 2: inner stride 2
    want = parent[:, 0:3:2].astype(np.float64)
    assert abs(hip.sum(f) - want.sum()) <= 1e-9 * np.abs(want).sum()
    assert hip.mean(f) == pytest.approx(want.mean(), rel=1e-12)
