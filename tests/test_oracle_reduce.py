"""Pins the CPU restatement of reductions, softmax and max pooling (oracle/reduce_pool.c):
the reference's literal vectors, then NumPy / exact arithmetic on random strided inputs."""
from fractions import Fraction

import numpy as np
import pytest

from conftest import DTYPES, seed_of, view_of, VIEW_KINDS, PARENT_SHAPE

NP_OPS = {"sum": np.add, "product": np.multiply, "min": np.minimum, "max": np.maximum}


@pytest.mark.parametrize("sfx", list(DTYPES))
def test_reference_aggregate_vectors(vectors, oracle, sfx):
    g = vectors["aggregate"]
    dt = DTYPES[sfx]
    t = np.array(g["t"], dtype=dt)
    assert oracle.reduce_all("sum", t) == g["sum"]
    assert np.array_equal(oracle.reduce_axis("sum", t, 0), np.array(g["sum_axis0"], dtype=dt))
    assert np.array_equal(oracle.reduce_axis("sum", t, 1), np.array(g["sum_axis1"], dtype=dt))
    assert oracle.reduce_all("product", t) == g["product_t"]
    a = np.array(g["a"], dtype=dt)
    assert oracle.reduce_all("product", a) == g["product_a"]
    assert np.array_equal(oracle.reduce_axis("product", a, 0), np.array(g["product_a_axis0"], dtype=dt))
    assert np.array_equal(oracle.reduce_axis("product", a, 1), np.array(g["product_a_axis1"], dtype=dt))
    v, b = np.array(g["v"], dtype=dt), np.array(g["b"], dtype=dt)
    assert oracle.reduce_all("min", v) == g["min_v"] and oracle.reduce_all("max", v) == g["max_v"]
    for op in ("min", "max"):
        for ax in (0, 1):
            assert np.array_equal(oracle.reduce_axis(op, b, ax), np.array(g[f"{op}_b_axis{ax}"], dtype=dt))
    if np.dtype(dt).kind == "f":
        assert oracle.mean(t) == g["mean_float"]
        assert np.array_equal(oracle.mean(t, 0), np.array(g["mean_axis0"], dtype=dt))
        assert np.array_equal(oracle.mean(t, 1), np.array(g["mean_axis1"], dtype=dt))


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_reference_variance_std_vectors(vectors, oracle, sfx):
    """tests/tensor/test_aggregate.nim:88-110 (its bar is 1e-8 in float64)."""
    g = vectors["aggregate_float"]
    dt = DTYPES[sfx]
    tol = 1e-8 if sfx == "f64" else 2e-6
    a, b = np.array(g["a"], dtype=dt), np.array(g["b"], dtype=dt)
    assert abs(oracle.variance(a) - g["variance_a"]) < tol * 5
    assert abs(oracle.std(a) - g["std_a"]) < tol * 5
    for ax in (0, 1):
        assert np.abs(oracle.variance(b, ax) - np.array(g[f"variance_b_axis{ax}"])).sum() < tol * 50
        assert np.abs(oracle.std(b, ax) - np.array(g[f"std_b_axis{ax}"])).sum() < tol * 10
    assert np.array_equal(oracle.variance(b.astype(dt), 0), np.array(g["variance_b_axis0"], dtype=dt))   # exact in the reference's test


def test_variance_against_float64_closed_form(oracle):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((37, 53)).astype(np.float32) * 3 + 1
    assert abs(oracle.variance(x) - np.var(x.astype(np.float64), ddof=1)) < 1e-4
    for ax in (0, 1):
        want = np.var(x.astype(np.float64), axis=ax, ddof=1, keepdims=True)
        got = oracle.variance(x, ax)
        assert got.shape == want.shape and np.allclose(got, want, rtol=1e-5)
        assert np.allclose(oracle.std(x, ax), np.sqrt(want), rtol=1e-5)
    x64 = x.astype(np.float64)
    assert np.allclose(oracle.variance(x64.T, 0), np.var(x64.T, axis=0, ddof=1, keepdims=True), rtol=1e-12)


@pytest.mark.parametrize("sfx", list(DTYPES))
def test_reference_argmax_argmin_vectors(vectors, oracle, sfx):
    """tests/tensor/test_aggregate.nim:112-215."""
    dt = DTYPES[sfx]
    for case in vectors["argmax_argmin"]["cases"]:
        a = np.array(case["a"], dtype=dt)
        for name, op in (("argmax", "max"), ("argmin", "min")):
            for ax, want in case[name].items():
                idx, val = oracle.argreduce(op, a, int(ax))
                assert idx.dtype == np.int64 and np.array_equal(idx, np.array(want)), (name, ax)
                assert np.array_equal(val, np.take_along_axis(a, idx, int(ax)))


def test_argreduce_first_extremum_and_nan_rules(oracle):
    """Ties keep the lowest position (NumPy's argmax / argmin agree on NaN-free data); a NaN in slice 0
    stays, a NaN elsewhere is never taken (what `if val > dmax` does, aggregate.nim:191, 248)."""
    rng = np.random.default_rng(3)
    for dt in DTYPES.values():
        x = rng.integers(-4, 5, (7, 33, 5)).astype(dt)      # many ties
        for v in (x, x.transpose(2, 0, 1), x[::-1, ::2]):
            for ax in range(3):
                for op, ref in (("max", np.argmax), ("min", np.argmin)):
                    idx, val = oracle.argreduce(op, v, ax)
                    assert np.array_equal(idx, np.expand_dims(ref(v, axis=ax), ax))
                    assert np.array_equal(val, np.take_along_axis(v, idx, ax))
    nan = np.nan
    x = np.array([[nan, 1, 2], [1, nan, 3], [1, nan, 0], [nan, nan, nan], [2, 2, nan]], dtype=np.float64)
    idx, val = oracle.argreduce("max", x, 1)
    assert idx.ravel().tolist() == [0, 2, 0, 0, 0] and np.isnan(val[0, 0]) and val[1, 0] == 3 and np.isnan(val[3, 0])
    idx, val = oracle.argreduce("min", x, 1)
    assert idx.ravel().tolist() == [0, 0, 2, 0, 0] and val[2, 0] == 0


def test_reference_maxpool_vectors(vectors, oracle):
    g = vectors["maxpool"]
    for dt in DTYPES.values():
        x = np.array(g["input"], dtype=dt).reshape(g["input_shape"])
        idx, pooled = oracle.maxpool2d(x, g["kernel"], g["padding"], g["stride"])
        assert np.array_equal(pooled, np.array(g["pooled"], dtype=dt).reshape(g["pooled_shape"]))
        assert np.array_equal(idx, np.array(g["max_indices"], dtype=np.int64))
        # backward with gradOutput = pooled (tests/nn_primitives/test_nnp_maxpool.nim:34-45)
        grad = oracle.maxpool2d_backward(x.shape, idx, pooled)
        assert np.array_equal(grad.reshape(4, 4), np.array(g["backward"]["grad_input"], dtype=dt))


def test_maxpool_backward_is_the_serial_scatter(oracle):
    """Overlapping windows record the same input element several times: the last output in index
    order wins (a NumPy fancy assignment applies the same rule); without overlap the result is the
    gradient of sum(maxpooled * G), checked by differences on a tie-free input."""
    rng = np.random.default_rng(8)
    x = rng.integers(-3, 4, (2, 3, 7, 6)).astype(np.float64)
    idx, pooled = oracle.maxpool2d(x, (3, 3), (1, 1), (1, 1))
    g = rng.standard_normal(pooled.shape)
    want = np.zeros(x.size)
    want[idx] = g.reshape(-1)
    assert np.array_equal(oracle.maxpool2d_backward(x.shape, idx, g).reshape(-1), want)
    x = rng.permutation(2 * 2 * 6 * 6).reshape(2, 2, 6, 6).astype(np.float64)   # no ties
    idx, pooled = oracle.maxpool2d(x, (2, 2), (0, 0), (2, 2))
    g = rng.standard_normal(pooled.shape)
    grad = oracle.maxpool2d_backward(x.shape, idx, g)
    h = 1e-3
    for pos in [(0, 0, 0, 0), (1, 1, 3, 2), (0, 1, 5, 5), (1, 0, 2, 4)]:
        xp, xm = x.copy(), x.copy()
        xp[pos] += h; xm[pos] -= h
        num = ((oracle.maxpool2d(xp, (2, 2), (0, 0), (2, 2))[1] - oracle.maxpool2d(xm, (2, 2), (0, 0), (2, 2))[1]) * g).sum() / (2 * h)
        assert abs(num - grad[pos]) < 1e-9


@pytest.mark.parametrize("sfx", ["i32", "i64"])
@pytest.mark.parametrize("kind", VIEW_KINDS)
def test_integer_reductions_against_numpy(oracle, sfx, kind):
    """Wrapping sums / products and min / max of integer views: NumPy's ufunc.reduce wraps the same
    way and is order independent for these operations."""
    dt = DTYPES[sfx]
    info = np.iinfo(dt)
    rng = np.random.default_rng(seed_of("red-int", sfx, kind))
    shape = (13, 21)
    parent = rng.integers(info.min, info.max, size=PARENT_SHAPE[kind](*shape), endpoint=True).astype(dt)
    v = view_of(parent, kind, shape)
    for op, uf in NP_OPS.items():
        with np.errstate(over="ignore"):
            assert oracle.reduce_all(op, v) == uf.reduce(v, axis=None, dtype=dt)
            for ax in range(v.ndim):
                assert np.array_equal(oracle.reduce_axis(op, v, ax), uf.reduce(v, axis=ax, dtype=dt, keepdims=True)), (op, ax)


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_float_sum_is_the_serial_fold(oracle, sfx):
    """A float sum is pinned by its order: the restatement must equal a left-to-right Python fold
    in the tensor's own precision, element order = C order of the view (not of memory)."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("fold", sfx))
    parent = rng.uniform(-1, 1, (7, 9, 5)).astype(dt)
    for v in (parent, parent.transpose(2, 0, 1), parent[::2, ::-1, 1:4]):
        acc = None
        for x in v.reshape(-1):          # reshape of a view copies in C order
            acc = x if acc is None else dt(acc + x)
        assert oracle.reduce_all("sum", v) == acc
        for ax in range(3):
            want = np.take(v, 0, axis=ax).copy()
            for l in range(1, v.shape[ax]):
                want = (want + np.take(v, l, axis=ax)).astype(dt)
            assert np.array_equal(oracle.reduce_axis("sum", v, ax), np.expand_dims(want, ax))


def test_float_sum_close_to_exact(oracle):
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, 2000)
    exact = sum(Fraction(float(v)) for v in x)
    assert abs(Fraction(float(oracle.reduce_all("sum", x))) - exact) < Fraction(1, 10**12)


def test_integer_mean_truncates(oracle):
    for dt in (np.int32, np.int64):
        assert oracle.mean(np.array([-7, 2, 1], dtype=dt)) == -1          # -4 div 3
        assert oracle.mean(np.array([7, -2, -1], dtype=dt)) == 1
        m = oracle.mean(np.array([[-7, 5], [2, 2]], dtype=dt), 0)
        assert np.array_equal(m, np.array([[-2, 3]], dtype=dt))           # -5 div 2 = -2


def test_empty_and_bad_axis(oracle):
    e = np.empty((0, 3), dtype=np.float32)
    assert oracle.reduce_axis("sum", e, 0).shape == (0, 3)               # returnEmptyIfEmpty
    with pytest.raises(ValueError):
        oracle.reduce_all("sum", e)
    with pytest.raises(IndexError):
        oracle.reduce_axis("sum", np.zeros((2, 2), np.float32), 2)


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_softmax_closed_form(oracle, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("softmax", sfx))
    x = (rng.standard_normal((9, 37)) * 5).astype(dt)
    got = oracle.softmax(x)
    xl = x.astype(np.longdouble)
    e = np.exp(xl - xl.max(1, keepdims=True))
    want = e / e.sum(1, keepdims=True)
    tol = 5e-7 if sfx == "f32" else 1e-15
    assert np.max(np.abs(got - want) / want) < tol * 10
    assert np.allclose(got.sum(1), 1, atol=tol * 40)
    # shift invariance (exact up to rounding of x + c) and large magnitudes without overflow
    assert np.allclose(oracle.softmax((x + dt(3)).astype(dt)), got, rtol=1e-4 if sfx == "f32" else 1e-12)
    big = np.array([[1000, 1001, 999], [-1000, -1001, -999]], dtype=dt)
    sb = oracle.softmax(big)
    assert np.all(np.isfinite(sb)) and np.allclose(sb[0], sb[1][[0, 1, 2]] if False else sb[0])
    # strided input (transposed view)
    xt = np.ascontiguousarray(x.T).T
    assert np.array_equal(oracle.softmax(xt), got)


@pytest.mark.parametrize("sfx", list(DTYPES))
def test_maxpool_against_bruteforce(oracle, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("maxpool", sfx))
    x = rng.integers(-50, 50, (2, 3, 7, 9)).astype(dt)
    for kernel, pad, stride in [((2, 2), (0, 0), (2, 2)), ((3, 3), (1, 1), (1, 1)), ((3, 2), (1, 0), (2, 3)), ((2, 2), (2, 2), (1, 1))]:
        idx, out = oracle.maxpool2d(x, kernel, pad, stride)
        low = -np.inf if np.dtype(dt).kind == "f" else np.iinfo(dt).min
        N, C, H, W = x.shape
        oh, ow = out.shape[2:]
        flat = x.reshape(-1)
        for n in range(N):
            for c in range(C):
                for h in range(oh):
                    for w in range(ow):
                        best, arg = low, np.iinfo(np.int64).min
                        for ph in range(kernel[0]):
                            for pw in range(kernel[1]):
                                r, q = h * stride[0] + ph - pad[0], w * stride[1] + pw - pad[1]
                                if 0 <= r < H and 0 <= q < W and x[n, c, r, q] > best:
                                    best, arg = x[n, c, r, q], q + W * (r + H * (c + n * C))
                        o = w + ow * (h + oh * (c + n * C))
                        assert out[n, c, h, w] == best and idx[o] == arg
                        if arg >= 0:
                            assert flat[arg] == best


def _exact_sce(x, target):
    """The loss from its definition in extended precision: mean over rows of logsumexp(row) - <row, target row>."""
    xl, tl = x.astype(np.longdouble), target.astype(np.longdouble)
    m = xl.max(1, keepdims=True)
    lse = np.log(np.exp(xl - m).sum(1)) + m[:, 0]
    return np.mean(lse - (xl * tl).sum(1))


def test_cross_entropy_reference_literal(oracle):
    """tests/nn_primitives/test_nnp_loss.nim:31-44: one row of four scores, the fourth class true: 0.0709 within 2e-5,
    through the dense and the sparse form."""
    predicted = np.array([[-3.44, 1.16, -0.81, 3.91]])
    truth = np.array([[0.0, 0, 0, 1]])
    assert abs(oracle.softmax_cross_entropy(predicted, truth) - 0.0709) <= 2e-5
    assert abs(oracle.sparse_softmax_cross_entropy(predicted, np.array([3])) - 0.0709) <= 2e-5


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_cross_entropy_closed_forms_and_gradients(oracle, sfx):
    """What the mathematics fixes for the restated one-pass recurrence: the loss against its definition in extended
    precision (random soft targets; one-hot targets = the sparse form), shift invariance, ln(classes) for equal
    scores, no overflow at +-1000; the backward forms against central differences of the loss (the reference's own
    check, test_nnp_loss.nim:46-62 and 66-103) and against softmax - target entry by entry."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("sce-oracle", sfx))
    tol = 2e-6 if sfx == "f32" else 1e-14
    for rows, cols in ((1, 4), (7, 10), (256, 20), (5, 1), (3, 333)):
        x = (rng.standard_normal((rows, cols)) * 3).astype(dt)
        soft = rng.uniform(0, 1, (rows, cols))
        soft = (soft / soft.sum(1, keepdims=True)).astype(dt)
        labels = rng.integers(0, cols, rows)
        onehot = np.zeros((rows, cols), dtype=dt)
        onehot[np.arange(rows), labels] = 1
        for target in (soft, onehot):
            got = oracle.softmax_cross_entropy(x, target)
            want = _exact_sce(x, target)
            assert abs(got - want) <= tol * max(1.0, abs(want)) * 8, (rows, cols)
        assert abs(oracle.sparse_softmax_cross_entropy(x, labels) - _exact_sce(x, onehot)) <= tol * 8 * max(1.0, abs(_exact_sce(x, onehot)))
        assert abs(oracle.softmax_cross_entropy((x + dt(5)).astype(dt), onehot) - oracle.softmax_cross_entropy(x, onehot)) <= tol * 64
        # gradients: g * (softmax - target) / rows, and the numerical gradient of the float64 loss
        xl = x.astype(np.longdouble)
        e = np.exp(xl - xl.max(1, keepdims=True))
        sm = e / e.sum(1, keepdims=True)
        g = dt(0.37)
        for target, got in ((soft, oracle.softmax_cross_entropy_backward(g, x, soft)),
                            (onehot, oracle.sparse_softmax_cross_entropy_backward(g, x, labels)),
                            (onehot, oracle.softmax_cross_entropy_backward(g, x, onehot))):
            want = np.longdouble(g) * (sm - target.astype(np.longdouble)) / rows
            assert np.max(np.abs(got - want)) <= tol * 8, (rows, cols)
        if sfx == "f64" and rows * cols <= 200:
            num = np.zeros_like(x)
            for idx in np.ndindex(*x.shape):
                keep = x[idx]
                x[idx] = keep + 1e-5; up = oracle.softmax_cross_entropy(x, soft)
                x[idx] = keep - 1e-5; dn = oracle.softmax_cross_entropy(x, soft)
                x[idx] = keep
                num[idx] = (up - dn) / 2e-5
            assert np.max(np.abs(oracle.softmax_cross_entropy_backward(1.0, x, soft) - num)) < 1e-9
    flat = np.zeros((3, 8), dtype=dt)
    assert abs(oracle.sparse_softmax_cross_entropy(flat, np.array([0, 3, 7])) - np.log(8)) <= tol * 8
    big = np.array([[1000, -1000, 999], [-1000, -1001, -999]], dtype=dt)
    v = oracle.sparse_softmax_cross_entropy(big, np.array([0, 2]))
    # ln(sumexp) + max is rounded at the magnitude of the scores before the score of the true class is subtracted
    assert np.isfinite(v) and abs(v - _exact_sce(big, np.array([[1, 0, 0], [0, 0, 1]], dtype=dt))) <= np.finfo(dt).eps * 1000 * 2
    assert oracle.softmax_cross_entropy(np.zeros((0, 4), dtype=dt), np.zeros((0, 4), dtype=dt)) == 0


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_sigmoid_cross_entropy_closed_forms(oracle, sfx):
    """No vector in the reference's tests: the restated body -y x + max(x, 0) + ln1p(exp(-|x|)) against the definition of
    binary cross-entropy, -(y ln s + (1 - y) ln(1 - s)) with s = sigmoid(x), in extended precision (they are the same
    function; the body is the overflow-free form), ln 2 at x = 0, no overflow at +-1000, and the backward form against
    (s - y) / batch and central differences of the loss."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("sigmoid-ce-oracle", sfx))
    tol = 4e-6 if sfx == "f32" else 1e-13
    for rows, cols in ((1, 1), (7, 10), (64, 33)):
        x = (rng.standard_normal((rows, cols)) * 3).astype(dt)
        y = rng.uniform(0, 1, (rows, cols)).astype(dt)
        xl, yl = x.astype(np.longdouble), y.astype(np.longdouble)
        s = 1 / (1 + np.exp(-xl))
        want = float(np.sum(-(yl * np.log(s) + (1 - yl) * np.log1p(-s))) / rows)
        got = oracle.sigmoid_cross_entropy(x, y)
        assert abs(got - want) <= tol * max(1.0, abs(want)) * cols, (rows, cols)
        g = oracle.sigmoid_cross_entropy_backward(dt(0.7), x, y)
        assert np.max(np.abs(g - np.longdouble(0.7) * (s - yl) / rows)) <= tol
        if sfx == "f64" and rows * cols <= 70:
            num = np.zeros_like(x)
            for idx in np.ndindex(*x.shape):
                keep = x[idx]
                x[idx] = keep + 1e-5; up = oracle.sigmoid_cross_entropy(x, y)
                x[idx] = keep - 1e-5; dn = oracle.sigmoid_cross_entropy(x, y)
                x[idx] = keep
                num[idx] = (up - dn) / 2e-5
            assert np.max(np.abs(oracle.sigmoid_cross_entropy_backward(1.0, x, y) - num)) < 1e-9
    zero = np.zeros((4, 5), dtype=dt)
    assert abs(oracle.sigmoid_cross_entropy(zero, zero) - 5 * np.log(2)) <= tol * 8
    big = np.array([[1000.0, -1000.0]], dtype=dt)
    assert oracle.sigmoid_cross_entropy(big, np.array([[1.0, 0.0]], dtype=dt)) == 0
    assert oracle.sigmoid_cross_entropy(big, np.array([[0.0, 1.0]], dtype=dt)) == 2000
