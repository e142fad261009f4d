"""Softmax cross-entropy, dense and sparse, forward and backward, on the GPU through the C ABI: the reference's literal
(tests/nn_primitives/test_nnp_loss.nim:31-44), its own gradient checks (:46-62, :66-103: the backward forms against the
numerical gradient of the loss, mean relative error below 1e-6, dense against sparse), and the oracle's restatement
of the one-pass recurrence on batch sizes and class counts from one to vocabulary-sized rows, contiguous and strided.
Tolerances: loss within 4e-6 (f32) / 1e-13 (f64) of its definition in extended precision (and of the oracle on rows of
up to 4097 classes) relative to max(1, |loss|); gradient entries within
2e-6 / 1e-14 absolute of grad * (softmax - target) / batch (entries are at most |grad| / batch)."""
import numpy as np
import pytest

from conftest import DTYPES, seed_of

pytestmark = pytest.mark.gpu
FLT = ["f32", "f64"]
LOSS_TOL = {"f32": 4e-6, "f64": 1e-13}
GRAD_TOL = {"f32": 2e-6, "f64": 1e-14}


def say(*a):
    print(*a, flush=True)


def test_reference_literal(hip):
    predicted = hip.toHip(np.array([[-3.44, 1.16, -0.81, 3.91]]))
    truth = hip.toHip(np.array([[0.0, 0, 0, 1]]))
    sparse_truth = hip.toHip(np.array([3], dtype=np.int64))
    sce = hip.softmax_cross_entropy(predicted, truth)
    sparse = hip.sparse_softmax_cross_entropy(predicted, sparse_truth)
    assert abs(sce - 0.0709) <= 2e-5 and abs(sparse - 0.0709) <= 2e-5


def _exact_loss(x, target):
    xl, tl = x.astype(np.longdouble), target.astype(np.longdouble)
    m = xl.max(1, keepdims=True)
    return float(np.mean(np.log(np.exp(xl - m).sum(1)) + m[:, 0] - (xl * tl).sum(1)))


def _numerical_gradient(f, x, h=1e-5):
    g = np.zeros_like(x)
    for idx in np.ndindex(*x.shape):
        keep = x[idx]
        x[idx] = keep + h; up = f(x)
        x[idx] = keep - h; dn = f(x)
        x[idx] = keep
        g[idx] = (up - dn) / (2 * h)
    return g


def _mean_relative_error(a, b):
    d = np.maximum(np.abs(a), np.abs(b))
    return np.mean(np.where(d == 0, 0, np.abs(a - b) / np.where(d == 0, 1, d)))


@pytest.mark.parametrize("rows,cols", [(1, 4), (256, 20)])
def test_reference_gradient_checks(hip, oracle, rows, cols):
    """test_nnp_loss.nim:46-62 (one row) and :66-103 (batch 256, 20 classes): float64, expected gradient = loss times
    the numerical gradient of the loss, the device's backward called with the loss as upstream gradient."""
    rng = np.random.default_rng(seed_of("sce-reference", rows, cols))
    pred = rng.uniform(-1, 1, (rows, cols))
    labels = rng.integers(0, cols, rows)
    dense = np.zeros((rows, cols))
    dense[np.arange(rows), labels] = 1
    d_pred, d_dense, d_labels = hip.toHip(pred), hip.toHip(dense), hip.toHip(labels.astype(np.int64))
    sce, sparse = hip.softmax_cross_entropy(d_pred, d_dense), hip.sparse_softmax_cross_entropy(d_pred, d_labels)
    assert abs(sce - sparse) <= 2e-5
    expected = sce * _numerical_gradient(lambda p: oracle.softmax_cross_entropy(p, dense), pred.copy())
    expected_sparse = sparse * _numerical_gradient(lambda p: oracle.sparse_softmax_cross_entropy(p, labels), pred.copy())
    assert _mean_relative_error(expected, expected_sparse) < 1e-6
    assert _mean_relative_error(hip.softmax_cross_entropy_backward(sce, d_pred, d_dense).toCpu(), expected) < 1e-6
    assert _mean_relative_error(hip.sparse_softmax_cross_entropy_backward(sparse, d_pred, d_labels).toCpu(), expected_sparse) < 1e-6
    # the upstream gradient as a one-element device tensor, like the reference's Tensor overload
    g = hip.softmax_cross_entropy_backward(hip.toHip(np.array([sce])), d_pred, d_dense).toCpu()
    assert np.array_equal(g, hip.softmax_cross_entropy_backward(sce, d_pred, d_dense).toCpu())


SHAPES = [(1, 1), (1, 4), (3, 2), (64, 10), (256, 20), (1000, 17), (5000, 10), (33, 64), (70, 65), (129, 1000), (16, 4097),
          (2, 50000), (4, 262144)]


@pytest.mark.parametrize("sfx", FLT)
def test_loss_and_gradients_vs_oracle(hip, oracle, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("sce-gpu", sfx))
    for rows, cols in SHAPES:
        say("cross-entropy", sfx, rows, cols)
        x = (rng.standard_normal((rows, cols)) * 3).astype(dt)
        soft = rng.uniform(0, 1, (rows, cols))
        soft = (soft / soft.sum(1, keepdims=True)).astype(dt)
        labels = rng.integers(0, cols, rows).astype(np.int64)
        dx, dsoft, dlab = hip.toHip(x), hip.toHip(soft), hip.toHip(labels)
        # the loss from its definition in extended precision; the oracle's serial one-pass sums in the element type drift
        # from it on very long rows (like the reference's), the device's 64 partial recurrences per row less so
        onehot = np.zeros((rows, cols), dtype=dt)
        onehot[np.arange(rows), labels] = 1
        for target, got, oracle_value in ((soft, hip.softmax_cross_entropy(dx, dsoft), oracle.softmax_cross_entropy(x, soft)),
                                          (onehot, hip.sparse_softmax_cross_entropy(dx, dlab), oracle.sparse_softmax_cross_entropy(x, labels))):
            exact = _exact_loss(x, target)
            assert isinstance(got, dt) and abs(got - exact) <= LOSS_TOL[sfx] * max(1.0, abs(exact)), (rows, cols, got, exact)
            if cols <= 4097:
                assert abs(got - oracle_value) <= LOSS_TOL[sfx] * max(1.0, abs(oracle_value)), (rows, cols, got, oracle_value)
        g = dt(1.7)
        xl = x.astype(np.longdouble)
        e = np.exp(xl - xl.max(1, keepdims=True))
        sm = e / e.sum(1, keepdims=True)
        for target, got, oracle_value in ((soft, hip.softmax_cross_entropy_backward(g, dx, dsoft).toCpu(), oracle.softmax_cross_entropy_backward(g, x, soft)),
                                          (onehot, hip.sparse_softmax_cross_entropy_backward(g, dx, dlab).toCpu(), oracle.sparse_softmax_cross_entropy_backward(g, x, labels))):
            exact = np.longdouble(g) * (sm - target.astype(np.longdouble)) / rows
            assert np.max(np.abs(got - exact)) <= GRAD_TOL[sfx] * 1.7, (rows, cols)
            if cols <= 4097:
                assert np.max(np.abs(got - oracle_value)) <= GRAD_TOL[sfx] * 1.7, (rows, cols)
        # every row of the gradient sums to zero (softmax and the target both sum to one)
        assert np.max(np.abs(got.astype(np.float64).sum(1))) <= GRAD_TOL[sfx] * cols


@pytest.mark.parametrize("sfx", FLT)
def test_strided_operands(hip, oracle, sfx):
    """Transposed scores and targets, a column slice of a wider buffer, every other label of a longer vector: the same
    values as their contiguous copies."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("sce-views", sfx))
    rows, cols = 37, 21
    x = (rng.standard_normal((rows, cols)) * 2).astype(dt)
    t = rng.uniform(0, 1, (rows, cols))
    t = (t / t.sum(1, keepdims=True)).astype(dt)
    labels = rng.integers(0, cols, rows).astype(np.int64)
    base = hip.softmax_cross_entropy(hip.toHip(x), hip.toHip(t))
    base_sparse = hip.sparse_softmax_cross_entropy(hip.toHip(x), hip.toHip(labels))
    base_grad = hip.softmax_cross_entropy_backward(1.0, hip.toHip(x), hip.toHip(t)).toCpu()
    xt, tt = hip.toHip(np.ascontiguousarray(x.T)).transpose(), hip.toHip(np.ascontiguousarray(t.T)).transpose()
    assert hip.softmax_cross_entropy(xt, tt) == base
    assert np.array_equal(hip.softmax_cross_entropy_backward(1.0, xt, tt).toCpu(), base_grad)
    wide = np.zeros((rows, cols + 11), dtype=dt)
    wide[:, 5:5 + cols] = x
    xs = hip.toHip(wide)[:, 5:5 + cols]
    assert hip.softmax_cross_entropy(xs, hip.toHip(t)) == base
    every_other = np.zeros(2 * rows, dtype=np.int64)
    every_other[::2] = labels
    ls = hip.toHip(every_other)[::2]
    assert hip.sparse_softmax_cross_entropy(xs, ls) == base_sparse
    assert np.array_equal(hip.sparse_softmax_cross_entropy_backward(1.0, xs, ls).toCpu(),
                          hip.sparse_softmax_cross_entropy_backward(1.0, hip.toHip(x), hip.toHip(labels)).toCpu())


def test_edge_cases_and_errors(hip):
    f32 = np.float32
    assert hip.softmax_cross_entropy(hip.zeros((0, 5), f32), hip.zeros((0, 5), f32)) == 0          # empty batch: 0, like the reference
    assert hip.sparse_softmax_cross_entropy(hip.zeros((0, 5), f32), hip.toHip(np.zeros(0, np.int64))) == 0
    x = hip.toHip(np.array([[1000.0, -1000.0, 999.0], [-1000.0, -1001.0, -999.0]], dtype=f32))
    v = hip.sparse_softmax_cross_entropy(x, hip.toHip(np.array([0, 2], dtype=np.int64)))
    assert np.isfinite(v) and abs(v - 0.36043) < 2e-4                                                 # no overflow at +-1000
    # a label outside the row is not read: the loss is NaN, and so is that row of the gradient (the other rows are not touched by it)
    bad = hip.toHip(np.array([0, 7], dtype=np.int64))
    assert np.isnan(hip.sparse_softmax_cross_entropy(x, bad))
    g = hip.sparse_softmax_cross_entropy_backward(1.0, x, bad).toCpu()
    good = hip.sparse_softmax_cross_entropy_backward(1.0, x, hip.toHip(np.array([0, 2], dtype=np.int64))).toCpu()
    assert np.all(np.isnan(g[1])) and np.array_equal(g[0], good[0])
    g = hip.sparse_softmax_cross_entropy_backward(1.0, x, hip.toHip(np.array([-1, 2], dtype=np.int64))).toCpu()
    assert np.all(np.isnan(g[0])) and np.array_equal(g[1], good[1])
    with pytest.raises(ValueError):
        hip.softmax_cross_entropy(hip.zeros((2, 3), f32), hip.zeros((2, 4), f32))
    with pytest.raises(ValueError):
        hip.sparse_softmax_cross_entropy(hip.zeros((2, 3), f32), hip.toHip(np.zeros(3, np.int64)))
    with pytest.raises(TypeError):
        hip.sparse_softmax_cross_entropy(hip.zeros((2, 3), f32), hip.toHip(np.zeros(2, np.int32)))
    with pytest.raises((TypeError, ValueError)):
        hip.softmax_cross_entropy(hip.zeros((2, 3), np.int32), hip.zeros((2, 3), np.int32))


@pytest.mark.parametrize("sfx", FLT)
def test_sigmoid_cross_entropy(hip, oracle, sfx):
    """sigmoid_cross_entropy and its backward form (nnp_sigmoid_cross_entropy.nim:23-62; no vector in the reference's
    tests: pinned on the definition of binary cross-entropy in extended precision) on small, ragged, large and strided
    operands: loss within 4e-6 / 1e-13 of the definition relative to max(1, |loss|), gradient entries within 2e-6 / 1e-14,
    and both against the oracle's restatement where its serial sum is short."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("sigmoid-ce-gpu", sfx))
    for rows, cols in ((1, 1), (7, 10), (64, 33), (1000, 17), (513, 2049), (4096, 1000)):
        say("sigmoid cross-entropy", sfx, rows, cols)
        x = (rng.standard_normal((rows, cols)) * 3).astype(dt)
        y = rng.uniform(0, 1, (rows, cols)).astype(dt)
        dx, dy = hip.toHip(x), hip.toHip(y)
        xl, yl = x.astype(np.longdouble), y.astype(np.longdouble)
        s = 1 / (1 + np.exp(-xl))
        exact = float(np.sum(-(yl * np.log(s) + (1 - yl) * np.log1p(-s))) / rows)
        got = hip.sigmoid_cross_entropy(dx, dy)
        assert isinstance(got, dt) and abs(got - exact) <= LOSS_TOL[sfx] * max(1.0, abs(exact)), (rows, cols, got, exact)
        if rows * cols <= 20000:
            want = oracle.sigmoid_cross_entropy(x, y)
            assert abs(got - want) <= LOSS_TOL[sfx] * max(1.0, abs(want)) * 4, (rows, cols)
        g = hip.sigmoid_cross_entropy_backward(dt(1.3), dx, dy).toCpu()
        assert np.max(np.abs(g - np.longdouble(1.3) * (s - yl) / rows)) <= GRAD_TOL[sfx] * 1.3, (rows, cols)
        if rows * cols <= 20000:
            assert np.max(np.abs(g - oracle.sigmoid_cross_entropy_backward(dt(1.3), x, y))) <= GRAD_TOL[sfx] * 1.3
    # transposed operands: the same value and gradient as their contiguous copies
    x, y = (rng.standard_normal((37, 21)) * 2).astype(dt), rng.uniform(0, 1, (37, 21)).astype(dt)
    base = hip.sigmoid_cross_entropy(hip.toHip(x), hip.toHip(y))
    xt, yt = hip.toHip(np.ascontiguousarray(x.T)).transpose(), hip.toHip(np.ascontiguousarray(y.T)).transpose()
    assert hip.sigmoid_cross_entropy(xt, yt) == base
    assert np.array_equal(hip.sigmoid_cross_entropy_backward(1.0, xt, yt).toCpu(), hip.sigmoid_cross_entropy_backward(1.0, hip.toHip(x), hip.toHip(y)).toCpu())
    big = hip.toHip(np.array([[1000.0, -1000.0]], dtype=dt))
    assert hip.sigmoid_cross_entropy(big, hip.toHip(np.array([[1.0, 0.0]], dtype=dt))) == 0
    with pytest.raises(ValueError):
        hip.sigmoid_cross_entropy(hip.zeros((2, 3), dt), hip.zeros((3, 2), dt))
    with pytest.raises(ValueError):
        hip.sigmoid_cross_entropy(hip.zeros((0, 3), dt), hip.zeros((0, 3), dt))
