"""gemv / dot on the GPU through the C ABI: reference literals, oracle parity (the oracle's
gemm_strided with N = 1 is the same arithmetic), closed forms for wraparound."""
import numpy as np
import pytest

from conftest import DTYPES, seed_of

pytestmark = pytest.mark.gpu
ALL = ["f32", "f64", "i32", "i64"]
TOL = {"f32": 1e-4, "f64": 1e-12}


def say(*a):
    print(*a, flush=True)


def fill(rng, shape, dt, full=False):
    if np.dtype(dt).kind == "f":
        return rng.uniform(-1, 1, size=shape).astype(dt)
    info = np.iinfo(dt)
    lo, hi = (info.min, info.max) if full else (-100, 100)
    return rng.integers(lo, hi, size=shape, endpoint=True).astype(dt)


def check(oracle, sfx, got, want, what):
    if sfx in ("i32", "i64"):
        assert np.array_equal(got, want), what
    else:
        assert oracle.rel_frobenius(got, want) <= TOL[sfx], what


@pytest.mark.parametrize("sfx", ALL)
def test_reference_literals(hip, vectors, sfx):
    dt = DTYPES[sfx]
    m = vectors["matrices"]
    for a, x, want in [("gv_a33", "gv_x", "gv_ax"), ("gv_b", "gv_u", "gv_bu"), ("gv_d", "gv_e", "gv_de")]:
        A, X = hip.toHip(np.array(m[a], dtype=dt)), hip.toHip(np.array(m[x], dtype=dt).ravel())
        assert np.array_equal((A * X).toCpu(), np.array(m[want], dtype=dt).ravel())
    # tests/tensor/test_operators_blas.nim:195-201 and test_operators_blas_cuda.nim:115-119
    u, v = hip.toHip(np.array([1, 3, -5], dtype=dt)), hip.toHip(np.array([4, -2, -1], dtype=dt))
    assert hip.dot(u, v) == 3
    # negative-step slices, test_operators_blas.nim:347-365
    b = hip.toHip(np.array(m["gv_b"], dtype=dt))
    uu = hip.toHip(np.array(m["gv_u"], dtype=dt).ravel())
    assert np.array_equal((b[4:1:-2, 3:0:-2] * uu[2::-2]).toCpu(), np.array([10027, -3682], dtype=dt))
    assert np.array_equal((b[2:4, 3:0:-2] * uu[2::-2]).toCpu(), np.array([-3682, -4783], dtype=dt))


SHAPES = [(1, 1), (3, 5), (64, 64), (65, 129), (256, 33), (300, 1000), (1024, 4096), (4096, 260), (2048, 2050),
          # tall and skinny, both ways: several short rows per wavefront (C layout) / the workgroup-wide walk with a second
          # pass over chunk partials (F layout); few long rows: chunks of a row over several wavefronts
          (70_000, 64), (9_000, 16), (5_000, 24), (20_000, 128), (64, 70_000), (5, 300_000), (300, 20_000), (512, 9_000)]


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("layout", ["C", "F", "step"])
def test_gemv_vs_oracle(hip, oracle, sfx, shape, layout):
    dt = DTYPES[sfx]
    M, N = shape
    rng = np.random.default_rng(seed_of("gemv", sfx, shape, layout))
    full = True
    if layout == "C":
        A = fill(rng, (M, N), dt, full); dA = hip.toHip(A)
    elif layout == "F":
        P = fill(rng, (N, M), dt, full); A = P.T; dA = hip.toHip(P).transpose()
    else:
        P = fill(rng, (M, 2 * N), dt, full); A = P[:, ::2]; dA = hip.toHip(P)[:, ::2]
    x, y = fill(rng, (N,), dt, full), fill(rng, (M,), dt, full)
    for alpha, beta in [(1, 0), (3, -2)]:
        say("gemv", sfx, shape, layout, alpha, beta)
        want = oracle.gemm_strided(alpha, A, x.reshape(N, 1), beta, y.copy().reshape(M, 1)).ravel()
        dy = hip.toHip(y)
        hip.gemv(alpha, dA, hip.toHip(x), beta, dy)
        check(oracle, sfx, dy.toCpu(), want, f"{shape} {layout} {alpha} {beta}")
    # strided x and y
    say("gemv strided vectors", sfx, shape, layout)
    x2, y2 = fill(rng, (2 * N,), dt, full), fill(rng, (3 * M,), dt, full)
    w = oracle.gemm_strided(1, A, x2[::2].copy().reshape(N, 1), 1, y2[::3].copy().reshape(M, 1)).ravel()
    dy2 = hip.toHip(y2)
    hip.gemv(1, dA, hip.toHip(x2)[::2], 1, dy2[::3])
    got = dy2.toCpu()
    check(oracle, sfx, got[::3], w, "strided vectors")
    keep = np.ones(3 * M, dtype=bool); keep[::3] = False
    assert np.array_equal(got[keep], y2[keep])


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("n", [1, 5, 1000, 4097, 1 << 20])
def test_dot(hip, oracle, sfx, n):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("dot", sfx, n))
    a, b = fill(rng, (2 * n,), dt, True), fill(rng, (n,), dt, True)
    say("dot", sfx, n)
    got = hip.dot(hip.toHip(a)[::2], hip.toHip(b))
    if sfx in ("i32", "i64"):
        U = lambda v: v.astype(np.int64).view(np.uint64)
        with np.errstate(over="ignore"):
            s = int((U(a[::2]) * U(b)).sum(dtype=np.uint64))
        w = 32 if sfx == "i32" else 64
        s %= 1 << w
        want = s - (1 << w) if s >= 1 << (w - 1) else s
        assert int(got) == want
    else:
        want = float(np.dot(a[::2].astype(np.longdouble), b.astype(np.longdouble)))
        scale = float(np.sqrt(n)) + 1
        assert abs(float(got) - want) <= (1e-5 if sfx == "f32" else 1e-13) * scale
    assert hip.dot(hip.empty((0,), dt), hip.empty((0,), dt)) == 0


def test_gemv_errors(hip):
    A = hip.toHip(np.zeros((3, 4), np.float32))
    with pytest.raises(IndexError):
        A * hip.toHip(np.zeros(3, np.float32))
    with pytest.raises(ValueError):
        hip.dot(hip.toHip(np.zeros(3, np.float32)), hip.toHip(np.zeros(4, np.float32)))
