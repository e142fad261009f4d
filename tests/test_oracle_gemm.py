"""Pins the CPU oracle's gemm_strided restatement (oracle/laser_gemm.c) — CPU only.

Three independent anchors:
  1. the reference's own known-answer vectors (tests/golden/reference_vectors.json);
  2. closed forms the mathematics fixes: modular integer products (Python big ints / NumPy
     uint64), float64 and long-double products, exact rationals on tiny inputs;
  3. invariants: beta == 0 never reads C, K == 0 leaves C untouched, views == their copies.
"""
import numpy as np
import pytest

from conftest import seed_of, DTYPES, VIEW_KINDS, np_apply_ops, strided_view, view_of

TOL = {"f32": 1e-4, "f64": 1e-12}   # relative Frobenius error, the contract of the hot path


def _mat(vectors, name, dtype):
    return np.array(vectors["matrices"][name], dtype=dtype)


@pytest.mark.parametrize("sfx", ["f32", "f64", "i32", "i64"])
def test_reference_gemm_vectors(vectors, oracle, sfx):
    dt = DTYPES[sfx]
    for case in vectors["gemm"]:
        a, b, want = (_mat(vectors, case[k], dt) for k in ("a", "b", "expect"))
        got = oracle.matmul(a, b)
        assert np.array_equal(got, want), case["name"]


@pytest.mark.parametrize("sfx", ["f32", "f64", "i32", "i64"])
def test_reference_view_vectors(vectors, oracle, sfx):
    dt = DTYPES[sfx]
    for case in vectors["gemm_views"]:
        a = np_apply_ops(_mat(vectors, case["a"], dt), case["a_ops"])
        b = np_apply_ops(_mat(vectors, case["b"], dt), case["b_ops"])
        want = np.array(case["expect_literal"], dtype=dt) if "expect_literal" in case else _mat(vectors, case["expect"], dt)
        got = oracle.matmul(a, b)
        assert np.array_equal(got, want), case["name"]


def test_reference_colmajor_reversed_slice(vectors, oracle):
    c = vectors["gemm_colmajor_reversed_slice"]
    a = np.array(c["a"], dtype=np.float64)
    eig = np.asfortranarray(np.array(c["eigvecs_logical"], dtype=np.float64))
    b = np_apply_ops(eig, c["b_ops"])
    assert b.strides == (8, -16)            # column-major parent, columns reversed
    got = oracle.matmul(a, b)
    assert np.abs(got - np.array(c["expect"])).mean() < c["mean_abs_tol"]


def test_reference_fusion_vector(vectors, oracle):
    c = vectors["gemm_fusion"]
    A, x, b = (np.array(c[k], dtype=np.float64) for k in ("A", "x", "b"))
    out = b.copy()
    oracle.gemm_strided(1.0, A, x, 1.0, out)     # A*x + b  ==  gemm(1, A, x, 1, copy(b))
    assert np.array_equal(out, np.array(c["expect"])) and b[0, 0] == 0.0


# sizes around the register tile (6 x 16 / 6 x 8 / 6 x 4), the cache blocks (mc = 192 / 96,
# kc = 512 / 256) and a few primes
EDGE_SHAPES = [(1, 1, 1), (1, 7, 3), (5, 1, 9), (6, 16, 4), (7, 17, 5), (5, 15, 3), (13, 9, 1),
               (97, 33, 65), (191, 31, 513), (193, 17, 511), (95, 40, 257), (12, 130, 1025)]


@pytest.mark.parametrize("sfx", ["i32", "i64"])
@pytest.mark.parametrize("shape", EDGE_SHAPES)
def test_int_matches_modular_closed_form(oracle, sfx, shape):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, shape))
    M, N, K = shape
    info = np.iinfo(dt)
    # full-range entries: the products wrap many times over
    A = rng.integers(info.min, info.max, size=(M, K), dtype=dt, endpoint=True)
    B = rng.integers(info.min, info.max, size=(K, N), dtype=dt, endpoint=True)
    C = rng.integers(info.min, info.max, size=(M, N), dtype=dt, endpoint=True)
    for alpha, beta in [(1, 0), (1, 1), (3, -2), (-7, 5), (0, 1)]:
        want = oracle.closed_gemm_int_fast(alpha, A, B, beta, C)
        got = oracle.gemm_strided(alpha, A, B, beta, C.copy())
        assert np.array_equal(got, want), (alpha, beta)


def test_closed_forms_agree_with_bigint(oracle):
    """The fast uint64 closed form itself is checked against Python integers."""
    rng = np.random.default_rng(7)
    for dt in (np.int32, np.int64):
        info = np.iinfo(dt)
        A = rng.integers(info.min, info.max, size=(5, 9), dtype=dt, endpoint=True)
        B = rng.integers(info.min, info.max, size=(9, 4), dtype=dt, endpoint=True)
        C = rng.integers(info.min, info.max, size=(5, 4), dtype=dt, endpoint=True)
        for alpha, beta in [(1, 0), (-3, 7)]:
            assert np.array_equal(oracle.closed_gemm_int(alpha, A, B, beta, C),
                                  oracle.closed_gemm_int_fast(alpha, A, B, beta, C))


def test_int_wrap_known_answer(oracle):
    # (2^31 - 1) * 2 wraps to -2; 2^62 * 4 wraps to 0; hand-computed
    A = np.array([[2**31 - 1, 1]], dtype=np.int32)
    B = np.array([[2], [3]], dtype=np.int32)
    assert oracle.matmul(A, B)[0, 0] == -2 + 3
    A = np.array([[2**62, -1]], dtype=np.int64)
    B = np.array([[4], [5]], dtype=np.int64)
    assert oracle.matmul(A, B)[0, 0] == -5


@pytest.mark.parametrize("sfx", ["f32", "f64"])
@pytest.mark.parametrize("shape", EDGE_SHAPES)
def test_float_matches_wider_precision(oracle, sfx, shape):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, shape))
    M, N, K = shape
    A = rng.uniform(-1, 1, (M, K)).astype(dt)
    B = rng.uniform(-1, 1, (K, N)).astype(dt)
    C = rng.uniform(-1, 1, (M, N)).astype(dt)
    wide = np.float64 if sfx == "f32" else np.longdouble
    for alpha, beta in [(1, 0), (1, 1), (1.5, 0.5), (-0.25, 2)]:
        want = oracle.closed_gemm_float(alpha, A, B, beta, C, wide)
        got = oracle.gemm_strided(alpha, A, B, beta, C.copy())
        assert oracle.rel_frobenius(got, want) <= TOL[sfx], (alpha, beta)


def test_float_exact_rationals_tiny(oracle):
    """Dyadic inputs whose products and sums are exactly representable: any summation order
    must return the exact rational result."""
    rng = np.random.default_rng(11)
    A = (rng.integers(-64, 64, (7, 9)) / 8.0).astype(np.float64)
    B = (rng.integers(-64, 64, (9, 5)) / 4.0).astype(np.float64)
    C = (rng.integers(-64, 64, (7, 5)) / 2.0).astype(np.float64)
    want = oracle.closed_gemm_exact(0.5, A, B, 2, C)
    got = oracle.gemm_strided(0.5, A, B, 2.0, C.copy())
    assert all(float(w) == g for w, g in zip(want.ravel(), got.ravel()))


@pytest.mark.parametrize("sfx", ["f32", "f64", "i32", "i64"])
@pytest.mark.parametrize("ka", VIEW_KINDS)
@pytest.mark.parametrize("kb", ["C", "F", "colstep2", "neg_cols", "bcast_rows"])
def test_views_equal_their_copies(oracle, sfx, ka, kb):
    """A strided / transposed / reversed / broadcast operand gives the same bits as its
    contiguous copy (same algorithm, same order of operations)."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, ka, kb))
    M, N, K = 23, 19, 37
    A, _ = strided_view(rng, (M, K), dt, ka)
    B, _ = strided_view(rng, (K, N), dt, kb)
    got = oracle.matmul(A, B)
    want = oracle.matmul(np.ascontiguousarray(A), np.ascontiguousarray(B))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("sfx", ["f32", "f64", "i32", "i64"])
@pytest.mark.parametrize("kc", ["F", "rowstep2", "colstep2", "neg_rows", "inner_block"])
def test_strided_destination(oracle, sfx, kc):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, kc))
    M, N, K = 14, 21, 9
    A, _ = strided_view(rng, (M, K), dt, "C")
    B, _ = strided_view(rng, (K, N), dt, "C")
    Cv, parent = strided_view(rng, (M, N), dt, kc)
    before = parent.copy()
    want = oracle.gemm_strided(2, A, B, 3, np.ascontiguousarray(Cv))
    oracle.gemm_strided(2, A, B, 3, Cv)
    assert np.array_equal(Cv, want)
    # nothing outside the view was written
    inside = np.zeros(parent.shape, dtype=bool)
    view_of(inside, kc, (M, N))[...] = True
    assert np.array_equal(parent[~inside], before[~inside])


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_beta_zero_overwrites_nan(oracle, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(3)
    A = rng.uniform(-1, 1, (9, 20)).astype(dt)
    B = rng.uniform(-1, 1, (20, 33)).astype(dt)
    C = np.full((9, 33), np.nan, dtype=dt)
    oracle.gemm_strided(1, A, B, 0, C)
    assert np.isfinite(C).all()


@pytest.mark.parametrize("sfx", ["f32", "i64"])
def test_empty_k_leaves_c_untouched(oracle, sfx):
    dt = DTYPES[sfx]
    A = np.zeros((4, 0), dtype=dt)
    B = np.zeros((0, 5), dtype=dt)
    C = np.arange(20, dtype=dt).reshape(4, 5)
    oracle.gemm_strided(1, A, B, 0, C)          # beta is NOT applied: the loops never run
    assert np.array_equal(C, np.arange(20, dtype=dt).reshape(4, 5))


def test_alpha_zero_propagates_nan(oracle):
    A = np.array([[np.nan, 1.0]], dtype=np.float32)
    B = np.ones((2, 1), dtype=np.float32)
    C = np.zeros((1, 1), dtype=np.float32)
    oracle.gemm_strided(0.0, A, B, 1.0, C)
    assert np.isnan(C[0, 0])


def test_transpose_identity(oracle):
    """(A B)^T == B^T A^T through transposed views — bit for bit for integers."""
    rng = np.random.default_rng(5)
    A = rng.integers(-1000, 1000, (31, 45)).astype(np.int64)
    B = rng.integers(-1000, 1000, (45, 29)).astype(np.int64)
    assert np.array_equal(oracle.matmul(A, B).T, oracle.matmul(B.T, A.T))


def test_baseline_config_sizes_small(oracle):
    """Config 2 at 1500^3 is covered on the GPU; here the int32 path at a size that crosses
    every blocking boundary (M > mc, K > kc) against the closed form."""
    rng = np.random.default_rng(2001)
    A = rng.integers(-100, 101, (400, 600)).astype(np.int32)
    B = rng.integers(-100, 101, (600, 333)).astype(np.int32)
    want = oracle.closed_gemm_int_fast(1, A, B, 0, np.zeros((400, 333), np.int32))
    assert np.array_equal(oracle.matmul(A, B), want)
