"""GEMM parity on the GPU: the HIP kernels (through the C ABI) against the CPU oracle, the
reference's known-answer vectors, and size-independent properties at the full benchmark sizes.

Bars: integers bit-exact; float32 <= 1e-4, float64 <= 1e-12 relative Frobenius error."""
import numpy as np
import pytest

from conftest import seed_of, DTYPES, VIEW_KINDS, hip_apply_ops, np_apply_ops

pytestmark = pytest.mark.gpu

TOL = {"f32": 1e-4, "f64": 1e-12}
ALL = ["f32", "f64", "i32", "i64"]


def say(*a):
    print(*a, flush=True)


def _mat(vectors, name, dt):
    return np.array(vectors["matrices"][name], dtype=dt)


def fill(rng, shape, dt, lo=-100, hi=100):
    if np.dtype(dt).kind == "f":
        return rng.uniform(-1, 1, size=shape).astype(dt)
    return rng.integers(lo, hi, size=shape, endpoint=True).astype(dt)


def assert_parity(oracle, sfx, got, want, what=""):
    if sfx in ("i32", "i64"):
        assert np.array_equal(got, want), what
    else:
        err = oracle.rel_frobenius(got, want)
        assert err <= TOL[sfx], f"{what}: rel Frobenius {err:.3e}"


# ------------------------------------------------------------------ reference vectors
@pytest.mark.parametrize("sfx", ALL)
def test_reference_vectors(hip, vectors, sfx):
    dt = DTYPES[sfx]
    for case in vectors["gemm"]:
        say("gemm vector", case["name"], sfx)
        a, b = hip.toHip(_mat(vectors, case["a"], dt)), hip.toHip(_mat(vectors, case["b"], dt))
        assert np.array_equal((a * b).toCpu(), _mat(vectors, case["expect"], dt)), case["name"]


@pytest.mark.parametrize("sfx", ALL)
def test_reference_view_vectors(hip, vectors, sfx):
    dt = DTYPES[sfx]
    for case in vectors["gemm_views"]:
        say("gemm view vector", case["name"], sfx)
        a = hip_apply_ops(hip.toHip(_mat(vectors, case["a"], dt)), case["a_ops"])
        b = hip_apply_ops(hip.toHip(_mat(vectors, case["b"], dt)), case["b_ops"])
        want = np.array(case["expect_literal"], dtype=dt) if "expect_literal" in case else _mat(vectors, case["expect"], dt)
        assert np.array_equal((a * b).toCpu(), want), case["name"]


def test_reference_colmajor_reversed_slice(hip, vectors):
    c = vectors["gemm_colmajor_reversed_slice"]
    a = hip.toHip(np.array(c["a"], dtype=np.float64))
    # column-major parent made on the device: upload the transpose, view it transposed
    eig = hip.toHip(np.array(c["eigvecs_logical"], dtype=np.float64).T.copy()).transpose()
    assert eig.is_F_contiguous()
    b = hip_apply_ops(eig, c["b_ops"])
    assert b.strides == (1, -2)
    val = (a * b).toCpu()
    assert np.abs(val - np.array(c["expect"])).mean() < c["mean_abs_tol"]


def test_reference_fusion_vector(hip, vectors):
    c = vectors["gemm_fusion"]
    A, x, b = (hip.toHip(np.array(c[k], dtype=np.float64)) for k in ("A", "x", "b"))
    for _ in range(5):
        out = b.clone()
        hip.gemm(1.0, A, x, 1.0, out)
        assert out.toCpu()[0, 0] == 12.0 and b.toCpu()[0, 0] == 0.0


# ------------------------------------------------------------------ oracle parity, edge shapes
EDGE_SHAPES = [(1, 1, 1), (1, 7, 3), (5, 1, 9), (33, 31, 2), (64, 64, 16), (65, 63, 17), (127, 129, 15),
               (128, 128, 128), (255, 257, 33), (256, 256, 64), (300, 200, 100), (97, 513, 65)]


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("shape", EDGE_SHAPES)
def test_edge_shapes_vs_oracle(hip, oracle, sfx, shape):
    dt = DTYPES[sfx]
    M, N, K = shape
    rng = np.random.default_rng(seed_of(sfx, shape))
    info = None if np.dtype(dt).kind == "f" else np.iinfo(dt)
    lo, hi = (-100, 100) if info is None else (info.min, info.max)   # integers: full range, wraps
    A, B, C = fill(rng, (M, K), dt, lo, hi), fill(rng, (K, N), dt, lo, hi), fill(rng, (M, N), dt, lo, hi)
    for alpha, beta in [(1, 0), (1, 1), (3, -2)]:
        say("edge", sfx, shape, alpha, beta)
        want = oracle.gemm_strided(alpha, A, B, beta, C.copy())
        dC = hip.toHip(C)
        hip.gemm(alpha, hip.toHip(A), hip.toHip(B), beta, dC)
        assert_parity(oracle, sfx, dC.toCpu(), want, f"{shape} a={alpha} b={beta}")


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("tile", ["0", "1", "2", "3", "4", "5"])
def test_every_tile_shape(hip, oracle, sfx, tile, monkeypatch):
    """Forces each workgroup tile candidate on a ragged problem."""
    if sfx in ("i32", "i64") and int(tile) >= 2:
        pytest.skip("integer path has two tile candidates")
    monkeypatch.setenv(f"AM_HIP_GEMM_TILE_{sfx.upper()}", tile)
    dt = DTYPES[sfx]
    rng = np.random.default_rng(int(tile) + 17)
    M, N, K = 517, 389, 77
    A, B, C = fill(rng, (M, K), dt), fill(rng, (K, N), dt), fill(rng, (M, N), dt)
    say("tile", sfx, tile)
    want = oracle.gemm_strided(2, A, B, 1, C.copy())
    dC = hip.toHip(C)
    hip.gemm(2, hip.toHip(A), hip.toHip(B), 1, dC)
    assert_parity(oracle, sfx, dC.toCpu(), want, f"tile {tile}")


@pytest.mark.parametrize("layout", ["CC", "FC", "CF", "FF"])
def test_f32_128_tile_with_eight_wavefronts(hip, oracle, layout, monkeypatch):
    """More than 128 tiles of 128 x 128 and no split of k: the workgroup of eight wavefronts (32 x 64 each) that the
    library uses there, on ragged extents, every operand layout, alpha/beta and a strided destination."""
    monkeypatch.setenv("AM_HIP_GEMM_TILE_F32", "1")
    rng = np.random.default_rng(seed_of("tile128x8", layout))
    for (M, N, K) in [(1500, 1400, 77), (1409, 1537, 16), (1665, 1281, 131)]:
        A, B = fill(rng, (M, K), np.float32), fill(rng, (K, N), np.float32)
        C = fill(rng, (M, 2 * N), np.float32)
        dA = hip.toHip(np.ascontiguousarray(A.T)).transpose() if layout[0] == "F" else hip.toHip(A)
        dB = hip.toHip(np.ascontiguousarray(B.T)).transpose() if layout[1] == "F" else hip.toHip(B)
        say("tile128x8", layout, (M, N, K))
        want = C.copy()
        oracle.gemm_strided(-0.5, A, B, 2, want[:, ::2])
        dC = hip.toHip(C)
        hip.gemm(-0.5, dA, dB, 2, dC[:, ::2])
        assert_parity(oracle, "f32", dC.toCpu(), want, f"{(M, N, K)} {layout}")


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("layout", ["CC", "FC", "CF", "FF"])
def test_unit_stride_operands_of_any_pitch_and_alignment(hip, oracle, sfx, layout):
    """Operands with a unit stride are moved in 16-byte vectors whatever their row pitch, extent and base
    address: extents that are not a multiple of the vector (k, m and n all ragged), pitches that put every
    row at another offset within 16 bytes, base addresses one element off, and views that end exactly at the
    end of their allocation (so that a vector read past the last row would leave it)."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("ragged", sfx, layout))
    vk = 16 // np.dtype(dt).itemsize
    for (M, N, K) in [(259, 131, 67), (64 + 1, 4 * vk + 1, vk + 1), (300, 257, 2 * vk - 1)]:
        # parents sized to a whole number of 512-byte allocation granules, views that drop the FIRST row and
        # column: the view's last element is the allocation's last element
        def parent_and_view(rows, cols, fortran):
            pr, pc = (cols + 1, rows + 1) if fortran else (rows + 1, cols + 1)
            pad = (-(pr * pc * np.dtype(dt).itemsize)) % 512 // np.dtype(dt).itemsize
            return fill(rng, (pad + pr * pc,), dt), pad, pr, pc
        views_np, views_dev = [], []
        for (rows, cols), fortran in (((M, K), layout[0] == "F"), ((K, N), layout[1] == "F")):
            flat, pad, pr, pc = parent_and_view(rows, cols, fortran)
            host = flat[pad:].reshape(pr, pc)[1:, 1:]
            dflat = hip.toHip(flat)
            from arraymancer_amd import metadata as md
            from arraymancer_amd.tensor_hip import HipTensor
            dev = HipTensor(md.Layout((pr - 1, pc - 1), (pc, 1), pad + pc + 1), dflat.storage, dflat.dtype)
            if fortran:
                host, dev = host.T, dev.transpose()
            assert host.shape == (rows, cols) and dev.shape == (rows, cols)
            views_np.append(host); views_dev.append(dev)
        C = fill(rng, (M, N), dt)
        for alpha, beta in ((1, 0), (2, 1)):
            say("ragged", sfx, layout, (M, N, K), alpha, beta)
            want = oracle.gemm_strided(alpha, views_np[0], views_np[1], beta, C.copy())
            dC = hip.toHip(C)
            hip.gemm(alpha, views_dev[0], views_dev[1], beta, dC)
            assert_parity(oracle, sfx, dC.toCpu(), want, f"{layout} {(M, N, K)}")


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_extents_just_above_a_tile_multiple(hip, oracle, sfx, monkeypatch):
    """A float product with a few rows / columns more than a multiple of the tile edge runs as the aligned block
    plus strips of those rows and columns (three or two launches): every block of C, the bias and the views must
    be cut at the same place. Compared with the oracle and with the same product run whole (the cut is forced: the
    library's own estimate only cuts where a round of tiles is saved)."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("peel", sfx))
    for (M, N, K), trans in [((1030, 520, 300), ""), ((512 + 16, 2048 + 1, 96), "AB"), ((1024, 1024 + 3, 130), "B"), ((1024 + 2, 640, 77), "A")]:
        A = fill(rng, (K, M) if "A" in trans else (M, K), dt)
        B = fill(rng, (N, K) if "B" in trans else (K, N), dt)
        C, bias = fill(rng, (M, N), dt), fill(rng, (1, N), dt)
        dA, dB = hip.toHip(A), hip.toHip(B)
        vA, vB = (dA.transpose(), A.T) if "A" in trans else (dA, A), (dB.transpose(), B.T) if "B" in trans else (dB, B)
        results = {}
        for peel in ("1", "0"):
            monkeypatch.setenv("AM_HIP_GEMM_PEEL", peel)
            say("peel", sfx, (M, N, K), trans, "cut" if peel == "1" else "whole")
            dC = hip.toHip(C)
            hip.gemm(1.5, vA[0], vB[0], 0.5, dC, epilogue="bias_relu", bias=hip.toHip(bias))
            results[peel] = dC.toCpu()
            dP = hip.empty((M, N), dt)
            hip.gemm(1, vA[0], vB[0], 0, dP)
            results[peel + "plain"] = dP.toCpu()
        want = oracle.gemm_strided(1.5, vA[1], vB[1], 0.5, C.copy())
        want = oracle.map2("add_relu", want, oracle.broadcast(bias, want.shape))
        assert_parity(oracle, sfx, results["1"], want, f"cut {(M, N, K)} {trans}")
        assert_parity(oracle, sfx, results["1plain"], oracle.matmul(vA[1], vB[1]), f"cut, plain {(M, N, K)} {trans}")
        assert oracle.rel_frobenius(results["1"], results["0"]) <= TOL[sfx]
        assert oracle.rel_frobenius(results["1plain"], results["0plain"]) <= TOL[sfx]
        # a column-major destination (the library multiplies the transposed problem: the cut must follow the swap)
        monkeypatch.setenv("AM_HIP_GEMM_PEEL", "1")
        dCt = hip.toHip(np.ascontiguousarray(C.T))
        hip.gemm(1.5, vA[0], vB[0], 0.5, dCt.transpose(), epilogue="bias", bias=hip.toHip(bias))
        want_cm = oracle.map2("add", oracle.gemm_strided(1.5, vA[1], vB[1], 0.5, C.copy()), oracle.broadcast(bias, C.shape))
        assert_parity(oracle, sfx, dCt.toCpu().T, want_cm, f"cut, column-major C {(M, N, K)} {trans}")


# ------------------------------------------------------------------ strided / transposed views
def device_view(hip, parent_np, kind, shape):
    """The same geometry as conftest.strided_view, built with view ops on the device tensor."""
    m, n = shape
    t = hip.toHip(parent_np)
    if kind == "C":
        return t
    if kind == "F":
        return t.transpose()
    if kind == "rowstep2":
        return t[::2]
    if kind == "colstep2":
        return t[:, ::2]
    if kind == "neg_rows":
        return t[::-1]
    if kind == "neg_cols":
        return t[:, ::-1]
    if kind == "inner_block":
        return t[2:2 + m, 1:1 + n]
    if kind == "bcast_rows":
        return t.broadcast((m, n))
    raise KeyError(kind)


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("ka", VIEW_KINDS)
@pytest.mark.parametrize("kb", VIEW_KINDS)
def test_views_without_host_copy(hip, oracle, sfx, ka, kb):
    from conftest import strided_view
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, ka, kb))
    M, N, K = 72, 52, 40      # multiples of 4: the vector loaders are eligible where strides allow
    A, pa = strided_view(rng, (M, K), dt, ka)
    B, pb = strided_view(rng, (K, N), dt, kb)
    say("views", sfx, ka, kb)
    dA, dB = device_view(hip, pa, ka, (M, K)), device_view(hip, pb, kb, (K, N))
    assert dA.shape == A.shape and dB.shape == B.shape
    got = (dA * dB).toCpu()
    want = oracle.matmul(A, B)
    assert_parity(oracle, sfx, got, want, f"{ka} x {kb}")


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("kc", ["F", "rowstep2", "colstep2", "neg_rows", "inner_block"])
def test_strided_destination(hip, oracle, sfx, kc):
    from conftest import strided_view, view_of
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, kc))
    M, N, K = 37, 45, 29
    A, B = fill(rng, (M, K), dt), fill(rng, (K, N), dt)
    Cv, parent = strided_view(rng, (M, N), dt, kc)
    say("dest", sfx, kc)
    before = parent.copy()
    dC = device_view(hip, parent, kc, (M, N))               # uploads `parent`, views it on the device
    hip.gemm(2, hip.toHip(A), hip.toHip(B), 3, dC)
    oracle.gemm_strided(2, A, B, 3, Cv)                      # writes through the NumPy view into `parent`
    after = hip.HipTensor(hip.Layout(parent.shape, tuple(s // parent.itemsize for s in parent.strides), 0),
                          dC.storage, dC.dtype).toCpu()
    assert_parity(oracle, sfx, view_of(after, kc, (M, N)), Cv, kc)
    inside = np.zeros(parent.shape, dtype=bool)
    view_of(inside, kc, (M, N))[...] = True
    assert np.array_equal(after[~inside], before[~inside])   # nothing outside the view was written


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_float_semantics(hip, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(9)
    A, B = fill(rng, (70, 30), dt), fill(rng, (30, 90), dt)
    say("beta0 NaN", sfx)
    dC = hip.toHip(np.full((70, 90), np.nan, dtype=dt))
    hip.gemm(1, hip.toHip(A), hip.toHip(B), 0, dC)
    assert np.isfinite(dC.toCpu()).all()                      # beta == 0 never reads C
    say("alpha0 NaN", sfx)
    A2 = A.copy(); A2[3, 4] = np.nan
    dC = hip.toHip(np.zeros((70, 90), dtype=dt))
    hip.gemm(0, hip.toHip(A2), hip.toHip(B), 1, dC)
    assert np.isnan(dC.toCpu()[3]).all()                      # alpha == 0 is not special-cased


@pytest.mark.parametrize("sfx", ALL)
def test_empty_extents_leave_c_untouched(hip, sfx):
    dt = DTYPES[sfx]
    C = np.arange(20, dtype=dt).reshape(4, 5)
    dC = hip.toHip(C)
    hip.gemm(1, hip.empty((4, 0), dt), hip.empty((0, 5), dt), 0, dC)
    assert np.array_equal(dC.toCpu(), C)
    assert (hip.empty((0, 3), dt) * hip.empty((3, 4), dt)).shape == (0, 4)


@pytest.mark.parametrize("sfx", ALL)
def test_linear_backward(hip, oracle, sfx):
    """gradInput = gradOutput * weight, gradWeight = gradOutput.transpose * input,
    gradBias = sum(gradOutput, axis=0) (nnp_linear.nim:39-66) against the oracle's GEMM and fold,
    at the dense layer of the MNIST chain and at a ragged shape."""
    dt = DTYPES[sfx]
    for batch, fin, fout in ((64, 800, 500), (37, 129, 61)):
        rng = np.random.default_rng(batch)
        x, W, g = fill(rng, (batch, fin), dt), fill(rng, (fout, fin), dt), fill(rng, (batch, fout), dt)
        say("linear_backward", sfx, batch, fin, fout)
        gi, gw, gb = hip.linear_backward(hip.toHip(x), hip.toHip(W), hip.toHip(g))
        assert gi.shape == (batch, fin) and gw.shape == (fout, fin) and gb.shape == (1, fout)
        assert_parity(oracle, sfx, gi.toCpu(), oracle.matmul(g, W), "gradInput")
        assert_parity(oracle, sfx, gw.toCpu(), oracle.matmul(g.T, x), "gradWeight")
        assert_parity(oracle, sfx, gb.toCpu(), oracle.reduce_axis("sum", g, 0), "gradBias")
        gi2, gw2 = hip.linear_backward(hip.toHip(x), hip.toHip(W), hip.toHip(g), with_bias=False)
        assert np.array_equal(gi2.toCpu(), gi.toCpu()) and np.array_equal(gw2.toCpu(), gw.toCpu())


def test_linear_backward_is_the_gradient_of_linear(hip):
    """Central differences of L = sum(linear(x, W, b) *. G) through the device forward pass agree
    with linear_backward (float64, so the difference quotient is good to ~1e-9)."""
    rng = np.random.default_rng(5)
    x, W, b, G = (rng.standard_normal(s) for s in ((5, 7), (4, 7), (1, 4), (5, 4)))
    dG = hip.toHip(G)

    def loss(x_, W_, b_):
        return hip.sum(hip.bc_mul(hip.linear(hip.toHip(x_), hip.toHip(W_), hip.toHip(b_)), dG))

    gi, gw, gb = (t.toCpu() for t in hip.linear_backward(hip.toHip(x), hip.toHip(W), dG))
    h = 1e-5
    for arr, grad, pos in ((x, gi, 0), (W, gw, 1), (b, gb, 2)):
        num = np.zeros_like(arr)
        for idx in np.ndindex(arr.shape):
            args = [x.copy(), W.copy(), b.copy()]
            args[pos][idx] += h
            up = loss(*args)
            args[pos][idx] -= 2 * h
            num[idx] = (up - loss(*args)) / (2 * h)
        assert np.allclose(num, grad, rtol=1e-7, atol=1e-8), pos


def test_int_wrap_known_answers(hip):
    A = hip.toHip(np.array([[2**31 - 1, 1]], dtype=np.int32))
    B = hip.toHip(np.array([[2], [3]], dtype=np.int32))
    assert (A * B).toCpu()[0, 0] == 1
    A = hip.toHip(np.array([[2**62, -1]], dtype=np.int64))
    B = hip.toHip(np.array([[4], [5]], dtype=np.int64))
    assert (A * B).toCpu()[0, 0] == -5


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_fused_epilogue(hip, oracle, sfx):
    """linear + bias + ReLU in the GEMM epilogue == the reference's three passes
    (nnp_linear.nim:28-29 then relu)."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(21)
    x, W, b = fill(rng, (64, 100), dt), fill(rng, (50, 100), dt), fill(rng, (1, 50), dt)
    say("epilogue", sfx)
    out = oracle.matmul(x, W.T)
    oracle.map2("add", out, oracle.broadcast(b, out.shape), out=out)
    want_lin = out.copy()
    want_relu = oracle.unary("relu", out)
    dx, dW, db = hip.toHip(x), hip.toHip(W), hip.toHip(b)
    assert_parity(oracle, sfx, hip.linear(dx, dW, db).toCpu(), want_lin, "bias")
    got = hip.linear(dx, dW, db, relu=True).toCpu()
    assert_parity(oracle, sfx, got, want_relu, "bias+relu")
    assert (got >= 0).all() and (got == 0).any()
    # column-vector bias [M, 1]
    bcol = fill(rng, (64, 1), dt)
    o = hip.empty((64, 50), dt)
    hip.gemm(1, dx, dW.transpose(), 0, o, epilogue="bias", bias=hip.toHip(bcol))
    assert_parity(oracle, sfx, o.toCpu(), oracle.matmul(x, W.T) + bcol, "col bias")


# ------------------------------------------------------------------ the benchmark configurations
def test_config1_f32_1024(hip, oracle):
    rng_a, rng_b = np.random.default_rng(1001), np.random.default_rng(1002)
    A = rng_a.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    B = rng_b.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    say("config1 f32 1024^3")
    got = (hip.toHip(A) * hip.toHip(B)).toCpu()
    assert oracle.rel_frobenius(got, oracle.matmul(A, B)) <= 1e-4
    assert oracle.rel_frobenius(got, A.astype(np.float64) @ B.astype(np.float64)) <= 1e-4


def test_config2_i32_1500_bit_exact(hip, oracle):
    A = np.random.default_rng(2001).integers(-100, 100, (1500, 1500), endpoint=True).astype(np.int32)
    B = np.random.default_rng(2002).integers(-100, 100, (1500, 1500), endpoint=True).astype(np.int32)
    say("config2 i32 1500^3")
    got = (hip.toHip(A) * hip.toHip(B)).toCpu()
    assert np.array_equal(got, oracle.matmul(A, B))


@pytest.mark.parametrize("sfx", ["i32", "i64"])
def test_config2_4096_ring_checksum(hip, oracle, sfx):
    """Full size: every one of the 4096 x 4096 outputs against the oracle's blocked gemm_strided, and, as a
    second check that shares nothing with it, a property that holds exactly in Z / 2^w:
    (A B) v == A (B v) for any v."""
    dt = DTYPES[sfx]
    n = 4096
    A = np.random.default_rng(2001).integers(-100, 100, (n, n), endpoint=True).astype(dt)
    B = np.random.default_rng(2002).integers(-100, 100, (n, n), endpoint=True).astype(dt)
    say("config2 4096^3", sfx)
    C = (hip.toHip(A) * hip.toHip(B)).toCpu()
    v = np.random.default_rng(5).integers(-2**31, 2**31 - 1, (n, 1)).astype(np.int64).view(np.uint64)
    U = lambda x: x.astype(np.int64).view(np.uint64)
    with np.errstate(over="ignore"):
        lhs = U(C) @ v
        rhs = U(A) @ (U(B) @ v)
    mask = np.uint64(0xFFFFFFFF) if sfx == "i32" else np.uint64(0xFFFFFFFFFFFFFFFF)
    assert np.array_equal(lhs & mask, rhs & mask)
    assert np.array_equal(C, oracle.matmul(A, B))            # the whole matrix


def test_i64_4096_whole_range_all_digit_pairs(hip, oracle):
    """int64 4096^3 with entries over the whole int64 range: all 36 digit pairs of the matrix-core path are
    live and every accumulator wraps many times. Whole matrix through the ring checksum, a block of rows
    against the closed form in unsigned 64-bit arithmetic (NumPy's uint64 product wraps modulo 2^64) and
    against the oracle's blocked kernel."""
    n = 4096
    info = np.iinfo(np.int64)
    A = np.random.default_rng(2011).integers(info.min, info.max, (n, n), endpoint=True).astype(np.int64)
    B = np.random.default_rng(2012).integers(info.min, info.max, (n, n), endpoint=True).astype(np.int64)
    say("i64 4096^3 whole range")
    C = (hip.toHip(A) * hip.toHip(B)).toCpu()
    U = lambda x: x.view(np.uint64)
    v = np.random.default_rng(6).integers(info.min, info.max, (n, 1)).astype(np.int64)
    with np.errstate(over="ignore"):
        assert np.array_equal(U(C) @ U(v), U(A) @ (U(B) @ U(v)))
        rows = slice(3000, 3256)
        assert np.array_equal(U(C[rows]), U(np.ascontiguousarray(A[rows])) @ U(B))
    assert np.array_equal(C[rows], oracle.matmul(np.ascontiguousarray(A[rows]), B))


def test_config3_f64_views(hip, oracle):
    """gemm(1.5, A, B, 0.5, C): A a transposed view, B every other column of a 1024 x 6144 parent."""
    pa = np.random.default_rng(3001).standard_normal((1024, 2048))
    pb = np.random.default_rng(3002).standard_normal((1024, 6144))
    C = np.random.default_rng(3003).standard_normal((2048, 3072))
    dA = hip.toHip(pa).transpose()
    dB = hip.toHip(pb)[:, ::2]
    assert dA.strides == (1, 2048) and dB.strides == (6144, 2)
    dC = hip.toHip(C)
    say("config3 f64 2048x3072x1024 views")
    hip.gemm(1.5, dA, dB, 0.5, dC)
    got = dC.toCpu()
    want = oracle.gemm_strided(1.5, pa.T, pb[:, ::2], 0.5, C.copy())
    assert oracle.rel_frobenius(got, want) <= 1e-12
    rows = np.arange(0, 2048, 64)
    wide = 1.5 * (pa.T[rows].astype(np.longdouble) @ pb[:, ::2].astype(np.longdouble)) + 0.5 * C[rows].astype(np.longdouble)
    assert oracle.rel_frobenius(got[rows], wide) <= 1e-12


def test_config5_inference_chain(hip, oracle):
    rng = np.random.default_rng(5001)
    g = lambda *s: rng.normal(0, 0.1, s).astype(np.float32)
    k1, x1 = g(20, 25), g(25, 36864)
    k2, x2 = g(50, 500), g(500, 4096)
    x3, w3, b3 = g(64, 800), g(500, 800), g(1, 500)
    w4 = g(10, 500)
    say("config5 chain")
    f64 = lambda a: a.astype(np.float64)
    o1 = (hip.toHip(k1) * hip.toHip(x1)).toCpu()
    assert oracle.rel_frobenius(o1, f64(k1) @ f64(x1)) <= 1e-4
    o2 = (hip.toHip(k2) * hip.toHip(x2)).toCpu()
    assert oracle.rel_frobenius(o2, f64(k2) @ f64(x2)) <= 1e-4
    h = hip.linear(hip.toHip(x3), hip.toHip(w3), hip.toHip(b3), relu=True)
    want_h = np.maximum(f64(x3) @ f64(w3).T + f64(b3), 0)
    assert oracle.rel_frobenius(h.toCpu(), want_h) <= 1e-4
    o4 = (h * hip.toHip(w4).transpose()).toCpu()
    assert oracle.rel_frobenius(o4, want_h @ f64(w4).T) <= 1e-4


def test_fp32_4096_properties(hip, oracle):
    """Full headline size: the whole 4096 x 4096 result against the oracle's gemm_strided (<= 1e-4 relative
    Frobenius error, the float32 bar of the path) and against the float64 product, a row block on its own, and
    linearity in alpha."""
    n = 4096
    A = np.random.default_rng(1001).uniform(-1, 1, (n, n)).astype(np.float32)
    B = np.random.default_rng(1002).uniform(-1, 1, (n, n)).astype(np.float32)
    dA, dB = hip.toHip(A), hip.toHip(B)
    say("f32 4096^3")
    C1 = (dA * dB).toCpu()
    assert oracle.rel_frobenius(C1, oracle.matmul(A, B)) <= 1e-4                          # the whole matrix
    assert oracle.rel_frobenius(C1, A.astype(np.float64) @ B.astype(np.float64)) <= 1e-4
    rows = slice(2048, 2048 + 128)
    assert oracle.rel_frobenius(C1[rows], A[rows].astype(np.float64) @ B.astype(np.float64)) <= 1e-4
    dC = hip.empty((n, n), np.float32)
    hip.gemm(2.0, dA, dB, 0.0, dC)
    assert np.array_equal(dC.toCpu(), 2.0 * C1)       # scaling by 2 is exact in binary floating point


def test_hip_graph_replays_match_eager(hip, oracle):
    """The config-5 chain recorded once into a HIP graph: every replay, with eager work and
    synchronisation between replays, must reproduce the eager result bit for bit."""
    rng = np.random.default_rng(77)
    g = lambda *s: rng.normal(0, 0.1, s).astype(np.float32)
    x3, w3, b3, w4 = g(64, 800), g(500, 800), g(1, 500), g(10, 500)
    dx, dw3, db3, dw4 = hip.toHip(x3), hip.toHip(w3), hip.toHip(b3), hip.toHip(w4)
    h, o = hip.empty((64, 500), np.float32), hip.empty((64, 10), np.float32)
    scratch = hip.empty((64, 500), np.float32)

    def chain():
        hip.gemm(1.0, dx, dw3.transpose(), 0.0, h, epilogue="bias_relu", bias=db3)
        hip.gemm(1.0, h, dw4.transpose(), 0.0, o)
        hip.apply2("add", scratch, h)          # an element-wise node in the graph as well

    hip.unary("copy", h)                       # warm the library
    scratch_np = np.zeros((64, 500), np.float32)
    dscr0 = hip.toHip(scratch_np)
    scratch.storage, scratch.layout = dscr0.storage, dscr0.layout
    chain()
    eager_o, eager_h = o.toCpu().copy(), h.toCpu().copy()
    want_h = np.maximum(x3.astype(np.float64) @ w3.T.astype(np.float64) + b3, 0)
    assert oracle.rel_frobenius(eager_h, want_h) <= 1e-4
    say("graph capture")
    with hip.Graph() as graph:
        chain()
    try:                                       # allocation while capturing comes from the allocator's cache of freed blocks
        with hip.Graph():                      # or is refused (never from the driver); after the capture it works as ever
            hip.empty((4, 4), np.float32)
    except hip.HipAllocError:
        pass
    assert hip.empty((4, 4), np.float32).shape == (4, 4)
    expect_scratch = eager_h.copy()
    for rep in range(4):
        say("graph replay", rep)
        o_before = hip.scalar_op("mul", o, 0.0)            # eager work between replays
        hip.sync()
        graph.launch()
        hip.sync()
        assert np.array_equal(o.toCpu(), eager_o) and np.array_equal(h.toCpu(), eager_h)
        expect_scratch = expect_scratch + eager_h          # scratch accumulates h once per run
        assert np.array_equal(scratch.toCpu(), expect_scratch)


SPLITK_SHAPES = [(64, 10, 500), (64, 500, 800), (50, 4096, 500), (33, 47, 2049), (128, 128, 4096), (1, 1, 1000), (7, 300, 257),
                 # k long enough for the deep split factors (up to 128 ranges of k, larger tiles than the tile count alone would
                 # pick, partials folded by four wavefronts per column group)
                 (70, 70, 70_000), (128, 96, 100_000), (200, 200, 50_000), (300, 520, 20_000)]


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("shape", SPLITK_SHAPES)
def test_small_mn_long_k_split_k(hip, oracle, sfx, shape):
    """Few output tiles and a long K: the product is cut along K over several workgroups and the
    partial sums are added in a fixed order by a second kernel. Same bars as everywhere else, and
    two runs must agree bit for bit (deterministic reduction)."""
    dt = DTYPES[sfx]
    M, N, K = shape
    rng = np.random.default_rng(seed_of("splitk", sfx, shape))
    info = None if np.dtype(dt).kind == "f" else np.iinfo(dt)
    lo, hi = (-100, 100) if info is None else (info.min, info.max)
    A, B, C = fill(rng, (M, K), dt, lo, hi), fill(rng, (K, N), dt, lo, hi), fill(rng, (M, N), dt, lo, hi)
    dA, dB = hip.toHip(A), hip.toHip(B)
    for alpha, beta in [(1, 0), (2, 3)]:
        say("split-k", sfx, shape, alpha, beta)
        want = oracle.gemm_strided(alpha, A, B, beta, C.copy())
        dC = hip.toHip(C)
        hip.gemm(alpha, dA, dB, beta, dC)
        got = dC.toCpu().copy()
        assert_parity(oracle, sfx, got, want, f"{shape} a={alpha} b={beta}")
        dC2 = hip.toHip(C)
        hip.gemm(alpha, dA, dB, beta, dC2)
        assert np.array_equal(dC2.toCpu(), got)
    # transposed operands and a column-major destination through the same path
    say("split-k views", sfx, shape)
    dCt = hip.toHip(np.zeros((N, M), dtype=dt)).transpose()
    hip.gemm(1, hip.toHip(np.ascontiguousarray(A.T)).transpose(), dB, 0, dCt)
    assert_parity(oracle, sfx, dCt.toCpu(), oracle.matmul(A, B), f"{shape} views")


@pytest.mark.parametrize("sfx", ["i32", "i64"])
@pytest.mark.parametrize("tile", ["0", "1"])
@pytest.mark.parametrize("splits", ["1", "2", "3", "5", "16"])
def test_integer_forced_split_k(hip, oracle, sfx, tile, splits, monkeypatch):
    """Integer products may cut K into any number of ranges (ring arithmetic: no bit changes). Every
    tile candidate with forced split factors on ragged shapes, wrapping values, alpha/beta and a
    strided destination."""
    monkeypatch.setenv(f"AM_HIP_GEMM_TILE_{sfx.upper()}", tile)
    monkeypatch.setenv("AM_HIP_GEMM_SPLITK", splits)
    dt = DTYPES[sfx]
    info = np.iinfo(dt)
    for shape in [(150, 130, 333), (129, 257, 40), (64, 64, 16), (300, 5, 1000)]:
        M, N, K = shape
        rng = np.random.default_rng(seed_of("forced-splitk", sfx, shape, tile, splits))
        A, B, C = fill(rng, (M, K), dt, info.min, info.max), fill(rng, (K, N), dt, info.min, info.max), fill(rng, (M, 2 * N), dt, info.min, info.max)
        say("forced split-k", sfx, tile, splits, shape)
        want = C.copy()
        oracle.gemm_strided(-3, A, B, 7, want[:, ::2])
        dC = hip.toHip(C)
        hip.gemm(-3, hip.toHip(A), hip.toHip(B), 7, dC[:, ::2])
        assert np.array_equal(dC.toCpu(), want), f"{shape} tile {tile} splits {splits}"


@pytest.mark.parametrize("sfx", ["i32", "i64"])
def test_integer_mid_size_balanced_split(hip, oracle, sfx):
    """Sizes whose tile count does not fill the CUs evenly: the library cuts K on its own."""
    dt = DTYPES[sfx]
    for shape in [(1000, 900, 1100), (640, 640, 2048), (1500, 1500, 160)]:
        M, N, K = shape
        rng = np.random.default_rng(seed_of("balanced", sfx, shape))
        A, B = fill(rng, (M, K), dt, -1000, 1000), fill(rng, (K, N), dt, -1000, 1000)
        say("balanced split-k", sfx, shape)
        dC = hip.empty((M, N), dt)
        hip.gemm(1, hip.toHip(A), hip.toHip(B), 0, dC)
        assert np.array_equal(dC.toCpu(), oracle.matmul(A, B))


@pytest.mark.parametrize("tile", ["0", "1", "2", "3"])
def test_int32_digit_sliced_matrix_core_path(hip, oracle, tile, monkeypatch):
    """int32 products on the int8 matrix cores (four balanced base-256 digits, ten digit-pair
    products, Horner recombination modulo 2^32), forced on for every shape and all four tile shapes
    (256 x 128, 256 x 256, 128 x 128, 64 x 64):
    digit boundaries (±127, ±128, ±129 in every byte position), INT_MIN / INT_MAX, full-range random
    values with long K (accumulators wrap many times), ragged M / N / K, strided and transposed
    operands, column-major and strided destinations, every alpha / beta case. Bit-exact."""
    monkeypatch.setenv("AM_HIP_GEMM_I32_PATH", "mfma")
    monkeypatch.setenv("AM_HIP_GEMM_TILE_I8", tile)
    dt = np.int32
    info = np.iinfo(dt)
    edge = np.array([0, 1, -1, 127, 128, 129, -127, -128, -129, 255, 256, -255, -256, 32767, 32768, -32768, -32769,
                     2**23 - 1, 2**23, -2**23, 2**24 + 127, 2**24 + 128, -(2**24) - 129, info.max, info.min, info.max - 128,
                     info.min + 128, 0x7F7F7F7F, -0x7F7F7F80, 0x00800080 - 2**31], dtype=np.int64).astype(dt)
    rng = np.random.default_rng(seed_of("digits", tile))
    for shape in [(30, 30, 30), (1, 1, 1), (257, 129, 300), (64, 500, 1000), (300, 257, 4099), (513, 511, 129)]:
        M, N, K = shape
        say("digit path", tile, shape)
        A = rng.choice(edge, size=(M, K)) if K <= 300 else fill(rng, (M, K), dt, info.min, info.max)
        B = rng.choice(edge, size=(K, N)) if K <= 300 else fill(rng, (K, N), dt, info.min, info.max)
        C = fill(rng, (M, N), dt, info.min, info.max)
        dA, dB = hip.toHip(A), hip.toHip(B)
        for alpha, beta in [(1, 0), (1, 1), (-3, 7), (info.min, info.max)]:
            want = oracle.gemm_strided(alpha, A, B, beta, C.copy())
            assert np.array_equal(want, oracle.closed_gemm_int_fast(alpha, A, B, beta, C)) or K > 300
            dC = hip.toHip(C)
            hip.gemm(alpha, dA, dB, beta, dC)
            assert np.array_equal(dC.toCpu(), want), f"{shape} a={alpha} b={beta}"
        # transposed / stepped operands, column-major and stepped destinations
        dAt = hip.toHip(np.ascontiguousarray(A.T)).transpose()
        B2 = fill(rng, (K, 2 * N), dt, info.min, info.max)
        dCt = hip.toHip(np.zeros((N, M), dtype=dt)).transpose()
        hip.gemm(1, dAt, hip.toHip(B2)[:, ::2], 0, dCt)
        assert np.array_equal(dCt.toCpu(), oracle.matmul(A, np.ascontiguousarray(B2[:, ::2]))), f"{shape} views"
        wide = fill(rng, (M, 2 * N), dt, info.min, info.max)
        dW = hip.toHip(wide)
        want = wide.copy()
        oracle.gemm_strided(5, A, B, -2, want[:, ::2])
        hip.gemm(5, dA, dB, -2, dW[:, ::2])
        assert np.array_equal(dW.toCpu(), want), f"{shape} stepped destination"


@pytest.mark.parametrize("sfx", ["i32", "i64"])
@pytest.mark.parametrize("tile", ["", "0", "2", "3"])
def test_prepared_digit_planes(hip, oracle, sfx, tile, monkeypatch):
    """Products whose A and / or B operand was split into digit planes ahead of time (digits_prepare): the bits of
    the plain product and of the oracle, for one-plane entries and whole-range ones, contiguous / transposed / stepped
    operands on either side, ragged extents (the planes are padded to 256 rows whatever tile the product takes),
    row- and column-major destinations (the latter exchanges the operands' roles inside the library), every alpha /
    beta case; the same planes serve several products."""
    if tile:
        monkeypatch.setenv("AM_HIP_GEMM_TILE_I8", tile)
    dt = DTYPES[sfx]
    info = np.iinfo(dt)
    rng = np.random.default_rng(seed_of("prepared", sfx, tile))
    for (M, N, K), (lo, hi) in [((70, 90, 300), (-100, 100)), ((257, 129, 700), (info.min, info.max)), ((300, 513, 260), (-40000, 40000)),
                                ((64, 64, 256), (info.min, info.max)), ((1, 5, 3), (-5, 5))]:
        say("prepared digits", sfx, tile, (M, N, K), (lo, hi))
        A, B, C = fill(rng, (M, K), dt, lo, hi), fill(rng, (K, N), dt, lo, hi), fill(rng, (M, N), dt, info.min, info.max)
        # B as a transposed view of an [N x K] buffer, A as every other row of a taller one
        A2 = np.zeros((2 * M, K), dtype=dt); A2[::2] = A
        dA, dB = hip.toHip(A2)[::2], hip.toHip(np.ascontiguousarray(B.T)).transpose()
        pa, pb = hip.digits_prepare(dA, "left"), hip.digits_prepare(dB, "right")
        for alpha, beta in [(1, 0), (-3, 7), (info.min, info.max)]:
            want = oracle.gemm_strided(alpha, A, B, beta, C.copy())
            for a_d, b_d in [(pa, None), (None, pb), (pa, pb)]:
                dC = hip.toHip(C)
                hip.gemm(alpha, dA, dB, beta, dC, a_digits=a_d, b_digits=b_d)
                assert np.array_equal(dC.toCpu(), want), f"{(M, N, K)} a={alpha} b={beta} prepared={(a_d is not None, b_d is not None)}"
        dCt = hip.toHip(np.zeros((N, M), dtype=dt)).transpose()          # column-major C: roles exchanged inside
        hip.gemm(1, dA, dB, 0, dCt, a_digits=pa, b_digits=pb)
        assert np.array_equal(dCt.toCpu(), oracle.matmul(A, B))
        dCt = hip.toHip(np.zeros((N, M), dtype=dt)).transpose()
        hip.gemm(1, dA, dB, 0, dCt, b_digits=pb)
        assert np.array_equal(dCt.toCpu(), oracle.matmul(A, B))
        # the planes of B with another left operand
        A3 = fill(rng, (33, K), dt, lo, hi)
        out = hip.empty((33, N), dt)
        hip.gemm(1, hip.toHip(A3), dB, 0, out, b_digits=pb)
        assert np.array_equal(out.toCpu(), oracle.matmul(A3, B))
        # a handle of the wrong extents or side is refused, a released one too
        with pytest.raises(ValueError):
            hip.gemm(1, hip.toHip(A3), dB, 0, out, a_digits=pa, b_digits=pb)
        with pytest.raises(ValueError):
            hip.gemm(1, dA, dB, 0, hip.empty((M, N), dt), a_digits=pb)
        stale = hip.DigitPlanes(pa.handle, 0, pa.shape, pa.dtype)
        pa.release()
        with pytest.raises(ValueError):
            hip.gemm(1, dA, dB, 0, hip.empty((M, N), dt), a_digits=stale)
        with pytest.raises(ValueError):
            stale.release()
        stale.handle = 0


def test_prepared_digit_planes_at_size_and_in_a_graph(hip, oracle):
    """2048 x 1500 x 1700 int32 with entries in [-100, 100] and over the whole range, B prepared; and both operands
    prepared inside a captured graph (nothing left to allocate), replayed twice."""
    rng = np.random.default_rng(seed_of("prepared at size"))
    for lo, hi in [(-100, 100), (-2**31, 2**31 - 1)]:
        A, B = fill(rng, (2048, 1700), np.int32, lo, hi), fill(rng, (1700, 1500), np.int32, lo, hi)
        dA, dB = hip.toHip(A), hip.toHip(B)
        pb = hip.digits_prepare(dB, "right")
        out = hip.empty((2048, 1500), np.int32)
        hip.gemm(1, dA, dB, 0, out, b_digits=pb)
        assert np.array_equal(out.toCpu(), oracle.matmul(A, B))
    A, B = fill(rng, (300, 400), np.int64, -1000, 1000), fill(rng, (400, 200), np.int64, -1000, 1000)
    dA, dB, out = hip.toHip(A), hip.toHip(B), hip.zeros((300, 200), np.int64)
    pa, pb = hip.digits_prepare(dA, "left"), hip.digits_prepare(dB, "right")
    hip.gemm(1, dA, dB, 0, out, a_digits=pa, b_digits=pb)
    with hip.Graph() as g:
        hip.gemm(1, dA, dB, 1, out, a_digits=pa, b_digits=pb)
    want = oracle.matmul(A, B)
    for rep in range(2):
        g.launch()
        hip.sync()
        assert np.array_equal(out.toCpu(), (rep + 2) * want)


def test_int32_paths_agree_at_size(hip, oracle, monkeypatch):
    """2048^3 and a ragged 1500 x 1300 x 1700 product: the automatic choice, the matrix-core path
    and the VALU path give the same bits (and those of the CPU oracle)."""
    rng = np.random.default_rng(77)
    for shape in [(2048, 2048, 2048), (1500, 1300, 1700)]:
        M, N, K = shape
        A, B = fill(rng, (M, K), np.int32, -2**31, 2**31 - 1), fill(rng, (K, N), np.int32, -2**31, 2**31 - 1)
        dA, dB = hip.toHip(A), hip.toHip(B)
        want = oracle.matmul(A, B)
        for path in (None, "mfma", "valu"):
            say("i32 paths", shape, path)
            if path is None:
                monkeypatch.delenv("AM_HIP_GEMM_I32_PATH", raising=False)
            else:
                monkeypatch.setenv("AM_HIP_GEMM_I32_PATH", path)
            assert np.array_equal((dA * dB).toCpu(), want), f"{shape} path {path}"


@pytest.mark.parametrize("tile", ["0", "2", "3"])
def test_int64_digit_sliced_matrix_core_path(hip, oracle, tile, monkeypatch):
    """int64 products on the int8 matrix cores (eight balanced base-256 digits, 36 digit-pair
    products, each pair's exact 32-bit sums widened to 64 bits before the Horner shifts), forced on
    for every shape and each of its three tile shapes (256 x 128, 128 x 128, 64 x 64): digit boundaries in every byte position, INT64_MIN / INT64_MAX, full-range
    random values, ragged M / N / K, strided and transposed operands and destinations, every
    alpha / beta case. Bit-exact."""
    monkeypatch.setenv("AM_HIP_GEMM_I64_PATH", "mfma")
    monkeypatch.setenv("AM_HIP_GEMM_TILE_I8", tile)
    dt = np.int64
    info = np.iinfo(dt)
    base = [0, 1, -1, 127, 128, 129, -127, -128, -129, 255, 256, -255, -256, 32767, 32768, -32768, -32769]
    edge = list(base) + [info.max, info.min, info.max - 128, info.min + 128, 0x7F7F7F7F7F7F7F7F, 0x7F7F7F7F7F7F7F80,
                         -0x7F7F7F7F7F7F7F80, 0x0080008000800080]
    for byte in range(1, 8):
        edge += [sgn * (v << (8 * byte)) + off for sgn in (1, -1) for v in (127, 128, 129) for off in (0, 127, -128)
                 if info.min <= sgn * (v << (8 * byte)) + off <= info.max]
    edge = np.array(edge, dtype=dt)
    rng = np.random.default_rng(seed_of("digits64", tile))
    for shape in [(30, 30, 30), (1, 1, 1), (257, 129, 300), (64, 500, 1000), (300, 257, 4099), (513, 511, 129)]:
        M, N, K = shape
        say("int64 digit path", tile, shape)
        A = rng.choice(edge, size=(M, K)) if K <= 300 else fill(rng, (M, K), dt, info.min, info.max)
        B = rng.choice(edge, size=(K, N)) if K <= 300 else fill(rng, (K, N), dt, info.min, info.max)
        C = fill(rng, (M, N), dt, info.min, info.max)
        dA, dB = hip.toHip(A), hip.toHip(B)
        for alpha, beta in [(1, 0), (1, 1), (-3, 7), (info.min, info.max)]:
            want = oracle.gemm_strided(alpha, A, B, beta, C.copy())
            assert np.array_equal(want, oracle.closed_gemm_int_fast(alpha, A, B, beta, C)) or K > 300
            dC = hip.toHip(C)
            hip.gemm(alpha, dA, dB, beta, dC)
            assert np.array_equal(dC.toCpu(), want), f"{shape} a={alpha} b={beta}"
        dAt = hip.toHip(np.ascontiguousarray(A.T)).transpose()
        B2 = fill(rng, (K, 2 * N), dt, info.min, info.max)
        dCt = hip.toHip(np.zeros((N, M), dtype=dt)).transpose()
        hip.gemm(1, dAt, hip.toHip(B2)[:, ::2], 0, dCt)
        assert np.array_equal(dCt.toCpu(), oracle.matmul(A, np.ascontiguousarray(B2[:, ::2]))), f"{shape} views"
        wide = fill(rng, (M, 2 * N), dt, info.min, info.max)
        dW = hip.toHip(wide)
        want = wide.copy()
        oracle.gemm_strided(5, A, B, -2, want[:, ::2])
        hip.gemm(5, dA, dB, -2, dW[:, ::2])
        assert np.array_equal(dW.toCpu(), want), f"{shape} stepped destination"


def test_int64_digit_path_accumulator_limit(hip, oracle, monkeypatch):
    """Every digit of every entry is -128 and k = 131071: each pair's sum over k is 131071 * 2^14, the
    largest a 32-bit accumulator can be asked to hold exactly. One k more and the product is handed to
    the VALU kernel, forced or not. Entries with few digits take the same code with most planes skipped."""
    monkeypatch.setenv("AM_HIP_GEMM_I64_PATH", "mfma")
    v = np.array([0x7F7F7F7F7F7F7F80], dtype=np.int64)[0]    # = -128 * (1 + 2^8 + ... + 2^56) modulo 2^64
    for K in (131071, 131072):
        say("int64 digit path, accumulator limit", K)
        A = np.full((64, K), v, dtype=np.int64)
        B = np.full((K, 64), v, dtype=np.int64)
        B[::7, 3] = -1
        A[5, ::3] = 127
        got = (hip.toHip(A) * hip.toHip(B)).toCpu()
        assert np.array_equal(got, oracle.matmul(A, B)), K
    rng = np.random.default_rng(seed_of("digits64-small"))
    for lo, hi in [(-100, 100), (-40000, 40000), (-2**40, 2**40)]:
        say("int64 digit path, few digits", lo, hi)
        A, B = fill(rng, (300, 700), np.int64, lo, hi), fill(rng, (700, 260), np.int64, lo, hi)
        B[:, 5] = 0
        assert np.array_equal((hip.toHip(A) * hip.toHip(B)).toCpu(), oracle.matmul(A, B)), (lo, hi)
    Z = np.zeros((128, 512), dtype=np.int64)
    C = fill(rng, (128, 128), np.int64, -9, 9)
    dC = hip.toHip(C)
    hip.gemm(3, hip.toHip(Z), hip.toHip(fill(rng, (512, 128), np.int64, -9, 9)), 2, dC)     # all planes of A empty
    assert np.array_equal(dC.toCpu(), 2 * C)


def test_int64_paths_agree_at_size(hip, oracle, monkeypatch):
    """2048 x 1024 x 2048 and a ragged 1500 x 1300 x 1700 product: the automatic choice, the
    matrix-core path and the VALU path give the same bits (and those of the CPU oracle)."""
    rng = np.random.default_rng(78)
    for shape in [(2048, 1024, 2048), (1500, 1300, 1700)]:
        M, N, K = shape
        A, B = fill(rng, (M, K), np.int64, -2**63, 2**63 - 1), fill(rng, (K, N), np.int64, -2**63, 2**63 - 1)
        dA, dB = hip.toHip(A), hip.toHip(B)
        want = oracle.matmul(A, B)
        for path in (None, "mfma", "valu"):
            say("i64 paths", shape, path)
            if path is None:
                monkeypatch.delenv("AM_HIP_GEMM_I64_PATH", raising=False)
            else:
                monkeypatch.setenv("AM_HIP_GEMM_I64_PATH", path)
            assert np.array_equal((dA * dB).toCpu(), want), f"{shape} path {path}"


@pytest.mark.parametrize("sfx", ["i32", "i64"])
def test_digit_path_window_views(hip, oracle, sfx, monkeypatch):
    """Operands that are windows of larger 16-byte aligned buffers, with extents that are not
    multiples of the 16-byte load width: the vector loads of the digit-splitting passes must stop at
    the window's edge (what lies beyond is made large so that reading it would change the result)."""
    monkeypatch.setenv(f"AM_HIP_GEMM_{sfx.upper()}_PATH", "mfma")
    dt = DTYPES[sfx]
    info = np.iinfo(dt)
    rng = np.random.default_rng(seed_of("windows", sfx))
    for (M, N, K) in [(61, 67, 131), (130, 35, 257), (33, 129, 62)]:
        say("digit path windows", sfx, (M, N, K))
        bigA = fill(rng, (M + 8, K + 24), dt, info.min, info.max)
        bigB = fill(rng, (K + 8, N + 24), dt, info.min, info.max)
        A_small = fill(rng, (M, K), dt, -100, 100)
        B_small = fill(rng, (K, N), dt, -100, 100)
        for r0, c0 in [(0, 0), (4, 8), (3, 4)]:
            hostA, hostB = bigA.copy(), bigB.copy()
            hostA[r0:r0 + M, c0:c0 + K] = A_small
            hostB[r0:r0 + K, c0:c0 + N] = B_small
            dA = hip.toHip(hostA)[r0:r0 + M, c0:c0 + K]
            dB = hip.toHip(hostB)[r0:r0 + K, c0:c0 + N]
            assert np.array_equal((dA * dB).toCpu(), oracle.matmul(A_small, B_small)), (M, N, K, r0, c0)
            # the same windows transposed: unit stride along the other direction
            dAt = hip.toHip(np.ascontiguousarray(hostA.T))[c0:c0 + K, r0:r0 + M].transpose()
            dBt = hip.toHip(np.ascontiguousarray(hostB.T))[c0:c0 + N, r0:r0 + K].transpose()
            assert np.array_equal((dAt * dBt).toCpu(), oracle.matmul(A_small, B_small)), (M, N, K, r0, c0, "T")


SMALL_SHAPES = [(1, 1, 1), (20, 36864 // 64, 25), (50, 300, 500), (64, 500, 800), (64, 10, 500), (7, 33, 15), (16, 16, 16),
                (17, 47, 17), (64, 64, 4099), (33, 200, 1000), (3, 5, 8191), (500, 10, 64), (4096, 3, 129), (300, 64, 77),
                (37, 132, 40), (9, 70, 33), (16, 1028, 16)]


@pytest.mark.parametrize("nvec", ["0", "2"])
@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_small_row_path(hip, oracle, sfx, nvec, monkeypatch):
    """Products with at most 64 rows or columns on the kernel that loads matrix-instruction operands
    straight from global memory (forced on): every k tail (K < 16, K % 16 != 0, K % 4 != 0), ragged
    M and N, one to four wavefronts per tile, both orientations, every alpha / beta case, against
    the oracle and against the tiled kernel on the same inputs. nvec: the variant for a B with unit
    stride along n (16-byte loads along n, several tiles per wavefront) switched off / forced wherever
    the operand allows it."""
    monkeypatch.setenv("AM_HIP_GEMM_SMALL_NVEC", nvec)
    dt = DTYPES[sfx]
    eps = np.finfo(dt).eps
    rng = np.random.default_rng(seed_of("small", sfx))
    for (M, N, K) in SMALL_SHAPES:
        A, B, C = fill(rng, (M, K), dt), fill(rng, (K, N), dt), fill(rng, (M, N), dt)
        dA, dB = hip.toHip(A), hip.toHip(B)
        for alpha, beta in [(1, 0), (1, 1), (-0.75, 0.5), (2, -1)]:
            say("small path", sfx, (M, N, K), alpha, beta)
            want = oracle.closed_gemm_float(alpha, A, B, beta, C).astype(dt)
            got = {}
            for mode in ("1", "0"):
                monkeypatch.setenv("AM_HIP_GEMM_SMALL", mode)
                dC = hip.toHip(C)
                hip.gemm(alpha, dA, dB, beta, dC)
                got[mode] = dC.toCpu().copy()
                assert_parity(oracle, sfx, got[mode], want, f"{(M, N, K)} a={alpha} b={beta} small={mode}")
            scale = np.abs(alpha) * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)) + np.abs(beta * C)
            assert np.all(np.abs(got["1"].astype(np.float64) - want) <= 4 * (K + 4) * eps * scale + np.finfo(dt).tiny), (M, N, K)
    monkeypatch.setenv("AM_HIP_GEMM_SMALL", "1")
    # every number of wavefronts per tile on shares of k that are whole chunks, part chunks and a tail
    for (M, N, K) in [(40, 100, 1000), (64, 64, 333), (5, 20, 40)]:
        A, B = fill(rng, (M, K), dt), fill(rng, (K, N), dt)
        want = oracle.closed_gemm_float(1, A, B, 0, None).astype(dt)
        for w in ("1", "2", "4"):
            say("small path, wavefronts per tile", sfx, (M, N, K), w)
            monkeypatch.setenv("AM_HIP_GEMM_SMALL_W", w)
            assert_parity(oracle, sfx, (hip.toHip(A) * hip.toHip(B)).toCpu(), want, f"{(M, N, K)} W={w}")
    monkeypatch.delenv("AM_HIP_GEMM_SMALL_W")
    # beta == 0 must not read C: NaN there never reaches the result
    C = np.full((20, 70), np.nan, dtype=dt)
    A, B = fill(rng, (20, 40), dt), fill(rng, (40, 70), dt)
    dC = hip.toHip(C)
    hip.gemm(1, hip.toHip(A), hip.toHip(B), 0, dC)
    assert np.isfinite(dC.toCpu()).all()


@pytest.mark.parametrize("nvec", ["0", "2"])
@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_small_row_path_views_and_epilogue(hip, oracle, sfx, nvec, monkeypatch):
    """The same kernels on transposed, stepped, reversed and broadcast operands, strided and
    column-major destinations, and with the fused bias / ReLU epilogue (row and column bias)."""
    monkeypatch.setenv("AM_HIP_GEMM_SMALL", "1")
    monkeypatch.setenv("AM_HIP_GEMM_SMALL_NVEC", nvec)
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("small-views", sfx))
    for (M, N, K) in [(64, 500, 800), (20, 300, 25), (50, 96, 500), (300, 20, 123)]:
        say("small path views", sfx, (M, N, K))
        A, B = fill(rng, (M, K), dt), fill(rng, (K, N), dt)
        want = oracle.matmul(A, B)
        dA, dB = hip.toHip(A), hip.toHip(B)
        dAt = hip.toHip(np.ascontiguousarray(A.T)).transpose()          # unit stride along m
        dBt = hip.toHip(np.ascontiguousarray(B.T)).transpose()          # unit stride along k
        for a, b, what in [(dA, dBt, "C * F"), (dAt, dB, "F * C"), (dAt, dBt, "F * F")]:
            assert_parity(oracle, sfx, (a * b).toCpu(), want, f"{(M, N, K)} {what}")
        A2, B2 = fill(rng, (2 * M, K), dt), fill(rng, (K, 2 * N), dt)
        got = (hip.toHip(A2)[::2] * hip.toHip(B2)[:, ::2]).toCpu()
        assert_parity(oracle, sfx, got, oracle.matmul(np.ascontiguousarray(A2[::2]), np.ascontiguousarray(B2[:, ::2])), "stepped")
        got = (hip.toHip(A)[::-1] * dB).toCpu()
        assert_parity(oracle, sfx, got, oracle.matmul(np.ascontiguousarray(A[::-1]), B), "reversed rows")
        row = fill(rng, (1, K), dt)
        got = (hip.toHip(row).broadcast((M, K)) * dB).toCpu()
        assert_parity(oracle, sfx, got, oracle.matmul(np.ascontiguousarray(np.broadcast_to(row, (M, K))), B), "broadcast rows")
        # destinations: column-major, and every second column of a wider buffer
        dCt = hip.toHip(np.zeros((N, M), dtype=dt)).transpose()
        hip.gemm(1, dA, dB, 0, dCt)
        assert_parity(oracle, sfx, dCt.toCpu(), want, "column-major C")
        wide = fill(rng, (M, 2 * N), dt)
        dW = hip.toHip(wide)
        ref = wide.copy()
        ref[:, ::2] = oracle.closed_gemm_float(2, A, B, 0.5, wide[:, ::2]).astype(dt)
        hip.gemm(2, dA, dB, 0.5, dW[:, ::2])
        assert_parity(oracle, sfx, dW.toCpu(), ref, "stepped C")
        assert np.array_equal(dW.toCpu()[:, 1::2], wide[:, 1::2])
        # fused epilogue
        brow, bcol = fill(rng, (1, N), dt), fill(rng, (M, 1), dt)
        for bias, epi in [(brow, "bias"), (brow, "bias_relu"), (bcol, "bias_relu"), (None, "relu")]:
            o = hip.empty((M, N), dt)
            hip.gemm(1, dA, dB, 0, o, epilogue=epi, bias=None if bias is None else hip.toHip(bias))
            ref = want + (0 if bias is None else bias)
            if "relu" in epi:
                ref = np.where(0 >= ref, 0, ref)
            assert_parity(oracle, sfx, o.toCpu(), ref.astype(dt), f"{(M, N, K)} {epi}")


@pytest.mark.parametrize("sfx", ["i32", "i64"])
def test_integer_data_dependent_path(hip, oracle, sfx, monkeypatch):
    """Both integer kernels launched behind the digit scan, the one the data rules out leaving at
    once: for every limit on the number of live digit pairs and operands with one, a few and all
    digit planes in use, with and without a split of k in the vector-ALU kernel, with beta != 0
    (a product computed twice, or by neither kernel, would show). Bit-exact."""
    monkeypatch.setenv(f"AM_HIP_GEMM_{sfx.upper()}_PATH", "spec")
    dt = DTYPES[sfx]
    info = np.iinfo(dt)
    rng = np.random.default_rng(seed_of("spec", sfx))
    M, N, K = 300, 260, 700
    C = fill(rng, (M, N), dt, -1000, 1000)
    for lo, hi in [(-100, 100), (-40000, 40000), (info.min, info.max), (0, 0)]:
        A, B = fill(rng, (M, K), dt, lo, hi), fill(rng, (K, N), dt, lo, hi)
        dA, dB = hip.toHip(A), hip.toHip(B)
        want = oracle.gemm_strided(3, A, B, -2, C.copy())
        for limit in ("0", "1", "2", "4", "9", "10", "35", "36"):
            for splitk in (None, "3"):
                say("data-dependent integer path", sfx, (lo, hi), limit, splitk)
                monkeypatch.setenv("AM_HIP_GEMM_SPEC_PAIRS", limit)
                if splitk:
                    monkeypatch.setenv("AM_HIP_GEMM_SPLITK", splitk)
                else:
                    monkeypatch.delenv("AM_HIP_GEMM_SPLITK", raising=False)
                dC = hip.toHip(C)
                hip.gemm(3, dA, dB, -2, dC)
                assert np.array_equal(dC.toCpu(), want), (lo, hi, limit, splitk)


@pytest.mark.parametrize("sfx", ["i32", "i64"])
def test_digit_path_broadcast_and_reversed_operands(hip, oracle, sfx, monkeypatch):
    """Zero and negative strides reach the digit-splitting passes as element loads: a row broadcast
    over all rows of A, B with its rows and columns reversed, and both at once."""
    monkeypatch.setenv(f"AM_HIP_GEMM_{sfx.upper()}_PATH", "mfma")
    dt = DTYPES[sfx]
    info = np.iinfo(dt)
    rng = np.random.default_rng(seed_of("digit-bcast", sfx))
    M, N, K = 70, 130, 300
    row = fill(rng, (1, K), dt, info.min, info.max)
    B = fill(rng, (K, N), dt, info.min, info.max)
    A = fill(rng, (M, K), dt, -300, 300)
    dB = hip.toHip(B)
    say("digit path, broadcast A", sfx)
    got = (hip.toHip(row).broadcast((M, K)) * dB).toCpu()
    assert np.array_equal(got, oracle.matmul(np.ascontiguousarray(np.broadcast_to(row, (M, K))), B))
    say("digit path, reversed B", sfx)
    got = (hip.toHip(A) * dB[::-1, ::-1]).toCpu()
    assert np.array_equal(got, oracle.matmul(A, np.ascontiguousarray(B[::-1, ::-1])))
    say("digit path, both", sfx)
    got = (hip.toHip(row).broadcast((M, K)) * dB[::-1, ::-1]).toCpu()
    assert np.array_equal(got, oracle.matmul(np.ascontiguousarray(np.broadcast_to(row, (M, K))), np.ascontiguousarray(B[::-1, ::-1])))


def test_random_products_all_routes(hip, oracle):
    """120 seeded random products: element type, extents from 1 to 700 (log-uniform, so that the
    small-product, tiled, split-k, VALU and digit-sliced routes all get picked by the library on its
    own), layout of A, B and C, alpha / beta. Integers bit-exact, floats within the tolerance."""
    from conftest import strided_view, view_of
    rng = np.random.default_rng(20240607)
    dest_kinds = ["C", "F", "rowstep2", "colstep2", "inner_block"]
    for case in range(120):
        sfx = ALL[case % len(ALL)]
        dt = DTYPES[sfx]
        M, N, K = (int(round(np.exp(rng.uniform(0, np.log(700))))) for _ in range(3))
        ka, kb = rng.choice(VIEW_KINDS), rng.choice(VIEW_KINDS)
        kc = rng.choice(dest_kinds)
        alpha, beta = [(1, 0), (1, 1), (2, -1), (-3, 2), (0, 1)][int(rng.integers(0, 5))]
        A, pa = strided_view(rng, (M, K), dt, ka)
        B, pb = strided_view(rng, (K, N), dt, kb)
        Cv, pc = strided_view(rng, (M, N), dt, kc)
        say("random product", case, sfx, (M, N, K), ka, kb, kc, alpha, beta)
        dA, dB = device_view(hip, pa, ka, (M, K)), device_view(hip, pb, kb, (K, N))
        dC = device_view(hip, pc, kc, (M, N))
        hip.gemm(alpha, dA, dB, beta, dC)
        oracle.gemm_strided(alpha, A, B, beta, Cv)          # through the NumPy view into `pc`
        after = hip.HipTensor(hip.Layout(pc.shape, tuple(st // pc.itemsize for st in pc.strides), 0), dC.storage, dC.dtype).toCpu()
        assert_parity(oracle, sfx, view_of(after, kc, (M, N)), Cv, f"case {case}: {sfx} {(M, N, K)} {ka} {kb} {kc} a={alpha} b={beta}")
