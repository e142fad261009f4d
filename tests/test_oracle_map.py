"""Pins the CPU oracle's strided map / apply restatement (oracle/strided_map.c) — CPU only.

Anchors: the reference's literal vectors (test_broadcasting.nim, test_operators_blas*.nim,
test_higherorder.nim) and NumPy's own broadcasting / strided views (each element is one IEEE or
ring operation, so the comparison is bit-exact)."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from conftest import DTYPES, seed_of

INT = ["i32", "i64"]
FLT = ["f32", "f64"]


def _kinds(kind):
    return {"int": INT, "float": FLT, "any": INT + FLT, "float64_only": ["f64"]}[kind]


def test_reference_elementwise_vectors(vectors, oracle):
    for case in vectors["elementwise"]:
        for sfx in _kinds(case["kind"]):
            dt = DTYPES[sfx]
            a, b = np.array(case["a"], dtype=dt), np.array(case["b"], dtype=dt)
            ba, bb = oracle.broadcast2(a, b)
            got = oracle.map2(case["op"], ba, bb)
            assert np.array_equal(got, np.array(case["expect"], dtype=dt)), (case["name"], sfx)


def test_reference_explicit_broadcast(vectors, oracle):
    for case in vectors["explicit_broadcast"]:
        t = np.array(case["t"], dtype=np.int64)
        got = oracle.unary("copy", oracle.broadcast(t, case["shape"]))
        assert np.array_equal(got, np.array(case["expect"]))


def test_reference_inplace_broadcast(vectors, oracle):
    for case in vectors["inplace_broadcast"]:
        for sfx in _kinds(case["kind"]):
            dt = DTYPES[sfx]
            a, b = np.array(case["a"], dtype=dt), np.array(case["b"], dtype=dt)
            oracle.map2(case["op"], a, oracle.broadcast(b, a.shape), out=a)   # apply2: dst is a
            assert np.array_equal(a, np.array(case["expect"], dtype=dt)), (case["source"], sfx)


def test_reference_scalar_chains(vectors, oracle):
    for case in vectors["scalar_chains"]:
        for sfx in _kinds(case["kind"]):
            dt = DTYPES[sfx]
            t = np.array(case["a"], dtype=dt)
            for op, s, side in case["steps"]:
                t = oracle.scalar_op(op, t, s, scalar_on_left=(side == "left"))
            assert np.array_equal(t, np.array(case["expect"], dtype=dt)), (case["source"], sfx)


def test_reference_sigmoid_chain(vectors, oracle):
    c = vectors["sigmoid_chain"]
    t = np.array(c["t"], dtype=np.float32)
    # 1 /. (1 +. exp(0 -. t))
    e = oracle.unary("exp", oracle.scalar_op("sub", t, 0.0, scalar_on_left=True))
    got = oracle.scalar_op("div", oracle.scalar_op("add", e, 1.0, scalar_on_left=True), 1.0, scalar_on_left=True)
    assert np.array_equal(got, np.array(c["expect"], dtype=np.float32))
    assert np.array_equal(oracle.unary("sigmoid", t), np.array(c["expect"], dtype=np.float32))


def test_reference_sliced_add_sub(vectors, oracle):
    c = vectors["sliced_add_sub"]
    a = np.array(c["a"], dtype=np.float64)
    for case in c["cases"]:
        (r0, r1, _), (c0, c1, _) = case["slice"]
        got = oracle.map2(case["op"], a[r0:r1 + 1, c0:c1 + 1], a.T[r0:r1 + 1, c0:c1 + 1])
        assert np.array_equal(got, np.array(case["expect"], dtype=np.float64))


def test_reference_inplace_on_transposed(vectors, oracle):
    c = vectors["inplace_on_transposed"]
    t = np.array(c["vandermonde"], dtype=np.float32)
    z = t.copy().T                   # a transposed (column-major) view of its own buffer
    assert not z.flags["C_CONTIGUOUS"]
    oracle.map2("add", z, z, out=z)
    assert np.array_equal(z, np.array(c["after_z_plus_z"], dtype=np.float32))
    oracle.map2("add", z, t, out=z)
    assert np.array_equal(z, np.array(c["after_plus_t2"], dtype=np.float32))


def test_reference_map2_bool(vectors, oracle):
    c = vectors["map2_bool"]
    a, b = np.array(c["a"], dtype=np.int64), np.array(c["b"], dtype=np.int64)
    m = oracle.map2("mod", a, b)
    assert np.array_equal(m, np.array(c["expect_mod"]))
    assert np.array_equal(m == 0, np.array(c["expect"]))
    got = oracle.compare("mod_is_zero", a, b)      # the whole body, with its bool result
    assert got.dtype == np.bool_ and np.array_equal(got, np.array(c["expect"]))


_NP_CMP = {"==": np.equal, "!=": np.not_equal, "<": np.less, "<=": np.less_equal, ">": np.greater, ">=": np.greater_equal}


def test_reference_comparison_vectors(vectors, oracle):
    c = vectors["comparison"]
    for dt in (np.int32, np.int64, np.float32, np.float64):
        a, b = np.array(c["a"], dtype=dt), np.array(c["b"], dtype=dt)
        for case in c["tensor_tensor"]:
            assert np.array_equal(oracle.compare(case["cmp"], a, b), np.array(case["expect"]))
        for case in c["tensor_scalar"]:
            cmp = {"<=": ">=", ">=": "<=", "<": ">", ">": "<"}.get(case["cmp"], case["cmp"]) if case["scalar_on_left"] else case["cmp"]
            assert np.array_equal(oracle.compare(cmp, a, case["scalar"]), np.array(case["expect"]))


@pytest.mark.parametrize("dt", [np.int32, np.int64, np.float32, np.float64])
def test_comparisons_against_numpy_on_strided_operands(oracle, dt):
    """Each output element is one comparison: NumPy's broadcasting comparison fixes it, NaN included."""
    rng = np.random.default_rng(seed_of("cmp", str(dt)))
    a = rng.integers(-3, 3, (7, 1, 5)).astype(dt)
    b = rng.integers(-3, 3, (1, 6, 5)).astype(dt)
    if np.dtype(dt).kind == "f":
        a[0, 0, :3] = [np.nan, np.inf, -0.0]
        b[0, :3, 0] = [np.nan, 0.0, np.inf]
    ba, bb = oracle.broadcast2(a, b)
    for cmp, f in _NP_CMP.items():
        with np.errstate(invalid="ignore"):
            assert np.array_equal(oracle.compare(cmp, ba, bb), f(a, b)), cmp
            assert np.array_equal(oracle.compare(cmp, ba[::-1].transpose(2, 0, 1), bb[::-1].transpose(2, 0, 1)),
                                  f(a, b)[::-1].transpose(2, 0, 1)), cmp
            assert np.array_equal(oracle.compare(cmp, ba, 1), f(a, dt(1)) & np.ones(ba.shape, bool)), cmp


def test_reference_math_function_vectors(vectors, oracle):
    m = vectors["math_functions"]
    for dt in (np.float32, np.float64):
        s = m["sgn"]
        assert np.array_equal(oracle.sgn(np.array(s["a"], dtype=dt)), np.array(s["expect"], dtype=np.int64))
        cs = m["copysign"]
        got = oracle.map2("copysign", np.array(cs["a"], dtype=dt), np.array(cs["signs"], dtype=dt))
        want = np.array(cs["expect"], dtype=dt)
        assert np.array_equal(got, want) and np.array_equal(np.signbit(got), np.signbit(want))
        c = m["classify"]
        x = np.array([float(v) for v in c["a"]], dtype=dt)
        assert np.array_equal(oracle.predicate("isnan", x), np.array(c["isnan"]))
        assert np.array_equal(oracle.predicate("isnotnan", x), ~np.array(c["isnan"]))
        names = ("fcNormal", "fcSubnormal", "fcZero", "fcNegZero", "fcNan", "fcInf", "fcNegInf")
        assert [names[k] for k in oracle.predicate("classify", x)] == c["classes"]
        tiny = np.finfo(dt).tiny
        assert oracle.predicate("classify", np.array([tiny, tiny / 2, -tiny / 4, 1.0, -3.5], dtype=dt)).tolist() == [0, 1, 1, 0, 0]
    for dt in (np.int32, np.int64):
        assert oracle.sgn(np.array([-7, 0, 9, np.iinfo(dt).min], dtype=dt)).tolist() == [-1, 0, 1, -1]
        mm = m["minmax"]
        a, b = np.array(mm["a"], dtype=dt), np.array(mm["b"], dtype=dt)
        assert oracle.map2("min", a, b).tolist() == mm["min"] and oracle.map2("max", a, b).tolist() == mm["max"]
    f = m["floormod"]
    a = np.array([f["start"] + i * f["step"] for i in range(f["count"])])       # arange(-70.7, 50.0, 34.7)
    ts, st = oracle.scalar_op("floormod", a, 3.0), oracle.scalar_op("floormod", a, 3.0, scalar_on_left=True)
    assert np.mean(np.abs(ts - np.array(f["tensor_scalar_3"]))) < 1e-9 and np.signbit(ts[1])
    assert np.mean(np.abs(st - np.array(f["scalar_3_tensor"]))) < 1e-9


@pytest.mark.parametrize("dt", [np.int32, np.int64, np.float64])
def test_floormod_is_python_modulo(oracle, dt):
    """floorMod's result takes the divisor's sign: for integers it is Python's %, for floats np.mod
    wherever that is exact (it is np.fmod moved by one divisor)."""
    rng = np.random.default_rng(seed_of("floormod", str(dt)))
    a = rng.integers(-50, 50, 400).astype(dt)
    b = rng.integers(-9, 9, 400).astype(dt)
    b[b == 0] = 4
    got = oracle.map2("floormod", a, b)
    assert np.array_equal(got, np.array([int(x) % int(y) for x, y in zip(a, b)], dtype=dt))


def test_deg_rad_conversions(oracle):
    for dt in (np.float32, np.float64):
        x = np.array([0, 30, 45, 90, 180, -360, 1e-3], dtype=dt)
        r = oracle.unary("degtorad", x)
        np.testing.assert_allclose(r, np.deg2rad(x.astype(np.float64)), rtol=4 * np.finfo(dt).eps)
        np.testing.assert_allclose(oracle.unary("radtodeg", r), x, rtol=4 * np.finfo(dt).eps)
    assert oracle.unary("degtorad", np.array([180.0]))[0] == np.pi


def test_int_division_truncates_toward_zero(oracle):
    a = np.array([7, -7, 7, -7, 0, 5, -2**31], dtype=np.int32)
    b = np.array([2, 2, -2, -2, 3, 0, -1], dtype=np.int32)
    assert oracle.map2("div", a, b).tolist() == [3, -3, -3, 3, 0, 0, -2**31]
    assert oracle.map2("mod", a, b).tolist() == [1, -1, 1, -1, 0, 0, 0]
    assert np.array_equal(oracle.closed_map2("div", a, b), oracle.map2("div", a, b))
    assert np.array_equal(oracle.closed_map2("mod", a, b), oracle.map2("mod", a, b))


def test_relu_forms(oracle):
    x = np.array([-1.0, -0.0, 0.0, 2.5, np.nan, -np.inf, np.inf], dtype=np.float32)
    r = oracle.unary("relu", x)
    assert r[:4].tolist() == [0.0, 0.0, 0.0, 2.5] and not np.signbit(r[1])
    assert np.isnan(r[4]) and r[5] == 0 and r[6] == np.inf
    b = np.zeros_like(x)
    assert np.array_equal(oracle.map2("add_relu", x, b), r, equal_nan=True)


# ---- random shapes and strides against NumPy (hypothesis) ---------------------------------
@st.composite
def strided_pair(draw):
    rank = draw(st.integers(1, 6))
    shape = tuple(draw(st.integers(1, 5)) for _ in range(rank))
    views = []
    for _ in range(2):
        # parent twice as large in every axis; random start / step sign / broadcast per axis
        key, bcast = [], []
        for n in shape:
            mode = draw(st.sampled_from(["full", "step2", "rev", "bcast"]))
            bcast.append(mode == "bcast")
            key.append({"full": slice(0, n), "step2": slice(0, 2 * n, 2), "rev": slice(n - 1, None, -1),
                        "bcast": slice(0, 1)}[mode])
        perm = draw(st.permutations(range(rank)))
        views.append((tuple(key), tuple(bcast), tuple(perm)))
    return shape, views


def _make(rng, shape, dt, spec):
    key, bcast, perm = spec
    pshape = tuple(2 * n for n in shape)
    # build the parent in a permuted memory order so that inner strides are not always unit
    parent = np.empty([pshape[p] for p in perm], dtype=dt)
    if np.dtype(dt).kind == "f":
        parent[...] = rng.uniform(-4, 4, parent.shape)
    else:
        parent[...] = rng.integers(-50, 50, parent.shape)
    parent = parent.transpose(np.argsort(perm))
    v = parent[key]
    tgt = tuple(shape)
    strides = tuple(0 if b else s for b, s in zip(bcast, v.strides))
    return np.lib.stride_tricks.as_strided(v, shape=tgt, strides=strides, writeable=False)


@settings(max_examples=120, deadline=None)
@given(strided_pair(), st.sampled_from(["f32", "f64", "i32", "i64"]),
       st.sampled_from(["add", "sub", "mul", "div", "add_relu", "relu_bwd", "max", "min", "sigmoid_bwd", "tanh_bwd", "sqdiff"]),
       st.integers(0, 2**31))
def test_random_strides_match_numpy(oracle, spec, sfx, op, seed):
    shape, views = spec
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed)
    a, b = _make(rng, shape, dt, views[0]), _make(rng, shape, dt, views[1])
    got = oracle.map2(op, a, b)
    want = oracle.closed_map2(op, a, b)
    assert got.dtype == want.dtype and np.array_equal(got, want, equal_nan=True)


def test_block_split_large(oracle):
    """n >= 1000 takes the multi-block path of omp_parallel_blocks; result must not depend on it."""
    rng = np.random.default_rng(1)
    a = rng.uniform(-1, 1, (257, 129)).astype(np.float32)
    b = rng.uniform(-1, 1, (1, 129)).astype(np.float32)
    s = rng.uniform(-1, 1, (257, 1)).astype(np.float32)
    ba, bb = oracle.broadcast2(a, b)
    y = oracle.map2("add", ba, bb)
    assert np.array_equal(y, a + b)
    by, bs = oracle.broadcast2(y, s)
    assert np.array_equal(oracle.map2("mul", by, bs), y * s)
    assert np.array_equal(oracle.map2("add_relu", ba, bb), np.maximum(a + b, 0))


def test_transcendental_bodies_close_to_numpy(oracle):
    rng = np.random.default_rng(2)
    for dt, tol in ((np.float32, 2e-6), (np.float64, 1e-14)):
        a = rng.uniform(-3, 3, (33, 17)).astype(dt)
        b = rng.uniform(-3, 3, (33, 17)).astype(dt)
        np.testing.assert_allclose(oracle.map2("add_sigmoid", a, b), 1 / (1 + np.exp(-(a + b).astype(np.float64))), rtol=tol)
        np.testing.assert_allclose(oracle.map2("add_tanh", a, b), np.tanh((a + b).astype(np.float64)), rtol=tol, atol=tol)


def test_sqrt_and_square_bodies(oracle):
    """sqrt is one correctly rounded IEEE operation, square one multiplication (wrapping for
    integers): NumPy computes the same bits."""
    rng = np.random.default_rng(4)
    for dt in (np.float32, np.float64):
        x = rng.uniform(0, 1e6, (33, 17)).astype(dt)
        assert np.array_equal(oracle.unary("sqrt", x), np.sqrt(x))
        assert np.array_equal(oracle.unary("square", x.T), (x * x).T)
    for dt in (np.int32, np.int64):
        info = np.iinfo(dt)
        x = rng.integers(info.min, info.max, (9, 31), endpoint=True).astype(dt)
        assert np.array_equal(oracle.unary("square", x), x * x)
        with pytest.raises(ValueError):
            oracle.unary("sqrt", x)


def test_broadcast_errors(oracle):
    with pytest.raises(ValueError):
        oracle.broadcast2(np.zeros((3, 2)), np.zeros((2, 2)))
    with pytest.raises(ValueError):
        oracle.broadcast(np.zeros((3, 2)), (3, 3))


def test_float_mod_is_fmod(oracle):
    """`mod` on float tensors is Nim's std/math `mod`, C fmod: an exact operation (no rounding), result
    with the dividend's sign. Pinned on NumPy's fmod, on the exact identity x = trunc(x / y) * y + r for
    small integer-valued operands, and on the special values."""
    rng = np.random.default_rng(21)
    for dt in (np.float32, np.float64):
        x = (rng.uniform(-1e4, 1e4, (17, 33)) * 10.0 ** rng.integers(-3, 4, (17, 33))).astype(dt)
        y = rng.uniform(-50, 50, (17, 33)).astype(dt)
        assert np.array_equal(oracle.map2("mod", x, y), np.fmod(x, y))
        assert np.array_equal(oracle.scalar_op("mod", x, 3.5), np.fmod(x, dt(3.5)))
        assert np.array_equal(oracle.scalar_op("mod", y, 3.5, scalar_on_left=True), np.fmod(dt(3.5), y))
        xi, yi = rng.integers(-1000, 1000, 500).astype(dt), rng.integers(1, 40, 500).astype(dt)
        r = oracle.map2("mod", xi, yi)
        assert np.array_equal(np.trunc(xi / yi) * yi + r, xi) and np.all(np.abs(r) < yi)
        with np.errstate(invalid="ignore"):
            sp = oracle.map2("mod", np.array([5.5, -5.5, 1.0, np.inf, -0.0], dtype=dt), np.array([2.0, 2.0, 0.0, 2.0, 3.0], dtype=dt))
        assert sp[0] == 1.5 and sp[1] == -1.5 and np.isnan(sp[2]) and np.isnan(sp[3]) and sp[4] == 0 and np.signbit(sp[4])


def test_map3_bodies_match_numpy(oracle):
    """x*y+z and (1-y)*z+y*x are sequences of separately rounded IEEE operations: NumPy evaluates the
    same sequence, so the comparison is bit-exact; tanh(x+y*z) is checked to libm accuracy."""
    rng = np.random.default_rng(9)
    for dt in (np.float32, np.float64):
        base = rng.uniform(-2, 2, (3, 40, 48)).astype(dt)
        x, y, z = base[0][:, 0:16], base[1][:, 16:32], base[2].T[8:24].T   # column slices, like the GRU gates
        assert np.array_equal(oracle.map3("muladd", x, y, z), x * y + z)
        assert np.array_equal(oracle.map3("addmul", x, y, z), (x + y) * z)
        assert np.array_equal(oracle.map3("gru_blend", x, y, z), (dt(1) - y) * z + y * x)
        np.testing.assert_allclose(oracle.map3("gru_candidate", x, y, z), np.tanh((x + y * z).astype(np.float64)),
                                   rtol=2e-6 if dt == np.float32 else 1e-14, atol=1e-7 if dt == np.float32 else 1e-15)
        # apply3: destination is the first operand, written through its own strides
        dst = base[0].copy()
        want = dst.copy(); want[:, 0:16] = want[:, 0:16] * y + z
        oracle.map3("muladd", dst[:, 0:16], y, z, out=dst[:, 0:16])
        assert np.array_equal(dst, want)
    a = np.array([2**31 - 1, -5, 7], dtype=np.int32)
    assert oracle.map3("muladd", a, a, a).tolist() == [(((2**31 - 1) ** 2 + 2**31 - 1 + 2**31) % 2**32) - 2**31, 20, 56]
    assert oracle.map3("addmul", a, a, a).tolist() == [(((2**32 - 2) * (2**31 - 1)) % 2**32 + 2**31) % 2**32 - 2**31, 50, 98]
    with pytest.raises(ValueError):
        oracle.map3("gru_blend", a, a, a)


def test_reference_conv_vectors(vectors, oracle):
    """im2col + GEMM + bias against the reference's convolution literals
    (tests/nn_primitives/test_nnp_convolution.nim:21-134)."""
    for case in vectors["conv_im2col"]:
        for dt in (np.float32, np.int64, np.float64, np.int32):
            x = np.array(case["input"], dtype=dt)
            k = np.array(case["kernel"], dtype=dt)
            b = np.array(case["bias"], dtype=dt)
            got = oracle.conv2d(x, k, b, tuple(case["padding"]), tuple(case["stride"]))
            assert np.array_equal(got, np.array(case["target"], dtype=dt)), case["name"]


def _conv_direct(x, k, pad, st):
    """Cross-correlation straight from its definition (no column matrix), in the operands' own type."""
    N, C, H, W = x.shape
    co, _, kh, kw = k.shape
    ho, wo = (H + 2 * pad[0] - kh) // st[0] + 1, (W + 2 * pad[1] - kw) // st[1] + 1
    xp = np.zeros((N, C, H + 2 * pad[0], W + 2 * pad[1]), dtype=x.dtype)
    xp[:, :, pad[0]:pad[0] + H, pad[1]:pad[1] + W] = x
    y = np.zeros((N, co, ho, wo), dtype=x.dtype)
    for h in range(ho):
        for w in range(wo):
            patch = xp[:, :, h * st[0]:h * st[0] + kh, w * st[1]:w * st[1] + kw]
            y[:, :, h, w] = np.einsum("ncij,ocij->no", patch, k)
    return y


_BWD_GEOMS = [((2, 3, 4, 5), (2, 3, 3, 3), (1, 1), (1, 1)),      # the reference's own backward case (test_nnp_convolution.nim:137-168)
              ((2, 3, 5, 5), (2, 3, 3, 3), (1, 1), (2, 2)),
              ((3, 2, 7, 6), (4, 2, 3, 2), (0, 2), (2, 1)),
              ((1, 1, 6, 9), (3, 1, 2, 4), (2, 0), (1, 3)),
              ((2, 4, 5, 5), (1, 4, 5, 5), (0, 0), (1, 1))]


@pytest.mark.parametrize("geom", _BWD_GEOMS)
def test_conv_backward_against_numerical_gradient_and_adjoints(oracle, geom):
    """conv2d_backward the way the reference checks it (tests/nn_primitives/test_nnp_convolution.nim:137-168):
    against central differences of the pinned forward pass, in float64. The convolution is linear in each argument,
    so the differences are exact up to rounding. Beside that, with a random grad_output instead of ones: the two
    adjoint identities <conv(x, k), g> = <x, grad_input> = <k, grad_weight>, which no transposed or shifted index
    survives, with the forward pass taken from the definition rather than from the column matrix."""
    xs, ks, pad, st = geom
    rng = np.random.default_rng(seed_of("conv-bwd-oracle", geom))
    x, k, b = rng.uniform(-1, 1, xs), rng.uniform(-1, 1, ks), rng.uniform(-1, 1, (ks[0], 1, 1))
    y = oracle.conv2d(x, k, b, pad, st)
    assert np.allclose(y, _conv_direct(x, k, pad, st) + b.reshape(1, -1, 1, 1), rtol=0, atol=1e-13)
    ones = np.ones_like(y)
    gi, gw, gb = oracle.conv2d_backward(x, k, b, pad, st, ones)

    def numerical(arr, f, h=1e-3):
        g = np.zeros_like(arr)
        flat, gf = arr.reshape(-1), g.reshape(-1)
        for i in range(flat.size):
            keep = flat[i]
            flat[i] = keep + h; up = f()
            flat[i] = keep - h; dn = f()
            flat[i] = keep
            gf[i] = (up - dn) / (2 * h)
        return g

    total = lambda: oracle.conv2d(x, k, b, pad, st).sum()
    for got, arr in ((gi, x), (gw, k), (gb, b)):
        want = numerical(arr, total)
        assert np.mean(np.abs(got - want) / (np.abs(want) + 1e-30)) < 1e-6 or np.max(np.abs(got - want)) < 1e-9
    for trial in range(3):
        g = rng.uniform(-1, 1, y.shape)
        gi, gw, gb = oracle.conv2d_backward(x, k, b, pad, st, g)
        lhs = np.sum(_conv_direct(x, k, pad, st) * g)
        assert abs(lhs - np.sum(x * gi)) <= 1e-12 * max(1.0, abs(lhs))
        assert abs(lhs - np.sum(k * gw)) <= 1e-12 * max(1.0, abs(lhs))
        assert np.allclose(gb.reshape(-1), g.sum((0, 2, 3)), rtol=0, atol=1e-13)
        # every entry, not one inner product: grad_input[n, c, y, x] = <conv(e_ncyx, k), g>, grad_weight likewise
        e = np.zeros_like(x)
        for idx in [tuple(rng.integers(0, s) for s in xs) for _ in range(6)]:
            e[idx] = 1.0
            assert abs(np.sum(_conv_direct(e, k, pad, st) * g) - gi[idx]) <= 1e-12
            e[idx] = 0.0
        e = np.zeros_like(k)
        for idx in [tuple(rng.integers(0, s) for s in ks) for _ in range(6)]:
            e[idx] = 1.0
            assert abs(np.sum(_conv_direct(x, e, pad, st) * g) - gw[idx]) <= 1e-12
            e[idx] = 0.0


def test_col2im_is_the_adjoint_of_im2col_and_wraps(oracle):
    """col2im sums the entries im2col would have read from a pixel: <im2col(x), c> = <x, col2im(c)> exactly on
    integers (wrapping ones included), and col2im(im2col(ones)) counts the patches that cover each pixel."""
    rng = np.random.default_rng(seed_of("col2im-oracle"))
    for (C, H, W, kh, kw, pad, st) in [(2, 5, 6, 3, 3, (1, 1), (1, 1)), (1, 7, 4, 2, 3, (0, 2), (2, 1)), (3, 4, 4, 4, 4, (0, 0), (1, 1)),
                                       (2, 6, 6, 3, 3, (2, 2), (3, 2))]:
        x = rng.integers(-50, 50, (C, H, W)).astype(np.int64)
        col = oracle.im2col(x, (kh, kw), pad, st)
        c = rng.integers(-50, 50, col.shape).astype(np.int64)
        back = oracle.col2im(c, C, H, W, (kh, kw), pad, st)
        assert int(np.sum(col * c)) == int(np.sum(x * back))
        cover = oracle.col2im(oracle.im2col(np.ones_like(x), (kh, kw), pad, st), C, H, W, (kh, kw), pad, st)
        hc, wc = (H + 2 * pad[0] - kh) // st[0] + 1, (W + 2 * pad[1] - kw) // st[1] + 1
        brute = np.zeros((H, W), dtype=np.int64)
        for h in range(hc):
            for w in range(wc):
                for i in range(kh):
                    for j in range(kw):
                        r, q = h * st[0] + i - pad[0], w * st[1] + j - pad[1]
                        if 0 <= r < H and 0 <= q < W:
                            brute[r, q] += 1
        assert np.array_equal(cover, np.broadcast_to(brute, (C, H, W)))
    big = np.full((4, 4), 2**31 - 1, dtype=np.int32)         # a pixel covered by four patches: 4 * INT_MAX wraps to -4
    assert oracle.col2im(big, 1, 3, 3, (2, 2), (0, 0), (1, 1))[0, 1, 1] == np.int32(-4)


_UFUNC_NUMPY = dict(ln=np.log, log10=np.log10, log2=np.log2, sin=np.sin, cos=np.cos, tan=np.tan, sinh=np.sinh,
                    cosh=np.cosh, arcsin=np.arcsin, arccos=np.arccos, arctan=np.arctan, arcsinh=np.arcsinh,
                    arccosh=np.arccosh, arctanh=np.arctanh, cbrt=np.cbrt, floor=np.floor, ceil=np.ceil,
                    trunc=np.trunc)
_UFUNC_DOMAIN = dict(ln=(1e-3, 1e3), log10=(1e-3, 1e3), log2=(1e-3, 1e3), arcsin=(-1, 1), arccos=(-1, 1),
                     arccosh=(1, 50), arctanh=(-0.999, 0.999), sinh=(-20, 20), cosh=(-20, 20))


def test_reference_pow_and_ufunc_vectors(vectors, oracle):
    """`^.` / `^.=`, reciprocal, cos and ln on the reference's own literals. The reference compares
    pow with ==: so does this test (the host's pow is correctly rounded on these inputs)."""
    v = vectors["pow_and_ufunc"]
    a = np.array(v["a"])
    assert np.array_equal(oracle.scalar_op("pow", a, 2.0), np.array(v["pow_2"]))
    quot = np.array([[n / q] for n, q in v["pow_m1_as_quotients"]])
    assert np.array_equal(oracle.scalar_op("pow", a, -1.0), quot)
    assert np.array_equal(oracle.unary("reciprocal", a), quot)
    assert np.array_equal(oracle.scalar_op("pow", a, 2.0, scalar_on_left=True), np.array(v["two_pow_a"]))
    inplace = a.copy()
    oracle.scalar_op("pow", inplace, 2.0, out=inplace)
    assert np.array_equal(inplace, np.array(v["pow_2"]))
    import math
    c, l = np.array(v["cos_input"]), np.array(v["ln_input"])
    assert np.abs(oracle.unary("cos", c) - np.vectorize(math.cos)(c)).mean() <= 1e-15
    assert np.array_equal(oracle.unary("ln", l), np.vectorize(math.log)(l))


def test_ufunc_bodies_against_numpy_and_closed_forms(oracle):
    """Every universal function is the host libm's function of that name. Pinned against NumPy's own
    evaluation (2 units in the last place: NumPy may use its SIMD routines), against Python's math
    module for the ones NumPy lacks, and against closed forms a wrong function name would break."""
    import math
    rng = np.random.default_rng(11)
    for dt, ulp in ((np.float32, 2 ** -23), (np.float64, 2 ** -52)):
        for name, fn in _UFUNC_NUMPY.items():
            lo, hi = _UFUNC_DOMAIN.get(name, (-8, 8))
            x = rng.uniform(lo, hi, (13, 29)).astype(dt)
            got, want = oracle.unary(name, x.T), fn(x.T)
            assert got.dtype == dt
            if name in ("floor", "ceil", "trunc"):
                assert np.array_equal(got, want), name
            else:
                assert np.all(np.abs(got - want) <= 2 * ulp * np.maximum(np.abs(want), np.finfo(dt).tiny)), (name, dt)
        x = rng.uniform(-3, 3, 200).astype(dt)
        for name, fn in (("erf", math.erf), ("erfc", math.erfc), ("gamma", math.gamma), ("lgamma", math.lgamma)):
            want = np.array([fn(float(v)) for v in x])
            np.testing.assert_allclose(oracle.unary(name, x), want, rtol=8 * ulp, atol=8 * ulp, err_msg=name)
        # closed forms
        halves = np.array([-2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 0.49999997, -0.0, 3.0], dtype=dt)
        assert np.array_equal(oracle.unary("round", halves), np.array([-3, -2, -1, 1, 2, 3, 0, -0.0, 3], dtype=dt))
        assert np.signbit(oracle.unary("round", np.array([-0.25], dtype=dt)))[0]
        ints = np.arange(1, 11, dtype=dt)
        np.testing.assert_allclose(oracle.unary("gamma", ints), [math.factorial(int(i) - 1) for i in ints], rtol=2 * ulp)
        np.testing.assert_allclose(oracle.unary("cbrt", ints ** 3), ints, rtol=2 * ulp)
        assert np.array_equal(oracle.unary("log2", 2.0 ** ints), ints)
        assert np.array_equal(oracle.unary("reciprocal", x), dt(1) / x)
        np.testing.assert_allclose(oracle.unary("erf", x) + oracle.unary("erfc", x), 1, rtol=4 * ulp)
        s, c = oracle.unary("sin", x), oracle.unary("cos", x)
        np.testing.assert_allclose(s * s + c * c, 1, rtol=8 * ulp)
        # pow: tensor-tensor, both scalar sides; exact where the result is representable
        y = rng.uniform(-3, 3, x.shape).astype(dt)
        b = np.abs(x) + dt(0.5)
        want = np.power(b, y)
        assert np.all(np.abs(oracle.map2("pow", b, y) - want) <= 2 * ulp * np.abs(want))
        assert np.array_equal(oracle.scalar_op("pow", ints, 2), ints * ints)
        assert np.array_equal(oracle.scalar_op("pow", ints, 2, scalar_on_left=True), 2.0 ** ints)
    for dt in (np.int32, np.int64):
        with pytest.raises(ValueError):
            oracle.unary("ln", np.arange(4, dtype=dt))
        with pytest.raises(ValueError):
            oracle.map2("pow", np.arange(4, dtype=dt), np.arange(4, dtype=dt))


def test_clamp_body(oracle):
    """clamp(x, min, max) = min where x < min, max where x > max, else x (math_functions.nim:146-152; the
    comparisons of Nim's clamp): NumPy's clip computes the same on non-NaN input; a NaN stays a NaN."""
    rng = np.random.default_rng(31)
    for dt in (np.float32, np.float64, np.int32, np.int64):
        x = (rng.uniform(-100, 100, (19, 23))).astype(dt)
        lo, hi = np.broadcast_to(dt(-25), x.shape), np.broadcast_to(dt(40), x.shape)
        assert np.array_equal(oracle.map3("clamp", x.T, lo.T, hi.T), np.clip(x, -25, 40).T)
    x = np.array([np.nan, -np.inf, np.inf, -0.0, 5.0])
    got = oracle.map3("clamp", x, np.broadcast_to(0.0, x.shape), np.broadcast_to(1.0, x.shape))
    assert np.isnan(got[0]) and got[1] == 0 and got[2] == 1 and got[3] == 0 and np.signbit(got[3]) and got[4] == 1


def test_fac_is_the_factorial(oracle):
    """fac (tensor/ufunc.nim:84-85 -> Nim's std/math fac): n! for 0 .. 20 against Python's exact integers, wrapped into
    int32 from 13! on; 0 outside the table's range, where Nim raises."""
    import math
    n = np.arange(0, 21, dtype=np.int64)
    assert oracle.unary("fac", n).tolist() == [math.factorial(int(k)) for k in n]
    got32 = oracle.unary("fac", n.astype(np.int32))
    assert got32.tolist() == [((math.factorial(int(k)) + 2**31) % 2**32) - 2**31 for k in n]
    assert oracle.unary("fac", np.array([-1, 21, 5], dtype=np.int64)).tolist() == [0, 0, 120]
    with pytest.raises(ValueError):
        oracle.unary("fac", np.array([1.0, 2.0]))
