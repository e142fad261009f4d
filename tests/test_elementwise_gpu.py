"""Element-wise / broadcast / map parity on the GPU (through the C ABI): bit-exact against the CPU
oracle and NumPy for every single-operation body; transcendental bodies within a stated tolerance."""
import numpy as np
import pytest

from conftest import DTYPES, seed_of

pytestmark = pytest.mark.gpu
ALL = ["f32", "f64", "i32", "i64"]
INT, FLT = ["i32", "i64"], ["f32", "f64"]


def say(*a):
    print(*a, flush=True)


def _kinds(kind):
    return {"int": INT, "float": FLT, "any": ALL, "float64_only": ["f64"]}[kind]


def fill(rng, shape, dt, lo=-50, hi=50):
    if np.dtype(dt).kind == "f":
        return rng.uniform(-4, 4, size=shape).astype(dt)
    return rng.integers(lo, hi, size=shape, endpoint=True).astype(dt)


# ------------------------------------------------------------------ reference vectors
def test_reference_elementwise_vectors(hip, vectors):
    for case in vectors["elementwise"]:
        for sfx in _kinds(case["kind"]):
            dt = DTYPES[sfx]
            say("ew vector", case["name"], sfx)
            a, b = hip.toHip(np.array(case["a"], dtype=dt)), hip.toHip(np.array(case["b"], dtype=dt))
            op = {"add": "+.", "sub": "-.", "mul": "*.", "div": "/.", "mod": "mod"}[case["op"]]
            got = hip.OPERATORS[op](a, b).toCpu()
            assert np.array_equal(got, np.array(case["expect"], dtype=dt)), (case["name"], sfx)


def test_reference_explicit_broadcast(hip, vectors):
    for case in vectors["explicit_broadcast"]:
        t = hip.toHip(np.array(case["t"], dtype=np.int64))
        assert np.array_equal(t.bc(case["shape"]).clone().toCpu(), np.array(case["expect"]))
        assert np.array_equal(t.bc(case["shape"]).toCpu(), np.array(case["expect"]))


def test_reference_inplace_broadcast(hip, vectors):
    for case in vectors["inplace_broadcast"]:
        for sfx in _kinds(case["kind"]):
            dt = DTYPES[sfx]
            say("ew inplace", case["source"], sfx)
            a, b = hip.toHip(np.array(case["a"], dtype=dt)), hip.toHip(np.array(case["b"], dtype=dt))
            op = {"add": "+.=", "sub": "-.=", "mul": "*.=", "div": "/.="}[case["op"]]
            hip.OPERATORS[op](a, b)
            assert np.array_equal(a.toCpu(), np.array(case["expect"], dtype=dt))


def test_reference_scalar_chains(hip, vectors):
    for case in vectors["scalar_chains"]:
        for sfx in _kinds(case["kind"]):
            dt = DTYPES[sfx]
            say("ew scalar", case["source"], sfx)
            t = hip.toHip(np.array(case["a"], dtype=dt))
            for op, s, side in case["steps"]:
                f = hip.OPERATORS[{"add": "+.", "sub": "-.", "mul": "*.", "div": "/.", "mod": "mod"}[op]]
                t = f(s, t) if side == "left" else f(t, s)
            assert np.array_equal(t.toCpu(), np.array(case["expect"], dtype=dt)), (case["source"], sfx)


def test_reference_sigmoid_chain(hip, vectors):
    c = vectors["sigmoid_chain"]
    t = hip.toHip(np.array(c["t"], dtype=np.float32))
    e = hip.unary("exp", hip.bc_sub(0.0, t))
    got = hip.bc_div(1.0, hip.bc_add(1.0, e))
    assert np.array_equal(got.toCpu(), np.array(c["expect"], dtype=np.float32))
    assert np.array_equal(hip.sigmoid(t).toCpu(), np.array(c["expect"], dtype=np.float32))


def test_reference_sliced_add_sub(hip, vectors):
    c = vectors["sliced_add_sub"]
    a = hip.toHip(np.array(c["a"], dtype=np.float64))
    a_t = a.transpose()
    for case in c["cases"]:
        (r0, r1, _), (c0, c1, _) = case["slice"]
        x, y = a[r0:r1 + 1, c0:c1 + 1], a_t[r0:r1 + 1, c0:c1 + 1]
        got = (x + y) if case["op"] == "add" else (x - y)
        assert np.array_equal(got.toCpu(), np.array(case["expect"], dtype=np.float64))


def test_reference_inplace_on_transposed(hip, vectors):
    c = vectors["inplace_on_transposed"]
    t = np.array(c["vandermonde"], dtype=np.float32)
    z = hip.toHip(t).clone().transpose()
    z += z
    assert np.array_equal(z.toCpu(), np.array(c["after_z_plus_z"], dtype=np.float32))
    z += hip.toHip(t)
    assert np.array_equal(z.toCpu(), np.array(c["after_plus_t2"], dtype=np.float32))
    with pytest.raises(ValueError):
        z += hip.toHip(t)[0:2, 0:2]


def test_reference_map2_bool(hip, vectors):
    """The reference's fixture for a map body whose result type differs from the input's: x mod y == 0
    as ONE device pass that returns a bool tensor."""
    c = vectors["map2_bool"]
    for dt in (np.int64, np.int32):
        a, b = hip.toHip(np.array(c["a"], dtype=dt)), hip.toHip(np.array(c["b"], dtype=dt))
        m = hip.map2("mod_is_zero", a, b)
        assert m.dtype == np.bool_ and m.shape == (4,)
        assert np.array_equal(m.toCpu(), np.array(c["expect"]))
        assert np.array_equal(hip.map2("mod", a, b).toCpu(), np.array(c["expect_mod"], dtype=dt))


def test_reference_comparison_vectors(hip, vectors):
    c = vectors["comparison"]
    for sfx in ALL:
        dt = DTYPES[sfx]
        a, b = hip.toHip(np.array(c["a"], dtype=dt)), hip.toHip(np.array(c["b"], dtype=dt))
        for case in c["tensor_tensor"]:
            say("compare vector", sfx, case["cmp"])
            got = hip.OPERATORS[case["cmp"] + "."](a, b)
            assert got.dtype == np.bool_ and np.array_equal(got.toCpu(), np.array(case["expect"]))
        for case in c["tensor_scalar"]:
            f = hip.OPERATORS[case["cmp"] + "."]
            got = f(case["scalar"], a) if case["scalar_on_left"] else f(a, case["scalar"])
            assert np.array_equal(got.toCpu(), np.array(case["expect"])), case


def test_reference_math_function_vectors(hip, vectors):
    m = vectors["math_functions"]
    for sfx in FLT:
        dt = DTYPES[sfx]
        s = m["sgn"]
        got = hip.sgn(hip.toHip(np.array(s["a"], dtype=dt)))
        assert got.dtype == np.int64 and got.toCpu().tolist() == s["expect"]
        cs = m["copysign"]
        a = hip.toHip(np.array(cs["a"], dtype=dt))
        want = np.array(cs["expect"], dtype=dt)
        hip.mcopySign(a, hip.toHip(np.array(cs["signs"], dtype=dt)))
        assert np.array_equal(a.toCpu(), want) and np.array_equal(np.signbit(a.toCpu()), np.signbit(want))
        c = m["classify"]
        x = hip.toHip(np.array([float(v) for v in c["a"]], dtype=dt))
        assert np.array_equal(hip.isNaN(x).toCpu(), np.array(c["isnan"]))
        assert np.array_equal(hip.isNotNaN(x).toCpu(), ~np.array(c["isnan"]))
        assert [hip.FLOAT_CLASS[k] for k in hip.classify(x).toCpu()] == c["classes"]
    mm = m["minmax"]
    for sfx in INT:
        a, b = hip.toHip(np.array(mm["a"], dtype=DTYPES[sfx])), hip.toHip(np.array(mm["b"], dtype=DTYPES[sfx]))
        assert hip.map2("min", a, b).toCpu().tolist() == mm["min"] and hip.map2("max", a, b).toCpu().tolist() == mm["max"]
    f = m["floormod"]
    a = np.array([f["start"] + i * f["step"] for i in range(f["count"])])
    ts, st = hip.floorMod(hip.toHip(a), 3.0).toCpu(), hip.floorMod(3.0, hip.toHip(a)).toCpu()
    assert np.mean(np.abs(ts - np.array(f["tensor_scalar_3"]))) < 1e-9 and np.signbit(ts[1])
    assert np.mean(np.abs(st - np.array(f["scalar_3_tensor"]))) < 1e-9


# ------------------------------------------------------------------ oracle / NumPy parity
SHAPES = [(1,), (3,), (1000,), (4099,), (7, 13), (64, 4096), (33, 4100), (5, 6, 7), (2, 3, 4, 5, 6, 2), (300, 1), (1, 300)]
BIN_OPS = ["add", "sub", "mul", "div", "add_relu", "relu_bwd", "max", "min", "sigmoid_bwd", "tanh_bwd", "sqdiff"]


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("shape", SHAPES)
def test_same_shape_ops_bit_exact(hip, oracle, sfx, shape):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, shape))
    a, b = fill(rng, shape, dt), fill(rng, shape, dt)
    if sfx in INT:
        a.ravel()[:2] = [np.iinfo(dt).max, np.iinfo(dt).min][: min(2, a.size)]   # force wraparound cases
    da, db = hip.toHip(a), hip.toHip(b)
    for op in BIN_OPS + (["mod"] if sfx in INT else []):
        say("same-shape", sfx, shape, op)
        got = hip.map2(op, da, db).toCpu()
        want = oracle.map2(op, a, b)
        assert np.array_equal(got, want, equal_nan=True), op
        assert np.array_equal(got, oracle.closed_map2(op, a, b), equal_nan=True), op


BC_CASES = [((64, 4096), (1, 4096)), ((64, 4096), (64, 1)), ((1, 4096), (64, 4096)), ((64, 1), (64, 4096)),
            ((4, 1), (1, 3)), ((5, 1, 7), (1, 6, 1)), ((2, 3, 2048), (2, 1, 2048)), ((3, 1, 4096), (1, 5, 1)),
            ((1, 1), (9, 1031)),
            # rows far shorter than a column tile, whole 16-byte vectors per row: the flat form of the row kernel
            ((300, 64), (1, 64)), ((300, 64), (300, 1)), ((1, 64), (300, 64)), ((300, 1), (300, 64)), ((17, 8, 36), (1, 8, 1)),
            ((17, 8, 36), (17, 1, 36)), ((6, 5, 4, 24), (1, 5, 1, 1)), ((6, 5, 4, 24), (6, 1, 4, 1))]


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("shapes", BC_CASES)
def test_broadcast_ops_bit_exact(hip, oracle, sfx, shapes):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, shapes))
    a, b = fill(rng, shapes[0], dt), fill(rng, shapes[1], dt)
    b[b == 0] = 3
    da, db = hip.toHip(a), hip.toHip(b)
    for name, npf in [("+.", np.add), ("-.", np.subtract), ("*.", np.multiply)]:
        say("broadcast", sfx, shapes, name)
        got = hip.OPERATORS[name](da, db).toCpu()
        with np.errstate(over="ignore"):
            assert np.array_equal(got, npf(a, b)), name
    say("broadcast", sfx, shapes, "/.")
    ba, bb = oracle.broadcast2(a, b)
    assert np.array_equal(hip.bc_div(da, db).toCpu(), oracle.map2("div", ba, bb))
    assert np.array_equal(hip.bias_relu(da, db).toCpu(), oracle.map2("add_relu", ba, bb))


CMPS = ["==", "!=", "<", "<=", ">", ">="]
_NP_CMP = {"==": np.equal, "!=": np.not_equal, "<": np.less, "<=": np.less_equal, ">": np.greater, ">=": np.greater_equal}


def _with_specials(a, b, sfx):
    if sfx in FLT:   # NaN, infinities and signed zeros on both sides, some of them facing each other
        sp = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, np.nan], dtype=a.dtype)
        a.ravel()[: min(6, a.size)] = sp[: min(6, a.size)]
        b.ravel()[: min(6, b.size)] = sp[::-1][: min(6, b.size)]
    return a, b


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("shapes", BC_CASES + [((4099,), (4099,)), ((33, 4100), (33, 4100))])
def test_broadcast_comparisons_bit_exact(hip, oracle, sfx, shapes):
    """`==.` ... `>=.` with implicit broadcasting and in the scalar forms: each output byte is one comparison,
    so NumPy fixes it; the oracle's strided walk is compared as well. Small value range, so that equal
    elements occur."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("cmp", sfx, shapes))
    a = rng.integers(-3, 3, shapes[0], endpoint=True).astype(dt)
    b = rng.integers(-3, 3, shapes[1], endpoint=True).astype(dt)
    a, b = _with_specials(a, b, sfx)
    da, db = hip.toHip(a), hip.toHip(b)
    ba, bb = oracle.broadcast2(a, b)
    for cmp in CMPS:
        say("compare", sfx, shapes, cmp)
        got = hip.OPERATORS[cmp + "."](da, db)
        assert got.dtype == np.bool_ and got.is_C_contiguous()
        g = got.toCpu()
        with np.errstate(invalid="ignore"):
            assert np.array_equal(g, _NP_CMP[cmp](a, b)), cmp
        assert np.array_equal(g, oracle.compare(cmp, ba, bb)), cmp
        with np.errstate(invalid="ignore"):
            assert np.array_equal(hip.OPERATORS[cmp + "."](da, 1).toCpu(), _NP_CMP[cmp](a, dt(1))), cmp
            assert np.array_equal(hip.OPERATORS[cmp + "."](1, da).toCpu(), _NP_CMP[cmp](dt(1), a)), cmp
    if sfx in INT:
        b2 = b.copy(); b2[b2 == 0] = 2
        got = hip.map2("mod_is_zero", hip.toHip(ba.copy()), hip.toHip(np.broadcast_to(b2, ba.shape).copy())).toCpu()
        assert np.array_equal(got, np.fmod(ba, np.broadcast_to(b2, ba.shape)) == 0)


@pytest.mark.parametrize("sfx", ALL)
def test_short_rows_in_wider_buffers(hip, oracle, sfx):
    """Column windows of wider buffers whose rows are a few vectors long (the flat form of the row kernel, with row
    strides that differ between the operands): two windows, window and row / column vector, scalar and unary forms,
    comparisons, in place; a window that starts off a 16-byte boundary takes the generic kernel and must agree."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("short-rows", sfx))
    P, Q = fill(rng, (257, 200), dt), fill(rng, (257, 136), dt)
    dP, dQ = hip.toHip(P), hip.toHip(Q)
    row, col = fill(rng, (1, 72), dt), fill(rng, (257, 1), dt)
    drow, dcol = hip.toHip(row), hip.toHip(col)
    for lo_p, lo_q in [(8, 16), (64, 0), (3, 5)]:
        a, b = P[:, lo_p:lo_p + 72], Q[:, lo_q:lo_q + 72]
        da, db = dP[:, lo_p:lo_p + 72], dQ[:, lo_q:lo_q + 72]
        say("short rows", sfx, lo_p, lo_q)
        with np.errstate(over="ignore"):
            assert np.array_equal(hip.map2("sub", da, db).toCpu(), a - b)
            assert np.array_equal(hip.bc_add(da, drow).toCpu(), a + row)
            assert np.array_equal(hip.bc_mul(dcol, db).toCpu(), col * b)
            assert np.array_equal(hip.scalar_op("sub", da, 3, scalar_on_left=True).toCpu(), dt(3) - a)
            assert np.array_equal(hip.unary("neg", db).toCpu(), -b)
        assert np.array_equal(hip.bc_lt(da, db).toCpu(), a < b)
        assert np.array_equal(hip.bc_ge(da, dcol).toCpu(), a >= col)
    # in place on a window: the columns outside it stay as they were
    want = P.copy()
    with np.errstate(over="ignore"):
        want[:, 8:80] += Q[:, 16:88]
        want[:, 8:80] *= row
    w = dP[:, 8:80]
    w += dQ[:, 16:88]
    w.bc_imul(drow)
    assert np.array_equal(dP.toCpu(), want)


@pytest.mark.parametrize("sfx", ALL)
def test_comparisons_and_predicates_on_strided_views(hip, oracle, sfx):
    """Transposed, stepped, reversed and column-sliced operands (the generic and the LDS-tiled kernels with a
    one-byte destination), plus sgn / isNaN / classify on the same views."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("cmp-strided", sfx))
    P = rng.integers(-2, 2, (96, 80), endpoint=True).astype(dt)
    Q = rng.integers(-2, 2, (80, 96), endpoint=True).astype(dt)
    P, Q = _with_specials(P, Q, sfx)
    if sfx in FLT:
        P[5, 7:12] = [np.finfo(dt).tiny / 2, -np.finfo(dt).tiny / 8, np.finfo(dt).tiny, -1e-30, 3.5]
    dP, dQ = hip.toHip(P), hip.toHip(Q)
    cases = [("transposed b", dP, P, dQ.transpose(), Q.T),
             ("both stepped", dP[::2, ::2], P[::2, ::2], dQ.transpose()[::2, ::2], Q.T[::2, ::2]),
             ("reversed", dP[::-1, ::-1], P[::-1, ::-1], dQ.transpose(), Q.T),
             ("column block", dP[:, 16:48], P[:, 16:48], dP[:, 48:80], P[:, 48:80])]
    for name, da, a, db, b in cases:
        for cmp in ("==", "<", ">="):
            say("compare strided", sfx, name, cmp)
            assert np.array_equal(hip.map2(cmp, da, db).toCpu(), oracle.compare(cmp, a, b)), (name, cmp)
        assert np.array_equal(hip.sgn(da).toCpu(), oracle.sgn(a)), name
        if sfx in FLT:
            for pred, f in (("isnan", hip.isNaN), ("isnotnan", hip.isNotNaN), ("classify", hip.classify)):
                assert np.array_equal(f(da).toCpu(), oracle.predicate(pred, a)), (name, pred)
    with pytest.raises(TypeError):
        hip.map2("add", hip.map2("==", dP, dP), hip.map2("==", dP, dP))     # no arithmetic on bool tensors
    if sfx in INT:
        with pytest.raises(TypeError):
            hip.isNaN(dP)


@pytest.mark.parametrize("sfx", ALL)
def test_floormod_clamp_by_value_and_angle_conversions(hip, oracle, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("floormod", sfx))
    a, b = fill(rng, (37, 1028), dt), fill(rng, (37, 1028), dt, lo=-9, hi=9)
    b[b == 0] = 4
    da, db = hip.toHip(a), hip.toHip(b)
    assert np.array_equal(hip.floorMod(da, db).toCpu(), oracle.map2("floormod", a, b))
    assert np.array_equal(hip.floorMod(da, 3).toCpu(), oracle.scalar_op("floormod", a, 3))
    assert np.array_equal(hip.floorMod(-3, da.transpose()).toCpu(), oracle.scalar_op("floormod", a.T, -3, scalar_on_left=True))
    if sfx in INT:
        assert np.array_equal(hip.floorMod(da, db).toCpu(), np.mod(a, b))       # Python's %: sign of the divisor
    # clamp with both bounds by value, out of place on a view and in place
    lo, hi = (dt(-1.5), dt(2.25)) if sfx in FLT else (dt(-7), dt(11))
    assert np.array_equal(hip.clamp(da, lo, hi).toCpu(), np.clip(a, lo, hi))
    assert np.array_equal(hip.clamp(da.transpose()[::2], lo, hi).toCpu(), np.clip(a.T[::2], lo, hi))
    dc = hip.toHip(a)
    hip.mclamp(dc[:, 16:48], lo, hi)
    want = a.copy(); want[:, 16:48] = np.clip(a[:, 16:48], lo, hi)
    assert np.array_equal(dc.toCpu(), want)
    if sfx in FLT:
        x = np.concatenate([a.ravel()[:4000] * 90, [0.0, 180.0, -360.0, 1e-30]]).astype(dt)
        assert np.array_equal(hip.degToRad(hip.toHip(x)).toCpu(), oracle.unary("degtorad", x))
        assert np.array_equal(hip.radToDeg(hip.toHip(x)).toCpu(), oracle.unary("radtodeg", x))
        assert np.array_equal(hip.copySign(da, db).toCpu(), np.copysign(a, b))
        nan_clamped = hip.clamp(hip.toHip(np.array([np.nan, -9, 9], dtype=dt)), lo, hi).toCpu()
        assert np.isnan(nan_clamped[0]) and nan_clamped[1] == lo and nan_clamped[2] == hi


def test_clamp_inside_a_graph(hip):
    """Bounds by value: the call allocates nothing and copies nothing, so it can be recorded."""
    x = np.random.default_rng(5).uniform(-4, 4, (64, 4096)).astype(np.float32)
    dx, out = hip.toHip(x), hip.empty((64, 4096), np.float32)
    from arraymancer_amd import tensor_hip as th
    with hip.Graph() as g:
        th._clamp_into(out, dx, -1.0, 1.0)
    for _ in range(3):
        g.launch()
        assert np.array_equal(out.toCpu(), np.clip(x, -1, 1))
        th._unary_into("neg", out, out)   # eager work between replays


@pytest.mark.parametrize("sfx", ALL)
def test_strided_operands_and_destinations(hip, oracle, sfx):
    """Transposed, stepped, reversed and column-sliced operands, out of place and in place."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, "strided"))
    P, Q = fill(rng, (96, 80), dt), fill(rng, (80, 96), dt)
    dP, dQ = hip.toHip(P), hip.toHip(Q)
    cases = [
        ("transposed b", dP, P, dQ.transpose(), Q.T),
        ("both stepped", dP[::2, ::2], P[::2, ::2], dQ.transpose()[::2, ::2], Q.T[::2, ::2]),
        ("reversed", dP[::-1, ::-1], P[::-1, ::-1], dQ.transpose(), Q.T),
        ("column block (GRU gate slices)", dP[:, 16:48], P[:, 16:48], dP[:, 48:80], P[:, 48:80]),
    ]
    for name, da, a, db, b in cases:
        say("strided", sfx, name)
        assert np.array_equal(hip.map2("add", da, db).toCpu(), oracle.map2("add", a, b)), name
        assert np.array_equal(hip.map2("mul", da, db).toCpu(), oracle.map2("mul", a, b)), name
    # in place through a strided destination: parent[:, 16:48] +.= row vector
    say("strided inplace", sfx)
    v = fill(rng, (1, 32), dt)
    dP[:, 16:48].bc_iadd(hip.toHip(v))
    P2 = P.copy(); P2[:, 16:48] += v
    assert np.array_equal(dP.toCpu(), P2)
    # in place on a transposed destination
    dQt = dQ.transpose()
    dQt += dP
    assert np.array_equal(dQ.toCpu(), (Q.T + P2).T)


@pytest.mark.parametrize("sfx", ALL)
def test_scalar_and_unary(hip, oracle, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, "scalar"))
    a = fill(rng, (37, 1028), dt)
    a[a == 0] = 5
    da = hip.toHip(a)
    for op in ["add", "sub", "mul", "div", "max", "min"] + (["mod"] if sfx in INT else []):
        for left in (False, True):
            say("scalar", sfx, op, left)
            got = hip.scalar_op(op, da, 3, scalar_on_left=left).toCpu()
            assert np.array_equal(got, oracle.scalar_op(op, a, 3, scalar_on_left=left)), (op, left)
    for op in ["copy", "neg", "relu", "abs", "square"] + (["sqrt"] if sfx in FLT else []):
        say("unary", sfx, op)
        nan_ok = op == "sqrt"   # negative entries
        with np.errstate(invalid="ignore"):
            assert np.array_equal(hip.unary(op, da).toCpu(), oracle.unary(op, a), equal_nan=nan_ok), op
            assert np.array_equal(hip.unary(op, da.transpose()).toCpu(), oracle.unary(op, a.T), equal_nan=nan_ok), op
    assert np.array_equal((da * 2).toCpu(), a * dt(2))
    assert np.array_equal((2 * da).toCpu(), a * dt(2))
    assert np.array_equal((-da).toCpu(), -a)
    assert np.array_equal(da.transpose().clone().toCpu(), a.T)
    assert np.array_equal(da.reshape(1028, 37).toCpu(), a.reshape(1028, 37))
    assert np.array_equal(da.transpose().reshape(37, 1028).toCpu(), a.T.reshape(37, 1028))


@pytest.mark.parametrize("sfx", FLT)
def test_transcendental_bodies(hip, oracle, sfx):
    """exp / tanh / sigmoid come from the device math library: not bit-comparable with libm.
    Tolerance: 4 ulp-scale relative error (float32 4e-7 * 4, float64 1e-15 * 8)."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, "trans"))
    a, b = fill(rng, (64, 1024), dt), fill(rng, (1, 1024), dt)
    rtol = 2e-6 if sfx == "f32" else 1e-14
    da, db = hip.toHip(a), hip.toHip(b)
    ba, bb = oracle.broadcast2(a, b)
    for op in ("add_sigmoid", "add_tanh"):
        say("transcendental", sfx, op)
        la, lb = da, db.broadcast(a.shape)
        np.testing.assert_allclose(hip.map2(op, la, lb).toCpu(), oracle.map2(op, ba, bb), rtol=rtol, atol=rtol)
    for op in ("sigmoid", "tanh", "exp"):
        np.testing.assert_allclose(hip.unary(op, da).toCpu(), oracle.unary(op, a), rtol=rtol, atol=rtol)


@pytest.mark.parametrize("sfx", FLT)
def test_sqrt_is_correctly_rounded(hip, sfx):
    """IEEE square root: the same bits as NumPy's, NaN for negative input, signed zeros kept."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, "sqrt"))
    x = np.concatenate([rng.uniform(0, 1e6, 4093), 10.0 ** rng.uniform(-40, 38, 2000), [0.0, -0.0, np.inf, 1.0, 4.0, 2.0]]).astype(dt)
    got = hip.sqrt(hip.toHip(x)).toCpu()
    assert np.array_equal(got, np.sqrt(x))
    assert np.signbit(got[-5]) and got[-5] == 0
    with np.errstate(invalid="ignore"):
        assert np.isnan(hip.sqrt(hip.toHip(np.array([-1.0, np.nan], dtype=dt))).toCpu()).all()
    with pytest.raises(TypeError):
        hip.sqrt(hip.zeros((4,), np.int32))


def test_relu_special_values(hip):
    x = np.array([-1.0, -0.0, 0.0, 2.5, np.nan, -np.inf, np.inf] * 3, dtype=np.float32)
    r = hip.relu(hip.toHip(x)).toCpu()
    assert r[:4].tolist() == [0.0, 0.0, 0.0, 2.5] and not np.signbit(r[1])
    assert np.isnan(r[4]) and r[5] == 0 and r[6] == np.inf


def test_int_division_conventions(hip):
    a = hip.toHip(np.array([7, -7, 7, -7, 0, 5, -2**31], dtype=np.int32))
    b = hip.toHip(np.array([2, 2, -2, -2, 3, 0, -1], dtype=np.int32))
    assert hip.bc_div(a, b).toCpu().tolist() == [3, -3, -3, 3, 0, 0, -2**31]
    assert hip.bc_mod(a, b).toCpu().tolist() == [1, -1, 1, -1, 0, 0, 0]


def test_errors(hip):
    a = hip.toHip(np.zeros((4, 2), np.float32))
    with pytest.raises(ValueError):
        hip.bc_add(a, hip.toHip(np.zeros((1, 3), np.float32)))
    with pytest.raises(TypeError):
        hip.map2("add_tanh", hip.toHip(np.zeros(3, np.int32)), hip.toHip(np.zeros(3, np.int32)))
    with pytest.raises(ValueError):   # zero-stride destination
        hip.apply2("add", hip.toHip(np.zeros((1, 2), np.float32)).broadcast((4, 2)), a)
    empty = hip.empty((0, 5), np.float32)
    assert (empty + empty).shape == (0, 5)


# ------------------------------------------------------------------ the 8192 x 8192 broadcast configuration, full size
def test_config4_8192_bit_exact(hip):
    X = np.random.default_rng(4001).uniform(-1, 1, (8192, 8192)).astype(np.float32)
    b = np.random.default_rng(4002).uniform(-1, 1, (1, 8192)).astype(np.float32)
    s = np.random.default_rng(4003).uniform(-1, 1, (8192, 1)).astype(np.float32)
    dX, db, ds = hip.toHip(X), hip.toHip(b), hip.toHip(s)
    say("config4 +.")
    dY = hip.bc_add(dX, db)
    Y = X + b
    assert np.array_equal(dY.toCpu(), Y)
    say("config4 *.")
    assert np.array_equal(hip.bc_mul(dY, ds).toCpu(), Y * s)
    say("config4 bias+relu")
    assert np.array_equal(hip.bias_relu(dX, db).toCpu(), np.where(0 >= Y, np.float32(0), Y))


@pytest.mark.parametrize("sfx", FLT)
def test_gru_cell_gates_on_column_slices(hip, oracle, sfx):
    """The fused gate bodies of the reference's GRU cell (nn_primitives/nnp_gru.nim:73-88), applied in
    place to column slices of [batch, 3H] buffers, against the oracle doing the same on NumPy views."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, "gru"))
    batch, H = 48, 256
    W3x, U3h, hidden = fill(rng, (batch, 3 * H), dt), fill(rng, (batch, 3 * H), dt), fill(rng, (batch, H), dt)
    dW, dU, dh = hip.toHip(W3x), hip.toHip(U3h), hip.toHip(hidden)
    sr, sz, srz, s_ = slice(0, H), slice(H, 2 * H), slice(0, 2 * H), slice(2 * H, 3 * H)
    say("gru step 2", sfx)
    hip.apply2("add_sigmoid", dW[:, srz], dU[:, srz])
    oracle.map2("add_sigmoid", W3x[:, srz], U3h[:, srz], out=W3x[:, srz])
    say("gru step 3", sfx)
    hip.apply3("gru_candidate", dW[:, s_], dW[:, sr], dU[:, s_])
    oracle.map3("gru_candidate", W3x[:, s_], W3x[:, sr], U3h[:, s_], out=W3x[:, s_])
    say("gru step 4", sfx)
    hip.apply3("gru_blend", dh, dW[:, sz], dW[:, s_])
    oracle.map3("gru_blend", hidden, W3x[:, sz], W3x[:, s_], out=hidden)
    tol = 4e-6 if sfx == "f32" else 1e-13
    np.testing.assert_allclose(dW.toCpu(), W3x, rtol=tol, atol=tol)
    np.testing.assert_allclose(dh.toCpu(), hidden, rtol=tol, atol=tol)


@pytest.mark.parametrize("sfx", ALL)
def test_map3_muladd_bit_exact(hip, oracle, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, "map3"))
    for shape in [(5,), (33, 1030), (4, 6, 258), (64, 4096)]:
        a, b, c = fill(rng, shape, dt), fill(rng, shape, dt), fill(rng, shape, dt)
        say("map3 muladd", sfx, shape)
        got = hip.map3("muladd", hip.toHip(a), hip.toHip(b), hip.toHip(c)).toCpu()
        assert np.array_equal(got, oracle.map3("muladd", a, b, c))
        if len(shape) == 2:   # transposed operand -> generic kernel
            got = hip.map3("muladd", hip.toHip(a), hip.toHip(np.ascontiguousarray(b.T)).transpose(), hip.toHip(c)).toCpu()
            assert np.array_equal(got, oracle.map3("muladd", a, b, c))
    # (X +. b) *. s in one pass equals the two broadcast passes bit for bit (each step rounded on its own)
    X, r, col = fill(rng, (300, 1030), dt), fill(rng, (1, 1030), dt), fill(rng, (300, 1), dt)
    dX, dr, dc = hip.toHip(X), hip.toHip(r), hip.toHip(col)
    fused = hip.map3("addmul", dX, dr.broadcast(X.shape), dc.broadcast(X.shape)).toCpu()
    assert np.array_equal(fused, hip.bc_mul(hip.bc_add(dX, dr), dc).toCpu())
    assert np.array_equal(fused, oracle.map3("addmul", X, np.broadcast_to(r, X.shape), np.broadcast_to(col, X.shape)))
    if sfx in INT:
        with pytest.raises(TypeError):
            hip.map3("gru_blend", hip.toHip(a), hip.toHip(b), hip.toHip(c))
    else:
        x, y, z = (hip.toHip(t) for t in (a, b, c))
        assert np.array_equal(hip.map3("gru_blend", x, y, z).toCpu(), oracle.map3("gru_blend", a, b, c))


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("shape", [(16, 16), (130, 67), (257, 1031), (1024, 512), (128, 128), (260, 392), (136, 1028)])
def test_mixed_unit_stride_axes(hip, oracle, sfx, shape):
    """Operands whose unit stride is on different axes (the LDS-tiled 2-D kernels: the element form for small,
    odd or unaligned extents, the 16-byte-vector form with whole and ragged tiles otherwise): transposed inputs,
    transposed destinations, a broadcast row or column vector beside a transposed matrix, scalar and unary
    forms, windows of larger tensors."""
    dt = DTYPES[sfx]
    R, C = shape
    rng = np.random.default_rng(seed_of(sfx, "tiled", shape))
    A, Bt, v = fill(rng, (R, C), dt), fill(rng, (C, R), dt), fill(rng, (1, C), dt)
    dA, dBt, dv = hip.toHip(A), hip.toHip(Bt), hip.toHip(v)
    say("tiled a + b^T", sfx, shape)
    assert np.array_equal(hip.map2("add", dA, dBt.transpose()).toCpu(), A + Bt.T)
    assert np.array_equal(hip.map2("sub", dBt.transpose(), dA).toCpu(), Bt.T - A)
    say("tiled both transposed", sfx, shape)
    assert np.array_equal(hip.map2("mul", dBt.transpose(), dBt.transpose()).toCpu(), oracle.map2("mul", Bt.T, Bt.T))
    say("tiled clone / unary / scalar of a transposed view", sfx, shape)
    assert np.array_equal(dBt.transpose().clone().toCpu(), Bt.T)
    assert np.array_equal(hip.unary("neg", dBt.transpose()).toCpu(), oracle.unary("neg", Bt.T))
    assert np.array_equal(hip.scalar_op("sub", dBt.transpose(), 3, scalar_on_left=True).toCpu(),
                          oracle.scalar_op("sub", Bt.T, 3, scalar_on_left=True))
    say("tiled broadcast row vector + transposed", sfx, shape)
    assert np.array_equal(hip.bc_add(dBt.transpose(), dv).toCpu(), Bt.T + v)
    col = fill(rng, (R, 1), dt)
    assert np.array_equal(hip.bc_mul(dBt.transpose(), hip.toHip(col)).toCpu(), oracle.map2("mul", Bt.T, np.broadcast_to(col, (R, C))))
    if R > 24 and C > 24:
        say("tiled windows", sfx, shape)
        for r_lo, c_lo in [(8, 4), (4, 8), (1, 3)]:    # the last one breaks the 16-byte alignment: element form
            got = hip.map2("add", dA[r_lo:, c_lo:], dBt.transpose()[r_lo:, c_lo:]).toCpu()
            assert np.array_equal(got, A[r_lo:, c_lo:] + Bt.T[r_lo:, c_lo:]), (r_lo, c_lo)
            assert np.array_equal(dBt.transpose()[r_lo:, c_lo:].clone().toCpu(), Bt.T[r_lo:, c_lo:])
    say("tiled in place on a transposed destination", sfx, shape)
    dD = hip.toHip(Bt)
    dDt = dD.transpose()
    dDt += dA
    assert np.array_equal(dD.toCpu(), (Bt.T + A).T)
    dDt.bc_imul(dv)
    assert np.array_equal(dD.toCpu(), ((Bt.T + A) * v).T)


@pytest.mark.parametrize("sfx", FLT)
def test_activation_backward(hip, oracle, sfx):
    """relu / sigmoid / tanh backward (nnp_activation.nim:61-74): map2 over (cached output,
    gradient), bit-exact against the oracle and the NumPy statement; sigmoid and tanh backward
    agree with central differences of the device forward pass."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(77)
    x, g = fill(rng, (33, 130), dt), fill(rng, (33, 130), dt)
    dx, dg = hip.toHip(x), hip.toHip(g)
    say("activation backward", sfx)
    assert np.array_equal(hip.relu_backward(dg, dx).toCpu(), np.where(x <= 0, dt(0), g))
    s, t = hip.sigmoid(dx), hip.tanh(dx)
    cs, ct = s.toCpu(), t.toCpu()
    assert np.array_equal(hip.sigmoid_backward(dg, s).toCpu(), cs * (1 - cs) * g)
    assert np.array_equal(hip.tanh_backward(dg, t).toCpu(), g * (1 - ct * ct))
    assert np.array_equal(hip.sigmoid_backward(dg, s).toCpu(), oracle.map2("sigmoid_bwd", cs, g))
    assert np.array_equal(hip.tanh_backward(dg, t.transpose().clone().transpose()).toCpu(), oracle.map2("tanh_bwd", ct, g))
    if sfx == "f64":
        h = 1e-6
        up, dn = hip.toHip(x + h), hip.toHip(x - h)
        num = (hip.sigmoid(up).toCpu() - hip.sigmoid(dn).toCpu()) / (2 * h) * g
        assert np.allclose(num, hip.sigmoid_backward(dg, s).toCpu(), rtol=1e-6, atol=1e-9)
        num = (hip.tanh(up).toCpu() - hip.tanh(dn).toCpu()) / (2 * h) * g
        assert np.allclose(num, hip.tanh_backward(dg, t).toCpu(), rtol=1e-6, atol=1e-9)


# ------------------------------------------------------------------ `^.` and the universal functions
_UFUNC_DOMAIN = dict(ln=(1e-3, 1e3), log10=(1e-3, 1e3), log2=(1e-3, 1e3), arcsin=(-1, 1), arccos=(-1, 1),
                     arccosh=(1, 50), arctanh=(-0.999, 0.999), sinh=(-20, 20), cosh=(-20, 20), gamma=(-3.9, 12),
                     lgamma=(-3.9, 30), cbrt=(-1e3, 1e3))
_EXACT_UFUNCS = ("floor", "ceil", "trunc", "round", "reciprocal", "sqrt")
# Units in the last place allowed between the device math library and the host's libm (both are a few
# ulp from the true value; the reference's result is the host libm's).
_UFUNC_ULPS = dict(gamma=16, lgamma=16, erfc=8, tan=8)


def test_reference_pow_and_ufunc_vectors(hip, vectors):
    """The reference's literals for `^.`, `^.=`, reciprocal, cos and ln. The reference compares pow
    results with ==; the device pow is held to 2 units in the last place here, and the cases whose
    result the device also hits exactly are asserted as such."""
    import math
    v = vectors["pow_and_ufunc"]
    a = np.array(v["a"])
    da = hip.toHip(a)
    quot = np.array([[n / q] for n, q in v["pow_m1_as_quotients"]])
    say("pow literals")
    assert np.array_equal(hip.OPERATORS["^."](da, 2.0).toCpu(), np.array(v["pow_2"]))
    np.testing.assert_allclose(hip.OPERATORS["^."](da, -1.0).toCpu(), quot, rtol=2 ** -51, atol=0)
    np.testing.assert_allclose(hip.OPERATORS["^."](2.0, da).toCpu(), np.array(v["two_pow_a"]), rtol=2 ** -51, atol=0)
    b = da.clone()
    assert hip.OPERATORS["^.="](b, 2.0) is b
    assert np.array_equal(b.toCpu(), np.array(v["pow_2"]))
    assert np.array_equal(hip.reciprocal(da).toCpu(), quot)
    c = da.clone()
    hip.mreciprocal(c)
    assert np.array_equal(c.toCpu(), quot)
    ci, li = np.array(v["cos_input"]), np.array(v["ln_input"])
    assert np.abs(hip.cos(hip.toHip(ci)).toCpu() - np.vectorize(math.cos)(ci)).mean() <= 1e-15
    np.testing.assert_allclose(hip.ln(hip.toHip(li)).toCpu(), np.vectorize(math.log)(li), rtol=2 ** -52, atol=0)


@pytest.mark.parametrize("sfx", FLT)
def test_universal_functions(hip, oracle, sfx):
    """Every function of tensor/ufunc.nim against the oracle (the host's libm, which the reference
    calls): exact for the rounding functions and reciprocal, within a few units in the last place for
    the device math library's transcendental ones; contiguous, transposed and column-slice operands."""
    dt = DTYPES[sfx]
    ulp = np.finfo(dt).eps
    rng = np.random.default_rng(seed_of(sfx, "ufunc"))
    for name in hip.UFUNCS:
        lo, hi = _UFUNC_DOMAIN.get(name, (-8, 8))
        if name == "sqrt":
            lo, hi = 0, 1e6
        a = rng.uniform(lo, hi, (96, 1030)).astype(dt)
        da = hip.toHip(a)
        say("ufunc", sfx, name)
        want = oracle.unary(name, a)
        got = getattr(hip, name if name != "round" else "round")(da).toCpu()
        got_t = hip.unary(name, da.transpose()).toCpu()
        got_s = hip.unary(name, da[:, 3:900]).toCpu()
        if name in _EXACT_UFUNCS:
            assert np.array_equal(got, want), name
        else:
            floor = 1.0 if name == "lgamma" else float(np.finfo(dt).tiny)
            tol = _UFUNC_ULPS.get(name, 4) * ulp * np.maximum(np.abs(want), floor)
            err = np.abs(got.astype(np.float64) - want.astype(np.float64))
            assert np.all(err <= tol), (name, float((err / tol).max()))
        # the same kernel body whatever the strides: transposed and sliced operands give the same bits
        assert np.array_equal(got_t, got.T, equal_nan=True), name
        assert np.array_equal(got_s, got[:, 3:900], equal_nan=True), name


@pytest.mark.parametrize("sfx", FLT)
def test_rounding_functions_special_values(hip, sfx):
    dt = DTYPES[sfx]
    x = np.array([-2.5, -1.5, -0.5, -0.25, -0.0, 0.0, 0.25, 0.5, 1.5, 2.5, 1e30, -1e30, np.inf, -np.inf,
                  np.nextafter(dt(0.5), dt(0))], dtype=dt)
    d = hip.toHip(x)
    for name, fn in (("floor", np.floor), ("ceil", np.ceil), ("trunc", np.trunc)):
        got = hip.unary(name, d).toCpu()
        assert np.array_equal(got, fn(x)) and np.array_equal(np.signbit(got), np.signbit(fn(x))), name
    r = np.trunc(x)
    with np.errstate(invalid="ignore"):
        want = np.where(np.abs(x - r) >= 0.5, r + np.copysign(dt(1), x), r).astype(dt)   # halves away from zero
    got = hip.round(d).toCpu()
    assert np.array_equal(got, want) and np.array_equal(np.signbit(got), np.signbit(x))
    assert np.isnan(hip.floor(hip.toHip(np.array([np.nan], dtype=dt))).toCpu()[0])
    with np.errstate(divide="ignore"):
        assert np.array_equal(hip.reciprocal(d).toCpu(), dt(1) / x)


@pytest.mark.parametrize("sfx", FLT)
def test_pow_forms(hip, oracle, sfx):
    """pow as tensor ^. scalar, scalar ^. tensor, in place, and as a map2 body over broadcast operands."""
    dt = DTYPES[sfx]
    ulp = np.finfo(dt).eps
    rng = np.random.default_rng(seed_of(sfx, "pow"))
    base = rng.uniform(0.1, 6, (64, 1030)).astype(dt)
    expo = rng.uniform(-3, 3, (1, 1030)).astype(dt)
    db, de = hip.toHip(base), hip.toHip(expo)

    def close(got, want, what):
        # float32 pow is evaluated in double on the device and rounded once: the host's bits except at
        # rare near-ties; float64 pow is the device math library's, a few units in the last place off
        err = np.abs(got.astype(np.float64) - want.astype(np.float64))
        lim = (1 if sfx == "f32" else 4) * ulp * np.abs(want)
        assert np.all(err <= lim), (what, float((err / (ulp * np.abs(want))).max()))
        if sfx == "f32":
            assert np.mean(got == want) >= 0.999, (what, float(np.mean(got == want)))

    say("pow", sfx)
    close(hip.bc_pow(db, 2.5).toCpu(), oracle.scalar_op("pow", base, 2.5), "t ^. s")
    close(hip.bc_pow(1.5, db).toCpu(), oracle.scalar_op("pow", base, 1.5, scalar_on_left=True), "s ^. t")
    close(hip.bc_pow(db.transpose(), -0.5).toCpu(), oracle.scalar_op("pow", base.T, -0.5), "transposed")
    ba, bb = oracle.broadcast2(base, expo)
    close(hip.map2("pow", db, de.broadcast(base.shape)).toCpu(), oracle.map2("pow", ba, bb), "map2")
    c = db.clone()
    c.bc_ipow(2.0)
    close(c.toCpu(), oracle.scalar_op("pow", base, 2.0), "^.=")
    ints = np.arange(0, 24, dtype=dt)
    if sfx == "f32":
        assert np.array_equal(hip.bc_pow(2.0, hip.toHip(ints)).toCpu(), 2.0 ** ints)
        assert np.array_equal(c.toCpu(), base * base)        # pow(x, 2) correctly rounded = the rounded square
    else:
        close(hip.bc_pow(2.0, hip.toHip(ints)).toCpu(), 2.0 ** ints, "2 ^. n")
    with np.errstate(invalid="ignore"):
        sp = hip.bc_pow(hip.toHip(np.array([-8.0, 0.0, np.inf, -1.0], dtype=dt)), 0.5).toCpu()
    assert np.isnan(sp[0]) and sp[1] == 0 and sp[2] == np.inf and np.isnan(sp[3])
    assert hip.bc_pow(hip.empty((0, 3), dt), 2.0).shape == (0, 3)


@pytest.mark.parametrize("sfx", FLT)
def test_float_mod(hip, oracle, sfx):
    """`mod` on float tensors (C fmod) is exact: the oracle's bits in every form, special values included."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, "fmod"))
    x = (rng.uniform(-1e4, 1e4, (64, 1030)) * 10.0 ** rng.integers(-3, 4, (64, 1030))).astype(dt)
    y = rng.uniform(-50, 50, (1, 1030)).astype(dt)
    dx, dy = hip.toHip(x), hip.toHip(y)
    say("float mod", sfx)
    bx, by = oracle.broadcast2(x, y)
    assert np.array_equal(hip.bc_mod(dx, dy).toCpu(), oracle.map2("mod", bx, by))
    assert np.array_equal(hip.bc_mod(dx, 3.5).toCpu(), oracle.scalar_op("mod", x, 3.5))
    assert np.array_equal(hip.bc_mod(3.5, dx.transpose()).toCpu(), oracle.scalar_op("mod", x.T, 3.5, scalar_on_left=True))
    a, b = np.array([5.5, -5.5, 1.0, np.inf, -0.0, 7.0], dtype=dt), np.array([2.0, 2.0, 0.0, 2.0, 3.0, np.inf], dtype=dt)
    with np.errstate(invalid="ignore"):
        want = np.fmod(a, b)
    got = hip.bc_mod(hip.toHip(a), hip.toHip(b)).toCpu()
    ok = ~np.isnan(want)                         # the sign of a NaN is not specified
    assert np.array_equal(got, want, equal_nan=True) and np.array_equal(np.signbit(got)[ok], np.signbit(want)[ok])


def test_pow_and_ufunc_errors(hip):
    ti = hip.toHip(np.arange(6, dtype=np.int32))
    tf = hip.toHip(np.arange(6, dtype=np.float32))
    for call in (lambda: hip.bc_pow(ti, 2), lambda: hip.bc_pow(tf, tf), lambda: hip.bc_pow(2.0, 3.0),
                 lambda: hip.ln(ti), lambda: hip.unary("floor", ti), lambda: hip.scalar_op("pow", ti, 2),
                 lambda: hip.map2("pow", ti, ti), lambda: ti.bc_ipow(2), lambda: hip.mreciprocal(ti)):
        with pytest.raises(TypeError):
            call()


@pytest.mark.parametrize("sfx", ALL)
def test_clamp(hip, oracle, sfx):
    """clamp / mclamp in one pass (bounds as zero-stride operands), any element type, any strides."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of(sfx, "clamp"))
    x = rng.uniform(-100, 100, (70, 1030)).astype(dt)
    dx = hip.toHip(x)
    say("clamp", sfx)
    want = oracle.map3("clamp", x, np.broadcast_to(dt(-25), x.shape), np.broadcast_to(dt(40), x.shape))
    assert np.array_equal(want, np.clip(x, -25, 40))
    assert np.array_equal(hip.clamp(dx, -25, 40).toCpu(), want)
    assert np.array_equal(hip.clamp(dx.transpose(), -25, 40).toCpu(), want.T)
    assert np.array_equal(hip.clamp(dx[:, 5:77], -25, 40).toCpu(), want[:, 5:77])
    v = dx[:, 4:1028]
    assert hip.mclamp(v, -25, 40) is v
    got = dx.toCpu()
    assert np.array_equal(got[:, 4:1028], want[:, 4:1028]) and np.array_equal(got[:, :4], x[:, :4])
    assert hip.clamp(hip.empty((0, 4), dt), 0, 1).shape == (0, 4)
    if sfx in FLT:
        s = hip.clamp(hip.toHip(np.array([np.nan, -np.inf, np.inf, -0.0, 5.0], dtype=dt)), 0, 1).toCpu()
        assert np.isnan(s[0]) and s[1] == 0 and s[2] == 1 and s[3] == 0 and np.signbit(s[3]) and s[4] == 1


def test_more_than_2_pow_31_elements(hip):
    """A destination of 2^31 + 2^20 int32 elements (8 GiB): the streaming kernel's row / tile counters and the
    generic kernel's switch from 32- to 64-bit element indices are both past 2^31 here. Written through
    zero-stride (broadcast) operands and checked by folds on the device, so nothing of that size is copied."""
    n_rows, L = (1 << 15) + 16, 1 << 16                      # 32784 x 65536 = 2^31 + 2^20 elements
    col = np.arange(n_rows, dtype=np.int32).reshape(n_rows, 1) % 7 - 3
    row = (np.arange(L, dtype=np.int32).reshape(1, L) % 5) * 11
    dcol, drow = hip.toHip(col), hip.toHip(row)
    say("8 GiB destination, streaming kernel")
    big = hip.bc_add(dcol, drow)                             # [n_rows, L], rows kernel (row vector + one scalar per row)
    assert big.size > 2**31
    want_sum = int(col.astype(np.int64).sum()) * L + int(row.astype(np.int64).sum()) * n_rows
    wrap = lambda v: ((v + 2**31) % 2**32) - 2**31
    assert int(hip.sum(big)) == wrap(want_sum)               # int32 sums wrap
    assert int(hip.max(big)) == int(col.max() + row.max()) and int(hip.min(big)) == int(col.min() + row.min())
    # the first and the last row, each through a small device-side gather (toCpu of a view copies its whole storage)
    assert np.array_equal(big[:1, :].clone().toCpu(), col[:1] + row)
    assert np.array_equal(big[n_rows - 1:, :].clone().toCpu(), col[n_rows - 1:] + row)
    del big
    say("8 GiB destination, generic kernel (64-bit element index)")
    # inner stride -1 on an operand sends the same shape to the generic kernel
    rrow = hip.toHip(row[:, ::-1].copy())[:, ::-1]           # the same values seen through a reversed view
    big2 = hip.bc_add(dcol, rrow)
    assert int(hip.sum(big2)) == wrap(want_sum)
    assert np.array_equal(big2[n_rows - 1:, :].clone().toCpu(), col[n_rows - 1:] + row)
    assert np.array_equal(big2[:1, :].clone().toCpu(), col[:1] + row)


@pytest.mark.parametrize("sfx", ["i32", "i64"])
def test_fac(hip, oracle, sfx):
    """fac (tensor/ufunc.nim:84-85): n! of every element, 0 .. 20, bit for bit against the oracle (int32 wraps from 13!
    on) on contiguous and strided operands; an element outside the table's range raises, like Nim's assertion."""
    import math
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("fac", sfx))
    n = np.arange(0, 21).astype(dt)
    got = hip.fac(hip.toHip(n)).toCpu()
    assert got.tolist() == oracle.unary("fac", n).tolist()
    if sfx == "i64":
        assert got.tolist() == [math.factorial(int(k)) for k in n]
    a = rng.integers(0, 21, (257, 130)).astype(dt)
    da = hip.toHip(a)
    assert np.array_equal(hip.fac(da).toCpu(), oracle.unary("fac", a))
    assert np.array_equal(hip.fac(da.transpose()[3:, ::2]).toCpu(), oracle.unary("fac", np.ascontiguousarray(a.T[3:, ::2])))
    for bad in (-1, 21):
        b = a.copy()
        b[100, 7] = bad
        with pytest.raises(ValueError):
            hip.fac(hip.toHip(b))
    with pytest.raises(TypeError):
        hip.fac(hip.zeros((2, 2), np.float32))
    assert hip.fac(hip.zeros((0, 3), dt)).shape == (0, 3)


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_sgd_update_of_many_tensors_in_one_launch(hip, sfx):
    """am_hip_sgd_update_*: value - lr * gradient over a list of tensors (optimizers.nim:35-51 runs one pass per
    parameter) bit for bit against NumPy's same expression: sizes around the 4096-element pieces and the 16-byte
    vectors, an empty tensor in the list, more tensors than one launch takes, an unaligned window of a wider buffer."""
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("sgd", sfx))
    sizes = [1, 3, 4, 5, 500, 4095, 4096, 4097, 8191, 10, 0, 12289, 400_000] + [int(n) for n in rng.integers(1, 300, 70)]
    vals = [rng.standard_normal(n).astype(dt) for n in sizes]
    grads = [rng.standard_normal(n).astype(dt) for n in sizes]
    dv, dg = [hip.toHip(v) for v in vals], [hip.toHip(g) for g in grads]
    lr = dt(0.0375)
    hip.sgd_update(dv, dg, float(lr))
    for v, g, d, n in zip(vals, grads, dv, sizes):
        assert np.array_equal(d.toCpu(), v - lr * g), n
    # 2-D parameters and a window that starts at an odd element
    w, gw = rng.standard_normal((37, 53)).astype(dt), rng.standard_normal((37, 53)).astype(dt)
    wide = rng.standard_normal(1001).astype(dt)
    dwide = hip.toHip(wide)
    gwin = rng.standard_normal(998).astype(dt)
    dw = hip.toHip(w)
    hip.sgd_update([dw, dwide[3:]], [hip.toHip(gw), hip.toHip(gwin)], 0.5)
    assert np.array_equal(dw.toCpu(), w - dt(0.5) * gw)
    expect = wide.copy()
    expect[3:] = wide[3:] - dt(0.5) * gwin
    assert np.array_equal(dwide.toCpu(), expect)
    with pytest.raises(ValueError):
        hip.sgd_update([dw], [hip.toHip(gw.T.copy())], 0.1)                 # shapes differ
    with pytest.raises(ValueError):
        hip.sgd_update([dw.transpose()], [hip.toHip(gw).transpose()], 0.1)  # not contiguous
    with pytest.raises(TypeError):
        hip.sgd_update([hip.zeros((3,), np.int32)], [hip.zeros((3,), np.int32)], 0.1)
    hip.sgd_update([], [], 0.1)
