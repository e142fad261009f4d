"""The GRU primitives on the GPU (src/arraymancer/nn_primitives/nnp_gru.nim): the reference's own vectors
(tests/nn_primitives/test_nnp_gru.nim:10-57 one cell, :178-268 two stacked layers over four timesteps, values it took
from PyTorch / cuDNN, mean relative error below 1e-8 in float64), the cell's backward pass against the numerical
gradient of the forward pass as the reference checks it (:78-172, mean absolute error below 1e-8), and larger random
cells against the same chain through the oracle's operators."""
import numpy as np
import pytest

from conftest import seed_of

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


X = [[0.1, 0.2, 0.3, 0.4], [-0.1, -0.2, -0.3, -0.4], [0.5, 0.6, 0.7, 0.8]]
HIDDEN = [[-1.0, -1.0]] * 3
W3 = [[0.9, 0.8, 0.7, 0.6], [0.8, 0.7, 0.6, 0.5], [0.7, 0.6, 0.5, 0.4], [0.6, 0.5, 0.4, 0.3], [0.5, 0.4, 0.3, 0.2], [0.4, 0.3, 0.2, 0.1]]
U3 = [[-0.3, -0.1], [-0.2, 0.0], [-0.3, -0.1], [-0.2, 0.0], [-0.3, -0.1], [-0.2, 0.0]]
BW3 = [[0.1, 0.2, 0.3, 0.4, 0.5, 0.6]]
BU3 = [[-0.1, -0.2, -0.3, -0.4, -0.5, -0.6]]
PYTORCH_CELL = [[-0.5317437280, -0.4752916969], [-0.3930421219, -0.3209550879], [-0.7325259335, -0.6429624731]]


def mean_relative_error(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = np.maximum(np.abs(got), np.abs(want))
    return np.mean(np.where(d == 0, 0.0, np.abs(got - want) / np.where(d == 0, 1.0, d)))


@pytest.mark.parametrize("dt,tol", [(np.float64, 1e-8), (np.float32, 1e-6)])
def test_cell_reference_vectors(hip, dt, tol):
    arrs = [np.array(v, dtype=dt) for v in (X, W3, U3, BW3, BU3)]
    dev = [hip.toHip(a) for a in arrs]
    h = hip.toHip(np.array(HIDDEN, dtype=dt))
    assert hip.gru_cell_inference(*dev, h) is h
    assert mean_relative_error(h.toCpu(), PYTORCH_CELL) < tol
    h = hip.toHip(np.array(HIDDEN, dtype=dt))
    r, z, n, Uh = hip.gru_cell_forward(*dev, h)
    assert mean_relative_error(h.toCpu(), PYTORCH_CELL) < tol
    assert all(t.shape == (3, 2) for t in (r, z, n, Uh))
    # what was saved is what the forward pass used: h' = (1 - z) * n + z * h
    zz, nn = z.toCpu().astype(np.float64), n.toCpu().astype(np.float64)
    assert np.allclose((1 - zz) * nn + zz * np.array(HIDDEN), PYTORCH_CELL, rtol=0, atol=tol * 10)


SEQ_X = [[[0.1, 0.2, 0.3, 0.4, 0.5], [-0.1, -0.2, -0.3, -0.4, -0.5], [0.5, 0.6, 0.7, 0.8, 0.9]],
         [[-0.1, -0.2, -0.3, -0.4, -0.5], [-0.1, -0.2, -0.3, -0.4, -0.5], [0.5, 0.6, 0.7, 0.8, 0.9]],
         [[0.1, 0.2, 0.3, 0.4, 0.5], [-0.1, -0.2, -0.3, -0.4, -0.5], [-0.1, -0.2, -0.3, -0.4, -0.5]],
         [[-0.1, -0.2, -0.3, -0.4, -0.5], [-0.1, -0.2, -0.3, -0.4, -0.5], [-0.1, -0.2, -0.3, -0.4, -0.5]]]
SEQ_HIDDEN = [[[-1.0, -1.0]] * 3, [[2.0, 3.0]] * 3]
W3S0 = [[0.9, 0.8, 0.7, 0.6, 0.5], [0.8, 0.7, 0.6, 0.5, 0.4], [0.7, 0.6, 0.5, 0.4, 0.3], [0.6, 0.5, 0.4, 0.3, 0.2],
        [0.5, 0.4, 0.3, 0.2, 0.1], [0.4, 0.3, 0.2, 0.1, 0.0]]
W3SN = [[[0.5, 0.6], [0.4, 0.5], [0.3, 0.4], [0.2, 0.3], [0.1, 0.2], [0.0, 0.1]]]
U3S = [[[-0.3, -0.1], [-0.2, 0.0], [-0.3, -0.1], [-0.2, 0.0], [-0.3, -0.1], [-0.2, 0.0]],
       [[-0.4, -0.5], [-0.4, 0.5], [-0.4, -0.5], [-0.4, 0.5], [-0.4, -0.5], [-0.4, 0.5]]]
BW3S = [[[0.1, 0.2, 0.3, 0.4, 0.5, 0.6]], [[0.2, 0.3, 0.4, 0.2, 0.3, 0.4]]]
BU3S = [[[-0.1, -0.2, -0.3, -0.4, -0.5, -0.6]], [[0.1, 0.2, 0.3, 0.4, 0.5, 0.6]]]
PY_OUTPUT = [[[0.2564464804, 2.4324064858], [0.3212793315, 2.4821776260], [0.1983539289, 2.3849941275]],
             [[0.1323593874, 2.1939630024], [0.1591080583, 2.2447442148], [0.0683269257, 2.1121420346]],
             [[0.1233993158, 1.9977140846], [0.1320258443, 2.0434525564], [0.0904040251, 1.9111566097]],
             [[0.1355803839, 1.8195602154], [0.1369919053, 1.8612790359], [0.1230976350, 1.7381913793]]]
PY_HIDDEN_N = [[[0.0155439572, 0.1680427130], [-0.0038861287, 0.1854366532], [-0.0549487103, 0.1189245136]],
               [[0.1355803839, 1.8195602154], [0.1369919053, 1.8612790359], [0.1230976350, 1.7381913793]]]


@pytest.mark.parametrize("dt,tol", [(np.float64, 1e-8), (np.float32, 2e-6)])
def test_stacked_sequence_reference_vectors(hip, dt, tol):
    dev = [hip.toHip(np.array(v, dtype=dt)) for v in (SEQ_X, W3S0, W3SN, U3S, BW3S, BU3S)]
    h = hip.toHip(np.array(SEQ_HIDDEN, dtype=dt))
    out = hip.gru_inference(*dev, h)
    assert out.shape == (4, 3, 2)
    assert mean_relative_error(out.toCpu(), PY_OUTPUT) < tol
    assert mean_relative_error(h.toCpu(), PY_HIDDEN_N) < tol
    # one layer alone: W3sN empty or None
    h1 = hip.toHip(np.array(SEQ_HIDDEN[:1], dtype=dt))
    one = hip.gru_inference(dev[0], dev[1], None, dev[3][0:1], dev[4][0:1], dev[5][0:1], h1)
    assert np.array_equal(one.toCpu()[-1], h1.toCpu()[0])
    assert mean_relative_error(h1.toCpu()[0], PY_HIDDEN_N[0]) < tol
    with pytest.raises(ValueError):
        hip.gru_inference(dev[0], dev[1], None, dev[3], dev[4], dev[5], h)


def oracle_cell(oracle, x, W3_, U3_, bW3, bU3, h):
    """gru_cell_inference through the oracle's GEMM and map bodies; returns (h', r, z, n, Uh)."""
    H = h.shape[1]
    W3x = oracle.map2("add", oracle.matmul(x, W3_.T), oracle.broadcast(bW3, (x.shape[0], 3 * H)))
    U3h = oracle.map2("add", oracle.matmul(h, U3_.T), oracle.broadcast(bU3, (x.shape[0], 3 * H)))
    Uh = U3h[:, 2 * H:].copy()
    rz = oracle.map2("add_sigmoid", np.ascontiguousarray(W3x[:, :2 * H]), np.ascontiguousarray(U3h[:, :2 * H]))
    r, z = np.ascontiguousarray(rz[:, :H]), np.ascontiguousarray(rz[:, H:])
    n = oracle.map3("gru_candidate", np.ascontiguousarray(W3x[:, 2 * H:]), r, Uh)
    return oracle.map3("gru_blend", h, z, n), r, z, n, Uh


@pytest.mark.parametrize("dt,B,F,H", [(np.float64, 3, 4, 2), (np.float64, 64, 100, 96), (np.float32, 128, 256, 512), (np.float32, 5, 7, 3)])
def test_cell_forward_and_backward(hip, oracle, dt, B, F, H):
    rng = np.random.default_rng(seed_of("gru-cell", np.dtype(dt).name, B, F, H))
    scale = 1.0 if F < 50 else 0.1
    x, h = rng.uniform(0, 1, (B, F)).astype(dt), rng.uniform(0, 1, (B, H)).astype(dt)
    W3_, U3_ = (rng.uniform(0, 1, (3 * H, F)) * scale).astype(dt), (rng.uniform(0, 1, (3 * H, H)) * scale).astype(dt)
    bW3, bU3 = rng.uniform(0, 1, (1, 3 * H)).astype(dt), rng.uniform(0, 1, (1, 3 * H)).astype(dt)
    f32 = dt == np.float32
    say("gru cell", np.dtype(dt).name, B, F, H)
    dev = [hip.toHip(a) for a in (x, W3_, U3_, bW3, bU3)]
    dh = hip.toHip(h)
    r, z, n, Uh = hip.gru_cell_forward(*dev, dh)
    want_h, wr, wz, wn, wUh = oracle_cell(oracle, x, W3_, U3_, bW3, bU3, h)
    tol = 2e-5 if f32 else 1e-12
    for got, want, name in ((dh, want_h, "h'"), (r, wr, "r"), (z, wz, "z"), (n, wn, "n"), (Uh, wUh, "Uh")):
        assert np.max(np.abs(got.toCpu() - want)) <= tol * max(1.0, np.max(np.abs(want))), name
    h2 = hip.toHip(h)
    hip.gru_cell_inference(*dev, h2)
    assert np.max(np.abs(h2.toCpu() - dh.toCpu())) <= tol
    dnext = rng.uniform(0.5, 1.5, (B, H)).astype(dt) if B > 3 else np.ones((B, H), dtype=dt)
    grads = hip.gru_cell_backward(hip.toHip(dnext), dev[0], hip.toHip(h), dev[1], dev[2], r, z, n, Uh)
    names = ("dx", "dh", "dW3", "dU3", "dbW3", "dbU3")
    shapes = (x.shape, h.shape, W3_.shape, U3_.shape, bW3.shape, bU3.shape)
    for g, name, shape in zip(grads, names, shapes):
        assert g.shape == shape, name
    if B * F <= 100 and not f32:
        # the reference's check: numerical gradient of sum(dnext * h') with respect to every input, float64
        params = [x, h, W3_, U3_, bW3, bU3]

        def objective():
            return float(np.sum(dnext * oracle_cell(oracle, params[0], params[2], params[3], params[4], params[5], params[1])[0]))

        for g, arr, name in zip(grads, params, names):
            num = np.zeros_like(arr)
            flat, nf = arr.reshape(-1), num.reshape(-1)
            for i in range(flat.size):
                keep = flat[i]
                flat[i] = keep + 1e-5; up = objective()
                flat[i] = keep - 1e-5; dn = objective()
                flat[i] = keep
                nf[i] = (up - dn) / 2e-5
            err = np.mean(np.abs(g.toCpu() - num))
            say(f"  {name}: mean absolute error against the numerical gradient {err:.2e}")
            assert err < 1e-8, name
    # the same formulas in extended precision from the saved tensors
    L = np.longdouble
    rr, zz, nn, uu, hh, dn_ = (a.astype(L) for a in (r.toCpu(), z.toCpu(), n.toCpu(), Uh.toCpu(), h, dnext))
    dz, dnn = (hh - nn) * dn_, (1 - zz) * dn_
    dWx = dnn * (1 - nn * nn)
    dr, dUh = uu * dWx, rr * dWx
    dWzx, dWrx = zz * (1 - zz) * dz, rr * (1 - rr) * dr
    dW3x, dU3h = np.concatenate([dWrx, dWzx, dWx], 1), np.concatenate([dWrx, dWzx, dUh], 1)
    want = (dW3x @ W3_.astype(L), dU3h @ U3_.astype(L) + dn_ * zz, dW3x.T @ x.astype(L), dU3h.T @ hh, dW3x.sum(0, keepdims=True), dU3h.sum(0, keepdims=True))
    for g, w, name in zip(grads, want, names):
        rel = np.linalg.norm((g.toCpu().astype(L) - w).astype(np.float64)) / max(np.linalg.norm(w.astype(np.float64)), 1e-30)
        assert rel <= (1e-4 if f32 else 1e-12), (name, rel)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_fused_gates_equal_the_three_passes(hip, dt):
    """am_hip_gru_gates_* against the three separate bodies of the reference's cell (apply2 sigmoid(x + y) on the reset
    and update columns, apply3 tanh(x + y * z), apply3 (1 - y) * z + y * x) bit for bit: aligned buffers (16-byte
    lanes) and products / hidden states that are windows of wider buffers at odd offsets (element lanes)."""
    from arraymancer_amd import tensor_hip as th
    rng = np.random.default_rng(seed_of("gru-gates", np.dtype(dt).name))
    for B, H, pad in ((3, 2, 0), (64, 96, 0), (17, 33, 0), (40, 64, 3), (5, 8, 1)):
        wide_w = rng.standard_normal((B, 3 * H + 2 * pad)).astype(dt)
        wide_u = rng.standard_normal((B, 3 * H + 2 * pad)).astype(dt)
        wide_h = rng.standard_normal((B, H + 2 * pad)).astype(dt)
        win3, win1 = slice(pad, pad + 3 * H), slice(pad, pad + H)
        # three passes, in place on copies
        W, U, h = hip.toHip(wide_w)[:, win3], hip.toHip(wide_u)[:, win3], hip.toHip(wide_h)[:, win1]
        hip.apply2("add_sigmoid", W[:, 0:2 * H], U[:, 0:2 * H])
        hip.apply3("gru_candidate", W[:, 2 * H:], W[:, 0:H], U[:, 2 * H:])
        hip.apply3("gru_blend", h, W[:, H:2 * H], W[:, 2 * H:])
        # one pass
        W2, U2 = hip.toHip(wide_w)[:, win3], hip.toHip(wide_u)[:, win3]
        parent_h = hip.toHip(wide_h)
        h2 = parent_h[:, win1]
        keep = tuple(hip.empty((B, H), dt) for _ in range(4))
        th._gru_gates_inplace(W2, U2, h2, keep)
        assert np.array_equal(h2.toCpu(), h.toCpu()), (B, H, pad)
        assert np.array_equal(keep[0].toCpu(), W.toCpu()[:, 0:H]) and np.array_equal(keep[1].toCpu(), W.toCpu()[:, H:2 * H])
        assert np.array_equal(keep[2].toCpu(), W.toCpu()[:, 2 * H:]) and np.array_equal(keep[3].toCpu(), wide_u[:, pad + 2 * H:pad + 3 * H])
        assert np.array_equal(W2.toCpu(), wide_w[:, win3])                       # the products are only read
        full = parent_h.toCpu()
        assert np.array_equal(full[:, :pad], wide_h[:, :pad]) and np.array_equal(full[:, pad + H:], wide_h[:, pad + H:])
        h3 = hip.toHip(wide_h)[:, win1]
        th._gru_gates_inplace(W2, U2, h3)                                        # nothing kept: same hidden state
        assert np.array_equal(h3.toCpu(), h.toCpu())
    with pytest.raises(ValueError):
        th._gru_gates_inplace(hip.zeros((2, 5), dt), hip.zeros((2, 6), dt), hip.zeros((2, 2), dt))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_fused_backward_gates_equal_the_separate_passes(hip, dt):
    """am_hip_gru_gates_backward_* against the reference's sequence of `-.`, `*.`, tanh_backward, sigmoid_backward and
    concat (nnp_gru.nim:165-186) run as separate launches: both [batch, 3H] gradients bit for bit, on shapes that take
    the 16-byte lanes and on ones that take the element lanes."""
    from arraymancer_amd import tensor_hip as th
    rng = np.random.default_rng(seed_of("gru-gates-bwd", np.dtype(dt).name))
    for B, H in ((3, 2), (64, 96), (17, 33), (128, 512)):
        host = [rng.uniform(-1, 1, (B, H)).astype(dt) for _ in range(6)]          # dnext, h, r, z, n, Uh
        dev = [hip.toHip(a) for a in host]
        want_w, want_u = hip.empty((B, 3 * H), dt), hip.empty((B, 3 * H), dt)
        th._gru_gates_backward_passes(*dev, want_w, want_u)
        x = hip.toHip(rng.uniform(-1, 1, (B, 5)).astype(dt))
        W3_, U3_ = hip.toHip(rng.uniform(-1, 1, (3 * H, 5)).astype(dt)), hip.toHip(rng.uniform(-1, 1, (3 * H, H)).astype(dt))
        dx, dh, dW3, dU3, dbW3, dbU3 = hip.gru_cell_backward(dev[0], x, dev[1], W3_, U3_, *dev[2:])
        # the dense layers' gradients are functions of the two gate-gradient buffers alone
        wx, wW, wb = hip.linear_backward(x, W3_, want_w)
        wh, wU, wbu = hip.linear_backward(dev[1], U3_, want_u)
        assert np.array_equal(dx.toCpu(), wx.toCpu()) and np.array_equal(dW3.toCpu(), wW.toCpu()) and np.array_equal(dbW3.toCpu(), wb.toCpu())
        assert np.array_equal(dU3.toCpu(), wU.toCpu()) and np.array_equal(dbU3.toCpu(), wbu.toCpu())
        assert np.array_equal(dh.toCpu(), (host[0] * host[3] + wh.toCpu()).astype(dt))
        # and the gate gradients themselves, against NumPy (single IEEE operations in the same order)
        dnext, h, r, z, n, Uh = host
        one = dt(1)
        dz, dn = (h - n) * dnext, (one - z) * dnext
        dWx = dn * (one - n * n)
        dr, dUh = Uh * dWx, r * dWx
        dWzx, dWrx = z * (one - z) * dz, r * (one - r) * dr
        assert np.array_equal(want_w.toCpu(), np.concatenate([dWrx, dWzx, dWx], 1))
        assert np.array_equal(want_u.toCpu(), np.concatenate([dWrx, dWzx, dUh], 1))


def oracle_gru(oracle, x, W3s0, W3sN, U3s, bW3s, bU3s, hidden):
    """gru_inference (nnp_gru.nim:194-262) cell by cell through the oracle's operators; returns (output, hiddenN)."""
    T = x.shape[0]
    layers = U3s.shape[0]
    h = hidden.copy()
    out = np.empty((T, x.shape[1], hidden.shape[2]), dtype=x.dtype)
    for layer in range(layers):
        W3l = W3s0 if layer == 0 else W3sN[layer - 1]
        for t in range(T):
            src = np.ascontiguousarray(x[t] if layer == 0 else out[t])
            h[layer] = oracle_cell(oracle, src, W3l, U3s[layer], bW3s[layer], bU3s[layer], np.ascontiguousarray(h[layer]))[0]
            out[t] = h[layer]
    return out, h


@pytest.mark.parametrize("layers,T", [(1, 1), (1, 4), (2, 1), (2, 3), (3, 2)])
def test_sequence_forward_and_backward(hip, oracle, layers, T):
    """gru_forward / gru_backward (nnp_gru.nim:263-500) the way the reference checks them (test_nnp_gru.nim:295-470):
    forward equal to the inference pass, and every gradient against central differences of
    sum(wo * output) + sum(wh * hiddenN) through the inference pass, float64, for stacks of one to three layers."""
    B, F, H = 3, 4, 2
    rng = np.random.default_rng(seed_of("gru-seq", layers, T))
    u = lambda *s: rng.uniform(0, 1, s)
    x, hidden = u(T, B, F), u(layers, B, H)
    W3s0, W3sN, U3s = u(3 * H, F), u(max(layers - 1, 0), 3 * H, H), u(layers, 3 * H, H)
    bW3s, bU3s = u(layers, 1, 3 * H), u(layers, 1, 3 * H)
    wo, wh = u(T, B, H), u(layers, B, H)                   # the gradients flowing back
    say("gru sequence", layers, "layers", T, "steps")
    dev = lambda a: hip.toHip(a)
    dWN = dev(W3sN) if layers > 1 else None
    h = dev(hidden)
    out, cache = hip.gru_forward(dev(x), dev(W3s0), dWN, dev(U3s), dev(bW3s), dev(bU3s), h)
    want_out, want_h = oracle_gru(oracle, x, W3s0, W3sN, U3s, bW3s, bU3s, hidden)
    assert np.max(np.abs(out.toCpu() - want_out)) < 1e-12 and np.max(np.abs(h.toCpu() - want_h)) < 1e-12
    h2 = dev(hidden)
    assert np.max(np.abs(hip.gru_inference(dev(x), dev(W3s0), dWN, dev(U3s), dev(bW3s), dev(bU3s), h2).toCpu() - out.toCpu())) < 1e-13
    grads = hip.gru_backward(dev(wo), dev(wh), cache, dev(W3s0), dWN, dev(U3s))
    params = dict(dInput=x, dHidden0=hidden, dW3s0=W3s0, dW3sN=W3sN, dU3s=U3s, dbW3s=bW3s, dbU3s=bU3s)

    def objective():
        o, hn = oracle_gru(oracle, x, W3s0, W3sN, U3s, bW3s, bU3s, hidden)
        return float(np.sum(wo * o) + np.sum(wh * hn))

    for got, (name, arr) in zip(grads, params.items()):
        if arr.size == 0:
            assert got is None, name
            continue
        assert got.shape == arr.shape, name
        num = np.zeros_like(arr)
        flat, nf = arr.reshape(-1), num.reshape(-1)
        for i in range(flat.size):
            keep = flat[i]
            flat[i] = keep + 1e-5; up = objective()
            flat[i] = keep - 1e-5; dn = objective()
            flat[i] = keep
            nf[i] = (up - dn) / 2e-5
        err = np.mean(np.abs(got.toCpu() - num))
        say(f"  {name}: mean absolute error against the numerical gradient {err:.2e}")
        assert err < 1e-8, name
