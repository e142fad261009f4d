"""The forward pass of the reference's example 2 (examples/ex02_handwritten_digits_recognition.nim:36-46) on the
device against the same chain through the oracle: every stage on the device's own input for that stage (max-pooling
indices must then be identical), the whole chain end to end, eagerly and replayed from one HIP graph."""
import numpy as np
import pytest

from conftest import seed_of

pytestmark = pytest.mark.gpu
TOL = {"f32": 1e-4, "f64": 1e-12}     # relative Frobenius norm
DT = {"f32": np.float32, "f64": np.float64}


def say(*a):
    print(*a, flush=True)


def relu(oracle, x):
    return oracle.unary("relu", x)


def dense(oracle, x, w, b, act):
    out = oracle.matmul(x, w.T)                                    # nnp_linear.nim:20-29: x * weight.transpose, +.= bias
    out = oracle.map2("add", out, oracle.broadcast(b, out.shape))
    return relu(oracle, out) if act else out


def oracle_stages(oracle, x, p):
    """[(name, value)] of every stage of the chain, computed by the oracle from x."""
    a1 = relu(oracle, oracle.conv2d(x, p["cv1_w"], p["cv1_b"]))
    i1, p1 = oracle.maxpool2d(a1, (2, 2), (0, 0), (2, 2))
    a2 = relu(oracle, oracle.conv2d(p1, p["cv2_w"], p["cv2_b"]))
    i2, p2 = oracle.maxpool2d(a2, (2, 2), (0, 0), (2, 2))
    h = dense(oracle, p2.reshape(x.shape[0], -1), p["hidden_w"], p["hidden_b"], True)
    y = dense(oracle, h, p["classifier_w"], p["classifier_b"], False)
    return dict(a1=a1, idx1=i1, pool1=p1, a2=a2, idx2=i2, pool2=p2, hidden=h, logits=y)


@pytest.mark.parametrize("sfx", ["f32", "f64"])
@pytest.mark.parametrize("batch", [64, 3])
def test_ex02_forward(hip, oracle, sfx, batch):
    from arraymancer_amd import ex02
    dt = DT[sfx]
    rng = np.random.default_rng(seed_of("ex02", sfx, batch))
    p = ex02.random_params(rng, dt)
    x = rng.uniform(0, 1, (batch, 1, 28, 28)).astype(dt)
    say("ex02 forward", sfx, "batch", batch)
    net = ex02.DemoNet(batch, p, dt)
    dx = hip.toHip(x)
    logits = net.forward(dx).toCpu()
    assert logits.shape == (batch, 10)
    got = {n: getattr(net, n).toCpu() for n in ("a1", "idx1", "pool1", "a2", "idx2", "pool2", "hidden", "logits")}

    # end to end against the oracle's own chain
    want = oracle_stages(oracle, x, p)
    for name in ("a1", "pool1", "a2", "pool2", "hidden", "logits"):
        err = oracle.rel_frobenius(got[name], want[name])
        say(f"  end to end {name}: {err:.2e}")
        assert err <= TOL[sfx], name

    # stage by stage on the device's own inputs: pooling is exact, indices included
    for src, idx, out in (("a1", "idx1", "pool1"), ("a2", "idx2", "pool2")):
        wi, wo = oracle.maxpool2d(got[src], (2, 2), (0, 0), (2, 2))
        assert np.array_equal(got[idx], wi), idx
        assert np.array_equal(got[out], wo), out
    assert oracle.rel_frobenius(got["a2"], relu(oracle, oracle.conv2d(got["pool1"], p["cv2_w"], p["cv2_b"]))) <= TOL[sfx]
    flat = got["pool2"].reshape(batch, -1)
    assert oracle.rel_frobenius(got["hidden"], dense(oracle, flat, p["hidden_w"], p["hidden_b"], True)) <= TOL[sfx]
    assert oracle.rel_frobenius(got["logits"], dense(oracle, got["hidden"], p["classifier_w"], p["classifier_b"], False)) <= TOL[sfx]
    assert (got["a1"] >= 0).all() and (got["a2"] >= 0).all() and (got["hidden"] >= 0).all()

    # one HIP graph of the whole pass: every replay gives the eager result bit for bit, also after the input changed
    say("  graph replays")
    g = net.capture(dx)
    for rep in range(3):
        dx2 = hip.toHip(rng.uniform(0, 1, x.shape).astype(dt))
        eager = net.forward(dx2).toCpu().copy()
        hip.tensor_hip._unary_into("copy", dx, dx2)      # the graph reads dx: new values at the same address
        g.launch()
        hip.sync()
        assert np.array_equal(net.logits.toCpu(), eager), f"replay {rep}"


def oracle_backward(oracle, x, labels, p):
    """Loss and parameter gradients of one learning step through the oracle's primitives, in the reference's order."""
    st = oracle_stages(oracle, x, p)
    n = x.shape[0]
    loss = oracle.sparse_softmax_cross_entropy(st["logits"], labels)
    d_logits = oracle.sparse_softmax_cross_entropy_backward(1, st["logits"], labels)

    def linear_bwd(inp, w, go):                                   # nnp_linear.nim:39-55
        return oracle.matmul(go, w), oracle.matmul(go.T, inp), oracle.reduce_axis("sum", go, 0)

    relu_bwd = lambda g, cached: oracle.map2("relu_bwd", cached, g)   # nnp_activation.nim:65-70
    d_hidden, g_cw, g_cb = linear_bwd(st["hidden"], p["classifier_w"], d_logits)
    d_hidden = relu_bwd(d_hidden, st["hidden"])
    d_flat, g_hw, g_hb = linear_bwd(st["pool2"].reshape(n, -1), p["hidden_w"], d_hidden)
    d_a2 = oracle.maxpool2d_backward(st["a2"].shape, st["idx2"], np.ascontiguousarray(d_flat.reshape(st["pool2"].shape)))
    d_a2 = relu_bwd(d_a2, st["a2"])
    d_pool1, g_k2, g_b2 = oracle.conv2d_backward(st["pool1"], p["cv2_w"], p["cv2_b"], (0, 0), (1, 1), d_a2)
    d_a1 = oracle.maxpool2d_backward(st["a1"].shape, st["idx1"], d_pool1)
    d_a1 = relu_bwd(d_a1, st["a1"])
    _, g_k1, g_b1 = oracle.conv2d_backward(x, p["cv1_w"], p["cv1_b"], (0, 0), (1, 1), d_a1)
    return loss, dict(cv1_w=g_k1, cv1_b=g_b1, cv2_w=g_k2, cv2_b=g_b2, hidden_w=g_hw, hidden_b=g_hb, classifier_w=g_cw, classifier_b=g_cb)


@pytest.mark.parametrize("sfx", ["f32", "f64"])
def test_ex02_training_step(hip, oracle, sfx):
    """One step of the example's learning loop (examples/ex02_handwritten_digits_recognition.nim:58-72) on the device:
    forward, sparse softmax cross-entropy, the backward primitives in reverse order, the SGD update. The gradients
    against the same chain through the oracle; in float64 also against central differences of the oracle's loss for
    a few entries of every parameter; the update bit for bit against x - lr * y; and the loss of a fixed batch goes down."""
    from arraymancer_amd import ex02
    dt, batch = DT[sfx], 16
    rng = np.random.default_rng(seed_of("ex02-train", sfx))
    p = ex02.random_params(rng, dt)
    x = rng.uniform(0, 1, (batch, 1, 28, 28)).astype(dt)
    labels = rng.integers(0, 10, batch).astype(np.int64)
    net = ex02.DemoNet(batch, p, dt)
    dx, dl = hip.toHip(x), hip.toHip(labels)
    say("ex02 training step", sfx)
    loss, grads = net.loss_and_gradients(dx, dl)
    want_loss, want = oracle_backward(oracle, x, labels, p)
    assert abs(loss - want_loss) <= (1e-5 if sfx == "f32" else 1e-12) * max(1.0, abs(want_loss))
    for name, g in grads.items():
        assert g.shape == p[name].shape, name
        err = oracle.rel_frobenius(g.toCpu(), want[name].reshape(p[name].shape))
        say(f"  gradient of {name}: {err:.2e}")
        assert err <= (2e-4 if sfx == "f32" else 1e-11), name
    if sfx == "f64":
        def loss_at():
            return float(oracle.sparse_softmax_cross_entropy(oracle_stages(oracle, x, p)["logits"], labels))
        for name in p:
            flat = p[name].reshape(-1)
            got = grads[name].toCpu().reshape(-1)
            for i in rng.choice(flat.size, 3, replace=False):
                keep = flat[i]
                flat[i] = keep + 1e-5; up = loss_at()
                flat[i] = keep - 1e-5; dn = loss_at()
                flat[i] = keep
                num = (up - dn) / 2e-5
                assert abs(got[i] - num) <= 1e-6 * max(1e-3, abs(num)), (name, i, got[i], num)
    before = {k: v.toCpu().copy() for k, v in net.p.items()}
    host_grads = {k: g.toCpu().copy() for k, g in grads.items()}
    net.sgd_update(grads, 0.01)
    for name in p:
        assert np.array_equal(net.p[name].toCpu(), before[name] - dt(0.01) * host_grads[name].reshape(before[name].shape)), name
    losses = [float(loss)] + [float(net.train_step(dx, dl, 0.01)) for _ in range(5)]
    say("  losses over six steps on one batch:", [round(v, 4) for v in losses])
    assert losses[-1] < losses[0]


def test_ex02_training_step_as_one_graph(hip):
    """The whole learning step (forward, backward, SGD update; about forty kernels with their temporaries) recorded
    into ONE graph by Graph.record - a rehearsal that leaves the allocator one cached block per allocation, then the
    capture served from that cache - against the same steps issued one by one: parameters bit for bit after every
    step, with new images and labels in the same buffers each time; the recording itself must not count as a step."""
    from arraymancer_amd import ex02
    dt, batch = np.float32, 32
    rng = np.random.default_rng(seed_of("ex02-train-graph"))
    p = ex02.random_params(rng, dt)
    eager, replayed = ex02.DemoNet(batch, p, dt), ex02.DemoNet(batch, p, dt)
    x, labels = hip.empty((batch, 1, 28, 28), dt), hip.empty((batch,), np.int64)
    first_x, first_l = rng.uniform(0, 1, (batch, 1, 28, 28)).astype(dt), rng.integers(0, 10, batch).astype(np.int64)
    hip.tensor_hip._unary_into("copy", x, hip.toHip(first_x))
    hip.tensor_hip._unary_into("copy", labels, hip.toHip(first_l))
    say("ex02 training step as a graph: recording")
    graph = replayed.capture_train_step(x, labels, 0.05)
    for name in p:
        assert np.array_equal(replayed.p[name].toCpu(), np.asarray(p[name], dtype=dt).reshape(replayed.p[name].shape)), name
    live0, _ = memory(hip)
    for step in range(4):
        hx, hl = rng.uniform(0, 1, (batch, 1, 28, 28)).astype(dt), rng.integers(0, 10, batch).astype(np.int64)
        hip.tensor_hip._unary_into("copy", x, hip.toHip(hx))
        hip.tensor_hip._unary_into("copy", labels, hip.toHip(hl))
        eager.train_step(x, labels, 0.05)
        graph.launch()
        hip.sync()
        for name in p:
            assert np.array_equal(replayed.p[name].toCpu(), eager.p[name].toCpu()), (step, name)
    live1, _ = memory(hip)
    assert live1 <= live0, "replays must not allocate"
    # a sequence that was not rehearsed finds no cached block of an unusual size: a clear error, and the capture ends cleanly
    del graph, replayed, eager
    assert hip.load_library().am_hip_empty_cache() == 0
    with pytest.raises(hip.HipAllocError):
        with hip.Graph():
            hip.empty((12345, 77), np.float64)
    assert hip.empty((4,), dt).shape == (4,)


def memory(hip):
    import ctypes
    live, cached = ctypes.c_size_t(), ctypes.c_size_t()
    hip.load_library().am_hip_memory_stats(ctypes.byref(live), ctypes.byref(cached))
    return live.value, cached.value
