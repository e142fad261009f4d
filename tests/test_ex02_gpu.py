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
