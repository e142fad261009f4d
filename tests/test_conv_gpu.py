"""Device im2col + strided-batched GEMM (+ fused bias / ReLU) against the oracle's per-image
restatement of the reference's convolution, and the batched GEMM entry point on its own."""
import numpy as np
import pytest

from conftest import DTYPES, seed_of

pytestmark = pytest.mark.gpu
ALL = ["f32", "f64", "i32", "i64"]
TOL = {"f32": 1e-4, "f64": 1e-12}


def say(*a):
    print(*a, flush=True)


def fill(rng, shape, dt):
    if np.dtype(dt).kind == "f":
        return rng.uniform(-1, 1, size=shape).astype(dt)
    return rng.integers(-100, 100, size=shape, endpoint=True).astype(dt)


def check(oracle, sfx, got, want, what=""):
    if sfx in ("i32", "i64"):
        assert np.array_equal(got, want), what
    else:
        assert oracle.rel_frobenius(got, want) <= TOL[sfx], what


@pytest.mark.parametrize("sfx", ALL)
def test_reference_conv_literals(hip, vectors, sfx):
    dt = DTYPES[sfx]
    for case in vectors["conv_im2col"]:
        say("conv literal", case["name"], sfx)
        x, k, b = (hip.toHip(np.array(case[n], dtype=dt)) for n in ("input", "kernel", "bias"))
        out = hip.conv2d(x, k, b, tuple(case["padding"]), tuple(case["stride"]))
        assert np.array_equal(out.toCpu(), np.array(case["target"], dtype=dt)), case["name"]


GEOMS = [  # N, C, H, W, C_out, kH, kW, pad, stride
    (1, 1, 5, 5, 1, 3, 3, (0, 0), (1, 1)),
    (3, 2, 9, 7, 4, 3, 2, (1, 0), (2, 1)),
    (8, 3, 16, 16, 8, 5, 5, (2, 2), (1, 1)),
    (64, 1, 28, 28, 20, 5, 5, (0, 0), (1, 1)),      # MNIST conv1 of the reference's example (24 x 24 = 576 outputs)
    (16, 20, 12, 12, 50, 5, 5, (0, 0), (1, 1)),     # conv2 (8 x 8 = 64 outputs)
    (2, 3, 4, 8, 2, 3, 3, (0, 0), (1, 1)),          # 2 x 6 outputs: 16-byte groups of pixels straddle the output rows
    (4, 2, 16, 16, 3, 3, 3, (1, 1), (2, 2)),        # stride 2 with padding, 8 x 8 outputs
    (2, 5, 11, 13, 70, 1, 1, (0, 0), (1, 1)),       # 1 x 1 kernel (k is the channel alone), more output channels than a small tile
    (3, 8, 20, 20, 130, 3, 5, (2, 3), (1, 2)),      # padding wider than the kernel's reach on one side, 130 output channels
    (2, 16, 40, 40, 32, 3, 3, (1, 1), (1, 1)),      # 1600 outputs per image: the larger tiles
]


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("geom", GEOMS)
def test_im2col_and_conv_vs_oracle(hip, oracle, sfx, geom):
    dt = DTYPES[sfx]
    N, C, H, W, co, kh, kw, pad, stride = geom
    rng = np.random.default_rng(seed_of("conv", sfx, geom))
    x, k, b = fill(rng, (N, C, H, W), dt), fill(rng, (co, C, kh, kw), dt), fill(rng, (co,), dt)
    dx = hip.toHip(x)
    say("im2col", sfx, geom)
    col = hip.im2col(dx, (kh, kw), pad, stride).toCpu()
    for n in (0, N - 1):
        assert np.array_equal(col[n], oracle.im2col(x[n], (kh, kw), pad, stride))
    say("conv2d", sfx, geom)
    want = oracle.conv2d(x, k, b, pad, stride)
    # floats: the one-launch form (column matrix gathered by the GEMM's loader) and the im2col + batched GEMM form;
    # integers only have the second
    forms = (True, False, None) if sfx in ("f32", "f64") and C * kh * kw * np.dtype(dt).itemsize >= 16 else (False, None)
    for fused in forms:
        got = hip.conv2d(dx, hip.toHip(k), hip.toHip(b), pad, stride, fused=fused).toCpu()
        check(oracle, sfx, got, want, f"conv + bias, fused={fused}")
        got = hip.conv2d(dx, hip.toHip(k), hip.toHip(b), pad, stride, relu=True, fused=fused).toCpu()
        check(oracle, sfx, got, np.where(0 >= want, np.zeros_like(want), want), f"conv + bias + relu, fused={fused}")
        got = hip.conv2d(dx, hip.toHip(k), None, pad, stride, fused=fused).toCpu()
        check(oracle, sfx, got, oracle.conv2d(x, k, None, pad, stride), f"conv, fused={fused}")
        # a channel-sliced (strided) input goes through the same kernel
        if C > 1:
            got = hip.conv2d(dx[:, ::-1], hip.toHip(np.ascontiguousarray(k[:, ::-1])), None, pad, stride, fused=fused).toCpu()
            check(oracle, sfx, got, oracle.conv2d(x, k, None, pad, stride), f"reversed channels, fused={fused}")


@pytest.mark.parametrize("sfx", ALL)
def test_gemm_batched(hip, oracle, sfx):
    dt = DTYPES[sfx]
    rng = np.random.default_rng(seed_of("batched", sfx))
    batch, M, N, K = 7, 45, 52, 36
    A, B, C = fill(rng, (batch, M, K), dt), fill(rng, (batch, K, N), dt), fill(rng, (batch, M, N), dt)
    say("batched", sfx)
    dC = hip.toHip(C)
    hip.gemm_batched(2, hip.toHip(A), hip.toHip(B), 3, dC)
    want = np.stack([oracle.gemm_strided(2, A[z], B[z], 3, C[z].copy()) for z in range(batch)])
    check(oracle, sfx, dC.toCpu(), want, "batched")
    say("batched shared A, transposed B", sfx)
    Bt = np.ascontiguousarray(B.transpose(0, 2, 1))
    dC = hip.toHip(C)
    dBt = hip.toHip(Bt)
    dB_view = type(dBt)(hip.Layout((batch, K, N), (dBt.strides[0], dBt.strides[2], dBt.strides[1]), 0), dBt.storage, dBt.dtype)
    hip.gemm_batched(1, hip.toHip(A[0]), dB_view, 0, dC)
    want = np.stack([oracle.matmul(A[0], B[z]) for z in range(batch)])
    check(oracle, sfx, dC.toCpu(), want, "shared A")
    with pytest.raises(IndexError):
        hip.gemm_batched(1, hip.toHip(A[:3]), hip.toHip(B), 0, dC)
