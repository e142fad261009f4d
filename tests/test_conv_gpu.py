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
    (2, 4, 6, 4, 5, 3, 3, (1, 1), (1, 1)),          # image rows of one 16-byte float vector: every gathered vector but the middle one hangs over an edge
    (2, 3, 7, 12, 6, 2, 5, (0, 4), (1, 1)),         # padding as wide as a float vector: vectors wholly in the padding beside partial ones (16 outputs per row)
    (1, 2, 5, 6, 3, 1, 3, (0, 2), (2, 1)),          # unit stride along the width only, rows 6 wide: a hanging vector is shifted by up to 2 either way
    (3, 24, 28, 28, 40, 3, 3, (1, 1), (1, 1)),      # 784 outputs: whole tiles and an edge tile of 16 columns
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
        if fused:
            # every other column of an image twice as wide: the one-element gathers, where the contiguous image may take
            # 16-byte ones; the products are added in the same order, so the results agree to the bit
            wide = np.zeros((N, C, H, 2 * W), dt)
            wide[..., ::2] = x
            spaced = hip.conv2d(hip.toHip(wide)[:, :, :, ::2], hip.toHip(k), None, pad, stride, fused=True).toCpu()
            assert np.array_equal(spaced, got), "one-element and 16-byte gathers differ"
        # a channel-sliced (strided) input goes through the same kernel
        if C > 1:
            got = hip.conv2d(dx[:, ::-1], hip.toHip(np.ascontiguousarray(k[:, ::-1])), None, pad, stride, fused=fused).toCpu()
            check(oracle, sfx, got, oracle.conv2d(x, k, None, pad, stride), f"reversed channels, fused={fused}")


@pytest.mark.parametrize("geom", [(3, 8, 24, 24, 130, 3, 3, (1, 1), (1, 1)), (2, 6, 9, 11, 200, 3, 2, (1, 1), (2, 1))])
def test_fused_conv_tiles(hip, oracle, geom, monkeypatch):
    """Every workgroup tile of the one-launch float32 convolution, forced in turn on 130 and 200 output channels (edge
    tiles in both directions), with 16-byte gathers (first geometry) and one-element gathers (second): the oracle's
    result from each, and the same bits from the tiles that use the same matrix instruction."""
    N, C, H, W, co, kh, kw, pad, stride = geom
    rng = np.random.default_rng(seed_of("conv tiles", geom))
    x, k, b = fill(rng, (N, C, H, W), np.float32), fill(rng, (co, C, kh, kw), np.float32), fill(rng, (co,), np.float32)
    want = oracle.conv2d(x, k, b, pad, stride)
    got = {}
    for tile in (0, 1, 2):
        say("conv tile", tile, geom)
        monkeypatch.setenv("AM_HIP_CONV_TILE_F32", str(tile))
        got[tile] = hip.conv2d(hip.toHip(x), hip.toHip(k), hip.toHip(b), pad, stride, fused=True).toCpu()
        check(oracle, "f32", got[tile], want, f"tile {tile}")
    assert np.array_equal(got[0], got[2])


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


BWD_GEOMS = [  # N, C, H, W, C_out, kH, kW, pad, stride
    (2, 3, 4, 5, 2, 3, 3, (1, 1), (1, 1)),          # the reference's own backward case (test_nnp_convolution.nim:137-168)
    (1, 1, 5, 5, 1, 3, 3, (0, 0), (1, 1)),
    (3, 2, 9, 7, 4, 3, 2, (1, 0), (2, 1)),
    (4, 2, 16, 16, 3, 3, 3, (1, 1), (2, 2)),        # stride 2 with padding: pixels that no column covers get 0
    (3, 8, 20, 20, 13, 3, 5, (2, 3), (1, 2)),       # padding wider than the kernel's reach on one side
    (2, 5, 11, 13, 7, 1, 1, (0, 0), (1, 1)),        # 1 x 1 kernel
    (2, 3, 9, 9, 4, 2, 2, (0, 0), (3, 3)),          # stride beyond the kernel: rows and columns of the image left out
    (64, 1, 28, 28, 20, 5, 5, (0, 0), (1, 1)),      # conv1 of the reference's example 2 at batch 64
    (16, 20, 12, 12, 50, 5, 5, (0, 0), (1, 1)),     # conv2
    (2, 3, 6, 6, 4, 3, 3, (2, 2), (1, 1)),          # padding k - 1: the gradient as a convolution needs no padding of its own
    (2, 3, 6, 6, 4, 2, 2, (2, 2), (1, 1)),          # padding k: outputs made of padding alone; not a convolution any more
    (1, 2, 9, 10, 3, 3, 4, (1, 2), (1, 1)),         # kernel widths 4, 7 and 9 at unit stride
    (1, 1, 10, 12, 2, 2, 7, (0, 3), (1, 1)),
    (1, 1, 6, 14, 2, 2, 9, (0, 4), (1, 1)),
    (2, 100, 8, 8, 6, 3, 3, (1, 1), (1, 1)),        # more input channels than the one-launch form of grad_input takes on small images
    (1, 100, 24, 24, 6, 3, 3, (1, 1), (1, 1)),      # the same channels on 576 pixels: float32 takes the one-launch form, float64 the product + gather
    (3, 4, 6, 4, 5, 3, 3, (1, 1), (1, 1)),          # image rows of one float vector: the gathered weight gradient's vectors hang over both edges
    (2, 3, 7, 12, 6, 2, 5, (0, 4), (1, 1)),         # padding as wide as a float vector
    (5, 2, 9, 8, 140, 3, 3, (1, 1), (2, 1)),        # window stepping by 2 rows and 1 column; 140 output channels (edge tile of rows), k = 5 * 32 not a slab multiple in float64's tile
    (70, 3, 10, 10, 8, 3, 3, (0, 0), (1, 1)),       # k = 70 * 64 = 4480: split over workgroups
]


@pytest.mark.parametrize("sfx", ALL)
@pytest.mark.parametrize("geom", BWD_GEOMS)
def test_col2im_and_conv_backward_vs_oracle(hip, oracle, sfx, geom):
    """col2im and conv2d_backward (fallback/conv.nim:55-79, 107-145; nnp_convolution.nim:65-107) against the oracle's
    per-image restatement: col2im bit for bit in every type (same entries added in the same order), the gradients bit
    for bit on integers and within the float GEMM tolerance otherwise."""
    dt = DTYPES[sfx]
    N, C, H, W, co, kh, kw, pad, stride = geom
    rng = np.random.default_rng(seed_of("conv-bwd", sfx, geom))
    ho, wo = (H + 2 * pad[0] - kh) // stride[0] + 1, (W + 2 * pad[1] - kw) // stride[1] + 1
    x, k, b = fill(rng, (N, C, H, W), dt), fill(rng, (co, C, kh, kw), dt), fill(rng, (co, 1, 1), dt)
    g = fill(rng, (N, co, ho, wo), dt)
    say("col2im", sfx, geom)
    cols = fill(rng, (N, C * kh * kw, ho * wo), dt)
    got = hip.col2im(hip.toHip(cols), C, H, W, (kh, kw), pad, stride).toCpu()
    for n in (0, N - 1):
        assert np.array_equal(got[n], oracle.col2im(cols[n], C, H, W, (kh, kw), pad, stride)), n
    one = hip.col2im(hip.toHip(cols[0]), C, H, W, (kh, kw), pad, stride).toCpu()
    assert one.shape == (C, H, W) and np.array_equal(one, got[0])
    say("folded im2col", sfx, geom)
    folded = hip.im2col_folded(hip.toHip(x), (kh, kw), pad, stride).toCpu().reshape(C * kh * kw, N, ho * wo)
    for n in (0, N - 1):
        assert np.array_equal(folded[:, n], oracle.im2col(x[n], (kh, kw), pad, stride)), n
    say("conv2d_backward", sfx, geom)
    gi, gw, gb = hip.conv2d_backward(hip.toHip(x), hip.toHip(k), hip.toHip(b), pad, stride, hip.toHip(g))
    wi, ww, wb = oracle.conv2d_backward(x, k, b, pad, stride, g)
    assert gi.shape == x.shape and gw.shape == k.shape and gb.shape == b.shape
    check(oracle, sfx, gi.toCpu(), wi, "grad_input")
    check(oracle, sfx, gw.toCpu(), ww, "grad_weight")
    check(oracle, sfx, gb.toCpu(), wb, "grad_bias")
    gi2, gw2, gb2 = hip.conv2d_backward(hip.toHip(x), hip.toHip(k), None, pad, stride, hip.toHip(g))
    assert gb2 is None and np.array_equal(gi2.toCpu(), gi.toCpu()) and np.array_equal(gw2.toCpu(), gw.toCpu())
    # grad_weight from the written column matrix (where the call above gathered it), and from an input with other strides
    _, gw3, _ = hip.conv2d_backward(hip.toHip(x), hip.toHip(k), None, pad, stride, hip.toHip(g), need_input_grad=False,
                                    fused_weight_gradient=False)
    check(oracle, sfx, gw3.toCpu(), ww, "grad_weight, im2col + product")
    if C > 1:
        _, gw4, _ = hip.conv2d_backward(hip.toHip(np.ascontiguousarray(x[:, ::-1]))[:, ::-1], hip.toHip(k), None, pad, stride,
                                        hip.toHip(g), need_input_grad=False)
        check(oracle, sfx, gw4.toCpu(), ww, "grad_weight, reversed channel stride")


def test_conv_backward_reference_check(hip, oracle):
    """The reference's own check (test_nnp_convolution.nim:137-168): float32 gradients for grad_output = ones against
    the float64 numerical gradient of the forward pass, mean relative error below 1e-6."""
    rng = np.random.default_rng(seed_of("conv-bwd-reference"))
    x = rng.uniform(0, 1, (2, 3, 4, 5)).astype(np.float32)
    k = rng.uniform(0, 1, (2, 3, 3, 3)).astype(np.float32)
    b = rng.uniform(0, 1, (2, 1, 1)).astype(np.float32)
    pad, stride = (1, 1), (1, 1)
    out = hip.conv2d(hip.toHip(x), hip.toHip(k), hip.toHip(b), pad, stride)
    gi, gw, gb = hip.conv2d_backward(hip.toHip(x), hip.toHip(k), hip.toHip(b), pad, stride, hip.toHip(np.ones(out.shape, np.float32)))
    x64, k64, b64 = x.astype(np.float64), k.astype(np.float64), b.astype(np.float64)

    def numerical(arr, h=1e-3):
        grad = np.zeros_like(arr)
        flat, gf = arr.reshape(-1), grad.reshape(-1)
        for i in range(flat.size):
            keep = flat[i]
            flat[i] = keep + h; up = oracle.conv2d(x64, k64, b64, pad, stride).sum()
            flat[i] = keep - h; dn = oracle.conv2d(x64, k64, b64, pad, stride).sum()
            flat[i] = keep
            gf[i] = (up - dn) / (2 * h)
        return grad

    for got, arr, name in ((gi, x64, "grad_input"), (gw, k64, "grad_weight"), (gb, b64, "grad_bias")):
        want = numerical(arr)
        err = np.mean(np.abs(got.toCpu().astype(np.float64) - want) / np.abs(want))
        say("conv backward, reference check", name, err)
        assert err < 1e-6, name


def test_conv_backward_errors(hip):
    x, k = hip.zeros((2, 3, 5, 5), np.float32), hip.zeros((4, 3, 3, 3), np.float32)
    with pytest.raises(ValueError):
        hip.conv2d_backward(x, k, None, (0, 0), (1, 1), hip.zeros((2, 4, 4, 4), np.float32))     # wrong output extent
    with pytest.raises(ValueError):
        hip.conv2d_backward(x, hip.zeros((4, 2, 3, 3), np.float32), None, (0, 0), (1, 1), hip.zeros((2, 4, 3, 3), np.float32))
    with pytest.raises(ValueError):
        hip.col2im(hip.zeros((27, 8), np.float32), 3, 5, 5, (3, 3))                               # 9 columns expected


def test_gathered_weight_gradient_entry_point(hip):
    """am_hip_conv2d_grad_weight_* through the C ABI on its own: the geometries it refuses (AM_E_SHAPE, nothing
    launched, the result untouched), bad arguments, and a batch of no images, which leaves the result as it is."""
    import ctypes
    from arraymancer_amd import _lib
    L = _lib.load()
    fn = L.am_hip_conv2d_grad_weight_f32
    x = hip.toHip(np.ones((2, 3, 6, 8), np.float32))
    out = hip.toHip(np.full((4, 3, 3, 3), 7, np.float32))
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())

    def call(N, W, pad_w, stride_w, xs=None, g=None, o=out, in_ptr=None):
        wo = (W + 2 * pad_w - 3) // stride_w + 1
        g = g if g is not None else hip.toHip(np.ones((4, max(N, 1) * 4 * wo), np.float32))
        return fn(N, 3, 6, W, 4, 3, 3, 0, pad_w, 1, stride_w, in_ptr if in_ptr is not None else ptr(x), *(xs or x.strides), ptr(g), g.strides[0],
                  ptr(o) if o is not None else None)

    say("window stepping by two columns")
    assert call(2, 8, 1, 2) == _lib.AM_E_SHAPE
    say("output rows of 6 pixels")
    assert call(2, 8, 0, 1) == _lib.AM_E_SHAPE
    say("image with stride 2 along the width")
    assert call(2, 8, 1, 1, xs=(144, 48, 8, 2)) == _lib.AM_E_SHAPE
    say("null pointers, bad geometry")
    assert call(2, 8, 1, 1, o=None) == _lib.AM_E_ARG
    assert call(2, 8, 1, 1, in_ptr=ctypes.c_void_p(0)) == _lib.AM_E_ARG
    assert fn(2, 3, 6, 8, 4, 0, 3, 0, 1, 1, 1, ptr(x), *x.strides, ptr(x), 8, ptr(out)) == _lib.AM_E_ARG
    assert "am_hip_conv2d_grad_weight_f32" in _lib.last_error()
    assert np.array_equal(out.toCpu(), np.full((4, 3, 3, 3), 7, np.float32))
    say("no images")
    assert call(0, 8, 1, 1) == _lib.AM_OK and np.array_equal(out.toCpu(), np.full((4, 3, 3, 3), 7, np.float32))
    say("two images of ones: every entry counts the pixels its window position covers")
    assert call(2, 8, 1, 1) == _lib.AM_OK
    got = out.toCpu()
    want = np.empty((4, 3, 3, 3), np.float32)
    want[:, :, :, 0] = want[:, :, :, 2] = 2 * 4 * 7      # 4 output rows x 8 output columns, one of them in the padding
    want[:, :, :, 1] = 2 * 4 * 8
    assert np.array_equal(got, want)
