"""The HipTensor operator surface exercised the way the reference exercises its CUDA backend
(tests/tensor/test_operators_blas_cuda.nim, test_broadcasting_cuda.nim, test_init_cuda.nim,
test_shapeshifting_cuda.nim): small literals round-tripped toHip ... toCpu."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_round_trip_and_clone_of_reversed_slice(hip):
    # test_init_cuda.nim:20-33: clone of a reversed slice
    a = np.arange(1, 26, dtype=np.float64).reshape(5, 5)
    d = hip.toHip(a)
    assert np.array_equal(d.toCpu(), a)
    r = d[::-1, ::-1]
    assert np.array_equal(r.toCpu(), a[::-1, ::-1])
    c = r.clone()
    assert c.is_C_contiguous() and np.array_equal(c.toCpu(), a[::-1, ::-1])


def test_gemm_gemv_literals(hip):
    # test_operators_blas_cuda.nim:19-113
    a = hip.toHip(np.array([[1.0, 2, 3], [4, 5, 6]]))
    b = hip.toHip(np.array([[7.0, 8], [9, 10], [11, 12]]))
    assert np.array_equal((a * b).toCpu(), [[58, 64], [139, 154]])
    d = hip.toHip(np.array([[1.0, -1, 2], [0, -3, 1]]))
    e = hip.toHip(np.array([2.0, 1, 0]))
    assert np.array_equal((d * e).toCpu(), [1.0, -3.0])
    c = hip.toHip(np.array([[1, 2, 3], [4, 5, 6]], dtype=np.float32))
    with pytest.raises(IndexError):
        c * c
    with pytest.raises(ValueError):
        e * a


def test_inplace_and_out_of_place_add_sub(hip):
    # test_operators_blas_cuda.nim:121-227
    u = hip.toHip(np.array([1.0, 3, -5]))
    v = hip.toHip(np.array([4.0, -2, -1]))
    u += v
    assert np.array_equal(u.toCpu(), [5.0, 1, -6])
    u -= v
    assert np.array_equal(u.toCpu(), [1.0, 3, -5])
    assert np.array_equal((u + v).toCpu(), [5.0, 1, -6])
    assert np.array_equal((u - v).toCpu(), [-3.0, 5, -4])
    a = hip.toHip(np.array([7.0, 4, 3, 1, 8, 6, 8, 1, 6, 2]).reshape(5, 2))
    b = hip.toHip(np.array([6.0, 6, 2, 0, 4, 3, 2, 0, 0, 3]).reshape(5, 2))
    assert np.array_equal((a + b).toCpu().ravel(), [13.0, 10, 5, 1, 12, 9, 10, 1, 6, 5])
    a -= b
    assert np.array_equal(a.toCpu().ravel(), [1.0, -2, 1, 1, 4, 3, 6, 1, 6, -1])
    with pytest.raises(ValueError):
        a += b[0:2, 0:2]
    with pytest.raises(ValueError):
        a + b[0:2, 0:2]


def test_scalar_mul_div(hip):
    # test_operators_blas_cuda.nim:229-240
    u = hip.toHip(np.array([2.0, 6, -10]))
    assert np.array_equal((u / 2).toCpu(), [1.0, 3, -5])
    a = hip.toHip(np.array([1, 3, -5], dtype=np.float32))
    assert np.array_equal((2 * a).toCpu(), [2, 6, -10])
    assert np.array_equal((a * 2).toCpu(), [2, 6, -10])
    a *= 2
    assert np.array_equal(a.toCpu(), [2, 6, -10])
    a /= 2
    assert np.array_equal(a.toCpu(), [1, 3, -5])


def test_broadcast_literals(hip):
    # test_broadcasting_cuda.nim:18-189
    a = hip.toHip(np.array([0.0, 10, 20, 30]).reshape(4, 1))
    b = hip.toHip(np.array([0.0, 1, 2]).reshape(1, 3))
    assert np.array_equal(hip.bc_add(a, b).toCpu(), [[0, 1, 2], [10, 11, 12], [20, 21, 22], [30, 31, 32]])
    assert np.array_equal(hip.bc_sub(a, b).toCpu(), [[0, -1, -2], [10, 9, 8], [20, 19, 18], [30, 29, 28]])
    assert np.array_equal(hip.bc_mul(a, b).toCpu(), [[0, 0, 0], [0, 10, 20], [0, 20, 40], [0, 30, 60]])
    c = hip.toHip(np.array([100.0, 10, 20, 30]).reshape(4, 1))
    d = hip.toHip(np.array([2.0, 5, 10]).reshape(1, 3))
    assert np.array_equal(hip.bc_div(c, d).toCpu(), [[50, 20, 10], [5, 2, 1], [10, 4, 2], [15, 6, 3]])
    e = a.broadcast((4, 3)).clone()
    e.bc_iadd(b)
    assert np.array_equal(e.toCpu(), [[0, 1, 2], [10, 11, 12], [20, 21, 22], [30, 31, 32]])
    assert np.array_equal(hip.bc_add(hip.bc_add(100.0, a), 200.0).toCpu().ravel(), [300, 310, 320, 330])
    assert np.array_equal(hip.bc_sub(hip.bc_sub(100.0, a), 200.0).toCpu().ravel(), [-100, -110, -120, -130])


def test_views_share_storage(hip):
    # test_shapeshifting_cuda.nim:57-78 / test_accessors_slicer_cuda.nim:58-104
    a = hip.toHip(np.arange(24, dtype=np.int32).reshape(4, 6))
    t = a.transpose()
    assert t.storage is a.storage
    a[1:3, 2:5].bc_iadd(1000)
    want = np.arange(24, dtype=np.int32).reshape(4, 6)
    want[1:3, 2:5] += 1000
    assert np.array_equal(a.toCpu(), want) and np.array_equal(t.toCpu(), want.T)
    assert np.array_equal(a[::2, ::-3].toCpu(), want[::2, ::-3])


def test_conv_as_im2col_gemm(hip, vectors):
    """tests/nn_primitives/test_nnp_convolution.nim:21-134: im2col on the host (the reference's
    per-image loop, fallback/conv.nim:99-103), GEMM + bias on the device."""
    for case in vectors["conv_im2col"]:
        for dt in (np.float32, np.int32):
            x = np.array(case["input"], dtype=dt)[0]
            k = np.array(case["kernel"], dtype=dt)
            (ph, pw), (sh, sw) = case["padding"], case["stride"]
            C, H, W = x.shape
            Co, _, kh, kw = k.shape
            Ho, Wo = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
            xp = np.zeros((C, H + 2 * ph, W + 2 * pw), dtype=dt)
            xp[:, ph:ph + H, pw:pw + W] = x
            col = np.empty((C * kh * kw, Ho * Wo), dtype=dt)
            for c in range(C * kh * kw):
                wo, ho, co = c % kw, (c // kw) % kh, c // (kw * kh)
                col[c] = xp[co, ho:ho + sh * Ho:sh, wo:wo + sw * Wo:sw].reshape(-1)
            out = hip.toHip(k.reshape(Co, -1)) * hip.toHip(col)
            out.bc_iadd(hip.toHip(np.array(case["bias"], dtype=dt).reshape(Co, 1)))
            assert np.array_equal(out.toCpu().reshape(1, Co, Ho, Wo), np.array(case["target"], dtype=dt)), case["name"]


def test_caching_allocator(hip):
    """Freed device blocks are reused without a device synchronisation; results stay right when a
    block is handed out again while earlier kernels on the stream still read it."""
    import ctypes
    L = hip.load_library()
    live, cached = ctypes.c_size_t(), ctypes.c_size_t()

    def stats():
        assert L.am_hip_memory_stats(ctypes.byref(live), ctypes.byref(cached)) == 0
        return live.value, cached.value

    assert L.am_hip_empty_cache() == 0
    live0, cached0 = stats()
    assert cached0 == 0
    t = hip.empty((1000, 1000), np.float32)          # 4 000 000 B -> one 2 MiB-granule block of 4 MiB
    ptr = t.storage.ptr
    assert stats()[0] == live0 + 4 * 1024 * 1024
    del t
    assert stats() == (live0, 4 * 1024 * 1024)
    u = hip.empty((1024, 1024), np.float32)          # same rounded size: the cached block comes back
    assert u.storage.ptr == ptr and stats() == (live0 + 4 * 1024 * 1024, 0)
    del u
    small = hip.empty((3,), np.int32)                # 512-byte granule
    assert stats()[0] == live0 + 512
    del small
    # immediate reuse under load: each result of the chain frees its operand while the next kernel is queued
    rng = np.random.default_rng(11)
    x = rng.uniform(-1, 1, (512, 512)).astype(np.float32)
    d = hip.toHip(x)
    want = x.copy()
    for i in range(50):
        d = d + d if i % 2 == 0 else hip.scalar_op("mul", d, np.float32(0.5))
        want = want + want if i % 2 == 0 else want * np.float32(0.5)
    assert np.array_equal(d.toCpu(), want)
    assert L.am_hip_empty_cache() == 0 and stats()[1] == 0
    # a foreign pointer is rejected, not handed to the driver
    assert L.am_hip_free(ctypes.c_void_p(0x1000)) != 0


def test_display_of_device_tensors(hip):
    """`$t` / pretty on real device tensors, views included: the reference's table layout under a header that
    names this backend (format pinned on the reference's literals in tests/test_display.py)."""
    t = hip.toHip(np.arange(1, 25, dtype=np.int64).reshape(2, 3, 4))
    want = ('HipTensor[system.int] of shape "[2, 3, 4]" on backend "Hip"\n'
            "          0                      1\n"
            "|1      2     3     4| |13    14    15    16|\n"
            "|5      6     7     8| |17    18    19    20|\n"
            "|9     10    11    12| |21    22    23    24|")
    got = str(t)
    assert [l.rstrip() for l in got.rstrip("\n").split("\n")] == want.split("\n")
    v = hip.toHip(np.arange(1, 6, dtype=np.int32).reshape(1, 5)).transpose()
    assert v.pretty(specifier="||") == "| 1|\n| 2|\n| 3|\n| 4|\n| 5|"
    sl = hip.toHip(np.arange(12, dtype=np.float32).reshape(3, 4))[::2, 1::2]          # strided view
    assert sl.pretty(specifier="<>") == "HipTensor[float32]<2,2>:[[1, 3], [9, 11]]"
    assert hip.bc_ge(sl, 3.0).pretty(specifier="<>") == "HipTensor[bool]<2,2>:[[false, true], [true, true]]"
    assert hip.toHip(np.array([0.9532932, 0.12945823])).pretty(precision=4, specifier="[]") == "[0.9533, 0.1295]"
    assert str(hip.empty((0, 3), np.float64)) == 'HipTensor[system.float] of shape "[0, 3]" on backend "Hip"\n    [] (empty)'


def test_free_during_graph_capture_is_deferred_to_the_graph(hip):
    """A tensor dropped inside `with Graph()` is neither leaked nor handed out again while the graph can
    still replay the kernels that use it: the block stays live until the graph is destroyed, then goes back
    to the cache. Live / cached byte counts balance across the whole capture."""
    import ctypes
    import gc
    L = hip.load_library()
    live, cached = ctypes.c_size_t(), ctypes.c_size_t()

    def stats():
        assert L.am_hip_memory_stats(ctypes.byref(live), ctypes.byref(cached)) == 0
        return live.value, cached.value

    x = np.random.default_rng(3).uniform(-1, 1, (256, 1024)).astype(np.float32)
    dx, out = hip.toHip(x), hip.empty((256, 1024), np.float32)
    assert L.am_hip_empty_cache() == 0
    live0, _ = stats()
    tmp = hip.toHip(2 * x)                      # 1 MiB of data, allocated before the capture
    live_tmp, _ = stats()
    assert live_tmp > live0
    from arraymancer_amd import tensor_hip as th
    with hip.Graph() as g:
        th._binary_into("add", out, dx, tmp)    # the graph reads tmp ...
        del tmp                                 # ... and tmp goes out of scope inside the capture
        gc.collect()
    assert stats() == (live_tmp, 0)             # still live: the graph owns it; nothing was cached
    other = hip.empty((256, 1024), np.float32)  # must not receive tmp's block
    th._unary_into("copy", other, dx)
    for _ in range(3):
        g.launch()
        assert np.array_equal(out.toCpu(), x + 2 * x)
        th._unary_into("neg", out, out)
    del other
    del g
    gc.collect()
    assert L.am_hip_empty_cache() == 0
    assert stats() == (live0, 0)                # the deferred block came back when the graph went away


@pytest.mark.parametrize("dt", [np.uint32, np.uint64])
def test_unsigned_ring_operations_against_the_modular_closed_form(hip, dt):
    """uint32 / uint64 on the signed kernels (laser gemm.nim:275-307 casts the pointers the same way). Pinned on what the
    ring fixes: every result equals exact integer arithmetic reduced modulo 2^n (Python big integers), whatever the
    sign reading of the operands - entries over the whole unsigned range, so most have the twin's sign bit set."""
    bits = 8 * np.dtype(dt).itemsize
    mod = 1 << bits
    rng = np.random.default_rng(99001 + bits)
    A = rng.integers(0, mod - 1, (37, 53), dtype=dt, endpoint=True)
    B = rng.integers(0, mod - 1, (53, 29), dtype=dt, endpoint=True)
    C0 = rng.integers(0, mod - 1, (37, 29), dtype=dt, endpoint=True)
    big = lambda X: X.astype(object)
    exact = lambda X: np.array(X % mod, dtype=dt)
    dA, dB = hip.toHip(A), hip.toHip(B)
    assert dA.dtype == np.dtype(dt) and (dA * dB).dtype == np.dtype(dt)
    assert np.array_equal((dA * dB).toCpu(), exact(big(A) @ big(B)))
    alpha, beta = mod - 3, (mod >> 1) + 7                       # scalars above the twin's positive range
    dC = hip.toHip(C0)
    hip.gemm(alpha, dA, dB.transpose().clone().transpose(), beta, dC)   # B through a column-major view
    assert np.array_equal(dC.toCpu(), exact(alpha * (big(A) @ big(B)) + beta * big(C0)))
    # the reference's own small literal (gemm.nim:373-396), unsigned
    a = hip.toHip(np.array([[1, 2, 3], [4, 5, 6]], dtype=dt))
    b = hip.toHip(np.array([[7, 8], [9, 10], [11, 12]], dtype=dt))
    assert np.array_equal((a * b).toCpu(), [[58, 64], [139, 154]])
    v = rng.integers(0, mod - 1, 53, dtype=dt, endpoint=True)
    assert np.array_equal((dA * hip.toHip(v)).toCpu(), exact(big(A) @ big(v)))
    assert int(hip.dot(hip.toHip(v), hip.toHip(A[0]))) == int(sum(int(x) * int(y) for x, y in zip(v, A[0])) % mod)
    X, Y = A, rng.integers(0, mod - 1, A.shape, dtype=dt, endpoint=True)
    dX, dY = hip.toHip(X), hip.toHip(Y)
    assert np.array_equal((dX + dY).toCpu(), exact(big(X) + big(Y)))
    assert np.array_equal((dX - dY).toCpu(), exact(big(X) - big(Y)))
    assert np.array_equal(hip.bc_mul(dX, hip.toHip(Y[:1])).toCpu(), exact(big(X) * big(Y[:1])))
    assert np.array_equal((dX * (mod - 2)).toCpu(), exact(big(X) * (mod - 2)))
    assert np.array_equal(hip.bc_add(dX, mod - 1).toCpu(), exact(big(X) + (mod - 1)))
    assert np.array_equal((-dX).toCpu(), exact(-big(X)))
    assert int(hip.sum(dX)) == int(big(X).sum() % mod)
    assert np.array_equal(hip.sum(dX, 0).toCpu(), exact(big(X).sum(axis=0, keepdims=True)))
    assert int(hip.product(hip.toHip(X[0, :5]))) == int(np.prod(big(X[0, :5])) % mod)
    for refused in (lambda: hip.bc_div(dX, dY), lambda: dX / 3, lambda: hip.bc_le(dX, dY), lambda: hip.max(dX)):
        with pytest.raises(TypeError):
            refused()


def test_scalar_broadcast_is_one_element_with_zero_strides(hip):
    """broadcast(val, shape), shapeshifting.nim:136-176: storage of ONE element, every stride 0, usable as an operand."""
    t = hip.broadcast(2.5, (3, 4), np.float32)
    assert t.shape == (3, 4) and t.strides == (0, 0) and t.offset == 0 and t.storage.nelems == 1 and t.dtype == np.float32
    assert np.array_equal(t.toCpu(), np.full((3, 4), 2.5, np.float32))
    m = np.arange(12, dtype=np.float32).reshape(3, 4)
    assert np.array_equal((hip.toHip(m) + t).toCpu(), m + np.float32(2.5))
    assert np.array_equal(hip.bc_mul(hip.toHip(m), t).toCpu(), m * np.float32(2.5))
    c = t.clone()
    assert c.is_C_contiguous() and c.storage.nelems == 12 and np.array_equal(c.toCpu(), np.full((3, 4), 2.5, np.float32))
    i = hip.broadcast(-7, (2, 5))                      # a Python int: int64, like Nim's `int`
    assert i.dtype == np.int64 and np.array_equal(i.toCpu(), np.full((2, 5), -7))
    a = np.arange(10, dtype=np.int64).reshape(2, 5)
    assert np.array_equal((hip.toHip(a) * hip.broadcast(3, (5, 2), np.int64)).toCpu(), a @ np.full((5, 2), 3))   # as a GEMM operand
    assert hip.broadcast(1.0, (0, 3)).toCpu().shape == (0, 3)
    # the tensor form under the same name
    assert hip.broadcast(hip.toHip(np.ones((1, 4))), (3, 4)).strides == (0, 1)
