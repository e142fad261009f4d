"""am_hip_gemm_noalloc_f32 (split-K partials in the library's static device array, no allocation)
against am_hip_gemm_f32 (partials in a hipMalloc'ed workspace): same kernels, same plan, so the
results are held to bit equality, which is inside the float32 bar (<= 1e-4 relative Frobenius error)
that am_hip_gemm_f32 itself is held to against the oracle. Two calls in a row, the second smaller,
so that the second runs over whatever the first left in the array."""
import ctypes
import os

import numpy as np
import pytest

from arraymancer_amd._lib import last_error

pytestmark = pytest.mark.gpu


def _call(L, name, M, N, K, alpha, dA, dB, beta, dC):
    f = ctypes.c_float
    return getattr(L, name)(M, N, K, f(alpha), ctypes.c_void_p(dA.data_ptr()), dA.strides[0], dA.strides[1],
                            ctypes.c_void_p(dB.data_ptr()), dB.strides[0], dB.strides[1], f(beta),
                            ctypes.c_void_p(dC.data_ptr()), dC.strides[0], dC.strides[1])


def _pair(hip, oracle, rng, M, N, K, alpha=1.0, beta=0.0, transposed_b=False):
    L = hip.load_library()
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (N, K) if transposed_b else (K, N)).astype(np.float32)
    C0 = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    dA, dB = hip.toHip(A), hip.toHip(B)
    if transposed_b:
        dB, B = dB.transpose(), B.T
    d_ref, d_new = hip.toHip(C0), hip.toHip(C0)
    assert _call(L, "am_hip_gemm_f32", M, N, K, alpha, dA, dB, beta, d_ref) == 0, last_error()
    assert _call(L, "am_hip_gemm_noalloc_f32", M, N, K, alpha, dA, dB, beta, d_new) == 0, last_error()
    ref, new = d_ref.toCpu(), d_new.toCpu()
    assert np.array_equal(ref, new), f"{M}x{N}x{K}: results differ from am_hip_gemm_f32"
    want = oracle.gemm_strided(alpha, A, B, beta, C0.copy())
    assert oracle.rel_frobenius(new, want) <= 1e-4   # the float32 bar of the path
    return new


def test_no_alloc_gemm_matches_allocating_entry_point_two_calls_in_a_row(hip, oracle):
    rng = np.random.default_rng(77001)
    # few output tiles, long K: both calls are cut along K (16 and 32 ways), partials through the static array
    _pair(hip, oracle, rng, 256, 256, 4096)
    _pair(hip, oracle, rng, 128, 96, 2048, alpha=1.5, beta=0.5, transposed_b=True)   # smaller, over the first call's leftovers
    # a product that needs no split (no scratch at all) and one for the skinny-product kernel
    _pair(hip, oracle, rng, 512, 640, 128)
    _pair(hip, oracle, rng, 48, 300, 700, beta=1.0)


def test_no_alloc_gemm_allocates_nothing_and_rejects_what_does_not_fit(hip):
    L = hip.load_library()
    rng = np.random.default_rng(77002)
    M = N = 1536
    K = 1024
    dA = hip.toHip(rng.uniform(-1, 1, (M, K)).astype(np.float32))
    dB = hip.toHip(rng.uniform(-1, 1, (K, N)).astype(np.float32))
    dC = hip.empty((M, N), np.float32)
    live0, cached0, live1, cached1 = (ctypes.c_size_t() for _ in range(4))
    L.am_hip_memory_stats(ctypes.byref(live0), ctypes.byref(cached0))
    assert _call(L, "am_hip_gemm_noalloc_f32", M, N, K, 1.0, dA, dB, 0.0, dC) == 0, last_error()
    L.am_hip_memory_stats(ctypes.byref(live1), ctypes.byref(cached1))
    assert (live0.value, cached0.value) == (live1.value, cached1.value)
    # forced onto the 256 x 256 tile the same product is 36 tiles cut 3 ways: 28 MiB of partials > 16 MiB
    os.environ["AM_HIP_GEMM_TILE_F32"] = "0"
    try:
        rc = _call(L, "am_hip_gemm_noalloc_f32", M, N, K, 1.0, dA, dB, 0.0, dC)
    finally:
        del os.environ["AM_HIP_GEMM_TILE_F32"]
    assert rc == -2 and "static" in last_error() and "am_hip_gemm_f32" in last_error()
    hip.sync()
