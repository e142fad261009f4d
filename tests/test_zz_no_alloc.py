"""am_hip_gemm_noalloc_f32 (split-K partials in the library's static device array, no allocation)
against am_hip_gemm_f32 (partials in a hipMalloc'ed workspace): same kernels and, wherever the
allocating entry point's plan fits the 16 MiB array and cuts no strips off, the same plan, so those
results are held to bit equality, which is inside the float32 bar (<= 1e-4 relative Frobenius error)
that am_hip_gemm_f32 itself is held to against the oracle; shapes on which the two plans differ are
held to that bar alone. Two calls in a row, the second smaller, so that the second runs over whatever
the first left in the array."""
import ctypes
import os
import subprocess
import sys
import textwrap

import numpy as np
import pytest

from arraymancer_amd._lib import last_error

pytestmark = pytest.mark.gpu


def _call(L, name, M, N, K, alpha, dA, dB, beta, dC):
    f = ctypes.c_float
    return getattr(L, name)(M, N, K, f(alpha), ctypes.c_void_p(dA.data_ptr()), dA.strides[0], dA.strides[1],
                            ctypes.c_void_p(dB.data_ptr()), dB.strides[0], dB.strides[1], f(beta),
                            ctypes.c_void_p(dC.data_ptr()), dC.strides[0], dC.strides[1])


def _pair(hip, oracle, rng, M, N, K, alpha=1.0, beta=0.0, transposed_b=False, same_plan=True):
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
    if same_plan:
        assert np.array_equal(ref, new), f"{M}x{N}x{K}: results differ from am_hip_gemm_f32"
    want = oracle.gemm_strided(alpha, A, B, beta, C0.copy())
    assert oracle.rel_frobenius(new, want) <= 1e-4   # the float32 bar of the path
    assert oracle.rel_frobenius(ref, want) <= 1e-4
    return new


def test_no_alloc_gemm_matches_allocating_entry_point_two_calls_in_a_row(hip, oracle):
    rng = np.random.default_rng(77001)
    # few output tiles, long K: both calls are cut along K (16 and 32 ways), partials through the static array
    _pair(hip, oracle, rng, 256, 256, 4096)
    _pair(hip, oracle, rng, 128, 96, 2048, alpha=1.5, beta=0.5, transposed_b=True)   # smaller, over the first call's leftovers
    # a product that needs no split (no scratch at all) and one for the skinny-product kernel
    _pair(hip, oracle, rng, 512, 640, 128)
    _pair(hip, oracle, rng, 48, 300, 700, beta=1.0)


def test_no_alloc_gemm_where_the_plans_differ(hip, oracle):
    """Shapes on which am_hip_gemm_f32 plans something the allocation-free entry point does not: partial tiles
    beyond the 16 MiB array (a weight-gradient shape: few tiles, very long k), and an aligned block plus strips
    (extents one above a multiple of 64). Both answers meet the float32 bar; bit equality is not promised."""
    rng = np.random.default_rng(77003)
    _pair(hip, oracle, rng, 500, 800, 65536, same_plan=False)
    _pair(hip, oracle, rng, 2049, 2049, 192, same_plan=False)
    _pair(hip, oracle, rng, 200, 200, 8192)     # long k within the array: the joint plan of both entry points


_FRESH_PROCESS = textwrap.dedent("""
    import ctypes, sys
    import numpy as np
    sys.path.insert(0, sys.argv[1])
    import arraymancer_amd as hip
    from arraymancer_amd._lib import last_error
    L = hip.load_library()
    f = ctypes.c_float
    def call(name, M, N, K, dA, dB, dC):
        rc = getattr(L, name)(M, N, K, f(1.0), ctypes.c_void_p(dA.data_ptr()), K, 1, ctypes.c_void_p(dB.data_ptr()), N, 1,
                              f(0.0), ctypes.c_void_p(dC.data_ptr()), N, 1)
        assert rc == 0, last_error()
        hip.sync()
    def free_bytes():
        a, b = ctypes.c_size_t(), ctypes.c_size_t()
        assert L.am_hip_device_free_bytes(ctypes.byref(a), ctypes.byref(b)) == 0, last_error()
        return a.value
    rng = np.random.default_rng(1)
    M, N, K = 256, 256, 4096            # few tiles, long k: cut along k, partial tiles through scratch memory
    dA = hip.toHip(rng.uniform(-1, 1, (M, K)).astype(np.float32))
    dB = hip.toHip(rng.uniform(-1, 1, (K, N)).astype(np.float32))
    dC, dD = hip.empty((M, N), np.float32), hip.empty((M, N), np.float32)
    sA, sB, sC = hip.toHip(np.ones((64, 64), np.float32)), hip.toHip(np.ones((64, 64), np.float32)), hip.empty((64, 64), np.float32)
    call("am_hip_gemm_noalloc_f32", 64, 64, 64, sA, sB, sC)   # loads the code objects: what a first launch costs is not the point
    before = free_bytes()
    call("am_hip_gemm_noalloc_f32", M, N, K, dA, dB, dC)
    after = free_bytes()
    call("am_hip_gemm_f32", M, N, K, dA, dB, dD)              # the allocating twin takes its 64 MiB workspace now
    twin = free_bytes()
    assert np.array_equal(dC.toCpu(), dD.toCpu())
    print("FREE", before, after, twin)
""")


def test_no_alloc_gemm_takes_no_device_memory_in_a_fresh_process():
    """The driver's own count of free device memory (hipMemGetInfo sees every allocation of the process, the
    library's workspaces included) around a split-K call of the allocation-free entry point, in a process where no
    allocating GEMM has run yet: it must not move, while the same product through am_hip_gemm_f32 right afterwards
    takes the 64 MiB split-K workspace - which shows that the count would have seen it."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-c", _FRESH_PROCESS, root], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    before, after, twin = (int(x) for x in res.stdout.strip().splitlines()[-1].split()[1:])
    assert before - after < (1 << 20), f"am_hip_gemm_noalloc_f32 took {before - after} bytes of device memory"
    assert after - twin >= (48 << 20), f"the allocating entry point's workspace did not show ({after - twin} bytes): the count proves nothing"


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
