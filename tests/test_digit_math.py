"""The arithmetic behind the digit-sliced integer GEMM, checked on the CPU with NumPy alone:
balanced base-256 digits, their one-add-one-xor extraction, and the Horner recombination of the
digit-pair products modulo 2^32 / 2^64 (the device kernels are tested against the oracle elsewhere;
this pins the identities they rely on)."""
import numpy as np
import pytest


def balanced_digits(x, nd):
    """Digit d of x (as an unsigned nd-byte word): byte d of (x + 0x80..80) ^ 0x80..80, read as int8."""
    mask = int.from_bytes(b"\x80" * nd, "little")
    mod = 1 << (8 * nd)
    y = ((int(x) % mod + mask) % mod) ^ mask
    return [((y >> (8 * d)) & 0xFF) - (256 if (y >> (8 * d)) & 0x80 else 0) for d in range(nd)]


def reference_digits(x, nd):
    """The textbook loop: take the low byte as a signed digit, subtract it, shift."""
    mod = 1 << (8 * nd)
    u = int(x) % mod
    out = []
    for _ in range(nd):
        d = u & 0xFF
        d -= 256 if d >= 128 else 0
        out.append(d)
        u = ((u - d) % mod) >> 8
    return out


@pytest.mark.parametrize("nd", [4, 8])
def test_digit_extraction_matches_the_subtract_and_shift_loop(nd):
    rng = np.random.default_rng(nd)
    info = np.iinfo(np.int32 if nd == 4 else np.int64)
    edge = [0, 1, -1, 127, 128, 129, -127, -128, -129, 255, 256, -255, -256, info.max, info.min, info.max - 128, info.min + 128]
    edge += [s * (v << (8 * b)) + o for b in range(1, nd) for v in (127, 128, 129) for s in (1, -1) for o in (0, 127, -128)
             if info.min <= s * (v << (8 * b)) + o <= info.max]
    values = edge + [int(v) for v in rng.integers(info.min, info.max, 2000, endpoint=True)]
    mod = 1 << (8 * nd)
    for x in values:
        d = balanced_digits(x, nd)
        assert d == reference_digits(x, nd), x
        assert all(-128 <= v <= 127 for v in d)
        assert sum(v << (8 * i) for i, v in enumerate(d)) % mod == x % mod, x


@pytest.mark.parametrize("nd", [4, 8])
def test_pairs_with_i_plus_j_below_nd_suffice_and_horner_recombines(nd):
    """sum_{s} 256^s sum_{i+j=s} A_i B_j == A B (mod 2^(8 nd)), evaluated highest s first with a shift by
    8 between two values of s, each A_i B_j an exact int8 x int8 product summed in a wide accumulator."""
    rng = np.random.default_rng(100 + nd)
    dt = np.int32 if nd == 4 else np.int64
    info = np.iinfo(dt)
    mod = 1 << (8 * nd)
    M, N, K = 5, 6, 37
    A = rng.integers(info.min, info.max, (M, K), endpoint=True).astype(dt)
    B = rng.integers(info.min, info.max, (K, N), endpoint=True).astype(dt)
    Ad = np.array([[balanced_digits(v, nd) for v in row] for row in A], dtype=object)     # [M][K][nd]
    Bd = np.array([[balanced_digits(v, nd) for v in row] for row in B], dtype=object)     # [K][N][nd]
    want = (A.astype(object) @ B.astype(object)) % mod
    acc = np.zeros((M, N), dtype=object)
    for s in range(nd - 1, -1, -1):
        acc = (acc * 256) % mod if s != nd - 1 else acc
        for i in range(s + 1):
            j = s - i
            acc = (acc + Ad[:, :, i] @ Bd[:, :, j]) % mod
    assert np.array_equal(acc, want)
    # the pairs with i + j >= nd only contribute multiples of 2^(8 nd)
    for i in range(nd):
        for j in range(nd - i, nd):
            assert np.all(((Ad[:, :, i] @ Bd[:, :, j]) * (1 << (8 * (i + j)))) % mod == 0)


def test_int64_pair_sums_fit_32_bits_up_to_k_131071():
    """One digit pair's sum over k is at most k * 2^14 in magnitude: exact in an int32 accumulator for
    k <= 131071, the limit the int64 path applies."""
    assert 131071 * 128 * 128 <= 2**31 - 1 < 131072 * 128 * 128
    assert -(131071 * 128 * 127) >= -(2**31)
