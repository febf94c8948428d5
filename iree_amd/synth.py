"""Seeded synthetic inputs, integer-only so they are bit-identical on every
machine (no libm, no platform RNG): element i of stream `seed` is
splitmix64(seed * 0x9E3779B97F4A7C15 + i). Used by the tests, the benchmark and
the golden-fixture generator so that all three see the same bytes.
"""
import numpy as np

_GOLD = np.uint64(0x9E3779B97F4A7C15)


def splitmix64(seed, n, start=0):
    with np.errstate(over="ignore"):
        z = (np.uint64(seed) * _GOLD + np.arange(start, start + n, dtype=np.uint64))
        z = z + _GOLD
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def uniform_int8(seed, n):
    """Uniform over [-128, 127]."""
    return (splitmix64(seed, n) >> np.uint64(56)).astype(np.uint8).view(np.int8)


def uniform_u4_packed(seed, n):
    """n 4-bit values, two per byte (even index in the low nibble)."""
    r = splitmix64(seed, (n + 1) // 2)
    return (r >> np.uint64(56)).astype(np.uint8)


def uniform_pm1_f16(seed, n):
    """Uniform on [-1, 1) rounded to f16 (round-to-nearest-even by numpy)."""
    r = (splitmix64(seed, n) >> np.uint64(32)).astype(np.uint32).view(np.int32)
    return (r.astype(np.float64) / 2147483648.0).astype(np.float32).astype(np.float16)


def normal_f64(seed, n):
    """Approximately N(0,1): Irwin-Hall sum of twelve 16-bit uniforms (three
    64-bit draws), exact integer sum, unit variance."""
    acc = np.zeros(n, dtype=np.int64)
    for d in range(3):
        r = splitmix64(seed * 3 + d + 0x1000, n)
        for f in range(4):
            acc += ((r >> np.uint64(16 * f)) & np.uint64(0xFFFF)).astype(np.int64)
    return (acc.astype(np.float64) - 6.0 * 65535.0) / 65536.0


def normal_f16(seed, n, scale=1.0):
    return (normal_f64(seed, n) * scale).astype(np.float32).astype(np.float16)


def normal_f32(seed, n, scale=1.0):
    return (normal_f64(seed, n) * scale).astype(np.float32)


def uniform_f16(seed, n, lo, hi):
    r = (splitmix64(seed, n) >> np.uint64(40)).astype(np.float64) / float(1 << 24)
    return (lo + (hi - lo) * r).astype(np.float32).astype(np.float16)


def small_int_f16(seed, n, lo=-8, hi=8):
    """Small integers as f16: products and partial sums stay exact."""
    r = (splitmix64(seed, n) >> np.uint64(40)).astype(np.int64)
    return (lo + r % (hi - lo)).astype(np.float16)


# ---------------------------------------------------------------------------
# The operand generator of the reference's end-to-end matmul tests
# (tools/testing/e2e/test_utils.c:260-267, constants test_utils.h:99-100, used
# as tools/testing/e2e/iree-e2e-matmul-test.cc:641-660 does): a Lehmer step
# whose product is taken in 32-bit unsigned arithmetic, i.e. it wraps before
# the reduction modulo 2^31 - 1, then value = state % range + min.
# ---------------------------------------------------------------------------

# [min, max] per element type (tools/testing/e2e/test_utils.c:269-319).
E2E_RANGE = {"i8": (-2, 2), "i32": (-8, 8), "f16": (-4, 4), "bf16": (-2, 2), "f32": (-8, 8)}


def e2e_pseudorandom_ints(seed, n, lo, hi):
    """The n integers in [lo, hi] the reference's test runner draws from `seed`."""
    out = np.empty(n, dtype=np.int32)
    state, span = int(seed), hi - lo + 1
    for i in range(n):
        state = ((state * 48271) & 0xFFFFFFFF) % 2147483647
        out[i] = state % span + lo
    return out


def e2e_matrix(seed, n, elem):
    """n elements of type `elem` ("i8", "i32", "f16", "bf16", "f32") as the
    reference's generate_random_matrix fills them: small integers, converted
    exactly (bf16 as its 16 bits in a uint16 array)."""
    lo, hi = E2E_RANGE[elem]
    v = e2e_pseudorandom_ints(seed, n, lo, hi)
    if elem == "i8":
        return v.astype(np.int8)
    if elem == "i32":
        return v
    if elem == "f16":
        return v.astype(np.float16)
    if elem == "f32":
        return v.astype(np.float32)
    # bf16: the high half of the f32 (small integers have no low bits)
    return (v.astype(np.float32).view(np.uint32) >> np.uint32(16)).astype(np.uint16)
