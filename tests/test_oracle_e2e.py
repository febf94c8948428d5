"""Pins the oracle's restatement of the reference's end-to-end matmul checker
(its reference matmul and its operand generator) on the CPU."""
import numpy as np
import pytest

import e2e_matmul_cases as E
import ukref
from iree_amd import synth


def test_pseudorandom_stream_known_values():
    """The first states from seed 2, worked out by hand: 2 * 48271 = 96542;
    96542 * 48271 = 4660178882, which wraps to 365211586 in 32 bits BEFORE the
    reduction modulo 2^31 - 1 (a true Lehmer generator would give 365211588).
    Range 5, minimum -2: 96542 % 5 - 2 = 0, 365211586 % 5 - 2 = -1."""
    assert list(synth.e2e_pseudorandom_ints(2, 2, -2, 2)) == [0, -1]
    assert list(synth.e2e_pseudorandom_ints(2, 2, 0, 2 ** 31 - 2)) == [96542, 365211586]
    # big-integer restatement, and the oracle's C version of the same stream
    state, want = 7, []
    for _ in range(5000):
        state = ((state * 48271) % (1 << 32)) % 2147483647
        want.append(state % 17 - 8)
    assert list(synth.e2e_pseudorandom_ints(7, 5000, -8, 8)) == want
    out = np.empty(5000, np.int32)
    ukref.oracle().oracle_e2e_pseudorandom_fill(7, 5000, -8, 8, ukref.ptr(out))
    assert list(out) == want


def test_generated_matrices_are_exact_small_integers():
    for elem, (lo, hi) in synth.E2E_RANGE.items():
        x = synth.e2e_matrix(11, 4000, elem)
        assert x.dtype == E.NP_DTYPE[elem]
        v = E.to_int64(x, elem)
        assert v.min() == lo and v.max() == hi          # the whole range is drawn
        assert np.array_equal(v, synth.e2e_pseudorandom_ints(11, 4000, lo, hi))


@pytest.mark.parametrize("name", sorted(E.TYPES))
def test_reference_matmul_restatement_against_exact_integers(name):
    """oracle_e2e_reference_matmul (f32 accumulation in k order, one final
    rounding) against int64 products rounded once by numpy, on every shape of
    the reference's SMALL list and two large ones, with and without an
    accumulator."""
    type_flag, in_elem, out_elem = E.TYPES[name]
    o = ukref.oracle()
    for (m, k, n, accumulate, dynamic, ls, rs, accs) in list(E.cases(E.SMALL)) + list(E.cases(E.LARGE[:2])):
        if not dynamic:
            continue
        lhs, rhs, acc = E.operands(m, k, n, ls, rs, accs, in_elem, out_elem)
        got = np.zeros(m * n, E.NP_DTYPE[out_elem])
        assert o.oracle_e2e_reference_matmul(ukref.ptr(lhs), ukref.ptr(rhs),
                                             ukref.ptr(acc) if acc is not None else None,
                                             ukref.ptr(got), m, n, k, type_flag) == 0
        want = E.exact_result(lhs, rhs, acc, m, k, n, in_elem, out_elem)
        assert np.array_equal(got.reshape(m, n).view(np.uint8), want.view(np.uint8)), (m, k, n)


def test_reference_matmul_restatement_rounds_narrow_results_once():
    """Sums beyond what f16 / bf16 hold exactly: 999 products of 4 * 3 = 11988
    lies halfway between the f16 neighbours 11984 and 11992 (ties to even:
    11984); with an accumulator of 4 the sum 11992 is exact. bf16 (8 bits of
    significand): 999 * 2 * 2 = 3996 -> 4000 (step 16 from 2048)."""
    o = ukref.oracle()
    lhs, rhs = np.full(999, 4, np.float16), np.full(999, 3, np.float16)
    got = np.zeros(1, np.float16)
    from iree_amd import flags as F
    assert o.oracle_e2e_reference_matmul(ukref.ptr(lhs), ukref.ptr(rhs), None, ukref.ptr(got), 1, 1, 999,
                                         F.MMT4D_TYPE_F16F16F16) == 0
    assert float(got[0]) == 11984.0
    acc = np.full(1, 4, np.float16)
    assert o.oracle_e2e_reference_matmul(ukref.ptr(lhs), ukref.ptr(rhs), ukref.ptr(acc), ukref.ptr(got), 1, 1, 999,
                                         F.MMT4D_TYPE_F16F16F16) == 0
    assert float(got[0]) == 11992.0
    two = np.full(999, 0x4000, np.uint16)      # bf16 2.0
    gotb = np.zeros(1, np.uint16)
    assert o.oracle_e2e_reference_matmul(ukref.ptr(two), ukref.ptr(two), None, ukref.ptr(gotb), 1, 1, 999,
                                         F.MMT4D_TYPE_BF16BF16BF16) == 0
    assert ukref.bf16_bits_to_f32(gotb)[0] == 4000.0
