"""Pins oracle_pack / oracle_unpack: against the compiled reference library on
the reference's own test matrix (tools/pack_test.c:137-246,
tools/unpack_test.c:123-218), against a numpy pad/reshape/transpose closed form,
and through the round-trip and untouched-destination invariants."""
import itertools

import numpy as np
import pytest

import ukref
from iree_amd import flags as F

OUTER = [(0, 1), (1, 0), (1, 1), (3, 2), (9, 33)]           # pack_test.c:137-145
PADS = ["none", "one_incomplete_tile", "a_lot"]             # pack_test.c:146-151
PACK_TILES = [(F.PACK_TYPE_F32F32, 3, 5), (F.PACK_TYPE_I8I8, 4, 2),
              (F.PACK_TYPE_I32I32, 3, 4), (F.PACK_TYPE_F16F16, 6, 7),
              (F.PACK_TYPE_BF16BF16, 9, 2),
              # x86 shapes (pack_test.c:229-241)
              (F.PACK_TYPE_F32F32, 8, 1), (F.PACK_TYPE_I8I8, 8, 2),
              (F.PACK_TYPE_F32F32, 8, 8), (F.PACK_TYPE_I32I32, 8, 8),
              (F.PACK_TYPE_F32F32, 16, 1), (F.PACK_TYPE_BF16BF16, 16, 2),
              (F.PACK_TYPE_I8I8, 16, 2), (F.PACK_TYPE_F32F32, 16, 16),
              (F.PACK_TYPE_I32I32, 16, 16),
              # gfx950 shapes
              (F.PACK_TYPE_F16F16, 32, 8), (F.PACK_TYPE_F16F16, 32, 16),
              (F.PACK_TYPE_I8I8, 32, 16), (F.PACK_TYPE_I8I8, 32, 32),
              (F.PACK_TYPE_I32I32, 32, 32)]
UNPACK_TILES = [(F.UNPACK_TYPE_F32F32, 3, 5), (F.UNPACK_TYPE_I32I32, 3, 4),
                (F.UNPACK_TYPE_F16F16, 6, 7), (F.UNPACK_TYPE_BF16BF16, 9, 2),
                (F.UNPACK_TYPE_F32F32, 8, 8), (F.UNPACK_TYPE_I32I32, 8, 8),
                (F.UNPACK_TYPE_F32F32, 16, 16), (F.UNPACK_TYPE_I32I32, 16, 16),
                (F.UNPACK_TYPE_F32F32, 32, 32), (F.UNPACK_TYPE_F16F16, 32, 16)]


def _feature_sets():
    return [""] + [fs for fs in ("avx2_fma", "avx512_base") if ukref.host_supports(fs)]


@pytest.mark.parametrize("type_flag,t0,t1", PACK_TILES)
def test_pack_oracle_vs_reference_and_numpy(type_flag, t0, t1):
    rng = np.random.default_rng(31 * type_flag + 7 * t0 + t1)
    have_ref = ukref.reflib() is not None
    n = 0
    for (o0, o1), ti, to, pad in itertools.product(OUTER, (0, 1), (0, 1), PADS):
        case = ukref.PackCase(rng, type_flag, o0, o1, t0, t1, transpose_inner=ti,
                              transpose_outer=to, pad=pad,
                              loose_strides=bool(rng.integers(0, 2)), offsets=True,
                              in_stride1=1 + int(rng.integers(0, 2)))
        got = case.run_oracle()
        assert np.array_equal(got, case.run_numpy()), (o0, o1, ti, to, pad)
        if have_ref:
            for fs in _feature_sets():
                assert np.array_equal(got, case.run_ref(fs)), (o0, o1, ti, to, pad, fs)
        n += 1
    assert n == 60


@pytest.mark.parametrize("type_flag,t0,t1", UNPACK_TILES)
def test_unpack_oracle_vs_reference_and_numpy(type_flag, t0, t1):
    rng = np.random.default_rng(17 * type_flag + 5 * t0 + t1)
    have_ref = ukref.reflib() is not None
    for (o0, o1), ti, to, pad in itertools.product(OUTER, (0, 1), (0, 1), PADS):
        case = ukref.UnpackCase(rng, type_flag, o0, o1, t0, t1, transpose_inner=ti,
                                transpose_outer=to, pad=pad,
                                loose_strides=bool(rng.integers(0, 2)), offsets=True,
                                out_stride1=1 + int(rng.integers(0, 2)))
        got = case.run_oracle()
        assert np.array_equal(got, case.run_numpy()), (o0, o1, ti, to, pad)
        if have_ref:
            for fs in _feature_sets():
                assert np.array_equal(got, case.run_ref(fs)), (o0, o1, ti, to, pad, fs)


def test_unpack_of_pack_is_identity_and_padding_is_the_low_bits():
    import ctypes as C
    from iree_amd._lib import UnpackParams
    rng = np.random.default_rng(8)
    for ti, to in itertools.product((0, 1), (0, 1)):
        case = ukref.PackCase(rng, F.PACK_TYPE_F16F16, 5, 4, 6, 7, transpose_inner=ti,
                              transpose_outer=to, pad="one_incomplete_tile", in_size=(27, 23))
        packed = case.run_oracle()
        # every slot that is not a source element holds the low 16 bits of the pad
        src = set(case.inp[case.in_offset + r * case.in_stride0 + c] for r in range(27) for c in range(23))
        padv = case.padding_value & 0xFFFF
        region = packed[:case.out_size0 * case.out_stride0]
        assert int(np.count_nonzero(region == padv)) >= 5 * 4 * 42 - 27 * 23 - len(src & {padv})
        back = np.full(27 * 23 + 3, 0xBEEF, np.uint16)
        up = UnpackParams(ukref.ptr(packed).value, 0, case.out_stride0, case.out_stride1,
                          ukref.ptr(back).value, 0, 23, 1, case.out_size0, case.out_size1,
                          case.out_size2, case.out_size3, 27, 23, case.flags, None)
        assert ukref.oracle().oracle_unpack(C.byref(up)) == 0
        want = np.stack([case.inp[r * case.in_stride0:][:23] for r in range(27)]).ravel()
        assert np.array_equal(back[:27 * 23], want)
        assert (back[27 * 23:] == 0xBEEF).all()  # canary: nothing written past the end


def test_pack_unpack_reject_invalid():
    import ctypes as C
    rng = np.random.default_rng(2)
    case = ukref.PackCase(rng, F.PACK_TYPE_F32F32, 2, 2, 3, 5)
    out = case.out_init.copy()
    p = case.params(ukref.ptr(case.inp).value, ukref.ptr(out).value)
    p.out_stride1 += 1
    assert ukref.oracle().oracle_pack(C.byref(p)) == F.STATUS_INVALID_ARGUMENT
    p = case.params(ukref.ptr(case.inp).value, ukref.ptr(out).value)
    p.flags = 0x06
    assert ukref.oracle().oracle_pack(C.byref(p)) == F.STATUS_INVALID_ARGUMENT
    p = case.params(ukref.ptr(case.inp).value, ukref.ptr(out).value)
    p.in_size0 = 7  # 2 tiles of 3 rows cannot hold 7 rows
    assert ukref.oracle().oracle_pack(C.byref(p)) == F.STATUS_INVALID_ARGUMENT
    ucase = ukref.UnpackCase(rng, F.UNPACK_TYPE_F32F32, 2, 2, 3, 5)
    uout = ucase.out_init.copy()
    up = ucase.params(ukref.ptr(ucase.inp).value, ukref.ptr(uout).value)
    up.flags = F.PACK_TYPE_I8I8  # no 1-byte unpack in the ABI
    assert ukref.oracle().oracle_unpack(C.byref(up)) == F.STATUS_INVALID_ARGUMENT
