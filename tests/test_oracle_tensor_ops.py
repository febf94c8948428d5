"""The oracle (and the real reference library where it is built) on the pack /
unpack cases of the reference's end-to-end tensor-op tests: literal results and
pad + reshape + transpose constructions, not the oracle's own formula."""
import numpy as np
import pytest

import tensor_ops_cases as T
import ukref
from iree_amd import flags as F

PACK_FLAG = {"i32": F.PACK_TYPE_I32I32, "i8": F.PACK_TYPE_I8I8}


def make_pack_case(name, elem, rows, cols, tr, tc, ti, to, padding):
    src = T.pack_source(elem, rows, cols)
    o0, o1 = T.PACK_OUTER.get(name, (-(-rows // tr), -(-cols // tc)))
    case = ukref.PackCase(np.random.default_rng(1), PACK_FLAG[elem], o0, o1, tr, tc,
                          transpose_inner=ti, transpose_outer=to, in_size=(rows, cols))
    case.inp = np.ascontiguousarray(src).reshape(-1).view(case.dtype).copy()
    case.padding_value = 0 if padding is None else padding
    n = case.out_size0 * case.out_size1 * case.out_size2 * case.out_size3
    case.out_init = np.full(n, 0x55, dtype=case.dtype)
    want = T.pack_expected(name, src, tr, tc, ti, to, padding)
    assert want.shape == (case.out_size0, case.out_size1, case.out_size2, case.out_size3)
    return case, want.reshape(-1).view(case.dtype)


def make_unpack_case(name, rows, cols, tr, tc, ti, to):
    src, want = T.unpack_source_and_expected(name, rows, cols, tr, tc, ti, to)
    case = ukref.UnpackCase(np.random.default_rng(1), F.UNPACK_TYPE_I32I32, -(-rows // tr), -(-cols // tc), tr, tc,
                            transpose_inner=ti, transpose_outer=to, out_size=(rows, cols))
    assert src.shape == (case.in_size0, case.in_size1, case.in_size2, case.in_size3)
    case.inp = src.reshape(-1).view(case.dtype).copy()
    case.out_init = np.full(rows * cols, 0x55555555, dtype=case.dtype)
    return case, want.reshape(-1).view(case.dtype)


@pytest.mark.parametrize("spec", T.PACK_CASES, ids=[c[0] for c in T.PACK_CASES])
def test_pack_cases(spec):
    case, want = make_pack_case(*spec)
    assert np.array_equal(case.run_oracle(), want)
    if ukref.reflib() is not None:
        assert np.array_equal(case.run_ref(), want)


@pytest.mark.parametrize("spec", T.UNPACK_CASES, ids=[c[0] for c in T.UNPACK_CASES])
def test_unpack_cases(spec):
    case, want = make_unpack_case(*spec)
    assert np.array_equal(case.run_oracle(), want)
    if ukref.reflib() is not None:
        assert np.array_equal(case.run_ref(), want)
