"""The pack / unpack cases of the reference's end-to-end tensor-op tests
(tests/e2e/tensor_ops/{pack,pack_dynamic_inner_tiles,pack_i8,unpack}.mlir)
through the C ABI on the GPU: literal results and pad + reshape + transpose
constructions, bit-exact, the whole destination compared."""
import numpy as np
import pytest

import gpucase
import tensor_ops_cases as T
from test_oracle_tensor_ops import make_pack_case, make_unpack_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("spec", T.PACK_CASES, ids=[c[0] for c in T.PACK_CASES])
def test_pack_cases(uk, cuda, spec):
    case, want = make_pack_case(*spec)
    assert np.array_equal(gpucase.run_pack(case), want)


@pytest.mark.parametrize("spec", T.UNPACK_CASES, ids=[c[0] for c in T.UNPACK_CASES])
def test_unpack_cases(uk, cuda, spec):
    case, want = make_unpack_case(*spec)
    assert np.array_equal(gpucase.run_unpack(case), want)
