"""The reference's end-to-end matmul test suite through the data-tiled chain on
the GPU: its SMALL and LARGE shape lists x its six llvm-cpu element-type pairs
x accumulate as listed x dynamic / static sizes
(tests/e2e/matmul/generate_e2e_matmul_tests.py:134-213,
tests/e2e/matmul/CMakeLists.txt:606-942), operands from its own generator
(small integers, seeds counting up from 2: e2e_matmul_cases.py), through

    query tile -> pack LHS, pack RHS (transposing), [pack accumulator] -> mmt4d -> unpack

with the tile the library's query chooses: static sizes below 32 narrow M0 or
N0 (1x10x10 runs M0 = 1, 10x10x1 and 1000x1000x1 run N0 = 1 with the
transposing unpack), dynamic sizes keep 32 x 32. Every result is compared bit
for bit with the oracle's restatement of the test runner's reference matmul
(tools/testing/e2e/iree-e2e-matmul-test.cc:28-149) and with exact integer
arithmetic: all partial sums are integers below 2^24, so the order of the f32
additions cannot change a bit.
"""
import numpy as np
import pytest

import e2e_matmul_cases as E
import ukref
from iree_amd import flags as F

pytestmark = pytest.mark.gpu

TORCH_DTYPE = {"i8": "int8", "i32": "int32", "f16": "float16", "bf16": "int16", "f32": "float32"}


def _to_dev(x, elem):
    import torch
    if elem == "bf16":
        return torch.from_numpy(x.view(np.int16).copy()).cuda()
    return torch.from_numpy(x.copy()).cuda()


@pytest.mark.parametrize("shapes_id", ["small", "large"])
@pytest.mark.parametrize("name", sorted(E.TYPES))
def test_e2e_matmul_suite(uk, cuda, name, shapes_id):
    import torch
    type_flag, in_elem, out_elem = E.TYPES[name]
    o = ukref.oracle()
    element_wise = []
    for (m, k, n, accumulate, dynamic, ls, rs, accs) in E.cases(E.SMALL if shapes_id == "small" else E.LARGE):
        lhs, rhs, acc = E.operands(m, k, n, ls, rs, accs, in_elem, out_elem)
        want = np.zeros(m * n, E.NP_DTYPE[out_elem])
        assert o.oracle_e2e_reference_matmul(ukref.ptr(lhs), ukref.ptr(rhs),
                                             ukref.ptr(acc) if acc is not None else None,
                                             ukref.ptr(want), m, n, k, type_flag) == 0
        exact = E.exact_result(lhs, rhs, acc, m, k, n, in_elem, out_elem)
        assert np.array_equal(want.view(np.uint8), exact.reshape(-1).view(np.uint8))
        if acc is not None:
            c = _to_dev(acc, out_elem)
        else:
            # (the runner hands the function no accumulator: the result buffer starts as garbage)
            c = torch.full((m * n,), 77, dtype=getattr(torch, TORCH_DTYPE[out_elem]), device="cuda")
        tile = "dynamic" if dynamic else None
        op = uk.ukernel._MMT4D_TO_QUERY_OP[type_flag]
        M0, N0, K0 = uk.query_matmul_tile_sizes(op) if dynamic else uk.query_matmul_tile_sizes(op, m, n, k)
        if dynamic or (m >= 32 and n >= 32):
            assert (M0, N0) == (32, 32)
        elif n < m:
            assert M0 == 32 and N0 == max(1, 1 << (n - 1).bit_length())     # narrow N0, transposing unpack
        else:
            assert N0 == 32 and M0 == max(1, 1 << (m - 1).bit_length())
        uk.matmul_data_tiled(_to_dev(lhs, in_elem), _to_dev(rhs, in_elem), c, m, n, k, type_flag,
                             accumulate=accumulate, tile=tile)
        torch.cuda.synchronize()
        got = c.cpu().numpy().view(E.NP_DTYPE[out_elem])
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), \
            (name, (m, k, n), accumulate, "dynamic" if dynamic else "static", (M0, N0, K0))
        if not uk.last_kernel_path().startswith("mmt4d:mfma"):
            element_wise.append(((m, k, n), dynamic, (M0, N0, K0), uk.last_kernel_path()))
    # Every case of the suite runs on the matrix cores (a K that is not whole
    # instruction steps ends in a partial step, narrow tiles have their kernel).
    assert not element_wise, element_wise


@pytest.mark.parametrize("name", sorted(E.TYPES))
def test_e2e_matmul_suite_with_the_unpack_fused(uk, cuda, name):
    """The dynamic-size cases once more with the unpack (and the pack of the
    accumulator) folded into the matmul: the same bits."""
    import torch
    type_flag, in_elem, out_elem = E.TYPES[name]
    for (m, k, n, accumulate, dynamic, ls, rs, accs) in list(E.cases(E.SMALL)) + list(E.cases(E.LARGE)):
        if not dynamic:
            continue
        lhs, rhs, acc = E.operands(m, k, n, ls, rs, accs, in_elem, out_elem)
        want = E.exact_result(lhs, rhs, acc, m, k, n, in_elem, out_elem).reshape(-1)
        c = _to_dev(acc, out_elem) if acc is not None else \
            torch.full((m * n,), 77, dtype=getattr(torch, TORCH_DTYPE[out_elem]), device="cuda")
        uk.matmul_data_tiled(_to_dev(lhs, in_elem), _to_dev(rhs, in_elem), c, m, n, k, type_flag,
                             accumulate=accumulate, tile="dynamic", fuse_unpack=True)
        torch.cuda.synchronize()
        got = c.cpu().numpy().view(E.NP_DTYPE[out_elem])
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (name, (m, k, n), accumulate)
