"""The case list of the reference's end-to-end matmul tests, as data.

Shapes: the SMALL and LARGE lists of
tests/e2e/matmul/generate_e2e_matmul_tests.py:134-177; element types: the
llvm-cpu instantiations of tests/e2e/matmul/CMakeLists.txt:606-942 (i8 -> i32,
f32 -> f32, f16 -> f16, f16 -> f32, bf16 -> bf16, bf16 -> f32); every shape is
run with dynamic and with static sizes (its get_dynamicities, :203-213).
Operands are drawn as its generate_call does (:695-760): a seed counter that
starts at 1 per generated file and is incremented before each use, one seed
for the left-hand side, one for the right-hand side and, when accumulating,
one for the accumulator.
"""
import numpy as np

from iree_amd import flags as F
from iree_amd import synth

# (m, k, n, accumulate)
SMALL = [(1, 1, 1, True), (1, 1, 1, False), (2, 2, 2, True), (4, 4, 4, True), (8, 8, 8, True),
         (9, 9, 9, True), (6, 13, 3, True), (15, 37, 7, False), (81, 19, 41, True),
         (1, 10, 10, True), (1, 10, 10, False), (10, 1, 10, True), (10, 10, 1, True),
         (10, 10, 1, False)]
LARGE = [(123, 456, 789, True), (654, 321, 234, False), (1, 1000, 1000, True),
         (1000, 1000, 1, True), (1000, 1000, 1, False)]

# name -> (mmt4d type flag, operand element, accumulator / result element)
TYPES = {
    "i8_i32": (F.MMT4D_TYPE_S8S8S32, "i8", "i32"),
    "f32_f32": (F.MMT4D_TYPE_F32F32F32, "f32", "f32"),
    "f16_f16": (F.MMT4D_TYPE_F16F16F16, "f16", "f16"),
    "f16_f32": (F.MMT4D_TYPE_F16F16F32, "f16", "f32"),
    "bf16_bf16": (F.MMT4D_TYPE_BF16BF16BF16, "bf16", "bf16"),
    "bf16_f32": (F.MMT4D_TYPE_BF16BF16F32, "bf16", "f32"),
}

NP_DTYPE = {"i8": np.int8, "i32": np.int32, "f16": np.float16, "bf16": np.uint16, "f32": np.float32}


def cases(shapes):
    """Yields (m, k, n, accumulate, dynamic, lhs_seed, rhs_seed, acc_seed) in
    the generator's order: shapes outer, dynamicity inner, seeds counting on."""
    seed = 1
    for (m, k, n, accumulate) in shapes:
        for dynamic in (True, False):
            lhs_seed, rhs_seed = seed + 1, seed + 2
            seed += 2
            acc_seed = None
            if accumulate:
                seed += 1
                acc_seed = seed
            yield m, k, n, accumulate, dynamic, lhs_seed, rhs_seed, acc_seed


def to_int64(x, elem):
    """The exact integer values of a generated matrix."""
    if elem == "bf16":
        return (x.astype(np.uint32) << np.uint32(16)).view(np.float32).astype(np.int64)
    return x.astype(np.int64)


def exact_result(lhs, rhs, acc, m, k, n, lhs_elem, out_elem):
    """The matmul in exact integer arithmetic, then the one rounding the result
    type implies (every partial sum is an integer below 2^24, so f32
    accumulation in any order is exact; f16 / bf16 results round once, to
    nearest even)."""
    s = to_int64(lhs, lhs_elem).reshape(m, k) @ to_int64(rhs, lhs_elem).reshape(k, n)
    if acc is not None:
        s = s + to_int64(acc, out_elem).reshape(m, n)
    assert np.abs(s).max(initial=0) < (1 << 24)
    if out_elem == "i32":
        return s.astype(np.int32)
    f = s.astype(np.float32)
    if out_elem == "f32":
        return f
    if out_elem == "f16":
        return f.astype(np.float16)
    # bf16, round to nearest even on the 16 discarded bits
    u = f.view(np.uint32)
    u = u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return (u >> np.uint32(16)).astype(np.uint16)


def operands(m, k, n, lhs_seed, rhs_seed, acc_seed, lhs_elem, out_elem):
    lhs = synth.e2e_matrix(lhs_seed, m * k, lhs_elem)
    rhs = synth.e2e_matrix(rhs_seed, k * n, lhs_elem)
    acc = synth.e2e_matrix(acc_seed, m * n, out_elem) if acc_seed is not None else None
    return lhs, rhs, acc
