"""The pack / unpack cases of the reference's end-to-end tensor-op tests, as data.

tests/e2e/tensor_ops/pack.mlir, pack_dynamic_inner_tiles.mlir (the same cases
with the tile sizes as run-time values), pack_i8.mlir and unpack.mlir check
`tensor.pack` / `tensor.unpack` either against literal constants or against
what pad + reshape + transpose of the same source give. Those ops reach the
ukernels with `inner_dims_pos = [1, 0]` as the TRANSPOSE_INNER flag and
`outer_dims_perm = [1, 0]` as TRANSPOSE_OUTER
(compiler/src/iree/compiler/Codegen/Common/CPU/CPULowerToUKernels.cpp:325-345,
:445-465); the result tensor's four sizes are the ukernel's out_size0..3.

A case: source shape (rows, columns), element type, tile in MATRIX orientation
(rows, columns), the two transposes, the padding value (None: the source is
whole tiles), and either `literal` (source and expected values written out in
the reference's file) or the expectation by construction. Sources of the
large cases are the reference's generators: element (i, j) = i * width + j
(modulo 256 for i8; pack.mlir:1-19, pack_i8.mlir:1-21), and for unpack the 4-D
tensor whose element is its own linear index (unpack.mlir:1-22).
"""
import numpy as np

# name, elem, rows, cols, tile rows, tile cols, transpose inner, transpose outer, padding
PACK_CASES = [
    # pack.mlir:21-58 (static and dynamic forms share the values), literal results below
    ("pack_simple", "i32", 4, 4, 2, 2, False, False, None),
    ("pack_simple_pad_mode", "i32", 4, 4, 3, 3, False, False, 0),
    # pack.mlir:99-243 / pack_dynamic_inner_tiles.mlir:78-275
    ("pack_large", "i32", 128, 256, 32, 16, False, False, None),
    ("pack_transpose_inner_dims_large", "i32", 128, 256, 32, 16, True, False, None),
    ("pack_pad_large", "i32", 100, 250, 32, 16, False, False, 42),
    ("pack_pad_transpose_outer_dims_large", "i32", 100, 250, 32, 16, False, True, 42),
    ("pack_pad_transpose_inner_dims_large", "i32", 100, 250, 32, 16, True, False, 42),
    ("pack_pad_transpose_inner_and_outer_dims_large", "i32", 100, 250, 32, 16, True, True, 42),
    # pack_i8.mlir:23-117 (the VNNI layouts: 16x2 tiles, right-hand side with both transposes)
    ("pack_vnni_lhs_large", "i8", 128, 256, 16, 2, False, False, None),
    ("pack_vnni_rhs_large", "i8", 256, 512, 2, 16, True, True, None),
    ("pack_vnni_lhs_large_with_pad", "i8", 127, 255, 16, 2, False, False, 0),
    ("pack_vnni_rhs_large_with_pad", "i8", 255, 511, 2, 16, True, True, 0),
    # tests/e2e/regression/pack_pad_transpose_1x9_into_2x4x8x4_issue_12546.mlir: a 1 x 9 row of
    # 1..9 into 2x4x8x4 with both transposes (matrix tiles of 4 rows x 8 columns) and padding 0,
    # the result written out in the file: the nine values head the columns of the first tiles
    ("pack_pad_transpose_1x9_into_2x4x8x4", "i8", 1, 9, 4, 8, True, True, 0),
]

# Result tensors with more outer tiles than the source needs (whole tiles of
# padding): name -> (outer rows, outer columns) in matrix orientation.
PACK_OUTER = {"pack_pad_transpose_1x9_into_2x4x8x4": (4, 2)}

PACK_LITERALS = {
    "pack_simple": [[[[0, 1], [4, 5]], [[2, 3], [6, 7]]], [[[8, 9], [12, 13]], [[10, 11], [14, 15]]]],
    "pack_simple_pad_mode": [[[[0, 1, 2], [4, 5, 6], [8, 9, 10]], [[3, 0, 0], [7, 0, 0], [11, 0, 0]]],
                             [[[12, 13, 14], [0, 0, 0], [0, 0, 0]], [[15, 0, 0], [0, 0, 0], [0, 0, 0]]]],
}

# name, rows, cols of the result, tile rows, tile cols, transpose inner, transpose outer
# (the packed source is whole tiles; results smaller than that are the
# "extract_slice" cases, unpack.mlir:223-444)
UNPACK_CASES = [
    ("unpack_simple", 4, 4, 2, 2, False, False),
    ("unpack_simple_extract_slice", 4, 4, 3, 3, False, False),
    ("unpack_large", 128, 256, 32, 16, False, False),
    ("unpack_transpose_inner_dims_large", 128, 256, 32, 16, True, False),
    ("unpack_transpose_outer_dims_large", 128, 256, 32, 16, False, True),
    ("unpack_transpose_inner_and_outer_dims_large", 128, 256, 32, 16, True, True),
    ("unpack_extract_slice_large", 100, 250, 32, 16, False, False),
    ("unpack_extract_slice_transpose_inner_dims_large", 100, 250, 32, 16, True, False),
    ("unpack_extract_slice_transpose_outer_dims_large", 100, 250, 32, 16, False, True),
    ("unpack_extract_slice_transpose_inner_and_outer_dims_large", 100, 250, 32, 16, True, True),
]

UNPACK_LITERALS = {
    # name: (packed source, expected matrix)
    "unpack_simple": (PACK_LITERALS["pack_simple"],
                      [[0, 1, 2, 3], [4, 5, 6, 7], [8, 9, 10, 11], [12, 13, 14, 15]]),
    "unpack_simple_extract_slice": (PACK_LITERALS["pack_simple_pad_mode"],
                                    [[0, 1, 2, 3], [4, 5, 6, 7], [8, 9, 10, 11], [12, 13, 14, 15]]),
}

NP = {"i32": np.int32, "i8": np.int8}


def _issue_12546_result():
    out = np.zeros((2, 4, 8, 4), dtype=np.int8)
    out[0, 0, :, 0] = np.arange(1, 9)
    out[1, 0, 0, 0] = 9
    return out


def pack_source(elem, rows, cols):
    if (elem, rows, cols) == ("i8", 1, 9):
        return np.arange(1, 10, dtype=np.int8).reshape(1, 9)
    lin = np.arange(rows * cols, dtype=np.int64).reshape(rows, cols)
    return (lin % 256).astype(np.uint8).view(np.int8) if elem == "i8" else lin.astype(np.int32)


def pack_expected(name, src, tr, tc, ti, to, padding):
    """What the reference's test compares with: the literal, or tensor.pad up
    to whole tiles, expand_shape to (outer rows, tile rows, outer columns, tile
    columns) and linalg.transpose into the result's order."""
    if name in PACK_LITERALS:
        return np.array(PACK_LITERALS[name], dtype=src.dtype)
    if name == "pack_pad_transpose_1x9_into_2x4x8x4":
        return _issue_12546_result()
    rows, cols = src.shape
    o0, o1 = -(-rows // tr), -(-cols // tc)
    padded = np.full((o0 * tr, o1 * tc), 0 if padding is None else padding, dtype=src.dtype)
    padded[:rows, :cols] = src
    r = padded.reshape(o0, tr, o1, tc)
    perm = {(False, False): (0, 2, 1, 3), (True, False): (0, 2, 3, 1),
            (False, True): (2, 0, 1, 3), (True, True): (2, 0, 3, 1)}[(ti, to)]
    return np.ascontiguousarray(r.transpose(perm))


def unpack_source_and_expected(name, rows, cols, tr, tc, ti, to):
    """The packed 4-D source (its elements their own linear indices) and the
    matrix the reference's test expects: the inverse transpose, collapse_shape
    and extract_slice of it."""
    if name in UNPACK_LITERALS:
        src, want = UNPACK_LITERALS[name]
        return np.array(src, dtype=np.int32), np.array(want, dtype=np.int32)
    o0, o1 = -(-rows // tr), -(-cols // tc)
    dims = {(False, False): (o0, o1, tr, tc), (True, False): (o0, o1, tc, tr),
            (False, True): (o1, o0, tr, tc), (True, True): (o1, o0, tc, tr)}[(ti, to)]
    src = np.arange(int(np.prod(dims)), dtype=np.int32).reshape(dims)
    # back to (outer rows, tile rows, outer columns, tile columns)
    inverse = {(False, False): (0, 2, 1, 3), (True, False): (0, 3, 1, 2),
               (False, True): (1, 2, 0, 3), (True, True): (1, 3, 0, 2)}[(ti, to)]
    full = src.transpose(inverse).reshape(o0 * tr, o1 * tc)
    return src, np.ascontiguousarray(full[:rows, :cols])
