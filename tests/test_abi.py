"""The C-ABI library loads, exports every symbol include/iree_amd_uk.h
declares, agrees with the reference's flag values, and its host-only entry
points (validation, tile-size query, info) behave - all without a GPU."""
import ctypes as C
import os
import re
import subprocess
import tempfile

import pytest

import iree_amd
from iree_amd import flags as F
from iree_amd._lib import (Mmt4dParams, PackParams, QueryOutParams, QueryParams,
                           UnpackParams)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "iree_amd_uk.h")


def _header_text():
    with open(HEADER) as f:
        return f.read()


def test_every_declared_symbol_is_exported():
    text = re.sub(r"/\*.*?\*/", "", _header_text(), flags=re.S)
    names = re.findall(r"IREE_AMD_UK_EXPORT\s+[\w\s\*]+?\b(iree_amd_uk_\w+)\s*\(", text)
    assert len(names) >= 24, names
    lib = iree_amd.load_library()
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"


# Values of the reference's exported_bits.h:29-106 ("set in stone"), as data.
REFERENCE_FLAG_VALUES = {
    "MMT4D_TYPE_F32F32F32": 0x01, "MMT4D_TYPE_S8S8S32": 0x02, "MMT4D_TYPE_F16F16F32": 0x03,
    "MMT4D_TYPE_F16F16F16": 0x04, "MMT4D_TYPE_BF16BF16F32": 0x05, "MMT4D_TYPE_BF16BF16BF16": 0x06,
    "MMT4D_TYPE_S16S16S32": 0x07, "MMT4D_TYPE_S16U4S32": 0x08, "MMT4D_TYPE_S16S8S32": 0x09,
    "MMT4D_TYPE_S8S4S32": 0x0A, "MMT4D_ACCUMULATE": 0x100,
    "MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION": 0x200, "MMT4D_SKIP_INTERMEDIATE_ROUNDINGS": 0x400,
    "MMT4D_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION": 0x1,
    "PACK_TYPE_F32F32": 1, "PACK_TYPE_I8I8": 2, "PACK_TYPE_I32I32": 3, "PACK_TYPE_F16F16": 4,
    "PACK_TYPE_BF16BF16": 5, "PACK_TRANSPOSE_INNER": 0x100, "PACK_TRANSPOSE_OUTER": 0x200,
    "UNPACK_TYPE_F32F32": 1, "UNPACK_TYPE_I32I32": 3, "UNPACK_TYPE_F16F16": 4,
    "UNPACK_TYPE_BF16BF16": 5, "UNPACK_TRANSPOSE_INNER": 0x100, "UNPACK_TRANSPOSE_OUTER": 0x200,
    "QUERY_TILE_SIZES_OPERAND_ROLE_LHS": 1, "QUERY_TILE_SIZES_OPERAND_ROLE_RHS": 2,
    "QUERY_TILE_SIZES_OPERAND_ROLE_RESULT": 3,
    "QUERY_TILE_SIZES_OPERATION_MATMUL_F32F32F32": 0x100,
    "QUERY_TILE_SIZES_OPERATION_MATMUL_I8I8I32": 0x200,
    "QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F32": 0x300,
    "QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F16": 0x400,
    "QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16F32": 0x500,
    "QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16BF16": 0x600,
}


def test_flag_values_equal_the_reference():
    defs = dict(re.findall(r"#define IREE_AMD_UK_FLAG_(\w+)\s+(0x[0-9A-Fa-f]+|\d+)", _header_text()))
    for name, val in REFERENCE_FLAG_VALUES.items():
        assert int(defs[name], 0) == val, name
    # the Python mirror agrees with the header
    py = {"QUERY_ROLE_LHS": "QUERY_TILE_SIZES_OPERAND_ROLE_LHS",
          "QUERY_OP_MATMUL_I8I8I32": "QUERY_TILE_SIZES_OPERATION_MATMUL_I8I8I32",
          "QUERY_OP_MATMUL_F16F16F32": "QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F32"}
    for name in dir(F):
        hname = py.get(name, name)
        if hname in defs and isinstance(getattr(F, name), int):
            assert getattr(F, name) == int(defs[hname], 0), name
    # flag words the reference's compiler tests pin
    # (Codegen/Common/CPU/test/lower_to_ukernel_ops.mlir:212 and the blog walkthrough)
    assert (F.MMT4D_TYPE_F16F16F16 | F.MMT4D_ACCUMULATE | F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION |
            F.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) == 1796
    assert (F.MMT4D_TYPE_F32F32F32 | F.MMT4D_ACCUMULATE | F.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) == 1281


def test_struct_layout_matches_the_c_header():
    src = r'''
#include <stdio.h>
#include <stddef.h>
#include "iree_amd_uk.h"
int main(void) {
  printf("%zu %zu %zu %zu %zu\n", sizeof(iree_amd_uk_mmt4d_params_t), sizeof(iree_amd_uk_pack_params_t),
         sizeof(iree_amd_uk_unpack_params_t), sizeof(iree_amd_uk_query_tile_sizes_2d_params_t),
         sizeof(iree_amd_uk_query_tile_sizes_2d_out_params_t));
  printf("%zu %zu %zu %zu\n", offsetof(iree_amd_uk_mmt4d_params_t, M0), offsetof(iree_amd_uk_mmt4d_params_t, flags),
         offsetof(iree_amd_uk_pack_params_t, padding_value), offsetof(iree_amd_uk_unpack_params_t, flags));
  return 0;
}'''
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        with open(c, "w") as f:
            f.write(src)
        exe = os.path.join(d, "t")
        subprocess.check_call(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-I",
                               os.path.join(ROOT, "include"), c, "-o", exe])
        out = subprocess.check_output([exe]).decode().split()
    sizes = [int(x) for x in out]
    assert sizes[:5] == [C.sizeof(Mmt4dParams), C.sizeof(PackParams), C.sizeof(UnpackParams),
                         C.sizeof(QueryParams), C.sizeof(QueryOutParams)]
    assert sizes[5:] == [Mmt4dParams.M0.offset, Mmt4dParams.flags.offset,
                         PackParams.padding_value.offset, UnpackParams.flags.offset]


def test_query_tile_sizes_roles_and_narrowing():
    q = iree_amd.query_tile_sizes_2d
    # (M0, N0, K0) per operation: one 32x32 MFMA block, K0 = the 16 bytes a lane feeds it
    for op, (m0, n0, k0) in [(F.QUERY_OP_MATMUL_I8I8I32, (32, 32, 16)),
                             (F.QUERY_OP_MATMUL_F16F16F32, (32, 32, 8)),
                             (F.QUERY_OP_MATMUL_BF16BF16F32, (32, 32, 8)),
                             (F.QUERY_OP_MATMUL_F8E4M3F8E4M3F32, (32, 32, 16))]:
        assert q(op | F.QUERY_ROLE_LHS) == (m0, k0)
        assert q(op | F.QUERY_ROLE_RHS) == (n0, k0)
        assert q(op | F.QUERY_ROLE_RESULT) == (m0, n0)
        # role mapping equals the reference's (query_tile_sizes.c:43-63) via the oracle
        import ukref
        t0, t1 = C.c_int64(), C.c_int64()
        for role in (F.QUERY_ROLE_LHS, F.QUERY_ROLE_RHS, F.QUERY_ROLE_RESULT):
            assert ukref.oracle().oracle_query_role_tile(role, m0, n0, k0, C.byref(t0), C.byref(t1)) == 0
            assert q(op | role) == (t0.value, t1.value)
    # narrow static sizes shrink to the next power of two, never below 1
    op = F.QUERY_OP_MATMUL_F16F16F32
    assert q(op | F.QUERY_ROLE_LHS, 1, 4096) == (1, 8)
    assert q(op | F.QUERY_ROLE_LHS, 7, 4096) == (8, 8)
    assert q(op | F.QUERY_ROLE_LHS, 17, 4096) == (32, 8)
    assert q(op | F.QUERY_ROLE_RHS, 4096, 4096) == (32, 8)
    assert q(op | F.QUERY_ROLE_RHS, 5, 4096) == (8, 8)
    # the result role sees both sizes and narrows only the smaller one, N by
    # transposition only when it is the narrower of the two
    # (CPUMaterializeEncodingPass.cpp:296-303 of the reference)
    assert q(op | F.QUERY_ROLE_RESULT, 8, 3) == (32, 4)
    assert q(op | F.QUERY_ROLE_RESULT, 3, 8) == (4, 32)
    assert q(op | F.QUERY_ROLE_RESULT, 8, 8) == (8, 32)
    assert q(op | F.QUERY_ROLE_RESULT, 4096, 1) == (32, 1)
    assert q(op | F.QUERY_ROLE_RESULT, 16, 4096) == (16, 32)
    with pytest.raises(iree_amd.UkError) as e:
        q(0x0700 | F.QUERY_ROLE_LHS)
    assert e.value.status == F.STATUS_INVALID_ARGUMENT
    with pytest.raises(iree_amd.UkError):
        q(op | 0x7)


def test_mmt4d_info_reports_mfma_tiles():
    have = F.MMT4D_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION
    assert iree_amd.mmt4d_info(32, 32, 8, F.MMT4D_TYPE_F16F16F32) == have
    assert iree_amd.mmt4d_info(32, 32, 16, F.MMT4D_TYPE_F16F16F32) == have
    assert iree_amd.mmt4d_info(32, 32, 16, F.MMT4D_TYPE_S8S8S32) == have
    assert iree_amd.mmt4d_info(32, 32, 32, F.MMT4D_TYPE_S8S8S32) == have
    assert iree_amd.mmt4d_info(16, 16, 1, F.MMT4D_TYPE_F16F16F32) == 0
    # 16-bit left-hand sides run as int8 digit planes at 32 x 32 tiles of any K0
    assert iree_amd.mmt4d_info(32, 32, 8, F.MMT4D_TYPE_S16S16S32) == have
    assert iree_amd.mmt4d_info(32, 32, 2, F.MMT4D_TYPE_S16U4S32) == have
    assert iree_amd.mmt4d_info(16, 16, 2, F.MMT4D_TYPE_S16S16S32) == 0
    # ... and at narrow tiles of 1 to 31 rows (the reference's own s16 x u4 tile is 1 x 32 x 8)
    assert iree_amd.mmt4d_info(1, 32, 8, F.MMT4D_TYPE_S16U4S32) == have
    assert iree_amd.mmt4d_info(15, 32, 8, F.MMT4D_TYPE_S16S8S32) == have
    assert iree_amd.mmt4d_info(16, 32, 8, F.MMT4D_TYPE_S16S8S32) == have
    assert iree_amd.mmt4d_info(4, 32, 8, F.MMT4D_TYPE_S16S16S32) == have
    assert iree_amd.mmt4d_info(32, 16, 8, F.MMT4D_TYPE_S16S16S32) == 0


def test_enumerated_tiles_and_the_chooser_follow_the_reference():
    """enumerate_matmul_tiles / choose_matmul_tile against what
    CPUMaterializeEncodingPass.cpp:168-377 documents: tile lists are the full
    tile and its truncations in M; the example of its comment (narrow M = 7 with
    tiles of M = 8, 4, 2, 1 keeps M = 8); the reference's own avx512 f32 list
    for matvec / vecmat shapes; narrow N reduced to narrow M with M and N
    exchanged; upper bounds; and a brute-force restatement of the rating rule
    on random tile lists. query_tile_sizes_2d answers with the chooser's tile."""
    import itertools
    import random
    assert iree_amd.enumerate_matmul_tiles(F.QUERY_OP_MATMUL_F16F16F32) == [
        (32, 32, 8), (16, 32, 8), (8, 32, 8), (4, 32, 8), (2, 32, 8), (1, 32, 8)]
    assert iree_amd.enumerate_matmul_tiles(F.QUERY_OP_MATMUL_I8I8I32)[0] == (32, 32, 16)
    assert iree_amd.enumerate_matmul_tiles(F.QUERY_OP_MATMUL_F32F32F32)[-1] == (1, 32, 4)
    with pytest.raises(iree_amd.UkError):
        iree_amd.enumerate_matmul_tiles(0x7F)
    ch = iree_amd.choose_matmul_tile
    assert ch([(8, 8, 1), (4, 8, 1), (2, 8, 1), (1, 8, 1)], narrow_m=7) == (8, 8, 1)
    avx512 = [(16, 16, 1), (8, 16, 1), (4, 16, 1), (2, 16, 1), (1, 16, 1)]     # its lines 195-201
    assert ch(avx512) == (16, 16, 1)
    assert ch(avx512, narrow_m=1) == (1, 16, 1)
    assert ch(avx512, narrow_n=1) == (16, 1, 1)
    assert ch(avx512, narrow_m=3) == (4, 16, 1)
    assert ch(avx512, narrow_m=5, narrow_n=2) == (16, 2, 1)      # N the narrower: exchanged
    assert ch(avx512, narrow_m=2, narrow_n=5) == (2, 16, 1)
    assert ch(avx512, narrow_m=4, narrow_n=4) == (4, 16, 1)      # a tie stays a narrow-M problem
    assert ch(avx512, upper_bound=(4, 16, 1)) == (4, 16, 1)
    assert ch(avx512, narrow_m=1, upper_bound=(8, 16, 1)) == (1, 16, 1)
    with pytest.raises(iree_amd.UkError):
        ch(avx512, upper_bound=(16, 8, 1))

    def pow2ceil(v):
        return 1 << (v - 1).bit_length() if v > 1 else 1

    def restated(tiles, nm, nn, ub):
        if nn and (not nm or nn < nm):
            m, n, k = restated(tiles, nn, 0, ub)
            return n, m, k
        ok = [t for t in tiles if ub is None or (t[0] <= ub[0] and t[1] <= ub[1] and t[2] <= ub[2])]
        pen = [max(t[0] - pow2ceil(nm), 0) if nm else 0 for t in ok]
        best = [t for t, p in zip(ok, pen) if p == min(pen)]
        return max(best, key=lambda t: t[0] * t[1] * t[2])       # (max keeps the first of equals)

    rnd = random.Random(5)
    for _ in range(300):
        tiles = [(rnd.choice([1, 2, 4, 8, 16, 32]), rnd.choice([4, 8, 16, 32]), rnd.choice([1, 2, 4, 8, 16]))
                 for _ in range(rnd.randint(1, 7))]
        nm, nn = rnd.choice([0, 0, 1, 3, 7, 8, 20]), rnd.choice([0, 0, 1, 2, 5, 16])
        ub = rnd.choice([None, None, (32, 32, 16), (8, 32, 16)])
        try:
            want = restated(tiles, nm, nn, ub)
        except ValueError:
            with pytest.raises(iree_amd.UkError):
                ch(tiles, nm, nn, ub)
            continue
        assert ch(tiles, nm, nn, ub) == want, (tiles, nm, nn, ub)
    # the run-time query is this chooser on the enumerated tiles
    q = iree_amd.query_tile_sizes_2d
    for op in (F.QUERY_OP_MATMUL_I8I8I32, F.QUERY_OP_MATMUL_F16F16F32, F.QUERY_OP_MATMUL_F32F32F32,
               F.QUERY_OP_MATMUL_F8E4M3F8E4M3F32):
        tiles = iree_amd.enumerate_matmul_tiles(op)
        for m, n in itertools.product([1, 2, 3, 7, 8, 15, 17, 31, 32, 500], repeat=2):
            narrow_m, narrow_n = (m if m < 32 else 0), (n if n < 32 else 0)
            M0, N0, K0 = ch(tiles, narrow_m, narrow_n)
            assert q(op | F.QUERY_ROLE_RESULT, m, n) == (M0, N0), (hex(op), m, n)
            assert q(op | F.QUERY_ROLE_LHS, m if M0 < 32 else -2 ** 63, 4096) == (M0, K0)
            assert q(op | F.QUERY_ROLE_RHS, n if N0 < 32 else -2 ** 63, 4096) == (N0, K0)


def test_query_matmul_tile_sizes_gives_one_consistent_tile():
    """The three-size query: the chooser on the enumerated tiles with the
    static sizes below 32 as narrow sizes, so at most one of M0 / N0 is
    narrowed whatever the caller passes, it agrees with the RESULT role, and
    every answer has a matrix-core kernel."""
    have = F.MMT4D_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION
    dyn = -2 ** 63
    qm, q, ch = iree_amd.query_matmul_tile_sizes, iree_amd.query_tile_sizes_2d, iree_amd.choose_matmul_tile
    assert qm(F.QUERY_OP_MATMUL_F16F16F32, 4, 8, 4096) == (4, 32, 8)     # the wider of two narrow sizes stays full
    assert qm(F.QUERY_OP_MATMUL_F16F16F32, 8, 4, 4096) == (32, 4, 8)
    assert qm(F.QUERY_OP_MATMUL_I8I8I32, 1000, 1, 1000) == (32, 1, 16)
    assert qm(F.QUERY_OP_MATMUL_I8I8I32, 1, 1000, 1000) == (1, 32, 16)
    assert qm(F.QUERY_OP_MATMUL_F32F32F32) == (32, 32, 4)
    assert qm(F.QUERY_OP_MATMUL_F32F32F32, 9, dyn, dyn) == (16, 32, 4)
    for op, type_flag in [(F.QUERY_OP_MATMUL_I8I8I32, F.MMT4D_TYPE_S8S8S32),
                          (F.QUERY_OP_MATMUL_F16F16F16, F.MMT4D_TYPE_F16F16F16),
                          (F.QUERY_OP_MATMUL_BF16BF16F32, F.MMT4D_TYPE_BF16BF16F32),
                          (F.QUERY_OP_MATMUL_F32F32F32, F.MMT4D_TYPE_F32F32F32)]:
        tiles = iree_amd.enumerate_matmul_tiles(op)
        for m in (dyn, 0, 1, 2, 3, 9, 10, 15, 16, 31, 32, 81, 1000):
            for n in (dyn, 0, 1, 3, 7, 10, 16, 19, 32, 41, 1000):
                M0, N0, K0 = qm(op, m, n, 64)
                assert (M0, N0, K0) == ch(tiles, max(m, 1) if -1 < m < 32 else 0, max(n, 1) if -1 < n < 32 else 0)
                assert (M0, N0) == q(op | F.QUERY_ROLE_RESULT, m, n)
                assert M0 == 32 or N0 == 32
                assert iree_amd.mmt4d_info(M0, N0, K0, type_flag | F.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) == have
    with pytest.raises(iree_amd.UkError):
        qm(0x7F00, 1, 1, 1)


def test_every_tile_the_query_returns_has_an_architecture_kernel():
    """mmt4d_info reports a matrix-core kernel for each tile
    query_tile_sizes_2d can hand out: full tiles, narrow M0 (static M < 32) and
    narrow N0 (static N < 32, served with the operands exchanged)."""
    have = F.MMT4D_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION
    q = iree_amd.query_tile_sizes_2d
    dyn = -2 ** 63
    sizes = [dyn, 1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 32, 33, 4096]
    for op, type_flag in [(F.QUERY_OP_MATMUL_I8I8I32, F.MMT4D_TYPE_S8S8S32),
                          (F.QUERY_OP_MATMUL_F16F16F32, F.MMT4D_TYPE_F16F16F32),
                          (F.QUERY_OP_MATMUL_F16F16F16, F.MMT4D_TYPE_F16F16F16),
                          (F.QUERY_OP_MATMUL_BF16BF16F32, F.MMT4D_TYPE_BF16BF16F32),
                          (F.QUERY_OP_MATMUL_BF16BF16BF16, F.MMT4D_TYPE_BF16BF16BF16),
                          (F.QUERY_OP_MATMUL_F32F32F32, F.MMT4D_TYPE_F32F32F32),
                          (F.QUERY_OP_MATMUL_F8E4M3F8E4M3F32, F.MMT4D_TYPE_F8E4M3F8E4M3F32)]:
        flags = type_flag | F.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS
        for m in sizes:
            for n in sizes:
                m0, n0 = q(op | F.QUERY_ROLE_RESULT, m, n)
                assert m0 == 32 or n0 == 32, (m, n, m0, n0)
                # The operand queries a caller makes for this matmul. Only one
                # dimension is narrowed; a caller passes the other one, when it
                # is below 32 too, as dynamic, so that its operand keeps the
                # full tile.
                m_arg, n_arg = m, n
                if m0 < 32 and 0 < n < 32:
                    n_arg = dyn
                if n0 < 32 and 0 < m < 32:
                    m_arg = dyn
                lm0, k0 = q(op | F.QUERY_ROLE_LHS, m_arg, 4096)
                rn0, rk0 = q(op | F.QUERY_ROLE_RHS, n_arg, 4096)
                assert (lm0, rn0, rk0) == (m0, n0, k0), (m, n)
                assert iree_amd.mmt4d_info(m0, n0, k0, flags) == have, (hex(type_flag), m0, n0, k0)
        # each operand query on its own also only yields served tiles
        for sz in sizes:
            lm0, k0 = q(op | F.QUERY_ROLE_LHS, sz, 4096)
            assert iree_amd.mmt4d_info(lm0, 32, k0, flags) == have
            rn0, k0 = q(op | F.QUERY_ROLE_RHS, sz, 4096)
            assert iree_amd.mmt4d_info(32, rn0, k0, flags) == have


def test_validation_happens_before_any_device_work():
    """Invalid calls are rejected and degenerate calls return OK without a GPU
    (no compute is attempted in this test)."""
    lib = iree_amd.load_library()
    one = C.c_void_p(16)
    # unknown flag bits / unknown type / bad sub-byte K0 (reference mmt4d.c:12-48)
    assert lib.iree_amd_uk_mmt4d(one, 0, 8, one, 0, 8, one, 0, 8, 1, 1, 1, 2, 2, 2, 0x802, None, None) == 3
    assert lib.iree_amd_uk_mmt4d(one, 0, 8, one, 0, 8, one, 0, 8, 1, 1, 1, 2, 2, 2, 0x0C, None, None) == 3
    assert lib.iree_amd_uk_mmt4d(one, 0, 8, one, 0, 8, one, 0, 8, 1, 1, 1, 2, 2, 3, F.MMT4D_TYPE_S8S4S32, None, None) == 3
    assert lib.iree_amd_uk_mmt4d(one, 0, 8, one, 0, 8, one, 0, 8, 1, 1, 1, 40000, 2, 2, 2, None, None) == 3
    assert b"M0/N0/K0" in lib.iree_amd_uk_last_error()
    # early returns (reference mmt4d.c:105-113)
    assert lib.iree_amd_uk_mmt4d(None, 0, 8, None, 0, 8, None, 0, 8, 0, 5, 7, 2, 2, 2, 2, None, None) == 0
    assert lib.iree_amd_uk_mmt4d(None, 0, 8, None, 0, 8, None, 0, 8, 5, 7, 0, 2, 2, 2, 2 | 0x100, None, None) == 0
    # pack: out_stride1 must be the tile size (reference pack.c:72); I8 unpack does not exist
    assert lib.iree_amd_uk_pack(one, 0, 4, 1, one, 0, 99, 7, 2, 4, 1, 2, 2, 2, 0, 1, None, None) == 3
    assert lib.iree_amd_uk_pack(one, 0, 4, 1, one, 0, 8, 4, 5, 4, 1, 2, 2, 2, 0, 1, None, None) == 3
    assert lib.iree_amd_uk_pack(None, 0, 4, 1, None, 0, 8, 4, 0, 0, 0, 2, 2, 2, 0, 1, None, None) == 0
    assert lib.iree_amd_uk_unpack(one, 0, 8, 4, one, 0, 4, 1, 1, 2, 2, 2, 2, 4, 2, None, None) == 3
    assert lib.iree_amd_uk_unpack(None, 0, 8, 4, None, 0, 4, 1, 1, 2, 2, 2, 0, 4, 1, None, None) == 0
    assert lib.iree_amd_uk_dequant_matmul_i4(one, one, one, one, one, 1, 8, 100, 32, 0, None) == 3
    # the fused forms: size conditions of unpack for 32x32 tiles, row pitches, scale rules, empty calls
    f1 = C.c_float(1.0)
    mu = lib.iree_amd_uk_mmt4d_unpack
    assert mu(one, 0, 512, one, 0, 512, one, 0, 64, 32, 64, 2, 2, 2, 16, 2, f1, None) == 3    # 32 rows cannot need 2 outer rows
    assert mu(one, 0, 512, one, 0, 512, one, 0, 63, 33, 64, 2, 2, 2, 16, 2, f1, None) == 3    # pitch below a row
    assert mu(one, 0, 512, one, 0, 512, one, 0, 64, 33, 64, 2, 2, 2, 16, 2, C.c_float(2.0), None) == 3   # scale on integers
    assert mu(None, 0, 512, None, 0, 512, None, 0, 64, 0, 64, 0, 2, 2, 16, 2, f1, None) == 0
    mp = lib.iree_amd_uk_matmul_packed_rhs
    assert mp(one, 0, 64, one, 0, 2048, one, 0, 64, 33, 64, 64, 0, 2, f1, None) == 3        # K0 = 0
    assert mp(one, 0, 63, one, 0, 2048, one, 0, 64, 33, 64, 64, 16, 2, f1, None) == 3       # lhs pitch below a row
    assert mp(one, 0, 64, one, 0, 2048, one, 0, 64, 33, 64, 40, 16, 2, f1, None) == 12      # K not whole tiles
    assert mp(None, 0, 64, None, 0, 2048, None, 0, 64, 0, 64, 64, 16, 2, f1, None) == 0
    # their batch forms: the same checks, a negative batch, an empty batch
    bmu = lib.iree_amd_uk_batch_mmt4d_unpack
    assert bmu(one, 0, 512, one, 0, 512, one, 0, 64, 33, 64, 2, 2, 2, 16, 2, f1, -1, 0, 0, 0, None) == 3
    assert bmu(one, 0, 512, one, 0, 512, one, 0, 63, 33, 64, 2, 2, 2, 16, 2, f1, 3, 0, 0, 0, None) == 3
    assert bmu(None, 0, 512, None, 0, 512, None, 0, 64, 33, 64, 2, 2, 2, 16, 2, f1, 0, 0, 0, 0, None) == 0
    bmp = lib.iree_amd_uk_batch_matmul_packed_rhs
    assert bmp(one, 0, 64, one, 0, 2048, one, 0, 64, 33, 64, 64, 16, 2, f1, -2, 0, 0, 0, None) == 3
    assert bmp(one, 0, 64, one, 0, 2048, one, 0, 64, 33, 64, 40, 16, 2, f1, 2, 0, 0, 0, None) == 12
    assert bmp(None, 0, 64, None, 0, 2048, None, 0, 64, 33, 64, 64, 16, 2, f1, 0, 0, 0, 0, None) == 0
    assert lib.iree_amd_uk_mfma_probe(2, None, 1, None, None, None) == 3
    # the newer entry points: sizes are checked before buffers, buffers before any launch
    assert lib.iree_amd_uk_quantize_groups_i16(one, one, one, one, 2, 100, 32, None) == 3        # K not whole groups
    assert lib.iree_amd_uk_quantize_groups_i16(None, None, None, None, 0, 128, 32, None) == 0
    assert lib.iree_amd_uk_quantize_groups_i16(None, one, one, one, 2, 128, 32, None) == 3
    assert lib.iree_amd_uk_quantize_pack_f8e4m3(one, 40, one, 40 * 32, 3, 40, f1, None) == 3    # cols not whole tiles
    assert lib.iree_amd_uk_quantize_pack_f8e4m3(one, 16, one, 32 * 32, 3, 32, f1, None) == 3    # pitch below a row
    assert lib.iree_amd_uk_quantize_pack_f8e4m3(None, 32, None, 32 * 32, 0, 32, f1, None) == 0
    assert lib.iree_amd_uk_quantize_pack_f8e4m3(one, 32, None, 32 * 32, 3, 32, f1, None) == 3
    assert lib.iree_amd_uk_copy_probe(None, one, 8192, 0, 0, None) == 3
    assert lib.iree_amd_uk_dequant_matmul_i4(one, one, one, one, one, 1, 8, 128, 32, 0x8, None) == 3   # unknown flag bit
    assert lib.iree_amd_uk_mmt4d_noalloc_p(None, None) == 3
    assert lib.iree_amd_uk_release_scratch() == 0
    assert lib.iree_amd_uk_version() >= 1
