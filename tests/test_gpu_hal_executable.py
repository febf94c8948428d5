"""The code object of the mmt4d kernels for a HAL executable on a HIP device
(iree_amd/hal/mi355x_kernels.hip), loaded and dispatched the way the reference's
HIP HAL driver does (runtime/src/iree/hal/drivers/hip/native_executable.c:180-253,
stream_command_buffer.c:519-581) through include/iree_amd_hal_executable.h.
Every export is checked against the oracle bit for bit on the reference's
small-integer inputs (tools/mmt4d_test.c:430-436), and the row-major-result
exports against the library's own fused entry point on N(0,1) data."""
import itertools
import os
import re
import zlib

import numpy as np
import pytest

import ukref
from iree_amd import flags as F
from iree_amd import hal_executable as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TILED = [n for n in H.EXPORTS if "_unpack_" not in n]
UNPACK = [n for n in H.EXPORTS if "_unpack_" in n]
# outer shapes: one tile, ragged macro tiles both ways, more workgroups than
# XCDs, K tile counts with and without a partial last matrix-core step
SHAPES = [(1, 1, 1), (1, 1, 8), (3, 2, 6), (5, 7, 10), (9, 4, 19), (17, 9, 4), (4, 33, 2), (2, 3, 44)]


def test_export_table_matches_the_sources():
    """The Python table, the kernel source and the committed MLIR agree."""
    with open(os.path.join(ROOT, "iree_amd", "hal", "mi355x_kernels.hip")) as f:
        src = f.read()
    rows = re.findall(r"^MI355X_MMT4D_EXPORTS\((\w+), \w+, \d+, \d+, \d+, \d+, \d+, (\d+)\)", src, re.M)
    assert len(rows) * 2 == len(H.EXPORTS)
    for name, lds in rows:
        for prefix in ("mi355x_mmt4d_", "mi355x_mmt4d_unpack_"):
            e = H.EXPORTS[prefix + name]
            assert e.lds == int(lds) and e.tile == int(name[-1])
    with open(os.path.join(ROOT, "iree_amd", "hal", "mi355x_kernels.mlir")) as f:
        assert f.read() == H.mlir_source()
    assert H.workgroup_count("mi355x_mmt4d_s8s8s32_t8", 9, 17) == 2 * 3
    assert H.workgroup_count("mi355x_mmt4d_s8s8s32_t4", 9, 17) == 3 * 5
    # f16 8191 x 5001 -> 32 x 16 tiles: 256 x 313 tiles = 8192 rows of 626 chunks
    assert H.pack_workgroup_count("mi355x_pack_16bit", 8191, 5001, 32, 16) == 20 * 512
    assert H.pack_workgroup_count("mi355x_unpack_16bit", 8191, 5001, 32, 16) == 20 * 512
    assert H.pack_workgroup_count("mi355x_unpack_32bit", 17, 9, 8, 4) == 1 * 2
    # f16 4096 x 4096 in tiles of 8 rows x 32 columns: one row group per tile row
    assert H.pack_transpose_workgroup_count("mi355x_pack_transpose_16bit", 4096, 4096, 8, 32) == 64 * 32
    assert H.pack_transpose_workgroup_count("mi355x_pack_transpose_16bit", 1001, 333, 8, 32) == 6 * 8
    assert H.pack_transpose_workgroup_count("mi355x_unpack_transpose_32bit", 95, 257, 32, 8) == 5 * 2
    mm = re.findall(r"^MI355X_MATMUL_EXPORT\((\w+), \w+, \d+, \d+, \d+, \d+, \d+, (\d+)\)", src, re.M)
    assert len(mm) == len(H.MATMUL_EXPORTS)
    for name, lds in mm:
        assert H.MATMUL_EXPORTS["mi355x_matmul_packed_rhs_" + name].lds == int(lds)
    assert H.matmul_workgroup_count("mi355x_matmul_packed_rhs_s8s8s32_t4x8", 200, 333) == 2 * 2
    assert H.matmul_workgroup_count("mi355x_matmul_packed_rhs_s8s8s32_t8x8", 4096, 4096) == 16 * 16
    assert sorted(re.findall(r"^MI355X_DEQUANT_I4_EXPORT\((\w+), \d\)", src, re.M)) == ["r16", "r32"]
    assert H.dequant_workgroup_count(14336) == 256 and H.dequant_workgroup_count(96) == 3


def test_code_object_is_built_and_names_every_export():
    with open(H.CODE_OBJECT, "rb") as f:
        image = f.read()
    for name in (list(H.EXPORTS) + list(H.PACK_EXPORTS) + list(H.PACK_TRANSPOSE_EXPORTS) + list(H.MATMUL_EXPORTS) +
                 list(H.DEQUANT_EXPORTS)):
        assert name.encode() + b"\0" in image, name


def test_library_exports_the_declared_entry_points(uk):
    with open(os.path.join(ROOT, "include", "iree_amd_hal_executable.h")) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    names = re.findall(r"IREE_AMD_HAL_EXPORT\s+\w+\s+(iree_amd_hal_executable_\w+)\s*\(", text)
    assert sorted(names) == ["iree_amd_hal_executable_add_export", "iree_amd_hal_executable_dispatch",
                             "iree_amd_hal_executable_load", "iree_amd_hal_executable_release"]
    lib = uk.load_library()
    for n in names:
        assert hasattr(lib, n)


@pytest.fixture(scope="module")
def exe(uk, cuda):
    e = H.HalExecutable()
    yield e
    e.close()


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("name", TILED)
def test_tiled_exports_bit_exact_against_the_oracle(exe, name):
    import torch
    e = H.EXPORTS[name]
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    for K0 in e.k0:
        for (M, N, K), acc in itertools.product(SHAPES, (False, True)):
            case = ukref.Mmt4dCase(rng, e.type_flag, M, N, K, 32, 32, K0, accumulate=acc)
            lhs, rhs, out = _dev(case.lhs), _dev(case.rhs), _dev(case.out_init)
            exe.mmt4d(name, lhs, rhs, out, M, N, K, K0, case.flags)
            torch.cuda.synchronize()
            got = out.cpu().numpy().view(case.out_init.dtype)
            want = case.run_oracle(ukref.F16_IEEE)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (name, K0, (M, N, K), acc)


@pytest.mark.gpu
@pytest.mark.parametrize("name", UNPACK)
def test_row_major_exports_equal_the_library_entry_point(uk, cuda, exe, name):
    """Same kernel body as iree_amd_uk_mmt4d_unpack: identical bits on float data,
    with ragged M and N, a partial last K step, with and without accumulation;
    elements outside the matrix stay untouched (the buffers are exactly M x N)."""
    import torch
    e = H.EXPORTS[name]
    K0 = e.k0[0]
    M, N = 200, 333
    K1 = 37
    M1, N1 = -(-M // 32), -(-N // 32)
    rng = np.random.default_rng(21)

    def operand(n):
        if e.type_flag == F.MMT4D_TYPE_S8S8S32:
            return torch.from_numpy(rng.integers(-128, 128, n, dtype=np.int8)).cuda()
        if e.type_flag == F.MMT4D_TYPE_F8E4M3F8E4M3F32:
            # every byte but the two NaN encodings
            b = rng.integers(0, 256, n, dtype=np.uint8)
            b[(b & 0x7F) == 0x7F] = 0x38
            return torch.from_numpy(b).cuda()
        x = torch.from_numpy(rng.standard_normal(n).astype(np.float32)).cuda()
        return {F.MMT4D_TYPE_F16F16F32: x.half(), F.MMT4D_TYPE_BF16BF16F32: x.bfloat16(),
                F.MMT4D_TYPE_F32F32F32: x}[e.type_flag]

    lhs, rhs = operand(M1 * K1 * 32 * K0), operand(N1 * K1 * 32 * K0)
    odt = torch.int32 if e.type_flag == F.MMT4D_TYPE_S8S8S32 else torch.float32
    for acc in (0, F.MMT4D_ACCUMULATE):
        init = torch.from_numpy(rng.integers(-50, 50, M * N).astype(np.int32)).cuda().to(odt)
        one, two = init.clone(), init.clone()
        exe.mmt4d(name, lhs, rhs, one, M1, N1, K1, K0, e.type_flag | acc, out_rows=M, out_cols=N)
        uk.mmt4d_unpack(lhs, rhs, two, M, N, M1, N1, K1, K0, e.type_flag | acc)
        torch.cuda.synchronize()
        assert np.array_equal(one.cpu().numpy().view(np.uint32), two.cpu().numpy().view(np.uint32)), (name, acc)
        assert not torch.equal(one, init)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["mi355x_mmt4d_s8s8s32_t8", "mi355x_mmt4d_f16f16f32_t4",
                                  "mi355x_mmt4d_f8e4m3f8e4m3f32_t8"])
def test_tiled_exports_batch_planes_bit_exact_against_the_oracle(exe, name):
    """A grid of `batch` planes in y: every plane has the bits of the
    reference's per-entry mmt4d call on dense operands."""
    import torch
    e = H.EXPORTS[name]
    rng = np.random.default_rng(zlib.crc32(name.encode()) + 1)
    for (batch, M, N, K), acc in itertools.product([(3, 2, 3, 5), (5, 9, 4, 2), (19, 9, 10, 3)], (False, True)):
        case = ukref.BatchMmt4dCase(rng, e.type_flag, batch, M, N, K, 32, 32, e.k0[0], accumulate=acc)
        lhs, rhs, out = _dev(case.lhs), _dev(case.rhs), _dev(case.out_init)
        exe.mmt4d(name, lhs, rhs, out, M, N, K, e.k0[0], case.flags, batch=batch)
        torch.cuda.synchronize()
        got = out.cpu().numpy().view(case.out_init.dtype)
        want = case.run_oracle(ukref.F16_IEEE)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (name, batch, (M, N, K), acc)


@pytest.mark.gpu
def test_row_major_export_batch_planes_equal_single_dispatches(uk, cuda, exe):
    import torch
    name = "mi355x_mmt4d_unpack_f16f16f32_t4"
    batch, M, N, K1, K0 = 3, 100, 77, 9, 8
    M1, N1 = -(-M // 32), -(-N // 32)
    g = torch.Generator(device="cuda").manual_seed(11)
    lhs = torch.randn(batch, M1 * K1 * 32 * K0, device="cuda", generator=g).half()
    rhs = torch.randn(batch, N1 * K1 * 32 * K0, device="cuda", generator=g).half()
    out = torch.full((batch, M, N), 3.0, device="cuda")
    exe.mmt4d(name, lhs, rhs, out, M1, N1, K1, K0, F.MMT4D_TYPE_F16F16F32, out_rows=M, out_cols=N,
              batch=batch)
    for b in range(batch):
        one = torch.full((M, N), 3.0, device="cuda")
        exe.mmt4d(name, lhs[b], rhs[b], one, M1, N1, K1, K0, F.MMT4D_TYPE_F16F16F32, out_rows=M, out_cols=N)
        assert torch.equal(out[b], one), b


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(H.MATMUL_EXPORTS))
def test_matmul_exports_equal_the_library_entry_point(uk, cuda, exe, name):
    """mi355x_matmul_packed_rhs_*: the bits of iree_amd_uk_matmul_packed_rhs (same
    kernel body) on random data, ragged M and N, with and without accumulation;
    for i8 also the exact integer product."""
    import torch
    e = H.MATMUL_EXPORTS[name]
    K0 = e.k0[0]
    M, N, K = 200, 333, 9 * e.mfma_k
    N1, K1 = -(-N // 32), K // K0
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    if e.type_flag == F.MMT4D_TYPE_S8S8S32:
        A = rng.integers(-128, 128, (M, K), dtype=np.int8)
        B = rng.integers(-128, 128, (N, K), dtype=np.int8)
        a_dev, b_dev, ptype = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), F.PACK_TYPE_I8I8
    elif e.type_flag == F.MMT4D_TYPE_F8E4M3F8E4M3F32:
        A = rng.integers(0, 256, (M, K), dtype=np.uint8)
        B = rng.integers(0, 256, (N, K), dtype=np.uint8)
        A[(A & 0x7F) == 0x7F] = 0x38
        B[(B & 0x7F) == 0x7F] = 0x38
        a_dev, b_dev, ptype = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), F.PACK_TYPE_I8I8
    else:
        tdt = {F.MMT4D_TYPE_F16F16F32: torch.float16, F.MMT4D_TYPE_BF16BF16F32: torch.bfloat16,
               F.MMT4D_TYPE_F32F32F32: torch.float32}[e.type_flag]
        a_dev = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).cuda().to(tdt)
        b_dev = torch.from_numpy(rng.standard_normal((N, K)).astype(np.float32)).cuda().to(tdt)
        ptype = F.PACK_TYPE_F32F32 if tdt == torch.float32 else F.PACK_TYPE_F16F16
    rhs = torch.empty(N1 * K1 * 32 * K0, dtype=b_dev.dtype, device=cuda)
    uk.pack(b_dev, rhs, N, K, N1, K1, 32, K0, 0, ptype)
    odt = torch.int32 if e.type_flag == F.MMT4D_TYPE_S8S8S32 else torch.float32
    for acc in (0, F.MMT4D_ACCUMULATE):
        init = torch.from_numpy(rng.integers(-50, 50, M * N).astype(np.int32)).cuda().to(odt)
        one, two = init.clone(), init.clone()
        exe.matmul_packed_rhs(name, a_dev, rhs, one, M, N, K, K0, e.type_flag | acc)
        uk.matmul_packed_rhs(a_dev, rhs, two, M, N, K, K0, e.type_flag | acc)
        torch.cuda.synchronize()
        assert np.array_equal(one.cpu().numpy().view(np.uint32), two.cpu().numpy().view(np.uint32)), (name, acc)
        if e.type_flag == F.MMT4D_TYPE_S8S8S32:
            want = A.astype(np.int32) @ B.astype(np.int32).T
            if acc:
                want = want + init.cpu().numpy().reshape(M, N)
            assert np.array_equal(one.cpu().numpy().reshape(M, N), want)


PACK_CASES = [  # size0, size1, tile0, tile1 (elements)
    (1, 1, 1, 16), (33, 70, 32, 16), (100, 257, 8, 32), (64, 64, 32, 32), (17, 500, 16, 64),
    (300, 33, 1, 16), (129, 1000, 32, 16), (200, 300, 32, 8), (77, 130, 32, 4), (45, 260, 8, 8),
    # tiles that are not powers of two, or whose rows are not whole 16-byte chunks (single elements)
    (50, 77, 24, 16), (123, 200, 12, 48), (9, 9, 3, 5), (130, 95, 7, 1), (40, 300, 32, 6), (65, 64, 5, 24)]


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(H.PACK_EXPORTS))
def test_pack_and_unpack_exports_match_the_closed_form(uk, cuda, exe, name):
    """pack: out[o0][o1][t0][t1] = in[o0 t0 + i0][o1 t1 + i1] or the padding element
    (the reference's own statement of it, tools/pack_test.c:36-70); unpack: the
    inverse, elements outside the matrix untouched (tools/unpack_test.c:13-58).
    Also bit-identical to the library's iree_amd_uk_pack / _unpack."""
    import torch
    es, is_pack = H.PACK_EXPORTS[name]
    dt = {1: np.uint8, 2: np.uint16, 4: np.uint32}[es]
    lib_type = {1: F.PACK_TYPE_I8I8, 2: F.PACK_TYPE_F16F16, 4: F.PACK_TYPE_F32F32}[es]
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    for size0, size1, tile0, tile1 in PACK_CASES:
        o0, o1 = -(-size0 // tile0), -(-size1 // tile1)
        pad = int(rng.integers(1, 1 << (8 * es)))
        mat = rng.integers(0, 1 << (8 * es), (size0, size1), dtype=np.uint64).astype(dt)
        padded = np.full((o0 * tile0, o1 * tile1), pad, dtype=dt)
        padded[:size0, :size1] = mat
        tiles = np.ascontiguousarray(padded.reshape(o0, tile0, o1, tile1).transpose(0, 2, 1, 3))
        if is_pack:
            src = torch.from_numpy(mat.view(np.uint8).reshape(-1).copy()).cuda()
            got = torch.full((tiles.size * es,), 0xA5, dtype=torch.uint8, device=cuda)
            ref = torch.full((tiles.size * es,), 0x5A, dtype=torch.uint8, device=cuda)
            exe.pack(name, src, got, size0, size1, tile0, tile1, pad)
            uk.pack(src, ref, size0, size1, o0, o1, tile0, tile1, pad, lib_type)
            torch.cuda.synchronize()
            assert np.array_equal(got.cpu().numpy(), tiles.view(np.uint8).reshape(-1)), (name, size0, size1, tile0, tile1)
            assert torch.equal(got, ref)
        else:
            src = torch.from_numpy(tiles.view(np.uint8).reshape(-1).copy()).cuda()
            # a destination with a guard row behind the matrix: it must stay as it was
            got = torch.full(((size0 + 1) * size1 * es,), 0xA5, dtype=torch.uint8, device=cuda)
            exe.unpack(name, src, got, size0, size1, tile0, tile1)
            torch.cuda.synchronize()
            out = got.cpu().numpy()
            assert np.array_equal(out[:size0 * size1 * es], mat.view(np.uint8).reshape(-1)), (name, size0, size1, tile0, tile1)
            assert (out[size0 * size1 * es:] == 0xA5).all()


TRANSPOSE_CASES = [  # (size0, size1, tile0 rows, tile1 columns)
    (1001, 333, 8, 32), (200, 95, 16, 32), (64, 64, 32, 32), (515, 70, 4, 32), (95, 257, 32, 8),
    (4096, 70, 8, 32), (1, 1, 16, 1), (129, 1003, 16, 4),
    # tiles that are not powers of two, or of less than 16 bytes of rows (single elements)
    (50, 77, 24, 8), (123, 200, 12, 5), (9, 9, 3, 5), (130, 95, 1, 7), (300, 40, 6, 32), (8, 8, 24, 8), (33, 65, 2, 2)]


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(H.PACK_TRANSPOSE_EXPORTS))
def test_transposing_pack_and_unpack_exports_match_the_closed_form(uk, cuda, exe, name):
    """Tiles of tile0 rows x tile1 columns stored column by column
    (IREE_UK_FLAG_PACK_TRANSPOSE_INNER, pack.c:131-166; unpack.c:190-247):
    out[o0][o1][i1][i0] = in[o0 tile0 + i0][o1 tile1 + i1] or the padding
    element; unpack: the inverse, nothing outside the matrix written. Also
    bit-identical to the library's iree_amd_uk_pack / _unpack with the flag."""
    import torch
    es, is_pack = H.PACK_TRANSPOSE_EXPORTS[name]
    dt = {1: np.uint8, 2: np.uint16, 4: np.uint32}[es]
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    for size0, size1, tile0, tile1 in TRANSPOSE_CASES:
        o0, o1 = -(-size0 // tile0), -(-size1 // tile1)
        pad = int(rng.integers(1, 1 << (8 * es)))
        mat = rng.integers(0, 1 << (8 * es), (size0, size1), dtype=np.uint64).astype(dt)
        padded = np.full((o0 * tile0, o1 * tile1), pad, dtype=dt)
        padded[:size0, :size1] = mat
        tiles = np.ascontiguousarray(padded.reshape(o0, tile0, o1, tile1).transpose(0, 2, 3, 1))
        if is_pack:
            lib_type = {1: F.PACK_TYPE_I8I8, 2: F.PACK_TYPE_F16F16, 4: F.PACK_TYPE_F32F32}[es]
            src = torch.from_numpy(mat.view(np.uint8).reshape(-1).copy()).cuda()
            got = torch.full((tiles.size * es,), 0xA5, dtype=torch.uint8, device=cuda)
            ref = torch.full((tiles.size * es,), 0x5A, dtype=torch.uint8, device=cuda)
            exe.pack_transpose(name, src, got, size0, size1, tile0, tile1, pad)
            uk.pack(src, ref, size0, size1, o0, o1, tile1, tile0, pad, lib_type | F.PACK_TRANSPOSE_INNER)
            torch.cuda.synchronize()
            assert np.array_equal(got.cpu().numpy(), tiles.view(np.uint8).reshape(-1)), (name, size0, size1, tile0, tile1)
            assert torch.equal(got, ref)
        else:
            lib_type = {2: F.UNPACK_TYPE_F16F16, 4: F.UNPACK_TYPE_F32F32}[es]
            src = torch.from_numpy(tiles.view(np.uint8).reshape(-1).copy()).cuda()
            got = torch.full(((size0 + 1) * size1 * es,), 0xA5, dtype=torch.uint8, device=cuda)
            ref = torch.full(((size0 + 1) * size1 * es,), 0xA5, dtype=torch.uint8, device=cuda)
            exe.unpack_transpose(name, src, got, size0, size1, tile0, tile1)
            uk.unpack(src, ref, o0, o1, tile1, tile0, size0, size1, lib_type | F.UNPACK_TRANSPOSE_INNER)
            torch.cuda.synchronize()
            out = got.cpu().numpy()
            assert np.array_equal(out[:size0 * size1 * es], mat.view(np.uint8).reshape(-1)), (name, size0, size1, tile0, tile1)
            assert (out[size0 * size1 * es:] == 0xA5).all()
            assert torch.equal(got, ref)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(H.DEQUANT_EXPORTS))
def test_dequant_exports_equal_the_library_entry_point(uk, cuda, exe, name):
    """mi355x_dequant_matmul_i4_k4096_g128_*: the bits of
    iree_amd_uk_dequant_matmul_i4 (same kernel body) on the decode shape and on
    a narrow one, and within the stated tolerance of the oracle; row counts the
    export does not take leave the result untouched."""
    import torch
    from iree_amd import synth
    from test_gpu_dequant import ATOL, RTOL, tile_weights
    K, gs = 4096, 128
    G = K // gs
    rows = H.DEQUANT_EXPORTS[name]
    for N, Ms in ((14336, [1, 8, rows - 7, rows]), (96, [rows - 1])):
        w = synth.uniform_u4_packed(2, N * K)
        s = synth.uniform_f16(4, N * G, 0.005, 0.02)
        zp = synth.uniform_u4_packed(5, N * G)
        wd = torch.from_numpy(tile_weights(w, N, K)).cuda()
        sd = torch.from_numpy(s.view(np.int16)).cuda()
        zd = torch.from_numpy(zp).cuda()
        for M in Ms:
            x = synth.normal_f16(M, M * K)
            xd = torch.from_numpy(x.view(np.int16)).cuda()
            one = torch.full((M * N,), 0x7E00, dtype=torch.int16, device=cuda)
            two = torch.full((M * N,), 0x7E00, dtype=torch.int16, device=cuda)
            exe.dequant_matmul_i4(name, xd, wd, sd, zd, one, M, N)
            uk.dequant_matmul_i4(xd, wd, sd, zd, two, M, N, K, gs,
                                 F.DEQUANT_MATMUL_ZP_U4 | F.DEQUANT_MATMUL_W_TILED)
            torch.cuda.synchronize()
            assert torch.equal(one, two), (name, M, N)
            if N == 96 or M == 1:
                want = np.zeros(M * N, np.uint16)
                assert ukref.oracle().oracle_dequant_matmul_i4(
                    ukref.ptr(x.view(np.uint16)), ukref.ptr(w), ukref.ptr(s.view(np.uint16)), ukref.ptr(zp),
                    ukref.ptr(want), M, N, K, gs, 1) == 0
                got = one.cpu().numpy().view(np.float16).astype(np.float64)
                wantf = want.view(np.float16).astype(np.float64)
                assert np.all(np.abs(got - wantf) <= ATOL + RTOL * np.abs(wantf)), (name, M, N)
        out = torch.full((64 * N,), 0x7E00, dtype=torch.int16, device=cuda)
        xd = torch.zeros(64 * K, dtype=torch.int16, device=cuda)
        for bad_m in (0, rows + 1):
            exe.dispatch(name, H.dequant_workgroup_count(N), [xd, wd, sd, zd, out], [bad_m, N])
        exe.dispatch(name, 1, [xd, wd, sd, zd, out], [1, 48])
        torch.cuda.synchronize()
        assert bool((out == 0x7E00).all())


@pytest.mark.gpu
def test_pack_export_round_trip_at_full_size(uk, cuda, exe):
    """f16 8191 x 5001 <-> 32 x 16 tiles: the library's packed bytes, and the
    round trip returns the source."""
    import torch
    from iree_amd import synth
    R, Cc = 8191, 5001
    o0, o1 = 256, 313
    x = torch.from_numpy(synth.uniform_pm1_f16(1, R * Cc).view(np.int16)).cuda()
    p1 = torch.empty(o0 * o1 * 512, dtype=torch.int16, device=cuda)
    p2 = torch.empty_like(p1)
    back = torch.zeros_like(x)
    exe.pack("mi355x_pack_16bit", x, p1, R, Cc, 32, 16, 0)
    uk.pack(x, p2, R, Cc, o0, o1, 32, 16, 0, F.PACK_TYPE_F16F16)
    exe.unpack("mi355x_unpack_16bit", p1, back, R, Cc, 32, 16)
    torch.cuda.synchronize()
    assert torch.equal(p1, p2)
    assert torch.equal(back, x)


@pytest.mark.gpu
def test_full_size_f16_dispatch_equals_the_library(uk, cuda, exe):
    """4096^3 f16 through the 256x256 export: the bits of iree_amd_uk_mmt4d."""
    import torch
    from iree_amd import synth
    M1 = N1 = 128
    K0, K1 = 8, 512
    lhs = torch.from_numpy(synth.normal_f16(1, 4096 * 4096, scale=1 / 64).view(np.int16)).cuda()
    rhs = torch.from_numpy(synth.normal_f16(2, 4096 * 4096, scale=1 / 64).view(np.int16)).cuda()
    one = torch.empty(4096 * 4096, dtype=torch.float32, device=cuda)
    two = torch.empty(4096 * 4096, dtype=torch.float32, device=cuda)
    exe.mmt4d("mi355x_mmt4d_f16f16f32_t8", lhs, rhs, one, M1, N1, K1, K0, F.MMT4D_TYPE_F16F16F32)
    uk.mmt4d(lhs, rhs, two, M1, N1, K1, 32, 32, K0, F.MMT4D_TYPE_F16F16F32)
    torch.cuda.synchronize()
    assert float(two.abs().max()) > 0
    assert torch.equal(one.view(torch.int32), two.view(torch.int32))


@pytest.mark.gpu
def test_loader_rejects_what_the_driver_rejects(uk, cuda, exe):
    with pytest.raises(uk.UkError) as err:
        exe.add_export("mi355x_no_such_kernel", shared_memory_size=0)
    assert err.value.status == 5 and "not found" in str(err.value)
    with pytest.raises(uk.UkError) as err:
        exe.add_export("mi355x_mmt4d_s8s8s32_t8", shared_memory_size=1 << 20)
    assert err.value.status == 3 and "shared memory" in str(err.value)
    with pytest.raises(uk.UkError):
        exe.add_export("mi355x_mmt4d_s8s8s32_t8", block=(2048, 1, 1))
    import ctypes as C
    lib = uk.load_library()
    handle = C.c_void_p()
    assert lib.iree_amd_hal_executable_load(None, 0, C.byref(handle)) == 3
    junk = b"not a code object" * 16
    assert lib.iree_amd_hal_executable_load(junk, len(junk), C.byref(handle)) != 0
    assert not handle.value
    # an empty grid is a no-op
    import torch
    out = torch.full((1024,), 7, dtype=torch.int32, device=cuda)
    exe.dispatch("mi355x_mmt4d_s8s8s32_t4", 0, [out, out, out], [0, 0, 1, 16, 0])
    torch.cuda.synchronize()
    assert int(out.min()) == 7
