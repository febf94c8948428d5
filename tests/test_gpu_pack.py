"""GPU parity of pack / unpack against the oracle, bit-exact, through the C ABI:
the reference's own test matrix (tools/pack_test.c:137-246,
tools/unpack_test.c:123-218) plus the gfx950 tile shapes, which take the
streaming kernels, and the full-size bandwidth workload (f16 8191x5001 <-> 32x16)."""
import hashlib
import itertools
import json
import os

import numpy as np
import pytest

import gpucase
import ukref
from iree_amd import flags as F
from iree_amd import synth
from test_oracle_pack import OUTER, PACK_TILES, PADS, UNPACK_TILES

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "golden.json")


@pytest.mark.parametrize("type_flag,t0,t1", PACK_TILES)
def test_pack_matches_oracle(uk, cuda, type_flag, t0, t1):
    rng = np.random.default_rng(131 * type_flag + 7 * t0 + t1)
    for (o0, o1), ti, to, pad in itertools.product(OUTER, (0, 1), (0, 1), PADS):
        for aligned in (False, True):
            # `aligned`: tight strides, zero offsets, unit inner stride -> the
            # streaming kernel where the tile shape allows it
            case = ukref.PackCase(rng, type_flag, o0, o1, t0, t1, transpose_inner=ti,
                                  transpose_outer=to, pad=pad,
                                  loose_strides=(not aligned) and bool(rng.integers(0, 2)),
                                  offsets=not aligned,
                                  in_stride1=1 if aligned else 1 + int(rng.integers(0, 2)))
            got = gpucase.run_pack(case)
            assert np.array_equal(got, case.run_oracle()), (o0, o1, ti, to, pad, aligned)


@pytest.mark.parametrize("type_flag,t0,t1", UNPACK_TILES)
def test_unpack_matches_oracle(uk, cuda, type_flag, t0, t1):
    rng = np.random.default_rng(117 * type_flag + 5 * t0 + t1)
    for (o0, o1), ti, to, pad in itertools.product(OUTER, (0, 1), (0, 1), PADS):
        for aligned in (False, True):
            case = ukref.UnpackCase(rng, type_flag, o0, o1, t0, t1, transpose_inner=ti,
                                    transpose_outer=to, pad=pad,
                                    loose_strides=(not aligned) and bool(rng.integers(0, 2)),
                                    offsets=not aligned,
                                    out_stride1=1 if aligned else 1 + int(rng.integers(0, 2)))
            got = gpucase.run_unpack(case)
            # compares the WHOLE destination buffer: elements outside the
            # matrix (stride gaps, the tail) must be untouched
            assert np.array_equal(got, case.run_oracle()), (o0, o1, ti, to, pad, aligned)


@pytest.mark.parametrize("type_flag,t0,t1,rows,cols", [
    (F.PACK_TYPE_F16F16, 32, 16, 333, 1001),   # odd row pitch: 2-byte aligned rows
    (F.PACK_TYPE_F16F16, 32, 8, 95, 257),
    (F.PACK_TYPE_I8I8, 32, 16, 129, 1003),     # 1-byte aligned rows
    (F.PACK_TYPE_I8I8, 32, 32, 64, 4096),
    (F.PACK_TYPE_F32F32, 32, 32, 70, 515),
    (F.PACK_TYPE_I32I32, 8, 4, 37, 123),
    (F.PACK_TYPE_BF16BF16, 16, 64, 100, 700),
])
def test_streaming_shapes_with_ragged_edges(uk, cuda, type_flag, t0, t1, rows, cols):
    rng = np.random.default_rng(rows * cols)
    for to in (0, 1):
        o0, o1 = -(-rows // t0), -(-cols // t1)
        case = ukref.PackCase(rng, type_flag, o0, o1, t0, t1, transpose_outer=to,
                              in_size=(rows, cols))
        packed = gpucase.run_pack(case)
        assert np.array_equal(packed, case.run_oracle()), (to,)
        if type_flag != F.PACK_TYPE_I8I8:
            ucase = ukref.UnpackCase(rng, type_flag, o0, o1, t0, t1, transpose_outer=to,
                                     out_size=(rows, cols))
            assert np.array_equal(gpucase.run_unpack(ucase), ucase.run_oracle()), (to,)


@pytest.mark.parametrize("type_flag,tr,tc,rows,cols", [
    (F.PACK_TYPE_F16F16, 8, 32, 1001, 333),    # f16 right-hand side: K0 = 8 rows x N0 = 32 columns
    (F.PACK_TYPE_F16F16, 16, 32, 200, 95),     # two 16-byte row groups per tile
    (F.PACK_TYPE_I8I8, 16, 32, 1003, 129),
    (F.PACK_TYPE_I8I8, 32, 32, 4096, 64),
    (F.PACK_TYPE_F32F32, 4, 32, 515, 70),
    (F.PACK_TYPE_BF16BF16, 24, 5, 123, 77),    # odd tile width, three row groups
    # rows that start on 4-byte boundaries: the kernel with dword loads, whole and ragged blocks
    (F.PACK_TYPE_F16F16, 8, 32, 1000, 520),
    (F.PACK_TYPE_I8I8, 16, 32, 1003, 772),
    (F.PACK_TYPE_BF16BF16, 16, 64, 300, 1028),
    (F.PACK_TYPE_I8I8, 32, 8, 200, 1024),
    # 2-byte elements, 512 columns and more, enough blocks for every compute unit: the kernel that
    # loads 16 bytes per lane and passes the chunks through LDS (4 row groups per wave, 1, two row
    # groups per tile), ragged in both directions
    (F.PACK_TYPE_F16F16, 8, 32, 4100, 4200),
    (F.PACK_TYPE_F16F16, 8, 32, 1030, 4200),
    (F.PACK_TYPE_BF16BF16, 16, 64, 4100, 4130),
])
def test_transposing_pack_with_ragged_edges(uk, cuda, type_flag, tr, tc, rows, cols):
    """Packs with transposed inner tiles (what the right-hand side B[K][N] of a
    matmul needs): matrix tiles of tr rows x tc columns, stored column by column."""
    rng = np.random.default_rng(rows + cols)
    orows, ocols = -(-rows // tr), -(-cols // tc)
    for to in (0, 1):
        case = ukref.PackCase(rng, type_flag, orows, ocols, tr, tc, transpose_inner=1,
                              transpose_outer=to, in_size=(rows, cols))
        assert np.array_equal(gpucase.run_pack(case), case.run_oracle()), (to,)
        loose = ukref.PackCase(rng, type_flag, orows, ocols, tr, tc, transpose_inner=1,
                               transpose_outer=to, in_size=(rows, cols), loose_strides=True,
                               offsets=True)
        assert np.array_equal(gpucase.run_pack(loose), loose.run_oracle()), (to, "loose")


@pytest.mark.parametrize("type_flag,tr,tc,rows,cols", [
    (F.UNPACK_TYPE_F32F32, 32, 32, 333, 1001),
    (F.UNPACK_TYPE_I32I32, 32, 8, 95, 257),      # the transposed result tiles of a narrow matmul
    (F.UNPACK_TYPE_F16F16, 16, 32, 129, 1003),
    (F.UNPACK_TYPE_BF16BF16, 24, 5, 123, 77),    # odd tile width, three row groups
    (F.UNPACK_TYPE_F32F32, 8, 32, 4096, 70),
    (F.UNPACK_TYPE_F16F16, 32, 8, 2000, 130),    # lanes whose 8 columns end at the matrix edge
    (F.UNPACK_TYPE_F32F32, 32, 4, 77, 64),       # exactly one wave of blocks across
    (F.UNPACK_TYPE_I32I32, 32, 16, 1030, 1000),  # row groups past the matrix in the last quartet
    (F.UNPACK_TYPE_BF16BF16, 32, 32, 511, 515),
    # stored columns of 128 bytes and more: a wave takes 8 row groups and 8 blocks across
    (F.UNPACK_TYPE_F32F32, 64, 32, 333, 1001),
    (F.UNPACK_TYPE_F16F16, 64, 16, 1000, 130),
    (F.UNPACK_TYPE_I32I32, 32, 32, 4100, 37),
])
def test_transposing_unpack_with_ragged_edges(uk, cuda, type_flag, tr, tc, rows, cols):
    """Unpacks of tiles stored column by column (matrix tiles of tr rows x tc
    columns): the fast kernel for whole 16-byte stored rows; the whole
    destination buffer is compared, so nothing outside the matrix is touched."""
    rng = np.random.default_rng(rows * 3 + cols)
    orows, ocols = -(-rows // tr), -(-cols // tc)
    for to in (0, 1):
        case = ukref.UnpackCase(rng, type_flag, orows, ocols, tr, tc, transpose_inner=1,
                                transpose_outer=to, out_size=(rows, cols))
        assert np.array_equal(gpucase.run_unpack(case), case.run_oracle()), (to,)
        loose = ukref.UnpackCase(rng, type_flag, orows, ocols, tr, tc, transpose_inner=1,
                                 transpose_outer=to, out_size=(rows, cols), loose_strides=True,
                                 offsets=True)
        assert np.array_equal(gpucase.run_unpack(loose), loose.run_oracle()), (to, "loose")


@pytest.mark.parametrize("type_flag,t0,t1,rows,cols", [
    (F.UNPACK_TYPE_F16F16, 32, 16, 70, 1001),     # rows of 2002 bytes: every alignment of a row start mod 16
    (F.UNPACK_TYPE_F16F16, 32, 16, 9, 512),       # exactly 1 KiB per row
    (F.UNPACK_TYPE_BF16BF16, 8, 8, 37, 3000),
    (F.UNPACK_TYPE_F32F32, 32, 32, 45, 777),
    (F.UNPACK_TYPE_I32I32, 32, 32, 130, 257),
    (F.UNPACK_TYPE_F32F32, 16, 4, 33, 1030),
    # (that kernel serves tile rows of 32 bytes; the other shapes here take the kernels around it)
    (F.UNPACK_TYPE_F32F32, 32, 8, 50, 1000),
    (F.UNPACK_TYPE_BF16BF16, 16, 16, 37, 3000),
])
def test_unpack_with_line_aligned_stores_every_row_alignment(uk, cuda, type_flag, t0, t1, rows, cols):
    """Rows of 1 KiB and more in power-of-two tiles run the unpack kernel whose
    stores are aligned cache lines (every 16 stored bytes are a byte-shifted
    pair of tile chunks): row pitches and first-element offsets that give every
    alignment of a row start, rows that end inside their last window, row
    counts that are not whole blocks of 4; the whole destination buffer is
    compared, so the bytes before and behind every row are untouched."""
    rng = np.random.default_rng(rows * 7 + cols)
    o0, o1 = -(-rows // t0), -(-cols // t1)
    for to in (0, 1):
        for extra_pitch, out_offset in ((0, 0), (0, 3), (0, 17), (0, 63), (1, 3), (5, 64), (37, 1), (64, 17)):
            case = ukref.UnpackCase(rng, type_flag, o0, o1, t0, t1, transpose_outer=to, out_size=(rows, cols))
            case.out_stride0 = cols + extra_pitch
            case.out_offset = out_offset
            info = np.iinfo(case.dtype)
            case.out_init = rng.integers(0, int(info.max) + 1, size=out_offset + rows * case.out_stride0 + 131,
                                         dtype=np.uint64).astype(case.dtype)
            assert np.array_equal(gpucase.run_unpack(case), case.run_oracle()), (to, extra_pitch, out_offset)


def test_full_size_f16_8191x5001_pack_unpack_round_trip(uk, cuda):
    """The bandwidth workload at its real size: packed bytes equal the oracle's
    (and the committed SHA-256 produced by the reference library), the padded
    row and columns hold the padding value, and unpack restores the source."""
    import torch
    R, Cc, T0, T1 = 8191, 5001, 32, 16
    O0, O1 = -(-R // T0), -(-Cc // T1)
    x = synth.uniform_pm1_f16(1, R * Cc).view(np.uint16)
    xd = torch.from_numpy(x.view(np.int16)).cuda()
    packed = torch.full((O0 * O1 * T0 * T1,), 0x5A5A, dtype=torch.int16, device="cuda")
    uk.pack(xd, packed, R, Cc, O0, O1, T0, T1, 0, F.PACK_TYPE_F16F16)
    back = torch.full((R * Cc + 64,), 0x1234, dtype=torch.int16, device="cuda")
    uk.unpack(packed, back, O0, O1, T0, T1, R, Cc, F.UNPACK_TYPE_F16F16)
    torch.cuda.synchronize()
    got = packed.cpu().numpy().view(np.uint16)
    # oracle at full size (a few hundred ms of C)
    import ctypes as C
    from iree_amd._lib import PackParams
    want = np.full(O0 * O1 * T0 * T1, 0x5A5A, np.uint16)
    p = PackParams(ukref.ptr(x).value, 0, Cc, 1, ukref.ptr(want).value, 0, O1 * T0 * T1, T0 * T1,
                   R, Cc, O0, O1, T0, T1, 0, F.PACK_TYPE_F16F16, None)
    assert ukref.oracle().oracle_pack(C.byref(p)) == 0
    assert np.array_equal(got, want)
    with open(GOLDEN) as f:
        golden = json.load(f)
    assert hashlib.sha256(got.tobytes()).hexdigest() == golden["pack_f16_8191x5001_32x16_sha256"]
    t = got.reshape(O0, O1, T0, T1)
    assert not t[-1, :, R - (O0 - 1) * T0:, :].any()      # 1 padded row
    assert not t[:, -1, :, Cc - (O1 - 1) * T1:].any()     # 7 padded columns
    b = back.cpu().numpy().view(np.uint16)
    assert np.array_equal(b[:R * Cc], x)
    assert (b[R * Cc:] == 0x1234).all()


def test_copy_and_read_probes(uk, cuda):
    """The yardstick kernels bench.py times next to pack / unpack and the
    weight-streaming kernels: modes 0 and 1 copy every byte, modes 2 and 3 read
    only and leave the destination alone; sizes that are not whole 8 KiB chunks
    are refused."""
    import torch
    n = 8192 * 37
    src = torch.from_numpy(np.random.default_rng(5).integers(0, 256, n, dtype=np.uint8)).to(cuda)
    for mode in (0, 1, 4, 5):
        for bpc in (0, 2):
            dst = torch.zeros(n, dtype=torch.uint8, device=cuda)
            uk.copy_probe(src, dst, n, mode, bpc)
            torch.cuda.synchronize()
            assert torch.equal(src, dst)
    sink = torch.full((16,), 7, dtype=torch.int32, device=cuda)
    for mode in (2, 3, 6, 7):
        uk.copy_probe(src, sink, n, mode, 0)
        uk.copy_probe(src, sink, n, mode, 4)
    torch.cuda.synchronize()
    assert bool((sink == 7).all())
    with pytest.raises(uk.UkError):
        uk.copy_probe(src, sink, 8192 * 3 + 16, 0, 0)
    with pytest.raises(uk.UkError):
        uk.copy_probe(src, sink, n, 8, 0)
