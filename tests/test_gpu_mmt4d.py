"""GPU parity of mmt4d against the oracle through the C ABI. Integer types are
bit-exact; float types are bit-exact on the reference's small-integer inputs
(every partial sum exact, tools/mmt4d_test.c:430-436) and within 1e-2 relative
or 1e-3 absolute of the f64-accumulated oracle on N(0,1) inputs."""
import ctypes as C
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
from test_oracle_mmt4d import REF_TYPES, SHAPES, TILES

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "golden.json")
RTOL, ATOL = 1e-2, 1e-3   # the stated tolerance for f16 / fp8 / int4 results


@pytest.mark.parametrize("type_flag", REF_TYPES + [F.MMT4D_TYPE_F8E4M3F8E4M3F32])
def test_reference_test_matrix_bit_exact(uk, cuda, type_flag):
    rng = np.random.default_rng(3000 + type_flag)
    tiles = TILES.get(type_flag, [(3, 5, 8), (32, 32, 16)])
    for tile in tiles:
        M0, N0, K0 = tile
        for (M, N, K), acc in itertools.product(SHAPES, (False, True)):
            if type_flag in (F.MMT4D_TYPE_F16F16F16, F.MMT4D_TYPE_BF16BF16BF16) and K * K0 > 24:
                continue
            case = ukref.Mmt4dCase(rng, type_flag, M, N, K, M0, N0, K0, accumulate=acc,
                                   loose_strides=bool(rng.integers(0, 2)),
                                   offsets=bool(rng.integers(0, 2)))
            got = gpucase.run_mmt4d(case)
            want = case.run_oracle(ukref.F16_IEEE)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), \
                (hex(type_flag), tile, (M, N, K), acc)


MFMA_TILES = [(F.MMT4D_TYPE_S8S8S32, 32, 32, 16), (F.MMT4D_TYPE_S8S8S32, 32, 32, 32),
              (F.MMT4D_TYPE_F16F16F32, 32, 32, 8), (F.MMT4D_TYPE_F16F16F32, 32, 32, 16),
              (F.MMT4D_TYPE_BF16BF16F32, 32, 32, 8), (F.MMT4D_TYPE_BF16BF16F32, 32, 32, 16),
              (F.MMT4D_TYPE_F8E4M3F8E4M3F32, 32, 32, 16),
              (F.MMT4D_TYPE_F32F32F32, 32, 32, 4), (F.MMT4D_TYPE_F32F32F32, 32, 32, 8),
              # f16 / bf16 results: on the matrix cores when intermediate roundings are skipped
              (F.MMT4D_TYPE_F16F16F16, 32, 32, 8), (F.MMT4D_TYPE_BF16BF16BF16, 32, 32, 16)]
# outer shapes chosen to hit: single tile, ragged macro tiles in M and N, K
# tails that are not whole LDS stages, both macro-tile variants, > 8 XCD slices
MFMA_SHAPES = [(1, 1, 2), (1, 1, 8), (3, 2, 6), (5, 7, 10), (9, 4, 18), (8, 8, 8),
               (17, 9, 4), (4, 33, 2), (20, 20, 12), (9, 17, 28), (2, 3, 44),
               # K tile counts that are not whole MFMA steps (a partial last step)
               (2, 3, 1), (3, 2, 7), (9, 4, 19), (4, 5, 21), (2, 2, 3), (1, 2, 23), (8, 8, 13)]


@pytest.mark.parametrize("type_flag,M0,N0,K0", MFMA_TILES)
def test_mfma_kernels_bit_exact_on_exact_inputs(uk, cuda, type_flag, M0, N0, K0):
    assert uk.mmt4d_info(M0, N0, K0, type_flag | F.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) == 1
    rng = np.random.default_rng(4000 + type_flag + K0)
    for (M, N, K), acc in itertools.product(MFMA_SHAPES, (False, True)):
        case = ukref.Mmt4dCase(rng, type_flag, M, N, K, M0, N0, K0, accumulate=acc)
        got = gpucase.run_mmt4d(case)
        want = case.run_oracle(ukref.F16_IEEE)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), \
            (hex(type_flag), (M0, N0, K0), (M, N, K), acc)
        # The same call without the generic-fallback permission must also be
        # served (it is an MFMA tile) and give the same bits.
        got2 = gpucase.run_mmt4d(case, flags=case.flags & ~F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)
        assert np.array_equal(got2.view(np.uint8), want.view(np.uint8))
    # loose strides that keep 16-byte alignment stay on the MFMA path; odd ones
    # and odd offsets fall back to the generic kernel - both must be right
    for loose, offs in [(True, False), (False, True), (True, True)]:
        case = ukref.Mmt4dCase(rng, type_flag, 5, 3, 6, M0, N0, K0, accumulate=True,
                               loose_strides=loose, offsets=offs)
        assert np.array_equal(gpucase.run_mmt4d(case), case.run_oracle(ukref.F16_IEEE))
    case = ukref.Mmt4dCase(rng, type_flag, 5, 3, 6, M0, N0, K0)
    case.lhs_stride0 += 64
    case.rhs_stride0 += 32
    case.out_stride0 += 16
    case.lhs = np.resize(case.lhs, case.lhs.size + 5 * 64)
    case.rhs = np.resize(case.rhs, case.rhs.size + 3 * 32)
    case.out_init = np.resize(case.out_init, case.out_init.size + 5 * 16)
    assert np.array_equal(gpucase.run_mmt4d(case), case.run_oracle(ukref.F16_IEEE))


@pytest.mark.parametrize("type_flag,K0", [(F.MMT4D_TYPE_F16F16F32, 8), (F.MMT4D_TYPE_S8S8S32, 16),
                                          (F.MMT4D_TYPE_F8E4M3F8E4M3F32, 16)])
@pytest.mark.parametrize("M,N", [(64, 128), (4, 2048), (128, 8), (64, 130)])
def test_mfma_macro_tile_variants_bit_exact(uk, cuda, type_flag, K0, M, N):
    """Outer shapes for which, on 256 compute units, the launcher prefers the
    256x128, 128x256 and 256x256 macro tiles (the small shapes above all take
    128x128), including ragged last tiles and a partial last K step."""
    rng = np.random.default_rng(M * N + K0)
    for K, acc in ((5, False), (12, True)):
        case = ukref.Mmt4dCase(rng, type_flag, M, N, K, 32, 32, K0, accumulate=acc)
        got = gpucase.run_mmt4d(case)
        want = case.run_oracle(ukref.F16_IEEE)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (hex(type_flag), M, N, K, acc)


@pytest.mark.parametrize("K0", [16, 32])
def test_s8s4_on_the_matrix_cores_bit_exact(uk, cuda, K0):
    """S8S4S32 (signed 4-bit right-hand side, mmt4d_tile_generic.c:81-142) at the
    gfx950 tiles: the library widens the right-hand side to int8 in scratch
    memory and runs the s8 x s8 matrix-core kernels; mmt4d_info reports an
    architecture tile and the generic fallback is NOT allowed in these calls.
    Bits of the oracle for macro-tile and narrow shapes, accumulate, a partial
    last K step, loose strides; operands the widening pass cannot take (an odd
    element offset into the packed nibbles) go through the element-wise kernel
    with the same bits."""
    tf = F.MMT4D_TYPE_S8S4S32
    rng = np.random.default_rng(9100 + K0)
    assert uk.mmt4d_info(32, 32, K0, tf) == 1
    assert uk.mmt4d_info(8, 32, K0, tf) == 1
    assert uk.mmt4d_info(16, 16, 2, tf) == 0
    for M0, M, N, K, acc in ((32, 3, 5, 7, False), (32, 16, 9, 12, True), (32, 64, 64, 5, False),
                             (8, 1, 300, 26, True), (1, 1, 40, 64, False)):
        case = ukref.Mmt4dCase(rng, tf, M, N, K, M0, 32, K0, accumulate=acc)
        got = gpucase.run_mmt4d(case, flags=case.flags & ~F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)
        assert np.array_equal(got, case.run_oracle()), (M0, M, N, K, acc)
    case = ukref.Mmt4dCase(rng, tf, 5, 6, 9, 32, 32, K0, accumulate=True, loose_strides=True, offsets=True)
    assert np.array_equal(gpucase.run_mmt4d(case), case.run_oracle())


def _full_range_operand(rng, type_flag, which, n_elems):
    """Every bit pattern of the element type, the extremes over-represented:
    sums wrap around modulo 2^32 (the oracle accumulates in uint32_t)."""
    dt = ukref.mmt4d_operand_dtypes(type_flag)[which]
    bits = (F.MMT4D_TYPE_BITS[type_flag][0], F.MMT4D_TYPE_BITS[type_flag][1], 32)[which]
    if bits == 4:
        return rng.integers(0, 256, size=(n_elems + 1) // 2, dtype=np.uint8)
    info = np.iinfo(dt)
    v = rng.integers(info.min, info.max + 1, size=n_elems, dtype=np.int64)
    edge = rng.random(n_elems) < 0.05
    v[edge] = rng.choice(np.array([info.min, info.min + 1, -129, -128, -1, 0, 127, 128, 255, 256, info.max - 1,
                                   info.max]).clip(info.min, info.max), size=int(edge.sum()))
    return v.astype(dt)


@pytest.mark.parametrize("type_flag", [F.MMT4D_TYPE_S16S16S32, F.MMT4D_TYPE_S16S8S32, F.MMT4D_TYPE_S16U4S32])
def test_s16_on_the_matrix_cores_bit_exact(uk, cuda, type_flag):
    """16-bit left-hand sides (mmt4d_tile_generic.c:11-51,108-142) at 32 x 32
    tiles of any K0: above a size threshold the library splits the 16-bit
    operands into int8 digit planes in scratch memory, runs the s8 x s8
    matrix-core kernel on them and adds the digit products with their weights,
    modulo 2^32 like the reference's accumulators. Bits of the oracle for the
    reference's value ranges and for full-range operands whose sums wrap
    around; K0 = 2 (the reference's own tile), 8, 16, an odd one that leaves a
    ragged last 16-wide K tile; accumulate; loose strides and offsets; a
    problem below the threshold (element-wise kernel, same bits)."""
    rng = np.random.default_rng(9300 + type_flag)
    even = type_flag == F.MMT4D_TYPE_S16U4S32          # two 4-bit elements per byte
    assert uk.mmt4d_info(32, 32, 8, type_flag) == 1
    assert uk.mmt4d_info(32, 32, 2, type_flag) == 1
    assert uk.mmt4d_info(16, 16, 2, type_flag) == 0
    for M, N, K, K0, acc in ((4, 4, 128, 8, False), (3, 7, 100, 8, True), (4, 5, 129, 8, True), (5, 5, 400, 2, False),
                             (4, 5, 150 if even else 300, 6 if even else 3, True), (2, 9, 70, 16, False),
                             (1, 1, 3, 8, True)):
        for gen in (ukref.random_operand, _full_range_operand):
            case = ukref.Mmt4dCase(rng, type_flag, M, N, K, 32, 32, K0, accumulate=acc, generator=gen)
            got = gpucase.run_mmt4d(case, flags=case.flags & ~F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)
            assert np.array_equal(got, case.run_oracle()), (M, N, K, K0, acc, gen.__name__)
    case = ukref.Mmt4dCase(rng, type_flag, 5, 6, 90, 32, 32, 8, accumulate=True, loose_strides=True, offsets=True,
                           generator=_full_range_operand)
    assert np.array_equal(gpucase.run_mmt4d(case), case.run_oracle())
    # narrow left-hand side tiles (one outer row of 1..31 rows). Up to 15 rows
    # against an 8- or 4-bit right-hand side the planes are the rows of one
    # int8 tile for the narrow matrix-core kernel; 16 to 31 rows, and every
    # narrow tile against a 16-bit right-hand side, run as 32-row planes whose
    # rows past M0 are zeros. An odd count of 16-wide K tiles, accumulate,
    # offsets; the matrix-core route asserted.
    assert uk.mmt4d_info(1, 32, 8, type_flag) == 1
    assert uk.mmt4d_info(16, 32, 8, type_flag) == 1 and uk.mmt4d_info(31, 32, 2, type_flag) == 1
    for M0, N, K, K0, acc in ((1, 70, 520, 8, False), (1, 448, 512, 8, True), (4, 33, 300, 8, False),
                              (2, 40, 521, 8, True), (15, 10, 128, 16, False), (7, 24, 700, 2, True),
                              (16, 64, 512, 8, False), (17, 40, 300, 8, True), (31, 12, 256, 16, False),
                              (24, 33, 129, 2, True)):
        for gen in (ukref.random_operand, _full_range_operand):
            case = ukref.Mmt4dCase(rng, type_flag, 1, N, K, M0, 32, K0, accumulate=acc, offsets=acc, generator=gen)
            got = gpucase.run_mmt4d(case, flags=case.flags & ~F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)
            # (below 2^24 multiply-accumulates, 2^23 for the one-tile form, the three
            # extra launches cost more than the element-wise kernel takes)
            one_tile = M0 <= 15 and type_flag != F.MMT4D_TYPE_S16S16S32
            planes = M0 * 32 * N * K * K0 >= (1 << 23 if one_tile else 1 << 24)
            assert uk.last_kernel_path() == ("mmt4d:mfma-s16-planes" if planes else "mmt4d:element-wise"), \
                (M0, N, K, K0, uk.last_kernel_path())
            assert np.array_equal(got, case.run_oracle()), (M0, N, K, K0, acc, gen.__name__)
    # two outer rows of a narrow tile, and a problem below the size threshold: the element-wise kernel
    for M, M0, N, K in ((2, 16, 64, 512), (1, 16, 2, 8)):
        case = ukref.Mmt4dCase(rng, type_flag, M, N, K, M0, 32, 8, generator=_full_range_operand)
        assert np.array_equal(gpucase.run_mmt4d(case), case.run_oracle())
        assert uk.last_kernel_path() == "mmt4d:element-wise"
    # random K0, outer counts, strides and offsets, every case above the size threshold
    for _ in range(10):
        K0 = int(rng.choice([2, 4, 6, 8, 10, 16, 24, 32])) if even else int(rng.choice([1, 2, 3, 4, 5, 8, 16, 17, 32]))
        M, N = int(rng.integers(1, 9)), int(rng.integers(1, 9))
        K = -(-(1 << 24) // (M * N * 1024 * K0)) + int(rng.integers(0, 5))
        case = ukref.Mmt4dCase(rng, type_flag, M, N, K, 32, 32, K0, accumulate=bool(rng.integers(0, 2)),
                               loose_strides=bool(rng.integers(0, 2)), offsets=bool(rng.integers(0, 2)),
                               generator=_full_range_operand)
        assert np.array_equal(gpucase.run_mmt4d(case), case.run_oracle()), (M, N, K, K0)


@pytest.mark.parametrize("type_flag,K0", [(F.MMT4D_TYPE_F16F16F32, 8), (F.MMT4D_TYPE_F16F16F32, 16),
                                          (F.MMT4D_TYPE_BF16BF16F32, 8), (F.MMT4D_TYPE_S8S8S32, 16),
                                          (F.MMT4D_TYPE_S8S8S32, 32), (F.MMT4D_TYPE_F32F32F32, 4),
                                          (F.MMT4D_TYPE_F16F16F16, 8), (F.MMT4D_TYPE_BF16BF16BF16, 16),
                                          (F.MMT4D_TYPE_F8E4M3F8E4M3F32, 16)])
def test_narrow_lhs_tiles_bit_exact(uk, cuda, type_flag, K0):
    """Narrow left-hand-side tiles (M0 < 32, one outer row: the decode shapes
    the tile-size query hands out for a static M below 32) run the streaming
    MFMA kernel: K step counts that fill 8, 16 and 32 register slots per wave,
    ragged splits over the 8 waves, more outer columns than compute units,
    accumulate, long K. Calls that kernel does not take (two outer rows,
    unaligned operands) must give the same bits through the element-wise
    kernel."""
    rng = np.random.default_rng(7000 + type_flag + K0)
    mfma_k = {F.MMT4D_TYPE_S8S8S32: 32, F.MMT4D_TYPE_F32F32F32: 8,
              F.MMT4D_TYPE_F8E4M3F8E4M3F32: 64}.get(type_flag, 16)
    tps = mfma_k // K0                      # K tiles per MFMA step
    for M0 in (1, 2, 4, 8, 16):
        assert uk.mmt4d_info(M0, 32, K0, type_flag | F.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) == 1
        # (2100 and more outer columns of at most 16 steps: one column per wave)
        for N, steps, acc in ((1, 1, False), (5, 8, True), (300, 13, False), (3, 70, True),
                              (7, 128, False), (2, 255, True), (2100, 8, True), (2051, 13, False),
                              (2300, 3, False)):
            case = ukref.Mmt4dCase(rng, type_flag, 1, N, steps * tps, M0, 32, K0, accumulate=acc)
            got = gpucase.run_mmt4d(case, flags=case.flags & ~F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)
            assert np.array_equal(got.view(np.uint8), case.run_oracle(ukref.F16_IEEE).view(np.uint8)), \
                (hex(type_flag), M0, K0, N, steps, acc)
    # a K beyond what one launch row keeps in registers (and a K of 64 steps or
    # more with few outer columns) is split over workgroup rows whose partial
    # sums a second kernel adds
    if True:
        for M0, N, steps, acc in ((8, 40, 600, False), (1, 9, 896, True), (16, 3, 257, False),
                                  (4, 100, 300, True), (2, 128, 64, False)):
            case = ukref.Mmt4dCase(rng, type_flag, 1, N, steps * tps, M0, 32, K0, accumulate=acc)
            got = gpucase.run_mmt4d(case, flags=case.flags & ~F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)
            assert np.array_equal(got.view(np.uint8), case.run_oracle(ukref.F16_IEEE).view(np.uint8)), \
                (hex(type_flag), M0, K0, N, steps, acc)
    for M, N, K in ((2, 3, 4 * tps), (1, 3, 2 * tps + (1 if tps > 1 else 0)), (1, 2, 260 * tps)):
        case = ukref.Mmt4dCase(rng, type_flag, M, N, K, 8, 32, K0, accumulate=True,
                               loose_strides=True, offsets=True)
        assert np.array_equal(gpucase.run_mmt4d(case), case.run_oracle(ukref.F16_IEEE)), (M, N, K)


@pytest.mark.parametrize("type_flag,K0", [(F.MMT4D_TYPE_F16F16F32, 8), (F.MMT4D_TYPE_BF16BF16F32, 8),
                                          (F.MMT4D_TYPE_S8S8S32, 16), (F.MMT4D_TYPE_F32F32F32, 4),
                                          (F.MMT4D_TYPE_F16F16F16, 8), (F.MMT4D_TYPE_BF16BF16BF16, 8),
                                          (F.MMT4D_TYPE_F8E4M3F8E4M3F32, 16)])
def test_narrow_tiles_with_a_k_that_is_not_whole_instruction_steps(uk, cuda, type_flag, K0):
    """A packed K is whole tiles of K0, not whole matrix-core steps (two tiles of
    the queried K0 per step, four for fp8): K = 1000 f16 elements are 125
    tiles. The narrow-tile kernel ends such a K with a partial step whose
    missing tiles count as zeros on both sides; nothing may be read past the
    operands' ends (the right-hand side buffer ends with its last tile). Every
    tail length, in the one-column-per-wave form, the form that splits K over
    the waves (staged and direct left-hand sides), the K split over workgroup
    rows and the narrow right-hand side form; matrix-core kernel asserted."""
    rng = np.random.default_rng(7300 + type_flag)
    mfma_k = {F.MMT4D_TYPE_S8S8S32: 32, F.MMT4D_TYPE_F32F32F32: 8,
              F.MMT4D_TYPE_F8E4M3F8E4M3F32: 64}.get(type_flag, 16)
    tps = mfma_k // K0
    no_fallback = ~F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION
    for tail in range(1, tps):
        for M0, N, steps, acc in ((1, 1, 0, False), (1, 1, 0, True), (4, 7, 0, True), (8, 5, 3, False),
                                  (1, 32, 62, True), (16, 3, 70, False), (2, 2300, 5, True),
                                  (1, 9, 896, False), (16, 40, 600, True), (4, 300, 13, False)):
            K = steps * tps + tail
            case = ukref.Mmt4dCase(rng, type_flag, 1, N, K, M0, 32, K0, accumulate=acc)
            got = gpucase.run_mmt4d(case, flags=case.flags & no_fallback)
            assert uk.last_kernel_path() == "mmt4d:mfma-narrow", (hex(type_flag), M0, N, K)
            assert np.array_equal(got.view(np.uint8), case.run_oracle(ukref.F16_IEEE).view(np.uint8)), \
                (hex(type_flag), M0, N, K, acc)
        for N0, M, steps, acc in ((1, 1, 0, False), (1, 1000 // 32 + 1, 62, True), (8, 3, 70, False), (2, 40, 300, True)):
            K = steps * tps + tail
            case = ukref.Mmt4dCase(rng, type_flag, M, 1, K, 32, N0, K0, accumulate=acc)
            got = gpucase.run_mmt4d(case, flags=case.flags & no_fallback)
            assert uk.last_kernel_path() == "mmt4d:mfma-narrow", (hex(type_flag), N0, M, K)
            assert np.array_equal(got.view(np.uint8), case.run_oracle(ukref.F16_IEEE).view(np.uint8)), \
                (hex(type_flag), N0, M, K, acc)


@pytest.mark.parametrize("type_flag,K0", [(F.MMT4D_TYPE_F16F16F32, 8), (F.MMT4D_TYPE_F16F16F32, 16),
                                          (F.MMT4D_TYPE_BF16BF16F32, 8), (F.MMT4D_TYPE_S8S8S32, 16),
                                          (F.MMT4D_TYPE_S8S8S32, 32), (F.MMT4D_TYPE_F32F32F32, 4),
                                          (F.MMT4D_TYPE_F16F16F16, 8), (F.MMT4D_TYPE_BF16BF16BF16, 16),
                                          (F.MMT4D_TYPE_F8E4M3F8E4M3F32, 16)])
def test_narrow_rhs_tiles_bit_exact(uk, cuda, type_flag, K0):
    """Narrow right-hand-side tiles (N0 < 32, M0 = 32, one outer column: what
    the tile-size query hands out for a static N below 32, and the
    matrix-vector product at N0 = 1). The library runs them as the narrow
    left-hand-side problem with the operands exchanged and stores the tiles
    transposed (the reference does the transposition in the compiler,
    EncodingUtils.cpp:23-92). Same shape list as the narrow left-hand-side
    test, generic fallback NOT allowed, bits of the oracle; loose strides of
    the result (tiles not back to back), and what the kernel does not take
    (two outer columns, unaligned operands) through the element-wise kernel."""
    rng = np.random.default_rng(7100 + type_flag + K0)
    mfma_k = {F.MMT4D_TYPE_S8S8S32: 32, F.MMT4D_TYPE_F32F32F32: 8,
              F.MMT4D_TYPE_F8E4M3F8E4M3F32: 64}.get(type_flag, 16)
    tps = mfma_k // K0
    for N0 in (1, 2, 4, 8, 16):
        assert uk.mmt4d_info(32, N0, K0, type_flag | F.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) == 1
        for M, steps, acc in ((1, 1, False), (5, 8, True), (300, 13, False), (3, 70, True),
                              (7, 128, False), (2, 255, True), (2100, 8, True), (2051, 13, False),
                              (2300, 3, False)):
            case = ukref.Mmt4dCase(rng, type_flag, M, 1, steps * tps, 32, N0, K0, accumulate=acc)
            got = gpucase.run_mmt4d(case, flags=case.flags & ~F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)
            assert np.array_equal(got.view(np.uint8), case.run_oracle(ukref.F16_IEEE).view(np.uint8)), \
                (hex(type_flag), N0, K0, M, steps, acc)
    for N0, M, steps, acc in ((8, 40, 600, False), (1, 9, 896, True), (16, 3, 257, False),
                              (4, 100, 300, True), (2, 128, 64, False)):
        case = ukref.Mmt4dCase(rng, type_flag, M, 1, steps * tps, 32, N0, K0, accumulate=acc)
        got = gpucase.run_mmt4d(case, flags=case.flags & ~F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)
        assert np.array_equal(got.view(np.uint8), case.run_oracle(ukref.F16_IEEE).view(np.uint8)), \
            (hex(type_flag), N0, K0, M, steps, acc)
    # result tiles with gaps between them (16-byte aligned operand strides keep
    # the call on the matrix-core kernel): short K, long K in one launch row,
    # and a long K with few outer rows, which cannot be split through the
    # dense scratch buffer
    for M, steps, acc in ((6, 8, True), (300, 40, False), (3, 200, True)):
        case = ukref.Mmt4dCase(rng, type_flag, M, 1, steps * tps, 32, 4, K0, accumulate=acc)
        case.out_stride0 += 24
        case.out_init = np.resize(case.out_init, case.out_init.size + M * 24)
        got = gpucase.run_mmt4d(case, flags=case.flags & ~F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)
        assert np.array_equal(got.view(np.uint8), case.run_oracle(ukref.F16_IEEE).view(np.uint8)), \
            (hex(type_flag), M, steps, acc)
    for M, N, K in ((3, 2, 4 * tps), (3, 1, 2 * tps + (1 if tps > 1 else 0)), (2, 1, 260 * tps)):
        case = ukref.Mmt4dCase(rng, type_flag, M, N, K, 32, 8, K0, accumulate=True,
                               loose_strides=True, offsets=True)
        assert np.array_equal(gpucase.run_mmt4d(case), case.run_oracle(ukref.F16_IEEE)), (M, N, K)


def test_without_fallback_permission_unserved_tiles_are_refused(uk, cuda):
    rng = np.random.default_rng(1)
    case = ukref.Mmt4dCase(rng, F.MMT4D_TYPE_S8S8S32, 2, 2, 2, 9, 6, 3)
    with pytest.raises(uk.UkError) as e:
        gpucase.run_mmt4d(case, flags=F.MMT4D_TYPE_S8S8S32)
    assert e.value.status == F.STATUS_UNIMPLEMENTED


@pytest.mark.parametrize("K0", [8, 16])
def test_f16_normal_inputs_within_tolerance(uk, cuda, K0):
    """f16 x f16 -> f32 on N(0,1)/sqrt(K) inputs, with and without accumulate,
    against the f64-accumulated oracle: |got - want| <= 1e-3 + 1e-2 |want|."""
    rng = np.random.default_rng(6)
    M, N, K = 6, 5, 512 // K0
    scale = 1.0 / np.sqrt(K * K0)

    def gen(rng, tf, which, n):
        if which == 2:
            return rng.standard_normal(n).astype(np.float32)
        return (rng.standard_normal(n) * scale).astype(np.float16).view(np.uint16)

    for acc in (False, True):
        case = ukref.Mmt4dCase(rng, F.MMT4D_TYPE_F16F16F32, M, N, K, 32, 32, K0,
                               accumulate=acc, generator=gen)
        got = case.written_region(gpucase.run_mmt4d(case))
        want = case.written_region(case.run_oracle(f64=True))
        assert np.all(np.abs(got - want) <= ATOL + RTOL * np.abs(want))
        # and in practice far tighter than the stated tolerance
        assert np.max(np.abs(got - want)) < 1e-5


def _pack_chain_oracle_i8(A, B, M, N, K):
    want = np.zeros((M, N), np.int32)
    assert ukref.oracle().oracle_matmul_rowmajor(ukref.ptr(A), ukref.ptr(B), ukref.ptr(want),
                                                 M, N, K, F.MMT4D_TYPE_S8S8S32) == 0
    return want


@pytest.mark.parametrize("M,N,K", [(1024, 1024, 1024), (123, 456, 789), (81, 19, 41), (1, 1000, 1000)])
def test_i8_matmul_through_pack_mmt4d_unpack(uk, cuda, M, N, K):
    """linalg.matmul i8 x i8 -> i32 through data tiling, bit-exact against a
    plain row-major integer matmul (shapes: the 1024^3 configuration and ragged
    shapes from the reference's e2e generator,
    tests/e2e/matmul/generate_e2e_matmul_tests.py:134-177)."""
    import torch
    A = synth.uniform_int8(1, M * K)
    B = synth.uniform_int8(2, K * N)
    c = torch.zeros(M * N, dtype=torch.int32, device="cuda")
    uk.matmul_data_tiled(torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), c,
                         M, N, K, F.MMT4D_TYPE_S8S8S32)
    torch.cuda.synchronize()
    got = c.cpu().numpy().reshape(M, N)
    want = _pack_chain_oracle_i8(A, B, M, N, K)
    assert np.array_equal(got, want)
    if (M, N, K) == (1024, 1024, 1024):
        with open(GOLDEN) as f:
            golden = json.load(f)
        assert hashlib.sha256(got.tobytes()).hexdigest() == golden["matmul_i8_1024_sha256"]


def test_i8_matmul_accumulates_into_seeded_c(uk, cuda):
    import torch
    M, N, K = 200, 100, 300
    A, B = synth.uniform_int8(1, M * K), synth.uniform_int8(2, K * N)
    c0 = (synth.splitmix64(3, M * N) >> np.uint64(44)).astype(np.int64).astype(np.int32)
    c = torch.from_numpy(c0.copy()).cuda()
    uk.matmul_data_tiled(torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), c,
                         M, N, K, F.MMT4D_TYPE_S8S8S32, accumulate=True)
    want = c0.reshape(M, N) + _pack_chain_oracle_i8(A, B, M, N, K)
    assert np.array_equal(c.cpu().numpy().reshape(M, N), want)


@pytest.mark.parametrize("M,N,K", [(1024, 1024, 1024), (123, 456, 800), (40, 1000, 992)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_i8_matmul_chain_with_the_fused_forms(uk, cuda, M, N, K, accumulate):
    """The same chain with the unpack, and then also the pack of A, folded into
    the matmul (pack of B + mmt4d_unpack, pack of B + matmul_packed_rhs): the
    exact integer product both ways."""
    import torch
    A, B = synth.uniform_int8(1, M * K), synth.uniform_int8(2, K * N)
    c0 = (synth.splitmix64(3, M * N) >> np.uint64(44)).astype(np.int64).astype(np.int32)
    want = _pack_chain_oracle_i8(A, B, M, N, K)
    if accumulate:
        want = want + c0.reshape(M, N)
    for kw in ({"fuse_unpack": True}, {"fuse_pack_lhs": True}):
        c = torch.from_numpy(c0.copy()).cuda() if accumulate else torch.zeros(M * N, dtype=torch.int32, device="cuda")
        uk.matmul_data_tiled(torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), c,
                             M, N, K, F.MMT4D_TYPE_S8S8S32, accumulate=accumulate, **kw)
        torch.cuda.synchronize()
        assert np.array_equal(c.cpu().numpy().reshape(M, N), want), kw


def _sampled_f64_rows(A, B, rows, K, N):
    return A[rows].astype(np.float64) @ B.astype(np.float64)


@pytest.mark.parametrize("accumulate", [False, True])
def test_f16_4096_cubed_through_pack_mmt4d_unpack(uk, cuda, accumulate):
    """The headline configuration at full size: f16 4096^3 with N(0,1)/sqrt(K)
    inputs (second run accumulating into a seeded f32 C). Checked three ways:
    64 sampled rows against an f64 product (the stated tolerance), the
    checksum identity sum(C) = colsum(A) . rowsum(B), and bit-equality with the
    oracle on 4 whole output tiles."""
    import torch
    M = N = K = 4096
    A = synth.normal_f16(1, M * K, 1.0 / 64).reshape(M, K)
    B = synth.normal_f16(2, K * N, 1.0 / 64).reshape(K, N)
    C0 = synth.normal_f32(3, M * N).reshape(M, N) if accumulate else np.zeros((M, N), np.float32)
    c = torch.from_numpy(C0.copy().reshape(-1)).cuda()
    ws = uk.matmul_data_tiled(torch.from_numpy(A.reshape(-1).view(np.int16)).cuda().view(torch.float16),
                              torch.from_numpy(B.reshape(-1).view(np.int16)).cuda().view(torch.float16),
                              c, M, N, K, F.MMT4D_TYPE_F16F16F32, accumulate=accumulate)
    torch.cuda.synchronize()
    got = c.cpu().numpy().reshape(M, N)
    rows = (synth.splitmix64(9, 64) % np.uint64(M)).astype(np.int64)
    want = _sampled_f64_rows(A, B, rows, K, N) + C0[rows]
    err = np.abs(got[rows] - want)
    assert np.all(err <= ATOL + RTOL * np.abs(want)), float(err.max())
    assert float(err.max()) < 5e-5
    total = got.astype(np.float64).sum()
    ident = A.astype(np.float64).sum(axis=0) @ B.astype(np.float64).sum(axis=1) + C0.astype(np.float64).sum()
    assert abs(total - ident) <= 1e-6 * np.abs(got).astype(np.float64).sum()
    # packed-layout check of whole tiles against the oracle's f32 tile function
    M0, N0, K0 = 32, 32, 8
    lhs = ws["lhs"].cpu().numpy().view(np.uint16)
    rhs = ws["rhs"].cpu().numpy().view(np.uint16)
    out = ws["out"].cpu().numpy()
    K1, N1 = K // K0, N // N0
    from iree_amd._lib import Mmt4dParams
    for (i, j) in [(0, 0), (5, 77), (127, 127), (64, 3)]:
        tile = np.zeros(M0 * N0, np.float32)
        if accumulate:
            tile[:] = C0[i * M0:(i + 1) * M0, j * N0:(j + 1) * N0].reshape(-1)
        p = Mmt4dParams(ukref.ptr(lhs).value, i * K1 * M0 * K0, K1 * M0 * K0,
                        ukref.ptr(rhs).value, j * K1 * N0 * K0, K1 * N0 * K0,
                        ukref.ptr(tile).value, 0, M0 * N0, 1, 1, K1, M0, N0, K0,
                        F.MMT4D_TYPE_F16F16F32 | (F.MMT4D_ACCUMULATE if accumulate else 0), None)
        assert ukref.oracle().oracle_mmt4d_f64(C.byref(p)) == 0
        g = out[(i * N1 + j) * M0 * N0:][:M0 * N0]
        assert np.all(np.abs(g - tile) <= ATOL + RTOL * np.abs(tile))


def test_i8_4096_cubed_mmt4d_invariants(uk, cuda):
    """i8 4096^3 (the integer metric run) on packed operands: exact checksum
    identity in integers, and 6 whole tiles bit-equal to the oracle."""
    import torch
    M1 = N1 = 128
    M0 = N0 = 32
    K0, K1 = 16, 256
    lhs = synth.uniform_int8(1, M1 * K1 * M0 * K0)
    rhs = synth.uniform_int8(2, N1 * K1 * N0 * K0)
    out = torch.empty(M1 * N1 * M0 * N0, dtype=torch.int32, device="cuda")
    uk.mmt4d(torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda(), out, M1, N1, K1, M0, N0, K0,
             F.MMT4D_TYPE_S8S8S32)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    L = lhs.reshape(M1, K1, M0, K0).astype(np.int64)
    R = rhs.reshape(N1, K1, N0, K0).astype(np.int64)
    ident = int((L.sum(axis=(0, 2)) * R.sum(axis=(0, 2))).sum())
    assert int(got.astype(np.int64).sum()) == ident
    for (i, j) in [(0, 0), (1, 126), (127, 127), (63, 64), (100, 7), (8, 8)]:
        want = np.einsum("kac,kbc->ab", L[i], R[j]).astype(np.int32).reshape(-1)
        assert np.array_equal(got[(i * N1 + j) * 1024:][:1024], want), (i, j)


def test_host_pointer_variants(uk, cuda):
    """iree_amd_uk_{pack,mmt4d,unpack}_host: the entry points the HAL plugin's
    imports call with host buffers."""
    lib = uk.load_library()
    rng = np.random.default_rng(12)
    for tf, tile in [(F.MMT4D_TYPE_S8S8S32, (32, 32, 16)), (F.MMT4D_TYPE_F16F16F32, (4, 6, 5))]:
        case = ukref.Mmt4dCase(rng, tf, 3, 4, 6, *tile, accumulate=True, loose_strides=True, offsets=True)
        out = case.out_init.copy()
        p = case.params(ukref.ptr(case.lhs).value, ukref.ptr(case.rhs).value, ukref.ptr(out).value)
        assert lib.iree_amd_uk_mmt4d_host(C.byref(p)) == 0
        assert np.array_equal(out, case.run_oracle())
    pc = ukref.PackCase(rng, F.PACK_TYPE_F16F16, 3, 5, 32, 16, pad="one_incomplete_tile",
                        loose_strides=True, offsets=True)
    out = pc.out_init.copy()
    p = pc.params(ukref.ptr(pc.inp).value, ukref.ptr(out).value)
    assert lib.iree_amd_uk_pack_host(C.byref(p)) == 0
    assert np.array_equal(out, pc.run_oracle())
    ucase = ukref.UnpackCase(rng, F.UNPACK_TYPE_I32I32, 3, 5, 32, 32, pad="one_incomplete_tile",
                             loose_strides=True, offsets=True, out_stride1=2)
    out = ucase.out_init.copy()
    p = ucase.params(ukref.ptr(ucase.inp).value, ukref.ptr(out).value)
    assert lib.iree_amd_uk_unpack_host(C.byref(p)) == 0
    assert np.array_equal(out, ucase.run_oracle())


@pytest.mark.parametrize("accumulate", [False, True])
def test_host_pointer_mmt4d_in_row_blocks(uk, cuda, accumulate):
    """A host-pointer mmt4d large enough to be pipelined over blocks of outer
    rows (uploads of the next block overlapping the download of the finished
    one): bit-equal to the device-pointer entry point on the same operands,
    with a row count that the blocks do not divide, an offset left-hand side and
    a loose left-hand-side stride; twice through one pool."""
    import torch
    lib = uk.load_library()
    from iree_amd._lib import Mmt4dParams
    M1, N1, K1, M0, N0, K0 = 77, 96, 16, 32, 32, 16
    lhs_stride = K1 * M0 * K0 + 64
    lhs = synth.uniform_int8(31, 128 + M1 * lhs_stride)
    rhs = synth.uniform_int8(32, N1 * K1 * N0 * K0)
    init = np.arange(M1 * N1 * M0 * N0, dtype=np.int32) % 1000 - 500
    flags = F.MMT4D_TYPE_S8S8S32 | (F.MMT4D_ACCUMULATE if accumulate else 0)
    want = torch.from_numpy(init.copy()).cuda()
    uk.mmt4d(torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda(), want, M1, N1, K1, M0, N0, K0, flags,
             lhs_offset=128, lhs_stride0=lhs_stride)
    torch.cuda.synchronize()
    want = want.cpu().numpy()
    pool = C.c_void_p()
    assert lib.iree_amd_uk_host_pool_create(C.byref(pool)) == 0
    try:
        for _ in range(2):
            out = init.copy()
            p = Mmt4dParams(ukref.ptr(lhs).value, 128, lhs_stride, ukref.ptr(rhs).value, 0, K1 * N0 * K0,
                            ukref.ptr(out).value, 0, N1 * M0 * N0, M1, N1, K1, M0, N0, K0, flags, None)
            assert lib.iree_amd_uk_mmt4d_host_pooled(pool, C.byref(p)) == 0, lib.iree_amd_uk_last_error()
            assert np.array_equal(out, want)
    finally:
        lib.iree_amd_uk_host_pool_destroy(pool)


@pytest.mark.gpu
def test_mfma_probe_runs_and_counts_operations(uk, cuda):
    """The register-only matrix-core loop bench.py times: it launches for every
    type with a matrix-core kernel, reports 2 operations per multiply-add of
    one 4-wave workgroup per compute unit (k = the K extent of the instruction
    the mmt4d kernel uses for the type), leaves its sink alone, and refuses
    types without such a kernel."""
    import torch
    ops = torch.zeros(64 * 1024, dtype=torch.uint8, device=cuda)
    sink = torch.zeros(256, dtype=torch.float32, device=cuda)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    for flag, k in ((F.MMT4D_TYPE_F16F16F32, 32), (F.MMT4D_TYPE_BF16BF16F32, 32), (F.MMT4D_TYPE_S8S8S32, 64),
                    (F.MMT4D_TYPE_F8E4M3F8E4M3F32, 64), (F.MMT4D_TYPE_F32F32F32, 8)):
        n = uk.mfma_probe(flag, ops, 7, sink)
        assert n == cus * 4 * 7 * 2 * 128 * 128 * k       # a 128 x 128 x k update per wave and step
    torch.cuda.synchronize()
    assert float(sink.abs().sum()) == 0.0
    with pytest.raises(uk.UkError):
        uk.mfma_probe(F.MMT4D_TYPE_S16S16S32, ops, 7, sink)
    with pytest.raises(uk.UkError):
        uk.mfma_probe(F.MMT4D_TYPE_F16F16F32, ops, -1, sink)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(1024, 1024, 1024), (123, 456, 789), (81, 19, 41), (1, 1000, 1000),
                                   (300, 257, 48)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_i8_matmul_with_fused_unpack_is_bit_exact(uk, cuda, M, N, K, accumulate):
    """mmt4d_unpack (mmt4d writing / accumulating the row-major matrix itself)
    against the plain integer matmul of the oracle and against the two-call
    sequence, on the 1024^3 configuration and ragged shapes; the row pitch of C
    is wider than a row and the bytes between rows must stay untouched."""
    import torch
    A = synth.uniform_int8(1, M * K)
    B = synth.uniform_int8(2, K * N)
    ldc = N + 5
    c0 = (synth.uniform_int8(3, M * ldc).astype(np.int32) * 1000)
    c = torch.from_numpy(c0.copy()).cuda()
    a_d, b_d = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    M1, N1, K1 = -(-M // 32), -(-N // 32), -(-K // 16)
    lhs = torch.empty(M1 * K1 * 512, dtype=torch.int8, device=cuda)
    rhs = torch.empty(N1 * K1 * 512, dtype=torch.int8, device=cuda)
    uk.pack(a_d, lhs, M, K, M1, K1, 32, 16, 0, F.PACK_TYPE_I8I8)
    uk.pack(b_d, rhs, K, N, N1, K1, 32, 16, 0,
            F.PACK_TYPE_I8I8 | F.PACK_TRANSPOSE_INNER | F.PACK_TRANSPOSE_OUTER)
    flags = F.MMT4D_TYPE_S8S8S32 | (F.MMT4D_ACCUMULATE if accumulate else 0)
    uk.mmt4d_unpack(lhs, rhs, c, M, N, M1, N1, K1, 16, flags, out_stride0=ldc)
    torch.cuda.synchronize()
    got = c.cpu().numpy().reshape(M, ldc)
    want = _pack_chain_oracle_i8(A, B, M, N, K)
    before = c0.reshape(M, ldc)
    if accumulate:
        want = want + before[:, :N]
    assert np.array_equal(got[:, :N], want)
    assert np.array_equal(got[:, N:], before[:, N:])


@pytest.mark.gpu
@pytest.mark.parametrize("type_flag,K0,dt", [(F.MMT4D_TYPE_F16F16F32, 8, np.float16), (F.MMT4D_TYPE_F32F32F32, 4, np.float32)])
def test_fused_unpack_equals_mmt4d_then_unpack_bitwise(uk, cuda, type_flag, K0, dt):
    """Same kernel arithmetic, different store addresses: the fused form must
    reproduce mmt4d + unpack bit for bit on float data too (ragged M and N, a K
    with a partial last matrix-core step)."""
    import torch
    M, N, K = 200, 333, 8 * 37 + (4 if dt is np.float32 else 0)
    M1, N1, K1 = -(-M // 32), -(-N // 32), -(-K // K0)
    rng = np.random.default_rng(11)
    lhs = torch.from_numpy(rng.standard_normal(M1 * K1 * 32 * K0).astype(dt)).cuda()
    rhs = torch.from_numpy(rng.standard_normal(N1 * K1 * 32 * K0).astype(dt)).cuda()
    tiled = torch.zeros(M1 * N1 * 1024, dtype=torch.float32, device=cuda)
    two = torch.full((M * N,), -3.0, dtype=torch.float32, device=cuda)
    one = torch.full((M * N,), -3.0, dtype=torch.float32, device=cuda)
    uk.mmt4d(lhs, rhs, tiled, M1, N1, K1, 32, 32, K0, type_flag)
    uk.unpack(tiled, two, M1, N1, 32, 32, M, N, F.UNPACK_TYPE_F32F32)
    uk.mmt4d_unpack(lhs, rhs, one, M, N, M1, N1, K1, K0, type_flag)
    torch.cuda.synchronize()
    assert np.array_equal(one.cpu().numpy().view(np.uint32), two.cpu().numpy().view(np.uint32))


@pytest.mark.gpu
def test_fused_unpack_rejects_what_it_cannot_serve(uk, cuda):
    import torch
    lhs = torch.zeros(4 * 512, dtype=torch.int8, device=cuda)
    out = torch.zeros(64 * 64, dtype=torch.int32, device=cuda)
    ok = dict(out_size0=33, out_size1=64, M=2, N=2, K=2, K0=16, flags=F.MMT4D_TYPE_S8S8S32)
    uk.mmt4d_unpack(lhs, lhs, out, **ok)
    for bad in (dict(out_size0=32), dict(out_size0=65), dict(out_size1=0), dict(flags=0x0C),
                dict(out_stride0=63)):
        with pytest.raises(uk.UkError):
            uk.mmt4d_unpack(lhs, lhs, out, **{**ok, **bad})
    # a type without a matrix-core kernel: unimplemented, not a wrong result
    with pytest.raises(uk.UkError) as e:
        uk.mmt4d_unpack(lhs, lhs, out, **{**ok, "flags": F.MMT4D_TYPE_S16S16S32, "K0": 8})
    assert e.value.status == 12


@pytest.mark.gpu
def test_fused_unpack_applies_the_output_scale(uk, cuda):
    """out_scale multiplies a float result once on the store: the same single
    f32 multiplication as scale_f32 after mmt4d + unpack, so bit-identical.
    Integer types and accumulation refuse a scale."""
    import torch
    M, N, K = 96, 160, 128
    M1, N1, K1 = M // 32, N // 32, K // 16
    src = torch.from_numpy(synth.normal_f16(5, (M + N) * K).view(np.int16)).cuda()
    q = torch.empty((M + N) * K, dtype=torch.uint8, device=cuda)
    uk.quantize_f16_to_f8e4m3(src, q, (M + N) * K, 1.0)
    lhs, rhs = q[:M * K], q[M * K:]
    flags = F.MMT4D_TYPE_F8E4M3F8E4M3F32
    tiled = torch.zeros(M1 * N1 * 1024, dtype=torch.float32, device=cuda)
    two = torch.zeros(M * N, dtype=torch.float32, device=cuda)
    one = torch.zeros(M * N, dtype=torch.float32, device=cuda)
    uk.mmt4d(lhs, rhs, tiled, M1, N1, K1, 32, 32, 16, flags)
    uk.unpack(tiled, two, M1, N1, 32, 32, M, N, F.UNPACK_TYPE_F32F32)
    uk.scale_f32(two, M * N, 0.37)
    uk.mmt4d_unpack(lhs, rhs, one, M, N, M1, N1, K1, 16, flags, out_scale=0.37)
    torch.cuda.synchronize()
    assert float(two.abs().max()) > 0
    assert np.array_equal(one.cpu().numpy().view(np.uint32), two.cpu().numpy().view(np.uint32))
    with pytest.raises(uk.UkError):
        uk.mmt4d_unpack(lhs, rhs, one, M, N, M1, N1, K1, 16, flags | F.MMT4D_ACCUMULATE, out_scale=0.37)
    oi = torch.zeros(M * N, dtype=torch.int32, device=cuda)
    with pytest.raises(uk.UkError):
        uk.mmt4d_unpack(lhs, rhs, oi, M, N, M1, N1, K1, 16, F.MMT4D_TYPE_S8S8S32, out_scale=2.0)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(1024, 1024, 1024), (123, 456, 800), (81, 19, 64), (1, 1000, 992),
                                   (300, 257, 32), (77, 130, 1088), (530, 290, 2112)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_i8_matmul_with_packed_rhs_in_one_kernel_is_bit_exact(uk, cuda, M, N, K, accumulate):
    """matmul_packed_rhs: row-major LHS read by the matmul itself, pre-packed
    RHS, row-major result. Against the plain integer matmul of the oracle; row
    pitches of A and C wider than a row (the bytes between rows of C must stay
    untouched), ragged M and N, K in whole matrix-core steps of 32 (an even
    number of them runs the 16-row instruction on 64-byte steps, an odd number
    the 32-row one on 32-byte steps)."""
    import torch
    lda, ldc = K + 16, N + 5
    A = synth.uniform_int8(1, M * K).reshape(M, K)
    B = synth.uniform_int8(2, K * N)
    a_pad = synth.uniform_int8(9, M * lda).reshape(M, lda).copy()
    a_pad[:, :K] = A
    c0 = (synth.uniform_int8(3, M * ldc).astype(np.int32) * 1000)
    c = torch.from_numpy(c0.copy()).cuda()
    N1, K1 = -(-N // 32), K // 16
    rhs = torch.empty(N1 * K1 * 512, dtype=torch.int8, device=cuda)
    uk.pack(torch.from_numpy(B).cuda(), rhs, K, N, N1, K1, 32, 16, 0,
            F.PACK_TYPE_I8I8 | F.PACK_TRANSPOSE_INNER | F.PACK_TRANSPOSE_OUTER)
    flags = F.MMT4D_TYPE_S8S8S32 | (F.MMT4D_ACCUMULATE if accumulate else 0)
    uk.matmul_packed_rhs(torch.from_numpy(a_pad).cuda(), rhs, c, M, N, K, 16, flags,
                         lhs_stride0=lda, out_stride0=ldc)
    torch.cuda.synchronize()
    got = c.cpu().numpy().reshape(M, ldc)
    want = _pack_chain_oracle_i8(A.reshape(-1), B, M, N, K)
    before = c0.reshape(M, ldc)
    if accumulate:
        want = want + before[:, :N]
    assert np.array_equal(got[:, :N], want)
    assert np.array_equal(got[:, N:], before[:, N:])


@pytest.mark.gpu
@pytest.mark.parametrize("type_flag,K0,dt,K", [(F.MMT4D_TYPE_F16F16F32, 8, np.float16, 32 * 9),
                                               (F.MMT4D_TYPE_F16F16F32, 16, np.float16, 32 * 9),
                                               (F.MMT4D_TYPE_F32F32F32, 4, np.float32, 8 * 21),
                                               (F.MMT4D_TYPE_F8E4M3F8E4M3F32, 16, np.uint8, 64 * 5)])
def test_matmul_packed_rhs_equals_pack_mmt4d_unpack_bitwise(uk, cuda, type_flag, K0, dt, K):
    """The one-kernel form against the three-call sequence on float data: same
    bytes reach the same lanes, so the results are bit-identical."""
    import torch
    M, N = 200, 333
    M1, N1, K1 = -(-M // 32), -(-N // 32), K // K0
    rng = np.random.default_rng(17)
    if dt is np.uint8:
        a = rng.integers(0, 0x78, size=M * K).astype(np.uint8)       # finite e4m3 codes
        rhs_h = rng.integers(0, 0x78, size=N1 * K1 * 32 * K0).astype(np.uint8)
        pack_type = F.PACK_TYPE_I8I8
    else:
        a = rng.standard_normal(M * K).astype(dt)
        rhs_h = rng.standard_normal(N1 * K1 * 32 * K0).astype(dt)
        pack_type = F.PACK_TYPE_F16F16 if dt is np.float16 else F.PACK_TYPE_F32F32
    a_d, rhs = torch.from_numpy(a).cuda(), torch.from_numpy(rhs_h).cuda()
    lhs = torch.empty(M1 * K1 * 32 * K0, dtype=a_d.dtype, device=cuda)
    uk.pack(a_d, lhs, M, K, M1, K1, 32, K0, 0, pack_type)
    tiled = torch.zeros(M1 * N1 * 1024, dtype=torch.float32, device=cuda)
    three = torch.full((M * N,), -3.0, dtype=torch.float32, device=cuda)
    one = torch.full((M * N,), -3.0, dtype=torch.float32, device=cuda)
    uk.mmt4d(lhs, rhs, tiled, M1, N1, K1, 32, 32, K0, type_flag)
    uk.unpack(tiled, three, M1, N1, 32, 32, M, N, F.UNPACK_TYPE_F32F32)
    uk.matmul_packed_rhs(a_d, rhs, one, M, N, K, K0, type_flag)
    torch.cuda.synchronize()
    assert float(three.abs().max()) > 0
    assert np.array_equal(one.cpu().numpy().view(np.uint32), three.cpu().numpy().view(np.uint32))


@pytest.mark.gpu
def test_matmul_packed_rhs_rejects_what_it_cannot_serve(uk, cuda):
    import torch
    a = torch.zeros(64 * 64, dtype=torch.int8, device=cuda)
    out = torch.zeros(64 * 64, dtype=torch.int32, device=cuda)
    ok = dict(M=33, N=64, K=64, K0=16, flags=F.MMT4D_TYPE_S8S8S32)
    uk.matmul_packed_rhs(a, a, out, **ok)
    for bad, status in ((dict(K=48), 12), (dict(K=40), 12), (dict(lhs_stride0=63), 3), (dict(out_stride0=63), 3),
                        (dict(flags=0x0C), 3), (dict(flags=F.MMT4D_TYPE_S16S16S32, K0=8), 12),
                        (dict(lhs_offset=1), 12), (dict(out_scale=2.0), 3)):
        with pytest.raises(uk.UkError) as e:
            uk.matmul_packed_rhs(a, a, out, **{**ok, **bad})
        assert e.value.status == status, (bad, e.value.status)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N", [(9216, 2048), (2048, 9216)])
def test_i8_shapes_that_split_into_two_launches(uk, cuda, M, N):
    """288 large tiles on 256 compute units: the launcher runs one whole round of
    256x256 tiles and a second launch for the remaining rows (or columns).
    Tiled and row-major results, and the row-major left-hand side, against an
    exact float64 product (|sum| < 2^53)."""
    import torch
    K = 2048
    A = synth.uniform_int8(1, M * K).reshape(M, K)
    B = synth.uniform_int8(2, N * K).reshape(N, K)          # B^T, row-major [N][K]
    want = (A.astype(np.float64) @ B.astype(np.float64).T).astype(np.int64)
    a_d, b_d = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    M1, N1, K1 = M // 32, N // 32, K // 16
    lhs = torch.empty(M * K, dtype=torch.int8, device=cuda)
    rhs = torch.empty(N * K, dtype=torch.int8, device=cuda)
    uk.pack(a_d, lhs, M, K, M1, K1, 32, 16, 0, F.PACK_TYPE_I8I8)
    uk.pack(b_d, rhs, N, K, N1, K1, 32, 16, 0, F.PACK_TYPE_I8I8)
    tiled = torch.empty(M * N, dtype=torch.int32, device=cuda)
    uk.mmt4d(lhs, rhs, tiled, M1, N1, K1, 32, 32, 16, F.MMT4D_TYPE_S8S8S32)
    got = tiled.cpu().numpy().reshape(M1, N1, 32, 32).transpose(0, 2, 1, 3).reshape(M, N)
    assert np.array_equal(got, want)
    for fn in (lambda c: uk.mmt4d_unpack(lhs, rhs, c, M, N, M1, N1, K1, 16, F.MMT4D_TYPE_S8S8S32),
               lambda c: uk.matmul_packed_rhs(a_d, rhs, c, M, N, K, 16, F.MMT4D_TYPE_S8S8S32)):
        c = torch.full((M * N,), -1, dtype=torch.int32, device=cuda)
        fn(c)
        torch.cuda.synchronize()
        assert np.array_equal(c.cpu().numpy().reshape(M, N), want)


# Few macro tiles and a long K: the launcher splits K over workgroup rows and
# sums the partial results in slice order.
KSPLIT_TYPES = [(F.MMT4D_TYPE_S8S8S32, 16, 32), (F.MMT4D_TYPE_F16F16F32, 8, 32),
                (F.MMT4D_TYPE_F16F16F16, 16, 32), (F.MMT4D_TYPE_BF16BF16F32, 8, 32),
                (F.MMT4D_TYPE_F8E4M3F8E4M3F32, 16, 64), (F.MMT4D_TYPE_F32F32F32, 4, 8)]


@pytest.mark.gpu
@pytest.mark.parametrize("type_flag,K0,mfma_k", KSPLIT_TYPES)
def test_k_split_shapes_bit_exact(uk, cuda, type_flag, K0, mfma_k):
    """Outer shapes of a few tiles with 70 to 200 matrix-core K-steps (plus a
    partial last one where K0 allows it), tiled result, with and without
    accumulate: the bits of the oracle (every partial sum is exact)."""
    rng = np.random.default_rng(9100 + type_flag + K0)
    tps = mfma_k // K0
    for (M, N, steps), acc in itertools.product([(8, 16, 128), (3, 5, 70), (1, 40, 200)], (False, True)):
        K = steps * tps + (1 if tps > 1 else 0)
        case = ukref.Mmt4dCase(rng, type_flag, M, N, K, 32, 32, K0, accumulate=acc)
        got = gpucase.run_mmt4d(case)
        want = case.run_oracle(ukref.F16_IEEE)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (hex(type_flag), (M, N, K), acc)


@pytest.mark.gpu
@pytest.mark.parametrize("type_flag,K0,mfma_k,dt", [(F.MMT4D_TYPE_S8S8S32, 16, 32, np.int8),
                                                    (F.MMT4D_TYPE_F16F16F32, 8, 32, np.float16),
                                                    (F.MMT4D_TYPE_F32F32F32, 4, 8, np.float32)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_k_split_row_major_forms_equal_the_three_call_chain(uk, cuda, type_flag, K0, mfma_k, dt, accumulate):
    """The fused forms on a K-split shape (200 x 333, 96 K-steps) with random
    data: mmt4d_unpack and matmul_packed_rhs give the bits of pack + mmt4d +
    unpack (all three split alike and add the slices in the same order), and
    within the stated tolerance of a float64 matmul."""
    import torch
    M, N, K = 200, 333, 96 * mfma_k
    M1, N1, K1 = -(-M // 32), -(-N // 32), K // K0
    rng = np.random.default_rng(77)
    if dt is np.int8:
        A = rng.integers(-128, 128, (M, K), dtype=np.int8)
        B = rng.integers(-128, 128, (N, K), dtype=np.int8)
        odt, ptype = torch.int32, F.PACK_TYPE_I8I8
    else:
        A = (rng.standard_normal((M, K)) / 8).astype(dt)
        B = (rng.standard_normal((N, K)) / 8).astype(dt)
        odt, ptype = torch.float32, (F.PACK_TYPE_F16F16 if dt is np.float16 else F.PACK_TYPE_F32F32)
    a_dev, b_dev = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    lhs = torch.empty(M1 * K1 * 32 * K0, dtype=a_dev.dtype, device=cuda)
    rhs = torch.empty(N1 * K1 * 32 * K0, dtype=a_dev.dtype, device=cuda)
    uk.pack(a_dev, lhs, M, K, M1, K1, 32, K0, 0, ptype)
    uk.pack(b_dev, rhs, N, K, N1, K1, 32, K0, 0, ptype)
    init = torch.from_numpy(rng.integers(-40, 40, M * N).astype(np.int32)).cuda().to(odt)
    flags = type_flag | (F.MMT4D_ACCUMULATE if accumulate else 0)
    utype = F.UNPACK_TYPE_I32I32 if odt == torch.int32 else F.UNPACK_TYPE_F32F32
    # three calls (the tiled accumulator starts from the packed initial result)
    tiled = torch.zeros(M1 * N1 * 1024, dtype=odt, device=cuda)
    uk.pack(init, tiled, M, N, M1, N1, 32, 32, 0, F.PACK_TYPE_I32I32 if odt == torch.int32 else F.PACK_TYPE_F32F32)
    uk.mmt4d(lhs, rhs, tiled, M1, N1, K1, 32, 32, K0, flags)
    three = init.clone()
    uk.unpack(tiled, three, M1, N1, 32, 32, M, N, utype)
    fused = init.clone()
    uk.mmt4d_unpack(lhs, rhs, fused, M, N, M1, N1, K1, K0, flags)
    one = init.clone()
    uk.matmul_packed_rhs(a_dev, rhs, one, M, N, K, K0, flags)
    torch.cuda.synchronize()
    t3, tf, t1 = (x.cpu().numpy().view(np.uint32) for x in (three, fused, one))
    assert np.array_equal(tf, t3)
    assert np.array_equal(t1, t3)
    want = A.astype(np.float64) @ B.astype(np.float64).T
    if accumulate:
        want = want + init.cpu().numpy().reshape(M, N).astype(np.float64)
    got = three.cpu().numpy().reshape(M, N).astype(np.float64)
    if dt is np.int8:
        assert np.array_equal(got, want)
    else:
        assert np.all(np.abs(got - want) <= ATOL + RTOL * np.abs(want))


@pytest.mark.gpu
def test_k_split_scratch_grows_and_is_kept_per_stream(uk, cuda):
    """K-split calls of growing size on two streams, interleaved: the scratch
    buffer of a stream is replaced by a larger one while earlier work may still
    be queued, and the two streams never share one. Every result equals the
    exact integer product."""
    import torch
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    rng = np.random.default_rng(5)
    jobs = []
    # 16 MiB is the smallest buffer: 4 slices of 40 x 40 tiles need 26 MiB, 4 of 64 x 48 need 50
    for idx, (M1, N1, K1) in enumerate([(2, 3, 256), (40, 40, 256), (1, 2, 512), (64, 48, 256), (40, 40, 256)]):
        A = rng.integers(-128, 128, (M1 * 32, K1 * 16), dtype=np.int8)
        B = rng.integers(-128, 128, (N1 * 32, K1 * 16), dtype=np.int8)
        a_dev, b_dev = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
        N1b, K1b = N1, K1
        rhs = torch.empty(N1 * K1 * 512, dtype=torch.int8, device=cuda)
        uk.pack(b_dev, rhs, N1 * 32, K1 * 16, N1b, K1b, 32, 16, 0, F.PACK_TYPE_I8I8)
        outs = []
        for st in streams:
            out = torch.zeros(M1 * 32 * N1 * 32, dtype=torch.int32, device=cuda)
            # (no device synchronisation between the calls: earlier work of the
            # stream is still queued when its buffer is replaced; the stream
            # only waits for the operands prepared on the current one)
            st.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(st):
                uk.matmul_packed_rhs(a_dev, rhs, out, M1 * 32, N1 * 32, K1 * 16, 16, F.MMT4D_TYPE_S8S8S32,
                                     stream=st)
            outs.append(out)
        jobs.append((A, B, outs, a_dev, rhs))
    torch.cuda.synchronize()
    for A, B, outs, _, _ in jobs:
        want = A.astype(np.int32) @ B.astype(np.int32).T
        for out in outs:
            assert np.array_equal(out.cpu().numpy().reshape(want.shape), want)
    # the cached buffers can be given back (what a plugin's unload does) and
    # come back on demand
    lib = uk.load_library()
    free0 = torch.cuda.mem_get_info()[0]
    assert lib.iree_amd_uk_release_scratch() == 0
    assert torch.cuda.mem_get_info()[0] >= free0 + (16 << 20)
    A, B, outs, a_dev, rhs = jobs[1]
    again = torch.zeros_like(outs[0])
    uk.matmul_packed_rhs(a_dev, rhs, again, A.shape[0], B.shape[0], A.shape[1], 16, F.MMT4D_TYPE_S8S8S32)
    torch.cuda.synchronize()
    assert torch.equal(again, outs[0])


@pytest.mark.gpu
def test_random_outer_shapes_i8_exact(uk, cuda):
    """Seeded random outer shapes (1 to 70 tiles each way, 2 to 1100 K tiles of
    16) through every launch decision - the four macro tiles, the split of a
    partial last round into two launches, the K split - with and without
    accumulate, against the exact integer product (computed in float64, where
    every sum below 2^53 is exact)."""
    import torch
    rng = np.random.default_rng(20240)
    for case in range(24):
        M1, N1 = (int(v) for v in rng.integers(1, 71, 2))
        K1 = int(rng.choice([2, 7, 33, 128, 129, 260, 512, 900, 1100]))
        if case % 6 == 0:
            M1, N1, K1 = int(rng.integers(60, 100)), int(rng.integers(60, 100)), int(rng.choice([64, 128, 300]))
        acc = bool(case % 2)
        lhs = rng.integers(-128, 128, (M1, K1, 32, 16), dtype=np.int8)
        rhs = rng.integers(-128, 128, (N1, K1, 32, 16), dtype=np.int8)
        init = rng.integers(-1000, 1000, (M1, N1, 32, 32)).astype(np.int32)
        out = torch.from_numpy(init.copy()).cuda()
        uk.mmt4d(torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda(), out, M1, N1, K1, 32, 32, 16,
                 F.MMT4D_TYPE_S8S8S32 | (F.MMT4D_ACCUMULATE if acc else 0))
        torch.cuda.synchronize()
        A = lhs.transpose(0, 2, 1, 3).reshape(M1 * 32, K1 * 16).astype(np.float64)
        B = rhs.transpose(0, 2, 1, 3).reshape(N1 * 32, K1 * 16).astype(np.float64)
        want = (A @ B.T).reshape(M1, 32, N1, 32).transpose(0, 2, 1, 3)
        if acc:
            want = want + init
        got = out.cpu().numpy().reshape(M1, N1, 32, 32)
        assert np.array_equal(got.astype(np.float64), want), (case, M1, N1, K1, acc)


@pytest.mark.gpu
@pytest.mark.parametrize("accumulate", [False, True])
def test_matmul_packed_rhs_wide_result_packs_the_lhs_first(uk, cuda, accumulate):
    """16384 result columns and more (and 512 rows): matmul_packed_rhs packs its
    left-hand side into the stream's scratch buffer and runs the packed-operand
    kernel. Ragged M and N, a row pitch wider than the row, exact integers."""
    import torch
    M, N, K = 530, 16400, 160
    lda, ldc = K + 16, N + 8
    rng = np.random.default_rng(31)
    a_pad = rng.integers(-128, 128, (M, lda), dtype=np.int8)
    B = rng.integers(-128, 128, (N, K), dtype=np.int8)
    N1, K1 = -(-N // 32), K // 16
    rhs = torch.empty(N1 * K1 * 512, dtype=torch.int8, device=cuda)
    uk.pack(torch.from_numpy(B).cuda(), rhs, N, K, N1, K1, 32, 16, 0, F.PACK_TYPE_I8I8)
    c0 = rng.integers(-1000, 1000, (M, ldc)).astype(np.int32)
    c = torch.from_numpy(c0.copy()).cuda()
    uk.matmul_packed_rhs(torch.from_numpy(a_pad).cuda(), rhs, c, M, N, K, 16,
                         F.MMT4D_TYPE_S8S8S32 | (F.MMT4D_ACCUMULATE if accumulate else 0),
                         lhs_stride0=lda, out_stride0=ldc)
    torch.cuda.synchronize()
    got = c.cpu().numpy()
    want = a_pad[:, :K].astype(np.int32) @ B.astype(np.int32).T
    if accumulate:
        want = want + c0[:, :N]
    assert np.array_equal(got[:, :N], want)
    assert np.array_equal(got[:, N:], c0[:, N:])


BATCH_CASES = [
    # type, tile, batch, (M, N, K), gap (lhs, rhs, out) in elements
    (F.MMT4D_TYPE_S8S8S32, (32, 32, 16), 3, (2, 3, 4), (0, 0, 0)),
    (F.MMT4D_TYPE_S8S8S32, (32, 32, 16), 5, (9, 4, 19), (64, 32, 16)),
    (F.MMT4D_TYPE_F16F16F32, (32, 32, 8), 4, (5, 7, 10), (16, 8, 4)),
    (F.MMT4D_TYPE_F16F16F32, (32, 32, 8), 7, (1, 1, 2), (0, 0, 0)),
    (F.MMT4D_TYPE_BF16BF16F32, (32, 32, 16), 2, (17, 9, 4), (0, 0, 0)),
    (F.MMT4D_TYPE_F8E4M3F8E4M3F32, (32, 32, 16), 6, (3, 2, 6), (0, 0, 0)),
    (F.MMT4D_TYPE_F32F32F32, (32, 32, 4), 3, (4, 5, 21), (0, 0, 0)),
    (F.MMT4D_TYPE_F16F16F16, (32, 32, 8), 3, (2, 3, 3), (0, 0, 0)),
    # 8 and more entries of few macro tiles: whole entries are dealt to the XCDs
    (F.MMT4D_TYPE_S8S8S32, (32, 32, 16), 16, (9, 4, 19), (0, 0, 0)),
    (F.MMT4D_TYPE_F16F16F32, (32, 32, 8), 9, (5, 7, 10), (16, 8, 4)),
    (F.MMT4D_TYPE_BF16BF16F32, (32, 32, 8), 23, (17, 20, 4), (0, 0, 0)),
    # long K and few macro tiles per entry (a single mmt4d would split K)
    (F.MMT4D_TYPE_F16F16F32, (32, 32, 8), 2, (2, 2, 512), (0, 0, 0)),
    # batch strides the matrix-core kernel cannot address (odd byte alignment):
    # entry by entry
    (F.MMT4D_TYPE_S8S8S32, (32, 32, 16), 3, (2, 3, 4), (3, 5, 1)),
    # tiles of the element-wise kernel and of the narrow left-hand-side kernel
    (F.MMT4D_TYPE_S8S8S32, (4, 6, 2), 3, (2, 3, 4), (1, 2, 3)),
    (F.MMT4D_TYPE_F16F16F32, (8, 32, 8), 3, (1, 5, 12), (0, 0, 0)),
    (F.MMT4D_TYPE_S16U4S32, (3, 5, 8), 2, (2, 3, 4), (0, 0, 0)),
    # narrow left-hand sides (one outer row): the entries are planes of one
    # launch of the streaming kernel; odd gaps run entry by entry
    (F.MMT4D_TYPE_S8S8S32, (4, 32, 32), 9, (1, 7, 8), (0, 0, 0)),
    (F.MMT4D_TYPE_F8E4M3F8E4M3F32, (16, 32, 16), 5, (1, 3, 4), (0, 0, 0)),
    (F.MMT4D_TYPE_BF16BF16BF16, (2, 32, 16), 4, (1, 9, 6), (0, 0, 0)),
    (F.MMT4D_TYPE_F16F16F32, (1, 32, 16), 40, (1, 33, 8), (8, 16, 3)),
    (F.MMT4D_TYPE_F16F16F32, (1, 32, 8), 300, (1, 2, 16), (0, 0, 0)),
    (F.MMT4D_TYPE_S8S8S32, (8, 32, 16), 70, (1, 37, 26), (16, 0, 32)),
    (F.MMT4D_TYPE_BF16BF16BF16, (2, 32, 16), 33, (1, 70, 9), (0, 0, 0)),
    (F.MMT4D_TYPE_F32F32F32, (8, 32, 8), 3, (1, 5, 3), (3, 1, 0)),
]


@pytest.mark.parametrize("type_flag,tile,batch,shape,gap", BATCH_CASES)
@pytest.mark.parametrize("acc", [False, True])
def test_batch_mmt4d_bit_exact(uk, cuda, type_flag, tile, batch, shape, gap, acc):
    """Every entry of a batch has the bits of the reference's per-entry mmt4d
    call, and nothing between the entries is written."""
    rng = np.random.default_rng(8100 + type_flag + batch + shape[2])
    case = ukref.BatchMmt4dCase(rng, type_flag, batch, *shape, *tile, accumulate=acc, gap=gap)
    got = gpucase.run_batch_mmt4d(case)
    want = case.run_oracle(ukref.F16_IEEE)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


def test_batch_mmt4d_degenerate_and_large_batch(uk, cuda):
    rng = np.random.default_rng(8200)
    # batch == 0: nothing is touched
    case = ukref.BatchMmt4dCase(rng, F.MMT4D_TYPE_S8S8S32, 0, 2, 2, 2, 32, 32, 16)
    assert np.array_equal(gpucase.run_batch_mmt4d(case), case.out_init)
    # K == 0 zero-fills every entry (accumulate: leaves them)
    for acc in (False, True):
        case = ukref.BatchMmt4dCase(rng, F.MMT4D_TYPE_S8S8S32, 3, 2, 2, 0, 32, 32, 16, accumulate=acc,
                                    gap=(0, 0, 9))
        assert np.array_equal(gpucase.run_batch_mmt4d(case), case.run_oracle())
    # more entries than one launch has planes, shared right-hand side (batch stride 0)
    M0 = N0 = 32
    K0 = 16
    batch = 65535 + 300
    lhs = rng.integers(-128, 128, size=batch * M0 * K0, dtype=np.int8)
    rhs = rng.integers(-128, 128, size=N0 * K0, dtype=np.int8)
    import torch
    from iree_amd import ukernel
    d_lhs, d_rhs = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()
    d_out = torch.full((batch, M0, N0), 7, dtype=torch.int32, device="cuda")
    ukernel.batch_mmt4d(d_lhs, d_rhs, d_out, batch, 1, 1, 1, M0, N0, K0, F.MMT4D_TYPE_S8S8S32,
                        rhs_batch_stride=0)
    want = lhs.reshape(batch, M0, K0).astype(np.int32) @ rhs.reshape(N0, K0).astype(np.int32).T
    assert np.array_equal(d_out.cpu().numpy(), want)


def test_batch_mmt4d_large_entries_match_single_calls(uk, cuda):
    """At a size the oracle does not reach: a batch equals its entries run one
    by one through iree_amd_uk_mmt4d (itself checked against the oracle)."""
    import torch
    from iree_amd import ukernel
    g = torch.Generator(device="cuda").manual_seed(5)
    batch, M, N, K, K0 = 6, 24, 20, 48, 8
    lhs = torch.randn(batch, M, K, 32, K0, device="cuda", generator=g).half()
    rhs = torch.randn(batch, N, K, 32, K0, device="cuda", generator=g).half()
    out = torch.zeros(batch, M, N, 32, 32, device="cuda")
    ukernel.batch_mmt4d(lhs, rhs, out, batch, M, N, K, 32, 32, K0, F.MMT4D_TYPE_F16F16F32)
    for b in range(batch):
        one = torch.zeros(M, N, 32, 32, device="cuda")
        ukernel.mmt4d(lhs[b], rhs[b], one, M, N, K, 32, 32, K0, F.MMT4D_TYPE_F16F16F32)
        assert torch.equal(out[b], one), b


@pytest.mark.gpu
@pytest.mark.parametrize("type_flag,K0,dt", [(F.MMT4D_TYPE_S8S8S32, 16, np.int8), (F.MMT4D_TYPE_F16F16F32, 8, np.float16),
                                             (F.MMT4D_TYPE_F32F32F32, 4, np.float32)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_batch_forms_of_the_fused_entry_points_match_single_calls(uk, cuda, type_flag, K0, dt, accumulate):
    """batch_mmt4d_unpack and batch_matmul_packed_rhs (one launch, entries as
    workgroup planes) against one call of mmt4d_unpack / matmul_packed_rhs per
    entry, which the tests above pin to the oracle: the same bits, ragged M and
    N, gaps between the entries of every operand (whole 16 bytes for the
    operands, whose entries must be aligned like those of a single call; any
    for `out`), gaps in `out` untouched; a shared right-hand side (batch
    stride 0); batch 0 and 1; an entry that is not 16-byte aligned is refused
    like the single call refuses it."""
    import torch
    rng = np.random.default_rng(31 + K0)
    out_dt = np.int32 if dt is np.int8 else np.float32
    flags = type_flag | (F.MMT4D_ACCUMULATE if accumulate else 0)
    mfma_k = {np.int8: 32, np.float16: 32, np.float32: 8}[dt]

    def values(n):
        if dt is np.int8:
            return rng.integers(-128, 128, n).astype(np.int8)
        return rng.integers(-4, 5, n).astype(dt)

    for batch, M, N, K, gap in ((5, 70, 100, 3 * mfma_k, 64), (3, 200, 333, 9 * mfma_k, 0), (9, 32, 64, 2 * mfma_k, 16),
                                (2, 40, 40, 4 * mfma_k, 48), (1, 33, 65, mfma_k, 0), (0, 33, 65, mfma_k, 0),
                                # one row per entry against whole tiles of columns: the planes of the
                                # kernel for narrow left-hand side tiles
                                (4, 1, 96, 4 * mfma_k, 16), (3, 1, 64, 2 * mfma_k, 0)):
        M1, N1, K1 = -(-M // 32), -(-N // 32), K // K0
        lhs_bs, rhs_bs = M1 * K1 * 32 * K0 + gap, N1 * K1 * 32 * K0 + gap
        a_bs, out_bs = M * K + gap, M * N + gap + 7
        nb = max(batch, 1)
        lhs_t = torch.from_numpy(values(nb * lhs_bs)).cuda()       # packed left-hand sides
        rhs_t = torch.from_numpy(values(nb * rhs_bs)).cuda()       # packed right-hand sides
        a_rm = torch.from_numpy(values(nb * a_bs)).cuda()          # row-major left-hand sides
        out0 = torch.from_numpy(rng.integers(-50, 50, nb * out_bs).astype(out_dt)).cuda()
        for shared_rhs in (False, True):
            rbs = 0 if shared_rhs else rhs_bs
            # mmt4d_unpack
            got, want = out0.clone(), out0.clone()
            uk.batch_mmt4d_unpack(lhs_t, rhs_t, got, batch, M, N, M1, N1, K1, K0, flags,
                                  lhs_batch_stride=lhs_bs, rhs_batch_stride=rbs, out_batch_stride=out_bs)
            for b in range(batch):
                uk.mmt4d_unpack(lhs_t, rhs_t, want, M, N, M1, N1, K1, K0, flags, lhs_offset=b * lhs_bs,
                                rhs_offset=b * rbs, out_offset=b * out_bs)
            torch.cuda.synchronize()
            assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (batch, M, N, K, gap, shared_rhs)
            if batch:
                assert not torch.equal(got.view(torch.int32), out0.view(torch.int32))
            # matmul_packed_rhs
            got, want = out0.clone(), out0.clone()
            uk.batch_matmul_packed_rhs(a_rm, rhs_t, got, batch, M, N, K, K0, flags,
                                       lhs_batch_stride=a_bs, rhs_batch_stride=rbs, out_batch_stride=out_bs)
            for b in range(batch):
                uk.matmul_packed_rhs(a_rm, rhs_t, want, M, N, K, K0, flags, lhs_offset=b * a_bs,
                                     rhs_offset=b * rbs, out_offset=b * out_bs)
            torch.cuda.synchronize()
            assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (batch, M, N, K, gap, shared_rhs)
    with pytest.raises(uk.UkError):
        uk.batch_mmt4d_unpack(lhs_t, rhs_t, out0, -1, 33, 65, 2, 3, K1, K0, flags)
    lhs_t = torch.from_numpy(values(2 * (2 * K1 * 32 * K0) + 3)).cuda()
    rhs_t = torch.from_numpy(values(3 * K1 * 32 * K0)).cuda()
    out = torch.zeros(2 * 33 * 65, dtype=out0.dtype, device=cuda)
    with pytest.raises(uk.UkError):
        uk.batch_mmt4d_unpack(lhs_t, rhs_t, out, 2, 33, 65, 2, 3, K1, K0, flags,
                              lhs_batch_stride=2 * K1 * 32 * K0 + 3, rhs_batch_stride=0)
