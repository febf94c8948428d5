"""Pins oracle_mmt4d: against the compiled reference library (bit-exact, the
reference's own shape/tile/flag matrix of tools/mmt4d_test.c:459-608), against
an independent numpy einsum, and through tile-shape invariance."""
import ctypes as C
import itertools

import numpy as np
import pytest

import ukref
from iree_amd import flags as F

# tools/mmt4d_test.c:459-479
SHAPES = [(0, 1, 1), (0, 5, 7), (1, 0, 1), (5, 0, 7), (1, 1, 0), (5, 7, 0),
          (1, 1, 1), (1, 1, 2), (1, 1, 10), (1, 1, 100), (2, 1, 1), (1, 2, 1),
          (2, 2, 2), (5, 7, 13)]
# tools/mmt4d_test.c:541-608: odd tiles per type, then the x86 tile shapes; the
# gfx950 tile shapes are appended.
TILES = {
    F.MMT4D_TYPE_F32F32F32: [(3, 5, 7), (16, 16, 1), (8, 8, 1), (32, 32, 4)],
    F.MMT4D_TYPE_S8S8S32: [(9, 6, 3), (16, 16, 2), (8, 8, 2), (1, 16, 2), (32, 32, 16), (32, 32, 32)],
    F.MMT4D_TYPE_F16F16F32: [(4, 6, 5), (16, 16, 1), (8, 8, 1), (2, 16, 1), (32, 32, 8), (32, 32, 16)],
    F.MMT4D_TYPE_F16F16F16: [(3, 5, 8), (16, 16, 1), (4, 8, 1)],
    F.MMT4D_TYPE_BF16BF16F32: [(11, 4, 1), (16, 16, 2), (32, 32, 8)],
    F.MMT4D_TYPE_BF16BF16BF16: [(2, 9, 3), (16, 16, 2)],
    F.MMT4D_TYPE_S16S16S32: [(4, 5, 6), (16, 16, 2), (8, 8, 2)],
    F.MMT4D_TYPE_S16U4S32: [(5, 3, 2), (1, 32, 8)],
    F.MMT4D_TYPE_S16S8S32: [(3, 8, 4)],
    F.MMT4D_TYPE_S8S4S32: [(9, 12, 2), (4, 16, 2)],
}
REF_TYPES = sorted(TILES)


def _cases(rng, type_flag, tile, shapes=SHAPES):
    M0, N0, K0 = tile
    for (M, N, K), acc in itertools.product(shapes, (False, True)):
        # keep 16-bit accumulators exactly representable (mmt4d_test.c:457-458)
        if type_flag in (F.MMT4D_TYPE_F16F16F16, F.MMT4D_TYPE_BF16BF16BF16) and K * K0 > 24:
            continue
        loose = bool(rng.integers(0, 2))
        offs = bool(rng.integers(0, 2))
        yield ukref.Mmt4dCase(rng, type_flag, M, N, K, M0, N0, K0, accumulate=acc,
                              loose_strides=loose, offsets=offs)


@pytest.mark.parametrize("type_flag", REF_TYPES)
def test_oracle_matches_reference_library(type_flag):
    if ukref.reflib() is None:
        pytest.skip("oracle/_ref not built (reference sources absent)")
    rng = np.random.default_rng(1000 + type_flag)
    feature_sets = [""] + [fs for fs in ("avx2_fma", "avx512_base", "avx512_vnni")
                           if ukref.host_supports(fs)]
    n = 0
    for tile in TILES[type_flag]:
        for case in _cases(rng, type_flag, tile):
            want_oracle = case.run_oracle(ukref.F16_IEEE)
            for fs in feature_sets:
                got = case.run_ref(fs)
                # small-integer inputs: every order of summation is exact, so the
                # flush-vs-IEEE f16 decode and the FMA-vs-mul+add paths coincide.
                assert np.array_equal(got.view(np.uint8), want_oracle.view(np.uint8)), \
                    (hex(type_flag), tile, case.dims, hex(case.flags), fs)
                n += 1
    assert n > 50


@pytest.mark.parametrize("type_flag", [F.MMT4D_TYPE_F16F16F16, F.MMT4D_TYPE_BF16BF16BF16])
@pytest.mark.parametrize("skip", [False, True])
def test_oracle_16bit_accumulators_match_reference_on_random_floats(type_flag, skip):
    """The 16-bit-output variants are order and rounding sensitive: compare the
    generic reference path on genuinely random inputs, bit for bit."""
    if ukref.reflib() is None:
        pytest.skip("oracle/_ref not built")
    rng = np.random.default_rng(77 + type_flag + int(skip))

    def gen(rng, tf, which, n):
        x = rng.standard_normal(n).astype(np.float32)
        if tf == F.MMT4D_TYPE_F16F16F16:
            return x.astype(np.float16).view(np.uint16)
        return ukref.f32_to_bf16_bits(x)

    for (M, N, K), acc in itertools.product([(1, 1, 1), (2, 3, 5), (3, 2, 17)], (False, True)):
        case = ukref.Mmt4dCase(rng, type_flag, M, N, K, 3, 5, 4, accumulate=acc,
                               skip_rounding=skip, generator=gen)
        got = case.run_ref("")  # generic tile functions
        want = case.run_oracle(ukref.F16_FLUSH)
        assert np.array_equal(got, want), (hex(type_flag), skip, (M, N, K), acc)


def test_oracle_f16_random_floats_match_reference_generic_and_avx512():
    """f16 x f16 -> f32 on N(0,1)/sqrt(K) inputs: the flush-subnormal mode must
    equal the reference's generic path bit for bit (same order, no FMA); the
    IEEE mode must agree with the AVX-512 path to a few ulp (FMA vs mul+add)."""
    if ukref.reflib() is None:
        pytest.skip("oracle/_ref not built")
    rng = np.random.default_rng(5)
    K = 24

    def gen(rng, tf, which, n):
        if which == 2:
            return rng.standard_normal(n).astype(np.float32)
        x = (rng.standard_normal(n) / np.sqrt(K * 16)).astype(np.float16)
        x[::97] = np.float16(3e-6)  # sprinkle subnormals
        return x.view(np.uint16)

    for acc in (False, True):
        case = ukref.Mmt4dCase(rng, F.MMT4D_TYPE_F16F16F32, 3, 2, K, 16, 16, 1,
                               accumulate=acc, generator=gen)
        assert np.array_equal(case.run_ref(""), case.run_oracle(ukref.F16_FLUSH))
        if ukref.host_supports("avx512_base"):
            a = case.run_ref("avx512_base")
            b = case.run_oracle(ukref.F16_IEEE)
            np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-6)
            f64 = case.run_oracle(f64=True)
            np.testing.assert_allclose(b, f64, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("type_flag", REF_TYPES + [F.MMT4D_TYPE_F8E4M3F8E4M3F32])
def test_oracle_matches_numpy_einsum(type_flag):
    rng = np.random.default_rng(2000 + type_flag)
    tiles = TILES.get(type_flag, [(3, 5, 8), (32, 32, 16)])
    for tile in tiles[:3]:
        for (M, N, K) in [(1, 1, 1), (2, 3, 4), (5, 7, 3)]:
            if type_flag in (F.MMT4D_TYPE_F16F16F16, F.MMT4D_TYPE_BF16BF16BF16) and K * tile[2] > 24:
                continue
            case = ukref.Mmt4dCase(rng, type_flag, M, N, K, *tile, loose_strides=True, offsets=True)
            got = case.written_region(case.run_oracle())
            want = case.run_numpy()
            if got.dtype == np.int32:
                assert np.array_equal(got.astype(np.int64), want)
            elif type_flag == F.MMT4D_TYPE_F16F16F16:
                assert np.array_equal(got.view(np.float16).astype(np.float64), want)
            elif type_flag == F.MMT4D_TYPE_BF16BF16BF16:
                assert np.array_equal(ukref.bf16_bits_to_f32(got).astype(np.float64), want)
            else:
                assert np.array_equal(got.astype(np.float64), want)


def test_oracle_accumulate_is_out_plus_product():
    rng = np.random.default_rng(9)
    for tf in (F.MMT4D_TYPE_S8S8S32, F.MMT4D_TYPE_F16F16F32):
        case = ukref.Mmt4dCase(rng, tf, 3, 2, 5, 4, 6, 2, accumulate=True)
        got = case.written_region(case.run_oracle()).astype(np.float64)
        base = case.written_region(case.out_init).astype(np.float64)
        assert np.array_equal(got, base + case.run_numpy())


def test_oracle_degenerate_shapes_follow_reference_early_return():
    rng = np.random.default_rng(3)
    # K == 0 without accumulate zero-fills; with accumulate leaves out untouched.
    c = ukref.Mmt4dCase(rng, F.MMT4D_TYPE_S8S8S32, 2, 3, 0, 4, 4, 2, accumulate=False)
    assert not c.written_region(c.run_oracle()).any()
    c = ukref.Mmt4dCase(rng, F.MMT4D_TYPE_S8S8S32, 2, 3, 0, 4, 4, 2, accumulate=True)
    assert np.array_equal(c.run_oracle(), c.out_init)
    for dims in [(0, 3, 2), (3, 0, 2)]:
        c = ukref.Mmt4dCase(rng, F.MMT4D_TYPE_F16F16F32, *dims, 4, 4, 2)
        assert np.array_equal(c.run_oracle(), c.out_init)


def test_rowmajor_result_is_independent_of_tile_shape():
    """pack -> mmt4d -> unpack through the oracle gives the plain matrix product
    whatever (M0, N0, K0): zero padding is neutral."""
    import ctypes as C
    from iree_amd._lib import PackParams, UnpackParams, Mmt4dParams
    rng = np.random.default_rng(11)
    M, N, K = 45, 37, 70
    A = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    B = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
    want = A.astype(np.int64) @ B.astype(np.int64)
    o = ukref.oracle()
    for (M0, N0, K0) in [(16, 16, 2), (32, 32, 16), (9, 6, 3)]:
        M1, N1, K1 = -(-M // M0), -(-N // N0), -(-K // K0)
        pa = np.zeros(M1 * K1 * M0 * K0, np.int8)
        pb = np.zeros(N1 * K1 * N0 * K0, np.int8)
        pc = np.zeros(M1 * N1 * M0 * N0, np.int32)
        c = np.zeros((M, N), np.int32)
        p = PackParams(ukref.ptr(A).value, 0, K, 1, ukref.ptr(pa).value, 0, K1 * M0 * K0, M0 * K0,
                       M, K, M1, K1, M0, K0, 0, F.PACK_TYPE_I8I8, None)
        assert o.oracle_pack(C.byref(p)) == 0
        p = PackParams(ukref.ptr(B).value, 0, N, 1, ukref.ptr(pb).value, 0, K1 * N0 * K0, N0 * K0,
                       K, N, N1, K1, N0, K0, 0,
                       F.PACK_TYPE_I8I8 | F.PACK_TRANSPOSE_INNER | F.PACK_TRANSPOSE_OUTER, None)
        assert o.oracle_pack(C.byref(p)) == 0
        mp = Mmt4dParams(ukref.ptr(pa).value, 0, K1 * M0 * K0, ukref.ptr(pb).value, 0, K1 * N0 * K0,
                         ukref.ptr(pc).value, 0, N1 * M0 * N0, M1, N1, K1, M0, N0, K0,
                         F.MMT4D_TYPE_S8S8S32, None)
        assert o.oracle_mmt4d(C.byref(mp), 0) == 0
        up = UnpackParams(ukref.ptr(pc).value, 0, N1 * M0 * N0, M0 * N0, ukref.ptr(c).value, 0, N, 1,
                          M1, N1, M0, N0, M, N, F.UNPACK_TYPE_I32I32, None)
        assert o.oracle_unpack(C.byref(up)) == 0
        assert np.array_equal(c.astype(np.int64), want), (M0, N0, K0)
        # and the oracle's own row-major matmul agrees
        c2 = np.zeros((M, N), np.int32)
        assert o.oracle_matmul_rowmajor(ukref.ptr(A), ukref.ptr(B), ukref.ptr(c2), M, N, K,
                                        F.MMT4D_TYPE_S8S8S32) == 0
        assert np.array_equal(c2, c)


def test_oracle_rejects_what_the_reference_asserts_on():
    import ctypes as C
    rng = np.random.default_rng(4)
    c = ukref.Mmt4dCase(rng, F.MMT4D_TYPE_S8S8S32, 1, 1, 1, 4, 4, 2)
    out = c.out_init.copy()
    bad = [
        c.params(ukref.ptr(c.lhs).value, ukref.ptr(c.rhs).value, ukref.ptr(out).value, flags=0x800 | 2),
        c.params(ukref.ptr(c.lhs).value, ukref.ptr(c.rhs).value, ukref.ptr(out).value, flags=0x0C),
        c.params(ukref.ptr(c.lhs).value, ukref.ptr(c.rhs).value, ukref.ptr(out).value, flags=0),
    ]
    for p in bad:
        assert ukref.oracle().oracle_mmt4d(C.byref(p), 0) == F.STATUS_INVALID_ARGUMENT
    p = c.params(ukref.ptr(c.lhs).value, ukref.ptr(c.rhs).value, ukref.ptr(out).value,
                 flags=F.MMT4D_TYPE_S8S4S32)
    p.K0 = 3  # 3 x 4 bits is not a whole number of bytes
    assert ukref.oracle().oracle_mmt4d(C.byref(p), 0) == F.STATUS_INVALID_ARGUMENT


def test_batch_oracle_is_one_mmt4d_per_entry_and_matches_numpy():
    """linalg.batch_mmt4d restated as the loop the reference lowers it to; the
    einsum over the batch pins the entry offsets (a wrong batch stride or a
    dropped entry changes the sums) and untouched gaps pin the extents."""
    rng = np.random.default_rng(77)
    for tf, tile in ((F.MMT4D_TYPE_S8S8S32, (4, 6, 2)), (F.MMT4D_TYPE_F16F16F32, (32, 32, 8)),
                     (F.MMT4D_TYPE_S8S8S32, (32, 32, 16))):
        for acc in (False, True):
            case = ukref.BatchMmt4dCase(rng, tf, 3, 2, 3, 4, *tile, accumulate=acc,
                                        gap=(5, 3, 7), offsets=True)
            out = case.run_oracle()
            got = case.written_regions(out).astype(np.float64)
            want = case.run_numpy().astype(np.float64)
            if acc:
                want = want + case.written_regions(case.out_init).astype(np.float64)
            assert np.array_equal(got, want)
            # nothing outside the batch entries is written
            mask = np.ones(out.size, bool)
            M, N, K, M0, N0, K0 = case.dims
            for b in range(case.batch):
                for i in range(M):
                    o = case.out_offset + b * case.out_batch_stride + i * case.out_stride0
                    mask[o:o + N * M0 * N0] = False
            assert np.array_equal(out[mask], case.out_init[mask])
            # and against the real reference library, entry by entry
            lib = ukref.reflib()
            if lib is not None:
                ref = case.out_init.copy()
                for b in range(case.batch):
                    p = case.entry_params(b, 0, 0, 0)
                    lib.iree_uk_mmt4d(ukref.ptr(case.lhs), p.lhs_offset, p.lhs_stride0,
                                      ukref.ptr(case.rhs), p.rhs_offset, p.rhs_stride0,
                                      ukref.ptr(ref), p.out_offset, p.out_stride0,
                                      M, N, K, M0, N0, K0, case.flags,
                                      C.cast(ukref.cpu_data(""), C.c_void_p))
                assert np.array_equal(ref, out)
