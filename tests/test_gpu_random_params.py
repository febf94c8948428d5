"""Seeded random sweeps over the parameter space of the three ukernels: every
type tuple, the gfx950 tiles (full, narrow on either side) and arbitrary small
tiles, ragged outer sizes, accumulate, loose strides and offsets, both
transposes of pack / unpack and every padding regime. Each case is compared
with the oracle bit for bit (the operands follow the reference's own test
generator, tools/util.c:122-168: small integers for the float types, so every
kernel the dispatcher may choose gives the same bits)."""
import numpy as np
import pytest

import gpucase
import ukref
from iree_amd import flags as F

pytestmark = pytest.mark.gpu

MMT4D_TYPES = [F.MMT4D_TYPE_F32F32F32, F.MMT4D_TYPE_S8S8S32, F.MMT4D_TYPE_F16F16F32, F.MMT4D_TYPE_F16F16F16,
               F.MMT4D_TYPE_BF16BF16F32, F.MMT4D_TYPE_BF16BF16BF16, F.MMT4D_TYPE_S16S16S32,
               F.MMT4D_TYPE_S16U4S32, F.MMT4D_TYPE_S16S8S32, F.MMT4D_TYPE_S8S4S32,
               F.MMT4D_TYPE_F8E4M3F8E4M3F32]
# K0 values that make a packed tile row 16 bytes (and twice that) per type
ARCH_K0 = {F.MMT4D_TYPE_F32F32F32: (4,), F.MMT4D_TYPE_S8S8S32: (16, 32), F.MMT4D_TYPE_F16F16F32: (8, 16),
           F.MMT4D_TYPE_F16F16F16: (8, 16), F.MMT4D_TYPE_BF16BF16F32: (8, 16), F.MMT4D_TYPE_BF16BF16BF16: (8, 16),
           F.MMT4D_TYPE_S16S16S32: (8,), F.MMT4D_TYPE_S16U4S32: (8,), F.MMT4D_TYPE_S16S8S32: (8,),
           F.MMT4D_TYPE_S8S4S32: (16, 32), F.MMT4D_TYPE_F8E4M3F8E4M3F32: (16,)}


@pytest.mark.parametrize("seed", range(6))
def test_random_mmt4d_calls_bit_exact(uk, cuda, seed):
    rng = np.random.default_rng(424200 + seed)
    for _ in range(150):
        tf = MMT4D_TYPES[int(rng.integers(0, len(MMT4D_TYPES)))]
        shape = int(rng.integers(0, 4))
        if shape == 0:       # the full gfx950 tile
            M0, N0, K0 = 32, 32, int(rng.choice(ARCH_K0[tf]))
        elif shape == 1:     # narrow left-hand side
            M0, N0, K0 = int(rng.choice([1, 2, 4, 8, 16])), 32, int(rng.choice(ARCH_K0[tf]))
        elif shape == 2:     # narrow right-hand side
            M0, N0, K0 = 32, int(rng.choice([1, 2, 4, 8, 16])), int(rng.choice(ARCH_K0[tf]))
        else:                # anything small (even K0 for the 4-bit operands)
            M0, N0 = int(rng.integers(1, 9)), int(rng.integers(1, 9))
            K0 = int(rng.integers(1, 5)) * (2 if tf in (F.MMT4D_TYPE_S16U4S32, F.MMT4D_TYPE_S8S4S32) else 1)
        narrow = shape in (1, 2)
        M = 1 if shape == 1 and rng.integers(0, 4) else int(rng.integers(1, 7))
        N = 1 if shape == 2 and rng.integers(0, 4) else int(rng.integers(1, 40 if narrow else 7))
        K = int(rng.integers(1, 70 if narrow else 20))
        loose = bool(rng.integers(0, 3) == 0)
        case = ukref.Mmt4dCase(rng, tf, M, N, K, M0, N0, K0, accumulate=bool(rng.integers(0, 2)),
                               loose_strides=loose, offsets=loose and bool(rng.integers(0, 2)))
        got = gpucase.run_mmt4d(case)
        want = case.run_oracle(ukref.F16_IEEE)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), \
            (seed, hex(tf), M, N, K, M0, N0, K0, case.flags, loose)


PACK_TYPES = [F.PACK_TYPE_F32F32, F.PACK_TYPE_I8I8, F.PACK_TYPE_I32I32, F.PACK_TYPE_F16F16, F.PACK_TYPE_BF16BF16]
UNPACK_TYPES = [F.UNPACK_TYPE_F32F32, F.UNPACK_TYPE_I32I32, F.UNPACK_TYPE_F16F16, F.UNPACK_TYPE_BF16BF16]
PADS = ["none", "one_incomplete_tile", "a_lot"]


def _random_tile(rng):
    if rng.integers(0, 2):
        return int(rng.choice([1, 2, 4, 8, 16, 32])), int(rng.choice([4, 8, 16, 32, 64]))
    return int(rng.integers(1, 20)), int(rng.integers(1, 20))


@pytest.mark.parametrize("seed", range(4))
def test_random_pack_and_unpack_calls_bit_exact(uk, cuda, seed):
    rng = np.random.default_rng(515100 + seed)
    for _ in range(150):
        t0, t1 = _random_tile(rng)
        o0, o1 = int(rng.integers(1, 12)), int(rng.integers(1, 40))
        loose = bool(rng.integers(0, 3) == 0)
        kw = dict(transpose_inner=int(rng.integers(0, 2)), transpose_outer=int(rng.integers(0, 2)),
                  pad=PADS[int(rng.integers(0, 3))], loose_strides=loose, offsets=loose and bool(rng.integers(0, 2)))
        pc = ukref.PackCase(rng, PACK_TYPES[int(rng.integers(0, 5))], o0, o1, t0, t1,
                            in_stride1=1 + int(rng.integers(0, 6) == 0), **kw)
        assert np.array_equal(gpucase.run_pack(pc), pc.run_oracle()), (seed, "pack", o0, o1, t0, t1, kw)
        uc = ukref.UnpackCase(rng, UNPACK_TYPES[int(rng.integers(0, 4))], o0, o1, t0, t1,
                              out_stride1=1 + int(rng.integers(0, 6) == 0), **kw)
        # (the whole destination buffer is compared: nothing outside the matrix may change)
        assert np.array_equal(gpucase.run_unpack(uc), uc.run_oracle()), (seed, "unpack", o0, o1, t0, t1, kw)


@pytest.mark.parametrize("seed", range(3))
def test_random_large_transposing_packs_bit_exact(uk, cuda, seed):
    """Transposing packs of 2-byte elements large enough for the kernel that
    loads 16 bytes per lane and passes the chunks through LDS (512 columns and
    more, a block for every compute unit), with ragged edges, any padding
    regime, both outer orders and row pitches that are or are not whole
    dwords; against the oracle."""
    rng = np.random.default_rng(626200 + seed)
    for _ in range(5):
        t0 = int(rng.choice([8, 16, 32]))
        t1 = int(rng.choice([8, 16, 32, 64]))
        rows, cols = int(rng.integers(1030, 4200)), int(rng.integers(600, 4200))
        # (enough row groups of 8 x 512-column blocks for 256 compute units)
        if (rows // 8) * (cols // 512 + 1) < 1100:
            rows = 4100
        kw = dict(transpose_inner=1, transpose_outer=int(rng.integers(0, 2)), in_size=(rows, cols),
                  pad=PADS[int(rng.integers(0, 3))], loose_strides=bool(rng.integers(0, 4) == 0))
        pc = ukref.PackCase(rng, F.PACK_TYPE_F16F16 if rng.integers(0, 2) else F.PACK_TYPE_BF16BF16,
                            -(-rows // t0), -(-cols // t1), t0, t1, **kw)
        assert np.array_equal(gpucase.run_pack(pc), pc.run_oracle()), (seed, rows, cols, t0, t1, kw)


@pytest.mark.parametrize("seed", range(3))
def test_random_int4_dequant_matmul_calls_within_tolerance(uk, cuda, seed):
    """The grouped int4 dequantising matmul over random row counts (both sides of
    every kernel boundary: 8, 16, 32 rows), column counts, K (the matrix-core
    kernels' 2048 / 4096, longer K in whole 2048s, and K only the element-wise
    kernel takes), group sizes, zero-point forms and weight layouts, in the
    plain and the reassociated form: the tolerances of test_gpu_dequant.py."""
    from test_gpu_dequant import run_case, run_reassoc_case
    rng = np.random.default_rng(616000 + seed)
    for _ in range(40):
        K = int(rng.choice([256, 384, 1024, 2048, 2048, 4096, 4096, 6144]))
        gs_options = [g for g in (32, 64, 128, 256, 512, K) if K % g == 0]
        gs = int(rng.choice(gs_options))
        tiled = bool(rng.integers(0, 2)) and K % 128 == 0
        N = 32 * int(rng.integers(1, 7)) if tiled else int(rng.integers(1, 200))
        M = int(rng.choice([1, 2, 3, 7, 8, 9, 15, 16, 17, 31, 32, 33, 40]))
        zp_u4 = bool(rng.integers(0, 2))
        run_case(uk, M, N, K, gs, zp_u4, tiled, seed=int(rng.integers(0, 1 << 20)))
        if rng.integers(0, 2):
            run_reassoc_case(uk, min(M, 17), N, K, gs, zp_u4, tiled, seed=int(rng.integers(0, 1 << 20)))


# (type, K0 values, elements of K per matrix-core step, integers that the type holds exactly)
FUSED_TYPES = [(F.MMT4D_TYPE_F16F16F32, (8, 16), 32, 8), (F.MMT4D_TYPE_BF16BF16F32, (8, 16), 32, 8),
               (F.MMT4D_TYPE_S8S8S32, (16, 32), 32, 128), (F.MMT4D_TYPE_F8E4M3F8E4M3F32, (16,), 64, 8),
               (F.MMT4D_TYPE_F32F32F32, (4, 8), 8, 8),
               # results rounded once to the operand type (intermediate roundings skipped)
               (F.MMT4D_TYPE_F16F16F16, (8, 16), 32, 8), (F.MMT4D_TYPE_BF16BF16BF16, (8, 16), 32, 8)]


def _encode(torch, tf, ints):
    """Integer-valued matrix -> device tensor of the type's elements."""
    t = torch.from_numpy(ints.astype(np.float32)).cuda()
    if tf == F.MMT4D_TYPE_S8S8S32:
        return torch.from_numpy(ints.astype(np.int8)).cuda()
    if tf in (F.MMT4D_TYPE_F16F16F32, F.MMT4D_TYPE_F16F16F16):
        return t.half()
    if tf in (F.MMT4D_TYPE_BF16BF16F32, F.MMT4D_TYPE_BF16BF16BF16):
        return t.bfloat16()
    if tf == F.MMT4D_TYPE_F8E4M3F8E4M3F32:
        return t.to(torch.float8_e4m3fn).view(torch.uint8)
    return t


@pytest.mark.parametrize("seed", range(4))
def test_random_fused_matmul_calls_exact(uk, cuda, seed):
    """mmt4d_unpack and matmul_packed_rhs (the matmul that writes the row-major
    result itself, and the one that also reads its left-hand side row-major)
    over random types, shapes, K0, row pitches and accumulate, on small
    integers: every sum is exact in the accumulator type, so any tile, K-step
    size or K split the launcher picks must give the integer product."""
    import torch
    rng = np.random.default_rng(515100 + seed)
    pack_type = {1: F.PACK_TYPE_I8I8, 2: F.PACK_TYPE_F16F16, 4: F.PACK_TYPE_F32F32}
    for _ in range(40):
        tf, k0s, mfma_k, lim = FUSED_TYPES[int(rng.integers(0, len(FUSED_TYPES)))]
        K0 = int(rng.choice(k0s))
        M = int(rng.integers(1, 700)) if rng.integers(0, 4) else int(rng.integers(1, 40))
        N = int(rng.integers(1, 700)) if rng.integers(0, 4) else int(rng.integers(1, 40))
        if rng.integers(0, 6) == 0:
            # one row against whole tiles of columns: the matrix-vector form, which
            # matmul_packed_rhs hands to the kernel for narrow left-hand side tiles
            M, N = 1, 32 * int(rng.integers(1, 60))
        steps = int(rng.integers(1, 12)) if rng.integers(0, 5) else int(rng.integers(64, 160))
        if rng.integers(0, 5) == 0:
            # a few rows against more than 128 tiles of columns: matmul_packed_rhs runs the
            # kernel for narrow left-hand side tiles on the row-major matrix itself
            # (any K that one launch holds: up to 128 steps of 64 bytes per row)
            M, N = int(rng.integers(2, 33)), int(rng.integers(4100, 5200))
            steps = int(rng.integers(1, 129))
        K = steps * mfma_k
        acc = bool(rng.integers(0, 2))
        A = rng.integers(-lim, lim, (M, K))
        B = rng.integers(-lim, lim, (N, K))
        narrow_out = tf in (F.MMT4D_TYPE_F16F16F16, F.MMT4D_TYPE_BF16BF16BF16)
        C0 = rng.integers(-128, 128, (M, N)) if narrow_out else rng.integers(-1000, 1000, (M, N))
        want = A @ B.T + (C0 if acc else 0)
        a_dev, b_dev = _encode(torch, tf, A), _encode(torch, tf, B)
        es = a_dev.element_size()
        # row pitches: the left-hand side's a multiple of 16 bytes, the result's anything
        lda = K + int(rng.integers(0, 3)) * (16 // es)
        ldc = N + int(rng.integers(0, 7))
        a_pad = torch.zeros(M, lda, dtype=a_dev.dtype, device=cuda)
        a_pad[:, :K] = a_dev
        M1, N1, K1 = -(-M // 32), -(-N // 32), K // K0
        rhs = torch.empty(N1 * K1 * 32 * K0, dtype=b_dev.dtype, device=cuda)
        lhs = torch.empty(M1 * K1 * 32 * K0, dtype=a_dev.dtype, device=cuda)
        uk.pack(b_dev, rhs, N, K, N1, K1, 32, K0, 0, pack_type[es])
        uk.pack(a_dev, lhs, M, K, M1, K1, 32, K0, 0, pack_type[es])
        odt = {F.MMT4D_TYPE_S8S8S32: torch.int32, F.MMT4D_TYPE_F16F16F16: torch.float16,
               F.MMT4D_TYPE_BF16BF16BF16: torch.bfloat16}.get(tf, torch.float32)
        flags = tf | (F.MMT4D_ACCUMULATE if acc else 0) | (F.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS if narrow_out else 0)
        if narrow_out:
            # the exact sum (it fits f32), rounded once to the result type
            want = torch.from_numpy(want.astype(np.float32)).to(odt).double().numpy()
        for form in ("matmul_packed_rhs", "mmt4d_unpack"):
            c = torch.full((M, ldc), 77, dtype=odt, device=cuda)
            c[:, :N] = torch.from_numpy(C0).cuda().to(odt)
            if form == "matmul_packed_rhs":
                uk.matmul_packed_rhs(a_pad, rhs, c, M, N, K, K0, flags, lhs_stride0=lda, out_stride0=ldc)
            else:
                uk.mmt4d_unpack(lhs, rhs, c, M, N, M1, N1, K1, K0, flags, out_stride0=ldc)
            torch.cuda.synchronize()
            got = c.double().cpu().numpy()
            case = (seed, form, hex(tf), M, N, K, K0, acc, lda, ldc)
            assert np.array_equal(got[:, :N], want.astype(np.float64)), case
            assert (got[:, N:] == 77).all(), case
