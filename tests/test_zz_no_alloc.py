"""iree_amd_uk_mmt4d_noalloc_p: the mmt4d entry point that allocates nothing
(its K-split partial sums live in a device array of the library's code
object) against iree_amd_uk_mmt4d_p, through the C ABI."""
import ctypes as C

import numpy as np
import pytest

import gpucase
import ukref
from iree_amd import flags as F

pytestmark = pytest.mark.gpu


def _run(entry, case, lhs, rhs, out_init):
    import torch
    out = out_init.clone()
    p = case.params(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(),
                    flags=case.flags & ~F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)
    st = entry(C.byref(p), C.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return st, out.cpu().numpy().view(case.out_init.dtype)


def test_noalloc_mmt4d_equals_the_allocating_entry_point(uk, cuda):
    """Two calls in a row per type, the second with a smaller input (the array
    keeps the first call's partial sums): K-split shapes, whose kernels use the
    scratch memory, and one unsplit shape. Bit-exact against
    iree_amd_uk_mmt4d_p (the same kernels and the same split, so even float
    sums agree to the bit) and against the oracle on exact inputs; no device
    memory is allocated by the calls."""
    import torch
    lib = uk.load_library()
    rng = np.random.default_rng(4242)
    for type_flag, K0, mfma_k in ((F.MMT4D_TYPE_S8S8S32, 16, 32), (F.MMT4D_TYPE_F16F16F32, 8, 32),
                                  (F.MMT4D_TYPE_F8E4M3F8E4M3F32, 16, 64)):
        tps = mfma_k // K0
        # (outer rows, outer columns, matrix-core K steps): 8 x 16 x 128 and
        # 3 x 5 x 70 split K; 20 x 20 x 12 does not; the narrow tile splits K
        # through the dense form of the same buffer
        shapes = [(8, 16, 128, 32, True), (3, 5, 70, 32, False), (20, 20, 12, 32, True),
                  (1, 40, 600, 8, False), (1, 9, 300, 8, True)]
        for i, (M, N, steps, M0, acc) in enumerate(shapes):
            case = ukref.Mmt4dCase(rng, type_flag, M, N, steps * tps, M0, 32, K0, accumulate=acc)
            lhs, rhs, out0 = gpucase._to_dev(case.lhs), gpucase._to_dev(case.rhs), gpucase._to_dev(case.out_init)
            st_a, want = _run(lib.iree_amd_uk_mmt4d_p, case, lhs, rhs, out0)
            assert st_a == 0
            if i == 0:
                # first call on the device looks up the array's address
                st, got = _run(lib.iree_amd_uk_mmt4d_noalloc_p, case, lhs, rhs, out0)
                assert st == 0, lib.iree_amd_uk_last_error()
                assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
            free_before = torch.cuda.mem_get_info()[0]
            st, got = _run(lib.iree_amd_uk_mmt4d_noalloc_p, case, lhs, rhs, out0)
            assert st == 0, lib.iree_amd_uk_last_error()
            assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the free device memory"
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (hex(type_flag), M, N, steps, M0)
            assert np.array_equal(got.view(np.uint8), case.run_oracle(ukref.F16_IEEE).view(np.uint8))


def test_noalloc_mmt4d_on_random_data_and_beyond_the_limit(uk, cuda):
    """N(0,1) f16 operands on a K-split shape: the bits of iree_amd_uk_mmt4d_p
    and within 1e-2 relative / 1e-3 absolute of the float64 oracle. A K split
    whose partial sums exceed the array is refused with RESOURCE_EXHAUSTED
    before anything runs; the next call works."""
    import torch
    lib = uk.load_library()
    rng = np.random.default_rng(77)

    def normal(rng, type_flag, which, n):
        if which == 2:
            return rng.standard_normal(n).astype(np.float32)
        return (rng.standard_normal(n) / 8).astype(np.float16).view(np.uint16)
    for (M, N, K) in ((8, 16, 512), (4, 6, 300)):
        case = ukref.Mmt4dCase(rng, F.MMT4D_TYPE_F16F16F32, M, N, K, 32, 32, 8, accumulate=True, generator=normal)
        lhs, rhs, out0 = gpucase._to_dev(case.lhs), gpucase._to_dev(case.rhs), gpucase._to_dev(case.out_init)
        st_a, want = _run(lib.iree_amd_uk_mmt4d_p, case, lhs, rhs, out0)
        st, got = _run(lib.iree_amd_uk_mmt4d_noalloc_p, case, lhs, rhs, out0)
        assert st_a == 0 and st == 0
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
        ref = case.run_oracle(f64=True)
        assert np.all(np.abs(got.astype(np.float64) - ref) <= 1e-3 + 1e-2 * np.abs(ref))
    # 56 x 76 outer tiles of i8 with K = 16384 (70 macro tiles of 256 x 256 on
    # 256 compute units, 512 K steps): the launcher splits K three ways and the
    # partial sums (3 x 17.4 MB) exceed the 32 MiB array
    M1, N1, K1 = 56, 76, 1024
    lhs = torch.from_numpy(rng.integers(-128, 128, M1 * K1 * 512, dtype=np.int8)).cuda()
    rhs = torch.from_numpy(rng.integers(-128, 128, N1 * K1 * 512, dtype=np.int8)).cuda()
    out = torch.full((M1 * N1 * 1024,), -5, dtype=torch.int32, device=cuda)
    from iree_amd._lib import Mmt4dParams
    p = Mmt4dParams(lhs.data_ptr(), 0, K1 * 512, rhs.data_ptr(), 0, K1 * 512, out.data_ptr(), 0, N1 * 1024,
                    M1, N1, K1, 32, 32, 16, F.MMT4D_TYPE_S8S8S32, None)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    st = lib.iree_amd_uk_mmt4d_noalloc_p(C.byref(p), stream)
    torch.cuda.synchronize()
    assert st == 8, st
    assert b"scratch" in lib.iree_amd_uk_last_error()
    assert bool((out == -5).all()), "a refused call wrote to its result"
    # the allocating entry point takes it; the no-allocation one still works afterwards
    assert lib.iree_amd_uk_mmt4d_p(C.byref(p), stream) == 0
    torch.cuda.synchronize()
    want_big = out.clone()
    p.M, p.N = 8, 16
    out.fill_(-5)
    assert lib.iree_amd_uk_mmt4d_noalloc_p(C.byref(p), stream) == 0
    torch.cuda.synchronize()
    got = out.view(M1 * N1, 1024)
    # outer rows of the small call are N1 tiles apart (out_stride0 unchanged)
    wb = want_big.view(M1, N1, 1024)
    gs = out.view(M1, N1, 1024)
    assert torch.equal(gs[:8, :16], wb[:8, :16])
    assert bool((gs[8:] == -5).all()) and bool((gs[:8, 16:] == -5).all())


def test_noalloc_mmt4d_with_16_bit_operands(uk, cuda):
    """The 16-bit left-hand-side types keep their int8 digit planes and the
    product of the planes in the same array when they fit (4 x 4 and 16 x 16
    outer tiles) and run the element-wise kernel when they do not (46 x 46:
    93 x 93 product tiles of 4 KiB): no allocation either way, the bits of
    iree_amd_uk_mmt4d_p and of the oracle, calls in a row with smaller ones
    after larger ones."""
    import torch
    lib = uk.load_library()
    rng = np.random.default_rng(616)
    for type_flag in (F.MMT4D_TYPE_S16S16S32, F.MMT4D_TYPE_S16S8S32):
        for M, N, K, K0, acc in ((46, 46, 8, 8, False), (16, 16, 64, 8, True), (4, 4, 128, 8, False)):
            case = ukref.Mmt4dCase(rng, type_flag, M, N, K, 32, 32, K0, accumulate=acc)
            lhs, rhs, out0 = gpucase._to_dev(case.lhs), gpucase._to_dev(case.rhs), gpucase._to_dev(case.out_init)
            st_a, want = _run(lib.iree_amd_uk_mmt4d_p, case, lhs, rhs, out0)
            assert st_a == 0
            # (the first launch of a kernel in a process makes the HIP runtime
            # load its code: measured around the second call)
            st, got = _run(lib.iree_amd_uk_mmt4d_noalloc_p, case, lhs, rhs, out0)
            assert st == 0, lib.iree_amd_uk_last_error()
            assert np.array_equal(got, want), (hex(type_flag), M, N, K)
            free_before = torch.cuda.mem_get_info()[0]
            st, got = _run(lib.iree_amd_uk_mmt4d_noalloc_p, case, lhs, rhs, out0)
            assert st == 0, lib.iree_amd_uk_last_error()
            assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the free device memory"
            assert np.array_equal(got, want), (hex(type_flag), M, N, K)
            assert np.array_equal(got, case.run_oracle()), (hex(type_flag), M, N, K)


def test_noalloc_mmt4d_with_a_4_bit_right_hand_side(uk, cuda):
    """S8S4S32 at the gfx950 tile widens its right-hand side to int8 in the
    same array when it fits (one byte per weight) and runs the element-wise
    kernel when it does not (72 x 1024 tiles of 32 x 16: 37.7 MB against the
    32 MiB array): no allocation and no error either way, the bits of
    iree_amd_uk_mmt4d_p and of the oracle, the large call first so that the
    small one finds the array used."""
    import torch
    lib = uk.load_library()
    rng = np.random.default_rng(404)
    for M, N, K, acc, path in ((1, 72, 1024, False, "mmt4d:element-wise"),
                               (4, 8, 64, True, "mmt4d:mfma-widened-s4"),
                               (2, 3, 10, False, "mmt4d:mfma-widened-s4")):
        case = ukref.Mmt4dCase(rng, F.MMT4D_TYPE_S8S4S32, M, N, K, 32, 32, 16, accumulate=acc)
        lhs, rhs, out0 = gpucase._to_dev(case.lhs), gpucase._to_dev(case.rhs), gpucase._to_dev(case.out_init)
        st_a, want = _run(lib.iree_amd_uk_mmt4d_p, case, lhs, rhs, out0)
        assert st_a == 0
        assert uk.last_kernel_path() == "mmt4d:mfma-widened-s4"
        st, got = _run(lib.iree_amd_uk_mmt4d_noalloc_p, case, lhs, rhs, out0)
        assert st == 0, lib.iree_amd_uk_last_error()
        assert np.array_equal(got, want), (M, N, K)
        free_before = torch.cuda.mem_get_info()[0]
        st, got = _run(lib.iree_amd_uk_mmt4d_noalloc_p, case, lhs, rhs, out0)
        assert st == 0, lib.iree_amd_uk_last_error()
        assert uk.last_kernel_path() == path, (M, N, K)
        assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the free device memory"
        assert np.array_equal(got, want), (M, N, K)
        assert np.array_equal(got, case.run_oracle()), (M, N, K)
