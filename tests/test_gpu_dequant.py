"""GPU parity of the grouped int4 dequantising matmul against the f64 oracle:
|got - want| <= 1e-3 + 1e-2 |want| (the stated tolerance for int4 results), on
decode shapes (MFMA kernel) and on shapes only the generic kernel serves."""
import numpy as np
import pytest

import ukref
from iree_amd import flags as F
from iree_amd import synth

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 1e-3


def tile_weights(w_bytes, N, K):
    """Row-major [N][K/2] nibble bytes -> the pre-tiled layout of the header:
    [N/32][K/128][32 columns][4 chunks j][4 dwords q], dword (j, q) = row-major
    dword 4q + j of the column's 64-byte span."""
    d = w_bytes.view(np.uint32).reshape(N // 32, 32, K // 128, 4, 4)   # [nt][c][s][q][j]
    return np.ascontiguousarray(d.transpose(0, 2, 1, 4, 3)).reshape(-1).view(np.uint8)


def run_case(uk, M, N, K, gs, zp_u4, tiled, seed=0, frac_zp=False, want_path=None, repeats=0):
    import torch
    G = K // gs
    x = synth.normal_f16(seed + 1, M * K)
    w = synth.uniform_u4_packed(seed + 2, N * K)
    s = synth.uniform_f16(seed + 4, N * G, 0.005, 0.02)
    if zp_u4:
        zp = synth.uniform_u4_packed(seed + 5, N * G)
        if zp.size * 2 < N * G + 1:
            zp = np.concatenate([zp, np.zeros(1, np.uint8)])
    else:
        zi = (synth.splitmix64(seed + 5, N * G) >> np.uint64(60)).astype(np.float32)
        if frac_zp:
            zi = zi + 0.5
        zp = zi.astype(np.float16)
    want = np.zeros(M * N, np.uint16)
    assert ukref.oracle().oracle_dequant_matmul_i4(
        ukref.ptr(x.view(np.uint16)), ukref.ptr(w), ukref.ptr(s.view(np.uint16)),
        ukref.ptr(zp.view(np.uint8) if zp_u4 else zp.view(np.uint16)), ukref.ptr(want),
        M, N, K, gs, int(zp_u4)) == 0
    wd = tile_weights(w, N, K) if tiled else w
    flags = (F.DEQUANT_MATMUL_ZP_U4 if zp_u4 else 0) | (F.DEQUANT_MATMUL_W_TILED if tiled else 0)
    out = torch.full((M * N,), 0x7E00, dtype=torch.int16, device="cuda")
    xd, wdev = torch.from_numpy(x.view(np.int16)).cuda(), torch.from_numpy(wd).cuda()
    sd, zd = torch.from_numpy(s.view(np.int16)).cuda(), torch.from_numpy(zp.view(np.uint8)).cuda()
    uk.dequant_matmul_i4(xd, wdev, sd, zd, out, M, N, K, gs, flags)
    torch.cuda.synchronize()
    bits = out.cpu().numpy().copy()
    if want_path is not None:
        assert uk.last_kernel_path() == want_path, (uk.last_kernel_path(), M, N, K, gs, tiled)
    for _ in range(repeats):
        # (the same call again, the result buffer refilled: the sums are added in
        # a fixed order, so every run gives the same bits)
        out.fill_(0x7E00)
        uk.dequant_matmul_i4(xd, wdev, sd, zd, out, M, N, K, gs, flags)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), bits), "two runs of the same call differ"
    got = bits.view(np.float16).astype(np.float64)
    wantf = want.view(np.float16).astype(np.float64)
    err = np.abs(got - wantf)
    assert np.all(err <= ATOL + RTOL * np.abs(wantf)), (M, N, K, gs, zp_u4, tiled, float(err.max()))
    return float(err.max()), float(np.abs(wantf).max())


@pytest.mark.parametrize("M", [1, 8, 32])
@pytest.mark.parametrize("tiled", [False, True])
def test_decode_shape_llama_ffn(uk, cuda, M, tiled):
    """The decode configuration: K = 4096, N = 14336, groups of 128, f16 scales,
    packed uint4 zero points."""
    err, mag = run_case(uk, M, 14336, 4096, 128, True, tiled, want_path="dequant_i4:mfma", repeats=3)
    # f32 accumulation of exact products: far inside the stated tolerance, at
    # most one f16 unit in the last place from the correctly rounded result
    assert err <= float(np.spacing(np.float16(max(1.0, mag))))


@pytest.mark.parametrize("K,gs", [(1024, 32), (1024, 64), (2048, 32), (2048, 64), (2048, 128), (2048, 256),
                                  (2048, 2048), (4096, 32), (4096, 64), (4096, 256), (4096, 512),
                                  (4096, 1024), (4096, 4096)])
@pytest.mark.parametrize("zp_u4", [False, True])
def test_mfma_kernel_group_sizes_and_zero_point_forms(uk, cuda, K, gs, zp_u4):
    # (rows: up to 16 stage the activations through LDS in one go, 8 or 16 rows
    # per wave; 17..32 in phases of 8 rows, three phases up to 24 rows and four
    # beyond; 40 = a pass of 32 and one of 8 from row 32 on)
    for M, N, tiled in [(3, 96, True), (32, 64, False), (40, 100, False), (17, 160, True), (12, 64, True),
                        (8, 32, False), (9, 64, False), (24, 96, False), (25, 64, True), (31, 64, False)]:
        run_case(uk, M, N, K, gs, zp_u4, tiled, seed=K + gs)


@pytest.mark.parametrize("K", [11008, 5120, 256, 768, 2304, 6400, 13824])
@pytest.mark.parametrize("gs,zp_u4", [(128, True), (128, False), (256, True), (64, True), (32, False)])
def test_mfma_kernel_serves_every_k_in_whole_256s(uk, cuda, K, gs, zp_u4):
    """K is not limited to whole 2048s (the pattern puts no such limit on it:
    11008 and 5120 are common decoder widths): the matrix-core kernel runs
    workgroup slices of 2048 whose last one is shorter, the trailing waves of
    that slice multiplying zeros. One row, few rows, 16, 17 and 32 rows (all
    staging forms), both weight layouts, against the f64 oracle, the kernel
    family asserted and two runs bit-identical."""
    if K % gs:
        pytest.skip("K is whole groups")
    for M, N, tiled in [(1, 14336 if K in (11008, 5120) else 96, True), (8, 64, True), (16, 96, False),
                        (17, 64, True), (32, 160, False), (3, 32, False)]:
        if gs < 128 and not tiled:
            continue
        run_case(uk, M, N, K, gs, zp_u4, tiled, seed=K + gs + M, want_path="dequant_i4:mfma", repeats=1)


@pytest.mark.parametrize("K,gs", [(6144, 128), (8192, 64), (14336, 128), (14336, 256), (2048, 64)])
@pytest.mark.parametrize("zp_u4", [False, True])
def test_long_k_small_batches(uk, cuda, K, gs, zp_u4):
    """K beyond 4096 (in whole 2048s): rows go through LDS in passes of as many
    as fit (one pass, several, and more than the 8 passes allowed, which the
    element-wise kernel serves), ragged N for row-major weights: all against
    the f64 oracle."""
    for M, N, tiled in [(1, 64, True), (1, 50, False), (4, 96, True), (5, 47, False), (16, 32, True),
                        (33, 64, True), (41, 40, False)]:
        if gs < 128 and not tiled:
            continue
        run_case(uk, M, N, K, gs, zp_u4, tiled, seed=K + gs + M)


@pytest.mark.parametrize("M,N,K,tiled", [(2, 4800, 6144, True), (1, 4112, 8192, False), (3, 1024, 14336, True),
                                        (1, 8192, 6144, True)])
def test_long_k_medium_n_splits_k_over_waves(uk, cuda, M, N, K, tiled):
    """Column counts between one and eight units per compute unit: the chunks of
    a unit are shared by 2, 4 or 8 waves (one part may be shorter or empty, some
    unit lanes of a workgroup have no unit) and summed through LDS."""
    run_case(uk, M, N, K, 128, True, tiled, seed=N + K)


@pytest.mark.parametrize("M,N,K,tiled", [(8, 4096, 14336, True), (16, 1024, 14336, False), (12, 4096, 8192, True),
                                        (32, 2048, 14336, True), (6, 36, 10240, False)])
def test_long_k_batches_split_k_over_workgroup_rows(uk, cuda, M, N, K, tiled):
    """More rows than fit LDS over all of K: K is split over workgroup rows whose
    f32 partial sums a second kernel adds (2 to 4 rows of K, one or two passes
    of 16 rows, few and many units per row)."""
    run_case(uk, M, N, K, 128, True, tiled, seed=M + N + K)


def test_fractional_f16_zero_points(uk, cuda):
    run_case(uk, 5, 64, 2048, 128, False, False, seed=3, frac_zp=True)
    run_case(uk, 5, 64, 2048, 128, False, True, seed=4, frac_zp=True)


@pytest.mark.parametrize("M,N,K,gs", [(2, 10, 96, 32), (5, 33, 192, 96), (1, 7, 640, 64), (3, 64, 1536, 128)])
def test_generic_kernel_shapes(uk, cuda, M, N, K, gs):
    for zp_u4 in (False, True):
        run_case(uk, M, N, K, gs, zp_u4, False, seed=M * N)
    if N % 32 == 0 and K % 128 == 0:
        run_case(uk, M, N, K, gs, True, True, seed=M * N + 1)


def test_pack_i4_weights_matches_the_documented_layout(uk, cuda):
    import torch
    for N, K in [(32, 128), (96, 512), (14336, 4096)]:
        w = synth.uniform_u4_packed(N + K, N * K)
        dst = torch.zeros(N * K // 2, dtype=torch.uint8, device="cuda")
        uk.pack_i4_weights(torch.from_numpy(w).cuda(), dst, N, K)
        torch.cuda.synchronize()
        assert np.array_equal(dst.cpu().numpy(), tile_weights(w, N, K)), (N, K)
    with pytest.raises(uk.UkError):
        uk.pack_i4_weights(dst, dst, 48, 128)
    with pytest.raises(uk.UkError):
        uk.pack_i4_weights(dst, dst, 32, 192)


def test_invalid_arguments(uk, cuda):
    import torch
    t = torch.zeros(64, dtype=torch.int16, device="cuda")
    with pytest.raises(uk.UkError) as e:
        uk.dequant_matmul_i4(t, t, t, t, t, 1, 8, 100, 32)       # K % group_size != 0
    assert e.value.status == F.STATUS_INVALID_ARGUMENT
    with pytest.raises(uk.UkError):
        uk.dequant_matmul_i4(t, t, t, t, t, 1, 8, 128, 48)       # group_size % 32 != 0
    with pytest.raises(uk.UkError):
        uk.dequant_matmul_i4(t, t, t, t, t, 1, 8, 128, 32, F.DEQUANT_MATMUL_W_TILED)  # N % 32
    uk.dequant_matmul_i4(t, t, t, t, t, 0, 8, 128, 32)           # M == 0: nothing to do


# ---------------------------------------------------------------------------
# The reassociated form (DEQUANT_MATMUL_REASSOCIATE): i16 activations, integer
# products, float epilogue.
# ---------------------------------------------------------------------------

def test_quantize_groups_i16_equals_the_oracle(uk, cuda):
    """q and scale_x bit for bit (one float32 division each, truncation); the
    group sums within float32 rounding of the oracle's sequential sums (the
    kernel adds lane-strided partial sums with a butterfly)."""
    import torch
    for M, K, gs in ((1, 4096, 128), (5, 512, 32), (33, 1024, 256), (3, 192, 64)):
        x = synth.normal_f16(700 + M, M * K)
        x[:gs] = 0
        G = K // gs
        q0 = np.zeros(M * K, np.int16)
        sx0 = np.zeros(M * G, np.float32)
        gs0 = np.zeros(M * G, np.float32)
        assert ukref.oracle().oracle_quantize_groups_i16(ukref.ptr(x.view(np.uint16)), M, K, gs, ukref.ptr(q0),
                                                          ukref.ptr(sx0), ukref.ptr(gs0)) == 0
        q = torch.full((M * K,), 77, dtype=torch.int16, device="cuda")
        sx = torch.full((M * G,), -1.0, dtype=torch.float32, device="cuda")
        sm = torch.full((M * G,), -1.0, dtype=torch.float32, device="cuda")
        uk.quantize_groups_i16(torch.from_numpy(x.view(np.int16)).cuda(), q, sx, sm, M, K, gs)
        torch.cuda.synchronize()
        assert np.array_equal(q.cpu().numpy(), q0), (M, K, gs)
        assert np.array_equal(sx.cpu().numpy(), sx0)
        xf = np.abs(x.astype(np.float64)).reshape(M * G, gs).sum(axis=1)
        assert np.all(np.abs(sm.cpu().numpy().astype(np.float64) - gs0) <= 1e-6 * xf + 1e-12)


def run_reassoc_case(uk, M, N, K, gs, zp_u4, tiled, seed=0, stream=None):
    import torch
    G = K // gs
    x = synth.normal_f16(seed + 1, M * K)
    w = synth.uniform_u4_packed(seed + 2, N * K)
    s = synth.uniform_f16(seed + 4, N * G, 0.005, 0.02)
    if zp_u4:
        zp = synth.uniform_u4_packed(seed + 5, N * G)
        if zp.size * 2 < N * G + 1:
            zp = np.concatenate([zp, np.zeros(1, np.uint8)])
    else:
        zp = ((synth.splitmix64(seed + 5, N * G) >> np.uint64(60)).astype(np.float32) + 0.5).astype(np.float16)
    zp_arg = ukref.ptr(zp.view(np.uint8) if zp_u4 else zp.view(np.uint16))
    want = np.zeros(M * N, np.uint16)
    assert ukref.oracle().oracle_dequant_matmul_i4_reassoc(
        ukref.ptr(x.view(np.uint16)), ukref.ptr(w), ukref.ptr(s.view(np.uint16)), zp_arg, ukref.ptr(want),
        M, N, K, gs, int(zp_u4), None) == 0
    plain = np.zeros(M * N, np.uint16)
    assert ukref.oracle().oracle_dequant_matmul_i4(
        ukref.ptr(x.view(np.uint16)), ukref.ptr(w), ukref.ptr(s.view(np.uint16)), zp_arg, ukref.ptr(plain),
        M, N, K, gs, int(zp_u4)) == 0
    wd = tile_weights(w, N, K) if tiled else w
    flags = (F.DEQUANT_MATMUL_ZP_U4 if zp_u4 else 0) | (F.DEQUANT_MATMUL_W_TILED if tiled else 0) | \
        F.DEQUANT_MATMUL_REASSOCIATE
    out = torch.full((M * N,), 0x7E00, dtype=torch.int16, device="cuda")
    uk.dequant_matmul_i4(torch.from_numpy(x.view(np.int16)).cuda(), torch.from_numpy(wd).cuda(),
                         torch.from_numpy(s.view(np.int16)).cuda(),
                         torch.from_numpy(zp.view(np.uint8)).cuda(), out, M, N, K, gs, flags, stream=stream)
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.float16).astype(np.float64)
    wantf = want.view(np.float16).astype(np.float64)
    # Against the oracle of the same algorithm: the integer sums are exact and
    # the quantisation is bit-identical, so only the order of the float32
    # additions over the groups (and the group sums) differs: far inside the
    # stated tolerance; two f16 units in the last place is what is allowed here.
    ulp = np.spacing(np.abs(want.view(np.float16))).astype(np.float64)
    err = np.abs(got - wantf)
    assert np.all(err <= 2 * ulp + 1e-4), (M, N, K, gs, zp_u4, tiled, float(err.max()))
    # Against the plain (unreassociated) float64 oracle: the rewrite itself
    # loses precision (16-bit activations, truncated; the reference says so,
    # FuseDequantizationMatmul.cpp:746-748), about 5e-4 absolute at these
    # magnitudes for groups of 128 and K = 4096, more with longer K (more
    # truncated terms) and with larger groups (truncation biases every term of a
    # group the same way, and one scale serves more activations: a single
    # group of 6144 reached 0.016). So results near zero can leave the stated
    # bound, and the oracle of the rewrite leaves it at the same elements.
    # Held: for every element twice the absolute part of the stated bound,
    # scaled by K / 4096 and by the group size / 512 where those exceed 1; the
    # stated bound itself for all but two in a thousand (1 of 114688 at the
    # decode shape; running the random sweeps under 160 other seeds gave up to
    # 3 of 3247), and a small result may hold three whatever its size.
    pf = plain.view(np.float16).astype(np.float64)
    dev = np.abs(got - pf)
    scale = max(1, K // 4096) * max(1, gs // 512)
    assert np.all(dev <= 2 * ATOL * scale + RTOL * np.abs(pf)), (M, N, K, gs, float(dev.max()))
    outside = int(np.count_nonzero(dev > ATOL + RTOL * np.abs(pf)))
    assert outside <= max(3, int(2e-3 * dev.size)), (M, N, K, gs, outside)


@pytest.mark.parametrize("M", [1, 8, 32])
def test_reassociated_decode_shape_llama_ffn(uk, cuda, M):
    """The decode configuration through the reassociated form on the matrix
    cores (tiled weights, groups of 128, packed uint4 zero points)."""
    run_reassoc_case(uk, M, 14336, 4096, 128, True, True, seed=50 + M)


class _PerThreadStream:
    """hipStreamPerThread, the handle ((hipStream_t)2) as a stream object."""
    cuda_stream = 2


@pytest.mark.parametrize("M,N,K,gs,tiled", [(8, 256, 4096, 128, True), (3, 40, 384, 64, False)])
def test_reassociated_on_the_per_thread_default_stream(uk, cuda, M, N, K, gs, tiled):
    """The library keys its cached scratch buffers by stream and never leases
    one for the per-thread default stream (one handle, a different stream in
    every host thread). The reassociated form cannot run without scratch
    memory: there it takes a buffer of its own in stream order and gives the
    same result (matrix-core and element-wise kernels)."""
    import torch
    torch.cuda.synchronize()
    run_reassoc_case(uk, M, N, K, gs, True, tiled, seed=900 + M, stream=_PerThreadStream())
    assert uk.last_kernel_path() == ("dequant_i4:reassociated" if tiled else "dequant_i4:reassociated-element-wise")


@pytest.mark.parametrize("M,N,K,gs,zp_u4,tiled", [
    (3, 64, 4096, 256, True, True), (17, 96, 4096, 512, False, True),    # larger groups, f16 zero points
    (40, 64, 2048, 128, True, True), (2, 32, 2048, 256, False, True),    # K = 2048, more than 32 rows
    (5, 40, 384, 64, True, False), (2, 64, 256, 32, False, True),        # element-wise kernel
    (9, 32, 4096, 1024, True, True),                                      # a group larger than a wave's slice
    (2100, 32, 16384, 128, True, False),                                  # element-wise kernel in two passes of rows
])
def test_reassociated_other_shapes(uk, cuda, M, N, K, gs, zp_u4, tiled):
    run_reassoc_case(uk, M, N, K, gs, zp_u4, tiled, seed=M + N)
