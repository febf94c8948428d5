"""Pins the oracle's reassociated int4 dequant-matmul (the opt-in rewrite of
compiler/src/iree/compiler/GlobalOptimization/FuseDequantizationMatmul.cpp:398-645
of the reference: per-group i16 quantisation of the activations, an integer
i16 x u4 -> i32 contraction per group, a float epilogue over the groups).
There is no runnable reference for the pattern (it is compiler IR), so each
stage is pinned by itself: the quantisation by numpy float32 arithmetic, the
integer core by a numpy integer product and by the reference's own
iree_uk_mmt4d S16U4S32 ukernel on its 1x32x8 tile (oracle/_ref), the epilogue
by the closed form in float64, the whole by the plain (unreassociated) oracle
on inputs the quantisation represents exactly."""
import ctypes as C

import numpy as np
import pytest

import ukref
from iree_amd import flags as F


def _inputs(rng, M, N, K, gs, zp_u4=True):
    G = K // gs
    x = (rng.standard_normal(M * K)).astype(np.float16)
    w = rng.integers(0, 256, N * K // 2, dtype=np.uint8)
    s = rng.uniform(0.005, 0.02, N * G).astype(np.float16)
    if zp_u4:
        zp = rng.integers(0, 256, (N * G + 1) // 2 + 1, dtype=np.uint8)
    else:
        zp = (rng.integers(0, 16, N * G) + 0.5).astype(np.float16)
    return x, w, s, zp


def _nibbles(w, N, K):
    n = np.empty(w.size * 2, np.int64)
    n[0::2] = w & 0xF
    n[1::2] = w >> 4
    return n[:N * K].reshape(N, K)


def _zp_values(zp, N, G, zp_u4):
    if not zp_u4:
        return zp.astype(np.float64).reshape(N, G)
    n = np.empty(zp.size * 2, np.float64)
    n[0::2] = zp & 0xF
    n[1::2] = zp >> 4
    return n[:N * G].reshape(N, G)


def _run(x, w, s, zp, M, N, K, gs, zp_u4):
    G = K // gs
    out = np.zeros(M * N, np.uint16)
    core = np.zeros(M * N * G, np.int32)
    st = ukref.oracle().oracle_dequant_matmul_i4_reassoc(
        ukref.ptr(x.view(np.uint16)), ukref.ptr(w), ukref.ptr(s.view(np.uint16)),
        ukref.ptr(zp.view(np.uint8) if zp_u4 else zp.view(np.uint16)), ukref.ptr(out),
        M, N, K, gs, int(zp_u4), ukref.ptr(core))
    assert st == 0
    return out.view(np.float16).reshape(M, N), core.reshape(M, N, G)


def _quantize(x, M, K, gs):
    G = K // gs
    q = np.zeros(M * K, np.int16)
    sx = np.zeros(M * G, np.float32)
    gsum = np.zeros(M * G, np.float32)
    assert ukref.oracle().oracle_quantize_groups_i16(ukref.ptr(x.view(np.uint16)), M, K, gs,
                                                      ukref.ptr(q), ukref.ptr(sx), ukref.ptr(gsum)) == 0
    return q.reshape(M, K), sx.reshape(M, G), gsum.reshape(M, G)


@pytest.mark.parametrize("M,K,gs", [(1, 256, 128), (5, 512, 32), (3, 384, 64)])
def test_quantisation_is_float32_divide_and_truncate(M, K, gs):
    rng = np.random.default_rng(M * K + gs)
    x = rng.standard_normal(M * K).astype(np.float16)
    x[:gs] = 0                                    # a group of zeros quantises to zeros
    q, sx, gsum = _quantize(x, M, K, gs)
    xf = x.astype(np.float32).reshape(M, K // gs, gs)
    mx = np.abs(xf).max(axis=2)
    want_sx = (mx / np.float32(32767.0)).astype(np.float32)
    assert np.array_equal(sx, want_sx)
    with np.errstate(divide="ignore", invalid="ignore"):
        ratio = (xf / want_sx[:, :, None]).astype(np.float32)
    want_q = np.where(want_sx[:, :, None] > 0, np.trunc(ratio), 0).astype(np.int16).reshape(M, K)
    assert np.array_equal(q, want_q)
    assert np.abs(q).max() <= 32767 and np.abs(q).max() >= 32766
    # the group sums are sequential float32 additions in k order
    want_sum = np.zeros((M, K // gs), np.float32)
    for k in range(gs):
        want_sum = (want_sum + xf[:, :, k]).astype(np.float32)
    assert np.array_equal(gsum, want_sum)


@pytest.mark.parametrize("M,N,K,gs,zp_u4", [(1, 64, 256, 128, True), (4, 32, 256, 32, False),
                                            (7, 96, 384, 128, True)])
def test_integer_core_and_epilogue(M, N, K, gs, zp_u4):
    rng = np.random.default_rng(N + K + gs)
    x, w, s, zp = _inputs(rng, M, N, K, gs, zp_u4)
    out, core = _run(x, w, s, zp, M, N, K, gs, zp_u4)
    q, sx, gsum = _quantize(x, M, K, gs)
    G = K // gs
    wn = _nibbles(w, N, K)
    want_core = np.einsum("mgk,ngk->mng", q.astype(np.int64).reshape(M, G, gs), wn.reshape(N, G, gs))
    assert np.array_equal(core, want_core)
    # epilogue in float64: sum_g (acc * scale_x * scale - zp * scale * group_sum)
    sv = s.astype(np.float64).reshape(N, G)
    zv = _zp_values(zp, N, G, zp_u4)
    want = (want_core * sx.astype(np.float64)[:, None, :] * sv[None] -
            (zv * sv)[None] * gsum.astype(np.float64)[:, None, :]).sum(axis=2)
    got = out.astype(np.float64)
    # f32 steps and one f16 rounding against float64
    assert np.all(np.abs(got - want) <= 2e-3 * np.abs(want) + 1e-3)
    # and against the plain oracle: the 16-bit quantisation loses little
    plain = np.zeros(M * N, np.uint16)
    assert ukref.oracle().oracle_dequant_matmul_i4(
        ukref.ptr(x.view(np.uint16)), ukref.ptr(w), ukref.ptr(s.view(np.uint16)),
        ukref.ptr(zp.view(np.uint8) if zp_u4 else zp.view(np.uint16)), ukref.ptr(plain),
        M, N, K, gs, int(zp_u4)) == 0
    pf = plain.view(np.float16).astype(np.float64).reshape(M, N)
    assert np.all(np.abs(got - pf) <= 1e-3 + 1e-2 * np.abs(pf))


def test_integer_core_equals_the_reference_s16u4_ukernel():
    """The contraction the rewrite produces is what the reference's
    iree_uk_mmt4d S16U4S32 computes on its 1x32x8 tile
    (arch/x86_64/mmt4d_x86_64_tiles.inl:75): one call per group."""
    lib = ukref.reflib()
    if lib is None:
        pytest.skip("oracle/_ref is not built here")
    rng = np.random.default_rng(99)
    M, N, K, gs = 3, 64, 256, 128
    x, w, s, zp = _inputs(rng, M, N, K, gs)
    _, core = _run(x, w, s, zp, M, N, K, gs, True)
    q, _, _ = _quantize(x, M, K, gs)
    wn = _nibbles(w, N, K)
    G, K1, N1 = K // gs, gs // 8, N // 32
    fs = ukref.best_host_feature_set()
    cd = ukref.cpu_data(fs)
    for m in range(M):
        for g in range(G):
            lhs = np.ascontiguousarray(q[m, g * gs:(g + 1) * gs]).astype(np.int16)        # [K1][1][8]
            r = wn[:, g * gs:(g + 1) * gs].reshape(N1, 32, K1, 8).transpose(0, 2, 1, 3)    # [N1][K1][32][8]
            flat = np.ascontiguousarray(r).reshape(-1).astype(np.uint8)
            rhs = (flat[0::2] | (flat[1::2] << 4)).astype(np.uint8)
            out = np.zeros(N1 * 32, np.int32)
            lib.iree_uk_mmt4d(ukref.ptr(lhs), 0, K1 * 8, ukref.ptr(rhs), 0, K1 * 32 * 8, ukref.ptr(out), 0,
                              N1 * 32, 1, N1, K1, 1, 32, 8,
                              F.MMT4D_TYPE_S16U4S32 | F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION,
                              C.cast(cd, C.c_void_p))
            assert np.array_equal(out, core[m, :, g]), (m, g)


def test_exactly_representable_activations_give_the_plain_result():
    """Activations that are 0 or +-(the group's maximum) quantise to 0 and
    +-32767 without error, so the reassociated result is the plain one up to
    the float32 steps: within one f16 unit in the last place."""
    rng = np.random.default_rng(5)
    M, N, K, gs = 4, 64, 512, 128
    x, w, s, zp = _inputs(rng, M, N, K, gs)
    mags = rng.uniform(0.25, 4.0, (M, K // gs, 1)).astype(np.float16)
    signs = rng.integers(-1, 2, (M, K // gs, gs)).astype(np.float16)
    signs[:, :, 0] = 1
    x = (mags * signs).astype(np.float16).reshape(-1)
    out, _ = _run(x, w, s, zp, M, N, K, gs, True)
    plain = np.zeros(M * N, np.uint16)
    assert ukref.oracle().oracle_dequant_matmul_i4(
        ukref.ptr(x.view(np.uint16)), ukref.ptr(w), ukref.ptr(s.view(np.uint16)), ukref.ptr(zp),
        ukref.ptr(plain), M, N, K, gs, 1) == 0
    pf = plain.view(np.float16).reshape(M, N)
    ulp = np.spacing(np.abs(pf).astype(np.float16)).astype(np.float64)
    assert np.all(np.abs(out.astype(np.float64) - pf.astype(np.float64)) <= ulp + 2e-4 * np.abs(pf.astype(np.float64)))
