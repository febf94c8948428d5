"""Pins the oracle's int4 dequant-matmul, SiLU and tile-role helpers against
closed forms evaluated with numpy."""
import ctypes as C

import numpy as np

import ukref
from iree_amd import flags as F


def _unpack_u4(b, n):
    out = np.empty(b.size * 2, np.int64)
    out[0::2] = b & 0xF
    out[1::2] = b >> 4
    return out[:n]


def test_dequant_matmul_i4_closed_form():
    rng = np.random.default_rng(0)
    o = ukref.oracle()
    for (M, N, K, gs, zp_u4) in [(1, 8, 64, 32, 0), (3, 5, 128, 32, 1), (2, 6, 256, 128, 1), (4, 3, 256, 64, 0)]:
        G = K // gs
        x = rng.standard_normal((M, K)).astype(np.float16)
        w = rng.integers(0, 256, size=N * K // 2, dtype=np.uint8)
        s = rng.uniform(0.005, 0.02, size=(N, G)).astype(np.float16)
        if zp_u4:
            zp = rng.integers(0, 256, size=(N * G + 1) // 2, dtype=np.uint8)
            zf = _unpack_u4(zp, N * G).reshape(N, G).astype(np.float64)
        else:
            zp = rng.integers(0, 16, size=(N, G)).astype(np.float16)
            zf = zp.astype(np.float64)
        out = np.zeros((M, N), np.uint16)
        st = o.oracle_dequant_matmul_i4(ukref.ptr(x), ukref.ptr(w), ukref.ptr(s), ukref.ptr(zp),
                                        ukref.ptr(out), M, N, K, gs, zp_u4)
        assert st == 0
        wq = _unpack_u4(w, N * K).reshape(N, G, gs).astype(np.float64)
        deq = (wq - zf[:, :, None]) * s.astype(np.float64)[:, :, None]
        want = x.astype(np.float64).reshape(M, G, gs)
        want = np.einsum("mgk,ngk->mn", want, deq)
        got = out.view(np.float16).astype(np.float64)
        # f64 accumulation in a different order, then one f16 rounding
        np.testing.assert_allclose(got, want, rtol=2 ** -10, atol=1e-6)
    # nibble order: byte 0x21 holds element 0 = 1 (low nibble), element 1 = 2
    x = np.array([[1.0, 0.0] + [0.0] * 30], np.float16)
    w = np.zeros(16, np.uint8)
    w[0] = 0x21
    s = np.ones((1, 1), np.float16)
    zp = np.zeros((1, 1), np.float16)
    out = np.zeros((1, 1), np.uint16)
    assert o.oracle_dequant_matmul_i4(ukref.ptr(x), ukref.ptr(w), ukref.ptr(s), ukref.ptr(zp),
                                      ukref.ptr(out), 1, 1, 32, 32, 0) == 0
    assert out.view(np.float16)[0, 0] == 1.0
    x[0, 0], x[0, 1] = 0.0, 1.0
    assert o.oracle_dequant_matmul_i4(ukref.ptr(x), ukref.ptr(w), ukref.ptr(s), ukref.ptr(zp),
                                      ukref.ptr(out), 1, 1, 32, 32, 0) == 0
    assert out.view(np.float16)[0, 0] == 2.0


def test_silu_mul():
    o = ukref.oracle()
    for g, u in [(0.0, 3.0), (1.0, 1.0), (-2.5, 0.7), (10.0, -1.0), (-30.0, 2.0)]:
        want = g * (1.0 / (1.0 + np.exp(-g))) * u
        assert abs(o.oracle_silu_mul(g, u) - want) <= 1e-15 * max(1.0, abs(want))
    assert o.oracle_silu_mul(0.0, 5.0) == 0.0


def test_query_role_mapping():
    o = ukref.oracle()
    t0, t1 = C.c_int64(), C.c_int64()
    for role, want in [(F.QUERY_ROLE_LHS, (32, 8)), (F.QUERY_ROLE_RHS, (16, 8)),
                       (F.QUERY_ROLE_RESULT, (32, 16))]:
        assert o.oracle_query_role_tile(role, 32, 16, 8, C.byref(t0), C.byref(t1)) == 0
        assert (t0.value, t1.value) == want
    assert o.oracle_query_role_tile(0, 1, 1, 1, C.byref(t0), C.byref(t1)) == F.STATUS_INVALID_ARGUMENT
