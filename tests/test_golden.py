"""The oracle reproduces the committed fixtures that tests/golden/make_golden.py
produced from the real reference library (digests of full outputs on seeded
inputs). This pins the oracle wherever the reference itself is unavailable."""
import ctypes as C
import hashlib
import json
import os

import numpy as np

import ukref
from iree_amd import flags as F
from iree_amd import synth
from iree_amd._lib import Mmt4dParams, PackParams, UnpackParams

with open(os.path.join(os.path.dirname(__file__), "golden", "golden.json")) as f:
    GOLDEN = json.load(f)


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def oracle_matmul(A, B, Cacc, M, N, K, tile, mm_type, in_pack, out_pack, out_dtype, f64=False):
    o = ukref.oracle()
    M0, N0, K0 = tile
    M1, N1, K1 = -(-M // M0), -(-N // N0), -(-K // K0)
    pa = np.zeros(M1 * K1 * M0 * K0, A.dtype)
    pb = np.zeros(N1 * K1 * N0 * K0, B.dtype)
    pc = np.zeros(M1 * N1 * M0 * N0, out_dtype)
    c = np.zeros(M * N, out_dtype) if Cacc is None else Cacc.copy()
    p = PackParams(ukref.ptr(A).value, 0, K, 1, ukref.ptr(pa).value, 0, K1 * M0 * K0, M0 * K0,
                   M, K, M1, K1, M0, K0, 0, in_pack, None)
    assert o.oracle_pack(C.byref(p)) == 0
    p = PackParams(ukref.ptr(B).value, 0, N, 1, ukref.ptr(pb).value, 0, K1 * N0 * K0, N0 * K0,
                   K, N, N1, K1, N0, K0, 0, in_pack | F.PACK_TRANSPOSE_INNER | F.PACK_TRANSPOSE_OUTER, None)
    assert o.oracle_pack(C.byref(p)) == 0
    flags = mm_type
    if Cacc is not None:
        p = PackParams(ukref.ptr(c).value, 0, N, 1, ukref.ptr(pc).value, 0, N1 * M0 * N0, M0 * N0,
                       M, N, M1, N1, M0, N0, 0, out_pack, None)
        assert o.oracle_pack(C.byref(p)) == 0
        flags |= F.MMT4D_ACCUMULATE
    mp = Mmt4dParams(ukref.ptr(pa).value, 0, K1 * M0 * K0, ukref.ptr(pb).value, 0, K1 * N0 * K0,
                     ukref.ptr(pc).value, 0, N1 * M0 * N0, M1, N1, K1, M0, N0, K0, flags, None)
    if f64:
        assert o.oracle_mmt4d_f64(C.byref(mp)) == 0
    else:
        assert o.oracle_mmt4d_mt(C.byref(mp), ukref.F16_IEEE, 8) == 0
    up = UnpackParams(ukref.ptr(pc).value, 0, N1 * M0 * N0, M0 * N0, ukref.ptr(c).value, 0, N, 1,
                      M1, N1, M0, N0, M, N, out_pack, None)
    assert o.oracle_unpack(C.byref(up)) == 0
    return c


def test_pack_f16_8191x5001_digest():
    R, Cc, T0, T1 = 8191, 5001, 32, 16
    O0, O1 = -(-R // T0), -(-Cc // T1)
    x = synth.uniform_pm1_f16(1, R * Cc).view(np.uint16)
    assert sha(x) == GOLDEN["input_f16_8191x5001_sha256"]
    packed = np.full(O0 * O1 * T0 * T1, 0x5A5A, np.uint16)
    p = PackParams(ukref.ptr(x).value, 0, Cc, 1, ukref.ptr(packed).value, 0, O1 * T0 * T1, T0 * T1,
                   R, Cc, O0, O1, T0, T1, 0, F.PACK_TYPE_F16F16, None)
    assert ukref.oracle().oracle_pack(C.byref(p)) == 0
    assert sha(packed) == GOLDEN["pack_f16_8191x5001_32x16_sha256"]


def test_i8_matmul_digests_with_cpu_and_gfx950_tiles():
    A, B = synth.uniform_int8(1, 256 * 256), synth.uniform_int8(2, 256 * 256)
    for tile in [(16, 16, 2), (32, 32, 16), (32, 32, 32)]:
        c = oracle_matmul(A, B, None, 256, 256, 256, tile, F.MMT4D_TYPE_S8S8S32,
                          F.PACK_TYPE_I8I8, F.PACK_TYPE_I32I32, np.int32)
        assert sha(c) == GOLDEN["matmul_i8_256_sha256"], tile
    M, N, K = 123, 77, 201
    A, B = synth.uniform_int8(1, M * K), synth.uniform_int8(2, K * N)
    c0 = (synth.splitmix64(3, M * N) >> np.uint64(44)).astype(np.int64).astype(np.int32)
    for tile in [(16, 16, 2), (32, 32, 16)]:
        c = oracle_matmul(A, B, c0, M, N, K, tile, F.MMT4D_TYPE_S8S8S32,
                          F.PACK_TYPE_I8I8, F.PACK_TYPE_I32I32, np.int32)
        assert sha(c) == GOLDEN["matmul_i8_123x77x201_acc_sha256"], tile


def test_i8_1024_rowmajor_digest():
    M = N = K = 1024
    A, B = synth.uniform_int8(1, M * K), synth.uniform_int8(2, K * N)
    c = np.zeros(M * N, np.int32)
    assert ukref.oracle().oracle_matmul_rowmajor(ukref.ptr(A), ukref.ptr(B), ukref.ptr(c), M, N, K,
                                                 F.MMT4D_TYPE_S8S8S32) == 0
    assert sha(c) == GOLDEN["matmul_i8_1024_sha256"]


def test_f16_digests_and_samples():
    M, N, K = 200, 120, 300
    A = synth.small_int_f16(1, M * K).view(np.uint16)
    B = synth.small_int_f16(2, K * N).view(np.uint16)
    for tile in [(16, 16, 1), (32, 32, 8)]:
        c = oracle_matmul(A, B, None, M, N, K, tile, F.MMT4D_TYPE_F16F16F32,
                          F.PACK_TYPE_F16F16, F.PACK_TYPE_F32F32, np.float32)
        assert sha(c) == GOLDEN["matmul_f16_exact_200x120x300_sha256"], tile
    M = N = K = 512
    A = synth.normal_f16(1, M * K, 1 / np.sqrt(K)).view(np.uint16)
    B = synth.normal_f16(2, K * N, 1 / np.sqrt(K)).view(np.uint16)
    c = oracle_matmul(A, B, None, M, N, K, (32, 32, 8), F.MMT4D_TYPE_F16F16F32,
                      F.PACK_TYPE_F16F16, F.PACK_TYPE_F32F32, np.float32, f64=True)
    s = GOLDEN["matmul_f16_normal_512_samples"]
    want = np.array([np.frombuffer(bytes.fromhex(h), np.float32)[0] for h in s["value_f32_hex"]])
    got = c[np.array(s["index"])]
    # reference x86 path (f32 FMA chain) vs f64 accumulation: a few f32 ulp
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-7)
