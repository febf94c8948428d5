"""Writes tests/golden/golden.json from the REAL reference ukernel library
(oracle/_ref/libiree_uk_ref.so, compiled from the reference's own sources by
oracle/Makefile). Run where the reference sources exist:

    make -C oracle ref && python tests/golden/make_golden.py

Inputs come from iree_amd.synth (integer-only, bit-reproducible), so the
fixtures are digests plus a few sampled values rather than bulk data.
"""
import ctypes as C
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import ukref  # noqa: E402
from iree_amd import flags as F  # noqa: E402
from iree_amd import synth  # noqa: E402


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def ref_matmul(lib, cd, A, B, Cacc, M, N, K, tile, mm_type, in_pack, out_pack, out_dtype):
    """The reference's end-to-end chain (tools/e2e_matmul_benchmark.c:173-186)."""
    M0, N0, K0 = tile
    M1, N1, K1 = -(-M // M0), -(-N // N0), -(-K // K0)
    pa = np.zeros(M1 * K1 * M0 * K0, A.dtype)
    pb = np.zeros(N1 * K1 * N0 * K0, B.dtype)
    pc = np.zeros(M1 * N1 * M0 * N0, out_dtype)
    c = np.zeros(M * N, out_dtype) if Cacc is None else Cacc.copy()
    cdp = C.cast(cd, C.c_void_p)
    lib.iree_uk_pack(ukref.ptr(A), 0, K, 1, ukref.ptr(pa), 0, K1 * M0 * K0, M0 * K0,
                     M, K, M1, K1, M0, K0, 0, in_pack, cdp)
    lib.iree_uk_pack(ukref.ptr(B), 0, N, 1, ukref.ptr(pb), 0, K1 * N0 * K0, N0 * K0,
                     K, N, N1, K1, N0, K0, 0,
                     in_pack | F.PACK_TRANSPOSE_INNER | F.PACK_TRANSPOSE_OUTER, cdp)
    flags = mm_type | F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION
    if Cacc is not None:
        lib.iree_uk_pack(ukref.ptr(c), 0, N, 1, ukref.ptr(pc), 0, N1 * M0 * N0, M0 * N0,
                         M, N, M1, N1, M0, N0, 0, out_pack, cdp)
        flags |= F.MMT4D_ACCUMULATE
    lib.iree_uk_mmt4d(ukref.ptr(pa), 0, K1 * M0 * K0, ukref.ptr(pb), 0, K1 * N0 * K0,
                      ukref.ptr(pc), 0, N1 * M0 * N0, M1, N1, K1, M0, N0, K0, flags, cdp)
    lib.iree_uk_unpack(ukref.ptr(pc), 0, N1 * M0 * N0, M0 * N0, ukref.ptr(c), 0, N, 1,
                       M1, N1, M0, N0, M, N, out_pack, cdp)
    return c


def main():
    lib = ukref.reflib()
    if lib is None:
        raise SystemExit("oracle/_ref/libiree_uk_ref.so is missing: run `make -C oracle ref`")
    fs = ukref.best_host_feature_set()
    cd = ukref.cpu_data(fs)
    g = {"_generated_by": "tests/golden/make_golden.py",
         "_source": "reference ukernel library compiled from its own sources (oracle/Makefile)",
         "_cpu_feature_set": fs}

    # pack f16 8191x5001 -> [256][313][32][16], padding value 0
    R, Cc, T0, T1 = 8191, 5001, 32, 16
    O0, O1 = -(-R // T0), -(-Cc // T1)
    x = synth.uniform_pm1_f16(1, R * Cc).view(np.uint16)
    packed = np.full(O0 * O1 * T0 * T1, 0x5A5A, np.uint16)
    lib.iree_uk_pack(ukref.ptr(x), 0, Cc, 1, ukref.ptr(packed), 0, O1 * T0 * T1, T0 * T1,
                     R, Cc, O0, O1, T0, T1, 0, F.PACK_TYPE_F16F16, C.cast(cd, C.c_void_p))
    g["pack_f16_8191x5001_32x16_sha256"] = sha(packed)
    back = np.zeros(R * Cc, np.uint16)
    lib.iree_uk_unpack(ukref.ptr(packed), 0, O1 * T0 * T1, T0 * T1, ukref.ptr(back), 0, Cc, 1,
                       O0, O1, T0, T1, R, Cc, F.UNPACK_TYPE_F16F16, C.cast(cd, C.c_void_p))
    assert np.array_equal(back, x)
    g["input_f16_8191x5001_sha256"] = sha(x)

    # i8 1024^3 through the reference's x86 tile (16x16x2) and through the
    # gfx950 tile (32x32x16, generic tile function): same row-major result
    M = N = K = 1024
    A, B = synth.uniform_int8(1, M * K), synth.uniform_int8(2, K * N)
    c1 = ref_matmul(lib, cd, A, B, None, M, N, K, (16, 16, 2), F.MMT4D_TYPE_S8S8S32,
                    F.PACK_TYPE_I8I8, F.PACK_TYPE_I32I32, np.int32)
    g["matmul_i8_1024_sha256"] = sha(c1)
    c2 = ref_matmul(lib, cd, A[:256 * 256], B[:256 * 256], None, 256, 256, 256, (32, 32, 16),
                    F.MMT4D_TYPE_S8S8S32, F.PACK_TYPE_I8I8, F.PACK_TYPE_I32I32, np.int32)
    g["matmul_i8_256_sha256"] = sha(c2)

    # ragged shape with accumulate (padded edges in all three dimensions)
    M, N, K = 123, 77, 201
    A, B = synth.uniform_int8(1, M * K), synth.uniform_int8(2, K * N)
    c0 = (synth.splitmix64(3, M * N) >> np.uint64(44)).astype(np.int64).astype(np.int32)
    c3 = ref_matmul(lib, cd, A, B, c0, M, N, K, (16, 16, 2), F.MMT4D_TYPE_S8S8S32,
                    F.PACK_TYPE_I8I8, F.PACK_TYPE_I32I32, np.int32)
    g["matmul_i8_123x77x201_acc_sha256"] = sha(c3)

    # f16 -> f32, small-integer inputs (exact): 200x120x300, tile 16x16x1
    M, N, K = 200, 120, 300
    A = synth.small_int_f16(1, M * K).view(np.uint16)
    B = synth.small_int_f16(2, K * N).view(np.uint16)
    c4 = ref_matmul(lib, cd, A, B, None, M, N, K, (16, 16, 1), F.MMT4D_TYPE_F16F16F32,
                    F.PACK_TYPE_F16F16, F.PACK_TYPE_F32F32, np.float32)
    g["matmul_f16_exact_200x120x300_sha256"] = sha(c4)

    # f16 -> f32, N(0,1)/sqrt(K) inputs at 512^3: 16 sampled outputs of the
    # reference's AVX-512 (or best available) path, for tolerance checks
    M = N = K = 512
    A = synth.normal_f16(1, M * K, 1 / np.sqrt(K)).view(np.uint16)
    B = synth.normal_f16(2, K * N, 1 / np.sqrt(K)).view(np.uint16)
    c5 = ref_matmul(lib, cd, A, B, None, M, N, K, (16, 16, 1), F.MMT4D_TYPE_F16F16F32,
                    F.PACK_TYPE_F16F16, F.PACK_TYPE_F32F32, np.float32)
    idx = (synth.splitmix64(77, 16) % np.uint64(M * N)).astype(np.int64)
    g["matmul_f16_normal_512_samples"] = {"index": [int(i) for i in idx],
                                          "value_f32_hex": [c5[i].tobytes().hex() for i in idx]}

    with open(os.path.join(HERE, "golden.json"), "w") as f:
        json.dump(g, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps(g, indent=1, sort_keys=True))


if __name__ == "__main__":
    main()
