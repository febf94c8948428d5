"""Test-side access to the two CPU checkers (test infrastructure only).

* ``oracle``  - this repository's C restatement, ``oracle/_build/liboracle.so``
* ``reflib``  - the real reference ukernel library compiled from its own sources
                by ``oracle/Makefile`` into ``oracle/_ref/libiree_uk_ref.so``
                (present wherever it was built beforehand; ``None`` otherwise)

Both take the same parameter structs as the device library; all pointers here
are host (numpy) pointers.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from iree_amd import flags as F
from iree_amd._lib import Mmt4dParams, PackParams, UnpackParams

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "_build", "liboracle.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libiree_uk_ref.so")

F16_IEEE = 0
F16_FLUSH = 1

_oracle = None
_ref = None
_ref_tried = False


def oracle():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_SO):
            subprocess.check_call(["make", "-C", ORACLE_DIR, "oracle"],
                                  stdout=subprocess.DEVNULL)
        lib = C.CDLL(ORACLE_SO)
        lib.oracle_mmt4d.restype = C.c_int
        lib.oracle_mmt4d.argtypes = [C.POINTER(Mmt4dParams), C.c_int]
        lib.oracle_mmt4d_f64.restype = C.c_int
        lib.oracle_mmt4d_f64.argtypes = [C.POINTER(Mmt4dParams)]
        lib.oracle_mmt4d_mt.restype = C.c_int
        lib.oracle_mmt4d_mt.argtypes = [C.POINTER(Mmt4dParams), C.c_int, C.c_int]
        lib.oracle_pack.restype = C.c_int
        lib.oracle_pack.argtypes = [C.POINTER(PackParams)]
        lib.oracle_unpack.restype = C.c_int
        lib.oracle_unpack.argtypes = [C.POINTER(UnpackParams)]
        lib.oracle_query_role_tile.restype = C.c_int
        lib.oracle_query_role_tile.argtypes = [C.c_uint32, C.c_int, C.c_int, C.c_int,
                                               C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
        lib.oracle_f16_to_f32.restype = C.c_float
        lib.oracle_f16_to_f32.argtypes = [C.c_uint16, C.c_int]
        lib.oracle_f32_to_f16.restype = C.c_uint16
        lib.oracle_f32_to_f16.argtypes = [C.c_float]
        lib.oracle_bf16_to_f32.restype = C.c_float
        lib.oracle_bf16_to_f32.argtypes = [C.c_uint16]
        lib.oracle_f32_to_bf16.restype = C.c_uint16
        lib.oracle_f32_to_bf16.argtypes = [C.c_float]
        lib.oracle_f8e4m3_to_f32.restype = C.c_float
        lib.oracle_f8e4m3_to_f32.argtypes = [C.c_uint8, C.c_int]
        lib.oracle_f32_to_f8e4m3.restype = C.c_uint8
        lib.oracle_f32_to_f8e4m3.argtypes = [C.c_float, C.c_int, C.c_int]
        lib.oracle_matmul_rowmajor.restype = C.c_int
        lib.oracle_matmul_rowmajor.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p,
                                               C.c_int64, C.c_int64, C.c_int64, C.c_uint32]
        lib.oracle_dequant_matmul_i4.restype = C.c_int
        lib.oracle_dequant_matmul_i4.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p,
                                                 C.c_void_p, C.c_void_p, C.c_int64,
                                                 C.c_int64, C.c_int64, C.c_int64, C.c_int]
        lib.oracle_quantize_groups_i16.restype = C.c_int
        lib.oracle_quantize_groups_i16.argtypes = [C.c_void_p, C.c_int64, C.c_int64, C.c_int64,
                                                   C.c_void_p, C.c_void_p, C.c_void_p]
        lib.oracle_dequant_matmul_i4_reassoc.restype = C.c_int
        lib.oracle_dequant_matmul_i4_reassoc.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p,
                                                         C.c_void_p, C.c_void_p, C.c_int64,
                                                         C.c_int64, C.c_int64, C.c_int64, C.c_int,
                                                         C.c_void_p]
        lib.oracle_e2e_reference_matmul.restype = C.c_int
        lib.oracle_e2e_reference_matmul.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                                    C.c_int64, C.c_int64, C.c_int64, C.c_uint32]
        lib.oracle_e2e_pseudorandom_fill.restype = C.c_uint32
        lib.oracle_e2e_pseudorandom_fill.argtypes = [C.c_uint32, C.c_int64, C.c_int32, C.c_int32,
                                                     C.c_void_p]
        lib.oracle_silu_mul.restype = C.c_double
        lib.oracle_silu_mul.argtypes = [C.c_double, C.c_double]
        _oracle = lib
    return _oracle


def reflib():
    """The compiled reference library, or None when it is not available."""
    global _ref, _ref_tried
    if not _ref_tried:
        _ref_tried = True
        if os.path.exists(REF_SO):
            lib = C.CDLL(REF_SO)
            lib.iree_uk_mmt4d.restype = None
            lib.iree_uk_mmt4d.argtypes = [C.c_void_p, C.c_int64, C.c_int64,
                                          C.c_void_p, C.c_int64, C.c_int64,
                                          C.c_void_p, C.c_int64, C.c_int64,
                                          C.c_int64, C.c_int64, C.c_int64,
                                          C.c_int32, C.c_int32, C.c_int32,
                                          C.c_uint32, C.c_void_p]
            lib.iree_uk_mmt4d_info.restype = C.c_uint32
            lib.iree_uk_mmt4d_info.argtypes = [C.c_int32, C.c_int32, C.c_int32,
                                               C.c_uint32, C.c_void_p]
            lib.iree_uk_pack.restype = None
            lib.iree_uk_pack.argtypes = [C.c_void_p] + [C.c_int64] * 3 + [C.c_void_p] + \
                [C.c_int64] * 3 + [C.c_int64] * 6 + [C.c_uint64, C.c_uint32, C.c_void_p]
            lib.iree_uk_unpack.restype = None
            lib.iree_uk_unpack.argtypes = [C.c_void_p] + [C.c_int64] * 3 + [C.c_void_p] + \
                [C.c_int64] * 3 + [C.c_int64] * 6 + [C.c_uint32, C.c_void_p]
            _ref = lib
    return _ref


# ---------------------------------------------------------------------------
# cpu_data bits for the reference's x86-64 dispatch
# (runtime/src/iree/schemas/cpu_feature_bits.inl:85-117, bit positions as data).
# ---------------------------------------------------------------------------
_X86_BITS = {"avx": 10, "fma": 11, "f16c": 14, "avx2": 15, "avx512f": 20,
             "avx512cd": 21, "avx512vl": 22, "avx512dq": 23, "avx512bw": 24,
             "avx512vnni": 28}
_NAMED = {
    "": [],
    "avx2_fma": ["avx", "avx2", "fma", "f16c"],
    "avx512_base": ["avx", "avx2", "fma", "f16c", "avx512f", "avx512bw",
                    "avx512dq", "avx512vl", "avx512cd"],
    "avx512_vnni": ["avx", "avx2", "fma", "f16c", "avx512f", "avx512bw",
                    "avx512dq", "avx512vl", "avx512cd", "avx512vnni"],
}


def host_cpu_flags():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    return set(line.split(":", 1)[1].split())
    except OSError:
        pass
    return set()


def host_supports(feature_set):
    have = host_cpu_flags()
    names = {"avx512vnni": "avx512_vnni"}
    return all(names.get(n, n) in have for n in _NAMED[feature_set])


def best_host_feature_set():
    for fs in ("avx512_vnni", "avx512_base", "avx2_fma"):
        if host_supports(fs):
            return fs
    return ""


def cpu_data(feature_set=""):
    arr = (C.c_uint64 * 8)()
    v = 0
    for n in _NAMED[feature_set]:
        v |= 1 << _X86_BITS[n]
    arr[0] = v
    return arr


# ---------------------------------------------------------------------------
# numpy helpers
# ---------------------------------------------------------------------------

def ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def f32_to_bf16_bits(x):
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f8e4m3_decode_table(ieee=True):
    """All 256 e4m3fn codes as float32 (closed form, numpy only)."""
    out = np.zeros(256, dtype=np.float32)
    for v in range(256):
        s, e, m = v >> 7, (v >> 3) & 0xF, v & 7
        if e == 15 and m == 7:
            val = np.nan
        elif e == 0:
            val = (m * 2.0 ** -9) if ieee else 0.0
        else:
            val = (1 + m / 8.0) * 2.0 ** (e - 7)
        out[v] = -val if s else val
    return out


# Element storage for one mmt4d operand: (numpy dtype of the byte container,
# bits per element).
def mmt4d_operand_dtypes(type_flag):
    T = F
    return {
        T.MMT4D_TYPE_F32F32F32: (np.float32, np.float32, np.float32),
        T.MMT4D_TYPE_S8S8S32: (np.int8, np.int8, np.int32),
        T.MMT4D_TYPE_F16F16F32: (np.uint16, np.uint16, np.float32),
        T.MMT4D_TYPE_F16F16F16: (np.uint16, np.uint16, np.uint16),
        T.MMT4D_TYPE_BF16BF16F32: (np.uint16, np.uint16, np.float32),
        T.MMT4D_TYPE_BF16BF16BF16: (np.uint16, np.uint16, np.uint16),
        T.MMT4D_TYPE_S16S16S32: (np.int16, np.int16, np.int32),
        T.MMT4D_TYPE_S16U4S32: (np.int16, np.uint8, np.int32),
        T.MMT4D_TYPE_S16S8S32: (np.int16, np.int8, np.int32),
        T.MMT4D_TYPE_S8S4S32: (np.int8, np.uint8, np.int32),
        T.MMT4D_TYPE_F8E4M3F8E4M3F32: (np.uint8, np.uint8, np.float32),
    }[type_flag]


_F8_SMALL = None


def random_operand(rng, type_flag, which, n_elems):
    """`n_elems` elements of operand `which` (0 lhs, 1 rhs, 2 out) with the value
    distributions of the reference's test generator
    (runtime/src/iree/builtins/ukernel/tools/util.c:122-168): small integers for
    floats so that every partial sum is exact, full range for 8-bit ints, random
    bytes for sub-byte types. Returns the storage array (bytes for 4-bit)."""
    global _F8_SMALL
    lhs_b, rhs_b, out_b = F.MMT4D_TYPE_BITS[type_flag]
    dt = mmt4d_operand_dtypes(type_flag)[which]
    T = F
    is_f16 = type_flag in (T.MMT4D_TYPE_F16F16F32, T.MMT4D_TYPE_F16F16F16)
    is_bf16 = type_flag in (T.MMT4D_TYPE_BF16BF16F32, T.MMT4D_TYPE_BF16BF16BF16)
    is_f8 = type_flag == T.MMT4D_TYPE_F8E4M3F8E4M3F32
    bits = (lhs_b, rhs_b, out_b * 8)[which]
    if bits == 4:
        return rng.integers(0, 256, size=(n_elems + 1) // 2, dtype=np.uint8)
    if which == 2:
        if out_b == 4 and dt == np.float32:
            return rng.integers(-2, 2, size=n_elems).astype(np.float32)
        if dt == np.int32:
            return rng.integers(-512, 1536, size=n_elems).astype(np.int32)
        if is_f16:
            return rng.integers(-8, 8, size=n_elems).astype(np.float16).view(np.uint16)
        return f32_to_bf16_bits(rng.integers(-2, 2, size=n_elems).astype(np.float32))
    if type_flag == T.MMT4D_TYPE_F32F32F32:
        return rng.integers(-2, 2, size=n_elems).astype(np.float32)
    if is_f16:
        return rng.integers(-8, 8, size=n_elems).astype(np.float16).view(np.uint16)
    if is_bf16:
        return f32_to_bf16_bits(rng.integers(-2, 2, size=n_elems).astype(np.float32))
    if is_f8:
        if _F8_SMALL is None:
            tab = f8e4m3_decode_table()
            _F8_SMALL = np.array([v for v in range(256) if np.isfinite(tab[v]) and
                                  abs(tab[v]) <= 4 and tab[v] == np.round(tab[v])],
                                 dtype=np.uint8)
        return rng.choice(_F8_SMALL, size=n_elems)
    if dt == np.int8:
        return rng.integers(-128, 128, size=n_elems).astype(np.int8)
    if dt == np.int16:
        return rng.integers(-512, 1536, size=n_elems).astype(np.int16)
    raise AssertionError("unhandled operand type")


def decode_operand(type_flag, which, storage, n_elems):
    """Storage array -> float64/int64 values (numpy only; independent of the
    oracle's C decoders)."""
    T = F
    lhs_b, rhs_b, _ = F.MMT4D_TYPE_BITS[type_flag]
    bits = (lhs_b, rhs_b)[which]
    if bits == 4:
        b = storage.astype(np.uint8)
        nib = np.empty(b.size * 2, dtype=np.int64)
        nib[0::2] = b & 0xF
        nib[1::2] = b >> 4
        nib = nib[:n_elems]
        if type_flag == T.MMT4D_TYPE_S8S4S32:
            nib = np.where(nib >= 8, nib - 16, nib)
        return nib
    if type_flag in (T.MMT4D_TYPE_F16F16F32, T.MMT4D_TYPE_F16F16F16):
        return storage.view(np.float16).astype(np.float64)
    if type_flag in (T.MMT4D_TYPE_BF16BF16F32, T.MMT4D_TYPE_BF16BF16BF16):
        return bf16_bits_to_f32(storage).astype(np.float64)
    if type_flag == T.MMT4D_TYPE_F8E4M3F8E4M3F32:
        return f8e4m3_decode_table()[storage].astype(np.float64)
    if type_flag == T.MMT4D_TYPE_F32F32F32:
        return storage.astype(np.float64)
    return storage.astype(np.int64)


class Mmt4dCase:
    """One mmt4d call on host buffers: operands, an output pre-filled with
    values (so accumulate and stride gaps are observable), and the params."""

    def __init__(self, rng, type_flag, M, N, K, M0, N0, K0, accumulate=False,
                 skip_rounding=True, loose_strides=False, offsets=False,
                 generator=random_operand):
        self.type_flag = type_flag
        self.dims = (M, N, K, M0, N0, K0)
        lhs_b, rhs_b, out_b = F.MMT4D_TYPE_BITS[type_flag]

        def stride(tight, bits):
            if not loose_strides:
                return tight
            extra = 1 if bits >= 8 else 2  # sub-byte strides stay on byte boundaries
            return tight + extra

        self.lhs_stride0 = stride(K * M0 * K0, lhs_b)
        self.rhs_stride0 = stride(K * N0 * K0, rhs_b)
        self.out_stride0 = stride(N * M0 * N0, 32)
        self.lhs_offset = 3 if offsets else 0
        self.rhs_offset = (2 if rhs_b < 8 else 5) if offsets else 0
        self.out_offset = 7 if offsets else 0
        n_lhs = self.lhs_offset + max(M, 1) * self.lhs_stride0 + 1
        n_rhs = self.rhs_offset + max(N, 1) * self.rhs_stride0 + 2
        n_out = self.out_offset + max(M, 1) * self.out_stride0 + 1
        self.lhs = generator(rng, type_flag, 0, n_lhs)
        self.rhs = generator(rng, type_flag, 1, n_rhs)
        self.out_init = generator(rng, type_flag, 2, n_out)
        self.flags = type_flag | F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION
        if accumulate:
            self.flags |= F.MMT4D_ACCUMULATE
        if skip_rounding:
            self.flags |= F.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS

    def params(self, lhs_ptr, rhs_ptr, out_ptr, flags=None):
        M, N, K, M0, N0, K0 = self.dims
        return Mmt4dParams(
            lhs_buffer=lhs_ptr, lhs_offset=self.lhs_offset, lhs_stride0=self.lhs_stride0,
            rhs_buffer=rhs_ptr, rhs_offset=self.rhs_offset, rhs_stride0=self.rhs_stride0,
            out_buffer=out_ptr, out_offset=self.out_offset, out_stride0=self.out_stride0,
            M=M, N=N, K=K, M0=M0, N0=N0, K0=K0,
            flags=self.flags if flags is None else flags, cpu_data=None)

    def run_oracle(self, f16_mode=F16_IEEE, f64=False):
        out = self.out_init.copy()
        p = self.params(ptr(self.lhs).value, ptr(self.rhs).value, ptr(out).value)
        st = oracle().oracle_mmt4d_f64(C.byref(p)) if f64 else \
            oracle().oracle_mmt4d(C.byref(p), f16_mode)
        assert st == 0, f"oracle_mmt4d status {st}"
        return out

    def run_ref(self, feature_set=""):
        lib = reflib()
        out = self.out_init.copy()
        M, N, K, M0, N0, K0 = self.dims
        cd = cpu_data(feature_set)
        lib.iree_uk_mmt4d(ptr(self.lhs), self.lhs_offset, self.lhs_stride0,
                          ptr(self.rhs), self.rhs_offset, self.rhs_stride0,
                          ptr(out), self.out_offset, self.out_stride0,
                          M, N, K, M0, N0, K0, self.flags, C.cast(cd, C.c_void_p))
        return out

    def run_numpy(self):
        """Independent numpy evaluation (einsum in int64 / float64); returns the
        expected values of the written region as an (M, N, M0, N0) array."""
        M, N, K, M0, N0, K0 = self.dims
        lhs_all = decode_operand(self.type_flag, 0, self.lhs, self.lhs.size * (2 if F.MMT4D_TYPE_BITS[self.type_flag][0] == 4 else 1))
        rhs_all = decode_operand(self.type_flag, 1, self.rhs, self.rhs.size * (2 if F.MMT4D_TYPE_BITS[self.type_flag][1] == 4 else 1))
        lhs = np.stack([lhs_all[self.lhs_offset + i * self.lhs_stride0:][:K * M0 * K0]
                        for i in range(M)]).reshape(M, K, M0, K0) if M else np.zeros((0, K, M0, K0))
        rhs = np.stack([rhs_all[self.rhs_offset + j * self.rhs_stride0:][:K * N0 * K0]
                        for j in range(N)]).reshape(N, K, N0, K0) if N else np.zeros((0, K, N0, K0))
        return np.einsum("ikac,jkbc->ijab", lhs, rhs)

    def written_region(self, out):
        M, N, K, M0, N0, K0 = self.dims
        rows = [out[self.out_offset + i * self.out_stride0:][:N * M0 * N0] for i in range(M)]
        return np.stack(rows).reshape(M, N, M0, N0) if M else np.zeros((0, N, M0, N0), out.dtype)


class BatchMmt4dCase(Mmt4dCase):
    """`batch` mmt4d problems of one shape (linalg.batch_mmt4d). The oracle runs
    them the way the reference lowers the op: one mmt4d call per batch entry on
    rank-reduced slices (compiler/src/iree/compiler/Codegen/Common/CPU/
    CPUPrepareUkernels.cpp:23-43,165-245). `gap`: elements between the end of
    one entry and the start of the next, per operand (lhs, rhs, out)."""

    def __init__(self, rng, type_flag, batch, M, N, K, M0, N0, K0, accumulate=False,
                 gap=(0, 0, 0), offsets=False, generator=random_operand):
        super().__init__(rng, type_flag, M, N, K, M0, N0, K0, accumulate=accumulate,
                         offsets=offsets, generator=generator)
        self.batch = batch
        self.lhs_batch_stride = M * self.lhs_stride0 + gap[0]
        self.rhs_batch_stride = N * self.rhs_stride0 + gap[1]
        self.out_batch_stride = M * self.out_stride0 + gap[2]
        nb = max(batch, 1)
        self.lhs = generator(rng, type_flag, 0, self.lhs_offset + nb * self.lhs_batch_stride + 1)
        self.rhs = generator(rng, type_flag, 1, self.rhs_offset + nb * self.rhs_batch_stride + 2)
        self.out_init = generator(rng, type_flag, 2, self.out_offset + nb * self.out_batch_stride + 1)

    def entry_params(self, b, lhs_ptr, rhs_ptr, out_ptr):
        p = self.params(lhs_ptr, rhs_ptr, out_ptr)
        p.lhs_offset += b * self.lhs_batch_stride
        p.rhs_offset += b * self.rhs_batch_stride
        p.out_offset += b * self.out_batch_stride
        return p

    def run_oracle(self, f16_mode=F16_IEEE, f64=False):
        out = self.out_init.copy()
        for b in range(self.batch):
            p = self.entry_params(b, ptr(self.lhs).value, ptr(self.rhs).value, ptr(out).value)
            st = oracle().oracle_mmt4d_f64(C.byref(p)) if f64 else \
                oracle().oracle_mmt4d(C.byref(p), f16_mode)
            assert st == 0, f"oracle_mmt4d status {st}"
        return out

    def run_numpy(self):
        """(batch, M, N, M0, N0) products by einsum in int64 / float64."""
        M, N, K, M0, N0, K0 = self.dims
        lhs_all = decode_operand(self.type_flag, 0, self.lhs, self.lhs.size)
        rhs_all = decode_operand(self.type_flag, 1, self.rhs, self.rhs.size)
        res = []
        for b in range(self.batch):
            lo = self.lhs_offset + b * self.lhs_batch_stride
            ro = self.rhs_offset + b * self.rhs_batch_stride
            lhs = np.stack([lhs_all[lo + i * self.lhs_stride0:][:K * M0 * K0]
                            for i in range(M)]).reshape(M, K, M0, K0)
            rhs = np.stack([rhs_all[ro + j * self.rhs_stride0:][:K * N0 * K0]
                            for j in range(N)]).reshape(N, K, N0, K0)
            res.append(np.einsum("ikac,jkbc->ijab", lhs, rhs))
        return np.stack(res)

    def written_regions(self, out):
        M, N, K, M0, N0, K0 = self.dims
        return np.stack([
            np.stack([out[self.out_offset + b * self.out_batch_stride + i * self.out_stride0:][:N * M0 * N0]
                      for i in range(M)]).reshape(M, N, M0, N0) for b in range(self.batch)])


PACK_NP_DTYPE = {F.PACK_TYPE_F32F32: np.uint32, F.PACK_TYPE_I8I8: np.uint8,
                 F.PACK_TYPE_I32I32: np.uint32, F.PACK_TYPE_F16F16: np.uint16,
                 F.PACK_TYPE_BF16BF16: np.uint16}


class PackCase:
    """One pack call on host buffers (bit patterns only; pack moves bytes)."""

    def __init__(self, rng, type_flag, outer0, outer1, tile0, tile1, *,
                 transpose_inner=False, transpose_outer=False, pad="none",
                 loose_strides=False, offsets=False, in_stride1=1, in_size=None):
        # (outer0, outer1, tile0, tile1) are in MATRIX orientation, as in the
        # reference's test (tools/pack_test.c:137-194); the stored order swaps
        # them when the transposes are set.
        dt = PACK_NP_DTYPE[type_flag]
        self.dtype = dt
        o0, o1 = outer0, outer1
        if pad == "a_lot":
            o0 += 16
            o1 += 16
        in0, in1 = outer0 * tile0, outer1 * tile1
        if pad == "one_incomplete_tile":
            in0 = max(0, in0 - int(rng.integers(0, tile0)))
            in1 = max(0, in1 - int(rng.integers(0, tile1)))
        if in_size is not None:
            in0, in1 = in_size
        self.in_size0, self.in_size1 = in0, in1
        self.out_size0, self.out_size1 = (o1, o0) if transpose_outer else (o0, o1)
        self.out_size2, self.out_size3 = (tile1, tile0) if transpose_inner else (tile0, tile1)
        self.flags = type_flag
        if transpose_inner:
            self.flags |= F.PACK_TRANSPOSE_INNER
        if transpose_outer:
            self.flags |= F.PACK_TRANSPOSE_OUTER
        self.in_stride1 = in_stride1
        self.in_stride0 = in1 * in_stride1 + (1 if loose_strides else 0)
        self.out_stride1 = self.out_size2 * self.out_size3
        self.out_stride0 = self.out_size1 * self.out_stride1 + (1 if loose_strides else 0)
        self.in_offset = int(rng.integers(0, 65536)) if offsets else 0
        self.out_offset = int(rng.integers(0, 65536)) if offsets else 0
        info = np.iinfo(dt)
        n_in = self.in_offset + max(in0, 1) * self.in_stride0 + 1
        n_out = self.out_offset + max(self.out_size0, 1) * self.out_stride0 + 1
        self.inp = rng.integers(0, int(info.max) + 1, size=n_in, dtype=np.uint64).astype(dt)
        self.out_init = rng.integers(0, int(info.max) + 1, size=n_out, dtype=np.uint64).astype(dt)
        self.padding_value = int(rng.integers(0, 1 << 63, dtype=np.uint64)) * 2 + int(rng.integers(0, 2))

    def params(self, in_ptr, out_ptr):
        return PackParams(
            in_buffer=in_ptr, in_offset=self.in_offset, in_stride0=self.in_stride0,
            in_stride1=self.in_stride1, out_buffer=out_ptr, out_offset=self.out_offset,
            out_stride0=self.out_stride0, out_stride1=self.out_stride1,
            in_size0=self.in_size0, in_size1=self.in_size1, out_size0=self.out_size0,
            out_size1=self.out_size1, out_size2=self.out_size2, out_size3=self.out_size3,
            padding_value=self.padding_value, flags=self.flags, cpu_data=None)

    def run_oracle(self):
        out = self.out_init.copy()
        p = self.params(ptr(self.inp).value, ptr(out).value)
        st = oracle().oracle_pack(C.byref(p))
        assert st == 0, f"oracle_pack status {st}"
        return out

    def run_ref(self, feature_set=""):
        out = self.out_init.copy()
        cd = cpu_data(feature_set)
        reflib().iree_uk_pack(ptr(self.inp), self.in_offset, self.in_stride0, self.in_stride1,
                              ptr(out), self.out_offset, self.out_stride0, self.out_stride1,
                              self.in_size0, self.in_size1, self.out_size0, self.out_size1,
                              self.out_size2, self.out_size3, self.padding_value, self.flags,
                              C.cast(cd, C.c_void_p))
        return out

    def run_numpy(self):
        """Closed form with numpy pad/reshape/transpose; returns the full output
        buffer (untouched elements keep out_init)."""
        ti = bool(self.flags & F.PACK_TRANSPOSE_INNER)
        to = bool(self.flags & F.PACK_TRANSPOSE_OUTER)
        O0, O1 = (self.out_size1, self.out_size0) if to else (self.out_size0, self.out_size1)
        T0, T1 = (self.out_size3, self.out_size2) if ti else (self.out_size2, self.out_size3)
        out = self.out_init.copy()
        if 0 in (self.out_size0, self.out_size1, self.out_size2, self.out_size3):
            return out
        rows = np.arange(self.in_size0)[:, None] * self.in_stride0
        cols = np.arange(self.in_size1)[None, :] * self.in_stride1
        mat = self.inp[self.in_offset + rows + cols] if self.in_size0 and self.in_size1 else \
            np.zeros((self.in_size0, self.in_size1), self.dtype)
        padv = np.array(self.padding_value & int(np.iinfo(self.dtype).max), dtype=np.uint64).astype(self.dtype)
        full = np.full((O0 * T0, O1 * T1), padv, dtype=self.dtype)
        full[:self.in_size0, :self.in_size1] = mat
        t = full.reshape(O0, T0, O1, T1).transpose(0, 2, 1, 3)  # [O0][O1][T0][T1]
        if to:
            t = t.transpose(1, 0, 2, 3)
        if ti:
            t = t.transpose(0, 1, 3, 2)
        t = np.ascontiguousarray(t).reshape(self.out_size0, -1)
        for d0 in range(self.out_size0):
            s = self.out_offset + d0 * self.out_stride0
            out[s:s + t.shape[1]] = t[d0]
        return out


class UnpackCase:
    def __init__(self, rng, type_flag, outer0, outer1, tile0, tile1, *,
                 transpose_inner=False, transpose_outer=False, pad="none",
                 loose_strides=False, offsets=False, out_stride1=1, out_size=None):
        dt = PACK_NP_DTYPE[type_flag]
        self.dtype = dt
        o0, o1 = outer0, outer1
        if pad == "a_lot":
            o0 += 16
            o1 += 16
        out0, out1 = outer0 * tile0, outer1 * tile1
        if pad == "one_incomplete_tile":
            out0 = max(0, out0 - int(rng.integers(0, tile0)))
            out1 = max(0, out1 - int(rng.integers(0, tile1)))
        if out_size is not None:
            out0, out1 = out_size
        self.out_size0, self.out_size1 = out0, out1
        self.in_size0, self.in_size1 = (o1, o0) if transpose_outer else (o0, o1)
        self.in_size2, self.in_size3 = (tile1, tile0) if transpose_inner else (tile0, tile1)
        self.flags = type_flag
        if transpose_inner:
            self.flags |= F.UNPACK_TRANSPOSE_INNER
        if transpose_outer:
            self.flags |= F.UNPACK_TRANSPOSE_OUTER
        self.in_stride1 = self.in_size2 * self.in_size3
        self.in_stride0 = self.in_size1 * self.in_stride1 + (1 if loose_strides else 0)
        self.out_stride1 = out_stride1
        self.out_stride0 = out1 * out_stride1 + (1 if loose_strides else 0)
        self.in_offset = int(rng.integers(0, 65536)) if offsets else 0
        self.out_offset = int(rng.integers(0, 65536)) if offsets else 0
        info = np.iinfo(dt)
        n_in = self.in_offset + max(self.in_size0, 1) * self.in_stride0 + 1
        n_out = self.out_offset + max(out0, 1) * self.out_stride0 + 1
        self.inp = rng.integers(0, int(info.max) + 1, size=n_in, dtype=np.uint64).astype(dt)
        self.out_init = rng.integers(0, int(info.max) + 1, size=n_out, dtype=np.uint64).astype(dt)

    def params(self, in_ptr, out_ptr):
        return UnpackParams(
            in_buffer=in_ptr, in_offset=self.in_offset, in_stride0=self.in_stride0,
            in_stride1=self.in_stride1, out_buffer=out_ptr, out_offset=self.out_offset,
            out_stride0=self.out_stride0, out_stride1=self.out_stride1,
            in_size0=self.in_size0, in_size1=self.in_size1, in_size2=self.in_size2,
            in_size3=self.in_size3, out_size0=self.out_size0, out_size1=self.out_size1,
            flags=self.flags, cpu_data=None)

    def run_oracle(self):
        out = self.out_init.copy()
        p = self.params(ptr(self.inp).value, ptr(out).value)
        st = oracle().oracle_unpack(C.byref(p))
        assert st == 0, f"oracle_unpack status {st}"
        return out

    def run_ref(self, feature_set=""):
        out = self.out_init.copy()
        cd = cpu_data(feature_set)
        reflib().iree_uk_unpack(ptr(self.inp), self.in_offset, self.in_stride0, self.in_stride1,
                                ptr(out), self.out_offset, self.out_stride0, self.out_stride1,
                                self.in_size0, self.in_size1, self.in_size2, self.in_size3,
                                self.out_size0, self.out_size1, self.flags,
                                C.cast(cd, C.c_void_p))
        return out

    def run_numpy(self):
        ti = bool(self.flags & F.UNPACK_TRANSPOSE_INNER)
        to = bool(self.flags & F.UNPACK_TRANSPOSE_OUTER)
        out = self.out_init.copy()
        if self.out_size0 == 0 or self.out_size1 == 0:
            return out
        t = np.stack([self.inp[self.in_offset + d0 * self.in_stride0:][:self.in_size1 * self.in_stride1]
                      for d0 in range(self.in_size0)])
        t = t.reshape(self.in_size0, self.in_size1, self.in_size2, self.in_size3)
        if ti:
            t = t.transpose(0, 1, 3, 2)
        if to:
            t = t.transpose(1, 0, 2, 3)
        O0, O1, T0, T1 = t.shape
        full = t.transpose(0, 2, 1, 3).reshape(O0 * T0, O1 * T1)
        rows = np.arange(self.out_size0)[:, None] * self.out_stride0
        cols = np.arange(self.out_size1)[None, :] * self.out_stride1
        out[self.out_offset + rows + cols] = full[:self.out_size0, :self.out_size1]
        return out
