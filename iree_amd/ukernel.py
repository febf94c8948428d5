"""Host mirror of the reference's ukernel entry points over the C-ABI library.

Function names, argument names and meaning follow
runtime/src/iree/builtins/ukernel/{mmt4d.h:14-21, pack.h:26-34, unpack.h:17-25,
query_tile_sizes.h:29-31} of the reference; buffers are torch CUDA tensors used
only as owners of device memory (their ``data_ptr()`` is the base pointer,
offsets and strides are in elements exactly as in the reference). Work is
enqueued on torch's current stream. Errors from the library raise ``UkError``.
"""
import ctypes as C

import torch

from . import flags as F
from ._lib import (MatmulTile, Mmt4dParams, PackParams, QueryOutParams, QueryParams,
                   UnpackParams, load_library)


class UkError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"iree_amd_uk status {status}: {message}")
        self.status = status


def _check(status):
    if status != 0:
        msg = load_library().iree_amd_uk_last_error()
        raise UkError(status, msg.decode() if msg else "")


def last_kernel_path():
    """Name of the kernel family that served this thread's last mmt4d or
    dequant_matmul_i4 call (see include/iree_amd_uk.h)."""
    return load_library().iree_amd_uk_last_kernel_path().decode()


def _ptr(t):
    # (plain ints: the declared argtypes convert them, which is cheaper than
    # building a c_void_p per argument)
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("ukernel buffers must be CUDA (HIP) tensors")
    return t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(stream):
    if stream is None:
        if _raw_stream is not None:
            return _raw_stream(torch.cuda.current_device())
        stream = torch.cuda.current_stream()
    return stream.cuda_stream


def mmt4d(lhs_buffer, rhs_buffer, out_buffer, M, N, K, M0, N0, K0, flags, *,
          lhs_offset=0, lhs_stride0=None, rhs_offset=0, rhs_stride0=None,
          out_offset=0, out_stride0=None, stream=None):
    """iree_uk_mmt4d (reference mmt4d.h:14-21). Strides default to tight."""
    if lhs_stride0 is None:
        lhs_stride0 = K * M0 * K0
    if rhs_stride0 is None:
        rhs_stride0 = K * N0 * K0
    if out_stride0 is None:
        out_stride0 = N * M0 * N0
    lib = load_library()
    _check(lib.iree_amd_uk_mmt4d(
        _ptr(lhs_buffer), lhs_offset, lhs_stride0, _ptr(rhs_buffer), rhs_offset,
        rhs_stride0, _ptr(out_buffer), out_offset, out_stride0, M, N, K, M0, N0,
        K0, flags, None, _stream(stream)))


def batch_mmt4d(lhs_buffer, rhs_buffer, out_buffer, batch, M, N, K, M0, N0, K0, flags, *,
                lhs_offset=0, lhs_stride0=None, rhs_offset=0, rhs_stride0=None,
                out_offset=0, out_stride0=None, lhs_batch_stride=None,
                rhs_batch_stride=None, out_batch_stride=None, stream=None):
    """linalg.batch_mmt4d: `batch` mmt4d problems of one shape, which the
    reference runs as one mmt4d ukernel call per entry (reference
    CPUPrepareUkernels.cpp:23-43,165-245). Strides default to tight."""
    if lhs_stride0 is None:
        lhs_stride0 = K * M0 * K0
    if rhs_stride0 is None:
        rhs_stride0 = K * N0 * K0
    if out_stride0 is None:
        out_stride0 = N * M0 * N0
    if lhs_batch_stride is None:
        lhs_batch_stride = M * lhs_stride0
    if rhs_batch_stride is None:
        rhs_batch_stride = N * rhs_stride0
    if out_batch_stride is None:
        out_batch_stride = M * out_stride0
    p = Mmt4dParams(_ptr(lhs_buffer), lhs_offset, lhs_stride0, _ptr(rhs_buffer), rhs_offset,
                    rhs_stride0, _ptr(out_buffer), out_offset, out_stride0, M, N, K, M0, N0,
                    K0, flags, None)
    _check(load_library().iree_amd_uk_batch_mmt4d(
        C.byref(p), batch, lhs_batch_stride, rhs_batch_stride, out_batch_stride, _stream(stream)))


def mmt4d_info(M0, N0, K0, flags):
    """iree_uk_mmt4d_info (reference mmt4d.h:23-25)."""
    return load_library().iree_amd_uk_mmt4d_info(M0, N0, K0, flags, None)


def pack(in_buffer, out_buffer, in_size0, in_size1, out_size0, out_size1,
         out_size2, out_size3, padding_value, flags, *, in_offset=0,
         in_stride0=None, in_stride1=1, out_offset=0, out_stride0=None,
         out_stride1=None, stream=None):
    """iree_uk_pack (reference pack.h:26-34). Strides default to tight."""
    if in_stride0 is None:
        in_stride0 = in_size1 * in_stride1
    if out_stride1 is None:
        out_stride1 = out_size2 * out_size3
    if out_stride0 is None:
        out_stride0 = out_size1 * out_stride1
    lib = load_library()
    _check(lib.iree_amd_uk_pack(
        _ptr(in_buffer), in_offset, in_stride0, in_stride1, _ptr(out_buffer),
        out_offset, out_stride0, out_stride1, in_size0, in_size1, out_size0,
        out_size1, out_size2, out_size3, padding_value & 0xFFFFFFFFFFFFFFFF,
        flags, None, _stream(stream)))


def unpack(in_buffer, out_buffer, in_size0, in_size1, in_size2, in_size3,
           out_size0, out_size1, flags, *, in_offset=0, in_stride0=None,
           in_stride1=None, out_offset=0, out_stride0=None, out_stride1=1,
           stream=None):
    """iree_uk_unpack (reference unpack.h:17-25). Strides default to tight."""
    if in_stride1 is None:
        in_stride1 = in_size2 * in_size3
    if in_stride0 is None:
        in_stride0 = in_size1 * in_stride1
    if out_stride0 is None:
        out_stride0 = out_size1 * out_stride1
    lib = load_library()
    _check(lib.iree_amd_uk_unpack(
        _ptr(in_buffer), in_offset, in_stride0, in_stride1, _ptr(out_buffer),
        out_offset, out_stride0, out_stride1, in_size0, in_size1, in_size2,
        in_size3, out_size0, out_size1, flags, None, _stream(stream)))


_INT64_MIN = -(1 << 63)


def query_tile_sizes_2d(flags, size0=_INT64_MIN, size1=_INT64_MIN):
    """iree_uk_query_tile_sizes_2d (reference query_tile_sizes.h:29-31).
    Returns (tile_size0, tile_size1). Needs no device."""
    p = QueryParams(flags=flags, size0=size0, size1=size1, cpu_data=None)
    o = QueryOutParams()
    _check(load_library().iree_amd_uk_query_tile_sizes_2d(C.byref(p), C.byref(o)))
    return int(o.tile_size0), int(o.tile_size1)


def enumerate_matmul_tiles(operation):
    """The (M, N, K) tiles the gfx950 kernels serve for a QUERY_OP_* operation:
    the full tile and its truncations in M (the reference's
    enumerateMatmulTile*, CPUMaterializeEncodingPass.cpp:168-281)."""
    n = C.c_int32(0)
    _check(load_library().iree_amd_uk_enumerate_matmul_tiles(operation, None, 0, C.byref(n)))
    tiles = (MatmulTile * n.value)()
    _check(load_library().iree_amd_uk_enumerate_matmul_tiles(operation, tiles, n.value, C.byref(n)))
    return [(t.M, t.N, t.K) for t in tiles]


def choose_matmul_tile(tiles, narrow_m=0, narrow_n=0, upper_bound=None):
    """The reference's chooseMatmulTile (CPUMaterializeEncodingPass.cpp:284-377)
    over a list of (M, N, K) tiles; returns the chosen (M, N, K)."""
    arr = (MatmulTile * max(len(tiles), 1))(*[MatmulTile(*t) for t in tiles])
    ub = (C.c_int64 * 3)(*upper_bound) if upper_bound is not None else None
    out = MatmulTile()
    _check(load_library().iree_amd_uk_choose_matmul_tile(arr, len(tiles), narrow_m, narrow_n, ub, C.byref(out)))
    return out.M, out.N, out.K


def query_matmul_tile_sizes(operation, M=_INT64_MIN, N=_INT64_MIN, K=_INT64_MIN):
    """The (M0, N0, K0) tile of one matmul from its three sizes at once
    (``_INT64_MIN`` = dynamic): at most one of M0 and N0 is narrowed, the one of
    the smaller static size (the reference's chooseMatmulTile,
    CPUMaterializeEncodingPass.cpp:296-303)."""
    out = MatmulTile()
    _check(load_library().iree_amd_uk_query_matmul_tile_sizes(operation, M, N, K, C.byref(out)))
    return out.M, out.N, out.K


def dequant_matmul_i4(x, w, scale, zp, out, M, N, K, group_size, flags=0,
                      stream=None):
    """Grouped int4-weight dequantising matmul (see include/iree_amd_uk.h)."""
    _check(load_library().iree_amd_uk_dequant_matmul_i4(
        _ptr(x), _ptr(w), _ptr(scale), _ptr(zp), _ptr(out), M, N, K, group_size,
        flags, _stream(stream)))


def quantize_groups_i16(x, q, scale_x, group_sum, M, K, group_size, stream=None):
    """Per-group 16-bit quantisation of f16 activations: the first step of the
    reassociated dequantising matmul (see include/iree_amd_uk.h)."""
    _check(load_library().iree_amd_uk_quantize_groups_i16(
        _ptr(x), _ptr(q), _ptr(scale_x), _ptr(group_sum), M, K, group_size, _stream(stream)))


def pack_i4_weights(w_rowmajor, w_tiled, N, K, stream=None):
    """Row-major [N][K/2] 4-bit weights -> the DEQUANT_MATMUL_W_TILED layout."""
    _check(load_library().iree_amd_uk_pack_i4_weights(
        _ptr(w_rowmajor), _ptr(w_tiled), N, K, _stream(stream)))


def quantize_f16_to_f8e4m3(inp, out, n, inv_scale, stream=None):
    _check(load_library().iree_amd_uk_quantize_f16_to_f8e4m3(
        _ptr(inp), _ptr(out), n, inv_scale, _stream(stream)))


def quantize_pack_f8e4m3(inp, out_tiles, rows, cols, inv_scale, *, ld=None, out_stride0=None, stream=None):
    """quantize_f16_to_f8e4m3 and the pack of its result into 32x16 left-hand-side
    tiles in one pass (rows past ``rows`` zero); strides default to tight."""
    if ld is None:
        ld = cols
    if out_stride0 is None:
        out_stride0 = cols * 32
    _check(load_library().iree_amd_uk_quantize_pack_f8e4m3(
        _ptr(inp), ld, _ptr(out_tiles), out_stride0, rows, cols, inv_scale, _stream(stream)))


def silu_mul_quantize(gate, up, out, rows, cols, ld, gate_scale, up_scale,
                      inv_out_scale, stream=None):
    _check(load_library().iree_amd_uk_silu_mul_quantize(
        _ptr(gate), _ptr(up), _ptr(out), rows, cols, ld, gate_scale, up_scale,
        inv_out_scale, _stream(stream)))


def silu_mul_quantize_tiled(acc, acc_stride0, gate_tile0, up_tile0, out, out_stride0,
                            M1, N1, gate_scale, up_scale, inv_out_scale, stream=None):
    _check(load_library().iree_amd_uk_silu_mul_quantize_tiled(
        _ptr(acc), acc_stride0, gate_tile0, up_tile0, _ptr(out), out_stride0, M1, N1,
        gate_scale, up_scale, inv_out_scale, _stream(stream)))


def mmt4d_silu_mul_f8e4m3(lhs_buffer, rhs_buffer, out_buffer, M, N, K, K0, flags,
                          gate_scale, up_scale, inv_out_scale, *, lhs_offset=0,
                          lhs_stride0=None, rhs_offset=0, rhs_stride0=None, out_offset=0,
                          out_stride0=None, stream=None):
    """mmt4d over interleaved gate/up right-hand-side tiles with the SiLU * up
    product quantised to e4m3 in the epilogue (see include/iree_amd_uk.h)."""
    if lhs_stride0 is None:
        lhs_stride0 = K * 32 * K0
    if rhs_stride0 is None:
        rhs_stride0 = K * 32 * K0
    if out_stride0 is None:
        out_stride0 = N // 2 * 1024
    _check(load_library().iree_amd_uk_mmt4d_silu_mul_f8e4m3(
        _ptr(lhs_buffer), lhs_offset, lhs_stride0, _ptr(rhs_buffer), rhs_offset, rhs_stride0,
        _ptr(out_buffer), out_offset, out_stride0, M, N, K, K0, flags,
        gate_scale, up_scale, inv_out_scale, _stream(stream)))


def mmt4d_unpack(lhs_buffer, rhs_buffer, out_buffer, out_size0, out_size1, M, N, K, K0, flags, *,
                 lhs_offset=0, lhs_stride0=None, rhs_offset=0, rhs_stride0=None, out_offset=0,
                 out_stride0=None, out_scale=1.0, stream=None):
    """mmt4d (tiles 32x32xK0) whose result is written / accumulated as the
    row-major ``out_size0`` x ``out_size1`` matrix an unpack would produce,
    float results times ``out_scale``."""
    if lhs_stride0 is None:
        lhs_stride0 = K * 32 * K0
    if rhs_stride0 is None:
        rhs_stride0 = K * 32 * K0
    if out_stride0 is None:
        out_stride0 = out_size1
    _check(load_library().iree_amd_uk_mmt4d_unpack(
        _ptr(lhs_buffer), lhs_offset, lhs_stride0, _ptr(rhs_buffer), rhs_offset, rhs_stride0,
        _ptr(out_buffer), out_offset, out_stride0, out_size0, out_size1, M, N, K, K0, flags,
        out_scale, _stream(stream)))


def matmul_packed_rhs(lhs, rhs_packed, out, M, N, K, K0, flags, *, lhs_offset=0, lhs_stride0=None,
                      rhs_offset=0, rhs_stride0=None, out_offset=0, out_stride0=None, out_scale=1.0,
                      stream=None):
    """Row-major ``out[M][N] (+)= lhs[M][K] * rhs`` with ``rhs`` already packed
    into 32 x K0 tiles: pack(LHS), mmt4d and unpack in one kernel. M, N, K are
    element counts."""
    if lhs_stride0 is None:
        lhs_stride0 = K
    if rhs_stride0 is None:
        rhs_stride0 = K * 32
    if out_stride0 is None:
        out_stride0 = N
    _check(load_library().iree_amd_uk_matmul_packed_rhs(
        _ptr(lhs), lhs_offset, lhs_stride0, _ptr(rhs_packed), rhs_offset, rhs_stride0,
        _ptr(out), out_offset, out_stride0, M, N, K, K0, flags, out_scale, _stream(stream)))


def batch_mmt4d_unpack(lhs_buffer, rhs_buffer, out_buffer, batch, out_size0, out_size1, M, N, K, K0, flags, *,
                       lhs_offset=0, lhs_stride0=None, rhs_offset=0, rhs_stride0=None, out_offset=0,
                       out_stride0=None, lhs_batch_stride=None, rhs_batch_stride=None,
                       out_batch_stride=None, out_scale=1.0, stream=None):
    """``batch`` problems of ``mmt4d_unpack`` in one launch; strides default to tight."""
    if lhs_stride0 is None:
        lhs_stride0 = K * 32 * K0
    if rhs_stride0 is None:
        rhs_stride0 = K * 32 * K0
    if out_stride0 is None:
        out_stride0 = out_size1
    if lhs_batch_stride is None:
        lhs_batch_stride = M * lhs_stride0
    if rhs_batch_stride is None:
        rhs_batch_stride = N * rhs_stride0
    if out_batch_stride is None:
        out_batch_stride = out_size0 * out_stride0
    _check(load_library().iree_amd_uk_batch_mmt4d_unpack(
        _ptr(lhs_buffer), lhs_offset, lhs_stride0, _ptr(rhs_buffer), rhs_offset, rhs_stride0,
        _ptr(out_buffer), out_offset, out_stride0, out_size0, out_size1, M, N, K, K0, flags,
        out_scale, batch, lhs_batch_stride, rhs_batch_stride, out_batch_stride, _stream(stream)))


def batch_matmul_packed_rhs(lhs, rhs_packed, out, batch, M, N, K, K0, flags, *, lhs_offset=0,
                            lhs_stride0=None, rhs_offset=0, rhs_stride0=None, out_offset=0,
                            out_stride0=None, lhs_batch_stride=None, rhs_batch_stride=None,
                            out_batch_stride=None, out_scale=1.0, stream=None):
    """``batch`` problems of ``matmul_packed_rhs`` in one launch; strides default
    to tight (``rhs_batch_stride=0`` shares one packed right-hand side)."""
    if lhs_stride0 is None:
        lhs_stride0 = K
    if rhs_stride0 is None:
        rhs_stride0 = K * 32
    if out_stride0 is None:
        out_stride0 = N
    if lhs_batch_stride is None:
        lhs_batch_stride = M * lhs_stride0
    if rhs_batch_stride is None:
        rhs_batch_stride = -(-N // 32) * rhs_stride0
    if out_batch_stride is None:
        out_batch_stride = M * out_stride0
    _check(load_library().iree_amd_uk_batch_matmul_packed_rhs(
        _ptr(lhs), lhs_offset, lhs_stride0, _ptr(rhs_packed), rhs_offset, rhs_stride0,
        _ptr(out), out_offset, out_stride0, M, N, K, K0, flags, out_scale, batch,
        lhs_batch_stride, rhs_batch_stride, out_batch_stride, _stream(stream)))


def scale_f32(buf, n, scale, stream=None):
    _check(load_library().iree_amd_uk_scale_f32(_ptr(buf), n, scale, _stream(stream)))


def mfma_probe(type_flag, operands, iters, sink, stream=None):
    """Register-only matrix-core loop on the bit content of ``operands`` (at
    least 64 KiB); returns the operation count (2 per multiply-add) of the
    launch. A measurement aid, not part of the reference's interface."""
    ops = C.c_int64(0)
    _check(load_library().iree_amd_uk_mfma_probe(type_flag, _ptr(operands), iters, _ptr(sink),
                                                 C.byref(ops), _stream(stream)))
    return ops.value


def copy_probe(src, dst, nbytes, mode=0, blocks_per_cu=0, stream=None):
    """Plain out-of-place copy of ``nbytes`` (whole 8 KiB chunks): the yardstick
    for the pack / unpack streams; modes 2 and 3 only read (the yardstick for
    the weight-streaming kernels). A measurement aid, not part of the
    reference's interface."""
    _check(load_library().iree_amd_uk_copy_probe(_ptr(src), _ptr(dst), nbytes, mode, blocks_per_cu,
                                                 _stream(stream)))


# ---------------------------------------------------------------------------
# The reference's end-to-end chain: pack LHS, pack RHS (inner+outer transposed),
# [pack accumulator], mmt4d, unpack
# (runtime/src/iree/builtins/ukernel/tools/e2e_matmul_benchmark.c:173-186,
# parameters built as at :208-285).
# ---------------------------------------------------------------------------

_MMT4D_TO_QUERY_OP = {
    F.MMT4D_TYPE_F32F32F32: F.QUERY_OP_MATMUL_F32F32F32,
    F.MMT4D_TYPE_S8S8S32: F.QUERY_OP_MATMUL_I8I8I32,
    F.MMT4D_TYPE_F16F16F32: F.QUERY_OP_MATMUL_F16F16F32,
    F.MMT4D_TYPE_F16F16F16: F.QUERY_OP_MATMUL_F16F16F16,
    F.MMT4D_TYPE_BF16BF16F32: F.QUERY_OP_MATMUL_BF16BF16F32,
    F.MMT4D_TYPE_BF16BF16BF16: F.QUERY_OP_MATMUL_BF16BF16BF16,
    F.MMT4D_TYPE_F8E4M3F8E4M3F32: F.QUERY_OP_MATMUL_F8E4M3F8E4M3F32,
}
_IN_PACK_TYPE = {
    F.MMT4D_TYPE_F32F32F32: F.PACK_TYPE_F32F32,
    F.MMT4D_TYPE_S8S8S32: F.PACK_TYPE_I8I8,
    F.MMT4D_TYPE_F16F16F32: F.PACK_TYPE_F16F16,
    F.MMT4D_TYPE_F16F16F16: F.PACK_TYPE_F16F16,
    F.MMT4D_TYPE_BF16BF16F32: F.PACK_TYPE_BF16BF16,
    F.MMT4D_TYPE_BF16BF16BF16: F.PACK_TYPE_BF16BF16,
    F.MMT4D_TYPE_F8E4M3F8E4M3F32: F.PACK_TYPE_I8I8,
}
_OUT_PACK_TYPE = {
    F.MMT4D_TYPE_F32F32F32: F.PACK_TYPE_F32F32,
    F.MMT4D_TYPE_S8S8S32: F.PACK_TYPE_I32I32,
    F.MMT4D_TYPE_F16F16F32: F.PACK_TYPE_F32F32,
    F.MMT4D_TYPE_F16F16F16: F.PACK_TYPE_F16F16,
    F.MMT4D_TYPE_BF16BF16F32: F.PACK_TYPE_F32F32,
    F.MMT4D_TYPE_BF16BF16BF16: F.PACK_TYPE_BF16BF16,
    F.MMT4D_TYPE_F8E4M3F8E4M3F32: F.PACK_TYPE_F32F32,
}


def _ceil_div(a, b):
    return -(-a // b)


def matmul_data_tiled(a, b, c, M, N, K, mmt4d_type, *, accumulate=False,
                      tile=None, workspace=None, fuse_unpack=False, fuse_pack_lhs=False):
    """Row-major C[M][N] (+)= A[M][K] * B[K][N] through pack -> mmt4d -> unpack.
    With ``fuse_unpack`` the last two (and the pack of C when accumulating) are
    the one kernel ``mmt4d_unpack``; it needs a tile with a matrix-core kernel.
    With ``fuse_pack_lhs`` the matmul also reads A row-major itself
    (``matmul_packed_rhs``): the chain is the pack of B and one matmul launch;
    K must then be whole matrix-core steps.

    ``a``/``b``/``c`` are flat CUDA tensors holding the row-major matrices with
    the element types of ``mmt4d_type``. ``tile`` = (M0, N0, K0); by default the
    tile the library's query_matmul_tile_sizes reports for these static sizes
    (narrow for M or N below 32), with ``"dynamic"`` the one for unknown sizes. ``workspace`` may
    carry pre-allocated packed buffers as a dict {"lhs","rhs","out"}.
    Returns the dict of packed buffers used (so callers can reuse them).
    """
    if tile is None:
        M0, N0, K0 = query_matmul_tile_sizes(_MMT4D_TO_QUERY_OP[mmt4d_type], M, N, K)
    elif tile == "dynamic":
        # (the tile of a matmul whose sizes the compiler did not know)
        M0, N0, K0 = query_matmul_tile_sizes(_MMT4D_TO_QUERY_OP[mmt4d_type])
    else:
        M0, N0, K0 = tile
    M1, N1, K1 = _ceil_div(M, M0), _ceil_div(N, N0), _ceil_div(K, K0)
    in_type = _IN_PACK_TYPE[mmt4d_type]
    out_type = _OUT_PACK_TYPE[mmt4d_type]
    ws = workspace if workspace is not None else {}
    fuse_unpack = fuse_unpack or fuse_pack_lhs
    if "lhs" not in ws and not fuse_pack_lhs:
        ws["lhs"] = torch.empty(M1 * K1 * M0 * K0, dtype=a.dtype, device=a.device)
    if "rhs" not in ws:
        ws["rhs"] = torch.empty(N1 * K1 * N0 * K0, dtype=b.dtype, device=b.device)
    if "out" not in ws and not fuse_unpack:
        ws["out"] = torch.empty(M1 * N1 * M0 * N0, dtype=c.dtype, device=c.device)
    if not fuse_pack_lhs:
        pack(a, ws["lhs"], M, K, M1, K1, M0, K0, 0, in_type)
    pack(b, ws["rhs"], K, N, N1, K1, N0, K0, 0,
         in_type | F.PACK_TRANSPOSE_INNER | F.PACK_TRANSPOSE_OUTER)
    mm_flags = mmt4d_type | F.MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION | \
        F.MMT4D_SKIP_INTERMEDIATE_ROUNDINGS
    if fuse_pack_lhs:
        if (M0, N0) != (32, 32) or K % K0:
            raise ValueError("fuse_pack_lhs needs 32x32 tiles and K in whole tiles")
        if accumulate:
            mm_flags |= F.MMT4D_ACCUMULATE
        matmul_packed_rhs(a, ws["rhs"], c, M, N, K, K0, mm_flags)
        return ws
    if fuse_unpack:
        if (M0, N0) != (32, 32):
            raise ValueError("fuse_unpack needs 32x32 tiles")
        if accumulate:
            mm_flags |= F.MMT4D_ACCUMULATE
        mmt4d_unpack(ws["lhs"], ws["rhs"], c, M, N, M1, N1, K1, K0, mm_flags)
        return ws
    if accumulate:
        pack(c, ws["out"], M, N, M1, N1, M0, N0, 0, out_type)
        mm_flags |= F.MMT4D_ACCUMULATE
    mmt4d(ws["lhs"], ws["rhs"], ws["out"], M1, N1, K1, M0, N0, K0, mm_flags)
    unpack(ws["out"], c, M1, N1, M0, N0, M, N, out_type)
    return ws


class Fp8Mlp:
    """Llama-style MLP block ``y = (silu(x Wg^T) * (x Wu^T)) Wd^T`` on fp8 e4m3
    operands with per-tensor f32 scales, as the chain of dispatches the
    reference's patterns give (gate and up fused horizontally into one matmul,
    compiler/src/iree/compiler/GlobalOptimization/FuseSiluHorizontalMatmul.cpp:113-140):

        quantize x -> pack LHS -> mmt4d [gate|up] -> silu*up -> fp8 LHS tiles
        -> mmt4d down -> unpack -> scale

    With ``fused`` (the default) the gate/up matmul and the SiLU * up step are one
    kernel (``mmt4d_silu_mul_f8e4m3``) and the f32 gate/up values never reach memory.

    Weights arrive as e4m3 bytes, row-major ``[N][K]`` (the transpose_b form),
    and are packed once into right-hand-side tiles 32x16. ``sx``/``sh`` are the
    static activation scales (value = code * scale), ``sg``/``su``/``sd`` the
    weight scales. M, hidden and ffn must be multiples of 32.
    """

    def __init__(self, hidden, ffn, wg_q, wu_q, wd_q, sg, su, sd, sx, sh, max_tokens, fused=True):
        if hidden % 32 or ffn % 32 or max_tokens % 32:
            raise ValueError("hidden, ffn and max_tokens must be multiples of 32")
        self.hidden, self.ffn, self.max_tokens, self.fused = hidden, ffn, max_tokens, fused
        self.sg, self.su, self.sd, self.sx, self.sh = sg, su, sd, sx, sh
        dev = wg_q.device
        u8 = torch.uint8
        t = F.PACK_TYPE_I8I8
        self.wgu = torch.empty(2 * ffn * hidden, dtype=u8, device=dev)
        F1, H1 = ffn // 32, hidden // 32
        row = hidden * 32          # bytes of one outer row of right-hand-side tiles
        if fused:
            # gate tile row j at outer row 2j, up tile row j at 2j + 1
            pack(wg_q, self.wgu, ffn, hidden, F1, hidden // 16, 32, 16, 0, t, out_stride0=2 * row)
            pack(wu_q, self.wgu, ffn, hidden, F1, hidden // 16, 32, 16, 0, t, out_stride0=2 * row,
                 out_offset=row)
        else:
            # gate tiles occupy outer rows [0, F1), up tiles [F1, 2 F1)
            pack(wg_q, self.wgu, ffn, hidden, F1, hidden // 16, 32, 16, 0, t)
            pack(wu_q, self.wgu, ffn, hidden, F1, hidden // 16, 32, 16, 0, t,
                 out_offset=ffn * hidden)
        self.wd = torch.empty(hidden * ffn, dtype=u8, device=dev)
        pack(wd_q, self.wd, hidden, ffn, H1, ffn // 16, 32, 16, 0, t)
        M = max_tokens
        self.xq = torch.empty(M * hidden, dtype=u8, device=dev)
        self.x_tiles = torch.empty(M * hidden, dtype=u8, device=dev)
        self.acc = None if fused else torch.empty(M * 2 * ffn, dtype=torch.float32, device=dev)
        self.h_tiles = torch.empty(M * ffn, dtype=u8, device=dev)
        self.acc2 = torch.empty(M * hidden, dtype=torch.float32, device=dev)

    def __call__(self, x_f16, y_f32, M):
        hidden, ffn = self.hidden, self.ffn
        if M % 32 or M > self.max_tokens:
            raise ValueError("M must be a multiple of 32 within max_tokens")
        M1, F1, H1 = M // 32, ffn // 32, hidden // 32
        mm = F.MMT4D_TYPE_F8E4M3F8E4M3F32
        if self.fused:
            quantize_pack_f8e4m3(x_f16, self.x_tiles, M, hidden, 1.0 / self.sx)
        else:
            quantize_f16_to_f8e4m3(x_f16, self.xq, M * hidden, 1.0 / self.sx)
            pack(self.xq, self.x_tiles, M, hidden, M1, hidden // 16, 32, 16, 0, F.PACK_TYPE_I8I8)
        if self.fused:
            mmt4d_silu_mul_f8e4m3(self.x_tiles, self.wgu, self.h_tiles, M1, 2 * F1, hidden // 16, 16, mm,
                                  self.sx * self.sg, self.sx * self.su, 1.0 / self.sh)
        else:
            mmt4d(self.x_tiles, self.wgu, self.acc, M1, 2 * F1, hidden // 16, 32, 32, 16, mm)
            silu_mul_quantize_tiled(self.acc, 2 * F1 * 1024, 0, F1, self.h_tiles, ffn * 32, M1, F1,
                                    self.sx * self.sg, self.sx * self.su, 1.0 / self.sh)
        if self.fused:
            mmt4d_unpack(self.h_tiles, self.wd, y_f32, M, hidden, M1, H1, ffn // 16, 16, mm,
                         out_scale=self.sh * self.sd)
        else:
            mmt4d(self.h_tiles, self.wd, self.acc2, M1, H1, ffn // 16, 32, 32, 16, mm)
            unpack(self.acc2, y_f32, M1, H1, 32, 32, M, hidden, F.UNPACK_TYPE_F32F32)
            scale_f32(y_f32, M * hidden, self.sh * self.sd)
