"""ctypes binding of the C-ABI library declared in include/iree_amd_uk.h.

The library must have been built (``python -m iree_amd.build`` or
``__graft_entry__.build()``); there is no fallback of any kind: a missing or
stale library raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_NAME = "libiree_amd_uk.so"
_lib = None

index_t = C.c_int64


class Mmt4dParams(C.Structure):
    """iree_amd_uk_mmt4d_params_t (same field order as the reference's
    runtime/src/iree/builtins/ukernel/mmt4d_internal.h:14-32)."""

    _fields_ = [
        ("lhs_buffer", C.c_void_p), ("lhs_offset", index_t), ("lhs_stride0", index_t),
        ("rhs_buffer", C.c_void_p), ("rhs_offset", index_t), ("rhs_stride0", index_t),
        ("out_buffer", C.c_void_p), ("out_offset", index_t), ("out_stride0", index_t),
        ("M", index_t), ("N", index_t), ("K", index_t),
        ("M0", C.c_int32), ("N0", C.c_int32), ("K0", C.c_int32),
        ("flags", C.c_uint32), ("cpu_data", C.c_void_p),
    ]


class PackParams(C.Structure):
    """iree_amd_uk_pack_params_t (reference pack_internal.h:12-30)."""

    _fields_ = [
        ("in_buffer", C.c_void_p), ("in_offset", index_t),
        ("in_stride0", index_t), ("in_stride1", index_t),
        ("out_buffer", C.c_void_p), ("out_offset", index_t),
        ("out_stride0", index_t), ("out_stride1", index_t),
        ("in_size0", index_t), ("in_size1", index_t),
        ("out_size0", index_t), ("out_size1", index_t),
        ("out_size2", index_t), ("out_size3", index_t),
        ("padding_value", C.c_uint64), ("flags", C.c_uint32),
        ("cpu_data", C.c_void_p),
    ]


class UnpackParams(C.Structure):
    """iree_amd_uk_unpack_params_t (reference unpack_internal.h:12-29)."""

    _fields_ = [
        ("in_buffer", C.c_void_p), ("in_offset", index_t),
        ("in_stride0", index_t), ("in_stride1", index_t),
        ("out_buffer", C.c_void_p), ("out_offset", index_t),
        ("out_stride0", index_t), ("out_stride1", index_t),
        ("in_size0", index_t), ("in_size1", index_t),
        ("in_size2", index_t), ("in_size3", index_t),
        ("out_size0", index_t), ("out_size1", index_t),
        ("flags", C.c_uint32), ("cpu_data", C.c_void_p),
    ]


class MatmulTile(C.Structure):
    """iree_amd_uk_matmul_tile_t."""
    _fields_ = [("M", C.c_int32), ("N", C.c_int32), ("K", C.c_int32)]


class QueryParams(C.Structure):
    _fields_ = [("flags", C.c_uint32), ("size0", index_t), ("size1", index_t),
                ("cpu_data", C.c_void_p)]


class QueryOutParams(C.Structure):
    _fields_ = [("tile_size0", index_t), ("tile_size1", index_t)]


def library_path():
    """The built library; IREE_AMD_UK_LIBRARY (the variable the HAL plugin reads
    as well) names another build of it."""
    return os.environ.get("IREE_AMD_UK_LIBRARY") or os.path.join(_HERE, "csrc", _LIB_NAME)


def _declare(lib):
    vp, i64, i32, u32, u64 = C.c_void_p, C.c_int64, C.c_int32, C.c_uint32, C.c_uint64
    lib.iree_amd_uk_mmt4d.restype = C.c_int
    lib.iree_amd_uk_mmt4d.argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i64,
                                       i64, i64, i64, i32, i32, i32, u32, vp, vp]
    lib.iree_amd_uk_mmt4d_p.restype = C.c_int
    lib.iree_amd_uk_mmt4d_p.argtypes = [C.POINTER(Mmt4dParams), vp]
    lib.iree_amd_uk_mmt4d_noalloc_p.restype = C.c_int
    lib.iree_amd_uk_mmt4d_noalloc_p.argtypes = [C.POINTER(Mmt4dParams), vp]
    lib.iree_amd_uk_batch_mmt4d.restype = C.c_int
    lib.iree_amd_uk_batch_mmt4d.argtypes = [C.POINTER(Mmt4dParams), i64, i64, i64, i64, vp]
    lib.iree_amd_uk_mmt4d_info.restype = u32
    lib.iree_amd_uk_mmt4d_info.argtypes = [i32, i32, i32, u32, vp]
    lib.iree_amd_uk_pack.restype = C.c_int
    lib.iree_amd_uk_pack.argtypes = [vp, i64, i64, i64, vp, i64, i64, i64,
                                      i64, i64, i64, i64, i64, i64, u64, u32, vp, vp]
    lib.iree_amd_uk_pack_p.restype = C.c_int
    lib.iree_amd_uk_pack_p.argtypes = [C.POINTER(PackParams), vp]
    lib.iree_amd_uk_unpack.restype = C.c_int
    lib.iree_amd_uk_unpack.argtypes = [vp, i64, i64, i64, vp, i64, i64, i64,
                                        i64, i64, i64, i64, i64, i64, u32, vp, vp]
    lib.iree_amd_uk_unpack_p.restype = C.c_int
    lib.iree_amd_uk_unpack_p.argtypes = [C.POINTER(UnpackParams), vp]
    lib.iree_amd_uk_enumerate_matmul_tiles.restype = C.c_int
    lib.iree_amd_uk_enumerate_matmul_tiles.argtypes = [C.c_uint32, C.POINTER(MatmulTile), C.c_int32,
                                                       C.POINTER(C.c_int32)]
    lib.iree_amd_uk_choose_matmul_tile.restype = C.c_int
    lib.iree_amd_uk_choose_matmul_tile.argtypes = [C.POINTER(MatmulTile), C.c_int32, i64, i64,
                                                   C.POINTER(C.c_int64), C.POINTER(MatmulTile)]
    lib.iree_amd_uk_query_matmul_tile_sizes.restype = C.c_int
    lib.iree_amd_uk_query_matmul_tile_sizes.argtypes = [C.c_uint32, i64, i64, i64, C.POINTER(MatmulTile)]
    lib.iree_amd_uk_query_tile_sizes_2d.restype = C.c_int
    lib.iree_amd_uk_query_tile_sizes_2d.argtypes = [C.POINTER(QueryParams),
                                                     C.POINTER(QueryOutParams)]
    lib.iree_amd_uk_dequant_matmul_i4.restype = C.c_int
    lib.iree_amd_uk_dequant_matmul_i4.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64,
                                                   i64, u32, vp]
    lib.iree_amd_uk_quantize_groups_i16.restype = C.c_int
    lib.iree_amd_uk_quantize_groups_i16.argtypes = [vp, vp, vp, vp, i64, i64, i64, vp]
    lib.iree_amd_uk_pack_i4_weights.restype = C.c_int
    lib.iree_amd_uk_pack_i4_weights.argtypes = [vp, vp, i64, i64, vp]
    lib.iree_amd_uk_quantize_f16_to_f8e4m3.restype = C.c_int
    lib.iree_amd_uk_quantize_f16_to_f8e4m3.argtypes = [vp, vp, i64, C.c_float, vp]
    lib.iree_amd_uk_quantize_pack_f8e4m3.restype = C.c_int
    lib.iree_amd_uk_quantize_pack_f8e4m3.argtypes = [vp, i64, vp, i64, i64, i64, C.c_float, vp]
    lib.iree_amd_uk_silu_mul_quantize.restype = C.c_int
    lib.iree_amd_uk_silu_mul_quantize.argtypes = [vp, vp, vp, i64, i64, i64,
                                                   C.c_float, C.c_float, C.c_float, vp]
    lib.iree_amd_uk_silu_mul_quantize_tiled.restype = C.c_int
    lib.iree_amd_uk_silu_mul_quantize_tiled.argtypes = [vp, i64, i64, i64, vp, i64, i64, i64,
                                                         C.c_float, C.c_float, C.c_float, vp]
    lib.iree_amd_uk_mmt4d_silu_mul_f8e4m3.restype = C.c_int
    lib.iree_amd_uk_mmt4d_silu_mul_f8e4m3.argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i64,
                                                       i64, i64, i64, i32, u32,
                                                       C.c_float, C.c_float, C.c_float, vp]
    lib.iree_amd_uk_mmt4d_unpack.restype = C.c_int
    lib.iree_amd_uk_mmt4d_unpack.argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i64, i64, i64,
                                             i64, i64, i64, C.c_int32, C.c_uint32, C.c_float, vp]
    lib.iree_amd_uk_matmul_packed_rhs.restype = C.c_int
    lib.iree_amd_uk_matmul_packed_rhs.argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i64,
                                                  i64, i64, i64, C.c_int32, C.c_uint32, C.c_float, vp]
    lib.iree_amd_uk_batch_mmt4d_unpack.restype = C.c_int
    lib.iree_amd_uk_batch_mmt4d_unpack.argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i64, i64, i64,
                                                   i64, i64, i64, C.c_int32, C.c_uint32, C.c_float,
                                                   i64, i64, i64, i64, vp]
    lib.iree_amd_uk_batch_matmul_packed_rhs.restype = C.c_int
    lib.iree_amd_uk_batch_matmul_packed_rhs.argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i64,
                                                        i64, i64, i64, C.c_int32, C.c_uint32, C.c_float,
                                                        i64, i64, i64, i64, vp]
    lib.iree_amd_uk_scale_f32.restype = C.c_int
    lib.iree_amd_uk_scale_f32.argtypes = [vp, i64, C.c_float, vp]
    lib.iree_amd_uk_mfma_probe.restype = C.c_int
    lib.iree_amd_uk_mfma_probe.argtypes = [C.c_uint32, vp, i64, vp, C.POINTER(C.c_int64), vp]
    lib.iree_amd_uk_copy_probe.restype = C.c_int
    lib.iree_amd_uk_copy_probe.argtypes = [vp, vp, i64, i32, i32, vp]
    lib.iree_amd_uk_device_count.restype = C.c_int
    lib.iree_amd_uk_device_count.argtypes = [C.POINTER(C.c_int)]
    lib.iree_amd_uk_device_set.restype = C.c_int
    lib.iree_amd_uk_device_set.argtypes = [C.c_int]
    lib.iree_amd_uk_device_malloc.restype = C.c_int
    lib.iree_amd_uk_device_malloc.argtypes = [C.POINTER(vp), u64]
    lib.iree_amd_uk_device_free.restype = C.c_int
    lib.iree_amd_uk_device_free.argtypes = [vp]
    lib.iree_amd_uk_memcpy_h2d.restype = C.c_int
    lib.iree_amd_uk_memcpy_h2d.argtypes = [vp, vp, u64, vp]
    lib.iree_amd_uk_memcpy_d2h.restype = C.c_int
    lib.iree_amd_uk_memcpy_d2h.argtypes = [vp, vp, u64, vp]
    lib.iree_amd_uk_stream_create.restype = C.c_int
    lib.iree_amd_uk_stream_create.argtypes = [C.POINTER(vp)]
    lib.iree_amd_uk_stream_destroy.restype = C.c_int
    lib.iree_amd_uk_stream_destroy.argtypes = [vp]
    lib.iree_amd_uk_stream_synchronize.restype = C.c_int
    lib.iree_amd_uk_stream_synchronize.argtypes = [vp]
    lib.iree_amd_uk_release_scratch.restype = C.c_int
    lib.iree_amd_uk_release_scratch.argtypes = []
    lib.iree_amd_uk_last_kernel_path.restype = C.c_char_p
    lib.iree_amd_uk_last_kernel_path.argtypes = []
    lib.iree_amd_uk_last_error.restype = C.c_char_p
    lib.iree_amd_uk_last_error.argtypes = []
    lib.iree_amd_uk_version.restype = u32
    lib.iree_amd_uk_version.argtypes = []
    lib.iree_amd_uk_host_pool_create.restype = C.c_int
    lib.iree_amd_uk_host_pool_create.argtypes = [C.POINTER(vp)]
    lib.iree_amd_uk_host_pool_destroy.restype = None
    lib.iree_amd_uk_host_pool_destroy.argtypes = [vp]
    lib.iree_amd_uk_mmt4d_host_pooled.restype = C.c_int
    lib.iree_amd_uk_mmt4d_host_pooled.argtypes = [vp, C.POINTER(Mmt4dParams)]
    lib.iree_amd_uk_pack_host_pooled.restype = C.c_int
    lib.iree_amd_uk_pack_host_pooled.argtypes = [vp, C.POINTER(PackParams)]
    lib.iree_amd_uk_unpack_host_pooled.restype = C.c_int
    lib.iree_amd_uk_unpack_host_pooled.argtypes = [vp, C.POINTER(UnpackParams)]
    lib.iree_amd_uk_mmt4d_host.restype = C.c_int
    lib.iree_amd_uk_mmt4d_host.argtypes = [C.POINTER(Mmt4dParams)]
    lib.iree_amd_uk_pack_host.restype = C.c_int
    lib.iree_amd_uk_pack_host.argtypes = [C.POINTER(PackParams)]
    lib.iree_amd_uk_unpack_host.restype = C.c_int
    lib.iree_amd_uk_unpack_host.argtypes = [C.POINTER(UnpackParams)]
    # include/iree_amd_hal_executable.h
    lib.iree_amd_hal_executable_load.restype = C.c_int
    lib.iree_amd_hal_executable_load.argtypes = [vp, C.c_size_t, C.POINTER(vp)]
    lib.iree_amd_hal_executable_add_export.restype = C.c_int
    lib.iree_amd_hal_executable_add_export.argtypes = [vp, C.c_char_p, u32, u32, u32, u32,
                                                       C.POINTER(i32)]
    lib.iree_amd_hal_executable_dispatch.restype = C.c_int
    lib.iree_amd_hal_executable_dispatch.argtypes = [vp, i32, u32, u32, u32, C.POINTER(vp),
                                                     C.c_size_t, C.POINTER(u32), C.c_size_t, vp]
    lib.iree_amd_hal_executable_release.restype = None
    lib.iree_amd_hal_executable_release.argtypes = [vp]


def load_library():
    """Returns the loaded C-ABI library; raises if it has not been built."""
    global _lib
    if _lib is None:
        path = library_path()
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} is missing: the HIP extension has not been built "
                "(run `python -m iree_amd.build`). There is no CPU fallback.")
        lib = C.CDLL(path)
        _declare(lib)
        _lib = lib
    return _lib
