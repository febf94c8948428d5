"""MI355X (gfx950) implementation of IREE's data-tiled matmul microkernels.

The product is the C-ABI shared library built from ``iree_amd/csrc`` (declared in
``include/iree_amd_uk.h``). This package is the thin Python host mirror of the
reference's ukernel entry points (``iree_uk_pack`` / ``iree_uk_mmt4d`` /
``iree_uk_unpack`` / ``iree_uk_query_tile_sizes_2d``) over that library; torch is
used only to own device memory and streams.
"""
from . import flags  # noqa: F401
from ._lib import load_library, library_path  # noqa: F401
from .ukernel import (  # noqa: F401
    Fp8Mlp,
    UkError,
    dequant_matmul_i4,
    matmul_data_tiled,
    matmul_packed_rhs,
    mfma_probe,
    quantize_groups_i16,
    copy_probe,
    batch_matmul_packed_rhs,
    choose_matmul_tile,
    enumerate_matmul_tiles,
    last_kernel_path,
    batch_mmt4d,
    batch_mmt4d_unpack,
    mmt4d,
    mmt4d_info,
    mmt4d_silu_mul_f8e4m3,
    mmt4d_unpack,
    pack,
    pack_i4_weights,
    quantize_f16_to_f8e4m3,
    quantize_pack_f8e4m3,
    query_matmul_tile_sizes,
    query_tile_sizes_2d,
    scale_f32,
    silu_mul_quantize,
    silu_mul_quantize_tiled,
    unpack,
)
