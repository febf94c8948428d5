"""The mmt4d, pack and unpack kernels as a HAL executable object for a HIP device.

``iree_amd/hal/mi355x_kernels.hip`` builds into ``mi355x_kernels_gfx950.co``: a
code object of ``extern "C"`` kernels that IREE links into a
``hal.executable.source`` (reference
samples/custom_dispatch/hip/kernels/example.mlir:36-118). This module holds the
table of its exports (what the ``hal.executable.export`` ops must declare),
writes that MLIR, and loads and dispatches the object the way the HIP HAL
driver does (runtime/src/iree/hal/drivers/hip/native_executable.c:180-253,
stream_command_buffer.c:519-581) through the C-ABI of
``include/iree_amd_hal_executable.h`` - which is how the tests run it without
an IREE runtime.
"""
import ctypes as C
import os
from collections import namedtuple

from . import flags as F
from ._lib import load_library
from .ukernel import _check, _ptr, _stream

HERE = os.path.dirname(os.path.abspath(__file__))
CODE_OBJECT = os.path.join(HERE, "hal", "mi355x_kernels_gfx950.co")
WORKGROUP_SIZE = 256

# name: element-type tuple of the reference's flag enum; tile: outer tiles (of
# 32 rows) per workgroup in both directions; lds: workgroup_local_memory in
# bytes; k0: the K0 values served (the first is what the tile-size query answers).
Export = namedtuple("Export", "name type_flag tile lds k0 lhs_bytes out_bytes")


def _exports():
    kib = 1024
    rows = [
        ("f16f16f32", F.MMT4D_TYPE_F16F16F32, 160 * kib, 64 * kib, (8, 16), 2, 4),
        ("bf16bf16f32", F.MMT4D_TYPE_BF16BF16F32, 160 * kib, 64 * kib, (8, 16), 2, 4),
        ("s8s8s32", F.MMT4D_TYPE_S8S8S32, 160 * kib, 64 * kib, (16, 32), 1, 4),
        ("f8e4m3f8e4m3f32", F.MMT4D_TYPE_F8E4M3F8E4M3F32, 160 * kib, 128 * kib, (16,), 1, 4),
        ("f32f32f32", F.MMT4D_TYPE_F32F32F32, 128 * kib, 64 * kib, (4, 8), 4, 4),
    ]
    out = {}
    for name, flag, lds8, lds4, k0, lb, ob in rows:
        for tile, lds in ((8, lds8), (4, lds4)):
            for prefix in ("mi355x_mmt4d_", "mi355x_mmt4d_unpack_"):
                full = f"{prefix}{name}_t{tile}"
                out[full] = Export(full, flag, tile, lds, k0, lb, ob)
    return out


EXPORTS = _exports()

# The whole linear layer on a row-major left-hand side and pre-packed weights:
# name -> (type flag, macro tile in outer tiles (rows, columns), LDS bytes, K0
# served, elements of K per matrix-core step).
MatmulExport = namedtuple("MatmulExport", "name type_flag tile_m tile_n lds k0 mfma_k")


def _matmul_exports():
    kib = 1024
    rows = [("f16f16f32", F.MMT4D_TYPE_F16F16F32, 160 * kib, (8, 16), 32),
            ("bf16bf16f32", F.MMT4D_TYPE_BF16BF16F32, 160 * kib, (8, 16), 32),
            ("s8s8s32", F.MMT4D_TYPE_S8S8S32, 128 * kib, (16, 32), 32),
            ("s8s8s32_k64", F.MMT4D_TYPE_S8S8S32, 160 * kib, (16,), 64),
            ("f8e4m3f8e4m3f32", F.MMT4D_TYPE_F8E4M3F8E4M3F32, 160 * kib, (16,), 64),
            ("f32f32f32", F.MMT4D_TYPE_F32F32F32, 128 * kib, (4, 8), 8)]
    out = {}
    for name, flag, lds8, k0, mk in rows:
        for tm, lds in ((4, 72 * kib), (8, lds8)):
            full = f"mi355x_matmul_packed_rhs_{name}_t{tm}x8"
            out[full] = MatmulExport(full, flag, tm, 8, lds, k0, mk)
    return out


MATMUL_EXPORTS = _matmul_exports()


def matmul_workgroup_count(name, M, N):
    """Grid of a matmul export for an M x N result (elements)."""
    e = MATMUL_EXPORTS[name]
    return -(-(-(-M // 32)) // e.tile_m) * -(-(-(-N // 32)) // e.tile_n)


# pack / unpack without transposes, by element size: name -> (bytes per element,
# True for pack). Any tile size; power-of-two tiles whose rows are whole
# 16-byte chunks run the streaming kernel, others move single elements.
PACK_EXPORTS = {"mi355x_pack_8bit": (1, True), "mi355x_pack_16bit": (2, True),
                "mi355x_pack_32bit": (4, True), "mi355x_unpack_16bit": (2, False),
                "mi355x_unpack_32bit": (4, False)}


# The same with transposed inner tiles (a tile covers tile0 rows x tile1 columns
# of the matrix and is stored column by column): any tile size; power-of-two
# tiles with tile0 * bytes >= 16 move 16-byte chunks, others single elements.
PACK_TRANSPOSE_EXPORTS = {"mi355x_pack_transpose_8bit": (1, True), "mi355x_pack_transpose_16bit": (2, True),
                          "mi355x_pack_transpose_32bit": (4, True),
                          "mi355x_unpack_transpose_16bit": (2, False),
                          "mi355x_unpack_transpose_32bit": (4, False)}


def pack_transpose_workgroup_count(name, size0, size1, tile0, tile1):
    """Grid of a transposing pack / unpack export: blocks of 64 columns x 16
    groups of rows, a group being the 16 / bytes rows of one 16-byte chunk,
    over the padded columns (pack) or the matrix's own (unpack)."""
    es, is_pack = PACK_TRANSPOSE_EXPORTS[name]
    groups = -(-size0 // tile0) * -(-tile0 * es // 16)
    cols = -(-size1 // tile1) * tile1 if is_pack else size1
    return -(-cols // 64) * -(-groups // 16)


def pack_workgroup_count(name, size0, size1, tile0, tile1):
    """Grid of a pack / unpack export: blocks of 16 rows x 32 chunks of 16 bytes
    over the padded extent (pack) or the matrix itself (unpack)."""
    es, is_pack = PACK_EXPORTS[name]
    if is_pack:
        cols = -(-(-(-size1 // tile1) * tile1 * es) // 16)
        rows = -(-size0 // tile0) * tile0
    else:
        cols = -(-size1 * es // 16)
        rows = size0
    return -(-cols // 32) * -(-rows // 16)


# The int4-weight dequantising matmul of the decode step (K = 4096, groups of
# 128, packed uint4 zero points, tiled weights): name -> rows served.
DEQUANT_EXPORTS = {"mi355x_dequant_matmul_i4_k4096_g128_r16": 16,
                   "mi355x_dequant_matmul_i4_k4096_g128_r32": 32}
DEQUANT_WORKGROUP_SIZE = 512
DEQUANT_LDS = 128 * 1024
DEQUANT_MAX_WORKGROUPS = 256


def dequant_workgroup_count(N):
    """Grid of the dequant exports: one workgroup per compute unit at most,
    each walking tiles of 32 columns."""
    return min(N // 32, DEQUANT_MAX_WORKGROUPS)


def workgroup_count(export, M, N):
    """Grid of an export for M x N outer tiles: what its count region returns."""
    t = EXPORTS[export].tile if isinstance(export, str) else export.tile
    return -(-M // t) * -(-N // t)


class HalExecutable:
    """A loaded code object; `dispatch` launches one export."""

    def __init__(self, path=CODE_OBJECT):
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `python -m iree_amd.build`")
        with open(path, "rb") as f:
            self._image = f.read()
        self._lib = load_library()
        handle = C.c_void_p()
        _check(self._lib.iree_amd_hal_executable_load(self._image, len(self._image), C.byref(handle)))
        self._handle = handle
        self._ordinals = {}

    def add_export(self, name, block=(WORKGROUP_SIZE, 1, 1), shared_memory_size=None):
        if shared_memory_size is None:
            shared_memory_size = (0 if name in PACK_EXPORTS or name in PACK_TRANSPOSE_EXPORTS else
                                  DEQUANT_LDS if name in DEQUANT_EXPORTS else
                                  MATMUL_EXPORTS[name].lds if name in MATMUL_EXPORTS else EXPORTS[name].lds)
        if name in DEQUANT_EXPORTS and block == (WORKGROUP_SIZE, 1, 1):
            block = (DEQUANT_WORKGROUP_SIZE, 1, 1)
        ordinal = C.c_int32(-1)
        _check(self._lib.iree_amd_hal_executable_add_export(
            self._handle, name.encode(), block[0], block[1], block[2], shared_memory_size,
            C.byref(ordinal)))
        self._ordinals[name] = ordinal.value
        return ordinal.value

    def dispatch(self, name, workgroups, bindings, push_constants, stream=None):
        """bindings: CUDA tensors (or raw device addresses); push_constants: ints,
        each passed as one 32-bit value."""
        if name not in self._ordinals:
            self.add_export(name)
        if isinstance(workgroups, int):
            workgroups = (workgroups, 1, 1)
        ptrs = (C.c_void_p * max(len(bindings), 1))(
            *[b if isinstance(b, int) else _ptr(b) for b in bindings])
        consts = (C.c_uint32 * max(len(push_constants), 1))(
            *[int(c) & 0xFFFFFFFF for c in push_constants])
        _check(self._lib.iree_amd_hal_executable_dispatch(
            self._handle, self._ordinals[name], workgroups[0], workgroups[1], workgroups[2],
            ptrs, len(bindings), consts, len(push_constants), _stream(stream)))

    def mmt4d(self, name, lhs, rhs, out, M, N, K, K0, flags, out_rows=None, out_cols=None,
              batch=1, stream=None):
        """One mmt4d export over dense operands (see the table in
        iree_amd/hal/mi355x_kernels.hip for the layouts); `batch` problems laid
        one after the other in each binding run as workgroup planes in y."""
        e = EXPORTS[name]
        consts = [M, N, K, K0, flags]
        if "_unpack_" in name:
            consts += [out_rows, out_cols]
        self.dispatch(name, (workgroup_count(e, M, N), batch, 1), [lhs, rhs, out], consts, stream)

    def matmul_packed_rhs(self, name, lhs, rhs_packed, out, M, N, K, K0, flags, stream=None):
        """mi355x_matmul_packed_rhs_*: out[M][N] (+)= lhs[M][K] * rhs, all dense,
        M, N, K in elements."""
        self.dispatch(name, matmul_workgroup_count(name, M, N), [lhs, rhs_packed, out],
                      [M, N, K, K0, flags], stream)

    def pack(self, name, matrix, tiles, size0, size1, tile0, tile1, padding=0, stream=None):
        """mi355x_pack_*: matrix (size0 x size1, dense) -> tiles; `padding` is the
        bit pattern of the padding element."""
        assert PACK_EXPORTS[name][1]
        self.dispatch(name, pack_workgroup_count(name, size0, size1, tile0, tile1), [matrix, tiles],
                      [size0, size1, tile0, tile1, padding], stream)

    def unpack(self, name, tiles, matrix, size0, size1, tile0, tile1, stream=None):
        """mi355x_unpack_*: tiles -> matrix (size0 x size1, dense)."""
        assert not PACK_EXPORTS[name][1]
        self.dispatch(name, pack_workgroup_count(name, size0, size1, tile0, tile1), [tiles, matrix],
                      [size0, size1, tile0, tile1], stream)

    def pack_transpose(self, name, matrix, tiles, size0, size1, tile0, tile1, padding=0, stream=None):
        """mi355x_pack_transpose_*: matrix (size0 x size1, dense) -> tiles of
        tile0 rows x tile1 columns stored column by column."""
        assert PACK_TRANSPOSE_EXPORTS[name][1]
        self.dispatch(name, pack_transpose_workgroup_count(name, size0, size1, tile0, tile1), [matrix, tiles],
                      [size0, size1, tile0, tile1, padding], stream)

    def unpack_transpose(self, name, tiles, matrix, size0, size1, tile0, tile1, stream=None):
        """mi355x_unpack_transpose_*: tiles stored column by column -> matrix."""
        assert not PACK_TRANSPOSE_EXPORTS[name][1]
        self.dispatch(name, pack_transpose_workgroup_count(name, size0, size1, tile0, tile1), [tiles, matrix],
                      [size0, size1, tile0, tile1], stream)

    def dequant_matmul_i4(self, name, x, w_tiled, scale, zp, out, M, N, stream=None):
        """mi355x_dequant_matmul_i4_k4096_g128_*: out[M][N] f16 = x[M][4096] f16
        times int4 weights (tiled layout) with f16 scales [N][32] and packed
        uint4 zero points [N][32]."""
        assert 1 <= M <= DEQUANT_EXPORTS[name] and N >= 32 and N % 32 == 0
        self.dispatch(name, dequant_workgroup_count(N), [x, w_tiled, scale, zp, out], [M, N], stream)

    def close(self):
        if self._handle:
            self._lib.iree_amd_hal_executable_release(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


_MLIR_HEADER = """\
// hal.executable.source for iree_amd/hal/mi355x_kernels_gfx950.co: the gfx950
// mmt4d, pack, unpack and int4 dequantising matmul kernels as hand-written dispatches on a HIP device, after the
// reference's samples/custom_dispatch/hip/kernels/example.mlir:16-118.
// Written by iree_amd.hal_executable.mlir_source(); NOT compiled here (this
// build has no iree-compile).
//
// Every mmt4d export: bindings lhs (read only), rhs (read only), out; push constants
// M, N, K (outer tile counts), K0, flags (0x100 = accumulate), and for
// mi355x_mmt4d_unpack_* also out_rows, out_cols. The workload of a dispatch is
// (M, N, batch): batch = 1 for linalg.mmt4d, the batch size of a
// linalg.batch_mmt4d on dense operands (workgroup planes in y).

#rocm_gfx950_target = #hal.executable.target<"rocm", "rocm-hsaco-fb", {
  target_arch = "gfx950"
}>

hal.executable.source public @mi355x_mmt4d attributes {
  objects = #hal.executable.objects<{
    #rocm_gfx950_target = [
      #hal.executable.object<{path = "iree_amd/hal/mi355x_kernels_gfx950.co"}>
    ]
  }>
} {
"""

_MLIR_EXPORT = """\
  hal.executable.export public @{name} ordinal({ordinal})
      layout(#hal.pipeline.layout<push_constants = {constants}, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {{
    workgroup_size = [{wg} : index, 1 : index, 1 : index],
    workgroup_local_memory = {lds} : index
  }} {{
  ^bb0(%device: !hal.device, %m: index, %n: index, %batch: index):
    %x = affine.apply affine_map<()[s0, s1] -> ((s0 ceildiv {tile}) * (s1 ceildiv {tile}))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %batch, %c1 : index, index, index
  }}
"""

_MLIR_MATMUL_EXPORT = """\
  // out[M][N] (+)= lhs[M][K] * rhs (packed); push constants M, N, K (elements), K0, flags; workload (M, N)
  // limits: M * K elements of lhs below 2 GiB, K a multiple of the matrix-core K extent (else nothing is written)
  hal.executable.export public @{name} ordinal({ordinal})
      layout(#hal.pipeline.layout<push_constants = 5, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer>
        ]>
      ]>) attributes {{
    workgroup_size = [{wg} : index, 1 : index, 1 : index],
    workgroup_local_memory = {lds} : index
  }} {{
  ^bb0(%device: !hal.device, %m: index, %n: index):
    %x = affine.apply affine_map<()[s0, s1] -> (((s0 ceildiv 32) ceildiv {tile_m}) * ((s1 ceildiv 32) ceildiv {tile_n}))>()[%m, %n]
    %c1 = arith.constant 1 : index
    hal.return %x, %c1, %c1 : index, index, index
  }}
"""

_MLIR_PACK_EXPORT = """\
  // {what}; push constants size0, size1, tile0, tile1{extra}; workload (size0, size1, tile0, tile1)
  // any tile size, no transposes; power-of-two tiles whose rows are whole 16-byte chunks stream 16-byte chunks, others move single elements
  hal.executable.export public @{name} ordinal({ordinal})
      layout(#hal.pipeline.layout<push_constants = {constants}, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {{
    workgroup_size = [{wg} : index, 1 : index, 1 : index]
  }} {{
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c32 = arith.constant 32 : index
    %bytes = arith.constant {es} : index
{extent}
    %chunks = arith.ceildivui %row_bytes, %c16 : index
    %bx = arith.ceildivui %chunks, %c32 : index
    %by = arith.ceildivui {rows}, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }}
"""

_MLIR_PACK_TRANSPOSE_EXPORT = """\
  // {what}, tiles of tile0 rows x tile1 columns stored column by column; push constants size0, size1, tile0, tile1{extra}; workload (size0, size1, tile0, tile1)
  // any tile size; power-of-two tiles with tile0 * {es} >= 16 move 16-byte chunks, others single elements
  hal.executable.export public @{name} ordinal({ordinal})
      layout(#hal.pipeline.layout<push_constants = {constants}, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer>
        ]>
      ]>) attributes {{
    workgroup_size = [{wg} : index, 1 : index, 1 : index]
  }} {{
  ^bb0(%device: !hal.device, %size0: index, %size1: index, %tile0: index, %tile1: index):
    %c1 = arith.constant 1 : index
    %c16 = arith.constant 16 : index
    %c64 = arith.constant 64 : index
    %bytes = arith.constant {es} : index
    %o0 = arith.ceildivui %size0, %tile0 : index
    %tile_bytes = arith.muli %tile0, %bytes : index
    %per_tile = arith.ceildivui %tile_bytes, %c16 : index
    %groups = arith.muli %o0, %per_tile : index
{extent}    %bx = arith.ceildivui {cols}, %c64 : index
    %by = arith.ceildivui %groups, %c16 : index
    %x = arith.muli %bx, %by : index
    hal.return %x, %c1, %c1 : index, index, index
  }}
"""

_MLIR_DEQUANT_EXPORT = """\
  // out[M][N] f16 = x[M][4096] f16 * int4 weights (tiled), groups of 128: f16 scales [N][32], packed uint4 zero points [N][32]
  // push constants M, N; workload (N); limits: 1 <= M <= {rows}, N a multiple of 32 (else nothing is written)
  hal.executable.export public @{name} ordinal({ordinal})
      layout(#hal.pipeline.layout<push_constants = 2, sets = [
        <0, bindings = [
            <0, storage_buffer, ReadOnly>,
            <1, storage_buffer, ReadOnly>,
            <2, storage_buffer, ReadOnly>,
            <3, storage_buffer, ReadOnly>,
            <4, storage_buffer>
        ]>
      ]>) attributes {{
    workgroup_size = [{wg} : index, 1 : index, 1 : index],
    workgroup_local_memory = {lds} : index
  }} {{
  ^bb0(%device: !hal.device, %n: index):
    %c1 = arith.constant 1 : index
    %c32 = arith.constant 32 : index
    %cmax = arith.constant {max_wg} : index
    %tiles = arith.divui %n, %c32 : index
    %x = arith.minui %tiles, %cmax : index
    hal.return %x, %c1, %c1 : index, index, index
  }}
"""

_MLIR_PACK_TRANSPOSE_EXTENT = """\
    %o1 = arith.ceildivui %size1, %tile1 : index
    %cols = arith.muli %o1, %tile1 : index
"""

_MLIR_PACK_EXTENT = """\
    %o0 = arith.ceildivui %size0, %tile0 : index
    %rows = arith.muli %o0, %tile0 : index
    %o1 = arith.ceildivui %size1, %tile1 : index
    %cols = arith.muli %o1, %tile1 : index
    %row_bytes = arith.muli %cols, %bytes : index"""

_MLIR_UNPACK_EXTENT = """\
    %row_bytes = arith.muli %size1, %bytes : index"""

_MLIR_FOOTER = """\
}

// A dispatch site (f16, 4096^3: M = N = 128 outer tiles, K = 512 tiles of K0 = 8):
//   %out = flow.dispatch @mi355x_mmt4d::@mi355x_mmt4d_f16f16f32_t8[%c128, %c128, %c1](
//       %c128_i32, %c128_i32, %c512_i32, %c8_i32, %c0_i32, %lhs, %rhs)
//     : (i32, i32, i32, i32, i32, tensor<128x512x32x8xf16>, tensor<128x512x32x8xf16>)
//       -> tensor<128x128x32x32xf32>
// (primitive operands come first and must be i32, example.mlir:128-140; with
// the accumulate flag the result is tied to a third tensor operand: `-> %acc`.)
"""


def mlir_source():
    """Text of the hal.executable.source that declares every export."""
    parts = [_MLIR_HEADER]
    for ordinal, e in enumerate(EXPORTS.values()):
        parts.append(_MLIR_EXPORT.format(
            name=e.name, ordinal=ordinal, constants=7 if "_unpack_" in e.name else 5,
            wg=WORKGROUP_SIZE, lds=e.lds, tile=e.tile))
    ordinal = len(EXPORTS)
    for e in MATMUL_EXPORTS.values():
        parts.append(_MLIR_MATMUL_EXPORT.format(name=e.name, ordinal=ordinal, wg=WORKGROUP_SIZE,
                                                lds=e.lds, tile_m=e.tile_m, tile_n=e.tile_n))
        ordinal += 1
    for name, (es, is_pack) in PACK_EXPORTS.items():
        parts.append(_MLIR_PACK_EXPORT.format(
            name=name, ordinal=ordinal, es=es, wg=WORKGROUP_SIZE, constants=5 if is_pack else 4,
            what=("pack: in = matrix, out = tiles" if is_pack else "unpack: in = tiles, out = matrix"),
            extra=", padding" if is_pack else "",
            extent=_MLIR_PACK_EXTENT if is_pack else _MLIR_UNPACK_EXTENT,
            rows="%rows" if is_pack else "%size0"))
        ordinal += 1
    for name, (es, is_pack) in PACK_TRANSPOSE_EXPORTS.items():
        parts.append(_MLIR_PACK_TRANSPOSE_EXPORT.format(
            name=name, ordinal=ordinal, es=es, wg=WORKGROUP_SIZE, constants=5 if is_pack else 4,
            what=("pack: in = matrix, out = tiles" if is_pack else "unpack: in = tiles, out = matrix"),
            extra=", padding" if is_pack else "",
            extent=_MLIR_PACK_TRANSPOSE_EXTENT if is_pack else "",
            cols="%cols" if is_pack else "%size1"))
        ordinal += 1
    for name, rows in DEQUANT_EXPORTS.items():
        parts.append(_MLIR_DEQUANT_EXPORT.format(name=name, ordinal=ordinal, rows=rows,
                                                 wg=DEQUANT_WORKGROUP_SIZE, lds=DEQUANT_LDS,
                                                 max_wg=DEQUANT_MAX_WORKGROUPS))
        ordinal += 1
    parts.append(_MLIR_FOOTER)
    return "".join(parts)
