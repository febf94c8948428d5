/*
 * iree_amd_hal_executable.h - loads a gfx950 code object of hand-written kernels
 * and dispatches its exports the way IREE's HIP HAL driver does, so that the
 * kernels linked into a `hal.executable.source`
 * (REF samples/custom_dispatch/hip/kernels/example.mlir:36-118) can be run and
 * tested without the IREE runtime.
 *
 * What each call stands for in the reference:
 *   load      iree_hal_hip_native_executable_create: hipModuleLoadDataEx on the
 *             code object bytes        REF runtime/src/iree/hal/drivers/hip/native_executable.c:180-200
 *   add_export  per entry point: hipModuleGetFunction, the check of the shared
 *             memory size against the device limit, hipFuncSetAttribute(
 *             MAX_DYNAMIC_SHARED_SIZE_BYTES), block size kept for the launches
 *                                      REF native_executable.c:213-253
 *   dispatch  iree_hal_hip_stream_command_buffer_dispatch: kernel parameters =
 *             the binding device pointers in order, then every push constant as
 *             a 32-bit value in a parameter slot of its own; hipModuleLaunchKernel
 *             with the export's block size and shared memory size
 *                                      REF runtime/src/iree/hal/drivers/hip/stream_command_buffer.c:519-581
 * Status codes are those of iree_amd_uk.h (0 = OK); the message of a failure is
 * read with iree_amd_uk_last_error().
 *
 * Limits of the exports in mi355x_kernels_gfx950.co (a kernel cannot report an
 * error: a dispatch outside them returns without writing anything):
 *   mi355x_mmt4d_*, mi355x_mmt4d_unpack_*   one outer row of an operand
 *       (32 x K elements) below 2 GiB; K whole K0 tiles; dense operands.
 *   mi355x_matmul_packed_rhs_*              the row-major left-hand side
 *       (M x K elements) below 2 GiB: its rows are addressed with 32-bit byte
 *       offsets; K a multiple of the matrix-core K extent (s8s8s32_k64: of
 *       64, with K0 = 16: the faster i8 form).
 *   mi355x_pack_*, mi355x_unpack_*          power-of-two tile sizes whose rows
 *       are whole 16-byte chunks, no transposes.
 *   mi355x_pack_transpose_*, mi355x_unpack_transpose_*   transposed inner
 *       tiles: power-of-two tile sizes whose stored rows (the tile's matrix
 *       rows) are whole 16-byte chunks.
 *   mi355x_dequant_matmul_i4_k4096_g128_r16, _r32   1..16 or 1..32 rows of
 *       4096 f16 activations; N a multiple of 32; weights in the layout
 *       iree_amd_uk_pack_i4_weights writes, f16 scales and packed uint4 zero
 *       points [N][32]; 512 threads and 131072 bytes of dynamic shared memory.
 */
#ifndef IREE_AMD_HAL_EXECUTABLE_H_
#define IREE_AMD_HAL_EXECUTABLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(_WIN32)
#define IREE_AMD_HAL_EXPORT
#else
#define IREE_AMD_HAL_EXPORT __attribute__((visibility("default")))
#endif

typedef struct iree_amd_hal_executable_t iree_amd_hal_executable_t;

/* Loads the code object `data[0..size)` on the current device. */
IREE_AMD_HAL_EXPORT int iree_amd_hal_executable_load(const void* data, size_t size,
                                 iree_amd_hal_executable_t** out_executable);

/* Registers the export `name` with the block size and dynamic shared memory
 * size its hal.executable.export declares (workgroup_size,
 * workgroup_local_memory); *out_ordinal is its index for dispatch. */
IREE_AMD_HAL_EXPORT int iree_amd_hal_executable_add_export(iree_amd_hal_executable_t* executable, const char* name,
                                       uint32_t block_x, uint32_t block_y, uint32_t block_z,
                                       uint32_t shared_memory_size, int32_t* out_ordinal);

/* Launches export `ordinal` over workgroup_x * _y * _z workgroups on `stream`
 * (a hipStream_t; NULL = the default stream). `bindings` are device pointers. */
IREE_AMD_HAL_EXPORT int iree_amd_hal_executable_dispatch(iree_amd_hal_executable_t* executable, int32_t ordinal,
                                     uint32_t workgroup_x, uint32_t workgroup_y,
                                     uint32_t workgroup_z, const void* const* bindings,
                                     size_t binding_count, const uint32_t* push_constants,
                                     size_t push_constant_count, void* stream);

/* Unloads the module and frees the handle (NULL is accepted). */
IREE_AMD_HAL_EXPORT void iree_amd_hal_executable_release(iree_amd_hal_executable_t* executable);

#ifdef __cplusplus
}
#endif

#endif /* IREE_AMD_HAL_EXECUTABLE_H_ */
