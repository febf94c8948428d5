// C-ABI entry points of the gfx950 ukernel library (include/iree_amd_uk.h):
// argument packing, validation, early returns, kernel selection, the thin
// device ABI and the host-pointer staging variants. No kernels live here.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "uk_common.h"

namespace uk {

static thread_local char g_last_error[512] = "";

int fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof g_last_error, fmt, ap);
  va_end(ap);
  return status;
}

static thread_local const char* g_kernel_path = "";
void note_kernel_path(const char* name) { g_kernel_path = name; }

int check_hip(hipError_t err, const char* what) {
  if (err == hipSuccess) return 0;
  int status = IREE_AMD_UK_STATUS_INTERNAL;
  if (err == hipErrorNoDevice || err == hipErrorInvalidDevice ||
      err == hipErrorNotInitialized || err == hipErrorInsufficientDriver) {
    status = IREE_AMD_UK_STATUS_UNAVAILABLE;
  } else if (err == hipErrorOutOfMemory) {
    status = 8;  // RESOURCE_EXHAUSTED
  }
  // The error is reported here: take it off the runtime's "last error", or the
  // caller's next HIP call (torch's, say) reports it a second time.
  (void)hipGetLastError();
  return fail(status, "%s: %s", what, hipGetErrorString(err));
}

bool mmt4d_type_info(uint32_t flags, Mmt4dTypeInfo* out) {
  switch (flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32: *out = {32, 32, 4}; return true;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32: *out = {8, 8, 4}; return true;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32: *out = {16, 16, 4}; return true;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16: *out = {16, 16, 2}; return true;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32: *out = {16, 16, 4}; return true;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16: *out = {16, 16, 2}; return true;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S16S32: *out = {16, 16, 4}; return true;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S16U4S32: *out = {16, 4, 4}; return true;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32: *out = {16, 8, 4}; return true;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S4S32: *out = {8, 4, 4}; return true;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32: *out = {8, 8, 4}; return true;
    default: return false;
  }
}

int pack_elem_bytes(uint32_t flags) {
  switch (flags & IREE_AMD_UK_FLAG_PACK_TYPE_MASK) {
    case IREE_AMD_UK_FLAG_PACK_TYPE_F32F32:
    case IREE_AMD_UK_FLAG_PACK_TYPE_I32I32: return 4;
    case IREE_AMD_UK_FLAG_PACK_TYPE_F16F16:
    case IREE_AMD_UK_FLAG_PACK_TYPE_BF16BF16: return 2;
    case IREE_AMD_UK_FLAG_PACK_TYPE_I8I8: return 1;
    default: return 0;
  }
}

int unpack_elem_bytes(uint32_t flags) {
  // Same table minus the 1-byte type, which the reference reserves but does
  // not define for unpack (exported_bits.h:75-79).
  if ((flags & IREE_AMD_UK_FLAG_UNPACK_TYPE_MASK) == IREE_AMD_UK_FLAG_PACK_TYPE_I8I8)
    return 0;
  return pack_elem_bytes(flags);
}

static bool fits_i32(int64_t v) { return v >= 0 && v <= 0x7FFFFFFFll; }
static bool fits_i16(int64_t v) { return v >= 0 && v <= 0x7FFFll; }

// Mirrors the asserts of the reference's iree_uk_mmt4d_validate (mmt4d.c:12-48).
int validate_mmt4d(const iree_amd_uk_mmt4d_params_t& p) {
  const uint32_t known =
      IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK | IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE |
      IREE_AMD_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS |
      IREE_AMD_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION;
  if (p.flags & ~known)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: unknown flag bits 0x%x", p.flags & ~known);
  Mmt4dTypeInfo ti;
  if (!mmt4d_type_info(p.flags, &ti))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: unknown type 0x%x", p.flags & 0xFF);
  if (!fits_i32(p.M) || !fits_i32(p.N) || !fits_i32(p.K))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: M/N/K outside [0, 2^31)");
  if (!fits_i16(p.M0) || !fits_i16(p.N0) || !fits_i16(p.K0))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: M0/N0/K0 outside [0, 2^15)");
  if ((p.K0 * ti.lhs_bits) % 8 || (p.K0 * ti.rhs_bits) % 8)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: K0 rows are not whole bytes");
  if ((p.lhs_stride0 * ti.lhs_bits) % 8 || (p.rhs_stride0 * ti.rhs_bits) % 8 ||
      (p.lhs_offset * ti.lhs_bits) % 8 || (p.rhs_offset * ti.rhs_bits) % 8)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: sub-byte stride/offset not on a byte boundary");
  return 0;
}

// Mirrors iree_uk_pack_validate (pack.c:51-103). The reference also caps one
// tile at 4 KiB because of its stack temporary (pack.c:9-49); the GPU kernels
// have no such buffer, so larger tiles are accepted here.
int validate_pack(const iree_amd_uk_pack_params_t& p) {
  const uint32_t known = IREE_AMD_UK_FLAG_PACK_TYPE_MASK |
                         IREE_AMD_UK_FLAG_PACK_TRANSPOSE_INNER |
                         IREE_AMD_UK_FLAG_PACK_TRANSPOSE_OUTER;
  if (p.flags & ~known)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack: unknown flag bits 0x%x", p.flags & ~known);
  if (!pack_elem_bytes(p.flags))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack: unknown type 0x%x", p.flags & 0xFF);
  if (p.in_size0 < 0 || p.in_size1 < 0 || p.out_size0 < 0 || p.out_size1 < 0 ||
      p.out_size2 < 0 || p.out_size3 < 0 || p.in_stride0 < 0 ||
      p.in_stride1 < 0 || p.out_stride0 < 0)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack: negative size or stride");
  if (p.out_stride1 != p.out_size2 * p.out_size3)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack: out_stride1 must equal out_size2*out_size3");
  int64_t o0 = p.out_size0, o1 = p.out_size1, t0 = p.out_size2, t1 = p.out_size3;
  if (p.flags & IREE_AMD_UK_FLAG_PACK_TRANSPOSE_OUTER) { int64_t t = o0; o0 = o1; o1 = t; }
  if (p.flags & IREE_AMD_UK_FLAG_PACK_TRANSPOSE_INNER) { int64_t t = t0; t0 = t1; t1 = t; }
  if (o0 * t0 < p.in_size0 || o1 * t1 < p.in_size1)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack: tiled shape does not cover the source");
  return 0;
}

// Mirrors iree_uk_unpack_validate (unpack.c:31-81).
int validate_unpack(const iree_amd_uk_unpack_params_t& p) {
  const uint32_t known = IREE_AMD_UK_FLAG_UNPACK_TYPE_MASK |
                         IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_INNER |
                         IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_OUTER;
  if (p.flags & ~known)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "unpack: unknown flag bits 0x%x", p.flags & ~known);
  if (!unpack_elem_bytes(p.flags))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "unpack: unknown type 0x%x", p.flags & 0xFF);
  if (p.in_size0 < 0 || p.in_size1 < 0 || p.in_size2 < 0 || p.in_size3 < 0 ||
      p.out_size0 < 0 || p.out_size1 < 0 || p.in_stride0 < 0 ||
      p.out_stride0 < 0 || p.out_stride1 < 0)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "unpack: negative size or stride");
  if (p.in_stride1 != p.in_size2 * p.in_size3)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "unpack: in_stride1 must equal in_size2*in_size3");
  int64_t o0 = p.in_size0, o1 = p.in_size1, t0 = p.in_size2, t1 = p.in_size3;
  if (p.flags & IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_OUTER) { int64_t t = o0; o0 = o1; o1 = t; }
  if (p.flags & IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_INNER) { int64_t t = t0; t0 = t1; t1 = t; }
  if (o0 * t0 < p.out_size0 || o1 * t1 < p.out_size1)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "unpack: tiled shape does not cover the destination");
  return 0;
}

int device_cu_count() {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (!cached[dev]) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

// The tile the gfx950 kernels are built around, per operation:
// M0 = N0 = 32 (one MFMA 32x32 block) and K0 = half the K extent of one MFMA,
// i.e. exactly the 16 bytes one lane feeds the instruction, so that a packed
// tile is already in MFMA operand register order.
struct MatmulTile { int M0, N0, K0; };
static bool matmul_tile_for_op(uint32_t op, MatmulTile* t) {
  switch (op) {
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_I8I8I32:
      *t = {32, 32, 16}; return true;
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F32:
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F16:
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16F32:
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16BF16:
      *t = {32, 32, 8}; return true;
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F8E4M3F8E4M3F32:
      *t = {32, 32, 16}; return true;
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F32F32F32:
      *t = {32, 32, 4}; return true;
    default: return false;
  }
}

// Narrow dimension handling: a static size below the full tile shrinks the tile
// to the next power of two that holds it (the reference's compile-time chooser
// accepts padding up to that power of two and no further,
// CPUMaterializeEncodingPass.cpp:343-353).
static int narrow(int full, int64_t size) {
  if (size < 0 || size >= full) return full;  // dynamic (INT64_MIN) or wide
  int t = 1;
  while (t < size) t <<= 1;
  return t < full ? t : full;
}

}  // namespace uk

using namespace uk;

//===----------------------------------------------------------------------===//
// mmt4d
//===----------------------------------------------------------------------===//

extern "C" int iree_amd_uk_mmt4d_p(const iree_amd_uk_mmt4d_params_t* params,
                                   void* stream) {
  if (!params) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: null params");
  const iree_amd_uk_mmt4d_params_t& p = *params;
  UK_RETURN_IF_ERROR(validate_mmt4d(p));
  // Early return exactly as the reference (mmt4d.c:105-113).
  if (p.M == 0 || p.N == 0 ||
      (p.K == 0 && (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE)))
    return 0;
  if (p.M0 == 0 || p.N0 == 0) return 0;  // empty tiles: nothing to write
  if (!p.lhs_buffer && p.K && p.K0) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: null lhs");
  if (!p.rhs_buffer && p.K && p.K0) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: null rhs");
  if (!p.out_buffer) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: null out");
  hipStream_t s = (hipStream_t)stream;
  // (what served the call is recorded for iree_amd_uk_last_kernel_path)
  auto generic = [&]() {
    note_kernel_path("mmt4d:element-wise");
    return launch_mmt4d_generic(p, s);
  };
  if (mmt4d_skinny_supported(p.flags, p.M0, p.N0, p.K0)) {
    // Narrow left-hand-side tiles (a matrix of fewer than 32 rows): the
    // streaming MFMA kernel, or the element-wise one for what it cannot take.
    int st = launch_mmt4d_skinny(p, s);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) { note_kernel_path("mmt4d:mfma-narrow"); return st; }
    return generic();
  }
  if (mmt4d_mfma_supported(p.flags, p.M0, p.N0, p.K0)) {
    int st = launch_mmt4d_mfma(p, s);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) { note_kernel_path("mmt4d:mfma"); return st; }
    // A gfx950 tile whose operands the MFMA kernel cannot take (not 16-byte
    // aligned, or a K extent that is not whole MFMA steps): the tile is still
    // an architecture tile, served by the element-wise kernel whether or not
    // the caller allowed the generic fallback.
    return generic();
  }
  if (mmt4d_s8s4_widened_supported(p.flags, p.M0, p.N0, p.K0)) {
    int st = launch_mmt4d_s8s4_widened(p, s);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) { note_kernel_path("mmt4d:mfma-widened-s4"); return st; }
    return generic();     // (an architecture tile all the same)
  }
  if (mmt4d_s16_planes_supported(p.flags, p.M0, p.N0, p.K0)) {
    int st = launch_mmt4d_s16_planes(p, s);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) { note_kernel_path("mmt4d:mfma-s16-planes"); return st; }
    return generic();     // (likewise)
  }
  if (!(p.flags & IREE_AMD_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION)) {
    // The reference asserts here (mmt4d.c:128-138); a release build would
    // crash on a null tile function. Report instead.
    return fail(IREE_AMD_UK_STATUS_UNIMPLEMENTED,
                "mmt4d: no gfx950 MFMA kernel for type 0x%x tile %dx%dx%d and "
                "generic fallback not allowed",
                p.flags & 0xFF, p.M0, p.N0, p.K0);
  }
  return generic();
}

extern "C" int iree_amd_uk_mmt4d(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t M0, int32_t N0,
    int32_t K0, uint32_t flags, const uint64_t* cpu_data, void* stream) {
  iree_amd_uk_mmt4d_params_t p = {lhs_buffer, lhs_offset, lhs_stride0,
                                  rhs_buffer, rhs_offset, rhs_stride0,
                                  out_buffer, out_offset, out_stride0,
                                  M, N, K, M0, N0, K0, flags, cpu_data};
  return iree_amd_uk_mmt4d_p(&p, stream);
}

extern "C" int iree_amd_uk_batch_mmt4d(const iree_amd_uk_mmt4d_params_t* params,
                                       iree_amd_uk_index_t batch,
                                       iree_amd_uk_index_t lhs_batch_stride,
                                       iree_amd_uk_index_t rhs_batch_stride,
                                       iree_amd_uk_index_t out_batch_stride, void* stream) {
  if (!params) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "batch_mmt4d: null params");
  if (batch < 0) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "batch_mmt4d: negative batch");
  const iree_amd_uk_mmt4d_params_t& p = *params;
  UK_RETURN_IF_ERROR(validate_mmt4d(p));
  if (batch == 0) return 0;
  if (batch == 1) return iree_amd_uk_mmt4d_p(params, stream);
  // One launch over all batch entries where the matrix-core kernel takes the
  // problem; the same early returns as a single mmt4d come first.
  const bool nothing_to_do = p.M == 0 || p.N == 0 || p.M0 == 0 || p.N0 == 0 ||
                             (p.K == 0 && (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE));
  if (nothing_to_do) return 0;
  if (p.lhs_buffer && p.rhs_buffer && p.out_buffer && mmt4d_skinny_supported(p.flags, p.M0, p.N0, p.K0)) {
    // (narrow left-hand sides: the entries of a decode step)
    const int st = launch_batch_mmt4d_skinny(p, batch, lhs_batch_stride, rhs_batch_stride,
                                             out_batch_stride, (hipStream_t)stream);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) return st;
  } else if (p.lhs_buffer && p.rhs_buffer && p.out_buffer && mmt4d_mfma_supported(p.flags, p.M0, p.N0, p.K0)) {
    const int st = launch_batch_mmt4d_mfma(p, batch, lhs_batch_stride, rhs_batch_stride,
                                           out_batch_stride, (hipStream_t)stream);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) return st;
  }
  // Otherwise entry by entry, the way the reference lowers the op (batch tiled
  // to 1, then rank-reduced to mmt4d: CPUPrepareUkernels.cpp:23-43,165-245).
  for (iree_amd_uk_index_t b = 0; b < batch; ++b) {
    iree_amd_uk_mmt4d_params_t q = p;
    q.lhs_offset += b * lhs_batch_stride;
    q.rhs_offset += b * rhs_batch_stride;
    q.out_offset += b * out_batch_stride;
    UK_RETURN_IF_ERROR(iree_amd_uk_mmt4d_p(&q, stream));
  }
  return 0;
}

extern "C" uint32_t iree_amd_uk_mmt4d_info(int32_t M0, int32_t N0, int32_t K0,
                                           uint32_t flags,
                                           const uint64_t* cpu_data) {
  (void)cpu_data;
  return (mmt4d_mfma_supported(flags, M0, N0, K0) || mmt4d_skinny_supported(flags, M0, N0, K0) ||
          mmt4d_s8s4_widened_supported(flags, M0, N0, K0) || mmt4d_s16_planes_supported(flags, M0, N0, K0))
             ? IREE_AMD_UK_FLAG_MMT4D_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION
             : 0u;
}

//===----------------------------------------------------------------------===//
// pack / unpack
//===----------------------------------------------------------------------===//

extern "C" int iree_amd_uk_pack_p(const iree_amd_uk_pack_params_t* params,
                                  void* stream) {
  if (!params) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack: null params");
  const iree_amd_uk_pack_params_t& p = *params;
  UK_RETURN_IF_ERROR(validate_pack(p));
  // Early return as the reference (pack.c:106-109).
  if (p.out_size0 == 0 || p.out_size1 == 0 || p.out_size2 == 0 || p.out_size3 == 0)
    return 0;
  if (!p.out_buffer) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack: null out");
  if (!p.in_buffer && p.in_size0 && p.in_size1)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack: null in");
  return launch_pack(p, (hipStream_t)stream);
}

extern "C" int iree_amd_uk_pack(
    const void* in_buffer, iree_amd_uk_index_t in_offset,
    iree_amd_uk_index_t in_stride0, iree_amd_uk_index_t in_stride1,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t out_stride1,
    iree_amd_uk_index_t in_size0, iree_amd_uk_index_t in_size1,
    iree_amd_uk_index_t out_size0, iree_amd_uk_index_t out_size1,
    iree_amd_uk_index_t out_size2, iree_amd_uk_index_t out_size3,
    uint64_t padding_value, uint32_t flags, const uint64_t* cpu_data,
    void* stream) {
  iree_amd_uk_pack_params_t p = {in_buffer, in_offset, in_stride0, in_stride1,
                                 out_buffer, out_offset, out_stride0, out_stride1,
                                 in_size0, in_size1, out_size0, out_size1,
                                 out_size2, out_size3, padding_value, flags,
                                 cpu_data};
  return iree_amd_uk_pack_p(&p, stream);
}

extern "C" int iree_amd_uk_unpack_p(const iree_amd_uk_unpack_params_t* params,
                                    void* stream) {
  if (!params) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "unpack: null params");
  const iree_amd_uk_unpack_params_t& p = *params;
  UK_RETURN_IF_ERROR(validate_unpack(p));
  // Early return as the reference (unpack.c:84-86).
  if (p.out_size0 == 0 || p.out_size1 == 0) return 0;
  if (!p.out_buffer || !p.in_buffer)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "unpack: null buffer");
  return launch_unpack(p, (hipStream_t)stream);
}

extern "C" int iree_amd_uk_unpack(
    const void* in_buffer, iree_amd_uk_index_t in_offset,
    iree_amd_uk_index_t in_stride0, iree_amd_uk_index_t in_stride1,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t out_stride1,
    iree_amd_uk_index_t in_size0, iree_amd_uk_index_t in_size1,
    iree_amd_uk_index_t in_size2, iree_amd_uk_index_t in_size3,
    iree_amd_uk_index_t out_size0, iree_amd_uk_index_t out_size1,
    uint32_t flags, const uint64_t* cpu_data, void* stream) {
  iree_amd_uk_unpack_params_t p = {in_buffer, in_offset, in_stride0, in_stride1,
                                   out_buffer, out_offset, out_stride0, out_stride1,
                                   in_size0, in_size1, in_size2, in_size3,
                                   out_size0, out_size1, flags, cpu_data};
  return iree_amd_uk_unpack_p(&p, stream);
}

//===----------------------------------------------------------------------===//
// query_tile_sizes_2d
//===----------------------------------------------------------------------===//

extern "C" int iree_amd_uk_query_tile_sizes_2d(
    const iree_amd_uk_query_tile_sizes_2d_params_t* params,
    iree_amd_uk_query_tile_sizes_2d_out_params_t* out_params) {
  if (!params || !out_params)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "query_tile_sizes: null params");
  MatmulTile t;
  if (!matmul_tile_for_op(params->flags & IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MASK, &t))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "query_tile_sizes: unknown operation 0x%x",
                params->flags & IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MASK);
  // Role mapping of the reference (query_tile_sizes.c:43-63).
  switch (params->flags & IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_MASK) {
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_LHS:
      out_params->tile_size0 = narrow(t.M0, params->size0);
      out_params->tile_size1 = t.K0;
      return 0;
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RHS:
      out_params->tile_size0 = narrow(t.N0, params->size0);
      out_params->tile_size1 = t.K0;
      return 0;
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RESULT: {
      // Both dimensions are known here. At most ONE is narrowed, the smaller
      // one (the reference's chooser reduces narrow-N to narrow-M by
      // transposition only when N is the narrower of the two and keeps the
      // other dimension's full tile: CPUMaterializeEncodingPass.cpp:296-303).
      const int m0 = narrow(t.M0, params->size0), n0 = narrow(t.N0, params->size1);
      const bool m_narrow = m0 < t.M0, n_narrow = n0 < t.N0;
      // (an empty dimension counts as one of size 1, as in the three-size query)
      const int64_t s0 = params->size0 > 0 ? params->size0 : 1, s1 = params->size1 > 0 ? params->size1 : 1;
      const bool pick_n = n_narrow && (!m_narrow || s1 < s0);
      out_params->tile_size0 = pick_n ? t.M0 : m0;
      out_params->tile_size1 = pick_n ? n0 : t.N0;
      return 0;
    }
    default:
      return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "query_tile_sizes: unknown operand role 0x%x",
                  params->flags & IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_MASK);
  }
}

extern "C" int iree_amd_uk_enumerate_matmul_tiles(uint32_t operation, iree_amd_uk_matmul_tile_t* tiles,
                                                  int32_t capacity, int32_t* out_count) {
  if (!out_count || capacity < 0 || (capacity > 0 && !tiles))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "enumerate_matmul_tiles: null argument or negative capacity");
  MatmulTile t;
  if (!matmul_tile_for_op(operation & IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MASK, &t))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "enumerate_matmul_tiles: unknown operation 0x%x", operation);
  int32_t n = 0;
  for (int m = t.M0; m >= 1; m >>= 1, ++n)
    if (n < capacity) tiles[n] = {m, t.N0, t.K0};
  *out_count = n;
  return 0;
}

namespace {
int64_t power_of_2_ceil(int64_t v) {
  int64_t p = 1;
  while (p < v) p <<= 1;
  return p;
}
}  // namespace

extern "C" int iree_amd_uk_choose_matmul_tile(const iree_amd_uk_matmul_tile_t* tiles, int32_t count,
                                              iree_amd_uk_index_t narrow_m, iree_amd_uk_index_t narrow_n,
                                              const iree_amd_uk_index_t* upper_bound,
                                              iree_amd_uk_matmul_tile_t* out_tile) {
  if (!tiles || !out_tile || count <= 0 || narrow_m < 0 || narrow_n < 0)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "choose_matmul_tile: null argument, no tiles or a negative size");
  // narrow N: reduce to narrow M, exchange M and N of the answer
  if (narrow_n && (!narrow_m || narrow_n < narrow_m)) {
    const int st = iree_amd_uk_choose_matmul_tile(tiles, count, narrow_n, 0, upper_bound, out_tile);
    if (st) return st;
    const int32_t m = out_tile->M;
    out_tile->M = out_tile->N;
    out_tile->N = m;
    return 0;
  }
  int64_t best_penalty = INT64_MAX;
  for (int pass = 0; pass < 2; ++pass) {
    int64_t best_product = 0;
    bool found = false;
    for (int32_t i = 0; i < count; ++i) {
      const iree_amd_uk_matmul_tile_t& t = tiles[i];
      if (upper_bound && (t.M > upper_bound[0] || t.N > upper_bound[1] || t.K > upper_bound[2])) continue;
      int64_t penalty = 0;
      if (narrow_m) {
        penalty = (int64_t)t.M - power_of_2_ceil(narrow_m);
        if (penalty < 0) penalty = 0;
      }
      if (pass == 0) {
        if (penalty < best_penalty) best_penalty = penalty;
        found = true;
      } else if (penalty == best_penalty) {
        const int64_t product = (int64_t)t.M * t.N * t.K;
        if (best_product < product) {
          best_product = product;
          *out_tile = t;
          found = true;
        }
      }
    }
    if (!found)
      return fail(IREE_AMD_UK_STATUS_NOT_FOUND, "choose_matmul_tile: no tile within the upper bound");
  }
  return 0;
}

extern "C" int iree_amd_uk_query_matmul_tile_sizes(uint32_t operation, iree_amd_uk_index_t M,
                                                   iree_amd_uk_index_t N, iree_amd_uk_index_t K,
                                                   iree_amd_uk_matmul_tile_t* out_tile) {
  (void)K;   // (no gfx950 tile depends on the size of K)
  if (!out_tile) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "query_matmul_tile_sizes: null out_tile");
  iree_amd_uk_matmul_tile_t tiles[8];
  int32_t count = 0;
  UK_RETURN_IF_ERROR(iree_amd_uk_enumerate_matmul_tiles(operation, tiles, 8, &count));
  if (count > 8) count = 8;
  // A static size below the widest tile marks the matmul as narrow in that
  // dimension; the chooser then narrows the narrower of the two only.
  const int64_t full_m = tiles[0].M, full_n = tiles[0].N;
  const int64_t narrow_m = (M >= 0 && M < full_m) ? (M > 0 ? M : 1) : 0;
  const int64_t narrow_n = (N >= 0 && N < full_n) ? (N > 0 ? N : 1) : 0;
  return iree_amd_uk_choose_matmul_tile(tiles, count, narrow_m, narrow_n, nullptr, out_tile);
}

//===----------------------------------------------------------------------===//
// int4 dequant matmul, fp8 helpers
//===----------------------------------------------------------------------===//

extern "C" int iree_amd_uk_dequant_matmul_i4(
    const void* x_buffer, const void* w_buffer, const void* scale_buffer,
    const void* zp_buffer, void* out_buffer, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K,
    iree_amd_uk_index_t group_size, uint32_t flags, void* stream) {
  if (flags & ~7u) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "dequant_matmul_i4: unknown flag bits");
  if (M < 0 || N < 0 || K < 0 || group_size <= 0)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "dequant_matmul_i4: bad sizes");
  if (K % group_size || group_size % 32)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT,
                "dequant_matmul_i4: need K %% group_size == 0 and group_size %% 32 == 0");
  if (M == 0 || N == 0) return 0;
  if (!x_buffer || !w_buffer || !scale_buffer || !zp_buffer || !out_buffer)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "dequant_matmul_i4: null buffer");
  if (flags & IREE_AMD_UK_FLAG_DEQUANT_MATMUL_REASSOCIATE)
    return launch_dequant_matmul_i4_reassoc(x_buffer, w_buffer, scale_buffer, zp_buffer,
                                            out_buffer, M, N, K, group_size, flags,
                                            (hipStream_t)stream);
  return launch_dequant_matmul_i4(x_buffer, w_buffer, scale_buffer, zp_buffer,
                                  out_buffer, M, N, K, group_size, flags,
                                  (hipStream_t)stream);
}

extern "C" int iree_amd_uk_quantize_groups_i16(const void* x_f16, void* q_i16, void* scale_x_f32,
                                               void* group_sum_f32, iree_amd_uk_index_t M,
                                               iree_amd_uk_index_t K, iree_amd_uk_index_t group_size,
                                               void* stream) {
  if (M < 0 || K < 0 || group_size <= 0 || K % group_size)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "quantize_groups_i16: need K %% group_size == 0");
  if (M == 0 || K == 0) return 0;
  if (!x_f16 || !q_i16 || !scale_x_f32 || !group_sum_f32)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "quantize_groups_i16: null buffer");
  return launch_quantize_groups_i16(x_f16, q_i16, scale_x_f32, group_sum_f32, M, K, group_size,
                                    (hipStream_t)stream);
}

extern "C" int iree_amd_uk_pack_i4_weights(const void* w_rowmajor, void* w_tiled,
                                           iree_amd_uk_index_t N, iree_amd_uk_index_t K,
                                           void* stream) {
  if (N < 0 || K < 0 || N % 32 || K % 128)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT,
                "pack_i4_weights: need N %% 32 == 0 and K %% 128 == 0");
  if (N == 0 || K == 0) return 0;
  if (!w_rowmajor || !w_tiled)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack_i4_weights: null buffer");
  if (((uintptr_t)w_rowmajor | (uintptr_t)w_tiled) % 4)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack_i4_weights: buffers must be 4-byte aligned");
  return launch_pack_i4_weights(w_rowmajor, w_tiled, N, K, (hipStream_t)stream);
}

extern "C" int iree_amd_uk_quantize_f16_to_f8e4m3(const void* in_f16,
                                                  void* out_fp8,
                                                  iree_amd_uk_index_t n,
                                                  float inv_scale, void* stream) {
  if (n < 0) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "quantize: negative n");
  if (n == 0) return 0;
  if (!in_f16 || !out_fp8) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "quantize: null buffer");
  return launch_quantize_f16_to_f8e4m3(in_f16, out_fp8, n, inv_scale, (hipStream_t)stream);
}

extern "C" int iree_amd_uk_quantize_pack_f8e4m3(const void* in_f16, iree_amd_uk_index_t ld, void* out_tiles,
                                               iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t rows,
                                               iree_amd_uk_index_t cols, float inv_scale, void* stream) {
  if (rows < 0 || cols < 0 || ld < cols || cols % 16)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "quantize_pack: cols must be whole tiles of 16 and ld >= cols");
  if (rows == 0 || cols == 0) return 0;
  if (!in_f16 || !out_tiles) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "quantize_pack: null buffer");
  if (out_stride0 < cols * 32 || out_stride0 % 16 || ((uintptr_t)out_tiles & 15))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT,
                "quantize_pack: the tiled buffer must be 16-byte aligned with an outer pitch of whole 16 bytes, at least cols * 32");
  return launch_quantize_pack_f8e4m3(in_f16, ld, out_tiles, out_stride0, rows, cols, inv_scale, (hipStream_t)stream);
}

extern "C" int iree_amd_uk_silu_mul_quantize(
    const void* gate_f32, const void* up_f32, void* out_fp8,
    iree_amd_uk_index_t rows, iree_amd_uk_index_t cols, iree_amd_uk_index_t ld,
    float gate_scale, float up_scale, float inv_out_scale, void* stream) {
  if (rows < 0 || cols < 0 || ld < cols)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "silu_mul_quantize: bad sizes");
  if (rows == 0 || cols == 0) return 0;
  if (!gate_f32 || !up_f32 || !out_fp8)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "silu_mul_quantize: null buffer");
  return launch_silu_mul_quantize(gate_f32, up_f32, out_fp8, rows, cols, ld,
                                  gate_scale, up_scale, inv_out_scale,
                                  (hipStream_t)stream);
}

extern "C" int iree_amd_uk_silu_mul_quantize_tiled(
    const void* acc_tiled, iree_amd_uk_index_t acc_stride0,
    iree_amd_uk_index_t gate_tile0, iree_amd_uk_index_t up_tile0,
    void* out_tiled, iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t M1,
    iree_amd_uk_index_t N1, float gate_scale, float up_scale,
    float inv_out_scale, void* stream) {
  if (M1 < 0 || N1 < 0 || gate_tile0 < 0 || up_tile0 < 0)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "silu_mul_quantize_tiled: bad sizes");
  if (M1 == 0 || N1 == 0) return 0;
  if (!acc_tiled || !out_tiled)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "silu_mul_quantize_tiled: null buffer");
  const iree_amd_uk_index_t last = (gate_tile0 > up_tile0 ? gate_tile0 : up_tile0) + N1;
  if (acc_stride0 < last * 1024 || out_stride0 < N1 * 1024)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT,
                "silu_mul_quantize_tiled: outer row pitch smaller than the tiles of a row");
  if (((uintptr_t)acc_tiled | (uintptr_t)out_tiled) % 16 || acc_stride0 % 4 || out_stride0 % 16)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT,
                "silu_mul_quantize_tiled: buffers and pitches must be 16-byte aligned");
  return launch_silu_mul_quantize_tiled(acc_tiled, acc_stride0, gate_tile0, up_tile0, out_tiled,
                                        out_stride0, M1, N1, gate_scale, up_scale,
                                        inv_out_scale, (hipStream_t)stream);
}

extern "C" int iree_amd_uk_mmt4d_silu_mul_f8e4m3(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float gate_scale, float up_scale, float inv_out_scale, void* stream) {
  iree_amd_uk_mmt4d_params_t p = {lhs_buffer, lhs_offset, lhs_stride0,
                                  rhs_buffer, rhs_offset, rhs_stride0,
                                  out_buffer, out_offset, out_stride0,
                                  M, N, K, 32, 32, K0, flags, nullptr};
  UK_RETURN_IF_ERROR(validate_mmt4d(p));
  if (flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d_silu_mul: accumulate is not supported");
  if (N % 2) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d_silu_mul: N counts gate and up tiles and must be even");
  if (out_stride0 < N / 2 * 1024)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d_silu_mul: out_stride0 smaller than one outer row");
  if (M == 0 || N == 0) return 0;
  if (!lhs_buffer || !rhs_buffer || !out_buffer)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d_silu_mul: null buffer");
  int st = IREE_AMD_UK_STATUS_NOT_FOUND;
  if (mmt4d_mfma_supported(flags, 32, 32, K0) &&
      (flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) != IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32)
    st = launch_mmt4d_silu_mul_mfma(p, gate_scale, up_scale, inv_out_scale, (hipStream_t)stream);
  if (st == IREE_AMD_UK_STATUS_NOT_FOUND)
    return fail(IREE_AMD_UK_STATUS_UNIMPLEMENTED,
                "mmt4d_silu_mul: needs an MFMA float type at its queried K0, K > 0 and "
                "16-byte aligned operands");
  return st;
}

namespace {
// Entry b of a batch works on operands b * {lhs,rhs,out}_batch_stride elements
// after those of entry 0; batch = 1 is the plain call.
struct BatchStrides {
  iree_amd_uk_index_t batch, lhs, rhs, out;
};

int mmt4d_unpack_impl(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t out_size0,
    iree_amd_uk_index_t out_size1, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float out_scale, const BatchStrides& b, void* stream) {
  if (b.batch < 0) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d_unpack: negative batch");
  iree_amd_uk_mmt4d_params_t p = {lhs_buffer, lhs_offset, lhs_stride0,
                                  rhs_buffer, rhs_offset, rhs_stride0,
                                  out_buffer, out_offset, out_stride0,
                                  M, N, K, 32, 32, K0, flags, nullptr};
  UK_RETURN_IF_ERROR(validate_mmt4d(p));
  if (out_scale != 1.0f) {
    const uint32_t type = flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK;
    const bool integer = type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32 ||
                         type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S16S32 ||
                         type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S16U4S32 ||
                         type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32 ||
                         type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S4S32;
    if (integer || (flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE))
      return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT,
                  "mmt4d_unpack: out_scale other than 1 needs a float type and no accumulate flag");
  }
  // the size conditions of unpack (unpack.c:31-80 of the reference) for 32x32 tiles
  if (out_size0 < 0 || out_size1 < 0 || out_size0 > M * 32 || out_size1 > N * 32 ||
      (M > 0 && out_size0 <= (M - 1) * 32) || (N > 0 && out_size1 <= (N - 1) * 32))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT,
                "mmt4d_unpack: matrix size does not match the outer tile counts");
  if (out_stride0 < out_size1)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d_unpack: out_stride0 smaller than a row");
  if (M == 0 || N == 0 || b.batch == 0) return 0;
  if (!lhs_buffer || !rhs_buffer || !out_buffer)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d_unpack: null buffer");
  int st = IREE_AMD_UK_STATUS_NOT_FOUND;
  if (mmt4d_mfma_supported(flags, 32, 32, K0))
    st = launch_mmt4d_unpack_mfma(p, out_size0, out_size1, out_scale, b.batch, b.lhs, b.rhs, b.out,
                                  (hipStream_t)stream);
  if (st == IREE_AMD_UK_STATUS_NOT_FOUND && b.batch > 1) {
    // (batch strides that one launch cannot take: entry by entry)
    for (iree_amd_uk_index_t e = 0; e < b.batch; ++e) {
      st = mmt4d_unpack_impl(lhs_buffer, lhs_offset + e * b.lhs, lhs_stride0, rhs_buffer, rhs_offset + e * b.rhs,
                             rhs_stride0, out_buffer, out_offset + e * b.out, out_stride0, out_size0, out_size1,
                             M, N, K, K0, flags, out_scale, BatchStrides{1, 0, 0, 0}, stream);
      if (st) return st;
    }
    return 0;
  }
  if (st == IREE_AMD_UK_STATUS_NOT_FOUND)
    return fail(IREE_AMD_UK_STATUS_UNIMPLEMENTED,
                "mmt4d_unpack: needs a type and K0 with a matrix-core kernel, K > 0 and "
                "16-byte aligned operands");
  return st;
}
}  // namespace

extern "C" int iree_amd_uk_mmt4d_unpack(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t out_size0,
    iree_amd_uk_index_t out_size1, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float out_scale, void* stream) {
  return mmt4d_unpack_impl(lhs_buffer, lhs_offset, lhs_stride0, rhs_buffer, rhs_offset, rhs_stride0, out_buffer,
                           out_offset, out_stride0, out_size0, out_size1, M, N, K, K0, flags, out_scale,
                           BatchStrides{1, 0, 0, 0}, stream);
}

extern "C" int iree_amd_uk_batch_mmt4d_unpack(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t out_size0,
    iree_amd_uk_index_t out_size1, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float out_scale, iree_amd_uk_index_t batch, iree_amd_uk_index_t lhs_batch_stride,
    iree_amd_uk_index_t rhs_batch_stride, iree_amd_uk_index_t out_batch_stride, void* stream) {
  return mmt4d_unpack_impl(lhs_buffer, lhs_offset, lhs_stride0, rhs_buffer, rhs_offset, rhs_stride0, out_buffer,
                           out_offset, out_stride0, out_size0, out_size1, M, N, K, K0, flags, out_scale,
                           BatchStrides{batch, lhs_batch_stride, rhs_batch_stride, out_batch_stride}, stream);
}

namespace {
int matmul_packed_rhs_impl(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float out_scale, const BatchStrides& b, void* stream) {
  if (b.batch < 0) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "matmul_packed_rhs: negative batch");
  if (M < 0 || N < 0 || K < 0 || K0 <= 0)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "matmul_packed_rhs: negative size or K0 <= 0");
  if (K % K0)
    return fail(IREE_AMD_UK_STATUS_UNIMPLEMENTED, "matmul_packed_rhs: K must be whole K0 tiles");
  // the equivalent mmt4d: outer counts and K tiles
  iree_amd_uk_mmt4d_params_t p = {lhs_buffer, lhs_offset, lhs_stride0,
                                  rhs_buffer, rhs_offset, rhs_stride0,
                                  out_buffer, out_offset, out_stride0,
                                  (M + 31) / 32, (N + 31) / 32, K / K0, 32, 32, K0, flags, nullptr};
  UK_RETURN_IF_ERROR(validate_mmt4d(p));
  if (out_scale != 1.0f) {
    const uint32_t type = flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK;
    const bool integer = type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32 ||
                         type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S16S32 ||
                         type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S16U4S32 ||
                         type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32 ||
                         type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S4S32;
    if (integer || (flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE))
      return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT,
                  "matmul_packed_rhs: out_scale other than 1 needs a float type and no accumulate flag");
  }
  if (lhs_stride0 < K || out_stride0 < N)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "matmul_packed_rhs: a row pitch smaller than a row");
  if (M == 0 || N == 0 || b.batch == 0) return 0;
  if (!lhs_buffer || !rhs_buffer || !out_buffer)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "matmul_packed_rhs: null buffer");
  int st = IREE_AMD_UK_STATUS_NOT_FOUND;
  // One row (the matrix-vector product of a decode step): the row is its own
  // tile row of 1 x K0 tiles and a row of 1 x 32 result tiles is the row-major
  // result, so this is the mmt4d with narrow left-hand side tiles that the
  // tile-size query gives for a static M of 1, which streams the right-hand
  // side once (N = 14336, K = 4096, f16: 23 us against 28 for the macro-tile
  // kernel with its K split).
  if (M == 1 && N % 32 == 0 && out_scale == 1.0f && mmt4d_skinny_supported(flags, 1, 32, K0)) {
    const iree_amd_uk_mmt4d_params_t row = {lhs_buffer, lhs_offset, K, rhs_buffer, rhs_offset, rhs_stride0,
                                            out_buffer, out_offset, N, 1, N / 32, K / K0, 1, 32, K0, flags, nullptr};
    // (a batch of such rows, the attention scores of a decode step say: the planes of one launch)
    st = b.batch == 1 ? launch_mmt4d_skinny(row, (hipStream_t)stream)
                      : launch_batch_mmt4d_skinny(row, b.batch, b.lhs, b.rhs, b.out, (hipStream_t)stream);
  }
  // A few rows (2 to 32): the same kernel with the rows of the matrix as the
  // rows of its one narrow tile, reading them and writing the result row-major.
  if (st == IREE_AMD_UK_STATUS_NOT_FOUND && M > 1 && M <= 32 && b.batch == 1 && out_scale == 1.0f)
    st = launch_matmul_rows_skinny(p, M, N, (hipStream_t)stream);
  if (st == IREE_AMD_UK_STATUS_NOT_FOUND && mmt4d_mfma_supported(flags, 32, 32, K0))
    st = launch_matmul_packed_rhs_mfma(p, M, N, out_scale, b.batch, b.lhs, b.rhs, b.out, (hipStream_t)stream);
  if (st == IREE_AMD_UK_STATUS_NOT_FOUND && b.batch > 1) {
    for (iree_amd_uk_index_t e = 0; e < b.batch; ++e) {
      st = matmul_packed_rhs_impl(lhs_buffer, lhs_offset + e * b.lhs, lhs_stride0, rhs_buffer,
                                  rhs_offset + e * b.rhs, rhs_stride0, out_buffer, out_offset + e * b.out,
                                  out_stride0, M, N, K, K0, flags, out_scale, BatchStrides{1, 0, 0, 0}, stream);
      if (st) return st;
    }
    return 0;
  }
  if (st == IREE_AMD_UK_STATUS_NOT_FOUND)
    return fail(IREE_AMD_UK_STATUS_UNIMPLEMENTED,
                "matmul_packed_rhs: needs a type and K0 with a matrix-core kernel, K > 0 in whole "
                "matrix-core steps and 16-byte aligned rows and tiles");
  return st;
}
}  // namespace

extern "C" int iree_amd_uk_matmul_packed_rhs(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float out_scale, void* stream) {
  return matmul_packed_rhs_impl(lhs_buffer, lhs_offset, lhs_stride0, rhs_buffer, rhs_offset, rhs_stride0,
                                out_buffer, out_offset, out_stride0, M, N, K, K0, flags, out_scale,
                                BatchStrides{1, 0, 0, 0}, stream);
}

extern "C" int iree_amd_uk_batch_matmul_packed_rhs(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float out_scale, iree_amd_uk_index_t batch, iree_amd_uk_index_t lhs_batch_stride,
    iree_amd_uk_index_t rhs_batch_stride, iree_amd_uk_index_t out_batch_stride, void* stream) {
  return matmul_packed_rhs_impl(lhs_buffer, lhs_offset, lhs_stride0, rhs_buffer, rhs_offset, rhs_stride0,
                                out_buffer, out_offset, out_stride0, M, N, K, K0, flags, out_scale,
                                BatchStrides{batch, lhs_batch_stride, rhs_batch_stride, out_batch_stride},
                                stream);
}

extern "C" int iree_amd_uk_scale_f32(void* buf_f32, iree_amd_uk_index_t n, float scale,
                                     void* stream) {
  if (n < 0) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "scale_f32: negative n");
  if (n == 0) return 0;
  if (!buf_f32 || (uintptr_t)buf_f32 % 4)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "scale_f32: null or misaligned buffer");
  return launch_scale_f32(buf_f32, n, scale, (hipStream_t)stream);
}

extern "C" int iree_amd_uk_mfma_probe(uint32_t type_flag, const void* operands,
                                      iree_amd_uk_index_t iters, void* sink,
                                      int64_t* out_ops_per_launch, void* stream) {
  if (!operands || !sink || (uintptr_t)operands % 16 || (uintptr_t)sink % 4)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mfma_probe: null or misaligned buffer");
  if (iters < 0 || iters > (1 << 24))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mfma_probe: iters out of range");
  return launch_mfma_probe(type_flag, operands, iters, sink, out_ops_per_launch,
                           (hipStream_t)stream);
}

extern "C" int iree_amd_uk_copy_probe(const void* src, void* dst, iree_amd_uk_index_t bytes, int32_t mode,
                                      int32_t blocks_per_cu, void* stream) {
  if (!src || !dst) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "copy_probe: null buffer");
  return launch_copy_probe(src, dst, bytes, mode, blocks_per_cu, (hipStream_t)stream);
}

//===----------------------------------------------------------------------===//
// Thin device ABI
//===----------------------------------------------------------------------===//

extern "C" int iree_amd_uk_device_count(int* out_count) {
  if (!out_count) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "device_count: null");
  *out_count = 0;
  hipError_t e = hipGetDeviceCount(out_count);
  if (e == hipErrorNoDevice) { *out_count = 0; return 0; }
  return check_hip(e, "hipGetDeviceCount");
}
extern "C" int iree_amd_uk_device_set(int ordinal) {
  return check_hip(hipSetDevice(ordinal), "hipSetDevice");
}
extern "C" int iree_amd_uk_device_malloc(void** out_ptr, uint64_t bytes) {
  if (!out_ptr) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "device_malloc: null");
  *out_ptr = nullptr;
  if (!bytes) return 0;
  return check_hip(hipMalloc(out_ptr, bytes), "hipMalloc");
}
extern "C" int iree_amd_uk_device_free(void* ptr) {
  if (!ptr) return 0;
  return check_hip(hipFree(ptr), "hipFree");
}
extern "C" int iree_amd_uk_memcpy_h2d(void* dst, const void* src, uint64_t bytes, void* stream) {
  if (!bytes) return 0;
  return check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream), "hipMemcpyAsync(h2d)");
}
extern "C" int iree_amd_uk_memcpy_d2h(void* dst, const void* src, uint64_t bytes, void* stream) {
  if (!bytes) return 0;
  return check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream), "hipMemcpyAsync(d2h)");
}
extern "C" int iree_amd_uk_stream_create(void** out_stream) {
  if (!out_stream) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "stream_create: null");
  hipStream_t s = nullptr;
  // Default priority on purpose: mixed stream priorities are not used.
  UK_RETURN_IF_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *out_stream = (void*)s;
  return 0;
}
extern "C" int iree_amd_uk_stream_destroy(void* stream) {
  if (!stream) return 0;
  return check_hip(hipStreamDestroy((hipStream_t)stream), "hipStreamDestroy");
}
extern "C" int iree_amd_uk_stream_synchronize(void* stream) {
  return check_hip(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
}
extern "C" int iree_amd_uk_release_scratch(void) {
  (void)scratch_release_idle();
  return 0;
}
extern "C" const char* iree_amd_uk_last_error(void) { return g_last_error; }
extern "C" const char* iree_amd_uk_last_kernel_path(void) { return g_kernel_path; }
extern "C" uint32_t iree_amd_uk_version(void) { return (0u << 16) | 1u; }
