// mmt4d with a signed 4-bit right-hand side (S8S4S32, reference
// runtime/src/iree/builtins/ukernel/mmt4d_tile_generic.c:81-142,
// exported_bits.h:29-41) on the matrix cores: the packed right-hand side is
// widened to int8 once, tile layout unchanged, into the stream's scratch
// buffer, and the s8 x s8 kernels run on that copy. The widening pass reads
// half a byte and writes one byte per weight, against 2 x M operations per
// weight in the matmul, so it is noise for anything but a handful of rows; the
// integer results are those of the element-wise kernel bit for bit.
#include "uk_common.h"

namespace uk {
namespace {

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 4 nibbles held in the low halves of 4 bytes -> 4 sign-extended bytes:
// (x ^ 8) - 8 per byte, the subtraction kept from borrowing across bytes.
__device__ __forceinline__ uint32_t sign_extend_nibbles(uint32_t low_halves) {
  const uint32_t t = low_halves ^ 0x08080808u;
  return ((t | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
}

// Element 2 i is the low nibble of byte i, element 2 i + 1 the high one.
__device__ __forceinline__ u32x2 widen_word(uint32_t w) {
  const uint32_t lo = sign_extend_nibbles(w & 0x0F0F0F0Fu), hi = sign_extend_nibbles((w >> 4) & 0x0F0F0F0Fu);
  return u32x2{__builtin_amdgcn_perm(hi, lo, 0x05010400u), __builtin_amdgcn_perm(hi, lo, 0x07030602u)};
}

// rows x units_per_row units of 8 source bytes -> 16 destination bytes.
__global__ __launch_bounds__(256) void widen_s4_kernel(const uint8_t* src, int64_t src_row_bytes, uint8_t* dst,
                                                       int64_t units_per_row, int64_t rows) {
  const int64_t total = rows * units_per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = i / units_per_row, u = i - row * units_per_row;
    const u32x2 v = *(const u32x2*)(src + row * src_row_bytes + u * 8);
    const u32x2 a = widen_word(v.x), b = widen_word(v.y);
    *(u32x4*)(dst + i * 16) = u32x4{a.x, a.y, b.x, b.y};
  }
}

}  // namespace

bool mmt4d_s8s4_widened_supported(uint32_t flags, int M0, int N0, int K0) {
  if ((flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) != IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S4S32) return false;
  const uint32_t as_s8 = (flags & ~(uint32_t)IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) | IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32;
  return mmt4d_mfma_supported(as_s8, M0, N0, K0) || mmt4d_skinny_supported(as_s8, M0, N0, K0);
}

int launch_mmt4d_s8s4_widened(const iree_amd_uk_mmt4d_params_t& p, hipStream_t s) {
  if (!mmt4d_s8s4_widened_supported(p.flags, p.M0, p.N0, p.K0)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int64_t row_elems = p.K * p.N0 * p.K0;       // of one outer row of the right-hand side
  // whole 8-byte units, 8-byte aligned, in every outer row
  if (p.K == 0 || row_elems % 16 || p.rhs_offset % 16 || p.rhs_stride0 % 16) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const uint8_t* src = (const uint8_t*)p.rhs_buffer + p.rhs_offset / 2;
  if ((uintptr_t)src % 8) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int64_t bytes = p.N * row_elems;
  ScratchLease lease(s, (size_t)bytes);
  // (no memory, or a caller that brings too little of its own: the element-wise
  // kernel needs none)
  if (!lease.ptr()) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int64_t units = row_elems / 16, total = units * p.N;
  int64_t blocks = ceil_div(total, (int64_t)256);
  const int64_t max_blocks = (int64_t)device_cu_count() * 32;
  if (blocks > max_blocks) blocks = max_blocks;
  hipLaunchKernelGGL(widen_s4_kernel, dim3((unsigned)blocks), dim3(256), 0, s, src, p.rhs_stride0 / 2,
                     (uint8_t*)lease.ptr(), units, p.N);
  UK_RETURN_IF_HIP(hipGetLastError());
  iree_amd_uk_mmt4d_params_t q = p;
  q.flags = (p.flags & ~(uint32_t)IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) | IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32;
  q.rhs_buffer = lease.ptr();
  q.rhs_offset = 0;
  q.rhs_stride0 = row_elems;
  // The stream's scratch buffer holds the widened operand until the matmul has
  // been queued: the matmul itself runs without scratch memory (no K split).
  ScratchOverride none(nullptr, 0, /*strict=*/false);
  return iree_amd_uk_mmt4d_p(&q, s);
}

}  // namespace uk
