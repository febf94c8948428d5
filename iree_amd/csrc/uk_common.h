// Shared declarations of the gfx950 ukernel library (internal, C++/HIP only).
//
// The public boundary is include/iree_amd_uk.h. Everything here is private to
// the .hip translation units: error plumbing, element-type tables and the
// launch functions each kernel file exports to uk_api.hip.
#ifndef IREE_AMD_CSRC_UK_COMMON_H_
#define IREE_AMD_CSRC_UK_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "iree_amd_uk.h"

namespace uk {

// Records a message for iree_amd_uk_last_error() on this thread and returns
// `status`, so call sites read `return fail(STATUS, "...")`.
int fail(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Records which kernel family served the calling thread's last call, for
// iree_amd_uk_last_kernel_path() (a static string; tests and callers that tune
// use it to tell a matrix-core kernel from the element-wise one).
void note_kernel_path(const char* name);

// Converts a hipError_t of a runtime call or of a kernel launch to a status.
int check_hip(hipError_t err, const char* what);

#define UK_RETURN_IF_HIP(expr)                                   \
  do {                                                           \
    int uk_status_ = ::uk::check_hip((expr), #expr);             \
    if (uk_status_) return uk_status_;                           \
  } while (0)

#define UK_RETURN_IF_ERROR(expr)       \
  do {                                 \
    int uk_status_ = (expr);           \
    if (uk_status_) return uk_status_; \
  } while (0)

// One bit per device ordinal on which a kernel's attributes have been set
// (hipFuncSetAttribute belongs to the kernel on ONE device). Host threads call
// concurrently: test() / set() are atomic; two threads may both find the bit
// clear and both make the idempotent call.
class PerDeviceOnce {
 public:
  bool done(int dev) const {
    return dev >= 0 && dev < 64 && ((bits_.load(std::memory_order_acquire) >> dev) & 1);
  }
  void mark(int dev) {
    if (dev >= 0 && dev < 64) bits_.fetch_or(1ull << dev, std::memory_order_release);
  }

 private:
  std::atomic<unsigned long long> bits_{0};
};

// Element-type facts of an mmt4d type tuple.
struct Mmt4dTypeInfo {
  int lhs_bits;
  int rhs_bits;
  int out_bytes;
};
// Returns false for an unknown type value.
bool mmt4d_type_info(uint32_t flags, Mmt4dTypeInfo* out);
// 0 for an unknown / unsupported type value.
int pack_elem_bytes(uint32_t flags);
int unpack_elem_bytes(uint32_t flags);

// Validation shared by the device and the host-pointer entry points.
int validate_mmt4d(const iree_amd_uk_mmt4d_params_t& p);
int validate_pack(const iree_amd_uk_pack_params_t& p);
int validate_unpack(const iree_amd_uk_unpack_params_t& p);

// Kernel launchers (each defined next to its kernels). All assume validated
// parameters and non-degenerate sizes.
int launch_mmt4d_generic(const iree_amd_uk_mmt4d_params_t& p, hipStream_t s);
// Returns true when a MFMA kernel exists for (type, M0, N0, K0).
bool mmt4d_mfma_supported(uint32_t flags, int M0, int N0, int K0);
bool mmt4d_skinny_supported(uint32_t flags, int M0, int N0, int K0);
int launch_mmt4d_skinny(const iree_amd_uk_mmt4d_params_t& p, hipStream_t s);
int launch_matmul_rows_skinny(const iree_amd_uk_mmt4d_params_t& p, int64_t M, int64_t out_cols, hipStream_t s);
// S8S4S32 through the s8 x s8 kernels on a widened copy of the right-hand side
// (uk_mmt4d_s8s4.hip); NOT_FOUND when the call must take the element-wise kernel.
bool mmt4d_s8s4_widened_supported(uint32_t flags, int M0, int N0, int K0);
int launch_mmt4d_s8s4_widened(const iree_amd_uk_mmt4d_params_t& p, hipStream_t s);
// 16-bit left-hand sides as int8 digit planes on the matrix cores
// (uk_mmt4d_s16.hip); NOT_FOUND when the call must take the element-wise kernel
// (small problems, no scratch memory).
bool mmt4d_s16_planes_supported(uint32_t flags, int M0, int N0, int K0);
int launch_mmt4d_s16_planes(const iree_amd_uk_mmt4d_params_t& p, hipStream_t s);
// Also needs alignment / stride properties of the actual call; returns
// NOT_FOUND (without recording an error) when the call must take the generic
// kernel instead.
int launch_mmt4d_mfma(const iree_amd_uk_mmt4d_params_t& p, hipStream_t s);
int launch_batch_mmt4d_skinny(const iree_amd_uk_mmt4d_params_t& p, int64_t batch, int64_t lhs_batch_stride,
                              int64_t rhs_batch_stride, int64_t out_batch_stride, hipStream_t s);
int launch_batch_mmt4d_mfma(const iree_amd_uk_mmt4d_params_t& p, int64_t batch, int64_t lhs_batch_stride,
                            int64_t rhs_batch_stride, int64_t out_batch_stride, hipStream_t s);
// (`batch` problems whose operands lie `*_batch_stride` elements apart run as
// the planes of one launch; NOT_FOUND when the strides are not whole 16 bytes)
int launch_mmt4d_unpack_mfma(const iree_amd_uk_mmt4d_params_t& p, int64_t out_rows,
                             int64_t out_cols, float out_scale, int64_t batch, int64_t lhs_batch_stride,
                             int64_t rhs_batch_stride, int64_t out_batch_stride, hipStream_t s);
int launch_matmul_packed_rhs_mfma(const iree_amd_uk_mmt4d_params_t& p, int64_t out_rows,
                                  int64_t out_cols, float out_scale, int64_t batch, int64_t lhs_batch_stride,
                                  int64_t rhs_batch_stride, int64_t out_batch_stride, hipStream_t s);
int launch_mmt4d_silu_mul_mfma(const iree_amd_uk_mmt4d_params_t& p, float gate_scale,
                               float up_scale, float inv_out_scale, hipStream_t s);

// Sums the partial results of a K split (tiled, accumulator type) in slice
// order into the result, tiled or row-major: what the kernel's own epilogue
// would have written (defined in uk_mmt4d_mfma.hip).
struct KSplitReduceArgs {
  const void* partials;      // slices x M x N tiles of 32x32 accumulator elements
  int slices;
  int M, N;                  // outer tile counts
  int64_t flat_elems;        // > 0: partials and result are dense arrays of so many elements (a multiple of 4) instead
  void* out;                 // offset applied
  int64_t out_stride_bytes;
  int accumulate, row_major_out, out_rows, out_cols;
  float out_scale;
  int acc_is_float;          // else int32
  int out_kind;              // 0 = accumulator type, 1 = f16, 2 = bf16
};
int launch_ksplit_reduce(const KSplitReduceArgs& r, hipStream_t s);
// Device memory beyond a call's operands (the partial sums of a K split, a
// packed copy of a row-major left-hand side) on stream `s` of the current
// device: one buffer per stream, kept and reused by later calls (work on one
// stream is ordered, so they cannot overlap), grown when a call needs more.
// The object must stay alive until the last launch that uses the memory has
// been queued: until then the buffer is neither evicted nor replaced. ptr() is
// nullptr when the memory cannot be had (the call then takes its fallback).
//
// A ScratchOverride on the calling thread replaces the cache for the calls made
// under it: they get `ptr` when they need at most `bytes` and nothing
// otherwise. With `strict`, a call that needs more does not fall back but fails
// (overflowed() below): that is the entry point that allocates nothing.
class ScratchLease {
 public:
  ScratchLease(hipStream_t s, size_t bytes);
  ~ScratchLease();
  ScratchLease(const ScratchLease&) = delete;
  ScratchLease& operator=(const ScratchLease&) = delete;
  void* ptr() const { return ptr_; }
  // The calling thread runs under a strict override that is too small for
  // this request: the caller returns scratch_overflow_status() instead of
  // falling back.
  bool overflowed() const { return overflowed_; }

 private:
  void* ptr_ = nullptr;
  uint64_t id_ = 0;
  bool overflowed_ = false;
};
// Scratch memory a call cannot do without: the stream's cached buffer when it
// can be leased, otherwise an allocation of the call's own, made and freed in
// stream order on the caller's stream (hipMallocAsync / hipFreeAsync: some
// tens of microseconds of host time, which is why it is only the fallback).
// That covers the per-thread default stream, a buffer another thread holds on
// the same stream, and a full cache. ptr() is nullptr only under a strict
// override that is too small, or when the device is out of memory.
class CallScratch {
 public:
  CallScratch(hipStream_t s, size_t bytes) : lease_(s, bytes), stream_(s) {
    if (!lease_.ptr() && !lease_.overflowed() && bytes) {
      if (hipMallocAsync(&own_, bytes, s) != hipSuccess) {
        (void)hipGetLastError();
        own_ = nullptr;
      }
    }
  }
  ~CallScratch() {
    if (own_ && hipFreeAsync(own_, stream_) != hipSuccess) (void)hipGetLastError();
  }
  CallScratch(const CallScratch&) = delete;
  CallScratch& operator=(const CallScratch&) = delete;
  void* ptr() const { return lease_.ptr() ? lease_.ptr() : own_; }
  bool overflowed() const { return lease_.overflowed(); }

 private:
  ScratchLease lease_;
  void* own_ = nullptr;
  hipStream_t stream_;
};
class ScratchOverride {
 public:
  ScratchOverride(void* ptr, size_t bytes, bool strict);
  ~ScratchOverride();
  ScratchOverride(const ScratchOverride&) = delete;
  ScratchOverride& operator=(const ScratchOverride&) = delete;

 private:
  void* prev_ptr_;
  size_t prev_bytes_;
  bool prev_strict_, prev_active_;
};
// Records the error of a request of `bytes` that a strict override cannot
// serve and returns its status (RESOURCE_EXHAUSTED).
int scratch_overflow_status(const char* what, size_t bytes);
// Frees the cached buffers that no call is using; returns how many.
size_t scratch_release_idle();

int launch_pack(const iree_amd_uk_pack_params_t& p, hipStream_t s);
int launch_unpack(const iree_amd_uk_unpack_params_t& p, hipStream_t s);

int launch_dequant_matmul_i4(const void* x, const void* w, const void* scale,
                             const void* zp, void* out, int64_t M, int64_t N,
                             int64_t K, int64_t group_size, uint32_t flags,
                             hipStream_t s);
int launch_dequant_matmul_i4_reassoc(const void* x, const void* w, const void* scale,
                                     const void* zp, void* out, int64_t M, int64_t N,
                                     int64_t K, int64_t group_size, uint32_t flags,
                                     hipStream_t s);
int launch_quantize_groups_i16(const void* x, void* q, void* scale_x, void* group_sum, int64_t M,
                               int64_t K, int64_t gs, hipStream_t s);
int launch_pack_i4_weights(const void* src, void* dst, int64_t N, int64_t K, hipStream_t s);
int launch_quantize_f16_to_f8e4m3(const void* in, void* out, int64_t n,
                                  float inv_scale, hipStream_t s);
int launch_quantize_pack_f8e4m3(const void* in, int64_t ld, void* out, int64_t out_stride0, int64_t rows,
                                int64_t cols, float inv_scale, hipStream_t s);
int launch_silu_mul_quantize(const void* gate, const void* up, void* out,
                             int64_t rows, int64_t cols, int64_t ld,
                             float gate_scale, float up_scale,
                             float inv_out_scale, hipStream_t s);
int launch_silu_mul_quantize_tiled(const void* acc, int64_t acc_stride0, int64_t gate_tile0,
                                   int64_t up_tile0, void* out, int64_t out_stride0, int64_t M1,
                                   int64_t N1, float gate_scale, float up_scale,
                                   float inv_out_scale, hipStream_t s);
int launch_scale_f32(void* buf, int64_t n, float scale, hipStream_t s);
int launch_mfma_probe(uint32_t type_flag, const void* operands, int64_t iters, void* sink,
                      int64_t* out_ops_per_launch, hipStream_t s);

int launch_copy_probe(const void* src, void* dst, int64_t bytes, int mode, int blocks_per_cu, hipStream_t s);

// Number of compute units of the current device (cached per device).
int device_cu_count();

__host__ __device__ static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace uk

#endif  // IREE_AMD_CSRC_UK_COMMON_H_
