// mmt4d through an entry point that allocates nothing.
//
// Some callers cannot call hipMalloc: code under HIP graph capture, tight
// serving loops, harnesses that forbid it. iree_amd_uk_mmt4d_p keeps the
// partial sums of a K split in a buffer it allocates per stream on first use;
// iree_amd_uk_mmt4d_noalloc_p runs the same kernels with that buffer in a device
// array that is part of the library's code object. Contract:
// include/iree_amd_uk.h.
#include "uk_common.h"

#include <mutex>

// Every GPU the library runs on holds its own copy of this array from the
// moment the code object is loaded until the process ends. In host code the
// name is only a handle for hipGetSymbolAddress; the device address obtained
// from it is what kernels are given.
static __device__ __align__(256) unsigned char scratch[IREE_AMD_UK_NOALLOC_SCRATCH_BYTES];

namespace {
// Device address of `scratch` on each device, looked up once per device with
// that device current (every device has its own copy at its own address).
int static_scratch_address(void** out_ptr) {
  static std::mutex mutex;
  static void* address[64] = {nullptr};
  int device = 0;
  UK_RETURN_IF_HIP(hipGetDevice(&device));
  if (device < 0 || device >= 64)
    return uk::fail(IREE_AMD_UK_STATUS_OUT_OF_RANGE, "mmt4d_noalloc: device ordinal %d beyond 63", device);
  std::lock_guard<std::mutex> lock(mutex);
  if (!address[device]) {
    void* ptr = nullptr;
    UK_RETURN_IF_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return uk::fail(IREE_AMD_UK_STATUS_INTERNAL, "mmt4d_noalloc: no address for the scratch array");
    address[device] = ptr;
  }
  *out_ptr = address[device];
  return 0;
}
}  // namespace

extern "C" int iree_amd_uk_mmt4d_noalloc_p(const iree_amd_uk_mmt4d_params_t* params, void* stream) {
  if (!params) return uk::fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: null params");
  // (invalid parameters are reported as by iree_amd_uk_mmt4d_p, before any device call)
  UK_RETURN_IF_ERROR(uk::validate_mmt4d(*params));
  void* ptr = nullptr;
  UK_RETURN_IF_ERROR(static_scratch_address(&ptr));
  // Every scratch request of the call is served from the static array or
  // fails: nothing below reaches the allocating cache.
  uk::ScratchOverride no_allocation(ptr, (size_t)IREE_AMD_UK_NOALLOC_SCRATCH_BYTES, /*strict=*/true);
  return iree_amd_uk_mmt4d_p(params, stream);
}
