// Loader and dispatcher of a code object of hand-written kernels, doing what
// IREE's HIP HAL driver does with a `hal.executable.source` object (contract:
// include/iree_amd_hal_executable.h; reference:
// runtime/src/iree/hal/drivers/hip/native_executable.c:180-253 and
// runtime/src/iree/hal/drivers/hip/stream_command_buffer.c:519-581).
// Host code only.
#include "iree_amd_hal_executable.h"

#include <string>
#include <vector>

#include "uk_common.h"

struct iree_amd_hal_executable_t {
  hipModule_t module = nullptr;
  int device = 0;
  int max_shared_memory = 0;
  struct Export {
    std::string name;
    hipFunction_t function;
    uint32_t block[3];
    uint32_t shared_memory_size;
  };
  std::vector<Export> exports;
};

using namespace uk;

extern "C" int iree_amd_hal_executable_load(const void* data, size_t size,
                                            iree_amd_hal_executable_t** out_executable) {
  if (!out_executable) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "hal_executable_load: null out pointer");
  *out_executable = nullptr;
  if (!data || size < 64)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "hal_executable_load: no code object given");
  iree_amd_hal_executable_t* e = new iree_amd_hal_executable_t();
  int st = check_hip(hipGetDevice(&e->device), "hipGetDevice");
  if (!st) st = check_hip(hipModuleLoadDataEx(&e->module, data, 0, nullptr, nullptr), "hipModuleLoadDataEx");
  if (!st)
    st = check_hip(hipDeviceGetAttribute(&e->max_shared_memory, hipDeviceAttributeMaxSharedMemoryPerBlock,
                                         e->device),
                   "hipDeviceGetAttribute");
  if (st) {
    if (e->module) (void)hipModuleUnload(e->module);
    delete e;
    return st;
  }
  *out_executable = e;
  return 0;
}

extern "C" int iree_amd_hal_executable_add_export(iree_amd_hal_executable_t* e, const char* name,
                                                  uint32_t block_x, uint32_t block_y,
                                                  uint32_t block_z, uint32_t shared_memory_size,
                                                  int32_t* out_ordinal) {
  if (!e || !name || !out_ordinal)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "hal_executable_add_export: null argument");
  if (block_x == 0 || block_y == 0 || block_z == 0 || (uint64_t)block_x * block_y * block_z > 1024)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "hal_executable_add_export: block size %u x %u x %u",
                block_x, block_y, block_z);
  hipFunction_t fn = nullptr;
  if (hipModuleGetFunction(&fn, e->module, name) != hipSuccess || !fn) {
    (void)hipGetLastError();
    return fail(IREE_AMD_UK_STATUS_NOT_FOUND, "exported module function '%s' not found", name);
  }
  if ((int64_t)shared_memory_size > e->max_shared_memory)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT,
                "function '%s' requested shared memory size of %u bytes larger than allowed size of %d bytes",
                name, shared_memory_size, e->max_shared_memory);
  UK_RETURN_IF_HIP(hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)shared_memory_size));
  e->exports.push_back({name, fn, {block_x, block_y, block_z}, shared_memory_size});
  *out_ordinal = (int32_t)e->exports.size() - 1;
  return 0;
}

extern "C" int iree_amd_hal_executable_dispatch(iree_amd_hal_executable_t* e, int32_t ordinal,
                                                uint32_t workgroup_x, uint32_t workgroup_y,
                                                uint32_t workgroup_z, const void* const* bindings,
                                                size_t binding_count, const uint32_t* push_constants,
                                                size_t push_constant_count, void* stream) {
  if (!e || ordinal < 0 || (size_t)ordinal >= e->exports.size())
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "hal_executable_dispatch: no export %d", ordinal);
  if ((binding_count && !bindings) || (push_constant_count && !push_constants) ||
      binding_count + push_constant_count > 256)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "hal_executable_dispatch: bad parameter lists");
  // an empty grid is a no-op (HIP rejects it)
  if (workgroup_x == 0 || workgroup_y == 0 || workgroup_z == 0) return 0;
  int dev = -1;
  UK_RETURN_IF_HIP(hipGetDevice(&dev));
  if (dev != e->device)
    return fail(IREE_AMD_UK_STATUS_FAILED_PRECONDITION,
                "hal_executable_dispatch: loaded on device %d, current device is %d", e->device, dev);
  const iree_amd_hal_executable_t::Export& x = e->exports[ordinal];
  // One pointer-sized payload slot per kernel parameter: the bindings, then the
  // push constants, each a 32-bit value at the start of its slot.
  const size_t count = binding_count + push_constant_count;
  std::vector<uint64_t> payload(count ? count : 1, 0);
  std::vector<void*> params(count ? count : 1, nullptr);
  for (size_t i = 0; i < count; ++i) params[i] = &payload[i];
  for (size_t i = 0; i < binding_count; ++i) payload[i] = (uint64_t)(uintptr_t)bindings[i];
  for (size_t i = 0; i < push_constant_count; ++i)
    *(uint32_t*)&payload[binding_count + i] = push_constants[i];
  return check_hip(hipModuleLaunchKernel(x.function, workgroup_x, workgroup_y, workgroup_z, x.block[0],
                                         x.block[1], x.block[2], x.shared_memory_size,
                                         (hipStream_t)stream, params.data(), nullptr),
                   "hipModuleLaunchKernel");
}

extern "C" void iree_amd_hal_executable_release(iree_amd_hal_executable_t* e) {
  if (!e) return;
  if (e->module) (void)hipModuleUnload(e->module);
  delete e;
}
