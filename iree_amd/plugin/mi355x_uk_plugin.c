/*
 * HAL executable plugin that serves IREE's data-tiling microkernel imports
 * (iree_uk_mmt4d / iree_uk_pack / iree_uk_unpack) from the MI355X library.
 *
 * Shape of a plugin: REF samples/custom_dispatch/cpu/plugin/system_plugin.c
 * (query -> {load, unload, resolve}); a "system" plugin because it opens a
 * shared library and talks to the GPU driver. The runtime loads it with
 *   iree-run-module --device=local-sync --executable_plugin=<this .so> ...
 *
 * What an import receives: the LLVMCPU backend turns a call to an external
 * function that is not linked as bitcode into a call through the import table
 * with ONE pointer to a struct of [results..., arguments..., extra fields...]
 * (REF compiler/src/iree/compiler/Codegen/LLVMCPU/DispatchABI.cpp:1142-1196,
 * 1312-1358). For the microkernel ops the arguments are, per buffer, (base
 * pointer, offset, stride of the outer dimension), then the sizes and flags,
 * then the "processor_data" extra field
 * (REF compiler/src/iree/compiler/Codegen/Common/CPU/CPULowerToUKernels.cpp:104-125,
 * 252-274): field for field the reference's own iree_uk_*_params_t
 * (REF runtime/src/iree/builtins/ukernel/mmt4d_internal.h:14-32,
 * pack_internal.h:12-30, unpack_internal.h:12-29), which is also the layout of
 * iree_amd_uk_*_params_t. Buffers of a local-CPU HAL device are host memory,
 * so the host-pointer entry points are used (they stage through device memory).
 *
 * Two spellings of each import, because results come first in the struct:
 *   mi355x_uk_{mmt4d,pack,unpack}  the op has only its tensor result (which
 *       bufferisation removes), as in example.mlir next to this file and in
 *       REF samples/custom_dispatch/cpu/plugin/system_ukernel.mlir:50-62: the
 *       struct IS the parameter struct.
 *   iree_uk_{mmt4d,pack,unpack}    the op as the llvm-cpu lowering builds it,
 *       with an extra i32 result (REF CPULowerToUKernels.cpp:157-168): the
 *       struct is {int32 result; <padding to 8>; parameter struct}; the import
 *       stores 0 into the result.
 *
 * Load parameters (--executable_plugin=path?key=value pairs reach load()):
 *   uk_library=<path>   the MI355X microkernel library; default: the
 *                       IREE_AMD_UK_LIBRARY environment variable, else
 *                       libiree_amd_uk.so next to ../csrc relative to this
 *                       plugin, else the dynamic loader's search path.
 */
#define _GNU_SOURCE
#include <dlfcn.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "iree_amd_hal_plugin_abi.h"
#include "iree_amd_uk.h"

typedef int (*pool_create_fn_t)(iree_amd_uk_host_pool_t**);
typedef void (*pool_destroy_fn_t)(iree_amd_uk_host_pool_t*);
typedef int (*mmt4d_host_fn_t)(iree_amd_uk_host_pool_t*, const iree_amd_uk_mmt4d_params_t*);
typedef int (*pack_host_fn_t)(iree_amd_uk_host_pool_t*, const iree_amd_uk_pack_params_t*);
typedef int (*unpack_host_fn_t)(iree_amd_uk_host_pool_t*, const iree_amd_uk_unpack_params_t*);
typedef int (*release_scratch_fn_t)(void);
typedef const char* (*last_error_fn_t)(void);

/* One per load(): several instances may live in one process
 * (REF runtime/src/iree/hal/local/executable_plugin.h:415-418), so everything a
 * call needs hangs off this struct - the staging pool included - and nothing is
 * global. The imports are called from arbitrary threads concurrently
 * (REF samples/custom_dispatch/cpu/plugin/system_plugin.c:21-25): the struct is
 * read-only after load and the pool hands every call a slot of its own. */
typedef struct mi355x_plugin_t {
  iree_amd_hal_plugin_allocator_t host_allocator;
  void* library;
  iree_amd_uk_host_pool_t* pool;
  pool_destroy_fn_t pool_destroy;
  mmt4d_host_fn_t mmt4d;
  pack_host_fn_t pack;
  unpack_host_fn_t unpack;
  release_scratch_fn_t release_scratch;
  last_error_fn_t last_error;
} mi355x_plugin_t;

static int report(mi355x_plugin_t* plugin, const char* what, int status) {
  if (status != 0) {
    const char* msg = plugin->last_error ? plugin->last_error() : "";
    fprintf(stderr, "mi355x_uk plugin: %s failed with status %d: %s\n", what, status, msg);
  }
  return status;
}

/* Imports: int fn(void* params, void* context, void* reserved), 0 = success. */
static int import_mmt4d(void* params, void* context, void* reserved) {
  (void)reserved;
  mi355x_plugin_t* plugin = (mi355x_plugin_t*)context;
  return report(plugin, "mmt4d", plugin->mmt4d(plugin->pool, (const iree_amd_uk_mmt4d_params_t*)params));
}
static int import_pack(void* params, void* context, void* reserved) {
  (void)reserved;
  mi355x_plugin_t* plugin = (mi355x_plugin_t*)context;
  return report(plugin, "pack", plugin->pack(plugin->pool, (const iree_amd_uk_pack_params_t*)params));
}
static int import_unpack(void* params, void* context, void* reserved) {
  (void)reserved;
  mi355x_plugin_t* plugin = (mi355x_plugin_t*)context;
  return report(plugin, "unpack", plugin->unpack(plugin->pool, (const iree_amd_uk_unpack_params_t*)params));
}

/* The llvm-cpu form: a leading i32 result, then the parameters at the next
 * 8-byte boundary (the first parameter is a pointer). */
typedef struct with_result_t {
  int32_t result;
  int32_t padding;
  char params[];
} with_result_t;
static int import_mmt4d_r(void* params, void* context, void* reserved) {
  with_result_t* w = (with_result_t*)params;
  w->result = 0;
  return import_mmt4d(w->params, context, reserved);
}
static int import_pack_r(void* params, void* context, void* reserved) {
  with_result_t* w = (with_result_t*)params;
  w->result = 0;
  return import_pack(w->params, context, reserved);
}
static int import_unpack_r(void* params, void* context, void* reserved) {
  with_result_t* w = (with_result_t*)params;
  w->result = 0;
  return import_unpack(w->params, context, reserved);
}

static int key_is(const iree_amd_hal_plugin_string_view_t* key, const char* name) {
  return key->size == strlen(name) && memcmp(key->data, name, key->size) == 0;
}

/* Opens the microkernel library: explicit path, environment, beside the plugin, search path. */
static void* open_uk_library(const char* explicit_path) {
  if (explicit_path && explicit_path[0]) return dlopen(explicit_path, RTLD_NOW | RTLD_LOCAL);
  const char* env = getenv("IREE_AMD_UK_LIBRARY");
  if (env && env[0]) return dlopen(env, RTLD_NOW | RTLD_LOCAL);
  Dl_info info;
  if (dladdr((void*)&open_uk_library, &info) && info.dli_fname) {
    char path[4096];
    const char* slash = strrchr(info.dli_fname, '/');
    const int dir_len = slash ? (int)(slash - info.dli_fname) : 0;
    if (dir_len > 0 && dir_len + 32 < (int)sizeof(path)) {
      snprintf(path, sizeof(path), "%.*s/../csrc/libiree_amd_uk.so", dir_len, info.dli_fname);
      void* lib = dlopen(path, RTLD_NOW | RTLD_LOCAL);
      if (lib) return lib;
      snprintf(path, sizeof(path), "%.*s/libiree_amd_uk.so", dir_len, info.dli_fname);
      lib = dlopen(path, RTLD_NOW | RTLD_LOCAL);
      if (lib) return lib;
    }
  }
  return dlopen("libiree_amd_uk.so", RTLD_NOW | RTLD_LOCAL);
}

static iree_amd_hal_plugin_status_t plugin_load(
    const iree_amd_hal_plugin_environment_v0_t* environment, size_t param_count,
    const iree_amd_hal_plugin_string_pair_t* params, void** out_self) {
  *out_self = NULL;
  mi355x_plugin_t* plugin = NULL;
  iree_amd_hal_plugin_alloc_params_t alloc = {sizeof(*plugin)};
  iree_amd_hal_plugin_status_t status = environment->host_allocator.ctl(
      environment->host_allocator.self, IREE_AMD_HAL_PLUGIN_ALLOCATOR_MALLOC, &alloc,
      (void**)&plugin);
  if (status) return status;
  memset(plugin, 0, sizeof(*plugin));
  plugin->host_allocator = environment->host_allocator;

  char path[4096] = {0};
  for (size_t i = 0; i < param_count; ++i) {
    if (key_is(&params[i].key, "uk_library") && params[i].value.size < sizeof(path)) {
      memcpy(path, params[i].value.data, params[i].value.size);  /* views are not NUL-terminated */
      path[params[i].value.size] = 0;
    }
  }
  plugin->library = open_uk_library(path);
  pool_create_fn_t pool_create = NULL;
  if (plugin->library) {
    pool_create = (pool_create_fn_t)dlsym(plugin->library, "iree_amd_uk_host_pool_create");
    plugin->pool_destroy = (pool_destroy_fn_t)dlsym(plugin->library, "iree_amd_uk_host_pool_destroy");
    plugin->mmt4d = (mmt4d_host_fn_t)dlsym(plugin->library, "iree_amd_uk_mmt4d_host_pooled");
    plugin->pack = (pack_host_fn_t)dlsym(plugin->library, "iree_amd_uk_pack_host_pooled");
    plugin->unpack = (unpack_host_fn_t)dlsym(plugin->library, "iree_amd_uk_unpack_host_pooled");
    plugin->release_scratch = (release_scratch_fn_t)dlsym(plugin->library, "iree_amd_uk_release_scratch");
    plugin->last_error = (last_error_fn_t)dlsym(plugin->library, "iree_amd_uk_last_error");
  }
  const int have_entry_points = plugin->library && pool_create && plugin->pool_destroy && plugin->mmt4d &&
                                plugin->pack && plugin->unpack;
  /* (creating the pool touches no device: its streams and buffers come with the first call) */
  if (!have_entry_points || pool_create(&plugin->pool) != 0 || !plugin->pool) {
    fprintf(stderr, "mi355x_uk plugin: cannot load the microkernel library: %s\n",
            !plugin->library ? dlerror() : !have_entry_points ? "missing entry points" : "no staging pool");
    if (plugin->library) dlclose(plugin->library);
    void* p = plugin;
    environment->host_allocator.ctl(environment->host_allocator.self,
                                    IREE_AMD_HAL_PLUGIN_ALLOCATOR_FREE, NULL, &p);
    return iree_amd_hal_plugin_status_from_code(IREE_AMD_HAL_PLUGIN_STATUS_UNAVAILABLE);
  }
  *out_self = plugin;
  return iree_amd_hal_plugin_status_from_code(IREE_AMD_HAL_PLUGIN_STATUS_OK);
}

static void plugin_unload(void* self) {
  mi355x_plugin_t* plugin = (mi355x_plugin_t*)self;
  if (!plugin) return;
  iree_amd_hal_plugin_allocator_t allocator = plugin->host_allocator;
  /* Everything is freed here: the library may be closed right after
   * (REF executable_plugin.h:424-427). No import is running any more. */
  if (plugin->pool) plugin->pool_destroy(plugin->pool);
  if (plugin->release_scratch) plugin->release_scratch();
  if (plugin->library) dlclose(plugin->library);
  void* p = plugin;
  allocator.ctl(allocator.self, IREE_AMD_HAL_PLUGIN_ALLOCATOR_FREE, NULL, &p);
}

static const struct {
  const char* name;
  iree_amd_hal_plugin_import_fn_t fn;
} kImports[] = {
    {"iree_uk_mmt4d", import_mmt4d_r},   {"iree_uk_pack", import_pack_r},
    {"iree_uk_unpack", import_unpack_r}, {"mi355x_uk_mmt4d", import_mmt4d},
    {"mi355x_uk_pack", import_pack},     {"mi355x_uk_unpack", import_unpack},
};

static iree_amd_hal_plugin_status_t plugin_resolve(
    void* self, const iree_amd_hal_plugin_resolve_params_v0_t* params,
    uint32_t* out_resolution) {
  *out_resolution = 0;
  int any_required_not_found = 0;
  for (size_t i = 0; i < params->count; ++i) {
    if (params->out_fn_ptrs[i]) continue;  /* another provider already resolved it */
    const char* name = params->symbol_names[i];
    const int optional = name && name[0] == '?';
    if (optional) ++name;
    int found = 0;
    for (size_t j = 0; name && j < sizeof(kImports) / sizeof(kImports[0]); ++j) {
      if (strcmp(name, kImports[j].name) == 0) {
        params->out_fn_ptrs[i] = (void*)kImports[j].fn;
        params->out_fn_contexts[i] = self;
        found = 1;
        break;
      }
    }
    if (!found) {
      if (optional) *out_resolution |= IREE_AMD_HAL_PLUGIN_RESOLUTION_MISSING_OPTIONAL;
      else any_required_not_found = 1;
    }
  }
  return iree_amd_hal_plugin_status_from_code(any_required_not_found
                                                  ? IREE_AMD_HAL_PLUGIN_STATUS_NOT_FOUND
                                                  : IREE_AMD_HAL_PLUGIN_STATUS_OK);
}

__attribute__((visibility("default"))) const iree_amd_hal_plugin_header_t**
iree_hal_executable_plugin_query(uint32_t max_version, void* reserved) {
  (void)reserved;
  static const iree_amd_hal_plugin_header_t header = {
      .version = IREE_AMD_HAL_PLUGIN_VERSION_0_1,
      .name = "mi355x_uk",
      .description = "MI355X (gfx950) data-tiled matmul microkernels: iree_uk_mmt4d / pack / unpack",
      .features = 0, /* not standalone: opens a shared library and the GPU driver */
      .sanitizer = IREE_AMD_HAL_PLUGIN_SANITIZER_KIND,
  };
  static const iree_amd_hal_plugin_v0_t plugin = {
      .header = &header,
      .load = plugin_load,
      .unload = plugin_unload,
      .resolve = plugin_resolve,
  };
  return max_version <= IREE_AMD_HAL_PLUGIN_VERSION_0_1
             ? (const iree_amd_hal_plugin_header_t**)&plugin
             : NULL;
}
