/*
 * iree_amd_hal_plugin_abi.h - the binary interface between IREE's local HAL
 * executable loader and an executable plugin, restated so that the MI355X
 * plugin builds without the IREE tree.
 *
 * Every type, field order and constant here must stay binary-identical to
 * REF runtime/src/iree/hal/local/executable_plugin.h (version 0.1):
 *   header            :152-176     query function  :185-194
 *   status codes      :221-252     allocator       :278-318
 *   string views      :324-340     resolution bits :345-351
 *   environment       :379-384     resolve params  :386-391
 *   plugin v0 vtable  :404-455
 * Only what a plugin needs is declared; names carry the iree_amd_ prefix so
 * that including the reference header next to this one does not clash.
 */
#ifndef IREE_AMD_HAL_PLUGIN_ABI_H_
#define IREE_AMD_HAL_PLUGIN_ABI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IREE_AMD_HAL_PLUGIN_VERSION_0_1 0x00000001u
#define IREE_AMD_HAL_PLUGIN_QUERY_SYMBOL "iree_hal_executable_plugin_query"

/* feature bits */
#define IREE_AMD_HAL_PLUGIN_FEATURE_STANDALONE (1u << 0)
#define IREE_AMD_HAL_PLUGIN_FEATURE_FULL_STATUS (1u << 1)

/* Status: a pointer-sized value whose low 5 bits are the code; 0 is OK. The
 * codes used here equal iree_amd_uk status codes (both mirror iree_status_code_t). */
typedef struct iree_amd_hal_status_handle_t* iree_amd_hal_plugin_status_t;
#define IREE_AMD_HAL_PLUGIN_STATUS_OK 0
#define IREE_AMD_HAL_PLUGIN_STATUS_INVALID_ARGUMENT 3
#define IREE_AMD_HAL_PLUGIN_STATUS_NOT_FOUND 5
#define IREE_AMD_HAL_PLUGIN_STATUS_RESOURCE_EXHAUSTED 8
#define IREE_AMD_HAL_PLUGIN_STATUS_FAILED_PRECONDITION 9
#define IREE_AMD_HAL_PLUGIN_STATUS_UNAVAILABLE 14
#define iree_amd_hal_plugin_status_from_code(code) \
  ((iree_amd_hal_plugin_status_t)((uintptr_t)(code) & 0x1Fu))

/* Sanitizer the plugin was compiled with (executable_plugin.h:76-100); the
 * runtime refuses a plugin whose sanitizer it was not built with itself. */
#define IREE_AMD_HAL_PLUGIN_SANITIZER_NONE 0
#define IREE_AMD_HAL_PLUGIN_SANITIZER_ADDRESS 1
#define IREE_AMD_HAL_PLUGIN_SANITIZER_MEMORY 2
#define IREE_AMD_HAL_PLUGIN_SANITIZER_THREAD 3
#define IREE_AMD_HAL_PLUGIN_SANITIZER_UNDEFINED 4
/* The kind in force for the translation unit that includes this header, for
 * the header's `sanitizer` field (executable_plugin.h:102-121): clang reports
 * it through __has_feature, gcc through __SANITIZE_ADDRESS__ / _THREAD__. */
#if defined(__has_feature)
#if __has_feature(address_sanitizer)
#define IREE_AMD_HAL_PLUGIN_SANITIZER_KIND IREE_AMD_HAL_PLUGIN_SANITIZER_ADDRESS
#elif __has_feature(memory_sanitizer)
#define IREE_AMD_HAL_PLUGIN_SANITIZER_KIND IREE_AMD_HAL_PLUGIN_SANITIZER_MEMORY
#elif __has_feature(thread_sanitizer)
#define IREE_AMD_HAL_PLUGIN_SANITIZER_KIND IREE_AMD_HAL_PLUGIN_SANITIZER_THREAD
#endif
#endif
#if !defined(IREE_AMD_HAL_PLUGIN_SANITIZER_KIND) && defined(__SANITIZE_ADDRESS__)
#define IREE_AMD_HAL_PLUGIN_SANITIZER_KIND IREE_AMD_HAL_PLUGIN_SANITIZER_ADDRESS
#endif
#if !defined(IREE_AMD_HAL_PLUGIN_SANITIZER_KIND) && defined(__SANITIZE_THREAD__)
#define IREE_AMD_HAL_PLUGIN_SANITIZER_KIND IREE_AMD_HAL_PLUGIN_SANITIZER_THREAD
#endif
#if !defined(IREE_AMD_HAL_PLUGIN_SANITIZER_KIND)
#define IREE_AMD_HAL_PLUGIN_SANITIZER_KIND IREE_AMD_HAL_PLUGIN_SANITIZER_NONE
#endif

typedef struct iree_amd_hal_plugin_header_t {
  uint32_t version;
  const char* name;
  const char* description;
  uint32_t features;
  int32_t sanitizer; /* IREE_AMD_HAL_PLUGIN_SANITIZER_* */
  uint64_t reserved[8];
} iree_amd_hal_plugin_header_t;

/* Host allocator handed to the plugin: ctl(self, command, params, inout_ptr). */
enum {
  IREE_AMD_HAL_PLUGIN_ALLOCATOR_MALLOC = 0,
  IREE_AMD_HAL_PLUGIN_ALLOCATOR_CALLOC = 1,
  IREE_AMD_HAL_PLUGIN_ALLOCATOR_REALLOC = 2,
  IREE_AMD_HAL_PLUGIN_ALLOCATOR_FREE = 3,
};
typedef struct iree_amd_hal_plugin_alloc_params_t {
  size_t byte_length;
} iree_amd_hal_plugin_alloc_params_t;
typedef iree_amd_hal_plugin_status_t (*iree_amd_hal_plugin_allocator_ctl_fn_t)(
    void* self, int32_t command, const void* params, void** inout_ptr);
typedef struct iree_amd_hal_plugin_allocator_t {
  void* self;
  iree_amd_hal_plugin_allocator_ctl_fn_t ctl;
} iree_amd_hal_plugin_allocator_t;

typedef struct iree_amd_hal_plugin_string_view_t {
  const char* data;
  size_t size;
} iree_amd_hal_plugin_string_view_t;
typedef struct iree_amd_hal_plugin_string_pair_t {
  iree_amd_hal_plugin_string_view_t key;
  iree_amd_hal_plugin_string_view_t value;
} iree_amd_hal_plugin_string_pair_t;

#define IREE_AMD_HAL_PLUGIN_RESOLUTION_MISSING_OPTIONAL (1u << 0)

typedef struct iree_amd_hal_plugin_environment_v0_t {
  iree_amd_hal_plugin_allocator_t host_allocator;
} iree_amd_hal_plugin_environment_v0_t;

typedef struct iree_amd_hal_plugin_resolve_params_v0_t {
  size_t count;
  const char* const* symbol_names; /* a leading '?' marks an optional import */
  void** out_fn_ptrs;
  void** out_fn_contexts;
} iree_amd_hal_plugin_resolve_params_v0_t;

typedef struct iree_amd_hal_plugin_v0_t {
  const iree_amd_hal_plugin_header_t* header;
  iree_amd_hal_plugin_status_t (*load)(
      const iree_amd_hal_plugin_environment_v0_t* environment,
      size_t param_count, const iree_amd_hal_plugin_string_pair_t* params,
      void** out_self);
  void (*unload)(void* self);
  iree_amd_hal_plugin_status_t (*resolve)(
      void* self, const iree_amd_hal_plugin_resolve_params_v0_t* params,
      uint32_t* out_resolution);
} iree_amd_hal_plugin_v0_t;

/* The one exported symbol of a plugin library. */
typedef const iree_amd_hal_plugin_header_t** (*iree_amd_hal_plugin_query_fn_t)(
    uint32_t max_version, void* reserved);

/* An import as the generated code calls it, 0 = success
 * (REF runtime/src/iree/hal/local/executable_library.h:157-158,
 * iree_hal_executable_import_v0_t). */
typedef int (*iree_amd_hal_plugin_import_fn_t)(void* params, void* context,
                                               void* reserved);

#ifdef __cplusplus
}
#endif
#endif /* IREE_AMD_HAL_PLUGIN_ABI_H_ */
