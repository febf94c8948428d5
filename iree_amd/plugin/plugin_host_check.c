/*
 * A host program in plain C that drives the plugin the way IREE's executable
 * plugin manager does (REF runtime/src/iree/hal/local/executable_plugin_manager.c
 * and plugins/system_library_plugin.c): dlopen, query, load with a host
 * allocator, resolve the three imports, call them on HOST buffers with the
 * reference's parameter structs, unload. It computes a small i8 matmul through
 * pack -> mmt4d -> unpack and compares it with a plain triple loop.
 *
 *   plugin_host_check <plugin.so> [<libiree_amd_uk.so>]
 *
 * Exit status 0 and "OK" on success. Needs a GPU (the imports run there).
 */
#define _GNU_SOURCE
#include <dlfcn.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "iree_amd_hal_plugin_abi.h"
#include "iree_amd_uk.h"

static int g_live_allocations = 0;

static iree_amd_hal_plugin_status_t host_allocator_ctl(void* self, int32_t command,
                                                       const void* params, void** inout_ptr) {
  (void)self;
  switch (command) {
    case IREE_AMD_HAL_PLUGIN_ALLOCATOR_MALLOC:
    case IREE_AMD_HAL_PLUGIN_ALLOCATOR_CALLOC: {
      const size_t n = ((const iree_amd_hal_plugin_alloc_params_t*)params)->byte_length;
      *inout_ptr = calloc(1, n);
      if (!*inout_ptr) return iree_amd_hal_plugin_status_from_code(IREE_AMD_HAL_PLUGIN_STATUS_RESOURCE_EXHAUSTED);
      ++g_live_allocations;
      return 0;
    }
    case IREE_AMD_HAL_PLUGIN_ALLOCATOR_FREE:
      free(*inout_ptr);
      --g_live_allocations;
      return 0;
    default:
      return iree_amd_hal_plugin_status_from_code(12 /* unimplemented */);
  }
}

#define CHECK(cond, ...)                       \
  do {                                         \
    if (!(cond)) {                             \
      fprintf(stderr, "FAILED: " __VA_ARGS__); \
      fprintf(stderr, "\n");                   \
      return 1;                                \
    }                                          \
  } while (0)

int main(int argc, char** argv) {
  CHECK(argc >= 2, "usage: %s <plugin.so> [<libiree_amd_uk.so>]", argv[0]);
  void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  CHECK(lib, "dlopen %s: %s", argv[1], dlerror());
  iree_amd_hal_plugin_query_fn_t query =
      (iree_amd_hal_plugin_query_fn_t)dlsym(lib, IREE_AMD_HAL_PLUGIN_QUERY_SYMBOL);
  CHECK(query, "no %s", IREE_AMD_HAL_PLUGIN_QUERY_SYMBOL);
  const iree_amd_hal_plugin_v0_t* plugin =
      (const iree_amd_hal_plugin_v0_t*)query(IREE_AMD_HAL_PLUGIN_VERSION_0_1, NULL);
  CHECK(plugin && plugin->header->version == IREE_AMD_HAL_PLUGIN_VERSION_0_1, "query");
  printf("plugin %s: %s\n", plugin->header->name, plugin->header->description);

  iree_amd_hal_plugin_environment_v0_t env = {{NULL, host_allocator_ctl}};
  iree_amd_hal_plugin_string_pair_t param;
  size_t param_count = 0;
  if (argc >= 3) {
    param.key.data = "uk_library"; param.key.size = strlen("uk_library");
    param.value.data = argv[2]; param.value.size = strlen(argv[2]);
    param_count = 1;
  }
  void* self = NULL;
  CHECK(plugin->load(&env, param_count, &param, &self) == 0 && self, "load");

  const char* names[3] = {"mi355x_uk_pack", "mi355x_uk_mmt4d", "mi355x_uk_unpack"};
  void* fns[3] = {NULL, NULL, NULL};
  void* ctxs[3] = {NULL, NULL, NULL};
  iree_amd_hal_plugin_resolve_params_v0_t rp = {3, names, fns, ctxs};
  uint32_t resolution = 0;
  CHECK(plugin->resolve(self, &rp, &resolution) == 0 && fns[0] && fns[1] && fns[2], "resolve");
  iree_amd_hal_plugin_import_fn_t pack_fn = (iree_amd_hal_plugin_import_fn_t)fns[0];
  iree_amd_hal_plugin_import_fn_t mmt4d_fn = (iree_amd_hal_plugin_import_fn_t)fns[1];
  iree_amd_hal_plugin_import_fn_t unpack_fn = (iree_amd_hal_plugin_import_fn_t)fns[2];

  /* C[M][N] = A[M][K] * B[K][N], i8 x i8 -> i32, gfx950 tiles 32 x 32 x 16 */
  enum { M = 75, N = 130, K = 200, M0 = 32, N0 = 32, K0 = 16 };
  enum { M1 = (M + M0 - 1) / M0, N1 = (N + N0 - 1) / N0, K1 = (K + K0 - 1) / K0 };
  int8_t* A = malloc(M * K);
  int8_t* B = malloc(K * N);
  int8_t* lhs = malloc(M1 * K1 * M0 * K0);
  int8_t* rhs = malloc(N1 * K1 * N0 * K0);
  int32_t* acc = malloc(sizeof(int32_t) * M1 * N1 * M0 * N0);
  int32_t* C = malloc(sizeof(int32_t) * M * N);
  uint32_t seed = 12345;
  for (int i = 0; i < M * K; ++i) A[i] = (int8_t)((seed = seed * 1664525u + 1013904223u) >> 24);
  for (int i = 0; i < K * N; ++i) B[i] = (int8_t)((seed = seed * 1664525u + 1013904223u) >> 24);
  memset(C, 0x7F, sizeof(int32_t) * M * N);

  iree_amd_uk_pack_params_t pl = {A, 0, K, 1, lhs, 0, K1 * M0 * K0, M0 * K0, M, K, M1, K1, M0, K0, 0,
                                  IREE_AMD_UK_FLAG_PACK_TYPE_I8I8, NULL};
  CHECK(pack_fn(&pl, ctxs[0], NULL) == 0, "pack lhs");
  iree_amd_uk_pack_params_t pr = {B, 0, N, 1, rhs, 0, K1 * N0 * K0, N0 * K0, K, N, N1, K1, N0, K0, 0,
                                  IREE_AMD_UK_FLAG_PACK_TYPE_I8I8 | IREE_AMD_UK_FLAG_PACK_TRANSPOSE_INNER |
                                      IREE_AMD_UK_FLAG_PACK_TRANSPOSE_OUTER,
                                  NULL};
  CHECK(pack_fn(&pr, ctxs[0], NULL) == 0, "pack rhs");
  iree_amd_uk_mmt4d_params_t mm = {lhs, 0, K1 * M0 * K0, rhs, 0, K1 * N0 * K0, acc, 0, N1 * M0 * N0,
                                   M1, N1, K1, M0, N0, K0,
                                   IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32 |
                                       IREE_AMD_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION,
                                   NULL};
  CHECK(mmt4d_fn(&mm, ctxs[1], NULL) == 0, "mmt4d");
  iree_amd_uk_unpack_params_t up = {acc, 0, N1 * M0 * N0, M0 * N0, C, 0, N, 1, M1, N1, M0, N0, M, N,
                                    IREE_AMD_UK_FLAG_UNPACK_TYPE_I32I32, NULL};
  CHECK(unpack_fn(&up, ctxs[2], NULL) == 0, "unpack");

  long mismatches = 0;
  for (int i = 0; i < M; ++i)
    for (int j = 0; j < N; ++j) {
      int32_t want = 0;
      for (int k = 0; k < K; ++k) want += (int32_t)A[i * K + k] * (int32_t)B[k * N + j];
      if (C[i * N + j] != want) ++mismatches;
    }
  CHECK(mismatches == 0, "%ld of %d results differ from the triple loop", mismatches, M * N);

  plugin->unload(self);
  CHECK(g_live_allocations == 0, "plugin leaked %d host allocations", g_live_allocations);
  dlclose(lib);
  free(A); free(B); free(lhs); free(rhs); free(acc); free(C);
  printf("OK: %dx%dx%d i8 matmul through the plugin imports is bit-exact\n", M, N, K);
  return 0;
}
