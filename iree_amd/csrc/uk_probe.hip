// Measurement aid: the MFMA issue pattern of the mmt4d kernel (a wave holds the
// A and B fragments of its 128 x 128 tile and updates all accumulator blocks
// once per K-step, with the instruction shape the kernel uses for the type)
// with ALL data movement removed: the fragments are loaded from a
// small buffer once and stay in registers. What it sustains is the ceiling of
// the matrix cores for operands with that bit pattern: on MI355X the rate
// depends strongly on the data (constant operands reach the nominal peak,
// random ones far less: the pipe is power-limited by operand toggling).
#include "uk_common.h"
#include "uk_mfma_cfg.h"

namespace uk {
namespace {

typedef uint32_t u32x4p __attribute__((ext_vector_type(4)));

template <typename Cfg>
__global__ __launch_bounds__(256) void mfma_probe_kernel(const char* operands, int64_t iters, float* sink) {
  typedef typename Cfg::frag_t frag_t;
  typedef typename Cfg::acc_t acc_t;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  constexpr int kFragBytes = sizeof(frag_t);
  // a wave's tile is 128 x 128: W x W blocks of the instruction's shape
  constexpr int W = 128 / Cfg::kRows, kAccRegs = Cfg::kRows * Cfg::kRows / 64;
  // 2 W fragments per wave: operands[(wave * 2 W + f) * 64 + lane]
  frag_t a[W], b[W];
#pragma unroll
  for (int f = 0; f < W; ++f) {
    a[f] = *(const frag_t*)(operands + ((size_t)(wave * 2 * W + f) * 64 + lane) * kFragBytes);
    b[f] = *(const frag_t*)(operands + ((size_t)(wave * 2 * W + W + f) * 64 + lane) * kFragBytes);
  }
  acc_t acc[W][W];
#pragma unroll
  for (int x = 0; x < W; ++x)
#pragma unroll
    for (int y = 0; y < W; ++y)
#pragma unroll
      for (int v = 0; v < kAccRegs; ++v) acc[x][y][v] = 0;
  for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int x = 0; x < W; ++x)
#pragma unroll
      for (int y = 0; y < W; ++y) acc[x][y] = Cfg::mfma(a[x], b[y], acc[x][y]);
  }
  // keep the result alive without storing it in the common case
  float s = 0.f;
#pragma unroll
  for (int x = 0; x < W; ++x)
#pragma unroll
    for (int y = 0; y < W; ++y)
#pragma unroll
      for (int v = 0; v < kAccRegs; ++v) s += (float)acc[x][y][v];
  if (s == 12345.678f) sink[threadIdx.x] = s;
}

// Second measurement aid: a plain out-of-place copy, the yardstick for the pack
// / unpack streams (what the reference's own benchmarks do with memcpy,
// runtime/src/iree/builtins/ukernel/tools/memcpy_benchmark.c:24-52). Every lane
// moves 16 bytes per access; a wave keeps kCopyUnroll accesses of 1 KiB in
// flight; workgroups walk contiguous chunks, XCD by XCD, like the pack kernel.
// Two geometries: 256 threads with two accesses in flight per lane (8 KiB per
// workgroup and step), and single waves with one (1 KiB: the unit of work the
// pack / unpack kernels settled on).
template <bool kNonTemporal, int kThreads, int kCopyUnroll>
__global__ __launch_bounds__(kThreads) void copy_probe_kernel(const u32x4p* src, u32x4p* dst, int64_t chunks) {
  // chunk = kCopyUnroll * kThreads lanes * 16 bytes
  for (int64_t c = blockIdx.x; c < chunks; c += gridDim.x) {
    const int64_t base = c * (kCopyUnroll * kThreads) + threadIdx.x;
    u32x4p v[kCopyUnroll];
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u)
      v[u] = kNonTemporal ? __builtin_nontemporal_load(src + base + u * kThreads) : src[base + u * kThreads];
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) {
      if (kNonTemporal) __builtin_nontemporal_store(v[u], dst + base + u * kThreads);
      else dst[base + u * kThreads] = v[u];
    }
  }
}

// The read half alone: what a kernel that only streams its input (a matrix of
// weights against a few activation rows) can reach. Every workgroup folds what
// it reads into one word and stores it only if it has a value that the data
// never produce in practice, so the loads stay and nothing is written.
template <bool kNonTemporal, int kThreads, int kCopyUnroll>
__global__ __launch_bounds__(kThreads) void read_probe_kernel(const u32x4p* src, uint32_t* sink, int64_t chunks) {
  uint32_t fold = 0;
  for (int64_t c = blockIdx.x; c < chunks; c += gridDim.x) {
    const int64_t base = c * (kCopyUnroll * kThreads) + threadIdx.x;
    u32x4p v[kCopyUnroll];
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u)
      v[u] = kNonTemporal ? __builtin_nontemporal_load(src + base + u * kThreads) : src[base + u * kThreads];
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) fold ^= v[u].x ^ (v[u].y * 3u) ^ (v[u].z * 5u) ^ (v[u].w * 7u);
  }
  if (fold == 0x9E3779B9u) sink[0] = fold;
}

template <int kThreads, int kCopyUnroll>
int launch_copy_geometry(const void* src, void* dst, int64_t bytes, int mode, int blocks_per_cu, hipStream_t s) {
  const int64_t chunks = bytes / ((int64_t)kCopyUnroll * kThreads * 16);
  int64_t blocks = blocks_per_cu > 0 ? (int64_t)device_cu_count() * blocks_per_cu : chunks;
  if (blocks > chunks) blocks = chunks;
  if (blocks > 0x7FFFFFFF) blocks = 0x7FFFFFFF;
  const dim3 g((unsigned)blocks), b(kThreads);
  switch (mode & 3) {
    case 0: hipLaunchKernelGGL((copy_probe_kernel<false, kThreads, kCopyUnroll>), g, b, 0, s, (const u32x4p*)src, (u32x4p*)dst, chunks); break;
    case 1: hipLaunchKernelGGL((copy_probe_kernel<true, kThreads, kCopyUnroll>), g, b, 0, s, (const u32x4p*)src, (u32x4p*)dst, chunks); break;
    case 2: hipLaunchKernelGGL((read_probe_kernel<false, kThreads, kCopyUnroll>), g, b, 0, s, (const u32x4p*)src, (uint32_t*)dst, chunks); break;
    default: hipLaunchKernelGGL((read_probe_kernel<true, kThreads, kCopyUnroll>), g, b, 0, s, (const u32x4p*)src, (uint32_t*)dst, chunks); break;
  }
  return check_hip(hipGetLastError(), "copy_probe launch");
}

template <typename Cfg>
int launch(const void* operands, int64_t iters, void* sink, int blocks, hipStream_t s) {
  hipLaunchKernelGGL((mfma_probe_kernel<Cfg>), dim3(blocks), dim3(256), 0, s, (const char*)operands,
                     iters, (float*)sink);
  return check_hip(hipGetLastError(), "mfma_probe launch");
}

}  // namespace

int launch_mfma_probe(uint32_t type_flag, const void* operands, int64_t iters, void* sink,
                      int64_t* out_ops_per_launch, hipStream_t s) {
  const int blocks = device_cu_count();   // one workgroup of 4 waves per compute unit, as the large tile
  int st;
  int64_t k;
  switch (type_flag & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
    // (the shapes the mmt4d kernel uses for each type)
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32: st = launch<F16Cfg16>(operands, iters, sink, blocks, s); k = 32; break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32: st = launch<BF16Cfg16>(operands, iters, sink, blocks, s); k = 32; break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32: st = launch<S8Cfg16>(operands, iters, sink, blocks, s); k = 64; break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32: st = launch<F8Cfg>(operands, iters, sink, blocks, s); k = 64; break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32: st = launch<F32Cfg>(operands, iters, sink, blocks, s); k = 8; break;
    default: return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mfma_probe: type has no MFMA kernel");
  }
  // per wave and iteration: a 128 x 128 x k update
  if (out_ops_per_launch) *out_ops_per_launch = (int64_t)blocks * 4 * iters * 2 * 128 * 128 * k;
  return st;
}

// bytes: a multiple of 8 KiB; mode 0 = plain accesses, 1 = non-temporal, 2 and
// 3 = the same two without the stores (dst then needs 4 bytes only), + 4 = the
// same in single-wave workgroups of 1 KiB per step;
// blocks_per_cu workgroups per compute unit (0 = one workgroup per chunk).
int launch_copy_probe(const void* src, void* dst, int64_t bytes, int mode, int blocks_per_cu, hipStream_t s) {
  if (bytes <= 0 || bytes % 8192 || ((uintptr_t)src | (uintptr_t)dst) % 16 || mode < 0 || mode > 7)
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT,
                "copy_probe: bytes must be whole chunks of 8192, buffers 16-byte aligned, mode 0..7");
  if (mode & 4) return launch_copy_geometry<64, 1>(src, dst, bytes, mode, blocks_per_cu, s);
  return launch_copy_geometry<256, 2>(src, dst, bytes, mode, blocks_per_cu, s);
}

}  // namespace uk
