// mmt4d on the gfx950 matrix cores: the host side. Picks the macro tile for a
// call, launches the kernel of uk_mmt4d_mfma_kernel.h and serves the fused
// forms (row-major result, row-major left-hand side, SiLU epilogue).
//
// Contract: include/iree_amd_uk.h (mirrors iree_uk_mmt4d,
// runtime/src/iree/builtins/ukernel/mmt4d.h:14-21 of the reference).
#include "uk_common.h"
#include "uk_mmt4d_mfma_kernel.h"
#include "uk_mmt4d_mfma_launch.h"
#include "uk_scratch_cache.h"

#include <mutex>

namespace uk {
namespace {

// Sum of the partial results of a K split. One thread owns 4 consecutive
// columns of one tile row: it adds the slices in order (after the old result,
// when accumulating) and writes what the matmul kernel's epilogue would have.
template <typename AccT, typename OutT>
__global__ __launch_bounds__(256) void ksplit_reduce_kernel(KSplitReduceArgs r) {
  typedef AccT acc4_t __attribute__((ext_vector_type(4)));
  typedef OutT out4_t __attribute__((ext_vector_type(4), aligned(sizeof(OutT))));
  const int64_t groups = r.flat_elems > 0 ? r.flat_elems / 4 : (int64_t)r.M * r.N * 256;
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= groups) return;
  const int64_t tile = g >> 8;
  const int in_tile = (int)(g & 255);
  const int row_in_tile = in_tile >> 3, col_in_tile = (in_tile & 7) * 4;
  const int i = (int)(tile / r.N), j = (int)(tile % r.N);
  OutT* dst;
  int valid = 4;   // leading elements of the group that exist in the result
  if (r.flat_elems > 0) {
    dst = (OutT*)r.out + g * 4;
  } else if (r.row_major_out) {
    const int row = i * 32 + row_in_tile, col = j * 32 + col_in_tile;
    if (row >= r.out_rows || col >= r.out_cols) return;
    valid = r.out_cols - col < 4 ? r.out_cols - col : 4;
    dst = (OutT*)((char*)r.out + (int64_t)row * r.out_stride_bytes) + col;
  } else {
    dst = (OutT*)((char*)r.out + (int64_t)i * r.out_stride_bytes) + (int64_t)j * 1024 + in_tile * 4;
  }
  acc4_t sum = {0, 0, 0, 0};
  if (r.accumulate) {
    if (valid == 4) {
      const out4_t old = *(const out4_t*)dst;
#pragma unroll
      for (int e = 0; e < 4; ++e) sum[e] = (AccT)old[e];
    } else {
      for (int e = 0; e < valid; ++e) sum[e] = (AccT)dst[e];
    }
  }
  const acc4_t* p = (const acc4_t*)r.partials + g;
  for (int sl = 0; sl < r.slices; ++sl) sum += p[(int64_t)sl * groups];
  out4_t v;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if constexpr (std::is_floating_point<AccT>::value)
      v[e] = r.row_major_out ? (OutT)(sum[e] * r.out_scale) : (OutT)sum[e];
    else
      v[e] = (OutT)sum[e];
  }
  if (valid == 4) {
    *(out4_t*)dst = v;
  } else {
    for (int e = 0; e < valid; ++e) dst[e] = v[e];
  }
}

}  // namespace

namespace {

// The cache's allocator: plain hipMalloc / hipFree (which waits for the
// device) / hipFreeAsync in stream order.
void* scratch_alloc(size_t bytes, void*) {
  void* p = nullptr;
  if (hipMalloc(&p, bytes) != hipSuccess || !p) { (void)hipGetLastError(); return nullptr; }
  return p;
}
void scratch_free_now(void* p, void*) {
  if (hipFree(p) != hipSuccess) (void)hipGetLastError();
}
void scratch_free_ordered(void* p, void* stream, void*) {
  if (hipFreeAsync(p, (hipStream_t)stream) != hipSuccess) { (void)hipGetLastError(); (void)hipFree(p); }
}

// 16 MiB at least per buffer, 512 MiB at most (larger problems run unsplit),
// 64 (device, stream) pairs.
ScratchCache& scratch_cache() {
  static ScratchCache cache(ScratchAllocator{scratch_alloc, scratch_free_now, scratch_free_ordered, nullptr},
                            (size_t)16 << 20, (size_t)512 << 20, 64);
  return cache;
}

struct OverrideState { void* ptr; size_t bytes; bool strict, active; };
thread_local OverrideState g_override = {nullptr, 0, false, false};

}  // namespace

ScratchLease::ScratchLease(hipStream_t s, size_t bytes) {
  if (g_override.active) {
    if (bytes != 0 && bytes <= g_override.bytes) ptr_ = g_override.ptr;
    else overflowed_ = g_override.strict && bytes > g_override.bytes;
    return;
  }
  // (the per-thread default stream is one handle for a different stream in
  // every host thread: a buffer keyed by it would be shared by unordered work)
  if (s == hipStreamPerThread) return;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) { (void)hipGetLastError(); return; }
  const ScratchCache::Lease lease = scratch_cache().acquire(device, (void*)s, bytes);
  ptr_ = lease.ptr;
  id_ = lease.id;
}

ScratchLease::~ScratchLease() {
  if (id_) {
    ScratchCache::Lease lease;
    lease.ptr = ptr_;
    lease.id = id_;
    scratch_cache().release(lease);
  }
}

ScratchOverride::ScratchOverride(void* ptr, size_t bytes, bool strict)
    : prev_ptr_(g_override.ptr), prev_bytes_(g_override.bytes), prev_strict_(g_override.strict),
      prev_active_(g_override.active) {
  g_override = {ptr, bytes, strict, true};
}
ScratchOverride::~ScratchOverride() { g_override = {prev_ptr_, prev_bytes_, prev_strict_, prev_active_}; }

int scratch_overflow_status(const char* what, size_t bytes) {
  return fail(8 /* RESOURCE_EXHAUSTED */,
              "%s needs %zu bytes of scratch memory; this entry point allocates nothing and has %zu",
              what, bytes, g_override.bytes);
}

size_t scratch_release_idle() { return scratch_cache().release_idle(); }

int launch_ksplit_reduce(const KSplitReduceArgs& r, hipStream_t s) {
  const int64_t groups = r.flat_elems > 0 ? r.flat_elems / 4 : (int64_t)r.M * r.N * 256;
  const int64_t blocks = (groups + 255) / 256;
  if (blocks < 1 || blocks > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const dim3 grid((unsigned)blocks), block(256);
  if (!r.acc_is_float) {
    hipLaunchKernelGGL((ksplit_reduce_kernel<int32_t, int32_t>), grid, block, 0, s, r);
  } else if (r.out_kind == 1) {
    hipLaunchKernelGGL((ksplit_reduce_kernel<float, _Float16>), grid, block, 0, s, r);
  } else if (r.out_kind == 2) {
    hipLaunchKernelGGL((ksplit_reduce_kernel<float, __bf16>), grid, block, 0, s, r);
  } else {
    hipLaunchKernelGGL((ksplit_reduce_kernel<float, float>), grid, block, 0, s, r);
  }
  return check_hip(hipGetLastError(), "ksplit_reduce launch");
}

namespace {

// mfma_k: K extent of the instruction the call runs on. f16 / bf16 use the
// 16x16x32 shapes, except with the fused SiLU epilogue (32x32x16).
struct Served { int mfma_k; };
bool served(uint32_t flags, int M0, int N0, int K0, bool silu, Served* out) {
  int mfma_k = 0;
  bool half_type = false;
  switch (flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32:
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32: mfma_k = silu ? 16 : 32; half_type = true; break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16:
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16:
      // f32 accumulation with one final rounding is only the reference's
      // arithmetic when intermediate roundings are skipped
      if (!(flags & IREE_AMD_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS)) return false;
      mfma_k = silu ? 16 : 32;
      half_type = true;
      break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32: mfma_k = 8; break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32: mfma_k = 32; break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32: mfma_k = 64; break;
    default: return false;
  }
  if (M0 != 32 || N0 != 32) return false;
  if (mfma_k == 64) {
    if (K0 != 16) return false;
  } else if (half_type) {
    if (K0 != 8 && K0 != 16) return false;   // a quarter / half (or half / all) of the K extent
  } else if (K0 != mfma_k && K0 * 2 != mfma_k) {
    return false;
  }
  if (out) out->mfma_k = mfma_k;
  return true;
}

}  // namespace

bool mmt4d_mfma_supported(uint32_t flags, int M0, int N0, int K0) {
  return served(flags, M0, N0, K0, false, nullptr);
}

namespace {
// Fills `a` from the parameters; NOT_FOUND when the MFMA kernels cannot take the call.
int make_args(const iree_amd_uk_mmt4d_params_t& p, int out_elem_bytes, bool silu, MfmaArgs* out_args) {
  Served sv;
  if (!served(p.flags, p.M0, p.N0, p.K0, silu, &sv)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  Mmt4dTypeInfo ti;
  mmt4d_type_info(p.flags, &ti);
  const int eb = ti.lhs_bits / 8;
  const int64_t k_elems = p.K * p.K0;
  // Every operand block must be 16-byte aligned. K need not be whole MFMA
  // steps: the kernel finishes with a partial step.
  if (p.K == 0) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const char* lhs = (const char*)p.lhs_buffer + p.lhs_offset * eb;
  const char* rhs = (const char*)p.rhs_buffer + p.rhs_offset * eb;
  if (((uintptr_t)lhs | (uintptr_t)rhs) % 16) return IREE_AMD_UK_STATUS_NOT_FOUND;
  if ((p.lhs_stride0 * eb) % 16 || (p.rhs_stride0 * eb) % 16) return IREE_AMD_UK_STATUS_NOT_FOUND;
  // (the kernel addresses an outer row of 32 x K elements with 32-bit byte offsets)
  if (k_elems * 32 * eb + 4096 > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  MfmaArgs& a = *out_args;
  a.lhs = lhs; a.rhs = rhs;
  a.out = (char*)p.out_buffer + p.out_offset * out_elem_bytes;
  a.lhs_stride_bytes = p.lhs_stride0 * eb;
  a.rhs_stride_bytes = p.rhs_stride0 * eb;
  a.out_stride_bytes = p.out_stride0 * out_elem_bytes;
  a.M = (int)p.M; a.N = (int)p.N;
  a.ksteps = (int)(k_elems / sv.mfma_k);
  a.tail_tiles = (int)((k_elems % sv.mfma_k) / p.K0);
  a.tiles_m = a.tiles_n = 0;
  a.k_slices = 0; a.slice_ksteps = 0; a.slice_out_bytes = 0;
  a.batch = 1; a.lhs_batch_bytes = a.rhs_batch_bytes = a.out_batch_bytes = 0;
  a.batch_by_xcd = 0;
  a.stream_out = p.M * p.N * 1024 * out_elem_bytes > (32ll << 20);
  a.accumulate = (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  a.k0_div = sv.mfma_k / p.K0;
  a.row_major_out = 0; a.out_rows = a.out_cols = 0;
  a.lhs_row_major = 0;
  a.gate_scale = a.up_scale = a.inv_out_scale = a.out_scale = 1.0f;
  return 0;
}
}  // namespace

namespace {
int launch_typed(const iree_amd_uk_mmt4d_params_t& p, const MfmaArgs& a, hipStream_t s);
}  // namespace

int launch_mmt4d_mfma(const iree_amd_uk_mmt4d_params_t& p, hipStream_t s) {
  Mmt4dTypeInfo ti;
  mmt4d_type_info(p.flags, &ti);
  MfmaArgs a;
  const int st = make_args(p, ti.out_bytes, false, &a);
  if (st) return st;
  return launch_typed(p, a, s);
}

// `batch` mmt4d problems of one shape, operands `*_batch_stride` elements
// apart: one launch whose workgroup planes are the batch entries (at most
// 65535 planes a launch).
namespace {
int launch_planes(const iree_amd_uk_mmt4d_params_t& p, MfmaArgs a, int64_t batch, int64_t lhs_batch_stride,
                  int64_t rhs_batch_stride, int64_t out_batch_stride, hipStream_t s);
}  // namespace

int launch_batch_mmt4d_mfma(const iree_amd_uk_mmt4d_params_t& p, int64_t batch, int64_t lhs_batch_stride,
                            int64_t rhs_batch_stride, int64_t out_batch_stride, hipStream_t s) {
  Mmt4dTypeInfo ti;
  mmt4d_type_info(p.flags, &ti);
  MfmaArgs a;
  const int st = make_args(p, ti.out_bytes, false, &a);
  if (st) return st;
  return launch_planes(p, a, batch, lhs_batch_stride, rhs_batch_stride, out_batch_stride, s);
}

namespace {
// Launches `a` (any operand form) over `batch` planes.
int launch_planes(const iree_amd_uk_mmt4d_params_t& p, MfmaArgs a, int64_t batch, int64_t lhs_batch_stride,
                  int64_t rhs_batch_stride, int64_t out_batch_stride, hipStream_t s) {
  Mmt4dTypeInfo ti;
  mmt4d_type_info(p.flags, &ti);
  const int eb = ti.lhs_bits / 8;
  a.lhs_batch_bytes = lhs_batch_stride * eb;
  a.rhs_batch_bytes = rhs_batch_stride * eb;
  a.out_batch_bytes = out_batch_stride * ti.out_bytes;
  if (a.lhs_batch_bytes % 16 || a.rhs_batch_bytes % 16) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int64_t kPlanes = 65535;
  for (int64_t b0 = 0; b0 < batch; b0 += kPlanes) {
    MfmaArgs c = a;
    c.batch = (int)(batch - b0 < kPlanes ? batch - b0 : kPlanes);
    c.stream_out = p.M * p.N * 1024 * (int64_t)ti.out_bytes * c.batch > (32ll << 20);
    c.lhs = a.lhs + b0 * a.lhs_batch_bytes;
    c.rhs = a.rhs + b0 * a.rhs_batch_bytes;
    c.out = a.out + b0 * a.out_batch_bytes;
    const int lst = launch_typed(p, c, s);
    if (lst) return lst;      // (NOT_FOUND can only come from the first launch)
  }
  return 0;
}
}  // namespace

// mmt4d whose result goes to a row-major out_rows x out_cols matrix (element
// pitch p.out_stride0 between rows) instead of tiles: what mmt4d followed by
// an unpack without transposes writes, and reads when accumulating; float
// results are multiplied by out_scale on the store.
int launch_mmt4d_unpack_mfma(const iree_amd_uk_mmt4d_params_t& p, int64_t out_rows,
                             int64_t out_cols, float out_scale, int64_t batch, int64_t lhs_batch_stride,
                             int64_t rhs_batch_stride, int64_t out_batch_stride, hipStream_t s) {
  Mmt4dTypeInfo ti;
  mmt4d_type_info(p.flags, &ti);
  MfmaArgs a;
  const int st = make_args(p, ti.out_bytes, false, &a);
  if (st) return st;
  if (out_rows > 0x7FFFFFFF || out_cols > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  a.row_major_out = 1;
  a.out_scale = out_scale;
  a.out_rows = (int)out_rows;
  a.out_cols = (int)out_cols;
  if (batch > 1) return launch_planes(p, a, batch, lhs_batch_stride, rhs_batch_stride, out_batch_stride, s);
  return launch_typed(p, a, s);
}

// The same with a row-major left-hand side as well: `p` describes the
// equivalent mmt4d (outer counts, K tiles, packed right-hand side), except that
// p.lhs_buffer / lhs_offset / lhs_stride0 are the out_rows x (K * K0) matrix,
// its first element and its row pitch in elements.
int launch_matmul_packed_rhs_mfma(const iree_amd_uk_mmt4d_params_t& p, int64_t out_rows,
                                  int64_t out_cols, float out_scale, int64_t batch, int64_t lhs_batch_stride,
                                  int64_t rhs_batch_stride, int64_t out_batch_stride, hipStream_t s) {
  Mmt4dTypeInfo ti;
  mmt4d_type_info(p.flags, &ti);
  MfmaArgs a;
  const int st = make_args(p, ti.out_bytes, false, &a);
  if (st) return st;
  // whole matrix-core K-steps only (a partial one would read past the row end),
  // and a matrix that 32-bit byte offsets can address
  if (a.tail_tiles != 0 || out_rows > 0x7FFFFFFF || out_cols > 0x7FFFFFFF ||
      out_rows * a.lhs_stride_bytes + 4096 > 0x7FFFFFFF)
    return IREE_AMD_UK_STATUS_NOT_FOUND;
  a.row_major_out = 1;
  a.out_rows = (int)out_rows;
  a.out_cols = (int)out_cols;
  a.out_scale = out_scale;
  // Reading the row-major matrix inside the matmul costs 1-4 % of the matmul's
  // time (half cache lines per row and K-step, fetched again by every column
  // of macro tiles); packing it first costs one pass over it. With 16384
  // result columns and more the pass is the cheaper of the two (measured,
  // f16 / i8 / fp8: 2048 x 28672 x 4096 411 / 247 / 219 us packed first
  // against 422 / 252 / 227; 4096 x 14336 x 4096 410 / 242 / 205 against
  // 418 / 239 / 204; 8192^3 886 / 526 / 489 against 834 / 517 / 481): the
  // left-hand side is then packed into the stream's scratch buffer and the
  // packed-operand kernel runs. That buffer is also where a K split keeps its
  // partial sums, so the two exclude each other (K is only ever split for
  // problems of few macro tiles).
  const int eb = ti.lhs_bits / 8;
  const int64_t packed_bytes = p.M * p.K * 32 * p.K0 * eb;
  if (batch > 1) {
    // (a batch reads its row-major left-hand sides in the kernel)
    a.lhs_row_major = 1;
    return launch_planes(p, a, batch, lhs_batch_stride, rhs_batch_stride, out_batch_stride, s);
  }
  if (out_cols >= 16384 && out_rows >= 512) {
    // (held until the matmul that reads the packed copy has been queued)
    ScratchLease lease(s, (size_t)packed_bytes);
    void* packed = lease.ptr();
    if (packed) {
      iree_amd_uk_pack_params_t pp;
      pp.in_buffer = p.lhs_buffer; pp.in_offset = p.lhs_offset;
      pp.in_stride0 = p.lhs_stride0; pp.in_stride1 = 1;
      pp.out_buffer = packed; pp.out_offset = 0;
      pp.out_stride0 = p.K * 32 * p.K0; pp.out_stride1 = 32 * p.K0;
      pp.in_size0 = out_rows; pp.in_size1 = p.K * p.K0;
      pp.out_size0 = p.M; pp.out_size1 = p.K; pp.out_size2 = 32; pp.out_size3 = p.K0;
      pp.padding_value = 0;
      pp.flags = eb == 1 ? IREE_AMD_UK_FLAG_PACK_TYPE_I8I8
                 : eb == 2 ? IREE_AMD_UK_FLAG_PACK_TYPE_F16F16 : IREE_AMD_UK_FLAG_PACK_TYPE_F32F32;
      pp.cpu_data = nullptr;
      const int pst = launch_pack(pp, s);
      if (pst) return pst;
      a.lhs = (const char*)packed;
      a.lhs_stride_bytes = p.K * 32 * p.K0 * eb;
      a.lhs_row_major = 0;
      a.k_slices = -1;     // no K split: the scratch buffer is taken
      return launch_typed(p, a, s);
    }
  }
  a.lhs_row_major = 1;
  return launch_typed(p, a, s);
}

namespace {
int launch_typed(const iree_amd_uk_mmt4d_params_t& p, const MfmaArgs& a, hipStream_t s) {
  switch (p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32: return launch_mfma_f16f16f32(a, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32: return launch_mfma_bf16bf16f32(a, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32: return launch_mfma_s8s8s32(a, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32: return launch_mfma_f8f8f32(a, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32: return launch_mfma_f32f32f32(a, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16: return launch_mfma_f16f16f16(a, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16: return launch_mfma_bf16bf16bf16(a, s);
    default: return IREE_AMD_UK_STATUS_NOT_FOUND;
  }
}
}  // namespace

// mmt4d whose epilogue is e4m3(silu(gate) * up): `p.N` counts gate AND up outer
// columns (interleaved, so it is even); the output has N / 2 outer columns of
// 1024 bytes and `out_offset` / `out_stride0` are in bytes.
int launch_mmt4d_silu_mul_mfma(const iree_amd_uk_mmt4d_params_t& p, float gate_scale,
                               float up_scale, float inv_out_scale, hipStream_t s) {
  MfmaArgs a;
  const int st = make_args(p, 1, true, &a);
  if (st) return st;
  a.gate_scale = gate_scale; a.up_scale = up_scale; a.inv_out_scale = inv_out_scale;
  a.accumulate = 0;
  switch (p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32: return launch_mfma_silu_f16(a, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32: return launch_mfma_silu_bf16(a, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32: return launch_mfma_silu_f8(a, s);
    default: return IREE_AMD_UK_STATUS_NOT_FOUND;
  }
}

}  // namespace uk
