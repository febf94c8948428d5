// Host-pointer entry points (include/iree_amd_uk.h): the same three ukernels on
// HOST buffers, which is what an import of IREE's local-CPU HAL receives
// (samples/custom_dispatch/cpu/plugin/README.md:90-97 of the reference). Each
// call stages the touched byte ranges into device memory, runs the device entry
// point and copies the destination range back.
//
// A pool keeps what the staging needs between calls: slots of one stream and
// three device buffers that grow on demand. A call takes a free slot for its
// duration, so calls from several host threads (the contract of an import,
// samples/custom_dispatch/cpu/plugin/system_plugin.c:21-25) run concurrently on
// slots of their own and share nothing; when every slot is taken a call waits
// for one. The pool holds no global state: a plugin instance owns its pool and
// destroys it on unload (executable_plugin.h:415-418).
#include "uk_common.h"

#include <condition_variable>
#include <mutex>
#include <vector>

namespace {

using namespace uk;

constexpr size_t kMaxSlots = 8;

struct HostSlot {
  int device = 0;
  hipStream_t stream = nullptr;
  void* dev[3] = {nullptr, nullptr, nullptr};
  size_t cap[3] = {0, 0, 0};
  bool busy = false;

  int init() {
    UK_RETURN_IF_HIP(hipGetDevice(&device));
    // (default priority on purpose: mixed stream priorities are not used)
    return check_hip(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking), "hipStreamCreate");
  }
  void destroy() {
    for (int i = 0; i < 3; ++i) {
      if (dev[i] && hipFree(dev[i]) != hipSuccess) (void)hipGetLastError();
      dev[i] = nullptr;
      cap[i] = 0;
    }
    if (stream && hipStreamDestroy(stream) != hipSuccess) (void)hipGetLastError();
    stream = nullptr;
  }
  // Device buffer `i` of at least `bytes`. The slot's stream is idle between
  // calls (every call ends with a synchronisation), so a smaller buffer can be
  // freed on the spot.
  int ensure(int i, int64_t bytes) {
    if (bytes <= 0 || (size_t)bytes <= cap[i]) return 0;
    if (dev[i]) {
      UK_RETURN_IF_HIP(hipFree(dev[i]));
      dev[i] = nullptr;
      cap[i] = 0;
    }
    const size_t want = ((size_t)bytes + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
    UK_RETURN_IF_HIP(hipMalloc(&dev[i], want));
    cap[i] = want;
    return 0;
  }
  int upload(int i, const void* host, int64_t byte_off, int64_t bytes, bool copy) {
    if (bytes <= 0) return 0;
    UK_RETURN_IF_ERROR(ensure(i, bytes));
    if (copy)
      UK_RETURN_IF_HIP(hipMemcpyAsync(dev[i], (const char*)host + byte_off, (size_t)bytes,
                                      hipMemcpyHostToDevice, stream));
    return 0;
  }
  int download(int i, void* host, int64_t byte_off, int64_t bytes) {
    if (bytes > 0)
      UK_RETURN_IF_HIP(hipMemcpyAsync((char*)host + byte_off, dev[i], (size_t)bytes,
                                      hipMemcpyDeviceToHost, stream));
    return check_hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
  }
};

}  // namespace

struct iree_amd_uk_host_pool_t {
  std::mutex mutex;
  std::condition_variable freed;
  std::vector<HostSlot*> slots;
};

namespace {

// A slot of `pool` on the current device for the duration of one call.
class SlotLease {
 public:
  explicit SlotLease(iree_amd_uk_host_pool_t* pool) : pool_(pool) {}
  ~SlotLease() {
    if (!slot_) return;
    {
      std::lock_guard<std::mutex> lock(pool_->mutex);
      slot_->busy = false;
    }
    pool_->freed.notify_one();
  }
  int acquire() {
    int device = 0;
    UK_RETURN_IF_HIP(hipGetDevice(&device));
    std::unique_lock<std::mutex> lock(pool_->mutex);
    for (;;) {
      size_t on_device = 0;
      for (HostSlot* s : pool_->slots) {
        if (s->device != device) continue;
        ++on_device;
        if (!s->busy) {
          s->busy = true;
          slot_ = s;
          return 0;
        }
      }
      if (on_device < kMaxSlots) {
        HostSlot* s = new HostSlot();
        const int st = s->init();
        if (st) {
          delete s;
          return st;
        }
        s->busy = true;
        pool_->slots.push_back(s);
        slot_ = s;
        return 0;
      }
      pool_->freed.wait(lock);
    }
  }
  HostSlot* operator->() { return slot_; }

 private:
  iree_amd_uk_host_pool_t* pool_;
  HostSlot* slot_ = nullptr;
};

// Bytes spanned by `rows` rows of `row_elems` contiguous elements, `stride`
// elements apart, for an element of `bits` bits.
int64_t span_bytes(int64_t rows, int64_t stride, int64_t row_elems, int bits) {
  if (rows <= 0 || row_elems <= 0) return 0;
  return (((rows - 1) * stride + row_elems) * bits + 7) / 8;
}

int mmt4d_on(iree_amd_uk_host_pool_t* pool, const iree_amd_uk_mmt4d_params_t* params) {
  if (!params) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d_host: null params");
  iree_amd_uk_mmt4d_params_t p = *params;
  UK_RETURN_IF_ERROR(validate_mmt4d(p));
  if (p.M == 0 || p.N == 0 || (p.K == 0 && (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE))) return 0;
  if (p.M0 == 0 || p.N0 == 0) return 0;
  Mmt4dTypeInfo ti;
  mmt4d_type_info(p.flags, &ti);
  const int64_t lhs_bytes = span_bytes(p.M, p.lhs_stride0, p.K * p.M0 * p.K0, ti.lhs_bits);
  const int64_t rhs_bytes = span_bytes(p.N, p.rhs_stride0, p.K * p.N0 * p.K0, ti.rhs_bits);
  const int64_t out_bytes = span_bytes(p.M, p.out_stride0, p.N * p.M0 * p.N0, ti.out_bytes * 8);
  const bool out_tight = p.out_stride0 == p.N * p.M0 * p.N0;
  const bool need_out_in = (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) || !out_tight;
  SlotLease slot(pool);
  UK_RETURN_IF_ERROR(slot.acquire());
  UK_RETURN_IF_ERROR(slot->upload(0, p.lhs_buffer, p.lhs_offset * ti.lhs_bits / 8, lhs_bytes, true));
  UK_RETURN_IF_ERROR(slot->upload(1, p.rhs_buffer, p.rhs_offset * ti.rhs_bits / 8, rhs_bytes, true));
  UK_RETURN_IF_ERROR(slot->upload(2, p.out_buffer, p.out_offset * ti.out_bytes, out_bytes, need_out_in));
  void* host_out = p.out_buffer;
  const int64_t host_out_off = p.out_offset * ti.out_bytes;
  p.lhs_buffer = slot->dev[0]; p.lhs_offset = 0;
  p.rhs_buffer = slot->dev[1]; p.rhs_offset = 0;
  p.out_buffer = slot->dev[2]; p.out_offset = 0;
  {
    // The copies over PCIe dwarf the kernel: K is never split here, so the call
    // needs no scratch memory and stays out of the per-stream cache.
    ScratchOverride no_scratch(nullptr, 0, /*strict=*/false);
    UK_RETURN_IF_ERROR(iree_amd_uk_mmt4d_p(&p, slot->stream));
  }
  return slot->download(2, host_out, host_out_off, out_bytes);
}

int pack_on(iree_amd_uk_host_pool_t* pool, const iree_amd_uk_pack_params_t* params) {
  if (!params) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack_host: null params");
  iree_amd_uk_pack_params_t p = *params;
  UK_RETURN_IF_ERROR(validate_pack(p));
  if (p.out_size0 == 0 || p.out_size1 == 0 || p.out_size2 == 0 || p.out_size3 == 0) return 0;
  const int es = pack_elem_bytes(p.flags);
  const int64_t in_row = p.in_size1 > 0 ? (p.in_size1 - 1) * p.in_stride1 + 1 : 0;
  const int64_t in_bytes = span_bytes(p.in_size0, p.in_stride0, in_row, es * 8);
  const int64_t out_bytes = span_bytes(p.out_size0, p.out_stride0, p.out_size1 * p.out_stride1, es * 8);
  const bool out_tight = p.out_stride0 == p.out_size1 * p.out_stride1;
  SlotLease slot(pool);
  UK_RETURN_IF_ERROR(slot.acquire());
  UK_RETURN_IF_ERROR(slot->upload(0, p.in_buffer, p.in_offset * es, in_bytes, true));
  UK_RETURN_IF_ERROR(slot->upload(2, p.out_buffer, p.out_offset * es, out_bytes, !out_tight));
  void* host_out = p.out_buffer;
  const int64_t host_out_off = p.out_offset * es;
  p.in_buffer = slot->dev[0]; p.in_offset = 0;
  p.out_buffer = slot->dev[2]; p.out_offset = 0;
  UK_RETURN_IF_ERROR(iree_amd_uk_pack_p(&p, slot->stream));
  return slot->download(2, host_out, host_out_off, out_bytes);
}

int unpack_on(iree_amd_uk_host_pool_t* pool, const iree_amd_uk_unpack_params_t* params) {
  if (!params) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "unpack_host: null params");
  iree_amd_uk_unpack_params_t p = *params;
  UK_RETURN_IF_ERROR(validate_unpack(p));
  if (p.out_size0 == 0 || p.out_size1 == 0) return 0;
  const int es = unpack_elem_bytes(p.flags);
  const int64_t in_bytes = span_bytes(p.in_size0, p.in_stride0, p.in_size1 * p.in_stride1, es * 8);
  const int64_t out_row = (p.out_size1 - 1) * p.out_stride1 + 1;
  const int64_t out_bytes = span_bytes(p.out_size0, p.out_stride0, out_row, es * 8);
  // The destination may have gaps (strides) the kernel must not disturb: start
  // from the caller's bytes unless the destination is dense.
  const bool out_dense = p.out_stride1 == 1 && p.out_stride0 == p.out_size1;
  SlotLease slot(pool);
  UK_RETURN_IF_ERROR(slot.acquire());
  UK_RETURN_IF_ERROR(slot->upload(0, p.in_buffer, p.in_offset * es, in_bytes, true));
  UK_RETURN_IF_ERROR(slot->upload(2, p.out_buffer, p.out_offset * es, out_bytes, !out_dense));
  void* host_out = p.out_buffer;
  const int64_t host_out_off = p.out_offset * es;
  p.in_buffer = slot->dev[0]; p.in_offset = 0;
  p.out_buffer = slot->dev[2]; p.out_offset = 0;
  UK_RETURN_IF_ERROR(iree_amd_uk_unpack_p(&p, slot->stream));
  return slot->download(2, host_out, host_out_off, out_bytes);
}

void destroy_pool_contents(iree_amd_uk_host_pool_t* pool) {
  for (HostSlot* s : pool->slots) {
    s->destroy();
    delete s;
  }
  pool->slots.clear();
}

// The entry points without a pool argument stage through a pool of their own
// that lives for the one call.
struct OneCallPool {
  iree_amd_uk_host_pool_t pool;
  ~OneCallPool() { destroy_pool_contents(&pool); }
};

}  // namespace

extern "C" int iree_amd_uk_host_pool_create(iree_amd_uk_host_pool_t** out_pool) {
  if (!out_pool) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "host_pool_create: null");
  *out_pool = new (std::nothrow) iree_amd_uk_host_pool_t();
  if (!*out_pool) return fail(8 /* RESOURCE_EXHAUSTED */, "host_pool_create: out of host memory");
  return 0;
}

extern "C" void iree_amd_uk_host_pool_destroy(iree_amd_uk_host_pool_t* pool) {
  if (!pool) return;
  destroy_pool_contents(pool);
  delete pool;
}

extern "C" int iree_amd_uk_mmt4d_host_pooled(iree_amd_uk_host_pool_t* pool,
                                             const iree_amd_uk_mmt4d_params_t* params) {
  if (!pool) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d_host_pooled: null pool");
  return mmt4d_on(pool, params);
}
extern "C" int iree_amd_uk_pack_host_pooled(iree_amd_uk_host_pool_t* pool,
                                            const iree_amd_uk_pack_params_t* params) {
  if (!pool) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "pack_host_pooled: null pool");
  return pack_on(pool, params);
}
extern "C" int iree_amd_uk_unpack_host_pooled(iree_amd_uk_host_pool_t* pool,
                                              const iree_amd_uk_unpack_params_t* params) {
  if (!pool) return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "unpack_host_pooled: null pool");
  return unpack_on(pool, params);
}

extern "C" int iree_amd_uk_mmt4d_host(const iree_amd_uk_mmt4d_params_t* params) {
  OneCallPool one;
  return mmt4d_on(&one.pool, params);
}
extern "C" int iree_amd_uk_pack_host(const iree_amd_uk_pack_params_t* params) {
  OneCallPool one;
  return pack_on(&one.pool, params);
}
extern "C" int iree_amd_uk_unpack_host(const iree_amd_uk_unpack_params_t* params) {
  OneCallPool one;
  return unpack_on(&one.pool, params);
}
