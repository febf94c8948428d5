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
//
// A large mmt4d is pipelined over blocks of outer rows: the calling thread
// uploads the right-hand side once and then, block by block, the left-hand-side
// rows, and launches the kernel on each block; helper threads that belong to
// the slot copy every finished block of the result back while the next
// blocks are still going up. Copies from and to pageable host memory block the
// thread that issues them, so the two directions of the PCIe link are only
// busy at the same time with a thread for each.
#include "uk_common.h"

#include <algorithm>
#include <condition_variable>
#include <deque>
#include <mutex>
#include <thread>
#include <vector>

namespace {

using namespace uk;

constexpr size_t kMaxSlots = 8;

constexpr int kMaxBlocks = 16;
// Helper threads per slot. One thread's copy to pageable memory runs at the
// speed of the runtime's staging copy on that thread, well below the link's.
constexpr int kWorkers = 3;

struct HostSlot {
  int device = 0;
  hipStream_t stream = nullptr;
  void* dev[3] = {nullptr, nullptr, nullptr};
  size_t cap[3] = {0, 0, 0};
  bool busy = false;
  // the helper thread that downloads finished blocks (started with the first
  // pipelined call, joined when the slot is destroyed)
  struct Job { hipEvent_t ready; const void* src; void* dst; size_t bytes; bool to_device; };   // ready: may be null
  hipStream_t out_stream[kWorkers] = {};
  hipEvent_t events[kMaxBlocks] = {};
  std::thread worker[kWorkers];
  std::mutex job_mutex;
  std::condition_variable job_cv, done_cv;
  std::deque<Job> jobs;
  int jobs_open = 0;        // queued or running
  int job_status = 0;       // first failure of the current call
  bool quit = false;

  int init() {
    UK_RETURN_IF_HIP(hipGetDevice(&device));
    // (default priority on purpose: mixed stream priorities are not used)
    return check_hip(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking), "hipStreamCreate");
  }
  void destroy() {
    {
      std::lock_guard<std::mutex> lock(job_mutex);
      quit = true;
    }
    job_cv.notify_all();
    for (std::thread& w : worker)
      if (w.joinable()) w.join();
    for (hipEvent_t& e : events) {
      if (e && hipEventDestroy(e) != hipSuccess) (void)hipGetLastError();
      e = nullptr;
    }
    for (hipStream_t& o : out_stream) {
      if (o && hipStreamDestroy(o) != hipSuccess) (void)hipGetLastError();
      o = nullptr;
    }
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

  // ---- the download helper -------------------------------------------------
  void worker_main(int w) {
    if (hipSetDevice(device) != hipSuccess) (void)hipGetLastError();
    hipStream_t mine = out_stream[w];
    for (;;) {
      Job job;
      {
        std::unique_lock<std::mutex> lock(job_mutex);
        job_cv.wait(lock, [&] { return quit || !jobs.empty(); });
        if (jobs.empty()) return;      // quit
        job = jobs.front();
        jobs.pop_front();
      }
      hipError_t err = job.ready ? hipStreamWaitEvent(mine, job.ready, 0) : hipSuccess;
      if (err == hipSuccess)
        err = hipMemcpyAsync(job.dst, job.src, job.bytes, job.to_device ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost,
                             mine);
      if (err == hipSuccess) err = hipStreamSynchronize(mine);
      if (err != hipSuccess) (void)hipGetLastError();
      {
        std::lock_guard<std::mutex> lock(job_mutex);
        if (err != hipSuccess && !job_status) job_status = IREE_AMD_UK_STATUS_INTERNAL;
        --jobs_open;
      }
      done_cv.notify_all();
    }
  }
  int start_worker() {
    if (worker[kWorkers - 1].joinable()) return 0;
    for (hipStream_t& o : out_stream)
      if (!o) UK_RETURN_IF_HIP(hipStreamCreateWithFlags(&o, hipStreamNonBlocking));
    for (hipEvent_t& e : events)
      if (!e) UK_RETURN_IF_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    for (int w = 0; w < kWorkers; ++w)
      if (!worker[w].joinable()) worker[w] = std::thread([this, w] { worker_main(w); });
    return 0;
  }
  void submit(const Job& job) {
    {
      std::lock_guard<std::mutex> lock(job_mutex);
      jobs.push_back(job);
      ++jobs_open;
    }
    job_cv.notify_one();
  }
  // Waits for every submitted copy; returns the first failure.
  int drain() {
    std::unique_lock<std::mutex> lock(job_mutex);
    done_cv.wait(lock, [&] { return jobs_open == 0; });
    const int st = job_status;
    job_status = 0;
    return st ? fail(st, "host-pointer mmt4d: a copy on a helper thread failed") : 0;
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
    pool_->freed.notify_all();     // (waiters may be after slots of different devices)
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
        // The new slot is entered as busy first and set up (a stream is
        // created) with the pool unlocked, so other threads' calls do not
        // wait behind the driver.
        HostSlot* s = new HostSlot();
        s->device = device;
        s->busy = true;
        pool_->slots.push_back(s);
        lock.unlock();
        const int st = s->init();
        if (st) {
          lock.lock();
          auto& v = pool_->slots;
          v.erase(std::remove(v.begin(), v.end(), s), v.end());
          lock.unlock();
          delete s;
          pool_->freed.notify_all();
          return st;
        }
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
  // Large problems with a dense result: blocks of outer rows, downloads of
  // finished blocks overlapping the uploads of the next ones.
  const int64_t lhs_row_bytes = p.lhs_stride0 * ti.lhs_bits / 8;
  const int64_t out_row_bytes = p.out_stride0 * ti.out_bytes;
  if (out_tight && p.M >= 4 && out_bytes >= ((int64_t)8 << 20) && (p.lhs_stride0 * ti.lhs_bits) % 8 == 0 &&
      lhs_row_bytes % 16 == 0) {
    UK_RETURN_IF_ERROR(slot->start_worker());
    UK_RETURN_IF_ERROR(slot->ensure(0, lhs_bytes));
    UK_RETURN_IF_ERROR(slot->ensure(2, out_bytes));
    {
      // the right-hand side, which the first block already needs whole: one
      // part per thread, the helpers' parts finished (on the host's clock)
      // before the first launch is queued
      UK_RETURN_IF_ERROR(slot->ensure(1, rhs_bytes));
      const char* host_rhs = (const char*)p.rhs_buffer + p.rhs_offset * ti.rhs_bits / 8;
      const int64_t part = ((rhs_bytes / (kWorkers + 1)) + 255) & ~(int64_t)255;
      for (int w = 1; w <= kWorkers; ++w) {
        const int64_t at = w * part;
        if (at >= rhs_bytes) break;
        const int64_t n = rhs_bytes - at < part ? rhs_bytes - at : part;
        slot->submit(HostSlot::Job{nullptr, host_rhs + at, (char*)slot->dev[1] + at, (size_t)n, true});
      }
      const int first = check_hip(hipMemcpyAsync(slot->dev[1], host_rhs, (size_t)(part < rhs_bytes ? part : rhs_bytes),
                                                 hipMemcpyHostToDevice, slot->stream), "hipMemcpyAsync(h2d)");
      const int others = slot->drain();
      UK_RETURN_IF_ERROR(first);
      UK_RETURN_IF_ERROR(others);
    }
    const char* host_lhs = (const char*)p.lhs_buffer + p.lhs_offset * ti.lhs_bits / 8;
    char* host_out = (char*)p.out_buffer + p.out_offset * ti.out_bytes;
    const int64_t blocks = p.M < kMaxBlocks ? p.M : kMaxBlocks;
    const int64_t rows_per_block = (p.M + blocks - 1) / blocks;
    int status = 0, b = 0;
    for (int64_t r0 = 0; r0 < p.M && !status; r0 += rows_per_block, ++b) {
      const int64_t rows = p.M - r0 < rows_per_block ? p.M - r0 : rows_per_block;
      const int64_t up = span_bytes(rows, p.lhs_stride0, p.K * p.M0 * p.K0, ti.lhs_bits);
      const int64_t down = rows * out_row_bytes;
      status = check_hip(hipMemcpyAsync((char*)slot->dev[0] + r0 * lhs_row_bytes, host_lhs + r0 * lhs_row_bytes,
                                        (size_t)up, hipMemcpyHostToDevice, slot->stream), "hipMemcpyAsync(h2d)");
      if (!status && (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE))
        status = check_hip(hipMemcpyAsync((char*)slot->dev[2] + r0 * out_row_bytes, host_out + r0 * out_row_bytes,
                                          (size_t)down, hipMemcpyHostToDevice, slot->stream), "hipMemcpyAsync(h2d)");
      if (status) break;
      iree_amd_uk_mmt4d_params_t q = p;
      q.lhs_buffer = (char*)slot->dev[0] + r0 * lhs_row_bytes; q.lhs_offset = 0;
      q.rhs_buffer = slot->dev[1]; q.rhs_offset = 0;
      q.out_buffer = (char*)slot->dev[2] + r0 * out_row_bytes; q.out_offset = 0;
      q.M = rows;
      {
        ScratchOverride no_scratch(nullptr, 0, /*strict=*/false);
        status = iree_amd_uk_mmt4d_p(&q, slot->stream);
      }
      if (!status) status = check_hip(hipEventRecord(slot->events[b], slot->stream), "hipEventRecord");
      if (!status)
        slot->submit(HostSlot::Job{slot->events[b], (char*)slot->dev[2] + r0 * out_row_bytes,
                                   host_out + r0 * out_row_bytes, (size_t)down, false});
    }
    const int drained = slot->drain();      // (also after a failure: the helper must be idle again)
    if (status) {
      (void)hipStreamSynchronize(slot->stream);
      (void)hipGetLastError();
      return status;
    }
    return drained;
  }
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
