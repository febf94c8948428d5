// Policy of the library's scratch-buffer cache, free of any HIP dependency so
// that it can be unit-tested on a CPU with a counting allocator.
//
// Some kernels need device memory beyond their operands (the partial sums of a
// K split, a packed copy of a row-major left-hand side). The library keeps one
// buffer per (device, stream): work on one stream is ordered, so two calls on
// it never use the buffer at the same time. A caller takes a LEASE on the
// buffer before it builds its launches and drops it after the last of them has
// been queued; while a lease is out the entry is neither evicted nor replaced
// by a larger one (a second host thread on the same stream that needs more
// gets nothing and runs its fallback). An entry without a lease can be
//   * grown:   the old buffer is freed in stream order (everything that uses
//              it has already been queued on that stream),
//   * evicted: least recently used first, with a free that waits for the
//              device, when the table is full (streams come and go),
//   * released by release_idle() (a plugin's unload).
#ifndef IREE_AMD_UK_SCRATCH_CACHE_H_
#define IREE_AMD_UK_SCRATCH_CACHE_H_

#include <stddef.h>
#include <stdint.h>

#include <mutex>
#include <vector>

namespace uk {

struct ScratchAllocator {
  void* (*alloc)(size_t bytes, void* user);                      // nullptr when it fails
  void (*free_now)(void* ptr, void* user);                       // waits for work that uses ptr
  void (*free_ordered)(void* ptr, void* stream, void* user);     // behind the work queued on stream
  void* user;
};

class ScratchCache {
 public:
  struct Lease {
    void* ptr = nullptr;
    uint64_t id = 0;     // 0 = no lease held
  };

  ScratchCache(ScratchAllocator allocator, size_t min_bytes, size_t max_bytes, size_t max_entries)
      : allocator_(allocator), min_bytes_(min_bytes), max_bytes_(max_bytes), max_entries_(max_entries) {}

  size_t max_bytes() const { return max_bytes_; }

  // The buffer of (device, stream), at least `bytes` large, or a Lease without
  // a pointer when it cannot be had. Every Lease with an id must be released.
  Lease acquire(int device, void* stream, size_t bytes) {
    Lease none;
    if (bytes == 0 || bytes > max_bytes_) return none;
    std::unique_lock<std::mutex> lock(mutex_);
    for (Entry& e : entries_) {
      if (e.device != device || e.stream != stream) continue;
      if (e.bytes < bytes) {
        if (e.leases > 0) return none;      // in use: not replaced under its user
        const size_t want = bytes * 2 < max_bytes_ ? bytes * 2 : max_bytes_;
        void* bigger = allocator_.alloc(want, allocator_.user);
        if (!bigger) return none;
        allocator_.free_ordered(e.ptr, stream, allocator_.user);
        e.ptr = bigger;
        e.bytes = want;
      }
      return lease_of(e);
    }
    // A new entry. When the table is full the least recently used idle buffer
    // makes room; it leaves the table here and is freed (a free that waits for
    // the device) only after the lock has been dropped, so that other threads'
    // calls do not queue behind that wait.
    void* evicted = nullptr;
    if (entries_.size() >= max_entries_) {
      size_t victim = entries_.size();
      for (size_t i = 0; i < entries_.size(); ++i)
        if (entries_[i].leases == 0 && (victim == entries_.size() || entries_[i].last_use < entries_[victim].last_use))
          victim = i;
      if (victim == entries_.size()) return none;   // every buffer is in use
      evicted = entries_[victim].ptr;
      entries_.erase(entries_.begin() + (long)victim);
    }
    const size_t want = bytes < min_bytes_ ? min_bytes_ : bytes;
    void* ptr = allocator_.alloc(want, allocator_.user);
    if (!ptr && evicted) {
      // (out of memory with the victim still allocated: free it first after all)
      allocator_.free_now(evicted, allocator_.user);
      evicted = nullptr;
      ptr = allocator_.alloc(want, allocator_.user);
    }
    Lease lease;
    if (ptr) {
      entries_.push_back(Entry{device, stream, ptr, want, 0, 0, next_id_++});
      lease = lease_of(entries_.back());
    }
    lock.unlock();
    if (evicted) allocator_.free_now(evicted, allocator_.user);
    return lease;
  }

  void release(const Lease& lease) {
    if (!lease.id) return;
    std::lock_guard<std::mutex> lock(mutex_);
    for (Entry& e : entries_)
      if (e.id == lease.id) {
        if (e.leases > 0) --e.leases;
        return;
      }
  }

  // Frees every buffer without a lease; returns how many were freed.
  size_t release_idle() {
    std::vector<void*> idle;
    {
      std::lock_guard<std::mutex> lock(mutex_);
      for (size_t i = 0; i < entries_.size();) {
        if (entries_[i].leases == 0) {
          idle.push_back(entries_[i].ptr);
          entries_.erase(entries_.begin() + (long)i);
        } else {
          ++i;
        }
      }
    }
    // (freed outside the lock: each free waits for the device)
    for (void* p : idle) allocator_.free_now(p, allocator_.user);
    return idle.size();
  }

  size_t entry_count() {
    std::lock_guard<std::mutex> lock(mutex_);
    return entries_.size();
  }

 private:
  struct Entry {
    int device;
    void* stream;
    void* ptr;
    size_t bytes;
    int leases;
    uint64_t last_use;
    uint64_t id;       // survives reordering of the table; a grown buffer keeps it
  };

  Lease lease_of(Entry& e) {
    ++e.leases;
    e.last_use = ++clock_;
    Lease l;
    l.ptr = e.ptr;
    l.id = e.id;
    return l;
  }

  ScratchAllocator allocator_;
  size_t min_bytes_, max_bytes_, max_entries_;
  std::mutex mutex_;
  std::vector<Entry> entries_;
  uint64_t clock_ = 0, next_id_ = 1;
};

}  // namespace uk

#endif  // IREE_AMD_UK_SCRATCH_CACHE_H_
