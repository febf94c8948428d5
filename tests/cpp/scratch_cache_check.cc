// CPU-only check of the scratch cache policy (iree_amd/csrc/uk_scratch_cache.h)
// with a counting allocator: no GPU, no HIP. Prints "ok" and exits 0, or the
// failed condition and exits 1.
#include <stdio.h>
#include <stdlib.h>

#include <atomic>
#include <set>
#include <thread>
#include <vector>

#include "uk_scratch_cache.h"

#define CHECK(cond)                                               \
  do {                                                            \
    if (!(cond)) {                                                \
      fprintf(stderr, "%s:%d: CHECK(%s)\n", __FILE__, __LINE__, #cond); \
      exit(1);                                                    \
    }                                                             \
  } while (0)

namespace {

struct Counting {
  std::mutex m;
  std::set<void*> live;
  int allocs = 0, frees_now = 0, frees_ordered = 0;
  size_t fail_above = ~(size_t)0;
};

void* c_alloc(size_t bytes, void* user) {
  Counting* c = (Counting*)user;
  std::lock_guard<std::mutex> l(c->m);
  if (bytes > c->fail_above) return nullptr;
  void* p = malloc(16);
  c->live.insert(p);
  ++c->allocs;
  return p;
}
void c_free(Counting* c, void* p) {
  std::lock_guard<std::mutex> l(c->m);
  CHECK(c->live.count(p) == 1);     // no double free, no foreign pointer
  c->live.erase(p);
  free(p);
}
void c_free_now(void* p, void* user) { ++((Counting*)user)->frees_now; c_free((Counting*)user, p); }
void c_free_ordered(void* p, void*, void* user) { ++((Counting*)user)->frees_ordered; c_free((Counting*)user, p); }

uk::ScratchAllocator allocator(Counting* c) { return uk::ScratchAllocator{c_alloc, c_free_now, c_free_ordered, c}; }
void* stream(int i) { return (void*)(uintptr_t)(0x1000 + i); }

}  // namespace

int main() {
  // reuse, minimum size, growth in stream order
  {
    Counting c;
    uk::ScratchCache cache(allocator(&c), 100, 1000, 4);
    auto a = cache.acquire(0, stream(0), 10);
    CHECK(a.ptr && a.id && c.allocs == 1);
    cache.release(a);
    auto b = cache.acquire(0, stream(0), 90);
    CHECK(b.ptr == a.ptr && c.allocs == 1);          // the 100-byte minimum already holds 90
    cache.release(b);
    auto g = cache.acquire(0, stream(0), 300);
    CHECK(g.ptr && g.ptr != a.ptr && c.allocs == 2 && c.frees_ordered == 1 && c.frees_now == 0);
    cache.release(g);
    CHECK(!cache.acquire(0, stream(0), 0).ptr);       // nothing asked for
    CHECK(!cache.acquire(0, stream(0), 1001).ptr);    // beyond the maximum
    CHECK(cache.entry_count() == 1);
    // another device with the same stream handle is another entry
    auto d1 = cache.acquire(1, stream(0), 10);
    CHECK(d1.ptr && d1.ptr != g.ptr && cache.entry_count() == 2);
    cache.release(d1);
    CHECK(cache.release_idle() == 2 && c.live.empty());
  }
  // a leased buffer is not grown under its user
  {
    Counting c;
    uk::ScratchCache cache(allocator(&c), 100, 1000, 4);
    auto a = cache.acquire(0, stream(0), 50);
    auto b = cache.acquire(0, stream(0), 500);        // second host thread, same stream, needs more
    CHECK(a.ptr && !b.ptr && !b.id && c.allocs == 1 && c.frees_ordered == 0);
    auto s = cache.acquire(0, stream(0), 60);         // what fits is shared (same stream = ordered work)
    CHECK(s.ptr == a.ptr);
    cache.release(s);
    cache.release(a);
    auto g = cache.acquire(0, stream(0), 500);
    CHECK(g.ptr && c.allocs == 2 && c.frees_ordered == 1);
    cache.release(g);
    cache.release_idle();
    CHECK(c.live.empty());
  }
  // eviction: least recently used entry WITHOUT a lease; none when all are leased
  {
    Counting c;
    uk::ScratchCache cache(allocator(&c), 100, 1000, 3);
    auto l0 = cache.acquire(0, stream(0), 10);
    auto l1 = cache.acquire(0, stream(1), 10);
    auto l2 = cache.acquire(0, stream(2), 10);
    CHECK(l0.ptr && l1.ptr && l2.ptr && cache.entry_count() == 3);
    CHECK(!cache.acquire(0, stream(3), 10).ptr && c.frees_now == 0);   // all in use: nothing evicted
    cache.release(l1);
    cache.release(l2);
    auto t = cache.acquire(0, stream(2), 10);         // touch stream 2: stream 1 is now the oldest idle one
    cache.release(t);
    auto l3 = cache.acquire(0, stream(3), 10);
    CHECK(l3.ptr && c.frees_now == 1 && cache.entry_count() == 3);
    CHECK(c.live.count(l1.ptr) == 0);                 // stream 1's buffer went
    CHECK(c.live.count(l0.ptr) == 1 && c.live.count(l2.ptr) == 1);   // the leased and the recent one stayed
    cache.release(l3);
    CHECK(cache.release_idle() == 2);                 // stream 0 is still leased
    CHECK(cache.entry_count() == 1 && c.live.count(l0.ptr) == 1);
    cache.release(l0);
    CHECK(cache.release_idle() == 1 && c.live.empty());
  }
  // allocation failure leaves the table as it was
  {
    Counting c;
    c.fail_above = 200;
    uk::ScratchCache cache(allocator(&c), 100, 1000, 2);
    auto a = cache.acquire(0, stream(0), 50);
    cache.release(a);
    CHECK(!cache.acquire(0, stream(0), 150).ptr);     // grows to 300: refused
    auto again = cache.acquire(0, stream(0), 50);
    CHECK(again.ptr == a.ptr && c.frees_ordered == 0);
    cache.release(again);
    CHECK(!cache.acquire(0, stream(1), 250).ptr && cache.entry_count() == 1);
    cache.release_idle();
    CHECK(c.live.empty());
  }
  // many threads, more streams than entries: every lease is exclusive of
  // eviction for as long as it is held
  {
    Counting c;
    uk::ScratchCache cache(allocator(&c), 100, 1000, 4);
    std::atomic<int> bad{0}, served{0};
    std::vector<std::thread> threads;
    for (int t = 0; t < 8; ++t)
      threads.emplace_back([&, t] {
        for (int i = 0; i < 2000; ++i) {
          auto l = cache.acquire(0, stream(t), 10 + (size_t)(i % 7) * 40);
          if (!l.ptr) continue;
          ++served;
          {
            std::lock_guard<std::mutex> g(c.m);
            if (c.live.count(l.ptr) != 1) ++bad;      // freed while leased
          }
          std::this_thread::yield();
          {
            std::lock_guard<std::mutex> g(c.m);
            if (c.live.count(l.ptr) != 1) ++bad;
          }
          cache.release(l);
        }
      });
    for (auto& th : threads) th.join();
    CHECK(bad == 0 && served > 0);
    cache.release_idle();
    CHECK(c.live.empty() && cache.entry_count() == 0);
  }
  printf("ok\n");
  return 0;
}
