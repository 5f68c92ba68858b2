// Three producer threads and a consumer drive the ring bookkeeping (ring_logic.h) under the thread
// sanitizer. The ring itself is host memory standing in for the device buffer. With back-pressure on,
// every transfer must reach the consumer exactly once with the bytes its producer wrote: no window handed
// out twice, no publication lost, no slot overwritten before it was read.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>
#include <map>
#include <mutex>
#include <sys/mman.h>

#include "arena_logic.h"
#include "ring_logic.h"

using namespace bikv;

static void die(const char* what) {
  fprintf(stderr, "ring_threads: %s\n", what);
  abort();
}

// The arena bookkeeping behind the torch allocator hooks, driven from four threads at once over a backend
// that hands out address space only: every block a thread holds lies inside a live backend allocation and
// overlaps no block of any other thread (each thread stamps its block's first and last byte address into a
// shared map under its own lock and checks for intruders).
static std::mutex g_backend_mu;
static std::map<char*, int64_t> g_backend_live;
static void* arena_backend_alloc(int, int64_t bytes) {
  void* p = mmap(nullptr, (size_t)bytes, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
  if (p == MAP_FAILED) die("mmap");
  std::lock_guard<std::mutex> lk(g_backend_mu);
  g_backend_live[(char*)p] = bytes;
  return p;
}
static void arena_backend_free(void* base) {
  int64_t bytes;
  {
    std::lock_guard<std::mutex> lk(g_backend_mu);
    auto it = g_backend_live.find((char*)base);
    if (it == g_backend_live.end()) die("release of memory the backend did not hand out");
    bytes = it->second;
    g_backend_live.erase(it);
  }
  munmap(base, (size_t)bytes);
}
static void arena_threads() {
  bikv::arena::Book book(int64_t(2) << 30, arena_backend_alloc, arena_backend_free);
  std::mutex held_mu;
  std::map<char*, int64_t> held;                 // every block currently held by any thread
  std::vector<std::thread> threads;
  for (int t = 0; t < 4; ++t)
    threads.emplace_back([&, t] {
      uint64_t x = 88172645463325252ull + (uint64_t)t * 977;
      auto rnd = [&] { x ^= x << 13; x ^= x >> 7; x ^= x << 17; return x; };
      std::vector<std::pair<char*, int64_t>> mine;
      for (int step = 0; step < 600; ++step) {
        if (mine.empty() || rnd() % 3) {
          const int64_t sz = (int64_t)(rnd() % 1300 + 1) << 20;          // some above half an arena
          char* q = (char*)book.take((int)(rnd() % 2), sz);
          if (!q) die("take failed");
          const int64_t r = bikv::arena::round_up(sz, bikv::arena::kAlign);
          {
            std::lock_guard<std::mutex> lk(g_backend_mu);
            auto it = g_backend_live.upper_bound(q);
            if (it == g_backend_live.begin()) die("block below every backend allocation");
            --it;
            if (q + r > it->first + it->second) die("block sticks out of its backend allocation");
          }
          {
            std::lock_guard<std::mutex> lk(held_mu);
            auto nx = held.lower_bound(q);
            if (nx != held.end() && q + r > nx->first) die("block overlaps another thread's block");
            if (nx != held.begin()) { --nx; if (nx->first + nx->second > q) die("block overlaps another thread's block"); }
            held[q] = r;
          }
          mine.emplace_back(q, r);
        } else {
          const size_t k = (size_t)(rnd() % mine.size());
          { std::lock_guard<std::mutex> lk(held_mu); held.erase(mine[k].first); }
          if (!book.give(mine[k].first)) die("give refused a live block");
          mine.erase(mine.begin() + (long)k);
        }
      }
      for (auto& b : mine) {
        { std::lock_guard<std::mutex> lk(held_mu); held.erase(b.first); }
        if (!book.give(b.first)) die("give refused a live block");
      }
    });
  for (auto& th : threads) th.join();
  if (book.live_blocks() != 0) die("blocks left behind");
  std::lock_guard<std::mutex> lk(g_backend_mu);
  if (g_backend_live.size() > 2) die("more than the two kept arenas (one per device) left with the backend");
  for (auto& b : g_backend_live) munmap(b.first, (size_t)b.second);
  g_backend_live.clear();
}

int main() {
  arena_threads();
  const int kProducers = 3, kPerProducer = 400;
  const size_t kRing = 4096;
  bikv_shared_control* c = static_cast<bikv_shared_control*>(malloc(sizeof(bikv_shared_control)));
  unsigned char* ring_mem = static_cast<unsigned char*>(malloc(kRing));
  bikv_shared_control image;
  memset(&image, 0, sizeof(image));
  image.buffer_size = kRing;
  ring::describe_ring(c, image);
  ring::Producer p;
  p.ctrl = c;
  p.backpressure = true;
  p.bp_timeout_ms = 20000;

  std::vector<int> seen((size_t)(kProducers * kPerProducer), 0);
  std::thread consumer([&] {
    for (int k = 0; k < kProducers * kPerProducer; ++k) {
      if (ring::wait_ms(ring::sem_of(c->sem_start), 20000) != ring::WAIT_OK) die("consumer timed out");
      const size_t at = c->last_valid_offset, n = c->data_size;
      const int64_t tag = c->tensor_shape[0];
      if (c->tensor_dim != 2 || (size_t)c->tensor_shape[1] != n || at + n > kRing) die("bad publication");
      if (tag < 0 || tag >= (int64_t)seen.size()) die("bad tag");
      for (size_t i = 0; i < n; ++i)
        if (ring_mem[at + i] != (unsigned char)(tag * 7 + (int64_t)i)) die("window holds somebody else's bytes");
      seen[(size_t)tag] += 1;
      sem_post(ring::sem_of(c->sem_complete));   // release: the producer may publish the next one
    }
  });
  std::vector<std::thread> producers;
  for (int t = 0; t < kProducers; ++t)
    producers.emplace_back([&, t] {
      for (int k = 0; k < kPerProducer; ++k) {
        const int64_t tag = (int64_t)t * kPerProducer + k;
        const size_t n = 64 + (size_t)((tag * 37) % 1500);
        std::lock_guard<std::mutex> lk(p.mu);                  // one transfer is one step
        size_t at = 0;
        if (ring::reserve_window(p, n, &at) != ring::WAIT_OK) die("reserve timed out");
        for (size_t i = 0; i < n; ++i) ring_mem[at + i] = (unsigned char)(tag * 7 + (int64_t)i);   // "the copy"
        if (ring::wait_slot(p) != ring::WAIT_OK) die("slot wait timed out");
        const int64_t shape[2] = {tag, (int64_t)n};
        ring::publish_transfer(p, at, n, shape, 2, 0);
      }
    });
  for (auto& th : producers) th.join();
  consumer.join();
  for (int v : seen)
    if (v != 1) die("a transfer was lost or delivered twice");
  free(ring_mem);
  free(c);
  printf("ring_threads ok\n");
  return 0;
}
