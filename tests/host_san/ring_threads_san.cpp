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

#include "ring_logic.h"

using namespace bikv;

static void die(const char* what) {
  fprintf(stderr, "ring_threads: %s\n", what);
  abort();
}

int main() {
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
