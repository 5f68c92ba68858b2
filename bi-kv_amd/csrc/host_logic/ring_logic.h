// Bookkeeping of the producer/consumer ring over the shared control block: the reference's wrap and
// publish rules (Bi-KV/SharedMemory/CUDA_Shared/copy_kernel.cu:84-89,115-128, ipc_service.cpp:130-142),
// the optional back-pressure through sem_complete, and the lock that makes a producer's transfer one
// step for the other threads of its process. Pure host logic (no HIP): ipc_ring.hip builds the roles on
// it, and the sanitizer-built host tests drive it from several threads over a malloc'd control block.
#pragma once
#include <errno.h>
#include <semaphore.h>
#include <stdint.h>
#include <string.h>
#include <time.h>

#include <deque>
#include <mutex>
#include <utility>

#include "../../../include/bikv_pagecopy.h"

namespace bikv {
namespace ring {

enum : int { WAIT_OK = 0, WAIT_TIMEOUT = 1, WAIT_ERROR = 2 };   // WAIT_ERROR: errno says why

inline sem_t* sem_of(unsigned char* raw) { return reinterpret_cast<sem_t*>(raw); }

// sem_wait with a timeout in milliseconds (< 0: wait forever); restarted after signals.
inline int wait_ms(sem_t* s, int64_t timeout_ms) {
  int rc;
  if (timeout_ms < 0) {
    do { rc = sem_wait(s); } while (rc == -1 && errno == EINTR);
  } else {
    struct timespec ts;
    clock_gettime(CLOCK_REALTIME, &ts);
    ts.tv_sec += timeout_ms / 1000;
    ts.tv_nsec += (timeout_ms % 1000) * 1000000L;
    if (ts.tv_nsec >= 1000000000L) {
      ts.tv_sec += 1;
      ts.tv_nsec -= 1000000000L;
    }
    do { rc = sem_timedwait(s, &ts); } while (rc == -1 && errno == EINTR);
  }
  if (rc == 0) return WAIT_OK;
  return errno == ETIMEDOUT ? WAIT_TIMEOUT : WAIT_ERROR;
}

// The reference's ring advance (copy_kernel.cu:87-89): a batch that does not fit behind the current
// offset restarts at 0. Returns the write offset; the offset itself only moves when the transfer is
// published.
inline size_t wrap_offset(bikv_shared_control* c, size_t data_size) {
  if (c->current_offset + data_size > c->buffer_size) c->current_offset = 0;
  return c->current_offset;
}

// The reference's publish step (copy_kernel.cu:116-128, ipc_service.cpp:130-142) for the transfer
// written at offset `at` (the value wrap_offset returned for it).
inline void publish(bikv_shared_control* c, size_t at, size_t data_size, const int64_t* shape, size_t ndim,
                    int32_t dtype_code) {
  c->last_valid_offset = at;
  c->current_offset = at + data_size;
  c->tensor_dim = ndim;
  for (size_t i = 0; i < ndim && i < BIKV_MAX_DIM; ++i) c->tensor_shape[i] = shape[i];
  c->data_size = data_size;
  c->dtype_code = dtype_code;
  sem_post(sem_of(c->sem_start));
}

// Producer-side state of one process. `mu` is held for the whole of a transfer — window, copy,
// publication — because the ring's write offset only moves at publication: two threads that reserved
// at the same time would be handed the same window (the reference's process-global statics,
// ipc_service.cpp:9-17, have exactly that race under its 20-thread gRPC pools).
struct Producer {
  std::mutex mu;
  bikv_shared_control* ctrl = nullptr;
  // back-pressure: transfers published and not yet released by the consumer, oldest first, as
  // (ring offset, bytes)
  bool backpressure = false;
  int64_t bp_timeout_ms = -1;
  std::deque<std::pair<size_t, size_t>> in_flight;
  // window handed out by the two-step form (reserve ... publish) and not published yet
  bool reserved = false;
  size_t reserved_at = 0, reserved_bytes = 0;
};

// Ring advance for the producer (caller holds p.mu). Without back-pressure this is wrap_offset. With it,
// the window [at, at+data_size) must not touch a transfer the consumer still holds: the consumer posts
// sem_complete once per transfer it is done with, in order, and the producer blocks here until every
// overlapping transfer has been released (the reference declares sem_complete, ipc_wrapper.h:16,
// initialises it, ipc_service.cpp:47, and never uses it: a wrapping producer overwrites tensors the
// consumer may still read).
inline int reserve_window(Producer& p, size_t data_size, size_t* at_out) {
  bikv_shared_control* c = p.ctrl;
  const size_t at = wrap_offset(c, data_size);
  *at_out = at;
  if (!p.backpressure) return WAIT_OK;
  sem_t* done = sem_of(c->sem_complete);
  while (!p.in_flight.empty() && sem_trywait(done) == 0) p.in_flight.pop_front();
  for (;;) {
    bool overlap = false;
    for (const auto& t : p.in_flight)
      if (t.second > 0 && data_size > 0 && t.first < at + data_size && at < t.first + t.second) overlap = true;
    if (!overlap) return WAIT_OK;
    const int rc = wait_ms(done, p.bp_timeout_ms);
    if (rc != WAIT_OK) return rc;
    p.in_flight.pop_front();
  }
}

// The control block has ONE slot for the published offset and shape (ipc_wrapper.h:21-27), so with
// back-pressure a transfer is published only once the consumer has released the previous one: the copy
// of transfer k+1 overlaps the consumer's use of transfer k, its publication does not. Caller holds p.mu.
inline int wait_slot(Producer& p) {
  if (!p.backpressure) return WAIT_OK;
  sem_t* done = sem_of(p.ctrl->sem_complete);
  while (!p.in_flight.empty()) {
    const int rc = wait_ms(done, p.bp_timeout_ms);
    if (rc != WAIT_OK) return rc;
    p.in_flight.pop_front();
  }
  return WAIT_OK;
}

// Publishes the transfer written at `at` and, with back-pressure, notes it as in flight. Caller holds p.mu.
inline void publish_transfer(Producer& p, size_t at, size_t data_size, const int64_t* shape, size_t ndim,
                             int32_t dtype_code) {
  publish(p.ctrl, at, data_size, shape, ndim, dtype_code);
  if (p.backpressure) p.in_flight.emplace_back(at, data_size);
}

// Fills a fresh control block so that a producer which maps it at any moment sees either "no ring yet"
// (buffer_size == 0) or the finished description: everything but buffer_size is written first, the
// semaphores are initialised, and buffer_size is stored last with release order. describes_ring() is
// the matching acquire load on the producer's side.
inline void describe_ring(bikv_shared_control* c, const bikv_shared_control& image) {
  bikv_shared_control tmp = image;
  tmp.buffer_size = 0;
  memcpy(c, &tmp, sizeof(tmp));
  sem_init(sem_of(c->sem_start), 1, 0);
  sem_init(sem_of(c->sem_complete), 1, 0);
  __atomic_store_n(&c->buffer_size, image.buffer_size, __ATOMIC_RELEASE);
}
inline size_t describes_ring(const bikv_shared_control* c) {
  return __atomic_load_n(&c->buffer_size, __ATOMIC_ACQUIRE);
}

}  // namespace ring
}  // namespace bikv
