// Sub-allocation of torch's memory-pool segments out of large placed arenas. HIP-free: the device memory
// comes from two callbacks, so the bookkeeping can be driven on the CPU under the sanitizers.
//
// Why arenas: bikv_device_alloc spreads ONE allocation over both halves of HBM chunk by chunk, and a chunk is at
// least 256 MiB. The reference allocates its Worker pool as 28 tensors of 160 MiB (Bi-KV/Worker/Worker.py:74-78);
// given a placement each, every tensor would be one chunk, lying wherever the driver put it. Carved out of one
// arena one after the other, consecutive tensors land on consecutive chunks, which alternate between the halves.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <mutex>
#include <vector>

namespace bikv {
namespace arena {

constexpr int64_t kAlign = int64_t(2) << 20;        // torch asks for multiples of 2 MiB; keep its alignment

inline int64_t round_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

// backend(device, bytes) -> base or nullptr; release(base)
typedef void* (*BackendAlloc)(int device, int64_t bytes);
typedef void (*BackendFree)(void* base);

class Book {
 public:
  Book(int64_t arena_bytes, BackendAlloc alloc, BackendFree release)
      : arena_bytes_(arena_bytes), alloc_(alloc), release_(release) {}

  // A block of at least `size` bytes on `device`, 2 MiB aligned inside its arena; nullptr when the backend fails.
  // Requests above half an arena get an allocation of their own (which the backend spreads by itself).
  void* take(int device, int64_t size) {
    if (size <= 0) return nullptr;
    const int64_t sz = round_up(size, kAlign);
    std::lock_guard<std::mutex> lk(mu_);
    if (sz > arena_bytes_ / 2) {
      void* p = alloc_(device, sz);
      if (p) blocks_[p] = Block{-1, sz};
      return p;
    }
    // only the device's newest arena is filled, front to back, and nothing in it is reused while any of its
    // blocks is alive: neighbours in allocation order are neighbours in memory
    int newest = -1;
    for (size_t i = 0; i < arenas_.size(); ++i) {
      const Arena& a = arenas_[i];
      if (a.base && a.device == device && (newest < 0 || a.serial > arenas_[(size_t)newest].serial)) newest = (int)i;
    }
    if (newest >= 0 && arenas_[(size_t)newest].used + sz <= arenas_[(size_t)newest].bytes) return carve(newest, sz);
    void* base = alloc_(device, arena_bytes_);
    if (!base) return nullptr;
    int idx = -1;
    for (size_t i = 0; i < arenas_.size(); ++i)
      if (!arenas_[i].base) idx = (int)i;
    if (idx < 0) {
      arenas_.push_back(Arena());
      idx = (int)arenas_.size() - 1;
    }
    arenas_[(size_t)idx] = Arena{static_cast<char*>(base), arena_bytes_, 0, 0, device, ++serial_};
    return carve(idx, sz);
  }

  // Gives a block back; an arena whose last block is gone is released (or, when it is its device's newest,
  // rewound and kept for the next request). Returns false for a pointer take() did not hand out.
  bool give(void* p) {
    std::lock_guard<std::mutex> lk(mu_);
    auto it = blocks_.find(p);
    if (it == blocks_.end()) return false;
    const Block b = it->second;
    blocks_.erase(it);
    if (b.arena < 0) {
      release_(p);
      return true;
    }
    Arena& a = arenas_[(size_t)b.arena];
    if (--a.live > 0) return true;
    bool newest = true;
    for (const Arena& o : arenas_)
      if (o.base && o.device == a.device && o.serial > a.serial) newest = false;
    if (newest) {
      a.used = 0;
    } else {
      release_(a.base);
      a = Arena();
    }
    return true;
  }

  // for tests
  size_t live_blocks() {
    std::lock_guard<std::mutex> lk(mu_);
    return blocks_.size();
  }
  size_t live_arenas() {
    std::lock_guard<std::mutex> lk(mu_);
    size_t n = 0;
    for (const Arena& a : arenas_) n += a.base != nullptr;
    return n;
  }

 private:
  struct Arena {
    char* base = nullptr;
    int64_t bytes = 0, used = 0;
    int live = 0;
    int device = 0;
    uint64_t serial = 0;
  };
  struct Block {
    int arena;      // -1: an allocation of its own
    int64_t bytes;
  };
  void* carve(int idx, int64_t sz) {
    Arena& a = arenas_[(size_t)idx];
    void* p = a.base + a.used;
    a.used += sz;
    ++a.live;
    blocks_[p] = Block{idx, sz};
    return p;
  }

  const int64_t arena_bytes_;
  const BackendAlloc alloc_;
  const BackendFree release_;
  std::mutex mu_;
  std::vector<Arena> arenas_;
  std::map<void*, Block> blocks_;
  uint64_t serial_ = 0;
};

}  // namespace arena
}  // namespace bikv
