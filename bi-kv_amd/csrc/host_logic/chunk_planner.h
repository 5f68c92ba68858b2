// Cuts the staging image of a batch into the pieces the host stager moves, one lane buffer at a time.
// Pure host logic (no HIP): the stager uses it, bikv_plan_chunks exposes it, and the sanitizer-built
// host tests drive it directly.
#pragma once
#include <stdint.h>

#include "../../../include/bikv_pagecopy.h"

namespace bikv {

// One contiguous byte range of the staging image together with the rectangle of
// (batch pages x planes) that fills it.
struct Chunk {
  int64_t first_page, n_pages;  // batch entries
  int plane_begin, plane_count;
  int64_t first_slot, n_slots;  // staging slots covered
};

// Pieces of at most `max_slots` slots, one per call of next(). Requests are packed back to back in batch
// order. An iterator: it holds no memory of its own, so the allocation-free entry point can use it.
class ChunkPlanner {
 public:
  ChunkPlanner(const int64_t* req_pages, int64_t n_req, int n_planes, int layout, int64_t max_slots)
      : req_(req_pages), n_req_(n_req), planes_(n_planes), layout_(layout), max_(max_slots) {
    if (layout_ == BIKV_LAYOUT_PAGE_MAJOR)
      for (int64_t r = 0; r < n_req_; ++r) total_ += req_[r];
  }

  bool next(Chunk* out) {
    if (layout_ == BIKV_LAYOUT_PAGE_MAJOR) {
      // slot = global_page * n_planes + plane: any run of whole pages is contiguous, across requests
      if (p_ >= total_) return false;
      if (max_ >= planes_) {
        const int64_t per = max_ / planes_;
        const int64_t n = total_ - p_ < per ? total_ - p_ : per;
        *out = Chunk{p_, n, 0, planes_, p_ * planes_, n * planes_};
        p_ += n;
      } else {
        // a piece is smaller than one page: cut every page into runs of consecutive planes
        const int c = planes_ - q_ < (int)max_ ? planes_ - q_ : (int)max_;
        *out = Chunk{p_, 1, q_, c, p_ * planes_ + q_, c};
        q_ += c;
        if (q_ >= planes_) { q_ = 0; ++p_; }
      }
      return true;
    }
    while (r_ < n_req_ && req_[r_] == 0) ++r_;
    if (r_ >= n_req_) return false;
    const int64_t m = req_[r_];
    if (m <= max_) {
      int64_t k = max_ / m;  // whole plane rows per piece
      if (k > planes_) k = planes_;
      const int c = planes_ - q_ < (int)k ? planes_ - q_ : (int)k;
      *out = Chunk{first_page_, m, q_, c, base_slot_ + (int64_t)q_ * m, (int64_t)c * m};
      q_ += c;
    } else {
      const int64_t n = m - j_ < max_ ? m - j_ : max_;
      *out = Chunk{first_page_ + j_, n, q_, 1, base_slot_ + (int64_t)q_ * m + j_, n};
      j_ += n;
      if (j_ >= m) { j_ = 0; ++q_; }
    }
    if (q_ >= planes_) {
      q_ = 0;
      first_page_ += m;
      base_slot_ += m * planes_;
      ++r_;
    }
    return true;
  }

 private:
  const int64_t* req_;
  int64_t n_req_;
  int planes_, layout_;
  int64_t max_;
  int64_t total_ = 0, p_ = 0;                       // page-major walk
  int64_t r_ = 0, j_ = 0, first_page_ = 0, base_slot_ = 0;
  int q_ = 0;
};

}  // namespace bikv
