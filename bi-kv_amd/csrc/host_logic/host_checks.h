// Host-side checks and orderings that need no GPU. Pure host logic (no HIP).
#pragma once
#include <stdint.h>

#include <algorithm>
#include <utility>
#include <vector>

namespace bikv {

// Looks for an id that occurs more than once in ids[0..n). Of all repeated ids it reports the one whose
// SECOND occurrence comes first in the caller's order: *id, and the two entries *first < *second that hold
// it. Returns false when all ids differ.
inline bool find_first_duplicate(const int64_t* ids, int64_t n, int64_t* id, int64_t* first, int64_t* second) {
  std::vector<std::pair<int64_t, int64_t>> v((size_t)(n > 0 ? n : 0));
  for (int64_t i = 0; i < n; ++i) v[(size_t)i] = {ids[i], i};
  std::sort(v.begin(), v.end());
  // within a group of equal ids the positions ascend, because the pairs were sorted
  int64_t best = -1, best_first = 0, best_id = 0;
  for (size_t i = 0; i + 1 < v.size();) {
    size_t j = i + 1;
    while (j < v.size() && v[j].first == v[i].first) ++j;
    if (j - i >= 2 && (best < 0 || v[i + 1].second < best)) {
      best = v[i + 1].second;
      best_first = v[i].second;
      best_id = v[i].first;
    }
    i = j;
  }
  if (best < 0) return false;
  *id = best_id;
  *first = best_first;
  *second = best;
  return true;
}

// The order in which bikv_device_alloc maps the physical chunks of an allocation: out[k] = true when
// position k takes a chunk of the "other" kind. The n_other chunks are spread as evenly as the counts
// allow over the n_same + n_other positions, so that every window of the allocation holds both kinds in
// (nearly) the proportion of the whole.
inline std::vector<bool> interleave_order(size_t n_same, size_t n_other) {
  const size_t n = n_same + n_other;
  std::vector<bool> out(n, false);
  size_t is = 0, io = 0;
  for (size_t k = 0; k < n; ++k) {
    const bool take_other = io < n_other && (is >= n_same || (io + 1) * n <= (k + 1) * n_other + n / 2);
    out[k] = take_other;
    if (take_other) ++io; else ++is;
  }
  return out;
}

}  // namespace bikv
