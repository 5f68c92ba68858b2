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

// How bikv_device_alloc tells the two kinds of physical chunks apart and deals them out. Every chunk but the
// first is probed as a pair with the first; a pair that straddles the two halves of HBM is faster than a pair
// inside one half. The yardstick is the SLOWEST pair seen (`ref_ms`), which only grows while chunks are being
// created: kinds are therefore derived from the times whenever they are needed and never stored, so that
// chunks met before the first slow pair — the driver handing out the OTHER half first — are not stuck with the
// kind they seemed to have then.
constexpr float kOtherBelow = 0.92f;     // other half: pair time below 0.92 x the slowest pair time

inline bool chunk_is_other(float pair_ms, float ref_ms) { return pair_ms > 0 && pair_ms < kOtherBelow * ref_ms; }

inline size_t count_other_chunks(const std::vector<float>& pair_ms, float ref_ms) {
  size_t k = 0;
  for (float t : pair_ms) k += chunk_is_other(t, ref_ms) ? 1 : 0;
  return k;
}

enum ChunkUse : int { CHUNK_SAME = 0, CHUNK_OTHER = 1, CHUNK_FILLER = 2 };

// Deals the created chunks out for an allocation of n = want_same + want_other chunks: the wanted number of
// each kind; what one kind lacks is made up from the other's surplus; the rest are fillers (released by the
// caller). Fewer than n chunks in all: every chunk is used.
inline std::vector<int> deal_chunks(const std::vector<float>& pair_ms, float ref_ms, size_t want_same, size_t want_other) {
  std::vector<int> use(pair_ms.size(), CHUNK_FILLER);
  size_t n_same = 0, n_other = 0;
  for (size_t i = 0; i < pair_ms.size(); ++i) {
    if (chunk_is_other(pair_ms[i], ref_ms)) {
      if (n_other < want_other) { use[i] = CHUNK_OTHER; ++n_other; }
    } else if (n_same < want_same) {
      use[i] = CHUNK_SAME;
      ++n_same;
    }
  }
  const size_t n = want_same + want_other;
  for (size_t i = 0; i < pair_ms.size() && n_same + n_other < n; ++i) {
    if (use[i] != CHUNK_FILLER) continue;
    if (chunk_is_other(pair_ms[i], ref_ms)) { use[i] = CHUNK_OTHER; ++n_other; }
    else { use[i] = CHUNK_SAME; ++n_same; }
  }
  return use;
}

}  // namespace bikv
