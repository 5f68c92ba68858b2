// Drives the library's pure host logic under the address and undefined-behaviour sanitizers.
// Every check aborts with a message on failure; "host_logic ok" on stdout means all passed.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <map>
#include <random>
#include <vector>
#include <sys/mman.h>

#include "arena_logic.h"
#include "chunk_planner.h"
#include "host_checks.h"
#include "ring_logic.h"

using namespace bikv;

#define REQUIRE(cond, ...)                                                   \
  do {                                                                       \
    if (!(cond)) {                                                           \
      fprintf(stderr, "%s:%d: %s failed: ", __FILE__, __LINE__, #cond);      \
      fprintf(stderr, __VA_ARGS__);                                          \
      fprintf(stderr, "\n");                                                 \
      abort();                                                               \
    }                                                                        \
  } while (0)

// Every slot of the staging image is covered exactly once, in ascending order, by pieces of at most
// max_slots slots whose (pages x planes) rectangle maps onto exactly the slots they claim.
static void check_plan(const std::vector<int64_t>& req, int planes, int layout, int64_t max_slots) {
  int64_t total_pages = 0;
  for (int64_t m : req) total_pages += m;
  std::vector<int64_t> req_first(req.size() + 1, 0);
  for (size_t r = 0; r < req.size(); ++r) req_first[r + 1] = req_first[r] + req[r];
  ChunkPlanner plan(req.data(), (int64_t)req.size(), planes, layout, max_slots);
  Chunk c;
  int64_t next_slot = 0, steps = 0;
  std::vector<unsigned char> seen((size_t)(total_pages * planes), 0);
  while (plan.next(&c)) {
    ++steps;
    REQUIRE(steps <= total_pages * planes + 1, "planner does not terminate");
    REQUIRE(c.n_slots >= 1 && c.n_slots <= max_slots, "n_slots %lld max %lld", (long long)c.n_slots, (long long)max_slots);
    REQUIRE(c.first_slot == next_slot, "pieces not back to back: %lld vs %lld", (long long)c.first_slot, (long long)next_slot);
    REQUIRE(c.n_slots == c.n_pages * c.plane_count, "rectangle %lld x %d != %lld slots", (long long)c.n_pages, c.plane_count, (long long)c.n_slots);
    REQUIRE(c.plane_begin >= 0 && c.plane_begin + c.plane_count <= planes && c.plane_count >= 1, "planes");
    REQUIRE(c.first_page >= 0 && c.first_page + c.n_pages <= total_pages, "pages");
    // the slots the kernel will compute for this rectangle (slot = base + j + q*m, or page*planes + q)
    size_t r = 0;
    while (req_first[r + 1] <= c.first_page) ++r;
    for (int64_t i = c.first_page; i < c.first_page + c.n_pages; ++i) {
      if (layout == BIKV_LAYOUT_LAYER_MAJOR) REQUIRE(i < req_first[r + 1], "a piece spans two requests");
      for (int q = c.plane_begin; q < c.plane_begin + c.plane_count; ++q) {
        const int64_t slot = layout == BIKV_LAYOUT_PAGE_MAJOR
                                 ? i * planes + q
                                 : req_first[r] * planes + (i - req_first[r]) + (int64_t)q * req[r];
        REQUIRE(slot >= c.first_slot && slot < c.first_slot + c.n_slots, "slot %lld outside its piece", (long long)slot);
        REQUIRE(!seen[(size_t)slot], "slot %lld covered twice", (long long)slot);
        seen[(size_t)slot] = 1;
      }
    }
    next_slot += c.n_slots;
  }
  REQUIRE(next_slot == total_pages * planes, "image not covered: %lld of %lld", (long long)next_slot, (long long)(total_pages * planes));
}

static void test_planner() {
  std::mt19937_64 rng(7);
  for (int it = 0; it < 3000; ++it) {
    const int n_req = (int)(rng() % 6);
    std::vector<int64_t> req((size_t)n_req);
    for (auto& m : req) m = (int64_t)(rng() % 4 == 0 ? 0 : rng() % 40);
    const int planes = 1 + (int)(rng() % 9);
    const int layout = (int)(rng() % 2);
    const int64_t max_slots = 1 + (int64_t)(rng() % 70);
    check_plan(req, planes, layout, max_slots);
  }
  // extremes: one-slot pieces, a lane buffer far larger than anything, single-page requests with a huge
  // budget (the rows-per-piece quotient is then enormous)
  check_plan({5, 1, 3}, 4, BIKV_LAYOUT_LAYER_MAJOR, 1);
  check_plan({5, 1, 3}, 4, BIKV_LAYOUT_PAGE_MAJOR, 1);
  check_plan({1, 1, 1}, 3, BIKV_LAYOUT_LAYER_MAJOR, std::numeric_limits<int64_t>::max() / 2);
  check_plan({7, 2}, 160, BIKV_LAYOUT_PAGE_MAJOR, std::numeric_limits<int64_t>::max() / 2);
  check_plan({}, 3, BIKV_LAYOUT_LAYER_MAJOR, 8);
  check_plan({0, 0}, 3, BIKV_LAYOUT_PAGE_MAJOR, 8);
}

static void test_duplicates() {
  std::mt19937_64 rng(11);
  const int64_t lo = std::numeric_limits<int64_t>::min(), hi = std::numeric_limits<int64_t>::max();
  for (int it = 0; it < 4000; ++it) {
    const int n = (int)(rng() % 12);
    std::vector<int64_t> ids((size_t)n);
    for (auto& x : ids) {
      const unsigned k = (unsigned)(rng() % 10);
      x = k == 0 ? lo : k == 1 ? hi : (int64_t)(rng() % 9) - 4;
    }
    // brute force: the smallest position that repeats an earlier one
    int64_t want_second = -1, want_first = -1;
    for (int j = 1; j < n && want_second < 0; ++j)
      for (int i = 0; i < j; ++i)
        if (ids[(size_t)i] == ids[(size_t)j]) { want_second = j; want_first = i; break; }
    int64_t id = 0, first = 0, second = 0;
    const bool got = find_first_duplicate(ids.data(), n, &id, &first, &second);
    REQUIRE(got == (want_second >= 0), "presence");
    if (got) {
      REQUIRE(second == want_second, "second occurrence %lld want %lld", (long long)second, (long long)want_second);
      REQUIRE(ids[(size_t)first] == id && ids[(size_t)second] == id && first < second, "entries");
      // `first` is the FIRST entry holding that id
      for (int i = 0; i < first; ++i) REQUIRE(ids[(size_t)i] != id, "first is not the first");
      (void)want_first;
    }
  }
  int64_t a = 0, b = 0, c = 0;
  REQUIRE(!find_first_duplicate(nullptr, 0, &a, &b, &c), "empty");
}

static void test_interleave() {
  for (size_t n_same = 0; n_same <= 40; ++n_same)
    for (size_t n_other = 0; n_other <= 40; ++n_other) {
      const std::vector<bool> o = interleave_order(n_same, n_other);
      const size_t n = n_same + n_other;
      REQUIRE(o.size() == n, "size");
      size_t others = 0;
      for (size_t k = 0; k < n; ++k) {
        others += o[k] ? 1 : 0;
        // every prefix holds the "other" kind in the proportion of the whole, to within one chunk
        const double ideal = n ? (double)(k + 1) * (double)n_other / (double)n : 0.0;
        REQUIRE((double)others >= ideal - 1.0 && (double)others <= ideal + 1.0, "prefix %zu of (%zu, %zu): %zu others, ideal %.2f",
                k, n_same, n_other, others, ideal);
      }
      REQUIRE(others == n_other, "count");
    }
}

static void test_ring() {
  bikv_shared_control* c = static_cast<bikv_shared_control*>(malloc(sizeof(bikv_shared_control)));
  memset(c, 0xEE, sizeof(*c));
  bikv_shared_control image;
  memset(&image, 0, sizeof(image));
  image.buffer_size = 1000;
  image.device_id = 3;
  strcpy(image.hostname, "host-a");
  ring::describe_ring(c, image);
  REQUIRE(ring::describes_ring(c) == 1000 && c->device_id == 3 && c->current_offset == 0, "describe_ring");
  ring::Producer p;
  p.ctrl = c;
  // the reference's wrap sequence for transfers of 400 bytes in a ring of 1000: 0, 400, 0, 400, 0
  const int64_t shape[5] = {4, 5, 2, 10, 1};
  const size_t want[5] = {0, 400, 0, 400, 0};
  for (int k = 0; k < 5; ++k) {
    size_t at = 77;
    REQUIRE(ring::reserve_window(p, 400, &at) == ring::WAIT_OK && at == want[k], "wrap step %d: %zu", k, at);
    ring::publish_transfer(p, at, 400, shape, 5, 0);
    REQUIRE(c->last_valid_offset == want[k] && c->current_offset == want[k] + 400 && c->data_size == 400 && c->tensor_dim == 5 &&
                c->tensor_shape[3] == 10, "publish step %d", k);
    REQUIRE(ring::wait_ms(ring::sem_of(c->sem_start), 0) == ring::WAIT_OK, "one post per transfer");
  }
  REQUIRE(ring::wait_ms(ring::sem_of(c->sem_start), 1) == ring::WAIT_TIMEOUT, "no extra post");
  // a transfer that exactly fills the rest does not wrap; one byte more does
  c->current_offset = 600;
  size_t at = 0;
  ring::reserve_window(p, 400, &at);
  REQUIRE(at == 600, "exact fit");
  c->current_offset = 601;
  ring::reserve_window(p, 400, &at);
  REQUIRE(at == 0, "wrap");
  // back-pressure: a published transfer blocks the publication of the next until it is released, and
  // a window that overlaps it until then; with a timeout both report WAIT_TIMEOUT and change nothing
  p.backpressure = true;
  p.bp_timeout_ms = 20;
  c->current_offset = 0;
  ring::reserve_window(p, 600, &at);
  REQUIRE(at == 0 && ring::wait_slot(p) == ring::WAIT_OK, "first transfer");
  ring::publish_transfer(p, at, 600, shape, 5, 0);
  REQUIRE(p.in_flight.size() == 1, "in flight");
  REQUIRE(ring::reserve_window(p, 300, &at) == ring::WAIT_OK && at == 600, "disjoint window needs no wait");
  REQUIRE(ring::wait_slot(p) == ring::WAIT_TIMEOUT && p.in_flight.size() == 1, "the slot is taken");
  REQUIRE(ring::reserve_window(p, 600, &at) == ring::WAIT_TIMEOUT, "overlapping window waits");   // wraps to 0
  sem_post(ring::sem_of(c->sem_complete));      // the consumer releases
  REQUIRE(ring::reserve_window(p, 600, &at) == ring::WAIT_OK && at == 0 && p.in_flight.empty(), "released");
  REQUIRE(ring::wait_slot(p) == ring::WAIT_OK, "slot free");
  sem_destroy(ring::sem_of(c->sem_start));
  sem_destroy(ring::sem_of(c->sem_complete));
  free(c);
}

// The arena bookkeeping behind the torch allocator hooks, over a malloc backend: blocks never overlap, stay
// inside what the backend handed out, follow each other in memory in allocation order, big requests get
// allocations of their own, and everything the backend gave is returned once the last block is gone.
static std::map<void*, int64_t> g_backend;      // base -> bytes, what the backend currently has out
static int g_backend_fail_after = -1;
static void* backend_alloc(int /*device*/, int64_t bytes) {
  if (g_backend_fail_after == 0) return nullptr;
  if (g_backend_fail_after > 0) --g_backend_fail_after;
  // address space only: the bookkeeping compares addresses and never touches the memory
  void* p = mmap(nullptr, (size_t)bytes, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
  REQUIRE(p != MAP_FAILED, "mmap of %lld bytes of address space", (long long)bytes);
  g_backend[p] = bytes;
  return p;
}
static void backend_drop(void* base) {
  munmap(base, (size_t)g_backend[base]);
  g_backend.erase(base);
}
static void backend_free(void* base) {
  REQUIRE(g_backend.count(base) == 1, "release of %p, which the backend did not hand out", base);
  backend_drop(base);
}
static void backend_drop_all() {
  while (!g_backend.empty()) backend_drop(g_backend.begin()->first);
}
static void test_arena() {
  const int64_t A = int64_t(2) << 30;
  {
    arena::Book book(A, backend_alloc, backend_free);
    std::vector<void*> p;
    for (int i = 0; i < 28; ++i) p.push_back(book.take(0, int64_t(160) << 20));       // the Worker's 28 layer tensors
    for (void* q : p) REQUIRE(q != nullptr, "take failed");
    REQUIRE(book.live_arenas() == 3 && g_backend.size() == 3, "28 x 160 MiB fill three arenas of 2 GiB, got %zu", book.live_arenas());
    for (int i = 1; i < 12; ++i)
      REQUIRE((char*)p[(size_t)i] - (char*)p[(size_t)i - 1] == (int64_t(160) << 20), "blocks of one arena are neighbours");
    void* big = book.take(0, (int64_t(1) << 30) + 1);
    REQUIRE(big && g_backend.size() == 4, "a request above half an arena is an allocation of its own");
    void* other_dev = book.take(1, int64_t(2) << 20);
    REQUIRE(other_dev && g_backend.size() == 5, "another device gets its own arena");
    REQUIRE(!book.give((char*)p[0] + 4096), "an address inside a block is not a block");
    for (int i = 0; i < 12; ++i) REQUIRE(book.give(p[(size_t)i]), "give");
    REQUIRE(g_backend.size() == 4, "an older arena is released with its last block");
    REQUIRE(!book.give(p[0]), "a block is given back once");
    for (int i = 12; i < 28; ++i) REQUIRE(book.give(p[(size_t)i]), "give");
    REQUIRE(book.give(big) && book.give(other_dev), "give");
    REQUIRE(book.live_blocks() == 0, "no block left");
    // the newest arena of each device is rewound and kept
    REQUIRE(g_backend.size() == 2 && book.live_arenas() == 2, "kept arenas: %zu", g_backend.size());
    void* again = book.take(0, int64_t(4) << 20);
    REQUIRE(again && g_backend.size() == 2, "a kept arena serves the next request");
    REQUIRE(book.give(again), "give");
    backend_drop_all();
  }
  {
    // random traffic: blocks are disjoint and inside a backend allocation
    arena::Book book(A, backend_alloc, backend_free);
    std::mt19937_64 rng(7);
    std::map<char*, int64_t> live;
    for (int step = 0; step < 4000; ++step) {
      if (live.empty() || rng() % 3) {
        const int64_t sz = (int64_t)(rng() % 700 + 1) << 20;
        char* q = (char*)book.take(0, sz);
        REQUIRE(q != nullptr, "take");
        const int64_t r = arena::round_up(sz, arena::kAlign);
        bool inside = false;
        for (auto& b : g_backend) inside |= q >= (char*)b.first && q + r <= (char*)b.first + b.second;
        REQUIRE(inside, "block outside every backend allocation");
        auto nx = live.lower_bound(q);
        REQUIRE(nx == live.end() || q + r <= nx->first, "block overlaps its successor");
        if (nx != live.begin()) { --nx; REQUIRE(nx->first + nx->second <= q, "block overlaps its predecessor"); }
        live[q] = r;
      } else {
        auto it = live.begin();
        std::advance(it, (long)(rng() % live.size()));
        REQUIRE(book.give(it->first), "give");
        live.erase(it);
      }
    }
    for (auto& b : live) REQUIRE(book.give(b.first), "give");
    REQUIRE(book.live_blocks() == 0 && g_backend.size() <= 1, "all but the kept arena returned");
    backend_drop_all();
  }
  {
    // the backend running dry: take reports it and leaves nothing behind
    arena::Book book(A, backend_alloc, backend_free);
    g_backend_fail_after = 1;
    void* a = book.take(0, int64_t(900) << 20);
    void* b = book.take(0, int64_t(900) << 20);
    void* c = book.take(0, int64_t(900) << 20);     // needs a second arena: refused
    REQUIRE(a && b && !c && book.live_blocks() == 2, "out of memory is reported");
    g_backend_fail_after = -1;
    REQUIRE(book.give(a) && book.give(b), "give");
    backend_drop_all();
  }
}

// The allocator's search for chunks of both kinds, replayed on the CPU with scripted halves: chunk k lies in
// half halves[k] (the first chunk is the reference), a pair inside one half probes slow, a straddling pair
// fast. The search creates chunks until it has want_same + want_other of the right kinds (or the script / the
// filler budget ends) and deals them out. Whatever order the driver hands the halves out in, the result must
// hold the wanted number of each kind whenever the script contains them.
struct Dealt { size_t same_in_ref_half, same_in_other_half, other_in_ref_half, other_in_other_half, fillers, created; };
static Dealt search_and_deal(const std::vector<int>& halves, size_t n, size_t max_fillers, std::mt19937_64& rng) {
  const size_t want_other = n / 2, want_same = n - want_other;
  std::vector<float> pair_ms;
  float ref_ms = 0;
  size_t k = 0;
  for (;;) {
    const size_t n_other = count_other_chunks(pair_ms, ref_ms), n_same = pair_ms.size() - n_other;
    if (n_same >= want_same && n_other >= want_other) break;
    if (pair_ms.size() >= n && pair_ms.size() - n >= max_fillers) break;
    if (k >= halves.size()) break;                                   // "out of memory"
    float t = 0;
    if (k > 0) t = (halves[k] == halves[0] ? 0.382f : 0.319f) * (1.0f + 0.01f * (float)((int)(rng() % 5) - 2));
    if (t > ref_ms) ref_ms = t;
    pair_ms.push_back(t);
    ++k;
  }
  const std::vector<int> use = deal_chunks(pair_ms, ref_ms, want_same, want_other);
  Dealt d = {0, 0, 0, 0, 0, pair_ms.size()};
  for (size_t i = 0; i < use.size(); ++i) {
    const bool in_ref_half = halves[i] == halves[0];
    if (use[i] == CHUNK_SAME) (in_ref_half ? d.same_in_ref_half : d.same_in_other_half)++;
    else if (use[i] == CHUNK_OTHER) (in_ref_half ? d.other_in_ref_half : d.other_in_other_half)++;
    else d.fillers++;
  }
  return d;
}
static void test_deal() {
  std::mt19937_64 rng(11);
  auto script = [](std::initializer_list<std::pair<int, int>> runs) {
    std::vector<int> h;
    for (auto& r : runs) h.insert(h.end(), (size_t)r.second, r.first);
    return h;
  };
  // the usual order: the reference's half first, then the other
  Dealt d = search_and_deal(script({{0, 40}, {1, 40}}), 18, 384, rng);
  REQUIRE(d.same_in_ref_half == 9 && d.other_in_other_half == 9 && d.same_in_other_half == 0 && d.other_in_ref_half == 0,
          "usual order: %zu/%zu", d.same_in_ref_half, d.other_in_other_half);
  REQUIRE(d.fillers == 31 && d.created == 49, "fillers %zu created %zu", d.fillers, d.created);
  // the reference is the last free chunk of its half: sixty chunks of the other half come first (all fast pairs,
  // nothing to compare them with yet), then the reference's half again
  d = search_and_deal(script({{0, 1}, {1, 60}, {0, 30}}), 18, 384, rng);
  REQUIRE(d.same_in_ref_half == 9 && d.other_in_other_half == 9 && d.same_in_other_half == 0 && d.other_in_ref_half == 0,
          "other half first: same %zu (+%zu misplaced), other %zu (+%zu misplaced)", d.same_in_ref_half, d.same_in_other_half,
          d.other_in_other_half, d.other_in_ref_half);
  // alternating halves: no fillers at all
  {
    std::vector<int> h;
    for (int i = 0; i < 40; ++i) h.push_back(i & 1);
    d = search_and_deal(h, 18, 384, rng);
    REQUIRE(d.same_in_ref_half == 9 && d.other_in_other_half == 9 && d.fillers == 0, "alternating: fillers %zu", d.fillers);
  }
  // a filler budget that does not reach the other half: complete, all of one kind, nothing labelled "other"
  d = search_and_deal(script({{0, 100}, {1, 40}}), 18, 10, rng);
  REQUIRE(d.created == 28 && d.same_in_ref_half == 18 && d.other_in_other_half + d.other_in_ref_half == 0 && d.fillers == 10,
          "budget: created %zu same %zu fillers %zu", d.created, d.same_in_ref_half, d.fillers);
  // memory runs out with too few chunks of the reference's half: the other kind makes up the difference
  d = search_and_deal(script({{0, 3}, {1, 40}}), 18, 384, rng);
  REQUIRE(d.same_in_ref_half == 3 && d.other_in_other_half + d.same_in_other_half == 15 && d.fillers == 25,
          "short half: same %zu other %zu fillers %zu", d.same_in_ref_half, d.other_in_other_half, d.fillers);
  // an odd count and a single chunk
  d = search_and_deal(script({{0, 10}, {1, 10}}), 7, 384, rng);
  REQUIRE(d.same_in_ref_half == 4 && d.other_in_other_half == 3, "odd count");
  d = search_and_deal(script({{0, 10}}), 1, 384, rng);
  REQUIRE(d.same_in_ref_half == 1 && d.created == 1 && d.fillers == 0, "single chunk");
  // random scripts: never more than wanted of a kind, every wanted chunk present when the script has it
  for (int trial = 0; trial < 300; ++trial) {
    std::vector<int> h;
    const size_t len = 20 + rng() % 200;
    int cur = 0;
    while (h.size() < len) {
      const size_t run = 1 + rng() % 40;
      h.insert(h.end(), run, cur);
      cur ^= 1;
    }
    const size_t n = 2 + rng() % 18;
    size_t have_ref = 0, have_other = 0;
    for (int x : h) (x == h[0] ? have_ref : have_other)++;
    d = search_and_deal(h, n, ~size_t(0), rng);
    const size_t want_other = n / 2, want_same = n - want_other;
    REQUIRE(d.same_in_ref_half + d.same_in_other_half + d.other_in_ref_half + d.other_in_other_half == std::min(n, h.size()), "complete");
    REQUIRE(d.other_in_ref_half == 0, "a chunk of the reference's half is never labelled other");
    if (have_ref >= want_same && have_other >= want_other)
      REQUIRE(d.same_in_ref_half == want_same && d.other_in_other_half == want_other,
              "trial %d: same %zu of %zu, other %zu of %zu", trial, d.same_in_ref_half, want_same, d.other_in_other_half, want_other);
  }
}

int main() {
  test_arena();
  test_deal();
  test_planner();
  test_duplicates();
  test_interleave();
  test_ring();
  printf("host_logic ok\n");
  return 0;
}
