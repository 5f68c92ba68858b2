// Pool memory placed for the MI355X memory system.
//
// Measured on MI355X (random 16 KiB tiles, one 64-lane workgroup per KiB, 4 GiB moved per launch): the
// physical address space behaves as two halves. A copy whose RANDOM WRITES all land in one half runs at
// 5.6-5.7 TB/s wherever its reads come from; the same writes spread over both halves run at 6.6-6.7 TB/s
// (+18 %). Reads do not care (6.25-6.45 TB/s either way), sequential writes hardly do. Which half a piece
// of memory lies in is a property of its PHYSICAL address: inside one hipMalloc of 112 GiB the boundary
// sat at an offset of 64 GiB; 1 GiB physical chunks created one after the other were 95 in one half, then
// 17 in the other. A KV pool that fits one half (every pool below ~100 GB on an otherwise empty GPU, and a
// big pool whenever the driver happens to place it so) therefore scatters 15-18 % slower than it could,
// and how a big pool straddles the boundary is what moved whole-process results by several percent from
// one allocation to the next.
//
// Nothing in HIP names the half, but it is easy to observe: a short scatter into two chunks is ~19 %
// faster when they lie in different halves. bikv_device_alloc builds an allocation out of physical chunks
// (hipMemCreate), classifies every chunk against the first one with that probe, keeps equal numbers of
// both kinds (creating — and afterwards releasing — as many filler chunks as it takes to reach the other
// half) and maps them alternately into one virtual range (hipMemAddressReserve / hipMemMap). Every
// window of such a pool, however small, then spreads its writes over both halves.
#include "../../include/bikv_pagecopy.h"
#include "host_logic/arena_logic.h"
#include "host_logic/host_checks.h"
#include "pagecopy_internal.h"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cerrno>
#include <chrono>
#include <cstdio>
#include <map>
#include <mutex>
#include <vector>
#include <fcntl.h>
#include <sys/file.h>
#include <sys/stat.h>
#include <unistd.h>

using namespace bikv;

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// The probe: every workgroup copies one KiB from a small source window into a pseudo-random 16 KiB tile of
// target a or target b (the same shape of traffic as a page scatter). Contents are garbage: the targets are
// fresh chunks that hold no data yet.
__global__ __launch_bounds__(64) void probe_kernel(const char* src, uint64_t src_mask, char* a, char* b,
                                                   uint32_t tiles_each) {
  const uint32_t w = blockIdx.x;
  uint32_t x = (w >> 4) * 2654435761u;          // one hash per 16 KiB tile; its 16 pieces are neighbours
  x ^= x >> 15;
  x *= 2246822519u;
  x ^= x >> 13;
  const uint32_t t = x % (2 * tiles_each);
  char* base = t < tiles_each ? a : b;
  const uint64_t off = (uint64_t)(t < tiles_each ? t : t - tiles_each) * 16384u + (w & 15u) * 1024u + threadIdx.x * 16u;
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + (((uint64_t)w * 1024u + threadIdx.x * 16u) & src_mask)));
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(base + off));
}

struct Allocation {
  int device = 0;
  void* va = nullptr;
  size_t bytes = 0, chunk = 0;
  std::vector<hipMemGenericAllocationHandle_t> handles;   // in mapping order
  int n_other = 0;                                         // chunks classified "other half"
  int n_fillers = 0;                                       // chunks created and released again
  int n_reprobed = 0;                                      // chunks whose first probe was too close to call
  double seconds = 0;                                      // wall time of the allocation
  float pair_ms_same = 0, pair_ms_other = 0;               // slowest / fastest pair probe seen
};

std::mutex g_mu;                 // guards g_allocs
std::mutex g_alloc_mu;           // one placement at a time per process
std::map<void*, Allocation> g_allocs;

size_t pow2_floor(size_t x) {
  size_t p = 1;
  while (p * 2 <= x) p *= 2;
  return p;
}

// One placement at a time per GPU across PROCESSES too: Bi-KV runs a cache process and a worker process
// on each GPU, and two placements at once would disturb each other's probe timings and compete for the
// filler chunks. An advisory lock on a file named after the GPU's PCI address; the kernel drops it when
// the process ends, whatever way it ends. Best effort: if the file cannot be opened the placement runs
// unlocked.
class DeviceFileLock {
 public:
  explicit DeviceFileLock(int device) {
    char bus[64] = "";
    if (hipDeviceGetPCIBusId(bus, sizeof(bus), device) != hipSuccess) {
      (void)hipGetLastError();
      snprintf(bus, sizeof(bus), "index%d", device);
    }
    for (char* c = bus; *c; ++c)
      if (*c == ':' || *c == '.' || *c == '/') *c = '_';
    char path[128];
    snprintf(path, sizeof(path), "/dev/shm/bikv_device_alloc_%s.lock", bus);
    fd_ = open(path, O_CREAT | O_RDWR, 0666);
    if (fd_ >= 0) {
      (void)fchmod(fd_, 0666);
      int rc;
      do { rc = flock(fd_, LOCK_EX); } while (rc == -1 && errno == EINTR);
    }
  }
  ~DeviceFileLock() {
    if (fd_ >= 0) {
      (void)flock(fd_, LOCK_UN);
      close(fd_);
    }
  }
  DeviceFileLock(const DeviceFileLock&) = delete;
  DeviceFileLock& operator=(const DeviceFileLock&) = delete;

 private:
  int fd_ = -1;
};

struct Prober {
  hipStream_t stream = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  char* src = nullptr;
  size_t src_bytes = size_t(1) << 30;   // far beyond the caches: the probe's reads come from HBM like a scatter's
  void* window = nullptr;      // two chunks of virtual space: [0] the reference chunk, [1] the candidate
  bool mapped[2] = {false, false};
  size_t chunk = 0;
  hipMemAccessDesc acc;

  int init(int device, size_t chunk_bytes) {
    chunk = chunk_bytes;
    acc = hipMemAccessDesc();
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = device;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    BIKV_HIP(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    BIKV_HIP(hipEventCreate(&e0));
    BIKV_HIP(hipEventCreate(&e1));
    BIKV_HIP(hipMalloc((void**)&src, src_bytes));
    BIKV_HIP(hipMemAddressReserve(&window, 2 * chunk, 0, nullptr, 0));
    return BIKV_OK;
  }
  // Whatever is still mapped in the window is unmapped first: releasing the address range, or a handle,
  // with a live mapping leaks it.
  void destroy() {
    if (stream) (void)hipStreamSynchronize(stream);
    for (int slot = 0; slot < 2; ++slot)
      if (window && mapped[slot]) {
        (void)hipMemUnmap(static_cast<char*>(window) + (size_t)slot * chunk, chunk);
        mapped[slot] = false;
      }
    if (window) (void)hipMemAddressFree(window, 2 * chunk);
    if (src) (void)hipFree(src);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (stream) (void)hipStreamDestroy(stream);
    window = nullptr;
    src = nullptr;
    e0 = e1 = nullptr;
    stream = nullptr;
  }
  int map(int slot, hipMemGenericAllocationHandle_t h) {
    char* at = static_cast<char*>(window) + (size_t)slot * chunk;
    BIKV_HIP(hipMemMap(at, chunk, 0, h, 0));
    mapped[slot] = true;
    BIKV_HIP(hipMemSetAccess(at, chunk, &acc, 1));
    return BIKV_OK;
  }
  int unmap(int slot) {
    if (!mapped[slot]) return BIKV_OK;
    BIKV_HIP(hipStreamSynchronize(stream));
    BIKV_HIP(hipMemUnmap(static_cast<char*>(window) + (size_t)slot * chunk, chunk));
    mapped[slot] = false;
    return BIKV_OK;
  }
  // milliseconds of one probe launch scattering ~1 GiB into the pair (slot 0, slot 1)
  int time_pair(float* ms) {
    char* a = static_cast<char*>(window);
    char* b = a + chunk;
    const uint32_t tiles = (uint32_t)(chunk / 16384);
    const uint32_t grid = 1u << 20;                       // 1 Mi workgroups x 1 KiB
    for (int i = 0; i < 2; ++i)
      hipLaunchKernelGGL(probe_kernel, dim3(grid), dim3(64), 0, stream, src, (uint64_t)src_bytes - 1, a, b, tiles);
    BIKV_HIP(hipEventRecord(e0, stream));
    for (int i = 0; i < 3; ++i)
      hipLaunchKernelGGL(probe_kernel, dim3(grid), dim3(64), 0, stream, src, (uint64_t)src_bytes - 1, a, b, tiles);
    BIKV_HIP(hipEventRecord(e1, stream));
    BIKV_HIP(hipEventSynchronize(e1));
    BIKV_HIP(hipGetLastError());
    BIKV_HIP(hipEventElapsedTime(ms, e0, e1));
    *ms /= 3;
    return BIKV_OK;
  }
};

void release_all(std::vector<hipMemGenericAllocationHandle_t>& v) {
  for (auto h : v) (void)hipMemRelease(h);
  v.clear();
}

// A pair that straddles the halves scatters ~19 % faster than a pair inside one half. Every candidate is
// probed as a PAIR with the first chunk (equal footprint for every probe), and judged against the slowest
// pair seen so far — pairs inside the first chunk's half. A time inside the band between the two groups is
// not trusted: the chunk is probed again (twice more at most) and the median decides.
constexpr float kBandLo = 0.88f, kBandHi = 0.96f;

}  // namespace

extern "C" int bikv_device_alloc_bounded(int device, int64_t bytes, int32_t placement, int64_t max_filler_bytes,
                                         void** out) {
  if (!out) return fail(BIKV_EINVAL, "null out");
  *out = nullptr;
  if (bytes <= 0) return fail(BIKV_EINVAL, "bytes must be positive");
  if (placement != BIKV_PLACE_SPREAD && placement != BIKV_PLACE_SEQUENTIAL)
    return fail(BIKV_EINVAL, "unknown placement %d", placement);
  BIKV_DEVICE(device);
  const auto t_begin = std::chrono::steady_clock::now();
  std::lock_guard<std::mutex> process_lock(g_alloc_mu);
  DeviceFileLock gpu_lock(device);
  hipMemAllocationProp prop = hipMemAllocationProp();
  prop.type = hipMemAllocationTypePinned;
  prop.location.type = hipMemLocationTypeDevice;
  prop.location.id = device;
  size_t gran = 0;
  BIKV_HIP(hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityRecommended));
  // chunks of 256 MiB .. 1 GiB, about 32 per allocation: small enough to interleave a 5 GB pool 20 ways,
  // large enough that the probe's footprint is far beyond any cache
  size_t chunk = std::min<size_t>(size_t(1) << 30, std::max<size_t>(size_t(256) << 20, pow2_floor((size_t)bytes / 32)));
  if (gran > 0 && chunk % gran) chunk = (chunk + gran - 1) / gran * gran;
  const size_t n = ((size_t)bytes + chunk - 1) / chunk;
  const size_t want_other = placement == BIKV_PLACE_SPREAD ? n / 2 : 0;
  const size_t want_same = n - want_other;
  const size_t max_fillers = max_filler_bytes < 0 ? ~size_t(0) : (size_t)max_filler_bytes / chunk;

  const size_t reserve = size_t(2) << 30;     // never take the last 2 GiB of the device
  {
    size_t free_now = 0, total_now = 0;
    BIKV_HIP(hipMemGetInfo(&free_now, &total_now));
    if (n * chunk + reserve > free_now)
      return fail(BIKV_EHIP, "out of device memory: %zu bytes asked for (%zu chunks of %zu), %zu free, 2 GiB kept back",
                  (size_t)bytes, n, chunk, free_now);
  }
  // Every chunk created, with the time of its pair probe against the first one (0 for the first chunk itself,
  // and for everything when nothing is probed). A chunk's kind is judged against the SLOWEST pair seen — pairs
  // inside the first chunk's half are the slow ones — and that reference only grows during the search, so kinds
  // are always derived from the times, never stored: a chunk that looked "same" while only fast pairs had been
  // seen (the driver handing out the other half first) turns into "other" as soon as a slow pair shows up.
  std::vector<hipMemGenericAllocationHandle_t> all;     // every chunk created, in creation order
  std::vector<float> pair_ms;                           // ... and the time of its pair probe
  std::vector<hipMemGenericAllocationHandle_t> same, other, fillers;
  Prober pr;
  int rc = BIKV_OK;
  auto cleanup = [&]() {
    pr.destroy();
    release_all(all);
    release_all(same);
    release_all(other);
    release_all(fillers);
  };
  if (placement == BIKV_PLACE_SPREAD && n >= 2) {
    rc = pr.init(device, chunk);
    if (rc) { cleanup(); return rc; }
  }
  float ref_ms = 0;
  // Create chunks until both kinds are complete. Chunks beyond the wanted number of a kind are fillers:
  // they only push the driver's allocator on towards the other half and are released at the end. The
  // search ends with whatever balance was reached when a creation fails (memory exhausted) or the filler
  // budget is spent.
  int n_reprobed = 0;
  size_t free_b = 0, total_b = 0;
  for (;;) {
    const size_t n_other_now = count_other_chunks(pair_ms, ref_ms), n_same_now = all.size() - n_other_now;
    if (n_same_now >= want_same && n_other_now >= want_other) break;
    if (all.size() >= n && all.size() - n >= max_fillers) break;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess || free_b < chunk + reserve) break;
    hipMemGenericAllocationHandle_t h;
    if (hipMemCreate(&h, chunk, &prop, 0) != hipSuccess) {
      (void)hipGetLastError();
      break;
    }
    float t = 0;
    if (pr.window) {
      if (all.empty()) {
        rc = pr.map(0, h);           // the first chunk is the reference every candidate is paired with
      } else {
        rc = pr.map(1, h);
        if (!rc) rc = pr.time_pair(&t);
        if (!rc && ref_ms > 0 && t > kBandLo * ref_ms && t < kBandHi * ref_ms) {
          // too close to call: two more probes, the median of the three decides
          float t2 = 0, t3 = 0;
          rc = pr.time_pair(&t2);
          if (!rc) rc = pr.time_pair(&t3);
          if (!rc) {
            float v[3] = {t, t2, t3};
            std::sort(v, v + 3);
            t = v[1];
            ++n_reprobed;
          }
        }
        // unmapped whether or not the probes worked: the handle is about to be released or kept for the
        // final mapping, and neither may happen while the window still maps it
        const int rc_unmap = pr.unmap(1);
        if (!rc) rc = rc_unmap;
      }
      if (rc) {
        (void)pr.unmap(all.empty() ? 0 : 1);
        (void)hipMemRelease(h);
        break;
      }
      if (t > ref_ms) ref_ms = t;                // pairs inside one half are the slow ones
    }
    all.push_back(h);
    pair_ms.push_back(t);
  }
  if (pr.window) (void)pr.unmap(0);
  if (rc) { cleanup(); return rc; }
  // Hand the chunks out by their final kinds (deal_chunks): the wanted number of each, what one kind lacks made
  // up from the other's surplus (then from freshly created chunks), everything else released as fillers.
  float fastest_ms = 0;
  {
    const std::vector<int> use = deal_chunks(pair_ms, ref_ms, want_same, want_other);
    for (size_t i = 0; i < all.size(); ++i) {
      if (chunk_is_other(pair_ms[i], ref_ms) && (fastest_ms == 0 || pair_ms[i] < fastest_ms)) fastest_ms = pair_ms[i];
      (use[i] == CHUNK_OTHER ? other : use[i] == CHUNK_SAME ? same : fillers).push_back(all[i]);
    }
    all.clear();
  }
  while (same.size() + other.size() < n) {
    hipMemGenericAllocationHandle_t h;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess || free_b < chunk + reserve ||
        hipMemCreate(&h, chunk, &prop, 0) != hipSuccess) {
      (void)hipGetLastError();
      break;
    }
    same.push_back(h);
  }
  if (same.size() + other.size() < n) {
    const size_t got = same.size() + other.size();
    cleanup();
    return fail(BIKV_EHIP, "out of device memory: %zu of %zu chunks of %zu bytes could be created", got, n, chunk);
  }
  const int n_fillers = (int)fillers.size();
  release_all(fillers);
  pr.destroy();

  // map alternately: position k takes an "other" chunk whenever that keeps the two kinds evenly mixed
  Allocation al;
  al.device = device;
  al.bytes = n * chunk;
  al.chunk = chunk;
  al.n_other = (int)other.size();
  al.n_fillers = n_fillers;
  al.n_reprobed = n_reprobed;
  al.pair_ms_same = ref_ms;
  al.pair_ms_other = fastest_ms;
  hipError_t e = hipMemAddressReserve(&al.va, al.bytes, 0, nullptr, 0);
  if (e != hipSuccess) { cleanup(); return fail_hip(e, "hipMemAddressReserve"); }
  const std::vector<bool> order = interleave_order(same.size(), other.size());
  size_t is = 0, io = 0;
  for (size_t k = 0; k < n && e == hipSuccess; ++k) {
    hipMemGenericAllocationHandle_t h = order[k] ? other[io++] : same[is++];
    e = hipMemMap(static_cast<char*>(al.va) + k * chunk, chunk, 0, h, 0);
    if (e == hipSuccess) al.handles.push_back(h);
  }
  if (e == hipSuccess) {
    hipMemAccessDesc acc = hipMemAccessDesc();
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = device;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    e = hipMemSetAccess(al.va, al.bytes, &acc, 1);
  }
  if (e != hipSuccess) {
    if (!al.handles.empty()) (void)hipMemUnmap(al.va, al.handles.size() * chunk);
    (void)hipMemAddressFree(al.va, al.bytes);
    cleanup();
    return fail_hip(e, "hipMemMap / hipMemSetAccess");
  }
  same.clear();
  other.clear();
  al.seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t_begin).count();
  {
    std::lock_guard<std::mutex> lk(g_mu);
    g_allocs[al.va] = al;
  }
  *out = al.va;
  return BIKV_OK;
}

extern "C" int bikv_device_alloc(int device, int64_t bytes, int32_t placement, void** out) {
  return bikv_device_alloc_bounded(device, bytes, placement, BIKV_DEFAULT_MAX_FILLER_BYTES, out);
}

extern "C" int bikv_device_free(void* p) {
  if (!p) return BIKV_OK;
  Allocation al;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_allocs.find(p);
    if (it == g_allocs.end()) return fail(BIKV_EINVAL, "pointer was not returned by bikv_device_alloc");
    al = it->second;
    g_allocs.erase(it);
  }
  BIKV_DEVICE(al.device);
  BIKV_HIP(hipDeviceSynchronize());
  hipError_t e = hipMemUnmap(al.va, al.bytes);
  release_all(al.handles);
  const hipError_t e2 = hipMemAddressFree(al.va, al.bytes);
  if (e != hipSuccess) return fail_hip(e, "hipMemUnmap");
  if (e2 != hipSuccess) return fail_hip(e2, "hipMemAddressFree");
  return BIKV_OK;
}

// Entry points with the signatures torch.cuda.memory.CUDAPluggableAllocator binds, so that a torch memory pool
// (torch.cuda.MemPool) can take its segments from bikv_device_alloc and the reference's torch.empty call sites
// (kvcache.py:38-43, Worker.py:74-78) stay as they are. Segments of up to 1 GiB are carved, one after the other,
// out of placed arenas of 2 GiB (host_logic/arena_logic.h), so that a pool made of many tensors smaller than a
// chunk still alternates between the halves; larger ones are placements of their own. A null return makes
// torch report out-of-memory.
constexpr int64_t kTorchArenaBytes = int64_t(2) << 30;
static void* torch_backend_alloc(int device, int64_t bytes) {
  void* p = nullptr;
  return bikv_device_alloc(device, bytes, BIKV_PLACE_SPREAD, &p) == BIKV_OK ? p : nullptr;
}
static void torch_backend_free(void* base) { (void)bikv_device_free(base); }
static arena::Book& torch_book() {
  static arena::Book* book = new arena::Book(kTorchArenaBytes, torch_backend_alloc, torch_backend_free);   // never destroyed
  return *book;
}

// torch releases what its pools still hold while the process exits, when this library's bookkeeping and the
// HIP runtime may already be gone; from the first exit handler on, releasing is left to the driver.
static std::atomic<bool> g_exiting{false};
static void mark_exiting() { g_exiting.store(true); }

extern "C" void* bikv_torch_alloc(int64_t size, int device, void* /*stream*/) {
  static std::once_flag once;
  std::call_once(once, [] { atexit(mark_exiting); });   // registered late, so it runs before any static destructor
  if (size <= 0 || g_exiting.load()) return nullptr;
  return torch_book().take(device, size);
}

extern "C" void bikv_torch_free(void* p, size_t /*size*/, int /*device*/, void* /*stream*/) {
  if (g_exiting.load()) return;
  (void)torch_book().give(p);
}

extern "C" int bikv_device_alloc_info(const void* p, bikv_alloc_info* info) {
  if (!p || !info) return fail(BIKV_EINVAL, "null argument");
  std::lock_guard<std::mutex> lk(g_mu);
  // any address inside an allocation names it (tensors carved out of an arena start past its base)
  auto it = g_allocs.upper_bound(const_cast<void*>(p));
  if (it == g_allocs.begin()) return fail(BIKV_EINVAL, "address is not inside memory from bikv_device_alloc");
  --it;
  if (static_cast<const char*>(p) >= static_cast<const char*>(it->first) + it->second.bytes)
    return fail(BIKV_EINVAL, "address is not inside memory from bikv_device_alloc");
  info->bytes = (int64_t)it->second.bytes;
  info->chunk_bytes = (int64_t)it->second.chunk;
  info->n_chunks = (int32_t)it->second.handles.size();
  info->n_other_half = it->second.n_other;
  info->n_fillers = it->second.n_fillers;
  info->n_reprobed = it->second.n_reprobed;
  info->seconds = it->second.seconds;
  info->pair_ms_same = it->second.pair_ms_same;
  info->pair_ms_other = it->second.pair_ms_other;
  return BIKV_OK;
}
