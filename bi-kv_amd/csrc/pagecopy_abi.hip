// C ABI of libbikv_pagecopy.so: argument validation, per-device context, pool handles, the layered
// gather/scatter entry points, the run copy and the device->pinned-host staging pipeline.
// Declarations and the reference call sites each entry point replaces: include/bikv_pagecopy.h.
#include "../../include/bikv_pagecopy.h"
#include "host_logic/chunk_planner.h"
#include "host_logic/host_checks.h"
#include "pagecopy_internal.h"
#include "pagecopy_kernels.h"

#include <algorithm>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <utility>
#include <vector>

namespace bikv {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int fail_hip(hipError_t e, const char* what) {
  return fail(BIKV_EHIP, "%s failed: %s", what, hipGetErrorString(e));
}

// ---- scratch of the allocation-free entry point ---------------------------------------------
// bikv_gather_to_host_noalloc stages through this array instead of a stager's hipMalloc'd buffers:
// kScratchPayload bytes for payload tiles followed by kScratchScale bytes for scale tiles. Every GPU the
// library runs on holds its own copy (16 MiB + 64 KiB) until the process ends. In host code the name is
// only a handle: the device address is taken once per device with hipGetSymbolAddress (device_status
// below) and that pointer is what kernels and copies are given.
constexpr int64_t kScratchPayload = int64_t(16) << 20;
constexpr int64_t kScratchScale = int64_t(64) << 10;
constexpr int64_t kScratchCopy = int64_t(8) << 20;     // bytes per hipMemcpyAsync out of the scratch (only when an
                                                        // address is not 16-byte aligned and the copy kernel cannot be used)
static __device__ __align__(256) unsigned char scratch[kScratchPayload + kScratchScale];

// ---- per-device context: the host-mapped status block and the scratch address ---------------
struct DevCtx {
  uint32_t* status_host = nullptr;  // pinned, mapped
  uint32_t* status_dev = nullptr;   // the same memory as the device sees it
  char* scratch_dev = nullptr;      // this device's copy of `scratch`
  bool bank_used[ST_BANKS] = {};    // banks handed out to stagers (the fixed ones are never marked)
};
static std::mutex g_ctx_mu;
static DevCtx g_ctx[64];

int device_status(int device, int bank, uint32_t** dev_ptr) {
  if (device < 0 || device >= 64) return fail(BIKV_EINVAL, "device index %d out of range", device);
  if (bank < 0 || bank >= ST_BANKS) return fail(BIKV_EINVAL, "internal: status bank %d", bank);
  std::lock_guard<std::mutex> lk(g_ctx_mu);
  DevCtx& c = g_ctx[device];
  if (!c.status_host) {
    BIKV_DEVICE(device);
    void* h = nullptr;
    BIKV_HIP(hipHostMalloc(&h, ST_SLOTS * sizeof(uint32_t) * ST_BANKS, hipHostMallocMapped | hipHostMallocPortable));
    memset(h, 0, ST_SLOTS * sizeof(uint32_t) * ST_BANKS);
    void* d = nullptr;
    hipError_t e = hipHostGetDevicePointer(&d, h, 0);
    if (e != hipSuccess) {
      (void)hipHostFree(h);
      return fail_hip(e, "hipHostGetDevicePointer");
    }
    // this device's address of the scratch array (the device is current here)
    void* sp = nullptr;
    e = hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !sp) {
      (void)hipHostFree(h);
      return fail_hip(e != hipSuccess ? e : hipErrorInvalidSymbol, "hipGetSymbolAddress(scratch)");
    }
    c.status_host = static_cast<uint32_t*>(h);
    c.status_dev = static_cast<uint32_t*>(d);
    c.scratch_dev = static_cast<char*>(sp);
  }
  *dev_ptr = c.status_dev + bank * ST_SLOTS;
  return BIKV_OK;
}

int acquire_bank(int device, int* bank_out) {
  uint32_t* st = nullptr;
  const int rc = device_status(device, ST_BANK_SHARED, &st);   // creates the block on first use
  if (rc) return rc;
  std::lock_guard<std::mutex> lk(g_ctx_mu);
  DevCtx& c = g_ctx[device];
  for (int b = ST_BANK_DYNAMIC; b < ST_BANKS; ++b) {
    if (c.bank_used[b]) continue;
    c.bank_used[b] = true;
    volatile uint32_t* s = c.status_host + b * ST_SLOTS;
    for (int i = 0; i < ST_SLOTS; ++i) s[i] = 0;
    *bank_out = b;
    return BIKV_OK;
  }
  return fail(BIKV_ERANGE, "device %d already has %d host stagers: no status words are left for another",
              device, ST_BANKS - ST_BANK_DYNAMIC);
}

void release_bank(int device, int bank) {
  if (device < 0 || device >= 64 || bank < ST_BANK_DYNAMIC || bank >= ST_BANKS) return;
  std::lock_guard<std::mutex> lk(g_ctx_mu);
  g_ctx[device].bank_used[bank] = false;
}

// The scratch address of a device whose context already exists; never creates one (the allocation-free
// entry point must not allocate, and creating a context allocates the status block).
static char* scratch_of(int device) {
  if (device < 0 || device >= 64) return nullptr;
  std::lock_guard<std::mutex> lk(g_ctx_mu);
  return g_ctx[device].status_host ? g_ctx[device].scratch_dev : nullptr;
}

static uint32_t take_status(int device, int bank) {
  std::lock_guard<std::mutex> lk(g_ctx_mu);
  DevCtx& c = g_ctx[device];
  if (!c.status_host) return 0;
  volatile uint32_t* s = c.status_host + bank * ST_SLOTS;
  uint32_t bits = 0;
  if (s[ST_SLOT_SRC]) bits |= BIKV_ST_SRC_RANGE;
  if (s[ST_SLOT_DST]) bits |= BIKV_ST_DST_RANGE;
  if (s[ST_SLOT_PAGE]) bits |= BIKV_ST_PAGE_ID;
  s[ST_SLOT_SRC] = 0;
  s[ST_SLOT_DST] = 0;
  s[ST_SLOT_PAGE] = 0;
  return bits;
}

static int status_error(uint32_t bits) {
  if (!bits) return BIKV_OK;
  return fail(BIKV_EBOUNDS, "kernel skipped out-of-range work (status bits 0x%x:%s%s%s)", bits,
              (bits & BIKV_ST_SRC_RANGE) ? " source-range" : "",
              (bits & BIKV_ST_DST_RANGE) ? " destination-range" : "",
              (bits & BIKV_ST_PAGE_ID) ? " page-id" : "");
}

int sync_and_check(int device, int bank, hipStream_t stream) {
  BIKV_HIP(hipStreamSynchronize(stream));
  return status_error(take_status(device, bank));
}

int check_bank(int device, int bank) { return status_error(take_status(device, bank)); }

static int current_device(int* dev) {
  BIKV_HIP(hipGetDevice(dev));
  return BIKV_OK;
}

static int lowbit_width(uint64_t x) {
  int w = 16;
  while (w > 1 && (x & (uint64_t)(w - 1))) w >>= 1;
  return w;
}

}  // namespace bikv

using namespace bikv;

// ---- pool handle --------------------------------------------------------------------------
struct bikv_pool {
  int device;
  int n_planes;
  int64_t n_pages;
  int64_t tile_bytes, page_stride;
  int64_t row_bytes, row_stride;    // row_bytes == tile_bytes: contiguous tiles
  int64_t scale_tile_bytes, scale_page_stride;
  const char** d_plane_base;        // device table: payload planes, then scale planes
  uint64_t align_bits;              // OR of every base, stride and tile size (payload)
  uint64_t scale_align_bits;
};

extern "C" int bikv_abi_version(void) { return BIKV_ABI_VERSION; }

extern "C" int bikv_init(int device) {
  uint32_t* st = nullptr;
  return device_status(device, ST_BANK_SHARED, &st);
}
extern "C" const char* bikv_last_error(void) { return g_err; }

extern "C" int bikv_check_status(int device, void* stream, uint32_t* bits_out) {
  if (device < 0 || device >= 64) return fail(BIKV_EINVAL, "device index %d out of range", device);
  BIKV_DEVICE(device);
  BIKV_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  const uint32_t bits = take_status(device, ST_BANK_SHARED);
  if (bits_out) *bits_out = bits;
  return status_error(bits);
}

extern "C" void bikv_reset_tuning(void) {
  std::lock_guard<std::mutex> lk(tuning_mutex());
  tuning_shared() = Tuning();
}

extern "C" int bikv_set_tuning(const char* key, int64_t value) {
  if (!key) return fail(BIKV_EINVAL, "null tuning key");
  std::lock_guard<std::mutex> lk(tuning_mutex());
  Tuning& t = tuning_shared();
  if (!strcmp(key, "seg")) {
    if (value < 0 || value > kMaxSeg) return fail(BIKV_EINVAL, "seg must be in [0, %d]", kMaxSeg);
    t.seg = (int)value;
  } else if (!strcmp(key, "unroll")) {
    if (value != 1 && value != 2 && value != 4 && value != 8)
      return fail(BIKV_EINVAL, "unroll must be 1, 2, 4 or 8");
    t.unroll = (int)value;
  } else if (!strcmp(key, "wave_block")) {
    if (value != 64 && value != 128 && value != 256)
      return fail(BIKV_EINVAL, "wave_block must be 64, 128 or 256");
    t.wave_block = (int)value;
  } else if (!strcmp(key, "order")) {
    if (value < -1 || value > 1) return fail(BIKV_EINVAL, "order must be -1, 0 or 1");
    t.order = (int)value;
  } else if (!strcmp(key, "log2_chunk")) {
    if (value < -1 || value > 16) return fail(BIKV_EINVAL, "log2_chunk must be in [-1, 16]");
    t.log2_chunk = (int)value;
  } else if (!strcmp(key, "nontemporal")) {
    if (value > 4) return fail(BIKV_EINVAL, "nontemporal must be -1, 0, 1, 2 (loads only), 3 (stores only) or 4 (nt + sc1)");
    t.nontemporal = value < 0 ? -1 : (int)value;
  } else if (!strcmp(key, "transpose_lds_kib")) {
    if (value < 2 || value > 60) return fail(BIKV_EINVAL, "transpose_lds_kib must be in [2, 60]");
    t.transpose_lds_kib = (int)value;
  } else if (!strcmp(key, "transpose_dsplit")) {
    if (value < 0 || value > 16 || (value & (value - 1))) return fail(BIKV_EINVAL, "transpose_dsplit must be 0 or a power of two <= 16");
    t.transpose_dsplit = (int)value;
  } else if (!strcmp(key, "run_group")) {
    t.run_group = value ? 1 : 0;
  } else if (!strcmp(key, "small_run_max")) {
    if (value < 16 || value > (1 << 20)) return fail(BIKV_EINVAL, "small_run_max must be in [16, 1 MiB]");
    t.small_run_max = (int)value;
  } else if (!strcmp(key, "transpose_block")) {
    if (value != 0 && value != 128 && value != 256 && value != 512 && value != 1024)
      return fail(BIKV_EINVAL, "transpose_block must be 0 (chosen per direction), 128, 256, 512 or 1024");
    t.transpose_block = (int)value;
  } else if (!strcmp(key, "transpose_sc1")) {
    t.transpose_sc1 = value ? 1 : 0;
  } else if (!strcmp(key, "transpose_kvswap")) {
    t.transpose_kvswap = value ? 1 : 0;
  } else if (!strcmp(key, "transpose_pairs")) {
    t.transpose_pairs = value ? 1 : 0;
  } else if (!strcmp(key, "debug_unique")) {
    t.debug_unique = value ? 1 : 0;
  } else {
    return fail(BIKV_EINVAL, "unknown tuning key '%s'", key);
  }
  return BIKV_OK;
}

extern "C" int bikv_pool_create(const bikv_pool_desc* d, bikv_pool** out) {
  if (!d || !out) return fail(BIKV_EINVAL, "null argument");
  *out = nullptr;
  if (d->n_planes <= 0 || d->n_planes > 65536) return fail(BIKV_EINVAL, "n_planes %d out of range", d->n_planes);
  if (d->n_pages <= 0) return fail(BIKV_EINVAL, "n_pages must be positive");
  if (d->tile_bytes <= 0 || d->page_stride_bytes < d->tile_bytes)
    return fail(BIKV_EINVAL, "need 0 < tile_bytes <= page_stride_bytes (got %lld, %lld)",
                (long long)d->tile_bytes, (long long)d->page_stride_bytes);
  if (!d->plane_base) return fail(BIKV_EINVAL, "plane_base is null");
  const bool has_scale = d->scale_tile_bytes > 0;
  if (has_scale && (!d->scale_plane_base || d->scale_page_stride_bytes < d->scale_tile_bytes))
    return fail(BIKV_EINVAL, "scale class needs scale_plane_base and scale_page_stride_bytes >= scale_tile_bytes");
  if (d->scale_tile_bytes < 0) return fail(BIKV_EINVAL, "negative scale_tile_bytes");
  int64_t row_bytes = d->tile_bytes, row_stride = d->tile_bytes;
  if (d->row_bytes < 0 || d->row_stride_bytes < 0) return fail(BIKV_EINVAL, "negative row_bytes or row_stride_bytes");
  if (d->row_bytes > 0 && d->row_bytes != d->tile_bytes) {
    row_bytes = d->row_bytes;
    row_stride = d->row_stride_bytes;
    if (d->tile_bytes % row_bytes != 0 || row_stride < row_bytes)
      return fail(BIKV_EINVAL, "need tile_bytes %% row_bytes == 0 and row_stride_bytes >= row_bytes (got %lld, %lld, %lld)",
                  (long long)d->tile_bytes, (long long)row_bytes, (long long)row_stride);
  }

  std::vector<const char*> table((size_t)d->n_planes * 2, nullptr);
  uint64_t ab = (uint64_t)d->tile_bytes | (uint64_t)d->page_stride_bytes | (uint64_t)row_bytes |
                (uint64_t)row_stride, sab = 0;
  for (int q = 0; q < d->n_planes; ++q) {
    if (!d->plane_base[q]) return fail(BIKV_EINVAL, "plane_base[%d] is null", q);
    table[q] = static_cast<const char*>(d->plane_base[q]);
    ab |= (uint64_t)d->plane_base[q];
  }
  if (has_scale) {
    sab = (uint64_t)d->scale_tile_bytes | (uint64_t)d->scale_page_stride_bytes;
    for (int q = 0; q < d->n_planes; ++q) {
      if (!d->scale_plane_base[q]) return fail(BIKV_EINVAL, "scale_plane_base[%d] is null", q);
      table[d->n_planes + q] = static_cast<const char*>(d->scale_plane_base[q]);
      sab |= (uint64_t)d->scale_plane_base[q];
    }
  }
  uint32_t* st = nullptr;
  int rc = device_status(d->device, ST_BANK_SHARED, &st);
  if (rc) return rc;
  BIKV_DEVICE(d->device);
  void* dtab = nullptr;
  BIKV_HIP(hipMalloc(&dtab, table.size() * sizeof(char*)));
  hipError_t e = hipMemcpy(dtab, table.data(), table.size() * sizeof(char*), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(dtab);
    return fail_hip(e, "hipMemcpy(plane table)");
  }
  bikv_pool* p = new bikv_pool();
  p->device = d->device;
  p->n_planes = d->n_planes;
  p->n_pages = d->n_pages;
  p->tile_bytes = d->tile_bytes;
  p->page_stride = d->page_stride_bytes;
  p->row_bytes = row_bytes;
  p->row_stride = row_stride;
  p->scale_tile_bytes = has_scale ? d->scale_tile_bytes : 0;
  p->scale_page_stride = has_scale ? d->scale_page_stride_bytes : 0;
  p->d_plane_base = static_cast<const char**>(dtab);
  p->align_bits = ab;
  p->scale_align_bits = sab;
  *out = p;
  return BIKV_OK;
}

extern "C" int bikv_pool_destroy(bikv_pool* p) {
  if (!p) return BIKV_OK;
  DeviceGuard guard_(p->device);
  hipError_t e = hipFree((void*)p->d_plane_base);
  delete p;
  if (e != hipSuccess) return fail_hip(e, "hipFree(plane table)");
  return BIKV_OK;
}

namespace bikv {

// Fills MoveArgs for one launch; `staging`/`scale_staging` are slot 0 of the (possibly windowed)
// staging image after slot_bias has been applied.
static int build_move(int bank, const bikv_pool* pool, const bikv_page_batch* b, const void* staging,
                      int64_t staging_bytes, const void* scale_staging, int64_t scale_bytes,
                      MoveArgs* m) {
  if (!pool || !b) return fail(BIKV_EINVAL, "null pool or batch");
  if (b->n_pages < 0) return fail(BIKV_EINVAL, "negative n_pages");
  int pb = b->plane_begin, pc = b->plane_count;
  if (pc <= 0) { pb = 0; pc = pool->n_planes; }
  if (pb < 0 || pb + pc > pool->n_planes)
    return fail(BIKV_EINVAL, "planes [%d, %d) outside [0, %d)", pb, pb + pc, pool->n_planes);
  memset(m, 0, sizeof(*m));
  m->n_batch = b->n_pages;
  m->plane_begin = pb;
  m->plane_count = pc;
  m->layout_hint = b->layout_hint;
  if (b->n_pages == 0) return BIKV_OK;
  if (!b->page_ids || !b->slots || !b->slot_strides)
    return fail(BIKV_EINVAL, "page_ids, slots and slot_strides must be non-null");
  if (!staging || staging_bytes < 0) return fail(BIKV_EINVAL, "staging buffer is null or negative-sized");
  const bool has_scale = pool->scale_tile_bytes > 0;
  if (has_scale && (!scale_staging || scale_bytes < 0))
    return fail(BIKV_EINVAL, "pool has a scale class: scale_staging must be given");
  uint32_t* st = nullptr;
  int rc = device_status(pool->device, bank, &st);
  if (rc) return rc;
  m->page_ids = b->page_ids;
  m->slots = b->slots;
  m->slot_strides = b->slot_strides;
  m->n_pool_pages = pool->n_pages;
  m->slot_bias = b->slot_bias;
  m->status = st;
  m->payload.plane_base = pool->d_plane_base;
  m->payload.staging = static_cast<char*>(const_cast<void*>(staging));
  m->payload.n_slots = staging_bytes / pool->tile_bytes;
  m->payload.tile_bytes = pool->tile_bytes;
  m->payload.page_stride = pool->page_stride;
  m->payload.row_bytes = pool->row_bytes;
  m->payload.row_stride = pool->row_stride;
  m->payload.log2_row = -1;
  if ((pool->row_bytes & (pool->row_bytes - 1)) == 0)
    for (m->payload.log2_row = 0; (int64_t(1) << m->payload.log2_row) < pool->row_bytes;) ++m->payload.log2_row;
  m->payload.vec_width = lowbit_width(pool->align_bits | (uint64_t)staging);
  if (has_scale) {
    m->scale.plane_base = pool->d_plane_base + pool->n_planes;
    m->scale.staging = static_cast<char*>(const_cast<void*>(scale_staging));
    m->scale.n_slots = scale_bytes / pool->scale_tile_bytes;
    m->scale.tile_bytes = pool->scale_tile_bytes;
    m->scale.page_stride = pool->scale_page_stride;
    m->scale.row_bytes = pool->scale_tile_bytes;
    m->scale.row_stride = pool->scale_tile_bytes;
    m->scale.log2_row = -1;
    m->scale.vec_width = lowbit_width(pool->scale_align_bits | (uint64_t)scale_staging);
  }
  return BIKV_OK;
}

static int move_pages(int bank, int dir, const bikv_pool* pool, const bikv_page_batch* b, const void* staging,
                      int64_t staging_bytes, const void* scale_staging, int64_t scale_bytes,
                      void* stream) {
  MoveArgs m;
  int rc = build_move(bank, pool, b, staging, staging_bytes, scale_staging, scale_bytes, &m);
  if (rc) return rc;
  if (m.n_batch == 0) return BIKV_OK;
  BIKV_DEVICE(pool->device);
  hipError_t e = launch_tile_move(dir, m, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail_hip(e, dir == 0 ? "gather launch" : "scatter launch");
  return BIKV_OK;
}

}  // namespace bikv

// ---- duplicate destinations ---------------------------------------------------------------------
// Two runs of one launch that write the same destination race (the reference's kernel has the same
// property, copy_kernel.cu:29-35: whichever block stores last wins). bikv_find_duplicate is the check
// on a host array; with BIKV_DEBUG_UNIQUE=1 in the environment the scattering entry points run it on a
// copy of the caller's device ids before they launch (a debugging aid: it synchronises the stream).
extern "C" int bikv_find_duplicate(const int64_t* ids, int64_t n, int64_t* dup_out) {
  if (n < 0 || (n > 0 && !ids)) return fail(BIKV_EINVAL, "bad find_duplicate arguments");
  int64_t best_id = 0, best_first = 0, best = 0;
  if (!find_first_duplicate(ids, n, &best_id, &best_first, &best)) return BIKV_OK;
  if (dup_out) *dup_out = best_id;
  return fail(BIKV_EINVAL, "destination id %lld is named more than once (entries %lld and %lld): a scatter's "
                           "destinations must be unique", (long long)best_id, (long long)best_first, (long long)best);
}

namespace bikv {

static bool debug_unique() {
  static const bool env_on = [] {
    const char* e = getenv("BIKV_DEBUG_UNIQUE");
    return e && e[0] && e[0] != '0';
  }();
  refresh_tuning();
  return env_on || tuning().debug_unique != 0;
}

// Debug path: fetches `n` device ids behind `stream` and fails if one repeats.
int check_unique_on_device(int device, const int64_t* dev_ids, int64_t n, hipStream_t stream) {
  if (!debug_unique() || n <= 1 || !dev_ids) return BIKV_OK;
  BIKV_DEVICE(device);
  std::vector<int64_t> host((size_t)n);
  BIKV_HIP(hipStreamSynchronize(stream));
  BIKV_HIP(hipMemcpy(host.data(), dev_ids, (size_t)n * sizeof(int64_t), hipMemcpyDeviceToHost));
  return bikv_find_duplicate(host.data(), n, nullptr);
}

}  // namespace bikv

extern "C" int bikv_gather_pages(const bikv_pool* pool, const bikv_page_batch* batch, void* staging,
                                 int64_t staging_bytes, void* scale_staging,
                                 int64_t scale_staging_bytes, void* stream) {
  return move_pages(ST_BANK_SHARED, 0, pool, batch, staging, staging_bytes, scale_staging, scale_staging_bytes, stream);
}

extern "C" int bikv_scatter_pages(const bikv_pool* pool, const bikv_page_batch* batch,
                                  const void* staging, int64_t staging_bytes,
                                  const void* scale_staging, int64_t scale_staging_bytes,
                                  void* stream) {
  if (pool && batch) {
    const int rc = check_unique_on_device(pool->device, batch->page_ids, batch->n_pages, static_cast<hipStream_t>(stream));
    if (rc) return rc;
  }
  return move_pages(ST_BANK_SHARED, 1, pool, batch, staging, staging_bytes, scale_staging, scale_staging_bytes, stream);
}

// The device that owns the memory behind `p`, or -1 when the runtime does not know the pointer or it is
// host memory.
static int device_of_pointer(const void* p) {
  hipPointerAttribute_t at;
  memset(&at, 0, sizeof(at));
  if (hipPointerGetAttributes(&at, p) != hipSuccess) {
    (void)hipGetLastError();   // an unknown pointer is not an error of this call
    return -1;
  }
  return at.type == hipMemoryTypeDevice ? at.device : -1;
}

int bikv::copy_runs_banked(int bank, const void* src, int64_t src_bytes, void* dst, int64_t dst_bytes,
                           const int64_t* src_off, const int64_t* dst_off, const int64_t* run_len,
                           int64_t n_runs, int64_t run_bytes, int64_t unit_bytes, void* stream) {
  if (n_runs < 0 || run_bytes < 0) return fail(BIKV_EINVAL, "negative n_runs or run_bytes");
  if (n_runs == 0 || run_bytes == 0) return BIKV_OK;
  if (!src || !dst || !src_off || !dst_off) return fail(BIKV_EINVAL, "null pointer argument");
  if (unit_bytes <= 0) return fail(BIKV_EINVAL, "unit_bytes must be positive");
  if (n_runs >= (int64_t(1) << 31)) return fail(BIKV_EINVAL, "too many runs");
  if (!run_len && (run_bytes > src_bytes || run_bytes > dst_bytes))
    return fail(BIKV_EINVAL, "run_bytes %lld exceeds a buffer (src %lld, dst %lld bytes)",
                (long long)run_bytes, (long long)src_bytes, (long long)dst_bytes);
  // The launch and its status words belong to the device that holds the data: the destination's, else
  // the source's (one of the two may be pinned host memory), else the offset tables', and the calling
  // thread's current device only when the runtime knows none of the pointers.
  int dev = device_of_pointer(dst);
  if (dev < 0) dev = device_of_pointer(src);
  if (dev < 0) dev = device_of_pointer(src_off);
  int rc = BIKV_OK;
  if (dev < 0) {
    rc = current_device(&dev);
    if (rc) return rc;
  }
  BIKV_DEVICE(dev);
  RunArgs a;
  a.src = static_cast<const char*>(src);
  a.dst = static_cast<char*>(dst);
  a.src_bytes = src_bytes;
  a.dst_bytes = dst_bytes;
  a.src_off = src_off;
  a.dst_off = dst_off;
  a.n_runs = n_runs;
  a.run_bytes = run_bytes;
  a.unit_bytes = unit_bytes;
  a.run_lens = run_len;
  rc = device_status(dev, bank, &a.status);
  if (rc) return rc;
  hipError_t e = launch_copy_runs(a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail_hip(e, "copy_runs launch");
  return BIKV_OK;
}

extern "C" int bikv_copy_runs(const void* src, int64_t src_bytes, void* dst, int64_t dst_bytes,
                              const int64_t* src_off, const int64_t* dst_off, int64_t n_runs,
                              int64_t run_bytes, int64_t unit_bytes, void* stream) {
  return copy_runs_banked(ST_BANK_SHARED, src, src_bytes, dst, dst_bytes, src_off, dst_off, nullptr, n_runs,
                          run_bytes, unit_bytes, stream);
}

extern "C" int bikv_copy_runs_ragged(const void* src, int64_t src_bytes, void* dst, int64_t dst_bytes,
                                     const int64_t* src_off, const int64_t* dst_off,
                                     const int64_t* run_len, int64_t n_runs, int64_t max_run_bytes,
                                     int64_t unit_bytes, void* stream) {
  if (n_runs > 0 && !run_len) return fail(BIKV_EINVAL, "run_len is null");
  return copy_runs_banked(ST_BANK_SHARED, src, src_bytes, dst, dst_bytes, src_off, dst_off, run_len, n_runs,
                          max_run_bytes, unit_bytes, stream);
}

// ---- pinned host memory -------------------------------------------------------------------
extern "C" int bikv_host_alloc(int64_t bytes, void** out) {
  if (!out || bytes <= 0) return fail(BIKV_EINVAL, "bad host_alloc arguments");
  BIKV_HIP(hipHostMalloc(out, (size_t)bytes, hipHostMallocMapped | hipHostMallocPortable));
  return BIKV_OK;
}

extern "C" int bikv_host_free(void* p) {
  if (!p) return BIKV_OK;
  BIKV_HIP(hipHostFree(p));
  return BIKV_OK;
}

static int link_copy(int device, void* dst, const void* src, int64_t bytes, int64_t chunk_bytes,
                     hipMemcpyKind kind, double* seconds_out) {
  if (!dst || !src || bytes <= 0) return fail(BIKV_EINVAL, "bad host-link copy arguments");
  BIKV_DEVICE(device);
  hipStream_t s;
  BIKV_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  if (chunk_bytes <= 0) chunk_bytes = bytes;
  const auto t0 = std::chrono::steady_clock::now();
  hipError_t e = hipSuccess;
  for (int64_t off = 0; off < bytes && e == hipSuccess; off += chunk_bytes) {
    const int64_t n = bytes - off < chunk_bytes ? bytes - off : chunk_bytes;
    e = hipMemcpyAsync(static_cast<char*>(dst) + off, static_cast<const char*>(src) + off,
                       (size_t)n, kind, s);
  }
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  const auto t1 = std::chrono::steady_clock::now();
  (void)hipStreamDestroy(s);
  if (e != hipSuccess) return fail_hip(e, "hipMemcpyAsync(host link)");
  if (seconds_out) *seconds_out = std::chrono::duration<double>(t1 - t0).count();
  return BIKV_OK;
}

extern "C" int bikv_d2h_copy(int device, void* host_dst, const void* dev_src, int64_t bytes,
                             int64_t chunk_bytes, double* seconds_out) {
  return link_copy(device, host_dst, dev_src, bytes, chunk_bytes, hipMemcpyDeviceToHost, seconds_out);
}

extern "C" int bikv_h2d_copy(int device, void* dev_dst, const void* host_src, int64_t bytes,
                             int64_t chunk_bytes, double* seconds_out) {
  return link_copy(device, dev_dst, host_src, bytes, chunk_bytes, hipMemcpyHostToDevice, seconds_out);
}

// ---- device <-> pinned-host staging pipeline -----------------------------------------------
// The stager owns n_buffers "lanes": a HIP stream with its own buffer in HBM. Launch k of the pipeline
// runs on lane k % n_buffers: ONE gather kernel fills the lane's buffer with `group` chunks' worth of the
// staging image, then `group` hipMemcpyAsync calls of chunk_bytes each move it to the host, all in the
// lane's stream order (for the receiving direction: the copies first, then one scatter kernel). Lanes
// never wait on each other: while one lane's copies occupy the host link the next lane's kernel has
// long finished (it moves its bytes ~100x faster than the link does) and its copies are queued.
//
// What shaped this (measured on MI355X, 64 KiB tiles, 1 GiB per pass, copies timed by rocprofv3's
// memory-copy trace):
//   * the DMA engine leaves ~9.5 us between two consecutive copies whatever stream they come from, so
//     4 MiB copies cannot exceed ~88 % of the link and 8 / 16 / 32 MiB reach 93 / 96 / 98 %;
//   * a kernel between two copies of one stream costs one more hand-over each way: one lane alone loses
//     another 5-10 %, two lanes hide it, more than two add nothing;
//   * host -> device, one kernel per copy makes small chunks erratic (4 MiB x 4 lanes: 72-95 % from pass
//     to pass) while one kernel per 4-8 copies stays at 95-98 %: hence `group`;
//   * ordering a copy stream behind a kernel stream with events loses 10-30 % below 16 MiB;
//   * the device -> host DMA path has two speeds on this platform, ~30 and ~57 GB/s, and a process can
//     sit in either for minutes (the host -> device path and kernels storing into mapped pinned memory
//     do not show it): BIKV_STAGE_DIRECT keeps 55 GB/s in both states, which is why BIKV_STAGE_AUTO
//     sends with the kernel and receives with the DMA engine.
// One step of a lane as the optional trace records it: two events around the launch or copy.
struct TraceOp {
  hipEvent_t e0, e1;
  int32_t lane, kind;
  int64_t bytes;
};

struct bikv_stager {
  int device;
  int bank;                  // this stager's own status words
  int64_t chunk_bytes;       // bytes of one host copy
  int group;                 // copies per kernel launch
  int64_t lane_bytes;        // chunk_bytes * group: HBM buffer of one lane
  int n_buf;
  char* ring;
  char* scale_ring;          // grown on demand: n_buf buffers of scale tiles
  int64_t scale_ring_bytes;
  std::vector<hipStream_t> lanes;
  hipEvent_t after;          // orders the lanes behind a caller's stream
  uint64_t next_launch;      // launches issued since creation (lane = next_launch % n_buf)
  // since the last bikv_stager_wait
  int64_t pending_bytes, pending_copies;
  bool timing;
  std::chrono::steady_clock::time_point t_first;
  // opt-in trace (bikv_stager_trace): up to trace_cap steps, each between two timing events
  int64_t trace_cap = 0;
  std::vector<TraceOp> trace;
};

extern "C" int bikv_stager_create(int device, int64_t chunk_bytes, int32_t chunks_per_launch,
                                  int32_t n_buffers, bikv_stager** out) {
  if (!out) return fail(BIKV_EINVAL, "null out");
  *out = nullptr;
  if (chunk_bytes < 4096 || n_buffers < 1 || n_buffers > 16 || chunks_per_launch < 1 || chunks_per_launch > 64)
    return fail(BIKV_EINVAL, "need chunk_bytes >= 4096, 1 <= chunks_per_launch <= 64 and 1 <= n_buffers <= 16");
  if (chunk_bytes > (int64_t(1) << 36) / chunks_per_launch) return fail(BIKV_EINVAL, "lane buffer too large");
  int bank = -1;
  int rc = acquire_bank(device, &bank);
  if (rc) return rc;
  DeviceGuard guard_(device);
  if (guard_.error() != hipSuccess) {
    release_bank(device, bank);
    return fail_hip(guard_.error(), "hipSetDevice");
  }
  bikv_stager* st = new bikv_stager();
  st->device = device;
  st->bank = bank;
  st->chunk_bytes = chunk_bytes;
  st->group = chunks_per_launch;
  st->lane_bytes = chunk_bytes * chunks_per_launch;
  st->n_buf = n_buffers;
  st->ring = nullptr;
  st->scale_ring = nullptr;
  st->scale_ring_bytes = 0;
  st->after = nullptr;
  st->next_launch = 0;
  st->pending_bytes = st->pending_copies = 0;
  st->timing = false;
  hipError_t e = hipMalloc((void**)&st->ring, (size_t)st->lane_bytes * n_buffers);
  if (e == hipSuccess) e = hipEventCreateWithFlags(&st->after, hipEventDisableTiming);
  for (int i = 0; i < n_buffers && e == hipSuccess; ++i) {
    hipStream_t s = nullptr;
    e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);  // default priority
    if (e == hipSuccess) st->lanes.push_back(s);
  }
  if (e != hipSuccess) {
    bikv_stager_destroy(st);
    return fail_hip(e, "stager setup");
  }
  *out = st;
  return BIKV_OK;
}

extern "C" int bikv_stager_destroy(bikv_stager* st) {
  if (!st) return BIKV_OK;
  DeviceGuard guard_(st->device);
  for (hipStream_t s : st->lanes) {
    (void)hipStreamSynchronize(s);
    (void)hipStreamDestroy(s);
  }
  if (st->after) (void)hipEventDestroy(st->after);
  if (st->ring) (void)hipFree(st->ring);
  if (st->scale_ring) (void)hipFree(st->scale_ring);
  for (TraceOp& op : st->trace) {
    (void)hipEventDestroy(op.e0);
    (void)hipEventDestroy(op.e1);
  }
  release_bank(st->device, st->bank);
  delete st;
  return BIKV_OK;
}

namespace bikv {

// The lanes a pipeline call runs on: the stager's own, or (allocation-free entry point) the caller's
// stream with a buffer that already exists.
struct LaneSet {
  int n;
  hipStream_t* streams;
  char* buf;               // lane l uses buf + l*lane_bytes
  char* scale_buf;         // lane l uses scale_buf + l*scale_lane_bytes (null: pool has no scale class)
  int64_t lane_bytes, scale_lane_bytes, chunk_bytes;
  uint64_t* next_launch;
  int bank;
  // device -> host hop done by the library's copy kernel through these device views of the two pinned
  // images (null: hipMemcpyAsync)
  char* host_dev = nullptr;
  char* host_scale_dev = nullptr;
  // opt-in trace: steps are appended to *trace while it holds fewer than trace_cap
  std::vector<TraceOp>* trace = nullptr;
  int64_t trace_cap = 0;
};

enum : int { TRACE_KERNEL = 0, TRACE_COPY_D2H = 1, TRACE_COPY_H2D = 2, TRACE_COPY_KERNEL = 3 };

// Records the first event of a traced step on `s`; returns its index in the trace or -1 (not traced).
static int trace_begin(const LaneSet& L, int lane, int kind, int64_t bytes, hipStream_t s) {
  if (!L.trace || (int64_t)L.trace->size() >= L.trace_cap) return -1;
  TraceOp op;
  op.lane = lane;
  op.kind = kind;
  op.bytes = bytes;
  if (hipEventCreate(&op.e0) != hipSuccess) return -1;
  if (hipEventCreate(&op.e1) != hipSuccess) {
    (void)hipEventDestroy(op.e0);
    return -1;
  }
  (void)hipEventRecord(op.e0, s);
  L.trace->push_back(op);
  return (int)L.trace->size() - 1;
}
static void trace_end(const LaneSet& L, int idx, hipStream_t s) {
  if (idx >= 0) (void)hipEventRecord((*L.trace)[(size_t)idx].e1, s);
}

static int validate_stage_args(const bikv_pool* pool, const bikv_page_batch* batch, const int64_t* req_pages,
                               int64_t n_requests, int32_t layout, const void* host, int64_t host_bytes,
                               const void* host_scale, int64_t host_scale_bytes, int64_t* total_pages_out) {
  if (!pool || !batch || !req_pages || !host) return fail(BIKV_EINVAL, "null argument");
  const bool has_scale = pool->scale_tile_bytes > 0;
  if (has_scale && !host_scale)
    return fail(BIKV_EINVAL, "pool has a scale class: the host scale image must be given");
  if (layout != BIKV_LAYOUT_LAYER_MAJOR && layout != BIKV_LAYOUT_PAGE_MAJOR)
    return fail(BIKV_EINVAL, "unknown layout %d", layout);
  if (batch->plane_count > 0 && (batch->plane_begin != 0 || batch->plane_count != pool->n_planes))
    return fail(BIKV_EINVAL, "the host staging pipeline moves all planes");
  if (batch->slot_bias != 0) return fail(BIKV_EINVAL, "slot_bias must be 0");
  int64_t total_pages = 0;
  for (int64_t r = 0; r < n_requests; ++r) {
    if (req_pages[r] < 0) return fail(BIKV_EINVAL, "negative req_pages[%lld]", (long long)r);
    total_pages += req_pages[r];
  }
  if (total_pages != batch->n_pages)
    return fail(BIKV_EINVAL, "req_pages sums to %lld but the batch has %lld pages",
                (long long)total_pages, (long long)batch->n_pages);
  const int64_t image_bytes = total_pages * pool->n_planes * pool->tile_bytes;
  const int64_t scale_image_bytes = total_pages * pool->n_planes * pool->scale_tile_bytes;
  if (host_bytes < image_bytes)
    return fail(BIKV_ERANGE, "host buffer holds %lld bytes, staging image needs %lld",
                (long long)host_bytes, (long long)image_bytes);
  if (has_scale && host_scale_bytes < scale_image_bytes)
    return fail(BIKV_ERANGE, "host scale buffer holds %lld bytes, scale image needs %lld",
                (long long)host_scale_bytes, (long long)scale_image_bytes);
  *total_pages_out = total_pages;
  return BIKV_OK;
}

// Enqueues the pipelined transfer of a batch on `L` and returns without waiting. dir 0: pool -> lane
// buffer -> host image; dir 1: host image -> lane buffer -> pool. A lane's stream orders the steps of a
// launch and keeps its buffer safe from the lane's next launch.
static int issue_pipelined(int dir, const bikv_pool* pool, const bikv_page_batch* batch,
                           const int64_t* req_pages, int64_t n_requests, int32_t layout, char* host,
                           char* host_scale, const LaneSet& L, int64_t* n_copies) {
  const int64_t T = pool->tile_bytes, S = pool->scale_tile_bytes;
  const bool has_scale = S > 0;
  int64_t max_slots = L.lane_bytes / T;
  if (max_slots < 1)
    return fail(BIKV_ERANGE, "chunk_bytes %lld is smaller than one tile (%lld bytes)",
                (long long)L.lane_bytes, (long long)T);
  if (has_scale && max_slots * S > L.scale_lane_bytes) max_slots = L.scale_lane_bytes / S;
  if (max_slots < 1) return fail(BIKV_ERANGE, "the scale buffer of a lane is smaller than one scale tile");
  ChunkPlanner plan(req_pages, n_requests, pool->n_planes, layout, max_slots);
  Chunk ch;
  while (plan.next(&ch)) {
    const int lane = (int)(*L.next_launch % (uint64_t)L.n);
    ++*L.next_launch;
    hipStream_t stream = L.streams[lane];
    char* dev_chunk = L.buf + (int64_t)lane * L.lane_bytes;
    char* dev_scale = has_scale ? L.scale_buf + (int64_t)lane * L.scale_lane_bytes : nullptr;
    bikv_page_batch sub = *batch;
    sub.page_ids = batch->page_ids + ch.first_page;
    sub.slots = batch->slots + ch.first_page;
    sub.slot_strides = batch->slot_strides + ch.first_page;
    sub.n_pages = ch.n_pages;
    sub.plane_begin = ch.plane_begin;
    sub.plane_count = ch.plane_count;
    sub.slot_bias = ch.first_slot;
    const int64_t bytes = ch.n_slots * T;
    char* host_chunk = host + ch.first_slot * T;
    char* host_scale_chunk = has_scale ? host_scale + ch.first_slot * S : nullptr;
    if (dir == 0) {
      const int t = trace_begin(L, lane, TRACE_KERNEL, bytes, stream);
      const int rc = move_pages(L.bank, 0, pool, &sub, dev_chunk, bytes, dev_scale, ch.n_slots * S, stream);
      if (rc) return rc;
      trace_end(L, t, stream);
    }
    // the hop between lane buffer and pinned image: the library's copy kernel through the mapped image when
    // the call asked for it and both ends are 16-byte aligned, else one hipMemcpyAsync per chunk_bytes
    char* img_dev = L.host_dev ? L.host_dev + ch.first_slot * T : nullptr;
    const bool kernel_hop = img_dev && (((uint64_t)img_dev | (uint64_t)dev_chunk) & 15) == 0;
    if (kernel_hop) {
      // one launch moves the whole lane buffer: thousands of waves' accesses are in flight at once, and
      // no copy engine is involved
      const int t = trace_begin(L, lane, TRACE_COPY_KERNEL, bytes, stream);
      BIKV_HIP(dir == 0 ? launch_linear_copy(dev_chunk, img_dev, bytes, stream)
                        : launch_linear_copy(img_dev, dev_chunk, bytes, stream));
      trace_end(L, t, stream);
      ++*n_copies;
    } else {
      for (int64_t off = 0; off < bytes; off += L.chunk_bytes) {
        const int64_t n = bytes - off < L.chunk_bytes ? bytes - off : L.chunk_bytes;
        const int t = trace_begin(L, lane, dir == 0 ? TRACE_COPY_D2H : TRACE_COPY_H2D, n, stream);
        BIKV_HIP(dir == 0 ? hipMemcpyAsync(host_chunk + off, dev_chunk + off, (size_t)n, hipMemcpyDeviceToHost, stream)
                          : hipMemcpyAsync(dev_chunk + off, host_chunk + off, (size_t)n, hipMemcpyHostToDevice, stream));
        trace_end(L, t, stream);
        ++*n_copies;
      }
    }
    if (has_scale) {
      const int64_t sb = ch.n_slots * S;
      char* simg_dev = L.host_scale_dev ? L.host_scale_dev + ch.first_slot * S : nullptr;
      if (kernel_hop && simg_dev && (((uint64_t)simg_dev | (uint64_t)dev_scale) & 15) == 0)
        BIKV_HIP(dir == 0 ? launch_linear_copy(dev_scale, simg_dev, sb, stream)
                          : launch_linear_copy(simg_dev, dev_scale, sb, stream));
      else
        BIKV_HIP(dir == 0 ? hipMemcpyAsync(host_scale_chunk, dev_scale, (size_t)sb, hipMemcpyDeviceToHost, stream)
                          : hipMemcpyAsync(dev_scale, host_scale_chunk, (size_t)sb, hipMemcpyHostToDevice, stream));
    }
    if (dir == 1) {
      const int t = trace_begin(L, lane, TRACE_KERNEL, bytes, stream);
      const int rc = move_pages(L.bank, 1, pool, &sub, dev_chunk, bytes, dev_scale, ch.n_slots * S, stream);
      if (rc) return rc;
      trace_end(L, t, stream);
    }
  }
  return BIKV_OK;
}

}  // namespace bikv

extern "C" int64_t bikv_plan_chunks(const int64_t* req_pages, int64_t n_requests, int32_t n_planes,
                                    int32_t layout, int64_t max_slots, int64_t* out, int64_t cap) {
  if (!req_pages || n_requests < 0 || n_planes <= 0 || max_slots < 1 || (cap > 0 && !out))
    return fail(BIKV_EINVAL, "bad plan_chunks arguments");
  if (layout != BIKV_LAYOUT_LAYER_MAJOR && layout != BIKV_LAYOUT_PAGE_MAJOR)
    return fail(BIKV_EINVAL, "unknown layout %d", layout);
  for (int64_t r = 0; r < n_requests; ++r)
    if (req_pages[r] < 0) return fail(BIKV_EINVAL, "negative req_pages[%lld]", (long long)r);
  ChunkPlanner plan(req_pages, n_requests, n_planes, layout, max_slots);
  Chunk ch;
  int64_t c = 0;
  for (; plan.next(&ch); ++c) {
    if (c >= cap) continue;
    int64_t* o = out + 6 * c;
    o[0] = ch.first_page; o[1] = ch.n_pages;
    o[2] = ch.plane_begin; o[3] = ch.plane_count;
    o[4] = ch.first_slot; o[5] = ch.n_slots;
  }
  return c;
}

static void drain_lanes(bikv_stager* st) {
  for (hipStream_t s : st->lanes) (void)hipStreamSynchronize(s);
}

// Both directions of the host staging pipeline, enqueue only.
static int stage_issue(int dir, bikv_stager* st, const bikv_pool* pool, const bikv_page_batch* batch,
                       const int64_t* req_pages, int64_t n_requests, int32_t layout, void* host,
                       int64_t host_bytes, void* host_scale, int64_t host_scale_bytes, int32_t mode,
                       void* after_stream) {
  if (!st) return fail(BIKV_EINVAL, "null argument");
  int64_t total_pages = 0;
  int rc = validate_stage_args(pool, batch, req_pages, n_requests, layout, host, host_bytes, host_scale,
                               host_scale_bytes, &total_pages);
  if (rc) return rc;
  if (pool->device != st->device) return fail(BIKV_EINVAL, "pool and stager are on different devices");
  if (mode == BIKV_STAGE_AUTO) mode = BIKV_STAGE_DIRECT;
  if (mode != BIKV_STAGE_DIRECT && mode != BIKV_STAGE_PIPELINED && mode != BIKV_STAGE_PIPELINED_KERNEL)
    return fail(BIKV_EINVAL, "unknown staging mode %d", mode);
  if (total_pages == 0) return BIKV_OK;
  const bool has_scale = pool->scale_tile_bytes > 0;
  const int64_t T = pool->tile_bytes, S = pool->scale_tile_bytes;
  const int64_t image_bytes = total_pages * pool->n_planes * T;
  const int64_t scale_image_bytes = total_pages * pool->n_planes * S;
  BIKV_DEVICE(st->device);
  if (dir == 1) {
    rc = check_unique_on_device(st->device, batch->page_ids, batch->n_pages, static_cast<hipStream_t>(after_stream));
    if (rc) return rc;
  }
  if (!st->timing) {
    st->timing = true;
    st->t_first = std::chrono::steady_clock::now();
  }
  const int n_lanes_used = mode == BIKV_STAGE_DIRECT ? 1 : st->n_buf;
  if (after_stream) {
    // the caller's stream may still be uploading the index arrays: the lanes start behind it
    BIKV_HIP(hipEventRecord(st->after, static_cast<hipStream_t>(after_stream)));
    for (int l = 0; l < n_lanes_used; ++l) {
      const int lane = (int)((st->next_launch + (uint64_t)l) % (uint64_t)st->n_buf);
      BIKV_HIP(hipStreamWaitEvent(st->lanes[lane], st->after, 0));
    }
  }
  int64_t copies = 0;
  if (mode == BIKV_STAGE_DIRECT) {
    void* dptr = nullptr;
    void* sptr = nullptr;
    BIKV_HIP(hipHostGetDevicePointer(&dptr, host, 0));
    if (has_scale) BIKV_HIP(hipHostGetDevicePointer(&sptr, host_scale, 0));
    const int lane = (int)(st->next_launch++ % (uint64_t)st->n_buf);
    LaneSet T0;                       // only the trace fields are used
    T0.trace = st->trace_cap > 0 ? &st->trace : nullptr;
    T0.trace_cap = st->trace_cap;
    const int t = trace_begin(T0, lane, TRACE_KERNEL, image_bytes, st->lanes[lane]);
    rc = move_pages(st->bank, dir, pool, batch, dptr, image_bytes, sptr, scale_image_bytes, st->lanes[lane]);
    if (rc) return rc;
    trace_end(T0, t, st->lanes[lane]);
  } else {
    // the scale tiles of a launch ride in a second, much smaller buffer per lane
    const int64_t max_slots = st->lane_bytes / T;
    const int64_t scale_lane = has_scale ? ((max_slots * S + 255) & ~int64_t(255)) : 0;
    if (scale_lane * st->n_buf > st->scale_ring_bytes) {
      drain_lanes(st);
      if (st->scale_ring) BIKV_HIP(hipFree(st->scale_ring));
      st->scale_ring = nullptr;
      st->scale_ring_bytes = 0;
      BIKV_HIP(hipMalloc((void**)&st->scale_ring, (size_t)(scale_lane * st->n_buf)));
      st->scale_ring_bytes = scale_lane * st->n_buf;
    }
    LaneSet L;
    L.n = st->n_buf;
    L.streams = st->lanes.data();
    L.buf = st->ring;
    L.scale_buf = has_scale ? st->scale_ring : nullptr;
    L.lane_bytes = st->lane_bytes;
    L.scale_lane_bytes = has_scale ? st->scale_ring_bytes / st->n_buf : 0;
    L.chunk_bytes = st->chunk_bytes;
    L.next_launch = &st->next_launch;
    L.bank = st->bank;
    L.trace = st->trace_cap > 0 ? &st->trace : nullptr;
    L.trace_cap = st->trace_cap;
    if (mode == BIKV_STAGE_PIPELINED_KERNEL) {
      void* dptr = nullptr;
      BIKV_HIP(hipHostGetDevicePointer(&dptr, host, 0));
      L.host_dev = static_cast<char*>(dptr);
      if (has_scale) {
        BIKV_HIP(hipHostGetDevicePointer(&dptr, host_scale, 0));
        L.host_scale_dev = static_cast<char*>(dptr);
      }
    }
    rc = issue_pipelined(dir, pool, batch, req_pages, n_requests, layout, static_cast<char*>(host),
                         static_cast<char*>(host_scale), L, &copies);
    if (rc) {
      drain_lanes(st);   // nothing is left in flight on an error path
      return rc;
    }
  }
  st->pending_bytes += image_bytes + scale_image_bytes;
  st->pending_copies += mode == BIKV_STAGE_DIRECT ? 1 : copies;
  return BIKV_OK;
}

extern "C" int bikv_stager_wait(bikv_stager* st, bikv_stage_stats* stats) {
  if (!st) return fail(BIKV_EINVAL, "null argument");
  BIKV_DEVICE(st->device);
  hipError_t es = hipSuccess;
  for (hipStream_t s : st->lanes) {
    const hipError_t e1 = hipStreamSynchronize(s);
    if (e1 != hipSuccess) es = e1;
  }
  const auto t1 = std::chrono::steady_clock::now();
  if (stats) {
    stats->bytes = st->pending_bytes;
    stats->n_chunks = st->pending_copies;
    stats->wall_seconds = st->timing ? std::chrono::duration<double>(t1 - st->t_first).count() : 0.0;
  }
  st->pending_bytes = st->pending_copies = 0;
  st->timing = false;
  if (es != hipSuccess) return fail_hip(es, "hipStreamSynchronize(lane)");
  return check_bank(st->device, st->bank);
}

// Opt-in trace of a stager's lanes: while it is on, every kernel launch and host copy the stager enqueues is
// bracketed by two timing events on its lane, up to `max_steps` steps (0 switches it off and drops what was
// recorded). bikv_stager_trace_read, after bikv_stager_wait, turns the events into start / end times in
// milliseconds relative to the first recorded step.
extern "C" int bikv_stager_trace(bikv_stager* st, int64_t max_steps) {
  if (!st || max_steps < 0 || max_steps > (int64_t(1) << 20)) return fail(BIKV_EINVAL, "bad stager_trace arguments");
  BIKV_DEVICE(st->device);
  drain_lanes(st);
  for (TraceOp& op : st->trace) {
    (void)hipEventDestroy(op.e0);
    (void)hipEventDestroy(op.e1);
  }
  st->trace.clear();
  st->trace_cap = max_steps;
  if (max_steps > 0) st->trace.reserve((size_t)max_steps);
  return BIKV_OK;
}

extern "C" int64_t bikv_stager_trace_read(bikv_stager* st, bikv_trace_step* out, int64_t cap) {
  if (!st || cap < 0 || (cap > 0 && !out)) return fail(BIKV_EINVAL, "bad stager_trace_read arguments");
  if (st->trace.empty()) return 0;
  BIKV_DEVICE(st->device);
  drain_lanes(st);
  const hipEvent_t base = st->trace[0].e0;
  int64_t n = 0;
  for (const TraceOp& op : st->trace) {
    if (n >= cap) break;
    float a = -1.0f, b = -1.0f;
    // a step whose launch failed has no second event: it is reported with end_ms = -1
    if (hipEventElapsedTime(&a, base, op.e0) != hipSuccess) { a = -1.0f; (void)hipGetLastError(); }
    if (hipEventElapsedTime(&b, base, op.e1) != hipSuccess) { b = -1.0f; (void)hipGetLastError(); }
    out[n].lane = op.lane;
    out[n].kind = op.kind;
    out[n].bytes = op.bytes;
    out[n].start_ms = a;
    out[n].end_ms = b;
    ++n;
  }
  return (int64_t)st->trace.size();
}

extern "C" int bikv_gather_to_host_async(bikv_stager* st, const bikv_pool* pool, const bikv_page_batch* batch,
                                         const int64_t* req_pages, int64_t n_requests, int32_t layout,
                                         void* host_dst, int64_t host_bytes, void* host_scale_dst,
                                         int64_t host_scale_bytes, int32_t mode, void* after_stream) {
  return stage_issue(0, st, pool, batch, req_pages, n_requests, layout, host_dst, host_bytes, host_scale_dst,
                     host_scale_bytes, mode, after_stream);
}

extern "C" int bikv_scatter_from_host_async(bikv_stager* st, const bikv_pool* pool, const bikv_page_batch* batch,
                                            const int64_t* req_pages, int64_t n_requests, int32_t layout,
                                            const void* host_src, int64_t host_bytes,
                                            const void* host_scale_src, int64_t host_scale_bytes,
                                            int32_t mode, void* after_stream) {
  return stage_issue(1, st, pool, batch, req_pages, n_requests, layout, const_cast<void*>(host_src), host_bytes,
                     const_cast<void*>(host_scale_src), host_scale_bytes, mode, after_stream);
}

// The synchronous forms: whatever earlier asynchronous calls left in flight is awaited first, so that the
// statistics and the status cover this call alone.
static int stage_sync(int dir, bikv_stager* st, const bikv_pool* pool, const bikv_page_batch* batch,
                      const int64_t* req_pages, int64_t n_requests, int32_t layout, void* host,
                      int64_t host_bytes, void* host_scale, int64_t host_scale_bytes, int32_t mode,
                      bikv_stage_stats* stats) {
  if (!st) return fail(BIKV_EINVAL, "null argument");
  if (stats) { stats->bytes = 0; stats->n_chunks = 0; stats->wall_seconds = 0.0; }
  if (st->timing) {
    const int rc0 = bikv_stager_wait(st, nullptr);
    if (rc0) return rc0;
  }
  int rc = stage_issue(dir, st, pool, batch, req_pages, n_requests, layout, host, host_bytes, host_scale,
                       host_scale_bytes, mode, nullptr);
  if (rc) return rc;
  return bikv_stager_wait(st, stats);
}

extern "C" int bikv_gather_to_host(bikv_stager* st, const bikv_pool* pool,
                                   const bikv_page_batch* batch, const int64_t* req_pages,
                                   int64_t n_requests, int32_t layout, void* host_dst,
                                   int64_t host_bytes, void* host_scale_dst,
                                   int64_t host_scale_bytes, int32_t mode,
                                   bikv_stage_stats* stats) {
  return stage_sync(0, st, pool, batch, req_pages, n_requests, layout, host_dst, host_bytes,
                    host_scale_dst, host_scale_bytes, mode, stats);
}

extern "C" int bikv_scatter_from_host(bikv_stager* st, const bikv_pool* pool,
                                      const bikv_page_batch* batch, const int64_t* req_pages,
                                      int64_t n_requests, int32_t layout, const void* host_src,
                                      int64_t host_bytes, const void* host_scale_src,
                                      int64_t host_scale_bytes, int32_t mode,
                                      bikv_stage_stats* stats) {
  return stage_sync(1, st, pool, batch, req_pages, n_requests, layout,
                    const_cast<void*>(host_src), host_bytes,
                    const_cast<void*>(host_scale_src), host_scale_bytes, mode, stats);
}

// The allocation-free form of bikv_gather_to_host: the lane pipeline on ONE lane — the caller's stream —
// whose buffer is this device's `scratch` array, with the library's copy kernel as the hop to the host
// (BIKV_STAGE_PIPELINED_KERNEL's shape). Enqueue only. Nothing here allocates or frees: the
// device context (status block, scratch address) was set up by bikv_init / bikv_pool_create, the planner
// is an iterator, errors go to a thread-local buffer.
extern "C" int bikv_gather_to_host_noalloc(const bikv_pool* pool, const bikv_page_batch* batch,
                                           const int64_t* req_pages, int64_t n_requests, int32_t layout,
                                           void* host_dst, int64_t host_bytes, void* host_scale_dst,
                                           int64_t host_scale_bytes, void* stream) {
  int64_t total_pages = 0;
  int rc = validate_stage_args(pool, batch, req_pages, n_requests, layout, host_dst, host_bytes,
                               host_scale_dst, host_scale_bytes, &total_pages);
  if (rc) return rc;
  if (pool->tile_bytes > kScratchPayload)
    return fail(BIKV_ERANGE, "tile of %lld bytes exceeds the %lld-byte scratch of the allocation-free entry point",
                (long long)pool->tile_bytes, (long long)kScratchPayload);
  if (pool->scale_tile_bytes > kScratchScale)
    return fail(BIKV_ERANGE, "scale tile of %lld bytes exceeds the %lld-byte scale scratch of the allocation-free entry point",
                (long long)pool->scale_tile_bytes, (long long)kScratchScale);
  char* base = scratch_of(pool->device);
  if (!base) return fail(BIKV_ESTATE, "device %d is not set up (bikv_init)", pool->device);
  if (total_pages == 0) return BIKV_OK;
  BIKV_DEVICE(pool->device);
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint64_t launches = 0;
  int64_t copies = 0;
  LaneSet L;
  L.n = 1;
  L.streams = &s;
  L.buf = base;
  L.scale_buf = pool->scale_tile_bytes > 0 ? base + kScratchPayload : nullptr;
  L.lane_bytes = kScratchPayload;
  L.scale_lane_bytes = pool->scale_tile_bytes > 0 ? kScratchScale : 0;
  L.chunk_bytes = kScratchCopy;
  L.next_launch = &launches;
  L.bank = ST_BANK_SHARED;
  // the hop to the host is the library's copy kernel storing through the mapped image: kernels only, so the
  // call can be captured into a HIP graph, and no copy engine is involved
  void* dptr = nullptr;
  BIKV_HIP(hipHostGetDevicePointer(&dptr, host_dst, 0));
  L.host_dev = static_cast<char*>(dptr);
  if (pool->scale_tile_bytes > 0) {
    BIKV_HIP(hipHostGetDevicePointer(&dptr, host_scale_dst, 0));
    L.host_scale_dev = static_cast<char*>(dptr);
  }
  return issue_pipelined(0, pool, batch, req_pages, n_requests, layout, static_cast<char*>(host_dst),
                         static_cast<char*>(host_scale_dst), L, &copies);
}

// ---- per-layer paged NHD pool and the fused layout change ------------------------------------
struct bikv_nhd {
  int device;
  int n_layers, kv_heads, head_dim, block_tokens, elem_bytes;
  int64_t n_blocks;
  int64_t block_stride, kv_stride, token_stride;   // elements
  const char** d_layer_base;
};

extern "C" int bikv_nhd_create(const bikv_nhd_desc* d, bikv_nhd** out) {
  if (!d || !out) return fail(BIKV_EINVAL, "null argument");
  *out = nullptr;
  if (d->n_layers <= 0 || d->n_layers > 65536 || d->kv_heads <= 0 || d->head_dim <= 0 ||
      d->block_tokens <= 0 || d->n_blocks <= 0)
    return fail(BIKV_EINVAL, "layers, kv_heads, head_dim, block_tokens and n_blocks must be positive");
  if (d->elem_bytes != 1 && d->elem_bytes != 2 && d->elem_bytes != 4)
    return fail(BIKV_EINVAL, "elem_bytes must be 1, 2 or 4");
  const int ve = 16 / d->elem_bytes;
  const int64_t cols = (int64_t)d->kv_heads * d->n_layers * 2;
  if (d->head_dim % ve != 0 || cols % ve != 0)
    return fail(BIKV_EINVAL, "head_dim (%d) and kv_heads*layers*2 (%lld) must be multiples of %d elements (16 bytes)",
                d->head_dim, (long long)cols, ve);
  if (cols >= (int64_t(1) << 24) || (int64_t)d->head_dim * (ve + 4 / d->elem_bytes) * d->elem_bytes > 48 * 1024)
    return fail(BIKV_EINVAL, "token shape too large for the layout-change kernel");
  if (!d->layer_base) return fail(BIKV_EINVAL, "layer_base is null");
  if (d->kv_stride_elems < 0 || d->token_stride_elems < d->kv_heads * (int64_t)d->head_dim ||
      d->block_stride_elems < (int64_t)d->block_tokens * 2 * d->kv_heads * d->head_dim)
    return fail(BIKV_EINVAL, "strides are smaller than the data they separate");
  std::vector<const char*> table((size_t)d->n_layers);
  for (int l = 0; l < d->n_layers; ++l) {
    if (!d->layer_base[l]) return fail(BIKV_EINVAL, "layer_base[%d] is null", l);
    if (((uint64_t)d->layer_base[l]) & 15) return fail(BIKV_EINVAL, "layer_base[%d] is not 16-byte aligned", l);
    table[l] = static_cast<const char*>(d->layer_base[l]);
  }
  if (((d->block_stride_elems | d->kv_stride_elems | d->token_stride_elems) * d->elem_bytes) & 15)
    return fail(BIKV_EINVAL, "strides must be multiples of 16 bytes");
  uint32_t* st = nullptr;
  int rc = device_status(d->device, ST_BANK_SHARED, &st);
  if (rc) return rc;
  BIKV_DEVICE(d->device);
  void* dtab = nullptr;
  BIKV_HIP(hipMalloc(&dtab, table.size() * sizeof(char*)));
  hipError_t e = hipMemcpy(dtab, table.data(), table.size() * sizeof(char*), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(dtab);
    return fail_hip(e, "hipMemcpy(layer table)");
  }
  bikv_nhd* p = new bikv_nhd();
  p->device = d->device;
  p->n_layers = d->n_layers;
  p->kv_heads = d->kv_heads;
  p->head_dim = d->head_dim;
  p->block_tokens = d->block_tokens;
  p->elem_bytes = d->elem_bytes;
  p->n_blocks = d->n_blocks;
  p->block_stride = d->block_stride_elems;
  p->kv_stride = d->kv_stride_elems;
  p->token_stride = d->token_stride_elems;
  p->d_layer_base = static_cast<const char**>(dtab);
  *out = p;
  return BIKV_OK;
}

extern "C" int bikv_nhd_destroy(bikv_nhd* p) {
  if (!p) return BIKV_OK;
  DeviceGuard guard_(p->device);
  hipError_t e = hipFree((void*)p->d_layer_base);
  delete p;
  if (e != hipSuccess) return fail_hip(e, "hipFree(layer table)");
  return BIKV_OK;
}

static int transpose_pages(int dir, const bikv_nhd* nhd, void* tm, int64_t tm_bytes,
                           const int64_t* block_ids, const int64_t* tm_pages, int64_t n_pages,
                           void* stream) {
  if (!nhd) return fail(BIKV_EINVAL, "null pool");
  if (n_pages < 0) return fail(BIKV_EINVAL, "negative n_pages");
  if (n_pages == 0) return BIKV_OK;
  if (!tm || !block_ids || !tm_pages) return fail(BIKV_EINVAL, "null pointer argument");
  if (((uint64_t)tm) & 15) return fail(BIKV_EINVAL, "token-major buffer is not 16-byte aligned");
  const int64_t cols = (int64_t)nhd->kv_heads * nhd->n_layers * 2;
  const int64_t page_bytes = (int64_t)nhd->block_tokens * nhd->head_dim * cols * nhd->elem_bytes;
  if (tm_bytes < page_bytes) return fail(BIKV_EINVAL, "token-major buffer is smaller than one page");
  TransposeArgs a;
  memset(&a, 0, sizeof(a));
  a.layer_base = nhd->d_layer_base;
  a.tm_base = static_cast<char*>(tm);
  a.block_ids = block_ids;
  a.tm_pages = tm_pages;
  a.n_pages = n_pages;
  a.n_blocks = nhd->n_blocks;
  a.n_tm_pages = tm_bytes / page_bytes;
  a.block_stride = nhd->block_stride;
  a.kv_stride = nhd->kv_stride;
  a.token_stride = nhd->token_stride;
  a.n_layers = nhd->n_layers;
  a.head_dim = nhd->head_dim;
  a.n_cols = (int32_t)cols;
  a.block_tokens = nhd->block_tokens;
  a.elem_bytes = nhd->elem_bytes;
  int rc = device_status(nhd->device, ST_BANK_SHARED, &a.status);
  if (rc) return rc;
  BIKV_DEVICE(nhd->device);
  hipError_t e = launch_transpose_pages(dir, a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail_hip(e, "layout-change launch");
  return BIKV_OK;
}

extern "C" int bikv_nhd_store_token_major(const bikv_nhd* nhd, void* tm, int64_t tm_bytes,
                                          const int64_t* block_ids, const int64_t* tm_pages,
                                          int64_t n_pages, void* stream) {
  return transpose_pages(0, nhd, tm, tm_bytes, block_ids, tm_pages, n_pages, stream);
}

extern "C" int bikv_nhd_load_token_major(const bikv_nhd* nhd, const void* tm, int64_t tm_bytes,
                                         const int64_t* block_ids, const int64_t* tm_pages,
                                         int64_t n_pages, void* stream) {
  if (nhd) {
    const int rc = check_unique_on_device(nhd->device, block_ids, n_pages, static_cast<hipStream_t>(stream));
    if (rc) return rc;
  }
  return transpose_pages(1, nhd, const_cast<void*>(tm), tm_bytes, block_ids, tm_pages, n_pages, stream);
}
