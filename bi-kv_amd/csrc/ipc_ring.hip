// Producer/consumer ring of the `ipc_service` operator: a control block in POSIX shared memory,
// a device ring buffer owned by the consumer, and the producer-side bookkeeping that follows every
// copy. Behaviour follows Bi-KV/SharedMemory/CUDA_Shared/ipc_service.cpp:20-202 (init, send,
// receive, cleanup) and copy_kernel.cu:84-89,115-128 (ring advance and shape publishing).
//
// Deliberate differences from the reference, all on error paths or internal:
//   - sizes are 64-bit and use the real element size (reference: int, sizeof(half));
//   - a batch larger than the whole ring is refused (reference: wraps to 0 and overruns);
//   - the copy is awaited with a stream synchronise (reference: cudaDeviceSynchronize);
//   - a producer in the consumer's own process uses the consumer's pointer instead of opening an
//     IPC handle (a process cannot open its own handle);
//   - consumer_receive can time out.
#include "../../include/bikv_pagecopy.h"
#include "host_logic/ring_logic.h"
#include "pagecopy_internal.h"
#include "pagecopy_kernels.h"

#include <cerrno>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <shared_mutex>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

using namespace bikv;

static_assert(sizeof(sem_t) == 32, "sem_t is 32 bytes on x86-64 glibc; SharedControl depends on it");
static_assert(sizeof(hipIpcMemHandle_t) <= BIKV_IPC_HANDLE_SIZE, "IPC handle must fit the control block");

namespace {

// What a role has mapped: the control block and the ring.
struct Role {
  int fd = -1;
  bikv_shared_control* ctrl = nullptr;
  void* mem = nullptr;
  int device = 0;
  bool ipc_mapped = false;  // producer only: mem came from hipIpcOpenMemHandle
  char shm_name[256] = "";
};

// One producer role and one consumer role per process, as in the reference (ipc_service.cpp:9-17), whose
// callers are gRPC thread pools: every entry point takes its role's lock, so concurrent callers are
// serialised instead of interleaving their bookkeeping.
//   g_prod.mu (inside ring::Producer)  held for the whole of a producer call, GPU copy included: the
//                                      ring's write offset only moves at publication
//   g_cons_mu                          exclusive for init / cleanup, shared for receive / release (a
//                                      receive blocked on the semaphore must not keep the release that
//                                      a producer under back-pressure is waiting for from running)
// Where both are needed (a producer attaching to the ring of a consumer in its own process, a consumer
// retiring such a producer) the consumer's lock is taken first.
Role g_producer, g_consumer;
ring::Producer g_prod;
std::shared_mutex g_cons_mu;

// Rings of this many bytes or more are neither exported nor mapped across processes.
constexpr size_t kMaxIpcBytes = size_t(2) << 30;

// Between bikv_producer_reserve and bikv_producer_publish the ring's write offset belongs to the
// reservation: any other producer call would be handed the same window.
const char kReservedMsg[] = "a reserved ring window is waiting for bikv_producer_publish (or bikv_producer_cancel)";

using ring::sem_of;

void unmap_role(Role& r) {
  if (r.ctrl) {
    munmap(r.ctrl, sizeof(bikv_shared_control));
    r.ctrl = nullptr;
  }
  if (r.fd != -1) {
    close(r.fd);
    r.fd = -1;
  }
}

// ring::reserve_window with the producer's messages (caller holds g_prod.mu)
int producer_reserve(size_t data_size, size_t* at_out) {
  const int rc = ring::reserve_window(g_prod, data_size, at_out);
  if (rc == ring::WAIT_TIMEOUT)
    return fail(BIKV_ESTATE, "producer timed out after %lld ms waiting for the consumer to release the ring space it needs",
                (long long)g_prod.bp_timeout_ms);
  if (rc == ring::WAIT_ERROR) return fail(BIKV_ESYS, "sem_wait(sem_complete) failed: %s", strerror(errno));
  return BIKV_OK;
}

int producer_wait_slot() {
  const int rc = ring::wait_slot(g_prod);
  if (rc == ring::WAIT_TIMEOUT)
    return fail(BIKV_ESTATE, "producer timed out after %lld ms waiting for the consumer to release the previous transfer",
                (long long)g_prod.bp_timeout_ms);
  if (rc == ring::WAIT_ERROR) return fail(BIKV_ESYS, "sem_wait(sem_complete) failed: %s", strerror(errno));
  return BIKV_OK;
}

void producer_cleanup_locked() {
  if (g_producer.mem && g_producer.ipc_mapped) (void)hipIpcCloseMemHandle(g_producer.mem);
  g_producer.mem = nullptr;
  unmap_role(g_producer);
  g_producer = Role();
  g_prod.ctrl = nullptr;
  g_prod.backpressure = false;
  g_prod.bp_timeout_ms = -1;
  g_prod.in_flight.clear();
  g_prod.reserved = false;
}

}  // namespace

// Maps the named control block into this process: `create` makes a fresh object of the block's size
// (replacing a stale one of the same name, exclusive, mode 0666 as ipc_service.cpp:33-35 does), otherwise an
// existing object is opened and must be at least that large. On failure nothing is left open, and a
// created object is removed again.
static int map_control(const char* name, bool create, const char* who, Role* r) {
  if (create) shm_unlink(name);
  r->fd = shm_open(name, create ? (O_CREAT | O_RDWR | O_EXCL) : O_RDWR, 0666);
  if (r->fd == -1) return fail(BIKV_ESYS, "%s shm_open failed: %s", who, strerror(errno));
  const char* what = nullptr;
  int err = 0;
  if (create) {
    if (ftruncate(r->fd, sizeof(bikv_shared_control)) == -1) what = "ftruncate", err = errno;
  } else {
    struct stat sb;
    if (fstat(r->fd, &sb) == -1 || (size_t)sb.st_size < sizeof(bikv_shared_control)) {
      close(r->fd);
      r->fd = -1;
      return fail(BIKV_ESYS, "%s: shared object is smaller than the control block", who);
    }
  }
  if (!what) {
    void* m = mmap(nullptr, sizeof(bikv_shared_control), PROT_READ | PROT_WRITE, MAP_SHARED, r->fd, 0);
    if (m == MAP_FAILED) what = "mmap", err = errno;
    else r->ctrl = static_cast<bikv_shared_control*>(m);
  }
  if (what) {
    close(r->fd);
    r->fd = -1;
    if (create) shm_unlink(name);
    return fail(BIKV_ESYS, "%s %s failed: %s", who, what, strerror(err));
  }
  return BIKV_OK;
}

// The consumer owns the ring: device memory first, then the control block that describes it. The block is
// filled from a local image with its ring size stored last (ring::describe_ring), so a producer that opens
// it early sees either "no ring yet" (refused) or the finished description, never half of one.
extern "C" int bikv_consumer_init(int device, const char* shm_name, size_t buffer_bytes) {
  if (!shm_name || !*shm_name) return fail(BIKV_EINVAL, "shm_name is empty");
  if (strlen(shm_name) >= sizeof(g_consumer.shm_name)) return fail(BIKV_EINVAL, "shm_name too long");
  if (buffer_bytes == 0) return fail(BIKV_EINVAL, "buffer_size must be positive");
  std::unique_lock<std::shared_mutex> lk(g_cons_mu);
  if (g_consumer.ctrl) return fail(BIKV_ESTATE, "consumer already initialised (call consumer_cleanup first)");
  BIKV_HIP(hipSetDevice(device));
  Role r;
  r.device = device;
  strncpy(r.shm_name, shm_name, sizeof(r.shm_name) - 1);

  bikv_shared_control image;
  memset(&image, 0, sizeof(image));
  image.device_id = device;
  image.buffer_size = buffer_bytes;
  gethostname(image.hostname, sizeof(image.hostname));
  hipError_t e = hipMalloc(&r.mem, buffer_bytes);
  if (e != hipSuccess) return fail(BIKV_EHIP, "consumer_init hipMalloc failed: %s", hipGetErrorString(e));
  // A ring of 2 GiB or more is never exported: IPC mappings that large have been seen not to return
  // on some ROCm hosts. Its handle stays zeroed, a producer in another process is refused
  // (bikv_producer_init), and a producer in this process uses the pointer directly.
  if (buffer_bytes < kMaxIpcBytes) {
    static_assert(sizeof(hipIpcMemHandle_t) <= sizeof(image.ipc_handle), "IPC handle does not fit the control block");
    hipIpcMemHandle_t handle;
    memset(&handle, 0, sizeof(handle));
    e = hipIpcGetMemHandle(&handle, r.mem);
    if (e != hipSuccess) {
      (void)hipFree(r.mem);
      return fail(BIKV_EHIP, "consumer_init hipIpcGetMemHandle failed: %s", hipGetErrorString(e));
    }
    memcpy(image.ipc_handle, &handle, sizeof(handle));
  }
  const int rc = map_control(shm_name, true, "consumer_init", &r);
  if (rc != BIKV_OK) {
    (void)hipFree(r.mem);
    return rc;
  }
  ring::describe_ring(r.ctrl, image);
  g_consumer = r;
  return BIKV_OK;
}

// The producer attaches to a ring some consumer described: the control block is opened and checked before
// the GPU is touched, so that a missing object or a foreign host is reported as such whatever the state of
// the device.
extern "C" int bikv_producer_init(int device, const char* shm_name) {
  if (!shm_name || !*shm_name) return fail(BIKV_EINVAL, "shm_name is empty");
  std::shared_lock<std::shared_mutex> lkc(g_cons_mu);     // the consumer of this process, if any, stays put
  std::lock_guard<std::mutex> lk(g_prod.mu);
  if (g_producer.ctrl) return fail(BIKV_ESTATE, "producer already initialised (call producer_cleanup first)");
  Role r;
  r.device = device;
  strncpy(r.shm_name, shm_name, sizeof(r.shm_name) - 1);
  int rc = map_control(shm_name, false, "producer_init", &r);
  if (rc != BIKV_OK) return rc;
  const bool same_process = g_consumer.ctrl && strcmp(g_consumer.shm_name, shm_name) == 0;
  const size_t ring_bytes = ring::describes_ring(r.ctrl);   // acquire: what follows it in the block is complete
  char host[sizeof(r.ctrl->hostname)];
  memset(host, 0, sizeof(host));
  gethostname(host, sizeof(host));
  const bool foreign = strncmp(host, r.ctrl->hostname, sizeof(host)) != 0;
  if (ring_bytes == 0 && (r.ctrl->hostname[0] == '\0' || !foreign))
    rc = fail(BIKV_ESTATE, "producer_init: the control block describes no ring yet (the consumer is still initialising)");
  else if (foreign)
    rc = fail(BIKV_ESTATE, "Processes must run on the same host");
  else if (!same_process && ring_bytes >= kMaxIpcBytes)
    // Mapping another process's allocation of 2 GiB or more has been seen not to return on some ROCm
    // hosts; the consumer does not export a handle for such a ring and it is refused here.
    rc = fail(BIKV_ERANGE, "the consumer's ring is %zu bytes: IPC mappings of 2 GiB or more are refused "
                           "(use a ring below 2 GiB, or run producer and consumer in one process)", ring_bytes);
  if (rc == BIKV_OK) {
    const hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) rc = fail_hip(e, "hipSetDevice");
  }
  if (rc == BIKV_OK) {
    if (same_process) {
      r.mem = g_consumer.mem;  // same process: no IPC mapping needed (or possible)
      r.ipc_mapped = false;
    } else {
      hipIpcMemHandle_t handle;
      memcpy(&handle, r.ctrl->ipc_handle, sizeof(handle));
      const hipError_t e = hipIpcOpenMemHandle(&r.mem, handle, hipIpcMemLazyEnablePeerAccess);
      if (e != hipSuccess) rc = fail(BIKV_EHIP, "producer_init hipIpcOpenMemHandle failed: %s", hipGetErrorString(e));
      r.ipc_mapped = e == hipSuccess;
    }
  }
  if (rc != BIKV_OK) {
    unmap_role(r);
    return rc;
  }
  g_producer = r;
  g_prod.ctrl = r.ctrl;
  return BIKV_OK;
}

extern "C" void bikv_producer_cleanup(void) {
  std::lock_guard<std::mutex> lk(g_prod.mu);
  producer_cleanup_locked();
}

extern "C" void bikv_consumer_cleanup(void) {
  std::unique_lock<std::shared_mutex> lkc(g_cons_mu);
  {
    std::lock_guard<std::mutex> lk(g_prod.mu);
    // a same-process producer borrows the consumer's buffer: retire it first
    if (g_producer.ctrl && !g_producer.ipc_mapped && g_producer.mem == g_consumer.mem) producer_cleanup_locked();
  }
  if (g_consumer.mem) {
    DeviceGuard guard_(g_consumer.device);
    (void)hipFree(g_consumer.mem);
    g_consumer.mem = nullptr;
  }
  if (g_consumer.ctrl) {
    sem_destroy(sem_of(g_consumer.ctrl->sem_start));
    sem_destroy(sem_of(g_consumer.ctrl->sem_complete));
  }
  const bool had = g_consumer.fd != -1;
  unmap_role(g_consumer);
  if (had) shm_unlink(g_consumer.shm_name);
  g_consumer = Role();
}

static int producer_copy(const void* src, int64_t src_bytes, const int64_t* src_off,
                         const int64_t* dst_off, const int64_t* run_tokens, int64_t n_runs,
                         int64_t page_size, int64_t total_tokens, const bikv_tensor_dims* dims,
                         int64_t elem_bytes, int32_t dtype_code, void* stream) {
  std::lock_guard<std::mutex> lk(g_prod.mu);
  if (!g_producer.ctrl || !g_producer.mem) return fail(BIKV_ESTATE, "producer is not initialised");
  if (g_prod.reserved) return fail(BIKV_ESTATE, kReservedMsg);
  if (!dims) return fail(BIKV_EINVAL, "dims is null");
  if (n_runs < 0 || page_size <= 0 || elem_bytes <= 0) return fail(BIKV_EINVAL, "bad n_runs, page_size or elem_bytes");
  if (dims->head_size <= 0 || dims->num_kv_heads <= 0 || dims->num_layers <= 0 || dims->kv_pair <= 0)
    return fail(BIKV_EINVAL, "TensorDims fields must be positive");
  if (total_tokens < 0 || total_tokens > n_runs * page_size)
    return fail(BIKV_EINVAL, "total_tokens %lld is outside [0, n_runs*page_size]", (long long)total_tokens);
  bikv_shared_control* c = g_producer.ctrl;
  const int64_t elems_per_token = dims->head_size * dims->num_kv_heads * dims->num_layers * dims->kv_pair;
  const int64_t token_bytes = elems_per_token * elem_bytes;
  const int64_t run_bytes = page_size * token_bytes;
  const int64_t data_size = total_tokens * token_bytes;
  if ((size_t)data_size > c->buffer_size)
    return fail(BIKV_ERANGE, "batch of %lld bytes does not fit the %zu-byte ring", (long long)data_size, c->buffer_size);
  BIKV_DEVICE(g_producer.device);
  size_t at = 0;
  {
    const int rc = producer_reserve((size_t)data_size, &at);
    if (rc) return rc;
  }
  if (n_runs > 0) {
    // the window handed to the kernel ends where this transfer ends: a run that would write past
    // the published bytes is skipped and reported
    char* window = static_cast<char*>(g_producer.mem) + at;
    if (!src_off || !dst_off) return fail(BIKV_EINVAL, "null pointer argument");
    int rc = run_tokens
        ? copy_runs_banked(ST_BANK_RING, src, src_bytes, window, data_size, src_off, dst_off, run_tokens,
                           n_runs, run_bytes, token_bytes, stream)
        : copy_runs_banked(ST_BANK_RING, src, src_bytes, window, data_size, src_off, dst_off, nullptr,
                           n_runs, run_bytes, elem_bytes, stream);
    if (rc) return rc;
    rc = sync_and_check(g_producer.device, ST_BANK_RING, static_cast<hipStream_t>(stream));
    if (rc) return rc;
  }
  const int64_t shape[5] = {total_tokens, dims->head_size, dims->num_kv_heads, dims->num_layers, dims->kv_pair};
  {
    const int rc = producer_wait_slot();
    if (rc) return rc;
  }
  ring::publish_transfer(g_prod, at, (size_t)data_size, shape, 5, dtype_code);
  return BIKV_OK;
}

extern "C" int bikv_producer_copy_pages(const void* src, int64_t src_bytes, const int64_t* src_off,
                                        const int64_t* dst_off, int64_t n_runs, int64_t page_size,
                                        const bikv_tensor_dims* dims, int64_t elem_bytes,
                                        int32_t dtype_code, void* stream) {
  if (n_runs < 0 || page_size <= 0) return fail(BIKV_EINVAL, "bad n_runs, page_size or elem_bytes");
  return producer_copy(src, src_bytes, src_off, dst_off, nullptr, n_runs, page_size, n_runs * page_size,
                       dims, elem_bytes, dtype_code, stream);
}

extern "C" int bikv_producer_copy_tokens(const void* src, int64_t src_bytes, const int64_t* src_off,
                                         const int64_t* dst_off, const int64_t* run_tokens,
                                         int64_t n_runs, int64_t page_size, int64_t total_tokens,
                                         const bikv_tensor_dims* dims, int64_t elem_bytes,
                                         int32_t dtype_code, void* stream) {
  if (n_runs > 0 && !run_tokens) return fail(BIKV_EINVAL, "run_tokens is null");
  return producer_copy(src, src_bytes, src_off, dst_off, run_tokens, n_runs, page_size, total_tokens,
                       dims, elem_bytes, dtype_code, stream);
}

extern "C" int bikv_producer_send(const void* dev_src, size_t bytes, const int64_t* shape,
                                  size_t ndim, int32_t dtype_code, void* stream) {
  std::lock_guard<std::mutex> lk(g_prod.mu);
  if (!g_producer.ctrl || !g_producer.mem) return fail(BIKV_ESTATE, "producer is not initialised");
  if (g_prod.reserved) return fail(BIKV_ESTATE, kReservedMsg);
  if (ndim > BIKV_MAX_DIM) return fail(BIKV_EINVAL, "at most %d dimensions can be published", BIKV_MAX_DIM);
  if ((bytes > 0 && !dev_src) || (ndim > 0 && !shape)) return fail(BIKV_EINVAL, "null pointer argument");
  bikv_shared_control* c = g_producer.ctrl;
  if (bytes > c->buffer_size)
    return fail(BIKV_ERANGE, "tensor of %zu bytes does not fit the %zu-byte ring", bytes, c->buffer_size);
  BIKV_DEVICE(g_producer.device);
  size_t at = 0;
  {
    const int rc = producer_reserve(bytes, &at);
    if (rc) return rc;
  }
  if (bytes > 0) {
    // the library's own copy kernel where both ends are 16-byte aligned (a plain copy at 6.8 TB/s against the
    // 4.6 TB/s of a device-to-device hipMemcpyAsync, and no copy engine involved), hipMemcpyAsync otherwise
    char* dst = static_cast<char*>(g_producer.mem) + at;
    if ((((uint64_t)dst | (uint64_t)dev_src) & 15) == 0)
      BIKV_HIP(launch_linear_copy(dev_src, dst, (int64_t)bytes, static_cast<hipStream_t>(stream)));
    else
      BIKV_HIP(hipMemcpyAsync(dst, dev_src, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
    BIKV_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  }
  {
    const int rc = producer_wait_slot();
    if (rc) return rc;
  }
  ring::publish_transfer(g_prod, at, bytes, shape, ndim, dtype_code);
  return BIKV_OK;
}

// Two-step producer for callers that fill the ring themselves (a layered gather whose staging image
// IS the consumer's ring window, the way block_per_page_copy_kernel writes straight into the mapped
// buffer, copy_kernel.cu:92-113): reserve applies the reference's wrap rule and hands out the write
// pointer; publish performs the reference's bookkeeping for exactly the reserved bytes.
extern "C" int bikv_producer_reserve(size_t bytes, void** ptr) {
  std::lock_guard<std::mutex> lk(g_prod.mu);
  if (!g_producer.ctrl || !g_producer.mem) return fail(BIKV_ESTATE, "producer is not initialised");
  if (g_prod.reserved) return fail(BIKV_ESTATE, kReservedMsg);
  if (!ptr) return fail(BIKV_EINVAL, "null pointer argument");
  bikv_shared_control* c = g_producer.ctrl;
  if (bytes > c->buffer_size)
    return fail(BIKV_ERANGE, "reservation of %zu bytes does not fit the %zu-byte ring", bytes, c->buffer_size);
  size_t at = 0;
  const int rc = producer_reserve(bytes, &at);
  if (rc) return rc;
  g_prod.reserved = true;
  g_prod.reserved_at = at;
  g_prod.reserved_bytes = bytes;
  *ptr = static_cast<char*>(g_producer.mem) + at;
  return BIKV_OK;
}

extern "C" int bikv_producer_publish(const int64_t* shape, size_t ndim, int32_t dtype_code, void* stream) {
  std::lock_guard<std::mutex> lk(g_prod.mu);
  if (!g_producer.ctrl || !g_producer.mem) return fail(BIKV_ESTATE, "producer is not initialised");
  if (!g_prod.reserved) return fail(BIKV_ESTATE, "nothing is reserved (call bikv_producer_reserve first)");
  if (ndim > BIKV_MAX_DIM) return fail(BIKV_EINVAL, "at most %d dimensions can be published", BIKV_MAX_DIM);
  if (ndim > 0 && !shape) return fail(BIKV_EINVAL, "null pointer argument");
  BIKV_DEVICE(g_producer.device);
  // the bytes must be in the ring before the consumer is woken; a kernel that skipped work is an error
  // (the caller's own launches report into the shared status bank: a flag raised by ANY unchecked
  // launch on this device since the last bikv_check_status fails the publication)
  int rc = sync_and_check(g_producer.device, ST_BANK_SHARED, static_cast<hipStream_t>(stream));
  if (rc == BIKV_EBOUNDS) g_prod.reserved = false;   // the window is incomplete: it is never published
  if (rc) return rc;
  rc = producer_wait_slot();
  if (rc) return rc;
  g_prod.reserved = false;
  ring::publish_transfer(g_prod, g_prod.reserved_at, g_prod.reserved_bytes, shape, ndim, dtype_code);
  return BIKV_OK;
}

extern "C" int bikv_producer_cancel(void) {
  std::lock_guard<std::mutex> lk(g_prod.mu);
  if (!g_producer.ctrl) return fail(BIKV_ESTATE, "producer is not initialised");
  g_prod.reserved = false;   // nothing was published: the window is handed out again next time
  return BIKV_OK;
}

extern "C" int bikv_producer_set_backpressure(int enabled, int64_t timeout_ms) {
  std::lock_guard<std::mutex> lk(g_prod.mu);
  if (!g_producer.ctrl) return fail(BIKV_ESTATE, "producer is not initialised");
  g_prod.backpressure = enabled != 0;
  g_prod.bp_timeout_ms = timeout_ms;
  if (!enabled) g_prod.in_flight.clear();
  return BIKV_OK;
}

extern "C" int bikv_consumer_release(void) {
  std::shared_lock<std::shared_mutex> lk(g_cons_mu);
  if (!g_consumer.ctrl) return fail(BIKV_ESTATE, "consumer is not initialised");
  if (sem_post(sem_of(g_consumer.ctrl->sem_complete)) != 0)
    return fail(BIKV_ESYS, "sem_post(sem_complete) failed: %s", strerror(errno));
  return BIKV_OK;
}

extern "C" int bikv_consumer_receive(int64_t timeout_ms, void** ptr, int64_t shape[BIKV_MAX_DIM],
                                     size_t* ndim, size_t* data_bytes, int32_t* device_id,
                                     int32_t* dtype_code) {
  // shared: the role cannot be cleaned up while this call waits, and a release can still run beside it
  std::shared_lock<std::shared_mutex> lk(g_cons_mu);
  if (!g_consumer.ctrl || !g_consumer.mem) return fail(BIKV_ESTATE, "consumer is not initialised");
  if (!ptr || !shape || !ndim) return fail(BIKV_EINVAL, "null pointer argument");
  bikv_shared_control* c = g_consumer.ctrl;
  const int rc = ring::wait_ms(sem_of(c->sem_start), timeout_ms);
  if (rc == ring::WAIT_TIMEOUT) return fail(BIKV_ESTATE, "consumer_receive timed out after %lld ms", (long long)timeout_ms);
  if (rc == ring::WAIT_ERROR) return fail(BIKV_ESYS, "consumer_receive sem_wait failed: %s", strerror(errno));
  if (c->tensor_dim > BIKV_MAX_DIM) return fail(BIKV_ESTATE, "control block holds %zu dimensions", c->tensor_dim);
  *ptr = static_cast<char*>(g_consumer.mem) + c->last_valid_offset;
  *ndim = c->tensor_dim;
  for (size_t i = 0; i < c->tensor_dim; ++i) shape[i] = c->tensor_shape[i];
  if (data_bytes) *data_bytes = c->data_size;
  if (device_id) *device_id = c->device_id;
  if (dtype_code) *dtype_code = c->dtype_code;
  return BIKV_OK;
}

extern "C" const bikv_shared_control* bikv_producer_control(void) { return g_producer.ctrl; }
extern "C" const bikv_shared_control* bikv_consumer_control(void) { return g_consumer.ctrl; }
extern "C" void* bikv_consumer_buffer(void) { return g_consumer.mem; }
