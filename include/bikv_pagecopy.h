/*
 * bikv_pagecopy.h — C ABI of libbikv_pagecopy.so, the MI355X (gfx950) KV page-copy library.
 *
 * The library replaces the device side of Bi-KV's `ipc_service` extension
 * (Bi-KV/SharedMemory/CUDA_Shared/{copy_kernel.cu, ipc_service.cpp, ipc_wrapper.h}) and adds the
 * layered (per layer, per K/V plane) page gather/scatter and the device->pinned-host staging pipeline.
 * Everything here is plain C: raw pointers, sizes, and two small PODs. No torch types cross the
 * boundary; a `void* stream` is a hipStream_t (NULL = the legacy default stream).
 *
 * Conventions
 *   - Every function returning int returns BIKV_OK (0) or a negative BIKV_E* code; the text of the
 *     last failure on the calling thread is available from bikv_last_error().
 *   - "device array" = memory the GPU can dereference (HBM, or pinned host memory mapped into the
 *     device address space). The library never reads device arrays on the host.
 *   - All offsets and sizes are 64-bit. (The reference computes sizes in `int`,
 *     copy_kernel.cu:81-84, and overflows at 2 GiB.)
 *   - Kernels bounds-check every run/tile against the extents passed here. A violating run/tile is
 *     skipped (nothing is read or written for it) and a bit is raised in a per-device status word;
 *     the synchronous entry points and bikv_check_status() turn that into BIKV_EBOUNDS.
 */
#ifndef BIKV_PAGECOPY_H
#define BIKV_PAGECOPY_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BIKV_ABI_VERSION 4

enum {
  BIKV_OK = 0,
  BIKV_EINVAL = -1,   /* bad argument (null pointer, negative size, misuse) */
  BIKV_EHIP = -2,     /* a HIP runtime call failed; message carries hipGetErrorString */
  BIKV_ESYS = -3,     /* shm_open/mmap/ftruncate/... failed; message carries strerror */
  BIKV_ESTATE = -4,   /* role not initialised / already initialised */
  BIKV_EBOUNDS = -5,  /* a kernel skipped at least one run/tile that fell outside its buffers */
  BIKV_ERANGE = -6    /* request larger than a fixed capacity (ring buffer, chunk) */
};

/* Bits of the per-device status word raised by kernels. */
enum {
  BIKV_ST_SRC_RANGE = 1u,   /* a source run/tile was outside the source extent */
  BIKV_ST_DST_RANGE = 2u,   /* a destination run/tile was outside the destination extent */
  BIKV_ST_PAGE_ID = 4u      /* a page id was outside [0, n_pages) */
};

int bikv_abi_version(void);
const char* bikv_last_error(void);

/* Sets up the library's per-device state on `device` (a small host-mapped status block, and the device
 * address of the library's static scratch array). Idempotent. Every handle-creating call does the same
 * on first use of a device; callers that must not allocate later call this up front. */
int bikv_init(int device);

/* Reads and clears the status word of `device` after synchronising `stream`.
 * Returns BIKV_OK, or BIKV_EBOUNDS with *bits_out (nullable) holding the BIKV_ST_* bits.
 * There is ONE status word per device, shared by every stream and host thread: a check reports (and
 * clears) whatever any launch on that device has raised since the previous check, so callers that run
 * several streams should treat a report as "some launch since the last check skipped work". Memory
 * safety never depends on the check: out-of-range units are skipped by the kernels themselves. */
int bikv_check_status(int device, void* stream, uint32_t* bits_out);

/* Kernel launch knobs, for measurement. Keys: "seg" (0 = default: the wave mover, one 16-byte
 * vector per lane, whenever the tile shape qualifies; n > 0 = the LDS-staged segment mover with n
 * batch pages per workgroup), "wave_block" (lanes per workgroup of the wave mover: 64, 128, 256),
 * "order" (wave mover walk: 0 = plane by plane, 1 = chunks of pages with their planes together,
 * -1 = default: chosen from the batch's layout hint), "log2_chunk" (order 1: pages per chunk,
 * -1 = chosen),
 * "unroll" (segment mover: 16-byte vectors in flight per lane: 1, 2, 4, 8), "nontemporal" (nt hint on
 * payload accesses: 1 on, 0 off, 4 = nt with system scope, -1 = default: chosen per direction and
 * layout; the run copy also takes 2 = loads only, 3 = stores only),
 * "small_run_max" (runs up to this
 * many bytes use one lane per 16-byte piece instead of one wave per KiB), "run_group" (1 = several
 * short runs share a row of the launch grid, default; 0 = one row per run), "transpose_lds_kib" and
 * "transpose_dsplit" (LDS tile budget and head_dim slices of the layout-change kernel),
 * "transpose_pairs" (1 = the K/V-pair kernel, default; 0 = the element-wise kernel), "transpose_block"
 * (its lanes per workgroup: 128, 256, 512, 1024; 0 = default: 256 for the load, 512 for the store) and
 * "transpose_sc1" (1 = its payload stores are nt with system scope, default; 0 = nt only),
 * "transpose_kvswap" (1 = where K and V rows of a token are adjacent halves of one KiB — the Worker's own
 * tensors at 2 KV heads x 128 x fp16 — the pair kernel reads and writes whole KiB on the pool side and
 * exchanges half-waves between lanes; 0 = default: every lane addresses its own rows, which measures 1.7 %
 * faster for the store and 0.6 % slower for the load),
 * "debug_unique" (1 = what BIKV_DEBUG_UNIQUE=1 in the environment switches on, see bikv_find_duplicate).
 * Process-wide and safe to set from any thread: a launch works on the snapshot of the knobs it took
 * when it began. */
int bikv_set_tuning(const char* key, int64_t value);
/* Every knob back to its default. */
void bikv_reset_tuning(void);

/* Host-side check for scatters: BIKV_OK when the n ids (HOST array) are pairwise different, else
 * BIKV_EINVAL with a message naming the repeated id and the two entries that hold it, and *dup_out
 * (nullable) set to that id. Two runs of one launch that write the same destination race here exactly
 * as in the reference's kernel (copy_kernel.cu:29-35: whichever block stores last wins), so callers
 * that cannot vouch for their page lists check them with this. With BIKV_DEBUG_UNIQUE=1 in the
 * environment, bikv_scatter_pages, bikv_scatter_from_host and bikv_nhd_load_token_major run the same
 * check on a copy of their device ids before launching (a debugging aid: it synchronises the stream). */
int bikv_find_duplicate(const int64_t* ids, int64_t n, int64_t* dup_out);

/* --------------------------------------------------------------------------------------------
 * 1. Run copy — the reference's generic offset->offset page copy.
 *
 * Replaces block_per_page_copy_kernel (copy_kernel.cu:9-36) and zero_copy_page_kernel
 * (copy_kernel.cu:39-66): for every run i < n_runs
 *     dst[dst_off[i]*unit .. +run_bytes) = src[src_off[i]*unit .. +run_bytes)
 * Gather = scattered src_off, dense dst_off; scatter = the same call with the roles swapped.
 * `src`/`dst` may be HBM or device-mapped pinned host memory (the zero-copy variant reads the
 * pinned host pool directly, copy_kernel.cu:142). `src_off`/`dst_off` are int64 device arrays in
 * units of `unit_bytes` (the reference passes element offsets; pass unit_bytes = element size, or
 * 1 for byte offsets). Source runs may overlap or repeat; destination runs must be disjoint.
 * Asynchronous on `stream`.
 * ------------------------------------------------------------------------------------------ */
int bikv_copy_runs(const void* src, int64_t src_bytes,
                   void* dst, int64_t dst_bytes,
                   const int64_t* src_off, const int64_t* dst_off,
                   int64_t n_runs, int64_t run_bytes, int64_t unit_bytes,
                   void* stream);

/* Ragged runs: run i moves run_len[i]*unit bytes (int64 device array, 0 <= run_len[i]*unit <=
 * max_run_bytes; a length outside that range skips the run and sets BIKV_ST_SRC_RANGE). This is what
 * a packed destination needs: the reference packs the partial last page of an item tighter than a
 * page (kvcache.py:169-174) but still copies whole pages (copy_kernel.cu:29-35), so its
 * destinations overlap; with the tail length given per run they do not. */
int bikv_copy_runs_ragged(const void* src, int64_t src_bytes,
                          void* dst, int64_t dst_bytes,
                          const int64_t* src_off, const int64_t* dst_off, const int64_t* run_len,
                          int64_t n_runs, int64_t max_run_bytes, int64_t unit_bytes,
                          void* stream);

/* --------------------------------------------------------------------------------------------
 * 2. Layered paged pool — gather/scatter of (page, layer, K/V) tiles.
 *
 * The pool is the Worker-side paged KV cache (Worker.py:74-78, Model/qwen2.py:532-536): one plane
 * per (layer, K/V) — plane index q = layer*kv_planes + kv — each holding n_pages tiles of
 * tile_bytes contiguous bytes, consecutive pages page_stride_bytes apart. A second, optional tile
 * class ("scale") describes per-page side data that must travel with the payload (fp32 scales of an
 * fp8 pool): same planes and page ids, its own base pointers, tile size and stride.
 *
 * The staging side is an array of tile-sized slots. Page i of a call lands, for plane q, in slot
 *     slot[i] + q * slot_stride[i]
 * i.e. byte offset slot*tile_bytes of `staging` (and slot*scale_tile_bytes of `scale_staging`).
 *   layer-major request buffer [L][2][m][tile]: slot = base_r + j,           slot_stride = m
 *   page-major  request buffer [m][L][2][tile]: slot = base_r + j*n_planes,  slot_stride = 1
 * (page-major at page granularity is the reference's token-major transfer layout, qwen2.py:519-522).
 * ------------------------------------------------------------------------------------------ */
typedef struct bikv_pool bikv_pool; /* opaque; owns a small device-resident plane table */

typedef struct bikv_pool_desc {
  int32_t device;
  int32_t n_planes;                /* layers * kv_planes */
  int64_t n_pages;                 /* pages per plane; page ids are checked against it */
  int64_t tile_bytes;              /* contiguous bytes of one (page, plane) tile */
  int64_t page_stride_bytes;       /* >= tile_bytes */
  const void* const* plane_base;   /* HOST array of n_planes device pointers */
  int64_t scale_tile_bytes;        /* 0 = no scale class */
  int64_t scale_page_stride_bytes;
  const void* const* scale_plane_base; /* HOST array of n_planes device pointers, or NULL */
  /* Tiles that are not contiguous in the pool: row_bytes > 0 cuts the payload tile into
   * tile_bytes/row_bytes rows of row_bytes bytes that sit row_stride_bytes apart (in staging the
   * tile stays contiguous). This is the Worker's own per-layer tensor [tokens, 2, heads, dim]
   * (Worker.py:74-78), where K and V interleave token by token: plane (l, k) has plane_base =
   * layer l + k*heads*dim elements, row = heads*dim elements, row stride = 2 rows, page stride =
   * block_tokens row strides. 0 = contiguous tiles. */
  int64_t row_bytes;
  int64_t row_stride_bytes;
} bikv_pool_desc;

int bikv_pool_create(const bikv_pool_desc* desc, bikv_pool** out);
int bikv_pool_destroy(bikv_pool* pool);

/* One batch of page moves. All three index arrays are int64 device arrays of n_pages entries.
 * Only planes [plane_begin, plane_begin+plane_count) are moved (plane_count <= 0 = all planes).
 * `slot_bias` is subtracted from every slot before it is scaled, so a window of a larger logical
 * staging buffer can be targeted (used by the chunked host pipeline). */
typedef struct bikv_page_batch {
  const int64_t* page_ids;
  const int64_t* slots;
  const int64_t* slot_strides;
  int64_t n_pages;
  int32_t plane_begin;
  int32_t plane_count;
  int64_t slot_bias;
  int32_t layout_hint;  /* BIKV_HINT_*: how slots were laid out; affects speed only, never results */
  int32_t reserved;
} bikv_page_batch;

enum { BIKV_HINT_NONE = 0, BIKV_HINT_LAYER_MAJOR = 1, BIKV_HINT_PAGE_MAJOR = 2 };

/* gather: pool -> staging. Duplicate and out-of-order page ids are legal. Asynchronous on stream.
 * Replaces the per-layer form of the reference's gather (kvcache.py:132-239 driving
 * copy_kernel.cu:9-36) for the paged compute layout. scale_staging may be NULL iff the pool has no
 * scale class. */
int bikv_gather_pages(const bikv_pool* pool, const bikv_page_batch* batch,
                      void* staging, int64_t staging_bytes,
                      void* scale_staging, int64_t scale_staging_bytes,
                      void* stream);

/* scatter: staging -> pool; the exact inverse. Page ids must be unique within the call.
 * Replaces the Worker's disabled host scatter `send_tensor[send_indices] = compute_buffer[...]`
 * (Worker.py:207) and the swapped-offset use of copy_kernel.cu:9-36. */
int bikv_scatter_pages(const bikv_pool* pool, const bikv_page_batch* batch,
                       const void* staging, int64_t staging_bytes,
                       const void* scale_staging, int64_t scale_staging_bytes,
                       void* stream);

/* --------------------------------------------------------------------------------------------
 * 3. Device <-> pinned-host staging pipeline.
 *
 * The reference stages KV for the transport in host tensors (kvcache.py:105-108, Worker.py:203-206)
 * that the RDMA endpoint sends from a pinned host region (onesided_rdma.h:301-337). This pipeline
 * fills such a region straight from the paged pool. A stager owns n_buffers lanes, each a HIP stream
 * with an HBM buffer of chunks_per_launch * chunk_bytes. Launch k runs on lane k % n_buffers: one
 * gather kernel fills the lane's buffer with the next contiguous piece of the staging image, then one
 * hipMemcpyAsync per chunk_bytes moves it to `host_dst`, all in the lane's stream order, so the copies
 * of one lane overlap the kernel (and queued copies) of the others. Two lanes are enough to keep the
 * link busy and are the steady choice: hipMemcpyAsync on three or four streams at once has whole passes at
 * two thirds of the link's rate, and a HIP process has 4 hardware queues by default (GPU_MAX_HW_QUEUES), its
 * streams dealt onto them in turn, so a fourth lane shares a queue with another lane.
 *
 * `req_pages` (HOST array, n_requests entries) gives the number of pages of each request; pages of
 * request r occupy batch entries [sum(req_pages[:r]), +req_pages[r]) and, in staging, a contiguous
 * block of req_pages[r]*n_planes slots whose layout is `layout`. Pieces are cut on request, plane
 * and page boundaries so that each is one contiguous byte range of the staging image.
 * `host_dst` must be pinned (hipHostMalloc / torch pin_memory) and hold the whole staging image; the
 * scale tiles of a pool with a scale class go, slot for slot, into a second pinned image.
 *
 * Modes: BIKV_STAGE_PIPELINED as above; BIKV_STAGE_DIRECT lets the kernel store into (read from) the
 * mapped pinned image itself, no HBM hop and no copy engine; BIKV_STAGE_PIPELINED_KERNEL keeps lanes and
 * lane buffers but makes the hop between lane buffer and pinned image with the library's own copy kernel
 * (one launch per lane buffer, through the mapped image) instead of hipMemcpyAsync; BIKV_STAGE_AUTO is
 * DIRECT in both directions. Why: on MI355X every hipMemcpyAsync between device and host, in either
 * direction, drops from ~57 to ~30 GB/s for as long as the driver is scrubbing device memory that some
 * hipFree (this process's or, at start-up, bikv_device_alloc's released filler chunks) has given back —
 * about one second per 15 GB freed, and hipFree itself returns at once, so nothing announces it. Kernels
 * that store to or load from mapped pinned memory hold 54-56 GB/s through it. PIPELINED is 1-2 % faster
 * than the other modes while nothing is being scrubbed and half as fast while something is.
 *
 * Every stager has status words of its own: a page id or slot that one stager's kernel rejects is
 * reported by THAT stager's wait (or synchronous call) and by no other's, so stagers are independent
 * objects that different host threads can drive on one GPU at the same time. A device serves up to 254
 * stagers at once (BIKV_ERANGE beyond). One stager is not re-entrant: one thread at a time per stager.
 * ------------------------------------------------------------------------------------------ */
typedef struct bikv_stager bikv_stager; /* opaque; owns n_buffers HIP streams, each with an HBM buffer */

enum { BIKV_LAYOUT_LAYER_MAJOR = 0, BIKV_LAYOUT_PAGE_MAJOR = 1 };
enum { BIKV_STAGE_PIPELINED = 0, BIKV_STAGE_DIRECT = 1, BIKV_STAGE_AUTO = 2, BIKV_STAGE_PIPELINED_KERNEL = 3 };

int bikv_stager_create(int device, int64_t chunk_bytes, int32_t chunks_per_launch, int32_t n_buffers,
                       bikv_stager** out);
int bikv_stager_destroy(bikv_stager* st);

typedef struct bikv_stage_stats {
  int64_t bytes;        /* payload bytes delivered */
  int64_t n_chunks;     /* host copies issued (1 per direct launch) */
  double wall_seconds;  /* host wall time from the first enqueue to the end of the wait */
} bikv_stage_stats;

/* Synchronous: returns when all bytes are in host memory; BIKV_EBOUNDS if a page id or slot was
 * rejected by a kernel of THIS call (every stager has status words of its own). */
int bikv_gather_to_host(bikv_stager* st, const bikv_pool* pool, const bikv_page_batch* batch,
                        const int64_t* req_pages, int64_t n_requests, int32_t layout,
                        void* host_dst, int64_t host_bytes,
                        void* host_scale_dst /* pinned; NULL iff the pool has no scale class */,
                        int64_t host_scale_bytes, int32_t mode,
                        bikv_stage_stats* stats /* nullable */);

/* The receiving side: the transport has landed a staging image (same layout as above) in pinned
 * host memory (the reference holds received KV in host tensors, Worker.py:166-169, and reads a
 * pinned host pool from the GPU in kvcache.py:241-366); each piece is copied host -> lane buffer and
 * scattered from there into the pool. Page ids must be unique (a scatter). Synchronous. */
int bikv_scatter_from_host(bikv_stager* st, const bikv_pool* pool, const bikv_page_batch* batch,
                           const int64_t* req_pages, int64_t n_requests, int32_t layout,
                           const void* host_src, int64_t host_bytes,
                           const void* host_scale_src /* pinned; NULL iff no scale class */,
                           int64_t host_scale_bytes, int32_t mode,
                           bikv_stage_stats* stats /* nullable */);

/* The same two transfers, enqueued only: the call returns as soon as kernels and copies are queued on
 * the stager's lanes, so the calling thread can build the next request while the link is busy, and
 * consecutive calls follow each other on the lanes without a drain in between (each request of the
 * reference is one blocking call, kvcache.py:219-225). `after_stream` (nullable hipStream_t): work
 * already queued there — typically the upload of the index arrays — is awaited by the lanes first.
 * The batch's device arrays, the pool and both host images must stay valid until bikv_stager_wait
 * returns; host images of calls in flight together must not overlap. bikv_stager_wait drains the
 * lanes, reports everything enqueued since the previous wait in `stats` (nullable) and returns
 * BIKV_EBOUNDS if any of those launches skipped out-of-range work. */
int bikv_gather_to_host_async(bikv_stager* st, const bikv_pool* pool, const bikv_page_batch* batch,
                              const int64_t* req_pages, int64_t n_requests, int32_t layout,
                              void* host_dst, int64_t host_bytes, void* host_scale_dst,
                              int64_t host_scale_bytes, int32_t mode, void* after_stream);
int bikv_scatter_from_host_async(bikv_stager* st, const bikv_pool* pool, const bikv_page_batch* batch,
                                 const int64_t* req_pages, int64_t n_requests, int32_t layout,
                                 const void* host_src, int64_t host_bytes, const void* host_scale_src,
                                 int64_t host_scale_bytes, int32_t mode, void* after_stream);
int bikv_stager_wait(bikv_stager* st, bikv_stage_stats* stats);

/* Opt-in trace of a stager's lanes, for finding out where the time of a transfer goes (no counterpart in
 * the reference; its stage timers are host-side prints, kvcache.py:155-238). While it is on, every kernel
 * launch and every host copy the stager enqueues is bracketed by two timing events on its lane, up to
 * `max_steps` steps; max_steps = 0 switches it off and drops what was recorded. bikv_stager_trace_read
 * (after bikv_stager_wait) writes up to `cap` steps in issue order and returns how many were recorded;
 * times are milliseconds from the start of the first recorded step. Tracing allocates events as it goes
 * and costs a few percent of throughput: a diagnostic, not a mode to serve in. */
enum { BIKV_TRACE_KERNEL = 0, BIKV_TRACE_COPY_D2H = 1, BIKV_TRACE_COPY_H2D = 2, BIKV_TRACE_COPY_KERNEL = 3 };
typedef struct bikv_trace_step {
  int32_t lane;
  int32_t kind;       /* BIKV_TRACE_*: gather/scatter kernel, hipMemcpyAsync out, hipMemcpyAsync in, copy kernel */
  int64_t bytes;
  float start_ms;
  float end_ms;       /* -1 when the step was never completed (its launch failed) */
} bikv_trace_step;
int bikv_stager_trace(bikv_stager* st, int64_t max_steps);
int64_t bikv_stager_trace_read(bikv_stager* st, bikv_trace_step* out, int64_t cap);

/* bikv_gather_to_host for callers that cannot allocate: code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc. It has no counterpart in the reference. The pipeline is that of
 * BIKV_STAGE_PIPELINED_KERNEL on ONE lane, the caller's `stream`: gather kernel into a buffer, then the
 * library's copy kernel from the buffer into `host_dst` through its device mapping, piece after piece in
 * stream order — kernel launches only, so a capturing stream records nothing but kernel nodes. (Only when a
 * tile size is not a multiple of 16 bytes does the hop fall back to hipMemcpyAsync calls of at most 8 MiB.)
 * The buffer is not a stager's: it is a static array inside the library's device code, 16 MiB for payload
 * tiles plus 64 KiB for scale tiles, which every GPU the library runs on holds until the process ends. The
 * call allocates and frees nothing (no hipMalloc, no stream or event creation) and only enqueues: it returns
 * when the kernels are queued on `stream`; rejected page ids / slots are reported by bikv_check_status
 * like those of bikv_gather_pages.
 * Limits: tile_bytes <= 16 MiB and scale_tile_bytes <= 64 KiB (BIKV_ERANGE otherwise); the device must
 * have been set up by bikv_init or any bikv_pool_create (BIKV_ESTATE otherwise — a valid pool implies it).
 * All calls on one GPU share that GPU's array: calls whose work overlaps in time (two streams, or two
 * threads) race on it and deliver wrong bytes; issue them on one stream, or wait between them. */
int bikv_gather_to_host_noalloc(const bikv_pool* pool, const bikv_page_batch* batch,
                                const int64_t* req_pages, int64_t n_requests, int32_t layout,
                                void* host_dst, int64_t host_bytes,
                                void* host_scale_dst /* pinned; NULL iff the pool has no scale class */,
                                int64_t host_scale_bytes, void* stream);

/* The pieces a stager whose lane buffer holds `max_slots_per_chunk` tiles cuts a batch into, without touching a GPU: writes up to `cap` pieces
 * as 6 int64 each (first_page, n_pages, plane_begin, plane_count, first_slot, n_slots) into `out`
 * and returns the total number of chunks (which may exceed cap), or a negative code. */
int64_t bikv_plan_chunks(const int64_t* req_pages, int64_t n_requests, int32_t n_planes,
                         int32_t layout, int64_t max_slots_per_chunk, int64_t* out, int64_t cap);

/* Plain pinned-buffer copy, for measuring the host link on the same box. Synchronous. */
int bikv_d2h_copy(int device, void* host_dst, const void* dev_src, int64_t bytes,
                  int64_t chunk_bytes /* 0 = one copy */, double* seconds_out);
int bikv_h2d_copy(int device, void* dev_dst, const void* host_src, int64_t bytes,
                  int64_t chunk_bytes /* 0 = one copy */, double* seconds_out);

/* --------------------------------------------------------------------------------------------
 * 3a. Device memory placed for this GPU's memory system (optional; no counterpart in the reference,
 * which allocates its pools with torch: kvcache.py:38-43, Worker.py:74-78).
 *
 * On MI355X the physical address space behaves as two halves: a copy whose random writes all land in
 * one half runs at 5.6-5.7 TB/s, the same writes spread over both at 6.6-6.7 TB/s; reads and sequential
 * writes hardly care. Which half memory lies in depends on where the driver put it: a pool that fits one
 * half (any pool below ~100 GB on an empty GPU) scatters 15-18 % slower than it could, and how a large
 * hipMalloc straddles the boundary changes from one allocation to the next.
 * bikv_device_alloc(BIKV_PLACE_SPREAD) builds the allocation from physical chunks (256 MiB - 1 GiB,
 * hipMemCreate), tells the halves apart with a short timed scatter into pairs of chunks (a pair that
 * straddles the halves runs ~19 % faster; a time too close to call is measured twice more), keeps equal
 * numbers of both kinds and maps them alternately into one virtual range, so that every window of the
 * pool spreads its writes over both halves. To reach the second half it may transiently create (and
 * release again) filler chunks: at most `max_filler_bytes` of them (bikv_device_alloc_bounded; < 0 = as
 * many as the free memory of the device less 2 GiB allows; bikv_device_alloc uses
 * BIKV_DEFAULT_MAX_FILLER_BYTES). When the budget does not reach the other half the allocation is
 * completed with what there is and bikv_device_alloc_info shows the imbalance. Two costs of fillers to
 * know: they are device memory other tenants of the GPU cannot have for the second or two the placement
 * takes, and the driver scrubs released memory in the background at ~15 GB/s, during which every
 * hipMemcpyAsync between host and device runs at about half its rate — so place pools at start-up, before
 * other large allocations and before traffic starts. Placements are serialised: within a process by a lock,
 * between the processes that share a GPU (Bi-KV runs a cache process and a worker process per GPU) by an
 * advisory file lock named after the GPU's PCI address, so that neither disturbs the other's probe timings
 * nor takes the chunks the other is counting on.
 * BIKV_PLACE_SEQUENTIAL maps the chunks in creation order, unprobed.
 * The memory behaves like hipMalloc'd memory for kernels and copies; it cannot be exported over HIP IPC.
 * Sizes are rounded up to whole chunks. ------------------------------------------------------------ */
enum { BIKV_PLACE_SPREAD = 0, BIKV_PLACE_SEQUENTIAL = 1 };
#define BIKV_DEFAULT_MAX_FILLER_BYTES ((int64_t)96 << 30)
typedef struct bikv_alloc_info {
  int64_t bytes;          /* mapped size (a whole number of chunks) */
  int64_t chunk_bytes;
  int32_t n_chunks;
  int32_t n_other_half;   /* chunks the probe placed in the other half than the first chunk */
  int32_t n_fillers;      /* chunks created on the way and released again */
  int32_t n_reprobed;     /* chunks whose first probe fell between the two groups and was repeated */
  double seconds;         /* wall time the placement took, waiting for the locks included */
  float pair_ms_same;     /* slowest pair probe seen (a pair inside the first chunk's half); 0 = nothing probed */
  float pair_ms_other;    /* fastest pair probe classified "other half"; 0 = none seen */
} bikv_alloc_info;
int bikv_device_alloc(int device, int64_t bytes, int32_t placement, void** out);
int bikv_device_alloc_bounded(int device, int64_t bytes, int32_t placement, int64_t max_filler_bytes, void** out);
int bikv_device_free(void* p);
int bikv_device_alloc_info(const void* p, bikv_alloc_info* info);
/* The same allocator behind the two function signatures torch.cuda.memory.CUDAPluggableAllocator binds
 * (alloc(size, device, stream) / free(ptr, size, device, stream); BIKV_PLACE_SPREAD, the default filler
 * budget; null on failure, which torch reports as out of memory). A torch.cuda.MemPool built on them lets
 * the reference's own torch.empty call sites (kvcache.py:38-43, Worker.py:74-78) produce placed pools;
 * segments of up to 1 GiB are carved one after the other out of placed arenas of 2 GiB (so a pool made of
 * many tensors smaller than a chunk still alternates between the halves), larger ones are placements of
 * their own; use such a pool for the KV pools only. bikv_device_alloc_info accepts any address inside a
 * placed allocation. */
void* bikv_torch_alloc(int64_t size, int device, void* stream);   /* ssize_t on the caller's side */
void bikv_torch_free(void* p, size_t size, int device, void* stream);

/* Pinned host memory (hipHostMalloc, mapped + portable). */
int bikv_host_alloc(int64_t bytes, void** out);
int bikv_host_free(void* p);

/* --------------------------------------------------------------------------------------------
 * 3b. Fused page move + layout change: token-major pages <-> per-layer paged NHD pool.
 *
 * Bi-KV keeps KV in two layouts and never converts between them: the storage / transfer layout is
 * token-major, one token = [head_dim][kv_heads][layers][2] elements (Model/qwen2.py:519-522; pools
 * (tokens,)+token_shape at kvcache.py:38-43, Worker.py:57-62), while the model reads a per-layer
 * paged pool whose rows are head_dim contiguous elements: [blocks*block, 2, heads, dim] per layer at
 * Worker.py:74-78, [blocks, 2, block, heads, dim] at Model/qwen2.py:532-536. Worker.receive_kvcache_
 * data_batch (Worker.py:162-191) stops at the received token-major tensor; these two calls are the
 * missing step, fused with the page scatter/gather:
 *   load : compute[l][block_ids[i]][k][t][h][:] = tm[tm_pages[i]][t][:, h, l, k]   (received KV -> pool)
 *   store: the inverse                                                             (pool -> KV to send)
 * for every page i < n_pages and every token t < block_tokens of it. The compute side is addressed
 *   layer_base[l] + (block*block_stride + k*kv_stride + t*token_stride + h*head_dim + d) * elem_bytes
 * which covers both reference forms (Worker.py form: block_stride = block*2*H*D, kv_stride = H*D,
 * token_stride = 2*H*D; qwen2.py form: block_stride = 2*block*H*D, kv_stride = block*H*D,
 * token_stride = H*D). `tm` is an array of token-major pages of block_tokens tokens each; `block_ids`
 * and `tm_pages` are int64 device arrays. Block ids must be unique in a load, page indices in a store.
 * Requires head_dim and kv_heads*layers*2 to be multiples of 16 bytes' worth of elements.
 * ------------------------------------------------------------------------------------------ */
typedef struct bikv_nhd bikv_nhd; /* opaque; owns a device-resident table of layer base pointers */

typedef struct bikv_nhd_desc {
  int32_t device;
  int32_t n_layers;
  int32_t kv_heads;
  int32_t head_dim;
  int32_t block_tokens;
  int32_t elem_bytes;            /* 1, 2 or 4 */
  int64_t n_blocks;
  int64_t block_stride_elems;
  int64_t kv_stride_elems;
  int64_t token_stride_elems;
  const void* const* layer_base; /* HOST array of n_layers device pointers, 16-byte aligned */
} bikv_nhd_desc;

int bikv_nhd_create(const bikv_nhd_desc* desc, bikv_nhd** out);
int bikv_nhd_destroy(bikv_nhd* pool);
int bikv_nhd_load_token_major(const bikv_nhd* pool, const void* tm, int64_t tm_bytes,
                              const int64_t* block_ids, const int64_t* tm_pages, int64_t n_pages,
                              void* stream);
int bikv_nhd_store_token_major(const bikv_nhd* pool, void* tm, int64_t tm_bytes,
                               const int64_t* block_ids, const int64_t* tm_pages, int64_t n_pages,
                               void* stream);

/* --------------------------------------------------------------------------------------------
 * 4. Producer/consumer ring — the `ipc_service` roles.
 *
 * The control block lives in POSIX shared memory and is byte-compatible with the reference's
 * SharedControl (ipc_wrapper.h:14-28): sizeof 480, field offsets asserted below. The consumer
 * creates the shm object and the device ring buffer and stores a 64-byte hipIpcMemHandle_t in
 * `ipc_handle`; a producer in another process maps it, a producer in the SAME process uses the
 * consumer's pointer directly. One producer role and one consumer role per process, as in the
 * reference (ipc_service.cpp:9-17), whose callers are gRPC thread pools: unlike the reference's, these
 * entry points may be called from several threads at once. A producer call holds the producer's lock from
 * its ring window to its publication (the copy included), so concurrent producer calls run one after the
 * other and every transfer gets a window and a publication of its own; init and cleanup exclude
 * everything else of their role; bikv_consumer_receive and bikv_consumer_release may run side by side.
 * ------------------------------------------------------------------------------------------ */
#define BIKV_IPC_HANDLE_SIZE 64
#define BIKV_MAX_DIM 5

typedef struct bikv_shared_control {
  unsigned char sem_start[32];    /* sem_t */
  unsigned char sem_complete[32]; /* sem_t; initialised, never waited on (as in the reference) */
  int32_t dtype_code;             /* reference: `data_ready`, never written. 0 = float16 */
  int32_t error_code;             /* unused, as in the reference */
  int32_t device_id;
  char hostname[256];
  size_t data_size;
  size_t tensor_dim;
  size_t current_offset;
  size_t last_valid_offset;
  size_t buffer_size;
  unsigned char ipc_handle[BIKV_IPC_HANDLE_SIZE];
  int64_t tensor_shape[BIKV_MAX_DIM];
} bikv_shared_control;

#if defined(__cplusplus)
static_assert(sizeof(bikv_shared_control) == 480, "SharedControl ABI");
static_assert(offsetof(bikv_shared_control, dtype_code) == 64, "SharedControl ABI");
static_assert(offsetof(bikv_shared_control, device_id) == 72, "SharedControl ABI");
static_assert(offsetof(bikv_shared_control, hostname) == 76, "SharedControl ABI");
static_assert(offsetof(bikv_shared_control, data_size) == 336, "SharedControl ABI");
static_assert(offsetof(bikv_shared_control, tensor_dim) == 344, "SharedControl ABI");
static_assert(offsetof(bikv_shared_control, current_offset) == 352, "SharedControl ABI");
static_assert(offsetof(bikv_shared_control, last_valid_offset) == 360, "SharedControl ABI");
static_assert(offsetof(bikv_shared_control, buffer_size) == 368, "SharedControl ABI");
static_assert(offsetof(bikv_shared_control, ipc_handle) == 376, "SharedControl ABI");
static_assert(offsetof(bikv_shared_control, tensor_shape) == 440, "SharedControl ABI");
#endif

/* TensorDims (ipc_wrapper.h:41-47). total_tokens is carried but ignored, as in the reference. */
typedef struct bikv_tensor_dims {
  int64_t total_tokens;
  int64_t head_size;
  int64_t num_kv_heads;
  int64_t num_layers;
  int64_t kv_pair;
} bikv_tensor_dims;

/* consumer_init (ipc_service.cpp:20-74): allocates the device ring and its IPC handle, then creates the
 * named control block (a stale object of that name is replaced) and fills it in one go: hostname, device,
 * ring size, handle, both semaphores at 0. Unlike the reference, which creates the block first and fills it
 * field by field around the allocation, a producer never finds a half-described ring. A ring of 2 GiB or
 * more is not exported (its handle stays zeroed): only a producer in the consumer's own process can use it. */
int bikv_consumer_init(int device, const char* shm_name, size_t buffer_bytes);
/* producer_init (ipc_service.cpp:77-110): open shm, same-host check, map the ring. A control block that
 * describes no ring yet (all zeros: the consumer is between creating and filling it) is BIKV_ESTATE. A producer in
 * ANOTHER process than the consumer refuses a ring of 2 GiB or more with BIKV_ERANGE (opening an IPC
 * mapping that large has been seen not to return on some ROCm hosts). */
int bikv_producer_init(int device, const char* shm_name);
/* producer_cleanup / consumer_cleanup (ipc_service.cpp:171-202). Idempotent. */
void bikv_producer_cleanup(void);
void bikv_consumer_cleanup(void);

/* producer_copy_pages / producer_zero_copy_pages (ipc_service.cpp:205-239 ->
 * copy_kernel.cu:68-129,133-196): run copy from `src` into the ring at the current write offset,
 * then the reference's bookkeeping — wrap to 0 if the batch does not fit behind current_offset,
 * last_valid_offset = current_offset, current_offset += data_size, tensor_dim = 5,
 * tensor_shape = [n_runs*page_size, head, kv_heads, layers, kv_pair], sem_post(sem_start).
 * data_size = n_runs*page_size*head*kv_heads*layers*kv_pair*elem_bytes (the reference hard-codes
 * sizeof(half), copy_kernel.cu:84). Offsets are int64 device arrays in ELEMENTS. `src` may be HBM
 * or mapped pinned host memory. Blocks until the copy has finished (stream sync, where the
 * reference uses cudaDeviceSynchronize). dtype_code is published for the consumer. */
int bikv_producer_copy_pages(const void* src, int64_t src_bytes,
                             const int64_t* src_off, const int64_t* dst_off, int64_t n_runs,
                             int64_t page_size, const bikv_tensor_dims* dims,
                             int64_t elem_bytes, int32_t dtype_code, void* stream);

/* The same transfer with offsets and run lengths in TOKENS (one token = head*kv_heads*layers*kv
 * elements), which is the unit kvcache.py:161-196 computes: run i copies run_tokens[i] <= page_size
 * tokens from token src_off[i] of the pool to token dst_off[i] of the ring window, so that a packed
 * destination (partial last pages) holds exactly `total_tokens` tokens with no overlap. Publishes
 * shape [total_tokens, head, kv_heads, layers, kv]; `total_tokens` is the host-side sum of
 * run_tokens, and a run that would write past it is skipped and reported (BIKV_EBOUNDS). */
int bikv_producer_copy_tokens(const void* src, int64_t src_bytes, const int64_t* src_off,
                              const int64_t* dst_off, const int64_t* run_tokens, int64_t n_runs,
                              int64_t page_size, int64_t total_tokens, const bikv_tensor_dims* dims,
                              int64_t elem_bytes, int32_t dtype_code, void* stream);

/* producer_send (ipc_service.cpp:113-143): contiguous device tensor -> ring, publishes the real
 * shape (ndim <= 5). */
int bikv_producer_send(const void* dev_src, size_t bytes, const int64_t* shape, size_t ndim,
                       int32_t dtype_code, void* stream);

/* The producer's two halves on their own, for callers that fill the ring themselves — a layered
 * gather whose staging image IS the consumer's ring window, the way block_per_page_copy_kernel
 * writes straight into the mapped buffer (copy_kernel.cu:92-113). bikv_producer_reserve applies the
 * reference's wrap rule (copy_kernel.cu:87-89) and returns the device pointer to write `bytes` at;
 * bikv_producer_publish waits for `stream`, fails with BIKV_EBOUNDS (publishing nothing) if a kernel
 * skipped work (the reservation is then dropped), and then does the reference's bookkeeping
 * (copy_kernel.cu:116-128) for exactly the reserved bytes. One reservation at a time: until it is
 * published or given up with bikv_producer_cancel, every other producer call (send, copy_pages,
 * copy_tokens, a second reserve) fails with BIKV_ESTATE, because it would be handed the same window.
 * The caller's launches report into the status word bikv_check_status reads, so a flag left by any
 * unchecked launch on the device since the last check also fails the publication. */
int bikv_producer_reserve(size_t bytes, void** ptr);
int bikv_producer_publish(const int64_t* shape, size_t ndim, int32_t dtype_code, void* stream);
int bikv_producer_cancel(void);

/* consumer_receive (ipc_service.cpp:146-168): sem_wait(sem_start) (timeout_ms < 0 = wait forever,
 * as the reference does; on timeout returns BIKV_ESTATE), then hands out a NON-OWNING pointer into
 * the ring, valid until the producer wraps over it. */
int bikv_consumer_receive(int64_t timeout_ms, void** ptr, int64_t shape[BIKV_MAX_DIM],
                          size_t* ndim, size_t* data_bytes, int32_t* device_id,
                          int32_t* dtype_code);

/* Back-pressure (off by default: a reference consumer never posts sem_complete). The reference
 * declares and initialises SharedControl.sem_complete (ipc_wrapper.h:16, ipc_service.cpp:47) but
 * never uses it, so a producer that runs ahead overwrites the single published offset/shape slot,
 * and one that wraps overwrites tensors the consumer may still be reading (ipc_service.cpp:146-168
 * hands out non-owning views). With back-pressure enabled on the producer, a transfer stays "in
 * flight" until the consumer calls bikv_consumer_release() (once per received transfer). A producer
 * call (i) blocks before copying while its ring window overlaps the in-flight transfer, (ii) copies,
 * then (iii) blocks before publishing until the in-flight transfer is released: the copy of the next
 * transfer overlaps the consumer's use of the current one. Either wait fails with BIKV_ESTATE after
 * timeout_ms (< 0 = wait forever) with nothing published. */
int bikv_producer_set_backpressure(int enabled, int64_t timeout_ms);
int bikv_consumer_release(void);

/* Read-only views for tests and diagnostics (NULL when the role is not initialised). */
const bikv_shared_control* bikv_producer_control(void);
const bikv_shared_control* bikv_consumer_control(void);
void* bikv_consumer_buffer(void);

#ifdef __cplusplus
}
#endif
#endif /* BIKV_PAGECOPY_H */
