/* A plain-C caller of libbikv_pagecopy.so: no HIP headers, no C++, no Python. It shows that the
 * boundary really is a C ABI (what a cgo / JNI / C++ host such as the reference's ipc_service.cpp
 * would link against) and checks one run copy, one ragged run copy and the layered gather/scatter
 * against loops written here.
 *
 * All buffers come from bikv_host_alloc: pinned host memory that the GPU reads and writes in place,
 * so a program without a device allocator can still drive every kernel (the reference's zero-copy
 * path does the same for its source, copy_kernel.cu:133-196).
 *
 * Prints "abi_client: ok" and exits 0, or prints what differed and exits 1. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "bikv_pagecopy.h"

#define CHECK(call)                                                              \
  do {                                                                           \
    int rc_ = (call);                                                            \
    if (rc_ != BIKV_OK) {                                                        \
      fprintf(stderr, "abi_client: %s -> %d: %s\n", #call, rc_, bikv_last_error()); \
      return 1;                                                                  \
    }                                                                            \
  } while (0)

static uint32_t rng_state = 12345u;
static uint32_t rnd(void) {
  rng_state = rng_state * 1664525u + 1013904223u;
  return rng_state >> 8;
}

int main(void) {
  if (bikv_abi_version() != BIKV_ABI_VERSION) {
    fprintf(stderr, "abi_client: library ABI %d, header %d\n", bikv_abi_version(), BIKV_ABI_VERSION);
    return 1;
  }
  enum { N_PAGES = 40, N_PLANES = 3, TILE = 4096, N_RUNS = 9, N_BATCH = 7 };
  void *pool_v, *stg_v, *idx_v, *dst_v;
  CHECK(bikv_host_alloc((int64_t)N_PLANES * N_PAGES * TILE, &pool_v));
  CHECK(bikv_host_alloc((int64_t)N_PLANES * N_BATCH * TILE, &stg_v));
  CHECK(bikv_host_alloc(64 * 8, &idx_v));
  CHECK(bikv_host_alloc((int64_t)N_RUNS * TILE, &dst_v));
  uint8_t* pool = (uint8_t*)pool_v;
  uint8_t* stg = (uint8_t*)stg_v;
  uint8_t* dst = (uint8_t*)dst_v;
  int64_t* idx = (int64_t*)idx_v;
  for (int64_t i = 0; i < (int64_t)N_PLANES * N_PAGES * TILE; ++i) pool[i] = (uint8_t)rnd();

  /* 1. run copy: nine runs of one tile out of plane 0, destinations in reverse order */
  int64_t* so = idx;
  int64_t* dof = idx + 16;
  int64_t* len = idx + 32;
  for (int i = 0; i < N_RUNS; ++i) {
    so[i] = (int64_t)(rnd() % N_PAGES) * TILE;
    dof[i] = (int64_t)(N_RUNS - 1 - i) * TILE;
    len[i] = (int64_t)(rnd() % (TILE + 1));
  }
  len[0] = 0;
  len[1] = TILE;
  memset(dst, 0xA5, (size_t)N_RUNS * TILE);
  CHECK(bikv_copy_runs(pool, (int64_t)N_PAGES * TILE, dst, (int64_t)N_RUNS * TILE, so, dof, N_RUNS, TILE, 1, NULL));
  CHECK(bikv_check_status(0, NULL, NULL));
  for (int i = 0; i < N_RUNS; ++i)
    if (memcmp(dst + dof[i], pool + so[i], TILE) != 0) {
      fprintf(stderr, "abi_client: run %d differs\n", i);
      return 1;
    }

  /* 2. ragged run copy: the same runs with their own lengths; bytes past a run's length stay 0xA5 */
  memset(dst, 0xA5, (size_t)N_RUNS * TILE);
  CHECK(bikv_copy_runs_ragged(pool, (int64_t)N_PAGES * TILE, dst, (int64_t)N_RUNS * TILE, so, dof, len, N_RUNS, TILE, 1, NULL));
  CHECK(bikv_check_status(0, NULL, NULL));
  for (int i = 0; i < N_RUNS; ++i)
    for (int64_t e = 0; e < TILE; ++e) {
      const uint8_t want = e < len[i] ? pool[so[i] + e] : 0xA5;
      if (dst[dof[i] + e] != want) {
        fprintf(stderr, "abi_client: ragged run %d byte %lld differs\n", i, (long long)e);
        return 1;
      }
    }

  /* 3. layered gather of 7 pages (one duplicate) over 3 planes, layer-major image, then scatter of the
   *    image into 7 other pages */
  const void* planes[N_PLANES];
  for (int q = 0; q < N_PLANES; ++q) planes[q] = pool + (int64_t)q * N_PAGES * TILE;
  bikv_pool_desc pd;
  memset(&pd, 0, sizeof(pd));
  pd.device = 0;
  pd.n_planes = N_PLANES;
  pd.n_pages = N_PAGES;
  pd.tile_bytes = TILE;
  pd.page_stride_bytes = TILE;
  pd.plane_base = planes;
  bikv_pool* handle = NULL;
  CHECK(bikv_pool_create(&pd, &handle));
  int64_t* ids = idx;
  int64_t* slots = idx + 16;
  int64_t* strides = idx + 32;
  const int64_t gather_ids[N_BATCH] = {5, 17, 5, 39, 0, 22, 8};
  const int64_t scatter_ids[N_BATCH] = {30, 31, 1, 2, 33, 12, 13};
  for (int i = 0; i < N_BATCH; ++i) {
    ids[i] = gather_ids[i];
    slots[i] = i;
    strides[i] = N_BATCH;
  }
  bikv_page_batch b;
  memset(&b, 0, sizeof(b));
  b.page_ids = ids;
  b.slots = slots;
  b.slot_strides = strides;
  b.n_pages = N_BATCH;
  b.layout_hint = BIKV_HINT_LAYER_MAJOR;
  memset(stg, 0xA5, (size_t)N_PLANES * N_BATCH * TILE);
  CHECK(bikv_gather_pages(handle, &b, stg, (int64_t)N_PLANES * N_BATCH * TILE, NULL, 0, NULL));
  CHECK(bikv_check_status(0, NULL, NULL));
  for (int q = 0; q < N_PLANES; ++q)
    for (int i = 0; i < N_BATCH; ++i)
      if (memcmp(stg + ((int64_t)q * N_BATCH + i) * TILE, pool + ((int64_t)q * N_PAGES + gather_ids[i]) * TILE, TILE) != 0) {
        fprintf(stderr, "abi_client: gathered tile (plane %d, entry %d) differs\n", q, i);
        return 1;
      }
  for (int i = 0; i < N_BATCH; ++i) ids[i] = scatter_ids[i];
  CHECK(bikv_scatter_pages(handle, &b, stg, (int64_t)N_PLANES * N_BATCH * TILE, NULL, 0, NULL));
  CHECK(bikv_check_status(0, NULL, NULL));
  for (int q = 0; q < N_PLANES; ++q)
    for (int i = 0; i < N_BATCH; ++i)
      if (memcmp(pool + ((int64_t)q * N_PAGES + scatter_ids[i]) * TILE, stg + ((int64_t)q * N_BATCH + i) * TILE, TILE) != 0) {
        fprintf(stderr, "abi_client: scattered tile (plane %d, entry %d) differs\n", q, i);
        return 1;
      }

  /* 4. a page id outside the pool is skipped and reported, not dereferenced */
  ids[3] = N_PAGES + 5;
  if (bikv_gather_pages(handle, &b, stg, (int64_t)N_PLANES * N_BATCH * TILE, NULL, 0, NULL) != BIKV_OK) return 1;
  uint32_t bits = 0;
  if (bikv_check_status(0, NULL, &bits) != BIKV_EBOUNDS || !(bits & BIKV_ST_PAGE_ID)) {
    fprintf(stderr, "abi_client: bad page id not reported (bits 0x%x)\n", bits);
    return 1;
  }

  /* 5. staging pipeline: two requests enqueued back to back into two pinned images, one wait; then the
   *    first image travels back into other pages through the synchronous call */
  {
    enum { R0 = 3, R1 = 4 };
    const int64_t r0_ids[R0] = {9, 3, 27};
    const int64_t r1_ids[R1] = {14, 9, 0, 38};
    const int64_t back_ids[R0] = {20, 21, 4};
    void *img0_v, *img1_v;
    CHECK(bikv_host_alloc((int64_t)N_PLANES * R0 * TILE, &img0_v));
    CHECK(bikv_host_alloc((int64_t)N_PLANES * R1 * TILE, &img1_v));
    uint8_t* img[2];
    img[0] = (uint8_t*)img0_v;
    img[1] = (uint8_t*)img1_v;
    bikv_stager* stager = NULL;
    CHECK(bikv_stager_create(0, 2 * TILE, 2, 2, &stager));
    /* index arrays of both requests live side by side in the pinned index block */
    for (int i = 0; i < R0; ++i) { ids[i] = r0_ids[i]; slots[i] = i; strides[i] = R0; }
    for (int i = 0; i < R1; ++i) { ids[8 + i] = r1_ids[i]; slots[8 + i] = i; strides[8 + i] = R1; }
    bikv_page_batch b0, b1;
    memset(&b0, 0, sizeof(b0));
    b0.page_ids = ids; b0.slots = slots; b0.slot_strides = strides; b0.n_pages = R0;
    b0.layout_hint = BIKV_HINT_LAYER_MAJOR;
    b1 = b0;
    b1.page_ids = ids + 8; b1.slots = slots + 8; b1.slot_strides = strides + 8; b1.n_pages = R1;
    const int64_t n0 = R0, n1 = R1;
    memset(img[0], 0xA5, (size_t)N_PLANES * R0 * TILE);
    memset(img[1], 0xA5, (size_t)N_PLANES * R1 * TILE);
    CHECK(bikv_gather_to_host_async(stager, handle, &b0, &n0, 1, BIKV_LAYOUT_LAYER_MAJOR, img[0],
                                    (int64_t)N_PLANES * R0 * TILE, NULL, 0, BIKV_STAGE_PIPELINED, NULL));
    CHECK(bikv_gather_to_host_async(stager, handle, &b1, &n1, 1, BIKV_LAYOUT_LAYER_MAJOR, img[1],
                                    (int64_t)N_PLANES * R1 * TILE, NULL, 0, BIKV_STAGE_AUTO, NULL));
    bikv_stage_stats stats;
    CHECK(bikv_stager_wait(stager, &stats));
    if (stats.bytes != (int64_t)N_PLANES * (R0 + R1) * TILE) {
      fprintf(stderr, "abi_client: stager reports %lld bytes\n", (long long)stats.bytes);
      return 1;
    }
    for (int q = 0; q < N_PLANES; ++q) {
      for (int i = 0; i < R0; ++i)
        if (memcmp(img[0] + ((int64_t)q * R0 + i) * TILE, pool + ((int64_t)q * N_PAGES + r0_ids[i]) * TILE, TILE) != 0) {
          fprintf(stderr, "abi_client: staged tile (request 0, plane %d, entry %d) differs\n", q, i);
          return 1;
        }
      for (int i = 0; i < R1; ++i)
        if (memcmp(img[1] + ((int64_t)q * R1 + i) * TILE, pool + ((int64_t)q * N_PAGES + r1_ids[i]) * TILE, TILE) != 0) {
          fprintf(stderr, "abi_client: staged tile (request 1, plane %d, entry %d) differs\n", q, i);
          return 1;
        }
    }
    for (int i = 0; i < R0; ++i) ids[i] = back_ids[i];
    CHECK(bikv_find_duplicate(ids, R0, NULL));
    CHECK(bikv_scatter_from_host(stager, handle, &b0, &n0, 1, BIKV_LAYOUT_LAYER_MAJOR, img[0],
                                 (int64_t)N_PLANES * R0 * TILE, NULL, 0, BIKV_STAGE_AUTO, &stats));
    for (int q = 0; q < N_PLANES; ++q)
      for (int i = 0; i < R0; ++i)
        if (memcmp(pool + ((int64_t)q * N_PAGES + back_ids[i]) * TILE, img[0] + ((int64_t)q * R0 + i) * TILE, TILE) != 0) {
          fprintf(stderr, "abi_client: tile scattered from the host (plane %d, entry %d) differs\n", q, i);
          return 1;
        }
    CHECK(bikv_stager_destroy(stager));
    CHECK(bikv_host_free(img0_v));
    CHECK(bikv_host_free(img1_v));
  }
  CHECK(bikv_pool_destroy(handle));
  CHECK(bikv_host_free(pool_v));
  CHECK(bikv_host_free(stg_v));
  CHECK(bikv_host_free(idx_v));
  CHECK(bikv_host_free(dst_v));
  printf("abi_client: ok\n");
  return 0;
}
