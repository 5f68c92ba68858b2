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
  CHECK(bikv_pool_destroy(handle));
  CHECK(bikv_host_free(pool_v));
  CHECK(bikv_host_free(stg_v));
  CHECK(bikv_host_free(idx_v));
  CHECK(bikv_host_free(dst_v));
  printf("abi_client: ok\n");
  return 0;
}
