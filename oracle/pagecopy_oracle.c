/*
 * pagecopy_oracle.c — CPU restatement of Bi-KV's KV page-copy path. TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker for the HIP library, never a code path of it: only tests, the smoke
 * check and the benchmark's CPU-baseline leg may build, load or call it.
 *
 * Each function restates one piece of the reference (paths relative to the Bi-KV repository):
 *   oracle_copy_runs        SharedMemory/CUDA_Shared/copy_kernel.cu:9-36 (block_per_page_copy_kernel)
 *                           and :39-66 (zero_copy_page_kernel) — the same formula, host-side source
 *   oracle_copy_runs_ragged the same copy with a length per run: what the packed destination offsets
 *                           of kvcache.py:169-174 need (tail tokens of a partial last page)
 *   oracle_ring_step        copy_kernel.cu:84-89,116-127 and ipc_service.cpp:118-138 (ring advance,
 *                           shape publishing)
 *   oracle_build_offsets    DistributedStorage/kvcache.py:161-174,187-196 (page list -> offsets)
 *   oracle_gather_layered / oracle_scatter_layered
 *                           the per-(page, layer, K/V) form of the same copy over the Worker's paged
 *                           pool (Worker/Worker.py:74-78, Model/qwen2.py:532-536); scatter is the
 *                           vectorised form of the disabled host line Worker.py:207
 *   oracle_transpose_pages  page move fused with the change between the token-major layout
 *                           (Model/qwen2.py:519-522) and the per-layer paged layout (Worker.py:74-78,
 *                           qwen2.py:532-536); the reference has no code for it, the index formulas
 *                           are the two layouts' definitions
 *
 * How each is pinned (tests/test_oracle.py): the two known-answer scenarios the reference's own
 * scripts hold (test_page_ipc.py:41-65,127-150; test_zero_copy.py:30-48,86-103), the library
 * routines the formula reduces to (numpy fancy indexing, torch.index_select / index_copy_),
 * per-byte brute force on tiny inputs, and permutation / duplicate / canary invariants. The ragged
 * copy is pinned by its reduction to the uniform copy, by brute force, and by an offset-free
 * statement of the packed transfer ("each item's rows, cut to its token count, back to back") reached
 * through the reference's own packed offsets. No function here is "parity unpinned".
 */
#include <stdint.h>
#include <string.h>

/* dst[do[i]*unit + e] = src[so[i]*unit + e], e < run_bytes  (copy_kernel.cu:22-34, 52-64).
 * Returns the number of runs that fell outside either buffer (those are skipped; the reference
 * would read or write out of bounds). */
int64_t oracle_copy_runs(const uint8_t* src, int64_t src_bytes, uint8_t* dst, int64_t dst_bytes,
                         const int64_t* src_off, const int64_t* dst_off, int64_t n_runs,
                         int64_t run_bytes, int64_t unit_bytes) {
  int64_t skipped = 0;
  for (int64_t p = 0; p < n_runs; ++p) {
    const int64_t s0 = src_off[p] * unit_bytes;
    const int64_t d0 = dst_off[p] * unit_bytes;
    if (s0 < 0 || d0 < 0 || s0 + run_bytes > src_bytes || d0 + run_bytes > dst_bytes) {
      ++skipped;
      continue;
    }
    for (int64_t e = 0; e < run_bytes; ++e) dst[d0 + e] = src[s0 + e];
  }
  return skipped;
}

/* Ragged form: run p moves run_len[p]*unit bytes. The packed destination of kvcache.py:169-174
 * (a partial last page takes only `tail` tokens) is consistent only with this: copying a whole page
 * there, as copy_kernel.cu:29-35 does, overwrites the start of the next item. Runs are applied in
 * order. Returns the number of runs skipped (length outside [0, max_run_bytes] or out of range). */
int64_t oracle_copy_runs_ragged(const uint8_t* src, int64_t src_bytes, uint8_t* dst, int64_t dst_bytes,
                                const int64_t* src_off, const int64_t* dst_off, const int64_t* run_len,
                                int64_t n_runs, int64_t max_run_bytes, int64_t unit_bytes) {
  int64_t skipped = 0;
  for (int64_t p = 0; p < n_runs; ++p) {
    const int64_t s0 = src_off[p] * unit_bytes;
    const int64_t d0 = dst_off[p] * unit_bytes;
    const int64_t n = run_len[p] * unit_bytes;
    if (run_len[p] < 0 || n > max_run_bytes || s0 < 0 || d0 < 0 || s0 + n > src_bytes ||
        d0 + n > dst_bytes) {
      ++skipped;
      continue;
    }
    for (int64_t e = 0; e < n; ++e) dst[d0 + e] = src[s0 + e];
  }
  return skipped;
}

/* Ring-buffer bookkeeping of one producer call. State mirrors the SharedControl fields the
 * reference touches (ipc_wrapper.h:21-27). */
typedef struct oracle_ring {
  uint64_t data_size;
  uint64_t tensor_dim;
  uint64_t current_offset;
  uint64_t last_valid_offset;
  uint64_t buffer_size;
  int64_t tensor_shape[5];
} oracle_ring;

/* copy_kernel.cu:81-89,116-127: data_size = n_pages*page_size*elems_per_token*elem_bytes; wrap to 0
 * when the batch does not fit behind current_offset; publish. Returns the write offset used.
 * (The reference computes these in `int` with elem_bytes fixed to sizeof(half); 64-bit here.) */
uint64_t oracle_ring_step(oracle_ring* r, int64_t n_pages, int64_t page_size, int64_t head_size,
                          int64_t num_kv_heads, int64_t num_layers, int64_t kv_pair,
                          int64_t elem_bytes) {
  const int64_t elements_per_token = head_size * num_kv_heads * num_layers * kv_pair;
  const int64_t page_elements = page_size * elements_per_token;
  const uint64_t data_size = (uint64_t)(n_pages * page_elements * elem_bytes);
  if (r->current_offset + data_size > r->buffer_size) r->current_offset = 0;
  const uint64_t at = r->current_offset;
  r->last_valid_offset = r->current_offset;
  r->current_offset += data_size;
  r->tensor_dim = 5;
  r->tensor_shape[0] = n_pages * page_size;
  r->tensor_shape[1] = head_size;
  r->tensor_shape[2] = num_kv_heads;
  r->tensor_shape[3] = num_layers;
  r->tensor_shape[4] = kv_pair;
  r->data_size = data_size;
  return at;
}

/* ipc_service.cpp:118-138 (producer_send): same wrap rule, real shape. */
uint64_t oracle_ring_send(oracle_ring* r, uint64_t data_size, const int64_t* shape, uint64_t ndim) {
  if (r->current_offset + data_size > r->buffer_size) r->current_offset = 0;
  const uint64_t at = r->current_offset;
  r->data_size = data_size;
  r->tensor_dim = ndim;
  r->last_valid_offset = r->current_offset;
  r->current_offset += data_size;
  for (uint64_t i = 0; i < ndim && i < 5; ++i) r->tensor_shape[i] = shape[i];
  return at;
}

/* kvcache.py:161-174,187-196. pages: the concatenated page lists; item_pages[k]: pages of item k;
 * item_tokens[k]: its token count. Writes src_off[i] = page*page_size*scale and dst_off[i] =
 * running sum of sizes * scale, where the last page of an item has size tokens%page_size when that
 * is non-zero. scale = 1 reproduces the reference's token units. Returns the total size. */
int64_t oracle_build_offsets(const int64_t* pages, const int64_t* item_pages,
                             const int64_t* item_tokens, int64_t n_items, int64_t page_size,
                             int64_t scale, int64_t* src_off, int64_t* dst_off) {
  int64_t i = 0, current_offset = 0;
  for (int64_t idx = 0; idx < n_items; ++idx) {
    const int64_t item_token_num = item_tokens[idx];
    for (int64_t page_idx = 0; page_idx < item_pages[idx]; ++page_idx) {
      int64_t size = page_size;
      if (page_idx == item_pages[idx] - 1 && item_token_num % page_size != 0)
        size = item_token_num % page_size;
      src_off[i] = pages[i] * page_size * scale;
      dst_off[i] = current_offset * scale;
      current_offset += size;
      ++i;
    }
  }
  return current_offset;
}

/* Layered gather. plane_base[q] points at plane q's pages (page p at + p*page_stride). Requests
 * are packed back to back in `staging`; request r with m pages occupies m*n_planes tile slots:
 *   layout 0 (layer-major): slot(q, j) = base_r + q*m + j
 *   layout 1 (page-major):  slot(q, j) = base_r + j*n_planes + q
 * Returns the number of page ids outside [0, n_pool_pages) (skipped). */
int64_t oracle_gather_layered(const uint8_t* const* plane_base, int32_t n_planes,
                              int64_t n_pool_pages, int64_t tile_bytes, int64_t page_stride,
                              const int64_t* page_ids, const int64_t* req_pages, int64_t n_req,
                              int32_t layout, uint8_t* staging) {
  int64_t first = 0, base = 0, bad = 0;
  for (int64_t r = 0; r < n_req; ++r) {
    const int64_t m = req_pages[r];
    for (int32_t q = 0; q < n_planes; ++q)
      for (int64_t j = 0; j < m; ++j) {
        const int64_t pid = page_ids[first + j];
        if (pid < 0 || pid >= n_pool_pages) { if (q == 0) ++bad; continue; }
        const int64_t slot = layout == 0 ? base + (int64_t)q * m + j : base + j * n_planes + q;
        const uint8_t* s = plane_base[q] + pid * page_stride;
        uint8_t* d = staging + slot * tile_bytes;
        for (int64_t e = 0; e < tile_bytes; ++e) d[e] = s[e];
      }
    first += m;
    base += m * n_planes;
  }
  return bad;
}

/* The exact inverse: staging -> pool. Page ids must be unique for a defined result. */
int64_t oracle_scatter_layered(uint8_t* const* plane_base, int32_t n_planes, int64_t n_pool_pages,
                               int64_t tile_bytes, int64_t page_stride, const int64_t* page_ids,
                               const int64_t* req_pages, int64_t n_req, int32_t layout,
                               const uint8_t* staging) {
  int64_t first = 0, base = 0, bad = 0;
  for (int64_t r = 0; r < n_req; ++r) {
    const int64_t m = req_pages[r];
    for (int32_t q = 0; q < n_planes; ++q)
      for (int64_t j = 0; j < m; ++j) {
        const int64_t pid = page_ids[first + j];
        if (pid < 0 || pid >= n_pool_pages) { if (q == 0) ++bad; continue; }
        const int64_t slot = layout == 0 ? base + (int64_t)q * m + j : base + j * n_planes + q;
        uint8_t* d = plane_base[q] + pid * page_stride;
        const uint8_t* s = staging + slot * tile_bytes;
        for (int64_t e = 0; e < tile_bytes; ++e) d[e] = s[e];
      }
    first += m;
    base += m * n_planes;
  }
  return bad;
}

/* Fused page move + layout change between the reference's two KV layouts (it holds both and no
 * code between them, so there is no reference vector; the index formulas ARE the two layouts):
 *   token-major page: element (t, d, h, l, k) of page p at ((((p*P + t)*D + d)*H + h)*L + l)*2 + k
 *     (token_shape = (head_size, num_kv_heads, num_layers, 2), Model/qwen2.py:519-522);
 *   compute pool, layer l: element (block b, k, t, h, d) at
 *     b*block_stride + k*kv_stride + t*token_stride + h*D + d
 *     (Worker/Worker.py:74-78: [blocks*P, 2, H, D] -> strides (P*2*H*D, H*D, 2*H*D);
 *      Model/qwen2.py:532-536: [blocks, 2, P, H, D] -> strides (2*P*H*D, P*H*D, H*D)).
 * dir 1: token-major -> compute; dir 0: compute -> token-major. Returns the number of pages whose
 * block id or token-major page index is out of range (skipped). */
int64_t oracle_transpose_pages(uint8_t* const* layer_base, int32_t n_layers, int32_t kv_heads,
                               int32_t head_dim, int32_t block_tokens, int32_t elem_bytes,
                               int64_t n_blocks, int64_t block_stride, int64_t kv_stride,
                               int64_t token_stride, uint8_t* tm, int64_t n_tm_pages,
                               const int64_t* block_ids, const int64_t* tm_pages, int64_t n,
                               int32_t dir) {
  const int64_t P = block_tokens, D = head_dim, H = kv_heads, L = n_layers;
  int64_t bad = 0;
  for (int64_t i = 0; i < n; ++i) {
    const int64_t b = block_ids[i], p = tm_pages[i];
    if (b < 0 || b >= n_blocks || p < 0 || p >= n_tm_pages) { ++bad; continue; }
    for (int64_t t = 0; t < P; ++t)
      for (int64_t d = 0; d < D; ++d)
        for (int64_t h = 0; h < H; ++h)
          for (int64_t l = 0; l < L; ++l)
            for (int64_t k = 0; k < 2; ++k) {
              const int64_t ti = ((((p * P + t) * D + d) * H + h) * L + l) * 2 + k;
              const int64_t ci = b * block_stride + k * kv_stride + t * token_stride + h * D + d;
              uint8_t* tp = tm + ti * elem_bytes;
              uint8_t* cp = layer_base[l] + ci * elem_bytes;
              for (int32_t e = 0; e < elem_bytes; ++e) {
                if (dir) cp[e] = tp[e]; else tp[e] = cp[e];
              }
            }
  }
  return bad;
}
