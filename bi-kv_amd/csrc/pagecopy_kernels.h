// Internal launch interface between the C ABI (pagecopy_abi.hip, ipc_ring.hip) and the gfx950
// kernels (pagecopy_kernels.hip). Not installed; the public surface is include/bikv_pagecopy.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

namespace bikv {

// Status slots written by kernels (one 32-bit word per condition, plain stores of 1, so no
// atomics are needed on the host-mapped status block).
enum : int { ST_SLOT_SRC = 0, ST_SLOT_DST = 1, ST_SLOT_PAGE = 2, ST_SLOTS = 8 };

// One tile class of a layered pool as the kernels see it.
struct TileClass {
  const char* const* plane_base;  // device-resident table, n_planes entries
  char* staging;                  // slot 0 of the staging window
  int64_t n_slots;                // slots available in the staging window
  int64_t tile_bytes;
  int64_t page_stride;
  int64_t row_bytes;              // pool side: the tile is tile_bytes/row_bytes rows of row_bytes bytes,
  int64_t row_stride;             // row_stride apart (row_bytes == tile_bytes: one contiguous tile)
  int32_t log2_row;               // log2(row_bytes) when that is a power of two, else -1
  int32_t vec_width;              // widest power of two (<=16) dividing every address and size
  int32_t log2_rows;              // segment mover: tile_bytes == 4096 << log2_rows; wave mover: pieces
                                  // per tile == 1 << log2_rows, or -1 when that is not a power of two
  uint32_t n_parts;               // wave mover: pieces per tile
  int32_t seg;                    // batch pages per workgroup
  uint32_t segs_per_plane;        // ceil(n_batch / seg)
  uint32_t n_blocks;              // plane_count * segs_per_plane
};

struct MoveArgs {
  TileClass payload;
  TileClass scale;                // n_blocks == 0 when the pool has no scale class
  const int64_t* page_ids;
  const int64_t* slots;
  const int64_t* slot_strides;
  int64_t n_batch;
  int64_t n_pool_pages;
  int64_t slot_bias;
  int32_t plane_begin;
  int32_t plane_count;
  int32_t order;                  // wave mover: 0 = plane by plane, 1 = page chunk by page chunk
  int32_t log2_chunk;             // order 1: pages per chunk = 2^log2_chunk
  int32_t layout_hint;            // host side only: 0 none, 1 layer-major, 2 page-major staging
  uint32_t* status;
};

struct Tuning {
  int seg = 0;          // 0 = wave mover when the shape qualifies, else segment movers with an
                        // automatic segment; > 0 = segment movers with this many pages per workgroup
  int wave_block = 64;  // lanes per workgroup of the wave mover (64, 128 or 256)
  int order = -1;       // wave mover walk: 0 = plane by plane, 1 = chunk of pages by chunk of pages,
                        // -1 = chosen from the batch's layout hint
  int log2_chunk = -1;  // order 1: 2^log2_chunk pages per chunk; -1 = chosen
  int unroll = 4;       // 16-byte vectors in flight per lane (1, 2, 4 or 8)
  int nontemporal = -1; // cache policy of payload accesses: 0 none, 1 nt, 4 nt + system scope,
                        // -1 = chosen per direction and layout (run copy also: 2 loads, 3 stores only)
  int run_group = 1;           // wave run kernel: several short runs share one grid row (0 = off)
  int small_run_max = 1023;    // runs up to this many bytes go to the one-lane-per-piece kernel
  int transpose_lds_kib = 60;  // LDS tile budget of the layout-change kernels, KiB
  int transpose_dsplit = 0;    // slices of head_dim per tile; 0 = default (1: whole compute rows)
  int transpose_pairs = 1;     // the K/V-pair kernel where the shape allows (0 = element-wise kernel)
  int transpose_block = 0;     // lanes per workgroup of the K/V-pair kernel: 128, 256, 512, 1024;
                               // 0 = chosen per direction (256 for the load, 512 for the store)
  int transpose_sc1 = 1;       // K/V-pair kernel: payload stores are nt with system scope (0 = nt only)
  int transpose_kvswap = 0;    // K/V-pair kernel: 1 = whole-KiB compute-side accesses by exchanging half-waves, where
                               // the pool's shape allows; 0 = every lane addresses its own K and V rows (default:
                               // measured, the exchange costs the store 1.7 % and gains the load 0.6 %)
  int debug_unique = 0;        // 1 = scattering entry points check their destination ids on the host first
};
// The knobs are process-wide and may be set from any thread. Setters change the shared copy under
// tuning_mutex(); every launch first copies it into a snapshot of the calling thread (refresh_tuning) and
// reads only that (tuning()), so one launch sees one consistent set of knobs whatever is set meanwhile.
std::mutex& tuning_mutex();
Tuning& tuning_shared();
const Tuning& tuning();
void refresh_tuning();

constexpr int kBlock = 256;      // 4 wavefronts
constexpr int kMaxSeg = 256;     // LDS descriptor slots per workgroup
constexpr int kRowBytes = kBlock * 16;  // one 16-byte vector per lane

// dir: 0 = gather (pool -> staging), 1 = scatter (staging -> pool).
hipError_t launch_tile_move(int dir, MoveArgs& a, hipStream_t stream);

struct RunArgs {
  const char* src;
  char* dst;
  int64_t src_bytes;
  int64_t dst_bytes;
  const int64_t* src_off;
  const int64_t* dst_off;
  int64_t n_runs;
  int64_t run_bytes;              // every run (run_lens null) or the longest run allowed
  int64_t unit_bytes;
  const int64_t* run_lens;        // nullable, device: length of each run in units (ragged runs)
  uint32_t* status;
};
hipError_t launch_copy_runs(const RunArgs& a, hipStream_t stream);
// Plain copy of `bytes` bytes between two 16-byte aligned device-visible addresses (either may be mapped
// pinned host memory).
hipError_t launch_linear_copy(const void* src, void* dst, int64_t bytes, hipStream_t stream);

// Fused page move + layout change between token-major pages and a per-layer paged NHD pool.
struct TransposeArgs {
  const char* const* layer_base;  // device-resident table, n_layers entries
  char* tm_base;                  // token-major side: pages of block_tokens tokens
  const int64_t* block_ids;       // compute-side block of each page
  const int64_t* tm_pages;        // token-major page index of each page
  int64_t n_pages;
  int64_t n_blocks;               // compute-side blocks (bounds check)
  int64_t n_tm_pages;             // token-major pages available (bounds check)
  int64_t block_stride, kv_stride, token_stride;  // compute side, in elements
  int32_t n_layers, head_dim, n_cols;             // n_cols = kv_heads * n_layers * 2
  int32_t block_tokens, elem_bytes;
  int32_t chunk_cols, chunk_rows, pitch;      // filled by the launcher
  int32_t swz_mask;                           // pair kernel: XOR mask of the 16-byte groups of an LDS row
  uint32_t n_chunks, n_dchunks, tile_words;
  // pair kernel, filled by the launcher: multipliers that replace divisions (m = ceil(2^32 / n), 0 for
  // n = 1) and the per-step advance of its two index walks for the chosen workgroup size
  uint32_t n_heads, m_heads, m_layers, m_vpr, m_dgs, m_chunks;
  uint32_t q_tm, r_tm, q_cp, r_cp;
  uint32_t sys_scope;             // payload stores carry system scope besides nt
  uint32_t kv_swap;               // pair kernel: K and V rows of a (token, layer) are the halves of one KiB and a
                                  // half-wave covers a layer's K rows: compute-side accesses exchange half-waves
  uint32_t* status;
};
// dir 0: compute -> token-major, dir 1: token-major -> compute.
hipError_t launch_transpose_pages(int dir, TransposeArgs& a, hipStream_t stream);

}  // namespace bikv
