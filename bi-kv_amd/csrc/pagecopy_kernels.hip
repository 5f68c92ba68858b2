// gfx950 kernels of the KV page-copy path. Pure data movement: every lane moves 16-byte vectors
// (global_load_dwordx4 / global_store_dwordx4) and a wavefront moves 1 KiB per instruction. No
// arithmetic on the payload, so the kernels are dtype-agnostic and bit-exact by construction (NaN
// payloads and fp8 bit patterns are never routed through a floating-point type).
//
// Semantics follow the reference's two kernels, block_per_page_copy_kernel and
// zero_copy_page_kernel (Bi-KV/SharedMemory/CUDA_Shared/copy_kernel.cu:9-36, 39-66):
//   dst[dst_off[i] + e] = src[src_off[i] + e]   for every run i and every byte e of the run.
// The reference moves one 2-byte scalar per thread per iteration with one 1024-thread block per
// page. Here the default movers (tile_move_wave_kernel for the layered pool, copy_runs_wave_kernel
// for the reference's runs) give every 1 KiB piece its own 64-lane workgroup, one vector per lane,
// with the piece's descriptor fetched by scalar loads: millions of tiny independent workgroups are
// what this GPU copies fastest with. The LDS-staged segment movers further down (a segment of pages
// per 256-lane workgroup, descriptors resolved once into LDS and broadcast) take the shapes the
// wave movers do not: tiles that are not 16-byte aligned, tiny tiles, misaligned pools.
#include "pagecopy_kernels.h"

#include <mutex>

namespace bikv {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int VW> struct VecOf;
template <> struct VecOf<16> { using T = u32x4; };
template <> struct VecOf<8> { using T = u32x2; };
template <> struct VecOf<4> { using T = uint32_t; };
template <> struct VecOf<2> { using T = uint16_t; };
template <> struct VecOf<1> { using T = uint8_t; };

// Every payload access goes through an explicit global-address-space pointer: addresses here are
// assembled from integers, and without the address space the compiler would have to emit flat_*
// instructions (which also probe the LDS and scratch apertures) instead of global_*.
#define BIKV_GLOBAL __attribute__((address_space(1)))

template <bool NT, class T>
__device__ __forceinline__ T ld(uint64_t addr) {
  const BIKV_GLOBAL T* p = (const BIKV_GLOBAL T*)addr;
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool NT, class T>
__device__ __forceinline__ void st(uint64_t addr, T v) {
  BIKV_GLOBAL T* p = (BIKV_GLOBAL T*)addr;
  if constexpr (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

// One 16-byte vector from s to d under a cache policy: 0 = default, 1 = nt on both accesses, 2 = nt
// plus system scope (sc1) on both. The last has no C++ spelling for 16-byte accesses, hence the two
// instructions written out; the load's result is awaited before the store reads it. Measured on
// MI355X against policy 1: +1.3 % on a linear copy, +1.8 % on random 16 KiB gathers.
template <int POL>
__device__ __forceinline__ void move16(uint64_t s, uint64_t d) {
  if constexpr (POL == 2) {
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1 nt\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(s) : "memory");
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" : : "v"(d), "v"(v) : "memory");
  } else {
    st<POL == 1, u32x4>(d, ld<POL == 1, u32x4>(s));
  }
}

// A value that is the same in every lane, moved to scalar registers so that the address of a
// vector access becomes (scalar base + per-lane offset).
__device__ __forceinline__ uint64_t uniform64(uint64_t x) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)x);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
  return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ void raise(uint32_t* status, int slot) {
  *reinterpret_cast<volatile uint32_t*>(status + slot) = 1u;
}

// ---------------------------------------------------------------------------------------------
// Layered tile move
// ---------------------------------------------------------------------------------------------

// Pool-side offset of byte `t` of a tile. A tile is contiguous in staging; in the pool it may be cut
// into rows that sit row_stride apart (the Worker's per-layer tensors [tokens, 2, heads, dim],
// Bi-KV/Worker/Worker.py:74-78, interleave K and V token by token: a (page, K|V) tile is block_tokens
// rows of heads*dim elements, two rows apart).
__device__ __forceinline__ uint64_t pool_offset(const TileClass& c, uint64_t t) {
  if (c.row_bytes == c.tile_bytes) return t;
  const uint64_t r = c.log2_row >= 0 ? t >> c.log2_row : t / (uint64_t)c.row_bytes;
  return r * (uint64_t)c.row_stride + (t - r * (uint64_t)c.row_bytes);
}

// Resolves the (pool address, staging address) pair of every page of this workgroup's segment
// into LDS. A tile that fails a bounds check gets a null pair and is skipped by the movers.
template <int DIR>
__device__ __forceinline__ int stage_descriptors(const TileClass& c, const MoveArgs& a,
                                                 uint32_t blk, uint64_t* s_pool,
                                                 uint64_t* s_stage, bool* any_bad) {
  const uint32_t q_rel = blk / c.segs_per_plane;
  const uint32_t sidx = blk - q_rel * c.segs_per_plane;
  const int64_t q = a.plane_begin + (int64_t)q_rel;
  const int64_t i0 = (int64_t)sidx * c.seg;
  const int64_t rem = a.n_batch - i0;
  const int nseg = rem < (int64_t)c.seg ? (int)rem : c.seg;
  const int tid = threadIdx.x;
  bool bad = false;
  if (tid < nseg) {
    const int64_t pid = a.page_ids[i0 + tid];
    const int64_t slot = a.slots[i0 + tid] + q * a.slot_strides[i0 + tid] - a.slot_bias;
    const bool bad_page = (uint64_t)pid >= (uint64_t)a.n_pool_pages;
    const bool bad_slot = (uint64_t)slot >= (uint64_t)c.n_slots;
    uint64_t pp = 0, sp = 0;
    if (bad_page) raise(a.status, ST_SLOT_PAGE);
    if (bad_slot) raise(a.status, DIR == 0 ? ST_SLOT_DST : ST_SLOT_SRC);
    if (!bad_page && !bad_slot) {
      pp = (uint64_t)(c.plane_base[q] + pid * c.page_stride);
      sp = (uint64_t)(c.staging + slot * c.tile_bytes);
    }
    s_pool[tid] = pp;
    s_stage[tid] = sp;
    bad = bad_page || bad_slot;
  }
  // also the barrier that publishes the descriptors
  *any_bad = __syncthreads_or(bad ? 1 : 0) != 0;
  return nseg;
}

// Fast mover: tiles are a power-of-two number of 4 KiB rows, everything is 16-byte aligned and
// every tile of the segment passed its bounds checks. The segment's tiles are walked as one flat
// sequence of rows, UNROLL rows at a time: UNROLL independent 16-byte loads per lane are issued
// back to back, then the UNROLL stores. An 8 KiB tile with UNROLL 4 therefore keeps two tiles in
// flight and a 64 KiB tile takes four passes. The loop body is branch-free so that the loads of one
// pass are never serialised behind each other.
template <int DIR, int UNROLL, bool NT>
__device__ __forceinline__ void move_rows(const TileClass& c, int nseg, const uint64_t* s_pool,
                                          const uint64_t* s_stage) {
  const int lr = c.log2_rows;
  const int mask = (1 << lr) - 1;
  const int total = nseg << lr;
  const int full = total & ~(UNROLL - 1);
  const uint32_t lane_off = threadIdx.x * 16u;
  for (int base = 0; base < full; base += UNROLL) {
    u32x4 v[UNROLL];
    uint64_t d[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int r = base + u;
      const int tt = r >> lr;
      const uint64_t row_off = (uint64_t)(r & mask) << 12;
      const uint64_t pool = uniform64(s_pool[tt]) + row_off;
      const uint64_t stg = uniform64(s_stage[tt]) + row_off;
      d[u] = DIR == 0 ? stg : pool;
      v[u] = ld<NT, u32x4>((DIR == 0 ? pool : stg) + lane_off);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) st<NT, u32x4>(d[u] + lane_off, v[u]);
  }
  for (int r = full; r < total; ++r) {
    const int tt = r >> lr;
    const uint64_t row_off = (uint64_t)(r & mask) << 12;
    const uint64_t pool = uniform64(s_pool[tt]) + row_off;
    const uint64_t stg = uniform64(s_stage[tt]) + row_off;
    st<NT, u32x4>((DIR == 0 ? stg : pool) + lane_off,
                  ld<NT, u32x4>((DIR == 0 ? pool : stg) + lane_off));
  }
}

// General mover: any tile size and alignment, VW-byte accesses (VW = the widest power of two that
// divides every base address, stride and the tile size). Used for the 32-byte scale tiles, for
// tiles that are not a whole number of 4 KiB rows, and for misaligned pools.
template <int DIR, int VW>
__device__ __forceinline__ void move_generic_vw(const TileClass& c, int nseg,
                                                const uint64_t* s_pool, const uint64_t* s_stage) {
  using T = typename VecOf<VW>::T;
  const uint32_t vpt = (uint32_t)(c.tile_bytes / VW);
  const uint32_t total = (uint32_t)nseg * vpt;  // the launcher keeps seg*vpt below 2^31
  for (uint32_t v = threadIdx.x; v < total; v += kBlock) {
    const uint32_t tt = v / vpt;
    const uint32_t ww = v - tt * vpt;
    const uint64_t pool = s_pool[tt];
    if (pool == 0) continue;
    const uint64_t stg = s_stage[tt];
    const uint64_t off = (uint64_t)ww * VW;
    const uint64_t poff = pool_offset(c, off);      // VW divides row_bytes and row_stride
    st<false, T>(DIR == 0 ? stg + off : pool + poff, ld<false, T>(DIR == 0 ? pool + poff : stg + off));
  }
}

template <int DIR>
__device__ __forceinline__ void move_generic(const TileClass& c, int nseg, const uint64_t* s_pool,
                                             const uint64_t* s_stage) {
  switch (c.vec_width) {
    case 16: move_generic_vw<DIR, 16>(c, nseg, s_pool, s_stage); break;
    case 8: move_generic_vw<DIR, 8>(c, nseg, s_pool, s_stage); break;
    case 4: move_generic_vw<DIR, 4>(c, nseg, s_pool, s_stage); break;
    case 2: move_generic_vw<DIR, 2>(c, nseg, s_pool, s_stage); break;
    default: move_generic_vw<DIR, 1>(c, nseg, s_pool, s_stage); break;
  }
}

// One launch moves both tile classes: workgroups [0, payload.n_blocks) take the payload,
// the rest take the scale tiles, so payload and scales of a page always travel together.
// Workgroup b of a class handles plane b / segs_per_plane and batch pages
// [(b % segs_per_plane)*seg, +seg): consecutive workgroups write consecutive staging ranges of one
// plane and read one plane's region of the pool.
template <int DIR, int UNROLL, bool NT, bool ROWS>
__global__ __launch_bounds__(kBlock) void tile_move_kernel(const MoveArgs a) {
  __shared__ uint64_t s_pool[kMaxSeg];
  __shared__ uint64_t s_stage[kMaxSeg];
  uint32_t blk = blockIdx.x;
  bool any_bad;
  if (blk < a.payload.n_blocks) {
    const int nseg = stage_descriptors<DIR>(a.payload, a, blk, s_pool, s_stage, &any_bad);
    if constexpr (ROWS) {
      // a segment holding a rejected tile takes the general mover, which skips null descriptors
      if (!any_bad) move_rows<DIR, UNROLL, NT>(a.payload, nseg, s_pool, s_stage);
      else move_generic<DIR>(a.payload, nseg, s_pool, s_stage);
    } else {
      move_generic<DIR>(a.payload, nseg, s_pool, s_stage);
    }
  } else {
    blk -= a.payload.n_blocks;
    const int nseg = stage_descriptors<DIR>(a.scale, a, blk, s_pool, s_stage, &any_bad);
    move_generic<DIR>(a.scale, nseg, s_pool, s_stage);
  }
}

template <int DIR, int UNROLL, bool NT>
static hipError_t launch_rows(const MoveArgs& a, uint32_t grid, hipStream_t s) {
  hipLaunchKernelGGL((tile_move_kernel<DIR, UNROLL, NT, true>), dim3(grid), dim3(kBlock), 0, s, a);
  return hipGetLastError();
}

template <int DIR>
static hipError_t launch_dir(const MoveArgs& a, bool rows, uint32_t grid, hipStream_t s) {
  if (!rows) {
    hipLaunchKernelGGL((tile_move_kernel<DIR, 1, false, false>), dim3(grid), dim3(kBlock), 0, s, a);
    return hipGetLastError();
  }
  const bool nt = tuning().nontemporal > 0 || (tuning().nontemporal < 0 && DIR == 0);
  switch (tuning().unroll) {
    case 1: return nt ? launch_rows<DIR, 1, true>(a, grid, s) : launch_rows<DIR, 1, false>(a, grid, s);
    case 2: return nt ? launch_rows<DIR, 2, true>(a, grid, s) : launch_rows<DIR, 2, false>(a, grid, s);
    case 8: return nt ? launch_rows<DIR, 8, true>(a, grid, s) : launch_rows<DIR, 8, false>(a, grid, s);
    default: return nt ? launch_rows<DIR, 4, true>(a, grid, s) : launch_rows<DIR, 4, false>(a, grid, s);
  }
}

// ---------------------------------------------------------------------------------------------
// Wave mover: the layout that measures fastest on MI355X for a pure copy — one 16-byte load and one
// 16-byte store per lane, one small workgroup (64 lanes = 1 KiB by default) per piece of a tile,
// millions of independent workgroups. Nothing is unrolled: with a single vector per lane the store
// of a wave follows its load immediately, reads and writes stay finely interleaved at the memory
// controllers, and the occupancy of the many tiny waves hides the latency.
//
// Grid: x = (batch page, piece of the tile), y = plane. The descriptor of a workgroup (page id,
// slot, slot stride, plane base) depends only on blockIdx, so it is fetched with scalar loads
// through the constant address space: the scalar cache does the broadcast that the LDS does in the
// segment movers above, without a barrier. Consecutive workgroups walk the pieces of one tile, then
// the next page of the same plane, so each plane's staging range is written front to back.
//
// Workgroups with blockIdx.x >= payload.n_blocks move the scale class (tiny tiles): one lane per
// vector, each lane fetching the descriptor of its own tile.
// ---------------------------------------------------------------------------------------------
#define BIKV_CONST __attribute__((address_space(4)))

template <class T>
__device__ __forceinline__ T cload(const T* p) {
  return *(const BIKV_CONST T*)(uint64_t)p;
}

template <int DIR, int VW>
__device__ __forceinline__ void move_one(uint64_t pool, uint64_t stg) {
  using T = typename VecOf<VW>::T;
  st<false, T>(DIR == 0 ? stg : pool, ld<false, T>(DIR == 0 ? pool : stg));
}

template <int DIR, int POL, int B>
__global__ __launch_bounds__(B) void tile_move_wave_kernel(const MoveArgs a) {
  const uint32_t bx = blockIdx.x;
  // pieces per tile: 2^lp when lp >= 0 (shift and mask), else n_parts (one uniform division per wave)
  const int32_t lp = a.payload.log2_rows;
  const uint32_t np = a.payload.n_parts;
  const bool payload = bx < a.payload.n_blocks;
  const uint32_t bt = payload ? (lp >= 0 ? bx >> lp : bx / np) : 0u;   // x index without the piece
  // Two walks over the same (page, plane, piece) space, chosen by the launcher:
  //   order 0: x = (page, piece), y = plane — one plane at a time, pages in batch order
  //   order 1: x = (plane, page within a chunk of 2^lc pages, piece), (y, z) = chunk — the planes of
  //            a few pages together: neighbouring workgroups touch pool planes gigabytes apart
  //            while each still writes runs of 2^lc tiles
  const uint32_t lc = (uint32_t)a.log2_chunk;
  int64_t q;
  uint32_t i;
  if (a.order == 0) {
    q = a.plane_begin + (int64_t)blockIdx.y;
    i = bt;
  } else {
    const uint64_t chunk = (uint64_t)blockIdx.y + (uint64_t)blockIdx.z * gridDim.y;
    const uint32_t t = bt;
    const uint64_t page = (chunk << lc) + (t & ((1u << lc) - 1u));
    if (page >= (uint64_t)a.n_batch) return;
    i = (uint32_t)page;
    q = a.plane_begin + (int64_t)(t >> lc);
  }
  if (payload) {
    const uint32_t part = lp >= 0 ? (bx & ((1u << lp) - 1u)) : bx - bt * np;
    const int64_t pid = cload(a.page_ids + i);
    const int64_t slot = cload(a.slots + i) + q * cload(a.slot_strides + i) - a.slot_bias;
    const uint64_t plane = (uint64_t)cload(a.payload.plane_base + q);  // issued with the others
    const bool bad_page = (uint64_t)pid >= (uint64_t)a.n_pool_pages;
    const bool bad_slot = (uint64_t)slot >= (uint64_t)a.payload.n_slots;
    if (bad_page || bad_slot) {
      if (threadIdx.x == 0 && part == 0) {
        if (bad_page) raise(a.status, ST_SLOT_PAGE);
        if (bad_slot) raise(a.status, DIR == 0 ? ST_SLOT_DST : ST_SLOT_SRC);
      }
      return;
    }
    const uint64_t pool = plane + (uint64_t)(pid * a.payload.page_stride);
    const uint64_t stg = (uint64_t)a.payload.staging + (uint64_t)(slot * a.payload.tile_bytes);
    const uint64_t off = (uint64_t)part * (B * 16u) + threadIdx.x * 16u;
    if (off < (uint64_t)a.payload.tile_bytes) { // the last piece of a tile may be ragged
      const uint64_t poff = pool_offset(a.payload, off);   // 16 divides row_bytes and row_stride
      move16<POL>(DIR == 0 ? pool + poff : stg + off, DIR == 0 ? stg + off : pool + poff);
    }
  } else {
    // scale class: one lane per vector; order 0 spreads the lanes over the pages of plane q,
    // order 1 over the planes of page i. The launcher keeps (scale workgroups * B) below 2^32.
    const uint32_t vpt = a.scale.segs_per_plane;  // vectors per scale tile (wave mover's meaning)
    const uint32_t v = (bx - a.payload.n_blocks) * (uint32_t)B + threadIdx.x;
    const uint32_t t = v / vpt;
    const uint32_t w = v - t * vpt;
    if (a.order == 0) {
      if ((uint64_t)t >= (uint64_t)a.n_batch) return;
      i = t;
    } else {
      const uint64_t chunk = (uint64_t)blockIdx.y + (uint64_t)blockIdx.z * gridDim.y;
      const uint64_t page = (chunk << lc) + (t & ((1u << lc) - 1u));
      if ((t >> lc) >= (uint32_t)a.plane_count || page >= (uint64_t)a.n_batch) return;
      i = (uint32_t)page;
      q = a.plane_begin + (int64_t)(t >> lc);
    }
    const int64_t pid = a.page_ids[i];
    const int64_t slot = a.slots[i] + q * a.slot_strides[i] - a.slot_bias;
    const bool bad_page = (uint64_t)pid >= (uint64_t)a.n_pool_pages;
    const bool bad_slot = (uint64_t)slot >= (uint64_t)a.scale.n_slots;
    if (bad_page) raise(a.status, ST_SLOT_PAGE);
    if (bad_slot) raise(a.status, DIR == 0 ? ST_SLOT_DST : ST_SLOT_SRC);
    if (bad_page || bad_slot) return;
    const uint64_t off = (uint64_t)w * (uint64_t)a.scale.vec_width;
    const uint64_t pool = (uint64_t)a.scale.plane_base[q] + (uint64_t)(pid * a.scale.page_stride) + off;
    const uint64_t stg = (uint64_t)a.scale.staging + (uint64_t)(slot * a.scale.tile_bytes) + off;
    switch (a.scale.vec_width) {
      case 16: move_one<DIR, 16>(pool, stg); break;
      case 8: move_one<DIR, 8>(pool, stg); break;
      case 4: move_one<DIR, 4>(pool, stg); break;
      case 2: move_one<DIR, 2>(pool, stg); break;
      default: move_one<DIR, 1>(pool, stg); break;
    }
  }
}

// How the wave mover walks a batch, and whether it marks its accesses non-temporal. Measured on
// MI355X with 8-64 KiB tiles and 56-160 planes of 2 GiB each:
//   * random accesses confined to ONE plane's few GiB run ~10 % slower than the same accesses spread
//     over all planes (6.3 vs 5.7 TB/s for scattered writes), so the pool side wants neighbouring
//     workgroups on different planes (order 1);
//   * the dense side wants runs: with a page-major staging image the planes of one page are already
//     adjacent (chunk of 1 page); with a layer-major image a scatter reads runs of 64 tiles per
//     plane (64 beat 16 by 1-1.5 % on pools spread over both halves of HBM and is within 0.4 % on
//     others; 256 helps 16 KiB tiles and hurts 8 KiB ones), and a gather — whose dense side is the WRITTEN one — does best writing each plane's
//     range front to back (order 0);
//   * the nt hint helps every case above, nt with system scope (policy 2 of move16) another 1-3 %;
//     without a layout hint hints are kept off for scatters, where nt is neutral to slightly
//     negative in order 0.
struct WavePolicy {
  int order, log2_chunk;
  int nt;   // cache policy of move16: 0, 1 or 2
};

static WavePolicy choose_wave_policy(int dir, int layout_hint) {
  WavePolicy p;
  if (layout_hint == 2) {          // page-major staging image
    p = {1, 0, 2};
  } else if (layout_hint == 1) {   // layer-major staging image
    p = dir == 0 ? WavePolicy{0, 0, 2} : WavePolicy{1, 6, 2};
  } else {
    p = {0, 0, dir == 0 ? 2 : 0};
  }
  const Tuning& t = tuning();
  if (t.order >= 0) p.order = t.order;
  if (t.log2_chunk >= 0) p.log2_chunk = t.log2_chunk;
  if (t.nontemporal >= 0) p.nt = t.nontemporal == 4 ? 2 : (t.nontemporal != 0 ? 1 : 0);
  return p;
}

template <int DIR, int B>
static hipError_t launch_wave_b(const MoveArgs& a, int nt, dim3 grid, hipStream_t s) {
  if (nt == 2)
    hipLaunchKernelGGL((tile_move_wave_kernel<DIR, 2, B>), grid, dim3(B), 0, s, a);
  else if (nt == 1)
    hipLaunchKernelGGL((tile_move_wave_kernel<DIR, 1, B>), grid, dim3(B), 0, s, a);
  else
    hipLaunchKernelGGL((tile_move_wave_kernel<DIR, 0, B>), grid, dim3(B), 0, s, a);
  return hipGetLastError();
}

template <int DIR>
static hipError_t launch_wave(const MoveArgs& a, int block, int nt, dim3 grid, hipStream_t s) {
  switch (block) {
    case 128: return launch_wave_b<DIR, 128>(a, nt, grid, s);
    case 256: return launch_wave_b<DIR, 256>(a, nt, grid, s);
    default: return launch_wave_b<DIR, 64>(a, nt, grid, s);
  }
}

// The wave mover takes any payload made of 16-byte aligned tiles of at least half a piece
// (piece = block*16 bytes); smaller or misaligned tiles go to the segment movers.
// Returns false when the shape does not qualify.
static bool plan_wave(MoveArgs& a, int block, int order, int log2_chunk, dim3* grid) {
  const int64_t piece = (int64_t)block * 16;
  TileClass& p = a.payload;
  if (p.vec_width != 16 || p.tile_bytes % 16 != 0 || p.tile_bytes * 2 < piece) return false;
  const int64_t parts = (p.tile_bytes + piece - 1) / piece;
  if (parts >= (int64_t(1) << 31)) return false;
  int lp = -1;
  if ((parts & (parts - 1)) == 0) {
    lp = 0;
    while ((int64_t(1) << lp) < parts) ++lp;
  }
  // order 0: x walks the batch pages of one plane; order 1: x walks the planes of one page
  if (order == 0) log2_chunk = 0;
  const int64_t walk = order == 0 ? a.n_batch : ((int64_t)a.plane_count << log2_chunk);
  const int64_t px = walk * parts;
  int64_t sx = 0;
  if (a.scale.tile_bytes > 0) {
    const int64_t vpt = a.scale.tile_bytes / a.scale.vec_width;
    if (vpt >= (int64_t(1) << 31)) return false;
    a.scale.segs_per_plane = (uint32_t)vpt;
    sx = (walk * vpt + block - 1) / block;
  }
  if (px + sx >= (int64_t(1) << 32) / block) return false;
  if (order == 0) {
    if (a.plane_count > 65535) return false;
    *grid = dim3((uint32_t)(px + sx), (uint32_t)a.plane_count, 1);
  } else {
    const int64_t chunks = (a.n_batch + (int64_t(1) << log2_chunk) - 1) >> log2_chunk;
    const int64_t gy = chunks < 32768 ? chunks : 32768;
    const int64_t gz = (chunks + gy - 1) / gy;
    if (gz > 65535) return false;
    *grid = dim3((uint32_t)(px + sx), (uint32_t)gy, (uint32_t)gz);
  }
  p.log2_rows = lp;
  p.n_parts = (uint32_t)parts;
  p.n_blocks = (uint32_t)px;
  a.scale.n_blocks = (uint32_t)sx;
  a.order = order;
  a.log2_chunk = log2_chunk;
  return true;
}

// Picks the number of batch pages per workgroup: enough bytes per workgroup to amortise the
// descriptor staging, but never so few workgroups that 256 CUs are left idle.
static int choose_seg(int forced, int64_t n_batch, int plane_count, int64_t tile_bytes,
                      int64_t units_per_tile) {
  int seg;
  if (forced > 0) {
    seg = forced;
  } else {
    // aim at ~256 KiB per workgroup
    int64_t want = (256 * 1024) / (tile_bytes > 0 ? tile_bytes : 1);
    if (want < 1) want = 1;
    seg = 1;
    while (seg * 2 <= want && seg * 2 <= kMaxSeg) seg *= 2;
    // keep at least ~8 workgroups per CU in the grid when the batch allows it
    const int64_t min_blocks = 8 * 256;
    while (seg > 1 && ((n_batch + seg - 1) / seg) * plane_count < min_blocks) seg /= 2;
  }
  if (seg > kMaxSeg) seg = kMaxSeg;
  if (seg < 1) seg = 1;
  while (seg > 1 && (int64_t)seg * units_per_tile >= (int64_t(1) << 31)) seg /= 2;
  return seg;
}

static bool finish_class(TileClass& c, int forced_seg, int64_t n_batch, int plane_count) {
  if (c.tile_bytes <= 0) { c.n_blocks = 0; c.seg = 1; c.segs_per_plane = 0; return true; }
  const int64_t units = c.tile_bytes / c.vec_width;
  if (units >= (int64_t(1) << 31)) return false;
  c.seg = choose_seg(forced_seg, n_batch, plane_count, c.tile_bytes, units);
  const int64_t spp = (n_batch + c.seg - 1) / c.seg;
  const int64_t nb = spp * plane_count;
  if (nb >= (int64_t(1) << 31)) return false;
  c.segs_per_plane = (uint32_t)spp;
  c.n_blocks = (uint32_t)nb;
  return true;
}

hipError_t launch_tile_move(int dir, MoveArgs& a, hipStream_t stream) {
  if (a.n_batch <= 0 || a.plane_count <= 0) return hipSuccess;
  refresh_tuning();
  if (tuning().seg == 0) {
    // default: the wave mover, whenever the payload shape qualifies
    dim3 grid;
    const WavePolicy pol = choose_wave_policy(dir, a.layout_hint);
    if (plan_wave(a, tuning().wave_block, pol.order, pol.log2_chunk, &grid))
      return dir == 0 ? launch_wave<0>(a, tuning().wave_block, pol.nt, grid, stream)
                      : launch_wave<1>(a, tuning().wave_block, pol.nt, grid, stream);
  }
  if (!finish_class(a.payload, tuning().seg, a.n_batch, a.plane_count)) return hipErrorInvalidValue;
  // scale tiles are tiny: pack as many pages per workgroup as LDS descriptors allow
  if (a.scale.tile_bytes > 0) {
    if (!finish_class(a.scale, kMaxSeg, a.n_batch, a.plane_count)) return hipErrorInvalidValue;
  } else {
    a.scale.n_blocks = 0;
  }
  const uint64_t grid = (uint64_t)a.payload.n_blocks + a.scale.n_blocks;
  if (grid == 0) return hipSuccess;
  if (grid >= (uint64_t(1) << 31) / kBlock * 2) return hipErrorInvalidValue;  // grid*block < 2^32
  // fast mover: 16-byte aligned tiles of 2^k rows of 4 KiB
  const int64_t nrows = a.payload.tile_bytes / kRowBytes;
  const bool rows = a.payload.vec_width == 16 && (a.payload.tile_bytes % kRowBytes) == 0 &&
                    (nrows & (nrows - 1)) == 0 && a.payload.row_bytes == a.payload.tile_bytes;
  a.payload.log2_rows = 0;
  if (rows)
    while ((int64_t(1) << a.payload.log2_rows) < nrows) ++a.payload.log2_rows;
  return dir == 0 ? launch_dir<0>(a, rows, (uint32_t)grid, stream)
                  : launch_dir<1>(a, rows, (uint32_t)grid, stream);
}

// ---------------------------------------------------------------------------------------------
// Run copy (reference API)
// ---------------------------------------------------------------------------------------------

template <int VW>
__device__ __forceinline__ void copy_span_vw(uint64_t s, uint64_t d, int64_t bytes) {
  using T = typename VecOf<VW>::T;
  const int64_t n = bytes / VW;
  for (int64_t i = threadIdx.x; i < n; i += kBlock)
    st<false, T>(d + (uint64_t)i * VW, ld<false, T>(s + (uint64_t)i * VW));
  const int64_t done = n * VW;
  for (int64_t i = done + threadIdx.x; i < bytes; i += kBlock)
    st<false, uint8_t>(d + (uint64_t)i, ld<false, uint8_t>(s + (uint64_t)i));
}

// Small runs (below 1 KiB by default): one lane per 16-byte piece, many runs per workgroup.
template <bool NT>
__global__ __launch_bounds__(kBlock) void copy_small_runs_kernel(const RunArgs a,
                                                                 uint32_t pieces_per_run,
                                                                 int64_t total_pieces) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= total_pieces) return;
  const int64_t run = p / pieces_per_run;
  const int64_t piece = p - run * pieces_per_run;
  const int64_t so_u = a.src_off[run];
  const int64_t do_u = a.dst_off[run];
  const int64_t so = so_u * a.unit_bytes;
  const int64_t dof = do_u * a.unit_bytes;
  const bool bad_src = so_u < 0 || so < 0 || so > a.src_bytes - a.run_bytes;
  const bool bad_dst = do_u < 0 || dof < 0 || dof > a.dst_bytes - a.run_bytes;
  if (bad_src) raise(a.status, ST_SLOT_SRC);
  if (bad_dst) raise(a.status, ST_SLOT_DST);
  if (bad_src || bad_dst) return;
  const int64_t lo = piece << 4;
  const int64_t n = a.run_bytes - lo < 16 ? a.run_bytes - lo : 16;
  const uint64_t s = (uint64_t)(a.src + so + lo);
  const uint64_t d = (uint64_t)(a.dst + dof + lo);
  if (n == 16 && (((s | d) & 15) == 0)) {
    st<NT, u32x4>(d, ld<NT, u32x4>(s));
  } else {
    for (int64_t i = 0; i < n; ++i)
      st<false, uint8_t>(d + (uint64_t)i, ld<false, uint8_t>(s + (uint64_t)i));
  }
}

// Moves up to 16 bytes between two addresses of any alignment with the widest accesses both allow.
__device__ __forceinline__ void move_upto16(uint64_t s, uint64_t d, int n) {
  const uint64_t al = s | d;
  int done = 0;
  if ((al & 7) == 0) {
    for (; done + 8 <= n; done += 8) st<false, u32x2>(d + done, ld<false, u32x2>(s + done));
  } else if ((al & 3) == 0) {
    for (; done + 4 <= n; done += 4) st<false, uint32_t>(d + done, ld<false, uint32_t>(s + done));
  } else if ((al & 1) == 0) {
    for (; done + 2 <= n; done += 2) st<false, uint16_t>(d + done, ld<false, uint16_t>(s + done));
  }
  for (; done < n; ++done) st<false, uint8_t>(d + done, ld<false, uint8_t>(s + done));
}

// Large runs, wave style (same shape as the wave mover above): grid x = 1 KiB piece of the run,
// (y, z) = run; one 16-byte vector per lane; the run's two offsets come in through scalar loads.
// A run whose addresses are not 16-byte aligned, and the ragged end of a run, fall back to narrower
// accesses lane by lane.
// `group_shift` >= 0 packs 2^group_shift runs into one row of the grid (x = run in group, piece;
// pieces per run = 2^piece_shift): rows of only a few workgroups dispatch slowly (runs of 2-8 pieces
// were capped near 4.85 TB/s whatever the kernel did).
template <bool NTL, bool NTS, int B, bool STREAM = false>
__global__ __launch_bounds__(B) void copy_runs_wave_kernel(const RunArgs a, int piece_shift,
                                                           int group_shift) {
  uint64_t run = (uint64_t)blockIdx.y + (uint64_t)blockIdx.z * gridDim.y;
  uint32_t piece = blockIdx.x;
  if (group_shift >= 0) {
    run = (run << group_shift) + (blockIdx.x >> piece_shift);
    piece = blockIdx.x & ((1u << piece_shift) - 1u);
  }
  if (run >= (uint64_t)a.n_runs) return;
  const int64_t so_u = cload(a.src_off + run);
  const int64_t do_u = cload(a.dst_off + run);
  const int64_t so = so_u * a.unit_bytes;
  const int64_t dof = do_u * a.unit_bytes;
  // ragged runs: this run's own length (a length outside [0, run_bytes] skips the run and is
  // reported as a source-range fault)
  int64_t rb = a.run_bytes;
  bool bad_len = false;
  if (a.run_lens) {
    const int64_t len_u = cload(a.run_lens + run);
    rb = len_u * a.unit_bytes;
    bad_len = len_u < 0 || rb < 0 || rb > a.run_bytes;
    if (bad_len) rb = 0;
  }
  const bool bad_src = bad_len || so_u < 0 || so < 0 || so > a.src_bytes - rb;
  const bool bad_dst = do_u < 0 || dof < 0 || dof > a.dst_bytes - rb;
  if (bad_src || bad_dst) {
    if (threadIdx.x == 0 && piece == 0) {
      if (bad_src) raise(a.status, ST_SLOT_SRC);
      if (bad_dst) raise(a.status, ST_SLOT_DST);
    }
    return;
  }
  const int64_t lo = (int64_t)piece * (B * 16) + threadIdx.x * 16;
  if (lo >= rb) return;
  const uint64_t s = (uint64_t)(a.src + so + lo);
  const uint64_t d = (uint64_t)(a.dst + dof + lo);
  const int64_t left = rb - lo;
  if (left >= 16 && ((s | d) & 15) == 0) {
    if constexpr (STREAM) move16<2>(s, d);
    else st<NTS, u32x4>(d, ld<NTL, u32x4>(s));
  } else {
    move_upto16(s, d, left < 16 ? (int)left : 16);
  }
}

template <int B>
static hipError_t launch_runs_wave(const RunArgs& a, hipStream_t stream) {
  const int64_t piece = (int64_t)B * 16;
  int64_t gx = (a.run_bytes + piece - 1) / piece;
  if (gx >= (int64_t(1) << 32) / B) return hipErrorInvalidValue;
  int64_t rows = a.n_runs;
  int piece_shift = 0, group_shift = -1;
  if (gx < 256 && (gx & (gx - 1)) == 0 && tuning().run_group != 0) {
    while ((int64_t(1) << piece_shift) < gx) ++piece_shift;
    group_shift = 0;
    while ((gx << group_shift) < 1024 && (int64_t(1) << group_shift) < a.n_runs) ++group_shift;
    rows = (a.n_runs + (int64_t(1) << group_shift) - 1) >> group_shift;
    gx <<= group_shift;
  }
  const int64_t gy = rows < 32768 ? rows : 32768;
  const int64_t gz = (rows + gy - 1) / gy;
  if (gz > 65535) return hipErrorInvalidValue;
  const dim3 grid((uint32_t)gx, (uint32_t)gy, (uint32_t)gz);
  const int nt = tuning().nontemporal;   // -1/1 both sides, 0 none, 2 loads only, 3 stores only, 4 sc1 nt
  if (nt == 4 || nt < 0)
    hipLaunchKernelGGL((copy_runs_wave_kernel<true, true, B, true>), grid, dim3(B), 0, stream, a, piece_shift, group_shift);
  else if (nt == 0)
    hipLaunchKernelGGL((copy_runs_wave_kernel<false, false, B>), grid, dim3(B), 0, stream, a, piece_shift, group_shift);
  else if (nt == 2)
    hipLaunchKernelGGL((copy_runs_wave_kernel<true, false, B>), grid, dim3(B), 0, stream, a, piece_shift, group_shift);
  else if (nt == 3)
    hipLaunchKernelGGL((copy_runs_wave_kernel<false, true, B>), grid, dim3(B), 0, stream, a, piece_shift, group_shift);
  else
    hipLaunchKernelGGL((copy_runs_wave_kernel<true, true, B>), grid, dim3(B), 0, stream, a, piece_shift, group_shift);
  return hipGetLastError();
}

hipError_t launch_copy_runs(const RunArgs& a, hipStream_t stream) {
  if (a.n_runs <= 0 || a.run_bytes <= 0) return hipSuccess;
  refresh_tuning();
  const int64_t small_max = tuning().small_run_max;
  if (a.run_lens || a.run_bytes > small_max) {
    switch (tuning().wave_block) {
      case 128: return launch_runs_wave<128>(a, stream);
      case 256: return launch_runs_wave<256>(a, stream);
      default: return launch_runs_wave<64>(a, stream);
    }
  }
  const int64_t ppr = (a.run_bytes + 15) >> 4;
  const int64_t total = ppr * a.n_runs;
  const int64_t grid = (total + kBlock - 1) / kBlock;
  if (grid >= (int64_t(1) << 24)) return hipErrorInvalidValue;
  if (tuning().nontemporal != 0)
    hipLaunchKernelGGL(copy_small_runs_kernel<true>, dim3((uint32_t)grid), dim3(kBlock), 0, stream, a,
                       (uint32_t)ppr, total);
  else
    hipLaunchKernelGGL(copy_small_runs_kernel<false>, dim3((uint32_t)grid), dim3(kBlock), 0, stream, a,
                       (uint32_t)ppr, total);
  return hipGetLastError();
}

// A plain copy of `bytes` bytes between two 16-byte aligned addresses in the wave movers' shape (one
// 16-byte vector per lane, 64-lane workgroups, nt + system scope): the hop between a stager's lane buffer
// and the mapped pinned image when the library moves those bytes itself.
__global__ __launch_bounds__(64) void linear_copy_kernel(const char* src, char* dst, int64_t bytes) {
  const int64_t lo = ((int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x) * 1024 + threadIdx.x * 16;
  if (lo >= bytes) return;
  const int64_t left = bytes - lo;
  if (left >= 16) move16<2>((uint64_t)(src + lo), (uint64_t)(dst + lo));
  else move_upto16((uint64_t)(src + lo), (uint64_t)(dst + lo), (int)left);
}

hipError_t launch_linear_copy(const void* src, void* dst, int64_t bytes, hipStream_t stream) {
  if (bytes <= 0) return hipSuccess;
  if ((((uint64_t)src | (uint64_t)dst) & 15) != 0) return hipErrorInvalidValue;
  const int64_t groups = (bytes + 1023) / 1024;
  const int64_t gx = groups < 65536 ? groups : 65536;
  const int64_t gy = (groups + gx - 1) / gx;
  if (gy > 65535) return hipErrorInvalidValue;
  hipLaunchKernelGGL(linear_copy_kernel, dim3((uint32_t)gx, (uint32_t)gy), dim3(64), 0, stream,
                     static_cast<const char*>(src), static_cast<char*>(dst), bytes);
  return hipGetLastError();
}

// Launch knobs: one shared copy that the setters change under a mutex, and one snapshot per thread that
// a launch takes when it begins and reads from then on.
static std::mutex g_tuning_mu;
static Tuning g_tuning;
static thread_local Tuning t_tuning;

std::mutex& tuning_mutex() { return g_tuning_mu; }
Tuning& tuning_shared() { return g_tuning; }
const Tuning& tuning() { return t_tuning; }
void refresh_tuning() {
  std::lock_guard<std::mutex> lk(g_tuning_mu);
  t_tuning = g_tuning;
}

}  // namespace bikv
