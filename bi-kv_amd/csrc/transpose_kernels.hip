// Fused page move + layout change between Bi-KV's two KV layouts, which the reference never converts:
//
//   token-major (storage / transfer): one token = [head_dim D][kv_heads H][layers L][2] elements,
//     Bi-KV/Model/qwen2.py:519-522 (token_shape), pools (tokens,)+token_shape at
//     Bi-KV/DistributedStorage/kvcache.py:38-43 and Bi-KV/Worker/Worker.py:57-62;
//   per-layer paged NHD (compute): L tensors addressed (block, kv, token, head, d) with D contiguous,
//     [blocks*block, 2, H, D] at Bi-KV/Worker/Worker.py:74-78 and [blocks, 2, block, H, D] at
//     Bi-KV/Model/qwen2.py:532-536 (the layout flashinfer's paged prefill reads).
//
// Per token this is the transpose of a [D][C] matrix (C = H*L*2, column c = (h*L + l)*2 + k) into
// C rows of D contiguous elements, each row landing in its own layer tensor. A workgroup stages one
// token (or a column chunk [D][Cc] of it when the token exceeds the LDS budget) in LDS; both sides move
// 16-byte vectors in global memory. Two kernels:
//   transpose_pairs_kernel (the default): K and V of one (head, layer) are neighbouring columns, so a
//     token-major row is a sequence of units {K[d], V[d]} and the layout change is a transpose of UNITS
//     plus a split / join of their halves in registers (v_perm_b32, or register selection for 4-byte
//     elements). The tile lies in LDS transposed, [column pair][d], unpadded, with the 16-byte groups of
//     a row XOR-swizzled so that the 16-byte accesses along d stay whole and the unit accesses of the
//     token-major side spread over all banks. No integer division: index splits are multiplications
//     by launch-time constants and incremental walks.
//   transpose_pages_kernel (the first version, selectable with transpose_pairs = 0 and kept as a second
//     implementation for the tests): element-wise LDS accesses, the compute side assembled from (or
//     split into) single elements, LDS pitch padded by 4 bytes.
#include "pagecopy_kernels.h"

namespace bikv {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define BIKV_GLOBAL __attribute__((address_space(1)))
#define BIKV_CONST __attribute__((address_space(4)))

template <class T>
__device__ __forceinline__ T tload(const T* p) {
  return *(const BIKV_CONST T*)(uint64_t)p;
}

template <int ES> struct ElemOf;
template <> struct ElemOf<1> { using T = uint8_t; };
template <> struct ElemOf<2> { using T = uint16_t; };
template <> struct ElemOf<4> { using T = uint32_t; };

// DIR 0: compute -> token-major (a Worker sending its KV to the cache)
// DIR 1: token-major -> compute (received KV landing in the paged pool)
template <int DIR, int ES>
__global__ __launch_bounds__(kBlock) void transpose_pages_kernel(const TransposeArgs a) {
  using E = typename ElemOf<ES>::T;
  constexpr int VE = 16 / ES;            // elements per 16-byte vector
  extern __shared__ uint32_t lds_words[];
  E* lds = reinterpret_cast<E*>(lds_words);
  uint64_t* row_addr = reinterpret_cast<uint64_t*>(lds_words + a.tile_words);  // Cc entries

  const uint32_t chunk = blockIdx.x % a.n_chunks;              // column chunk
  const uint32_t rest = blockIdx.x / a.n_chunks;
  const uint32_t dchunk = rest % a.n_dchunks;                  // slice of head_dim
  const uint32_t t = rest / a.n_dchunks;                       // token within the page
  const uint64_t i = (uint64_t)blockIdx.y + (uint64_t)blockIdx.z * gridDim.y;
  if (i >= (uint64_t)a.n_pages) return;
  const int64_t blk = tload(a.block_ids + i);
  const int64_t tmp = tload(a.tm_pages + i);
  const bool bad_blk = (uint64_t)blk >= (uint64_t)a.n_blocks;
  const bool bad_tm = (uint64_t)tmp >= (uint64_t)a.n_tm_pages;
  if (bad_blk || bad_tm) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
      if (bad_blk) *reinterpret_cast<volatile uint32_t*>(a.status + ST_SLOT_PAGE) = 1u;
      if (bad_tm) *reinterpret_cast<volatile uint32_t*>(a.status + (DIR == 0 ? ST_SLOT_DST : ST_SLOT_SRC)) = 1u;
    }
    return;
  }
  // the tile is rows [d0, d0+D) x columns [c0, c0+Cc) of the token's [head_dim][C] matrix
  const int D = a.chunk_rows, C = a.n_cols, Cc = a.chunk_cols, PC = a.pitch;
  const int c0 = (int)chunk * Cc;
  const int d0 = (int)dchunk * D;
  // compute-side address of every row (column c of the token) handled by this workgroup
  for (int c = threadIdx.x; c < Cc; c += kBlock) {
    const int cg = c0 + c;
    const int k = cg & 1;
    const int hl = cg >> 1;
    const int h = hl / a.n_layers;
    const int l = hl - h * a.n_layers;
    const int64_t off = blk * a.block_stride + (int64_t)k * a.kv_stride + (int64_t)t * a.token_stride +
                        (int64_t)h * a.head_dim + d0;
    row_addr[c] = (uint64_t)a.layer_base[l] + (uint64_t)off * ES;
  }
  // token-major side: row d of the tile starts at tm_tok + d*C
  const uint64_t tm_tok = (uint64_t)a.tm_base +
                          (((uint64_t)(tmp * a.block_tokens + t) * a.head_dim + d0) * C + c0) * ES;
  const int vec_per_row = Cc / VE;       // 16-byte vectors along c per matrix row
  const int n_tm_vec = D * vec_per_row;
  const int dgs = D / VE;                // 16-byte vectors along d per compute row
  const int n_cp_vec = Cc * ((dgs + 3) & ~3);   // lanes walk (4 vectors of a row, row, group of 4)

  // Global loads are issued U at a time before any of them is consumed, so that a lane keeps U
  // 16-byte requests in flight instead of one.
  constexpr int U = 8;
  if (DIR == 1) {
    for (int base = 0; base < n_tm_vec; base += kBlock * U) {
      u32x4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        // out-of-range lanes re-read the last vector instead of branching around the load: a
        // branch here makes the compiler wait for each load before issuing the next
        int v = base + u * kBlock + threadIdx.x;
        v = v < n_tm_vec ? v : n_tm_vec - 1;
        const int d = v / vec_per_row, cv = v - d * vec_per_row;
        x[u] = __builtin_nontemporal_load(
            (const BIKV_GLOBAL u32x4*)(tm_tok + ((uint64_t)d * C + cv * VE) * ES));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int v = base + u * kBlock + threadIdx.x;
        if (v < n_tm_vec) {
          const int d = v / vec_per_row, cv = v - d * vec_per_row;
          uint32_t* w = lds_words + (d * PC + cv * VE) * ES / 4;   // 4-byte aligned by construction
          w[0] = x[u].x; w[1] = x[u].y; w[2] = x[u].z; w[3] = x[u].w;
        }
      }
    }
  }
  __syncthreads();   // row_addr (and, for DIR 1, the tile) are in LDS
  if (DIR == 0) {
    for (int base = 0; base < n_cp_vec; base += kBlock * U) {
      u32x4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        int o = base + u * kBlock + threadIdx.x;
        o = o < n_cp_vec ? o : n_cp_vec - 1;
        const int dgl = o & 3, c = (o >> 2) % Cc;
        int dg = ((o >> 2) / Cc) * 4 + dgl;
        dg = dg < dgs ? dg : dgs - 1;              // branch-free, as above
        x[u] = *(const BIKV_GLOBAL u32x4*)(row_addr[c] + (uint64_t)dg * 16);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int o = base + u * kBlock + threadIdx.x;
        const int dgl = o & 3, c = (o >> 2) % Cc, dg = ((o >> 2) / Cc) * 4 + dgl;
        if (o < n_cp_vec && dg < dgs) {
          E e[VE];
          __builtin_memcpy(e, &x[u], 16);
#pragma unroll
          for (int j = 0; j < VE; ++j) lds[(dg * VE + j) * PC + c] = e[j];
        }
      }
    }
    __syncthreads();
    for (int v = threadIdx.x; v < n_tm_vec; v += kBlock) {
      const int d = v / vec_per_row, cv = v - d * vec_per_row;
      const uint32_t* w = lds_words + (d * PC + cv * VE) * ES / 4;
      u32x4 x = {w[0], w[1], w[2], w[3]};
      __builtin_nontemporal_store(x, (BIKV_GLOBAL u32x4*)(tm_tok + ((uint64_t)d * C + cv * VE) * ES));
    }
  } else {
    for (int o = threadIdx.x; o < n_cp_vec; o += kBlock) {
      const int dgl = o & 3, c = (o >> 2) % Cc, dg = ((o >> 2) / Cc) * 4 + dgl;
      if (dg >= dgs) continue;
      E e[VE];
#pragma unroll
      for (int j = 0; j < VE; ++j) e[j] = lds[(dg * VE + j) * PC + c];
      u32x4 x;
      __builtin_memcpy(&x, e, 16);
      *(BIKV_GLOBAL u32x4*)(row_addr[c] + (uint64_t)dg * 16) = x;
    }
  }
}

// ---- K/V pairs as units -------------------------------------------------------------------------
// Column c = (h*L + l)*2 + k puts the K and the V element of one (head, layer) next to each other,
// so a token row is a sequence of UNITS {K[d], V[d]} of 2*ES bytes and the layout change is a
// transpose of units ([D][C/2] -> [C/2][D]) followed by a split of each unit in registers.
// LDS holds the tile transposed, [column pair][d] units, no padding. A lane on the compute side
// reads 32 contiguous bytes of a pair's row (16/ES values of d) and turns them into one K vector and
// one V vector; a lane on the token-major side moves the 16/(2*ES) units of one vector to or from as
// many pair rows. The 16-byte groups of a row are permuted by XOR with (vector index mod 8), which
// keeps the 16-byte accesses along d intact and spreads the unit-wise accesses of the other side
// (consecutive lanes = consecutive vectors of a token-major row) over all banks. For 2-byte elements
// this takes 5.5 LDS and ~60 VALU instructions per 16-byte vector moved; the element-wise kernel
// above takes 11 and ~105 (three integer divisions per vector).
// The XOR mask is the largest 2^k - 1 <= 7 with 2^k dividing the groups of a row, so that the permuted
// index stays inside the row for every head_dim the entry points accept.
// 32 bytes of units {K,V} (g0 = the first 16, g1 = the next 16) -> a K vector and a V vector.
template <int ES>
__device__ __forceinline__ void split_kv(const u32x4& g0, const u32x4& g1, u32x4& kx, u32x4& vx) {
  if constexpr (ES == 4) {
    kx = u32x4{g0.x, g0.z, g1.x, g1.z};
    vx = u32x4{g0.y, g0.w, g1.y, g1.w};
  } else {
    constexpr uint32_t SK = ES == 2 ? 0x05040100u : 0x06040200u;   // K halves / K bytes of two words
    constexpr uint32_t SV = ES == 2 ? 0x07060302u : 0x07050301u;
    kx.x = __builtin_amdgcn_perm(g0.y, g0.x, SK);
    kx.y = __builtin_amdgcn_perm(g0.w, g0.z, SK);
    kx.z = __builtin_amdgcn_perm(g1.y, g1.x, SK);
    kx.w = __builtin_amdgcn_perm(g1.w, g1.z, SK);
    vx.x = __builtin_amdgcn_perm(g0.y, g0.x, SV);
    vx.y = __builtin_amdgcn_perm(g0.w, g0.z, SV);
    vx.z = __builtin_amdgcn_perm(g1.y, g1.x, SV);
    vx.w = __builtin_amdgcn_perm(g1.w, g1.z, SV);
  }
}
// The inverse: a K vector and a V vector -> 32 bytes of units.
template <int ES>
__device__ __forceinline__ void join_kv(const u32x4& kx, const u32x4& vx, u32x4& g0, u32x4& g1) {
  if constexpr (ES == 4) {
    g0 = u32x4{kx.x, vx.x, kx.y, vx.y};
    g1 = u32x4{kx.z, vx.z, kx.w, vx.w};
  } else {
    constexpr uint32_t SL = ES == 2 ? 0x05040100u : 0x05010400u;   // units from the low / high half of
    constexpr uint32_t SH = ES == 2 ? 0x07060302u : 0x07030602u;   // a K word and a V word
    g0.x = __builtin_amdgcn_perm(vx.x, kx.x, SL);
    g0.y = __builtin_amdgcn_perm(vx.x, kx.x, SH);
    g0.z = __builtin_amdgcn_perm(vx.y, kx.y, SL);
    g0.w = __builtin_amdgcn_perm(vx.y, kx.y, SH);
    g1.x = __builtin_amdgcn_perm(vx.z, kx.z, SL);
    g1.y = __builtin_amdgcn_perm(vx.z, kx.z, SH);
    g1.z = __builtin_amdgcn_perm(vx.w, kx.w, SL);
    g1.w = __builtin_amdgcn_perm(vx.w, kx.w, SH);
  }
}

template <int ES> struct UnitOf;
template <> struct UnitOf<1> { using T = uint16_t; };
template <> struct UnitOf<2> { using T = uint32_t; };
template <> struct UnitOf<4> { using T = uint64_t; };

// Division of a small index by a divisor fixed at launch: the launcher passes m = ceil(2^32 / n) (0 when
// n == 1) and the quotient is the high word of x * m, exact for x, n < 2^16. An integer division costs
// ~25 instructions; a lane of this kernel moves only a handful of vectors, so three or four divisions
// in its prologue were a third of all the vector instructions it issued.
__device__ __forceinline__ uint32_t udiv_small(uint32_t x, uint32_t m) {
  return m ? __umulhi(x, m) : x;
}
struct UWalk {       // (outer, inner) of a linear index that advances by the block size per step
  uint32_t outer, inner;
};
__device__ __forceinline__ UWalk uwalk_start(uint32_t idx, uint32_t n_inner, uint32_t m) {
  UWalk w;
  w.outer = udiv_small(idx, m);
  w.inner = idx - w.outer * n_inner;
  return w;
}
__device__ __forceinline__ void uwalk_step(UWalk& w, uint32_t q, uint32_t r, uint32_t n_inner) {
  w.outer += q;
  w.inner += r;
  if (w.inner >= n_inner) {
    w.inner -= n_inner;
    w.outer += 1;
  }
}

// 16-byte payload store: nt, or nt with system scope (sc1), which has no C++ spelling for 16-byte accesses.
__device__ __forceinline__ void store16(uint64_t p, const u32x4& v, bool sys) {
  if (sys)
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt" : : "v"(p), "v"(v) : "memory");
  else
    __builtin_nontemporal_store(v, (BIKV_GLOBAL u32x4*)p);
}

// lanes 32-63 of x <-> lanes 0-31 of y, all four dwords. With x = {K of layer A | K of layer B} and
// y = {V of layer A | V of layer B} (half-waves) this yields {K A | V A} and {K B | V B}, and back: the
// exchange is its own inverse.
__device__ __forceinline__ void swap_half_waves(u32x4& x, u32x4& y) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const auto r = __builtin_amdgcn_permlane32_swap(x[i], y[i], false, false);
    x[i] = r[0];
    y[i] = r[1];
  }
}
// the 64-bit value lane `src` of this wave holds, as a wave-uniform value
__device__ __forceinline__ uint64_t from_lane(uint64_t v, int src) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, src);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), src);
  return ((uint64_t)hi << 32) | lo;
}

template <int DIR, int ES, int B>
__global__ __launch_bounds__(B) void transpose_pairs_kernel(const TransposeArgs a) {
  using Unit = typename UnitOf<ES>::T;
  constexpr uint32_t UB = 2 * ES;               // bytes of a unit
  constexpr uint32_t UPV = 16 / UB;             // units in a 16-byte vector
  constexpr uint32_t UPV_SHIFT = ES == 1 ? 3 : (ES == 2 ? 2 : 1);
  constexpr uint32_t DPV = 16 / ES;             // values of d in a compute-side vector
  extern __shared__ uint32_t lds_words[];
  u32x4* lds_vec = reinterpret_cast<u32x4*>(lds_words);
  Unit* lds_unit = reinterpret_cast<Unit*>(lds_words);
  uint64_t* row_addr = reinterpret_cast<uint64_t*>(lds_words + a.tile_words);  // K row of each pair

  const uint32_t tid = threadIdx.x;
  const bool sys = a.sys_scope != 0;
  const uint32_t t = udiv_small(blockIdx.x, a.m_chunks);       // token within the page
  const uint32_t chunk = blockIdx.x - t * a.n_chunks;          // column chunk
  const uint64_t i = (uint64_t)blockIdx.y + (uint64_t)blockIdx.z * gridDim.y;
  if (i >= (uint64_t)a.n_pages) return;
  const int64_t blk = tload(a.block_ids + i);
  const int64_t tmp = tload(a.tm_pages + i);
  const bool bad_blk = (uint64_t)blk >= (uint64_t)a.n_blocks;
  const bool bad_tm = (uint64_t)tmp >= (uint64_t)a.n_tm_pages;
  if (bad_blk || bad_tm) {
    if (tid == 0 && blockIdx.x == 0) {
      if (bad_blk) *reinterpret_cast<volatile uint32_t*>(a.status + ST_SLOT_PAGE) = 1u;
      if (bad_tm) *reinterpret_cast<volatile uint32_t*>(a.status + (DIR == 0 ? ST_SLOT_DST : ST_SLOT_SRC)) = 1u;
    }
    return;
  }
  const uint32_t D = (uint32_t)a.head_dim, C = (uint32_t)a.n_cols, L = (uint32_t)a.n_layers;
  const uint32_t Cw = (uint32_t)a.chunk_cols >> 1;   // column pairs in the tile
  const uint32_t vpr = Cw >> UPV_SHIFT;              // 16-byte vectors per token-major row piece
  const uint32_t dgs = D / DPV;                      // 16-byte vectors per compute row
  const uint32_t gpr = (D * UB) >> 4;                // 16-byte groups per LDS row (even)
  const uint32_t sm = (uint32_t)a.swz_mask;          // 2^k - 1 with 2^k dividing gpr, at most 7
  const uint32_t cp0 = chunk * Cw;
  // The compute side is walked layer by layer (all heads of a layer, K rows then V rows, are
  // neighbours in memory), the LDS tile is indexed by column pair (head-major): entry j of the table
  // holds the K row address of the j-th pair in walking order and, in its top 16 bits, that pair's
  // index in the tile. A tile that is only a column chunk of the token is walked in column order.
  const uint64_t tok_off = (uint64_t)(blk * a.block_stride + (int64_t)t * a.token_stride) * ES;   // uniform
  auto pair_of = [&](uint32_t j, uint32_t& l, uint32_t& h, uint32_t& cp) {
    if (a.n_chunks == 1) {
      l = udiv_small(j, a.m_heads);
      h = j - l * a.n_heads;
      cp = h * L + l;
    } else {
      cp = j;
      h = udiv_small(cp0 + cp, a.m_layers);
      l = (cp0 + cp) - h * L;
    }
  };
  for (uint32_t j = tid; j < Cw; j += B) {
    uint32_t h, l, cp;
    pair_of(j, l, h, cp);
    row_addr[j] = ((uint64_t)a.layer_base[l] + tok_off + (uint64_t)(h * D * ES)) | ((uint64_t)cp << 48);
  }
  const uint64_t kv_bytes = (uint64_t)a.kv_stride * ES;
  // token-major side: a uniform base and 32-bit offsets inside the token (a token is far below 4 GiB)
  BIKV_GLOBAL char* tm_tok = (BIKV_GLOBAL char*)(uint64_t)a.tm_base +
                             (((uint64_t)(tmp * a.block_tokens + t) * D) * C + (uint64_t)cp0 * 2) * ES;
  const uint32_t tm_row_bytes = C * ES;
  const uint32_t n_tm = D * vpr;                // vectors on the token-major side
  const uint32_t n_cp = Cw * dgs;               // (pair, 16/ES values of d) items on the compute side
  // Unit (pair cp, d) sits in group (d / UPV) ^ s of row cp, s = (cp / UPV) & sm = the index of the
  // token-major vector the pair belongs to, mod 8 (mod a smaller power of two when the row has fewer
  // aligned groups, e.g. head_dim 80 at 2 bytes: 20 groups, mod 4).

  if (DIR == 1) {
    // token-major rows -> LDS, the units of a vector to as many pair rows
    constexpr uint32_t U = 8;
    UWalk w = uwalk_start(tid, vpr, a.m_vpr);                  // (d, vector within the row piece)
    for (uint32_t base = 0; base < n_tm; base += B * U) {
      u32x4 x[U];
      UWalk wu = w;
#pragma unroll
      for (uint32_t u = 0; u < U; ++u) {
        if (base + u * B >= n_tm) break;                       // whole workgroup past the end: nothing to load
        const uint32_t d = wu.outer < D ? wu.outer : 0;        // a lane past the end re-reads row 0
        x[u] = __builtin_nontemporal_load((const BIKV_GLOBAL u32x4*)(tm_tok + (d * tm_row_bytes + wu.inner * 16)));
        uwalk_step(wu, a.q_tm, a.r_tm, vpr);
      }
#pragma unroll
      for (uint32_t u = 0; u < U; ++u) {
        if (base + u * B >= n_tm) break;
        if (w.outer < D) {
          const uint32_t cv = w.inner, d = w.outer;
          // unit index inside row (cv*UPV + j): group (d/UPV ^ s) * UPV + d % UPV
          Unit* row = lds_unit + (cv * UPV) * D + ((((d >> UPV_SHIFT) ^ (cv & sm)) << UPV_SHIFT) | (d & (UPV - 1)));
          Unit e[UPV];
          __builtin_memcpy(e, &x[u], 16);
#pragma unroll
          for (uint32_t j = 0; j < UPV; ++j) row[j * D] = e[j];
        }
        uwalk_step(w, a.q_tm, a.r_tm, vpr);
      }
    }
    __syncthreads();
    // LDS -> compute rows: 32 bytes of units become one K vector and one V vector
    UWalk o = uwalk_start(tid, dgs, a.m_dgs);                  // (pair, group of d)
    if (a.kv_swap) {
      // K rows and V rows of a (token, layer) are the two halves of ONE contiguous KiB, and a half-wave
      // covers exactly the K rows of a layer: lanes 0-31 hold {K, V} of layer A, lanes 32-63 of layer B.
      // Exchanging half-waves turns {K A | K B}, {V A | V B} into {K A | V A}, {K B | V B}: each store
      // instruction then writes one whole KiB instead of two half-KiB pieces in two layer tensors.
      const uint32_t lane = tid & 63u;
      for (uint32_t base = 0; base < n_cp; base += B) {
        const bool valid = o.outer < Cw;
        const uint64_t entry = row_addr[valid ? o.outer : 0];
        const uint32_t cp = (uint32_t)(entry >> 48), dg = o.inner;
        const uint32_t s = (cp >> UPV_SHIFT) & sm;
        const uint32_t flip = (dg >> 2) & 1;
        const u32x4 lo = lds_vec[cp * gpr + ((2 * dg + flip) ^ s)];
        const u32x4 hi = lds_vec[cp * gpr + ((2 * dg + 1 - flip) ^ s)];
        const u32x4 g0 = flip ? hi : lo, g1 = flip ? lo : hi;
        u32x4 kx, vx;
        split_kv<ES>(g0, g1, kx, vx);
        swap_half_waves(kx, vx);                               // kx = {K A | V A}, vx = {K B | V B}
        const uint64_t ra = entry & 0xFFFFFFFFFFFFull;         // K row of this lane's pair
        const uint64_t kib_a = from_lane(ra, 0), kib_b = from_lane(ra, 32);   // lane 0 / 32: head 0 of its layer
        const bool valid_a = __builtin_amdgcn_readlane((int)valid, 0) != 0;
        const bool valid_b = __builtin_amdgcn_readlane((int)valid, 32) != 0;
        if (valid_a) store16(kib_a + lane * 16u, kx, sys);
        if (valid_b) store16(kib_b + lane * 16u, vx, sys);
        uwalk_step(o, a.q_cp, a.r_cp, dgs);
      }
    } else {
      for (uint32_t base = 0; base < n_cp; base += B) {
        if (o.outer < Cw) {
          const uint64_t entry = row_addr[o.outer];
          const uint32_t cp = (uint32_t)(entry >> 48), dg = o.inner;
          const uint32_t s = (cp >> UPV_SHIFT) & sm;
          const uint32_t flip = (dg >> 2) & 1;                   // lanes 0-3 and 4-7 start on different halves
          const u32x4 lo = lds_vec[cp * gpr + ((2 * dg + flip) ^ s)];
          const u32x4 hi = lds_vec[cp * gpr + ((2 * dg + 1 - flip) ^ s)];
          const u32x4 g0 = flip ? hi : lo, g1 = flip ? lo : hi;
          u32x4 kx, vx;
          split_kv<ES>(g0, g1, kx, vx);
          const uint64_t ra = (entry & 0xFFFFFFFFFFFFull) + (uint64_t)(dg * 16);
          store16(ra, kx, sys);
          store16(ra + kv_bytes, vx, sys);
        }
        uwalk_step(o, a.q_cp, a.r_cp, dgs);
      }
    }
  } else {
    // compute rows -> LDS: a K vector and a V vector interleave into 32 bytes of units
    __syncthreads();                                            // row_addr
    constexpr uint32_t U = 4;
    UWalk o = uwalk_start(tid, dgs, a.m_dgs);
    for (uint32_t base = 0; base < n_cp; base += B * U) {
      u32x4 kx[U], vx[U];
      uint32_t cps[U];
      UWalk ou = o;
#pragma unroll
      for (uint32_t u = 0; u < U; ++u) {
        if (base + u * B >= n_cp) break;                       // whole workgroup past the end: nothing to load
        const uint32_t jj = ou.outer < Cw ? ou.outer : 0;      // a lane past the end re-reads row 0
        const uint64_t entry = row_addr[jj];
        cps[u] = (uint32_t)(entry >> 48);
        if (a.kv_swap) {
          // one contiguous KiB per load instruction: the whole wave reads {K | V} of layer A, then of layer B
          // (see the store side of the other direction); the exchange after the loads gives every lane the
          // K vector and the V vector of its own pair
          const uint64_t row = entry & 0xFFFFFFFFFFFFull;
          const uint64_t kib_a = from_lane(row, 0), kib_b = from_lane(row, 32);
          const uint32_t lane = tid & 63u;
          kx[u] = __builtin_nontemporal_load((const BIKV_GLOBAL u32x4*)(kib_a + lane * 16u));
          vx[u] = __builtin_nontemporal_load((const BIKV_GLOBAL u32x4*)(kib_b + lane * 16u));
        } else {
          const uint64_t ra = (entry & 0xFFFFFFFFFFFFull) + (uint64_t)(ou.inner * 16);
          kx[u] = __builtin_nontemporal_load((const BIKV_GLOBAL u32x4*)ra);
          vx[u] = __builtin_nontemporal_load((const BIKV_GLOBAL u32x4*)(ra + kv_bytes));
        }
        uwalk_step(ou, a.q_cp, a.r_cp, dgs);
      }
#pragma unroll
      for (uint32_t u = 0; u < U; ++u) {
        if (base + u * B >= n_cp) break;
        if (a.kv_swap) swap_half_waves(kx[u], vx[u]);          // {K A | V A}, {K B | V B} -> {K A | K B}, {V A | V B}
        if (o.outer < Cw) {
          const uint32_t cp = cps[u], dg = o.inner;
          const uint32_t s = (cp >> UPV_SHIFT) & sm;
          const uint32_t flip = (dg >> 2) & 1;                 // as in the load: lanes 0-3 and 4-7 on different halves
          u32x4 g0, g1;
          join_kv<ES>(kx[u], vx[u], g0, g1);
          lds_vec[cp * gpr + ((2 * dg + flip) ^ s)] = flip ? g1 : g0;
          lds_vec[cp * gpr + ((2 * dg + 1 - flip) ^ s)] = flip ? g0 : g1;
        }
        uwalk_step(o, a.q_cp, a.r_cp, dgs);
      }
    }
    __syncthreads();
    UWalk w = uwalk_start(tid, vpr, a.m_vpr);
    for (uint32_t base = 0; base < n_tm; base += B) {
      if (w.outer < D) {
        const uint32_t cv = w.inner, d = w.outer;
        const Unit* row = lds_unit + (cv * UPV) * D + ((((d >> UPV_SHIFT) ^ (cv & sm)) << UPV_SHIFT) | (d & (UPV - 1)));
        Unit e[UPV];
#pragma unroll
        for (uint32_t j = 0; j < UPV; ++j) e[j] = row[j * D];
        u32x4 x;
        __builtin_memcpy(&x, e, 16);
        store16((uint64_t)(tm_tok + (d * tm_row_bytes + cv * 16)), x, sys);
      }
      uwalk_step(w, a.q_tm, a.r_tm, vpr);
    }
  }
}

template <int DIR>
static hipError_t launch_transpose_dir(const TransposeArgs& a, dim3 grid, size_t lds, hipStream_t s) {
  switch (a.elem_bytes) {
    case 1: hipLaunchKernelGGL((transpose_pages_kernel<DIR, 1>), grid, dim3(kBlock), lds, s, a); break;
    case 2: hipLaunchKernelGGL((transpose_pages_kernel<DIR, 2>), grid, dim3(kBlock), lds, s, a); break;
    case 4: hipLaunchKernelGGL((transpose_pages_kernel<DIR, 4>), grid, dim3(kBlock), lds, s, a); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

// Chooses the column chunk (a divisor of C that is a whole number of 16-byte vectors and keeps the
// LDS tile near 32 KiB) and launches. Returns hipErrorInvalidValue for shapes the kernel does not
// take (the caller has already validated them; this is a second line of defence).
hipError_t launch_transpose_pages(int dir, TransposeArgs& a, hipStream_t stream) {
  if (a.n_pages <= 0) return hipSuccess;
  refresh_tuning();
  const int ES = a.elem_bytes;
  if (ES != 1 && ES != 2 && ES != 4) return hipErrorInvalidValue;
  const int VE = 16 / ES;
  const int C = a.n_cols, D = a.head_dim;
  if (C <= 0 || D <= 0 || C % VE != 0 || D % VE != 0 || (C & 1)) return hipErrorInvalidValue;
  // Tile = [Dd rows of head_dim] x [Cc columns]. Measured on MI355X (Qwen2-1.5B/7B and Llama-3-8B
  // token shapes): throughput follows the width of the contiguous pieces on BOTH sides — whole
  // compute rows (Dd = head_dim) and the widest column chunk that fits LDS. Cutting head_dim to make
  // room for wider chunks lost 10-25 %, a 16 KiB tile lost 30-60 %, so the default is the full
  // head_dim with a ~60 KiB tile (two workgroups per CU).
  if (tuning().transpose_pairs != 0 && tuning().transpose_dsplit <= 1) {
    // the pair kernel: unpadded tile [Cc/2 pairs][D] units, the widest column chunk that fits
    const int64_t budget = (int64_t)tuning().transpose_lds_kib * 1024;
    int best = 0;
    for (int cc = VE; cc <= C; cc += VE)
      if (C % cc == 0 && (int64_t)D * cc * ES + (cc / 2) * 8 <= budget) best = cc;
    if (best > 0) {
      a.chunk_rows = D;
      a.n_dchunks = 1;
      a.chunk_cols = best;
      a.pitch = 0;
      const int gpr = D * ES / 8;               // 16-byte groups per LDS row
      int low = gpr & -gpr;
      a.swz_mask = (low > 8 ? 8 : low) - 1;
      a.n_chunks = (uint32_t)(C / best);
      a.tile_words = (uint32_t)((int64_t)D * best * ES / 4);
      const size_t lds = (size_t)a.tile_words * 4 + (size_t)(best / 2) * 8;
      const int64_t gx = (int64_t)a.n_chunks * a.block_tokens;
      const int64_t gy = a.n_pages < 32768 ? a.n_pages : 32768;
      const int64_t gz = (a.n_pages + gy - 1) / gy;
      if (gx >= (int64_t(1) << 24) || gx * a.n_chunks > (int64_t(1) << 32) || gz > 65535) return hipErrorInvalidValue;
      const dim3 grid((uint32_t)gx, (uint32_t)gy, (uint32_t)gz);
      // The load writes the pool in KiB pieces and does best with many small workgroups in flight; the store
      // reads them and does best with the waves of a tile sharing one workgroup (measured: 256 / 512 lanes).
      const int block = tuning().transpose_block > 0 ? tuning().transpose_block : (dir == 1 ? 256 : 512);
      // divisors of the kernel's index arithmetic as multipliers (see udiv_small); all are far below 2^16
      const uint32_t cw = (uint32_t)best / 2, upv = 16u / (2u * (uint32_t)ES);
      const uint32_t vpr = cw / upv, dgs = (uint32_t)D / (uint32_t)VE;
      const uint32_t n_heads = (uint32_t)C / (2u * (uint32_t)a.n_layers);
      if (vpr == 0 || dgs == 0 || n_heads == 0 || C >= 65536 || D >= 65536) return hipErrorInvalidValue;
      auto magic = [](uint32_t n) { return n <= 1 ? 0u : (uint32_t)(((uint64_t(1) << 32) + n - 1) / n); };
      a.n_heads = n_heads;
      a.m_heads = magic(n_heads);
      a.m_layers = magic((uint32_t)a.n_layers);
      a.m_vpr = magic(vpr);
      a.m_dgs = magic(dgs);
      a.m_chunks = magic(a.n_chunks);
      a.sys_scope = (uint32_t)tuning().transpose_sc1;
      // K rows and V rows of a (token, layer) adjacent (the Worker's [tokens, 2, heads, dim] tensors), half a
      // KiB each, whole token in one tile: half-waves can be exchanged so that every global access of a wave
      // on the compute side is one contiguous KiB
      a.kv_swap = (tuning().transpose_kvswap != 0 && a.n_chunks == 1 && n_heads * dgs == 32 &&
                   a.kv_stride * ES == 512 && (uint32_t)block % 64u == 0) ? 1u : 0u;
      a.q_tm = (uint32_t)block / vpr;
      a.r_tm = (uint32_t)block % vpr;
      a.q_cp = (uint32_t)block / dgs;
      a.r_cp = (uint32_t)block % dgs;
#define BIKV_LAUNCH_PAIRS(DIR_, ES_, B_) \
  hipLaunchKernelGGL((transpose_pairs_kernel<DIR_, ES_, B_>), grid, dim3(B_), lds, stream, a)
#define BIKV_LAUNCH_PAIRS_B(DIR_, ES_)                         \
  do {                                                         \
    if (block == 256) BIKV_LAUNCH_PAIRS(DIR_, ES_, 256);       \
    else if (block == 1024) BIKV_LAUNCH_PAIRS(DIR_, ES_, 1024); \
    else if (block == 128) BIKV_LAUNCH_PAIRS(DIR_, ES_, 128);  \
    else BIKV_LAUNCH_PAIRS(DIR_, ES_, 512);                    \
  } while (0)
      if (dir == 0) {
        if (ES == 1) BIKV_LAUNCH_PAIRS_B(0, 1);
        else if (ES == 2) BIKV_LAUNCH_PAIRS_B(0, 2);
        else BIKV_LAUNCH_PAIRS_B(0, 4);
      } else {
        if (ES == 1) BIKV_LAUNCH_PAIRS_B(1, 1);
        else if (ES == 2) BIKV_LAUNCH_PAIRS_B(1, 2);
        else BIKV_LAUNCH_PAIRS_B(1, 4);
      }
#undef BIKV_LAUNCH_PAIRS_B
#undef BIKV_LAUNCH_PAIRS
      return hipGetLastError();
    }
  }
  const int budget_elems = (tuning().transpose_lds_kib * 1024) / ES;
  int dsplit = tuning().transpose_dsplit;
  if (dsplit <= 0) dsplit = 1;
  if (D % (dsplit * VE) != 0) return hipErrorInvalidValue;
  const int Dd = D / dsplit;
  int best = VE;
  for (int cc = VE; cc <= C; cc += VE) {
    if (C % cc != 0) continue;
    const int pitch = cc + 4 / ES;
    if ((int64_t)Dd * pitch <= budget_elems) best = cc;
  }
  a.chunk_rows = Dd;
  a.n_dchunks = (uint32_t)dsplit;
  a.chunk_cols = best;
  a.pitch = best + 4 / ES;                      // +4 bytes: strided element accesses hit distinct banks
  a.n_chunks = (uint32_t)(C / best);
  a.tile_words = (uint32_t)(((int64_t)Dd * a.pitch * ES + 7) / 8 * 2);   // keeps row_addr 8-byte aligned
  const size_t lds = (size_t)a.tile_words * 4 + (size_t)best * 8;
  if (lds > 64 * 1024) return hipErrorInvalidValue;
  const int64_t gx = (int64_t)a.n_chunks * a.n_dchunks * a.block_tokens;
  const int64_t gy = a.n_pages < 32768 ? a.n_pages : 32768;
  const int64_t gz = (a.n_pages + gy - 1) / gy;
  if (gx >= (int64_t(1) << 24) || gz > 65535) return hipErrorInvalidValue;
  const dim3 grid((uint32_t)gx, (uint32_t)gy, (uint32_t)gz);
  return dir == 0 ? launch_transpose_dir<0>(a, grid, lds, stream)
                  : launch_transpose_dir<1>(a, grid, lds, stream);
}

}  // namespace bikv
